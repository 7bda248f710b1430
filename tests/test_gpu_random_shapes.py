"""Seeded random shapes and options against the CPU oracle, to the same bars as the hand-picked cases: row counts,
row lengths, formats, scale layouts, masks and weights are drawn at random so that the tile shape, the bounds handling
and the scale layout of a call vary together.  Every seed collects its failing cases and fails once at the end."""
import os
import random

import pytest
import torch

from oracle import torch_ref
from tests._util import assert_same
from tests.test_gpu_swiglu import check_fused
from tests.test_gpu_swiglu_backward import check_backward, make_inputs, run_gpu

pytestmark = pytest.mark.gpu


def _tk():
    import tilekernels_amd
    return tilekernels_amd


# TK_FUZZ_SEEDS=101,102,... adds runs with other seeds to the committed ones
EXTRA_SEEDS = [int(v) for v in os.getenv('TK_FUZZ_SEEDS', '').split(',') if v.strip()]


def _modes(rng):
    return rng.choice([(False, False, False), (False, True, False), (True, False, False), (True, True, False), (True, True, True)])


@pytest.mark.parametrize('seed', [11, 12] + EXTRA_SEEDS)
def test_random_casts_swiglu_and_moe_rows(seed):
    """per_token_cast, cast_back, per_block_cast, the fused SwiGLU cast, expand_to_fused and reduce_fused."""
    tk = _tk()
    rng = random.Random(seed)
    N_CASES, failures, desc = 120, [], ''
    for case in range(N_CASES):
        kind = rng.choice(['cast', 'cast', 'back', 'swiglu', 'swiglu', 'block', 'expand', 'reduce'])
        try:
            if kind in ('cast', 'back'):
                N = rng.choice([16, 32, 64, 128])
                K = rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 11, 13, 14, 16, 22]) * rng.choice([128, 256, 512, 1024]) if rng.random() < 0.8 else rng.randrange(1, 60) * 64
                if K % N: K = (K // N + 1) * N
                M = rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 33, 63, 130, 257])
                fmt = rng.choice(['e4m3', 'e2m1'])
                dt = rng.choice([torch.bfloat16, torch.float32])
                col, rnd, pk = _modes(rng)
                desc = f'{kind} M={M} K={K} N={N} {fmt} {dt} col={col} rnd={rnd} pk={pk}'
                x = (torch.randn((M, K)) * rng.choice([0.01, 1.0, 100.0])).to(dt)
                kw = dict(use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=pk)
                want = torch_ref.cast(x, fmt, (1, N), **kw)
                got = tk.quant.per_token_cast(x.cuda(), fmt, N, **kw)
                assert_same(got[0], want[0], 'codes'); assert_same(got[1], want[1], 'sf')
                if kind == 'back':
                    o = rng.choice(['bf16', 'fp32'])
                    assert_same(tk.quant.cast_back(got, o, (1, N)), torch_ref.cast_back(want, o, (1, N)), 'back ' + o)
            elif kind == 'block':
                blk = rng.choice([(128, 128), (32, 32), (32, 128), (128, 32)])
                M = rng.choice([1, 31, 32, 33, 127, 128, 129, 300])
                K = rng.randrange(1, 40) * 64
                fmt = rng.choice(['e4m3', 'e2m1'])
                col, rnd, pk = _modes(rng)
                desc = f'block M={M} K={K} {blk} {fmt} col={col} rnd={rnd} pk={pk}'
                x = torch.randn((M, K)).to(torch.bfloat16)
                kw = dict(use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=pk)
                want = torch_ref.cast(x, fmt, blk, **kw)
                got = tk.quant.per_block_cast(x.cuda(), fmt, blk, **kw)
                assert_same(got[0], want[0], 'codes'); assert_same(got[1], want[1], 'sf')
                o = rng.choice(['bf16', 'fp32'])
                assert_same(tk.quant.cast_back(got, o, blk), torch_ref.cast_back(want, o, blk), 'back ' + o)
            elif kind == 'swiglu':
                H = rng.choice([1, 2, 3, 4, 5, 7, 8, 11, 16, 22]) * rng.choice([128, 256, 512, 1024]) if rng.random() < 0.8 else rng.randrange(1, 40) * 128
                whole = rng.random() < 0.2
                N = H if whole else 128
                col, rnd, pk = (False, rng.random() < 0.5, False) if whole else _modes(rng)
                dt = rng.choice([torch.bfloat16, torch.bfloat16, torch.float32])
                T, topk, E = rng.choice([(1, 1, 1), (5, 2, 3), (17, 4, 8), (40, 3, 5)]); desc = "swiglu setup"
                g = torch.Generator().manual_seed(case)
                pe, ptt, w = tk.testing.generate_moe_layout(T, E, topk, rng.choice([1, 4, 16]), g, drop_fraction=0.1)
                R = pe.numel()
                with_mask, with_w = rng.random() < 0.5, rng.random() < 0.5
                clamp = rng.choice([None, None, 5.0, 0.5])
                desc = f'swiglu R={R} H={H} N={N} {dt} col={col} rnd={rnd} pk={pk} mask={with_mask} w={with_w} clamp={clamp}'
                x = torch.randn((R, 2 * H), generator=g) * 2
                x[pe < 0] = 0
                x = x.to(dt)
                kw = dict(use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=pk, swiglu_clamp_value=clamp)
                want = torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', N, ptt if with_w else None, w if with_w else None, pe if with_mask else None, **kw)
                got = tk.quant.swiglu_forward_and_per_token_cast(x.cuda(), 'e4m3', N, ptt.cuda() if with_w else None, w.cuda() if with_w else None, pe.cuda() if with_mask else None, **kw)
                check_fused(got, want, H // N, pk, desc)
            elif kind in ('expand', 'reduce'):
                T, topk, E = rng.choice([(1, 1, 1), (9, 2, 3), (65, 4, 8), (130, 8, 16), (33, 6, 7), (50, 1, 4)])
                hidden = rng.choice([64, 128, 256, 320, 512, 576, 1024, 2048, 2304, 4096]) if kind == 'expand' else rng.choice([256, 512, 768, 1024, 2048, 2304, 3584])
                dt = rng.choice([torch.bfloat16, torch.float32] + ([torch.float8_e4m3fn] if kind == 'expand' else []))
                desc = f'{kind} T={T} topk={topk} E={E} hidden={hidden} {dt}'
                g = torch.Generator().manual_seed(case)
                idx = torch.stack([torch.randperm(max(E, topk), generator=g)[:topk] % E for _ in range(T)]).to(torch.int64)
                if rng.random() < 0.3: idx[torch.rand(idx.shape, generator=g) < 0.1] = -1
                m = tk.moe.get_fused_mapping(idx.cuda(), E, 0, rng.choice([1, 16, 128]))
                pe, t2p = m[0], m[3]
                x = torch.randn((T, hidden), generator=g).to(dt)
                y = tk.moe.expand_to_fused(x.cuda(), t2p, pe)
                want = torch_ref.expand_to_fused(x, t2p.cpu(), pe.cpu())
                assert_same(y, want, 'expanded')
                if kind == 'reduce':
                    w = torch.rand((T, topk), generator=g)
                    fp8 = rng.choice(['', 'e4m3'])
                    got = tk.moe.reduce_fused(y, w.cuda(), t2p, fp8_format=fp8)
                    wr = torch_ref.reduce_fused(want, w, t2p.cpu(), fp8_format=fp8)
                    assert_same(got, wr, 'reduced ' + fp8)
        except AssertionError as e:
            failures.append(f'case {case}: {desc}: {str(e)[:300]}')
        except Exception as e:
            failures.append(f'case {case}: {desc}: {type(e).__name__}: {str(e)[:300]}')
    assert not failures, '\n'.join(failures)


@pytest.mark.parametrize('seed', [21, 22] + EXTRA_SEEDS)
def test_random_operators_around_the_path(seed):
    """The fused backward, the per-channel family, E5M6, the lossless re-blocking, the mapping, expansion with scales
    and re-quantisation of quantised input."""
    tk = _tk()
    rng = random.Random(seed)
    N_CASES, failures, desc = 120, [], ''
    for case in range(N_CASES):
        kind = rng.choice(['backward', 'pc', 'pct', 'pcs', 'e5m6', 'lossless', 'mapping', 'expand_sf', 'requant'])
        desc = kind + ' setup'
        try:
            if kind == 'backward':
                T, K, E = rng.choice([(1, 1, 1), (7, 2, 4), (33, 4, 8), (20, 3, 5)])
                H = rng.choice([128, 256, 384, 512, 640, 1024, 1280, 1536, 2048, 2560])
                N = rng.choice([32, 128]); rnd = rng.random() < 0.5; clamp = rng.choice([None, 10.0, 0.5])
                desc = f'backward T={T} K={K} E={E} H={H} N={N} rnd={rnd} clamp={clamp}'
                xq, go, w, ptt, t2p = make_inputs(T, K, E, H, N, seed=case, drop=rng.choice([0.0, 0.1]), alignment=rng.choice([1, 16]))
                if xq[0].shape[0] == 0: continue
                want = torch_ref.swiglu_backward_and_per_token_cast(xq, go, w, ptt, t2p, N, rnd, clamp)
                check_backward(run_gpu(tk, xq, go, w, ptt, t2p, N, rnd, clamp), want, rnd, desc)
            elif kind in ('pc', 'pct', 'pcs'):
                M = rng.choice([128, 256, 384, 640]); K = rng.randrange(1, 24) * 64
                npt = rng.choice([32, 128]); rnd = rng.random() < 0.5
                if kind == 'pc':
                    K = rng.randrange(1, 24) * 128
                    desc = f'per_channel M={M} K={K} rnd={rnd}'
                    x = torch.randn((M, K)).to(rng.choice([torch.bfloat16, torch.float32]))
                    want = torch_ref.cast(x, 'e4m3', (128, 1), round_sf=rnd)
                    got = tk.quant.per_channel_cast(x.cuda(), 'e4m3', 128, rnd)
                elif kind == 'pct':
                    desc = f'per_channel_T M={M} K={K} npt={npt} rnd={rnd}'
                    x = torch.randn((M, K)).to(torch.bfloat16)
                    want = torch_ref.per_channel_cast_and_transpose(x, npt, rnd)
                    got = tk.quant.per_channel_cast_and_transpose(x.cuda(), 'e4m3', npt, rnd)
                else:
                    K = rng.randrange(1, 16) * 128; wt = rng.random() < 0.5; clamp = rng.choice([None, 3.0])
                    desc = f'swiglu_per_channel M={M} K2={K} npt={npt} rnd={rnd} without_T={wt} clamp={clamp}'
                    x = (torch.randn((M, K)) * 2).to(torch.bfloat16)
                    want = torch_ref.swiglu_forward_and_per_channel_cast_and_transpose(x, npt, rnd, wt, clamp)
                    got = tk.quant.swiglu_forward_and_per_channel_cast_and_transpose(x.cuda(), 'e4m3', npt, rnd, wt, clamp)
                assert_same(got[0], want[0], 'codes'); assert_same(got[1], want[1], 'sf')
            elif kind == 'e5m6':
                M = rng.choice([1, 3, 8, 65]); K = rng.randrange(1, 300) * 8
                dt = rng.choice([torch.bfloat16, torch.float32])
                col, rnd, pk = rng.choice([(False, False, False), (False, True, False), (True, True, False), (True, True, True)])
                desc = f'e5m6 M={M} K={K} {dt} col={col} rnd={rnd} pk={pk}'
                x = (torch.randn((M, K)) * rng.choice([1e-3, 1.0, 1e3])).to(dt)
                want = torch_ref.cast_to_e5m6(x, K, col, rnd, pk)
                got = tk.quant.per_token_cast(x.cuda(), 'e5m6', K, use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=pk)
                assert_same(got[0], want[0], 'codes'); assert_same(got[1], want[1], 'sf')
                o = rng.choice(['bf16', 'fp32'])
                assert_same(tk.quant.cast_back(got, o, (1, K), x_special_fmt='e5m6'), torch_ref.cast_back_from_e5m6(want, o, (1, K)), 'back')
            elif kind == 'lossless':
                M = rng.choice([1, 5, 32, 100, 129, 260]); K = rng.randrange(1, 40) * 128
                ib = rng.choice([(1, 32), (1, 32), (32, 32), (1, 128)])
                ob = rng.choice([(1, 128), (128, 128), (32, 32), (32, 128), (128, 32)])
                if ob[0] % ib[0] or ob[1] % ib[1]: continue
                desc = f'lossless M={M} K={K} in={ib} out={ob}'
                x = torch.randn((M, K)).to(torch.bfloat16)
                x4 = torch_ref.cast(x, 'e2m1', ib, round_sf=True)
                want = torch_ref.per_block_cast_lossless(x4, 'e4m3', ib, ob, round_sf=True)
                got = tk.quant.per_block_cast_lossless((x4[0].cuda(), x4[1].cuda()), 'e4m3', ib, ob, round_sf=True)
                assert_same(got[0], want[0], 'codes'); assert_same(got[1], want[1], 'sf')
            elif kind in ('mapping', 'expand_sf'):
                T, K, E = rng.choice([(1, 1, 1), (9, 2, 3), (300, 8, 64), (1000, 6, 17), (513, 9, 32), (64, 1, 128)])
                al = rng.choice([1, 16, 64, 128])
                desc = f'{kind} T={T} K={K} E={E} align={al}'
                g = torch.Generator().manual_seed(case)
                idx = torch.topk(torch.rand((T, E), generator=g), K, dim=-1).indices
                if rng.random() < 0.5: idx = idx.masked_fill(torch.rand(idx.shape, generator=g) < 0.15, -1)
                want = torch_ref.get_fused_mapping(idx.contiguous(), E, al)
                got = tk.moe.get_fused_mapping(idx.contiguous().cuda(), E, 0, al)
                # positions inside an expert follow the flat index in both
                for i, name in enumerate(['pos_to_expert', 'pos_to_token', 'pos_to_token_topk', 'token_topk_to_pos', 'expert_start', 'expert_end', 'num_tokens_per_expert']):
                    assert torch.equal(got[i].cpu(), want[i].to(got[i].dtype)), name
                if kind == 'expand_sf' and want[0].numel() > 0:
                    hidden = rng.choice([128, 256, 576, 1024, 2048, 4096]); npc = rng.choice([32, 128])
                    col, rnd = rng.choice([(False, False), (False, True), (True, True), (True, False)])
                    desc += f' hidden={hidden} npc={npc} col={col}'
                    x = torch.randn((T, hidden), generator=g).to(torch.bfloat16)
                    xq = torch_ref.cast(x, 'e4m3', (1, npc), round_sf=rnd)
                    we = torch_ref.expand_to_fused_with_sf(xq, npc, want[3], want[0], col)
                    ge = tk.moe.expand_to_fused_with_sf((xq[0].cuda(), xq[1].cuda()), npc, got[3], got[0], col)
                    assert_same(ge[0], we[0], 'rows'); assert_same(ge[1], we[1], 'sf')
            elif kind == 'requant':
                M = rng.choice([1, 4, 7, 33, 130]); K = rng.choice([1, 2, 3, 4, 5, 8, 11]) * rng.choice([128, 512, 1024])
                xb = rng.choice([(1, 128), (1, 32), (32, 32), (128, 128)]); N = rng.choice([16, 32, 64, 128])
                fin, fout = rng.choice([('e4m3', 'e2m1'), ('e4m3', 'e4m3'), ('e2m1', 'e4m3')])
                col, rnd, pk = rng.choice([(False, False, False), (False, True, False), (True, True, False), (True, True, True)])
                desc = f'requant M={M} K={K} in={fin}{xb} out={fout}/{N} col={col} rnd={rnd} pk={pk}'
                x = torch.randn((M, K)).to(torch.bfloat16)
                xq = torch_ref.cast(x, fin, xb, round_sf=True)
                kw = dict(use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=pk)
                want = torch_ref.cast(xq, fout, (1, N), x_block_size=xb, **kw)
                got = tk.quant.per_token_cast((xq[0].cuda(), xq[1].cuda()), fout, N, x_block_size=xb, **kw)
                assert_same(got[0], want[0], 'codes'); assert_same(got[1], want[1], 'sf')
        except AssertionError as e:
            failures.append(f'case {case}: {desc}: {str(e)[:300]}')
        except Exception as e:
            failures.append(f'case {case}: {desc}: {type(e).__name__}: {str(e)[:300]}')
    assert not failures, '\n'.join(failures)
