"""Every compiled variant of the kernels at least once: the library picks a kernel by input type, group size, format,
scale layout, mode, row length and by whether the shape fits the tiles exactly (those variants carry no bounds checks), so
the cases here are grids over exactly these choices, on small shapes, each against the CPU oracle to the bars of the
other tests.  A grid collects its failing cases and fails once at the end."""
import itertools

import pytest
import torch

from oracle import torch_ref
from tests._util import assert_same
from tests.test_gpu_swiglu import check_fused

pytestmark = pytest.mark.gpu

# (column-major, power-of-two scales, packed UE8M0)
LAYOUTS = [(False, False, False), (False, True, False), (True, False, False), (True, True, False), (True, True, True)]


def _tk():
    import tilekernels_amd
    return tilekernels_amd


def _kw(layout):
    col, rnd, pk = layout
    return dict(use_tma_aligned_col_major_sf=col, round_sf=rnd, use_packed_ue8m0=pk)


class Failures:
    def __init__(self):
        self.items, self.ran = [], 0

    def run(self, desc, fn):
        self.ran += 1
        try:
            fn()
        except AssertionError as e:
            self.items.append(f'{desc}: {str(e)[:300]}')
        except Exception as e:      # noqa: BLE001
            self.items.append(f'{desc}: {type(e).__name__}: {str(e)[:300]}')

    def check(self, at_least):
        assert self.ran >= at_least, f'only {self.ran} cases ran'
        assert not self.items, f'{len(self.items)} of {self.ran} cases failed:\n' + '\n'.join(self.items[:40])


def _randn(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


# Row lengths of the per-token cast: one strip (stacked tiles), two and four strips (row-wise tiles for plain input, whose
# waves take two pieces; wide tiles in the scale-only mode), three strips (wide tiles), four (row-wise for quantised input
# too), a ragged two-strip and a ragged three-strip row, and a row short enough for the flattened kernel.
PT_K = [512, 1024, 1536, 2048, 896, 1408, 320]


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32], ids=['bf16', 'fp32'])
@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
def test_per_token_cast_variants(dtype, fmt):
    """Group sizes x layouts x row lengths x (rows that fit the tiles, rows that do not) x the three modes."""
    tk, f = _tk(), Failures()
    for N, layout, K, M in itertools.product([16, 32, 64, 128], LAYOUTS, PT_K, [16, 13]):
        if K % N:
            continue
        kw = _kw(layout)
        x = _randn((M, K), dtype, M * 7 + K + N, 3.0)
        xd = x.cuda()
        want = torch_ref.cast(x, fmt, (1, N), **kw)

        def full():
            got = tk.quant.per_token_cast(xd, fmt, N, **kw)
            assert_same(got[0], want[0], 'codes')
            assert_same(got[1], want[1], 'sf')

        def only():
            assert_same(tk.quant.per_token_cast_with_sf_only(xd, fmt, N, **kw), want[1], 'sf alone')

        def given():
            # (the multiplier is 1 / sf here, 448 / amax in the full cast: the codes may differ from the full cast's)
            expect = torch_ref.cast(x, fmt, (1, N), sf=want[1], **kw)
            assert_same(tk.quant.per_token_cast_with_precomputed_sf(xd, fmt, N, want[1].cuda(), **kw), expect, 'codes for given sf')

        def strided():
            # rows 16 bytes further apart than they are long; given scales in rows with three unused words behind them
            wide = torch.zeros((M, K + 16 // x.element_size()), dtype=dtype, device='cuda')
            view = wide[:, :K]
            view.copy_(xd)
            got = tk.quant.per_token_cast(view, fmt, N, **kw)
            assert_same(got[0], want[0], 'codes of strided rows')
            assert_same(got[1], want[1], 'sf of strided rows')
            assert_same(tk.quant.per_token_cast_with_sf_only(view, fmt, N, **kw), want[1], 'sf alone of strided rows')
            if not layout[0]:
                sf_wide = torch.zeros((M, K // N + 3), dtype=torch.float32, device='cuda')
                sf_view = sf_wide[:, :K // N]
                sf_view.copy_(want[1].cuda())
                expect = torch_ref.cast(x, fmt, (1, N), sf=want[1], **kw)
                assert_same(tk.quant.per_token_cast_with_precomputed_sf(view, fmt, N, sf_view, **kw), expect, 'codes for given strided sf')

        desc = f'M={M} K={K} N={N} {layout}'
        f.run(desc, full)
        f.run(desc + ' sf only', only)
        if not layout[0]:
            f.run(desc + ' given sf', given)
        if layout in (LAYOUTS[0], LAYOUTS[4]):
            f.run(desc + ' strided', strided)
    f.check(500)


@pytest.mark.parametrize('in_fmt', ['e4m3', 'e2m1'])
@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
def test_per_token_cast_of_quantised_input_variants(in_fmt, fmt):
    """Input blocks x group sizes x layouts x row lengths x rows that fit 16-row tiles or not."""
    tk, f = _tk(), Failures()
    for xb, N, layout, K, M in itertools.product([(128, 128), (32, 32), (1, 128), (1, 32)], [16, 32, 64, 128], LAYOUTS,
                                                 [512, 1536, 2048, 4096, 896, 1408], [16, 32, 13]):
        kw = _kw(layout)
        src = _randn((M, K), torch.bfloat16, M + K + N + xb[0], 2.0)
        xq = torch_ref.cast(src, in_fmt, xb)
        want = torch_ref.cast(xq, fmt, (1, N), x_block_size=xb, **kw)

        def full():
            got = tk.quant.per_token_cast(tuple(t.cuda() for t in xq), fmt, N, x_block_size=xb, **kw)
            assert_same(got[0], want[0], 'codes')
            assert_same(got[1], want[1], 'sf')

        f.run(f'M={M} K={K} N={N} in {xb} {layout}', full)
    f.check(1000)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32], ids=['bf16', 'fp32'])
@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
@pytest.mark.parametrize('hidden', [1024, 2048, 2560, 4224, 6144, 8192, 8320, 16384, 16448])
def test_per_token_cast_with_one_scale_per_row(dtype, fmt, hidden):
    """Rows held in one to four register pieces per thread (workgroups of one to four waves), rows of exactly that many
    pieces and rows that end inside one, and rows too long for registers (two passes)."""
    tk, f = _tk(), Failures()
    for h, rnd in itertools.product([hidden, hidden - 64], [False, True]):
        x = _randn((5, h), dtype, h, 2.0)
        want = torch_ref.cast(x, fmt, (1, h), round_sf=rnd)

        def full():
            got = tk.quant.per_token_cast(x.cuda(), fmt, h, round_sf=rnd)
            assert_same(got[0], want[0], 'codes')
            assert_same(got[1], want[1], 'sf')

        f.run(f'hidden={h} round_sf={rnd}', full)
    f.check(4)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32], ids=['bf16', 'fp32'])
@pytest.mark.parametrize('block', [(128, 128), (32, 32), (32, 128), (128, 32)], ids=lambda b: '%dx%d' % b)
def test_per_block_cast_variants(dtype, block):
    """128 x 128 tiles and the 128 x 512 tiles of mid-sized matrices (512 to 1280 blocks of 128 x 128), each on shapes
    that are whole tiles and on shapes that are not."""
    tk, f = _tk(), Failures()
    shapes = [(256, 1024), (200, 960), (4096, 2048), (4000, 2048)]
    for fmt, layout, (M, K) in itertools.product(['e4m3', 'e2m1'], LAYOUTS, shapes):
        if M * K > 1 << 20 and layout in LAYOUTS[1:4]:
            continue        # the large shapes with the plain and the packed layout only
        kw = _kw(layout)
        x = _randn((M, K), dtype, M + K, 2.0)
        xd = x.cuda()
        want = torch_ref.cast(x, fmt, block, **kw)

        def full():
            got = tk.quant.per_block_cast(xd, fmt, block, **kw)
            assert_same(got[0], want[0], 'codes')
            assert_same(got[1], want[1], 'sf')

        def only():
            assert_same(tk.quant.per_block_cast_with_sf_only(xd, fmt, block, **kw), want[1], 'sf alone')

        def given():
            expect = torch_ref.cast(x, fmt, block, sf=want[1], **kw)
            assert_same(tk.quant.per_block_cast_with_precomputed_sf(xd, fmt, block, want[1].cuda(), **kw), expect, 'codes for given sf')

        desc = f'{fmt} M={M} K={K} {layout}'
        f.run(desc, full)
        f.run(desc + ' sf only', only)
        if not layout[0]:
            f.run(desc + ' given sf', given)
    f.check(60)


def _swiglu_case(tk, dtype, R, H, N, layout, with_mask, with_weights, clamp_mode, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn((R, 2 * H), generator=g) * 2).to(dtype)
    pe = ptt = w = None
    if with_mask:
        pe = torch.randint(0, 4, (R,), generator=g).to(torch.int32)
        pe[torch.rand(R, generator=g) < 0.25] = -1
        x[pe < 0] = 0
    if with_weights:
        ptt = torch.randperm(R, generator=g).to(torch.int32)
        ptt[torch.rand(R, generator=g) < 0.1] = -1
        if pe is not None:
            ptt[pe < 0] = -1
        w = torch.rand(((R + 3) // 4, 4), generator=g) + 0.25
    clamp = None if clamp_mode == 0 else 0.75
    count = torch.tensor([5, 0, 2], dtype=torch.int64) if clamp_mode == 2 else None
    count_ref = None if count is None else count.clone()
    kw = dict(swiglu_clamp_value=clamp, **_kw(layout))
    want = torch_ref.swiglu_forward_and_per_token_cast(x, 'e4m3', N, ptt, w, pe, clamped_count=count_ref, **kw)
    dev = lambda t: None if t is None else t.cuda()
    cg = dev(count)
    got = tk.quant.swiglu_forward_and_per_token_cast(x.cuda(), 'e4m3', N, dev(ptt), dev(w), dev(pe), clamped_count=cg, **kw)
    check_fused(got, want, H // N, layout[2])
    if count is not None:
        assert cg.cpu().tolist() == count_ref.tolist(), f'counts {cg.cpu().tolist()} != {count_ref.tolist()}'


# bf16 waves take four 512-column pieces, fp32 waves two: row-wise tiles for H a multiple of that (one column of tiles, two
# columns), stacked tiles otherwise (H a multiple of 512, and not), short rows laid end to end over the lanes
SWIGLU_H = {torch.bfloat16: [2048, 4096, 1536, 640, 256], torch.float32: [1024, 2048, 1536, 640, 256]}


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32], ids=['bf16', 'fp32'])
@pytest.mark.parametrize('clamp_mode', [0, 1, 2], ids=['noclamp', 'clamp', 'clampcount'])
def test_swiglu_forward_variants(dtype, clamp_mode):
    """Tile shapes x layouts x (rows that fit the tiles, rows that do not) x mask x routing weights."""
    tk, f = _tk(), Failures()
    for H, layout, R, with_mask, with_weights in itertools.product(SWIGLU_H[dtype], [LAYOUTS[0], LAYOUTS[2], LAYOUTS[4]], [16, 13],
                                                                   [False, True], [False, True]):
        desc = f'R={R} H={H} {layout} mask={with_mask} weights={with_weights}'
        f.run(desc, lambda: _swiglu_case(tk, dtype, R, H, 128, layout, with_mask, with_weights, clamp_mode, R + H))
    f.check(100)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32], ids=['bf16', 'fp32'])
@pytest.mark.parametrize('clamp_mode', [0, 1, 2], ids=['noclamp', 'clamp', 'clampcount'])
def test_swiglu_forward_with_one_scale_per_row_variants(dtype, clamp_mode):
    """One to four register pieces per thread, and rows too long for registers."""
    tk, f = _tk(), Failures()
    for H, rnd, with_mask in itertools.product([1024, 2560, 4224, 6144, 8192, 8320], [False, True], [False, True]):
        desc = f'H={H} round_sf={rnd} mask={with_mask}'
        f.run(desc, lambda: _swiglu_case(tk, dtype, 6, H, H, (False, rnd, False), with_mask, True, clamp_mode, H))
    f.check(20)


# One scale per row: the row is held in 1, 2, 3, 4, 6 or 8 register pieces per thread by one to four waves; rows of exactly
# 256 threads x pieces x 8 elements run without bounds checks; rows beyond 16384 elements take two passes.
ROW_K = [2048, 2560, 3584, 4096, 4224, 5120, 6144, 7168, 8192, 8320, 10240, 12288, 14336, 16384, 16448, 20480]


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32], ids=['bf16', 'fp32'])
@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1', 'e5m6'])
def test_per_token_cast_with_one_scale_per_row_every_piece_count(dtype, fmt):
    tk, f = _tk(), Failures()
    for h, rnd in itertools.product(ROW_K, [False, True]):
        x = _randn((3, h), dtype, h, 2.0)
        want = torch_ref.cast_to_e5m6(x, h, round_sf=rnd) if fmt == 'e5m6' else torch_ref.cast(x, fmt, (1, h), round_sf=rnd)

        def full():
            got = tk.quant.per_token_cast(x.cuda(), fmt, h, round_sf=rnd)
            assert_same(got[0], want[0], 'codes')
            assert_same(got[1], want[1], 'sf')

        f.run(f'hidden={h} round_sf={rnd}', full)
    f.check(2 * len(ROW_K))


def test_per_token_cast_of_quantised_rows_that_are_not_16_byte_aligned():
    """E4M3 input to E2M1 with row-major scales takes 16 codes per lane where the rows allow 16-byte loads; rows 8 bytes
    off that (a view into a wider tensor) take the general kernel, here with row-wise tiles (K a multiple of 2048)."""
    tk, f = _tk(), Failures()
    for N, M, K in itertools.product([32, 64, 128], [16, 13], [2048, 4096]):
        src = _randn((M, K), torch.bfloat16, N + M + K, 2.0)
        xq = torch_ref.cast(src, 'e4m3', (1, 128))
        want = torch_ref.cast(xq, 'e2m1', (1, N), x_block_size=(1, 128))
        wide = torch.zeros((M, K + 8), dtype=torch.uint8, device='cuda').view(torch.float8_e4m3fn)
        view = wide[:, :K]
        view.copy_(xq[0].cuda())

        def full():
            got = tk.quant.per_token_cast((view, xq[1].cuda()), 'e2m1', N, x_block_size=(1, 128))
            assert_same(got[0], want[0], 'codes')
            assert_same(got[1], want[1], 'sf')

        f.run(f'N={N} M={M} K={K}', full)
    f.check(12)


@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
@pytest.mark.parametrize('out_fmt', ['bf16', 'fp32'])
def test_cast_back_variants(fmt, out_fmt):
    """Scale blocks x layouts x row lengths (stacked, wide, ragged, short) x rows that fit the tiles or not."""
    tk, f = _tk(), Failures()
    blocks = [(1, 128), (1, 32), (32, 32), (128, 128), (128, 1), (128, 2), (128, 4)]
    for blk, layout, K, M in itertools.product(blocks, [LAYOUTS[0], LAYOUTS[2], LAYOUTS[4]], [512, 1536, 1408, 896, 320], [16, 13]):
        if blk[1] < 8 and layout[0]:
            continue
        src = _randn((M, K), torch.bfloat16, M + K + blk[0] + blk[1], 2.0)
        xq = torch_ref.cast(src, fmt, blk, **_kw(layout))
        want = torch_ref.cast_back(xq, out_fmt, blk)
        f.run(f'{blk} {layout} M={M} K={K}',
              lambda: assert_same(tk.quant.cast_back(tuple(t.cuda() for t in xq), out_fmt, blk), want, 'values'))
    f.check(100)


@pytest.mark.parametrize('out_fmt', ['bf16', 'fp32'])
def test_cast_back_e5m6_variants(out_fmt):
    """12-bit codes with every block shape the dequantisation knows, on stacked, wide, ragged and short rows."""
    tk, f = _tk(), Failures()
    for blk, K, M in itertools.product([(1, 128), (128, 128), (1, 0), (128, 1), (128, 4)], [512, 1536, 1408, 896, 320], [16, 13]):
        blk = (blk[0], blk[1] or K)
        g = torch.Generator().manual_seed(K + M + blk[0])
        codes = torch.randint(0, 4096, (M, K), generator=g, dtype=torch.int32)
        codes[(codes & 0x7C0) == 0x7C0] &= 0xFBF         # no infinities or NaNs: values must compare as numbers
        packed = torch_ref.pack_e5m6(codes)
        sf = torch.exp2(torch.randint(-6, 6, (-(-M // blk[0]), -(-K // blk[1])), generator=g).float())
        want = torch_ref.cast_back_from_e5m6((packed, sf), out_fmt, blk)
        f.run(f'{blk} M={M} K={K}',
              lambda: assert_same(tk.quant.cast_back((packed.cuda(), sf.cuda()), out_fmt, blk, x_special_fmt='e5m6'), want, 'values'))
    f.check(50)


def test_per_channel_cast_c_abi_variants():
    """tk_per_channel_cast over input type x tokens per scale x transposed output x row gather, including the combinations
    the Python wrappers never ask for, and FP8 input whose buffers are only 8-byte aligned."""
    from tilekernels_amd import _ffi
    lib, f = _ffi.load(), Failures()
    T, K = 200, 384
    g = torch.Generator().manual_seed(3)
    for kind, npt, transpose, gather, shift in itertools.product(['bf16', 'fp32', 'e4m3'], [32, 128], [False, True], [False, True], [0, 8]):
        if (kind == 'fp32' and transpose) or (shift and (kind != 'e4m3' or transpose)):
            continue
        M = 16 * 21 if gather else 128
        x = torch.randn((T, K), generator=g)
        x = x if kind == 'fp32' else x.to(torch.bfloat16)
        pos = torch.randint(-1, T, (M,), generator=g, dtype=torch.int32) if gather else None
        xin = torch_ref.cast(x, 'e4m3', (1, 128)) if kind == 'e4m3' else x
        src = xin if gather else ((xin[0][:M], xin[1][:M]) if kind == 'e4m3' else xin[:M])
        want_codes, want_sf = torch_ref.per_channel_cast_fused(src, npt, 128 if kind == 'e4m3' else None, False, pos)
        if transpose:
            want_codes = want_codes.T.contiguous()

        def call():
            data = xin[0].view(torch.uint8) if kind == 'e4m3' else xin
            xbuf = torch.zeros(data.numel() * data.element_size() + 16, dtype=torch.uint8, device='cuda')
            xbuf[shift:shift + data.numel() * data.element_size()].copy_(data.contiguous().view(torch.uint8).flatten().cuda())
            sfd = xin[1].cuda() if kind == 'e4m3' else None
            posd = None if pos is None else pos.cuda()
            obuf = torch.zeros(want_codes.numel() + 16, dtype=torch.uint8, device='cuda')
            out_sf = torch.empty(tuple(want_sf.shape), dtype=torch.float32, device='cuda')
            rc = lib.tk_per_channel_cast(xbuf.data_ptr() + shift, 1 if kind == 'fp32' else 0, _ffi.ptr(sfd), T if gather else M, K, _ffi.ptr(posd), M,
                                         obuf.data_ptr() + shift, out_sf.data_ptr(), npt, 0, int(transpose), 0, 0, 0.0,
                                         _ffi.current_stream(obuf.device))
            assert rc == 0, rc
            torch.cuda.synchronize()
            got = obuf[shift:shift + want_codes.numel()].view(torch.float8_e4m3fn).reshape(want_codes.shape)
            assert_same(got, want_codes, 'codes')
            assert_same(out_sf, want_sf, 'scales')

        f.run(f'{kind} npt={npt} transpose={transpose} gather={gather} shift={shift}', call)
    f.check(24)


@pytest.mark.parametrize('in_block,out_block,hidden', [((1, 8), (32, 8), 512), ((1, 8), (128, 128), 1024), ((8, 8), (8, 8), 288)])
def test_per_block_cast_lossless_with_8_codes_per_lane(in_block, out_block, hidden):
    """Blocks that are no multiple of 16 columns wide: the re-blocking moves 8 codes per lane instead of 16."""
    from tests.test_oracle_lossless import reference_style_input
    tk = _tk()
    x = reference_style_input(150, hidden, seed=hidden)
    x_fp4 = torch_ref.cast(x, 'e2m1', in_block, round_sf=True)
    want = torch_ref.per_block_cast_lossless(x_fp4, 'e4m3', in_block, out_block, round_sf=True)
    got = tk.quant.per_block_cast_lossless((x_fp4[0].cuda(), x_fp4[1].cuda()), 'e4m3', in_block, out_block, round_sf=True)
    assert_same(got[0], want[0], 'codes')
    assert_same(got[1], want[1], 'scales')


def test_stream_floor_flat_moves_every_byte():
    """The traffic-only kernel for any ratio of bytes read to bytes written: what it writes is the XOR fold of what it
    read, for every width of loads and stores and every number of pieces per wave."""
    import numpy as np
    from tilekernels_amd import _ffi
    lib, f = _ffi.load(), Failures()
    stream = torch.cuda.current_stream().cuda_stream
    pieces = 37        # not a multiple of any wave's piece count: the last wave's surplus pieces must write nothing
    for I, O, P in itertools.product([16, 8, 4], [16, 8, 4, 0], [1, 2, 4, 8]):
        n_in = pieces * 64 * I
        data = torch.randint(0, 256, (n_in,), dtype=torch.uint8, generator=torch.Generator().manual_seed(I + O + P))
        words = np.zeros((pieces * 64, 4), dtype=np.uint32)
        words[:, :I // 4] = data.numpy().view(np.uint32).reshape(pieces * 64, I // 4)
        if O == 16:
            expect = words
        elif O == 8:
            expect = np.stack([words[:, 0] ^ words[:, 2], words[:, 1] ^ words[:, 3]], axis=1)
        else:
            expect = (words[:, 0] ^ words[:, 1] ^ words[:, 2] ^ words[:, 3])[:, None]

        def call():
            out = torch.full((pieces * 64 * max(O, 4) + 64,), 0xA5, dtype=torch.uint8, device='cuda')
            rc = lib.tk_stream_floor_flat(data.cuda().data_ptr(), n_in, I, out.data_ptr(), O, P, stream)
            assert rc == 0, rc
            torch.cuda.synchronize()
            got = out.cpu().numpy()
            n_out = pieces * 64 * O
            if O:
                assert np.array_equal(got[:n_out].view(np.uint32).reshape(expect.shape), expect), 'written words'
            assert (got[n_out:] == 0xA5).all(), 'bytes beyond the output were written'

        f.run(f'in {I} out {O} pieces {P}', call)
    assert lib.tk_stream_floor_flat(0, 64 * 16, 16, 0, 0, 1, stream) != 0       # null input
    f.check(48)


@pytest.mark.parametrize('spec', ['0:0', '0:1', '0:2', '0:8', '1:0', '2:0', '3:0', '4:0', '5:500', '6:1', '6:2', '7:1', '7:2', '8:25'])
def test_swiglu_cast_variants_match_the_product(spec):
    """The alternative structures of the headline kernel kept for measurements produce the product's codes and scales."""
    from tilekernels_amd import _ffi
    tk, lib = _tk(), _ffi.load()
    variant, param = (int(v) for v in spec.split(':'))
    R, H = 1024, 2048
    x = _randn((R, 2 * H), torch.bfloat16, 5, 2.0).cuda()
    codes, sf = tk.quant.swiglu_forward_and_per_token_cast(x, 'e4m3', 128)
    out = torch.full((R, H), 0xAB, dtype=torch.uint8, device='cuda')
    out_sf = torch.full((R, H // 128), -1.0, dtype=torch.float32, device='cuda')
    rc = lib.tk_swiglu_cast_variant(x.data_ptr(), R, H, out.data_ptr(), out_sf.data_ptr(), variant, param, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.equal(out, codes.view(torch.uint8)), 'codes'
    assert torch.equal(out_sf, sf), 'scales'


def test_smallest_shapes():
    """One to three rows of one or two groups: every lane but a few is beyond the data."""
    tk, f = _tk(), Failures()
    for N, layout, groups, M, fmt, dtype in itertools.product([16, 32, 64, 128], [LAYOUTS[0], LAYOUTS[2], LAYOUTS[4]], [1, 2], [1, 2, 3],
                                                              ['e4m3', 'e2m1'], [torch.bfloat16, torch.float32]):
        K = N * groups
        kw = _kw(layout)
        x = _randn((M, K), dtype, N + K + M, 2.0)
        want = torch_ref.cast(x, fmt, (1, N), **kw)

        def token():
            got = tk.quant.per_token_cast(x.cuda(), fmt, N, **kw)
            assert_same(got[0], want[0], 'codes')
            assert_same(got[1], want[1], 'sf')
            if K % 64 == 0:     # (dequantisation takes rows of a multiple of 64 elements, like the reference's)
                assert_same(tk.quant.cast_back(got, 'fp32', (1, N)), torch_ref.cast_back(want, 'fp32', (1, N)), 'values')

        f.run(f'per-token M={M} K={K} N={N} {fmt} {layout}', token)
    for blk, (M, K), fmt in itertools.product([(128, 128), (32, 32)], [(1, 64), (2, 128), (3, 192)], ['e4m3', 'e2m1']):
        x = _randn((M, K), torch.bfloat16, M + K, 2.0)
        want = torch_ref.cast(x, fmt, blk)

        def block():
            got = tk.quant.per_block_cast(x.cuda(), fmt, blk)
            assert_same(got[0], want[0], 'codes')
            assert_same(got[1], want[1], 'sf')

        f.run(f'per-block M={M} K={K} {blk} {fmt}', block)
    for R, H, layout in itertools.product([1, 2, 3], [128, 256], [LAYOUTS[0], LAYOUTS[2], LAYOUTS[4]]):
        f.run(f'swiglu R={R} H={H} {layout}', lambda: _swiglu_case(tk, torch.bfloat16, R, H, 128, layout, False, False, 0, R + H))
    f.check(300)


@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
def test_per_block_cast_into_a_buffer_that_is_only_8_byte_aligned(fmt):
    """The wide tiles of mid-sized matrices store 16 codes per lane; the entry point only asks for 8-byte alignment of the codes."""
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    M, K = 4096, 2048
    x = _randn((M, K), torch.bfloat16, 17, 2.0)
    want = torch_ref.cast(x, fmt, (128, 128))
    nbytes = want[0].numel()
    buf = torch.full((nbytes + 32,), 0x5A, dtype=torch.uint8, device='cuda')
    sf = torch.empty((M // 128, K // 128), dtype=torch.float32, device='cuda')
    xd = x.cuda()
    rc = lib.tk_per_block_cast(xd.data_ptr(), 0, M, K, buf.data_ptr() + 8, sf.data_ptr(), K // 128, 0 if fmt == 'e4m3' else 1, 128, 128, 0, 0, 0,
                               torch.cuda.current_stream().cuda_stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.equal(buf[8:8 + nbytes].cpu(), want[0].view(torch.uint8).flatten()), 'codes'
    assert bool((buf[:8] == 0x5A).all()) and bool((buf[8 + nbytes:] == 0x5A).all()), 'bytes around the codes were written'
    assert_same(sf, want[1], 'sf')


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
def test_masked_swiglu_cast_into_a_buffer_that_is_only_8_byte_aligned(dtype):
    """Padding rows of the row-wise kernel are written as 16-byte stores where the buffer allows it and as 8-byte stores
    otherwise; both must give the zeros (and nothing around the buffer) that the wrapper's 256-byte-aligned tensors get."""
    import tilekernels_amd as tk
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    R, H = 1031, 2048
    g = torch.Generator().manual_seed(23)
    x = (torch.randn((R, 2 * H), generator=g) * 2.0).to(dtype).cuda()
    pos_to_expert = torch.randint(0, 4, (R,), generator=g).to(torch.int32)
    pos_to_expert[5:77] = -1
    pos_to_expert[torch.rand((R,), generator=g) < 0.3] = -1
    pos_to_expert[-1] = -1
    pos_to_expert = pos_to_expert.cuda()
    want, want_sf = tk.quant.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, pos_to_expert=pos_to_expert)
    dead = (pos_to_expert < 0).cpu()
    assert bool((want.view(torch.uint8)[dead.cuda()] == 0).all()) and bool((want_sf[dead.cuda()] == 0).all())
    assert bool((want_sf[(~dead).cuda()] > 0).all())
    for shift in (8, 16):
        buf = torch.full((R * H + 64,), 0x5A, dtype=torch.uint8, device='cuda')
        sf = torch.full((R, H // 128), -1.0, dtype=torch.float32, device='cuda')
        rc = lib.tk_swiglu_per_token_cast(x.data_ptr(), _ffi.dtype_code(x), R, H, buf.data_ptr() + shift, sf.data_ptr(), H // 128, 128,
                                          _ffi.TK_SF_ROW_F32, 0, -1.0, None, None, 0, pos_to_expert.data_ptr(), 0, 0.0, None, 0,
                                          torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
        assert torch.equal(buf[shift:shift + R * H].view(R, H), want.view(torch.uint8)), f'codes at +{shift}'
        assert bool((buf[:shift] == 0x5A).all()) and bool((buf[shift + R * H:] == 0x5A).all()), f'bytes around the codes were written at +{shift}'
        assert torch.equal(sf, want_sf), f'scales at +{shift}'


@pytest.mark.parametrize('dtype,R,H', [(torch.bfloat16, 40003, 2048), (torch.bfloat16, 9001, 8192), (torch.float32, 17001, 2048)])
def test_swiglu_cast_of_a_launch_that_refills_the_gpu_many_times(dtype, R, H):
    """Launches of more than 3.5 times the GPU's wave slots run one-wave workgroups; rows are independent, so the result
    must equal that of the same rows cast in pieces small enough for the other launch shapes (which the oracle tests cover)."""
    import tilekernels_amd as tk
    g = torch.Generator().manual_seed(R)
    x = (torch.randn((R, 2 * H), generator=g) * 2.5).to(dtype).cuda()
    ptt = torch.randint(-1, R, (R,), generator=g).to(torch.int32).cuda()
    w = torch.rand((R // 8 + 1, 8), generator=g).cuda()
    for kw in ({}, dict(swiglu_clamp_value=2.0), dict(round_sf=True)):
        for weighted in (False, True):
            args = (ptt, w) if weighted else ()
            out, sf = tk.quant.swiglu_forward_and_per_token_cast(x, 'e4m3', 128, *args, **kw)
            step = 2048
            for r0 in range(0, R, step):
                r1 = min(R, r0 + step)
                part_args = (ptt[r0:r1].contiguous(), w) if weighted else ()
                o, s = tk.quant.swiglu_forward_and_per_token_cast(x[r0:r1], 'e4m3', 128, *part_args, **kw)
                assert torch.equal(out[r0:r1].view(torch.uint8), o.view(torch.uint8)), f'codes of rows {r0}..{r1} {kw} weighted={weighted}'
                assert torch.equal(sf[r0:r1], s), f'scales of rows {r0}..{r1} {kw} weighted={weighted}'


@pytest.mark.parametrize('fmt', ['e4m3', 'e2m1'])
@pytest.mark.parametrize('group', [16, 32, 64, 128])
def test_per_token_cast_of_fp32_rows_beyond_one_grid_plane(fmt, group):
    """fp32 input runs one-wave workgroups on the row-wise tiles, so only a grid that overhangs along z (more than 32768
    row tiles, not a multiple of that) has workgroups beyond the last row.  Rows are independent: the result must equal
    that of the same rows cast in launches of one grid plane (which the oracle tests cover), with computed and given scales."""
    import tilekernels_amd as tk
    M, K = 32768 + 3, 2048
    g = torch.Generator().manual_seed(group)
    x = (torch.randn((M, K), generator=g) * 3.0).cuda()
    out, sf = tk.quant.per_token_cast(x, fmt, group)
    given = tk.quant.per_token_cast_with_precomputed_sf(x, fmt, group, sf)
    given = given[0] if isinstance(given, tuple) else given
    step = 8192
    for r0 in range(0, M, step):
        r1 = min(M, r0 + step)
        o, s = tk.quant.per_token_cast(x[r0:r1], fmt, group)
        assert torch.equal(out[r0:r1].view(torch.uint8), o.view(torch.uint8)), f'codes of rows {r0}..{r1}'
        assert torch.equal(sf[r0:r1], s), f'scales of rows {r0}..{r1}'
        og = tk.quant.per_token_cast_with_precomputed_sf(x[r0:r1], fmt, group, s)
        og = og[0] if isinstance(og, tuple) else og
        assert torch.equal(given[r0:r1].view(torch.uint8), og.view(torch.uint8)), f'codes for given scales of rows {r0}..{r1}'
