"""Shape grids and synthetic inputs for the parity tests and the benchmark."""
import os

import torch

from ..utils import align


def _full_test() -> bool:
    return os.getenv('TK_FULL_TEST') in ('1', 'true', 'True')


def generate_num_tokens(alignment: int = 1, is_benchmark: bool = False):
    """Token counts of the reference's grid (tile_kernels/testing/generator.py:10-17)."""
    sizes = [4001, 8001]
    if _full_test() and not is_benchmark:
        sizes = [0] + sizes
    return [align(n, alignment) for n in sizes]


def generate_hidden_sizes(alignment: int = 64):
    return [h for h in (576, 2048, 2560, 3072, 4096, 6144, 7168) if h % alignment == 0]


def generate_num_sms():
    """Compute-unit limits to test with (tile_kernels/testing/generator.py:26-32)."""
    from ..config import get_device_num_sms
    n = get_device_num_sms()
    base = [n - 20, n]
    return [1] + base if _full_test() else base


def generate_moe_params(is_benchmark: bool = False):
    """Routing configurations of the reference's MoE-shaped tests, as seen by one expert-parallel rank
    (tile_kernels/testing/generator.py:35-51): ``num_experts`` is the rank's local expert count."""
    full = _full_test()
    if full and not is_benchmark:
        yield {'num_send_tokens': 0, 'num_topk': 1, 'num_experts': 1, 'num_ep_ranks': 1}
    for num_tokens in (4001,):
        for num_topk in (2, 6, 8, 9) + ((1, 7) if full else ()):
            for num_experts in (72, 256) + ((288, 384) if full else ()):
                for num_ep_ranks in (8, 64) + ((1, 72, 256) if full else ()):
                    if num_experts % num_ep_ranks == 0:
                        yield {'num_send_tokens': num_tokens, 'num_topk': num_topk,
                               'num_experts': num_experts // num_ep_ranks, 'num_ep_ranks': num_ep_ranks}


def generate_topk_idx(params: dict, device='cuda') -> torch.Tensor:
    """Top-k expert ids of the tokens that reach this rank (tile_kernels/testing/generator.py:54-69):
    every token of every rank picks ``num_topk`` of all experts; ids outside this rank's first
    ``num_experts`` become -1 and tokens with no local expert are dropped.  int64 ``[tokens, num_topk]``."""
    n, e, k, ranks = params['num_send_tokens'], params['num_experts'], params['num_topk'], params['num_ep_ranks']
    if n == 0:
        return torch.empty((0, k), dtype=torch.int64, device=device)
    scores = torch.rand((n * ranks, e * ranks), dtype=torch.bfloat16, device=device)
    topk_idx = torch.topk(scores, k=k, dim=-1, sorted=False).indices
    away = topk_idx >= e
    topk_idx = topk_idx.masked_fill(away, -1)
    return topk_idx[~away.all(dim=1)].contiguous()


# E5M6 keeps the top 12 bits of an fp16: its subnormals are k * 2^-20 for k = 1 .. 63, its smallest normal is 2^-14
E5M6_SPECIAL_VALUES = (2.0 ** -20, 2.0 ** -14 * 63 / 64, 2.0 ** -14)


def generate_e5m6_inputs(num_tokens: int, hidden: int, dtype: torch.dtype, device='cuda'):
    """``(x, is_special)`` pairs for the E5M6 tests (tile_kernels/testing/generator.py:70-89): one random
    tensor, then one constant tensor per special value whose last column holds 65024, so that the scale is 1
    and the constant is cast as it stands."""
    yield torch.randn((num_tokens, hidden), dtype=dtype, device=device), False
    for value in E5M6_SPECIAL_VALUES:
        x = torch.full((num_tokens, hidden), value, dtype=dtype, device=device)
        x[:, -1] = 65024.0
        yield x, True


def generate_rand_float(shape, device='cuda') -> torch.Tensor:
    """Normal values scaled by a power of two drawn uniformly from 2^-110 .. 2^126, non-finite values redrawn
    and magnitudes capped at an eighth of the fp32 range (tile_kernels/testing/generator.py:92-105)."""
    import random
    x = torch.randn(shape, dtype=torch.float32, device=device) * float(2 ** random.randint(-110, 126))
    bad = ~torch.isfinite(x)
    if bad.any():
        x[bad] = torch.randn((int(bad.sum()),), dtype=torch.float32, device=device)
    cap = torch.finfo(torch.float32).max / 8
    return x.clamp(-cap, cap)


def generate_moe_layout(num_tokens: int, num_experts: int, num_topk: int, alignment: int, generator: torch.Generator,
                        drop_fraction: float = 0.0):
    """Expert-major expanded layout of a top-k routed batch, built on the CPU.

    Every (token, k) pair whose expert is >= 0 gets one row; rows are grouped by expert and every
    expert's segment is padded to a multiple of ``alignment`` rows.  Same contract as the
    reference's fused mapping (tile_kernels/moe/get_fused_mapping_kernel.py:166-250):

      pos_to_expert[R]      expert of the row, -1 for padding
      pos_to_token_topk[R]  token * num_topk + k of the row, -1 for padding
      topk_weights[T, k]    softmax probabilities of the chosen experts (fp32)
    """
    logits = torch.randn((num_tokens, num_experts), generator=generator)
    prob = torch.softmax(logits, dim=-1)
    topk_w, topk_idx = torch.topk(prob, num_topk, dim=-1)
    if drop_fraction > 0:
        drop = torch.rand(topk_idx.shape, generator=generator) < drop_fraction
        topk_idx = topk_idx.masked_fill(drop, -1)
    flat = topk_idx.reshape(-1)
    order = torch.argsort(torch.where(flat < 0, num_experts, flat), stable=True)
    order = order[flat[order] >= 0]
    experts = flat[order]
    counts = torch.bincount(experts, minlength=num_experts)
    padded = (counts + alignment - 1) // alignment * alignment
    seg_start = torch.cumsum(padded, 0) - padded
    rank_in_expert = torch.arange(order.numel()) - (torch.cumsum(counts, 0) - counts)[experts]
    pos = seg_start[experts] + rank_in_expert
    R = int(padded.sum())
    pos_to_expert = torch.full((R,), -1, dtype=torch.int32)
    pos_to_token_topk = torch.full((R,), -1, dtype=torch.int32)
    pos_to_expert[pos] = experts.to(torch.int32)
    pos_to_token_topk[pos] = order.to(torch.int32)
    return pos_to_expert, pos_to_token_topk, topk_w.to(torch.float32).contiguous()


def make_baseline_input(cfg: int, scale_rows: float = 1.0):
    """Seeded CPU input of benchmark configuration ``cfg`` (1..5); ``scale_rows`` < 1 shrinks the
    row count for quick checks.  Returns a dict with ``x`` (bf16) and, for cfg 4, the MoE layout."""
    g = torch.Generator().manual_seed(1000 + cfg)
    rows = lambda n: max(1, int(n * scale_rows))
    if cfg == 1:      # activations with 0.1 % outliers x100
        x = torch.randn((rows(4096), 7168), generator=g)
        x[torch.rand(x.shape, generator=g) < 0.001] *= 100
        return {'x': x.to(torch.bfloat16)}
    if cfg == 2:      # weights N(0, 0.02) with 16 rows x50
        m = rows(7168)
        w = 0.02 * torch.randn((m, 2048), generator=g)
        w[torch.randperm(m, generator=g)[: min(16, m)]] *= 50
        return {'x': w.to(torch.bfloat16)}
    if cfg == 3:
        return {'x': torch.randn((rows(8192), 4096), generator=g).to(torch.bfloat16)}
    if cfg == 4:
        pe, ptt, w = generate_moe_layout(rows(4096), 256, 8, 128, g)
        x = torch.randn((pe.numel(), 4096), generator=g)
        x[pe < 0] = 0
        return {'x': x.to(torch.bfloat16), 'pos_to_expert': pe, 'pos_to_token_topk': ptt, 'topk_weights': w}
    if cfg == 5:      # Student-t, 4 degrees of freedom
        m = rows(16384)
        z = torch.randn((m, 7168), generator=g)
        chi = torch.zeros_like(z)
        for _ in range(4):
            chi += torch.randn((m, 7168), generator=g) ** 2
        return {'x': (z / torch.sqrt(chi / 4)).to(torch.bfloat16)}
    raise ValueError(cfg)
