"""GPU parity of the lossless FP4 -> FP8 re-blocking against the CPU oracle (bit for bit) and against the property
the reference tests (tests/quant/test_per_block_cast_lossless.py:90-104): dequantising the result equals
dequantising the input."""
import pytest
import torch

from oracle import torch_ref
from tests._util import assert_same
from tests.test_oracle_lossless import OUT_BLOCKS, SF_MODES, reference_style_input

pytestmark = pytest.mark.gpu


def _tk():
    import tilekernels_amd
    return tilekernels_amd


@pytest.mark.parametrize('out_mode', SF_MODES + [(False, False, False), (True, True, False)],
                         ids=lambda m: 'out-col%d-round%d-packed%d' % tuple(int(v) for v in m))
@pytest.mark.parametrize('in_mode', SF_MODES + [(True, True, False)], ids=lambda m: 'in-col%d-round%d-packed%d' % tuple(int(v) for v in m))
@pytest.mark.parametrize('out_block', OUT_BLOCKS + [(1, 32), (128, 32), (32, 128)])
@pytest.mark.parametrize('num_tokens,hidden', [(401, 576), (130, 2048), (257, 7168), (5, 32), (0, 256)])
def test_per_block_cast_lossless(num_tokens, hidden, out_block, in_mode, out_mode):
    tk = _tk()
    x = reference_style_input(num_tokens, hidden, seed=3 * hidden + num_tokens)
    x_fp4 = torch_ref.cast(x, 'e2m1', (1, 32), use_tma_aligned_col_major_sf=in_mode[0], round_sf=in_mode[1], use_packed_ue8m0=in_mode[2])
    want = torch_ref.per_block_cast_lossless(x_fp4, 'e4m3', (1, 32), out_block, *out_mode)
    got = tk.quant.per_block_cast_lossless((x_fp4[0].cuda(), x_fp4[1].cuda()), 'e4m3', x_block_size=(1, 32), out_block_size=out_block,
                                           use_tma_aligned_col_major_sf=out_mode[0], round_sf=out_mode[1], use_packed_ue8m0=out_mode[2])
    assert_same(got[0], want[0], 'codes')
    assert_same(got[1], want[1], 'scales')
    before = torch_ref.cast_back(x_fp4, 'fp32', (1, 32))
    after = torch_ref.cast_back((got[0].cpu(), got[1].cpu()), 'fp32', out_block)
    assert torch.equal(before.view(torch.int32), after.view(torch.int32))


@pytest.mark.parametrize('in_block,out_block', [((32, 32), (128, 128)), ((1, 128), (128, 128)), ((32, 32), (32, 32))])
def test_per_block_cast_lossless_other_input_blocks(in_block, out_block):
    tk = _tk()
    x = reference_style_input(300, 1024, seed=11)
    x_fp4 = torch_ref.cast(x, 'e2m1', in_block, round_sf=True)
    want = torch_ref.per_block_cast_lossless(x_fp4, 'e4m3', in_block, out_block, round_sf=True)
    got = tk.quant.per_block_cast_lossless((x_fp4[0].cuda(), x_fp4[1].cuda()), 'e4m3', in_block, out_block, round_sf=True)
    assert_same(got[0], want[0], 'codes')
    assert_same(got[1], want[1], 'scales')


def test_per_block_cast_lossless_after_the_gpu_fp4_cast():
    """The chain a weight conversion runs: GPU FP4 cast (1 x 32, packed scales) -> lossless re-blocking to 128 x 128."""
    tk = _tk()
    w = reference_style_input(1024, 4096, seed=5).to(torch.bfloat16).cuda()
    w4 = tk.quant.per_token_cast(w, 'e2m1', 32, use_tma_aligned_col_major_sf=True, round_sf=True, use_packed_ue8m0=True)
    w8 = tk.quant.per_block_cast_lossless(w4, 'e4m3', (1, 32), (128, 128), round_sf=True)
    a = tk.quant.cast_back(w4, 'fp32', (1, 32))
    b = tk.quant.cast_back(w8, 'fp32', (128, 128))
    assert torch.equal(a.view(torch.int32), b.view(torch.int32))


def test_per_block_cast_lossless_with_exponents_far_apart():
    """Input scales more than 127 binades apart inside one output block: the small values vanish (+-0), nothing wraps."""
    tk = _tk()
    g = torch.Generator().manual_seed(17)
    rows, hidden = 256, 1024
    codes = torch.randint(-128, 128, (rows, hidden // 2), generator=g, dtype=torch.int16).to(torch.int8)
    biased = torch.tensor([1, 10, 100, 121, 122, 150, 249, 250], dtype=torch.int32)
    e = biased[torch.randint(0, len(biased), (rows, hidden // 32), generator=g)]
    sf = (e << 23).view(torch.float32)
    for out_block in [(128, 128), (32, 32), (1, 128)]:
        want = torch_ref.per_block_cast_lossless((codes, sf), 'e4m3', (1, 32), out_block, round_sf=True)
        got = tk.quant.per_block_cast_lossless((codes.cuda(), sf.cuda()), 'e4m3', (1, 32), out_block, round_sf=True)
        assert_same(got[0], want[0], 'codes')
        assert_same(got[1], want[1], 'scales')
