"""tk_stream_floor (the traffic-only kernel bench.py times beside the operators) reads every input word and writes
every output byte it claims to: its output is a fixed XOR fold of the input, checked here against numpy."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('rows,cols,two', [(37, 2048, True), (64, 4096, False), (5, 1024, False), (130, 7168, False), (9, 3072, True)])
def test_stream_floor_reads_and_writes_everything(rows, cols, two):
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    width = cols * (2 if two else 1)
    xs = np.random.default_rng(rows * cols).integers(0, 2 ** 16, size=(rows, width), dtype=np.uint16)
    xd = torch.from_numpy(xs.view(np.int16)).cuda()
    out = torch.full((rows, cols), 0xAB, dtype=torch.uint8, device='cuda')
    sf = torch.full((rows, cols // 128), -1, dtype=torch.int32, device='cuda')
    rc = lib.tk_stream_floor(xd.data_ptr(), rows, cols, int(two), out.data_ptr(), sf.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    # per 8 input elements (four 32-bit words a, b, c, d; XORed with the other half's words when two halves are read)
    # the kernel stores the two words a ^ c, b ^ d
    w = xs.view(np.uint32).reshape(rows, width // 2)
    if two:
        w = w[:, : cols // 2] ^ w[:, cols // 2:]
    q = w.reshape(rows, cols // 8, 4)
    want = np.stack([q[:, :, 0] ^ q[:, :, 2], q[:, :, 1] ^ q[:, :, 3]], axis=-1).reshape(rows, cols // 4).view(np.uint8).reshape(rows, cols)
    assert np.array_equal(out.cpu().numpy(), want)
    assert not bool((sf == -1).all(dim=1).any())          # every row's words were written


def test_stream_floor_rejects_bad_shapes():
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    p = torch.zeros(16, dtype=torch.int64, device='cuda').data_ptr()
    assert lib.tk_stream_floor(p, 4, 1000, 0, p, 0, None) != 0          # columns not a multiple of 1024
    assert lib.tk_stream_floor(0, 4, 1024, 0, p, 0, None) != 0          # null input
    assert lib.tk_stream_floor(0, 0, 1024, 0, 0, 0, None) == 0          # no rows: nothing to do
