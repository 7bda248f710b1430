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
    # the word of group 4 * p + g (p: piece of 512 columns, g: its 128-column group) is written by lane 16 * g + (p mod P)
    # of the wave that holds the piece, P pieces per wave, and is the XOR of the first word that lane loaded of each of
    # the wave's pieces
    P = 4 if cols % 2048 == 0 else 2
    want_sf = np.zeros((rows, cols // 128), dtype=np.uint32)
    for tile in range(cols // (P * 512)):
        for j in range(P):
            for g in range(4):
                lane = 16 * g + j
                fold = np.zeros(rows, dtype=np.uint32)
                for r in range(P):
                    fold ^= w[:, ((tile * P + r) * 512 + lane * 8) // 2]
                want_sf[:, (tile * P + j) * 4 + g] = fold
    assert np.array_equal(sf.cpu().numpy().view(np.uint32), want_sf)


@pytest.mark.parametrize('rows,cols,two,r2,r1', [(64, 2048, True, 24, 12), (40, 4096, False, 20, 8), (16, 2048, True, 0, 16), (16, 2048, True, 16, 0), (8, 6144, True, 0, 0)])
def test_stream_floor_with_smaller_waves_at_the_end_writes_the_same(rows, cols, two, r2, r1):
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    width = cols * (2 if two else 1)
    xd = torch.randint(-2 ** 15, 2 ** 15, (rows, width), dtype=torch.int16, device='cuda')
    stream = torch.cuda.current_stream().cuda_stream
    out = [torch.full((rows, cols), 0xAB, dtype=torch.uint8, device='cuda') for _ in range(2)]
    assert lib.tk_stream_floor(xd.data_ptr(), rows, cols, int(two), out[0].data_ptr(), 0, stream) == 0
    sf = torch.full((rows, cols // 128), -1, dtype=torch.int32, device='cuda')
    assert lib.tk_stream_floor_tailed(xd.data_ptr(), rows, cols, int(two), out[1].data_ptr(), sf.data_ptr(), r2, r1, stream) == 0
    assert lib.tk_stream_floor_tailed(xd.data_ptr(), rows, cols, int(two), out[1].data_ptr(), sf.data_ptr(), rows, 4, stream) != 0   # more than there are
    torch.cuda.synchronize()
    assert torch.equal(out[0], out[1])
    # a scale word is the XOR of the first word its lane loaded of each of its wave's pieces: with one piece per wave that
    # is the first word of the group's own piece at lane 16 * g + (piece mod 1) = 16 * g
    w = xd.cpu().numpy().view(np.uint32).reshape(rows, width // 2)
    if two:
        w = w[:, : cols // 2] ^ w[:, cols // 2:]
    got = sf.cpu().numpy().view(np.uint32)
    for row in range(rows - r1, rows):
        for piece in range(cols // 512):
            for g in range(4):
                assert got[row, piece * 4 + g] == w[row, (piece * 512 + 16 * g * 8) // 2]
    assert not bool((sf == -1).any())


def test_stream_floor_rejects_bad_shapes():
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    p = torch.zeros(16, dtype=torch.int64, device='cuda').data_ptr()
    assert lib.tk_stream_floor(p, 4, 1000, 0, p, 0, None) != 0          # columns not a multiple of 1024
    assert lib.tk_stream_floor(0, 4, 1024, 0, p, 0, None) != 0          # null input
    assert lib.tk_stream_floor(0, 0, 1024, 0, 0, 0, None) == 0          # no rows: nothing to do


@pytest.mark.parametrize('rows,cols,two', [(37, 2048, True), (64, 4096, False), (9, 3072, True), (21, 1024, False)])
def test_stream_floor_timeline_stamps_every_wave(rows, cols, two):
    """The time-stamped variant writes the same output and, per wave, four non-decreasing times and its place."""
    from tilekernels_amd import _ffi
    lib = _ffi.load()
    width = cols * (2 if two else 1)
    xd = torch.randint(-2 ** 15, 2 ** 15, (rows, width), dtype=torch.int16, device='cuda')
    stream = torch.cuda.current_stream().cuda_stream
    out = [torch.zeros((rows, cols), dtype=torch.uint8, device='cuda') for _ in range(2)]
    sf = [torch.zeros((rows, cols // 128), dtype=torch.int32, device='cuda') for _ in range(2)]
    words = lib.tk_stream_floor_stamp_words(rows, cols)
    assert words == rows * (cols // (2048 if cols % 2048 == 0 else 1024)) * 6
    stamps = torch.zeros(words, dtype=torch.int64, device='cuda')
    assert lib.tk_stream_floor(xd.data_ptr(), rows, cols, int(two), out[0].data_ptr(), sf[0].data_ptr(), stream) == 0
    assert lib.tk_stream_floor_timeline(xd.data_ptr(), rows, cols, int(two), out[1].data_ptr(), sf[1].data_ptr(), stamps.data_ptr(), stream) == 0
    assert lib.tk_stream_floor_timeline(xd.data_ptr(), rows, cols, int(two), out[1].data_ptr(), sf[1].data_ptr(), 0, stream) != 0     # no stamp buffer
    torch.cuda.synchronize()
    assert torch.equal(out[0], out[1]) and torch.equal(sf[0], sf[1])
    t = stamps.cpu().numpy().reshape(-1, 6)
    assert (t[:, 0] > 0).all()
    assert (t[:, 0] <= t[:, 1]).all() and (t[:, 1] <= t[:, 2]).all() and (t[:, 2] <= t[:, 3]).all()
    assert ((t[:, 3] - t[:, 0]) < 100 * 1000).all()             # well under a millisecond at 100 MHz
    assert ((t[:, 5] & 0xF) < 8).all()                          # XCD number
