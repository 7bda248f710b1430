"""C-ABI checks that need no GPU: the library loads, exports every symbol the header declares, and
its host-side validation returns the documented status codes (no kernel is ever launched here)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, 'include', 'tk_quant.h')


@pytest.fixture(scope='module')
def lib():
    from tilekernels_amd import _ffi
    return _ffi.load()


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(tk_[a-z_0-9]+)\s*\(', text)))


def test_header_symbols_are_exported_and_bound(lib):
    from tilekernels_amd import _ffi
    names = declared_symbols()
    assert len(names) >= 8
    for n in names:
        assert hasattr(lib, n), f'{n} declared in tk_quant.h but not exported'
        assert n in _ffi.SIGNATURES, f'{n} has no ctypes signature'
    assert sorted(_ffi.SIGNATURES) == names


def test_version_and_strerror(lib):
    text = open(HEADER).read()
    want = int(re.search(r'#define TK_QUANT_VERSION (\d+)', text).group(1))
    assert lib.tk_version() == want
    assert lib.tk_strerror(0) == b'ok'
    for code in range(-11, 0):
        assert lib.tk_strerror(code) not in (b'', b'ok', b'unknown status')
    assert lib.tk_strerror(-99) == b'unknown status'
    assert lib.tk_strerror(700) == b'hip error'


# status codes of enum tk_status
OK, NULLP, SHAPE, DTYPE, FMT, GROUP, LAYOUT, MODE, STRIDE, ALIGN, LARGE, VALUE = 0, -1, -2, -3, -4, -5, -6, -7, -8, -9, -10, -11
P = 0x10000   # a fake, well-aligned, non-null device address (never dereferenced by the checks)


def check_pt(lib, x=P, dt=0, M=64, K=1024, ld=None, out=P, sf=P, sf_ld=None, fmt=0, group=128, layout=0, rnd=0, mode=0):
    ld = K if ld is None else ld
    nk = -(-K // group) if group > 0 else 1
    if sf_ld is None:
        sf_ld = nk if layout == 0 else (M + 3) // 4 * 4 if layout == 1 else (4 * M + 15) // 16 * 16
    return lib.tk_check_per_token_cast(x, dt, M, K, ld, out, sf, sf_ld, fmt, group, layout, rnd, mode)


def test_per_token_cast_validation(lib):
    assert check_pt(lib) == OK
    assert check_pt(lib, M=0, x=0, out=0, sf=0) == OK                  # empty input: nothing to check
    assert check_pt(lib, dt=2) == DTYPE
    assert check_pt(lib, fmt=3) == FMT
    assert check_pt(lib, fmt=2) == GROUP                               # E5M6: one scale per row only
    assert check_pt(lib, fmt=2, K=1000, group=1000) == OK              # ... for any K % 8 == 0
    assert check_pt(lib, fmt=2, K=1024, group=1024, layout=2, rnd=1) == OK
    assert check_pt(lib, fmt=2, K=1024, group=1024, mode=1) == MODE
    assert check_pt(lib, fmt=2, K=1024, group=1024, mode=2) == MODE
    assert check_pt(lib, mode=3) == MODE
    assert check_pt(lib, layout=3) == LAYOUT
    assert check_pt(lib, layout=2, rnd=0) == LAYOUT                    # UE8M0 bytes need power-of-two scales
    assert check_pt(lib, layout=2, rnd=1) == OK
    assert check_pt(lib, K=1020) == SHAPE
    assert check_pt(lib, M=-1) == SHAPE
    assert check_pt(lib, group=48) == GROUP
    assert check_pt(lib, K=1024, group=1024) == OK                     # one scale per row
    assert check_pt(lib, K=1000, group=1000) == GROUP                  # ... needs K % 64 == 0
    assert check_pt(lib, K=1024, group=1024, mode=1) == MODE
    assert check_pt(lib, x=0) == NULLP
    assert check_pt(lib, out=0) == NULLP
    assert check_pt(lib, out=0, mode=1) == OK                          # sf-only needs no output
    assert check_pt(lib, sf=0) == NULLP
    assert check_pt(lib, ld=512) == STRIDE
    assert check_pt(lib, sf_ld=4) == STRIDE
    assert check_pt(lib, x=P + 2) == ALIGN
    assert check_pt(lib, ld=1028) == ALIGN
    assert check_pt(lib, out=P + 4) == ALIGN
    assert check_pt(lib, M=2 ** 31) == LARGE


def check_pb(lib, x=P, dt=0, M=256, K=512, out=P, sf=P, sf_ld=None, fmt=0, bm=128, bk=128, layout=0, rnd=0, mode=0):
    if sf_ld is None:
        nm, nk = -(-M // bm), -(-K // bk)
        sf_ld = nk if layout == 0 else (nm + 3) // 4 * 4 if layout == 1 else (4 * nm + 15) // 16 * 16
    return lib.tk_check_per_block_cast(x, dt, M, K, out, sf, sf_ld, fmt, bm, bk, layout, rnd, mode)


def test_per_block_cast_validation(lib):
    assert check_pb(lib) == OK
    for bm, bk in ((32, 32), (32, 128), (128, 32)):
        assert check_pb(lib, bm=bm, bk=bk) == OK
    assert check_pb(lib, bm=64) == GROUP
    assert check_pb(lib, bk=1) == GROUP
    assert check_pb(lib, K=96) == SHAPE                                 # K % 64
    assert check_pb(lib, mode=2, layout=1) == LAYOUT                    # given scales are row-major only
    assert check_pb(lib, layout=2, rnd=0) == LAYOUT
    assert check_pb(lib, x=P + 8) == ALIGN
    assert check_pb(lib, sf=0) == NULLP
    assert check_pb(lib, sf_ld=1) == STRIDE
    assert check_pb(lib, M=0, x=0, out=0, sf=0) == OK
    assert check_pb(lib, dt=7) == DTYPE


def check_sw(lib, x=P, dt=0, R=64, H=2048, out=P, sf=P, sf_ld=None, group=128, layout=0, rnd=0, floor=-1.0,
             ptt=0, w=0, nw=0, pe=0, use_clamp=0, clamp=0.0, cnt=0):
    if sf_ld is None:
        nk = H // group if group else 1
        sf_ld = nk if layout == 0 else (R + 3) // 4 * 4 if layout == 1 else (4 * R + 15) // 16 * 16
    return lib.tk_check_swiglu_per_token_cast(x, dt, R, H, out, sf, sf_ld, group, layout, rnd, floor, ptt, w, nw, pe,
                                              use_clamp, clamp, cnt)


def test_swiglu_validation(lib):
    assert check_sw(lib) == OK
    assert check_sw(lib, group=2048) == OK
    assert check_sw(lib, group=2048, layout=1) == LAYOUT                # one scale per row: row-major only
    assert check_sw(lib, group=256) == GROUP
    assert check_sw(lib, H=2000) == SHAPE
    assert check_sw(lib, R=-5) == SHAPE
    assert check_sw(lib, dt=1, H=2 ** 29) == LARGE                      # an fp32 row of 4 GiB: byte offsets inside a row are 32-bit
    assert check_sw(lib, dt=0, H=2 ** 29, sf_ld=2 ** 22) == OK
    assert check_sw(lib, cnt=P) == MODE                                 # counters need a clamp
    assert check_sw(lib, cnt=P, use_clamp=1, clamp=1.0) == OK
    assert check_sw(lib, cnt=P + 4, use_clamp=1, clamp=1.0) == ALIGN
    assert check_sw(lib, use_clamp=1, clamp=float('nan')) == VALUE
    assert check_sw(lib, floor=float('nan')) == VALUE
    assert check_sw(lib, ptt=P) == NULLP                                # index without weights
    assert check_sw(lib, ptt=P, w=P, nw=128) == OK
    assert check_sw(lib, layout=2, rnd=0) == LAYOUT
    assert check_sw(lib, layout=2, rnd=1) == OK
    assert check_sw(lib, x=P + 4) == ALIGN
    assert check_sw(lib, out=0) == NULLP
    assert check_sw(lib, R=0, x=0, out=0, sf=0) == OK
    assert check_sw(lib, sf_ld=3) == STRIDE


def check_bwd(lib, x=P, x_sf=P, R=64, H=2048, group=128, go=P, w=P, ptt=P, t2p=P, nw=512, out=P, q=P, q_sf=P, xg=P, wg=P,
              rnd=0, use_clamp=0, clamp=0.0):
    return lib.tk_check_swiglu_backward_per_token_cast(x, x_sf, R, H, group, go, w, ptt, t2p, nw, out, q, q_sf, xg, wg, rnd,
                                                       use_clamp, clamp)


def test_swiglu_backward_validation(lib):
    assert check_bwd(lib) == OK
    assert check_bwd(lib, group=32) == OK
    assert check_bwd(lib, group=64) == GROUP
    assert check_bwd(lib, H=2080, group=128) == SHAPE                   # H % group
    assert check_bwd(lib, R=-1) == SHAPE
    assert check_bwd(lib, use_clamp=1, clamp=float('nan')) == VALUE
    assert check_bwd(lib, go=0) == NULLP
    assert check_bwd(lib, wg=0) == NULLP                                # needed whenever there are (token, k) pairs
    assert check_bwd(lib, R=0, x=0, x_sf=0, go=0, w=0, ptt=0, out=0, q=0, q_sf=0, xg=0) == OK   # no rows: only weight_grad
    assert check_bwd(lib, R=0, nw=0, x=0, x_sf=0, go=0, w=0, ptt=0, t2p=0, out=0, q=0, q_sf=0, xg=0, wg=0) == OK
    assert check_bwd(lib, go=P + 8) == ALIGN
    assert check_bwd(lib, x=P + 4) == ALIGN
    assert check_bwd(lib, R=2 ** 31) == LARGE


def check_pc(lib, x=P, dt=0, x_sf=0, T=256, K=512, p2t=0, M=256, out=P, out_sf=P, npt=128, rnd=0, tr=0, sw=0, use_clamp=0,
             clamp=0.0):
    return lib.tk_check_per_channel_cast(x, dt, x_sf, T, K, p2t, M, out, out_sf, npt, rnd, tr, sw, use_clamp, clamp)


def test_per_channel_cast_validation(lib):
    assert check_pc(lib) == OK
    assert check_pc(lib, npt=32, tr=1) == OK
    assert check_pc(lib, npt=64) == GROUP
    assert check_pc(lib, dt=1) == OK                                    # fp32: plain and gathered casts only
    assert check_pc(lib, dt=1, T=128, p2t=P) == OK
    assert check_pc(lib, dt=1, tr=1) == DTYPE
    assert check_pc(lib, dt=1, sw=1) == DTYPE
    assert check_pc(lib, dt=1, x_sf=P, K=256) == DTYPE
    assert check_pc(lib, dt=2) == DTYPE
    assert check_pc(lib, M=250) == SHAPE                                # M % 16
    assert check_pc(lib, K=20) == SHAPE                                 # K % 8
    assert check_pc(lib, T=128) == SHAPE                                # without a gather the input must hold M rows
    assert check_pc(lib, T=128, p2t=P) == OK
    assert check_pc(lib, T=0, p2t=P) == SHAPE                           # a gather needs at least one input row (row 0 stands in for dropped ones)
    assert check_pc(lib, x_sf=P, K=192) == MODE                         # FP8 input comes with 1 x 128 scales
    assert check_pc(lib, x_sf=P, K=256) == OK
    assert check_pc(lib, x_sf=P, sw=1) == MODE
    assert check_pc(lib, sw=1, p2t=P) == MODE
    assert check_pc(lib, use_clamp=1, clamp=1.0) == VALUE               # the clamp belongs to the SwiGLU form
    assert check_pc(lib, sw=1, use_clamp=1, clamp=1.0) == OK
    assert check_pc(lib, x=P + 8) == ALIGN
    assert check_pc(lib, x=P + 8, x_sf=P, K=256) == OK                  # codes need 8-byte alignment only
    assert check_pc(lib, out=P + 8, tr=1) == ALIGN
    assert check_pc(lib, out=0) == NULLP
    assert check_pc(lib, M=0, T=0, x=0, out=0, out_sf=0) == OK


def check_ll(lib, x=P, M=256, K=512, x_sf=P, x_ld=None, x_layout=0, ibm=1, ibk=32, out=P, out_sf=P, o_ld=None, o_layout=0, obm=128, obk=128):
    inm, ink, onm, onk = -(-M // ibm), -(-K // ibk), -(-M // obm), -(-K // obk)
    if x_ld is None:
        x_ld = ink if x_layout == 0 else (inm + 3) // 4 * 4 if x_layout == 1 else (4 * inm + 15) // 16 * 16
    if o_ld is None:
        o_ld = onk if o_layout == 0 else (onm + 3) // 4 * 4 if o_layout == 1 else (4 * onm + 15) // 16 * 16
    return lib.tk_check_per_block_cast_lossless(x, M, K, x_sf, x_ld, x_layout, ibm, ibk, out, out_sf, o_ld, o_layout, obm, obk)


def test_per_block_cast_lossless_validation(lib):
    assert check_ll(lib) == OK
    assert check_ll(lib, obm=1) == OK and check_ll(lib, obm=32, obk=32) == OK
    assert check_ll(lib, x_layout=2, o_layout=2) == OK
    assert check_ll(lib, x_layout=3) == LAYOUT and check_ll(lib, o_layout=-1) == LAYOUT
    assert check_ll(lib, K=500) == SHAPE
    assert check_ll(lib, obk=96) == GROUP                               # output blocks divide the 128 x 128 tile
    assert check_ll(lib, obm=256) == GROUP
    assert check_ll(lib, ibk=64, obk=32) == GROUP                       # ... and hold whole input blocks
    assert check_ll(lib, ibm=32, obm=1) == GROUP
    assert check_ll(lib, ibk=4) == GROUP
    assert check_ll(lib, x=0) == NULLP and check_ll(lib, out_sf=0) == NULLP
    assert check_ll(lib, x=P + 2) == ALIGN and check_ll(lib, out=P + 4) == ALIGN
    assert check_ll(lib, x_ld=3) == STRIDE and check_ll(lib, o_ld=1) == STRIDE
    assert check_ll(lib, M=0, x=0, x_sf=0, out=0, out_sf=0) == OK


def check_rf(lib, x=P, dt=0, R=1024, hidden=2048, x_sf=0, w=0, pos=P, T=128, K=8, out=P, odt=None, sf=0):
    return lib.tk_check_reduce_fused(x, dt, R, hidden, x_sf, w, pos, T, K, out, dt if odt is None else odt, sf)


def test_reduce_fused_validation(lib):
    assert check_rf(lib) == OK and check_rf(lib, dt=1) == OK
    assert check_rf(lib, odt=2) == OK and check_rf(lib, dt=1, odt=2, sf=P, w=P, x_sf=P) == OK     # FP8 output
    assert check_rf(lib, dt=0, odt=1) == DTYPE                          # otherwise the output has the input's type
    assert check_rf(lib, dt=2) == DTYPE
    assert check_rf(lib, hidden=2052) == SHAPE and check_rf(lib, K=0) == SHAPE
    assert check_rf(lib, pos=0) == NULLP and check_rf(lib, out=0) == NULLP and check_rf(lib, x=0) == NULLP
    assert check_rf(lib, x=P + 8) == ALIGN and check_rf(lib, out=P + 8) == ALIGN
    assert check_rf(lib, out=P + 8, odt=2) == OK                        # FP8 rows need 8-byte alignment only
    assert check_rf(lib, T=0, pos=0, out=0, x=0) == OK


def test_cast_back_validation(lib):
    def check(x=P, fmt=0, M=64, K=1024, sf=P, ld=None, layout=0, bm=1, bk=128, out=P, dt=0):
        ld = (-(-K // bk) if bk > 0 else K) if ld is None else ld
        return lib.tk_check_cast_back(x, fmt, M, K, sf, ld, layout, bm, bk, out, dt)
    assert check() == OK
    assert check(bm=128, bk=1) == OK and check(bm=128, bk=2) == OK and check(bm=128, bk=4) == OK     # per-channel scales
    assert check(bk=3) == GROUP and check(bk=12) == GROUP and check(bk=0) == GROUP and check(bm=0) == GROUP
    assert check(bm=128, bk=1, ld=1000) == STRIDE                       # one scale per column: the row of scales is K long
    assert check(K=1020) == SHAPE
    assert check(fmt=7) == FMT and check(dt=5) == DTYPE
    assert check(out=0) == NULLP and check(sf=0) == NULLP
    assert check(M=0, x=0, sf=0, out=0) == OK


def test_moe_layout_validation(lib):
    ws = lib.tk_fused_mapping_workspace_bytes(4096, 8, 256)
    assert ws > 0

    def check_map(idx=P, T=4096, K=8, E=256, align=128, R=49152, ws_ptr=P, ws_bytes=ws, outs=P):
        return lib.tk_check_get_fused_mapping(idx, T, K, E, align, R, outs, outs, outs, outs, outs, outs, outs, ws_ptr, ws_bytes)
    assert check_map() == OK
    assert check_map(E=2048) != OK                                      # more experts than the per-wave histogram holds
    assert check_map(align=0) == VALUE
    assert check_map(ws_bytes=ws - 4) == STRIDE                         # workspace too small
    assert check_map(idx=0) == NULLP
    assert check_map(outs=0) == NULLP

    def check_exp(x=P, T=64, rb=4096, t2p=P, K=2, p2e=P, R=256, out=P, x_sf=0, cols=0, out_sf=0, ld=0, cm=0):
        return lib.tk_check_expand_to_fused(x, T, rb, t2p, K, p2e, R, out, x_sf, cols, out_sf, ld, cm)
    assert check_exp() == OK
    assert check_exp(rb=4100) == ALIGN                                  # rows move as 16-byte pieces
    assert check_exp(out=0) == NULLP
    assert check_exp(x_sf=P, cols=32, out_sf=P, ld=32) == OK
    assert check_exp(x_sf=P, cols=32, out_sf=P, ld=16) == STRIDE
    assert check_exp(x_sf=P, cols=32, out_sf=0, ld=32) == NULLP


def test_launching_entry_points_reject_before_touching_the_device(lib):
    """A rejected call returns the status from the same validation and launches nothing, so it is safe
    without a GPU."""
    assert lib.tk_per_token_cast(P, 0, 64, 1020, 1020, P, P, 8, 0, 128, 0, 0, 0, None) == SHAPE
    assert lib.tk_per_block_cast(P, 0, 64, 512, P, P, 4, 0, 64, 64, 0, 0, 0, None) == GROUP
    assert lib.tk_swiglu_per_token_cast(P, 0, 64, 2000, P, P, 16, 128, 0, 0, -1.0, None, None, 0, None, 0, 0.0, None, 0, None) == SHAPE
    assert lib.tk_per_token_cast(None, 0, 0, 1024, 1024, None, None, 8, 0, 128, 0, 0, 0, None) == OK     # M == 0
    # the entry point with library-owned scratch refuses what its table cannot hold before any device call
    assert lib.tk_fused_mapping_workspace_bytes(262145, 4, 1024) > (4 << 20)
    assert lib.tk_get_fused_mapping_static(P, 262145, 4, 1024, 16, 1 << 20, P, P, P, P, P, P, P, None) == LARGE


def test_host_side_geometry_matches_the_oracle_layouts():
    """Scale-tensor shapes/strides produced by the host wrapper (allocation + epilogue) equal the oracle's."""
    import torch
    from oracle import torch_ref
    from tilekernels_amd.quant.common import alloc_scaling_factors, cast_epilogue, get_cast_output_config, sf_leading_dim
    for (M, K, blk) in ((37, 576, (1, 128)), (4001, 7168, (1, 32)), (130, 2560, (128, 128)), (1, 64, (1, 64)), (5, 512, (32, 32))):
        x = torch.zeros((M, K), dtype=torch.bfloat16)
        for col, rnd, packed in ((False, False, False), (True, False, False), (True, True, True)):
            cfg = get_cast_output_config('e4m3', blk, col, rnd, packed)
            store = alloc_scaling_factors((M, K), cfg, 'cpu')
            got = cast_epilogue(store, M, K, cfg)
            _, want = torch_ref.cast(x, 'e4m3', blk, round_sf=rnd, use_tma_aligned_col_major_sf=col, use_packed_ue8m0=packed)
            assert got.dtype == want.dtype and got.shape == want.shape and got.stride() == want.stride(), (M, K, blk, col, packed)
            nm, nk = -(-M // blk[0]), -(-K // blk[1])
            need = nk if not col else (4 * nm if packed else nm)
            assert sf_leading_dim(store) >= need


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from tilekernels_amd import _ffi
    monkeypatch.setattr(_ffi, '_lib', None)
    monkeypatch.setattr(_ffi, 'LIB_PATH', str(tmp_path / 'nope.so'))
    with pytest.raises(ImportError):
        _ffi.load()
