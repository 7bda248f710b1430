// Dequantisation of block-scaled E4M3 / packed E2M1 codes back to bf16 or fp32 for gfx950.
//
// out[m, k] = float(code[m, k]) * sf[m / bm, k / bk], one fp32 product, then (for bf16) one
// round-to-nearest-even conversion (v_cvt_pk_bf16_f32).  Pure streaming: for bf16 a lane takes 8
// consecutive codes (8 or 4 bytes), their shared scale, and writes 16 bytes; for fp32 it takes 4 codes
// of two pieces 256 columns apart and writes 16 bytes of each, so that every store instruction of a
// wave covers whole cache lines.  A workgroup covers 2 rows x up to 4096 columns (row-major scales) or
// 8 rows x 512 columns; half as many rows for fp32 output.
//
// Reference semantics: tile_kernels/quant/cast_back_kernel.py:19-75 (kernel) and :77-143 (wrappers),
// tile_kernels/torch/cast.py:40-59 (oracle).
#include "tk_device.hpp"
#include "tk_host.hpp"

namespace tk {

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// Rows per wave.  Measured on MI355X, E4M3 [8192, 4096] (us per call, 1 / 2 / 4 rows): to bf16 18.8 / 17.4 / 18.4, to fp32
// (whose lanes already hold two pieces per row) 28.8 / 29.6 / 31.4.
template <bool OUT_F32> constexpr int back_rows_per_wave() { return OUT_F32 ? 1 : 2; }

// WIDE: the workgroup's waves stand side by side on the same RPW rows (row-major scales: one
// workgroup then reads a row's scales once, instead of eight workgroups on eight L2s each fetching
// the line for 16 bytes of it); otherwise the 4 waves are stacked, 512 columns wide.
template <typename InT, bool OUT_F32, bool WIDE, bool FULL>
__global__ __launch_bounds__(WIDE ? 64 * kMaxWideWaves : kThreads) void cast_back_kernel(const void *x, void *out, void *a_sf, int64_t a_sf_ld,
                                                                                         int M, int K, int geom, int bm, int bk, int a_sf_layout,
                                                                                         int nm, int nk) {
    constexpr int RPW = back_rows_per_wave<OUT_F32>(), ROWS = WIDE ? RPW : kWaves * RPW;
    const SfRef sf{a_sf, a_sf_ld, a_sf_layout, nm, nk};
    // geom: wide tiles: waves per tile, the tile index comes from the grid (x = column tile, y and z = row
    // tile); otherwise the number of column tiles of a 1-D grid
    const bool one_col = geom * kStripCols >= K;   // wide tiles: the waves of one tile cover a whole row
    const int tile_m = WIDE ? tile_grid_row(one_col) : (int)blockIdx.x / geom;
    const int tile_k = WIDE ? tile_grid_col(one_col) : (int)blockIdx.x - tile_m * geom;
    const int lane = threadIdx.x & 63, wave = wave_id();
    const int strip = WIDE ? tile_k * geom + wave : tile_k;
    const int col = strip * kStripCols + lane * 8;
    const bool col_ok = FULL || col < K;
    const int row0 = tile_m * ROWS + (WIDE ? 0 : wave * RPW);

    if constexpr (OUT_F32) {
        // fp32 output: 8 values are 32 bytes, two 16-byte stores.  Were they a lane's own piece, each store
        // instruction would write every other 16 bytes of its cache lines (half lines: 49.8 us for 8192 x 4096
        // E4M3).  So a lane takes 4 codes of two pieces instead, columns 4 * lane and 256 + 4 * lane of the strip,
        // and each store instruction writes 1024 consecutive bytes.  Two lanes load the same piece; the
        // second load is served by the same fetch.
        const bool hi = lane & 1;
        const int pcol = strip * kStripCols + (lane >> 1) * 8;
        Raw8<InT> raw[RPW][2];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int c = pcol + h * (kStripCols / 2);
                // no branch around the loads: a lane beyond the last row or column reads the first codes and the first
                // scale, and writes nothing
                const bool ok = (FULL || c < K) && (FULL || row0 + r < M);
                raw[r][h].load(ok ? elem_ptr<InT>(x, row0 + r, K, c) : x);
                vmem_issue_gap();
                raw[r][h].s = sf_load(sf, ok ? (row0 + r) / bm : 0, ok ? c / bk : 0);
                vmem_issue_gap();
            }
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int c = pcol + h * (kStripCols / 2);
                if (!((FULL || c < K) && (FULL || row0 + r < M))) continue;
                float v[4];
                raw[r][h].get4(v, hi);
                const int64_t idx = (int64_t)(row0 + r) * K + c + (hi ? 4 : 0);
                __builtin_nontemporal_store(u32x4{f2u(v[0]), f2u(v[1]), f2u(v[2]), f2u(v[3])},
                                            reinterpret_cast<u32x4 *>(reinterpret_cast<float *>(out) + idx));
            }
        }
    } else {
        Raw8<InT> raw[RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const bool ok = col_ok && (FULL || row0 + r < M);
            raw[r].load(ok ? elem_ptr<InT>(x, row0 + r, K, col) : x);
            vmem_issue_gap();
            raw[r].s = sf_load(sf, ok ? (row0 + r) / bm : 0, ok ? col / bk : 0);
            vmem_issue_gap();
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            if (!(col_ok && (FULL || row0 + r < M))) continue;
            float v[8];
            raw[r].get(v);
            const int64_t idx = (int64_t)(row0 + r) * K + col;
            u32x4 w;
            w.x = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[0], v[1]}), bf16x2));
            w.y = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[2], v[3]}), bf16x2));
            w.z = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[4], v[5]}), bf16x2));
            w.w = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[6], v[7]}), bf16x2));
            __builtin_nontemporal_store(w, reinterpret_cast<u32x4 *>(reinterpret_cast<uint16_t *>(out) + idx));
        }
    }
}

// Short rows: the rows laid end to end in pieces of 8 codes, lane slot L serving piece L of the sequence, so that every
// lane has a piece whatever the row length (with 512-column strips a row of 576 columns keeps 72 of every 128 lanes
// busy, one of 64 columns 8 of 64).  fp32 output as in the tiled kernel: a lane takes 4 codes of two pieces 32 pieces
// apart, so that a store instruction of the wave covers consecutive bytes wherever the pieces are consecutive.
template <typename InT, bool OUT_F32>
__global__ __launch_bounds__(kThreads) void cast_back_flat_kernel(const void *x, void *out, void *a_sf, int64_t a_sf_ld, int M, int K, int ppr,
                                                                  unsigned ppr_recip, int bm, int bk, int a_sf_layout, int nm, int nk, int bm_sh, int bk_sh) {
    constexpr int RPW = 2;
    // block indices by shifts where the block extents are powers of two (bm_sh, bk_sh >= 0), which they nearly always are
    auto blk_m = [&](int row) { return bm_sh >= 0 ? row >> bm_sh : row / bm; };
    auto blk_k = [&](int col) { return bk_sh >= 0 ? col >> bk_sh : col / bk; };
    const SfRef sf{a_sf, a_sf_ld, a_sf_layout, nm, nk};
    const int lane = threadIdx.x & 63, wave = wave_id();
    const unsigned total = (unsigned)M * (unsigned)ppr;
    // All loads of the wave's slots go out before its first store: with a slot's store in front of the next slot's loads
    // the compiler must keep that order (input and output may overlap for all it knows) and the wave has one slot's
    // loads in flight at a time.
    if constexpr (OUT_F32) {
        const bool hi = lane & 1;
        Raw8<InT> raw[RPW][2];
        int row[RPW][2], col[RPW][2];
        bool ok[RPW][2];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const unsigned slot = (unsigned)((blockIdx.x * kWaves + wave) * RPW + r);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const unsigned piece = slot * 64u + (unsigned)(h * 32 + (lane >> 1));
                ok[r][h] = piece < total;
                // piece / ppr by multiplication: with floor(2^32 / ppr) the quotient comes out exact or one too small
                unsigned q = __umulhi(piece, ppr_recip), rem = piece - q * (unsigned)ppr;
                if (rem >= (unsigned)ppr) { ++q; rem -= (unsigned)ppr; }
                row[r][h] = (int)q;
                col[r][h] = (int)rem * 8;
                raw[r][h].load(ok[r][h] ? elem_ptr<InT>(x, row[r][h], K, col[r][h]) : x);
                vmem_issue_gap();
                raw[r][h].s = sf_load(sf, ok[r][h] ? blk_m(row[r][h]) : 0, ok[r][h] ? blk_k(col[r][h]) : 0);
                vmem_issue_gap();
            }
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                if (!ok[r][h]) continue;
                float v[4];
                raw[r][h].get4(v, hi);
                const int64_t idx = (int64_t)row[r][h] * K + col[r][h] + (hi ? 4 : 0);
                __builtin_nontemporal_store(u32x4{f2u(v[0]), f2u(v[1]), f2u(v[2]), f2u(v[3])},
                                            reinterpret_cast<u32x4 *>(reinterpret_cast<float *>(out) + idx));
            }
        }
    } else {
        Raw8<InT> raw[RPW];
        int row[RPW], col[RPW];
        bool ok[RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const unsigned piece = (unsigned)((blockIdx.x * kWaves + wave) * RPW + r) * 64u + (unsigned)lane;
            ok[r] = piece < total;
            unsigned q = __umulhi(piece, ppr_recip), rem = piece - q * (unsigned)ppr;
            if (rem >= (unsigned)ppr) { ++q; rem -= (unsigned)ppr; }
            row[r] = (int)q;
            col[r] = (int)rem * 8;
            raw[r].load(ok[r] ? elem_ptr<InT>(x, row[r], K, col[r]) : x);
            vmem_issue_gap();
            raw[r].s = sf_load(sf, ok[r] ? blk_m(row[r]) : 0, ok[r] ? blk_k(col[r]) : 0);
            vmem_issue_gap();
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            if (!ok[r]) continue;
            float v[8];
            raw[r].get(v);
            u32x4 w;
            w.x = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[0], v[1]}), bf16x2));
            w.y = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[2], v[3]}), bf16x2));
            w.z = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[4], v[5]}), bf16x2));
            w.w = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[6], v[7]}), bf16x2));
            __builtin_nontemporal_store(w, reinterpret_cast<u32x4 *>(reinterpret_cast<uint16_t *>(out) + (int64_t)row[r] * K + col[r]));
        }
    }
}

// Scale blocks narrower than a lane's 8 codes (bk = 1, 2 or 4: per-channel scales, as tile_kernels.quant.cast_back is
// called with x_block_size (128, 1)): every code of a piece has its own scale column, so a lane fetches 8 / bk scales
// beside its codes.  Pieces are laid end to end as in the kernel above; a lane writes its own 8 values (fp32: two
// 16-byte stores).
template <typename InT, bool OUT_F32>
__global__ __launch_bounds__(kThreads) void cast_back_fine_kernel(const void *x, void *out, void *a_sf, int64_t a_sf_ld, int M, int K, int ppr,
                                                                  unsigned ppr_recip, int bm, int bk, int a_sf_layout, int nm, int nk) {
    const SfRef sf{a_sf, a_sf_ld, a_sf_layout, nm, nk};
    const unsigned total = (unsigned)M * (unsigned)ppr;
    const unsigned piece = blockIdx.x * (unsigned)kThreads + threadIdx.x;
    if (piece >= total) return;
    unsigned q = __umulhi(piece, ppr_recip), rem = piece - q * (unsigned)ppr;
    if (rem >= (unsigned)ppr) { ++q; rem -= (unsigned)ppr; }
    const int row = (int)q, col = (int)rem * 8;
    Raw8<InT> raw;
    raw.load(elem_ptr<InT>(x, row, K, col));
    raw.s = 1.0f;                       // exact: the one rounding is the product with the element's own scale below
    const int mb = row / bm;
    float sc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) sc[i] = sf_load_select(sf, mb, (col + i) / bk);
    float v[8];
    raw.get(v);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = v[i] * sc[i];
    const int64_t idx = (int64_t)row * K + col;
    if constexpr (OUT_F32) {
        u32x4 *dst = reinterpret_cast<u32x4 *>(reinterpret_cast<float *>(out) + idx);
        __builtin_nontemporal_store(u32x4{f2u(v[0]), f2u(v[1]), f2u(v[2]), f2u(v[3])}, dst);
        __builtin_nontemporal_store(u32x4{f2u(v[4]), f2u(v[5]), f2u(v[6]), f2u(v[7])}, dst + 1);
    } else {
        u32x4 w;
        w.x = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[0], v[1]}), bf16x2));
        w.y = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[2], v[3]}), bf16x2));
        w.z = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[4], v[5]}), bf16x2));
        w.w = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[6], v[7]}), bf16x2));
        __builtin_nontemporal_store(w, reinterpret_cast<u32x4 *>(reinterpret_cast<uint16_t *>(out) + idx));
    }
}

template <typename InT, bool OUT_F32, bool WIDE>
static void launch_cast_back_2(const void *x, void *out, const void *sf, int64_t sf_ld, int M, int K, int sf_layout, int bm, int bk,
                               hipStream_t stream) {
    const int strips = (K + kStripCols - 1) / kStripCols;
    const int waves = WIDE ? wide_tile_waves(strips) : kWaves;
    constexpr int RPW = back_rows_per_wave<OUT_F32>();
    const int rows = WIDE ? RPW : kWaves * RPW;
    const int cols = WIDE ? waves * kStripCols : kStripCols;
    const int tiles_m = (M + rows - 1) / rows, tiles_k = (K + cols - 1) / cols;
    const int nm = (M + bm - 1) / bm, nk = (K + bk - 1) / bk;
    const dim3 block(64 * waves);
    const dim3 grid = WIDE ? tile_grid(tiles_k, tiles_m) : dim3((unsigned)(tiles_m * tiles_k));
    const int geom = WIDE ? waves : tiles_k;
    void *sfp = const_cast<void *>(sf);
    if (M % rows == 0 && K % cols == 0 && (!WIDE || tile_grid_exact(tiles_k, tiles_m)))
        hipLaunchKernelGGL((cast_back_kernel<InT, OUT_F32, WIDE, true>), grid, block, 0, stream, x, out, sfp, sf_ld, M, K, geom, bm, bk, sf_layout, nm, nk);
    else
        hipLaunchKernelGGL((cast_back_kernel<InT, OUT_F32, WIDE, false>), grid, block, 0, stream, x, out, sfp, sf_ld, M, K, geom, bm, bk, sf_layout, nm, nk);
}

// log2 of a power of two, -1 for any other value
inline int log2_or_minus1(int v) {
    for (int s = 0; s < 31; ++s)
        if ((1 << s) == v) return s;
    return -1;
}

template <typename InT, bool OUT_F32>
static hipError_t launch_cast_back(const void *x, void *out, const void *sf, int64_t sf_ld, int M, int K, int sf_layout,
                                   int bm, int bk, hipStream_t stream) {
    // (one row per wave with its pieces along the row, the shape that pays in the per-token cast, measured within 2 % here
    // either way: E4M3 [8192, 4096] to bf16 17.25 -> 17.43 us, to fp32 29.63 -> 29.08 us)
    // wide tiles with column-major scales are no faster (E4M3 [8192, 4096]) and slower with 32 x 32 blocks (20.9 us
    // against 16.2 us): a 2-row tile then uses 8 bytes of each scale line it touches
    // rows that fill less than 80 % of their 512-column strips
    const int64_t strips = (K + kStripCols - 1) / kStripCols, pieces = (int64_t)M * (K / 8);
    if (bk < 8) {
        const int64_t blocks = (pieces + kThreads - 1) / kThreads;
        hipLaunchKernelGGL((cast_back_fine_kernel<InT, OUT_F32>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, x, out,
                           const_cast<void *>(sf), sf_ld, M, K, K / 8,
                           (unsigned)(K == 8 ? 0xFFFFFFFFull : (1ull << 32) / (uint64_t)(K / 8)), bm, bk, sf_layout, (M + bm - 1) / bm, (K + bk - 1) / bk);
        return hipGetLastError();
    }
    if (K * 5 < strips * kStripCols * 4 && pieces < INT32_MAX - 4 * kThreads) {   // pieces are numbered in 32 bits
        const int64_t blocks = (pieces + 2 * kThreads - 1) / (2 * kThreads);
        hipLaunchKernelGGL((cast_back_flat_kernel<InT, OUT_F32>), dim3((unsigned)blocks), dim3(kThreads), 0, stream, x, out,
                           const_cast<void *>(sf), sf_ld, M, K, K / 8,
                           (unsigned)(K == 8 ? 0xFFFFFFFFull : (1ull << 32) / (uint64_t)(K / 8)), bm, bk, sf_layout, (M + bm - 1) / bm, (K + bk - 1) / bk,
                           log2_or_minus1(bm), log2_or_minus1(bk));
        return hipGetLastError();
    }
    if (sf_layout == TK_SF_ROW_F32 && wide_tiles_pay(K)) launch_cast_back_2<InT, OUT_F32, true>(x, out, sf, sf_ld, M, K, sf_layout, bm, bk, stream);
    else launch_cast_back_2<InT, OUT_F32, false>(x, out, sf, sf_ld, M, K, sf_layout, bm, bk, stream);
    return hipGetLastError();
}

}  // namespace tk

using namespace tk;

extern "C" int tk_check_cast_back(const void *x, int x_fmt, int64_t M, int64_t K, const void *x_sf, int64_t x_sf_ld,
                                  int x_sf_layout, int bm, int bk, const void *out, int out_dtype) {
    if (x_fmt != TK_E4M3 && x_fmt != TK_E2M1 && x_fmt != TK_E5M6) return TK_ERR_BAD_FORMAT;
    if (out_dtype != TK_BF16 && out_dtype != TK_F32) return TK_ERR_BAD_DTYPE;
    if (x_sf_layout < TK_SF_ROW_F32 || x_sf_layout > TK_SF_COL_UE8M0) return TK_ERR_BAD_LAYOUT;
    if (M < 0 || K <= 0 || K % 8 != 0) return TK_ERR_BAD_SHAPE;
    if (M > INT32_MAX - 64 || K > INT32_MAX - 1024) return TK_ERR_TOO_LARGE;
    if (bm < 1 || bk < 1 || (bk < 8 ? 8 % bk != 0 : bk % 8 != 0)) return TK_ERR_BAD_GROUP;   // 1, 2, 4 or a multiple of 8 columns per scale
    if (bk < 8 && M * (K / 8) > INT32_MAX - 4 * kThreads) return TK_ERR_TOO_LARGE;
    if (M == 0) return TK_OK;
    if (!x || !x_sf || !out) return TK_ERR_NULL_POINTER;
    if (!aligned_to(x, x_fmt == TK_E4M3 ? 8 : 4) || !aligned_to(out, 16)) return TK_ERR_MISALIGNED;   // E5M6: 12-byte pieces of 4-byte words
    if (!aligned_to(x_sf, 4) || (x_sf_layout == TK_SF_COL_UE8M0 && x_sf_ld % 4 != 0)) return TK_ERR_MISALIGNED;
    const int64_t nm = (M + bm - 1) / bm, nk = (K + bk - 1) / bk;
    const int64_t need = x_sf_layout == TK_SF_ROW_F32 ? nk : (x_sf_layout == TK_SF_COL_F32 ? nm : 4 * nm);
    if (x_sf_ld < need) return TK_ERR_BAD_STRIDE;
    if (((M + 1) / 2) * ((K + kStripCols - 1) / kStripCols) > INT32_MAX - 8) return TK_ERR_TOO_LARGE;
    return TK_OK;
}

extern "C" int tk_cast_back(const void *x, int x_fmt, int64_t M, int64_t K, const void *x_sf, int64_t x_sf_ld,
                            int x_sf_layout, int bm, int bk, void *out, int out_dtype, void *stream) {
    const int rc = tk_check_cast_back(x, x_fmt, M, K, x_sf, x_sf_ld, x_sf_layout, bm, bk, out, out_dtype);
    if (rc != TK_OK || M == 0) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e;
    if (x_fmt == TK_E4M3)
        e = out_dtype == TK_F32 ? launch_cast_back<e4m3in_t, true>(x, out, x_sf, x_sf_ld, (int)M, (int)K, x_sf_layout, bm, bk, s)
                                : launch_cast_back<e4m3in_t, false>(x, out, x_sf, x_sf_ld, (int)M, (int)K, x_sf_layout, bm, bk, s);
    else if (x_fmt == TK_E2M1)
        e = out_dtype == TK_F32 ? launch_cast_back<e2m1in_t, true>(x, out, x_sf, x_sf_ld, (int)M, (int)K, x_sf_layout, bm, bk, s)
                                : launch_cast_back<e2m1in_t, false>(x, out, x_sf, x_sf_ld, (int)M, (int)K, x_sf_layout, bm, bk, s);
    else
        e = out_dtype == TK_F32 ? launch_cast_back<e5m6in_t, true>(x, out, x_sf, x_sf_ld, (int)M, (int)K, x_sf_layout, bm, bk, s)
                                : launch_cast_back<e5m6in_t, false>(x, out, x_sf, x_sf_ld, (int)M, (int)K, x_sf_layout, bm, bk, s);
    return (int)e;
}
