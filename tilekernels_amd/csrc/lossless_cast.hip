// Lossless re-blocking of packed FP4 E2M1 codes (power-of-two scales per small block, e.g. 1 x 32) into FP8 E4M3
// codes with power-of-two scales per larger block (1 x 128, 32 x 32, 128 x 128, ...) for gfx950.
//
// Nothing is rounded.  An output block takes the exponent  e_out = max(e_in over its input blocks) - 6  (not below
// 0), and every value becomes  code * 2^(e_in - e_out): an E2M1 magnitude (0.5 .. 6, one mantissa bit) shifted by
// at most 6 binades up stays at or below 384 <= 448, and shifted down by at most 5 stays a normal E4M3 number, so
// E4M3 holds it exactly as long as the input exponents of one output block differ by no more than 11.  Beyond that
// the reference asserts (tile_kernels/quant/per_block_cast_lossless_kernel.py:126); here the small values are
// rounded by the conversion like any other (to +-0 once they are 127 or more binades below the output exponent).
//
// A workgroup of 512 threads owns a 128 x 256 tile (every supported output block divides 128 x 128): a lane takes 16
// consecutive codes (8 bytes; 8 codes where a block is narrower than 16 columns) of rows r, r + 32, ..., 4 in all, each
// with the exponent of its input block.  The exponent maxima of the output blocks are formed along the rows with DPP (a
// tile row is one DPP row of 16 lanes), down a lane's own rows in registers, and across lanes and waves with a few
// integer atomics on a small LDS table; then every lane shifts, converts and stores 16 bytes per row, and the first
// threads store the tile's output scales.
//
// Reference semantics: tile_kernels/quant/per_block_cast_lossless_kernel.py:15-147 (kernel) and :150-209 (wrapper).
#include <type_traits>

#include "tk_device.hpp"
#include "tk_host.hpp"

namespace tk {

constexpr int kLlTile = 128;                            // rows per tile; also the largest output block extent
constexpr int kLlTileK = 256;                           // columns per tile: a tile row is 128 bytes of codes, one whole cache line
                                                        // (with 128 columns, two workgroups fetched each line: 2.0 x the reads)
constexpr int kLlThreads = 512;

// CODES: codes per lane and row, 8 (a 4-byte load, an 8-byte store) or 16 (8 and 16 bytes: half the memory
// instructions; needs input and output blocks at least 16 columns wide, so that a lane's codes share one input scale
// and one output block).  Measured on MI355X, E2M1 1 x 32 -> E4M3 128 x 128: [7168, 2048] 6.3 us with 8, 5.2 us with 16
// (at [32768, 4096] both take 44 us).
template <int CODES>
__global__ __launch_bounds__(kLlThreads) void lossless_fp4_to_fp8_kernel(const uint8_t *x, void *a_xsf, int64_t a_xsf_ld, int M, int K,
                                                                       int a_xsf_layout, int ibm_sh, int ibk_sh, int obm_sh, int obk_sh,
                                                                       uint8_t *out, void *a_sf, int64_t a_sf_ld, int a_sf_layout,
                                                                       int in_nm, int in_nk, int out_nm, int out_nk) {
    constexpr int kPieces = kLlTileK / CODES;           // pieces per tile row = lanes per row: 32 (two DPP rows) or 16 (one)
    constexpr int kRowsPerPass = kLlThreads / kPieces;  // 16 or 32
    constexpr int kPasses = kLlTile / kRowsPerPass;     // rows per lane: 8 or 4
    constexpr int kCodesSh = CODES == 8 ? 3 : 4;
    typedef typename std::conditional<CODES == 8, uint32_t, u32x2>::type Codes;
    const SfRef xsf{a_xsf, a_xsf_ld, a_xsf_layout, in_nm, in_nk};
    const SfRef sf{a_sf, a_sf_ld, a_sf_layout, out_nm, out_nk};
    __shared__ int32_t blk_max[kLlTile][kLlTileK / 8];   // [output block row][output block column] of the tile; at most 128 x 32 used
    const int tile_m = blockIdx.y, tile_k = blockIdx.x;
    const int piece = threadIdx.x % kPieces, r0 = threadIdx.x / kPieces;
    const int col = tile_k * kLlTileK + piece * CODES;
    const bool col_ok = col < K;
    // every block extent is a power of two (the output blocks divide 128, the input blocks divide them): shifts, no divisions
    const int bcols_sh = 8 - obk_sh, bcols = 1 << bcols_sh, brows = kLlTile >> obm_sh;   // output blocks of a tile along the columns / rows
    const int lpb_sh = obk_sh - kCodesSh, lanes_per_block = 1 << lpb_sh;   // pieces of a row inside one output block: 1 .. 16
    const int bk_idx = piece >> lpb_sh;

    for (int i = threadIdx.x; i < brows * bcols; i += kLlThreads) blk_max[i >> bcols_sh][i & (bcols - 1)] = 0;

    // All loads first, without a branch around them (a branch per row makes the compiler finish one row's loads
    // before it issues the next): rows and columns outside the matrix read the tile's first element and count as 0.
    Codes code[kPasses];
    int e_in[kPasses];
    const int row_first = tile_m * kLlTile, col_first = tile_k * kLlTileK;
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
        const int row = row_first + p * kRowsPerPass + r0;
        const bool ok = col_ok && row < M;
        const int rr = ok ? row : row_first, cc = ok ? col : col_first;
        code[p] = __builtin_nontemporal_load(reinterpret_cast<const Codes *>(x + (((int64_t)rr * K + cc) >> 1)));
        vmem_issue_gap();
        e_in[p] = (int)(f2u(sf_load_select(xsf, rr >> ibm_sh, cc >> ibk_sh)) >> 23);
        if (!ok) { code[p] = Codes{}; e_in[p] = 0; }
    }

    __syncthreads();
    // Block maxima.  Along a row: 16 lanes (one DPP row) cover the widest output block (128 columns) or more, so the lanes
    // that share an output block reduce without LDS.  Down the rows: a lane folds its own consecutive rows while they stay in
    // one block, and only then does the first lane of each group touch the LDS table (a few atomics per 128 x 128 block, not 2048).
    uint32_t run = 0u;
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
        uint32_t m = (uint32_t)e_in[p];
        if (lanes_per_block >= 2) m = umax(m, dpp_u32<kDppXor1>(m));
        if (lanes_per_block >= 4) m = umax(m, dpp_u32<kDppXor2>(m));
        if (lanes_per_block >= 8) m = umax(m, dpp_u32<kDppHalfMirror>(m));
        if (lanes_per_block >= 16) m = umax(m, dpp_u32<kDppMirror>(m));
        run = umax(run, m);
        const int br = (p * kRowsPerPass + r0) >> obm_sh;
        const int br_next = p + 1 < kPasses ? ((p + 1) * kRowsPerPass + r0) >> obm_sh : -1;
        if (br != br_next) {
            if ((piece & (lanes_per_block - 1)) == 0 && run != 0u) atomicMax(&blk_max[br][bk_idx], (int32_t)run);
            run = 0u;
        }
    }
    __syncthreads();

#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
        const int row_in_tile = p * kRowsPerPass + r0;
        const int row = tile_m * kLlTile + row_in_tile;
        if (!(col_ok && row < M)) continue;
        const int top = blk_max[row_in_tile >> obm_sh][bk_idx];
        const int e_out = top >= 6 ? top - 6 : 0;
        // 2^(e_in - e_out) as a float: biased exponent e_in - e_out + 127.  Input exponents 127 or more below the
        // output's give 0 (such values are far below the smallest E4M3 step and become +-0, as with any scale below
        // 2^-126; the reference asserts that a block's exponents lie within its range instead)
        const int biased = e_in[p] - e_out + 127;
        const float scale = u2f((uint32_t)(biased > 0 ? biased : 0) << 23);
        if constexpr (CODES == 8) {
            Raw8<e2m1in_t> raw;
            raw.w = code[p];
            raw.s = scale;
            float v[8];
            raw.get(v);
            st_stream8(out + (int64_t)row * K + col, pack_e4m3x8<false>(v));
        } else {
            Raw8<e2m1in_t> lo, hi;
            lo.w = code[p].x;
            hi.w = code[p].y;
            lo.s = hi.s = scale;
            float v[8], w[8];
            lo.get(v);
            hi.get(w);
            const u32x2 a = pack_e4m3x8<false>(v), b = pack_e4m3x8<false>(w);
            __builtin_nontemporal_store(u32x4{a.x, a.y, b.x, b.y}, reinterpret_cast<u32x4 *>(out + (int64_t)row * K + col));
        }
    }

    for (int i = threadIdx.x; i < brows * bcols; i += kLlThreads) {
        const int bm_i = i >> bcols_sh, bk_i = i & (bcols - 1);
        const int m = tile_m * brows + bm_i, k = tile_k * bcols + bk_i;
        if (m < out_nm && k < out_nk) {
            const int top = blk_max[bm_i][bk_i];
            Scale sc;
            sc.e8 = (uint32_t)(top >= 6 ? top - 6 : 0);
            sc.sf = u2f(sc.e8 << 23);
            sc.inv = 0.0f;
            sf_store(sf, m, k, sc);
        }
    }
}

}  // namespace tk

using namespace tk;

extern "C" int tk_check_per_block_cast_lossless(const void *x, int64_t M, int64_t K, const void *x_sf, int64_t x_sf_ld,
                                                int x_sf_layout, int x_bm, int x_bk, const void *out, const void *out_sf,
                                                int64_t out_sf_ld, int out_sf_layout, int out_bm, int out_bk) {
    if (x_sf_layout < TK_SF_ROW_F32 || x_sf_layout > TK_SF_COL_UE8M0) return TK_ERR_BAD_LAYOUT;
    if (out_sf_layout < TK_SF_ROW_F32 || out_sf_layout > TK_SF_COL_UE8M0) return TK_ERR_BAD_LAYOUT;
    if (M < 0 || K <= 0 || K % 8 != 0) return TK_ERR_BAD_SHAPE;
    if (M > INT32_MAX - 256 || K > INT32_MAX - 256) return TK_ERR_TOO_LARGE;
    if (x_bm < 1 || x_bk < 8 || x_bk % 8 != 0) return TK_ERR_BAD_GROUP;
    // output blocks divide the 128 x 128 tile, hold whole 8-code pieces and whole input blocks
    if (out_bm < 1 || out_bk < 8 || kLlTile % out_bm != 0 || kLlTile % out_bk != 0 || out_bk % 8 != 0) return TK_ERR_BAD_GROUP;
    if (out_bm % x_bm != 0 || out_bk % x_bk != 0) return TK_ERR_BAD_GROUP;
    if (M == 0) return TK_OK;
    if (!x || !x_sf || !out || !out_sf) return TK_ERR_NULL_POINTER;
    if (!aligned_to(x, 4) || !aligned_to(out, 8) || !aligned_to(x_sf, 4) || !aligned_to(out_sf, 4)) return TK_ERR_MISALIGNED;
    const int64_t inm = (M + x_bm - 1) / x_bm, ink = (K + x_bk - 1) / x_bk;
    const int64_t onm = (M + out_bm - 1) / out_bm, onk = (K + out_bk - 1) / out_bk;
    const int64_t xneed = x_sf_layout == TK_SF_ROW_F32 ? ink : (x_sf_layout == TK_SF_COL_F32 ? inm : 4 * inm);
    const int64_t oneed = out_sf_layout == TK_SF_ROW_F32 ? onk : (out_sf_layout == TK_SF_COL_F32 ? onm : 4 * onm);
    if (x_sf_ld < xneed || out_sf_ld < oneed) return TK_ERR_BAD_STRIDE;
    if (out_sf_layout == TK_SF_COL_UE8M0 && out_sf_ld % 4 != 0) return TK_ERR_MISALIGNED;
    if ((M + kLlTile - 1) / kLlTile > 65535) return TK_ERR_TOO_LARGE;   // row tiles ride on grid.y
    return TK_OK;
}

extern "C" int tk_per_block_cast_lossless(const void *x, int64_t M, int64_t K, const void *x_sf, int64_t x_sf_ld, int x_sf_layout,
                                          int x_bm, int x_bk, void *out, void *out_sf, int64_t out_sf_ld, int out_sf_layout,
                                          int out_bm, int out_bk, void *stream) {
    const int rc = tk_check_per_block_cast_lossless(x, M, K, x_sf, x_sf_ld, x_sf_layout, x_bm, x_bk, out, out_sf, out_sf_ld,
                                                    out_sf_layout, out_bm, out_bk);
    if (rc != TK_OK || M == 0) return rc;
    const dim3 grid((unsigned)((K + kLlTileK - 1) / kLlTileK), (unsigned)((M + kLlTile - 1) / kLlTile));
    auto log2i = [](int v) { int s = 0; while ((1 << s) < v) ++s; return s; };
#define TK_LL_LAUNCH(CODES)                                                                                                          \
    hipLaunchKernelGGL(lossless_fp4_to_fp8_kernel<CODES>, grid, dim3(kLlThreads), 0, static_cast<hipStream_t>(stream),                  \
                       static_cast<const uint8_t *>(x), const_cast<void *>(x_sf), x_sf_ld, (int)M, (int)K, x_sf_layout, log2i(x_bm),     \
                       log2i(x_bk), log2i(out_bm), log2i(out_bk), static_cast<uint8_t *>(out), out_sf, out_sf_ld, out_sf_layout,          \
                       (int)((M + x_bm - 1) / x_bm), (int)((K + x_bk - 1) / x_bk), (int)((M + out_bm - 1) / out_bm),                     \
                       (int)((K + out_bk - 1) / out_bk))
    // 16 codes per lane need K and the column extents of the blocks to be multiples of 16, and 16-byte aligned output rows
    if (K % 16 == 0 && x_bk % 16 == 0 && out_bk % 16 == 0 && aligned_to(x, 8) && aligned_to(out, 16)) TK_LL_LAUNCH(16);
    else TK_LL_LAUNCH(8);
#undef TK_LL_LAUNCH
    return (int)hipGetLastError();
}
