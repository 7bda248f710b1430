// Per-block (bm x bk, bm/bk in {32, 128}) block-scaled cast to E4M3 / E2M1 for gfx950.
//
// A workgroup owns one tile of 128 rows x TW columns (TW = 128 with 512 threads, or 512 with 1024 threads: see the
// table at the launch code), i.e. 1 to 64 scale blocks.  With TW = 128, thread (t, c) = (tid / 16, tid % 16) holds
// the 8 elements at columns 8c.. of rows t, t+32, t+64, t+96: four 16-byte streaming loads per thread (bf16), all
// issued up front; the tile stays in registers between the amax reduction and the conversion, so HBM is read once.  The amax of a block is
// reduced over the bk/8 lanes that share it with DPP, then across row slots and waves through one
// LDS exchange (a partial per 16-lane row, one barrier, vector reads).
//
// Reference semantics: tile_kernels/quant/per_block_cast_kernel.py:52-136.
#include "tk_device.hpp"
#include "tk_host.hpp"

namespace tk {

constexpr int kBlockTile = 128;
constexpr int kPerBlockThreads = 512, kWideTile = 512, kWideThreads = 1024;   // the two tile shapes: see the table at the launch code

struct PerBlockParams {
    const void *x;
    uint8_t *out;
    SfRef sf;
    int M, K;
    int tiles_m, tiles_k;
    int round_sf, mode;
};

// Parameters travel as individual scalars (16 dwords in all) so that they are preloaded into SGPRs
// at wave start (the library is built with -amdgpu-kernarg-preload-count=16).
#define TK_PB_KERNEL_ARGS                                                                                  \
    const void *a_x, uint8_t *a_out, void *a_sf, int64_t a_sf_ld, int a_M, int a_K, int a_tiles_m, int a_tiles_k, \
        int a_round_sf, int a_mode, int a_sf_layout, int a_nm, int a_nk
#define TK_PB_KERNEL_UNPACK \
    const PerBlockParams p{a_x, a_out, SfRef{a_sf, a_sf_ld, a_sf_layout, a_nm, a_nk}, a_M, a_K, a_tiles_m, a_tiles_k, a_round_sf, a_mode}
#define TK_PB_LAUNCH_ARGS(p) \
    (p).x, (p).out, (p).sf.base, (p).sf.ld, (p).M, (p).K, (p).tiles_m, (p).tiles_k, (p).round_sf, (p).mode, (p).sf.layout, (p).sf.nm, (p).sf.nk

// TW: columns of a tile (128, 256 or 512); a tile is 128 rows x TW columns.
// THREADS: threads per tile.
// FULL: the tile lies wholly inside the matrix, so no bounds checks are compiled in.
template <typename InT, int FMT, int BM, int BK, int TW, int THREADS, bool FULL>
__device__ __forceinline__ void per_block_cast_tile(const PerBlockParams &p) {
    constexpr int LPR = TW / 8;                                      // lanes along a row of the tile
    constexpr int SUBM = kBlockTile / BM, SUBK = TW / BK;            // scale blocks per tile
    constexpr int LPG = BK / 8;                                      // lanes sharing a block in one row
    constexpr int TR = THREADS / LPR;                                // rows covered by one pass of the workgroup
    constexpr int NI = kBlockTile / TR;                              // rows per thread
    constexpr int IPB = BM / TR;                                     // of which per scale block
    static_assert(IPB >= 1, "a pass of the workgroup must not span two scale blocks");
    // partial maxima: one per (scale block, 16-row slot of the workgroup); no atomics, no zeroing
    __shared__ __attribute__((aligned(16))) uint32_t part[SUBM][SUBK][TR];

    const int tile_m = blockIdx.y, tile_k = blockIdx.x;   // 2-D grid: no division on the way to the first load

    const int t = threadIdx.x / LPR, c = threadIdx.x % LPR;
    const int col = tile_k * TW + c * 8;
    const int bj = (c * 8) / BK;
    const bool col_ok = FULL || col < p.K;
    const int row0 = tile_m * kBlockTile + t;
    const InT *x = reinterpret_cast<const InT *>(p.x) + (int64_t)row0 * p.K + col;
    const int64_t out_ld = FMT == TK_E4M3 ? p.K : p.K / 2;

    // fp32 input: the LPR lanes of a tile row read its 32 * LPR bytes as two whole-line loads and deal them out through LDS
    constexpr int XB = Raw8<InT>::kXchgBytes;
    constexpr int RUN = LPR < 64 ? LPR : 64;     // lanes of one run: a tile row, or the part of it that one wave holds
    __shared__ __attribute__((aligned(16))) uint8_t xchg[XB ? THREADS * XB : 16];
    Raw8<InT> raw[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        if (FULL) raw[i].template load_run<RUN>(x + (int64_t)(TR * i) * p.K, c % RUN);
        else raw[i].load(x + (int64_t)(TR * i) * p.K, col_ok && row0 + TR * i < p.M);
        if (i + 1 < NI) vmem_issue_gap();
    }
    if constexpr (FULL && XB != 0) {
#pragma unroll
        for (int i = 0; i < NI; ++i) raw[i].template settle<RUN>(xchg + (threadIdx.x / RUN) * (RUN * XB), c % RUN);
    }

    float inv[SUBM];
    if (p.mode != TK_CAST_GIVEN_SF) {
#pragma unroll
        for (int b = 0; b < SUBM; ++b) {
            float m = 0.0f;
#pragma unroll
            for (int i = b * IPB; i < (b + 1) * IPB; ++i) {
                float v[8];
                raw[i].get(v);
                m = __builtin_fmaxf(m, absmax8(v));
            }
            m = group_allmax<LPG>(m);
            if ((c % LPG) == 0) part[b][bj][t] = f2u(m);
        }
        __syncthreads();
#pragma unroll
        for (int b = 0; b < SUBM; ++b) {
            uint32_t m = 0;
#pragma unroll
            for (int q = 0; q < TR; q += 4) {
                const u32x4 w = *reinterpret_cast<const u32x4 *>(&part[b][bj][q]);
                m = umax(umax(m, umax(w.x, w.y)), umax(w.z, w.w));
            }
            const Scale sc = make_scale<Fmt<FMT>::qmax>(u2f(m), Fmt<FMT>::floor_, p.round_sf != 0);
            inv[b] = sc.inv;
            // one thread per scale block stores it: the first row slot's first lane of the block
            if (t == 0 && (c % LPG) == 0) {
                const int mb = tile_m * SUBM + b, kb = tile_k * SUBK + bj;
                if (mb < p.sf.nm && kb < p.sf.nk) sf_store(p.sf, mb, kb, sc);
            }
        }
    } else {
#pragma unroll
        for (int b = 0; b < SUBM; ++b) {
            const int m = tile_m * SUBM + b, k = tile_k * SUBK + bj;
            const float s = (m < p.sf.nm && k < p.sf.nk) ? sf_load(p.sf, m, k) : 1.0f;
            inv[b] = 1.0f / s;
        }
    }
    if (p.mode == TK_SF_ONLY) return;

    // Wide tiles: the two lanes that hold 16 neighbouring columns exchange the codes of two row slots, so that each stores
    // 16 consecutive codes of one row with one instruction: half as many store instructions, each twice as wide.  A launch of
    // wide tiles fits the GPU in one round, all its workgroups finish loading at about the same time (measured: the last load
    // of every workgroup of [7168, 2048] arrives between 3.4 and 4.7 us after the start) and the rest of the launch is one
    // burst of stores, which drains faster in fewer, wider instructions: bf16 [7168, 2048] -> E4M3 8.54 -> 8.20 us,
    // [4096, 4096] 9.22 -> 8.66, [8192, 2048] 9.94 -> 9.07.  (128-column tiles, whose workgroups finish at different times so
    // that loads and stores overlap, do not gain: [8192, 4096] 17.43 -> 17.65 us.)
    constexpr bool PAIRED = FULL && TW == kWideTile && NI % 2 == 0;
    if constexpr (PAIRED) {
        const bool odd = threadIdx.x & 1;
#pragma unroll
        for (int i = 0; i < NI; i += 2) {
            float v[8];
            raw[i].get(v);
            const u32x2 a = p.mode == TK_CAST_GIVEN_SF ? quantise8<FMT, true>(v, inv[i / IPB]) : quantise8<FMT, false>(v, inv[i / IPB]);
            raw[i + 1].get(v);
            const u32x2 b = p.mode == TK_CAST_GIVEN_SF ? quantise8<FMT, true>(v, inv[(i + 1) / IPB]) : quantise8<FMT, false>(v, inv[(i + 1) / IPB]);
            // the even lane keeps slot i and takes its neighbour's half of it, the odd lane likewise with slot i + 1
            const u32x2 send = odd ? a : b;
            const u32x2 recv = {dpp_u32<kDppXor1>(send.x), FMT == TK_E4M3 ? dpp_u32<kDppXor1>(send.y) : 0u};
            const u32x2 lo = odd ? recv : a, hi = odd ? b : recv;
            uint8_t *out_row = p.out + (int64_t)(row0 + TR * (i + (odd ? 1 : 0))) * out_ld;
            if (FMT == TK_E4M3) st_stream16(out_row + (col & ~15), u32x4{lo.x, lo.y, hi.x, hi.y});
            else st_stream8(out_row + ((col & ~15) >> 1), u32x2{lo.x, hi.x});
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int row = row0 + TR * i;
        if (FULL || (col_ok && row < p.M)) {
            float v[8];
            raw[i].get(v);
            uint8_t *out_row = p.out + (int64_t)row * out_ld;
            if (p.mode == TK_CAST_GIVEN_SF) quantise_store8<FMT, true>(v, inv[i / IPB], out_row, col);
            else quantise_store8<FMT, false>(v, inv[i / IPB], out_row, col);
        }
    }
}

// FULL_GRID: M and K are multiples of 128.  Otherwise only the tiles on the lower and right edges take the
// bounds-checked path; the choice is uniform over the workgroup.  (With every tile checked, bf16 [32767, 4096] took
// 63.9 us against 59.1 us for [32768, 4096].)
template <typename InT, int FMT, int BM, int BK, int TW, int THREADS, bool FULL_GRID>
__global__ __launch_bounds__(THREADS) void per_block_cast_kernel(TK_PB_KERNEL_ARGS) {
    TK_PB_KERNEL_UNPACK;
    if constexpr (FULL_GRID) {
        per_block_cast_tile<InT, FMT, BM, BK, TW, THREADS, true>(p);
    } else {
        if (((int)blockIdx.y + 1) * kBlockTile <= p.M && ((int)blockIdx.x + 1) * TW <= p.K)
            per_block_cast_tile<InT, FMT, BM, BK, TW, THREADS, true>(p);
        else
            per_block_cast_tile<InT, FMT, BM, BK, TW, THREADS, false>(p);
    }
}

// Tile shapes, measured on MI355X for bf16 -> E4M3 128x128 (us per call):
//                                          [2048,2048]  [7168,2048]  [4096,4096]  [4096,7168]  [8192,4096]  [16384,7168]
//   128 x 128, 512 threads (4 rows/thread)     4.07         9.13        10.02        15.58        17.46        52.1
//   128 x 512, 1024 threads (8 rows/thread)    6.02         8.60         9.19        16.36        18.45
//   128 x 512, 512 threads (16 rows/thread)    6.31         8.87         9.82        16.59        20.37        58.8
//   128 x 256, 1024 threads                    4.72         9.30        10.57        16.39        18.06
// (128 x 128 with 256 threads: 9.4 at [7168,2048], with 1024: 9.8.)  A wave of a 512-column tile reads 1 KB of one
// row per load instruction instead of 256 bytes of four rows, which pays while the matrix has too few 128 x 128
// tiles to fill the GPU several times over (here 896 and 1024 tiles: 3.5 and 4 workgroups per CU) and costs where it
// has many, or so few that whole CUs would stay empty.  The wide tile is used inside that window (with the paired
// 16-byte stores: [7168,2048] 8.24).  fp32 input, same window: [7168,2048] 13.58 -> 12.31, [8192,4096] 30.16 -> 29.96.
constexpr int64_t kWideMinTiles = 512, kWideMaxTiles = 1280;     // in 128 x 128 tiles

template <typename InT, int FMT, int BM, int BK, int TW, int THREADS>
static void launch_per_block_3(const PerBlockParams &p, hipStream_t stream) {
    const dim3 grid((unsigned)((p.K + TW - 1) / TW), (unsigned)p.tiles_m), block(THREADS);
    if (p.M % kBlockTile == 0 && p.K % TW == 0)
        hipLaunchKernelGGL((per_block_cast_kernel<InT, FMT, BM, BK, TW, THREADS, true>), grid, block, 0, stream, TK_PB_LAUNCH_ARGS(p));
    else
        hipLaunchKernelGGL((per_block_cast_kernel<InT, FMT, BM, BK, TW, THREADS, false>), grid, block, 0, stream, TK_PB_LAUNCH_ARGS(p));
}

template <typename InT, int FMT, int BM, int BK>
static void launch_per_block_2(const PerBlockParams &p, hipStream_t stream) {
    const int64_t tiles = (int64_t)p.tiles_m * p.tiles_k;
    if (p.K % kWideTile == 0 && tiles >= kWideMinTiles && tiles <= kWideMaxTiles)
        launch_per_block_3<InT, FMT, BM, BK, kWideTile, kWideThreads>(p, stream);
    else
        launch_per_block_3<InT, FMT, BM, BK, kBlockTile, kPerBlockThreads>(p, stream);
}

template <typename InT, int FMT>
static hipError_t launch_per_block(const PerBlockParams &p, int bm, int bk, hipStream_t stream) {
    if (bm == 128 && bk == 128) launch_per_block_2<InT, FMT, 128, 128>(p, stream);
    else if (bm == 32 && bk == 32) launch_per_block_2<InT, FMT, 32, 32>(p, stream);
    else if (bm == 128 && bk == 32) launch_per_block_2<InT, FMT, 128, 32>(p, stream);
    else launch_per_block_2<InT, FMT, 32, 128>(p, stream);
    return hipGetLastError();
}

}  // namespace tk

using namespace tk;

extern "C" int tk_check_per_block_cast(const void *x, int x_dtype, int64_t M, int64_t K, const void *out,
                                       const void *sf, int64_t sf_ld, int fmt, int bm, int bk, int sf_layout,
                                       int round_sf, int mode) {
    if (x_dtype != TK_BF16 && x_dtype != TK_F32) return TK_ERR_BAD_DTYPE;
    if (fmt != TK_E4M3 && fmt != TK_E2M1) return TK_ERR_BAD_FORMAT;
    if (mode < TK_CAST_AND_SF || mode > TK_CAST_GIVEN_SF) return TK_ERR_BAD_MODE;
    if (sf_layout < TK_SF_ROW_F32 || sf_layout > TK_SF_COL_UE8M0) return TK_ERR_BAD_LAYOUT;
    if (mode == TK_CAST_GIVEN_SF && sf_layout != TK_SF_ROW_F32) return TK_ERR_BAD_LAYOUT;
    if (sf_layout == TK_SF_COL_UE8M0 && !round_sf) return TK_ERR_BAD_LAYOUT;
    if ((bm != 32 && bm != 128) || (bk != 32 && bk != 128)) return TK_ERR_BAD_GROUP;
    if (M < 0 || K <= 0 || K % 64 != 0) return TK_ERR_BAD_SHAPE;
    if (M > INT32_MAX - 256 || K > INT32_MAX - 256) return TK_ERR_TOO_LARGE;
    if (M == 0) return TK_OK;
    if (!x || !sf || (mode != TK_SF_ONLY && !out)) return TK_ERR_NULL_POINTER;
    if (!aligned_to(x, 16) || (mode != TK_SF_ONLY && !aligned_to(out, 8)) || !aligned_to(sf, 4)) return TK_ERR_MISALIGNED;
    const int64_t nm = (M + bm - 1) / bm, nk = (K + bk - 1) / bk;
    const int64_t need = sf_layout == TK_SF_ROW_F32 ? nk : (sf_layout == TK_SF_COL_F32 ? nm : 4 * nm);
    if (sf_ld < need) return TK_ERR_BAD_STRIDE;
    const int64_t tiles = ((M + kBlockTile - 1) / kBlockTile) * ((K + kBlockTile - 1) / kBlockTile);
    if (tiles > INT32_MAX - 8 || (M + kBlockTile - 1) / kBlockTile > 65535) return TK_ERR_TOO_LARGE;   // row tiles ride on grid.y
    return TK_OK;
}

extern "C" int tk_per_block_cast(const void *x, int x_dtype, int64_t M, int64_t K, void *out, void *sf,
                                 int64_t sf_ld, int fmt, int bm, int bk, int sf_layout, int round_sf, int mode,
                                 void *stream) {
    const int rc = tk_check_per_block_cast(x, x_dtype, M, K, out, sf, sf_ld, fmt, bm, bk, sf_layout, round_sf, mode);
    if (rc != TK_OK || M == 0) return rc;
    PerBlockParams p;
    p.x = x;
    p.out = static_cast<uint8_t *>(out);
    p.sf = SfRef{sf, sf_ld, sf_layout, (int)((M + bm - 1) / bm), (int)((K + bk - 1) / bk)};
    p.M = (int)M;
    p.K = (int)K;
    p.tiles_m = (int)((M + kBlockTile - 1) / kBlockTile);
    p.tiles_k = (int)((K + kBlockTile - 1) / kBlockTile);
    p.round_sf = round_sf;
    p.mode = mode;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e;
    if (x_dtype == TK_BF16)
        e = fmt == TK_E4M3 ? launch_per_block<bf16_t, TK_E4M3>(p, bm, bk, s) : launch_per_block<bf16_t, TK_E2M1>(p, bm, bk, s);
    else
        e = fmt == TK_E4M3 ? launch_per_block<float, TK_E4M3>(p, bm, bk, s) : launch_per_block<float, TK_E2M1>(p, bm, bk, s);
    return (int)e;
}
