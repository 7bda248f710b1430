// Per-token (1 x G) block-scaled cast to E4M3 / E2M1 for gfx950.
//
// Work decomposition: a workgroup of 4 waves owns a tile of 4*RPW rows x 512 columns.  Each wave
// takes RPW rows; in every row its 64 lanes cover 512 consecutive elements with one 16-byte (bf16)
// or two 16-byte (fp32) streaming loads per lane, all rows' loads issued before the first use.  A
// group of G elements therefore lives in G/8 neighbouring lanes of one DPP row and its amax needs
// no LDS.  The divisions that turn an amax into a scale are shared out over the lanes of a group
// (one row each) instead of being repeated by all of them.  Row-major scales are stored straight
// from the lanes that computed them; column-major layouts are staged in LDS and written out
// transposed so that neighbouring lanes fill one contiguous segment.
//
// Reference semantics: tile_kernels/quant/per_token_cast_kernel.py:65-154 (plain-tensor branch),
// tile_kernels/quant/common.py:196-244.
#include <type_traits>

#include "tk_device.hpp"
#include "tk_host.hpp"

namespace tk {

struct PerTokenParams {
    const void *x;
    uint8_t *out;
    SfRef sf;
    int64_t x_ld;     // (logical) elements between rows of x
    int M, K;
    int geom;         // wide tiles: waves per tile (grid: x = column tile, y and z = row tile); else column tiles (1-D grid)
    int round_sf, mode;
    SfRef xsf;        // quantised input only: its block scales ...
    int in_bm, in_bk; // ... and their block shape
};

// Parameters travel as individual scalars (16 dwords in all) so that they are preloaded into SGPRs
// at wave start (the library is built with -amdgpu-kernarg-preload-count=16).
// Arguments in the order they are needed: the first 14 dwords arrive preloaded in SGPRs and hold all that
// the input addresses (codes and, for a quantised input, its scales) are made of; the others are fetched
// from the argument buffer while the loads are in flight.
#define TK_PT_KERNEL_ARGS                                                                                          \
    const void *a_x, int64_t a_x_ld, void *a_xsf, int64_t a_xsf_ld, int a_M, int a_K, int a_geom, int a_xsf_layout,  \
        int a_in_bm, int a_in_bk, uint8_t *a_out, void *a_sf, int64_t a_sf_ld, int a_round_sf, int a_mode,           \
        int a_sf_layout, int a_nk, int a_xsf_nm, int a_xsf_nk
#define TK_PT_KERNEL_UNPACK                                                                                          \
    const PerTokenParams p{a_x, a_out, SfRef{a_sf, a_sf_ld, a_sf_layout, a_M, a_nk}, a_x_ld, a_M, a_K, a_geom,   \
                           a_round_sf, a_mode, SfRef{a_xsf, a_xsf_ld, a_xsf_layout, a_xsf_nm, a_xsf_nk}, a_in_bm, a_in_bk}
#define TK_PT_LAUNCH_ARGS(p)                                                                                        \
    (p).x, (p).x_ld, (p).xsf.base, (p).xsf.ld, (p).M, (p).K, (p).geom, (p).xsf.layout, (p).in_bm, (p).in_bk, (p).out, \
        (p).sf.base, (p).sf.ld, (p).round_sf, (p).mode, (p).sf.layout, (p).sf.nk, (p).xsf.nm, (p).xsf.nk

// Tile shapes (RPW = pieces of 8 elements per lane, i.e. of 512 columns per wave):
//   T_WIDE    (row-major scales):      RPW rows x (W*512) columns, W = blockDim.x/64 waves side by side on the same rows;
//             the tile's scales are RPW contiguous runs, staged in LDS and stored as whole segments
//   T_STACKED (column-major layouts, and row lengths whose strips do not split evenly over 3..8 waves):  4*RPW rows x 512
//             columns, the 4 waves stacked;
//             the staged scales are stored transposed, 4*RPW rows per contiguous segment (row-major: one short run per row)
//   T_ROWWISE (row-major scales, K a multiple of RPW*512): 4 rows x (RPW*512) columns, one row per
//             wave; the scales a wave produces are neighbours in the scale row and it stores them itself: no LDS
//             stage and no barrier
// FULL_GRID: the tile grid covers the matrix exactly, so no bounds checks are compiled in.
enum { T_STACKED = 0, T_WIDE = 1, T_ROWWISE = 2 };

// Waves per workgroup of the row-wise tiles (their waves share nothing, so this only sets how many rows are dispatched
// and retired together).  Measured on MI355X, us per call with 4 / 2 / 1 waves, 1 x 128 groups, row-major scales:
//   fp32 -> E4M3 [8192, 7168] 44.8 / 44.6 / 44.3, [16384, 4096] 51.4 / 50.0 / 50.5, [4096, 4096] 14.26 / 14.15 / 14.11;
//   fp32 -> E2M1 [8192, 7168] 41.6 / 41.8 / 40.6, [16384, 4096] 48.0 / 47.0 / 46.0, [4096, 4096] 13.7 / 13.3 / 13.1;
//   bf16 -> E2M1 [8192, 4096] 14.5 / 13.95 / 16.2, [4096, 7168] 13.0 / 12.7 / 14.6, [32768, 4096] 49.8 / 49.3 / 58.0, [65536, 2048] 49.5 / 48.8 / 58.0;
//   bf16 -> E4M3 [16384, 7168] 50.3 / 50.3 / 52.0, [32768, 4096] 56.95 / 57.3 / 59.1, [4096, 7168] 14.9 / 14.8 / 16.6 - 17.5.
template <typename InT, int FMT> constexpr int rowwise_waves() {
    return Elem<InT>::quantised ? kWaves : (sizeof(InT) == 4 ? 1 : (FMT == TK_E2M1 ? 2 : kWaves));
}

template <typename InT, int G, int FMT, int RPW, int TILE, bool FULL_GRID, bool GIVEN = false>
__global__ __launch_bounds__(TILE == T_WIDE ? 64 * kMaxWideWaves : kThreads) void per_token_cast_kernel(TK_PT_KERNEL_ARGS) {
    TK_PT_KERNEL_UNPACK;
    // GIVEN: the cast with caller-supplied scales, chosen at the launch (row-wise tiles).  The mode argument lies beyond the
    // preloaded ones; read at run time, the scale loads wait for that fetch: bf16 [4096, 7168] 15.6 us, 14.7 us this way.
    const int mode = GIVEN ? (int)TK_CAST_GIVEN_SF : p.mode;
    constexpr bool WIDE = TILE == T_WIDE, ROWW = TILE == T_ROWWISE;
    // row-wise tiles always fit the columns, and their waves share nothing: on a grid that overhangs the last row the
    // waves beyond it leave at once and the others run without bounds checks, like on an exact grid
    constexpr bool FULL = FULL_GRID || ROWW;
    constexpr int LPG = G / 8;            // lanes per group
    constexpr int GPS = kStripCols / G;   // groups per 512-column strip
    constexpr int ROWS = WIDE ? RPW : kWaves * RPW;       // rows per tile (stacked and wide)
    constexpr int SGPR = WIDE ? kMaxWideWaves * GPS : GPS;   // staged groups per row (capacity)
    // everything on the way to the first load comes from the preloaded arguments and the workgroup ids
    const int nwaves = WIDE ? p.geom : kWaves;
    using RS = RowScales<Fmt<FMT>::qmax, RPW, LPG>;
    __shared__ uint32_t stage[ROWW ? 1 : ROWS][ROWW ? 1 : SGPR];
    // fp32 input: a wave's 2 KB of one row arrive as two whole-line loads and are dealt out to their lanes through LDS
    constexpr int XB = Raw8<InT>::kXchgBytes;
    __shared__ __attribute__((aligned(16))) uint8_t xchg[XB ? (WIDE ? kMaxWideWaves : kWaves) : 1][XB ? 64 * XB : 16];

    // wide tiles: the waves of one tile cover a whole row; row-wise: one wave does
    const bool one_col = (ROWW ? RPW : p.geom) * kStripCols >= p.K;
    const int tile_m = (WIDE || ROWW) ? tile_grid_row(one_col) : (int)blockIdx.x / p.geom;
    const int tile_k = (WIDE || ROWW) ? tile_grid_col(one_col) : (int)blockIdx.x - tile_m * p.geom;
    const int lane = threadIdx.x & 63, wave = wave_id();
    // piece r of the wave: row `row0 + (ROWW ? 0 : r)`, columns from `col + (ROWW ? r * 512 : 0)`
    const int strip = WIDE ? tile_k * nwaves + wave : (ROWW ? tile_k * RPW : tile_k);
    const int col = strip * kStripCols + lane * 8;
    const int g_in_strip = lane / LPG;
    const int kgrp = strip * GPS + g_in_strip;
    const bool col_ok = FULL || col < p.K;
    const int srow = WIDE ? 0 : wave * RPW;                // first staged row of this wave
    const int row0 = ROWW ? tile_m * rowwise_waves<InT, FMT>() + wave : tile_m * ROWS + srow;
    if constexpr (ROWW && !FULL_GRID) {
        if (row0 >= p.M) return;
    }
    const int64_t out_ld = FMT == TK_E4M3 ? p.K : p.K / 2;
    constexpr int kRowStep = ROWW ? 0 : 1, kColStep = ROWW ? kStripCols : 0, kGrpStep = ROWW ? GPS : 0;

    Raw8<InT> raw[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        const void *xp = elem_ptr<InT>(p.x, row0 + r * kRowStep, p.x_ld, col + r * kColStep);
        // no branch around a load (the loads of the wave's rows then go out together): a lane beyond the last row or
        // column reads the first bytes of the matrix, and the first scale, and is cleared by value once all loads are out
        // (clearing a register that a load is still to fill means waiting for that load)
        const bool ok = col_ok && (FULL || row0 + r < p.M);
        if (FULL) raw[r].template load_run<64>(xp, lane);
        else raw[r].load(ok ? xp : p.x);
        if (r + 1 < RPW) vmem_issue_gap();
        if constexpr (Elem<InT>::quantised) {
            // the 8 codes of a lane share one input scale (input blocks are at least 32 columns wide)
            raw[r].s = sf_load(p.xsf, ok ? (row0 + r * kRowStep) / p.in_bm : 0, ok ? (col + r * kColStep) / p.in_bk : 0);
            vmem_issue_gap();
        }
    }
    if constexpr (!FULL || Elem<InT>::quantised) {
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const bool ok = col_ok && (FULL || row0 + r < p.M);
            if (!FULL && !ok) raw[r].zero();
            if constexpr (Elem<InT>::quantised) {
                if (!ok) raw[r].s = 0.0f;
            }
        }
    }

    if constexpr (FULL && XB != 0) {
#pragma unroll
        for (int r = 0; r < RPW; ++r) raw[r].template settle<64>(xchg[wave], lane);
    }

    float inv[RPW];
    if (mode == TK_CAST_GIVEN_SF) {
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const bool ok = col_ok && (FULL || row0 + r < p.M);
            inv[r] = 1.0f / (ok ? sf_load_select(p.sf, row0 + r * kRowStep, kgrp + r * kGrpStep) : 1.0f);
        }
    } else {
        float amax[RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            float v[8];
            raw[r].get(v);
            amax[r] = group_allmax<LPG>(absmax8(v));
        }
        RS rs;
        rs.compute(amax, Fmt<FMT>::floor_, p.round_sf != 0, lane);
#pragma unroll
        for (int r = 0; r < RPW; ++r) inv[r] = rs.inv[r];
        // lane j (< A) of a group computed the scale of piece c*A + j
        const int own = lane % LPG;
        if (own < RS::A) {
#pragma unroll
            for (int c = 0; c < RS::NC; ++c) {
                if constexpr (ROWW) {
                    // group g_in_strip of piece c*A + own: the wave's scales form one run of RPW * GPS floats
                    st_stream4(reinterpret_cast<float *>(p.sf.base) + (int64_t)row0 * p.sf.ld + kgrp + (c * RS::A + own) * GPS, f2u(rs.own[c].sf));
                } else {
                    stage[srow + c * RS::A + own][(WIDE ? wave * GPS : 0) + g_in_strip] =
                        p.sf.layout == TK_SF_COL_UE8M0 ? rs.own[c].e8 : f2u(rs.own[c].sf);
                }
            }
        }
    }
    if (mode != TK_SF_ONLY) {
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            if (col_ok && (FULL || row0 + r < p.M)) {
                float v[8];
                raw[r].get(v);
                uint8_t *out_row = p.out + (int64_t)(row0 + r * kRowStep) * out_ld;
                if (mode == TK_CAST_GIVEN_SF) quantise_store8<FMT, true>(v, inv[r], out_row, col + r * kColStep);
                else quantise_store8<FMT, false>(v, inv[r], out_row, col + r * kColStep);
            }
        }
    }
    if constexpr (!ROWW) {
        if (mode != TK_CAST_GIVEN_SF) {
            __syncthreads();
            if (WIDE) sf_store_tile_rowmajor<ROWS, SGPR>(p.sf, stage, nwaves * GPS, tile_m * ROWS, tile_k * nwaves * GPS);
            else if (p.sf.layout == TK_SF_ROW_F32) sf_store_tile_rowmajor<ROWS, SGPR>(p.sf, stage, GPS, tile_m * ROWS, tile_k * GPS);
            else sf_store_tile_colmajor<ROWS, SGPR>(p.sf, stage, tile_m * ROWS, tile_k * SGPR);
        }
    }
}

// E4M3 input with block scales -> E2M1, row-major output scales, K a multiple of RPW * 1024: one row per wave, a lane
// taking 16 consecutive codes (one 16-byte load) of each of its RPW pieces of 1024 columns and writing their 16
// output codes with one 8-byte store.  With 8 codes per lane, as in the kernel above, a wave's load instruction
// moves 512 bytes and its store 256.  Measured on MI355X, 1 x 128 -> E2M1 1 x 32 (us per call, 8 / 16 codes per
// lane): [8192, 4096] 12.0 / 10.9, [32768, 4096] 39.7 / 36.2, [16384, 8192] 39.6 / 35.1; with 4 pieces per wave
// instead of 2: 11.4, 35.3, 34.1.  (E4M3 output, whose stores are 8 bytes per lane already, did not gain: [32768, 4096]
// 43.5 -> 44.6.)  A group of G columns lives in G / 16 neighbouring lanes; the 16 codes of a lane share one input
// scale (input blocks are multiples of 16 columns wide here).  Waves share nothing: no LDS, no barrier.
template <int G, int RPW, bool FULL_GRID>
__global__ __launch_bounds__(kThreads) void per_token_cast_q16_kernel(TK_PT_KERNEL_ARGS) {
    TK_PT_KERNEL_UNPACK;
    constexpr int kWide = 1024;                  // columns per piece
    constexpr int LPG = G / 16, GPS = kWide / G;
    constexpr int FMT = TK_E2M1;
    using RS = RowScales<Fmt<FMT>::qmax, RPW, LPG>;
    const bool one_col = RPW * kWide >= p.K;
    const int tile_m = tile_grid_row(one_col), tile_k = tile_grid_col(one_col);
    const int lane = threadIdx.x & 63, wave = wave_id();
    const int strip = tile_k * RPW;
    const int col = strip * kWide + lane * 16;
    const int kgrp = strip * GPS + lane / LPG;
    const int row0 = tile_m * kWaves + wave;
    if constexpr (!FULL_GRID) {
        if (row0 >= p.M) return;
    }
    Raw8<e4m3in_t> lo[RPW], hi[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        const u32x4 w = ld_stream16(elem_ptr<e4m3in_t>(p.x, row0, p.x_ld, col + r * kWide));
        if (r + 1 < RPW) vmem_issue_gap();
        lo[r].w = u32x2{w.x, w.y};
        hi[r].w = u32x2{w.z, w.w};
        lo[r].s = hi[r].s = sf_load(p.xsf, row0 / p.in_bm, (col + r * kWide) / p.in_bk);
    }
    float amax[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        float a[8], b[8];
        lo[r].get(a);
        hi[r].get(b);
        amax[r] = group_allmax<LPG>(__builtin_fmaxf(absmax8(a), absmax8(b)));
    }
    RS rs;
    rs.compute(amax, Fmt<FMT>::floor_, p.round_sf != 0, lane);
    // lane j (< A) of a group computed the scale of piece c*A + j; the wave's scales form one run of RPW * GPS floats
    const int own = lane % LPG;
    if (own < RS::A) {
#pragma unroll
        for (int c = 0; c < RS::NC; ++c)
            st_stream4(reinterpret_cast<float *>(p.sf.base) + (int64_t)row0 * p.sf.ld + kgrp + (c * RS::A + own) * GPS, f2u(rs.own[c].sf));
    }
    uint8_t *out_row = p.out + (int64_t)row0 * (p.K / 2);
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        float a[8], b[8];
        lo[r].get(a);
        hi[r].get(b);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            a[i] = a[i] * rs.inv[r];
            b[i] = b[i] * rs.inv[r];
        }
        st_stream8(out_row + ((col + r * kWide) >> 1), u32x2{pack_e2m1x8(a), pack_e2m1x8(b)});
    }
}

// One scale per row (group == K): a workgroup per row.  Rows of up to 16384 elements are held in registers, ITER pieces
// of 8 elements per thread, between the amax and the conversion, so they are read once; ITER == 0 takes longer rows
// in two passes (the second one is served by L2).  Reference: the `hidden == num_per_channels` branch,
// tile_kernels/quant/per_token_cast_kernel.py:31-35, and the E5M6 cast, which knows no other grouping
// (per_token_cast_to_e5m6_kernel.py:88).
template <int FMT> __host__ __device__ constexpr int64_t code_row_bytes(int64_t k) {
    return FMT == TK_E4M3 ? k : (FMT == TK_E2M1 ? k / 2 : k / 8 * 12);
}

// NT: threads of the workgroup when known at compile time (256), else 0: the count is read from the arguments.
// EXACT: the row is exactly ITER * NT * 8 elements long, no bounds checks.  (Both for the common row lengths: the
// E5M6 cast of bf16 [8192, 4096] measures 20.4 us without them, 20.1 us with NT alone.)
template <typename InT, int FMT, int ITER, int NT, bool EXACT>
__global__ __launch_bounds__(kThreads) void per_token_rowgroup_kernel(TK_PT_KERNEL_ARGS) {
    TK_PT_KERNEL_UNPACK;
    __shared__ uint32_t part[kThreads / 16];
    const int row = blockIdx.x;
    const int nt = NT ? NT : p.geom;   // threads of the workgroup: 64, 128, 192 or 256, the fewest that cover the row in ITER pieces
    const InT *x = reinterpret_cast<const InT *>(p.x) + (int64_t)row * p.x_ld;   // plain (bf16 / fp32) inputs only
    constexpr int N = ITER > 0 ? ITER : 1;
    Raw8<InT> held[N];
    float amax = 0.0f;
    if constexpr (ITER > 0) {
#pragma unroll
        for (int i = 0; i < ITER; ++i) {
            // a lane beyond the end of the row reads the row's first elements (no branch around the loads)
            const int col = (i * nt + threadIdx.x) * 8;
            held[i].load(x + ((EXACT || col < p.K) ? col : 0));
            if (i + 1 < ITER) vmem_issue_gap();
        }
        // (all loads are out before the first piece is looked at: left to itself the compiler moves the first piece's arithmetic in
        // front of the later loads where the row may end inside a piece, and the pieces then arrive one round trip after the other)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < ITER; ++i) {
            const int col = (i * nt + threadIdx.x) * 8;
            float v[8];
            held[i].get(v);
            if (EXACT || col < p.K) amax = __builtin_fmaxf(amax, absmax8(v));
        }
    } else {
        for (int col = threadIdx.x * 8; col < p.K; col += kThreads * 8) {
            Raw8<InT> raw;
            raw.load_cached(x + col);
            float v[8];
            raw.get(v);
            amax = __builtin_fmaxf(amax, absmax8(v));
        }
    }
    amax = group_allmax<16>(amax);
    if ((threadIdx.x & 15) == 0) part[threadIdx.x >> 4] = f2u(amax);
    __syncthreads();
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < kThreads / 16; ++i) m = umax(m, i * 16 < nt ? part[i] : 0u);
    const Scale sc = make_scale<Fmt<FMT>::qmax>(u2f(m), Fmt<FMT>::floor_, p.round_sf != 0);
    if (threadIdx.x == 0) sf_store(p.sf, row, 0, sc);
    uint8_t *out_row = p.out + (int64_t)row * code_row_bytes<FMT>(p.K);
    if constexpr (ITER > 0) {
#pragma unroll
        for (int i = 0; i < ITER; ++i) {
            const int col = (i * nt + threadIdx.x) * 8;
            float v[8];
            held[i].get(v);
            if (EXACT || col < p.K) quantise_store8<FMT, false>(v, sc.inv, out_row, col);
        }
    } else {
        for (int col = threadIdx.x * 8; col < p.K; col += kThreads * 8) {
            Raw8<InT> raw;
            raw.load(x + col);
            float v[8];
            raw.get(v);
            quantise_store8<FMT, false>(v, sc.inv, out_row, col);
        }
    }
}

// Pieces per thread and threads per workgroup of the row kernel: the fewest pieces (of 1, 2, 3, 4, 6, 8) with which at
// most 256 threads cover the row, then the fewest whole waves that do.  Measured on MI355X, E5M6 cast of bf16, always
// 256 threads and at most 4 pieces against this: [131072, 512] 86.4 us, [65536, 1536] 67.6 us, [12160, 11008] 89.4 us
// (two passes).
template <typename InT, int FMT>
static void launch_per_token_rowgroup(PerTokenParams &p, hipStream_t stream) {
    static const int kPieces[] = {1, 2, 3, 4, 6, 8};
    int iters = 0, threads = kThreads;
    for (int it : kPieces) {
        const int64_t per_wave = (int64_t)it * 64 * 8;
        const int64_t waves = (p.K + per_wave - 1) / per_wave;
        if (waves <= kWaves) { iters = it; threads = (int)waves * 64; break; }
    }
    p.geom = threads;
    // PARTIAL: the thread count template argument of a row that needs fewer than four waves (0: read from the arguments).  With 4 and
    // 8 pieces, and in two passes, a row always takes all four waves (the piece count before would have covered it otherwise).
#define TK_ROWGROUP_LAUNCH_NT(I, NT, EXACT) \
    hipLaunchKernelGGL((per_token_rowgroup_kernel<InT, FMT, I, NT, EXACT>), dim3(p.M), dim3(threads), 0, stream, TK_PT_LAUNCH_ARGS(p))
#define TK_ROWGROUP_LAUNCH(I, PARTIAL)                                              \
    do {                                                                            \
        if (threads == kThreads && (I) != 0 && p.K == (I) * kThreads * 8)           \
            TK_ROWGROUP_LAUNCH_NT(I, kThreads, (I) != 0);                           \
        else if (threads == kThreads)                                               \
            TK_ROWGROUP_LAUNCH_NT(I, kThreads, false);                              \
        else                                                                        \
            TK_ROWGROUP_LAUNCH_NT(I, PARTIAL, false);                               \
    } while (0)
    switch (iters) {
        case 1: TK_ROWGROUP_LAUNCH(1, 0); break;
        case 2: TK_ROWGROUP_LAUNCH(2, 0); break;
        case 3: TK_ROWGROUP_LAUNCH(3, 0); break;
        case 4: TK_ROWGROUP_LAUNCH(4, kThreads); break;
        case 6: TK_ROWGROUP_LAUNCH(6, 0); break;
        case 8: TK_ROWGROUP_LAUNCH(8, kThreads); break;
        default: TK_ROWGROUP_LAUNCH(0, kThreads); break;
    }
#undef TK_ROWGROUP_LAUNCH
#undef TK_ROWGROUP_LAUNCH_NT
}

// Short rows (plain inputs): the strips of the tiled kernels are 512 columns wide, so a row of 576 columns keeps 72 of
// every 128 lanes busy.  Here the rows are laid end to end in units of one group instead: lane slot L serves group
// L / LPG of the sequence (row 0's groups, row 1's groups, ...), 8 elements per lane, and only the last group of a row
// can be partly empty (576 columns in groups of 128: 72 of 80 lanes).  A wave holds RPW slots of 64 lanes; every group
// is complete inside one slot, so the reductions and the shared scale arithmetic are those of the tiled kernel.  Each
// scale is stored by one lane (all three layouts).
template <typename InT, int G, int FMT, int RPW>
__global__ __launch_bounds__(kThreads) void per_token_cast_flat_kernel(TK_PT_KERNEL_ARGS) {
    TK_PT_KERNEL_UNPACK;
    constexpr int LPG = G / 8;
    using RS = RowScales<Fmt<FMT>::qmax, RPW, LPG>;
    const int lane = threadIdx.x & 63, wave = wave_id();
    const int gpr = p.geom;   // groups per row
    const int64_t out_ld = FMT == TK_E4M3 ? p.K : p.K / 2;
    const int own = lane % LPG;

    int row[RPW], grp[RPW];
    bool ok[RPW];
    Raw8<InT> raw[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        const unsigned slot = (unsigned)((blockIdx.x * kWaves + wave) * RPW + r);
        const unsigned gs = (slot * 64u + (unsigned)lane) / (unsigned)LPG;
        // gs / gpr by multiplication: with floor(2^32 / gpr) the quotient comes out exact or one too small
        unsigned q = __umulhi(gs, (unsigned)p.in_bm), rem = gs - q * (unsigned)gpr;
        if (rem >= (unsigned)gpr) { ++q; rem -= (unsigned)gpr; }
        row[r] = (int)q;
        grp[r] = (int)rem;
        const int col = grp[r] * G + own * 8;
        ok[r] = row[r] < p.M && col < p.K;
        // no branch around the load: a lane beyond the matrix reads its first bytes and is cleared by value
        raw[r].load(ok[r] ? elem_ptr<InT>(p.x, row[r], p.x_ld, col) : p.x);
        if (r + 1 < RPW) vmem_issue_gap();
        if (!ok[r]) raw[r].zero();
    }

    float inv[RPW];
    if (p.mode == TK_CAST_GIVEN_SF) {
#pragma unroll
        for (int r = 0; r < RPW; ++r) inv[r] = 1.0f / (ok[r] ? sf_load_select(p.sf, row[r], grp[r]) : 1.0f);
    } else {
        float amax[RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            float v[8];
            raw[r].get(v);
            amax[r] = group_allmax<LPG>(absmax8(v));
        }
        RS rs;
        rs.compute(amax, Fmt<FMT>::floor_, p.round_sf != 0, lane);
#pragma unroll
        for (int r = 0; r < RPW; ++r) inv[r] = rs.inv[r];
        // lane j (< A) of a group computed the scale of slot c*A + j
        if (own < RS::A) {
#pragma unroll
            for (int c = 0; c < RS::NC; ++c) {
                // the slot's row and group, chosen by value (no dynamic indexing of the arrays)
                int m = row[c * RS::A], k = grp[c * RS::A];
                if (RS::A >= 2 && own == 1) { m = row[c * RS::A + (RS::A >= 2 ? 1 : 0)]; k = grp[c * RS::A + (RS::A >= 2 ? 1 : 0)]; }
                if (RS::A >= 4 && own == 2) { m = row[c * RS::A + (RS::A >= 4 ? 2 : 0)]; k = grp[c * RS::A + (RS::A >= 4 ? 2 : 0)]; }
                if (RS::A >= 4 && own == 3) { m = row[c * RS::A + (RS::A >= 4 ? 3 : 0)]; k = grp[c * RS::A + (RS::A >= 4 ? 3 : 0)]; }
                if (m < p.M) sf_store(p.sf, m, k, rs.own[c]);
            }
        }
    }
    if (p.mode != TK_SF_ONLY) {
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            if (!ok[r]) continue;
            float v[8];
            raw[r].get(v);
            uint8_t *out_row = p.out + (int64_t)row[r] * out_ld;
            const int col = grp[r] * G + own * 8;
            if (p.mode == TK_CAST_GIVEN_SF) quantise_store8<FMT, true>(v, inv[r], out_row, col);
            else quantise_store8<FMT, false>(v, inv[r], out_row, col);
        }
    }
}

// Rows per wave.  Measured on MI355X (us per call): bf16 [4096, 7168] -> E4M3 1x128 row-major scales
// 18.1 / 16.3 / 17.0 for 1 / 2 / 4 rows; bf16 [16384, 7168] -> E2M1 1x32 packed scales 55.2 / 43.4 / 45.4.
// Quantised input: a lane's 8 codes are only 8 (or 4) bytes, so a wave takes more rows to amortise
// its fixed work; E4M3 1x128 [8192, 4096] -> E2M1 1x32: 14.3 / 12.0 / 12.2 for 2 / 4 / 8 rows.
template <typename InT> constexpr int rows_per_wave() { return Elem<InT>::quantised ? 4 : 2; }

template <typename InT, int G, int FMT, int TILE>
static void launch_per_token_tiled(PerTokenParams &p, hipStream_t stream) {
    constexpr int RPW = rows_per_wave<InT>();
    constexpr bool WIDE = TILE == T_WIDE, ROWW = TILE == T_ROWWISE;
    const int strips = (p.K + kStripCols - 1) / kStripCols;
    const int waves = WIDE ? wide_tile_waves(strips) : (ROWW ? rowwise_waves<InT, FMT>() : kWaves);
    const int rows = WIDE ? RPW : (ROWW ? waves : kWaves * RPW);
    const int cols = WIDE ? waves * kStripCols : (ROWW ? RPW * kStripCols : kStripCols);
    const int tiles_m = (p.M + rows - 1) / rows, tiles_k = (p.K + cols - 1) / cols;
    p.geom = WIDE ? waves : tiles_k;
    const dim3 block(64 * waves);
    const dim3 grid = (WIDE || ROWW) ? tile_grid(tiles_k, tiles_m) : dim3((unsigned)(tiles_m * tiles_k));
    const bool exact = p.M % rows == 0 && p.K % cols == 0 && (!(WIDE || ROWW) || tile_grid_exact(tiles_k, tiles_m));
    if constexpr (ROWW && !Elem<InT>::quantised) {
        if (p.mode == TK_CAST_GIVEN_SF) {
            if (exact) hipLaunchKernelGGL((per_token_cast_kernel<InT, G, FMT, RPW, TILE, true, true>), grid, block, 0, stream, TK_PT_LAUNCH_ARGS(p));
            else hipLaunchKernelGGL((per_token_cast_kernel<InT, G, FMT, RPW, TILE, false, true>), grid, block, 0, stream, TK_PT_LAUNCH_ARGS(p));
            return;
        }
    }
    if (exact)
        hipLaunchKernelGGL((per_token_cast_kernel<InT, G, FMT, RPW, TILE, true>), grid, block, 0, stream, TK_PT_LAUNCH_ARGS(p));
    else
        hipLaunchKernelGGL((per_token_cast_kernel<InT, G, FMT, RPW, TILE, false>), grid, block, 0, stream, TK_PT_LAUNCH_ARGS(p));
}

// Whether the flattened kernel keeps more lanes busy than 512-column strips do (and the strips less than 80 %).
inline bool short_rows_pay(int64_t K, int G) {
    const int64_t strips = (K + kStripCols - 1) / kStripCols, groups = (K + G - 1) / G;
    return K * 5 < strips * kStripCols * 4 && groups * G < strips * kStripCols;
}

template <typename InT, int G, int FMT>
static void launch_per_token_group(PerTokenParams &p, hipStream_t stream) {
    constexpr int RPW = rows_per_wave<InT>();
    if constexpr (!Elem<InT>::quantised) {
        if (short_rows_pay(p.K, G)) {
            const int64_t gpr = (p.K + G - 1) / G, lanes = (int64_t)p.M * gpr * (G / 8);
            const int64_t blocks = (lanes + kThreads * RPW - 1) / (kThreads * RPW);
            if (lanes < INT32_MAX - 2 * kThreads * RPW) {   // lane slots are numbered in 32 bits
            p.geom = (int)gpr;
            p.in_bm = (int)(uint32_t)(gpr == 1 ? 0xFFFFFFFFull : (1ull << 32) / (uint64_t)gpr);   // plain input: the field carries the reciprocal of gpr
            hipLaunchKernelGGL((per_token_cast_flat_kernel<InT, G, FMT, RPW>), dim3((unsigned)blocks), dim3(kThreads), 0, stream,
                               TK_PT_LAUNCH_ARGS(p));
            return;
            }
        }
    }
    if constexpr (std::is_same<InT, e4m3in_t>::value && G >= 32 && FMT == TK_E2M1) {
        constexpr int Q16_RPW = 2;
        if (p.sf.layout == TK_SF_ROW_F32 && p.K % (Q16_RPW * 1024) == 0 && p.in_bk % 16 == 0 && aligned_to(p.x, 16) && p.x_ld % 16 == 0) {
            const int tiles_m = (p.M + kWaves - 1) / kWaves, tiles_k = p.K / (Q16_RPW * 1024);
            p.geom = tiles_k;
            const dim3 grid = tile_grid(tiles_k, tiles_m);
            if (p.M % kWaves == 0 && tile_grid_exact(tiles_k, tiles_m))
                hipLaunchKernelGGL((per_token_cast_q16_kernel<G, Q16_RPW, true>), grid, dim3(kThreads), 0, stream, TK_PT_LAUNCH_ARGS(p));
            else
                hipLaunchKernelGGL((per_token_cast_q16_kernel<G, Q16_RPW, false>), grid, dim3(kThreads), 0, stream, TK_PT_LAUNCH_ARGS(p));
            return;
        }
    }
    // Row-wise tiles where they fit the columns exactly.  Measured on MI355X against wide tiles: bf16 [4096, 7168] -> E4M3 14.85 ->
    // 14.46 us, [32768, 4096] 59.4 -> 56.8 us, given scales 15.83 -> 15.61 us; the scale-only mode, whose only stores
    // are the scales, is better off with the staged runs of the wide tile (10.15 us against 10.85 us).
    if (p.sf.layout == TK_SF_ROW_F32 && p.mode != TK_SF_ONLY && p.K % (RPW * kStripCols) == 0)
        launch_per_token_tiled<InT, G, FMT, T_ROWWISE>(p, stream);
    // a caller-supplied scale tensor is only read, so either tile shape does
    else if (p.sf.layout == TK_SF_ROW_F32 && wide_tiles_pay(p.K)) launch_per_token_tiled<InT, G, FMT, T_WIDE>(p, stream);
    else launch_per_token_tiled<InT, G, FMT, T_STACKED>(p, stream);
}

// plain (bf16 / fp32) and quantised (codes + block scales) inputs alike; one scale per row (group == K
// and not one of the tiled sizes) exists for plain inputs only
template <typename InT, int FMT>
static hipError_t launch_per_token(PerTokenParams &p, int group, hipStream_t stream) {
    if constexpr (!Elem<InT>::quantised) {
        if (group == p.K && group != 16 && group != 32 && group != 64 && group != 128) {
            launch_per_token_rowgroup<InT, FMT>(p, stream);
            return hipGetLastError();
        }
    }
    switch (group) {
        case 16: launch_per_token_group<InT, 16, FMT>(p, stream); break;
        case 32: launch_per_token_group<InT, 32, FMT>(p, stream); break;
        case 64: launch_per_token_group<InT, 64, FMT>(p, stream); break;
        default: launch_per_token_group<InT, 128, FMT>(p, stream); break;
    }
    return hipGetLastError();
}

}  // namespace tk

using namespace tk;

extern "C" int tk_check_per_token_cast(const void *x, int x_dtype, int64_t M, int64_t K, int64_t x_row_stride,
                                       const void *out, const void *sf, int64_t sf_ld, int fmt, int group,
                                       int sf_layout, int round_sf, int mode) {
    if (x_dtype != TK_BF16 && x_dtype != TK_F32) return TK_ERR_BAD_DTYPE;
    if (fmt != TK_E4M3 && fmt != TK_E2M1 && fmt != TK_E5M6) return TK_ERR_BAD_FORMAT;
    if (mode < TK_CAST_AND_SF || mode > TK_CAST_GIVEN_SF) return TK_ERR_BAD_MODE;
    if (sf_layout < TK_SF_ROW_F32 || sf_layout > TK_SF_COL_UE8M0) return TK_ERR_BAD_LAYOUT;
    if (sf_layout == TK_SF_COL_UE8M0 && !round_sf && mode != TK_CAST_GIVEN_SF) return TK_ERR_BAD_LAYOUT;
    if (M < 0 || K <= 0 || K % 8 != 0) return TK_ERR_BAD_SHAPE;
    if (M > INT32_MAX - 64 || K > INT32_MAX - 1024) return TK_ERR_TOO_LARGE;
    const bool row_group = fmt == TK_E5M6 || (group == K && group != 16 && group != 32 && group != 64 && group != 128);
    if (fmt == TK_E5M6) {       // one scale per row, as the reference's kernel (per_token_cast_to_e5m6_kernel.py:88)
        if (group != K) return TK_ERR_BAD_GROUP;
        if (mode != TK_CAST_AND_SF) return TK_ERR_BAD_MODE;
    } else if (row_group) {
        if (K % 64 != 0) return TK_ERR_BAD_GROUP;
        if (mode != TK_CAST_AND_SF) return TK_ERR_BAD_MODE;
    } else if (group != 16 && group != 32 && group != 64 && group != 128) {
        return TK_ERR_BAD_GROUP;
    }
    if (M == 0) return TK_OK;
    if (!x || !sf || (mode != TK_SF_ONLY && !out)) return TK_ERR_NULL_POINTER;
    if (x_row_stride < K) return TK_ERR_BAD_STRIDE;
    const int64_t esz = x_dtype == TK_BF16 ? 2 : 4;
    if (!aligned_to(x, 16) || (x_row_stride * esz) % 16 != 0) return TK_ERR_MISALIGNED;
    if (mode != TK_SF_ONLY && !aligned_to(out, 8)) return TK_ERR_MISALIGNED;
    if (!aligned_to(sf, 4)) return TK_ERR_MISALIGNED;
    const int64_t nk = (K + group - 1) / group;
    if (M * nk > INT32_MAX) return TK_ERR_TOO_LARGE;
    if (((M + 3) / 4) * ((K + kStripCols - 1) / kStripCols) > INT32_MAX) return TK_ERR_TOO_LARGE;   // tile count
    const int64_t need = sf_layout == TK_SF_ROW_F32 ? nk : (sf_layout == TK_SF_COL_F32 ? M : 4 * M);
    if (sf_ld < need) return TK_ERR_BAD_STRIDE;
    if (sf_layout == TK_SF_COL_UE8M0 && sf_ld % 4 != 0) return TK_ERR_MISALIGNED;
    return TK_OK;
}

extern "C" int tk_per_token_cast(const void *x, int x_dtype, int64_t M, int64_t K, int64_t x_row_stride, void *out,
                                 void *sf, int64_t sf_ld, int fmt, int group, int sf_layout, int round_sf, int mode,
                                 void *stream) {
    const int rc = tk_check_per_token_cast(x, x_dtype, M, K, x_row_stride, out, sf, sf_ld, fmt, group, sf_layout,
                                           round_sf, mode);
    if (rc != TK_OK || M == 0) return rc;
    PerTokenParams p;
    p.x = x;
    p.out = static_cast<uint8_t *>(out);
    p.sf = SfRef{sf, sf_ld, sf_layout, (int)M, (int)((K + group - 1) / group)};
    p.x_ld = x_row_stride;
    p.M = (int)M;
    p.K = (int)K;
    p.geom = 0;
    p.round_sf = round_sf;
    p.mode = mode;
    p.xsf = SfRef{nullptr, 0, TK_SF_ROW_F32, 0, 0};
    p.in_bm = p.in_bk = 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e;
    if (fmt == TK_E5M6) {
        if (x_dtype == TK_BF16) launch_per_token_rowgroup<bf16_t, TK_E5M6>(p, s);
        else launch_per_token_rowgroup<float, TK_E5M6>(p, s);
        return (int)hipGetLastError();
    }
    if (x_dtype == TK_BF16)
        e = fmt == TK_E4M3 ? launch_per_token<bf16_t, TK_E4M3>(p, group, s) : launch_per_token<bf16_t, TK_E2M1>(p, group, s);
    else
        e = fmt == TK_E4M3 ? launch_per_token<float, TK_E4M3>(p, group, s) : launch_per_token<float, TK_E2M1>(p, group, s);
    return (int)e;
}

extern "C" int tk_check_per_token_cast_quantized(const void *x, int x_fmt, int64_t M, int64_t K, int64_t x_row_stride,
                                                 const void *x_sf, int64_t x_sf_ld, int x_sf_layout, int x_bm, int x_bk,
                                                 const void *out, const void *sf, int64_t sf_ld, int fmt, int group,
                                                 int sf_layout, int round_sf) {
    if (x_fmt != TK_E4M3 && x_fmt != TK_E2M1) return TK_ERR_BAD_DTYPE;
    if (fmt != TK_E4M3 && fmt != TK_E2M1) return TK_ERR_BAD_FORMAT;
    if (sf_layout < TK_SF_ROW_F32 || sf_layout > TK_SF_COL_UE8M0) return TK_ERR_BAD_LAYOUT;
    if (x_sf_layout < TK_SF_ROW_F32 || x_sf_layout > TK_SF_COL_UE8M0) return TK_ERR_BAD_LAYOUT;
    if (sf_layout == TK_SF_COL_UE8M0 && !round_sf) return TK_ERR_BAD_LAYOUT;
    if (M < 0 || K <= 0 || K % 8 != 0) return TK_ERR_BAD_SHAPE;
    if (M > INT32_MAX - 64 || K > INT32_MAX - 4096) return TK_ERR_TOO_LARGE;
    if (group != 16 && group != 32 && group != 64 && group != 128) return TK_ERR_BAD_GROUP;
    if (x_bm < 1 || x_bk < 8 || x_bk % 8 != 0) return TK_ERR_BAD_GROUP;
    if (M == 0) return TK_OK;
    if (!x || !x_sf || !out || !sf) return TK_ERR_NULL_POINTER;
    if (x_row_stride < K) return TK_ERR_BAD_STRIDE;
    const uintptr_t unit = x_fmt == TK_E4M3 ? 8 : 4;     // bytes a lane loads
    if (!aligned_to(x, unit) || x_row_stride % 8 != 0) return TK_ERR_MISALIGNED;
    if (!aligned_to(out, 8) || !aligned_to(sf, 4)) return TK_ERR_MISALIGNED;
    if (!aligned_to(x_sf, 4) || (x_sf_layout == TK_SF_COL_UE8M0 && x_sf_ld % 4 != 0)) return TK_ERR_MISALIGNED;
    const int64_t nk = (K + group - 1) / group;
    if (M * nk > INT32_MAX) return TK_ERR_TOO_LARGE;
    const int64_t need = sf_layout == TK_SF_ROW_F32 ? nk : (sf_layout == TK_SF_COL_F32 ? M : 4 * M);
    if (sf_ld < need) return TK_ERR_BAD_STRIDE;
    if (sf_layout == TK_SF_COL_UE8M0 && sf_ld % 4 != 0) return TK_ERR_MISALIGNED;
    const int64_t xnm = (M + x_bm - 1) / x_bm, xnk = (K + x_bk - 1) / x_bk;
    const int64_t xneed = x_sf_layout == TK_SF_ROW_F32 ? xnk : (x_sf_layout == TK_SF_COL_F32 ? xnm : 4 * xnm);
    if (x_sf_ld < xneed) return TK_ERR_BAD_STRIDE;
    return TK_OK;
}

extern "C" int tk_per_token_cast_quantized(const void *x, int x_fmt, int64_t M, int64_t K, int64_t x_row_stride,
                                           const void *x_sf, int64_t x_sf_ld, int x_sf_layout, int x_bm, int x_bk,
                                           void *out, void *sf, int64_t sf_ld, int fmt, int group, int sf_layout,
                                           int round_sf, void *stream) {
    const int rc = tk_check_per_token_cast_quantized(x, x_fmt, M, K, x_row_stride, x_sf, x_sf_ld, x_sf_layout, x_bm, x_bk,
                                                     out, sf, sf_ld, fmt, group, sf_layout, round_sf);
    if (rc != TK_OK || M == 0) return rc;
    PerTokenParams p;
    p.x = x;
    p.out = static_cast<uint8_t *>(out);
    p.sf = SfRef{sf, sf_ld, sf_layout, (int)M, (int)((K + group - 1) / group)};
    p.x_ld = x_row_stride;
    p.M = (int)M;
    p.K = (int)K;
    p.geom = 0;
    p.round_sf = round_sf;
    p.mode = TK_CAST_AND_SF;
    p.xsf = SfRef{const_cast<void *>(x_sf), x_sf_ld, x_sf_layout, (int)((M + x_bm - 1) / x_bm), (int)((K + x_bk - 1) / x_bk)};
    p.in_bm = x_bm;
    p.in_bk = x_bk;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e;
    if (x_fmt == TK_E4M3)
        e = fmt == TK_E4M3 ? launch_per_token<e4m3in_t, TK_E4M3>(p, group, s) : launch_per_token<e4m3in_t, TK_E2M1>(p, group, s);
    else
        e = fmt == TK_E4M3 ? launch_per_token<e2m1in_t, TK_E4M3>(p, group, s) : launch_per_token<e2m1in_t, TK_E2M1>(p, group, s);
    return (int)e;
}
