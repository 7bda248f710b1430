// Fused SwiGLU + per-token (1 x 128, or one scale per row) E4M3 quantisation for gfx950.
//
// x[R, 2H]: gate = columns [0, H), up = columns [H, 2H).  The activation never touches HBM: a lane
// loads 8 gate and 8 up values (two 16-byte loads for bf16), computes v = g/(1+exp(-g))*u in fp32,
// and the 16 lanes that share a 128-column group reduce |v| with DPP, derive the scale and
// convert straight to packed FP8.  A wave holds four 512-column pieces (of one row, or of four rows:
// see the tile shapes below), all eight loads of a lane in flight before first use.
// Padding rows (pos_to_expert < 0) are not read; zeros are written for their codes and scales.
//
// Reference semantics: tile_kernels/quant/swiglu_forward_and_per_token_cast_kernel.py:61-170,
// tile_kernels/torch/swiglu.py:62-86.
#include <stddef.h>

#include <algorithm>

#include "swiglu_math.hpp"
#include "tk_device.hpp"
#include "tk_host.hpp"

namespace tk {

struct SwigluParams {
    const void *x;
    uint8_t *out;
    SfRef sf;
    const int32_t *pos_to_token_topk;
    const float *topk_weights;
    const int32_t *pos_to_expert;
    unsigned long long *clamped_count;
    int64_t num_weights;
    int R, H;
    int nwaves, tiles_k;   // waves (= rows) of a T_ROW tile; tiles along the columns
    int round_sf;
    float floor_;        // amax lower clamp
    float clamp;
};

// The kernels take their parameters as individual scalars in the order they are needed: the leading
// 14 dwords of the kernel-argument segment arrive preloaded in SGPRs when a wave starts (the library is
// built with -amdgpu-kernarg-preload-count=16) and hold everything the input addresses are made of, plus the two
// values that every code path of the tiled kernel uses (the compiler computes what all paths share before the
// first branch, and would wait there for an argument that is not preloaded); the others are fetched from the
// argument buffer (host memory) while the first loads are in flight.
#define TK_SWIGLU_KERNEL_ARGS                                                                                      \
    const void *a_x, const int32_t *a_pe, int a_R, int a_H, int a_nwaves, int a_tiles_k, uint8_t *a_out, void *a_sf, \
        float a_floor, int a_round_sf, int64_t a_sf_ld, float a_clamp, int a_sf_layout, const int32_t *a_ptt,          \
        const float *a_w, unsigned long long *a_cnt, int64_t a_nw, int a_nk
#define TK_SWIGLU_KERNEL_UNPACK                                                                            \
    const SwigluParams p{a_x, a_out, SfRef{a_sf, a_sf_ld, a_sf_layout, a_R, a_nk}, a_ptt, a_w, a_pe, a_cnt, \
                         a_nw, a_R, a_H, a_nwaves, a_tiles_k, a_round_sf, a_floor, a_clamp}
// (the variant whose later arguments are fetched behind the loads: see fetch_late_arguments)
#define TK_SWIGLU_KERNEL_UNPACK_EARLY                                                                                   \
    SwigluParams p{a_x, a_out, SfRef{a_sf, (int64_t)reinterpret_cast<intptr_t>(a_pe), TK_SF_ROW_F32, a_R, 0}, nullptr, nullptr, \
                   nullptr, nullptr, 0, a_R, a_H, a_nwaves, a_tiles_k, a_round_sf, a_floor, 0.0f}
#define TK_SWIGLU_LAUNCH_ARGS(p)                                                                                  \
    (p).x, (p).pos_to_expert, (p).R, (p).H, (p).nwaves, (p).tiles_k, (p).out, (p).sf.base, (p).floor_, (p).round_sf, \
        (p).sf.ld, (p).clamp, (p).sf.layout, (p).pos_to_token_topk, (p).topk_weights, (p).clamped_count,            \
        (p).num_weights, (p).sf.nk

// sum over the 64 lanes, in every lane
__device__ __forceinline__ uint32_t wave_sum(uint32_t v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += (uint32_t)__shfl_xor((int)v, m, 64);
    return v;
}

// CLAMP: 0 none, 1 clamp, 2 clamp and count
template <int CLAMP> struct ClampCounter {
    uint32_t n0 = 0, n1 = 0, n2 = 0;    // per lane
    // `counted` leaves the element out of the counts (it is clamped all the same)
    __device__ __forceinline__ void apply(float &g, float &u, float c, bool counted = true) {
        if (CLAMP == 0) return;
        if (CLAMP == 2) { n0 += counted && g > c; n1 += counted && u > c; n2 += counted && u < -c; }
        g = __builtin_fminf(g, c);
        u = clamp_both_sides(u, c);
    }
    // min(max(u, -c), c) in one instruction: the median of u, -c and c.  (A negative limit makes every element the limit,
    // as the two-step form does: the lower bound is then the limit itself.)
    static __device__ __forceinline__ float clamp_both_sides(float u, float c) {
        return __builtin_amdgcn_fmed3f(u, c >= 0.0f ? -c : c, c);
    }
    // Eight elements of every lane at once.  Counting costs six instructions per element and clamped elements are rare
    // in practice, so the wave first takes the largest gate and the largest |up| of its 512 elements (two instructions
    // per element) and counts only if one of them is beyond the limit.  bf16 [8192, 2 x 2048] on MI355X with nothing
    // clamped: 17.3 -> 16.4 us on 1024 looping workgroups, 18.4 -> 15.7 us on 2048 (14.4 us without the counters).
    __device__ __forceinline__ void apply8(float (&g)[8], float (&u)[8], float c) {
        if (CLAMP == 0) return;
        if (CLAMP == 2) {
            float mg = g[0], mu = __builtin_fabsf(u[0]);
#pragma unroll
            for (int i = 1; i < 8; ++i) {
                mg = __builtin_fmaxf(mg, g[i]);
                mu = __builtin_fmaxf(mu, __builtin_fabsf(u[i]));
            }
            if (__builtin_amdgcn_ballot_w64(mg > c || mu > c) != 0ull) {      // wave-uniform
#pragma unroll
                for (int i = 0; i < 8; ++i) { n0 += g[i] > c; n1 += u[i] > c; n2 += u[i] < -c; }
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            g[i] = __builtin_fminf(g[i], c);
            u[i] = clamp_both_sides(u[i], c);
        }
    }
    // Lanes -> wave (DPP adds, only in waves that counted anything) -> workgroup (one LDS atomic per wave and counter) ->
    // one global atomic instruction per workgroup, whose three lanes carry the three counters.  Requests to one line are
    // served one after the other, about 10 ns each on MI355X, whoever sends them: up to some 1400 reporting workgroups
    // hide behind the 15 us of bf16 [8192, 2 x 2048], more do not (every one of 2048 workgroups reporting: 33.8 us; of 1024
    // looping ones: 22.9 us), which is why the caller may cap the grid.  (With every lane adding to LDS by itself the
    // 1024 workgroups took 28.6 us; counts taken per wave as bits of the compare masks, in scalar registers, 23.2 us, but
    // 20.4 instead of 17.1 us where nothing is clamped.)
    __device__ __forceinline__ void flush(unsigned long long *dst) {
        if (CLAMP != 2) return;
        __shared__ unsigned long long acc[3];
        if (threadIdx.x < 3) acc[threadIdx.x] = 0ull;
        __syncthreads();
        if (__builtin_amdgcn_ballot_w64((n0 | n1 | n2) != 0u) != 0ull) {      // wave-uniform
            const uint32_t s0 = wave_sum(n0), s1 = wave_sum(n1), s2 = wave_sum(n2);
            if ((threadIdx.x & 63) == 0) {
                if (s0) atomicAdd(&acc[0], (unsigned long long)s0);
                if (s1) atomicAdd(&acc[1], (unsigned long long)s1);
                if (s2) atomicAdd(&acc[2], (unsigned long long)s2);
            }
        }
        __syncthreads();
        if (threadIdx.x < 3 && acc[threadIdx.x]) atomicAdd(&dst[threadIdx.x], acc[threadIdx.x]);
    }
};

// The kernel-argument segment of TK_SWIGLU_KERNEL_ARGS, field for field.
struct SwigluLateKernargs {
    int64_t sf_ld; float clamp; int sf_layout; const int32_t *ptt; const float *w; unsigned long long *cnt; int64_t nw; int nk;
};
struct SwigluKernargs {
    const void *x; const int32_t *pe; int R, H, nwaves, tiles_k; uint8_t *out; void *sf; float floor_; int round_sf;
    SwigluLateKernargs late;
};
static_assert(offsetof(SwigluKernargs, late) == 56 && offsetof(SwigluLateKernargs, ptt) == 16 && offsetof(SwigluLateKernargs, nw) == 40,
              "the mirror of the argument segment follows TK_SWIGLU_KERNEL_ARGS: 14 preloaded dwords, then the later arguments");

// The arguments beyond the preloaded ones that the row-wise waves use after their vector loads, read from the argument
// segment here and now.  A kernel whose code paths part before the loads names these arguments nowhere else: named, their
// fetch and the first arithmetic on them (a null test, an address) would be placed where the paths still run together,
// i.e. in front of the loads, and every wave would wait for the fetch before it requests its data.  Each wave pays a round
// trip to the scalar cache per argument it looks at here, one after the other where a later one is only fetched if an
// earlier one says so; for the one- and two-piece waves at the end of a launch that is time their data does not cover
// (bf16 [8192, 2 x 2048]: 14.7 us with the routing arguments looked at by every wave, 14.3 us without), so only what the
// variant at hand uses is fetched: the clamp value, the routing list with its weights and their count.  (The leading
// dimension of the scales, which every wave needs, travels in a preloaded place: see the launch code.)
__device__ __forceinline__ void fetch_late_arguments(SwigluParams &p, bool with_clamp, bool with_weights, bool with_layout = false) {
    uintptr_t ka = (uintptr_t)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(ka) : : "memory");      // stays behind the loads issued before it
    const SwigluLateKernargs *k = &reinterpret_cast<const SwigluKernargs *>(ka)->late;
    if (with_clamp) p.clamp = uniform_load(&k->clamp);
    if (with_layout) {
        p.sf.layout = uniform_load(&k->sf_layout);
        p.sf.nk = uniform_load(&k->nk);
    }
    if (with_weights) {
        p.pos_to_token_topk = uniform_load(&k->ptt);
        p.topk_weights = uniform_load(&k->w);
        p.num_weights = uniform_load(&k->nw);
    }
}

// `row` must be wave-uniform
__device__ __forceinline__ float row_weight(const SwigluParams &p, int row) {
    const int pos = uniform_load(p.pos_to_token_topk + row);
    return (pos >= 0 && pos < p.num_weights) ? uniform_load(p.topk_weights + pos) : 0.0f;
}

// One wave on NP pieces (no mask; CLAMP 0 or 1), for the finer-grained waves at the end of a launch (see the tiled kernel):
// consecutive pieces of one row, as in a T_ROW or T_ROWC tile, or with STACK the same piece of NP consecutive rows, as in a
// T_STACKED tile.  SF says where the scales go: 0 row-major, stored by the wave itself; 1 column-major layouts: the
// workgroup's four waves hold consecutive rows of the same pieces (rows row0 - wave * (STACK ? NP : 1) onwards), their
// scales meet in LDS and leave as runs along the rows; 2 whichever the layout argument says (read behind the loads).
template <typename InT, int CLAMP, int NP, bool WEIGHTED, int SF = 0, bool STACK = false>
__device__ __forceinline__ void swiglu_row_wave(SwigluParams p, int row0, int strip) {
    static_assert(CLAMP != 2, "the counting variant loops over tiles");
    static_assert(Raw8<InT>::kXchgBytes == 0, "inputs whose pieces need no exchange between lanes");
    constexpr int GPS = kStripCols / 128;
    constexpr int SROWS = kWaves * (STACK ? NP : 1), SCOLS = STACK ? GPS : NP * GPS;      // staged scales of the workgroup
    using RS = RowScales<448, NP, 16>;
    const int lane = threadIdx.x & 63, own = lane & 15;
    const int col = strip * kStripCols + lane * 8;
    const int64_t rstep = STACK ? 2 * (int64_t)p.H : 0;       // from piece to piece, in elements of the input
    constexpr int cstep = STACK ? 0 : kStripCols;
    // (row, column and H are non-negative 32-bit numbers: unsigned, the row offset is one 32 x 32 -> 64-bit product and nothing
    // needs a sign extension on the way to the loads)
    // The addresses are a wave-uniform 64-bit base (in scalar registers) plus a 32-bit byte offset per lane, which is the form
    // the load instruction takes as it is; a 64-bit address per lane costs two more vector instructions before every load.
    const uint32_t uh = (uint32_t)p.H;
    const uint8_t *xrow = reinterpret_cast<const uint8_t *>(p.x) + (uint64_t)(uint32_t)row0 * (2u * uh * (uint32_t)sizeof(InT));
    const uint32_t lane_off = (uint32_t)strip * (uint32_t)(kStripCols * sizeof(InT)) + (uint32_t)lane * (uint32_t)(8 * sizeof(InT));
    __shared__ uint32_t stage[SF ? SROWS : 1][SF ? SCOLS : 1];
    Raw8<InT> rg[NP], ru[NP];
#pragma unroll
    for (int r = 0; r < NP; ++r) {
        const uint8_t *xg = xrow + (uint64_t)r * (uint64_t)rstep * sizeof(InT) + (uint32_t)(r * cstep) * (uint32_t)sizeof(InT);
        rg[r].load(xg + lane_off);
        vmem_issue_gap();
        ru[r].load(xg + uh * (uint32_t)sizeof(InT) + lane_off);
        if (r + 1 < NP) vmem_issue_gap();
    }
    fetch_late_arguments(p, CLAMP != 0, WEIGHTED, SF != 0);
    float w[NP];
#pragma unroll
    for (int r = 0; r < NP; ++r) w[r] = WEIGHTED ? ((STACK || r == 0) ? row_weight(p, row0 + (STACK ? r : 0)) : w[0]) : 0.0f;
    ClampCounter<CLAMP> clamp;
    float v[NP][8], amax[NP];
#pragma unroll
    for (int r = 0; r < NP; ++r) {
        float g[8], u[8];
        rg[r].get(g);
        ru[r].get(u);
        clamp.apply8(g, u, p.clamp);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[r][i] = silu_mul<InT>(g[i], u[i]);
        if (WEIGHTED) {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[r][i] = v[r][i] * w[r];
        }
        amax[r] = group_allmax<16>(absmax8(v[r]));
    }
    RS rs;
    rs.compute(amax, p.floor_, p.round_sf != 0, lane);
    const bool staged = SF == 1 || (SF == 2 && p.sf.layout != TK_SF_ROW_F32);      // uniform over the launch
    // lane j (< A) of a group computed the scale of piece c*A + j
    if (own < RS::A) {
#pragma unroll
        for (int c = 0; c < RS::NC; ++c) {
            const int pc = c * RS::A + own;
            if (SF != 0 && staged) {
                if (STACK) stage[wave_id() * NP + pc][lane >> 4] = p.sf.layout == TK_SF_COL_UE8M0 ? rs.own[c].e8 : f2u(rs.own[c].sf);
                else stage[wave_id()][pc * GPS + (lane >> 4)] = p.sf.layout == TK_SF_COL_UE8M0 ? rs.own[c].e8 : f2u(rs.own[c].sf);
            } else {
                st_stream4(reinterpret_cast<float *>(p.sf.base) + (int64_t)(row0 + (STACK ? pc : 0)) * p.sf.ld + (strip + (STACK ? 0 : pc)) * GPS + (lane >> 4),
                           f2u(rs.own[c].sf));
            }
        }
    }
#pragma unroll
    for (int r = 0; r < NP; ++r) quantise_store8<TK_E4M3, false>(v[r], rs.inv[r], p.out + (int64_t)(row0 + (STACK ? r : 0)) * p.H, col + r * cstep);
    if constexpr (SF != 0) {
        if (staged) {
            __syncthreads();
            sf_store_tile_colmajor<SROWS, SCOLS>(p.sf, stage, row0 - wave_id() * (STACK ? NP : 1), strip * GPS);
        }
    }
}

// Tile shapes (a wave always holds RPW pieces of 512 output columns, each with its gate and its up half):
//   T_ROW     (row-major scales, H a multiple of RPW*512): W rows x (RPW*512) columns, one row per wave.  The RPW*4
//             scales a wave produces are neighbours in the scale row, so the wave stores them itself as one
//             contiguous run: no LDS stage and no workgroup barrier at the end of the tile
//   T_ROWC    (column-major layouts, H a multiple of RPW*512): the same 4 rows x (RPW*512) columns, one row per wave; the
//             scales are staged in LDS and stored transposed, 4 rows per run.  Against stacked tiles, whose waves
//             read 1 KB from each of 8 row halves instead of 4 KB from 2 (us per call, bf16, packed scales):
//             [32768, 2 x 2048] 60.6 -> 52.4, [16384, 2 x 4096] 69.4 -> 53.9, [8192, 2 x 6144] 48.8 -> 40.9
//   T_STACKED (other H): 4*RPW rows x 512 columns, the 4 waves stacked; the scales are staged in LDS and stored
//             transposed (row-major: one short run per row)
// W = blockDim.x / 64.  FULL_GRID: the tile grid covers the matrix exactly: no bounds checks are compiled in.
// MASK: pos_to_expert is given.
enum { T_STACKED = 0, T_ROW = 2, T_ROWC = 3 };

// ONECOL: the grid is known to be a single column of tiles (else it is found out at run time)
// TAILED (tiles of four-piece waves, exact grids): the launch ends in finer-grained waves.  The grid's row tiles
// come in three runs: `yb` workgroups of one-row waves as described above, then `ym` workgroups whose waves take two
// pieces, then workgroups whose waves take one; all cover the rows in order.  The requests of a launch are served
// roughly in the order they were made, so what arrives last belongs to the last workgroups; with whole rows per wave
// the launch ends with the few waves that got their data last each working through a whole row alone on its SIMD while
// the rest of the GPU is idle, with small waves that work is spread over four times as many SIMDs, and the small waves
// start in the slots that finished waves free, so the second half of the bytes is requested while the first is being
// served.  Measured on MI355X, bf16 [8192, 2 x 2048] (us per call): all rows by one-row waves 14.55; the last 40 % of
// the rows by two-piece waves 14.35; by one-piece waves 14.35 - 14.45; the last 70 % in two-piece and of those the last
// 15 % in one-piece waves 14.06 (55 % / 15 % of the rows: 2.2 and 0.6 times the GPU's wave slots).  The arguments pack
// the run lengths into the two tile-geometry words (see the launch code) so that they arrive preloaded, and the place of
// the mask pointer (these launches have no mask) carries the leading dimension of the scales.  TAILED: 1 without, 2 with
// routing weights.  T_ROWC tiles end the same way, with the four waves of a workgroup on four consecutive rows of the same
// two pieces or one piece (swiglu_row_wave<..., ROWC>), so that their scales still leave as runs along the rows; layout
// and group count of the scales are among the arguments read behind the loads.  T_STACKED tiles (H a multiple of 512 but
// not of 2048) end in workgroups of 4 x 2 rows and then 4 x 1 rows of one 512-column strip, a wave's two pieces one below
// the other as in the tile (row-major scales, without / with: [10912, 2 x 1536] 14.57 / 14.31, [6544, 2 x 2560] 14.71 / 14.29,
// [16384, 2 x 1536] 20.89 / 20.34, [2048, 2 x 7168] 13.52 / 12.97, [49152, 2 x 512] 20.96 / 20.35; packed: 14.46 / 14.31,
// 14.42 / 14.20, 20.78 / 20.39, 13.12 / 12.83, 20.95 / 20.47).  bf16, us per call without / with,
// column-major fp32 scales: [8192, 2 x 2048] 15.39 / 14.74, [4096, 2 x 4096] 15.34 / 14.86, [12288, 2 x 2048] 21.40 / 20.89,
// [16384, 2 x 2048] 27.53 / 27.13; packed UE8M0: 14.79 / 14.36, 14.70 / 14.47, 21.11 / 20.61, 27.18 / 26.88.
template <typename InT, int CLAMP, int RPW, int TILE, bool FULL_GRID, bool MASK, bool ONECOL, int TAILED = 0>
__global__ __launch_bounds__(TILE == T_ROW ? 64 * kMaxWideWaves : kThreads) void swiglu_cast_kernel(TK_SWIGLU_KERNEL_ARGS) {
    static_assert(!TAILED || (FULL_GRID && !MASK && CLAMP != 2 && RPW == 4), "tail waves: exact unmasked grids of four-piece waves");
    if constexpr (TAILED) {
        // a_nwaves: waves per workgroup (bits 0-3), column tiles (4-15), two-piece workgroups (16-31); a_tiles_k: one-row workgroups
        const int yb = a_tiles_k, ym = (int)((unsigned)a_nwaves >> 16);
        a_tiles_k = (a_nwaves >> 4) & 0xFFF;
        a_nwaves &= 15;
        const bool one_col = ONECOL || a_tiles_k == 1;
        const int y = tile_grid_row(one_col);
        if (y >= yb) {
            TK_SWIGLU_KERNEL_UNPACK_EARLY;
            const int strip0 = tile_grid_col(one_col) * RPW, wave = wave_id();
            const int rb = yb * kWaves;                         // rows done by one-row waves (these launches run four waves per workgroup)
            int row, strip;
            if constexpr (TILE == T_STACKED) {
                // stacked tiles: a wave's pieces lie one below the other; workgroups of 4 x 2 rows, then of 4 x 1 row, of one strip
                strip = tile_grid_col(one_col);
                const int rbs = yb * (kWaves * RPW);
                if (y - yb < ym) {
                    row = rbs + (y - yb) * (2 * kWaves) + wave * 2;
                    swiglu_row_wave<InT, CLAMP, 2, TAILED == 2, 2, true>(p, row, strip);
                } else {
                    row = rbs + ym * (2 * kWaves) + (y - yb - ym) * kWaves + wave;
                    if (row < p.R) swiglu_row_wave<InT, CLAMP, 1, TAILED == 2, 2, true>(p, row, strip);    // (whole workgroups overhang)
                }
            } else if constexpr (TILE == T_ROWC) {
                // four rows per workgroup, one per wave, the same pieces in each
                if (y - yb < ym) {
                    const int sub = y - yb;                         // two workgroups per four rows
                    row = rb + (sub >> 1) * kWaves + wave;
                    strip = strip0 + (sub & 1) * 2;
                    swiglu_row_wave<InT, CLAMP, 2, TAILED == 2, 1>(p, row, strip);
                } else {
                    const int sub = y - yb - ym;                    // four workgroups per four rows
                    row = rb + ym * 2 + (sub >> 2) * kWaves + wave;
                    strip = strip0 + (sub & 3);
                    if (row < p.R) swiglu_row_wave<InT, CLAMP, 1, TAILED == 2, 1>(p, row, strip);    // (whole workgroups overhang)
                }
            } else if (y - yb < ym) {
                const int sub = (y - yb) * kWaves + wave;       // two waves per row
                row = rb + (sub >> 1);
                strip = strip0 + (sub & 1) * 2;
                swiglu_row_wave<InT, CLAMP, 2, TAILED == 2>(p, row, strip);
            } else {
                const int sub = (y - yb - ym) * kWaves + wave;        // four waves per row
                row = rb + ((ym * kWaves) >> 1) + (sub >> 2);
                strip = strip0 + (sub & 3);
                if (row < p.R) swiglu_row_wave<InT, CLAMP, 1, TAILED == 2>(p, row, strip);    // (the grid may overhang along z)
            }
            return;
        }
    }
    SwigluParams p = TAILED ? SwigluParams{a_x, a_out, SfRef{a_sf, (int64_t)reinterpret_cast<intptr_t>(a_pe), TK_SF_ROW_F32, a_R, 0}, nullptr, nullptr,
                                           nullptr, nullptr, 0, a_R, a_H, a_nwaves, a_tiles_k, a_round_sf, a_floor, 0.0f}
                            : SwigluParams{a_x, a_out, SfRef{a_sf, a_sf_ld, a_sf_layout, a_R, a_nk}, a_ptt, a_w, a_pe, a_cnt,
                                           a_nw, a_R, a_H, a_nwaves, a_tiles_k, a_round_sf, a_floor, a_clamp};
    // T_ROW tiles always fit the columns, and their waves share nothing: on a grid that overhangs the last row the waves
    // beyond it leave at once and the others run without bounds checks, like on an exact grid
    constexpr bool ROWGUARD = TILE == T_ROW && !FULL_GRID && CLAMP != 2;
    constexpr bool FULL = FULL_GRID || ROWGUARD;
    constexpr bool ROWC = TILE == T_ROWC, ROW = TILE == T_ROW || ROWC;   // ROW: a wave's pieces lie along one row
    constexpr bool DIRECT = TILE == T_ROW;  // the wave stores its scales itself
    constexpr int GPS = kStripCols / 128;   // 4 groups per strip
    constexpr int ROWS = ROWC ? kWaves : kWaves * RPW;   // rows per tile (T_ROW: blockDim.x / 64, not used as a constant)
    constexpr int SGPR = ROWC ? RPW * GPS : GPS;   // staged groups per row
    // The counting variant loops over tiles (its grid is capped so that few workgroups touch the global
    // counters); every other variant has one workgroup per tile on a 2-D grid, which keeps integer
    // divisions and further kernel-argument loads out of the path to the first memory load.
    constexpr bool LOOP = CLAMP == 2;
    const int nwaves = (DIRECT && !TAILED) ? p.nwaves : kWaves;      // (launches that end in smaller waves run four waves per workgroup)
    const int rows = DIRECT ? nwaves : ROWS;
    using RS = RowScales<448, RPW, 16>;
    __shared__ uint32_t stage[DIRECT ? 1 : ROWS][DIRECT ? 1 : SGPR];
    // fp32 input: a wave's 2 KB of one row arrive as two whole-line loads and are dealt out to their lanes through LDS
    constexpr int XB = Raw8<InT>::kXchgBytes;
    __shared__ __attribute__((aligned(16))) uint8_t xchg[XB ? kWaves : 1][XB ? 64 * XB : 16];

    const int total = LOOP ? ((p.R + rows - 1) / rows) * p.tiles_k : 1;
    const int lane = threadIdx.x & 63, wave = wave_id();
    const bool has_weight = TAILED ? TAILED == 2 : p.pos_to_token_topk != nullptr;
    const int own = lane & 15;
    const int srow = ROWC ? wave : wave * RPW;
    ClampCounter<CLAMP> counter;

    for (int tile = LOOP ? (int)blockIdx.x : 0; tile < total; tile += LOOP ? (int)gridDim.x : 1) {
        const int tile_m = LOOP ? tile / p.tiles_k : tile_grid_row(ONECOL || p.tiles_k == 1);
        const int tile_k = LOOP ? tile - tile_m * p.tiles_k : tile_grid_col(ONECOL || p.tiles_k == 1);
        // piece r of the wave: row `row0 + (ROW ? 0 : r)`, columns from `col + (ROW ? r * 512 : 0)`
        const int strip = ROW ? tile_k * RPW : tile_k;
        const int col = strip * kStripCols + lane * 8;
        const int row0 = ROW ? tile_m * nwaves + wave : tile_m * ROWS + srow;
        if constexpr (ROWGUARD) {
            if (row0 >= p.R) return;
        }
        const uint32_t uh = (uint32_t)p.H;      // (unsigned: see swiglu_row_wave)
        const InT *x = reinterpret_cast<const InT *>(p.x) + (uint64_t)(uint32_t)row0 * (2u * uh) + (uint32_t)col;
        constexpr int kRowStep = ROW ? 0 : 1, kColStep = ROW ? kStripCols : 0;

        Raw8<InT> rg[RPW], ru[RPW];
        bool live[RPW];   // wave-uniform
        bool unused[RPW];   // pieces that read the matrix's first bytes in place of data
        // the mask entries of all rows are fetched before the first of them is looked at: one scalar
        // round trip in front of the loads instead of one per row
        int expert[RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r)
            expert[r] = (MASK && (FULL || row0 + r * kRowStep < p.R)) ? uniform_load(p.pos_to_expert + row0 + r * kRowStep) : 0;
        if constexpr (MASK && RPW == 4 && !ROW)   // all four values must exist here, so their loads are issued together above
            asm volatile("" ::"s"(expert[0]), "s"(expert[1]), "s"(expert[2]), "s"(expert[3]));
        // A masked row-wise wave with routing weights asks for its row's slot in the weight list together with its mask entry
        // (one scalar round trip for both) and for the weight itself right behind its vector loads, so that neither is waited
        // for once the data is there.  Fetched where they are used, after the data, they cost [48128, 2 x 2048] with 32768 live
        // rows 0.6 us of 61 on MI355X (2.6 us of 59 when the input is still in the last-level cache).
        constexpr bool EARLY_WEIGHT = MASK && ROW;
        int wpos = -1;
        if constexpr (EARLY_WEIGHT) {
            if (has_weight && (FULL || row0 < p.R)) wpos = uniform_load(p.pos_to_token_topk + row0);
        }
        // A wave whose row is padding writes the row's zeros and leaves: no loads, no arithmetic.  The zeros go out as
        // non-temporal 16-byte stores that cover whole lines.  Measured on MI355X, bf16, us per call, padding rows flowing
        // through the arithmetic as zeros / this way: configuration with runs of padding (32768 live rows of 47488, H = 2048)
        // 59.5 / 58.8, every third row padding ([32768, 2 x 2048]) 40.6 / 39.6.  With the write-through stores of the live
        // rows the runs cost 63.0 (16 bytes per lane) and 63.4 (8 bytes per lane), the scattered padding 38.4: a burst of
        // such stores to one stretch of memory is served slowly, and the runs are the layout this operator is made for.
        if constexpr (MASK && DIRECT && FULL) {
            if (expert[0] < 0) {
                uint8_t *piece = p.out + (int64_t)row0 * p.H + strip * kStripCols;
                if (RPW % 2 == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0) {
#pragma unroll
                    for (int i = 0; i < RPW / 2; ++i)
                        __builtin_nontemporal_store(u32x4{0u, 0u, 0u, 0u}, reinterpret_cast<u32x4 *>(piece + i * 1024 + lane * 16));
                } else {
#pragma unroll
                    for (int r = 0; r < RPW; ++r) st_stream8(piece + r * kColStep + lane * 8, u32x2{0u, 0u});
                }
                if (lane < RPW * GPS) st_stream4(reinterpret_cast<float *>(p.sf.base) + (int64_t)row0 * p.sf.ld + strip * GPS + lane, 0u);
                if constexpr (LOOP) continue;
                else return;
            }
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            live[r] = (FULL || row0 + r * kRowStep < p.R) && expert[r] >= 0;
            const InT *xr = x + (uint64_t)(uint32_t)(r * kRowStep) * (2u * uh) + r * kColStep;
            const bool piece_ok = FULL || col + r * kColStep < p.H;
            if (FULL && !MASK) {
                // (a wave-uniform 64-bit base plus a 32-bit byte offset per lane: see swiglu_row_wave)
                const uint8_t *xg = reinterpret_cast<const uint8_t *>(p.x) + (uint64_t)(uint32_t)(row0 + r * kRowStep) * (2u * uh * (uint32_t)sizeof(InT)) +
                                    (uint32_t)(r * kColStep) * (uint32_t)sizeof(InT);
                const uint32_t lane_off = (uint32_t)strip * (uint32_t)(kStripCols * sizeof(InT)) + (uint32_t)lane * (uint32_t)(8 * sizeof(InT));
                rg[r].template load_run<64>(xg + lane_off, lane);
                vmem_issue_gap();
                ru[r].template load_run<64>(xg + uh * (uint32_t)sizeof(InT) + lane_off, lane);
                if (r + 1 < RPW) vmem_issue_gap();
            } else if (FULL && XB != 0) {
                // (a padding row reads the first 2 KB of the matrix, as one run)
                const bool ok = live[r];
                const InT *src = ok ? xr : reinterpret_cast<const InT *>(p.x) + lane * 8;
                rg[r].template load_run<64>(src, lane);
                vmem_issue_gap();
                ru[r].template load_run<64>(ok ? xr + uh : src, lane);
                if (r + 1 < RPW) vmem_issue_gap();
                unused[r] = !ok;
            } else {
                // no branch around the loads (a branch would make the compiler wait for all eight loads
                // before the first row is evaluated): a padding row, and a lane beyond the last row or column,
                // reads the first bytes of the matrix, which every wave shares, and is cleared by value
                const bool ok = live[r] && piece_ok;
                const InT *src = ok ? xr : reinterpret_cast<const InT *>(p.x);
                rg[r].load(src);
                vmem_issue_gap();
                ru[r].load(ok ? xr + uh : src);
                if (r + 1 < RPW) vmem_issue_gap();
                unused[r] = !ok;
                if constexpr (sizeof(InT) != 4) {
                    if (!ok) { rg[r].zero(); ru[r].zero(); }
                }
            }
        }
        // fp32 input (two loads per piece): cleared once all loads are out, since clearing a register that a load is still to
        // fill means waiting for that load (masked fp32 [16384, 2 x 2048] 40.3 -> 38.4 us; bf16 input, whose clearing the
        // compiler already places behind the loads, measured 21.0 -> 21.2 us on a ragged batch with it and keeps its place)
        if constexpr (!(FULL && !MASK) && sizeof(InT) == 4) {
#pragma unroll
            for (int r = 0; r < RPW; ++r)
                if (unused[r]) { rg[r].zero(); ru[r].zero(); }
        }

        // (in this variant the fetch of the later arguments starts at the head of the kernel, where its paths part)
        if constexpr (TAILED != 0) fetch_late_arguments(p, CLAMP != 0, TAILED == 2, TILE != T_ROW);
        if constexpr (FULL && XB != 0) {
#pragma unroll
            for (int r = 0; r < RPW; ++r) {
                rg[r].template settle<64>(xchg[wave], lane);
                ru[r].template settle<64>(xchg[wave], lane);
            }
        }
        float wrow = 0.0f;
        if constexpr (EARLY_WEIGHT) {
            if (has_weight && live[0] && wpos >= 0 && wpos < p.num_weights) wrow = uniform_load(p.topk_weights + wpos);
        }
        // dead rows hold zeros, so they flow through as v = 0 and only their scale is overridden
        float v[RPW][8], amax[RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            float g[8], u[8];
            rg[r].get(g);
            ru[r].get(u);
            counter.apply8(g, u, p.clamp);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[r][i] = silu_mul<InT>(g[i], u[i]);
            if (has_weight) {
                const float w = EARLY_WEIGHT ? wrow : (live[r] ? row_weight(p, row0 + r * kRowStep) : 0.0f);
#pragma unroll
                for (int i = 0; i < 8; ++i) v[r][i] = v[r][i] * w;
            }
            amax[r] = group_allmax<16>(absmax8(v[r]));
        }
        RS rs;
        rs.compute(amax, p.floor_, p.round_sf != 0, lane);
        if (MASK) {
#pragma unroll
            for (int c = 0; c < RS::NC; ++c) {
                const int pick = lane & (RS::A - 1);
                const bool l0 = live[c * RS::A];
                const bool l1 = RS::A >= 2 ? live[c * RS::A + (RS::A >= 2 ? 1 : 0)] : false;
                const bool l2 = RS::A >= 4 ? live[c * RS::A + (RS::A >= 4 ? 2 : 0)] : false;
                const bool l3 = RS::A >= 4 ? live[c * RS::A + (RS::A >= 4 ? 3 : 0)] : false;
                bool mine = l0;
                if (RS::A >= 2) mine = pick == 1 ? l1 : mine;
                if (RS::A >= 4) { mine = pick == 2 ? l2 : mine; mine = pick == 3 ? l3 : mine; }
                if (!mine) { rs.own[c].sf = 0.0f; rs.own[c].e8 = 0u; }
            }
#pragma unroll
            for (int r = 0; r < RPW; ++r) rs.inv[r] = live[r] ? rs.inv[r] : 0.0f;
        }
        // lane j (< A) of a group computed the scale of piece c*A + j
        if (own < RS::A) {
#pragma unroll
            for (int c = 0; c < RS::NC; ++c) {
                if constexpr (ROWC) {
                    stage[srow][(c * RS::A + own) * GPS + (lane >> 4)] = p.sf.layout == TK_SF_COL_UE8M0 ? rs.own[c].e8 : f2u(rs.own[c].sf);
                } else if constexpr (DIRECT) {
                    // group (lane >> 4) of piece c*A + own: the wave's scales form one run of RPW * 4 floats
                    const int k = (strip + c * RS::A + own) * GPS + (lane >> 4);
                    if (FULL || (row0 < p.R && k < p.sf.nk))
                        st_stream4(reinterpret_cast<float *>(p.sf.base) + (int64_t)row0 * p.sf.ld + k, f2u(rs.own[c].sf));
                } else {
                    stage[srow + c * RS::A + own][lane >> 4] =
                        p.sf.layout == TK_SF_COL_UE8M0 ? rs.own[c].e8 : f2u(rs.own[c].sf);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r)
            if ((FULL || col + r * kColStep < p.H) && (FULL || row0 + r * kRowStep < p.R))
                quantise_store8<TK_E4M3, false>(v[r], rs.inv[r], p.out + (int64_t)(row0 + r * kRowStep) * p.H, col + r * kColStep);
        if constexpr (!DIRECT) {
            __syncthreads();
            if (ROWC) sf_store_tile_colmajor<ROWS, SGPR>(p.sf, stage, tile_m * ROWS, tile_k * SGPR);
            else if (p.sf.layout == TK_SF_ROW_F32) sf_store_tile_rowmajor<ROWS, SGPR>(p.sf, stage, GPS, tile_m * ROWS, tile_k * GPS);
            else sf_store_tile_colmajor<ROWS, SGPR>(p.sf, stage, tile_m * ROWS, tile_k * SGPR);
            if (LOOP && (int)gridDim.x < total) __syncthreads();   // stage is reused by the next tile
        }
    }
    counter.flush(p.clamped_count);
}

// Short rows (H fills less than 80 % of its 512-column strips: 768, 384, 256 ...): the rows laid end to end in units
// of one 128-column group, lane slot L serving group L / 16 of the sequence, 8 outputs per lane; only the last group of
// a row can be partly empty.  Every group is complete inside 64 lanes, so the reduction and the shared scale arithmetic
// are those of the tiled kernel; rows differ from lane to lane, so mask and weight are read per lane, and each scale is
// stored by one lane (all three layouts).  CLAMP: 0 none, 1 clamp (the counting variant stays with the tiled kernel).
template <typename InT, int CLAMP, int RPW>
__global__ __launch_bounds__(kThreads) void swiglu_cast_flat_kernel(TK_SWIGLU_KERNEL_ARGS) {
    TK_SWIGLU_KERNEL_UNPACK;
    constexpr int LPG = 16;
    using RS = RowScales<448, RPW, LPG>;
    const int lane = threadIdx.x & 63, wave = wave_id(), own = lane & 15;
    const int gpr = p.tiles_k;   // groups per row
    const InT *xb = reinterpret_cast<const InT *>(p.x);
    ClampCounter<CLAMP> counter;

    // Mask entries and weight indices of all slots are asked for first, then the data of all slots, then the weights: a
    // load whose address hangs on a loaded value waits for every load issued before it, so with a slot's mask entry read
    // behind the previous slot's data a wave had one slot's data in flight at a time ([32768, 2 x 768] bf16 22.3 us).
    int row[RPW], grp[RPW], expert[RPW], wpos[RPW];
    bool inside[RPW], live[RPW];
    Raw8<InT> rg[RPW], ru[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        const unsigned slot = (unsigned)((blockIdx.x * kWaves + wave) * RPW + r);
        const unsigned gs = (slot * 64u + (unsigned)lane) / (unsigned)LPG;
        // gs / gpr by multiplication: with floor(2^32 / gpr) the quotient comes out exact or one too small
        unsigned q = __umulhi(gs, (unsigned)p.nwaves), rem = gs - q * (unsigned)gpr;
        if (rem >= (unsigned)gpr) { ++q; rem -= (unsigned)gpr; }
        row[r] = (int)q;
        grp[r] = (int)rem;
        inside[r] = row[r] < p.R && grp[r] * 128 + own * 8 < p.H;
        expert[r] = 0;
        wpos[r] = -1;
    }
    // (one branch per table with the loads of all slots inside: a value that is loaded on one side of a branch and set on the
    // other is waited for before the branch ends)
    if (p.pos_to_expert) {
#pragma unroll
        for (int r = 0; r < RPW; ++r) expert[r] = p.pos_to_expert[row[r] < p.R ? row[r] : 0];      // (lanes beyond the last row read row 0's entry)
    }
    if (p.pos_to_token_topk) {
#pragma unroll
        for (int r = 0; r < RPW; ++r) wpos[r] = p.pos_to_token_topk[row[r] < p.R ? row[r] : 0];
    }
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        const int col = grp[r] * 128 + own * 8;
        live[r] = row[r] < p.R && expert[r] >= 0;
        // no branch around the loads: a padding row, and a lane beyond the matrix, reads its first bytes and is cleared by value
        const bool ok = inside[r] && live[r];
        const InT *src = ok ? xb + (int64_t)row[r] * (2 * (int64_t)p.H) + col : xb;
        rg[r].load(src);
        vmem_issue_gap();
        ru[r].load(ok ? src + p.H : src);
        vmem_issue_gap();
    }
#pragma unroll
    for (int r = 0; r < RPW; ++r)      // (cleared once all loads are out)
        if (!(inside[r] && live[r])) { rg[r].zero(); ru[r].zero(); }
    float w[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) w[r] = 0.0f;
    if (p.pos_to_token_topk) {
        bool has[RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            has[r] = live[r] && wpos[r] >= 0 && wpos[r] < p.num_weights;
            w[r] = p.topk_weights[has[r] ? wpos[r] : 0];
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) w[r] = has[r] ? w[r] : 0.0f;
    }

    float v[RPW][8], amax[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        float g[8], u[8];
        rg[r].get(g);
        ru[r].get(u);
        counter.apply8(g, u, p.clamp);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[r][i] = silu_mul<InT>(g[i], u[i]);
        if (p.pos_to_token_topk) {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[r][i] = v[r][i] * w[r];
        }
        amax[r] = group_allmax<16>(absmax8(v[r]));
    }
    RS rs;
    rs.compute(amax, p.floor_, p.round_sf != 0, lane);
    // lane j (< A) of a group computed the scale of slot c*A + j: its row and group are chosen by value
    if (own < RS::A) {
#pragma unroll
        for (int c = 0; c < RS::NC; ++c) {
            int m = row[c * RS::A], k = grp[c * RS::A];
            bool alive = live[c * RS::A];
            if (RS::A >= 2 && own == 1) { m = row[c * RS::A + 1]; k = grp[c * RS::A + 1]; alive = live[c * RS::A + 1]; }
            Scale sc = rs.own[c];
            if (!alive) { sc.sf = 0.0f; sc.e8 = 0u; }      // padding rows carry zero scales
            if (m < p.R) sf_store(p.sf, m, k, sc);
        }
    }
#pragma unroll
    for (int r = 0; r < RPW; ++r)
        if (inside[r]) quantise_store8<TK_E4M3, false>(v[r], live[r] ? rs.inv[r] : 0.0f, p.out + (int64_t)row[r] * p.H, grp[r] * 128 + own * 8);
}

// One scale per row (group == H): a workgroup per row.  Rows of up to ITER * 2048 outputs (ITER = 1..4) are
// evaluated once and held in registers between the amax and the conversion; ITER == 0 takes longer rows and
// evaluates the activation twice (amax pass, then convert pass; the second read comes from L2).  Row-major scales
// only.  Measured on MI355X, bf16 [16384, 2 x 4096]: 79.2 us in two passes (90.7 us with the clamp), 51.4 us held;
// fp32: 150.7 -> 102.2 us.
template <typename InT, int CLAMP, int ITER>
__global__ __launch_bounds__(kThreads) void swiglu_rowgroup_kernel(TK_SWIGLU_KERNEL_ARGS) {
    TK_SWIGLU_KERNEL_UNPACK;
    __shared__ uint32_t part[kThreads / 16];
    const InT *xb = reinterpret_cast<const InT *>(p.x);
    const int nt = p.nwaves * 64;   // threads of the workgroup: the fewest whole waves that cover a row in ITER pieces
    ClampCounter<CLAMP> counter;
    for (int row = blockIdx.x; row < p.R; row += gridDim.x) {
        // (the row's entry comes through the scalar path: as a vector load it is waited for by every lane in front of the row's data)
        const bool live = p.pos_to_expert == nullptr || uniform_load(p.pos_to_expert + row) >= 0;
        uint8_t *out_row = p.out + (int64_t)row * p.H;
        float *sf_row = reinterpret_cast<float *>(p.sf.base) + (int64_t)row * p.sf.ld;
        if (!live) {
            for (int col = threadIdx.x * 8; col < p.H; col += nt * 8) st_stream8(out_row + col, u32x2{0u, 0u});
            if (threadIdx.x == 0) sf_row[0] = 0.0f;
            continue;
        }
        const InT *x = xb + (int64_t)row * (2 * (int64_t)p.H);
        const float w = p.pos_to_token_topk ? row_weight(p, row) : 1.0f;
        float amax = 0.0f, inv = 0.0f;
        constexpr int NH = ITER > 0 ? ITER : 1;
        float held[NH][8];
        if constexpr (ITER > 0) {
            Raw8<InT> rg[NH], ru[NH];
#pragma unroll
            for (int i = 0; i < ITER; ++i) {
                // a lane beyond the end of the row reads the row's first elements (no branch around the loads)
                const int col = (i * nt + threadIdx.x) * 8;
                const int c = col < p.H ? col : 0;
                rg[i].load(x + c);
                ru[i].load(x + p.H + c);
            }
#pragma unroll
            for (int i = 0; i < ITER; ++i) {
                const int col = (i * nt + threadIdx.x) * 8;
                float g[8], u[8];
                rg[i].get(g);
                ru[i].get(u);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    counter.apply(g[e], u[e], p.clamp, col < p.H);
                    held[i][e] = silu_mul<InT>(g[e], u[e]);
                    if (p.pos_to_token_topk) held[i][e] = held[i][e] * w;
                }
                if (col < p.H) amax = __builtin_fmaxf(amax, absmax8(held[i]));
            }
        }
        for (int pass = ITER > 0 ? 1 : 0; pass < 2; ++pass) {
            if (pass == 1) {
                amax = group_allmax<16>(amax);
                __syncthreads();   // previous row's readers of `part` are done
                if ((threadIdx.x & 15) == 0) part[threadIdx.x >> 4] = f2u(amax);
                __syncthreads();
                uint32_t m = 0;
#pragma unroll
                for (int i = 0; i < kThreads / 16; ++i) m = umax(m, i * 16 < nt ? part[i] : 0u);
                const Scale sc = make_scale<448>(u2f(m), p.floor_, p.round_sf != 0);
                inv = sc.inv;
                if (threadIdx.x == 0) sf_row[0] = sc.sf;
                if constexpr (ITER > 0) {
#pragma unroll
                    for (int i = 0; i < ITER; ++i) {
                        const int col = (i * nt + threadIdx.x) * 8;
                        if (col < p.H) quantise_store8<TK_E4M3, false>(held[i], inv, out_row, col);
                    }
                    continue;
                }
            }
            for (int col = threadIdx.x * 8; col < p.H; col += nt * 8) {
                Raw8<InT> rg, ru;
                rg.load_cached(x + col);
                ru.load_cached(x + p.H + col);
                float g[8], u[8], v[8];
                rg.get(g);
                ru.get(u);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    counter.apply(g[i], u[i], p.clamp, pass == 0);
                    v[i] = silu_mul<InT>(g[i], u[i]);
                    if (p.pos_to_token_topk) v[i] = v[i] * w;
                }
                if (pass == 0) amax = __builtin_fmaxf(amax, absmax8(v));
                else quantise_store8<TK_E4M3, false>(v, inv, out_row, col);
            }
        }
    }
    counter.flush(p.clamped_count);
}

// Pieces per wave of the tiled kernel.  Measured on MI355X at [8192, 4096] bf16 (us per call, row-major
// scales, pieces = rows): 1 row 16.5, 2 rows 15.7, 4 rows 15.0.  With the four pieces taken from one row
// (T_ROW) instead of four rows: 14.75 -> 14.63.  fp32 input, whose pieces are twice the bytes (sixteen
// 16-byte loads per lane with 4 pieces), is better off with 2: [16384, 2 x 2048] 59.5 -> 52.1 us,
// [16384, 2 x 4096] 116.2 -> 98.2 us.
template <typename InT> constexpr int swiglu_pieces() { return sizeof(InT) == 4 ? 2 : 4; }

// Waves the current GPU holds at once at this kernel's occupancy (8 per SIMD, 4 SIMDs per compute unit).
static int64_t wave_slots() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus = n;
    }
    return (int64_t)cus * 32;
}

template <typename InT, int CLAMP, int RPW, int TILE>
static void launch_swiglu_tiled(SwigluParams &p, int max_blocks, hipStream_t stream) {
    // T_ROW, rows per workgroup (= waves), us per call at [8192, 4096] dense / [48128, 4096] with a third of the rows
    // masked: 1: 14.9 / 61.6, 2: 14.85 / 62.1, 4: 14.68 / 62.9, 8: 15.15 / 63.4.  A masked batch is better off with
    // single-wave workgroups: a wave whose row is padding is done at once and frees its slot alone.  So is a launch of more
    // than 3.5 times the GPU's wave slots (beyond those that end in smaller waves, below), where the slots are refilled
    // several times over and a wave that is done need not wait for the three others of its workgroup to be replaced
    // (four waves / one, bf16: [47360, 2 x 2048] 73.6 / 72.5, [65536, 2 x 2048] 101.1 / 99.0, [16384, 2 x 8192] 100.5 / 98.4,
    // [131072, 2 x 2048] 211.1 / 209.2; fp32: [16384, 2 x 2048] 48.4 / 47.4, [32768, 2 x 2048] 93.9 / 92.1).
    const bool many_turns = CLAMP != 2 && (int64_t)p.R * (p.H / kStripCols) / RPW * 2 > wave_slots() * 7;
    const int waves = TILE == T_ROW && (p.pos_to_expert || many_turns) ? 1 : kWaves;
    const int rows = TILE == T_ROW || TILE == T_ROWC ? waves : kWaves * RPW;
    const int cols = TILE == T_ROW || TILE == T_ROWC ? RPW * kStripCols : kStripCols;
    const int tiles_m = (p.R + rows - 1) / rows;
    p.tiles_k = (p.H + cols - 1) / cols;
    p.nwaves = waves;
    const int total = tiles_m * p.tiles_k;
    const dim3 block(64 * waves);
    const dim3 grid = CLAMP == 2 ? dim3((unsigned)((max_blocks > 0 && max_blocks < total) ? max_blocks : total))
                                 : tile_grid(p.tiles_k, tiles_m);
    const bool full = p.R % rows == 0 && p.H % cols == 0 && (CLAMP == 2 || tile_grid_exact(p.tiles_k, tiles_m));
    // the row-wise tiles of the common widths (H = 2048: one column of tiles) get a kernel of their own: the
    // run-time test costs the [8192, 2 x 2048] call 0.2 us
    constexpr bool ROWWISE = TILE == T_ROW || TILE == T_ROWC;
    const bool onecol = ROWWISE && p.tiles_k == 1;
    if constexpr (CLAMP != 2 && RPW == 4) {
        // Finer-grained waves at the end of the launch (see the kernel): the last rows by two-piece waves, 2.2 times the GPU's
        // wave slots of them but at most 55 % of the rows, and of those the last by one-piece waves, 0.6 times the slots, at
        // most 15 % of the rows.  For launches of 0.75 to 3.5 times the GPU's wave slots in one-row waves, where it was
        // measured to pay (bf16, us per call without / with): [6144, 2 x 2048] 11.40 / 11.31, [8192, 2 x 2048] 14.54 / 14.13,
        // [10240, 2 x 2048] 17.84 / 17.18, [16384, 2 x 2048] 26.92 / 26.50, [8192, 2 x 4096] 26.59 / 26.17, [2048, 2 x 8192]
        // 14.77 / 14.32, [24576, 2 x 2048] 42.92 / 42.54; smaller and larger launches lose with it ([4096, 2 x 2048] 8.11 / 8.48,
        // [32768, 2 x 2048] 57.37 / 57.71), and so does a masked batch ([48128, 2 x 2048], a third of the rows padding, 59.9 / 61.8).
        const int64_t slots = wave_slots(), ppr = p.H / kStripCols, row_waves = (int64_t)p.R * ppr / RPW;
        int rs = (int)std::min<int64_t>((int64_t)p.R * 15 / 100, slots * 6 / 10 / ppr) / 4 * 4;
        int rm = (int)std::min<int64_t>((int64_t)p.R * 55 / 100, slots * 22 / 10 / ppr) / 4 * 4;
        int rb = p.R - rm - rs;
        int64_t ym = (int64_t)rm * 2 / waves, ys = (int64_t)rs * 4 / waves, yb = rb / waves;
        if constexpr (TILE == T_STACKED) {
            // stacked tiles of 16 rows, then workgroups of 8 rows (two per wave), then of 4 rows, each on one strip of 512 columns
            rs = rs / 8 * 8;
            rb = (p.R - rm - rs) / rows * rows;
            rm = p.R - rb - rs;
            yb = rb / rows; ym = rm / (2 * kWaves); ys = rs / kWaves;
        }
        if (full && !p.pos_to_expert && waves == kWaves && row_waves * 4 >= slots * 3 && row_waves * 2 <= slots * 7 && rs > 0 && p.tiles_k <= 0xFFF &&
            ym <= 0xFFFF) {
            const dim3 tgrid = tile_grid(p.tiles_k, (int)(yb + ym + ys));
            p.nwaves = waves | (p.tiles_k << 4) | ((int)ym << 16);
            p.tiles_k = (int)yb;
            p.pos_to_expert = reinterpret_cast<const int32_t *>(static_cast<intptr_t>(p.sf.ld));     // a preloaded place for it
#define TK_SWIGLU_LAUNCH_TAILED(W_)                                                                                             \
    do {                                                                                                                        \
        if (onecol)                                                                                                             \
            hipLaunchKernelGGL((swiglu_cast_kernel<InT, CLAMP, RPW, TILE, true, false, true, W_>), tgrid, block, 0, stream,     \
                               TK_SWIGLU_LAUNCH_ARGS(p));                                                                       \
        else                                                                                                                    \
            hipLaunchKernelGGL((swiglu_cast_kernel<InT, CLAMP, RPW, TILE, true, false, false, W_>), tgrid, block, 0, stream,    \
                               TK_SWIGLU_LAUNCH_ARGS(p));                                                                       \
    } while (0)
            if (p.pos_to_token_topk) TK_SWIGLU_LAUNCH_TAILED(2);
            else TK_SWIGLU_LAUNCH_TAILED(1);
#undef TK_SWIGLU_LAUNCH_TAILED
            return;
        }
    }
#define TK_SWIGLU_LAUNCH(FULL_, MASK_)                                                                                          \
    do {                                                                                                                        \
        if (onecol)                                                                                                             \
            hipLaunchKernelGGL((swiglu_cast_kernel<InT, CLAMP, RPW, TILE, FULL_, MASK_, ROWWISE>), grid, block, 0, stream,      \
                               TK_SWIGLU_LAUNCH_ARGS(p));                                                                       \
        else                                                                                                                    \
            hipLaunchKernelGGL((swiglu_cast_kernel<InT, CLAMP, RPW, TILE, FULL_, MASK_, false>), grid, block, 0, stream,        \
                               TK_SWIGLU_LAUNCH_ARGS(p));                                                                       \
    } while (0)
    if (p.pos_to_expert) {
        // A masked batch in row-wise tiles takes one row per workgroup, so its grid fits unless it has more than one plane of
        // row tiles (several columns of tiles, more than 32768 rows); the counting variant's grid is flat and always fits.
        constexpr bool kAlwaysExact = TILE == T_ROW && CLAMP == 2;
        if (full || kAlwaysExact) TK_SWIGLU_LAUNCH(true, true);
        else if constexpr (TILE == T_ROW && !kAlwaysExact)
            hipLaunchKernelGGL((swiglu_cast_kernel<InT, CLAMP, RPW, TILE, false, true, false>), grid, block, 0, stream, TK_SWIGLU_LAUNCH_ARGS(p));
        else if constexpr (!kAlwaysExact) TK_SWIGLU_LAUNCH(false, true);
    } else {
        if (full) TK_SWIGLU_LAUNCH(true, false);
        else TK_SWIGLU_LAUNCH(false, false);
    }
#undef TK_SWIGLU_LAUNCH
}

template <typename InT, int CLAMP>
static hipError_t launch_swiglu_2(SwigluParams &p, bool row_group, int max_blocks, hipStream_t stream) {
    constexpr int kPieces = swiglu_pieces<InT>();
    if constexpr (CLAMP != 2) {
        // rows that fill less than 80 % of their 512-column strips: [87296, 2 x 768] bf16 58.2 us tiled
        const int64_t strips = (p.H + kStripCols - 1) / kStripCols, gpr = p.H / 128, lanes = (int64_t)p.R * gpr * 16;
        if (!row_group && p.H * 5 < strips * kStripCols * 4 && lanes < INT32_MAX - 4 * kThreads) {
            constexpr int RPW = 2;   // slots per wave; [32768, 2 x 768] bf16: 24.1 / 23.7 / 30.6 us with 1 / 2 / 4
            static_assert(RowScales<448, RPW, 16>::A == 2, "the flat kernel selects between two slots");
            p.tiles_k = (int)gpr;
            p.nwaves = (int)(uint32_t)(gpr == 1 ? 0xFFFFFFFFull : (1ull << 32) / (uint64_t)gpr);   // reciprocal of gpr for the kernel's divisions
            hipLaunchKernelGGL((swiglu_cast_flat_kernel<InT, CLAMP, RPW>), dim3((unsigned)((lanes + kThreads * RPW - 1) / (kThreads * RPW))),
                               dim3(kThreads), 0, stream, TK_SWIGLU_LAUNCH_ARGS(p));
            return hipGetLastError();
        }
    }
    if (row_group) {
        const int grid = max_blocks > 0 && max_blocks < p.R ? max_blocks : p.R;
        // the fewest pieces per thread (1..4) with which at most 4 waves cover a row, then the fewest waves that do
        // (bf16 [65536, 2 x 512]: 65 us with 256 threads per row whatever its length)
        int iter = 0, waves = kWaves;
        for (int it = 1; it <= 4 && iter == 0; ++it) {
            const int w = (p.H + it * kStripCols - 1) / (it * kStripCols);
            if (w <= kWaves) { iter = it; waves = w; }
        }
        p.nwaves = waves;
#define TK_ROWGROUP_LAUNCH(ITER) \
    hipLaunchKernelGGL((swiglu_rowgroup_kernel<InT, CLAMP, ITER>), dim3(grid), dim3(64 * waves), 0, stream, TK_SWIGLU_LAUNCH_ARGS(p))
        switch (iter) {
            case 1: TK_ROWGROUP_LAUNCH(1); break;
            case 2: TK_ROWGROUP_LAUNCH(2); break;
            case 3: TK_ROWGROUP_LAUNCH(3); break;
            case 4: TK_ROWGROUP_LAUNCH(4); break;
            default: TK_ROWGROUP_LAUNCH(0); break;
        }
#undef TK_ROWGROUP_LAUNCH
    } else if (p.sf.layout != TK_SF_ROW_F32 && p.H % (kPieces * kStripCols) == 0) {
        // (other H, where the last column tile of a row is partly empty and the loads are bounds-checked, are
        // better off with stacked tiles: [16384, 2 x 2560] 35.6 us stacked, 44.2 us this way)
        launch_swiglu_tiled<InT, CLAMP, kPieces, T_ROWC>(p, max_blocks, stream);
    } else if (p.H % (kPieces * kStripCols) == 0) {
        launch_swiglu_tiled<InT, CLAMP, kPieces, T_ROW>(p, max_blocks, stream);
    } else {
        // (tiles of a few rows with the workgroup's waves side by side, as the per-token cast uses them for row-major
        // scales, are no faster here: bf16 [26112, 2 x 2560] 52.9 us against 51.2 us, [21760, 2 x 3072] 53.1 against 51.5)
        launch_swiglu_tiled<InT, CLAMP, kPieces, T_STACKED>(p, max_blocks, stream);
    }
    return hipGetLastError();
}

template <typename InT>
static hipError_t launch_swiglu_1(SwigluParams &p, int clamp_mode, bool row_group, int max_blocks, hipStream_t stream) {
    switch (clamp_mode) {
        case 0: return launch_swiglu_2<InT, 0>(p, row_group, max_blocks, stream);
        case 1: return launch_swiglu_2<InT, 1>(p, row_group, max_blocks, stream);
        default: return launch_swiglu_2<InT, 2>(p, row_group, max_blocks, stream);
    }
}

}  // namespace tk

using namespace tk;

extern "C" int tk_check_swiglu_per_token_cast(const void *x, int x_dtype, int64_t R, int64_t H, const void *out,
                                              const void *sf, int64_t sf_ld, int group, int sf_layout, int round_sf,
                                              float sf_clamp_min, const int32_t *pos_to_token_topk,
                                              const float *topk_weights, int64_t num_weights,
                                              const int32_t *pos_to_expert, int use_clamp, float clamp,
                                              const int64_t *clamped_count) {
    (void)pos_to_expert;
    if (x_dtype != TK_BF16 && x_dtype != TK_F32) return TK_ERR_BAD_DTYPE;
    if (sf_layout < TK_SF_ROW_F32 || sf_layout > TK_SF_COL_UE8M0) return TK_ERR_BAD_LAYOUT;
    if (sf_layout == TK_SF_COL_UE8M0 && !round_sf) return TK_ERR_BAD_LAYOUT;
    if (R < 0 || H <= 0 || H % 128 != 0) return TK_ERR_BAD_SHAPE;
    if (R > INT32_MAX - 64 || H > (INT32_MAX - 1024) / 2) return TK_ERR_TOO_LARGE;
    if (2 * H * (x_dtype == TK_BF16 ? 2 : 4) > (int64_t)UINT32_MAX) return TK_ERR_TOO_LARGE;   // byte offsets inside a row are 32-bit
    if (group != 128 && group != H) return TK_ERR_BAD_GROUP;
    if (group != 128 && sf_layout != TK_SF_ROW_F32) return TK_ERR_BAD_LAYOUT;
    if (clamped_count && !use_clamp) return TK_ERR_BAD_MODE;
    if (use_clamp && !(clamp == clamp)) return TK_ERR_BAD_VALUE;
    if (sf_clamp_min != sf_clamp_min) return TK_ERR_BAD_VALUE;
    if (pos_to_token_topk && (!topk_weights || num_weights <= 0)) return TK_ERR_NULL_POINTER;
    if (R == 0) return TK_OK;
    if (!x || !out || !sf) return TK_ERR_NULL_POINTER;
    if (!aligned_to(x, 16) || !aligned_to(out, 8) || !aligned_to(sf, 4)) return TK_ERR_MISALIGNED;
    if (clamped_count && !aligned_to(clamped_count, 8)) return TK_ERR_MISALIGNED;
    const int64_t nk = H / group;
    const int64_t need = sf_layout == TK_SF_ROW_F32 ? nk : (sf_layout == TK_SF_COL_F32 ? R : 4 * R);
    if (sf_ld < need) return TK_ERR_BAD_STRIDE;
    if (sf_layout == TK_SF_COL_UE8M0 && sf_ld % 4 != 0) return TK_ERR_MISALIGNED;
    const int64_t tiles = ((R + 3) / 4) * ((H + kStripCols - 1) / kStripCols);
    if (tiles > INT32_MAX - 8) return TK_ERR_TOO_LARGE;
    return TK_OK;
}

extern "C" int tk_swiglu_per_token_cast(const void *x, int x_dtype, int64_t R, int64_t H, void *out, void *sf,
                                        int64_t sf_ld, int group, int sf_layout, int round_sf, float sf_clamp_min,
                                        const int32_t *pos_to_token_topk, const float *topk_weights,
                                        int64_t num_weights, const int32_t *pos_to_expert, int use_clamp,
                                        float clamp, int64_t *clamped_count, int max_blocks, void *stream) {
    const int rc = tk_check_swiglu_per_token_cast(x, x_dtype, R, H, out, sf, sf_ld, group, sf_layout, round_sf,
                                                  sf_clamp_min, pos_to_token_topk, topk_weights, num_weights,
                                                  pos_to_expert, use_clamp, clamp, clamped_count);
    if (rc != TK_OK || R == 0) return rc;
    const bool row_group = group != 128;
    SwigluParams p;
    p.x = x;
    p.out = static_cast<uint8_t *>(out);
    p.sf = SfRef{sf, sf_ld, sf_layout, (int)R, (int)(H / group)};
    p.pos_to_token_topk = pos_to_token_topk;
    p.topk_weights = topk_weights;
    p.pos_to_expert = pos_to_expert;
    p.clamped_count = reinterpret_cast<unsigned long long *>(clamped_count);
    p.num_weights = num_weights;
    p.R = (int)R;
    p.H = (int)H;
    p.nwaves = p.tiles_k = 0;
    p.round_sf = round_sf;
    p.floor_ = sf_clamp_min < 0.0f ? 1e-4f : sf_clamp_min;
    p.clamp = clamp;
    const int clamp_mode = use_clamp ? (clamped_count ? 2 : 1) : 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const hipError_t e = x_dtype == TK_BF16 ? launch_swiglu_1<bf16_t>(p, clamp_mode, row_group, max_blocks, s)
                                            : launch_swiglu_1<float>(p, clamp_mode, row_group, max_blocks, s);
    return (int)e;
}
