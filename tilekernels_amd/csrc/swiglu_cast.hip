// Fused SwiGLU + per-token (1 x 128, or one scale per row) E4M3 quantisation for gfx950.
//
// x[R, 2H]: gate = columns [0, H), up = columns [H, 2H).  The activation never touches HBM: a lane
// loads 8 gate and 8 up values (two 16-byte loads for bf16), computes v = g/(1+exp(-g))*u in fp32,
// and the 16 lanes that share a 128-column group reduce |v| with DPP, derive the scale and
// convert straight to packed FP8.  Tiling is the one of the per-token cast: 16 rows x 512 output
// columns per workgroup, 4 rows per wave, all eight loads of a lane in flight before first use.
// Padding rows (pos_to_expert < 0) are not read; zeros are written for their codes and scales.
//
// Reference semantics: tile_kernels/quant/swiglu_forward_and_per_token_cast_kernel.py:61-170,
// tile_kernels/torch/swiglu.py:62-86.
#include <stdlib.h>

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
    int tiles_m, tiles_k;
    int round_sf;
    int persistent;      // 1: workgroups stride over tiles by gridDim.x
    float floor_;        // amax lower clamp
    float clamp;
};

// Math variants for silu(g) = g / (1 + exp(-g)):
//   0  v_exp_f32 on g * -log2(e), v_rcp_f32: ~12 issue slots per element, a few ulp
//   1  libm-grade expf and an IEEE-rounded division: closest to the CPU evaluation, most ALU work
//   2  v_exp_f32 with a two-term argument and an fma-corrected quotient: ~1.5 ulp
template <int MATH> __device__ __forceinline__ float silu_mul(float g, float u) {
    if (MATH == 1) {
        const float e = expf(-g);
        const float d = 1.0f + e;
        return g / d * u;
    } else if (MATH == 0) {
        const float e = __builtin_amdgcn_exp2f(g * -1.4426950408889634f);
        const float d = 1.0f + e;
        return g * __builtin_amdgcn_rcpf(d) * u;
    } else {
        // -g * log2(e) as hi + lo, so that the rounding of the product does not reach the result
        const float nh = -1.4426950216293335f;        // float(-log2 e)
        const float nl = -1.9259629911266175e-8f;     // -log2 e - nh
        const float tp = g * nh;
        const float tl = __builtin_fmaf(g, nl, __builtin_fmaf(g, nh, -tp));
        // exp(-g) overflows for g < -88.7; capping the exponent keeps e and d finite, so the
        // corrected quotient below underflows to -0 / a negligible value instead of inf * 0
        const float th = __builtin_fminf(tp, 127.0f);
        float e = __builtin_amdgcn_exp2f(th);
        e = __builtin_fmaf(e, tl * 0.6931471805599453f, e);
        const float d = 1.0f + e;
        const float r = __builtin_amdgcn_rcpf(d);
        const float q0 = g * r;
        const float q = __builtin_fmaf(__builtin_fmaf(-d, q0, g), r, q0);
        return q * u;
    }
}

// CLAMP: 0 none, 1 clamp, 2 clamp and count
template <int CLAMP> struct ClampCounter {
    uint32_t n0 = 0, n1 = 0, n2 = 0;
    __device__ __forceinline__ void apply(float &g, float &u, float c) {
        if (CLAMP == 0) return;
        if (CLAMP == 2) { n0 += g > c; n1 += u > c; n2 += u < -c; }
        g = __builtin_fminf(g, c);
        u = __builtin_fminf(__builtin_fmaxf(u, -c), c);
    }
    // one global atomic per counter and workgroup
    __device__ __forceinline__ void flush(unsigned long long *dst) {
        if (CLAMP != 2) return;
        __shared__ unsigned long long acc[3];
        if (threadIdx.x < 3) acc[threadIdx.x] = 0ull;
        __syncthreads();
        if (n0) atomicAdd(&acc[0], (unsigned long long)n0);
        if (n1) atomicAdd(&acc[1], (unsigned long long)n1);
        if (n2) atomicAdd(&acc[2], (unsigned long long)n2);
        __syncthreads();
        if (threadIdx.x < 3 && acc[threadIdx.x]) atomicAdd(&dst[threadIdx.x], acc[threadIdx.x]);
    }
};

__device__ __forceinline__ float row_weight(const SwigluParams &p, int row) {
    const int pos = p.pos_to_token_topk[row];
    return (pos >= 0 && pos < p.num_weights) ? p.topk_weights[pos] : 0.0f;
}

template <typename InT, int CLAMP, int MATH>
__global__ __launch_bounds__(kThreads) void swiglu_cast_kernel(const SwigluParams p) {
    constexpr int GPS = kStripCols / 128;   // 4 groups per strip
    constexpr int RPW = kTileRows / 4;
    __shared__ uint32_t stage[kTileRows][GPS];

    const int total = p.tiles_m * p.tiles_k;
    int tile = p.persistent ? (int)blockIdx.x : xcd_tile_index(total);
    const int step = p.persistent ? (int)gridDim.x : total;
    if (tile < 0) tile = total;   // surplus workgroup: no tile, but it still reaches the counter flush

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const bool leader = (lane & 15) == 0;
    const bool staged = p.sf.layout != TK_SF_ROW_F32;
    const InT *x = reinterpret_cast<const InT *>(p.x);
    ClampCounter<CLAMP> counter;

    for (; tile < total; tile += step) {
        const int tile_m = tile / p.tiles_k, tile_k = tile - tile_m * p.tiles_k;
        const int col = tile_k * kStripCols + lane * 8;
        const int kgrp = tile_k * GPS + (lane >> 4);
        const bool col_ok = col < p.H;
        const int row0 = tile_m * kTileRows + wave * RPW;

        Raw8<InT> rg[RPW], ru[RPW];
        bool live[RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const int row = row0 + r;
            live[r] = row < p.R && (p.pos_to_expert == nullptr || p.pos_to_expert[row] >= 0);
            const InT *xr = x + (int64_t)row * (2 * (int64_t)p.H) + col;
            rg[r].load(xr, live[r] && col_ok);
            ru[r].load(xr + p.H, live[r] && col_ok);
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const int row = row0 + r;
            const bool in_range = row < p.R && col_ok;
            float g[8], u[8], v[8];
            rg[r].get(g);
            ru[r].get(u);
            Scale sc;
            if (live[r]) {   // wave-uniform
                const float w = p.pos_to_token_topk ? row_weight(p, row) : 1.0f;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (col_ok) counter.apply(g[i], u[i], p.clamp);
                    v[i] = silu_mul<MATH>(g[i], u[i]);
                    if (p.pos_to_token_topk) v[i] = v[i] * w;
                }
                const float amax = group_allmax<16>(absmax8(v));
                sc = make_scale(amax, p.floor_, 448.0f, p.round_sf != 0);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = 0.0f;
                sc.sf = 0.0f; sc.inv = 0.0f; sc.e8 = 0u;
            }
            if (leader) {
                if (staged) stage[wave * RPW + r][lane >> 4] = p.sf.layout == TK_SF_COL_F32 ? f2u(sc.sf) : sc.e8;
                else if (in_range) reinterpret_cast<float *>(p.sf.base)[(int64_t)row * p.sf.ld + kgrp] = sc.sf;
            }
            if (in_range) quantise_store8<TK_E4M3, false>(v, sc.inv, p.out + (int64_t)row * p.H, col);
        }
        if (staged) {
            __syncthreads();
            sf_store_tile_colmajor<GPS>(p.sf, stage, tile_m * kTileRows, tile_k * GPS);
            __syncthreads();   // stage is reused by the next tile
        }
    }
    counter.flush(p.clamped_count);
}

// One scale per row (group == H): a workgroup per row, the activation is evaluated twice (amax
// pass, then convert pass; the second read comes from L2).  Row-major scales only.
template <typename InT, int CLAMP, int MATH>
__global__ __launch_bounds__(kThreads) void swiglu_rowgroup_kernel(const SwigluParams p) {
    __shared__ uint32_t part[kThreads / 16];
    const InT *xb = reinterpret_cast<const InT *>(p.x);
    ClampCounter<CLAMP> counter;
    for (int row = blockIdx.x; row < p.R; row += gridDim.x) {
        const bool live = p.pos_to_expert == nullptr || p.pos_to_expert[row] >= 0;
        uint8_t *out_row = p.out + (int64_t)row * p.H;
        float *sf_row = reinterpret_cast<float *>(p.sf.base) + (int64_t)row * p.sf.ld;
        if (!live) {
            for (int col = threadIdx.x * 8; col < p.H; col += kThreads * 8) *reinterpret_cast<uint2 *>(out_row + col) = make_uint2(0, 0);
            if (threadIdx.x == 0) sf_row[0] = 0.0f;
            continue;
        }
        const InT *x = xb + (int64_t)row * (2 * (int64_t)p.H);
        const float w = p.pos_to_token_topk ? row_weight(p, row) : 1.0f;
        float amax = 0.0f, inv = 0.0f;
        for (int pass = 0; pass < 2; ++pass) {
            for (int col = threadIdx.x * 8; col < p.H; col += kThreads * 8) {
                Raw8<InT> rg, ru;
                rg.load(x + col, true);
                ru.load(x + p.H + col, true);
                float g[8], u[8], v[8];
                rg.get(g);
                ru.get(u);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    if (pass == 0) counter.apply(g[i], u[i], p.clamp);
                    else ClampCounter<(CLAMP ? 1 : 0)>().apply(g[i], u[i], p.clamp);
                    v[i] = silu_mul<MATH>(g[i], u[i]);
                    if (p.pos_to_token_topk) v[i] = v[i] * w;
                }
                if (pass == 0) amax = __builtin_fmaxf(amax, absmax8(v));
                else quantise_store8<TK_E4M3, false>(v, inv, out_row, col);
            }
            if (pass == 0) {
                amax = group_allmax<16>(amax);
                __syncthreads();   // previous row's readers of `part` are done
                if ((threadIdx.x & 15) == 0) part[threadIdx.x >> 4] = f2u(amax);
                __syncthreads();
                uint32_t m = 0;
#pragma unroll
                for (int i = 0; i < kThreads / 16; ++i) m = umax(m, part[i]);
                const Scale sc = make_scale(u2f(m), p.floor_, 448.0f, p.round_sf != 0);
                inv = sc.inv;
                if (threadIdx.x == 0) sf_row[0] = sc.sf;
            }
        }
    }
    counter.flush(p.clamped_count);
}

static int swiglu_math_variant() {
    static const int v = [] {
        const char *e = getenv("TK_SWIGLU_MATH");
        const int m = e ? atoi(e) : 2;
        return (m < 0 || m > 2) ? 2 : m;
    }();
    return v;
}

template <typename InT, int CLAMP, int MATH>
static hipError_t launch_swiglu_3(const SwigluParams &p, bool row_group, int max_blocks, hipStream_t stream) {
    if (row_group) {
        const int grid = max_blocks > 0 && max_blocks < p.R ? max_blocks : p.R;
        hipLaunchKernelGGL((swiglu_rowgroup_kernel<InT, CLAMP, MATH>), dim3(grid), dim3(kThreads), 0, stream, p);
    } else {
        const int total = p.tiles_m * p.tiles_k;
        const int grid = p.persistent ? max_blocks : kNumXcd * ((total + kNumXcd - 1) / kNumXcd);
        hipLaunchKernelGGL((swiglu_cast_kernel<InT, CLAMP, MATH>), dim3(grid), dim3(kThreads), 0, stream, p);
    }
    return hipGetLastError();
}

template <typename InT, int CLAMP>
static hipError_t launch_swiglu_2(const SwigluParams &p, bool row_group, int max_blocks, hipStream_t stream) {
    switch (swiglu_math_variant()) {
        case 0: return launch_swiglu_3<InT, CLAMP, 0>(p, row_group, max_blocks, stream);
        case 1: return launch_swiglu_3<InT, CLAMP, 1>(p, row_group, max_blocks, stream);
        default: return launch_swiglu_3<InT, CLAMP, 2>(p, row_group, max_blocks, stream);
    }
}

template <typename InT>
static hipError_t launch_swiglu_1(const SwigluParams &p, int clamp_mode, bool row_group, int max_blocks, hipStream_t stream) {
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
    const int64_t tiles = ((R + kTileRows - 1) / kTileRows) * ((H + kStripCols - 1) / kStripCols);
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
    p.tiles_m = (int)((R + kTileRows - 1) / kTileRows);
    p.tiles_k = (int)((H + kStripCols - 1) / kStripCols);
    p.round_sf = round_sf;
    p.persistent = (max_blocks > 0 && max_blocks < p.tiles_m * p.tiles_k) ? 1 : 0;
    p.floor_ = sf_clamp_min < 0.0f ? 1e-4f : sf_clamp_min;
    p.clamp = clamp;
    const int clamp_mode = use_clamp ? (clamped_count ? 2 : 1) : 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const hipError_t e = x_dtype == TK_BF16 ? launch_swiglu_1<bf16_t>(p, clamp_mode, row_group, max_blocks, s)
                                            : launch_swiglu_1<float>(p, clamp_mode, row_group, max_blocks, s);
    return (int)e;
}
