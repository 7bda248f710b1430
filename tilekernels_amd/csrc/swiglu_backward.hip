// Fused SwiGLU backward + per-token (1 x 32 / 1 x 128) E4M3 quantisation of the input gradient for gfx950.
//
// Inputs : x[R, 2H] E4M3 codes with fp32 scales [R, 2H/N] (the forward input as it was quantised),
//          grad_out[R, H] bf16, routing weights [T*K] fp32 and the two index maps of the expanded layout.
// Outputs: out[R, H] bf16          = silu(g) * u * w            (the forward activation, recomputed)
//          x_grad[R, 2H] bf16      = [d/dgate | d/dup]
//          x_grad codes[R, 2H] E4M3 with scales [R, 2H/N] fp32, quantised from the fp32 gradient
//          weight_grad[T*K] fp32   = sum_c grad_out * silu(g) * u per routed row, 0 for unrouted pairs
//
// A workgroup owns RPW whole rows: its W waves stand side by side, 512 columns each, and step along
// the row together, so the row's dot product for weight_grad is finished inside the workgroup (lane
// partials, a wave reduction, one LDS exchange) and written exactly once, in a fixed order.  A lane
// holds 8 consecutive gate columns and the 8 matching up columns: two 8-byte code loads, one 16-byte
// gradient load and two scale loads per row, three 16-byte and two 8-byte stores.  Nothing but the
// results touches HBM: per column 4 bytes are read and 8 written (plus 16/N bytes of scales).
//
// Reference semantics: tile_kernels/quant/swiglu_backward_and_per_token_cast_kernel.py:16-164,
// tile_kernels/torch/swiglu.py:98-227.
#include "swiglu_math.hpp"
#include "tk_device.hpp"
#include "tk_host.hpp"

namespace tk {

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ u32x4 pack_bf16x8(const float (&v)[8]) {
    u32x4 w;
    w.x = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[0], v[1]}), bf16x2));
    w.y = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[2], v[3]}), bf16x2));
    w.z = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[4], v[5]}), bf16x2));
    w.w = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{v[6], v[7]}), bf16x2));
    return w;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}

constexpr int kBwdMaxWaves = 8;

// Waves per workgroup for a row of `strips` 512-column strips: all of them up to 8; beyond that the
// largest of 8..4 that divides the count (no idle wave in the last pass), else 8.
static int backward_waves(int strips) {
    if (strips <= kBwdMaxWaves) return strips;
    for (int w = kBwdMaxWaves; w >= 4; --w)
        if (strips % w == 0) return w;
    return kBwdMaxWaves;
}

// Kernel arguments, in the order they are needed: the first 14 dwords arrive preloaded in SGPRs and
// hold everything the input addresses are made of; the rest is fetched from the argument buffer
// while the first loads are in flight.
#define TK_BWD_KERNEL_ARGS                                                                                       \
    const uint8_t *x, const float *x_sf, const uint16_t *grad_out, int R, int H, int nwaves, int round_sf,        \
        uint16_t *out, uint16_t *x_grad, uint8_t *q, float *q_sf, float clamp, const int32_t *ptt,               \
        const float *weights, float *weight_grad, const int32_t *t2p, int64_t num_weights

// N: columns per scale (32 or 128), of the input and of the quantised gradient alike.
// CLAMP: the activation clamp is applied.  FULL: every wave's every strip is inside the matrix.
template <int N, bool CLAMP, int RPW, bool FULL>
__global__ __launch_bounds__(64 * kBwdMaxWaves) void swiglu_backward_kernel(TK_BWD_KERNEL_ARGS) {
    constexpr int LPG = N / 8;                 // lanes that share a scale
    using RS = RowScales<448, 2 * RPW, LPG>;   // "row" 2r is the gate half of row r, 2r+1 its up half
    __shared__ float part[kBwdMaxWaves][RPW];

    const int lane = threadIdx.x & 63, wave = wave_id();
    const int strips = (H + kStripCols - 1) / kStripCols;

    const int row0 = blockIdx.x * RPW;
    const int nsf = 2 * H / N, hsf = H / N;

    if (row0 < R) {
    float w[RPW], acc[RPW];   // w: wave-uniform
#pragma unroll
    for (int r = 0; r < RPW; ++r) w[r] = acc[r] = 0.0f;

    for (int strip = wave; strip < strips; strip += nwaves) {
        const int col = strip * kStripCols + lane * 8;
        const bool col_ok = FULL || col < H;
        const int grp = col / N;

        Raw8<e4m3in_t> rg[RPW], ru[RPW];
        Raw8<bf16_t> rgo[RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const bool ok = col_ok && (FULL || row0 + r < R);
            const int64_t row = row0 + r;
            const uint8_t *xr = x + row * (2 * (int64_t)H) + col;
            rg[r].load(xr, ok);
            vmem_issue_gap();
            ru[r].load(xr + H, ok);
            vmem_issue_gap();
            rgo[r].load(grad_out + row * (int64_t)H + col, ok);
            vmem_issue_gap();
            rg[r].s = ok ? x_sf[row * nsf + grp] : 0.0f;
            ru[r].s = ok ? x_sf[row * nsf + hsf + grp] : 0.0f;
        }

        // the rows' routing weights: two dependent scalar round trips, started only now that the
        // strip's loads are in flight (the barrier keeps the compiler from hoisting them in front)
        // arguments beyond the preloaded ones are first touched here, behind the loads: passing them
        // through an empty asm keeps the address arithmetic built on them (which is loop-invariant) from
        // being hoisted, together with the wait for their arrival, in front of the first strip's loads
        asm volatile("" : "+s"(q), "+s"(q_sf), "+s"(clamp), "+s"(ptt), "+s"(weights));
        if (strip == wave) {
            asm volatile("" ::: "memory");
#pragma unroll
            for (int r = 0; r < RPW; ++r) {
                int idx = (FULL || row0 + r < R) ? uniform_load(ptt + row0 + r) : -1;
                if (idx >= num_weights) idx = -1;
                w[r] = idx >= 0 ? uniform_load(weights + idx) : 0.0f;
            }
        }

        float dg[RPW][8], du[RPW][8], amax[2 * RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            float g[8], u[8], go[8], o[8];
            rg[r].get(g);
            ru[r].get(u);
            rgo[r].get(go);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                bool cg = false, cu = false;
                if (CLAMP) {
                    cg = g[i] > clamp;
                    cu = u[i] > clamp || u[i] < -clamp;
                    g[i] = cg ? clamp : g[i];
                    u[i] = u[i] > clamp ? clamp : u[i];
                    u[i] = u[i] < -clamp ? -clamp : u[i];
                }
                const float d = 1.0f + exp_neg<float>(g[i]);
                const float s = reciprocal(d);
                const float act = quotient_with(g[i], d, s) * u[i];
                acc[r] = __builtin_fmaf(go[i], act, acc[r]);
                o[i] = act * w[r];
                const float t = (go[i] * w[r]) * s;
                const float a = (t * u[i]) * __builtin_fmaf(g[i], 1.0f - s, 1.0f);
                const float b = t * g[i];
                dg[r][i] = cg ? 0.0f : a;
                du[r][i] = cu ? 0.0f : b;
            }
            amax[2 * r] = group_allmax<LPG>(absmax8(dg[r]));
            amax[2 * r + 1] = group_allmax<LPG>(absmax8(du[r]));
            if (col_ok && (FULL || row0 + r < R)) {
                const int64_t row = row0 + r;
                __builtin_nontemporal_store(pack_bf16x8(o), reinterpret_cast<u32x4 *>(out + row * (int64_t)H + col));
                uint16_t *xg = x_grad + row * (2 * (int64_t)H) + col;
                __builtin_nontemporal_store(pack_bf16x8(dg[r]), reinterpret_cast<u32x4 *>(xg));
                __builtin_nontemporal_store(pack_bf16x8(du[r]), reinterpret_cast<u32x4 *>(xg + H));
            }
        }

        RS rs;
        rs.compute(amax, Fmt<TK_E4M3>::floor_, round_sf != 0, lane);
        // lane j (< A) of a group computed the scale of half (c*A + j) & 1 of row (c*A + j) >> 1
        if ((lane & (LPG - 1)) < RS::A && col_ok) {
#pragma unroll
            for (int c = 0; c < RS::NC; ++c) {
                const int rp = c * RS::A + (lane & (RS::A - 1));
                const int64_t row = row0 + (rp >> 1);
                if (FULL || row < R) st_stream4(q_sf + row * nsf + (rp & 1) * hsf + grp, f2u(rs.own[c].sf));
            }
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            if (col_ok && (FULL || row0 + r < R)) {
                uint8_t *qr = q + (int64_t)(row0 + r) * (2 * (int64_t)H);
                quantise_store8<TK_E4M3, false>(dg[r], rs.inv[2 * r], qr, col);
                quantise_store8<TK_E4M3, false>(du[r], rs.inv[2 * r + 1], qr, H + col);
            }
        }
    }

    // weight_grad[index] = dot product of the whole row: lanes -> wave -> workgroup
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        const float s = wave_sum(acc[r]);
        if (lane == 0) part[wave][r] = s;
    }
    __syncthreads();
    if (threadIdx.x < RPW) {
        const int r = threadIdx.x;
        float s = part[0][r];
        for (int i = 1; i < nwaves; ++i) s += part[i][r];
        const int idx = (FULL || row0 + r < R) ? ptt[row0 + r] : -1;
        if (idx >= 0 && idx < num_weights) weight_grad[idx] = s;
    }
    }   // row0 < R

    // weight_grad of the (token, k) pairs that have no row: grid-stride over the whole table.  Last, so
    // that its arguments (beyond the preloaded ones) are not waited for in front of the row loads.
    {
        const int64_t step = (int64_t)gridDim.x * blockDim.x;
        for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < num_weights; i += step)
            if (t2p[i] < 0) weight_grad[i] = 0.0f;
    }
}

constexpr int kBwdRowsPerGroup = 2;

struct BackwardArgs {
    const uint8_t *x;
    const float *x_sf;
    const uint16_t *grad_out;
    uint16_t *out, *x_grad;
    uint8_t *q;
    float *q_sf;
    int R, H;
    float clamp;
    int round_sf;
    const int32_t *ptt;
    const float *weights;
    float *weight_grad;
    const int32_t *t2p;
    int64_t num_weights;
};

template <int N, bool CLAMP>
static hipError_t launch_backward(const BackwardArgs &a, hipStream_t stream) {
    constexpr int RPW = kBwdRowsPerGroup;
    const int strips = (a.H + kStripCols - 1) / kStripCols;
    const int waves = backward_waves(strips);
    const int blocks = a.R > 0 ? (a.R + RPW - 1) / RPW : 1;
    const bool full = a.R % RPW == 0 && a.H % kStripCols == 0 && strips % waves == 0 && a.R > 0;
    const dim3 grid((unsigned)blocks), block(64 * waves);
#define TK_BWD_LAUNCH(F)                                                                                            \
    hipLaunchKernelGGL((swiglu_backward_kernel<N, CLAMP, RPW, F>), grid, block, 0, stream, a.x, a.x_sf, a.grad_out, \
                       a.R, a.H, waves, a.round_sf, a.out, a.x_grad, a.q, a.q_sf, a.clamp, a.ptt, a.weights, a.weight_grad, \
                       a.t2p, a.num_weights)
    if (full) TK_BWD_LAUNCH(true);
    else TK_BWD_LAUNCH(false);
#undef TK_BWD_LAUNCH
    return hipGetLastError();
}

}  // namespace tk

using namespace tk;

extern "C" int tk_check_swiglu_backward_per_token_cast(const void *x, const float *x_sf, int64_t R, int64_t H, int group,
                                                       const void *grad_out, const float *topk_weights,
                                                       const int32_t *pos_to_token_topk, const int32_t *token_topk_to_pos,
                                                       int64_t num_weights, const void *out, const void *x_grad_codes,
                                                       const float *x_grad_sf, const void *x_grad,
                                                       const float *weight_grad, int round_sf, int use_clamp, float clamp) {
    (void)round_sf;
    if (group != 32 && group != 128) return TK_ERR_BAD_GROUP;
    if (R < 0 || H <= 0 || H % group != 0 || num_weights < 0) return TK_ERR_BAD_SHAPE;
    if (R > INT32_MAX - 64 || H > (INT32_MAX - 1024) / 2) return TK_ERR_TOO_LARGE;
    if (use_clamp && !(clamp == clamp)) return TK_ERR_BAD_VALUE;
    if (num_weights > 0 && (!token_topk_to_pos || !weight_grad)) return TK_ERR_NULL_POINTER;
    if (R == 0) return TK_OK;
    if (!x || !x_sf || !grad_out || !topk_weights || !pos_to_token_topk || !out || !x_grad_codes || !x_grad_sf || !x_grad)
        return TK_ERR_NULL_POINTER;
    if (!aligned_to(x, 8) || !aligned_to(grad_out, 16) || !aligned_to(out, 16) || !aligned_to(x_grad, 16) ||
        !aligned_to(x_grad_codes, 8) || !aligned_to(x_sf, 4) || !aligned_to(x_grad_sf, 4))
        return TK_ERR_MISALIGNED;
    return TK_OK;
}

extern "C" int tk_swiglu_backward_per_token_cast(const void *x, const float *x_sf, int64_t R, int64_t H, int group,
                                                 const void *grad_out, const float *topk_weights,
                                                 const int32_t *pos_to_token_topk, const int32_t *token_topk_to_pos,
                                                 int64_t num_weights, void *out, void *x_grad_codes, float *x_grad_sf,
                                                 void *x_grad, float *weight_grad, int round_sf, int use_clamp,
                                                 float clamp, void *stream) {
    const int rc = tk_check_swiglu_backward_per_token_cast(x, x_sf, R, H, group, grad_out, topk_weights, pos_to_token_topk,
                                                           token_topk_to_pos, num_weights, out, x_grad_codes, x_grad_sf,
                                                           x_grad, weight_grad, round_sf, use_clamp, clamp);
    if (rc != TK_OK) return rc;
    if (R == 0 && num_weights == 0) return TK_OK;
    BackwardArgs a;
    a.x = static_cast<const uint8_t *>(x);
    a.x_sf = x_sf;
    a.grad_out = static_cast<const uint16_t *>(grad_out);
    a.out = static_cast<uint16_t *>(out);
    a.x_grad = static_cast<uint16_t *>(x_grad);
    a.q = static_cast<uint8_t *>(x_grad_codes);
    a.q_sf = x_grad_sf;
    a.R = (int)R;
    a.H = (int)H;
    a.clamp = clamp;
    a.round_sf = round_sf;
    a.ptt = pos_to_token_topk;
    a.weights = topk_weights;
    a.weight_grad = weight_grad;
    a.t2p = token_topk_to_pos;
    a.num_weights = num_weights;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e;
    if (group == 128) e = use_clamp ? launch_backward<128, true>(a, s) : launch_backward<128, false>(a, s);
    else e = use_clamp ? launch_backward<32, true>(a, s) : launch_backward<32, false>(a, s);
    return (int)e;
}
