/*
 * Scalar C restatement of the quantisation path's arithmetic -- TEST INFRASTRUCTURE ONLY.
 *
 * Nothing that ships links or loads this file: only tests, the smoke check and the CPU-baseline
 * leg of the benchmark do, as the checker.  It exists as a second, independently written
 * statement of the same algorithm as oracle/torch_ref.py, so that a slip in either one shows up as
 * a bit mismatch between the two (tests/test_oracle_cast.py, tests/test_oracle_swiglu_backward.py), and so that full-size inputs can
 * be checked in seconds.
 *
 * Algorithm followed (reference file:line):
 *   block amax, clamp, scale, inverse scale, power-of-two rounding .. tile_kernels/torch/cast.py:128-164
 *   use of a caller-supplied scale (1/sf, clamp +-448) ............. tile_kernels/torch/cast.py:165-190
 *   E2M1 code assignment and nibble packing ....................... tile_kernels/torch/cast.py:192-196, 224-252
 *   SwiGLU g/(1+exp(-g))*u, clamp, counters, routing weight ....... tile_kernels/torch/swiglu.py:62-86
 *   SwiGLU backward on a dequantised input ........................ tile_kernels/torch/swiglu.py:98-227
 *
 * Pins: tkref_e4m3_encode / tkref_e2m1_encode are checked against brute-force nearest-value
 * searches over the OCP value tables and hand known answers (tests/test_oracle_encoders.py); the
 * block functions against a naive Python loop on tiny inputs and against torch_ref bit-for-bit.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC).
 * Floating point contraction must stay off: every product and sum here is one IEEE binary32
 * rounding, as in the reference.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

static inline float load_elem(const void *x, int is_f32, int64_t idx) {
    return is_f32 ? ((const float *)x)[idx] : bf16_to_f32(((const uint16_t *)x)[idx]);
}

/* fp32 -> OCP E4M3FN byte: clamp to +-448, round to nearest even, subnormals in steps of 2^-9,
 * sign kept on underflow, NaN -> 0x7f | sign. */
uint8_t tkref_e4m3_encode(float v) {
    uint32_t sign = (f2u(v) >> 24) & 0x80u;
    float a = fabsf(v);
    if (isnan(v)) return (uint8_t)(sign | 0x7f);
    if (a > 448.0f) a = 448.0f;
    if (a < 0.015625f) {                        /* below 2^-6: fixed point, unit 2^-9 */
        return (uint8_t)(sign | (uint32_t)nearbyintf(a * 512.0f));
    }
    uint32_t b = f2u(a);
    b += 0x7FFFFu + ((b >> 20) & 1u);           /* RTNE on the 20 dropped mantissa bits */
    uint32_t e = (b >> 23) - 127u + 7u;
    return (uint8_t)(sign | (e << 3) | ((b >> 20) & 7u));
}

/* fp32 -> E2M1 nibble (sign in bit 3): nearest of {0,.5,1,1.5,2,3,4,6}, ties to the even code,
 * saturating; NaN saturates to 7 like any exponent-255 input in the reference's bit routine. */
uint8_t tkref_e2m1_encode(float v) {
    uint32_t sign = (f2u(v) >> 28) & 0x8u;
    float a = fabsf(v);
    uint32_t c;
    if (isnan(v) || a >= 6.0f) c = 7;
    else if (a < 1.0f) c = (uint32_t)nearbyintf(a * 2.0f);
    else if (a < 2.0f) c = 2u + (uint32_t)nearbyintf((a - 1.0f) * 2.0f);
    else if (a < 4.0f) c = 4u + (uint32_t)nearbyintf(a - 2.0f);
    else c = 6u + (uint32_t)nearbyintf((a - 4.0f) * 0.5f);
    return (uint8_t)(sign | c);
}

/* dequant scale and quantisation multiplier of one block from its amax */
static inline void scale_pair(float amax, float qmax, float floor_, int round_sf, float *sf, float *inv) {
    float a = amax > floor_ ? amax : floor_;
    float s = a / qmax;
    if (round_sf) {
        uint32_t b = (f2u(s) + 0x007FFFFFu) & 0x7F800000u;
        s = u2f(b);
        *inv = (s == 0.0f) ? 0.0f : 1.0f / s;
    } else {
        *inv = (f2u(s) == 0u) ? 0.0f : qmax / a;
    }
    *sf = s;
}

/*
 * Block-scaled cast of x[M,K] (row stride x_ld elements, unit column stride).
 *   x_is_f32 : 0 = bf16 bits, 1 = fp32
 *   fmt      : 0 = E4M3 (one byte per element), 1 = E2M1 (two elements per byte, even one low)
 *   bm, bk   : block shape; partial edge blocks use their in-range part
 *   floor_   : lower clamp of the block amax; < 0 selects the format default
 *   given_sf : NULL, or caller-supplied dequant scales [ceil(M/bm), ceil(K/bk)] row-major
 *   codes    : [M, K] or [M, K/2] bytes, contiguous
 *   sf_out   : [ceil(M/bm), ceil(K/bk)] fp32 row-major dequant scales (ignored with given_sf)
 * Returns 0, or -1 on a bad argument.
 */
int tkref_cast(const void *x, int x_is_f32, int64_t M, int64_t K, int64_t x_ld, int bm, int bk,
               int fmt, int round_sf, float floor_, const float *given_sf, uint8_t *codes, float *sf_out) {
    if (M < 0 || K < 0 || bm <= 0 || bk <= 0 || (fmt != 0 && fmt != 1)) return -1;
    if (fmt == 1 && (K & 1)) return -1;
    const float qmax = fmt == 0 ? 448.0f : 6.0f;
    if (floor_ < 0) floor_ = fmt == 0 ? 1e-4f : 6.0f * 0x1p-126f;
    const int64_t nm = (M + bm - 1) / bm, nk = (K + bk - 1) / bk;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t bi = 0; bi < nm; ++bi) {
        for (int64_t bj = 0; bj < nk; ++bj) {
            const int64_t r0 = bi * bm, r1 = (r0 + bm < M) ? r0 + bm : M;
            const int64_t c0 = bj * bk, c1 = (c0 + bk < K) ? c0 + bk : K;
            float sf, inv;
            if (given_sf) {
                sf = given_sf[bi * nk + bj];
                inv = 1.0f / sf;
            } else {
                float amax = 0.0f;
                for (int64_t r = r0; r < r1; ++r)
                    for (int64_t c = c0; c < c1; ++c) {
                        float a = fabsf(load_elem(x, x_is_f32, r * x_ld + c));
                        if (a > amax) amax = a;
                    }
                scale_pair(amax, qmax, floor_, round_sf, &sf, &inv);
                sf_out[bi * nk + bj] = sf;
            }
            for (int64_t r = r0; r < r1; ++r) {
                if (fmt == 0) {
                    for (int64_t c = c0; c < c1; ++c)
                        codes[r * K + c] = tkref_e4m3_encode(load_elem(x, x_is_f32, r * x_ld + c) * inv);
                } else {
                    for (int64_t c = c0; c < c1; c += 2) {
                        uint8_t lo = tkref_e2m1_encode(load_elem(x, x_is_f32, r * x_ld + c) * inv);
                        uint8_t hi = tkref_e2m1_encode(load_elem(x, x_is_f32, r * x_ld + c + 1) * inv);
                        codes[r * (K / 2) + c / 2] = (uint8_t)(lo | (hi << 4));
                    }
                }
            }
        }
    }
    return 0;
}

/*
 * SwiGLU forward: out[r, c] = g/(1+exp(-g)) * u [* w_r], g = x[r, c], u = x[r, c+H], fp32.
 *   use_clamp : g = min(g, clamp), u = min(max(u, -clamp), clamp); counts (may be NULL) gets
 *               += {#g>clamp, #u>clamp, #u<-clamp} taken before clamping over every row
 *   pos_to_token_topk / topk_weights (flat) : per-row weight, 0 where the index is negative
 *   pos_to_expert : rows with a negative entry are written as zeros (the masked_fill the
 *               reference's test applies before the cast)
 */
int tkref_swiglu(const void *x, int x_is_f32, int64_t R, int64_t H, const int32_t *pos_to_token_topk,
                 const float *topk_weights, const int32_t *pos_to_expert, int use_clamp, float clamp,
                 int64_t *counts, float *out) {
    if (R < 0 || H <= 0) return -1;
    int64_t n0 = 0, n1 = 0, n2 = 0;
#pragma omp parallel for schedule(static) reduction(+ : n0, n1, n2)
    for (int64_t r = 0; r < R; ++r) {
        float w = 1.0f;
        if (pos_to_token_topk) w = pos_to_token_topk[r] >= 0 ? topk_weights[pos_to_token_topk[r]] : 0.0f;
        const int dead = pos_to_expert && pos_to_expert[r] < 0;
        for (int64_t c = 0; c < H; ++c) {
            float g = load_elem(x, x_is_f32, r * 2 * H + c);
            float u = load_elem(x, x_is_f32, r * 2 * H + H + c);
            if (use_clamp) {
                n0 += g > clamp; n1 += u > clamp; n2 += u < -clamp;
                g = g < clamp ? g : clamp;
                u = u > -clamp ? u : -clamp;
                u = u < clamp ? u : clamp;
            }
            float e = expf(-g);
            float d = 1.0f + e;
            float v = g / d;
            v = v * u;
            if (pos_to_token_topk) v = v * w;
            out[r * H + c] = dead ? 0.0f : v;
        }
    }
    if (counts) { counts[0] += n0; counts[1] += n1; counts[2] += n2; }
    return 0;
}

/* OCP E4M3FN byte -> fp32 (0x7f / 0xff are NaN) */
static inline float e4m3_decode(uint8_t c) {
    const uint32_t e = (c >> 3) & 15u, m = c & 7u;
    float a;
    if (e == 15u && m == 7u) a = NAN;
    else if (e == 0u) a = (float)m * 0x1p-9f;
    else a = u2f(((e + 120u) << 23) | (m << 20));
    return (c & 0x80u) ? -a : a;
}

/*
 * SwiGLU backward on a quantised forward input (tile_kernels/torch/swiglu.py:98-227).
 *   codes[R, 2H] E4M3 bytes, sf[R, 2H/N] fp32 (N = group), grad_out[R, H] bf16 bits,
 *   weight[T*K] fp32, pos_to_token_topk[R] (negative = padding row, weight 0).
 * Outputs, all fp32: out[R, H] = g/(1+exp(-g))*u*w, x_grad[R, 2H] = [d/dgate | d/dup],
 * weight_grad[T*K] (zero-filled first, then the row dot products sum(grad_out * act)).
 * The only fused operation is fma(g, 1 - s, 1); every other product is rounded once.
 */
int tkref_swiglu_backward(const uint8_t *codes, const float *sf, int64_t R, int64_t H, int group,
                          const uint16_t *grad_out, const float *weight, int64_t num_weights,
                          const int32_t *pos_to_token_topk, int use_clamp, float clamp, float *out,
                          float *x_grad, float *weight_grad) {
    if (R < 0 || H <= 0 || group <= 0 || H % group) return -1;
    const int64_t nsf = 2 * H / group;
    for (int64_t i = 0; i < num_weights; ++i) weight_grad[i] = 0.0f;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < R; ++r) {
        const int32_t idx = pos_to_token_topk[r];
        const float w = idx >= 0 ? weight[idx] : 0.0f;
        float dot = 0.0f;
        for (int64_t c = 0; c < H; ++c) {
            float g = e4m3_decode(codes[r * 2 * H + c]) * sf[r * nsf + c / group];
            float u = e4m3_decode(codes[r * 2 * H + H + c]) * sf[r * nsf + (H + c) / group];
            int cg = 0, cu = 0;
            if (use_clamp) {
                cg = g > clamp;
                if (cg) g = clamp;
                if (u > clamp) { u = clamp; cu = 1; }
                else if (u < -clamp) { u = -clamp; cu = 1; }
            }
            const float go = bf16_to_f32(grad_out[r * H + c]);
            const float d = 1.0f + expf(-g);
            const float s = 1.0f / d;
            float t = go * w;
            t = t * s;
            float dg = t * u;
            dg = dg * fmaf(g, 1.0f - s, 1.0f);
            const float du = t * g;
            float act = g / d;
            act = act * u;
            out[r * H + c] = act * w;
            x_grad[r * 2 * H + c] = cg ? 0.0f : dg;
            x_grad[r * 2 * H + H + c] = cu ? 0.0f : du;
            dot += go * act;
        }
        if (idx >= 0) weight_grad[idx] = dot;
    }
    return 0;
}

void tkref_fmaf_n(const float *a, const float *b, const float *c, int64_t n, float *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = fmaf(a[i], b[i], c[i]);
}

/* bulk helpers so Python can test the encoders over whole arrays */
void tkref_e4m3_encode_n(const float *v, int64_t n, uint8_t *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = tkref_e4m3_encode(v[i]);
}
void tkref_e2m1_encode_n(const float *v, int64_t n, uint8_t *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = tkref_e2m1_encode(v[i]);
}

/*
 * Support for the test that pins the GPU's three-instruction division by a constant:
 *   q = a * y;  q' = fma(fma(-c, q, a), y, q)   with y = fl(1 / c)
 * Counts the positive floats with bit patterns in [lo_bits, hi_bits) for which q' differs from the
 * IEEE quotient a / c (only inputs whose quotient is a normal number are counted: smaller operands
 * take an ordinary division on the GPU).  fmaf() is the correctly rounded libm/hardware fma.
 * `uncorrected` != 0 drops the fma step (q alone), which is NOT exact: the negative control.
 */
int64_t tkref_count_div_mismatches(float c, uint32_t lo_bits, uint32_t hi_bits, int uncorrected) {
    const float y = 1.0f / c;
    int64_t bad = 0;
#pragma omp parallel for schedule(static) reduction(+ : bad)
    for (int64_t b = lo_bits; b < (int64_t)hi_bits; ++b) {
        const float a = u2f((uint32_t)b);
        const float want = a / c;
        if (want < 0x1p-126f) continue;
        const float q = a * y;
        const float r = fmaf(-c, q, a);
        const float q2 = uncorrected ? q : fmaf(r, y, q);
        bad += q2 != want;
    }
    return bad;
}
