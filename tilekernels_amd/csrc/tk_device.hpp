// Device-side building blocks shared by the gfx950 quantisation kernels: 16-byte vector loads,
// DPP cross-lane maxima, scale arithmetic, OCP FP8 / FP4 packing and scale-factor addressing.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tk_quant.h"

namespace tk {

constexpr int kTileRows = 16;     // rows of one workgroup tile (4 waves x 4 rows)
constexpr int kStripCols = 512;   // columns one wave covers per row: 64 lanes x 8 elements
constexpr int kThreads = 256;
constexpr int kNumXcd = 8;        // MI355X: workgroup i is dispatched to XCD i % 8

struct bf16_t { uint16_t bits; };

__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// ---------------------------------------------------------------------------------------------
// Workgroup -> tile mapping.  Consecutive workgroup ids land on different XCDs (each with its own
// L2), so tile t is handed to workgroup (t % per) * 8 + t / per ... inverted here: the workgroups
// of one XCD walk a contiguous range of tiles, which keeps partially written scale-factor cache
// lines inside one L2 until they are complete.
// Launch with grid = kNumXcd * ceil(total / kNumXcd); returns -1 for the surplus workgroups.
__device__ __forceinline__ int xcd_tile_index(int total) {
    const int per = (total + kNumXcd - 1) / kNumXcd;
    const int bid = blockIdx.x;
    const int t = (bid % kNumXcd) * per + bid / kNumXcd;
    return t < total ? t : -1;
}

// ---------------------------------------------------------------------------------------------
// Loads of 8 consecutive elements as fp32.  `ok == false` yields zeros without touching memory.
__device__ __forceinline__ void unpack_bf16x8(const uint4 w, float (&v)[8]) {
    v[0] = u2f(w.x << 16); v[1] = u2f(w.x & 0xFFFF0000u);
    v[2] = u2f(w.y << 16); v[3] = u2f(w.y & 0xFFFF0000u);
    v[4] = u2f(w.z << 16); v[5] = u2f(w.z & 0xFFFF0000u);
    v[6] = u2f(w.w << 16); v[7] = u2f(w.w & 0xFFFF0000u);
}

template <typename T> struct Raw8;
template <> struct Raw8<bf16_t> {
    uint4 w;
    __device__ __forceinline__ void load(const bf16_t *p, bool ok) {
        w = ok ? *reinterpret_cast<const uint4 *>(p) : make_uint4(0, 0, 0, 0);
    }
    __device__ __forceinline__ void get(float (&v)[8]) const { unpack_bf16x8(w, v); }
};
template <> struct Raw8<float> {
    float4 a, b;
    __device__ __forceinline__ void load(const float *p, bool ok) {
        a = ok ? *reinterpret_cast<const float4 *>(p) : make_float4(0, 0, 0, 0);
        b = ok ? *reinterpret_cast<const float4 *>(p + 4) : make_float4(0, 0, 0, 0);
    }
    __device__ __forceinline__ void get(float (&v)[8]) const {
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
};

__device__ __forceinline__ float absmax8(const float (&v)[8]) {
    float m = __builtin_fmaxf(__builtin_fabsf(v[0]), __builtin_fabsf(v[1]));
#pragma unroll
    for (int i = 2; i < 8; ++i) m = __builtin_fmaxf(m, __builtin_fabsf(v[i]));
    return m;
}

// ---------------------------------------------------------------------------------------------
// Cross-lane maxima on DPP (no LDS).  Operands are non-negative floats, whose order is the order
// of their bit patterns as unsigned integers, so the steps use integer max.
template <int CTRL> __device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7-i inside each 8
constexpr int kDppMirror = 0x140;     // lane i <-> 15-i inside each 16
constexpr int kDppRowShl4 = 0x104;    // lane i reads lane i+4 of its 16-lane row (0 past the end)
constexpr int kDppRowShl8 = 0x108;

__device__ __forceinline__ uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }

// every lane of each aligned group of LANES (2, 4, 8 or 16) lanes receives the group's maximum
template <int LANES> __device__ __forceinline__ float group_allmax(float nonneg) {
    uint32_t v = f2u(nonneg);
    if (LANES >= 2) v = umax(v, dpp_u32<kDppXor1>(v));
    if (LANES >= 4) v = umax(v, dpp_u32<kDppXor2>(v));
    if (LANES >= 8) v = umax(v, dpp_u32<kDppHalfMirror>(v));
    if (LANES >= 16) v = umax(v, dpp_u32<kDppMirror>(v));
    return u2f(v);
}

// ---------------------------------------------------------------------------------------------
// Scale of one block from its amax.
//   sf  = max(amax, floor) / qmax            (one correctly rounded division)
//   inv = qmax / max(amax, floor)            (a second, separate division)
// round_sf: sf is raised to the next power of two by carrying its mantissa into the exponent and
// inv = 1 / sf exactly (tile_kernels/torch/cast.py:158-164, tile_kernels/quant/common.py:196-216).
struct Scale {
    float sf;       // dequantisation scale, as stored
    float inv;      // multiplier applied before conversion
    uint32_t e8;    // biased exponent of sf (UE8M0 byte), valid with round_sf
};

__device__ __forceinline__ Scale make_scale(float amax, float floor_, float qmax, bool round_sf) {
    const float a = __builtin_fmaxf(amax, floor_);
    const float s = a / qmax;
    Scale r;
    if (!round_sf) {
        r.sf = s;
        r.inv = f2u(s) == 0u ? 0.0f : qmax / a;
        r.e8 = f2u(s) >> 23;
    } else {
        const uint32_t b = (f2u(s) + 0x007FFFFFu) & 0x7F800000u;
        const uint32_t e = b >> 23;
        r.sf = u2f(b);
        r.e8 = e;
        // 1 / 2^(e-127) = 2^(127-e): biased exponent 254 - e; e = 254 gives the subnormal 2^-127
        r.inv = e == 0u ? 0.0f : (e >= 254u ? u2f(0x00400000u >> (e - 254u)) : u2f((254u - e) << 23));
    }
    return r;
}

template <int FMT> struct Fmt;
template <> struct Fmt<TK_E4M3> {
    static constexpr float qmax = 448.0f;
    static constexpr float floor_ = 1e-4f;
};
template <> struct Fmt<TK_E2M1> {
    static constexpr float qmax = 6.0f;
    static constexpr float floor_ = 6.0f * 0x1p-126f;
};

// ---------------------------------------------------------------------------------------------
// Conversions.  v_cvt_pk_fp8_f32 on gfx950 is OCP E4M3FN round-to-nearest-even; it does not
// saturate by itself, so inputs that may exceed 448 are clamped first (CLAMP).
template <bool CLAMP> __device__ __forceinline__ uint2 pack_e4m3x8(const float (&q)[8]) {
    float c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) c[i] = CLAMP ? __builtin_amdgcn_fmed3f(q[i], -448.0f, 448.0f) : q[i];
    int lo = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], 0, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], lo, true);
    int hi = __builtin_amdgcn_cvt_pk_fp8_f32(c[4], c[5], 0, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(c[6], c[7], hi, true);
    return make_uint2((uint32_t)lo, (uint32_t)hi);
}

// eight fp32 -> eight E2M1 nibbles in one dword, element 2t in the low nibble of byte t
__device__ __forceinline__ uint32_t pack_e2m1x8(const float (&q)[8]) {
    uint32_t w = 0;
    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, q[0], q[1], 1.0f, 0);
    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, q[2], q[3], 1.0f, 1);
    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, q[4], q[5], 1.0f, 2);
    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, q[6], q[7], 1.0f, 3);
    return w;
}

// scale 8 values, convert, store: 8 bytes (E4M3) or 4 bytes (E2M1) per lane
template <int FMT, bool CLAMP>
__device__ __forceinline__ void quantise_store8(const float (&v)[8], float inv, uint8_t *out_row, int col) {
    float q[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = v[i] * inv;
    if (FMT == TK_E4M3) {
        *reinterpret_cast<uint2 *>(out_row + col) = pack_e4m3x8<CLAMP>(q);
    } else {
        *reinterpret_cast<uint32_t *>(out_row + (col >> 1)) = pack_e2m1x8(q);
    }
}

// ---------------------------------------------------------------------------------------------
// Scale-factor storage (see the layout table in tk_quant.h).
struct SfRef {
    void *base;
    int64_t ld;
    int layout;
    int nm, nk;   // number of blocks along rows / columns
};

__device__ __forceinline__ float sf_load(const SfRef &s, int m, int k) {
    if (s.layout == TK_SF_ROW_F32) return reinterpret_cast<const float *>(s.base)[(int64_t)m * s.ld + k];
    if (s.layout == TK_SF_COL_F32) return reinterpret_cast<const float *>(s.base)[(int64_t)k * s.ld + m];
    const uint32_t e = reinterpret_cast<const uint8_t *>(s.base)[(int64_t)(k >> 2) * s.ld + 4 * (int64_t)m + (k & 3)];
    return u2f(e << 23);
}

// store from a single lane; for the packed layout the lane that owns the last block of a row also
// zeroes the unused bytes of that row's last word
__device__ __forceinline__ void sf_store(const SfRef &s, int m, int k, const Scale &sc) {
    if (s.layout == TK_SF_ROW_F32) {
        reinterpret_cast<float *>(s.base)[(int64_t)m * s.ld + k] = sc.sf;
    } else if (s.layout == TK_SF_COL_F32) {
        reinterpret_cast<float *>(s.base)[(int64_t)k * s.ld + m] = sc.sf;
    } else {
        uint8_t *p = reinterpret_cast<uint8_t *>(s.base) + (int64_t)(k >> 2) * s.ld + 4 * (int64_t)m;
        p[k & 3] = (uint8_t)sc.e8;
        if (k == s.nk - 1)
            for (int j = (k & 3) + 1; j < 4; ++j) p[j] = 0;
    }
}

// Write the scales of one 16-row tile, staged in LDS as stage[row][g] (fp32 bits or exponent
// byte), to a column-major layout so that 16 consecutive lanes fill one 64-byte segment.
//   GPS    : groups per row in the stage
//   m0, k0 : block coordinates of stage[0][0]
template <int GPS>
__device__ __forceinline__ void sf_store_tile_colmajor(const SfRef &s, const uint32_t (*stage)[GPS], int m0, int k0) {
    if (s.layout == TK_SF_COL_F32) {
        for (int e = threadIdx.x; e < GPS * kTileRows; e += kThreads) {
            const int g = e / kTileRows, r = e % kTileRows;
            const int m = m0 + r, k = k0 + g;
            if (m < s.nm && k < s.nk) reinterpret_cast<uint32_t *>(s.base)[(int64_t)k * s.ld + m] = stage[r][g];
        }
    } else {
        constexpr int WPS = (GPS + 3) / 4;   // words per row in the stage
        for (int e = threadIdx.x; e < WPS * kTileRows; e += kThreads) {
            const int wd = e / kTileRows, r = e % kTileRows;
            const int m = m0 + r, k = k0 + 4 * wd;
            if (m < s.nm && k < s.nk) {
                uint32_t word = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (4 * wd + j < GPS && k + j < s.nk) word |= (stage[r][4 * wd + j] & 0xFFu) << (8 * j);
                *reinterpret_cast<uint32_t *>(reinterpret_cast<uint8_t *>(s.base) + (int64_t)(k >> 2) * s.ld + 4 * (int64_t)m) = word;
            }
        }
    }
}

}  // namespace tk
