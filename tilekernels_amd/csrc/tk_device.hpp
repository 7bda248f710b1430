// Device-side building blocks shared by the gfx950 quantisation kernels: streaming 16-byte loads
// and stores, DPP cross-lane maxima, scale arithmetic, OCP FP8 / FP4 packing and scale-factor
// addressing.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tk_quant.h"

namespace tk {

constexpr int kStripCols = 512;   // columns one wave covers per row: 64 lanes x 8 elements
constexpr int kThreads = 256;     // 4 waves per workgroup (stacked tiles; wide tiles use 3..8 waves)
constexpr int kWaves = kThreads / 64;
constexpr int kMaxWideWaves = 8;

// Number of waves of a wide tile (waves side by side, 512 columns each) for a row of `strips`
// 512-column strips: the largest of 8..3 that divides it, so that no wave idles; 0 if none does.
inline int wide_tile_waves(int strips) {
    for (int w = kMaxWideWaves; w >= 3; --w)
        if (strips % w == 0) return w;
    return 0;
}

// Wide tiles are for rows whose strips split evenly over 3..8 waves.  Other rows take stacked tiles: one or two
// strips would leave most waves of a wide tile without columns (SwiGLU of bf16 [65536, 2 x 512]: 62 us wide, 27 us
// stacked), and 11 or 13 strips still idle one wave of a tile in 12 or 14 (per-token cast of bf16 [20096, 6656]:
// 62.7 us wide with 7 waves, 57.4 us stacked).
inline bool wide_tiles_pay(int64_t cols) { return wide_tile_waves((int)((cols + kStripCols - 1) / kStripCols)) != 0; }

// Grid of a kernel with one workgroup per tile: column tiles on x, row tiles on y and z (y alone ends at 65535).
// Workgroups are handed out in x-first order, so those that run together walk along rows and touch long
// consecutive runs of memory; with the row tiles on x they walked down a column of tiles, each on its own rows:
// dequantisation of E4M3 [5888, 22528] 76.8 us against 62.6 us, per-token cast of bf16 [4096, 7168] 15.13 against
// 14.89 us, SwiGLU cast of bf16 [6016, 2 x 11008] 71.6 against 51.3 us.  A single column of tiles goes on x alone
// (as y of a grid one workgroup wide it starts workgroups more slowly: 48128 one-wave workgroups 61.5 -> 75.6 us).
// A grid whose y * z exceeds the number of row tiles has workgroups beyond the last row, which only the kernels'
// bounds-checked variants tolerate: tile_grid_exact() says whether there are none.
constexpr int kGridRowsLog2 = 15;
inline dim3 tile_grid(int tiles_k, int tiles_m) {
    if (tiles_k == 1) return dim3((unsigned)tiles_m);
    const int per_z = 1 << kGridRowsLog2;
    return dim3((unsigned)tiles_k, (unsigned)(tiles_m < per_z ? tiles_m : per_z), (unsigned)((tiles_m + per_z - 1) >> kGridRowsLog2));
}
inline bool tile_grid_exact(int tiles_k, int tiles_m) {
    return tiles_k == 1 || tiles_m <= (1 << kGridRowsLog2) || tiles_m % (1 << kGridRowsLog2) == 0;
}

struct bf16_t { uint16_t bits; };
struct e4m3in_t {};   // input that is itself E4M3 codes with block scales
struct e2m1in_t {};   // input that is packed E2M1 codes (two per byte) with block scales
struct e5m6in_t {};   // input that is packed E5M6 codes (eight per 12 bytes) with block scales

template <typename T> struct Elem { static constexpr int bits = 8 * (int)sizeof(T); static constexpr bool quantised = false; };
template <> struct Elem<e4m3in_t> { static constexpr int bits = 8; static constexpr bool quantised = true; };
template <> struct Elem<e2m1in_t> { static constexpr int bits = 4; static constexpr bool quantised = true; };
template <> struct Elem<e5m6in_t> { static constexpr int bits = 12; static constexpr bool quantised = true; };

typedef float f32x2 __attribute__((ext_vector_type(2)));

// address of element (row, col) of a matrix with `ld` logical elements per row
template <typename T> __device__ __forceinline__ const void *elem_ptr(const void *base, int64_t row, int64_t ld, int col) {
    return reinterpret_cast<const uint8_t *>(base) + (((row * ld + col) * Elem<T>::bits) >> 3);
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
// the same three words at an address that is only 4-byte aligned (the 12-byte E5M6 pieces): the plain type claims 16
typedef u32x3 u32x3_a4 __attribute__((aligned(4)));

// one_col: the grid is a single column of tiles (wave-uniform)
__device__ __forceinline__ int tile_grid_row(bool one_col) { return (int)(one_col ? blockIdx.x : (blockIdx.z << kGridRowsLog2) + blockIdx.y); }
// (a single column reads its index, 0, from y rather than using the constant: the SwiGLU cast of bf16 [8192, 2 x 2048]
// measures 14.65 us this way and 14.75 - 14.85 us with the constant folded in)
__device__ __forceinline__ int tile_grid_col(bool one_col) { return (int)(one_col ? blockIdx.y : blockIdx.x); }

__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// Wave index as a scalar: everything derived from it (row numbers, row pointers, per-row flags)
// then lives in SGPRs and uses scalar loads.
__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

// Load through the scalar (constant) path: for small read-only tables indexed by a wave-uniform
// value, so that the result arrives in an SGPR and does not tie up the vector memory counter.
template <typename T> __device__ __forceinline__ T uniform_load(const T *p) {
    typedef const T __attribute__((address_space(4))) *const_ptr;
    return *(const_ptr)(uintptr_t)p;
}

// ---------------------------------------------------------------------------------------------
// Streaming memory access.  Inputs are read once and outputs written once.  Measured on MI355X for
// the SwiGLU traffic shape (64 MiB read, 16 MiB written per call, buffers rotated past the last-
// level cache), time per call with plain / hinted accesses:
//     plain loads, plain stores                15.5 us
//     non-temporal loads, plain stores         14.8 us
//     non-temporal loads, non-temporal stores  14.2 us
//     non-temporal loads, write-through stores 13.8 us   <- used here
// Loads carry the `nt` bit; stores are issued at system scope (`sc0 sc1`), which writes them
// through instead of leaving dirty lines to be flushed when the kernel ends.
// Between two vector memory instructions of a wave that follow each other directly: one wait state.  A wave that issues its
// loads back to back is served worse than one with anything at all between them (MI355X, the loads and stores of the fused
// SwiGLU cast of bf16 [8192, 2 x 2048] alone, eight 16-byte loads per lane: back to back 14.07 us, one s_nop 0 / s_nop 3 /
// s_nop 7 / 16 / 32 / 64 wait states between them 13.76 / 13.73 / 13.75 / 13.79 / 13.87 / 13.97; the order of the loads makes
// no difference; the operator itself 14.05 -> 13.85 us; the same between stores changes nothing).  The compiler packs loads
// whose addresses are ready together, so the gap is part of the text; the memory clobber keeps the loads on either side
// where they are.
#ifndef TK_VMEM_GAP
#define TK_VMEM_GAP 1
#endif
__device__ __forceinline__ void vmem_issue_gap() {
#if TK_VMEM_GAP
    asm volatile("s_nop 0" ::: "memory");
#endif
}

__device__ __forceinline__ u32x4 ld_stream16(const void *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
}
__device__ __forceinline__ void st_stream8(void *p, u32x2 v) {
    __hip_atomic_store(reinterpret_cast<uint64_t *>(p), __builtin_bit_cast(uint64_t, v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_SYSTEM);
}
// (The 16-byte form has no builtin with these cache bits.  A store of more than 8 bytes must not be followed at once by
// a VALU instruction that overwrites its data registers; for its own stores the compiler keeps that distance, for an
// instruction it cannot look into it does not, so the wait state is part of the text.  Without it a loop whose next
// iteration begins by computing an address in the first data register stored that address instead of the data.)
__device__ __forceinline__ void st_stream16(void *p, u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 0" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void st_stream4(void *p, uint32_t v) {
    __hip_atomic_store(reinterpret_cast<uint32_t *>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// 8 consecutive elements, as fp32.  `ok == false` yields zeros without touching memory.
template <typename T> struct Raw8;
template <> struct Raw8<bf16_t> {
    u32x4 w;
    __device__ __forceinline__ void load(const void *p) { w = ld_stream16(p); }
    __device__ __forceinline__ void load(const void *p, bool ok) {
        w = u32x4{0u, 0u, 0u, 0u};
        if (ok) w = ld_stream16(p);
    }
    // a lane's 16 bytes are one load already: the run interface of the fp32 loader, with nothing to exchange
    static constexpr int kXchgBytes = 0;
    template <int LANES> __device__ __forceinline__ void load_run(const void *p, int) { w = ld_stream16(p); }
    template <int LANES> __device__ __forceinline__ void settle(uint8_t *, int) {}
    // ordinary (cacheable) load, for data that is read again shortly
    __device__ __forceinline__ void load_cached(const void *p) { w = *reinterpret_cast<const u32x4 *>(p); }
    __device__ __forceinline__ void zero() { w = u32x4{0u, 0u, 0u, 0u}; }
    __device__ __forceinline__ void get(float (&v)[8]) const {
        v[0] = u2f(w.x << 16); v[1] = u2f(w.x & 0xFFFF0000u);
        v[2] = u2f(w.y << 16); v[3] = u2f(w.y & 0xFFFF0000u);
        v[4] = u2f(w.z << 16); v[5] = u2f(w.z & 0xFFFF0000u);
        v[6] = u2f(w.w << 16); v[7] = u2f(w.w & 0xFFFF0000u);
    }
};
// fp32: a lane's 8 elements are 32 bytes.  Read as two 16-byte loads of the lane's own bytes, each load instruction of a
// wave touches every other 16 bytes of the 2 KB it spans, i.e. half of every cache line, twice over.  load_run() reads the
// same bytes with both instructions covering whole lines: the LANES lanes that hold one contiguous run of 8 * LANES
// elements (lane i of the run owning elements 8i .. 8i + 7) read the run's first half with one instruction and its second
// half with the other, 16 consecutive bytes per lane; settle() then hands every lane its own 32 bytes through LDS (two
// 16-byte writes, two 16-byte reads; the run's 32 * LANES bytes of LDS are private to its lanes, which belong to one wave,
// so no barrier is involved).  Measured on MI355X, per-token cast of fp32 [4096, 7168]: 26.6 -> 23.5 us; fused SwiGLU cast of
// fp32 [8192, 2 x 2048]: 27.6 -> 25.6 us (timed with the exchange left out).  All lanes of the run must be in range.
template <> struct Raw8<float> {
    u32x4 a, b;
    static constexpr int kXchgBytes = 32;   // LDS bytes per lane of a run
    __device__ __forceinline__ void load(const void *p) { a = ld_stream16(p); vmem_issue_gap(); b = ld_stream16(reinterpret_cast<const float *>(p) + 4); }
    __device__ __forceinline__ void load(const void *p, bool ok) {
        zero();
        if (ok) load(p);
    }
    // p: the lane's own 8 elements; i: its index among the LANES lanes of the run
    template <int LANES> __device__ __forceinline__ void load_run(const void *p, int i) {
        const uint8_t *q = reinterpret_cast<const uint8_t *>(p) - 16 * i;
        a = ld_stream16(q);
        vmem_issue_gap();
        b = ld_stream16(q + 16 * LANES);
    }
    // run_lds: the 32 * LANES bytes of LDS of this lane's run, 16-byte aligned
    template <int LANES> __device__ __forceinline__ void settle(uint8_t *run_lds, int i) {
        u32x4 *w = reinterpret_cast<u32x4 *>(run_lds);
        w[i] = a;
        w[LANES + i] = b;
        a = w[2 * i];
        b = w[2 * i + 1];
    }
    __device__ __forceinline__ void load_cached(const void *p) {
        a = *reinterpret_cast<const u32x4 *>(p);
        b = *(reinterpret_cast<const u32x4 *>(p) + 1);
    }
    __device__ __forceinline__ void zero() { a = u32x4{0u, 0u, 0u, 0u}; b = a; }
    __device__ __forceinline__ void get(float (&v)[8]) const {
        v[0] = u2f(a.x); v[1] = u2f(a.y); v[2] = u2f(a.z); v[3] = u2f(a.w);
        v[4] = u2f(b.x); v[5] = u2f(b.y); v[6] = u2f(b.z); v[7] = u2f(b.w);
    }
};

// Quantised inputs: 8 codes plus the dequantisation scale of the block they sit in (`s`, set by the
// caller); get() yields code * s, one rounding, as in the reference's dequantise-then-cast
// (tile_kernels/torch/cast.py:87-99).
template <> struct Raw8<e4m3in_t> {
    u32x2 w;
    float s;
    __device__ __forceinline__ void load(const void *p) { w = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(p)); }
    static constexpr int kXchgBytes = 0;
    template <int LANES> __device__ __forceinline__ void load_run(const void *p, int) { load(p); }
    template <int LANES> __device__ __forceinline__ void settle(uint8_t *, int) {}
    __device__ __forceinline__ void load(const void *p, bool ok) {
        w = u32x2{0u, 0u};
        if (ok) load(p);
    }
    __device__ __forceinline__ void zero() { w = u32x2{0u, 0u}; s = 0.0f; }
    __device__ __forceinline__ void get(float (&v)[8]) const {
        const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w.x, false), b = __builtin_amdgcn_cvt_pk_f32_fp8((int)w.x, true);
        const f32x2 c = __builtin_amdgcn_cvt_pk_f32_fp8((int)w.y, false), d = __builtin_amdgcn_cvt_pk_f32_fp8((int)w.y, true);
        v[0] = a.x * s; v[1] = a.y * s; v[2] = b.x * s; v[3] = b.y * s;
        v[4] = c.x * s; v[5] = c.y * s; v[6] = d.x * s; v[7] = d.y * s;
    }
    // codes 0..3 (hi = false) or 4..7 of the piece
    __device__ __forceinline__ void get4(float (&v)[4], bool hi) const {
        const int h = (int)(hi ? w.y : w.x);
        const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8(h, false), b = __builtin_amdgcn_cvt_pk_f32_fp8(h, true);
        v[0] = a.x * s; v[1] = a.y * s; v[2] = b.x * s; v[3] = b.y * s;
    }
};
template <> struct Raw8<e2m1in_t> {
    uint32_t w;
    float s;
    __device__ __forceinline__ void load(const void *p) { w = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(p)); }
    static constexpr int kXchgBytes = 0;
    template <int LANES> __device__ __forceinline__ void load_run(const void *p, int) { load(p); }
    template <int LANES> __device__ __forceinline__ void settle(uint8_t *, int) {}
    __device__ __forceinline__ void load(const void *p, bool ok) {
        w = 0u;
        if (ok) load(p);
    }
    __device__ __forceinline__ void zero() { w = 0u; s = 0.0f; }
    __device__ __forceinline__ void get(float (&v)[8]) const {
        const f32x2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0), b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1);
        const f32x2 c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2), d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3);
        v[0] = a.x * s; v[1] = a.y * s; v[2] = b.x * s; v[3] = b.y * s;
        v[4] = c.x * s; v[5] = c.y * s; v[6] = d.x * s; v[7] = d.y * s;
    }
    __device__ __forceinline__ void get4(float (&v)[4], bool hi) const {
        const uint32_t h = hi ? w >> 16 : w;
        const f32x2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(h, 1.0f, 0), b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(h, 1.0f, 1);
        v[0] = a.x * s; v[1] = a.y * s; v[2] = b.x * s; v[3] = b.y * s;
    }
};

// E5M6: a 12-bit float, the top 12 bits of an IEEE fp16 (sign, 5 exponent bits, 6 mantissa bits).  Eight
// codes c0..c7 form a 96-bit string with c0 in the most significant bits, stored as three 32-bit words
// from the high word down (reference: float_to_e5m6 / e5m6_to_float,
// tile_kernels/quant/per_token_cast_to_e5m6_kernel.py:36-70, cast_back_e5m6_kernel.py:12-41).
__device__ __forceinline__ float e5m6_value(uint32_t top12_in_bits_15_4) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(top12_in_bits_15_4 & 0xFFF0u));
}
template <> struct Raw8<e5m6in_t> {
    u32x3 w;
    float s;
    __device__ __forceinline__ void load(const void *p) { w = __builtin_nontemporal_load(reinterpret_cast<const u32x3_a4 *>(p)); }
    static constexpr int kXchgBytes = 0;
    template <int LANES> __device__ __forceinline__ void load_run(const void *p, int) { load(p); }
    template <int LANES> __device__ __forceinline__ void settle(uint8_t *, int) {}
    __device__ __forceinline__ void load(const void *p, bool ok) {
        w = u32x3{0u, 0u, 0u};
        if (ok) load(p);
    }
    __device__ __forceinline__ void zero() { w = u32x3{0u, 0u, 0u}; s = 0.0f; }
    __device__ __forceinline__ void get(float (&v)[8]) const {
        v[0] = e5m6_value(w.x >> 16) * s;
        v[1] = e5m6_value(w.x >> 4) * s;
        v[2] = e5m6_value((w.x << 8) | (w.y >> 24)) * s;
        v[3] = e5m6_value(w.y >> 12) * s;
        v[4] = e5m6_value(w.y) * s;
        v[5] = e5m6_value((w.y << 12) | (w.z >> 20)) * s;
        v[6] = e5m6_value(w.z >> 8) * s;
        v[7] = e5m6_value(w.z << 4) * s;
    }
    // codes 0..3 are the first 48 bits of the string, codes 4..7 the last 48
    __device__ __forceinline__ void get4(float (&v)[4], bool hi) const {
        const uint32_t a = hi ? (w.y << 16) | (w.z >> 16) : w.x, b = hi ? w.z & 0xFFFFu : w.y >> 16;
        v[0] = e5m6_value(a >> 16) * s;
        v[1] = e5m6_value(a >> 4) * s;
        v[2] = e5m6_value((a << 8) | (b >> 8)) * s;
        v[3] = e5m6_value(b << 4) * s;
    }
};

__device__ __forceinline__ float absmax8(const float (&v)[8]) {
    float m = __builtin_fmaxf(__builtin_fabsf(v[0]), __builtin_fabsf(v[1]));
#pragma unroll
    for (int i = 2; i < 8; ++i) m = __builtin_fmaxf(m, __builtin_fabsf(v[i]));
    return m;
}

// ---------------------------------------------------------------------------------------------
// Cross-lane operations on DPP (no LDS).  Maxima take non-negative floats, whose order is the
// order of their bit patterns as unsigned integers, so the steps use integer max.
template <int CTRL> __device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7-i inside each 8
constexpr int kDppMirror = 0x140;     // lane i <-> 15-i inside each 16

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

// value held by lane j of every aligned set of A (1, 2 or 4) lanes
template <int A, int J> __device__ __forceinline__ float bcast_within(float v) {
    static_assert(A == 1 || A == 2 || A == 4, "A");
    if (A == 1) return v;
    constexpr int ctrl = A == 4 ? J * 0x55 : (J ? 0xF5 : 0xA0);   // quad_perm [j,j,j,j] / [j,j,2+j,2+j]
    return u2f(dpp_u32<ctrl>(f2u(v)));
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

// a / C for C in {448, 6}, correctly rounded, in three instructions: q = a*y, r = fma(-C, q, a),
// q + r*y with y = fl(1/C).  For these two constants the result equals the IEEE quotient for EVERY
// positive float whose quotient is a normal number (checked exhaustively over all 2^31 inputs on the
// CPU with a correctly rounded fmaf); smaller operands take the ordinary division.
template <int QMAX> __device__ __forceinline__ float div_by_qmax(float a) {
    constexpr float c = (float)QMAX;
    constexpr float y = 1.0f / c;
    if (QMAX != 448 && QMAX != 6) return a / c;   // E5M6 has one scale per row: the plain division costs nothing there
    if (a < 0x1p-100f) return a / c;
    const float q = a * y;
    return __builtin_fmaf(__builtin_fmaf(-c, q, a), y, q);
}

// QMAX / a for a in [2^-60, 2^60]: the instructions of the IEEE division (reciprocal, one refinement of it, the quotient,
// one refinement, the final residual step) without its operand scaling and its special-case fix-up; on this range
// v_div_scale_f32 returns its operands unchanged and v_div_fixup_f32 the quotient it is given, so the result is
// QMAX / a bit for bit (compared on MI355X with the compiler's division for each of the 1006632961 floats of the range,
// for 448 and for 6, together with the three-instruction a / QMAX above: no difference).
template <int QMAX> __device__ __forceinline__ float qmax_over_plain(float a) {
    constexpr float n = (float)QMAX;
    float r = __builtin_amdgcn_rcpf(a);
    r = __builtin_fmaf(__builtin_fmaf(-a, r, 1.0f), r, r);
    float q = n * r;
    q = __builtin_fmaf(__builtin_fmaf(-a, q, n), r, q);
    return __builtin_fmaf(__builtin_fmaf(-a, q, n), r, q);
}

template <int QMAX> __device__ __forceinline__ Scale make_scale(float amax, float floor_, bool round_sf) {
    const float a = __builtin_fmaxf(amax, floor_);
    Scale r;
    if constexpr (QMAX == 448 || QMAX == 6) {
        // Maxima between 2^-60 and 2^60 in every lane (what any real tensor gives): both divisions in their short forms, chosen
        // by one branch for the wave, so the long forms cost nothing where they are not needed
        const bool plain = f2u(a) - 0x21800000u <= 0x5D800000u - 0x21800000u;
        if (__builtin_expect(__builtin_amdgcn_ballot_w64(!plain) == 0, 1)) {
            constexpr float c = (float)QMAX;
            constexpr float y = 1.0f / c;
            const float q = a * y;
            const float s = __builtin_fmaf(__builtin_fmaf(-c, q, a), y, q);
            if (!round_sf) {
                r.sf = s;
                r.inv = qmax_over_plain<QMAX>(a);
                r.e8 = f2u(s) >> 23;
            } else {
                const uint32_t b = (f2u(s) + 0x007FFFFFu) & 0x7F800000u;
                r.sf = u2f(b);
                r.e8 = b >> 23;
                r.inv = u2f((254u << 23) - b);      // the exponent of s is between 58 and 179 here
            }
            return r;
        }
    }
    const float s = div_by_qmax<QMAX>(a);
    if (!round_sf) {
        r.sf = s;
        r.inv = f2u(s) == 0u ? 0.0f : (float)QMAX / a;
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
    static constexpr int qmax = 448;
    static constexpr float floor_ = 1e-4f;
};
template <> struct Fmt<TK_E2M1> {
    static constexpr int qmax = 6;
    static constexpr float floor_ = 6.0f * 0x1p-126f;
};
template <> struct Fmt<TK_E5M6> {
    static constexpr int qmax = 65024;     // (2 - 2^-6) * 2^15
    static constexpr float floor_ = 1e-4f;
};

// Scales of RPW rows at once.  All lanes of a group already hold the group's amax of every row, so
// instead of every lane repeating the same divisions for every row, lane i of each aligned set of
// A lanes computes the scale of row c*A + i only and the multipliers are handed round with DPP.
//   own[c] : scale computed by this lane, i.e. of row c*A + (lane % A)
//   inv[r] : multiplier of row r, valid in every lane
template <int QMAX, int RPW, int LPG> struct RowScales {
    static constexpr int A = RPW >= 4 && LPG >= 4 ? 4 : (RPW >= 2 ? 2 : 1);
    static constexpr int NC = RPW / A;
    static_assert(RPW % A == 0 && LPG % A == 0, "rows per wave and lanes per group must be multiples of A");
    Scale own[NC];
    float inv[RPW];

    __device__ __forceinline__ void compute(const float (&amax)[RPW], float floor_, bool round_sf, int lane) {
        const int pick = lane & (A - 1);
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            // all candidates are read unconditionally and chosen by value, so the array never has to
            // be addressed dynamically
            const float a0 = amax[c * A];
            const float a1 = A >= 2 ? amax[c * A + (A >= 2 ? 1 : 0)] : 0.0f;
            const float a2 = A >= 4 ? amax[c * A + (A >= 4 ? 2 : 0)] : 0.0f;
            const float a3 = A >= 4 ? amax[c * A + (A >= 4 ? 3 : 0)] : 0.0f;
            float a = a0;
            if (A >= 2) a = pick == 1 ? a1 : a;
            if (A >= 4) { a = pick == 2 ? a2 : a; a = pick == 3 ? a3 : a; }
            own[c] = make_scale<QMAX>(a, floor_, round_sf);
            inv[c * A] = bcast_within<A, 0>(own[c].inv);
            if (A >= 2) inv[c * A + (A >= 2 ? 1 : 0)] = bcast_within<A, 1>(own[c].inv);
            if (A >= 4) {
                inv[c * A + (A >= 4 ? 2 : 0)] = bcast_within<A, 2>(own[c].inv);
                inv[c * A + (A >= 4 ? 3 : 0)] = bcast_within<A, 3>(own[c].inv);
            }
        }
    }
};

// ---------------------------------------------------------------------------------------------
// Conversions.  v_cvt_pk_fp8_f32 on gfx950 is OCP E4M3FN round-to-nearest-even; it does not
// saturate by itself, so inputs that may exceed 448 are clamped first (CLAMP).
template <bool CLAMP> __device__ __forceinline__ u32x2 pack_e4m3x8(const float (&q)[8]) {
    float c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) c[i] = CLAMP ? __builtin_amdgcn_fmed3f(q[i], -448.0f, 448.0f) : q[i];
    // (the first conversion of a dword fills its low half and keeps the rest of its third operand, which the second one
    // overwrites: any register that is at hand serves, and a zero would have to be made first)
    int lo = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], (int)f2u(c[0]), false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], lo, true);
    int hi = __builtin_amdgcn_cvt_pk_fp8_f32(c[4], c[5], (int)f2u(c[4]), false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(c[6], c[7], hi, true);
    return u32x2{(uint32_t)lo, (uint32_t)hi};
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

// fp32 -> 12-bit E5M6 codes, as the reference computes them: the fp16 obtained by rounding toward zero is cut to its
// top 12 bits, and the result is bumped by one when (kept lsb) + (low 17 bits of the fp32 pattern) exceeds 0x10000.
// Where the fp16 is normal those 17 bits are exactly the dropped ones, i.e. round to nearest even; below 2^-14 the
// reference uses the same bits although others were dropped, and so does this.  v_cvt_pkrtz_f16_f32 gives the
// round-toward-zero fp16 of two values at once (subnormals included); the two codes are then formed side by side in
// the halves of one dword, which keeps the conversion at about 8 VALU instructions per element (done one element
// at a time, with compares and selects, the cast of bf16 [8192, 4096] was bound by the VALU: 21.9 us against 19.9).
// Magnitudes from 2^16 up, where the instruction saturates and the reference's fp16 step goes to infinity, cannot
// occur: the values converted are x * (65024 / amax) or x * 2^-k with 2^-k <= 65024 / amax.
__device__ __forceinline__ uint32_t e5m6_code_pair(float a, float b) {
    const uint32_t h2 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
    const uint32_t kept2 = (h2 >> 4) & 0x0FFF0FFFu;
    const uint32_t ta = (f2u(a) & 0x1FFFFu) + (kept2 & 1u);
    const uint32_t tb = (f2u(b) & 0x1FFFFu) + ((kept2 >> 16) & 1u);
    // t > 0x10000  <=>  (t + 0xFFFF) >> 17 is 1 (t is at most 0x20000)
    const uint32_t bump2 = ((ta + 0xFFFFu) >> 17) | (((tb + 0xFFFFu) >> 17) << 16);
    return (kept2 + bump2) & 0x0FFF0FFFu;     // code of a in bits 11..0, of b in bits 27..16
}

__device__ __forceinline__ u32x3 pack_e5m6x8(const float (&q)[8]) {
    const uint32_t c01 = e5m6_code_pair(q[0], q[1]), c23 = e5m6_code_pair(q[2], q[3]);
    const uint32_t c45 = e5m6_code_pair(q[4], q[5]), c67 = e5m6_code_pair(q[6], q[7]);
    const uint32_t c1 = c01 >> 16, c2 = c23 & 0xFFFFu, c3 = c23 >> 16, c4 = c45 & 0xFFFFu, c5 = c45 >> 16, c6 = c67 & 0xFFFFu, c7 = c67 >> 16;
    return u32x3{(c01 << 20) | (c1 << 8) | (c2 >> 4),
                 (c2 << 28) | (c3 << 16) | (c4 << 4) | (c5 >> 8),
                 (c5 << 24) | (c6 << 12) | c7};
}

// scale 8 values and convert: the 8 E4M3 codes, or the 8 E2M1 codes in the first word (the second is 0)
template <int FMT, bool CLAMP> __device__ __forceinline__ u32x2 quantise8(const float (&v)[8], float inv) {
    static_assert(FMT == TK_E4M3 || FMT == TK_E2M1, "formats with whole-word codes");
    float q[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = v[i] * inv;
    if (FMT == TK_E4M3) return pack_e4m3x8<CLAMP>(q);
    return u32x2{pack_e2m1x8(q), 0u};
}

// scale 8 values, convert, store: 8 bytes (E4M3), 4 bytes (E2M1) or 12 bytes (E5M6) per lane
template <int FMT, bool CLAMP>
__device__ __forceinline__ void quantise_store8(const float (&v)[8], float inv, uint8_t *out_row, int col) {
    float q[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = v[i] * inv;
    if (FMT == TK_E4M3) st_stream8(out_row + col, pack_e4m3x8<CLAMP>(q));
    else if (FMT == TK_E2M1) st_stream4(out_row + (col >> 1), pack_e2m1x8(q));
    else __builtin_nontemporal_store(pack_e5m6x8(q), reinterpret_cast<u32x3_a4 *>(out_row + (col >> 3) * 12));
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
    // Only the load sits inside the branches.  Arithmetic on the loaded value in there (the byte of the packed
    // layout shifted into an exponent) makes the compiler wait for the load before it leaves the branch, and the
    // loads of several rows then complete one after the other: dequantisation of E4M3 [8192, 4096] with packed
    // scales took 19.2 us against 17.2 us with fp32 scales.  So the packed layout reads the aligned word that
    // holds the byte, and the extraction happens after the branches with operands that are the identity for fp32.
    const bool packed = s.layout == TK_SF_COL_UE8M0;
    uint32_t w;
    if (s.layout == TK_SF_ROW_F32) w = reinterpret_cast<const uint32_t *>(s.base)[(int64_t)m * s.ld + k];
    else if (s.layout == TK_SF_COL_F32) w = reinterpret_cast<const uint32_t *>(s.base)[(int64_t)k * s.ld + m];
    else w = *reinterpret_cast<const uint32_t *>(reinterpret_cast<const uint8_t *>(s.base) + (int64_t)(k >> 2) * s.ld + 4 * (int64_t)m);
    const uint32_t down = packed ? 8u * (uint32_t)(k & 3) : 0u, keep = packed ? 0xFFu : 0xFFFFFFFFu, up = packed ? 23u : 0u;
    return u2f(((w >> down) & keep) << up);
}

// The same without a branch: the layout only selects how the byte offset is formed, and the packed layout
// is read as the aligned word that holds the byte (its storage consists of whole 4-byte words).  Loads of
// several rows then go out back to back instead of one per branch.  Measured on MI355X: the given-scale
// cast of bf16 [4096, 7168] 16.7 -> 16.0 us; the loaders of quantised input are better off with the
// branches (re-quantisation of E4M3 [8192, 4096] 11.9 us against 12.3 us, dequantisation unchanged).
__device__ __forceinline__ float sf_load_select(const SfRef &s, int m, int k) {
    const bool packed = s.layout == TK_SF_COL_UE8M0;
    const int64_t major = s.layout == TK_SF_ROW_F32 ? m : (packed ? k >> 2 : k);
    const int64_t minor = s.layout == TK_SF_ROW_F32 ? k : m;
    const int64_t off = packed ? major * s.ld + 4 * minor + (k & 3) : 4 * (major * s.ld + minor);
    const uint32_t w = *reinterpret_cast<const uint32_t *>(reinterpret_cast<const uint8_t *>(s.base) + (off & ~(int64_t)3));
    return u2f(packed ? ((w >> (8 * (k & 3))) & 0xFFu) << 23 : w);
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

// Write the fp32 scales of one tile, staged in LDS as stage[row][g] (g < gpr <= PITCH), to the
// row-major layout: consecutive lanes take consecutive groups of a row, so each row leaves as one
// contiguous run.
template <int ROWS, int PITCH>
__device__ __forceinline__ void sf_store_tile_rowmajor(const SfRef &s, const uint32_t (*stage)[PITCH], int gpr, int m0, int k0) {
    for (int e = threadIdx.x; e < ROWS * gpr; e += blockDim.x) {
        const int r = e / gpr, g = e - r * gpr;
        const int m = m0 + r, k = k0 + g;
        if (m < s.nm && k < s.nk) st_stream4(reinterpret_cast<uint32_t *>(s.base) + (int64_t)m * s.ld + k, stage[r][g]);
    }
}

// Write the scales of one tile of ROWS rows, staged in LDS as stage[row][g] (fp32 bits or exponent
// byte), to a column-major layout: consecutive lanes take consecutive rows, so ROWS lanes fill one
// contiguous 4*ROWS-byte segment.
//   GPS    : groups per row in the stage
//   m0, k0 : block coordinates of stage[0][0]
template <int ROWS, int GPS>
__device__ __forceinline__ void sf_store_tile_colmajor(const SfRef &s, const uint32_t (*stage)[GPS], int m0, int k0) {
    if (s.layout == TK_SF_COL_F32) {
        for (int e = threadIdx.x; e < GPS * ROWS; e += kThreads) {
            const int g = e / ROWS, r = e % ROWS;
            const int m = m0 + r, k = k0 + g;
            if (m < s.nm && k < s.nk) st_stream4(reinterpret_cast<uint32_t *>(s.base) + (int64_t)k * s.ld + m, stage[r][g]);
        }
    } else {
        constexpr int WPS = (GPS + 3) / 4;   // words per row in the stage
        for (int e = threadIdx.x; e < WPS * ROWS; e += kThreads) {
            const int wd = e / ROWS, r = e % ROWS;
            const int m = m0 + r, k = k0 + 4 * wd;
            if (m < s.nm && k < s.nk) {
                uint32_t word = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (4 * wd + j < GPS && k + j < s.nk) word |= (stage[r][4 * wd + j] & 0xFFu) << (8 * j);
                st_stream4(reinterpret_cast<uint8_t *>(s.base) + (int64_t)(k >> 2) * s.ld + 4 * (int64_t)m, word);
            }
        }
    }
}

}  // namespace tk
