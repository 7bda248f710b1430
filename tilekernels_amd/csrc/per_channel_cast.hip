// Per-channel (N tokens x 1 column, N in {32, 128}) E4M3 cast for gfx950, with the fusions the
// reference offers around it: row gather (pos_to_token), dequantisation of an E4M3 input with 1 x 128
// scales, SwiGLU in front, and a transposed ([K, M]) output.
//
// A workgroup of 8 waves owns a 128-token x 256-column tile and keeps it in registers between the
// amax and the conversion, so HBM is read once.  Half a wave (32 lanes x 8 columns = 256 columns)
// takes 8 consecutive tokens: wave w, half h holds tokens 16 w + 8 h + p, p = 0..7.  A lane
// therefore owns 8 columns over 8 tokens and reduces |x| down its columns without any cross-lane
// step; the 16 partial maxima per column (8 waves x 2 halves) meet in LDS, thread c < 256 derives
// the scale(s) of column c (one division per scale in the whole workgroup, stored as one coalesced
// run) and hands the multipliers back through LDS.
//   plain output      : a lane converts 8 columns of a token -> one 8-byte store, 256 bytes per half-wave
//   transposed output : a lane converts 8 tokens of a column -> 8 bytes of an output row; the tile is
//                       turned in LDS ([256 columns][128 tokens] bytes) and leaves as 128-byte row pieces
//
// Reference semantics: tile_kernels/quant/per_channel_cast_fused_kernel.py:16-203,
// per_channel_cast_and_transpose_kernel.py:8-123,
// swiglu_forward_and_per_channel_cast_and_transpose_kernel.py:9-231; oracle
// tile_kernels/torch/per_channel_cast_fused.py and tile_kernels/torch/cast.py with block (N, 1).
#include "swiglu_math.hpp"
#include "tk_device.hpp"
#include "tk_host.hpp"

namespace tk {

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kPcTileM = 128, kPcTileK = 256;
// Consecutive tokens per lane.  With 4 (1024 threads per tile) every mode measured slower on MI355X at
// [8192, 4096]: plain 17.7 -> 18.3 us, FP8 input 13.4 -> 14.6, transposed 21.1 -> 24.0, SwiGLU 17.3 -> 18.0.
constexpr int kPcRows = 8;
constexpr int kPcParts = kPcTileM / kPcRows;             // half-waves per tile = partial maxima per column: 16
constexpr int kPcThreads = 32 * kPcParts;                // 512
// Turned tile in LDS: one row of 128 token bytes per column, rows 144 bytes apart.  A lane writes the 8
// tokens it holds of column 8 hl + j as one 8-byte word; left at its natural place (8 part) the 32
// lanes of a half-wave would meet in two of the 32 8-byte bank pairs (rows 8 x 144 bytes apart).  So
// the 16-byte unit of a row is rotated by (hl >> 1) & 7 and the two halves of the unit are exchanged
// when hl >= 16: with the row pitch supplying hl & 1, the five bits of hl land in five different bits
// of the bank-pair index and a half-wave's writes touch every bank pair once.  Units stay whole, so
// the reader still takes 16 bytes at a time.
constexpr int kPcPitch = kPcTileM + 16;

enum { PC_BF16 = 0, PC_E4M3 = 1, PC_SWIGLU = 2, PC_F32 = 3 };

struct PerChannelParams {
    const void *x;
    const float *x_sf;
    const int32_t *pos_to_token;
    uint8_t *out;
    float *out_sf;
    int num_tokens, K, M;      // input rows, columns (of the output), output rows
    int tiles_k;
    int round_sf, use_clamp;
    float clamp;
};

#define TK_PC_KERNEL_ARGS                                                                                          \
    const void *a_x, uint8_t *a_out, float *a_out_sf, const float *a_x_sf, const int32_t *a_p2t, int a_T, int a_K, \
        int a_M, int a_tiles_k, int a_round_sf, int a_use_clamp, float a_clamp
#define TK_PC_KERNEL_UNPACK \
    const PerChannelParams p{a_x, a_x_sf, a_p2t, a_out, a_out_sf, a_T, a_K, a_M, a_tiles_k, a_round_sf, a_use_clamp, a_clamp}
#define TK_PC_LAUNCH_ARGS(p) \
    (p).x, (p).out, (p).out_sf, (p).x_sf, (p).pos_to_token, (p).num_tokens, (p).K, (p).M, (p).tiles_k, (p).round_sf, (p).use_clamp, (p).clamp

template <int MODE> struct PcRaw { typedef Raw8<bf16_t> type; };
template <> struct PcRaw<PC_E4M3> { typedef Raw8<e4m3in_t> type; };
template <> struct PcRaw<PC_F32> { typedef Raw8<float> type; };

// Makes the compiler treat the packed input as redefined here, so that what was unpacked from it before
// cannot be kept alive across this point.
__device__ __forceinline__ void forget_unpacked(Raw8<bf16_t> &r) { asm volatile("" : "+v"(r.w)); }
__device__ __forceinline__ void forget_unpacked(Raw8<e4m3in_t> &r) { asm volatile("" : "+v"(r.w)); }
__device__ __forceinline__ void forget_unpacked(Raw8<float> &) {}   // nothing is unpacked: the registers are the values

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{a, b}), bf16x2));
}

template <int MODE, int NPT, bool TRANS, bool GATHER>
__global__ __launch_bounds__(kPcThreads, 4) void per_channel_cast_kernel(TK_PC_KERNEL_ARGS) {
    TK_PC_KERNEL_UNPACK;
    constexpr int NB = kPcTileM / NPT;          // scale blocks per tile along the tokens: 1 or 4
    typedef typename PcRaw<MODE>::type Raw;
    // the partial maxima are dead once the scales exist (second barrier), so the turned tile reuses their space
    constexpr int kPartBytes = kPcParts * kPcTileK * 4, kTurnedBytes = TRANS ? kPcTileK * kPcPitch : 0;
    __shared__ __attribute__((aligned(16))) uint8_t lds[kPartBytes > kTurnedBytes ? kPartBytes : kTurnedBytes];
    __shared__ __attribute__((aligned(16))) float inv_s[NB][kPcTileK];
    float (*part)[kPcTileK] = reinterpret_cast<float (*)[kPcTileK]>(lds);    // [wave * 2 + half][column]
    uint8_t *turned = lds;

    // 2-D grid (x = column tile, y = token tile); the FP8-input mode runs on a 1-D grid that it reorders
    int tile_m = blockIdx.y, tile_k = blockIdx.x;
    if constexpr (MODE == PC_E4M3) {
        tile_m = blockIdx.x / p.tiles_k;
        tile_k = blockIdx.x - tile_m * p.tiles_k;
        // Workgroups are dealt to the 8 XCDs (each with its own L2) round-robin.  The tiles of one token
        // range share the 128-byte lines of the input scales, so they are given to one XCD: 8 token
        // ranges advance side by side, one per XCD.  (Without this the scale lines are fetched 8 times.)
        const int tiles_m = (p.M + kPcTileM - 1) / kPcTileM, striped = (tiles_m / 8) * 8 * p.tiles_k;
        if ((int)blockIdx.x < striped) {
            const int q = blockIdx.x >> 3;
            tile_k = q % p.tiles_k;
            tile_m = (q / p.tiles_k) * 8 + (blockIdx.x & 7);
        }
    }
    const int lane = threadIdx.x & 63, wave = wave_id();
    const int half = lane >> 5, hl = lane & 31;
    const int col0 = tile_k * kPcTileK, col = col0 + hl * 8;
    const bool col_ok = col < p.K;
    const int tok0 = tile_m * kPcTileM + (wave * 2 + half) * kPcRows;
    const bool rows_ok = tok0 < p.M;            // M is a multiple of 16: all 8 tokens of a lane or none
    const int64_t in_ld = MODE == PC_SWIGLU ? 2 * (int64_t)p.K : p.K;

    // ---- load (and, for SwiGLU, activate) 8 tokens x 8 columns.  Whether a lane has anything to load
    // does not depend on the token (M is a multiple of 16), so the loads sit in straight-line code
    // under one branch; a gathered row with a negative index is read from row 0 and zeroed by value.
    Raw raw[kPcRows];
#pragma unroll
    for (int r = 0; r < kPcRows; ++r) raw[r].zero();
    if (rows_ok && col_ok) {
        if constexpr (MODE == PC_SWIGLU) {
            // all sixteen loads of the lane go out before the first activation is evaluated (issuing them in batches of
            // 4 or 2 tokens brings the kernel from 92 to 67 / 61 VGPRs and more waves per SIMD, but measured 18-19 us
            // against 16.8 us for bf16 [8192, 4096])
            Raw8<bf16_t> rg[kPcRows], ru[kPcRows];
#pragma unroll
            for (int r = 0; r < kPcRows; ++r) {
                const uint16_t *xr = reinterpret_cast<const uint16_t *>(p.x) + (int64_t)(tok0 + r) * in_ld + col;
                rg[r].load(xr);
                vmem_issue_gap();
                ru[r].load(xr + p.K);
                vmem_issue_gap();
            }
            __builtin_amdgcn_sched_barrier(0);
            // the clamp arguments lie beyond the preloaded ones: touched only now, behind the loads.
            // No clamp = clamp at infinity, so there is no branch in the hot loop.
            float clamp_arg = p.clamp;
            int use_clamp = p.use_clamp;
            asm volatile("" : "+s"(clamp_arg), "+s"(use_clamp));
            const float cl = use_clamp ? clamp_arg : __builtin_inff();
            const float lo = cl >= 0.0f ? -cl : cl;      // (a negative limit makes every element the limit, as the two-step form does)
#pragma unroll
            for (int r = 0; r < kPcRows; ++r) {
                float g[8], u[8], a[8];
                rg[r].get(g);
                ru[r].get(u);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    g[i] = __builtin_fminf(g[i], cl);
                    u[i] = __builtin_amdgcn_fmed3f(u[i], lo, cl);      // min(max(u, -cl), cl) in one instruction
                    a[i] = silu_mul<bf16_t>(g[i], u[i]);
                }
                // the activation is rounded to bf16 before it is quantised, as in the reference
                raw[r].w = u32x4{pack_bf16x2(a[0], a[1]), pack_bf16x2(a[2], a[3]), pack_bf16x2(a[4], a[5]), pack_bf16x2(a[6], a[7])};
            }
        } else {
            // (the gather indices of all rows are asked for before the first row's data: a load whose address hangs on a loaded value
            // waits for every load issued before it)
            int gathered[kPcRows];
            bool valid[kPcRows];
            if constexpr (GATHER) {
#pragma unroll
                for (int r = 0; r < kPcRows; ++r) gathered[r] = p.pos_to_token[tok0 + r];
            }
#pragma unroll
            for (int r = 0; r < kPcRows; ++r) {
                int src = tok0 + r;
                valid[r] = true;
                if constexpr (GATHER) {
                    src = gathered[r];
                    valid[r] = src >= 0 && src < p.num_tokens;
                    src = valid[r] ? src : 0;
                }
                if constexpr (MODE == PC_E4M3) {
                    raw[r].load(reinterpret_cast<const uint8_t *>(p.x) + (int64_t)src * in_ld + col);
                    vmem_issue_gap();
                    raw[r].s = p.x_sf[(int64_t)src * (p.K >> 7) + (col >> 7)];
                    vmem_issue_gap();
                } else if constexpr (MODE == PC_F32) {
                    raw[r].load(reinterpret_cast<const float *>(p.x) + (int64_t)src * in_ld + col);
                    vmem_issue_gap();
                } else {
                    raw[r].load(reinterpret_cast<const uint16_t *>(p.x) + (int64_t)src * in_ld + col);
                    vmem_issue_gap();
                }
            }
            // (rows without a source are cleared once all loads are out: clearing a register a load is still to fill means waiting for it)
            if constexpr (GATHER) {
#pragma unroll
                for (int r = 0; r < kPcRows; ++r)
                    if (!valid[r]) raw[r].zero();
            }
        }
    }

    // ---- |x| maxima down this lane's 8 columns
    float m[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) m[j] = 0.0f;
#pragma unroll
    for (int r = 0; r < kPcRows; ++r) {
        float v[8];
        raw[r].get(v);
#pragma unroll
        for (int j = 0; j < 8; ++j) m[j] = __builtin_fmaxf(m[j], __builtin_fabsf(v[j]));
    }
    // the tile is unpacked a second time after the scales are known; without this the compiler keeps
    // all 64 unpacked values alive across the two barriers instead
#pragma unroll
    for (int r = 0; r < kPcRows; ++r) forget_unpacked(raw[r]);
    {
        u32x4 *dst = reinterpret_cast<u32x4 *>(&part[wave * 2 + half][hl * 8]);
        dst[0] = u32x4{f2u(m[0]), f2u(m[1]), f2u(m[2]), f2u(m[3])};
        dst[1] = u32x4{f2u(m[4]), f2u(m[5]), f2u(m[6]), f2u(m[7])};
    }
    __syncthreads();

    // ---- thread c: scale(s) of column c
    if (threadIdx.x < kPcTileK) {
        const int c = threadIdx.x;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            float a = 0.0f;
#pragma unroll
            for (int i = 0; i < kPcParts / NB; ++i) a = __builtin_fmaxf(a, part[b * (kPcParts / NB) + i][c]);
            const Scale sc = make_scale<448>(a, Fmt<TK_E4M3>::floor_, p.round_sf != 0);
            inv_s[b][c] = sc.inv;
            const int tok = tile_m * kPcTileM + b * NPT;
            if (tok < p.M && col0 + c < p.K) st_stream4(p.out_sf + (int64_t)(tok / NPT) * p.K + col0 + c, f2u(sc.sf));
        }
    }
    __syncthreads();

    float inv[8];
    {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(&inv_s[NB == 1 ? 0 : (wave * 2 * kPcRows) / 32][hl * 8]);
        const u32x4 a = src[0], b = src[1];
        inv[0] = u2f(a.x); inv[1] = u2f(a.y); inv[2] = u2f(a.z); inv[3] = u2f(a.w);
        inv[4] = u2f(b.x); inv[5] = u2f(b.y); inv[6] = u2f(b.z); inv[7] = u2f(b.w);
    }

    if constexpr (!TRANS) {
#pragma unroll
        for (int r = 0; r < kPcRows; ++r) {
            float v[8], q[8];
            raw[r].get(v);
#pragma unroll
            for (int j = 0; j < 8; ++j) q[j] = v[j] * inv[j];
            if (rows_ok && col_ok) st_stream8(p.out + (int64_t)(tok0 + r) * p.K + col, pack_e4m3x8<false>(q));
        }
    } else {
        // codes of the lane's 8 consecutive tokens per column: token pairs fill the 16-bit halves of a dword
        uint32_t acc[8][2];
#pragma unroll
        for (int d = 0; d < 2; ++d) {
            float v0[8], v1[8], v2[8], v3[8];
            raw[4 * d].get(v0);
            raw[4 * d + 1].get(v1);
            raw[4 * d + 2].get(v2);
            raw[4 * d + 3].get(v3);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int lo = __builtin_amdgcn_cvt_pk_fp8_f32(v0[j] * inv[j], v1[j] * inv[j], 0, false);
                acc[j][d] = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(v2[j] * inv[j], v3[j] * inv[j], lo, true);
            }
        }
        {
            const int part = wave * 2 + half;
            const int unit = ((part >> 1) + (hl >> 1)) & 7, low = (part & 1) ^ (hl >> 4);
            uint8_t *dst = &turned[hl * 8 * kPcPitch + unit * 16 + low * 8];
#pragma unroll
            for (int j = 0; j < 8; ++j) *reinterpret_cast<u32x2 *>(dst + j * kPcPitch) = u32x2{acc[j][0], acc[j][1]};
        }
        __syncthreads();
        // 8 lanes x 16 bytes = the 128 tokens of one output row; a wave stores 8 rows per step
        const int chunk = threadIdx.x & 7;
        const int tok = tile_m * kPcTileM + chunk * 16;
#pragma unroll
        for (int i = 0; i < kPcTileK / (kPcThreads / 8); ++i) {
            const int h = (threadIdx.x >> 3) + (kPcThreads / 8) * i;
            if (col0 + h < p.K && tok < p.M) {
                const int unit = (chunk + (h >> 4)) & 7;
                u32x4 d = *reinterpret_cast<const u32x4 *>(&turned[h * kPcPitch + unit * 16]);
                if (i >= 2) d = u32x4{d.z, d.w, d.x, d.y};          // rows of the lanes hl >= 16: h >= 128
                // (write-through stores against non-temporal ones, bf16 [8192, 4096] on MI355X: plain and FP8 input 19.6 -> 19.2 us,
                // behind the SwiGLU 16.7 -> 16.9 us; ordinary stores 19.6 and 18.4 us)
                if constexpr (MODE != PC_SWIGLU) st_stream16(p.out + (int64_t)(col0 + h) * p.M + tok, d);
                else __builtin_nontemporal_store(d, reinterpret_cast<u32x4 *>(p.out + (int64_t)(col0 + h) * p.M + tok));
            }
        }
    }
}

// E4M3 input with 1 x 128 scales, plain (not transposed) output, with 16 codes per lane instead of 8: a workgroup of 512
// threads owns 128 tokens x 512 columns, half a wave (32 lanes x 16 columns) takes 8 consecutive tokens, and every
// load and store instruction of a lane moves 16 bytes (8 bytes per lane make a half-wave's instruction 256 bytes
// long; measured on MI355X at [8192, 4096]: 13.8 us that way, 12.8 us this way).  The rest is the kernel above: maxima down the lane's columns, the 16 partial maxima per column meet in LDS,
// thread c derives the scale(s) of column c and hands the multipliers back.
constexpr int kPcWideK = 512;

template <int NPT, bool GATHER>
__global__ __launch_bounds__(kPcThreads, 4) void per_channel_cast_fp8in_kernel(TK_PC_KERNEL_ARGS) {
    TK_PC_KERNEL_UNPACK;
    constexpr int NB = kPcTileM / NPT;
    __shared__ __attribute__((aligned(16))) float part[kPcParts][kPcWideK];
    __shared__ __attribute__((aligned(16))) float inv_s[NB][kPcWideK];

    // the tiles of one token range share the 128-byte lines of the input scales: 8 token ranges advance side by
    // side, one per XCD (workgroups are dealt to the XCDs round-robin)
    int tile_m = blockIdx.x / p.tiles_k, tile_k = blockIdx.x - tile_m * p.tiles_k;
    const int tiles_m = (p.M + kPcTileM - 1) / kPcTileM, striped = (tiles_m / 8) * 8 * p.tiles_k;
    if ((int)blockIdx.x < striped) {
        const int q = blockIdx.x >> 3;
        tile_k = q % p.tiles_k;
        tile_m = (q / p.tiles_k) * 8 + (blockIdx.x & 7);
    }
    const int lane = threadIdx.x & 63, wave = wave_id();
    const int half = lane >> 5, hl = lane & 31;
    const int col0 = tile_k * kPcWideK, col = col0 + hl * 16;
    const bool col_ok = col < p.K;              // K is a multiple of 128: all 16 columns of a lane or none
    const int tok0 = tile_m * kPcTileM + (wave * 2 + half) * kPcRows;
    const bool rows_ok = tok0 < p.M;            // M is a multiple of 16: all 8 tokens of a lane or none

    Raw8<e4m3in_t> lo[kPcRows], hi[kPcRows];
#pragma unroll
    for (int r = 0; r < kPcRows; ++r) { lo[r].zero(); hi[r].zero(); }
    if (rows_ok && col_ok) {
        // (gather indices of all rows first: see per_channel_cast_kernel)
        int gathered[kPcRows];
        if constexpr (GATHER) {
#pragma unroll
            for (int r = 0; r < kPcRows; ++r) gathered[r] = p.pos_to_token[tok0 + r];
        }
#pragma unroll
        for (int r = 0; r < kPcRows; ++r) {
            int src = tok0 + r;
            bool valid = true;
            if constexpr (GATHER) {
                src = gathered[r];
                valid = src >= 0 && src < p.num_tokens;
                src = valid ? src : 0;
            }
            const u32x4 w = ld_stream16(reinterpret_cast<const uint8_t *>(p.x) + (int64_t)src * p.K + col);
            vmem_issue_gap();
            lo[r].w = u32x2{w.x, w.y};
            hi[r].w = u32x2{w.z, w.w};
            lo[r].s = hi[r].s = p.x_sf[(int64_t)src * (p.K >> 7) + (col >> 7)];
            vmem_issue_gap();
            gathered[r] = valid ? 1 : 0;
        }
        if constexpr (GATHER) {      // (cleared once all loads are out)
#pragma unroll
            for (int r = 0; r < kPcRows; ++r)
                if (!gathered[r]) { lo[r].zero(); hi[r].zero(); }
        }
    }

    float m[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) m[j] = 0.0f;
#pragma unroll
    for (int r = 0; r < kPcRows; ++r) {
        float a[8], b[8];
        lo[r].get(a);
        hi[r].get(b);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            m[j] = __builtin_fmaxf(m[j], __builtin_fabsf(a[j]));
            m[8 + j] = __builtin_fmaxf(m[8 + j], __builtin_fabsf(b[j]));
        }
    }
    // the tile is decoded a second time after the scales are known, instead of 128 values kept alive across the barriers
#pragma unroll
    for (int r = 0; r < kPcRows; ++r) { forget_unpacked(lo[r]); forget_unpacked(hi[r]); }
    {
        u32x4 *dst = reinterpret_cast<u32x4 *>(&part[wave * 2 + half][hl * 16]);
#pragma unroll
        for (int q = 0; q < 4; ++q) dst[q] = u32x4{f2u(m[4 * q]), f2u(m[4 * q + 1]), f2u(m[4 * q + 2]), f2u(m[4 * q + 3])};
    }
    __syncthreads();

    {
        const int c = threadIdx.x;               // 512 threads, 512 columns
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            float a = 0.0f;
#pragma unroll
            for (int i = 0; i < kPcParts / NB; ++i) a = __builtin_fmaxf(a, part[b * (kPcParts / NB) + i][c]);
            const Scale sc = make_scale<448>(a, Fmt<TK_E4M3>::floor_, p.round_sf != 0);
            inv_s[b][c] = sc.inv;
            const int tok = tile_m * kPcTileM + b * NPT;
            if (tok < p.M && col0 + c < p.K) st_stream4(p.out_sf + (int64_t)(tok / NPT) * p.K + col0 + c, f2u(sc.sf));
        }
    }
    __syncthreads();

    float inv[16];
    {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(&inv_s[NB == 1 ? 0 : (wave * 2 * kPcRows) / 32][hl * 16]);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const u32x4 v = src[q];
            inv[4 * q] = u2f(v.x); inv[4 * q + 1] = u2f(v.y); inv[4 * q + 2] = u2f(v.z); inv[4 * q + 3] = u2f(v.w);
        }
    }
#pragma unroll
    for (int r = 0; r < kPcRows; ++r) {
        float a[8], b[8];
        lo[r].get(a);
        hi[r].get(b);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            a[j] = a[j] * inv[j];
            b[j] = b[j] * inv[8 + j];
        }
        const u32x2 x0 = pack_e4m3x8<false>(a), x1 = pack_e4m3x8<false>(b);
        if (rows_ok && col_ok)
            __builtin_nontemporal_store(u32x4{x0.x, x0.y, x1.x, x1.y}, reinterpret_cast<u32x4 *>(p.out + (int64_t)(tok0 + r) * p.K + col));
    }
}

template <int MODE, int NPT>
static void launch_per_channel_2(const PerChannelParams &p, bool transpose, hipStream_t stream) {
    const int tiles_m = (p.M + kPcTileM - 1) / kPcTileM;
    const dim3 block(kPcThreads);
    if constexpr (MODE == PC_E4M3) {
        if (!transpose && aligned_to(p.x, 16) && aligned_to(p.out, 16)) {
            const int wide_k = (p.K + kPcWideK - 1) / kPcWideK;
            PerChannelParams q = p;
            q.tiles_k = wide_k;
            const dim3 wide_grid((unsigned)(tiles_m * wide_k));
            if (p.pos_to_token) hipLaunchKernelGGL((per_channel_cast_fp8in_kernel<NPT, true>), wide_grid, block, 0, stream, TK_PC_LAUNCH_ARGS(q));
            else hipLaunchKernelGGL((per_channel_cast_fp8in_kernel<NPT, false>), wide_grid, block, 0, stream, TK_PC_LAUNCH_ARGS(q));
            return;
        }
    }
    // (token tiles on x, so that successive workgroups write neighbouring pieces of the same transposed rows,
    // measured slower: 19.7 -> 21.1 us transposed, 17.4 -> 20.3 us with SwiGLU)
    const dim3 grid = MODE == PC_E4M3 ? dim3((unsigned)(tiles_m * p.tiles_k)) : dim3((unsigned)p.tiles_k, (unsigned)tiles_m);
#define TK_PC_LAUNCH(T, G) \
    hipLaunchKernelGGL((per_channel_cast_kernel<MODE, NPT, T, G>), grid, block, 0, stream, TK_PC_LAUNCH_ARGS(p))
    if constexpr (MODE == PC_SWIGLU) {
        if (transpose) TK_PC_LAUNCH(true, false);
        else TK_PC_LAUNCH(false, false);
    } else if constexpr (MODE == PC_F32) {   // checked before: no transposed output from fp32
        if (p.pos_to_token) TK_PC_LAUNCH(false, true);
        else TK_PC_LAUNCH(false, false);
    } else if (p.pos_to_token) {
        if (transpose) TK_PC_LAUNCH(true, true);
        else TK_PC_LAUNCH(false, true);
    } else {
        if (transpose) TK_PC_LAUNCH(true, false);
        else TK_PC_LAUNCH(false, false);
    }
#undef TK_PC_LAUNCH
}

template <int MODE>
static hipError_t launch_per_channel(const PerChannelParams &p, int num_per_tokens, bool transpose, hipStream_t stream) {
    if (num_per_tokens == 128) launch_per_channel_2<MODE, 128>(p, transpose, stream);
    else launch_per_channel_2<MODE, 32>(p, transpose, stream);
    return hipGetLastError();
}

}  // namespace tk

using namespace tk;

extern "C" int tk_check_per_channel_cast(const void *x, int x_dtype, const float *x_sf, int64_t num_tokens, int64_t K,
                                         const int32_t *pos_to_token, int64_t M, const void *out, const float *out_sf,
                                         int num_per_tokens, int round_sf, int transpose, int swiglu, int use_clamp,
                                         float clamp) {
    (void)round_sf;
    (void)pos_to_token;
    (void)transpose;
    if (x_dtype != TK_BF16 && x_dtype != TK_F32) return TK_ERR_BAD_DTYPE;
    if (x_dtype == TK_F32 && (x_sf || swiglu || transpose)) return TK_ERR_BAD_DTYPE;   // as the reference: plain and gathered casts only
    if (num_per_tokens != 32 && num_per_tokens != 128) return TK_ERR_BAD_GROUP;
    if (num_tokens < 0 || M < 0 || K <= 0 || K % 8 != 0 || M % 16 != 0) return TK_ERR_BAD_SHAPE;
    if (x_sf && (K % 128 != 0 || swiglu)) return TK_ERR_BAD_MODE;
    if (!pos_to_token && num_tokens < M) return TK_ERR_BAD_SHAPE;
    // gathered rows with a negative index are read from row 0 and zeroed by value, so that row must exist
    if (pos_to_token && num_tokens == 0 && M > 0) return TK_ERR_BAD_SHAPE;
    if (swiglu && pos_to_token) return TK_ERR_BAD_MODE;
    if (use_clamp && (!swiglu || !(clamp == clamp))) return TK_ERR_BAD_VALUE;
    if (num_tokens > INT32_MAX - 256 || M > INT32_MAX - 256 || K > (INT32_MAX - 1024) / 2) return TK_ERR_TOO_LARGE;
    if (M == 0) return TK_OK;
    if (!x || !out || !out_sf) return TK_ERR_NULL_POINTER;
    if (!aligned_to(x, x_sf ? 8 : 16) || !aligned_to(out, transpose ? 16 : 8) || !aligned_to(out_sf, 4) || !aligned_to(x_sf, 4))
        return TK_ERR_MISALIGNED;
    const int64_t tiles = ((M + kPcTileM - 1) / kPcTileM) * ((K + kPcTileK - 1) / kPcTileK);
    if (tiles > INT32_MAX - 8 || (M + kPcTileM - 1) / kPcTileM > 65535) return TK_ERR_TOO_LARGE;   // token tiles ride on grid.y
    return TK_OK;
}

extern "C" int tk_per_channel_cast(const void *x, int x_dtype, const float *x_sf, int64_t num_tokens, int64_t K,
                                   const int32_t *pos_to_token, int64_t M, void *out, float *out_sf, int num_per_tokens,
                                   int round_sf, int transpose, int swiglu, int use_clamp, float clamp, void *stream) {
    const int rc = tk_check_per_channel_cast(x, x_dtype, x_sf, num_tokens, K, pos_to_token, M, out, out_sf, num_per_tokens,
                                             round_sf, transpose, swiglu, use_clamp, clamp);
    if (rc != TK_OK || M == 0) return rc;
    PerChannelParams p;
    p.x = x;
    p.x_sf = x_sf;
    p.pos_to_token = pos_to_token;
    p.out = static_cast<uint8_t *>(out);
    p.out_sf = out_sf;
    p.num_tokens = (int)num_tokens;
    p.K = (int)K;
    p.M = (int)M;
    p.tiles_k = (int)((K + kPcTileK - 1) / kPcTileK);
    p.round_sf = round_sf;
    p.use_clamp = use_clamp;
    p.clamp = clamp;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e;
    if (swiglu) e = launch_per_channel<PC_SWIGLU>(p, num_per_tokens, transpose != 0, s);
    else if (x_sf) e = launch_per_channel<PC_E4M3>(p, num_per_tokens, transpose != 0, s);
    else if (x_dtype == TK_F32) e = launch_per_channel<PC_F32>(p, num_per_tokens, false, s);
    else e = launch_per_channel<PC_BF16>(p, num_per_tokens, transpose != 0, s);
    return (int)e;
}
