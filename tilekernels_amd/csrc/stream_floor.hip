// Measurement aid: a kernel with the memory traffic of the cast kernels and no arithmetic.
//
// A wave takes PIECES consecutive 512-column pieces of one row of a bf16 matrix, all its 16-byte loads issued
// before the first is used (the same streaming loads as the casts), and writes one byte per element (the same
// 8-byte write-through stores), plus one 4-byte word per 128 columns where the operator it stands beside writes
// scales.  With `two_halves` the row has 2 * cols elements and a lane reads the piece of both halves, as the fused
// SwiGLU cast does.  The bytes stored are the XOR of the words loaded, so no load can be dropped by the compiler;
// there is no reduction, no conversion, no cross-lane step.  What this kernel takes on a given shape is what the
// access pattern costs on the machine; the difference to the real operator is the operator's arithmetic.
//
// With STAMP every wave also reports when it ran: the 100 MHz real-time counter at its start, when its last load
// has arrived (this variant waits for all loads before its first store), when its stores are issued and when they
// are acknowledged, plus the hardware id registers that say where it ran (XCD, shader engine, CU, SIMD).  From these
// stamps of a few back-to-back launches one reads how a launch of this size is spent: the gap between two launches, how
// long the waves take to start, when the first data arrives, how evenly the XCDs finish.
#include "tk_device.hpp"
#include "tk_host.hpp"

namespace tk {

constexpr int kStampWords = 6;     // per wave: start, loads done, stores issued, stores acknowledged, HW_ID, XCC_ID

template <int PIECES, bool TWO, bool STAMP>
__global__ __launch_bounds__(kThreads) void stream_floor_kernel(const bf16_t *x, int rows, int cols, uint8_t *out, uint32_t *sf,
                                                                int tiles_k, unsigned long long *stamps) {
    unsigned long long t_start = 0, t_loaded = 0;
    if constexpr (STAMP) t_start = wall_clock64();
    const int lane = threadIdx.x & 63, wave = wave_id();
    const int tile_m = tile_grid_row(tiles_k == 1), tile_k = tile_grid_col(tiles_k == 1);
    const int row = tile_m * kWaves + wave;
    if (row >= rows) return;
    const int col = tile_k * PIECES * kStripCols + lane * 8;
    // addresses as the operators form them: a wave-uniform base plus a 32-bit byte offset per lane
    const uint32_t ucols = (uint32_t)cols;
    const uint8_t *xrow = reinterpret_cast<const uint8_t *>(x) + (uint64_t)(uint32_t)row * ((TWO ? 4u : 2u) * ucols);
    const uint32_t lane_off = (uint32_t)(tile_k * PIECES) * (uint32_t)(kStripCols * 2) + (uint32_t)lane * 16u;
    const uint8_t *xup = xrow + ucols * 2u;      // the second half of the row
    asm volatile("" : "+s"(xup));                // (kept in scalar registers)
    u32x4 a[PIECES], b[PIECES];
#pragma unroll
    for (int r = 0; r < PIECES; ++r) {
        a[r] = ld_stream16(xrow + lane_off + r * (kStripCols * 2));
        vmem_issue_gap();
        b[r] = TWO ? ld_stream16(xup + lane_off + r * (kStripCols * 2)) : u32x4{0u, 0u, 0u, 0u};
        if (TWO) vmem_issue_gap();
    }
    // every load is back before the first store goes out, as in the operators, whose stores follow all their arithmetic
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (STAMP) t_loaded = wall_clock64();
    uint32_t fold = 0;
#pragma unroll
    for (int r = 0; r < PIECES; ++r) {
        const u32x4 v = a[r] ^ b[r];
        st_stream8(out + (int64_t)row * cols + col + r * kStripCols, u32x2{v.x ^ v.z, v.y ^ v.w});
        fold ^= v.x;
    }
    // one word per 128-column group: 4 per piece, the wave's PIECES * 4 words are one contiguous run
    if (sf != nullptr && (lane & 15) < PIECES)
        st_stream4(sf + (int64_t)row * (cols / 128) + (tile_k * PIECES + (lane & 15)) * 4 + (lane >> 4), fold);
    if constexpr (STAMP) {
        const unsigned long long t_issued = wall_clock64();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        const unsigned long long t_acked = wall_clock64();
        if (lane == 0) {
            unsigned long long *q = stamps + ((int64_t)row * tiles_k + tile_k) * kStampWords;
            q[0] = t_start;
            q[1] = t_loaded;
            q[2] = t_issued;
            q[3] = t_acked;
            q[4] = __builtin_amdgcn_s_getreg(63492);     // hwreg(HW_ID): wave, SIMD, CU, shader array and engine
            q[5] = __builtin_amdgcn_s_getreg(63508);     // hwreg(XCC_ID)
        }
    }
}

// The traffic of a launch that ends in smaller waves, as tk_swiglu_per_token_cast arranges its launches of about one to
// three occupancy rounds: row tiles [0, yb) are four rows of four-piece waves, the next ym workgroups hold two rows of
// two-piece waves, the rest one row of one-piece waves.  Same loads, stores and scale words as stream_floor_kernel.
template <bool TWO>
__global__ __launch_bounds__(kThreads) void stream_floor_tailed_kernel(const bf16_t *x, int rows, int cols, uint8_t *out, uint32_t *sf,
                                                                       int tiles_k, int yb, int ym) {
    const int lane = threadIdx.x & 63, wave = wave_id();
    const int y = tile_grid_row(tiles_k == 1), strip0 = tile_grid_col(tiles_k == 1) * 4;
    int row, strip, np;
    if (y < yb) {
        row = y * kWaves + wave; strip = strip0; np = 4;
    } else if (y - yb < ym) {
        const int sub = (y - yb) * kWaves + wave;
        row = yb * kWaves + (sub >> 1); strip = strip0 + (sub & 1) * 2; np = 2;
    } else {
        const int sub = (y - yb - ym) * kWaves + wave;
        row = yb * kWaves + ym * 2 + (sub >> 2); strip = strip0 + (sub & 3); np = 1;
    }
    if (row >= rows) return;
    const int col = strip * kStripCols + lane * 8;
    // (addresses as in stream_floor_kernel)
    const uint32_t ucols = (uint32_t)cols;
    const uint8_t *xrow = reinterpret_cast<const uint8_t *>(x) + (uint64_t)(uint32_t)row * ((TWO ? 4u : 2u) * ucols);
    const uint8_t *xup = xrow + ucols * 2u;
    asm volatile("" : "+s"(xup));
    const uint32_t lane_off = (uint32_t)strip * (uint32_t)(kStripCols * 2) + (uint32_t)lane * 16u;
    u32x4 a[4], b[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (r < np) {      // wave-uniform
            a[r] = ld_stream16(xrow + lane_off + r * (kStripCols * 2));
            vmem_issue_gap();
            b[r] = TWO ? ld_stream16(xup + lane_off + r * (kStripCols * 2)) : u32x4{0u, 0u, 0u, 0u};
            if (TWO) vmem_issue_gap();
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // (as in stream_floor_kernel)
    uint32_t fold = 0;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (r < np) {
            const u32x4 v = a[r] ^ b[r];
            st_stream8(out + (int64_t)row * cols + col + r * kStripCols, u32x2{v.x ^ v.z, v.y ^ v.w});
            fold ^= v.x;
        }
    }
    if (sf != nullptr && (lane & 15) < np) st_stream4(sf + (int64_t)row * (cols / 128) + (strip + (lane & 15)) * 4 + (lane >> 4), fold);
}

// The same idea for any ratio of bytes read to bytes written: a lane reads IN (16, 8 or 4) bytes per piece and writes OUT
// (16, 8, 4 or 0) bytes per piece, a piece being 64 lanes side by side; a wave takes PIECES consecutive pieces, all loads
// issued before the first store.  Input and output are flat byte ranges.
template <int IN> __device__ __forceinline__ u32x4 floor_load(const uint8_t *p) {
    if constexpr (IN == 16) return ld_stream16(p);
    else if constexpr (IN == 8) { const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(p)); return u32x4{v.x, v.y, 0u, 0u}; }
    else { const uint32_t v = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(p)); return u32x4{v, 0u, 0u, 0u}; }
}
template <int OUT> __device__ __forceinline__ void floor_store(uint8_t *p, u32x4 v) {
    if constexpr (OUT == 16) st_stream16(p, v);
    else if constexpr (OUT == 8) st_stream8(p, u32x2{v.x ^ v.z, v.y ^ v.w});
    else if constexpr (OUT == 4) st_stream4(p, v.x ^ v.y ^ v.z ^ v.w);
}

template <int IN, int OUT, int PIECES>
__global__ __launch_bounds__(kThreads) void stream_floor_flat_kernel(const uint8_t *in, int64_t pieces, uint8_t *out, uint32_t *sink) {
    const int lane = threadIdx.x & 63;
    const int64_t first = ((int64_t)blockIdx.x * kWaves + wave_id()) * PIECES;
    if (first >= pieces) return;
    u32x4 v[PIECES];
#pragma unroll
    for (int r = 0; r < PIECES; ++r) {
        const int64_t piece = first + r < pieces ? first + r : first;       // (a wave's surplus pieces read its first again)
        v[r] = floor_load<IN>(in + (piece * 64 + lane) * IN);
        vmem_issue_gap();
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // (as in stream_floor_kernel)
    uint32_t fold = 0;
#pragma unroll
    for (int r = 0; r < PIECES; ++r) {
        if (OUT != 0 && first + r < pieces) floor_store<OUT>(out + ((first + r) * 64 + lane) * OUT, v[r]);
        fold ^= v[r].x ^ v[r].y ^ v[r].z ^ v[r].w;
    }
    // nothing written: the loads must still be used.  No fold of real data is ever this value in all lanes at once
    if (OUT == 0 && fold == 0x9E3779B9u && sink != nullptr) st_stream4(sink, fold);
}

}  // namespace tk

using namespace tk;

extern "C" int tk_stream_floor_flat(const void *in, int64_t in_bytes, int in_bytes_per_lane, void *out, int out_bytes_per_lane,
                                    int pieces_per_wave, void *stream) {
    const int I = in_bytes_per_lane, O = out_bytes_per_lane, P = pieces_per_wave;
    if ((I != 16 && I != 8 && I != 4) || (O != 16 && O != 8 && O != 4 && O != 0) || (P != 1 && P != 2 && P != 4 && P != 8)) return TK_ERR_BAD_MODE;
    if (in_bytes < 0 || in_bytes % (64 * I) != 0) return TK_ERR_BAD_SHAPE;
    if (in_bytes == 0) return TK_OK;
    if (!in || (O != 0 && !out)) return TK_ERR_NULL_POINTER;
    if (!aligned_to(in, 16) || !aligned_to(out, 16)) return TK_ERR_MISALIGNED;
    const int64_t pieces = in_bytes / (64 * I), waves = (pieces + P - 1) / P, blocks = (waves + kWaves - 1) / kWaves;
    if (blocks > INT32_MAX) return TK_ERR_TOO_LARGE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint8_t *ip = static_cast<const uint8_t *>(in);
    uint8_t *op = static_cast<uint8_t *>(out);
#define TK_FLAT_3(II, OO, PP) \
    hipLaunchKernelGGL((stream_floor_flat_kernel<II, OO, PP>), dim3((unsigned)blocks), dim3(kThreads), 0, s, ip, pieces, op, (uint32_t *)nullptr)
#define TK_FLAT_2(II, OO)                 \
    do {                                  \
        if (P == 1) TK_FLAT_3(II, OO, 1); \
        else if (P == 2) TK_FLAT_3(II, OO, 2); \
        else if (P == 4) TK_FLAT_3(II, OO, 4); \
        else TK_FLAT_3(II, OO, 8);        \
    } while (0)
#define TK_FLAT_1(II)                     \
    do {                                  \
        if (O == 16) TK_FLAT_2(II, 16);   \
        else if (O == 8) TK_FLAT_2(II, 8); \
        else if (O == 4) TK_FLAT_2(II, 4); \
        else TK_FLAT_2(II, 0);            \
    } while (0)
    if (I == 16) TK_FLAT_1(16);
    else if (I == 8) TK_FLAT_1(8);
    else TK_FLAT_1(4);
#undef TK_FLAT_1
#undef TK_FLAT_2
#undef TK_FLAT_3
    return (int)hipGetLastError();
}

static int stream_floor_launch(const void *x, int64_t rows, int64_t cols, int two_halves, void *out, void *sf, void *stamps,
                               bool stamp, void *stream) {
    if (rows < 0 || cols <= 0 || cols % 1024 != 0) return TK_ERR_BAD_SHAPE;
    if (rows > INT32_MAX - 64 || cols > (INT32_MAX - 1024) / 4) return TK_ERR_TOO_LARGE;      // (a row's bytes are counted in 32 bits)
    if (rows == 0) return TK_OK;
    if (!x || !out || (stamp && !stamps)) return TK_ERR_NULL_POINTER;
    if (!aligned_to(x, 16) || !aligned_to(out, 8) || !aligned_to(sf, 4) || !aligned_to(stamps, 8)) return TK_ERR_MISALIGNED;
    const int pieces = cols % 2048 == 0 ? 4 : 2;
    const int tiles_k = (int)(cols / (pieces * kStripCols)), tiles_m = (int)((rows + kWaves - 1) / kWaves);
    const dim3 grid = tile_grid(tiles_k, tiles_m);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bf16_t *xp = static_cast<const bf16_t *>(x);
    uint8_t *op = static_cast<uint8_t *>(out);
    uint32_t *sp = static_cast<uint32_t *>(sf);
    unsigned long long *tp = static_cast<unsigned long long *>(stamps);
#define TK_FLOOR_LAUNCH(P, T, S) \
    hipLaunchKernelGGL((stream_floor_kernel<P, T, S>), grid, dim3(kThreads), 0, s, xp, (int)rows, (int)cols, op, sp, tiles_k, tp)
#define TK_FLOOR_LAUNCH_2(P, T)          \
    do {                                 \
        if (stamp) TK_FLOOR_LAUNCH(P, T, true); \
        else TK_FLOOR_LAUNCH(P, T, false);      \
    } while (0)
    if (pieces == 4) {
        if (two_halves) TK_FLOOR_LAUNCH_2(4, true);
        else TK_FLOOR_LAUNCH_2(4, false);
    } else {
        if (two_halves) TK_FLOOR_LAUNCH_2(2, true);
        else TK_FLOOR_LAUNCH_2(2, false);
    }
#undef TK_FLOOR_LAUNCH_2
#undef TK_FLOOR_LAUNCH
    return (int)hipGetLastError();
}

extern "C" int tk_stream_floor(const void *x, int64_t rows, int64_t cols, int two_halves, void *out, void *sf, void *stream) {
    return stream_floor_launch(x, rows, cols, two_halves, out, sf, nullptr, false, stream);
}

extern "C" int tk_stream_floor_tailed(const void *x, int64_t rows, int64_t cols, int two_halves, void *out, void *sf, int64_t rows_two,
                                      int64_t rows_one, void *stream) {
    if (rows < 0 || cols <= 0 || cols % 2048 != 0 || rows % 4 != 0 || rows_two < 0 || rows_one < 0 || rows_two % 4 != 0 || rows_one % 4 != 0 ||
        rows_two + rows_one > rows)
        return TK_ERR_BAD_SHAPE;
    if (rows > INT32_MAX / 8 || cols > (INT32_MAX - 1024) / 4) return TK_ERR_TOO_LARGE;
    if (rows == 0) return TK_OK;
    if (!x || !out) return TK_ERR_NULL_POINTER;
    if (!aligned_to(x, 16) || !aligned_to(out, 8) || !aligned_to(sf, 4)) return TK_ERR_MISALIGNED;
    const int tiles_k = (int)(cols / (4 * kStripCols));
    const int yb = (int)((rows - rows_two - rows_one) / kWaves), ym = (int)(rows_two * 2 / kWaves), ys = (int)(rows_one * 4 / kWaves);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid = tile_grid(tiles_k, yb + ym + ys);
    if (two_halves)
        hipLaunchKernelGGL(stream_floor_tailed_kernel<true>, grid, dim3(kThreads), 0, s, static_cast<const bf16_t *>(x), (int)rows, (int)cols,
                           static_cast<uint8_t *>(out), static_cast<uint32_t *>(sf), tiles_k, yb, ym);
    else
        hipLaunchKernelGGL(stream_floor_tailed_kernel<false>, grid, dim3(kThreads), 0, s, static_cast<const bf16_t *>(x), (int)rows, (int)cols,
                           static_cast<uint8_t *>(out), static_cast<uint32_t *>(sf), tiles_k, yb, ym);
    return (int)hipGetLastError();
}

extern "C" int64_t tk_stream_floor_stamp_words(int64_t rows, int64_t cols) {
    if (rows < 0 || cols <= 0 || cols % 1024 != 0) return 0;
    const int pieces = cols % 2048 == 0 ? 4 : 2;
    return rows * (cols / (pieces * kStripCols)) * kStampWords;
}

extern "C" int tk_stream_floor_timeline(const void *x, int64_t rows, int64_t cols, int two_halves, void *out, void *sf,
                                        void *stamps, void *stream) {
    return stream_floor_launch(x, rows, cols, two_halves, out, sf, stamps, true, stream);
}
