// Expert-major ("fused") MoE layout for gfx950: the mapping between the (token, k) routing list and
// the expanded row order, and the row expansion that feeds the fused SwiGLU op.  Integer / byte
// work, HBM- and latency-bound; no LDS tiling beyond per-wave histograms.
//
// Reference semantics: tile_kernels/moe/get_fused_mapping_kernel.py:24-250,
// tile_kernels/moe/expand_to_fused_kernel.py:16-200, tile_kernels/torch/expand_to_fused.py,
// tile_kernels/moe/reduce_fused_kernel.py:12-135, tile_kernels/torch/reduce_fused.py.
#include <atomic>

#include "tk_device.hpp"
#include "tk_host.hpp"

namespace tk {

// ------------------------------------------------------------------------------------------------
// get_fused_mapping: a stable counting sort of the flat (token, k) list by expert, every expert's
// segment padded to a multiple of `alignment`.  Lists of more than 64 Ki pairs take three launches, no grid-wide
// barrier (a single workgroup doing all of it was measured at 70 us for 32 Ki pairs against 18 us for the three
// launches: one CU cannot absorb the scattered 4-byte stores of the hand-out); shorter lists take the single
// launch of several workgroups further down:
//   count  : each wave histograms its own 256-element slice            -> ws[slice][expert]
//   scan   : one workgroup turns the histograms into exclusive offsets  -> ws[slice][expert], expert_start/end
//   assign : each wave walks its slice again in order and hands out positions
// Positions inside an expert follow the flat index (the reference leaves that order open).
constexpr int kSliceElems = 256;   // elements per wave
constexpr int kMaxExperts = 1024;  // bound on the per-wave LDS histogram

__global__ __launch_bounds__(kThreads) void fused_mapping_count_kernel(const int64_t *topk_idx, int numel, int num_experts,
                                                                       int32_t *ws, int32_t *pos_to_expert, int32_t *pos_to_token,
                                                                       int32_t *pos_to_token_topk, int num_expanded) {
    extern __shared__ int32_t hist[];   // [kWaves][num_experts]
    const int lane = threadIdx.x & 63, wave = wave_id();
    const int slice = blockIdx.x * kWaves + wave;
    int32_t *h = hist + wave * num_experts;
    for (int e = lane; e < num_experts; e += 64) h[e] = 0;
    // padding positions keep -1; the assign launch overwrites the live ones
    for (int i = blockIdx.x * kThreads + threadIdx.x; i < num_expanded; i += gridDim.x * kThreads) {
        pos_to_expert[i] = -1;
        pos_to_token[i] = -1;
        pos_to_token_topk[i] = -1;
    }
    __syncthreads();
    const int base = slice * kSliceElems;
    for (int j = lane; j < kSliceElems; j += 64) {
        const int i = base + j;
        if (i < numel) {
            const int64_t e = topk_idx[i];
            if (e >= 0 && e < num_experts) atomicAdd(&h[(int)e], 1);
        }
    }
    __syncthreads();
    if (base < numel)
        for (int e = lane; e < num_experts; e += 64) ws[(int64_t)slice * num_experts + e] = h[e];
}

// Mask of the lanes that hold the same expert id as this lane (ids < 0 match nothing): the ballots
// of every bit of the id, intersected.
__device__ __forceinline__ unsigned long long same_expert_lanes(int e, int expert_bits) {
    unsigned long long peers = __ballot(e >= 0);
    for (int b = 0; b < expert_bits; ++b) {
        const bool bit = (e >> b) & 1;
        const unsigned long long m = __ballot(bit);
        peers &= bit ? m : ~m;
    }
    return peers;
}

// One wave hands out positions to the elements [base, base + 64 * STEPS) of the flat (token, k) list, in order, 64 at
// a time; nx[e] is the next free position of expert e for this wave.  The ids of the whole slice are loaded before the
// first is used: one memory round trip per slice instead of one per 64 elements.
template <int STEPS>
__device__ __forceinline__ void assign_range(const int64_t *topk_idx, int base, int numel, int num_topk, int num_experts,
                                             int expert_bits, int32_t *nx, int32_t *pos_to_expert, int32_t *pos_to_token,
                                             int32_t *pos_to_token_topk, int32_t *token_topk_to_pos, int num_expanded) {
    // pos_to_expert == nullptr: the caller fills that array itself (it is a function of the expert offsets alone)
    const int lane = threadIdx.x & 63;
    const unsigned long long below = (1ull << lane) - 1ull;
    int64_t ids[STEPS];
#pragma unroll
    for (int j = 0; j < STEPS; ++j) {
        const int i = base + j * 64 + lane;
        ids[j] = topk_idx[i < numel ? i : base];
    }
#pragma unroll
    for (int j = 0; j < STEPS; ++j) {
        const int i = base + j * 64 + lane;
        if (base + j * 64 >= numel) break;             // wave-uniform
        const int64_t v = ids[j];
        const int e = (i < numel && v >= 0 && v < num_experts) ? (int)v : -1;
        const unsigned long long peers = same_expert_lanes(e, expert_bits);
        int pos = -1;
        if (e >= 0) {
            const int first = nx[e];
            pos = first + __popcll(peers & below);
            __builtin_amdgcn_wave_barrier();          // every peer has read before the last one advances the counter
            if ((peers >> lane) == 1ull) nx[e] = first + __popcll(peers);
        }
        __builtin_amdgcn_wave_barrier();
        if (i < numel) token_topk_to_pos[i] = pos;
        if (pos >= 0 && pos < num_expanded) {
            if (pos_to_expert) pos_to_expert[pos] = e;
            pos_to_token[pos] = i / num_topk;
            pos_to_token_topk[pos] = i;
        }
    }
}

// Inclusive prefix sum over the experts with all 1024 threads of a workgroup (Hillis-Steele on two
// ping-pong buffers); returns the index of the buffer that holds the result.
__device__ __forceinline__ int scan_experts(int32_t (*scan)[kMaxExperts], const int32_t *padded, int num_experts) {
    const int t = threadIdx.x;
    scan[0][t] = t < num_experts ? padded[t] : 0;
    __syncthreads();
    int cur = 0;
    for (int d = 1; d < kMaxExperts; d <<= 1) {
        scan[cur ^ 1][t] = scan[cur][t] + (t >= d ? scan[cur][t - d] : 0);
        cur ^= 1;
        __syncthreads();
    }
    return cur;
}

// One workgroup of 1024 threads.  The slice axis is cut into C = 1024 / num_experts chunks (at least
// one) and thread (c, e) owns chunk c of expert e: it sums its chunk (independent loads, so their
// latencies overlap), the chunk totals are exchanged through LDS, and a second walk over the chunk
// (from L2) writes the exclusive offsets.  Expert starts come from a block-wide prefix sum.
__global__ __launch_bounds__(1024) void fused_mapping_scan_kernel(int32_t *ws, int num_slices, int num_experts, int alignment,
                                                                  int32_t *expert_start, int32_t *expert_end,
                                                                  int32_t *num_tokens_per_expert) {
    __shared__ int32_t total[1024];          // [chunk][expert], chunks * num_experts <= 1024
    __shared__ int32_t padded[kMaxExperts];
    __shared__ int32_t scan[2][kMaxExperts];
    const int chunks = num_experts >= 1024 ? 1 : 1024 / num_experts;
    const int per = (num_slices + chunks - 1) / chunks;
    const int c = threadIdx.x / num_experts, e = threadIdx.x - c * num_experts;
    const bool active = c < chunks;
    const int s0 = c * per, s1 = min(s0 + per, num_slices);

    if (active) {
        int32_t sum = 0;
#pragma unroll 8
        for (int s = s0; s < s1; ++s) sum += ws[(int64_t)s * num_experts + e];
        total[c * num_experts + e] = sum;
    }
    __syncthreads();
    int32_t run = 0;
    if (active) {
        for (int k = 0; k < c; ++k) run += total[k * num_experts + e];
        if (c == 0) {
            int32_t all = 0;
            for (int k = 0; k < chunks; ++k) all += total[k * num_experts + e];
            padded[e] = (all + alignment - 1) / alignment * alignment;
        }
#pragma unroll 8
        for (int s = s0; s < s1; ++s) {
            const int64_t at = (int64_t)s * num_experts + e;
            const int32_t n = ws[at];
            ws[at] = run;          // exclusive offset of this slice inside the expert
            run += n;
        }
    }
    __syncthreads();
    const int cur = scan_experts(scan, padded, num_experts);
    const int t = threadIdx.x;
    if (t < num_experts) {
        const int32_t end = scan[cur][t];
        expert_start[t] = end - padded[t];
        expert_end[t] = end;
        num_tokens_per_expert[t] = padded[t];
    }
}

// The whole mapping in one launch, for lists of up to kSingleLaunchPairs (token, k) pairs: no launch has to wait for
// another, and no table in global memory is needed.  A workgroup of 16 waves owns 16 consecutive slices of 64, and instead
// of being told how many entries of every expert precede them it counts them itself: every workgroup reads the whole
// list once (a few hundred KB that stay in the L2) into LDS histograms: all entries, the entries before its own
// range, and one per slice of its own.  From these every workgroup derives the same expert offsets (a prefix sum over
// the padded expert sizes) and its slices' first positions, hands out positions exactly as the assign launch does, and
// marks its share of the padding positions: the ends of the experts e = workgroup, workgroup + gridDim, ... and its
// stride of the unused tail of the buffers.  Measured on MI355X for 4096 tokens, top-8 of 256 experts: 9.1 us, of which
// the counting pass is 4.2 (its LDS atomics), against 17.8 us for the three launches.
constexpr int kSingleLaunchPairs = 64 * 1024 - 1;
constexpr int kSingleWaves = 16;
constexpr int kSingleSlice = 64;            // entries a wave hands out: 1024 per workgroup, so that the scattered stores of the
                                            // hand-out spread over many CUs (256 per wave, 8 workgroups for 32 Ki pairs: 13.6 us)
constexpr int kSingleMaxExperts = 512;      // (1 + kSingleWaves) histograms of 4-byte counters must fit the LDS of a workgroup

__global__ __launch_bounds__(64 * kSingleWaves) void fused_mapping_single_kernel(const int64_t *topk_idx, int numel, int num_topk,
                                                                                int num_experts, int expert_bits, int alignment,
                                                                                int32_t *pos_to_expert, int32_t *pos_to_token,
                                                                                int32_t *pos_to_token_topk, int32_t *token_topk_to_pos,
                                                                                int32_t *expert_start, int32_t *expert_end,
                                                                                int32_t *num_tokens_per_expert, int num_expanded) {
    // counts[e]: entries of expert e in the whole list (low half) and before this workgroup's range (high half): one
    // LDS atomic per entry for both, which is what this pass spends its time on (a list of fewer than 64 Ki pairs
    // cannot overflow a half); slice[w][e]: entries of expert e in slice w of the workgroup's own range
    extern __shared__ int32_t hist[];        // counts[E], slice[kSingleWaves][E]
    __shared__ int32_t padded[kSingleMaxExperts];
    __shared__ int32_t ends[kSingleMaxExperts];
    __shared__ int32_t wave_total[kSingleMaxExperts / 64];
    uint32_t *counts = reinterpret_cast<uint32_t *>(hist);
    int32_t *slice = hist + num_experts;
    const int tid = threadIdx.x, lane = tid & 63, wave = wave_id();
    const int nthreads = 64 * kSingleWaves;
    const int own_base = blockIdx.x * (kSingleWaves * kSingleSlice), own_end = own_base + kSingleWaves * kSingleSlice;

    for (int i = tid; i < (1 + kSingleWaves) * num_experts; i += nthreads) hist[i] = 0;
    __syncthreads();
    auto count = [&](int i, int64_t v) {
        if (v >= 0 && v < num_experts) {
            const int e = (int)v;
            atomicAdd(&counts[e], i < own_base ? 0x10001u : 1u);
            if (i >= own_base && i < own_end) atomicAdd(&slice[((i - own_base) / kSingleSlice) * num_experts + e], 1);
        }
    };
    // The list is read in 16-byte pieces (two ids), 16 of them per thread in flight at a time: with a load or four at a
    // time the pass took as many memory round trips as it has iterations (24 us for 32 Ki pairs).
    const int head = (int)((reinterpret_cast<uintptr_t>(topk_idx) >> 3) & 1);      // ids before the first 16-byte boundary
    const int pairs = (numel - head) / 2;
    const u32x4 *wide = reinterpret_cast<const u32x4 *>(topk_idx + head);
    constexpr int U = 16;
    for (int p0 = 0; p0 < pairs; p0 += U * nthreads) {
        u32x4 w[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int pi = p0 + j * nthreads + tid;
            w[j] = wide[pi < pairs ? pi : 0];
            vmem_issue_gap();
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int pi = p0 + j * nthreads + tid;
            if (pi < pairs) {
                count(head + 2 * pi, (int64_t)(((uint64_t)w[j].y << 32) | w[j].x));
                count(head + 2 * pi + 1, (int64_t)(((uint64_t)w[j].w << 32) | w[j].z));
            }
        }
    }
    if (tid == 0 && head) count(0, topk_idx[0]);
    if (tid == 1 && head + 2 * pairs < numel) count(numel - 1, topk_idx[numel - 1]);
    __syncthreads();
    // prefix sum over the padded expert sizes: inside each wave by shuffles, across the (at most 8) waves through LDS
    int32_t mine = 0, incl = 0;
    if (tid < kSingleMaxExperts) {
        mine = tid < num_experts ? (int32_t)(((counts[tid] & 0xFFFFu) + alignment - 1) / alignment * alignment) : 0;
        incl = mine;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int32_t up = __shfl_up(incl, d, 64);
            if (lane >= d) incl += up;
        }
        if (lane == 63) wave_total[wave] = incl;
    }
    __syncthreads();
    if (tid < num_experts) {
        int32_t offset = 0;
        for (int w = 0; w < wave; ++w) offset += wave_total[w];
        const int32_t end = offset + incl, start = end - mine;
        padded[tid] = mine;
        ends[tid] = end;
        if (blockIdx.x == 0) {
            expert_start[tid] = start;
            expert_end[tid] = end;
            num_tokens_per_expert[tid] = mine;
        }
        // first position of every slice of this workgroup inside the expert
        int32_t run = start + (int32_t)(counts[tid] >> 16);
        for (int w = 0; w < kSingleWaves; ++w) {
            const int32_t n = slice[w * num_experts + tid];
            slice[w * num_experts + tid] = run;
            run += n;
        }
    }
    __syncthreads();
    const int total = ends[num_experts - 1];
    const int base = own_base + wave * kSingleSlice;
    if (base < numel)
        assign_range<kSingleSlice / 64>(topk_idx, base, numel, num_topk, num_experts, expert_bits, slice + wave * num_experts, nullptr,
                                        pos_to_token, pos_to_token_topk, token_topk_to_pos, num_expanded);
    // The experts this workgroup looks after, a wave per expert: pos_to_expert of the whole segment (it follows from the
    // offsets, and written here it leaves as whole lines instead of one scattered word per entry: the hand-out above
    // is bound by the rate at which one CU issues scattered stores) and the padding marks at the segment's end.
    for (int e = (int)blockIdx.x + wave * (int)gridDim.x; e < num_experts; e += kSingleWaves * (int)gridDim.x) {
        const int end = ends[e], start = end - padded[e], first = start + (int)(counts[e] & 0xFFFFu);
        for (int i = start + lane; i < end && i < num_expanded; i += 64) pos_to_expert[i] = i < first ? e : -1;
        for (int i = first + lane; i < end && i < num_expanded; i += 64) {
            pos_to_token[i] = -1;
            pos_to_token_topk[i] = -1;
        }
    }
    // positions beyond the last expert
    for (int i = total + (int)blockIdx.x * nthreads + tid; i < num_expanded; i += (int)gridDim.x * nthreads) {
        pos_to_expert[i] = -1;
        pos_to_token[i] = -1;
        pos_to_token_topk[i] = -1;
    }
}

__global__ __launch_bounds__(kThreads) void fused_mapping_assign_kernel(const int64_t *topk_idx, int numel, int num_topk,
                                                                        int num_experts, int expert_bits, const int32_t *ws,
                                                                        const int32_t *expert_start, int32_t *pos_to_expert,
                                                                        int32_t *pos_to_token, int32_t *pos_to_token_topk,
                                                                        int32_t *token_topk_to_pos, int num_expanded) {
    extern __shared__ int32_t next[];   // [kWaves][num_experts]: next free position per expert, per wave
    const int lane = threadIdx.x & 63, wave = wave_id();
    const int slice = blockIdx.x * kWaves + wave;
    const int base = slice * kSliceElems;
    if (base >= numel) return;          // whole wave; no barrier below
    int32_t *nx = next + wave * num_experts;
    for (int e = lane; e < num_experts; e += 64) nx[e] = expert_start[e] + ws[(int64_t)slice * num_experts + e];
    __builtin_amdgcn_wave_barrier();
    assign_range<kSliceElems / 64>(topk_idx, base, numel, num_topk, num_experts, expert_bits, nx, pos_to_expert, pos_to_token,
                                   pos_to_token_topk, token_topk_to_pos, num_expanded);
}

// ------------------------------------------------------------------------------------------------
// expand_to_fused.  Rows are moved as raw 16-byte pieces, so any element type works; optional 4-byte
// scale rows travel the same way into a row-major or column-major scale tensor.
//
// One load and one store per thread.  What bounds this operator is the write stream (8 bytes written
// per byte read at top-8), and on MI355X that stream runs the faster the fewer stores a thread issues:
// filling 268 MB takes 40.6 us with one 16-byte store per thread, 44 us with 2 or 4, 47 us with 8 and
// 53 us with 16.  A workgroup therefore copies one 4 KB chunk of one token's row to ONE of its
// positions, and the row is read once per position instead of once: the re-reads hit the L2, because
// workgroups are dealt to the 8 XCDs (one L2 each) round-robin and the workgroups of a chunk are
// numbered 8 apart, which puts all of them on one XCD back to back.  (Measured for [4096, 4096] bf16,
// top-8, random positions, 268 MB written: 50.6 us this way, 57 us with the copies of a chunk on
// different XCDs, 61 us with one load and 8 stores per thread.)
// The workgroups after those each look at a few consecutive expanded rows (8 KB worth) and zero the ones
// that are padding.
constexpr int kExpandChunk = kThreads * 16;

// Non-temporal 16-byte stores: writing the same 268 MB as whole 8 KB rows per wave takes 52 us with them and
// 62 us with plain stores; pairs of 8-byte system-scope stores are several times slower still.
__device__ __forceinline__ void expand_store16(void *p, u32x4 v) { __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p)); }

// Padding workgroup `pb` of the short-rows kernel: zero the rows among its pad_rows consecutive expanded rows that no
// token maps to (the same loop as in the kernel for long rows, which keeps its own copy: sharing this function cost
// that kernel 2 % with scale rows).
__device__ __forceinline__ void expand_zero_padding(int pb, int pad_rows, int num_expanded, int64_t row_bytes, uint8_t *out,
                                                    const int32_t *pos_to_expert, bool with_sf, int sf_cols, uint32_t *out_sf,
                                                    int64_t out_sf_ld, int sf_col_major) {
    const int r0 = pb * pad_rows;
    for (int r = r0; r < r0 + pad_rows && r < num_expanded; ++r) {
        if (uniform_load(pos_to_expert + r) >= 0) continue;
        uint8_t *dst = out + (int64_t)r * row_bytes;
        for (int64_t off = (int64_t)threadIdx.x * 16; off < row_bytes; off += kExpandChunk) expand_store16(dst + off, u32x4{0u, 0u, 0u, 0u});
        if (with_sf)
            for (int j = threadIdx.x; j < sf_cols; j += kThreads) out_sf[sf_col_major ? (int64_t)j * out_sf_ld + r : (int64_t)r * out_sf_ld + j] = 0u;
    }
}

__global__ __launch_bounds__(kThreads) void expand_to_fused_kernel(const uint8_t *x, int64_t row_bytes, const int32_t *token_topk_to_pos,
                                                                   int num_topk, int chunks, int copy_blocks, int num_tokens,
                                                                   int num_expanded, uint8_t *out, const int32_t *pos_to_expert,
                                                                   const uint32_t *x_sf, int sf_cols, uint32_t *out_sf,
                                                                   int64_t out_sf_ld, int sf_col_major, int pad_rows) {
    const int b = blockIdx.x;
    if (b < copy_blocks) {
        // b = 8 * ((token group * chunks + chunk) * num_topk + k) + token within its group of 8
        const int q = b >> 3;
        const int k = q % num_topk, q2 = q / num_topk;
        const int c = q2 % chunks, t = (q2 / chunks) * 8 + (b & 7);
        if (t >= num_tokens) return;
        const int p = uniform_load(token_topk_to_pos + (int64_t)t * num_topk + k);
        const int64_t off = (int64_t)c * kExpandChunk + threadIdx.x * 16;
        u32x4 v = u32x4{0u, 0u, 0u, 0u};
        if (off < row_bytes) v = *reinterpret_cast<const u32x4 *>(x + (int64_t)t * row_bytes + off);   // cached: read num_topk times
        if (p < 0 || p >= num_expanded) return;
        if (off < row_bytes) expand_store16(out + (int64_t)p * row_bytes + off, v);
        if (x_sf && c == 0)
            for (int j = threadIdx.x; j < sf_cols; j += kThreads)
                out_sf[sf_col_major ? (int64_t)j * out_sf_ld + p : (int64_t)p * out_sf_ld + j] = x_sf[(int64_t)t * sf_cols + j];
    } else {
        const int r0 = (b - copy_blocks) * pad_rows;
        for (int r = r0; r < r0 + pad_rows && r < num_expanded; ++r) {
            if (uniform_load(pos_to_expert + r) >= 0) continue;
            uint8_t *dst = out + (int64_t)r * row_bytes;
            for (int64_t off = (int64_t)threadIdx.x * 16; off < row_bytes; off += kExpandChunk) expand_store16(dst + off, u32x4{0u, 0u, 0u, 0u});
            if (x_sf)
                for (int j = threadIdx.x; j < sf_cols; j += kThreads) out_sf[sf_col_major ? (int64_t)j * out_sf_ld + r : (int64_t)r * out_sf_ld + j] = 0u;
        }
    }
}

// Rows of at most 2 KB (a kernel of its own: as a branch of the one above it cost that one 5 %).  The workgroup's
// threads form kpw groups of tpr threads (tpr * 16 >= row_bytes), and group g copies the row to position kg * kpw + g
// of the token, still one load and one store per thread.  (With one position per workgroup half or more of the
// threads had nothing to copy: bf16 [32768, 1024], top-8: 198.7 us, 124.6 us this way.)
__global__ __launch_bounds__(kThreads) void expand_short_rows_kernel(const uint8_t *x, int64_t row_bytes, const int32_t *token_topk_to_pos,
                                                                     int num_topk, int kpw, int tpr, int copy_blocks, int num_tokens,
                                                                     int num_expanded, uint8_t *out, const int32_t *pos_to_expert,
                                                                     const uint32_t *x_sf, int sf_cols, uint32_t *out_sf,
                                                                     int64_t out_sf_ld, int sf_col_major, int pad_rows) {
    const int b = blockIdx.x;
    if (b < copy_blocks) {
        // b = 8 * ((token group * groups of positions) + kg) + token within its group of 8
        const int kgroups = (num_topk + kpw - 1) / kpw;
        const int q = b >> 3;
        const int kg = q % kgroups, t = (q / kgroups) * 8 + (b & 7);
        const int g = (int)threadIdx.x / tpr, i = (int)threadIdx.x - g * tpr;
        const int k = kg * kpw + g;
        const int64_t off = (int64_t)i * 16;
        if (t >= num_tokens || g >= kpw || k >= num_topk) return;
        const int p = token_topk_to_pos[(int64_t)t * num_topk + k];
        u32x4 v = u32x4{0u, 0u, 0u, 0u};
        if (off < row_bytes) v = *reinterpret_cast<const u32x4 *>(x + (int64_t)t * row_bytes + off);   // cached: read num_topk times
        if (p < 0 || p >= num_expanded) return;
        if (off < row_bytes) expand_store16(out + (int64_t)p * row_bytes + off, v);
        if (x_sf)
            for (int j = i; j < sf_cols; j += tpr)
                out_sf[sf_col_major ? (int64_t)j * out_sf_ld + p : (int64_t)p * out_sf_ld + j] = x_sf[(int64_t)t * sf_cols + j];
    } else {
        expand_zero_padding(b - copy_blocks, pad_rows, num_expanded, row_bytes, out, pos_to_expert, x_sf != nullptr, sf_cols, out_sf, out_sf_ld,
                            sf_col_major);
    }
}

// ------------------------------------------------------------------------------------------------
// reduce_fused: the inverse of the expansion.  out[t] = sum over k of x[pos(t, k)] * s(t, k), accumulated in fp32 with
// one fused multiply-add per term, in the order k = 0, 1, ... (so that results are reproducible bit for bit), where
// s = topk_weights[t, k] (or 1) times x_sf[pos] (if given); positions < 0 are skipped.  The sum is scaled by *sf (if
// given) and rounded to the output type.  A thread owns 8 consecutive elements of one token: up to 8 rows' pieces are
// loaded before the first is used, and there is one store per thread.
constexpr int kReduceUnroll = 8;

// fp32 rows whose length is a multiple of 512: a thread's 8 elements are two runs of 4, 256 columns apart, so that each
// of its 16-byte loads (and of its fp32 stores) is, over the wave, 1024 consecutive bytes.  With the 8 elements in one
// run, every instruction touches half of each cache line it names (fp32 [81792, 4096] -> fp32, top-8: 220.2 us that way).
struct SplitF32 {};
struct Raw8SplitF32 {
    u32x4 a, b;
    __device__ __forceinline__ void load(const float *p) { a = ld_stream16(p); vmem_issue_gap(); b = ld_stream16(p + 256); }
    __device__ __forceinline__ void get(float (&v)[8]) const {
        v[0] = u2f(a.x); v[1] = u2f(a.y); v[2] = u2f(a.z); v[3] = u2f(a.w);
        v[4] = u2f(b.x); v[5] = u2f(b.y); v[6] = u2f(b.z); v[7] = u2f(b.w);
    }
};
template <typename InT> struct ReduceIn;
template <> struct ReduceIn<bf16_t> { typedef Raw8<bf16_t> raw; typedef bf16_t elem; static constexpr bool split = false; };
template <> struct ReduceIn<float> { typedef Raw8<float> raw; typedef float elem; static constexpr bool split = false; };
template <> struct ReduceIn<SplitF32> { typedef Raw8SplitF32 raw; typedef float elem; static constexpr bool split = true; };

// U terms k0 .. k0 + U - 1 of one token: all U rows' pieces are loaded before the first is used
template <typename InT, int U>
__device__ __forceinline__ void reduce_terms(float (&acc)[8], const typename ReduceIn<InT>::elem *x, const int32_t *pos_row, int k0, int t, int num_topk, int hidden,
                                             int num_expanded, int col, const float *topk_weights, const float *x_sf) {
    typename ReduceIn<InT>::raw raw[U];
    float s[U];
    bool live[U];
#pragma unroll
    for (int j = 0; j < U; ++j) {
        const int k = k0 + j;
        const int p = uniform_load(pos_row + k);
        live[j] = p >= 0 && p < num_expanded;
        // a skipped term reads row 0 (no branch around the loads) and is not added
        const int row = live[j] ? p : 0;
        raw[j].load(x + (int64_t)row * hidden + col);
        vmem_issue_gap();
        s[j] = 1.0f;
        if (topk_weights) s[j] = live[j] ? uniform_load(topk_weights + (int64_t)t * num_topk + k) : 0.0f;
        if (x_sf) s[j] = s[j] * uniform_load(x_sf + row);
    }
#pragma unroll
    for (int j = 0; j < U; ++j) {
        if (!live[j]) continue;      // wave-uniform
        float v[8];
        raw[j].get(v);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_fmaf(v[i], s[j], acc[i]);
    }
}

// OUT: 0 bf16, 1 fp32, 2 E4M3
template <typename InT, int OUT>
__global__ __launch_bounds__(kThreads) void reduce_fused_kernel(const typename ReduceIn<InT>::elem *x, const int32_t *token_topk_to_pos, int num_topk,
                                                                int hidden, int num_expanded, const float *topk_weights, const float *x_sf,
                                                                const float *sf, void *out) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    constexpr bool SPLIT = ReduceIn<InT>::split;
    const int t = blockIdx.y;
    // SPLIT: elements col .. col + 3 and col + 256 .. col + 259 (the wave's 512 columns are all inside the row or all outside)
    const int col = SPLIT ? (blockIdx.x * kThreads + (threadIdx.x & ~63)) * 8 + (threadIdx.x & 63) * 4 : (blockIdx.x * kThreads + threadIdx.x) * 8;
    if (col >= hidden) return;
    const int32_t *pos_row = token_topk_to_pos + (int64_t)t * num_topk;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    // whole groups of 8 terms, then the rest in steps of 4, 2 and 1: padding a short list to 8 with skipped terms would
    // still issue their loads (top-2 of bf16 [8576, 7168]: 46.7 us that way)
    int k0 = 0;
    for (; k0 + kReduceUnroll <= num_topk; k0 += kReduceUnroll)
        reduce_terms<InT, kReduceUnroll>(acc, x, pos_row, k0, t, num_topk, hidden, num_expanded, col, topk_weights, x_sf);
    if ((num_topk - k0) & 4) { reduce_terms<InT, 4>(acc, x, pos_row, k0, t, num_topk, hidden, num_expanded, col, topk_weights, x_sf); k0 += 4; }
    if ((num_topk - k0) & 2) { reduce_terms<InT, 2>(acc, x, pos_row, k0, t, num_topk, hidden, num_expanded, col, topk_weights, x_sf); k0 += 2; }
    if ((num_topk - k0) & 1) reduce_terms<InT, 1>(acc, x, pos_row, k0, t, num_topk, hidden, num_expanded, col, topk_weights, x_sf);
    if (sf) {
        const float f = uniform_load(sf);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = acc[i] * f;
    }
    const int64_t idx = (int64_t)t * hidden + col;
    if (OUT == 1) {
        u32x4 *o = reinterpret_cast<u32x4 *>(reinterpret_cast<float *>(out) + idx);
        __builtin_nontemporal_store(u32x4{f2u(acc[0]), f2u(acc[1]), f2u(acc[2]), f2u(acc[3])}, o);
        __builtin_nontemporal_store(u32x4{f2u(acc[4]), f2u(acc[5]), f2u(acc[6]), f2u(acc[7])}, o + (SPLIT ? 64 : 1));
    } else if (OUT == 0) {
        u32x4 w;
        w.x = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{acc[0], acc[1]}), bf16x2));
        w.y = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{acc[2], acc[3]}), bf16x2));
        w.z = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{acc[4], acc[5]}), bf16x2));
        w.w = __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2{acc[6], acc[7]}), bf16x2));
        // (written through: bf16 [4096, 4096] from top-8 of 256 experts 50.3 -> 49.2 us on MI355X against a non-temporal
        // store; the stores of most other kernels here lose that way, the expansion 64 -> 110 us)
        st_stream16(reinterpret_cast<uint16_t *>(out) + idx, w);
    } else if (SPLIT) {
        const u32x2 codes = pack_e4m3x8<false>(acc);
        st_stream4(reinterpret_cast<uint8_t *>(out) + idx, codes.x);
        st_stream4(reinterpret_cast<uint8_t *>(out) + idx + 256, codes.y);
    } else {
        st_stream8(reinterpret_cast<uint8_t *>(out) + idx, pack_e4m3x8<false>(acc));
    }
}

// reduce_fused without a single expanded row: every term is skipped, the result is zeros.  (The reduction kernel
// cannot run then: its skipped terms read row 0, which does not exist.)
__global__ __launch_bounds__(kThreads) void reduce_zero_kernel(uint64_t *out, int64_t words) {
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < words; i += (int64_t)gridDim.x * kThreads) out[i] = 0ull;
}

}  // namespace tk

using namespace tk;

extern "C" int64_t tk_fused_mapping_workspace_bytes(int64_t num_tokens, int num_topk, int num_experts) {
    if (num_tokens < 0 || num_topk <= 0 || num_experts <= 0) return 0;
    const int64_t slices = (num_tokens * num_topk + kSliceElems - 1) / kSliceElems;
    const int64_t padded = (slices + kWaves - 1) / kWaves * kWaves;       // whole workgroups
    return padded * num_experts * (int64_t)sizeof(int32_t);
}

extern "C" int tk_check_get_fused_mapping(const int64_t *topk_idx, int64_t num_tokens, int num_topk, int num_experts,
                                          int alignment, int64_t num_expanded, const int32_t *pos_to_expert,
                                          const int32_t *pos_to_token, const int32_t *pos_to_token_topk,
                                          const int32_t *token_topk_to_pos, const int32_t *expert_start,
                                          const int32_t *expert_end, const int32_t *num_tokens_per_expert,
                                          const void *workspace, int64_t workspace_bytes) {
    if (num_tokens < 0 || num_topk <= 0 || num_expanded < 0) return TK_ERR_BAD_SHAPE;
    if (num_experts <= 0 || num_experts > kMaxExperts) return TK_ERR_BAD_GROUP;
    if (alignment <= 0) return TK_ERR_BAD_VALUE;
    if (num_tokens * num_topk > INT32_MAX - 1024 || num_expanded > INT32_MAX - 1024) return TK_ERR_TOO_LARGE;
    if (!expert_start || !expert_end || !num_tokens_per_expert) return TK_ERR_NULL_POINTER;
    if (num_tokens > 0 && (!topk_idx || !token_topk_to_pos || !workspace)) return TK_ERR_NULL_POINTER;
    if (num_expanded > 0 && (!pos_to_expert || !pos_to_token || !pos_to_token_topk)) return TK_ERR_NULL_POINTER;
    if (workspace_bytes < tk_fused_mapping_workspace_bytes(num_tokens, num_topk, num_experts)) return TK_ERR_BAD_STRIDE;
    if (!aligned_to(topk_idx, 8) || !aligned_to(workspace, 4)) return TK_ERR_MISALIGNED;
    return TK_OK;
}

// the three launches; `ws` holds at least tk_fused_mapping_workspace_bytes() bytes
static int launch_fused_mapping(const int64_t *topk_idx, int64_t num_tokens, int num_topk, int num_experts, int alignment,
                                int64_t num_expanded, int32_t *pos_to_expert, int32_t *pos_to_token, int32_t *pos_to_token_topk,
                                int32_t *token_topk_to_pos, int32_t *expert_start, int32_t *expert_end,
                                int32_t *num_tokens_per_expert, int32_t *ws, hipStream_t s) {
    const int numel = (int)(num_tokens * num_topk);
    const int slices = (numel + kSliceElems - 1) / kSliceElems;
    const int blocks = (slices + kWaves - 1) / kWaves;
    const size_t lds = (size_t)kWaves * num_experts * sizeof(int32_t);
    int bits = 0;
    while ((1 << bits) < num_experts) ++bits;
    if (numel > 0 && numel <= kSingleLaunchPairs && num_experts <= kSingleMaxExperts) {
        const int groups = (numel + kSingleWaves * kSingleSlice - 1) / (kSingleWaves * kSingleSlice);
        hipLaunchKernelGGL(fused_mapping_single_kernel, dim3(groups), dim3(64 * kSingleWaves),
                           (size_t)(1 + kSingleWaves) * num_experts * sizeof(int32_t), s, topk_idx, numel, num_topk, num_experts, bits,
                           alignment, pos_to_expert, pos_to_token, pos_to_token_topk, token_topk_to_pos, expert_start, expert_end,
                           num_tokens_per_expert, (int)num_expanded);
        return (int)hipGetLastError();
    }
    // the count launch also fills the padding markers, so it runs even when there are no tokens
    const int fill_blocks = (int)((num_expanded + kThreads - 1) / kThreads);
    const int count_grid = blocks > 0 ? blocks : (fill_blocks > 1024 ? 1024 : fill_blocks);
    if (count_grid > 0)
        hipLaunchKernelGGL(fused_mapping_count_kernel, dim3(count_grid), dim3(kThreads), lds, s, topk_idx, numel, num_experts, ws,
                           pos_to_expert, pos_to_token, pos_to_token_topk, (int)num_expanded);
    hipLaunchKernelGGL(fused_mapping_scan_kernel, dim3(1), dim3(1024), 0, s, ws, slices, num_experts, alignment, expert_start,
                       expert_end, num_tokens_per_expert);
    if (blocks > 0)
        hipLaunchKernelGGL(fused_mapping_assign_kernel, dim3(blocks), dim3(kThreads), lds, s, topk_idx, numel, num_topk, num_experts,
                           bits, ws, expert_start, pos_to_expert, pos_to_token, pos_to_token_topk, token_topk_to_pos,
                           (int)num_expanded);
    return (int)hipGetLastError();
}

extern "C" int tk_get_fused_mapping(const int64_t *topk_idx, int64_t num_tokens, int num_topk, int num_experts, int alignment,
                                    int64_t num_expanded, int32_t *pos_to_expert, int32_t *pos_to_token,
                                    int32_t *pos_to_token_topk, int32_t *token_topk_to_pos, int32_t *expert_start,
                                    int32_t *expert_end, int32_t *num_tokens_per_expert, void *workspace,
                                    int64_t workspace_bytes, void *stream) {
    const int rc = tk_check_get_fused_mapping(topk_idx, num_tokens, num_topk, num_experts, alignment, num_expanded, pos_to_expert,
                                              pos_to_token, pos_to_token_topk, token_topk_to_pos, expert_start, expert_end,
                                              num_tokens_per_expert, workspace, workspace_bytes);
    if (rc != TK_OK) return rc;
    return launch_fused_mapping(topk_idx, num_tokens, num_topk, num_experts, alignment, num_expanded, pos_to_expert, pos_to_token,
                                pos_to_token_topk, token_topk_to_pos, expert_start, expert_end, num_tokens_per_expert,
                                static_cast<int32_t *>(workspace), static_cast<hipStream_t>(stream));
}

// ------------------------------------------------------------------------------------------------
// The same mapping for callers that cannot allocate or pass a workspace: the slice x expert table lives in a
// device array owned by the library.  Every GPU holds its own copy of the array at its own address, which is
// looked up once per device (the array's name is only a host-side handle, never a device address) and passed
// to the kernels like the caller's workspace above.  The count launch writes every table entry the later
// launches read, so nothing has to be cleared between calls; calls that overlap on one GPU would share the
// table and race.
static __device__ __align__(256) unsigned char scratch[TK_FUSED_MAPPING_STATIC_BYTES];

// device address of `scratch` on the current device
static int static_scratch_address(void **out) {
    constexpr int kMaxDevices = 64;
    static std::atomic<void *> known[kMaxDevices];
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return TK_ERR_TOO_LARGE;
    void *ptr = known[dev].load(std::memory_order_acquire);
    if (!ptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!ptr) return TK_ERR_NULL_POINTER;
        known[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return TK_OK;
}

extern "C" int tk_get_fused_mapping_static(const int64_t *topk_idx, int64_t num_tokens, int num_topk, int num_experts,
                                           int alignment, int64_t num_expanded, int32_t *pos_to_expert, int32_t *pos_to_token,
                                           int32_t *pos_to_token_topk, int32_t *token_topk_to_pos, int32_t *expert_start,
                                           int32_t *expert_end, int32_t *num_tokens_per_expert, void *stream) {
    // sizes first, so that an oversized request is reported as such whatever else is wrong with it
    if (num_tokens >= 0 && num_topk > 0 && num_experts > 0 && num_experts <= kMaxExperts &&
        num_tokens * num_topk <= INT32_MAX - 1024 &&
        tk_fused_mapping_workspace_bytes(num_tokens, num_topk, num_experts) > (int64_t)TK_FUSED_MAPPING_STATIC_BYTES)
        return TK_ERR_TOO_LARGE;
    void *ws = nullptr;
    int rc = static_scratch_address(&ws);
    if (rc != TK_OK) return rc;
    rc = tk_check_get_fused_mapping(topk_idx, num_tokens, num_topk, num_experts, alignment, num_expanded, pos_to_expert,
                                    pos_to_token, pos_to_token_topk, token_topk_to_pos, expert_start, expert_end,
                                    num_tokens_per_expert, ws, (int64_t)TK_FUSED_MAPPING_STATIC_BYTES);
    if (rc != TK_OK) return rc;
    return launch_fused_mapping(topk_idx, num_tokens, num_topk, num_experts, alignment, num_expanded, pos_to_expert, pos_to_token,
                                pos_to_token_topk, token_topk_to_pos, expert_start, expert_end, num_tokens_per_expert,
                                static_cast<int32_t *>(ws), static_cast<hipStream_t>(stream));
}

extern "C" int tk_check_expand_to_fused(const void *x, int64_t num_tokens, int64_t row_bytes, const int32_t *token_topk_to_pos,
                                        int num_topk, const int32_t *pos_to_expert, int64_t num_expanded, const void *out,
                                        const void *x_sf, int sf_cols, const void *out_sf, int64_t out_sf_ld,
                                        int sf_col_major) {
    if (num_tokens < 0 || num_expanded < 0 || row_bytes <= 0 || num_topk <= 0) return TK_ERR_BAD_SHAPE;
    if (row_bytes % 16 != 0) return TK_ERR_MISALIGNED;
    if (num_tokens + num_expanded > INT32_MAX - 1024) return TK_ERR_TOO_LARGE;
    {   // one workgroup per (token, position, 4 KB chunk) and one per expanded row
        const int64_t chunks = (row_bytes + kExpandChunk - 1) / kExpandChunk;
        if (chunks > INT32_MAX / 8 || num_topk > INT32_MAX / 8) return TK_ERR_TOO_LARGE;
        if (((num_tokens + 7) / 8 * 8) > (INT32_MAX - 1024 - num_expanded) / (num_topk * chunks)) return TK_ERR_TOO_LARGE;
    }
    if (num_expanded > 0 && (!pos_to_expert || !out)) return TK_ERR_NULL_POINTER;
    if (num_tokens > 0 && (!x || !token_topk_to_pos)) return TK_ERR_NULL_POINTER;
    if (!aligned_to(x, 16) || !aligned_to(out, 16)) return TK_ERR_MISALIGNED;
    if (x_sf) {
        if (sf_cols <= 0) return TK_ERR_BAD_SHAPE;
        if (!out_sf) return TK_ERR_NULL_POINTER;
        if (!aligned_to(x_sf, 4) || !aligned_to(out_sf, 4)) return TK_ERR_MISALIGNED;
        if (out_sf_ld < (sf_col_major ? num_expanded : sf_cols)) return TK_ERR_BAD_STRIDE;
    }
    return TK_OK;
}

extern "C" int tk_expand_to_fused(const void *x, int64_t num_tokens, int64_t row_bytes, const int32_t *token_topk_to_pos,
                                  int num_topk, const int32_t *pos_to_expert, int64_t num_expanded, void *out, const void *x_sf,
                                  int sf_cols, void *out_sf, int64_t out_sf_ld, int sf_col_major, void *stream) {
    const int rc = tk_check_expand_to_fused(x, num_tokens, row_bytes, token_topk_to_pos, num_topk, pos_to_expert, num_expanded, out,
                                            x_sf, sf_cols, out_sf, out_sf_ld, sf_col_major);
    if (rc != TK_OK) return rc;
    const int64_t chunks = (row_bytes + kExpandChunk - 1) / kExpandChunk;
    // rows of at most half a chunk: several positions of a token per workgroup
    const int tpr = (int)((row_bytes + 15) / 16);
    const int kpw = tpr * 2 <= kThreads ? (kThreads / tpr < num_topk ? kThreads / tpr : num_topk) : 1;
    const int64_t copy_blocks = (num_tokens + 7) / 8 * 8 * (kpw > 1 ? (num_topk + kpw - 1) / kpw : num_topk * chunks);
    // padding workgroups take 8 KB of consecutive rows each, two stores per thread.  Measured (us per call, 1 / 2 / 4
    // rows per workgroup): 8 KB rows 64.4 / 69.7 / 71.0; 4 KB rows with scales 41.4 / 36.0 / 37.0
    const int pad_rows = row_bytes >= 8192 ? 1 : (int)(8192 / row_bytes > 8 ? 8 : 8192 / row_bytes);
    const int64_t grid = copy_blocks + (num_expanded + pad_rows - 1) / pad_rows;
    if (grid == 0) return TK_OK;
    if (kpw > 1)
        hipLaunchKernelGGL(expand_short_rows_kernel, dim3((unsigned)grid), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                           static_cast<const uint8_t *>(x), row_bytes, token_topk_to_pos, num_topk, kpw, tpr, (int)copy_blocks,
                           (int)num_tokens, (int)num_expanded, static_cast<uint8_t *>(out), pos_to_expert,
                           static_cast<const uint32_t *>(x_sf), sf_cols, static_cast<uint32_t *>(out_sf), out_sf_ld, sf_col_major, pad_rows);
    else
        hipLaunchKernelGGL(expand_to_fused_kernel, dim3((unsigned)grid), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                           static_cast<const uint8_t *>(x), row_bytes, token_topk_to_pos, num_topk, (int)chunks, (int)copy_blocks,
                           (int)num_tokens, (int)num_expanded, static_cast<uint8_t *>(out), pos_to_expert,
                           static_cast<const uint32_t *>(x_sf), sf_cols, static_cast<uint32_t *>(out_sf), out_sf_ld, sf_col_major, pad_rows);
    return (int)hipGetLastError();
}

extern "C" int tk_check_reduce_fused(const void *x, int x_dtype, int64_t num_expanded, int64_t hidden, const float *x_sf,
                                     const float *topk_weights, const int32_t *token_topk_to_pos, int64_t num_tokens, int num_topk,
                                     const void *out, int out_dtype, const float *sf) {
    (void)x_sf;
    (void)topk_weights;
    (void)sf;
    if (x_dtype != TK_BF16 && x_dtype != TK_F32) return TK_ERR_BAD_DTYPE;
    if (out_dtype != x_dtype && out_dtype != TK_OUT_E4M3) return TK_ERR_BAD_DTYPE;      // same type as the input, or FP8
    if (num_tokens < 0 || num_expanded < 0 || num_topk <= 0 || hidden <= 0 || hidden % 8 != 0) return TK_ERR_BAD_SHAPE;
    if (num_tokens > 65535LL * 65535 || num_expanded > INT32_MAX - 1 || hidden > INT32_MAX - 4096) return TK_ERR_TOO_LARGE;
    if (num_tokens == 0) return TK_OK;
    if (!token_topk_to_pos || !out) return TK_ERR_NULL_POINTER;
    if (num_expanded > 0 && !x) return TK_ERR_NULL_POINTER;
    if (!aligned_to(x, 16) || !aligned_to(out, out_dtype == TK_OUT_E4M3 ? 8 : 16)) return TK_ERR_MISALIGNED;
    if (x_dtype == TK_F32 && !aligned_to(x, 16)) return TK_ERR_MISALIGNED;
    return TK_OK;
}

extern "C" int tk_reduce_fused(const void *x, int x_dtype, int64_t num_expanded, int64_t hidden, const float *x_sf,
                               const float *topk_weights, const int32_t *token_topk_to_pos, int64_t num_tokens, int num_topk,
                               void *out, int out_dtype, const float *sf, void *stream) {
    const int rc = tk_check_reduce_fused(x, x_dtype, num_expanded, hidden, x_sf, topk_weights, token_topk_to_pos, num_tokens,
                                         num_topk, out, out_dtype, sf);
    if (rc != TK_OK || num_tokens == 0) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (num_expanded == 0) {
        const int64_t words = num_tokens * hidden * (out_dtype == TK_F32 ? 4 : (out_dtype == TK_BF16 ? 2 : 1)) / 8;   // hidden % 8 == 0
        const int64_t blocks = (words + kThreads - 1) / kThreads;
        hipLaunchKernelGGL(reduce_zero_kernel, dim3((unsigned)(blocks < 65536 ? blocks : 65536)), dim3(kThreads), 0, s,
                           static_cast<uint64_t *>(out), words);
        return (int)hipGetLastError();
    }
    const unsigned chunks = (unsigned)((hidden + kThreads * 8 - 1) / (kThreads * 8));
    // tokens ride on grid.y (at most 65535 per launch)
    for (int64_t t0 = 0; t0 < num_tokens; t0 += 65535) {
        const unsigned nt = (unsigned)(num_tokens - t0 < 65535 ? num_tokens - t0 : 65535);
        const dim3 grid(chunks, nt);
        const int32_t *pos = token_topk_to_pos + t0 * num_topk;
        const float *w = topk_weights ? topk_weights + t0 * num_topk : nullptr;
        const int64_t out_bytes = out_dtype == TK_F32 ? 4 : (out_dtype == TK_BF16 ? 2 : 1);
        void *o = static_cast<uint8_t *>(out) + t0 * hidden * out_bytes;
#define TK_REDUCE_LAUNCH(T, O)                                                                                              \
    hipLaunchKernelGGL((reduce_fused_kernel<T, O>), grid, dim3(kThreads), 0, s, static_cast<const ReduceIn<T>::elem *>(x), pos, num_topk, \
                       (int)hidden, (int)num_expanded, w, x_sf, sf, o)
        if (x_dtype == TK_BF16) {
            if (out_dtype == TK_OUT_E4M3) TK_REDUCE_LAUNCH(bf16_t, 2);
            else TK_REDUCE_LAUNCH(bf16_t, 0);
        } else if (hidden % 512 == 0) {
            if (out_dtype == TK_OUT_E4M3) TK_REDUCE_LAUNCH(SplitF32, 2);
            else TK_REDUCE_LAUNCH(SplitF32, 1);
        } else {
            if (out_dtype == TK_OUT_E4M3) TK_REDUCE_LAUNCH(float, 2);
            else TK_REDUCE_LAUNCH(float, 1);
        }
#undef TK_REDUCE_LAUNCH
    }
    return (int)hipGetLastError();
}
