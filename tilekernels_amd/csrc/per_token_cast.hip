// Per-token (1 x G) block-scaled cast to E4M3 / E2M1 for gfx950.
//
// Work decomposition: a workgroup of 4 waves owns a tile of 16 rows x 512 columns.  Each wave
// takes 4 rows; in every row its 64 lanes cover 512 consecutive elements with one 16-byte (bf16)
// or two 16-byte (fp32) loads per lane, all four rows' loads issued before the first use.  A group
// of G elements therefore lives in G/8 neighbouring lanes of one DPP row and its amax needs no LDS.
// Row-major scales are stored straight from the group's first lane; column-major layouts are
// staged in LDS and written out transposed so that 16 lanes fill one 64-byte segment.
//
// Reference semantics: tile_kernels/quant/per_token_cast_kernel.py:65-154 (plain-tensor branch),
// tile_kernels/quant/common.py:196-244.
#include "tk_device.hpp"
#include "tk_host.hpp"

namespace tk {

struct PerTokenParams {
    const void *x;
    uint8_t *out;
    SfRef sf;
    int64_t x_ld;     // elements between rows of x
    int M, K;
    int tiles_m, tiles_k;
    int round_sf, mode;
};

template <typename InT, int G, int FMT>
__global__ __launch_bounds__(kThreads) void per_token_cast_kernel(const PerTokenParams p) {
    constexpr int LPG = G / 8;            // lanes per group
    constexpr int GPS = kStripCols / G;   // groups per 512-column strip
    constexpr int RPW = kTileRows / 4;    // rows per wave
    __shared__ uint32_t stage[kTileRows][GPS];

    const int tile = xcd_tile_index(p.tiles_m * p.tiles_k);
    if (tile < 0) return;
    const int tile_m = tile / p.tiles_k, tile_k = tile - tile_m * p.tiles_k;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = tile_k * kStripCols + lane * 8;
    const int g_in_strip = lane / LPG;
    const int kgrp = tile_k * GPS + g_in_strip;
    const bool col_ok = col < p.K;
    const bool leader = (lane % LPG) == 0;
    const int row0 = tile_m * kTileRows + wave * RPW;
    const int64_t out_ld = FMT == TK_E4M3 ? p.K : p.K / 2;
    const InT *x = reinterpret_cast<const InT *>(p.x);

    Raw8<InT> raw[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        const int row = row0 + r;
        raw[r].load(x + (int64_t)row * p.x_ld + col, col_ok && row < p.M);
    }

    const bool staged = p.sf.layout != TK_SF_ROW_F32 && p.mode != TK_CAST_GIVEN_SF;
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        const int row = row0 + r;
        const bool ok = col_ok && row < p.M;
        float v[8];
        raw[r].get(v);
        Scale sc;
        if (p.mode == TK_CAST_GIVEN_SF) {
            const float s = ok ? sf_load(p.sf, row, kgrp) : 1.0f;
            sc.inv = 1.0f / s;
        } else {
            const float amax = group_allmax<LPG>(absmax8(v));
            sc = make_scale(amax, Fmt<FMT>::floor_, Fmt<FMT>::qmax, p.round_sf != 0);
            if (leader) {
                if (staged) {
                    stage[wave * RPW + r][g_in_strip] = p.sf.layout == TK_SF_COL_F32 ? f2u(sc.sf) : sc.e8;
                } else if (ok) {
                    reinterpret_cast<float *>(p.sf.base)[(int64_t)row * p.sf.ld + kgrp] = sc.sf;
                }
            }
        }
        if (p.mode != TK_SF_ONLY && ok) {
            uint8_t *out_row = p.out + (int64_t)row * out_ld;
            if (p.mode == TK_CAST_GIVEN_SF) quantise_store8<FMT, true>(v, sc.inv, out_row, col);
            else quantise_store8<FMT, false>(v, sc.inv, out_row, col);
        }
    }
    if (staged) {
        __syncthreads();
        sf_store_tile_colmajor<GPS>(p.sf, stage, tile_m * kTileRows, tile_k * GPS);
    }
}

// One scale per row (group == K): a workgroup per row, two passes over the row (the second one is
// served by L2).  Reference: the `hidden == num_per_channels` branch,
// tile_kernels/quant/per_token_cast_kernel.py:31-35.
template <typename InT, int FMT>
__global__ __launch_bounds__(kThreads) void per_token_rowgroup_kernel(const PerTokenParams p) {
    __shared__ uint32_t part[kThreads / 16];
    const int row = blockIdx.x;
    const InT *x = reinterpret_cast<const InT *>(p.x) + (int64_t)row * p.x_ld;
    float amax = 0.0f;
    for (int col = threadIdx.x * 8; col < p.K; col += kThreads * 8) {
        Raw8<InT> raw;
        raw.load(x + col, true);
        float v[8];
        raw.get(v);
        amax = __builtin_fmaxf(amax, absmax8(v));
    }
    amax = group_allmax<16>(amax);
    if ((threadIdx.x & 15) == 0) part[threadIdx.x >> 4] = f2u(amax);
    __syncthreads();
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < kThreads / 16; ++i) m = umax(m, part[i]);
    const Scale sc = make_scale(u2f(m), Fmt<FMT>::floor_, Fmt<FMT>::qmax, p.round_sf != 0);
    if (threadIdx.x == 0) sf_store(p.sf, row, 0, sc);
    const int64_t out_ld = FMT == TK_E4M3 ? p.K : p.K / 2;
    uint8_t *out_row = p.out + (int64_t)row * out_ld;
    for (int col = threadIdx.x * 8; col < p.K; col += kThreads * 8) {
        Raw8<InT> raw;
        raw.load(x + col, true);
        float v[8];
        raw.get(v);
        quantise_store8<FMT, false>(v, sc.inv, out_row, col);
    }
}

template <typename InT, int FMT>
static hipError_t launch_per_token(const PerTokenParams &p, int group, hipStream_t stream) {
    if (group == p.K && group != 16 && group != 32 && group != 64 && group != 128) {
        hipLaunchKernelGGL((per_token_rowgroup_kernel<InT, FMT>), dim3(p.M), dim3(kThreads), 0, stream, p);
        return hipGetLastError();
    }
    const int total = p.tiles_m * p.tiles_k;
    const dim3 grid(kNumXcd * ((total + kNumXcd - 1) / kNumXcd));
    switch (group) {
        case 16: hipLaunchKernelGGL((per_token_cast_kernel<InT, 16, FMT>), grid, dim3(kThreads), 0, stream, p); break;
        case 32: hipLaunchKernelGGL((per_token_cast_kernel<InT, 32, FMT>), grid, dim3(kThreads), 0, stream, p); break;
        case 64: hipLaunchKernelGGL((per_token_cast_kernel<InT, 64, FMT>), grid, dim3(kThreads), 0, stream, p); break;
        default: hipLaunchKernelGGL((per_token_cast_kernel<InT, 128, FMT>), grid, dim3(kThreads), 0, stream, p); break;
    }
    return hipGetLastError();
}

}  // namespace tk

using namespace tk;

extern "C" int tk_check_per_token_cast(const void *x, int x_dtype, int64_t M, int64_t K, int64_t x_row_stride,
                                       const void *out, const void *sf, int64_t sf_ld, int fmt, int group,
                                       int sf_layout, int round_sf, int mode) {
    if (x_dtype != TK_BF16 && x_dtype != TK_F32) return TK_ERR_BAD_DTYPE;
    if (fmt != TK_E4M3 && fmt != TK_E2M1) return TK_ERR_BAD_FORMAT;
    if (mode < TK_CAST_AND_SF || mode > TK_CAST_GIVEN_SF) return TK_ERR_BAD_MODE;
    if (sf_layout < TK_SF_ROW_F32 || sf_layout > TK_SF_COL_UE8M0) return TK_ERR_BAD_LAYOUT;
    if (sf_layout == TK_SF_COL_UE8M0 && !round_sf && mode != TK_CAST_GIVEN_SF) return TK_ERR_BAD_LAYOUT;
    if (M < 0 || K <= 0 || K % 8 != 0) return TK_ERR_BAD_SHAPE;
    if (M > INT32_MAX - 64 || K > INT32_MAX - 1024) return TK_ERR_TOO_LARGE;
    const bool row_group = group == K && group != 16 && group != 32 && group != 64 && group != 128;
    if (row_group) {
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
    p.tiles_m = (int)((M + kTileRows - 1) / kTileRows);
    p.tiles_k = (int)((K + kStripCols - 1) / kStripCols);
    p.round_sf = round_sf;
    p.mode = mode;
    if ((int64_t)p.tiles_m * p.tiles_k > INT32_MAX - 8) return TK_ERR_TOO_LARGE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e;
    if (x_dtype == TK_BF16)
        e = fmt == TK_E4M3 ? launch_per_token<bf16_t, TK_E4M3>(p, group, s) : launch_per_token<bf16_t, TK_E2M1>(p, group, s);
    else
        e = fmt == TK_E4M3 ? launch_per_token<float, TK_E4M3>(p, group, s) : launch_per_token<float, TK_E2M1>(p, group, s);
    return (int)e;
}
