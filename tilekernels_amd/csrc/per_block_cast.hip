// Per-block (bm x bk, bm/bk in {32, 128}) block-scaled cast to E4M3 / E2M1 for gfx950.
//
// A workgroup of 256 threads owns one 128 x 128 tile, i.e. 1, 4 or 16 scale blocks.  Thread
// (t, c) = (tid / 16, tid % 16) holds the 8 elements at columns 8c.. of rows t, t+16, .., t+112:
// eight 16-byte loads per thread (bf16), all issued up front; the tile stays in registers between
// the amax reduction and the conversion, so HBM is read once.  The amax of a block is reduced
// over the bk/8 lanes that share it with DPP, then across rows and waves with an LDS integer max.
//
// Reference semantics: tile_kernels/quant/per_block_cast_kernel.py:52-136.
#include "tk_device.hpp"
#include "tk_host.hpp"

namespace tk {

constexpr int kBlockTile = 128;

struct PerBlockParams {
    const void *x;
    uint8_t *out;
    SfRef sf;
    int M, K;
    int tiles_m, tiles_k;
    int round_sf, mode;
};

template <typename InT, int FMT, int BM, int BK>
__global__ __launch_bounds__(kThreads) void per_block_cast_kernel(const PerBlockParams p) {
    constexpr int SUBM = kBlockTile / BM, SUBK = kBlockTile / BK;   // scale blocks per tile
    constexpr int LPG = BK / 8;                                      // lanes sharing a block in one row
    constexpr int NI = kBlockTile / 16;                              // rows per thread
    constexpr int IPB = BM / 16;                                     // of which per scale block
    __shared__ uint32_t amax_lds[SUBM][SUBK];

    const int tile_m = blockIdx.x / p.tiles_k, tile_k = blockIdx.x - tile_m * p.tiles_k;

    const int t = threadIdx.x >> 4, c = threadIdx.x & 15;
    const int col = tile_k * kBlockTile + c * 8;
    const int bj = (c * 8) / BK;
    const bool col_ok = col < p.K;
    const int row0 = tile_m * kBlockTile + t;
    const InT *x = reinterpret_cast<const InT *>(p.x);
    const int64_t out_ld = FMT == TK_E4M3 ? p.K : p.K / 2;

    if (p.mode != TK_CAST_GIVEN_SF && threadIdx.x < SUBM * SUBK) amax_lds[threadIdx.x / SUBK][threadIdx.x % SUBK] = 0u;

    Raw8<InT> raw[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int row = row0 + 16 * i;
        raw[i].load(x + (int64_t)row * p.K + col, col_ok && row < p.M);
    }

    float inv[SUBM];
    if (p.mode != TK_CAST_GIVEN_SF) {
        __syncthreads();   // zeroes visible
#pragma unroll
        for (int b = 0; b < SUBM; ++b) {
            float m = 0.0f;
#pragma unroll
            for (int i = b * IPB; i < (b + 1) * IPB; ++i) {
                float v[8];
                raw[i].get(v);
                m = __builtin_fmaxf(m, absmax8(v));
            }
            m = group_allmax<LPG>(m);
            if ((c % LPG) == 0) atomicMax(&amax_lds[b][bj], f2u(m));
        }
        __syncthreads();
#pragma unroll
        for (int b = 0; b < SUBM; ++b)
            inv[b] = make_scale<Fmt<FMT>::qmax>(u2f(amax_lds[b][bj]), Fmt<FMT>::floor_, p.round_sf != 0).inv;
        if (threadIdx.x < SUBM * SUBK) {
            const int b = threadIdx.x / SUBK, j = threadIdx.x % SUBK;
            const int m = tile_m * SUBM + b, k = tile_k * SUBK + j;
            if (m < p.sf.nm && k < p.sf.nk)
                sf_store(p.sf, m, k, make_scale<Fmt<FMT>::qmax>(u2f(amax_lds[b][j]), Fmt<FMT>::floor_, p.round_sf != 0));
        }
    } else {
#pragma unroll
        for (int b = 0; b < SUBM; ++b) {
            const int m = tile_m * SUBM + b, k = tile_k * SUBK + bj;
            const float s = (m < p.sf.nm && k < p.sf.nk) ? sf_load(p.sf, m, k) : 1.0f;
            inv[b] = 1.0f / s;
        }
    }
    if (p.mode == TK_SF_ONLY) return;

#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int row = row0 + 16 * i;
        if (col_ok && row < p.M) {
            float v[8];
            raw[i].get(v);
            uint8_t *out_row = p.out + (int64_t)row * out_ld;
            if (p.mode == TK_CAST_GIVEN_SF) quantise_store8<FMT, true>(v, inv[i / IPB], out_row, col);
            else quantise_store8<FMT, false>(v, inv[i / IPB], out_row, col);
        }
    }
}

template <typename InT, int FMT>
static hipError_t launch_per_block(const PerBlockParams &p, int bm, int bk, hipStream_t stream) {
    const int total = p.tiles_m * p.tiles_k;
    const dim3 grid((unsigned)total), block(kThreads);
    if (bm == 128 && bk == 128) hipLaunchKernelGGL((per_block_cast_kernel<InT, FMT, 128, 128>), grid, block, 0, stream, p);
    else if (bm == 32 && bk == 32) hipLaunchKernelGGL((per_block_cast_kernel<InT, FMT, 32, 32>), grid, block, 0, stream, p);
    else if (bm == 128 && bk == 32) hipLaunchKernelGGL((per_block_cast_kernel<InT, FMT, 128, 32>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((per_block_cast_kernel<InT, FMT, 32, 128>), grid, block, 0, stream, p);
    return hipGetLastError();
}

}  // namespace tk

using namespace tk;

extern "C" int tk_check_per_block_cast(const void *x, int x_dtype, int64_t M, int64_t K, const void *out,
                                       const void *sf, int64_t sf_ld, int fmt, int bm, int bk, int sf_layout,
                                       int round_sf, int mode) {
    if (x_dtype != TK_BF16 && x_dtype != TK_F32) return TK_ERR_BAD_DTYPE;
    if (fmt != TK_E4M3 && fmt != TK_E2M1) return TK_ERR_BAD_FORMAT;
    if (mode < TK_CAST_AND_SF || mode > TK_CAST_GIVEN_SF) return TK_ERR_BAD_MODE;
    if (sf_layout < TK_SF_ROW_F32 || sf_layout > TK_SF_COL_UE8M0) return TK_ERR_BAD_LAYOUT;
    if (mode == TK_CAST_GIVEN_SF && sf_layout != TK_SF_ROW_F32) return TK_ERR_BAD_LAYOUT;
    if (sf_layout == TK_SF_COL_UE8M0 && !round_sf) return TK_ERR_BAD_LAYOUT;
    if ((bm != 32 && bm != 128) || (bk != 32 && bk != 128)) return TK_ERR_BAD_GROUP;
    if (M < 0 || K <= 0 || K % 64 != 0) return TK_ERR_BAD_SHAPE;
    if (M > INT32_MAX - 256 || K > INT32_MAX - 256) return TK_ERR_TOO_LARGE;
    if (M == 0) return TK_OK;
    if (!x || !sf || (mode != TK_SF_ONLY && !out)) return TK_ERR_NULL_POINTER;
    if (!aligned_to(x, 16) || (mode != TK_SF_ONLY && !aligned_to(out, 8)) || !aligned_to(sf, 4)) return TK_ERR_MISALIGNED;
    const int64_t nm = (M + bm - 1) / bm, nk = (K + bk - 1) / bk;
    const int64_t need = sf_layout == TK_SF_ROW_F32 ? nk : (sf_layout == TK_SF_COL_F32 ? nm : 4 * nm);
    if (sf_ld < need) return TK_ERR_BAD_STRIDE;
    const int64_t tiles = ((M + kBlockTile - 1) / kBlockTile) * ((K + kBlockTile - 1) / kBlockTile);
    if (tiles > INT32_MAX - 8) return TK_ERR_TOO_LARGE;
    return TK_OK;
}

extern "C" int tk_per_block_cast(const void *x, int x_dtype, int64_t M, int64_t K, void *out, void *sf,
                                 int64_t sf_ld, int fmt, int bm, int bk, int sf_layout, int round_sf, int mode,
                                 void *stream) {
    const int rc = tk_check_per_block_cast(x, x_dtype, M, K, out, sf, sf_ld, fmt, bm, bk, sf_layout, round_sf, mode);
    if (rc != TK_OK || M == 0) return rc;
    PerBlockParams p;
    p.x = x;
    p.out = static_cast<uint8_t *>(out);
    p.sf = SfRef{sf, sf_ld, sf_layout, (int)((M + bm - 1) / bm), (int)((K + bk - 1) / bk)};
    p.M = (int)M;
    p.K = (int)K;
    p.tiles_m = (int)((M + kBlockTile - 1) / kBlockTile);
    p.tiles_k = (int)((K + kBlockTile - 1) / kBlockTile);
    p.round_sf = round_sf;
    p.mode = mode;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e;
    if (x_dtype == TK_BF16)
        e = fmt == TK_E4M3 ? launch_per_block<bf16_t, TK_E4M3>(p, bm, bk, s) : launch_per_block<bf16_t, TK_E2M1>(p, bm, bk, s);
    else
        e = fmt == TK_E4M3 ? launch_per_block<float, TK_E4M3>(p, bm, bk, s) : launch_per_block<float, TK_E2M1>(p, bm, bk, s);
    return (int)e;
}
