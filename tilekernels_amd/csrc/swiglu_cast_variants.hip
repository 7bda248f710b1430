// Measurement aid: alternative structures of the fused SwiGLU + 1 x 128 E4M3 cast, for the plain case only (bf16
// input, row-major fp32 scales, no mask, no routing weights, no clamp, H a multiple of 2048 and R of 8), so that the
// figures quoted for them can be measured again:  python bench.py --variant <name>[:<param>]
//
// Every variant computes the same values as tk_swiglu_per_token_cast, bit for bit (bench.py checks that before it
// times one).  None of them is reachable from the Python API.
//
//   base[:w]     the structure of the product kernel: one row per wave, its four 512-column pieces (eight 16-byte
//                loads per lane) requested before the first is used, the four scale divisions of a 128-column group
//                shared out over four lanes, all stores at the end.  w = waves (rows) per workgroup: 1, 2, 4 (default), 8
//   pkfloor[:w]  base with the -88 cap of the gate applied to the packed bf16 pairs (one 16-bit packed minimum per two
//                gates instead of one 32-bit minimum per gate)
//   widest[:w]   base with neighbouring lanes exchanging halves of two pieces, so that a lane stores 16 consecutive
//                codes with one 16-byte store: two store instructions per wave instead of four
//   prio[:w]     base raising the wave's priority once its first piece has arrived
//   piecesf      a scale division per piece and lane, each piece stored as soon as it is converted
//   late:t       piecesf for the waves whose first piece arrives more than t * 10 ns after their start, base for the others
//   ahead:n      pieces requested n (1, 2) ahead of the one being evaluated instead of all at once; a piece's scales
//                are computed and its codes stored before the next piece is waited for
//   rounds:p     p (1, 2) pieces per wave instead of 4: 4 / p times the waves, in 4 / p occupancy rounds at [8192, 4096]
//   tail:t       (H = 2048 only) the last t per cent of the rows as four one-piece waves each, launched behind the one-row
//                waves of the other rows: the work that arrives last is then spread over four times as many SIMDs
#include "swiglu_math.hpp"
#include "tk_device.hpp"
#include "tk_host.hpp"

namespace tk {

enum { V_BASE = 0, V_PKFLOOR = 1, V_WIDEST = 2, V_PRIO = 3, V_PIECESF = 4, V_LATE = 5, V_AHEAD = 6, V_ROUNDS = 7, V_TAIL = 8 };

// the eight activations of one lane's piece
template <bool PKFLOOR> __device__ __forceinline__ void eval_piece(const u32x4 &gw, const u32x4 &uw, float (&v)[8]) {
    Raw8<bf16_t> rg, ru;
    rg.w = gw;
    ru.w = uw;
    float g[8], u[8];
    ru.get(u);
    if constexpr (PKFLOOR) {
        // bf16 patterns order like the fp32 patterns they are the top half of: the cap works on both halves of a word at once,
        // and the capped gate serves the quotient too (below -88 either form gives a magnitude under 1e-35, i.e. a zero code)
        typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
        const u16x2 cap = {0xC2B0, 0xC2B0};
        uint32_t w[4] = {gw.x, gw.y, gw.z, gw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u16x2 m = __builtin_elementwise_min(__builtin_bit_cast(u16x2, w[i]), cap);
            w[i] = __builtin_bit_cast(uint32_t, m);
        }
        rg.w = u32x4{w[0], w[1], w[2], w[3]};
        rg.get(g);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float d = 1.0f + __builtin_amdgcn_exp2f(g[i] * -1.4426950408889634f);
            v[i] = quotient(g[i], d) * u[i];
        }
    } else {
        rg.get(g);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = silu_mul<bf16_t>(g[i], u[i]);
    }
}

__device__ __forceinline__ u32x2 convert_piece(const float (&v)[8], float inv) {
    float q[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = v[i] * inv;
    return pack_e4m3x8<false>(q);
}

// scale of the lane's own group computed by the lane itself; the first lane of the group stores it
__device__ __forceinline__ float own_scale_store(float amax, float floor_, float *sf_row, int k, int lane) {
    const Scale sc = make_scale<448>(amax, floor_, false);
    if ((lane & 15) == 0) st_stream4(sf_row + k, f2u(sc.sf));
    return sc.inv;
}

template <int VARIANT, int RPW, int AHEAD>
__global__ __launch_bounds__(64 * kMaxWideWaves) void swiglu_variant_kernel(const bf16_t *x, int R, int H, int nwaves, int tiles_k,
                                                                            uint8_t *out, float *sf, int nk, float floor_, int param) {
    const int lane = threadIdx.x & 63, wave = wave_id();
    const int tile_m = tile_grid_row(tiles_k == 1), tile_k = tile_grid_col(tiles_k == 1);
    const int row = tile_m * nwaves + wave;
    if (row >= R) return;
    const int strip = tile_k * RPW;
    const int col = strip * kStripCols + lane * 8;
    const bf16_t *xr = x + (int64_t)row * (2 * (int64_t)H) + col;
    uint8_t *out_row = out + (int64_t)row * H;
    float *sf_row = sf + (int64_t)row * nk;
    constexpr int GPS = kStripCols / 128;
    using RS = RowScales<448, RPW, 16>;

    if constexpr (VARIANT == V_AHEAD) {
        // AHEAD pieces in flight ahead of the one being evaluated
        u32x4 gw[RPW], uw[RPW];
#pragma unroll
        for (int r = 0; r < AHEAD && r < RPW; ++r) {
            gw[r] = ld_stream16(xr + r * kStripCols);
            vmem_issue_gap();
            uw[r] = ld_stream16(xr + H + r * kStripCols);
            vmem_issue_gap();
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            if (r + AHEAD < RPW) {
                gw[r + AHEAD < RPW ? r + AHEAD : 0] = ld_stream16(xr + (r + AHEAD) * kStripCols);
                vmem_issue_gap();
                uw[r + AHEAD < RPW ? r + AHEAD : 0] = ld_stream16(xr + H + (r + AHEAD) * kStripCols);
                vmem_issue_gap();
            }
            float v[8];
            eval_piece<false>(gw[r], uw[r], v);
            const float inv = own_scale_store(group_allmax<16>(absmax8(v)), floor_, sf_row, (strip + r) * GPS + (lane >> 4), lane);
            st_stream8(out_row + col + r * kStripCols, convert_piece(v, inv));
        }
        return;
    }

    unsigned long long t_start = 0;
    if constexpr (VARIANT == V_LATE) t_start = wall_clock64();
    u32x4 gw[RPW], uw[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        gw[r] = ld_stream16(xr + r * kStripCols);
        vmem_issue_gap();
        uw[r] = ld_stream16(xr + H + r * kStripCols);
        vmem_issue_gap();
    }
    if constexpr (VARIANT == V_PRIO) asm volatile("s_waitcnt vmcnt(%0)\n\ts_setprio 3" ::"n"(2 * RPW - 1) : "memory");
    bool piecewise = VARIANT == V_PIECESF;
    if constexpr (VARIANT == V_LATE) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * RPW - 2) : "memory");
        piecewise = (long long)(wall_clock64() - t_start) > (long long)param;
    }
    if (VARIANT == V_PIECESF || (VARIANT == V_LATE && piecewise)) {
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            float v[8];
            eval_piece<false>(gw[r], uw[r], v);
            const float inv = own_scale_store(group_allmax<16>(absmax8(v)), floor_, sf_row, (strip + r) * GPS + (lane >> 4), lane);
            st_stream8(out_row + col + r * kStripCols, convert_piece(v, inv));
        }
        return;
    }

    float v[RPW][8], amax[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        eval_piece<VARIANT == V_PKFLOOR>(gw[r], uw[r], v[r]);
        amax[r] = group_allmax<16>(absmax8(v[r]));
    }
    RS rs;
    rs.compute(amax, floor_, false, lane);
    const int own = lane & 15;
    if (own < RS::A) {
#pragma unroll
        for (int c = 0; c < RS::NC; ++c)
            st_stream4(sf_row + (strip + c * RS::A + own) * GPS + (lane >> 4), f2u(rs.own[c].sf));
    }
    if constexpr (VARIANT == V_WIDEST && RPW % 2 == 0) {
        // pieces a = 2j and b = 2j + 1: the even lane of a pair ends up with the 16 codes of piece a that the pair holds, the
        // odd lane with those of piece b
        const bool odd = lane & 1;
#pragma unroll
        for (int j = 0; j < RPW / 2; ++j) {
            const u32x2 a = convert_piece(v[2 * j], rs.inv[2 * j]), b = convert_piece(v[2 * j + 1], rs.inv[2 * j + 1]);
            const u32x2 send = odd ? a : b;
            const u32x2 recv = {dpp_u32<kDppXor1>(send.x), dpp_u32<kDppXor1>(send.y)};
            const u32x2 lo = odd ? recv : a, hi = odd ? b : recv;
            const int c16 = (strip + 2 * j + (odd ? 1 : 0)) * kStripCols + (lane >> 1) * 16;
            st_stream16(out_row + c16, u32x4{lo.x, lo.y, hi.x, hi.y});
        }
    } else {
#pragma unroll
        for (int r = 0; r < RPW; ++r) st_stream8(out_row + col + r * kStripCols, convert_piece(v[r], rs.inv[r]));
    }
}

// H = 2048: workgroups below `big` hold four rows, one per wave (four pieces each); every later workgroup holds one row,
// one piece per wave
__global__ __launch_bounds__(kThreads) void swiglu_tail_kernel(const bf16_t *x, int R, int big, uint8_t *out, float *sf, float floor_) {
    constexpr int H = 2048, GPS = kStripCols / 128;
    const int lane = threadIdx.x & 63, wave = wave_id();
    const int wg = blockIdx.x;
    if (wg < big) {
        const int row = wg * kWaves + wave;
        const int col = lane * 8;
        const bf16_t *xr = x + (int64_t)row * (2 * H) + col;
        u32x4 gw[4], uw[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            gw[r] = ld_stream16(xr + r * kStripCols);
            vmem_issue_gap();
            uw[r] = ld_stream16(xr + H + r * kStripCols);
            vmem_issue_gap();
        }
        float v[4][8], amax[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            eval_piece<false>(gw[r], uw[r], v[r]);
            amax[r] = group_allmax<16>(absmax8(v[r]));
        }
        RowScales<448, 4, 16> rs;
        rs.compute(amax, floor_, false, lane);
        if ((lane & 15) < 4) st_stream4(sf + (int64_t)row * (H / 128) + (lane & 15) * GPS + (lane >> 4), f2u(rs.own[0].sf));
#pragma unroll
        for (int r = 0; r < 4; ++r) st_stream8(out + (int64_t)row * H + col + r * kStripCols, convert_piece(v[r], rs.inv[r]));
    } else {
        const int row = big * kWaves + (wg - big);
        const int col = wave * kStripCols + lane * 8;
        const bf16_t *xr = x + (int64_t)row * (2 * H) + col;
        const u32x4 gw = ld_stream16(xr);
        vmem_issue_gap();
        const u32x4 uw = ld_stream16(xr + H);
        float v[8];
        eval_piece<false>(gw, uw, v);
        const float inv = own_scale_store(group_allmax<16>(absmax8(v)), floor_, sf + (int64_t)row * (H / 128), wave * GPS + (lane >> 4), lane);
        st_stream8(out + (int64_t)row * H + col, convert_piece(v, inv));
    }
}

template <int VARIANT, int RPW, int AHEAD = 0>
static hipError_t launch_variant(const void *x, int R, int H, void *out, void *sf, int waves, int param, hipStream_t stream) {
    const int tiles_k = H / (RPW * kStripCols), tiles_m = (R + waves - 1) / waves;
    hipLaunchKernelGGL((swiglu_variant_kernel<VARIANT, RPW, AHEAD>), tile_grid(tiles_k, tiles_m), dim3(64 * waves), 0, stream,
                       static_cast<const bf16_t *>(x), R, H, waves, tiles_k, static_cast<uint8_t *>(out), static_cast<float *>(sf),
                       H / 128, 1e-4f, param);
    return hipGetLastError();
}

}  // namespace tk

using namespace tk;

extern "C" int tk_swiglu_cast_variant(const void *x, int64_t R, int64_t H, void *out, void *sf, int variant, int param,
                                      void *stream) {
    if (R < 0 || H <= 0 || H % 2048 != 0 || R % 8 != 0) return TK_ERR_BAD_SHAPE;
    if (R > (1 << 20) || H > (1 << 20)) return TK_ERR_TOO_LARGE;
    if (R == 0) return TK_OK;
    if (!x || !out || !sf) return TK_ERR_NULL_POINTER;
    if (!aligned_to(x, 16) || !aligned_to(out, 16) || !aligned_to(sf, 4)) return TK_ERR_MISALIGNED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int r = (int)R, h = (int)H;
    const int waves = param == 1 || param == 2 || param == 8 ? param : kWaves;    // variants whose parameter is the workgroup size
    hipError_t e;
    switch (variant) {
        case V_BASE: e = launch_variant<V_BASE, 4>(x, r, h, out, sf, waves, 0, s); break;
        case V_PKFLOOR: e = launch_variant<V_PKFLOOR, 4>(x, r, h, out, sf, waves, 0, s); break;
        case V_WIDEST: e = launch_variant<V_WIDEST, 4>(x, r, h, out, sf, waves, 0, s); break;
        case V_PRIO: e = launch_variant<V_PRIO, 4>(x, r, h, out, sf, waves, 0, s); break;
        case V_PIECESF: e = launch_variant<V_PIECESF, 4>(x, r, h, out, sf, kWaves, 0, s); break;
        case V_LATE:
            if (param < 0) return TK_ERR_BAD_VALUE;
            e = launch_variant<V_LATE, 4>(x, r, h, out, sf, kWaves, param, s);
            break;
        case V_AHEAD:
            if (param == 1) e = launch_variant<V_AHEAD, 4, 1>(x, r, h, out, sf, kWaves, 0, s);
            else if (param == 2) e = launch_variant<V_AHEAD, 4, 2>(x, r, h, out, sf, kWaves, 0, s);
            else return TK_ERR_BAD_VALUE;
            break;
        case V_ROUNDS:
            if (param == 2) e = launch_variant<V_BASE, 2>(x, r, h, out, sf, kWaves, 0, s);
            else if (param == 1) e = launch_variant<V_BASE, 1>(x, r, h, out, sf, kWaves, 0, s);
            else return TK_ERR_BAD_VALUE;
            break;
        case V_TAIL: {
            if (h != 2048 || param < 0 || param > 100) return TK_ERR_BAD_VALUE;
            const int small_rows = (int)((int64_t)r * param / 100) / kWaves * kWaves, big = (r - small_rows) / kWaves;
            hipLaunchKernelGGL(swiglu_tail_kernel, dim3((unsigned)(big + small_rows)), dim3(kThreads), 0, s, static_cast<const bf16_t *>(x), r,
                               big, static_cast<uint8_t *>(out), static_cast<float *>(sf), 1e-4f);
            e = hipGetLastError();
            break;
        }
        default: return TK_ERR_BAD_MODE;
    }
    return (int)e;
}
