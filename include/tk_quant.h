/*
 * tk_quant.h -- C ABI of libtk_quant.so: FP8 E4M3 / FP4 E2M1 block-scaled casts and the fused
 * SwiGLU + per-token FP8 quantisation for AMD MI355X (gfx950).
 *
 * The reference exposes this path as Python functions only (there is no FFI in it); each entry
 * point below is what a binding for one of those functions would call, and names the function
 * it stands behind.
 *
 * Conventions (all entry points):
 *   - plain pointers and sizes; every data pointer is DEVICE memory owned by the caller;
 *   - the call validates its arguments on the host, enqueues kernels on `stream` (a hipStream_t,
 *     NULL = the default stream) and returns without synchronising;
 *   - it never allocates, frees or copies memory;
 *   - return value: 0 = enqueued, < 0 = an argument was rejected and nothing was launched
 *     (tk_status below), > 0 = a hipError_t reported by the launch;
 *   - M == 0 (R == 0) is valid and launches nothing;
 *   - every tk_check_* twin runs the same validation and launches nothing, so error handling can
 *     be exercised on a machine without a GPU.
 *
 * Scale-factor ("sf") storage, selected by `sf_layout`; (m, k) is the block's row / column index,
 * nm x nk the number of blocks:
 *   TK_SF_ROW_F32    fp32, element (m, k) at sf[m * sf_ld + k]
 *   TK_SF_COL_F32    fp32, element (m, k) at sf[k * sf_ld + m]         (sf_ld >= nm)
 *   TK_SF_COL_UE8M0  one biased-exponent byte per block, at
 *                    ((uint8_t*)sf)[(k / 4) * sf_ld + 4 * m + (k % 4)]  (sf_ld in BYTES, >= 4 * nm, a
 *                    multiple of 4: the storage is an array of 4-byte words, 4-byte aligned);
 *                    needs round_sf = 1.  In cast modes the bytes of a partly filled last word
 *                    (k >= nk) are written as 0.
 * (reference: get_sf_shape / store_sf / load_sf, tile_kernels/quant/common.py:130-138, 219-244).
 */
#ifndef TK_QUANT_H
#define TK_QUANT_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TK_QUANT_VERSION 110 /* major*10000 + minor*100 + patch */

enum tk_dtype { TK_BF16 = 0, TK_F32 = 1, TK_OUT_E4M3 = 2 /* output of tk_reduce_fused only */ };
enum tk_fmt { TK_E4M3 = 0, TK_E2M1 = 1, TK_E5M6 = 2 };
enum tk_sf_layout { TK_SF_ROW_F32 = 0, TK_SF_COL_F32 = 1, TK_SF_COL_UE8M0 = 2 };
enum tk_mode {
    TK_CAST_AND_SF = 0, /* write codes and scales                                  */
    TK_SF_ONLY = 1,     /* write scales only (`out` may be NULL)                   */
    TK_CAST_GIVEN_SF = 2 /* read scales from `sf`, write codes (quant = x * (1/sf), clamped) */
};

enum tk_status {
    TK_OK = 0,
    TK_ERR_NULL_POINTER = -1,
    TK_ERR_BAD_SHAPE = -2,    /* negative size, K not a multiple of what the format needs, ... */
    TK_ERR_BAD_DTYPE = -3,
    TK_ERR_BAD_FORMAT = -4,
    TK_ERR_BAD_GROUP = -5,    /* group / block size not supported                          */
    TK_ERR_BAD_LAYOUT = -6,   /* sf_layout unknown or not allowed with this mode / round_sf */
    TK_ERR_BAD_MODE = -7,
    TK_ERR_BAD_STRIDE = -8,   /* row stride or sf_ld too small                              */
    TK_ERR_MISALIGNED = -9,   /* pointer or stride not aligned for 16-byte vector access    */
    TK_ERR_TOO_LARGE = -10,   /* more than 2^31-1 rows, columns or blocks                   */
    TK_ERR_BAD_VALUE = -11    /* clamp / floor value not usable                             */
};

/*
 * Per-token cast: every row of x[M, K] is cut into groups of `group` consecutive columns (the
 * last one may be partial); each group gets one scale.
 *   amax = max(max|x|, floor)   floor = 1e-4 (E4M3) or 6*2^-126 (E2M1)
 *   sf   = amax / QMAX          QMAX  = 448 or 6;  with round_sf: sf = 2^ceil(log2 sf)
 *   code = cvt(x * inv)         inv = QMAX / amax, or 1 / sf with round_sf
 * Stands behind tile_kernels.quant.per_token_cast, per_token_cast_with_sf_only and
 * per_token_cast_with_precomputed_sf (tile_kernels/quant/per_token_cast_kernel.py:223-302).
 *
 *   x            bf16 or fp32, unit column stride, `x_row_stride` elements between rows
 *   out          E4M3: M*K bytes;  E2M1: M*K/2 bytes, element 2t in the low nibble of byte t
 *   group        16, 32, 64, 128, or K (one scale per row; needs K % 64 == 0 and TK_CAST_AND_SF)
 *   requirements K % 8 == 0; x and x_row_stride 16-byte aligned; out 8-byte aligned
 *
 * fmt = TK_E5M6 (tile_kernels/quant/per_token_cast_to_e5m6_kernel.py:10-70, 172-215): a 12-bit float, the top
 * 12 bits of an IEEE fp16 (sign, 5 exponent bits, 6 mantissa bits), QMAX = 65024, floor = 1e-4, one scale per
 * row (group == K, any K % 8 == 0, TK_CAST_AND_SF only).  code = the fp16 of x * inv rounded toward zero, cut
 * to 12 bits and incremented when (kept lsb) + (low 17 bits of the fp32 pattern of x * inv) > 0x10000: round
 * to nearest even for |x * inv| >= 2^-14.  out: M * K * 3/2 bytes; codes c0..c7 of eight consecutive elements
 * form a 96-bit string, c0 in the most significant bits, stored as three 32-bit words, high word first.
 */
int tk_per_token_cast(const void *x, int x_dtype, int64_t M, int64_t K, int64_t x_row_stride, void *out,
                      void *sf, int64_t sf_ld, int fmt, int group, int sf_layout, int round_sf, int mode,
                      void *stream);
int tk_check_per_token_cast(const void *x, int x_dtype, int64_t M, int64_t K, int64_t x_row_stride,
                            const void *out, const void *sf, int64_t sf_ld, int fmt, int group, int sf_layout,
                            int round_sf, int mode);

/*
 * Per-token cast of an input that is itself quantised: x holds E4M3 bytes [M, K] or packed E2M1
 * bytes [M, K/2] (K, x_row_stride in logical elements) with one dequantisation scale per
 * x_bm x x_bk block in x_sf (any of the three layouts; UE8M0 bytes decode to 2^(e-127)).
 * Every element is first dequantised, value = code * scale (one fp32 rounding), then cast as above.
 * Stands behind tile_kernels.quant.per_token_cast(x=(data, sf), x_block_size=...) 
 * (tile_kernels/quant/per_token_cast_kernel.py:87-126, tile_kernels/quant/common.py:62-88; oracle
 * tile_kernels/torch/cast.py:87-99).  Cast-and-scale mode only, group in {16, 32, 64, 128}.
 *   requirements K % 8 == 0, x_row_stride % 8 == 0, x_bk % 8 == 0; x 8-byte (E4M3) / 4-byte (E2M1) aligned
 */
int tk_per_token_cast_quantized(const void *x, int x_fmt, int64_t M, int64_t K, int64_t x_row_stride,
                                const void *x_sf, int64_t x_sf_ld, int x_sf_layout, int x_bm, int x_bk, void *out,
                                void *sf, int64_t sf_ld, int fmt, int group, int sf_layout, int round_sf,
                                void *stream);
int tk_check_per_token_cast_quantized(const void *x, int x_fmt, int64_t M, int64_t K, int64_t x_row_stride,
                                      const void *x_sf, int64_t x_sf_ld, int x_sf_layout, int x_bm, int x_bk,
                                      const void *out, const void *sf, int64_t sf_ld, int fmt, int group,
                                      int sf_layout, int round_sf);

/*
 * Per-block cast: x[M, K] contiguous is cut into bm x bk blocks (bm, bk in {32, 128}; edge blocks
 * may be partial); one scale per block, same arithmetic as above.
 * Stands behind tile_kernels.quant.per_block_cast, per_block_cast_with_sf_only and
 * per_block_cast_with_precomputed_sf (tile_kernels/quant/per_block_cast_kernel.py:205-276).
 *   requirements K % 64 == 0; x 16-byte aligned; TK_CAST_GIVEN_SF only with TK_SF_ROW_F32
 */
int tk_per_block_cast(const void *x, int x_dtype, int64_t M, int64_t K, void *out, void *sf, int64_t sf_ld,
                      int fmt, int bm, int bk, int sf_layout, int round_sf, int mode, void *stream);
int tk_check_per_block_cast(const void *x, int x_dtype, int64_t M, int64_t K, const void *out, const void *sf,
                            int64_t sf_ld, int fmt, int bm, int bk, int sf_layout, int round_sf, int mode);

/*
 * Fused SwiGLU + per-token E4M3 quantisation of x[R, 2H] (contiguous; gate = columns [0, H),
 * up = columns [H, 2H)):
 *   g, u in fp32; with use_clamp: g = min(g, clamp), u = min(max(u, -clamp), clamp)
 *   v = g / (1 + exp(-g)) * u  [* topk_weights[pos_to_token_topk[r]], 0 where the index is < 0]
 *   then the per-token cast above over v with groups of `group` (128 or H) columns.
 * Stands behind tile_kernels.quant.swiglu_forward_and_per_token_cast
 * (tile_kernels/quant/swiglu_forward_and_per_token_cast_kernel.py:175-260).
 *
 *   sf_clamp_min        amax floor; < 0 selects the default 1e-4
 *   pos_to_token_topk   NULL, or int32[R] index into topk_weights (flat, `num_weights` entries)
 *   pos_to_expert       NULL, or int32[R]; rows with a negative entry are padding: their codes and
 *                       scales are written as zeros (the reference leaves them unwritten)
 *   clamped_count       NULL, or int64[3] incremented by {#g > clamp, #u > clamp, #u < -clamp} over
 *                       the non-padding rows, counted before clamping (needs use_clamp)
 *   max_blocks          with clamped_count: > 0 caps the number of workgroups, which then loop over tiles
 *                       (the reference's num_sms knob for the counting variant: every workgroup that clamped
 *                       anything sends one atomic request to the counters, and requests to one line are served
 *                       one at a time; the Python wrapper passes 8 per compute unit); <= 0 or without
 *                       clamped_count: one workgroup per tile
 *   requirements        H % 128 == 0; group == 128, or group == H with TK_SF_ROW_F32; x 16-byte aligned;
 *                       a row of x (2 H elements) shorter than 4 GiB (TK_ERR_TOO_LARGE otherwise)
 */
int tk_swiglu_per_token_cast(const void *x, int x_dtype, int64_t R, int64_t H, void *out, void *sf, int64_t sf_ld,
                             int group, int sf_layout, int round_sf, float sf_clamp_min,
                             const int32_t *pos_to_token_topk, const float *topk_weights, int64_t num_weights,
                             const int32_t *pos_to_expert, int use_clamp, float clamp, int64_t *clamped_count,
                             int max_blocks, void *stream);
int tk_check_swiglu_per_token_cast(const void *x, int x_dtype, int64_t R, int64_t H, const void *out, const void *sf,
                                   int64_t sf_ld, int group, int sf_layout, int round_sf, float sf_clamp_min,
                                   const int32_t *pos_to_token_topk, const float *topk_weights, int64_t num_weights,
                                   const int32_t *pos_to_expert, int use_clamp, float clamp,
                                   const int64_t *clamped_count);

/*
 * Fused SwiGLU backward + per-token E4M3 quantisation of the input gradient.  x is the forward input as
 * it was quantised: E4M3 codes [R, 2H] (gate = columns [0, H), up = [H, 2H)) with fp32 scales
 * x_sf[R, 2H/group], both contiguous.  In fp32, with g = code * sf, u likewise, go = grad_out:
 *   use_clamp: g = min(g, clamp), u = min(max(u, -clamp), clamp); the gradient of a clamped value is 0
 *   d = 1 + exp(-g), s = 1 / d, act = g / d * u, w = topk_weights[pos_to_token_topk[r]] (0 where < 0)
 *   out         [R, H]  bf16 = act * w
 *   x_grad      [R, 2H] bf16 = [ go*w*s * u * fma(g, 1 - s, 1) | go*w*s * g ]
 *   x_grad_codes[R, 2H] E4M3 with x_grad_sf[R, 2H/group] fp32 (row-major): the per-token cast of the
 *                       fp32 gradient over groups of `group` columns (round_sf as in tk_per_token_cast)
 *   weight_grad [num_weights] fp32 = sum over the row of go * act at index pos_to_token_topk[r] >= 0,
 *                       and 0 at every index i with token_topk_to_pos[i] < 0
 * Stands behind tile_kernels.quant.swiglu_backward_and_per_token_cast
 * (tile_kernels/quant/swiglu_backward_and_per_token_cast_kernel.py:166-244).
 *   requirements        group in {32, 128}; H % group == 0; grad_out, out, x_grad 16-byte aligned,
 *                       x and x_grad_codes 8-byte aligned; num_weights = num_tokens * num_topk
 */
int tk_swiglu_backward_per_token_cast(const void *x, const float *x_sf, int64_t R, int64_t H, int group,
                                      const void *grad_out, const float *topk_weights, const int32_t *pos_to_token_topk,
                                      const int32_t *token_topk_to_pos, int64_t num_weights, void *out,
                                      void *x_grad_codes, float *x_grad_sf, void *x_grad, float *weight_grad,
                                      int round_sf, int use_clamp, float clamp, void *stream);
int tk_check_swiglu_backward_per_token_cast(const void *x, const float *x_sf, int64_t R, int64_t H, int group,
                                            const void *grad_out, const float *topk_weights,
                                            const int32_t *pos_to_token_topk, const int32_t *token_topk_to_pos,
                                            int64_t num_weights, const void *out, const void *x_grad_codes,
                                            const float *x_grad_sf, const void *x_grad, const float *weight_grad,
                                            int round_sf, int use_clamp, float clamp);

/*
 * Per-channel cast: E4M3 with one scale per `num_per_tokens` (32 or 128) tokens x 1 column, scales fp32
 * row-major out_sf[ceil(M / num_per_tokens), K].  The input is
 *   x_sf == NULL, swiglu == 0 : bf16 x[num_tokens, K]; fp32 too when transpose == 0 (the reference's
 *                               transposing and SwiGLU forms take bf16 only)
 *   x_sf != NULL              : E4M3 codes x[num_tokens, K] with fp32 scales x_sf[num_tokens, K / 128]
 *                               (1 x 128 groups); every element is first dequantised, code * scale
 *   swiglu != 0               : bf16 x[num_tokens, 2K]; the value cast is bf16(g / (1 + exp(-g)) * u) with
 *                               g = x[:, :K], u = x[:, K:], clamped as in tk_swiglu_per_token_cast with use_clamp
 * pos_to_token (NULL, or int32[M]) gathers rows: output row r comes from input row pos_to_token[r], a
 * negative index gives a row of zeros; without it M rows are taken in order (num_tokens >= M).  A gather needs
 * num_tokens >= 1 (TK_ERR_BAD_SHAPE otherwise).
 * transpose == 0: out[M, K];  transpose != 0: out[K, M].
 * Stands behind tile_kernels.quant.per_channel_cast, per_channel_cast_fused
 * (tile_kernels/quant/per_channel_cast_fused_kernel.py:130-203), per_channel_cast_and_transpose
 * (per_channel_cast_and_transpose_kernel.py:84-123) and swiglu_forward_and_per_channel_cast_and_transpose
 * (swiglu_forward_and_per_channel_cast_and_transpose_kernel.py:178-231).
 *   requirements K % 8 == 0 (K % 128 == 0 with x_sf); M % 16 == 0; x 16-byte (codes: 8-byte) aligned;
 *                out 8-byte, transposed 16-byte aligned
 */
int tk_per_channel_cast(const void *x, int x_dtype, const float *x_sf, int64_t num_tokens, int64_t K,
                        const int32_t *pos_to_token, int64_t M, void *out, float *out_sf, int num_per_tokens, int round_sf,
                        int transpose, int swiglu, int use_clamp, float clamp, void *stream);
int tk_check_per_channel_cast(const void *x, int x_dtype, const float *x_sf, int64_t num_tokens, int64_t K,
                              const int32_t *pos_to_token, int64_t M, const void *out, const float *out_sf,
                              int num_per_tokens, int round_sf, int transpose, int swiglu, int use_clamp, float clamp);

/*
 * Weighted reduction of expanded rows back to tokens (the inverse of tk_expand_to_fused):
 *   out[t, :] = round( sf * sum_k  x[pos, :] * (topk_weights[t, k] * x_sf[pos]) ),   pos = token_topk_to_pos[t, k] >= 0
 * accumulated in fp32 with one fused multiply-add per term, k ascending; topk_weights, x_sf ([num_expanded]
 * fp32) and sf (one fp32 on the device) may each be NULL (factor 1).  x: bf16 or fp32 [num_expanded, hidden],
 * contiguous; out: the type of x, or E4M3 bytes with out_dtype = TK_OUT_E4M3.  Positions outside [0, num_expanded) are
 * skipped; with num_expanded == 0 (x may then be NULL) the result is zeros.  The E4M3 conversion does not saturate: a
 * scaled sum beyond +-448 becomes NaN (0x7F / 0xFF), as torch's conversion in the reference's statement of the operator does.
 * Stands behind tile_kernels.moe.reduce_fused (tile_kernels/moe/reduce_fused_kernel.py:70-135; oracle
 * tile_kernels/torch/reduce_fused.py:14-72).
 *   requirements hidden % 8 == 0; x and out 16-byte (E4M3 out: 8-byte) aligned
 */
int tk_reduce_fused(const void *x, int x_dtype, int64_t num_expanded, int64_t hidden, const float *x_sf,
                    const float *topk_weights, const int32_t *token_topk_to_pos, int64_t num_tokens, int num_topk, void *out,
                    int out_dtype, const float *sf, void *stream);
int tk_check_reduce_fused(const void *x, int x_dtype, int64_t num_expanded, int64_t hidden, const float *x_sf,
                          const float *topk_weights, const int32_t *token_topk_to_pos, int64_t num_tokens, int num_topk,
                          const void *out, int out_dtype, const float *sf);

/*
 * Lossless re-blocking of FP4 into FP8: x holds packed E2M1 bytes [M, K/2] (contiguous) with one power-of-two
 * scale per x_bm x x_bk block in x_sf (any layout; of an fp32 scale only the exponent is used); out receives
 * E4M3 bytes [M, K] with one power-of-two scale per out_bm x out_bk block:
 *   e_out = max(exponent of x_sf over the input blocks inside the output block) - 6, not below 0
 *   out   = code * 2^(e_in - e_out)   (exact while the input exponents of an output block span at most 11)
 *   out_sf = 2^(e_out - 127) as fp32, or the byte e_out in the packed layout
 * so that out * out_sf == x * x_sf for every element.
 * Stands behind tile_kernels.quant.per_block_cast_lossless
 * (tile_kernels/quant/per_block_cast_lossless_kernel.py:150-209).
 *   requirements K % 8 == 0; x_bk % 8 == 0; out_bm and out_bk divide 128 and are multiples of x_bm and x_bk;
 *                x 4-byte, out 8-byte aligned
 */
int tk_per_block_cast_lossless(const void *x, int64_t M, int64_t K, const void *x_sf, int64_t x_sf_ld, int x_sf_layout,
                               int x_bm, int x_bk, void *out, void *out_sf, int64_t out_sf_ld, int out_sf_layout,
                               int out_bm, int out_bk, void *stream);
int tk_check_per_block_cast_lossless(const void *x, int64_t M, int64_t K, const void *x_sf, int64_t x_sf_ld,
                                     int x_sf_layout, int x_bm, int x_bk, const void *out, const void *out_sf,
                                     int64_t out_sf_ld, int out_sf_layout, int out_bm, int out_bk);

/*
 * Dequantisation: out[m, k] = float(code[m, k]) * sf[m / bm, k / bk] (one fp32 product), stored as
 * fp32 or rounded to bf16 (nearest even).  x: E4M3 bytes [M, K], packed E2M1 bytes [M, K/2] or packed E5M6
 * words [M, K*3/2 bytes] (layout as written by tk_per_token_cast), contiguous (K in logical elements); x_sf in
 * any of the three layouts.
 * Stands behind tile_kernels.quant.cast_back and per_token_cast_back
 * (tile_kernels/quant/cast_back_kernel.py:77-143, cast_back_e5m6_kernel.py:12-41, 141-176).
 *   requirements K % 8 == 0; bk 1, 2, 4 (per-channel scales) or a multiple of 8; out 16-byte aligned;
 *                x 8-byte (E4M3) / 4-byte (E2M1, E5M6) aligned
 */
int tk_cast_back(const void *x, int x_fmt, int64_t M, int64_t K, const void *x_sf, int64_t x_sf_ld, int x_sf_layout,
                 int bm, int bk, void *out, int out_dtype, void *stream);
int tk_check_cast_back(const void *x, int x_fmt, int64_t M, int64_t K, const void *x_sf, int64_t x_sf_ld,
                       int x_sf_layout, int bm, int bk, const void *out, int out_dtype);

/*
 * Expert-major MoE layout (the step before the fused SwiGLU op in an MoE layer).
 *
 * tk_get_fused_mapping: stable counting sort of the flat (token, k) list by expert id (entries < 0 are
 * skipped); expert e occupies positions [expert_start[e], expert_end[e]), its length padded to a
 * multiple of `alignment`.  Outputs (int32): pos_to_expert / pos_to_token / pos_to_token_topk
 * [num_expanded] (-1 on padding), token_topk_to_pos [num_tokens * num_topk] (-1 where skipped),
 * expert_start / expert_end / num_tokens_per_expert [num_experts] (padded lengths).  Positions
 * inside an expert follow the flat index.  `workspace` is caller-provided scratch of at least
 * tk_fused_mapping_workspace_bytes() bytes; positions >= num_expanded are not written.
 * Stands behind tile_kernels.moe.get_fused_mapping (tile_kernels/moe/get_fused_mapping_kernel.py:166-250).
 *   requirements num_experts <= 1024
 */
int64_t tk_fused_mapping_workspace_bytes(int64_t num_tokens, int num_topk, int num_experts);
int tk_get_fused_mapping(const int64_t *topk_idx, int64_t num_tokens, int num_topk, int num_experts, int alignment,
                         int64_t num_expanded, int32_t *pos_to_expert, int32_t *pos_to_token, int32_t *pos_to_token_topk,
                         int32_t *token_topk_to_pos, int32_t *expert_start, int32_t *expert_end,
                         int32_t *num_tokens_per_expert, void *workspace, int64_t workspace_bytes, void *stream);
int tk_check_get_fused_mapping(const int64_t *topk_idx, int64_t num_tokens, int num_topk, int num_experts, int alignment,
                               int64_t num_expanded, const int32_t *pos_to_expert, const int32_t *pos_to_token,
                               const int32_t *pos_to_token_topk, const int32_t *token_topk_to_pos,
                               const int32_t *expert_start, const int32_t *expert_end,
                               const int32_t *num_tokens_per_expert, const void *workspace, int64_t workspace_bytes);

/*
 * tk_get_fused_mapping_static: tk_get_fused_mapping without the workspace argument, for callers that cannot
 * allocate device memory or carry a workspace around (code under HIP graph capture, tight serving loops,
 * harnesses that forbid allocation).  It has no counterpart in the reference.  The slice x expert table lives
 * in a device array of TK_FUSED_MAPPING_STATIC_BYTES bytes that the library holds on every GPU it runs on until
 * the process ends; the call allocates and frees nothing.  Inputs whose table would not fit
 * (tk_fused_mapping_workspace_bytes() > TK_FUSED_MAPPING_STATIC_BYTES, i.e. more than 1 Mi (token, k) pairs at
 * 256 experts) are rejected with TK_ERR_TOO_LARGE.  Same outputs, bit for bit, as tk_get_fused_mapping.
 * All calls on one GPU share that GPU's table: calls that overlap there (two streams, two threads) race.
 * The first call on a device looks up the array's address and should happen outside graph capture.
 */
#define TK_FUSED_MAPPING_STATIC_BYTES (4 << 20)
int tk_get_fused_mapping_static(const int64_t *topk_idx, int64_t num_tokens, int num_topk, int num_experts, int alignment,
                                int64_t num_expanded, int32_t *pos_to_expert, int32_t *pos_to_token,
                                int32_t *pos_to_token_topk, int32_t *token_topk_to_pos, int32_t *expert_start,
                                int32_t *expert_end, int32_t *num_tokens_per_expert, void *stream);

/*
 * tk_expand_to_fused: row t of x (row_bytes bytes, any element type) is copied to every position
 * token_topk_to_pos[t * num_topk + k] >= 0; rows with pos_to_expert < 0 are zero-filled.  With
 * x_sf != NULL the token's `sf_cols` 4-byte scale words (contiguous rows) are expanded the same way
 * into out_sf: row-major (word (p, j) at out_sf[p * out_sf_ld + j]) or column-major
 * (out_sf[j * out_sf_ld + p]).
 * Stands behind tile_kernels.moe.expand_to_fused and expand_to_fused_with_sf
 * (tile_kernels/moe/expand_to_fused_kernel.py:94-200).
 *   requirements row_bytes % 16 == 0; x, out 16-byte aligned
 */
int tk_expand_to_fused(const void *x, int64_t num_tokens, int64_t row_bytes, const int32_t *token_topk_to_pos, int num_topk,
                       const int32_t *pos_to_expert, int64_t num_expanded, void *out, const void *x_sf, int sf_cols,
                       void *out_sf, int64_t out_sf_ld, int sf_col_major, void *stream);
int tk_check_expand_to_fused(const void *x, int64_t num_tokens, int64_t row_bytes, const int32_t *token_topk_to_pos,
                             int num_topk, const int32_t *pos_to_expert, int64_t num_expanded, const void *out,
                             const void *x_sf, int sf_cols, const void *out_sf, int64_t out_sf_ld, int sf_col_major);

/*
 * tk_stream_floor: measurement aid with no counterpart in the reference.  A kernel with the memory traffic of the
 * cast kernels (the same streaming 16-byte loads of a bf16 matrix, one byte written per element with the same
 * write-through 8-byte stores, one 4-byte word per 128 columns if sf != NULL) and no arithmetic; with two_halves the
 * input has 2 * cols columns and both halves are read per output element, as by tk_swiglu_per_token_cast.  bench.py
 * times it beside the real operators: what it takes is what the access pattern costs on the machine.
 *   requirements cols % 1024 == 0; x 16-byte, out 8-byte aligned
 */
int tk_stream_floor(const void *x, int64_t rows, int64_t cols, int two_halves, void *out, void *sf, void *stream);

/*
 * tk_stream_floor_timeline: the same kernel reporting where and when each of its waves ran (no counterpart in the
 * reference; bench.py --timeline reads it).  stamps receives tk_stream_floor_stamp_words(rows, cols) 64-bit words, six
 * per wave in row order: the 100 MHz real-time counter at the wave's start, when its last load has arrived (this variant
 * waits for all loads before its first store), when its stores are issued and when they are acknowledged, then the
 * HW_ID and XCC_ID hardware registers.
 *   requirements as tk_stream_floor; stamps 8-byte aligned
 */
int tk_stream_floor_timeline(const void *x, int64_t rows, int64_t cols, int two_halves, void *out, void *sf, void *stamps,
                             void *stream);
int64_t tk_stream_floor_stamp_words(int64_t rows, int64_t cols);

/*
 * tk_stream_floor_tailed: the traffic-only kernel on a launch that ends in smaller waves, as tk_swiglu_per_token_cast
 * arranges its launches of about one to three occupancy rounds (measurement aid, no counterpart in the reference): the
 * last rows_one rows are read and written by four waves of one 512-column piece each, the rows_two rows before them by
 * two waves of two pieces, the others by one wave of four pieces per 2048 columns.  Same output as tk_stream_floor.
 *   requirements cols % 2048 == 0; rows, rows_two, rows_one multiples of 4; x 16-byte, out 8-byte aligned
 */
int tk_stream_floor_tailed(const void *x, int64_t rows, int64_t cols, int two_halves, void *out, void *sf, int64_t rows_two,
                           int64_t rows_one, void *stream);

/*
 * tk_stream_floor_flat: the traffic-only kernel for any ratio of bytes read to bytes written (measurement aid, no
 * counterpart in the reference; bench_ops.py times it beside the operators around the path).  The input is a flat range of
 * in_bytes bytes; a lane reads in_bytes_per_lane (16, 8 or 4) bytes per piece of 64 lanes and writes out_bytes_per_lane
 * (16, 8, 4 or 0) bytes per piece to the flat output; a wave takes pieces_per_wave (1, 2, 4 or 8) consecutive pieces, all
 * its loads issued before its first store.  What is written is an XOR fold of what was read.
 *   requirements in_bytes % (64 * in_bytes_per_lane) == 0; in and out 16-byte aligned
 */
int tk_stream_floor_flat(const void *in, int64_t in_bytes, int in_bytes_per_lane, void *out, int out_bytes_per_lane,
                         int pieces_per_wave, void *stream);

/*
 * tk_swiglu_cast_variant: measurement aid with no counterpart in the reference.  Alternative structures of the kernel
 * behind tk_swiglu_per_token_cast for its plain case (bf16 x[R, 2H], E4M3 codes, row-major fp32 1 x 128 scales, no mask,
 * weights or clamp), each producing the same codes and scales bit for bit; bench.py --variant times them beside the
 * product kernel, which is how the figures quoted for them can be measured again.  variant / param:
 *   0 the product's structure (param: rows per workgroup 1, 2, 4 or 8; 0 = 4)      4 a scale division per piece and lane,
 *   1 the gate's -88 cap on packed bf16 pairs (param as 0)                           each piece stored once converted
 *   2 16-byte code stores after a lane-pair exchange (param as 0)                  5 variant 4 for waves whose first piece
 *   3 wave priority raised once the first piece has arrived (param as 0)             arrives later than param * 10 ns
 *   6 pieces requested param (1, 2) ahead instead of all at once                   7 param (1, 2) pieces per wave, not 4
 *   8 the last param per cent of the rows as four one-piece waves each (H = 2048)
 *   requirements H % 2048 == 0, R % 8 == 0; x and out 16-byte aligned
 */
int tk_swiglu_cast_variant(const void *x, int64_t R, int64_t H, void *out, void *sf, int variant, int param, void *stream);

/* Text for a tk_status value (or "hip error" for positive codes). Never NULL. */
const char *tk_strerror(int status);
/* TK_QUANT_VERSION the library was built from. */
int tk_version(void);

#ifdef __cplusplus
}
#endif
#endif /* TK_QUANT_H */
