/*
 * dmf_block.h -- C ABI of the fused transformer-block glue kernels (gfx950)
 * that sit either side of the attention operator in a DiT block, each with an
 * optional forward-mode tangent stream computed in the same pass.
 *
 * Under `torch.func.jvp` (loss.py:165-170) the reference runs these pieces as
 * strings of separate primal + tangent elementwise / reduction kernels:
 *   - `modulate(norm(x), shift, scale)`   models/layers.py:28-29, 198, 200, 218-219
 *   - `x + gate * branch`                  models/layers.py:198, 200
 *   - `GELU(approximate="tanh")`           models/layers.py:162
 *   - `RMSNorm` on q and k                 models/layers.py:33-42, 148
 *   - `SiLU` of the conditioning vector    models/layers.py:185-188, 211-214
 * Every entry point below replaces one such string by a single HBM pass.
 *
 * Conventions
 *   - (B, L, C) activations are dense and row-major; per-sample modulation
 *     vectors (shift / scale / gate and their tangents) are (B, C) with unit
 *     channel stride and a caller-given batch stride in elements (they are
 *     chunks of one (B, 6C) adaLN output, models/layers.py:197).
 *   - dtype codes, return codes and `dmf_attn_strerror` are those of
 *     dmf_attn.h.  All arithmetic is fp32; results are rounded once on store.
 *   - A NULL tangent *input* means "zero tangent".  A NULL tangent *output*
 *     selects the primal-only kernel.
 *   - C (and the head dim D of the RMSNorm entry points) must be a multiple of
 *     8; C <= 2048, D <= 128; base pointers and batch strides must keep every
 *     row 16-byte aligned.
 *   - The caller owns all memory (including the fp32 `workspace` of the
 *     backward entry points, sized by dmf_block_workspace_floats); launches are
 *     asynchronous on `stream` (hipStream_t as void*, NULL = default stream);
 *     entry points are re-entrant.  The backward reductions are two-stage sums
 *     in a fixed order (no atomics): results are run-to-run deterministic.
 */
#ifndef DMF_BLOCK_H
#define DMF_BLOCK_H

#include "dmf_attn.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Number of fp32 workspace elements a backward entry point needs.
 * `which`: 0 = dmf_ln_modulate_bwd, 1 = dmf_gate_residual_bwd (rows = B*L, dim = C),
 *          2 = dmf_rmsnorm_bwd (dim = D; B, L ignored), 3 = dmf_colsum (rows = B*L, dim = C).
 * Returns 0 on bad input. */
DMF_ATTN_API int64_t dmf_block_workspace_floats(int which, int B, int L, int dim);

/*
 * y = LayerNorm(x) * (1 + scale) + shift, LayerNorm over C without affine
 * parameters (biased variance, `eps` inside the square root), and -- when `ty`
 * is given -- its tangent along (tx, tshift, tscale):
 *   xh = (x - mean) * rstd,  dxh = rstd * (tx - mean(tx) - xh * mean(xh * tx)),
 *   ty = dxh * (1 + scale) + xh * tscale + tshift.
 * Replaces `modulate(self.norm1(x), shift_msa, scale_msa)` and its norm2 /
 * norm_final twins (models/layers.py:198, 200, 219).
 * x, tx: (B, L, C) of x_dtype.  shift, scale, tshift, tscale: (B, C) of
 * mod_dtype with batch strides mod_strides[0..3] (in that order).  y, ty:
 * (B, L, C) of y_dtype.
 */
DMF_ATTN_API int dmf_ln_modulate_fwd(const void* x, const void* tx, const void* shift, const void* scale,
                                     const void* tshift, const void* tscale, void* y, void* ty,
                                     const int64_t* mod_strides, int B, int L, int C, float eps,
                                     int x_dtype, int mod_dtype, int y_dtype, void* stream);

/*
 * Backward of the primal of dmf_ln_modulate_fwd: given gy = dLoss/dy,
 *   gx     = gres + rstd * (g - mean(g) - xh * mean(g * xh)),  g = gy * (1 + scale)
 *   gshift = sum_l gy,   gscale = sum_l gy * xh.
 * gres (x_dtype, may be NULL = 0) is the gradient that reaches x from its other
 * consumers (the residual path), added here instead of by a separate kernel.
 * gx: (B, L, C) of x_dtype; gshift, gscale: dense (B, C) of mod_dtype.
 */
DMF_ATTN_API int dmf_ln_modulate_bwd(const void* gy, const void* x, const void* scale, const void* gres, void* gx,
                                     void* gshift, void* gscale, float* workspace, int64_t scale_stride, int B, int L, int C,
                                     float eps, int x_dtype, int mod_dtype, int gy_dtype, void* stream);

/*
 * y = x + gate * h and, when `ty` is given, ty = tx + tgate * h + gate * th.
 * Replaces `x + gate_msa * self.attn(...)` / `x + gate_mlp * self.mlp(...)`
 * (models/layers.py:198, 200).  x, tx, y, ty: (B, L, C) of x_dtype; h, th:
 * (B, L, C) of h_dtype; gate, tgate: (B, C) of mod_dtype with batch strides
 * gate_strides[0..1].
 */
DMF_ATTN_API int dmf_gate_residual_fwd(const void* x, const void* tx, const void* gate, const void* tgate,
                                       const void* h, const void* th, void* y, void* ty,
                                       const int64_t* gate_strides, int B, int L, int C,
                                       int x_dtype, int mod_dtype, int h_dtype, void* stream);

/*
 * Backward of the primal of dmf_gate_residual_fwd (dLoss/dx is gy itself and
 * needs no kernel): gh = gate * gy ((B, L, C) of h_dtype), ggate = sum_l gy * h
 * (dense (B, C) of mod_dtype).  gy: (B, L, C) of gy_dtype.
 */
DMF_ATTN_API int dmf_gate_residual_bwd(const void* gy, const void* gate, const void* h, void* gh, void* ggate,
                                       float* workspace, int64_t gate_stride, int B, int L, int C,
                                       int gy_dtype, int mod_dtype, int h_dtype, void* stream);

/*
 * The gated residual and the LayerNorm + modulate that consumes its result, in
 * one pass over the residual stream (`x = x + gate_msa * attn(...)` followed by
 * `modulate(self.norm2(x), shift_mlp, scale_mlp)`, models/layers.py:198-200, and
 * likewise across the block boundary, :200 -> next block's :198, or :219):
 *   y = x + gate * h,  z = LayerNorm(y) * (1 + scale) + shift,
 * with ty, tz as in the two separate entry points when ty and tz are given
 * (both or neither).  x, tx, y, ty: x_dtype; h, th: h_dtype; z, tz: z_dtype;
 * gate, tgate, shift, scale, tshift, tscale: (B, C) of mod_dtype with batch
 * strides mod_strides[0..5] in that order.
 */
DMF_ATTN_API int dmf_residual_ln_modulate_fwd(const void* x, const void* tx, const void* gate, const void* tgate,
                                              const void* h, const void* th, const void* shift, const void* scale,
                                              const void* tshift, const void* tscale, void* y, void* ty, void* z,
                                              void* tz, const int64_t* mod_strides, int B, int L, int C, float eps,
                                              int x_dtype, int mod_dtype, int h_dtype, int z_dtype, void* stream);

/* Backward of dmf_residual_ln_modulate_fwd = dmf_ln_modulate_bwd (with the gradient of y from its other
 * consumers passed as `gres`) followed by dmf_gate_residual_bwd on its result. */

/*
 * y = 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) over n elements and,
 * when `ty` is given, ty = gelu'(x) * tx.  Replaces `self.act(...)` of the MLP
 * (models/layers.py:162, 166).  n must be a multiple of 8.
 */
DMF_ATTN_API int dmf_gelu_tanh_fwd(const void* x, const void* tx, void* y, void* ty, int64_t n, int dtype,
                                   void* stream);

/* gx = gelu'(x) * gy over n elements (n a multiple of 8). */
DMF_ATTN_API int dmf_gelu_tanh_bwd(const void* gy, const void* x, void* gx, int64_t n, int dtype, void* stream);

/*
 * y = x * sigmoid(x) over n elements (n a multiple of 8) and, when `ty` is
 * given, ty = silu'(x) * tx with silu'(x) = s (1 + x (1 - s)), s = sigmoid(x).
 * Replaces the `nn.SiLU()` in front of every adaLN projection
 * (models/layers.py:185-188, 211-214).  x, tx: x_dtype; y, ty: y_dtype (the
 * conditioning vector is fp32 while the projection that follows wants bf16).
 */
DMF_ATTN_API int dmf_silu_fwd(const void* x, const void* tx, void* y, void* ty, int64_t n, int x_dtype, int y_dtype,
                              void* stream);

/* gx = silu'(x) * gy over n elements; gy: gy_dtype, x and gx: x_dtype. */
DMF_ATTN_API int dmf_silu_bwd(const void* gy, const void* x, void* gx, int64_t n, int x_dtype, int gy_dtype,
                              void* stream);

/*
 * Per-head RMS norm over D of a logical (B, L, H, D) tensor:
 *   r = rsqrt(mean(x^2) + eps),  y = x * r * gain,
 *   ty = (tx * r + x * dr) * gain,  dr = -r^3 * mean(x * tx)   (when `ty` is given).
 * Replaces `self.q_norm(q)` / `self.k_norm(k)` (models/layers.py:33-42, 148).
 * x and tx carry four element strides each ({sB, sL, sH, 1}; views into a
 * packed qkv buffer qualify, models/layers.py:143-147): strides = {x[4], tx[4]}.
 * y, ty: dense (B, L, H, D) of `dtype`.  gain: (D) of gain_dtype.
 */
DMF_ATTN_API int dmf_rmsnorm_fwd(const void* x, const void* tx, const void* gain, void* y, void* ty,
                                 const int64_t* strides, int B, int L, int H, int D, float eps,
                                 int dtype, int gain_dtype, void* stream);

/*
 * Backward of the primal of dmf_rmsnorm_fwd:
 *   g = gy * gain,  gx = r * g - x * r^3 * mean(x * g),  ggain = sum_rows gy * x * r.
 * x and gx: strided as above (strides = {x[4], gx[4]}; gx may be one slot of a
 * packed (B, L, 3, H, D) gradient buffer); gy: dense (B, L, H, D); ggain: (D) of
 * gain_dtype.
 */
DMF_ATTN_API int dmf_rmsnorm_bwd(const void* gy, const void* x, const void* gain, void* gx, void* ggain,
                                 float* workspace, const int64_t* strides, int B, int L, int H, int D, float eps,
                                 int dtype, int gain_dtype, void* stream);

/*
 * out[c] = sum_r x[r][c] for a dense (rows, C) matrix, C a multiple of 8: the
 * bias gradient of a Linear layer (the `grad_output.sum(0)` of torch's
 * `linear_backward`, reached from models/layers.py:131,137,161-165) as a
 * fixed-order two-stage sum, safe to record into a HIP graph.
 */
DMF_ATTN_API int dmf_colsum(const void* x, void* out, float* workspace, int64_t rows, int C, int x_dtype,
                            int out_dtype, void* stream);

/*
 * dmf_colsum without a workspace argument and without any allocation: the
 * partial sums of the first stage are kept in a file-scope device array inside
 * the library (DMF_COLSUM_STATIC_MAX_FLOATS fp32 values = 4 MiB, held by every
 * GPU the library runs on until the process ends).  This entry point has no
 * counterpart in the reference; it exists for callers that cannot allocate --
 * code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc -- and calls no hipMalloc / hipFree or allocating library routine.
 * Same kernels and the same bits as dmf_colsum.
 *   - Limit: ceil(rows / 64) * C <= DMF_COLSUM_STATIC_MAX_FLOATS, otherwise
 *     DMF_ATTN_ESCRATCH is returned and nothing is launched (e.g. 8192 x 4608
 *     or 32768 x 1152 fit; use dmf_colsum with your own workspace beyond).
 *   - All calls on one GPU share that GPU's array: two calls that overlap in
 *     time on the same GPU (different streams, or host threads launching
 *     concurrently) race on it.  Calls ordered on one stream are safe, and
 *     nothing needs clearing between them (every partial sum a call reads was
 *     written by that call).
 */
#define DMF_COLSUM_STATIC_MAX_FLOATS (1 << 20)
DMF_ATTN_API int dmf_colsum_static(const void* x, void* out, int64_t rows, int C, int x_dtype, int out_dtype,
                                   void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DMF_BLOCK_H */
