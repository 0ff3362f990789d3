/*
 * dmf_attn.h -- C ABI of the MI355X (gfx950) forward-mode attention library.
 *
 * This is the boundary a host binds instead of the reference's kernel-side
 * FFI for the attention path:
 *   - the Triton launches `_attn_fwd_dual[_split][grid](...)`
 *     (models/flash_attention_2_jvp.py:196-230, = flash_attention_3_jvp.py:183-217),
 *   - `flash_attn_2_cuda.fwd` / `torch.ops.flash_attn_3.fwd`
 *     (models/flash_attention_2_jvp.py:47-61, flash_attention_3_jvp.py:72-107),
 *   - `flash_attn_2_cuda.bwd` / `torch.ops.flash_attn_3.bwd`
 *     (models/flash_attention_2_jvp.py:119-139, flash_attention_3_jvp.py:136-159).
 *
 * Conventions shared by every entry point
 *   - Tensors are logical (B, L, H, D) arrays, exactly the layout of
 *     `attn_op` (models/layers.py:93-94).  Each tensor comes with four
 *     element strides {stride_B, stride_L, stride_H, stride_D}; stride_D must
 *     be 1 and every (b, l, h) row must start on a 16-byte boundary, which
 *     holds for contiguous tensors and for the q/k/v views into a packed
 *     (B, L, 3, H, D) qkv buffer (models/layers.py:143-147).
 *   - `strides` is a flat int64 array of n_tensors*4 entries in the order the
 *     tensor pointers appear in the signature (outputs included, lse/delta
 *     excluded: those are dense (B, H, Lq) fp32).
 *   - `dtype`: DMF_ATTN_F32 (fp32 in/out, fp32 MFMA products) or
 *     DMF_ATTN_BF16 (bf16 in/out, bf16 MFMA, fp32 accumulation and softmax).
 *   - `lse` is the natural-log logsumexp of the scaled scores
 *     (models/triton_utils.py:347).
 *   - Ownership: the caller allocates every buffer; the library neither
 *     allocates nor frees device memory and keeps no state between calls.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *     Launches are asynchronous; nothing synchronises the host.  Entry points
 *     are re-entrant.
 *   - Return value: DMF_ATTN_OK or a negative DMF_ATTN_E* code; no kernel is
 *     launched on error.  The reference performs no such validation (a
 *     sequence shorter than its 128-row tile silently yields an
 *     uninitialised output, flash_attention_2_jvp.py:192-193).
 *   - Supported head dims: 32, 64, 72, 80, 96, 128.  Any Lq, Lkv >= 1.
 */
#ifndef DMF_ATTN_H
#define DMF_ATTN_H

#include <stdint.h>

/* Exported symbol (the library is built with hidden default visibility). */
#define DMF_ATTN_API __attribute__((visibility("default")))

#ifdef __cplusplus
extern "C" {
#endif

enum { DMF_ATTN_F32 = 0, DMF_ATTN_BF16 = 1 };

enum {
  DMF_ATTN_OK = 0,
  DMF_ATTN_EDTYPE = -1,    /* dtype is not DMF_ATTN_F32 / DMF_ATTN_BF16        */
  DMF_ATTN_EHEADDIM = -2,  /* head dim not in the supported set                 */
  DMF_ATTN_ESHAPE = -3,    /* a dimension is < 1 or B*H exceeds the grid limit  */
  DMF_ATTN_ESTRIDE = -4,   /* last-dim stride != 1 or a stride breaks alignment */
  DMF_ATTN_ENULL = -5,     /* a required pointer is NULL                        */
  DMF_ATTN_EALIGN = -6,    /* a base pointer is not 16-byte aligned             */
  DMF_ATTN_ELAUNCH = -7,   /* the HIP runtime rejected the launch               */
  DMF_ATTN_ENOKERNEL = -8, /* no kernel implements this variant for the given shape / dtype; nothing was launched */
  DMF_ATTN_ESCRATCH = -9   /* the problem needs more scratch memory than the library's static buffer holds        */
};

/* Library version, (major << 16) | minor. */
DMF_ATTN_API int dmf_attn_version(void);

/* Static, human-readable text for a return code. */
DMF_ATTN_API const char* dmf_attn_strerror(int code);

/*
 * Fused forward + JVP, one streaming online-softmax pass:
 *   O  = softmax(s Q K^T) V
 *   dO = dP V + P dV,  dP = P * (dS - rowsum(P * dS)),  dS = s (dQ K^T + Q dK^T)
 * Replaces the `_attn_fwd_dual` / `_attn_fwd_dual_split` launches
 * (models/flash_attention_2_jvp.py:196-230; kernels models/triton_utils.py:258-500).
 * strides: 8 tensors {q, k, v, tq, tk, tv, o, to}.  lse: (B, H, Lq) fp32.
 * dlse: optional (may be NULL) (B, H, Lq) fp32 output, the tangent of lse,
 * which is rowsum(P * dS) -- the kernel's running `mu` (triton_utils.py:113).
 */
DMF_ATTN_API int dmf_attn_fwd_jvp(const void* q, const void* k, const void* v,
                     const void* tq, const void* tk, const void* tv,
                     void* o, void* to, float* lse, float* dlse,
                     const int64_t* strides,
                     int B, int H, int Lq, int Lkv, int D,
                     float scale, int dtype, void* stream);

/*
 * Primal-only forward (no tangents).  Replaces `flash_attn_2_cuda.fwd` as
 * called at models/flash_attention_2_jvp.py:233-243 (dropout 0, non-causal,
 * no window / softcap / alibi).  strides: 4 tensors {q, k, v, o}.
 * lse may be NULL when the caller does not need it (no-grad inference).
 */
DMF_ATTN_API int dmf_attn_fwd(const void* q, const void* k, const void* v,
                 void* o, float* lse,
                 const int64_t* strides,
                 int B, int H, int Lq, int Lkv, int D,
                 float scale, int dtype, void* stream);

/*
 * Forward (+ JVP when `to` is given) with the per-head RMS norm of q folded into
 * the kernel's Q load, so that normalised q (and its tangent) never travel
 * through HBM:
 *   r = rsqrt(mean_d(q^2) + q_eps),  q_hat = q r gain,
 *   tq_hat = (tq r + q dr) gain,  dr = -r^3 mean_d(q tq),
 * then attention on (q_hat, k, v) and tangents (tq_hat, tk, tv) as above; q_hat
 * and tq_hat are rounded to `dtype` before use, like the outputs of
 * dmf_rmsnorm_fwd (dmf_block.h).  Replaces `q = self.q_norm(q)` together with
 * the attention call that follows it (models/layers.py:148-151); k is read as
 * given (already normalised: each k row is shared by every q row, so its norm
 * stays a separate pass).  q_gain: (D) fp32, 16-byte aligned.
 * strides: 8 tensors {q, k, v, tq, tk, tv, o, to}; with to == NULL (primal
 * only) tq, tk, tv, dlse and their strides are ignored and lse may be NULL.
 * Only the tuned bf16 kernels implement this variant: DMF_ATTN_ENOKERNEL is
 * returned (and nothing launched) for fp32 or for a shape they do not cover --
 * the caller then normalises q itself and calls dmf_attn_fwd[_jvp].
 */
DMF_ATTN_API int dmf_attn_fwd_qnorm(const void* q, const void* k, const void* v,
                     const void* tq, const void* tk, const void* tv,
                     const float* q_gain, float q_eps,
                     void* o, void* to, float* lse, float* dlse,
                     const int64_t* strides,
                     int B, int H, int Lq, int Lkv, int D,
                     float scale, int dtype, void* stream);

/*
 * The same with the per-head RMS norm of k folded in as well -- the whole of
 * `q, k = self.q_norm(q), self.k_norm(k); x = self.attn(q, k, v)`
 * (models/layers.py:147-151) as one launch on the raw projections.  Every key
 * tile is normalised (primal and tangent, same formulas with k_gain and the same
 * eps, rounded to `dtype`) in on-chip memory between its arrival and its use;
 * a work-group does this for the tiles it consumes, so a head's keys are
 * normalised once per 256 query rows.
 * q_hat, k_hat: optional contiguous (B, L, H, D) outputs of `dtype` (16-byte
 * aligned) that receive the normalised primal rows -- what dmf_attn_bwd and
 * dmf_rmsnorm_bwd need later -- or NULL when no backward pass follows.
 * k_gain == NULL: k is read as given (already normalised) and k_hat is ignored,
 * i.e. dmf_attn_fwd_qnorm with the q_hat output.
 * Same strides table, optional arguments and DMF_ATTN_ENOKERNEL behaviour as
 * dmf_attn_fwd_qnorm.
 */
DMF_ATTN_API int dmf_attn_fwd_qknorm(const void* q, const void* k, const void* v,
                     const void* tq, const void* tk, const void* tv,
                     const float* q_gain, const float* k_gain, float eps,
                     void* o, void* to, float* lse, float* dlse,
                     void* q_hat, void* k_hat,
                     const int64_t* strides,
                     int B, int H, int Lq, int Lkv, int D,
                     float scale, int dtype, void* stream);

/*
 * Backward on the primal output: dQ, dK, dV from (dout, q, k, v, o, lse).
 * Replaces `flash_attn_2_cuda.bwd` as called at
 * models/flash_attention_2_jvp.py:262-275.  Deterministic (no atomics).
 * strides: 8 tensors {dout, q, k, v, o, dq, dk, dv}.
 * delta: caller-provided (B, H, Lq) fp32 workspace; on return it holds
 * rowsum(dout * o), the `softmax_d` the reference's backward returns.
 */
DMF_ATTN_API int dmf_attn_bwd(const void* dout, const void* q, const void* k, const void* v,
                 const void* o, const float* lse,
                 void* dq, void* dk, void* dv, float* delta,
                 const int64_t* strides,
                 int B, int H, int Lq, int Lkv, int D,
                 float scale, int dtype, void* stream);

/*
 * Host-only query: which kernel(s) a call of an entry point would launch for a
 * shape on the current device, written to `buf` (NUL-terminated, truncated to
 * buflen) in the spelling profilers print, e.g.
 * "dmf::attn_fwd_bf16_kernel<72, true, 8, false, false>"; the two kernels of
 * the backward pair are joined by " + ".  Launches nothing and reads no device
 * memory; the answer depends on the device's compute-unit count (work-group
 * width and single-pass-vs-pair policies) and assumes rows less than 2 GiB
 * apart.  No counterpart in the reference (its dispatch is the Python branch
 * at models/flash_attention_2_jvp.py:190-191); meant for tests and benchmarks
 * that must name the kernel they exercised.  DMF_ATTN_ENOKERNEL for a
 * q-norm / qk-norm entry that no tuned kernel covers.
 */
enum {
  DMF_ATTN_PLAN_FWD = 0,            /* dmf_attn_fwd                                  */
  DMF_ATTN_PLAN_FWD_JVP = 1,        /* dmf_attn_fwd_jvp                              */
  DMF_ATTN_PLAN_BWD = 2,            /* dmf_attn_bwd                                  */
  DMF_ATTN_PLAN_FWD_QNORM_JVP = 3,  /* dmf_attn_fwd_qnorm / _qknorm without k_gain   */
  DMF_ATTN_PLAN_FWD_QKNORM_JVP = 4  /* dmf_attn_fwd_qknorm with k_gain, with tangents */
};
DMF_ATTN_API int dmf_attn_plan(int entry, int B, int H, int Lq, int Lkv, int D, int dtype,
                  char* buf, int buflen);

#ifdef __cplusplus
}
#endif
#endif /* DMF_ATTN_H */
