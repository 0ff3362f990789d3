// Kernel parameter blocks and launcher prototypes shared between the C-ABI
// translation unit and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dmf {

// Strides are in elements: st[t] = {stride_B, stride_L, stride_H}; the head-dim
// stride is 1 by contract.
struct FwdParams {
  const void *q, *k, *v, *tq, *tk, *tv;
  void *o, *to;
  float* lse;               // (B, H, Lq) or nullptr
  float* dlse;              // (B, H, Lq) or nullptr: tangent of lse (JVP kernels only)
  int64_t st[8][3];         // q, k, v, tq, tk, tv, o, to
  int H, Lq, Lkv;
  float scale, scale_log2;  // softmax scale and scale * log2(e)
  // Optional per-head RMS norm of q (and of its tangent) folded into the kernel's Q load: gain (D) fp32, or
  // nullptr.  Only the tuned bf16 kernels implement it; the dispatcher reports kNoQNormKernel otherwise.
  const float* q_gain;
  float q_eps;
  // Optional per-head RMS norm of k (and of its tangent) applied to every key tile once it has landed in LDS: gain (D)
  // fp32 or nullptr (needs q_gain; same eps).  q_hat / k_hat: optional contiguous (B, L, H, D) outputs that receive the
  // normalised primal rows (what a backward pass needs), or nullptr.
  const float* k_gain;
  void *q_hat, *k_hat;
};

constexpr int kNoQNormKernel = -8;

struct BwdParams {
  const void *dout, *q, *k, *v, *o;
  const float* lse;         // (B, H, Lq)
  void *dq, *dk, *dv;
  float* delta;             // (B, H, Lq): written by the dQ kernel, read by the dK/dV kernel
  int64_t st[8][3];         // dout, q, k, v, o, dq, dk, dv
  int H, Lq, Lkv;
  float scale, scale_log2;
};

// Opt a kernel in to `bytes` of dynamic LDS on the current device.  The attribute is per device, so the
// "already done" flag is kept per (kernel instantiation, device); a race between two host threads at worst
// repeats the idempotent call.
template <typename K>
inline bool ensure_dynamic_lds(K kernel, int bytes, bool (&done)[64]) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
  if (!done[dev]) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return false;
    done[dev] = true;
  }
  return true;
}


// Compute units of the current device (asked once per device; 256 if the query fails).
inline int compute_units() {
  static int cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    cached[dev] = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0 ? n : 256;
  }
  return cached[dev];
}

// Launch `kernel(params)` and return 0 or -7 (DMF_ATTN_ELAUNCH).  The status is the one hipLaunchKernel returns for
// this launch.  An error left behind by somebody else's earlier call is neither reported as a failure of this library
// nor hidden from its owner: the process-wide "last error" is only read -- and thereby cleared -- when this very launch
// failed, so that the failure the caller already gets as a return code is not raised a second time by the next
// unrelated check of the runtime's error state.
template <typename P>
inline int launch_kernel(void (*kernel)(P), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream, P params) {
  void* args[] = {&params};
  if (hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, args, lds_bytes, stream) == hipSuccess) return 0;
  (void)hipGetLastError();
  return -7;
}

// Return 0 or a negative DMF_ATTN_E* code.
int launch_fwd(const FwdParams& p, int BH, int D, bool bf16, bool jvp, hipStream_t stream);
// Building blocks of launch_fwd: the generic kernels (fp32 and bf16, any length)
// and the tuned bf16 kernels (returns 1 when it has no kernel for the case).
int launch_fwd_generic(const FwdParams& p, int BH, int D, bool bf16, bool jvp, hipStream_t stream);
int launch_fwd_bf16_fast(const FwdParams& p, int BH, int D, bool jvp, hipStream_t stream);
int launch_bwd_generic(const BwdParams& p, int BH, int D, bool bf16, hipStream_t stream);
int launch_bwd_bf16_fast(const BwdParams& p, int BH, int D, hipStream_t stream);
int launch_bwd(const BwdParams& p, int BH, int D, bool bf16, hipStream_t stream);

// Host-only: the tuned kernel(s) the two *_bf16_fast launchers pick for a case, written to buf as profilers spell them
// ("dmf::attn_fwd_bf16_kernel<72, true, 8, false, false>", the backward pair joined by " + "), for rows less than
// 2 GiB apart.  Returns false when there is no tuned kernel (the generic ones run).
bool plan_fwd_bf16_fast(int Lq, int D, bool jvp, int BH, bool q_norm, bool k_norm, char* buf, size_t n);
bool plan_bwd_bf16_fast(int Lq, int Lkv, int D, int BH, char* buf, size_t n);

}  // namespace dmf
