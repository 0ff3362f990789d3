// C ABI of the attention library (declared in include/dmf_attn.h): argument
// validation and marshalling into the kernel parameter blocks.  Nothing here
// allocates, frees or synchronises.
#include "../../include/dmf_attn.h"
#include "attn_kernels.h"
#include <algorithm>
#include <cstdio>

namespace {

constexpr int kVersion = (0 << 16) | 1;

bool head_dim_ok(int D) { return D == 32 || D == 64 || D == 72 || D == 80 || D == 96 || D == 128; }

// Validates one tensor's pointer and strides; fills st3 = {sB, sL, sH}.
int check_tensor(const void* ptr, const int64_t* st4, int elem_bytes, int64_t (&st3)[3]) {
  if (ptr == nullptr) return DMF_ATTN_ENULL;
  if (reinterpret_cast<uintptr_t>(ptr) % 16) return DMF_ATTN_EALIGN;
  if (st4[3] != 1) return DMF_ATTN_ESTRIDE;
  for (int i = 0; i < 3; ++i) {
    if (st4[i] < 0 || (st4[i] * elem_bytes) % 16) return DMF_ATTN_ESTRIDE;
    st3[i] = st4[i];
  }
  return DMF_ATTN_OK;
}

int check_common(int B, int H, int Lq, int Lkv, int D, int dtype) {
  if (dtype != DMF_ATTN_F32 && dtype != DMF_ATTN_BF16) return DMF_ATTN_EDTYPE;
  if (!head_dim_ok(D)) return DMF_ATTN_EHEADDIM;
  if (B < 1 || H < 1 || Lq < 1 || Lkv < 1) return DMF_ATTN_ESHAPE;
  const int64_t blocks = (int64_t)B * H * ((std::max(Lq, Lkv) + 127) / 128);
  if (blocks > 0x7fffffffLL) return DMF_ATTN_ESHAPE;
  return DMF_ATTN_OK;
}

}  // namespace

extern "C" {

int dmf_attn_version(void) { return kVersion; }

const char* dmf_attn_strerror(int code) {
  switch (code) {
    case DMF_ATTN_OK: return "ok";
    case DMF_ATTN_EDTYPE: return "unsupported dtype (expected DMF_ATTN_F32 or DMF_ATTN_BF16)";
    case DMF_ATTN_EHEADDIM: return "unsupported head dim (supported: 32, 64, 72, 80, 96, 128)";
    case DMF_ATTN_ESHAPE: return "bad shape (a dimension is < 1 or the grid would overflow)";
    case DMF_ATTN_ESTRIDE: return "bad stride (last-dim stride must be 1, other strides non-negative multiples of 16 bytes)";
    case DMF_ATTN_ENULL: return "a required pointer is NULL";
    case DMF_ATTN_EALIGN: return "a base pointer is not 16-byte aligned";
    case DMF_ATTN_ELAUNCH: return "the HIP runtime rejected the kernel launch";
    case DMF_ATTN_ENOKERNEL: return "no kernel implements this variant for the given shape / dtype";
    case DMF_ATTN_ESCRATCH: return "the problem needs more scratch memory than the library's static buffer holds (use the entry point that takes a workspace)";
    default: return "unknown error code";
  }
}

static_assert(dmf::kNoQNormKernel == DMF_ATTN_ENOKERNEL, "dispatcher code and ABI code must agree");

static int fwd_impl(const void* q, const void* k, const void* v, const void* tq, const void* tk, const void* tv,
                    void* o, void* to, float* lse, float* dlse, const int64_t* strides, bool jvp,
                    int B, int H, int Lq, int Lkv, int D, float scale, int dtype, void* stream,
                    const float* q_gain = nullptr, float q_eps = 0.f, const float* k_gain = nullptr, void* q_hat = nullptr,
                    void* k_hat = nullptr) {
  if (int rc = check_common(B, H, Lq, Lkv, D, dtype)) return rc;
  if (strides == nullptr) return DMF_ATTN_ENULL;
  const int eb = dtype == DMF_ATTN_BF16 ? 2 : 4;
  dmf::FwdParams p{};
  // parameter-block slots: q k v tq tk tv o to
  const void* ptrs[8] = {q, k, v, tq, tk, tv, o, to};
  const int slots_jvp[8] = {0, 1, 2, 3, 4, 5, 6, 7};
  const int slots_fwd[4] = {0, 1, 2, 6};
  const int n = jvp ? 8 : 4;
  // the q-norm entry point always passes the 8-tensor stride table
  const bool wide = jvp || q_gain != nullptr;
  for (int i = 0; i < n; ++i) {
    const int slot = jvp ? slots_jvp[i] : slots_fwd[i];
    if (int rc = check_tensor(ptrs[slot], strides + 4 * (wide ? slot : i), eb, p.st[slot])) return rc;
  }
  if (jvp && lse == nullptr) return DMF_ATTN_ENULL;
  if (lse != nullptr && reinterpret_cast<uintptr_t>(lse) % 4) return DMF_ATTN_EALIGN;
  p.q = q; p.k = k; p.v = v; p.tq = tq; p.tk = tk; p.tv = tv; p.o = o; p.to = to; p.lse = lse; p.dlse = dlse;
  p.H = H; p.Lq = Lq; p.Lkv = Lkv;
  p.scale = scale; p.scale_log2 = scale * 1.4426950408889634f;
  p.q_gain = q_gain; p.q_eps = q_eps;
  p.k_gain = k_gain; p.q_hat = q_hat; p.k_hat = k_hat;
  return dmf::launch_fwd(p, B * H, D, dtype == DMF_ATTN_BF16, jvp, static_cast<hipStream_t>(stream));
}

int dmf_attn_fwd_qnorm(const void* q, const void* k, const void* v, const void* tq, const void* tk, const void* tv,
                       const float* q_gain, float q_eps, void* o, void* to, float* lse, float* dlse,
                       const int64_t* strides, int B, int H, int Lq, int Lkv, int D, float scale, int dtype,
                       void* stream) {
  if (q_gain == nullptr) return DMF_ATTN_ENULL;
  if (reinterpret_cast<uintptr_t>(q_gain) % 16) return DMF_ATTN_EALIGN;
  const bool jvp = to != nullptr;
  if (!jvp) tq = tk = tv = nullptr, dlse = nullptr;
  return fwd_impl(q, k, v, tq, tk, tv, o, to, lse, dlse, strides, jvp, B, H, Lq, Lkv, D, scale, dtype, stream, q_gain,
                  q_eps);
}

int dmf_attn_fwd_qknorm(const void* q, const void* k, const void* v, const void* tq, const void* tk, const void* tv,
                        const float* q_gain, const float* k_gain, float eps, void* o, void* to, float* lse, float* dlse,
                        void* q_hat, void* k_hat, const int64_t* strides, int B, int H, int Lq, int Lkv, int D, float scale,
                        int dtype, void* stream) {
  if (q_gain == nullptr) return DMF_ATTN_ENULL;
  if (k_gain == nullptr) k_hat = nullptr;   // k is taken as given
  if (reinterpret_cast<uintptr_t>(q_gain) % 16 || reinterpret_cast<uintptr_t>(k_gain) % 16 ||
      reinterpret_cast<uintptr_t>(q_hat) % 16 || reinterpret_cast<uintptr_t>(k_hat) % 16)
    return DMF_ATTN_EALIGN;
  const bool jvp = to != nullptr;
  if (!jvp) tq = tk = tv = nullptr, dlse = nullptr;
  return fwd_impl(q, k, v, tq, tk, tv, o, to, lse, dlse, strides, jvp, B, H, Lq, Lkv, D, scale, dtype, stream, q_gain, eps,
                  k_gain, q_hat, k_hat);
}

int dmf_attn_fwd_jvp(const void* q, const void* k, const void* v, const void* tq, const void* tk, const void* tv,
                     void* o, void* to, float* lse, float* dlse, const int64_t* strides,
                     int B, int H, int Lq, int Lkv, int D, float scale, int dtype, void* stream) {
  return fwd_impl(q, k, v, tq, tk, tv, o, to, lse, dlse, strides, true, B, H, Lq, Lkv, D, scale, dtype, stream);
}

int dmf_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse, const int64_t* strides,
                 int B, int H, int Lq, int Lkv, int D, float scale, int dtype, void* stream) {
  return fwd_impl(q, k, v, nullptr, nullptr, nullptr, o, nullptr, lse, nullptr, strides, false, B, H, Lq, Lkv, D, scale, dtype, stream);
}

int dmf_attn_plan(int entry, int B, int H, int Lq, int Lkv, int D, int dtype, char* buf, int buflen) {
  if (int rc = check_common(B, H, Lq, Lkv, D, dtype)) return rc;
  if (buf == nullptr || buflen < 1) return DMF_ATTN_ENULL;
  if (entry < DMF_ATTN_PLAN_FWD || entry > DMF_ATTN_PLAN_FWD_QKNORM_JVP) return DMF_ATTN_ESHAPE;
  const bool bf16 = dtype == DMF_ATTN_BF16;
  const char* t = bf16 ? "__bf16" : "float";
  const size_t n = (size_t)buflen;
  if (entry == DMF_ATTN_PLAN_BWD) {
    if (!(bf16 && dmf::plan_bwd_bf16_fast(Lq, Lkv, D, B * H, buf, n)))
      snprintf(buf, n, "dmf::attn_bwd_dq_kernel<%s, %d> + dmf::attn_bwd_dkv_kernel<%s, %d>", t, D, t, D);
    return DMF_ATTN_OK;
  }
  const bool jvp = entry == DMF_ATTN_PLAN_FWD_JVP || entry == DMF_ATTN_PLAN_FWD_QNORM_JVP || entry == DMF_ATTN_PLAN_FWD_QKNORM_JVP;
  const bool qn = entry >= DMF_ATTN_PLAN_FWD_QNORM_JVP, kn = entry == DMF_ATTN_PLAN_FWD_QKNORM_JVP;
  if (bf16 && dmf::plan_fwd_bf16_fast(Lq, D, jvp, B * H, qn, kn, buf, n)) return DMF_ATTN_OK;
  if (qn) return DMF_ATTN_ENOKERNEL;
  snprintf(buf, n, "dmf::attn_fwd_kernel<%s, %d, %s>", t, D, jvp ? "true" : "false");
  return DMF_ATTN_OK;
}

int dmf_attn_bwd(const void* dout, const void* q, const void* k, const void* v, const void* o, const float* lse,
                 void* dq, void* dk, void* dv, float* delta, const int64_t* strides,
                 int B, int H, int Lq, int Lkv, int D, float scale, int dtype, void* stream) {
  if (int rc = check_common(B, H, Lq, Lkv, D, dtype)) return rc;
  if (strides == nullptr || lse == nullptr || delta == nullptr) return DMF_ATTN_ENULL;
  const int eb = dtype == DMF_ATTN_BF16 ? 2 : 4;
  dmf::BwdParams p{};
  const void* ptrs[8] = {dout, q, k, v, o, dq, dk, dv};
  for (int i = 0; i < 8; ++i)
    if (int rc = check_tensor(ptrs[i], strides + 4 * i, eb, p.st[i])) return rc;
  p.dout = dout; p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse;
  p.dq = dq; p.dk = dk; p.dv = dv; p.delta = delta;
  p.H = H; p.Lq = Lq; p.Lkv = Lkv;
  p.scale = scale; p.scale_log2 = scale * 1.4426950408889634f;
  return dmf::launch_bwd(p, B * H, D, dtype == DMF_ATTN_BF16, static_cast<hipStream_t>(stream));
}

}  // extern "C"
