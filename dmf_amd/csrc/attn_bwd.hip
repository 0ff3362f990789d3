// Backward of the primal attention output for gfx950: dQ, dK, dV from
// (dout, q, k, v, o, lse).  Deterministic, no atomics: two kernels.
//
//   1. attn_bwd_dq_kernel  -- a work-group owns 128 query rows and streams the
//      keys.  Prologue computes delta = rowsum(dout * o) for its rows (and
//      publishes it for kernel 2).  Uses the forward's transposed layout:
//        S^T = K Q^T,  dP^T = V dout^T,  dS^T = P^T * (dP^T - delta),
//        dQ^T += K^T dS^T.
//   2. attn_bwd_dkv_kernel -- a work-group owns 128 key rows and streams the
//      queries; lanes own key columns:
//        S = Q K^T,  dP = dout V^T,  dS = P * (dP - delta),
//        dV^T += dout^T P,  dK^T += Q^T dS.
//
// This is the computation the reference hands to the third-party
// flash-attention backward (models/flash_attention_2_jvp.py:260-276); P is
// recomputed from the saved logsumexp as exp(s*QK^T - lse).
#include "attn_common.h"
#include "attn_kernels.h"

namespace dmf {

// ------------------------------------------------------------------ dQ kernel
template <typename T, int D>
__global__ __launch_bounds__(256) void attn_bwd_dq_kernel(const BwdParams p) {
  using C = Cfg<T, D>;
  constexpr int VEC = C::VEC, VPR = C::VPR, NCHUNK = C::NCHUNK, NDT = C::NDT;
  constexpr int STRIDE = C::STRIDE, BKV = C::BKV, NSUB = C::NSUB, PV_STEPS = C::PV_STEPS;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* Kt = reinterpret_cast<T*>(smem);
  T* Vt = reinterpret_cast<T*>(smem + C::TILE_BYTES);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c32 = lane & 31, g = lane >> 5;
  const uint32_t nqb = (p.Lq + 127) / 128;
  const uint32_t wg = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = wg / nqb, qb = wg % nqb;
  const int b = bh / p.H, h = bh % p.H;
  const int q0 = qb * 128;
  auto base = [&](int t) { return (int64_t)b * p.st[t][0] + (int64_t)h * p.st[t][2]; };

  zero_tile_padding<T, D, BKV>(Kt, tid);
  zero_tile_padding<T, D, BKV>(Vt, tid);

  // ---- per-lane query row: Q, dout chunks; delta from dout and o; lse
  const int qrow = q0 + wave * 32 + c32;
  const bool qok = qrow < p.Lq;
  u32x4 Qr[NCHUNK], dOr[NCHUNK];
  float dpart = 0.f;
  {
    const T* gq = reinterpret_cast<const T*>(p.q) + base(1) + (int64_t)qrow * p.st[1][1];
    const T* gdo = reinterpret_cast<const T*>(p.dout) + base(0) + (int64_t)qrow * p.st[0][1];
    const T* go = reinterpret_cast<const T*>(p.o) + base(4) + (int64_t)qrow * p.st[4][1];
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      const int cv = 2 * c + g;
      const bool in = qok && cv < VPR;
      Qr[c] = in ? *reinterpret_cast<const u32x4*>(gq + cv * VEC) : u32x4{0, 0, 0, 0};
      dOr[c] = in ? *reinterpret_cast<const u32x4*>(gdo + cv * VEC) : u32x4{0, 0, 0, 0};
      const u32x4 ov = in ? *reinterpret_cast<const u32x4*>(go + cv * VEC) : u32x4{0, 0, 0, 0};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if constexpr (C::BF) {
          // bf16 -> fp32 is a 16-bit shift
          dpart += __uint_as_float(dOr[c][e] << 16) * __uint_as_float(ov[e] << 16);
          dpart += __uint_as_float(dOr[c][e] & 0xffff0000u) * __uint_as_float(ov[e] & 0xffff0000u);
        } else {
          dpart += __uint_as_float(dOr[c][e]) * __uint_as_float(ov[e]);
        }
      }
    }
  }
  const float delta = xhalf_sum(dpart);
  float lse2 = INFINITY;   // log2-domain logsumexp; +inf switches padded rows off
  if (qok) {
    lse2 = p.lse[(int64_t)bh * p.Lq + qrow] * kLog2e;
    if (g == 0) p.delta[(int64_t)bh * p.Lq + qrow] = delta;
  }

  f32x16 dQ[NDT];
#pragma unroll
  for (int t = 0; t < NDT; ++t) dQ[t] = f32x16{0};
  const float c2 = p.scale_log2;

  TileStream<T, D, BKV, 2> stream;
  const T* gsrc[2] = {reinterpret_cast<const T*>(p.k) + base(2), reinterpret_cast<const T*>(p.v) + base(3)};
  const int64_t gstride[2] = {p.st[2][1], p.st[3][1]};
  T* ldst[2] = {Kt, Vt};

  const int ntiles = (p.Lkv + BKV - 1) / BKV;
  stream.issue(gsrc, gstride, 0, p.Lkv, tid);
  for (int it = 0; it < ntiles; ++it) {
    const int kv0 = it * BKV;
    __syncthreads();
    stream.commit(ldst, tid);
    __syncthreads();
    if (it + 1 < ntiles) stream.issue(gsrc, gstride, kv0 + BKV, p.Lkv, tid);

#pragma unroll
    for (int s = 0; s < NSUB; ++s) {
      f32x16 S = {0}, dP = {0};
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c) {
        mma_chunk<T>(S, lds_row_chunk<T, STRIDE>(Kt, s * 32 + c32, c, g), Qr[c]);
        mma_chunk<T>(dP, lds_row_chunk<T, STRIDE>(Vt, s * 32 + c32, c, g), dOr[c]);
      }
      f32x16 dS;
      const bool tail = kv0 + BKV > p.Lkv;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float pr = fast_exp2(fmaf(S[i], c2, -lse2));
        if (tail && kv0 + s * 32 + acc_row(i, g) >= p.Lkv) pr = 0.f;
        dS[i] = pr * (dP[i] - delta);
      }
#pragma unroll
      for (int st = 0; st < PV_STEPS; ++st) {
        const ColOperand ds = acc_operand<T>(dS, st);
#pragma unroll
        for (int t = 0; t < NDT; ++t)
          mma_col<T>(dQ[t], lds_col_operand<T, STRIDE>(Kt, s * 32, t * 32, st, lane), ds);
      }
    }
  }

  store_rows_transposed<T, D>(reinterpret_cast<T*>(smem), reinterpret_cast<T*>(p.dq) + base(5), p.st[5][1], q0, p.Lq, tid,
                              [&](int t, int i) { return dQ[t][i] * p.scale; });
}

// --------------------------------------------------------------- dK/dV kernel
template <typename T, int D>
__global__ __launch_bounds__(256) void attn_bwd_dkv_kernel(const BwdParams p) {
  using C = Cfg<T, D>;
  constexpr int VEC = C::VEC, VPR = C::VPR, NCHUNK = C::NCHUNK, NDT = C::NDT;
  constexpr int STRIDE = C::STRIDE, BQ = C::BKV, NSUB = C::NSUB, PV_STEPS = C::PV_STEPS;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* Qt = reinterpret_cast<T*>(smem);
  T* dOt = reinterpret_cast<T*>(smem + C::TILE_BYTES);
  float* rowstat = reinterpret_cast<float*>(smem + 2 * C::TILE_BYTES + 512);   // [2][BQ]: lse2, delta

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c32 = lane & 31, g = lane >> 5;
  const uint32_t nkb = (p.Lkv + 127) / 128;
  const uint32_t wg = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = wg / nkb, kb = wg % nkb;
  const int b = bh / p.H, h = bh % p.H;
  const int k0 = kb * 128;
  auto base = [&](int t) { return (int64_t)b * p.st[t][0] + (int64_t)h * p.st[t][2]; };

  zero_tile_padding<T, D, BQ>(Qt, tid);
  zero_tile_padding<T, D, BQ>(dOt, tid);

  // ---- per-lane key row: K and V operand chunks stay in registers
  u32x4 Kr[NCHUNK], Vr[NCHUNK];
  {
    const int krow = k0 + wave * 32 + c32;
    const bool ok = krow < p.Lkv;
    const T* gk = reinterpret_cast<const T*>(p.k) + base(2) + (int64_t)krow * p.st[2][1];
    const T* gv = reinterpret_cast<const T*>(p.v) + base(3) + (int64_t)krow * p.st[3][1];
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      const int cv = 2 * c + g;
      const bool in = ok && cv < VPR;
      Kr[c] = in ? *reinterpret_cast<const u32x4*>(gk + cv * VEC) : u32x4{0, 0, 0, 0};
      Vr[c] = in ? *reinterpret_cast<const u32x4*>(gv + cv * VEC) : u32x4{0, 0, 0, 0};
    }
  }

  f32x16 dK[NDT], dV[NDT];
#pragma unroll
  for (int t = 0; t < NDT; ++t) {
    dK[t] = f32x16{0};
    dV[t] = f32x16{0};
  }
  const float c2 = p.scale_log2;

  TileStream<T, D, BQ, 2> stream;
  const T* gsrc[2] = {reinterpret_cast<const T*>(p.q) + base(1), reinterpret_cast<const T*>(p.dout) + base(0)};
  const int64_t gstride[2] = {p.st[1][1], p.st[0][1]};
  T* ldst[2] = {Qt, dOt};
  const float* glse = p.lse + (int64_t)bh * p.Lq;
  const float* gdelta = p.delta + (int64_t)bh * p.Lq;

  const int ntiles = (p.Lq + BQ - 1) / BQ;
  stream.issue(gsrc, gstride, 0, p.Lq, tid);
  float stat_pre = 0.f;
  auto issue_stats = [&](int r0) {
    if (tid < 2 * BQ) {
      const int r = r0 + (tid % BQ);
      if (tid < BQ) stat_pre = r < p.Lq ? glse[r] * kLog2e : INFINITY;   // +inf => P = 0 for padded query rows
      else stat_pre = r < p.Lq ? gdelta[r] : 0.f;
    }
  };
  issue_stats(0);
  for (int it = 0; it < ntiles; ++it) {
    const int r0 = it * BQ;
    __syncthreads();
    stream.commit(ldst, tid);
    if (tid < 2 * BQ) rowstat[tid] = stat_pre;
    __syncthreads();
    if (it + 1 < ntiles) {
      stream.issue(gsrc, gstride, r0 + BQ, p.Lq, tid);
      issue_stats(r0 + BQ);
    }

#pragma unroll
    for (int s = 0; s < NSUB; ++s) {
      f32x16 S = {0}, dP = {0};
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c) {
        mma_chunk<T>(S, lds_row_chunk<T, STRIDE>(Qt, s * 32 + c32, c, g), Kr[c]);
        mma_chunk<T>(dP, lds_row_chunk<T, STRIDE>(dOt, s * 32 + c32, c, g), Vr[c]);
      }
      f32x16 P, dS;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(rowstat + s * 32 + j * 8 + 4 * g);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(rowstat + BQ + s * 32 + j * 8 + 4 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int i = 4 * j + e;
          P[i] = fast_exp2(fmaf(S[i], c2, -l4[e]));
          dS[i] = P[i] * (dP[i] - d4[e]);
        }
      }
#pragma unroll
      for (int st = 0; st < PV_STEPS; ++st) {
        const ColOperand pp = acc_operand<T>(P, st);
        const ColOperand ds = acc_operand<T>(dS, st);
#pragma unroll
        for (int t = 0; t < NDT; ++t) {
          mma_col<T>(dV[t], lds_col_operand<T, STRIDE>(dOt, s * 32, t * 32, st, lane), pp);
          mma_col<T>(dK[t], lds_col_operand<T, STRIDE>(Qt, s * 32, t * 32, st, lane), ds);
        }
      }
    }
  }

  T* stage = reinterpret_cast<T*>(smem);
  store_rows_transposed<T, D>(stage, reinterpret_cast<T*>(p.dk) + base(6), p.st[6][1], k0, p.Lkv, tid,
                              [&](int t, int i) { return dK[t][i] * p.scale; });
  store_rows_transposed<T, D>(stage, reinterpret_cast<T*>(p.dv) + base(7), p.st[7][1], k0, p.Lkv, tid,
                              [&](int t, int i) { return dV[t][i]; });
}

template <typename T, int D>
static int launch_bwd_t(const BwdParams& p, int BH, hipStream_t stream) {
  using C = Cfg<T, D>;
  constexpr int tiles = 2 * C::TILE_BYTES + 512 + 2 * C::BKV * 4;
  constexpr int stage = 128 * C::OROWV * 16;
  constexpr int smem = tiles > stage ? tiles : stage;
  auto k1 = attn_bwd_dq_kernel<T, D>;
  auto k2 = attn_bwd_dkv_kernel<T, D>;
  static bool lds_ok1[64] = {}, lds_ok2[64] = {};
  if (!ensure_dynamic_lds(k1, smem, lds_ok1) || !ensure_dynamic_lds(k2, smem, lds_ok2)) return -7;
  const uint32_t nqb = (p.Lq + 127) / 128, nkb = (p.Lkv + 127) / 128;
  if (int rc = launch_kernel(k1, dim3(nqb * (uint32_t)BH), dim3(256), smem, stream, p)) return rc;
  return launch_kernel(k2, dim3(nkb * (uint32_t)BH), dim3(256), smem, stream, p);
}

template <typename T>
static int launch_bwd_d(const BwdParams& p, int BH, int D, hipStream_t stream) {
  switch (D) {
    case 32: return launch_bwd_t<T, 32>(p, BH, stream);
    case 64: return launch_bwd_t<T, 64>(p, BH, stream);
    case 72: return launch_bwd_t<T, 72>(p, BH, stream);
    case 80: return launch_bwd_t<T, 80>(p, BH, stream);
    case 96: return launch_bwd_t<T, 96>(p, BH, stream);
    case 128: return launch_bwd_t<T, 128>(p, BH, stream);
    default: return -2;
  }
}

int launch_bwd_generic(const BwdParams& p, int BH, int D, bool bf16, hipStream_t stream) {
  return bf16 ? launch_bwd_d<__bf16>(p, BH, D, stream) : launch_bwd_d<float>(p, BH, D, stream);
}

int launch_bwd(const BwdParams& p, int BH, int D, bool bf16, hipStream_t stream) {
  if (bf16) {
    const int rc = launch_bwd_bf16_fast(p, BH, D, stream);
    if (rc != 1) return rc;   // 1 = no tuned kernel for this shape
  }
  return launch_bwd_generic(p, BH, D, bf16, stream);
}

}  // namespace dmf
