// Fused attention forward (+ optional JVP) for gfx950: one streaming
// online-softmax pass over the keys with unnormalised accumulators.
//
// Work decomposition: a work-group of 4 waves owns 128 query rows of one
// (batch, head); each wave owns 32 of them and keeps, per lane, everything of
// query column c32 = lane&31 -- scores are produced TRANSPOSED,
//     S^T[kv, q] = K[kv, :] . Q[q, :],
// so that the softmax reductions over kv are in-lane (plus one lane^32
// exchange), the rescale factors are per-lane scalars, and the probability
// tile P^T feeds the P*V product as the MFMA B operand without leaving
// registers.  O and dO are accumulated transposed as well (O^T[d, q]) and are
// transposed back through LDS for a coalesced store.
//
// Quantities follow models/triton_utils.py:92-118 of the reference (S, dS,
// P*dS, mu = rowsum(P*dS), lse = m + log l) but the accumulators are kept
// unnormalised and divided once in the epilogue.
#include "attn_common.h"
#include "attn_kernels.h"

namespace dmf {

template <typename T, int D, bool JVP>
__global__ __launch_bounds__(256) void attn_fwd_kernel(const FwdParams p) {
  using C = Cfg<T, D>;
  constexpr int VEC = C::VEC, VPR = C::VPR, NCHUNK = C::NCHUNK, NDT = C::NDT;
  constexpr int STRIDE = C::STRIDE, BKV = C::BKV, NSUB = C::NSUB, PV_STEPS = C::PV_STEPS;
  constexpr int NT = JVP ? 4 : 2;                       // tensors streamed per KV tile: K, V [, dK, dV]

  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* Kt = reinterpret_cast<T*>(smem);
  T* Vt = reinterpret_cast<T*>(smem + C::TILE_BYTES);
  T* dKt = reinterpret_cast<T*>(smem + 2 * C::TILE_BYTES);
  T* dVt = reinterpret_cast<T*>(smem + 3 * C::TILE_BYTES);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c32 = lane & 31, g = lane >> 5;

  const uint32_t nqb = (p.Lq + 127) / 128;
  const uint32_t wg = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = wg / nqb, qb = wg % nqb;
  const int b = bh / p.H, h = bh % p.H;
  const int q0 = qb * 128;

  auto base = [&](int t) { return (int64_t)b * p.st[t][0] + (int64_t)h * p.st[t][2]; };
  const T* gq = reinterpret_cast<const T*>(p.q) + base(0);
  const T* gk = reinterpret_cast<const T*>(p.k) + base(1);
  const T* gv = reinterpret_cast<const T*>(p.v) + base(2);
  const T* gtq = JVP ? reinterpret_cast<const T*>(p.tq) + base(3) : nullptr;
  const T* gtk = JVP ? reinterpret_cast<const T*>(p.tk) + base(4) : nullptr;
  const T* gtv = JVP ? reinterpret_cast<const T*>(p.tv) + base(5) : nullptr;

  // ---- zero the contraction padding of the K / dK tiles (never overwritten later)
  zero_tile_padding<T, D, BKV>(Kt, tid);
  if constexpr (JVP) zero_tile_padding<T, D, BKV>(dKt, tid);

  // ---- Q (and dQ) operand chunks of this lane's query row, straight from HBM
  u32x4 Qr[NCHUNK], dQr[JVP ? NCHUNK : 1];
  {
    const int qrow = q0 + wave * 32 + c32;
    const bool ok = qrow < p.Lq;
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      const int cv = 2 * c + g;
      const bool in = ok && cv < VPR;
      Qr[c] = in ? *reinterpret_cast<const u32x4*>(gq + (int64_t)qrow * p.st[0][1] + cv * VEC) : u32x4{0, 0, 0, 0};
      if constexpr (JVP)
        dQr[c] = in ? *reinterpret_cast<const u32x4*>(gtq + (int64_t)qrow * p.st[3][1] + cv * VEC) : u32x4{0, 0, 0, 0};
    }
  }

  // ---- streaming state
  f32x16 O[NDT], dO[JVP ? NDT : 1];
#pragma unroll
  for (int t = 0; t < NDT; ++t) {
    O[t] = f32x16{0};
    if constexpr (JVP) dO[t] = f32x16{0};
  }
  float m_run = -INFINITY, l_run = 0.f, mu_run = 0.f;  // per-lane partials of row q (halves g=0/1 merged at the end)
  const float c2 = p.scale_log2;                        // softmax scale * log2(e)

  TileStream<T, D, BKV, NT> stream;
  const T* gsrc[NT];
  int64_t gstride[NT];
  T* ldst[NT];
  gsrc[0] = gk; gstride[0] = p.st[1][1]; ldst[0] = Kt;
  gsrc[1] = gv; gstride[1] = p.st[2][1]; ldst[1] = Vt;
  if constexpr (JVP) {
    gsrc[2] = gtk; gstride[2] = p.st[4][1]; ldst[2] = dKt;
    gsrc[3] = gtv; gstride[3] = p.st[5][1]; ldst[3] = dVt;
  }

  const int ntiles = (p.Lkv + BKV - 1) / BKV;
  stream.issue(gsrc, gstride, 0, p.Lkv, tid);
  for (int it = 0; it < ntiles; ++it) {
    const int kv0 = it * BKV;
    __syncthreads();           // every wave is done reading the previous tile
    stream.commit(ldst, tid);
    __syncthreads();
    if (it + 1 < ntiles) stream.issue(gsrc, gstride, kv0 + BKV, p.Lkv, tid);   // in flight during the math below

    // ---- S^T and dS^T for the NSUB 32-row sub-tiles
    f32x16 S[NSUB], dS[JVP ? NSUB : 1];
#pragma unroll
    for (int s = 0; s < NSUB; ++s) {
      S[s] = f32x16{0};
      if constexpr (JVP) dS[s] = f32x16{0};
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c) {
        const u32x4 ka = lds_row_chunk<T, STRIDE>(Kt, s * 32 + c32, c, g);
        mma_chunk<T>(S[s], ka, Qr[c]);
        if constexpr (JVP) {
          const u32x4 dka = lds_row_chunk<T, STRIDE>(dKt, s * 32 + c32, c, g);
          mma_chunk<T>(dS[s], ka, dQr[c]);
          mma_chunk<T>(dS[s], dka, Qr[c]);
        }
      }
    }
    // ---- mask keys past the end (last tile only; uniform branch)
    if (kv0 + BKV > p.Lkv) {
#pragma unroll
      for (int s = 0; s < NSUB; ++s)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (kv0 + s * 32 + acc_row(i, g) >= p.Lkv) S[s][i] = -INFINITY;
    }
    // ---- running maximum (log2 domain) and rescale
    float mx = S[0][0];
#pragma unroll
    for (int s = 0; s < NSUB; ++s)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, S[s][i]);
    mx = xhalf_max(mx);
    const float m_new = fmaxf(m_run, mx * c2);
    const float alpha = fast_exp2(m_run - m_new);
    m_run = m_new;
    l_run *= alpha;
    if constexpr (JVP) mu_run *= alpha;
#pragma unroll
    for (int t = 0; t < NDT; ++t) {
      O[t] *= alpha;
      if constexpr (JVP) dO[t] *= alpha;
    }
    // ---- probabilities, weights, and the P*V-like products
#pragma unroll
    for (int s = 0; s < NSUB; ++s) {
      f32x16 E, G;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        E[i] = fast_exp2(fmaf(S[s][i], c2, -m_new));
        l_run += E[i];
        if constexpr (JVP) {
          G[i] = E[i] * (dS[s][i] * p.scale);
          mu_run += G[i];
        }
      }
#pragma unroll
      for (int st = 0; st < PV_STEPS; ++st) {
        const ColOperand pe = acc_operand<T>(E, st);
        ColOperand pg;
        if constexpr (JVP) pg = acc_operand<T>(G, st);
#pragma unroll
        for (int t = 0; t < NDT; ++t) {
          const ColOperand va = lds_col_operand<T, STRIDE>(Vt, s * 32, t * 32, st, lane);
          mma_col<T>(O[t], va, pe);
          if constexpr (JVP) {
            const ColOperand dva = lds_col_operand<T, STRIDE>(dVt, s * 32, t * 32, st, lane);
            mma_col<T>(dO[t], va, pg);
            mma_col<T>(dO[t], dva, pe);
          }
        }
      }
    }
  }

  // ---- epilogue: normalise, transpose through LDS, coalesced store
  const float l_tot = xhalf_sum(l_run);
  const float inv_l = 1.0f / l_tot;
  float mu_n = 0.f;
  if constexpr (JVP) mu_n = xhalf_sum(mu_run) * inv_l;
  {
    const int qrow = q0 + wave * 32 + c32;
    if (p.lse != nullptr && g == 0 && qrow < p.Lq)
      p.lse[(int64_t)bh * p.Lq + qrow] = (m_run + log2f(l_tot)) * kLn2;
    if constexpr (JVP)
      if (p.dlse != nullptr && g == 0 && qrow < p.Lq) p.dlse[(int64_t)bh * p.Lq + qrow] = mu_n;
  }
  T* stage = reinterpret_cast<T*>(smem);
  store_rows_transposed<T, D>(stage, reinterpret_cast<T*>(p.o) + base(6), p.st[6][1], q0, p.Lq, tid,
                              [&](int t, int i) { return O[t][i] * inv_l; });
  if constexpr (JVP)
    store_rows_transposed<T, D>(stage, reinterpret_cast<T*>(p.to) + base(7), p.st[7][1], q0, p.Lq, tid,
                                [&](int t, int i) { return fmaf(-mu_n, O[t][i] * inv_l, dO[t][i] * inv_l); });
}

template <typename T, int D, bool JVP>
static int launch_fwd_t(const FwdParams& p, int BH, hipStream_t stream) {
  using C = Cfg<T, D>;
  constexpr int tiles = (JVP ? 4 : 2) * C::TILE_BYTES + 512;   // + slack: P*V operands read a few columns past the last row
  constexpr int stage = 128 * C::OROWV * 16;
  constexpr int smem = tiles > stage ? tiles : stage;
  auto kern = attn_fwd_kernel<T, D, JVP>;
  static bool lds_ok[64] = {};
  if (!ensure_dynamic_lds(kern, smem, lds_ok)) return -7;
  const uint32_t nqb = (p.Lq + 127) / 128;
  return launch_kernel(kern, dim3(nqb * (uint32_t)BH), dim3(256), smem, stream, p);
}

template <typename T, bool JVP>
static int launch_fwd_d(const FwdParams& p, int BH, int D, hipStream_t stream) {
  switch (D) {
    case 32: return launch_fwd_t<T, 32, JVP>(p, BH, stream);
    case 64: return launch_fwd_t<T, 64, JVP>(p, BH, stream);
    case 72: return launch_fwd_t<T, 72, JVP>(p, BH, stream);
    case 80: return launch_fwd_t<T, 80, JVP>(p, BH, stream);
    case 96: return launch_fwd_t<T, 96, JVP>(p, BH, stream);
    case 128: return launch_fwd_t<T, 128, JVP>(p, BH, stream);
    default: return -2;
  }
}

int launch_fwd_generic(const FwdParams& p, int BH, int D, bool bf16, bool jvp, hipStream_t stream) {
  if (bf16) return jvp ? launch_fwd_d<__bf16, true>(p, BH, D, stream) : launch_fwd_d<__bf16, false>(p, BH, D, stream);
  return jvp ? launch_fwd_d<float, true>(p, BH, D, stream) : launch_fwd_d<float, false>(p, BH, D, stream);
}

int launch_fwd(const FwdParams& p, int BH, int D, bool bf16, bool jvp, hipStream_t stream) {
  if (bf16) {
    const int rc = launch_fwd_bf16_fast(p, BH, D, jvp, stream);
    if (rc != 1) return rc;   // 1 = no tuned kernel for this shape
  }
  if (p.q_gain != nullptr) return kNoQNormKernel;   // the generic kernels take already-normalised q
  return launch_fwd_generic(p, BH, D, bf16, jvp, stream);
}

}  // namespace dmf
