// Tuned bf16 backward (dQ kernel + dK/dV kernel) for gfx950.
//
// Same two-kernel, atomics-free scheme and the same register layouts as the
// generic kernels in attn_bwd.hip, with the throughput structure of the tuned
// forward: <= 256 VGPRs (two work-groups per CU), 32-row tiles streamed
// HBM -> LDS by bounds-checked buffer DMA into a double buffer with one barrier
// per tile, software-pipelined LDS operand reads, and the softmax scale and
// log2(e) folded into the register-resident operand (Q in the dQ kernel, K in
// the dK/dV kernel) so that P = exp2(S - lse*log2e) costs one VALU op + exp.
#include "attn_common.h"
#include "attn_kernels.h"
#include <algorithm>

namespace dmf {

template <int D>
struct BwdFastCfg {
  static constexpr int VPR = D / 8, NCHUNK = (D + 15) / 16, NDT = (D + 31) / 32;
  static constexpr int P = Cfg<__bf16, D>::ROWV;     // tile row pitch in 16-byte vectors (odd): tiles are read both by rows and transposed
  static constexpr int STR = P * 8;
  static constexpr int TBYTES = 32 * P * 16;          // one 32-row tile
  static constexpr int STAT = 256;                    // per stage: 32 x lse, 32 x delta (fp32)
  static constexpr bool TAIL = (D % 32) != 0 && (D % 32) <= 16;   // 16-wide remainder via 16x16x32 MFMAs (72, 80)
  static constexpr int NMT = TAIL ? D / 32 : NDT;                 // full 32-wide output tiles
};

// bf16x8 chunk times a scalar, re-rounded to bf16.
__device__ __forceinline__ u32x4 scale_bf16x8(u32x4 x, float s) {
  u32x4 y;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    y[e] = pack_bf16x2(__uint_as_float(x[e] << 16) * s, __uint_as_float(x[e] & 0xffff0000u) * s);
  return y;
}

template <int BYTES_PER_STAGE, int PADV, int P, int VPR>
__device__ __forceinline__ void zero_pads(char* smem, int tile_off, int tid) {
  if constexpr (PADV > 0) {
#pragma unroll
    for (int s = 0; s < 2; ++s)
      for (int i = tid; i < 32 * PADV; i += 256)
        *reinterpret_cast<u32x4*>(smem + s * BYTES_PER_STAGE + tile_off + ((i / PADV) * P + VPR + i % PADV) * 16) = u32x4{0, 0, 0, 0};
  }
}

// ------------------------------------------------------------------ dQ kernel
// SUB = 32-key tiles per stage (and per work-group barrier).
template <int D, int SUB>
__global__ __launch_bounds__(256, 2) void attn_bwd_dq_bf16_kernel(const BwdParams p) {
  using F = BwdFastCfg<D>;
  using T = __bf16;
  constexpr int VPR = F::VPR, NCHUNK = F::NCHUNK, NMT = F::NMT, P = F::P, STR = F::STR;
  constexpr bool TAIL = F::TAIL;
  constexpr int PAIR = 2 * F::TBYTES;    // one 32-key tile: K | V
  constexpr int STAGE = SUB * PAIR;
  constexpr int V_OFF = F::TBYTES;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, g = lane >> 5;
  const uint32_t nqb = (p.Lq + 127) / 128;
  const uint32_t wg = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = wg / nqb, qb = wg % nqb;
  const int b = bh / p.H, h = bh % p.H;
  const int q0 = qb * 128;
  auto base = [&](int t) { return (int64_t)b * p.st[t][0] + (int64_t)h * p.st[t][2]; };

#pragma unroll
  for (int sub = 0; sub < SUB; ++sub) {
    zero_pads<STAGE, P - VPR, P, VPR>(smem, sub * PAIR, tid);
    zero_pads<STAGE, P - VPR, P, VPR>(smem, sub * PAIR + V_OFF, tid);
  }

  // ---- this lane's query row: Q (times scale*log2e), dout, delta, lse
  const int qrow = q0 + wave * 32 + c32;
  const bool qok = qrow < p.Lq;
  u32x4 Qr[NCHUNK], dOr[NCHUNK];
  float dpart = 0.f;
  {
    u32x4 Or[NCHUNK];
    const uint32_t rb_q = (uint32_t)p.st[1][1] * 2, rb_do = (uint32_t)p.st[0][1] * 2, rb_o = (uint32_t)p.st[4][1] * 2;
    load_row_chunks<NCHUNK, VPR>(make_rows_rsrc(reinterpret_cast<const T*>(p.q) + base(1), rb_q, p.Lq, D * 2), rb_q, qrow, g, Qr);
    load_row_chunks<NCHUNK, VPR>(make_rows_rsrc(reinterpret_cast<const T*>(p.dout) + base(0), rb_do, p.Lq, D * 2), rb_do, qrow, g, dOr);
    load_row_chunks<NCHUNK, VPR>(make_rows_rsrc(reinterpret_cast<const T*>(p.o) + base(4), rb_o, p.Lq, D * 2), rb_o, qrow, g, Or);
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      Qr[c] = scale_bf16x8(Qr[c], p.scale_log2);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        dpart += __uint_as_float(dOr[c][e] << 16) * __uint_as_float(Or[c][e] << 16);
        dpart += __uint_as_float(dOr[c][e] & 0xffff0000u) * __uint_as_float(Or[c][e] & 0xffff0000u);
      }
    }
  }
  const float delta = xhalf_sum(dpart);
  float lse2 = INFINITY;   // +inf switches padded query rows off (P = 0)
  if (qok) {
    lse2 = p.lse[(int64_t)bh * p.Lq + qrow] * kLog2e;
    if (g == 0) p.delta[(int64_t)bh * p.Lq + qrow] = delta;
  }

  f32x16 dQ[NMT];
  f32x4 dQ16[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
#pragma unroll
  for (int t = 0; t < NMT; ++t) dQ[t] = f32x16{0};

  const uint32_t rb_k = (uint32_t)p.st[2][1] * 2, rb_v = (uint32_t)p.st[3][1] * 2;
  const __amdgpu_buffer_rsrc_t rs_k = make_rows_rsrc(reinterpret_cast<const T*>(p.k) + base(2), rb_k, p.Lkv, D * 2);
  const __amdgpu_buffer_rsrc_t rs_v = make_rows_rsrc(reinterpret_cast<const T*>(p.v) + base(3), rb_v, p.Lkv, D * 2);
  const int ntiles = (p.Lkv + 31) / 32;             // 32-key tiles
  const int nstages = (ntiles + SUB - 1) / SUB;
  auto issue = [&](int is) {
    char* st = smem + (is & 1) * STAGE;
#pragma unroll
    for (int sub = 0; sub < SUB; ++sub) {
      const int it = is * SUB + sub;
      if (it < ntiles) {   // wave-uniform
        issue_tile_rows<P, VPR>(rs_k, rb_k, (uint32_t)it * 32 * rb_k, st + sub * PAIR, wave, lane);
        issue_tile_rows<P, VPR>(rs_v, rb_v, (uint32_t)it * 32 * rb_v, st + sub * PAIR + V_OFF, wave, lane);
      }
    }
  };
  const uint32_t row_addr = lds_addr(smem) + c32 * STR * 2 + g * 16;
  const uint32_t col_addr = lds_addr(smem) + ((4 * g + ((lane & 15) >> 2)) * STR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;

  const uint32_t tail_addr = lds_addr(smem) + tail_lane_offset(lane, STR, 32 * NMT) * 2;

  issue(0);
  for (int is = 0; is < nstages; ++is) {
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    lds_barrier();
    if (is + 1 < nstages) issue(is + 1);
   for (int sub = 0; sub < SUB; ++sub) {
    const int it = is * SUB + sub;
    if (it >= ntiles) break;             // wave-uniform
    const uint32_t ra = row_addr + (is & 1) * STAGE + sub * PAIR, ca = col_addr + (is & 1) * STAGE + sub * PAIR;

    // ---- S^T = K Q^T (log2 units), dP^T = V dout^T
    f32x16 S = {0}, dP = {0};
    {
      u32x4 kc[2], vc[2];
      kc[0] = lds_read128_issue<0>(ra);
      vc[0] = lds_read128_issue<V_OFF>(ra);
      static_for<NCHUNK>([&](auto cc) {
        constexpr int c = decltype(cc)::value;
        constexpr bool more = c + 1 < NCHUNK;
        if constexpr (more) {
          kc[(c + 1) & 1] = lds_read128_issue<32 * (c + 1)>(ra);
          vc[(c + 1) & 1] = lds_read128_issue<32 * (c + 1) + V_OFF>(ra);
        }
        lds_read128_wait<more ? 2 : 0>(kc[c & 1], vc[c & 1]);
        mma_chunk<T>(S, kc[c & 1], Qr[c]);
        mma_chunk<T>(dP, vc[c & 1], dOr[c]);
      });
    }
    // ---- dS^T = P^T * (dP^T - delta)
    f32x16 dS;
    const bool tail = (it + 1) * 32 > p.Lkv;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float pr = fast_exp2(S[i] - lse2);
      if (tail && it * 32 + acc_row(i, g) >= p.Lkv) pr = 0.f;
      dS[i] = pr * (dP[i] - delta);
    }
    // ---- dQ^T += K^T dS^T
    {
      ColOperand ds[2] = {acc_operand<T>(dS, 0), acc_operand<T>(dS, 1)};
      constexpr int NG = 2 * NMT, NGT = NG + (TAIL ? 1 : 0);
      TrPair kk[2];
      auto lo_off = [](int gi) constexpr { return (16 * (gi / NMT) * STR + 32 * (gi % NMT)) * 2; };
      kk[0] = lds_tr16_issue<lo_off(0), lo_off(0) + 8 * STR * 2>(ca);
      static_for<NGT>([&](auto gc) {
        constexpr int gi = decltype(gc)::value;
        constexpr bool more = gi + 1 < NGT;
        if constexpr (gi + 1 < NG) kk[(gi + 1) & 1] = lds_tr16_issue<lo_off(gi + 1), lo_off(gi + 1) + 8 * STR * 2>(ca);
        else if constexpr (more) kk[(gi + 1) & 1] = lds_tr16_issue<0, 8 * STR * 2>(tail_addr + (is & 1) * STAGE + sub * PAIR);
        lds_tr16_wait<more ? 2 : 0>(kk[gi & 1]);
        if constexpr (gi < NG) {
          mma_col<T>(dQ[gi % NMT], tr_operand(kk[gi & 1]), ds[gi / NMT]);
        } else {
          ColOperand d0, d1;
          tail_operands(ds[0], ds[1], d0, d1);
          mma16(dQ16[0], tr_operand(kk[gi & 1]), d0);
          mma16(dQ16[1], tr_operand(kk[gi & 1]), d1);
        }
      });
    }
   }
  }
  store_rows_transposed<T, D, 4, NMT>(reinterpret_cast<T*>(smem), reinterpret_cast<T*>(p.dq) + base(5), p.st[5][1], q0, p.Lq, tid,
                                      [&](int t, int i) { return dQ[t][i] * p.scale; },
                                      [&](void* ws) {
                                        if constexpr (TAIL) store_tail16<T, D, NMT>(ws, lane, [&](int hq, int e) { return dQ16[hq][e] * p.scale; });
                                      });
}

// --------------------------------------------------------------- dK/dV kernel
template <int D>
__global__ __launch_bounds__(256, 2) void attn_bwd_dkv_bf16_kernel(const BwdParams p) {
  using F = BwdFastCfg<D>;
  using T = __bf16;
  constexpr int VPR = F::VPR, NCHUNK = F::NCHUNK, NMT = F::NMT, P = F::P, STR = F::STR;
  constexpr bool TAIL = F::TAIL;
  constexpr int STAGE = 2 * F::TBYTES + F::STAT;   // Q | dout | lse[32], delta[32]
  constexpr int DO_OFF = F::TBYTES, STAT_OFF = 2 * F::TBYTES;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, g = lane >> 5;
  const uint32_t nkb = (p.Lkv + 127) / 128;
  const uint32_t wg = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = wg / nkb, kb = wg % nkb;
  const int b = bh / p.H, h = bh % p.H;
  const int k0 = kb * 128;
  auto base = [&](int t) { return (int64_t)b * p.st[t][0] + (int64_t)h * p.st[t][2]; };

  zero_pads<STAGE, P - VPR, P, VPR>(smem, 0, tid);
  zero_pads<STAGE, P - VPR, P, VPR>(smem, DO_OFF, tid);

  // ---- this lane's key row: K (times scale*log2e) and V stay in registers
  u32x4 Kr[NCHUNK], Vr[NCHUNK];
  {
    const int krow = k0 + wave * 32 + c32;
    const uint32_t rb_k = (uint32_t)p.st[2][1] * 2, rb_v = (uint32_t)p.st[3][1] * 2;
    load_row_chunks<NCHUNK, VPR>(make_rows_rsrc(reinterpret_cast<const T*>(p.k) + base(2), rb_k, p.Lkv, D * 2), rb_k, krow, g, Kr);
    load_row_chunks<NCHUNK, VPR>(make_rows_rsrc(reinterpret_cast<const T*>(p.v) + base(3), rb_v, p.Lkv, D * 2), rb_v, krow, g, Vr);
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) Kr[c] = scale_bf16x8(Kr[c], p.scale_log2);
  }
  f32x16 dK[NMT], dV[NMT];
  f32x4 dK16[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}}, dV16[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
#pragma unroll
  for (int t = 0; t < NMT; ++t) {
    dK[t] = f32x16{0};
    dV[t] = f32x16{0};
  }

  const uint32_t rb_q = (uint32_t)p.st[1][1] * 2, rb_do = (uint32_t)p.st[0][1] * 2;
  const __amdgpu_buffer_rsrc_t rs_q = make_rows_rsrc(reinterpret_cast<const T*>(p.q) + base(1), rb_q, p.Lq, D * 2);
  const __amdgpu_buffer_rsrc_t rs_do = make_rows_rsrc(reinterpret_cast<const T*>(p.dout) + base(0), rb_do, p.Lq, D * 2);
  // per-row statistics: padded query rows read lse = delta = 0 and are masked where P is formed
  const __amdgpu_buffer_rsrc_t rs_lse = make_rows_rsrc(p.lse + (int64_t)bh * p.Lq, 4, p.Lq, 4);
  const __amdgpu_buffer_rsrc_t rs_dl = make_rows_rsrc(p.delta + (int64_t)bh * p.Lq, 4, p.Lq, 4);
  auto issue = [&](int it) {
    char* st = smem + (it & 1) * STAGE;
    issue_tile_rows<P, VPR>(rs_q, rb_q, (uint32_t)it * 32 * rb_q, st, wave, lane);
    issue_tile_rows<P, VPR>(rs_do, rb_do, (uint32_t)it * 32 * rb_do, st + DO_OFF, wave, lane);
    if (wave < 2 && lane < 32)   // wave 0: lse[32], wave 1: delta[32]
      __builtin_amdgcn_raw_ptr_buffer_load_lds(wave == 0 ? rs_lse : rs_dl,
                                               (__attribute__((address_space(3))) void*)(st + STAT_OFF + wave * 128), 4,
                                               lane * 4, (uint32_t)it * 128, 0, 0);
  };
  const uint32_t row_addr = lds_addr(smem) + c32 * STR * 2 + g * 16;
  const uint32_t col_addr = lds_addr(smem) + ((4 * g + ((lane & 15) >> 2)) * STR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;

  const uint32_t tail_addr = lds_addr(smem) + tail_lane_offset(lane, STR, 32 * NMT) * 2;

  const int ntiles = (p.Lq + 31) / 32;
  issue(0);
  for (int it = 0; it < ntiles; ++it) {
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    lds_barrier();
    if (it + 1 < ntiles) issue(it + 1);
    const uint32_t ra = row_addr + (it & 1) * STAGE, ca = col_addr + (it & 1) * STAGE;
    const float* stat = reinterpret_cast<const float*>(smem + (it & 1) * STAGE + STAT_OFF);

    // ---- S = Q K^T (log2 units), dP = dout V^T : rows = queries (in-lane), columns = keys (lanes)
    f32x16 S = {0}, dP = {0};
    {
      u32x4 qc[2], oc[2];
      qc[0] = lds_read128_issue<0>(ra);
      oc[0] = lds_read128_issue<DO_OFF>(ra);
      static_for<NCHUNK>([&](auto cc) {
        constexpr int c = decltype(cc)::value;
        constexpr bool more = c + 1 < NCHUNK;
        if constexpr (more) {
          qc[(c + 1) & 1] = lds_read128_issue<32 * (c + 1)>(ra);
          oc[(c + 1) & 1] = lds_read128_issue<32 * (c + 1) + DO_OFF>(ra);
        }
        lds_read128_wait<more ? 2 : 0>(qc[c & 1], oc[c & 1]);
        mma_chunk<T>(S, qc[c & 1], Kr[c]);
        mma_chunk<T>(dP, oc[c & 1], Vr[c]);
      });
    }
    // ---- P = exp2(S - lse*log2e), dS = P * (dP - delta).  Query rows past Lq are switched off here (P = 0): the
    //      bounds check zero-fills them only when consecutive rows are distinct addresses, and a broadcast operand
    //      (row stride 0, e.g. the gradient of a sum over the sequence) aliases them onto row 0 instead.
    f32x16 Pm, dS;
    const bool qtail = (it + 1) * 32 > p.Lq;   // wave-uniform
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const f32x4 l4 = *reinterpret_cast<const f32x4*>(stat + j * 8 + 4 * g);
      const f32x4 d4 = *reinterpret_cast<const f32x4*>(stat + 32 + j * 8 + 4 * g);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = 4 * j + e;
        float pr = fast_exp2(fmaf(l4[e], -kLog2e, S[i]));
        if (qtail && it * 32 + acc_row(i, g) >= p.Lq) pr = 0.f;
        Pm[i] = pr;
        dS[i] = pr * (dP[i] - d4[e]);
      }
    }
    // ---- dV^T += dout^T P ; dK^T += Q^T dS
    {
      ColOperand pp[2] = {acc_operand<T>(Pm, 0), acc_operand<T>(Pm, 1)};
      ColOperand ds[2] = {acc_operand<T>(dS, 0), acc_operand<T>(dS, 1)};
      constexpr int NG = 2 * NMT, NGT = NG + (TAIL ? 1 : 0);
      TrPair qq[2], oo[2];
      auto lo_off = [](int gi) constexpr { return (16 * (gi / NMT) * STR + 32 * (gi % NMT)) * 2; };
      qq[0] = lds_tr16_issue<lo_off(0), lo_off(0) + 8 * STR * 2>(ca);
      oo[0] = lds_tr16_issue<lo_off(0) + DO_OFF, lo_off(0) + 8 * STR * 2 + DO_OFF>(ca);
      static_for<NGT>([&](auto gc) {
        constexpr int gi = decltype(gc)::value;
        constexpr bool more = gi + 1 < NGT;
        if constexpr (gi + 1 < NG) {
          constexpr int LO = lo_off(gi + 1), HI = LO + 8 * STR * 2;
          qq[(gi + 1) & 1] = lds_tr16_issue<LO, HI>(ca);
          oo[(gi + 1) & 1] = lds_tr16_issue<LO + DO_OFF, HI + DO_OFF>(ca);
        } else if constexpr (more) {
          const uint32_t ta = tail_addr + (it & 1) * STAGE;
          qq[(gi + 1) & 1] = lds_tr16_issue<0, 8 * STR * 2>(ta);
          oo[(gi + 1) & 1] = lds_tr16_issue<DO_OFF, 8 * STR * 2 + DO_OFF>(ta);
        }
        lds_tr16_wait<more ? 4 : 0>(qq[gi & 1], oo[gi & 1]);
        if constexpr (gi < NG) {
          mma_col<T>(dV[gi % NMT], tr_operand(oo[gi & 1]), pp[gi / NMT]);
          mma_col<T>(dK[gi % NMT], tr_operand(qq[gi & 1]), ds[gi / NMT]);
        } else {
          ColOperand p0, p1, d0, d1;
          tail_operands(pp[0], pp[1], p0, p1);
          tail_operands(ds[0], ds[1], d0, d1);
          mma16(dV16[0], tr_operand(oo[gi & 1]), p0);
          mma16(dV16[1], tr_operand(oo[gi & 1]), p1);
          mma16(dK16[0], tr_operand(qq[gi & 1]), d0);
          mma16(dK16[1], tr_operand(qq[gi & 1]), d1);
        }
      });
    }
  }
  T* stage = reinterpret_cast<T*>(smem);
  store_rows_transposed<T, D, 4, NMT>(stage, reinterpret_cast<T*>(p.dk) + base(6), p.st[6][1], k0, p.Lkv, tid,
                                      [&](int t, int i) { return dK[t][i] * p.scale; },
                                      [&](void* ws) {
                                        if constexpr (TAIL) store_tail16<T, D, NMT>(ws, lane, [&](int hq, int e) { return dK16[hq][e] * p.scale; });
                                      });
  store_rows_transposed<T, D, 4, NMT>(stage, reinterpret_cast<T*>(p.dv) + base(7), p.st[7][1], k0, p.Lkv, tid,
                                      [&](int t, int i) { return dV[t][i]; },
                                      [&](void* ws) {
                                        if constexpr (TAIL) store_tail16<T, D, NMT>(ws, lane, [&](int hq, int e) { return dV16[hq][e]; });
                                      });
}

template <int D>
static int launch_bwd_fast_t(const BwdParams& p, int BH, hipStream_t stream) {
  using F = BwdFastCfg<D>;
  constexpr int tiles = 2 * (2 * F::TBYTES + F::STAT) + 512;
  constexpr int stage = 128 * Cfg<__bf16, D>::OROWV * 16;
  constexpr int smem = tiles > stage ? tiles : stage;
  constexpr int kDqSub = 2;   // two 32-key tiles per barrier in the dQ kernel (+3 % over one; four would leave one work-group per CU)
  constexpr int tiles1 = 2 * kDqSub * 2 * F::TBYTES + 512;
  constexpr int smem1 = tiles1 > stage ? tiles1 : stage;
  auto k1 = attn_bwd_dq_bf16_kernel<D, kDqSub>;
  auto k2 = attn_bwd_dkv_bf16_kernel<D>;
  static bool lds_ok1[64] = {}, lds_ok2[64] = {};
  if (!ensure_dynamic_lds(k1, smem1, lds_ok1) || !ensure_dynamic_lds(k2, smem, lds_ok2)) return -7;
  const uint32_t nqb = (p.Lq + 127) / 128, nkb = (p.Lkv + 127) / 128;
  if (int rc = launch_kernel(k1, dim3(nqb * (uint32_t)BH), dim3(256), smem1, stream, p)) return rc;
  return launch_kernel(k2, dim3(nkb * (uint32_t)BH), dim3(256), smem, stream, p);
}

// Returns 1 if there is no tuned kernel for the case (caller uses the generic ones).
int launch_bwd_bf16_fast(const BwdParams& p, int BH, int D, hipStream_t stream) {
  // 32-bit buffer addressing: every (batch, head) slab of rows must span < 2 GiB
  const int64_t max_row = std::max(std::max(std::max(p.st[0][1], p.st[1][1]), std::max(p.st[2][1], p.st[3][1])), p.st[4][1]);
  if (max_row * 2 * (int64_t)(std::max(p.Lq, p.Lkv) + 256) >= (int64_t)1 << 31) return 1;
  switch (D) {
    case 64: return launch_bwd_fast_t<64>(p, BH, stream);
    case 72: return launch_bwd_fast_t<72>(p, BH, stream);
    case 80: return launch_bwd_fast_t<80>(p, BH, stream);
    case 96: return launch_bwd_fast_t<96>(p, BH, stream);
    case 128: return launch_bwd_fast_t<128>(p, BH, stream);
    default: return 1;
  }
}

}  // namespace dmf
