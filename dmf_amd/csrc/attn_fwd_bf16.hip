// Tuned bf16 attention forward (+ JVP) for gfx950.
//
// Same math and register layout as the generic kernel in attn_fwd.hip
// (transposed scores S^T = K Q^T, per-lane softmax state, P^T fed back as the
// MFMA B operand, O^T / dO^T accumulators), restructured for throughput:
//   * <= 256 VGPRs so two work-groups (8 waves) share a CU and one wave's
//     softmax VALU work overlaps another wave's MFMAs;
//   * K, V, dK, dV tiles of 32 keys go HBM -> LDS with global_load_lds_dwordx4
//     (no staging registers), double-buffered, one barrier per tile; the four
//     load instructions of the next tile are issued one at a time between the
//     score MFMAs of the current one (issued together right after the barrier
//     they keep all eight waves off the matrix pipe for ~350 cycles per tile);
//   * 256-row work-groups fetch their Q / dQ rows the same way (whole rows by
//     DMA into LDS, operands read from there) instead of one scattered 16-byte
//     load per lane and chunk;
//   * Q and dQ are pre-multiplied by the softmax scale when loaded, so neither
//     S nor dS needs a per-element scale;
//   * lazy rescaling: the running maximum is only raised (and O, dO rescaled)
//     when a score exceeds it by more than 2^kLazyLog2, otherwise the stale
//     maximum is kept -- exact, because normalisation happens once at the end;
//   * for head dims that are not a multiple of 32 the spare row D of the last
//     O^T / dO^T tile is fed a column of ones (V) / zeros (dV), so the MFMAs
//     deliver the row sums l = sum(P) and mu = sum(P*dS) for free.
#include "attn_common.h"
#include "attn_kernels.h"
#include <algorithm>
#include <cstdio>

namespace dmf {

constexpr float kLazyLog2 = 6.0f;

template <int D>
struct FastCfg {
  static constexpr int VPR = D / 8, NCHUNK = (D + 15) / 16, NDT = (D + 31) / 32;
  static constexpr int KP = Cfg<__bf16, D>::ROWV;                         // K/dK row pitch in 16-byte vectors (odd)
  static constexpr int VP = NDT * 4 <= 4 ? 4 : (NDT * 4 <= 12 ? 12 : 20);  // V/dV pitch: 4 (mod 8) vectors => conflict-free transposed reads
  static constexpr int KSTR = KP * 8, VSTR = VP * 8;                       // pitches in elements
  static constexpr int BKV = 32;
  static constexpr int QP = VPR | 1;                                       // Q/dQ staging row pitch in vectors (odd => conflict-free b128 reads)
  static constexpr int KBYTES = BKV * KP * 16, VBYTES = BKV * VP * 16;
  // Head dims with a remainder of at most 16 over a multiple of 32 (72, 80): the
  // remainder columns of O^T / dO^T are produced by 16x16x32 MFMAs instead of a
  // mostly-padding 32-wide tile.
  static constexpr bool TAIL = (D % 32) != 0 && (D % 32) <= 16;
  static constexpr int NMT = TAIL ? D / 32 : NDT;                          // full 32-wide output tiles
  // A spare output row (index D) exists when D is not a multiple of the tile width.
  static constexpr bool PADROW = TAIL ? (D % 32) < 16 : (D % 32) != 0;
  static constexpr int PAD_IDX = 4 * ((D % 32) / 8) + (D % 4);             // 32-wide last tile: accumulator element holding row D%32 ...
  static constexpr int PAD_G = ((D % 32) % 8) / 4;                         // ... in the lanes of this half
  static constexpr int PAD16_ROW = (D % 32) / 4, PAD16_E = D % 4;          // 16-wide tail: lanes of 16-lane row PAD16_ROW, element PAD16_E
  // Spare contraction slots in the last score chunk (head dim 72: slots 72..79 of 5 x 16): slots D..D+2 carry the running
  // maximum -- Q's pad elements hold -m as a bf16 triple (hi + mid + lo, 2^-24 relative) against ones in the K rows, and Q
  // is pre-multiplied by scale*log2(e) -- so that the MFMAs deliver S*log2(e) - m and the exponentials take their argument
  // as it is (no multiply-add per score).
  static constexpr bool MFOLD = 2 * NCHUNK > VPR;
  // Head dim 128 with tangents needs more than 256 registers (four accumulator tile pairs, eight Q and dQ operand chunks):
  // the last QPARK chunks of Q and dQ are parked in LDS (each wave its own lanes, written once) and read back next to the
  // K / dK chunks they multiply, instead of being spilled to scratch memory (256-row work-groups only: two 128-row
  // work-groups per CU have no LDS to spare for it).
  static constexpr int QPARK_JVP = D == 128 ? 4 : 0;
};

// NW = waves per work-group: 4 (128 query rows, two work-groups per CU) or
// 8 (256 query rows, one work-group per CU: half the tile traffic per FLOP).
// QN: per-head RMS norm of q (and its tangent) applied while the Q operands are formed.
// KN: per-head RMS norm of k (and its tangent) applied to every key tile in LDS, between its arrival and its use.
template <int D, bool JVP, int NW, bool QN = false, bool KN = false>
__global__ __launch_bounds__(64 * NW, 8 / NW) void attn_fwd_bf16_kernel(const FwdParams p) {
  static_assert(!KN || QN, "the key norm is only built together with the query norm");
  constexpr int NTHR = 64 * NW, BQ = 32 * NW;
  using F = FastCfg<D>;
  using T = __bf16;
  constexpr int VPR = F::VPR, NCHUNK = F::NCHUNK, NDT = F::NDT, KP = F::KP, VP = F::VP;
  constexpr int KSTR = F::KSTR, VSTR = F::VSTR, BKV = F::BKV;
  constexpr int STAGE = (JVP ? 2 : 1) * (F::KBYTES + F::VBYTES);
  // Staging of this work-group's Q (and dQ) rows behind the two tile stages, when 160 KB of LDS have room for it.
  constexpr int QP = F::QP, QS_OFF = 2 * STAGE + 512, QS_BYTES = 32 * NW * QP * 16;
  constexpr bool QLDS = NW == 8 && QS_OFF + (JVP ? 2 : 1) * QS_BYTES <= 160 * 1024;
  constexpr int QPARK = JVP && NW == 8 ? F::QPARK_JVP : 0;                 // parked operand k of wave w: QX_OFF + ((k * NW + w) * 64 + lane) * 16
  constexpr int QX_OFF = 2 * STAGE + 512;
  static_assert(QPARK == 0 || !QLDS, "the parked operands use the space behind the tile stages");

  extern __shared__ __attribute__((aligned(16))) char smem[];
  auto Kt = [&](int s) { return smem + s * STAGE; };
  auto Vt = [&](int s) { return smem + s * STAGE + F::KBYTES; };
  auto dKt = [&](int s) { return smem + s * STAGE + F::KBYTES + F::VBYTES; };
  auto dVt = [&](int s) { return smem + s * STAGE + 2 * F::KBYTES + F::VBYTES; };

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, g = lane >> 5;

  const uint32_t nqb = (p.Lq + BQ - 1) / BQ;
  const uint32_t wg = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = wg / nqb, qb = wg % nqb;
  const int b = bh / p.H, h = bh % p.H;
  const int q0 = qb * BQ;
  auto base = [&](int t) { return (int64_t)b * p.st[t][0] + (int64_t)h * p.st[t][2]; };
  const T* gk = reinterpret_cast<const T*>(p.k) + base(1);
  const T* gv = reinterpret_cast<const T*>(p.v) + base(2);
  const T* gtk = JVP ? reinterpret_cast<const T*>(p.tk) + base(4) : nullptr;
  const T* gtv = JVP ? reinterpret_cast<const T*>(p.tv) + base(5) : nullptr;

  const uint32_t rb_k = (uint32_t)p.st[1][1] * 2, rb_v = (uint32_t)p.st[2][1] * 2;
  const uint32_t rb_tk = JVP ? (uint32_t)p.st[4][1] * 2 : 0, rb_tv = JVP ? (uint32_t)p.st[5][1] * 2 : 0;
  const __amdgpu_buffer_rsrc_t rs_k = make_rows_rsrc(gk, rb_k, p.Lkv, D * 2);
  const __amdgpu_buffer_rsrc_t rs_v = make_rows_rsrc(gv, rb_v, p.Lkv, D * 2);
  const __amdgpu_buffer_rsrc_t rs_tk = make_rows_rsrc(JVP ? gtk : gk, JVP ? rb_tk : rb_k, p.Lkv, D * 2);
  const __amdgpu_buffer_rsrc_t rs_tv = make_rows_rsrc(JVP ? gtv : gv, JVP ? rb_tv : rb_v, p.Lkv, D * 2);
  // A tile is fetched in NPART parts (one DMA instruction per wave each): K, dK, V, dV.
  constexpr int NPART = JVP ? 4 : 2;
  static_assert(NCHUNK >= NPART, "one part of the next tile is issued after each of the first NPART score chunks");
  constexpr int DMA_PER_TILE = (JVP ? 2 : 1) * ((32 / NW * KP + 63) / 64 + (32 / NW * VP + 63) / 64);   // vmcnt units per wave
  auto issue_part = [&](int it, auto pc) {
    constexpr int part = decltype(pc)::value;
    const int s = it & 1;
    const uint32_t r0 = (uint32_t)it * BKV;
    if constexpr (part == 0) issue_tile_rows<KP, VPR, NW>(rs_k, rb_k, r0 * rb_k, Kt(s), wave, lane);
    if constexpr (part == 1 && JVP) issue_tile_rows<KP, VPR, NW>(rs_tk, rb_tk, r0 * rb_tk, dKt(s), wave, lane);
    if constexpr (part == (JVP ? 2 : 1)) issue_tile_rows<VP, VPR, NW>(rs_v, rb_v, r0 * rb_v, Vt(s), wave, lane);
    if constexpr (part == 3 && JVP) issue_tile_rows<VP, VPR, NW>(rs_tv, rb_tv, r0 * rb_tv, dVt(s), wave, lane);
  };
  auto issue = [&](int it) { static_for<NPART>([&](auto pc) { issue_part(it, pc); }); };


  // ---- padding of both stages: zeros, and the ones column of V
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    for (int i = tid; i < BKV * (KP - VPR); i += NTHR) {
      const int off = ((i / (KP - VPR)) * KP + VPR + i % (KP - VPR)) * 16;
      const bool one = F::MFOLD && i % (KP - VPR) == 0;   // elements D..D+2 of a K row = 1.0 (bf16 0x3f80): they multiply the -m triple in Q's pad slots
      *reinterpret_cast<u32x4*>(Kt(s) + off) = u32x4{one ? 0x3f803f80u : 0u, one ? 0x3f80u : 0u, 0, 0};
      if constexpr (JVP) *reinterpret_cast<u32x4*>(dKt(s) + off) = u32x4{0, 0, 0, 0};
    }
    if constexpr (VP > VPR) {
      for (int i = tid; i < BKV * (VP - VPR); i += NTHR) {
        const int cv = VPR + i % (VP - VPR);
        const int off = ((i / (VP - VPR)) * VP + cv) * 16;
        const bool ones = F::PADROW && cv == VPR;          // element D of the row = 1.0 (bf16 0x3f80)
        *reinterpret_cast<u32x4*>(Vt(s) + off) = u32x4{ones ? 0x3f80u : 0u, 0, 0, 0};
        if constexpr (JVP) *reinterpret_cast<u32x4*>(dVt(s) + off) = u32x4{0, 0, 0, 0};
      }
    }
  }

  // ---- Q, dQ operand chunks, pre-multiplied by the softmax scale.  MFOLD: the score product takes QrS = q*scale*log2(e)
  //      (+ the pad slot), the dK product of the tangent scores still Qr = q*scale (kept only with tangents).
  constexpr bool MFOLD = F::MFOLD;
  u32x4 Qr[NCHUNK], dQr[JVP ? NCHUNK : 1], QrS[MFOLD ? NCHUNK : 1], mB = {0, 0, 0, 0};
  {
    const int qrow = q0 + wave * 32 + c32;
    const uint32_t rb_q = (uint32_t)p.st[0][1] * 2;
    if constexpr (QLDS) {
      // Every wave fetches and reads only its own 32 rows: no barrier, just its own vmcnt.
      char* qs = smem + QS_OFF + wave * 32 * QP * 16;
      issue_rows<QP, VPR, 32>(make_rows_rsrc(reinterpret_cast<const T*>(p.q) + base(0), rb_q, p.Lq, D * 2), rb_q,
                              (uint32_t)(q0 + wave * 32) * rb_q, qs, lane);
      if constexpr (JVP) {
        const uint32_t rb_tq = (uint32_t)p.st[3][1] * 2;
        issue_rows<QP, VPR, 32>(make_rows_rsrc(reinterpret_cast<const T*>(p.tq) + base(3), rb_tq, p.Lq, D * 2), rb_tq,
                                (uint32_t)(q0 + wave * 32) * rb_tq, qs + QS_BYTES, lane);
      }
      issue(0);   // the first key tile follows the Q rows; loads complete in order, so it may stay in flight below
      __builtin_amdgcn_s_waitcnt(0x0F70 | (DMA_PER_TILE & 15) | ((DMA_PER_TILE >> 4) << 14));
      const uint32_t qa = lds_addr(qs) + c32 * QP * 16;
      static_for<NCHUNK>([&](auto cc) {
        constexpr int c = decltype(cc)::value;
        // (the upper half of the last chunk of a head dim that is not a multiple of 16 does not exist: read the lower one, zeroed below)
        const uint32_t a = 2 * c + 1 < VPR ? qa + g * 16 : qa;
        Qr[c] = lds_read128_issue<32 * c>(a);
        if constexpr (JVP) dQr[c] = lds_read128_issue<32 * c + QS_BYTES>(a);
      });
      if constexpr (JVP) lds_read128_wait<0>(Qr[NCHUNK - 1], dQr[NCHUNK - 1]);
      else lds_read128_wait<0>(Qr[NCHUNK - 1]);
#pragma unroll
      for (int c = 0; c + 1 < NCHUNK; ++c) {   // the other chunks are valid after the same wait
        if constexpr (JVP) asm volatile("" : "+v"(Qr[c]), "+v"(dQr[c]));
        else asm volatile("" : "+v"(Qr[c]));
      }
      if constexpr (2 * NCHUNK > VPR) {
        if (g == 1) {
          Qr[NCHUNK - 1] = u32x4{0, 0, 0, 0};
          if constexpr (JVP) dQr[NCHUNK - 1] = u32x4{0, 0, 0, 0};
        }
      }
    } else {
      load_row_chunks<NCHUNK, VPR>(make_rows_rsrc(reinterpret_cast<const T*>(p.q) + base(0), rb_q, p.Lq, D * 2), rb_q, qrow, g, Qr);
      if constexpr (JVP) {
        const uint32_t rb_tq = (uint32_t)p.st[3][1] * 2;
        load_row_chunks<NCHUNK, VPR>(make_rows_rsrc(reinterpret_cast<const T*>(p.tq) + base(3), rb_tq, p.Lq, D * 2), rb_tq, qrow, g, dQr);
      }
    }
    auto lo = [](uint32_t w) { return __uint_as_float(w << 16); };
    auto hi = [](uint32_t w) { return __uint_as_float(w & 0xffff0000u); };
    if constexpr (QN) {
      // q_hat = q r g,  dq_hat = (dq r + q dr) g  with  r = (mean q^2 + eps)^-1/2,  dr = -r^3 mean(q dq)  (models/layers.py:39-42
      // and its tangent); this lane holds elements 16c + 8g + 0..7 of its row, the other half of the wave the rest.
      // Rounded to bf16 before the softmax scale is applied, exactly like a separate norm kernel followed by this one.
      float ss = 0.f, sd = 0.f;
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          ss = fmaf(lo(Qr[c][e]), lo(Qr[c][e]), fmaf(hi(Qr[c][e]), hi(Qr[c][e]), ss));
          if constexpr (JVP) sd = fmaf(lo(Qr[c][e]), lo(dQr[c][e]), fmaf(hi(Qr[c][e]), hi(dQr[c][e]), sd));
        }
      const float r = 1.f / sqrtf(xhalf_sum(ss) * (1.f / D) + p.q_eps);
      const float dr = JVP ? -r * r * r * xhalf_sum(sd) * (1.f / D) : 0.f;
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c) {
        float gn[8];
        if (2 * c + g < VPR) {
          const f32x4* gp = reinterpret_cast<const f32x4*>(p.q_gain + 16 * c + 8 * g);
          const f32x4 g0 = gp[0], g1 = gp[1];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            gn[e] = g0[e];
            gn[4 + e] = g1[e];
          }
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) gn[e] = 0.f;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float ql = lo(Qr[c][e]), qh = hi(Qr[c][e]);
          const uint32_t qn = pack_bf16x2(ql * r * gn[2 * e], qh * r * gn[2 * e + 1]);
          if constexpr (JVP) {
            const uint32_t dn = pack_bf16x2(fmaf(lo(dQr[c][e]), r, ql * dr) * gn[2 * e], fmaf(hi(dQr[c][e]), r, qh * dr) * gn[2 * e + 1]);
            dQr[c][e] = dn;
          }
          Qr[c][e] = qn;
        }
      }
      if (p.q_hat != nullptr && qrow < p.Lq) {   // normalised rows for the backward pass (before the softmax scale goes in)
        T* dst = reinterpret_cast<T*>(p.q_hat) + (((int64_t)b * p.Lq + qrow) * p.H + h) * D + 8 * g;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c)
          if (2 * c + g < VPR) *reinterpret_cast<u32x4*>(dst + 16 * c) = Qr[c];
      }
    }
    auto scaled = [&](u32x4 x) {
      u32x4 y;
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = pack_bf16x2(lo(x[e]) * p.scale, hi(x[e]) * p.scale);
      return y;
    };
    // MERGE (tangents, half-empty last chunk): the two last-chunk products of the tangent scores, K dQ^T and dK Q^T over
    // head-dim columns 16(NCHUNK-1) .., fill half of the contraction slots each; they are issued as ONE MFMA whose A
    // operand takes K in the lower half of the slots and dK in the upper half (a per-lane LDS address) against
    // mB = [dQ | Q] -- one MFMA and one LDS read fewer per tile.
    constexpr bool MERGE = JVP && 2 * NCHUNK > VPR;
    if constexpr (MERGE) {
      auto sc = [&](uint32_t w) { return pack_bf16x2(lo(w) * p.scale, hi(w) * p.scale); };
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t qs = sc(Qr[NCHUNK - 1][e]);
        auto r = __builtin_amdgcn_permlane32_swap(qs, qs, false, false);   // r[0] of a lane above 31 = the value of lane - 32
        mB[e] = g ? r[0] : sc(dQr[NCHUNK - 1][e]);
      }
    }
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
      if constexpr (MFOLD) {
#pragma unroll
        for (int e = 0; e < 4; ++e) QrS[c][e] = pack_bf16x2(lo(Qr[c][e]) * p.scale_log2, hi(Qr[c][e]) * p.scale_log2);
      }
      Qr[c] = scaled(Qr[c]);
      if constexpr (JVP) dQr[c] = scaled(dQr[c]);
    }
    if constexpr (QPARK > 0) {
#pragma unroll
      for (int k = 0; k < QPARK; ++k) {
        char* px = smem + QX_OFF + ((2 * k * NW + wave) * 64 + lane) * 16;
        *reinterpret_cast<u32x4*>(px) = Qr[NCHUNK - QPARK + k];
        *reinterpret_cast<u32x4*>(px + NW * 64 * 16) = dQr[NCHUNK - QPARK + k];
      }
    }
  }
  const uint32_t qx_lane_addr = lds_addr(smem) + QX_OFF + (wave * 64 + lane) * 16;

  // first key tile on its way (issued after the Q loads: measured faster than issuing it first)
  if constexpr (!QLDS) issue(0);

  constexpr int NMT = F::NMT;
  constexpr bool TAIL = F::TAIL;
  f32x16 O[NMT], dO[JVP ? NMT : 1];        // full 32-wide tiles of O^T / dO^T
  f32x4 O16[2], dO16[2];                   // TAIL: 16-wide remainder, one 16x16 tile per half of the wave's 32 queries
#pragma unroll
  for (int t = 0; t < NMT; ++t) {
    O[t] = f32x16{0};
    if constexpr (JVP) dO[t] = f32x16{0};
  }
#pragma unroll
  for (int hq = 0; hq < 2; ++hq) {
    O16[hq] = f32x4{0, 0, 0, 0};
    dO16[hq] = f32x4{0, 0, 0, 0};
  }
  float m_run = F::MFOLD ? 0.f : -INFINITY, l_run = 0.f, mu_run = 0.f;   // log2-domain running max; VALU row sums only when !PADROW

  // Lane address for the transposed V / dV operand reads (see lds_col_operand):
  // 16 lanes fetch a 4-row x 16-column block, lane i supplying row i/4, columns 4*(i%4)..+3.
  constexpr int DV_OFF = F::KBYTES + F::VBYTES;   // dV tile sits this many bytes after the V tile
  const uint32_t k_lane_addr = lds_addr(smem) + c32 * KSTR * 2 + g * 16;   // row-operand reads of K / dK
  // merged last tangent-score chunk: K's last valid vector for the lower half of the wave, dK's for the upper half
  constexpr bool MERGE = JVP && 2 * NCHUNK > VPR;
  const uint32_t m_lane_addr = lds_addr(smem) + c32 * KSTR * 2 + (VPR - 1) * 16 + g * (F::KBYTES + F::VBYTES);
  const uint32_t v_lane_addr =
      lds_addr(smem) + F::KBYTES + ((4 * g + ((lane & 15) >> 2)) * VSTR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
  // Remainder (16x16x32) operand: 16-lane row w covers keys 16*(w%2) + 4*(w/2) + {0..3, 8..11} -- the keys whose
  // probabilities that row receives from swap16 -- at head-dim columns 32*NMT .. 32*NMT+15.
  const uint32_t t_lane_addr = lds_addr(smem) + F::KBYTES + tail_lane_offset(lane, VSTR, 32 * F::NMT) * 2;

  // KN: a 16-lane group owns one key row of the tile (lane i of the group: elements 8i .. 8i+7), a wave 4 rows per pass.
  float kgain[8];
  if constexpr (KN) {
#pragma unroll
    for (int e = 0; e < 8; ++e) kgain[e] = (lane & 15) < VPR ? p.k_gain[8 * (lane & 15) + e] : 0.f;
  }

  const int ntiles = (p.Lkv + BKV - 1) / BKV;
  for (int it = 0; it < ntiles; ++it) {
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's share of tile `it` has landed in LDS
    const int s = it & 1;
    if constexpr (KN) {
      // k_hat = k r g, dk_hat = (dk r + k dr) g with r = (mean k^2 + eps)^-1/2, dr = -r^3 mean(k dk): models/layers.py:39-42 and
      // its tangent, element for element the arithmetic of the stand-alone norm kernel; rounded to bf16 in place.
      // A wave normalises exactly the rows that it fetched itself (issue_tile_rows: rows RPW*wave .. +RPW-1 of K and dK), so
      // its own vmcnt wait is all it needs and the barrier below publishes the normalised rows: no second barrier.
      constexpr int RPW = 32 / NW;
      auto lo = [](uint32_t w) { return __uint_as_float(w << 16); };
      auto hi = [](uint32_t w) { return __uint_as_float(w & 0xffff0000u); };
#pragma unroll
      for (int ps = 0; ps < RPW / 4; ++ps) {
        const int row = RPW * wave + 4 * ps + (lane >> 4), cv = lane & 15;
        const bool live = cv < VPR;
        char* ka = Kt(s) + (row * KP + (live ? cv : 0)) * 16;
        u32x4 kv = *reinterpret_cast<const u32x4*>(ka), tkv = u32x4{0, 0, 0, 0};
        if constexpr (JVP) tkv = *reinterpret_cast<const u32x4*>(ka + DV_OFF);
        if (!live) kv = tkv = u32x4{0, 0, 0, 0};
        float x[8], t[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          x[2 * e] = lo(kv[e]);
          x[2 * e + 1] = hi(kv[e]);
          t[2 * e] = lo(tkv[e]);
          t[2 * e + 1] = hi(tkv[e]);
        }
        float ss = 0.f, st = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          ss = fmaf(x[e], x[e], ss);
          if constexpr (JVP) st = fmaf(x[e], t[e], st);
        }
        // (rows past the end of the sequence were zero-filled and must stay zero: with eps == 0 their r would be infinite)
        const float r = it * BKV + row < p.Lkv ? 1.f / sqrtf(group16_sum(ss) * (1.f / D) + p.q_eps) : 0.f;
        const float dr = JVP ? -r * r * r * group16_sum(st) * (1.f / D) : 0.f;
        if (live) {
          u32x4 kn, tkn;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            kn[e] = pack_bf16x2(x[2 * e] * r * kgain[2 * e], x[2 * e + 1] * r * kgain[2 * e + 1]);
            if constexpr (JVP)
              tkn[e] = pack_bf16x2(fmaf(t[2 * e], r, x[2 * e] * dr) * kgain[2 * e], fmaf(t[2 * e + 1], r, x[2 * e + 1] * dr) * kgain[2 * e + 1]);
          }
          *reinterpret_cast<u32x4*>(ka) = kn;
          if constexpr (JVP) *reinterpret_cast<u32x4*>(ka + DV_OFF) = tkn;
          const int key = it * BKV + row;
          if (p.k_hat != nullptr && qb == 0 && key < p.Lkv)   // the first query block of the head hands the rows to the backward pass
            *reinterpret_cast<u32x4*>(reinterpret_cast<T*>(p.k_hat) + (((int64_t)b * p.Lkv + key) * p.H + h) * D + 8 * cv) = kn;
        }
      }
    }

    lds_barrier();                         // ... and everyone else's; also: all waves are done with the other stage
    const bool fetch = it + 1 < ntiles;    // tile it + 1 goes into the other stage, in parts between the score MFMAs
    // ---- S^T (already scaled) and dS^T; the LDS reads of chunk c+1 are in
    //      flight while the MFMAs of chunk c run
    f32x16 S = {0}, dS = {0};
    {
      const uint32_t ka = k_lane_addr + s * STAGE;
      u32x4 kc[2], dkc[2], qx[2], dqx[2];
      static_assert(QPARK < NCHUNK, "the first chunk's operands stay in registers");
      // Q operand of the score product: the copy pre-multiplied by scale * log2e where the maximum rides in the MFMA
      auto score_q = [&](auto cc, const u32x4& plain) -> const u32x4& {
        if constexpr (MFOLD) return QrS[decltype(cc)::value];
        else return plain;
      };
      kc[0] = lds_read128_issue<0>(ka);
      if constexpr (JVP) dkc[0] = lds_read128_issue<DV_OFF>(ka);
      static_for<NCHUNK>([&](auto cc) {
        constexpr int c = decltype(cc)::value;
        constexpr bool more = c + 1 < NCHUNK;
        constexpr bool parked = c >= NCHUNK - QPARK, next_parked = more && c + 1 >= NCHUNK - QPARK;
        if constexpr (more) {
          kc[(c + 1) & 1] = lds_read128_issue<32 * (c + 1)>(ka);
          if constexpr (MERGE && c + 2 == NCHUNK) dkc[(c + 1) & 1] = lds_read128_issue<0>(m_lane_addr + s * STAGE);   // [K | dK], last vectors
          else if constexpr (JVP) dkc[(c + 1) & 1] = lds_read128_issue<32 * (c + 1) + DV_OFF>(ka);
          if constexpr (next_parked) {
            constexpr int k = c + 1 - (NCHUNK - QPARK);
            qx[(c + 1) & 1] = lds_read128_issue<2 * k * NW * 64 * 16>(qx_lane_addr);
            dqx[(c + 1) & 1] = lds_read128_issue<(2 * k + 1) * NW * 64 * 16>(qx_lane_addr);
          }
        }
        if constexpr (JVP) {
          constexpr int newer = more ? (next_parked ? 4 : 2) : 0;   // reads issued since this chunk's
          if constexpr (parked) lds_read128_wait<newer>(kc[c & 1], dkc[c & 1], qx[c & 1], dqx[c & 1]);
          else lds_read128_wait<newer>(kc[c & 1], dkc[c & 1]);
          const u32x4& qc = parked ? qx[c & 1] : Qr[c];
          const u32x4& dqc = parked ? dqx[c & 1] : dQr[c];
          mma_chunk<T>(S, kc[c & 1], score_q(cc, qc));
          if constexpr (MERGE && c + 1 == NCHUNK) {
            mma_chunk<T>(dS, dkc[c & 1], mB);
          } else {
            mma_chunk<T>(dS, kc[c & 1], dqc);
            mma_chunk<T>(dS, dkc[c & 1], qc);
          }
        } else {
          lds_read128_wait<more ? 1 : 0>(kc[c & 1]);
          mma_chunk<T>(S, kc[c & 1], score_q(cc, Qr[c]));
        }
        if constexpr (c < NPART) {
          if (fetch) issue_part(it + 1, cc);
        }
      });
    }
    // ---- keys past the end: their K/V rows were zero-filled by the bounds check, mask the scores
    if ((it + 1) * BKV > p.Lkv) {
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (it * BKV + acc_row(i, g) >= p.Lkv) S[i] = -INFINITY;
    }
    // ---- lazy running maximum
    float mx = fmaxf(S[0], S[1]);
#pragma unroll
    for (int i = 2; i < 16; ++i) mx = fmaxf(mx, S[i]);
    mx = MFOLD ? xhalf_max(mx) : xhalf_max(mx) * kLog2e;   // MFOLD: the scores arrive as S*log2(e) - m_run
    if (MFOLD ? (it == 0 || __builtin_amdgcn_ballot_w64(mx > kLazyLog2) != 0) : __builtin_amdgcn_ballot_w64(mx > m_run + kLazyLog2) != 0) {
      float m_new, alpha;
      if constexpr (MFOLD) {
        // The first tile sets the maximum whatever its sign (m_run starts at 0, not -inf: it is a product term); later it is
        // only raised.  This tile's scores, formed against the old maximum, are shifted by hand.
        m_new = it == 0 ? m_run + mx : fmaxf(m_run, m_run + mx);
        const float shift = m_new - m_run;
#pragma unroll
        for (int i = 0; i < 16; ++i) S[i] -= shift;
        alpha = it == 0 ? 0.f : fast_exp2(-shift);          // (nothing accumulated yet behind the first tile)
        if (g == 1) QrS[NCHUNK - 1] = split3_bf16(-m_new);
      } else {
        m_new = fmaxf(m_run, mx);
        alpha = fast_exp2(m_run - m_new);
      }
      m_run = m_new;
      if constexpr (!F::PADROW) {
        l_run *= alpha;
        if constexpr (JVP) mu_run *= alpha;
      }
#pragma unroll
      for (int t = 0; t < NMT; ++t) {
        O[t] *= alpha;
        if constexpr (JVP) dO[t] *= alpha;
      }
      if constexpr (TAIL) {
        float a0, a1;   // alpha of query (lane % 16) and of query 16 + (lane % 16)
        swap16f(alpha, a0, a1);
        O16[0] *= a0;
        O16[1] *= a1;
        if constexpr (JVP) {
          dO16[0] *= a0;
          dO16[1] *= a1;
        }
      }
    }
    // ---- E = exp2(S log2e - m), G = E * dS
    f32x16 E, G;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      E[i] = MFOLD ? fast_exp2(S[i]) : fast_exp2(fmaf(S[i], kLog2e, -m_run));
      if constexpr (JVP) G[i] = E[i] * dS[i];
      if constexpr (!F::PADROW) {
        l_run += E[i];
        if constexpr (JVP) mu_run += G[i];
      }
    }
    // ---- O^T += V^T P^T ; dO^T += V^T G^T + dV^T P^T, over 2*NMT operand groups
    //      (step st, head-dim tile t) plus, with TAIL, one 16-wide remainder group;
    //      group i+1 is read while group i multiplies
    {
      const uint32_t va = v_lane_addr + s * STAGE;   // this lane's transposed-read address in the stage's V tile
      ColOperand pe[2], pg[2];
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        pe[st] = acc_operand<T>(E, st);
        if constexpr (JVP) pg[st] = acc_operand<T>(G, st);
      }
      constexpr int NG = 2 * NMT, NGT = NG + (TAIL ? 1 : 0);
      TrPair v[2], dv[2];
      auto lo_off = [](int gi) constexpr { return (16 * (gi / NMT) * VSTR + 32 * (gi % NMT)) * 2; };
      v[0] = lds_tr16_issue<lo_off(0), lo_off(0) + 8 * VSTR * 2>(va);
      if constexpr (JVP) dv[0] = lds_tr16_issue<lo_off(0) + DV_OFF, lo_off(0) + 8 * VSTR * 2 + DV_OFF>(va);
      static_for<NGT>([&](auto gc) {
        constexpr int gi = decltype(gc)::value;
        constexpr bool more = gi + 1 < NGT;
        if constexpr (gi + 1 < NG) {
          constexpr int LO = lo_off(gi + 1), HI = LO + 8 * VSTR * 2;
          v[(gi + 1) & 1] = lds_tr16_issue<LO, HI>(va);
          if constexpr (JVP) dv[(gi + 1) & 1] = lds_tr16_issue<LO + DV_OFF, HI + DV_OFF>(va);
        } else if constexpr (more) {   // the remainder group: all 32 keys in one 16x16x32 operand
          const uint32_t ta = t_lane_addr + s * STAGE;
          v[(gi + 1) & 1] = lds_tr16_issue<0, 8 * VSTR * 2>(ta);
          if constexpr (JVP) dv[(gi + 1) & 1] = lds_tr16_issue<DV_OFF, 8 * VSTR * 2 + DV_OFF>(ta);
        }
        if constexpr (JVP) lds_tr16_wait<more ? 4 : 0>(v[gi & 1], dv[gi & 1]);
        else lds_tr16_wait<more ? 2 : 0>(v[gi & 1]);
        if constexpr (gi < NG) {
          constexpr int st = gi / NMT, t = gi % NMT;
          mma_col<T>(O[t], tr_operand(v[gi & 1]), pe[st]);
          if constexpr (JVP) {
            mma_col<T>(dO[t], tr_operand(v[gi & 1]), pg[st]);
            mma_col<T>(dO[t], tr_operand(dv[gi & 1]), pe[st]);
          }
        } else {
          // B operands for the two query halves: lanes of 16-lane row w take (half g = w/2, step st = w%2)
          ColOperand pe0, pe1, pg0, pg1;
          tail_operands(pe[0], pe[1], pe0, pe1);
          if constexpr (JVP) tail_operands(pg[0], pg[1], pg0, pg1);
          mma16(O16[0], tr_operand(v[gi & 1]), pe0);
          mma16(O16[1], tr_operand(v[gi & 1]), pe1);
          if constexpr (JVP) {
            mma16(dO16[0], tr_operand(v[gi & 1]), pg0);
            mma16(dO16[1], tr_operand(v[gi & 1]), pg1);
            mma16(dO16[0], tr_operand(dv[gi & 1]), pe0);
            mma16(dO16[1], tr_operand(dv[gi & 1]), pe1);
          }
        }
      });
    }
  }

  // ---- epilogue
  float l_tot, mu_tot = 0.f;
  if constexpr (F::PADROW && TAIL) {
    // row D of the remainder tiles: 16-lane row PAD16_ROW holds it for query (lane % 16) [+16 in the second tile]
    const int src = 16 * F::PAD16_ROW + (c32 & 15);
    const float x0 = __shfl(O16[0][F::PAD16_E], src), x1 = __shfl(O16[1][F::PAD16_E], src);
    l_tot = c32 < 16 ? x0 : x1;
    if constexpr (JVP) {
      const float y0 = __shfl(dO16[0][F::PAD16_E], src), y1 = __shfl(dO16[1][F::PAD16_E], src);
      mu_tot = c32 < 16 ? y0 : y1;
    }
  } else if constexpr (F::PADROW) {
    auto pick = [&](float x) {
      auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
      return __uint_as_float(r[F::PAD_G]);
    };
    l_tot = pick(O[NMT - 1][F::PAD_IDX]);
    if constexpr (JVP) mu_tot = pick(dO[NMT - 1][F::PAD_IDX]);
  } else {
    l_tot = xhalf_sum(l_run);
    if constexpr (JVP) mu_tot = xhalf_sum(mu_run);
  }
  const float inv_l = 1.0f / l_tot;
  const float mu_n = mu_tot * inv_l;
  {
    const int qrow = q0 + wave * 32 + c32;
    if (g == 0 && qrow < p.Lq) {
      if (p.lse != nullptr) p.lse[(int64_t)bh * p.Lq + qrow] = (m_run + log2f(l_tot)) * kLn2;
      if constexpr (JVP)
        if (p.dlse != nullptr) p.dlse[(int64_t)bh * p.Lq + qrow] = mu_n;
    }
  }
  T* stage = reinterpret_cast<T*>(smem);
  // remainder columns: lane (i = lane % 16, w = lane / 16) holds head-dim 32*NMT + 4w .. +3 of query i (tile 0) / 16 + i (tile 1)
  float inv16[2] = {inv_l, inv_l}, mun16[2] = {mu_n, mu_n};
  if constexpr (TAIL) {
    swap16f(inv_l, inv16[0], inv16[1]);
    swap16f(mu_n, mun16[0], mun16[1]);
  }
  auto tail_o = [&](void* ws) {
    if constexpr (TAIL) store_tail16<T, D, NMT>(ws, lane, [&](int hq, int e) { return O16[hq][e] * inv16[hq]; });
  };
  auto tail_to = [&](void* ws) {
    if constexpr (TAIL && JVP)
      store_tail16<T, D, NMT>(ws, lane, [&](int hq, int e) { return fmaf(-mun16[hq], O16[hq][e] * inv16[hq], dO16[hq][e] * inv16[hq]); });
  };
  store_rows_transposed<T, D, NW, NMT>(stage, reinterpret_cast<T*>(p.o) + base(6), p.st[6][1], q0, p.Lq, tid,
                                       [&](int t, int i) { return O[t][i] * inv_l; }, tail_o);
  if constexpr (JVP)
    store_rows_transposed<T, D, NW, NMT>(stage, reinterpret_cast<T*>(p.to) + base(7), p.st[7][1], q0, p.Lq, tid,
                                         [&](int t, int i) { return fmaf(-mu_n, O[t][i] * inv_l, dO[t][i] * inv_l); }, tail_to);
}

template <int D, bool JVP, int NW, bool QN, bool KN>
static int launch_fast_q(const FwdParams& p, int BH, hipStream_t stream) {
  using F = FastCfg<D>;
  constexpr int tiles = 2 * (JVP ? 2 : 1) * (F::KBYTES + F::VBYTES) + 512;
  constexpr int stage = 32 * NW * Cfg<__bf16, D>::OROWV * 16;
  constexpr int qst = (JVP ? 2 : 1) * 32 * NW * F::QP * 16;                       // Q / dQ staging of the 8-wave kernel (see QLDS there)
  constexpr int park = (JVP && NW == 8 ? F::QPARK_JVP : 0) * 2 * NW * 64 * 16;                 // parked Q / dQ operand chunks
  constexpr int need = (NW == 8 && tiles + qst <= 160 * 1024) ? tiles + qst : tiles + park;
  static_assert(need <= 160 * 1024, "LDS budget");
  constexpr int smem = need > stage ? need : stage;
  auto kern = attn_fwd_bf16_kernel<D, JVP, NW, QN, KN>;
  static bool lds_ok[64] = {};
  if (!ensure_dynamic_lds(kern, smem, lds_ok)) return -7;
  const uint32_t nqb = (p.Lq + 32 * NW - 1) / (32 * NW);
  return launch_kernel(kern, dim3(nqb * (uint32_t)BH), dim3(64 * NW), smem, stream, p);
}

template <int D, bool JVP, int NW>
static int launch_fast_t(const FwdParams& p, int BH, hipStream_t stream) {
  if (p.q_gain != nullptr) {
    if (reinterpret_cast<uintptr_t>(p.q_gain) % 16) return -6;
    if (p.k_gain != nullptr) return launch_fast_q<D, JVP, NW, true, true>(p, BH, stream);
    return launch_fast_q<D, JVP, NW, true, false>(p, BH, stream);
  }
  return launch_fast_q<D, JVP, NW, false, false>(p, BH, stream);
}

// Work-group width policy.  256-row work-groups (8 waves, one per CU with tangents) fetch every key tile once per 256
// queries -- half the tile traffic per FLOP -- and are the default when the sequence fills them.  128-row work-groups
// are resident two per CU (three where the kernel needs at most 168 registers: head dim 64 with tangents), so one's
// first and last rows overlap another's tiles.  Measured on MI355X (fwd+JVP, 8 waves vs 4):
//   * head dim 64, three per CU: 4 waves win once the grid gives every CU three of them
//     (B64 N1024 0.779 -> 0.749 ms, B256 N256 0.293 -> 0.269, B64 H12 N256 0.056 -> 0.048; smaller grids lose);
//   * other head dims, N <= 256: 4 waves win only where 8-wave work-groups would run in two or three rounds
//     (B32 H16: 0.0438 -> 0.0413 ms, B48: 0.070 -> 0.062) and lose 2-3 % from four rounds on;
//   * without tangents the 8-wave kernel fits twice per CU and is slower only at head dim 64 on large grids.
static bool fwd_wide_workgroups(int Lq, int D, bool jvp, int BH) {
  if (Lq <= 128) return false;
  const int cus = compute_units();
  // (without tangents only head dim 64 on a grid of at least eight narrow work-groups per CU prefers them:
  //  B256 H16 N256 0.129 -> 0.123 ms, B64 N1024 0.331 -> 0.326; the DMFT-B/2 call B64 H12 N256 is equal either way)
  if (!jvp) return !(D == 64 && (int64_t)BH * ((Lq + 127) / 128) >= 8 * (int64_t)cus);
  if (D == 64) return (int64_t)BH * ((Lq + 127) / 128) < 3 * (int64_t)cus;
  if (Lq <= 256) {
    const int64_t rounds = ((int64_t)BH * ((Lq + 255) / 256) + cus - 1) / cus;
    return rounds < 2 || rounds > 3;
  }
  return true;
}

bool plan_fwd_bf16_fast(int Lq, int D, bool jvp, int BH, bool q_norm, bool k_norm, char* buf, size_t n) {
  if (D != 64 && D != 72 && D != 80 && D != 96 && D != 128) return false;
  const auto tf = [](bool x) { return x ? "true" : "false"; };
  snprintf(buf, n, "dmf::attn_fwd_bf16_kernel<%d, %s, %d, %s, %s>", D, tf(jvp), fwd_wide_workgroups(Lq, D, jvp, BH) ? 8 : 4,
           tf(q_norm), tf(q_norm && k_norm));
  return true;
}

// Returns 1 if this translation unit has no kernel for the case (caller falls
// back to the generic kernel), else 0 / negative error code.
int launch_fwd_bf16_fast(const FwdParams& p, int BH, int D, bool jvp, hipStream_t stream) {
  // 32-bit buffer addressing: every (batch, head) slab of K/V rows must span < 2 GiB
  int64_t max_row = std::max(std::max(p.st[0][1], p.st[1][1]), p.st[2][1]);
  if (jvp) max_row = std::max(max_row, std::max(std::max(p.st[3][1], p.st[4][1]), p.st[5][1]));
  if (max_row * 2 * (int64_t)(std::max(p.Lq, p.Lkv) + 256) >= (int64_t)1 << 31) return 1;
  const bool wide = fwd_wide_workgroups(p.Lq, D, jvp, BH);
#define DMF_CASE(DD)                                                                           \
  case DD:                                                                                     \
    if (wide) return jvp ? launch_fast_t<DD, true, 8>(p, BH, stream) : launch_fast_t<DD, false, 8>(p, BH, stream); \
    return jvp ? launch_fast_t<DD, true, 4>(p, BH, stream) : launch_fast_t<DD, false, 4>(p, BH, stream);
  switch (D) {
    DMF_CASE(64)
    DMF_CASE(72)
    DMF_CASE(80)
    DMF_CASE(96)
    DMF_CASE(128)
    default: return 1;
  }
#undef DMF_CASE
}

}  // namespace dmf
