// Tuned bf16 backward for gfx950: the dQ kernel + dK/dV kernel pair (any length) and the single-pass kernel for
// sequences of at most 256 rows (further down).
//
// The pair is the two-kernel, atomics-free scheme of the generic kernels in attn_bwd.hip with the same register
// layouts and the throughput structure of the tuned forward: 32-row tiles streamed HBM -> LDS by bounds-checked
// buffer DMA into a double buffer with one barrier per tile, software-pipelined LDS operand reads, the softmax scale
// and log2(e) folded into the register-resident operand (Q in the dQ kernel, K in the dK/dV kernel).  Per tile each
// kernel issues its products as separate MFMA runs with the P / dS arithmetic pinned between the MFMAs of the run that
// does not depend on it; the end-of-sequence selects sit behind wave-uniform branches (last tile only); at head dim 72
// the statistics (-lse*log2e, -delta) ride in spare head-dim columns so that S - lse and dP - delta come out of the
// MFMAs (BwdFastCfg::STATCOL); tile pitches are free of bank conflicts for row and transposed reads alike.
#include "attn_common.h"
#include "attn_kernels.h"
#include <algorithm>
#include <cstdio>

// Nothing is scheduled across a pin, and a block that holds one is not turned into selects.
#define DMF_PIN() __builtin_amdgcn_sched_barrier(0)

namespace dmf {

// Waves per dK/dV work-group: four (eight halve the L2 -> LDS tile traffic but measured equal at head dim 72 and 8 % slower
// at head dim 64, where they leave one work-group per CU instead of three).
constexpr int kKvWaves = 4;
// 32-key tiles per barrier in the dQ kernel: two (+3 % over one; four would leave one work-group per CU).
constexpr int kDqSub = 2;
// The single-pass kernel takes sequences of 129 .. 256 rows; up to 128 rows a (batch, head) unit would occupy half of
// its eight waves and the kernel pair is faster.
constexpr int kFusedMinRows = 129, kFusedMaxRows = 256;

// Tile row pitch in 16-byte vectors.  Odd, so that the row-operand reads (ds_read_b128, 16 lanes a cycle over 64 banks)
// are conflict-free; with TRFREE also such that four consecutive rows start at least two vectors apart modulo 16, so
// that a transposed read (ds_read_b64_tr_b16: 16 lanes fetch 32 bytes of each of four consecutive rows) is
// conflict-free too -- pitches of 11 or 17 vectors put rows 0 and 3 (0 and 1) on the same banks and cost the read a
// second cycle.
constexpr int bwd_tile_pitch(int min_vectors, bool trfree) {
  for (int p = min_vectors | 1;; p += 2) {
    const int m = p % 16;
    if (!trfree || m == 3 || m == 7 || m == 9 || m == 13) return p;
  }
}

template <int D, bool TRFREE = false>
struct BwdFastCfg {
  static constexpr int VPR = D / 8, NCHUNK = (D + 15) / 16, NDT = (D + 31) / 32;
  static constexpr int P = TRFREE ? bwd_tile_pitch(Cfg<__bf16, D>::ROWV0, true) : Cfg<__bf16, D>::ROWV;   // tiles are read both by rows and transposed
  static constexpr int STR = P * 8;
  static constexpr int TBYTES = 32 * P * 16;          // one 32-row tile
  static constexpr int STAT = 256;                    // per stage: 32 x lse, 32 x delta (fp32)
  static constexpr bool TAIL = (D % 32) != 0 && (D % 32) <= 16;   // 16-wide remainder via 16x16x32 MFMAs (72, 80)
  static constexpr int NMT = TAIL ? D / 32 : NDT;                 // full 32-wide output tiles
  // The last 16-wide chunk of the score products has spare columns D .. (head dims 72, 104, 120).  Three of them carry
  // a per-row constant as a bf16 triple against ones on the other side, so that the MFMA itself yields S - lse and
  // dP - delta and the VALU subtractions go away.
  static constexpr bool STATCOL = (D % 16) == 8;
};

// Pad vector of a tile row whose first three elements are 1.0 (see BwdFastCfg::STATCOL).
__device__ __forceinline__ u32x4 ones3_bf16() { return u32x4{0x3f803f80u, 0x00003f80u, 0u, 0u}; }

// bf16x8 chunk times a scalar, re-rounded to bf16.
__device__ __forceinline__ u32x4 scale_bf16x8(u32x4 x, float s) {
  u32x4 y;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    y[e] = pack_bf16x2(__uint_as_float(x[e] << 16) * s, __uint_as_float(x[e] & 0xffff0000u) * s);
  return y;
}

// Fills the pad vectors of a 32-row tile in both stages (the tile DMA never writes them) with zeros; the first pad
// vector of a row with the 1, 1, 1, 0 ... pattern instead (PAD_ONES) or not at all (PAD_SKIP: its owner writes it).
enum { PAD_ZERO = 0, PAD_ONES = 1, PAD_SKIP = 2 };
template <int BYTES_PER_STAGE, int PADV, int P, int VPR, int FIRST = PAD_ZERO, int NT = 256>
__device__ __forceinline__ void zero_pads(char* smem, int tile_off, int tid) {
  if constexpr (PADV > 0) {
#pragma unroll
    for (int s = 0; s < 2; ++s)
      for (int i = tid; i < 32 * PADV; i += NT) {
        if (FIRST == PAD_SKIP && i % PADV == 0) continue;
        *reinterpret_cast<u32x4*>(smem + s * BYTES_PER_STAGE + tile_off + ((i / PADV) * P + VPR + i % PADV) * 16) =
            FIRST == PAD_ONES && i % PADV == 0 ? ones3_bf16() : u32x4{0, 0, 0, 0};
      }
  }
}

// 8-byte LDS store issued as a raw instruction, for the same reason as the untracked reads in attn_common.h (a store
// the compiler knows about would be preceded by a full vmcnt(0) while a tile DMA is in flight).  The data is in LDS
// once a later `s_waitcnt lgkmcnt(0)` of this wave has passed (LDS operations complete in order).
template <int OFF>
__device__ __forceinline__ void lds_write64_untracked(uint32_t addr, u32x2 w) {
  asm volatile("ds_write_b64 %0, %1 offset:%2" : : "v"(addr), "v"(w), "n"(OFF) : "memory");
}

template <int OFF>
__device__ __forceinline__ void lds_write128_untracked(uint32_t addr, u32x4 w) {
  asm volatile("ds_write_b128 %0, %1 offset:%2" : : "v"(addr), "v"(w), "n"(OFF) : "memory");
}

// One transposed 8-byte LDS read issued as a raw instruction (see lds_tr16_issue in attn_common.h for the pair form).
template <int OFF>
__device__ __forceinline__ u32x2 lds_tr16_issue1(uint32_t lane_addr) {
  u32x2 r;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=&v"(r) : "v"(lane_addr), "n"(OFF));
  return r;
}

// 4-byte LDS read issued as a raw instruction; lgkmcnt must be waited for before the result is used.
__device__ __forceinline__ uint32_t lds_read32_issue(uint32_t addr) {
  uint32_t r;
  asm volatile("ds_read_b32 %0, %1" : "=v"(r) : "v"(addr));
  return r;
}

// ------------------------------------------------------------------ dQ kernel
// SUB = 32-key tiles per stage (and per work-group barrier).
template <int D, int SUB>
__global__ __launch_bounds__(256, 2) void attn_bwd_dq_bf16_kernel(const BwdParams p) {
  using F = BwdFastCfg<D, true>;
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
    zero_pads<STAGE, P - VPR, P, VPR, F::STATCOL ? PAD_ONES : PAD_ZERO>(smem, sub * PAIR, tid);
    zero_pads<STAGE, P - VPR, P, VPR, F::STATCOL ? PAD_ONES : PAD_ZERO>(smem, sub * PAIR + V_OFF, tid);
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
  float lse2 = 1e30f;   // switches padded query rows off (P = 0)
  if (qok) {
    lse2 = p.lse[(int64_t)bh * p.Lq + qrow] * kLog2e;
    if (g == 0) p.delta[(int64_t)bh * p.Lq + qrow] = delta;
  }
  if constexpr (F::STATCOL) {   // columns D .. D+2 of this row: -lse against the ones in the K tile, -delta against those in the V tile
    if (g == 1) {
      Qr[NCHUNK - 1] = split3_bf16(-lse2);
      dOr[NCHUNK - 1] = split3_bf16(-delta);
    }
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

    // ---- Three MFMA runs per 32-key tile: S^T = K Q^T (log2 units), dP^T = V dout^T, dQ^T += K^T dS^T.  P^T = exp2(S^T - lse)
    //      is formed between the MFMAs of the dP run and the second half of dS^T = P^T (dP^T - delta) behind the first MFMA of
    //      the dQ run (an MFMA holds the matrix pipe for 32 cycles but the issue port for 4, and a wave issues in order; left
    //      alone the scheduler gathers the MFMAs, hence the pins).
    f32x16 S = {0}, dP = {0}, Pm, dS;
    ColOperand ds[2];
    const bool tail = (it + 1) * 32 > p.Lkv;   // keys past the end (last tile only): the pin keeps the selects out of the common path
    auto p_slice = [&](auto jc) {
      constexpr int jj = decltype(jc)::value;
#pragma unroll
      for (int e = 0; e < 4; ++e) Pm[4 * jj + e] = fast_exp2(F::STATCOL ? S[4 * jj + e] : S[4 * jj + e] - lse2);
    };
    auto ds_half = [&](auto hc) {
      constexpr int hh = decltype(hc)::value;
#pragma unroll
      for (int i = 8 * hh; i < 8 * hh + 8; ++i) dS[i] = Pm[i] * (F::STATCOL ? dP[i] : dP[i] - delta);
      if (tail) {
        DMF_PIN();
#pragma unroll
        for (int i = 8 * hh; i < 8 * hh + 8; ++i)
          if (it * 32 + acc_row(i, g) >= p.Lkv) dS[i] = 0.f;
      }
      ds[hh] = acc_operand<T>(dS, hh);
    };
    constexpr int NG = 2 * NMT, NGT = NG + (TAIL ? 1 : 0);
    TrPair kk[2];
    auto lo_off = [](int gi) constexpr { return (16 * (gi / NMT) * STR + 32 * (gi % NMT)) * 2; };
    static_assert(NCHUNK >= 4, "the four P slices ride between the first four dP MFMAs");
    {
      u32x4 kc[2], vc[2];
      kc[0] = lds_read128_issue<0>(ra);
      static_for<NCHUNK>([&](auto cc) {   // run 1: S^T
        constexpr int c = decltype(cc)::value;
        if constexpr (c + 1 < NCHUNK) kc[(c + 1) & 1] = lds_read128_issue<32 * (c + 1)>(ra);
        else vc[0] = lds_read128_issue<V_OFF>(ra);   // first operand of the next run
        lds_read128_wait<1>(kc[c & 1]);
        mma_chunk<T>(S, kc[c & 1], Qr[c]);
      });
      static_for<NCHUNK>([&](auto cc) {   // run 2: dP^T, P^T formed meanwhile
        constexpr int c = decltype(cc)::value;
        if constexpr (c + 1 < NCHUNK) {
          vc[(c + 1) & 1] = lds_read128_issue<32 * (c + 1) + V_OFF>(ra);
          lds_read128_wait<1>(vc[c & 1]);
        } else {   // first operand of the next run
          kk[0] = lds_tr16_issue<lo_off(0), lo_off(0) + 8 * STR * 2>(ca);
          lds_read128_wait<2>(vc[c & 1]);
        }
        DMF_PIN();
        mma_chunk<T>(dP, vc[c & 1], dOr[c]);
        DMF_PIN();
        if constexpr (c < 4) p_slice(cc);
        DMF_PIN();
      });
    }
    ds_half(std::integral_constant<int, 0>{});
    static_for<NGT>([&](auto gc) {   // run 3: dQ^T
      constexpr int gi = decltype(gc)::value;
      constexpr bool more = gi + 1 < NGT;
      if constexpr (gi + 1 < NG) kk[(gi + 1) & 1] = lds_tr16_issue<lo_off(gi + 1), lo_off(gi + 1) + 8 * STR * 2>(ca);
      else if constexpr (more) kk[(gi + 1) & 1] = lds_tr16_issue<0, 8 * STR * 2>(tail_addr + (is & 1) * STAGE + sub * PAIR);
      lds_tr16_wait<more ? 2 : 0>(kk[gi & 1]);
      DMF_PIN();
      if constexpr (gi < NG) {
        mma_col<T>(dQ[gi % NMT], tr_operand(kk[gi & 1]), ds[gi / NMT]);
      } else {
        ColOperand d0, d1;
        tail_operands(ds[0], ds[1], d0, d1);
        mma16(dQ16[0], tr_operand(kk[gi & 1]), d0);
        mma16(dQ16[1], tr_operand(kk[gi & 1]), d1);
      }
      DMF_PIN();
      if constexpr (gi == 0) ds_half(std::integral_constant<int, 1>{});
      DMF_PIN();
    });
   }
  }
  store_rows_transposed<T, D, 4, NMT>(reinterpret_cast<T*>(smem), reinterpret_cast<T*>(p.dq) + base(5), p.st[5][1], q0, p.Lq, tid,
                                      [&](int t, int i) { return dQ[t][i] * p.scale; },
                                      [&](void* ws) {
                                        if constexpr (TAIL) store_tail16<T, D, NMT>(ws, lane, [&](int hq, int e) { return dQ16[hq][e] * p.scale; });
                                      });
}

// --------------------------------------------------------------- dK/dV kernel
// NW waves of 32 keys each per work-group.
template <int D, int NW>
__global__ __launch_bounds__(64 * NW, 8 / NW) void attn_bwd_dkv_bf16_kernel(const BwdParams p) {
  using F = BwdFastCfg<D, true>;
  using T = __bf16;
  constexpr int VPR = F::VPR, NCHUNK = F::NCHUNK, NMT = F::NMT, P = F::P, STR = F::STR;
  constexpr bool TAIL = F::TAIL;
  constexpr int STAGE = 2 * F::TBYTES + F::STAT;   // Q | dout | lse[32], delta[32]
  constexpr int DO_OFF = F::TBYTES, STAT_OFF = 2 * F::TBYTES;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, g = lane >> 5;
  const uint32_t nkb = (p.Lkv + 32 * NW - 1) / (32 * NW);
  const uint32_t wg = xcd_remap(blockIdx.x, gridDim.x);
  const int bh = wg / nkb, kb = wg % nkb;
  const int b = bh / p.H, h = bh % p.H;
  const int k0 = kb * 32 * NW;
  auto base = [&](int t) { return (int64_t)b * p.st[t][0] + (int64_t)h * p.st[t][2]; };

  // SC: column D .. D+2 of a Q row carries -lse*log2e and of a dout row -delta (bf16 triples) against ones in this lane's
  // K and V rows, so S - lse and dP - delta come out of the MFMAs.  The stage's statistics area then holds lse / delta of
  // the FOLLOWING tile, and one wave per tile turns them into the pad vectors of the other stage while that tile's rows
  // are still on their way.
  constexpr bool SC = F::STATCOL;
  zero_pads<STAGE, P - VPR, P, VPR, SC ? PAD_SKIP : PAD_ZERO, 64 * NW>(smem, 0, tid);
  zero_pads<STAGE, P - VPR, P, VPR, SC ? PAD_SKIP : PAD_ZERO, 64 * NW>(smem, DO_OFF, tid);

  // ---- this lane's key row: K (times scale*log2e) and V stay in registers
  u32x4 Kr[NCHUNK], Vr[NCHUNK];
  {
    const int krow = k0 + wave * 32 + c32;
    const uint32_t rb_k = (uint32_t)p.st[2][1] * 2, rb_v = (uint32_t)p.st[3][1] * 2;
    load_row_chunks<NCHUNK, VPR>(make_rows_rsrc(reinterpret_cast<const T*>(p.k) + base(2), rb_k, p.Lkv, D * 2), rb_k, krow, g, Kr);
    load_row_chunks<NCHUNK, VPR>(make_rows_rsrc(reinterpret_cast<const T*>(p.v) + base(3), rb_v, p.Lkv, D * 2), rb_v, krow, g, Vr);
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) Kr[c] = scale_bf16x8(Kr[c], p.scale_log2);
    if constexpr (SC) {
      if (g == 1) Kr[NCHUNK - 1] = Vr[NCHUNK - 1] = ones3_bf16();
    }
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
    issue_tile_rows<P, VPR, NW>(rs_q, rb_q, (uint32_t)it * 32 * rb_q, st, wave, lane);
    issue_tile_rows<P, VPR, NW>(rs_do, rb_do, (uint32_t)it * 32 * rb_do, st + DO_OFF, wave, lane);
    if (wave < 2 && lane < 32)   // wave 0: lse[32], wave 1: delta[32] -- of this tile, with SC of the next one
      __builtin_amdgcn_raw_ptr_buffer_load_lds(wave == 0 ? rs_lse : rs_dl,
                                               (__attribute__((address_space(3))) void*)(st + STAT_OFF + wave * 128), 4,
                                               lane * 4, (uint32_t)(it + (SC ? 1 : 0)) * 128, 0, 0);
  };
  // pad vector of row (lane % 32) of the Q tile (lanes 0..31: x = lse) or the dout tile (lanes 32..63: x = delta)
  auto stat_vector = [&](float x, int row) {
    if (lane < 32) return split3_bf16(row < p.Lq ? -x * kLog2e : -1e30f);   // rows past the end: P = 0
    return split3_bf16(row < p.Lq ? -x : 0.f);
  };
  const uint32_t pad_addr = lds_addr(smem) + (lane < 32 ? 0 : DO_OFF) + (c32 * P + VPR) * 16;
  if constexpr (SC) {
    if (wave == 0) {   // tile 0
      float x = 0.f;
      if (c32 < p.Lq) x = (lane < 32 ? p.lse : p.delta)[(int64_t)bh * p.Lq + c32];
      *reinterpret_cast<u32x4*>(smem + (lane < 32 ? 0 : DO_OFF) + (c32 * P + VPR) * 16) = stat_vector(x, c32);
    }
  }
  const uint32_t row_addr = lds_addr(smem) + c32 * STR * 2 + g * 16;
  const uint32_t col_addr = lds_addr(smem) + ((4 * g + ((lane & 15) >> 2)) * STR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;

  const uint32_t tail_addr = lds_addr(smem) + tail_lane_offset(lane, STR, 32 * NMT) * 2;

  const int ntiles = (p.Lq + 31) / 32;
  issue(0);
  for (int it = 0; it < ntiles; ++it) {
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    lds_barrier();
    if (it + 1 < ntiles) issue(it + 1);
    const uint32_t so = (it & 1) * STAGE;
    const uint32_t ra = row_addr + so, ca = col_addr + so;
    // Query rows past the end are switched off through their lse (P = 0): the bounds check zero-fills their operands only
    // when consecutive rows are distinct addresses; a broadcast operand -- row stride 0, e.g. the gradient of a sum over
    // the sequence -- aliases them onto row 0 instead.
    if constexpr (SC) {
      if (it + 1 < ntiles && wave == (it & (NW - 1))) {   // pad vectors of tile it + 1, in the other stage
        uint32_t x = lds_read32_issue(lds_addr(smem) + so + STAT_OFF + lane * 4);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(x));
        // (in LDS before this wave's last operand read of the tile returns: LDS operations complete in order)
        lds_write128_untracked<0>(pad_addr + (STAGE - so), stat_vector(__uint_as_float(x), (it + 1) * 32 + c32));
      }
    } else if ((it + 1) * 32 > p.Lq) {   // last tile, the whole work-group: lse = +inf
      if (tid < 32 && it * 32 + tid >= p.Lq) reinterpret_cast<float*>(smem + so + STAT_OFF)[tid] = INFINITY;
      lds_barrier();
    }

    // ---- Four MFMA runs per tile: S = Q K^T (log2 units) and dP = dout V^T (rows = queries, in-lane; columns = keys, lanes),
    //      then dV^T += dout^T P and dK^T += Q^T dS.  The arithmetic in between is issued inside the run that does not depend
    //      on it -- P = exp2(S - lse*log2e) between the MFMAs of dP, dS = P (dP - delta) between the MFMAs of dV -- because an
    //      MFMA holds the matrix pipe for 32 cycles but the issue port for 4, and a wave issues in order: only interleaved in
    //      program order do the two overlap (left alone the scheduler gathers the MFMAs, hence the pins).
    //      Head dims above 96 have no registers to spare for the overlap and do the arithmetic between the runs.
    constexpr bool IL = D <= 96;
    constexpr bool ST = IL && !SC;   // lse / delta slices are read between the MFMAs
    f32x16 S = {0}, dP = {0}, Pm, dS;
    ColOperand pp[2], ds[2];
    // lse / delta of a slice's four queries (8jj + 4g .. +3): raw reads like the operands, requested one slice ahead
    const uint32_t stat_addr = lds_addr(smem) + so + STAT_OFF + 16 * g;
    u32x4 sl[2], sd[2];
    auto p_slice = [&](auto jc) {
      constexpr int jj = decltype(jc)::value;
      const u32x4 l4 = sl[jj & 1];
#pragma unroll
      for (int e = 0; e < 4; ++e) Pm[4 * jj + e] = fast_exp2(SC ? S[4 * jj + e] : fmaf(__uint_as_float(l4[e]), -kLog2e, S[4 * jj + e]));
      if constexpr (jj & 1) pp[jj >> 1] = acc_operand<T>(Pm, jj >> 1);
    };
    auto ds_slice = [&](auto jc) {
      constexpr int jj = decltype(jc)::value;
      const u32x4 d4 = sd[jj & 1];
#pragma unroll
      for (int e = 0; e < 4; ++e) dS[4 * jj + e] = Pm[4 * jj + e] * (SC ? dP[4 * jj + e] : dP[4 * jj + e] - __uint_as_float(d4[e]));
      if constexpr (jj & 1) ds[jj >> 1] = acc_operand<T>(dS, jj >> 1);
    };
    static_assert(NCHUNK >= 4, "the four P slices ride between the first four dP MFMAs");
    {
      u32x4 qc[2], oc[2];
      qc[0] = lds_read128_issue<0>(ra);
      static_for<NCHUNK>([&](auto cc) {   // run 1: S
        constexpr int c = decltype(cc)::value;
        if constexpr (c + 1 < NCHUNK) {
          qc[(c + 1) & 1] = lds_read128_issue<32 * (c + 1)>(ra);
          lds_read128_wait<1>(qc[c & 1]);
        } else {   // first operand and first lse slice of the next run
          oc[0] = lds_read128_issue<DO_OFF>(ra);
          if constexpr (ST) sl[0] = lds_read128_issue<0>(stat_addr);
          lds_read128_wait<ST ? 2 : 1>(qc[c & 1]);
        }
        mma_chunk<T>(S, qc[c & 1], Kr[c]);
      });
      static_for<NCHUNK>([&](auto cc) {   // run 2: dP, P formed meanwhile
        constexpr int c = decltype(cc)::value;
        constexpr bool more = c + 1 < NCHUNK;
        if constexpr (more) oc[(c + 1) & 1] = lds_read128_issue<32 * (c + 1) + DO_OFF>(ra);
        if constexpr (ST && c + 1 < 4) sl[(c + 1) & 1] = lds_read128_issue<32 * (c + 1)>(stat_addr);   // 8 queries = 32 bytes per slice
        // operand c and lse slice c were requested one step ago: leave what has been requested since in flight
        if constexpr (ST && c < 4) lds_read128_wait<(more ? 1 : 0) + (c + 1 < 4 ? 1 : 0)>(oc[c & 1], sl[c & 1]);
        else lds_read128_wait<more ? 1 : 0>(oc[c & 1]);
        DMF_PIN();
        mma_chunk<T>(dP, oc[c & 1], Vr[c]);
        DMF_PIN();
        if constexpr (IL && c < 4) p_slice(cc);
        DMF_PIN();
      });
    }
    if constexpr (!IL) {   // all of the arithmetic between the runs
      static_for<4>([&](auto jc) {
        constexpr int jj = decltype(jc)::value;
        sl[jj & 1] = lds_read128_issue<32 * jj>(stat_addr);
        sd[jj & 1] = lds_read128_issue<128 + 32 * jj>(stat_addr);
        lds_read128_wait<0>(sl[jj & 1], sd[jj & 1]);
        p_slice(jc);
        ds_slice(jc);
      });
    }
    {
      constexpr int NG = 2 * NMT, NGT = NG + (TAIL ? 1 : 0);
      static_assert(NGT >= 4, "the four dS slices ride between the first four dV MFMAs");
      TrPair qq[2], oo[2];
      auto lo_off = [](int gi) constexpr { return (16 * (gi / NMT) * STR + 32 * (gi % NMT)) * 2; };
      const uint32_t ta = tail_addr + so;
      oo[0] = lds_tr16_issue<lo_off(0) + DO_OFF, lo_off(0) + 8 * STR * 2 + DO_OFF>(ca);
      if constexpr (ST) sd[0] = lds_read128_issue<128>(stat_addr);   // delta[32] follows lse[32]
      static_for<NGT>([&](auto gc) {   // run 3: dV^T += dout^T P, dS formed meanwhile
        constexpr int gi = decltype(gc)::value;
        if constexpr (gi + 1 < NG) {
          constexpr int LO = lo_off(gi + 1), HI = LO + 8 * STR * 2;
          oo[(gi + 1) & 1] = lds_tr16_issue<LO + DO_OFF, HI + DO_OFF>(ca);
        } else if constexpr (gi + 1 < NGT) {
          oo[(gi + 1) & 1] = lds_tr16_issue<DO_OFF, 8 * STR * 2 + DO_OFF>(ta);
        } else {
          qq[0] = lds_tr16_issue<lo_off(0), lo_off(0) + 8 * STR * 2>(ca);   // first operand of the next run
        }
        if constexpr (ST && gi + 1 < 4) sd[(gi + 1) & 1] = lds_read128_issue<128 + 32 * (gi + 1)>(stat_addr);
        if constexpr (ST && gi < 4) {
          asm volatile("s_waitcnt lgkmcnt(%[n])" : "+v"(oo[gi & 1].lo), "+v"(oo[gi & 1].hi), "+v"(sd[gi & 1]) : [n] "n"(gi + 1 < 4 ? 3 : 2));
        } else {
          lds_tr16_wait<2>(oo[gi & 1]);
        }
        DMF_PIN();
        if constexpr (gi < NG) {
          mma_col<T>(dV[gi % NMT], tr_operand(oo[gi & 1]), pp[gi / NMT]);
        } else {
          ColOperand p0, p1;
          tail_operands(pp[0], pp[1], p0, p1);
          mma16(dV16[0], tr_operand(oo[gi & 1]), p0);
          mma16(dV16[1], tr_operand(oo[gi & 1]), p1);
        }
        DMF_PIN();
        if constexpr (IL && gi < 4) ds_slice(gc);
        DMF_PIN();
      });
      static_for<NGT>([&](auto gc) {   // run 4: dK^T += Q^T dS
        constexpr int gi = decltype(gc)::value;
        constexpr bool more = gi + 1 < NGT;
        if constexpr (gi + 1 < NG) {
          constexpr int LO = lo_off(gi + 1), HI = LO + 8 * STR * 2;
          qq[(gi + 1) & 1] = lds_tr16_issue<LO, HI>(ca);
        } else if constexpr (more) {
          qq[(gi + 1) & 1] = lds_tr16_issue<0, 8 * STR * 2>(ta);
        }
        lds_tr16_wait<more ? 2 : 0>(qq[gi & 1]);
        if constexpr (gi < NG) {
          mma_col<T>(dK[gi % NMT], tr_operand(qq[gi & 1]), ds[gi / NMT]);
        } else {
          ColOperand d0, d1;
          tail_operands(ds[0], ds[1], d0, d1);
          mma16(dK16[0], tr_operand(qq[gi & 1]), d0);
          mma16(dK16[1], tr_operand(qq[gi & 1]), d1);
        }
      });
    }
  }
  T* stage = reinterpret_cast<T*>(smem);
  store_rows_transposed<T, D, NW, NMT>(stage, reinterpret_cast<T*>(p.dk) + base(6), p.st[6][1], k0, p.Lkv, tid,
                                      [&](int t, int i) { return dK[t][i] * p.scale; },
                                      [&](void* ws) {
                                        if constexpr (TAIL) store_tail16<T, D, NMT>(ws, lane, [&](int hq, int e) { return dK16[hq][e] * p.scale; });
                                      });
  store_rows_transposed<T, D, NW, NMT>(stage, reinterpret_cast<T*>(p.dv) + base(7), p.st[7][1], k0, p.Lkv, tid,
                                      [&](int t, int i) { return dV[t][i]; },
                                      [&](void* ws) {
                                        if constexpr (TAIL) store_tail16<T, D, NMT>(ws, lane, [&](int hq, int e) { return dV16[hq][e]; });
                                      });
}

// ------------------------------------------------ single-pass backward, whole (batch, head) unit per work-group
// For sequences of at most 256 rows one 8-wave work-group owns a whole (batch, head) unit and every score tile is
// formed exactly once -- 5 GEMM units per (query tile, key tile) pair instead of the 7 of the two-kernel scheme --
// with no atomics, no workspace and a fixed summation order:
//   * wave w owns keys 32w .. 32w+31: K (times scale*log2e) and V stay in registers as B operands, dK^T and dV^T are
//     its accumulators over the whole sequence ("phase 1", the dK/dV kernel's loop body: S = Q K^T, dP = dout V^T,
//     P, dS, dV^T += dout^T P, dK^T += Q^T dS, with Q / dout tiles of 32 queries streamed HBM -> LDS by DMA);
//   * dQ needs dS contracted over keys, i.e. across the waves.  Instead of summing eight fp32 partial tiles, the bf16
//     dS tiles themselves are exchanged: phase 1 leaves tile (query tile j, key block w) in an LDS array X, and after
//     four query tiles ("half" of the sequence; 64 KB of X) "phase 2" forms dQ^T = K^T dS^T for those 128 queries from X
//     and an LDS-resident copy of K.  The 3 (head dim 72: 2 + remainder) output tiles of a query tile are split
//     between wave jj (tiles of part 0) and wave jj + 4 (part 1) -- two waves of the same SIMD, so every SIMD gets the
//     same MFMA work and no partial sums have to be combined.
// LDS: K (8 tiles) | NST stages of Q, dout tiles | X (64 KB, reused as store staging) | lse, delta of all rows.
template <int D>
struct BwdFusedCfg {
  using F = BwdFastCfg<D, true>;
  static constexpr int TB = F::TBYTES;
  static constexpr int XBYTES = 65536, STATBYTES = 2 * 256 * 4;
  // Q / dout stages: as many as the LDS has room for next to tiles of the pitch that keeps the transposed reads free of
  // bank conflicts (head dims 72 and 80: three stages of 13-vector rows rather than four of 11, 1 % faster).  A third or
  // fourth stage only has to absorb jitter: the wait for a tile's delta rows at the end of every iteration already leaves
  // nothing but the newest tile request in flight, so a tile has two iterations to arrive whatever the depth.
  static constexpr int NST = (8 + 2 * 4) * TB + XBYTES + STATBYTES <= 160 * 1024 ? 4 : ((8 + 2 * 3) * TB + XBYTES + STATBYTES <= 160 * 1024 ? 3 : 2);
  static constexpr int K_OFF = 0, QS_OFF = 8 * TB, X_OFF = QS_OFF + 2 * NST * TB, STAT_OFF = X_OFF + XBYTES;
  static constexpr int LDS_BYTES = STAT_OFF + STATBYTES;
  static constexpr int XTILE = 32 * 32 * 2;                      // one exchanged dS tile: [32 keys][32 queries] bf16
  static constexpr int NT0 = (F::NMT + 1) / 2;                   // part 0: output tiles 0 .. NT0-1 (+ the 16-wide remainder); part 1: the rest
  static_assert(LDS_BYTES <= 160 * 1024, "head dim too large for the single-pass backward");
  static_assert(256 * Cfg<__bf16, D>::OROWV * 16 <= XBYTES, "store staging must fit the exchange area");
};

template <int D>
__global__ __launch_bounds__(512, 1) void attn_bwd_fused_bf16_kernel(const BwdParams p) {
  using F = BwdFastCfg<D, true>;
  using FC = BwdFusedCfg<D>;
  using T = __bf16;
  constexpr int VPR = F::VPR, NCHUNK = F::NCHUNK, NMT = F::NMT, P = F::P, STR = F::STR, TB = FC::TB;
  constexpr bool TAIL = F::TAIL;
  constexpr int DO_OFF = TB;               // dout tile sits after the Q tile of its stage
  constexpr int STAGE = 2 * TB;
  constexpr int NT0 = FC::NT0, NST = FC::NST;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31, g = lane >> 5;
  const int bh = xcd_remap(blockIdx.x, gridDim.x);
  const int b = bh / p.H, h = bh % p.H;
  auto base = [&](int t) { return (int64_t)b * p.st[t][0] + (int64_t)h * p.st[t][2]; };
  float* stat_lse = reinterpret_cast<float*>(smem + FC::STAT_OFF);
  float* stat_delta = stat_lse + 256;

  // SC: columns D .. D+2 of a Q row carry -lse*log2e and of a dout row -delta (bf16 triples, BwdFastCfg::STATCOL) against
  // ones in this lane's K and V rows, so that S - lse and dP - delta come out of the MFMAs; the lane that finishes a
  // row's delta writes both pad vectors.
  constexpr bool SC = F::STATCOL;
  // ---- zero the contraction padding of the K tiles and of both Q / dout stages (with SC not the first pad vector of
  //      the stage tiles: its owner writes it, for tile 0 before the first barrier)
  if constexpr (P > VPR) {
    constexpr int PADV = P - VPR;
    for (int i = tid; i < (8 + 2 * NST) * 32 * PADV; i += 512) {
      const int tile = i / (32 * PADV), r = (i / PADV) % 32, cv = VPR + i % PADV;
      if (SC && tile >= 8 && cv == VPR) continue;
      *reinterpret_cast<u32x4*>(smem + tile * TB + (r * P + cv) * 16) = u32x4{0, 0, 0, 0};
    }
  }

  const uint32_t rb_q = (uint32_t)p.st[1][1] * 2, rb_do = (uint32_t)p.st[0][1] * 2;
  const uint32_t rb_k = (uint32_t)p.st[2][1] * 2, rb_v = (uint32_t)p.st[3][1] * 2;
  const __amdgpu_buffer_rsrc_t rs_q = make_rows_rsrc(reinterpret_cast<const T*>(p.q) + base(1), rb_q, p.Lq, D * 2);
  const __amdgpu_buffer_rsrc_t rs_do = make_rows_rsrc(reinterpret_cast<const T*>(p.dout) + base(0), rb_do, p.Lq, D * 2);
  const __amdgpu_buffer_rsrc_t rs_k = make_rows_rsrc(reinterpret_cast<const T*>(p.k) + base(2), rb_k, p.Lkv, D * 2);
  const __amdgpu_buffer_rsrc_t rs_v = make_rows_rsrc(reinterpret_cast<const T*>(p.v) + base(3), rb_v, p.Lkv, D * 2);
  const int nqt = (p.Lq + 31) / 32, nkb = (p.Lkv + 31) / 32;   // query tiles / key blocks in use (<= 8 each)

  // ---- requests, in the order in which their data is needed (a work-group has its CU to itself, so whatever the
  //      first tile waits for is exposed; the memory system serves the requests roughly first come, first served):
  //      lse and the first tile's dout / o rows (for delta), the first Q / dout tile, this wave's K and V rows, further
  //      tiles.
  // Every wave issues exactly two DMA instructions per Q / dout tile, and
  // wait_tile() -- called when tile j is needed -- lets the ones issued after tile j stay in flight (vector memory operations
  // complete in order, and anything not counted here can only make the wait stricter).
  // Tiles 0 .. NST-2 are requested up front, then tile j+NST-1 at the top of iteration j: when tile j is waited for,
  // the tiles j+1 .. j+NST-2 were requested after it.
  auto issue_q = [&](int j) {   // tile j goes to stage j % NST
    char* st = smem + FC::QS_OFF + (j % NST) * STAGE;
    issue_tile_rows<P, VPR, 8>(rs_q, rb_q, (uint32_t)j * 32 * rb_q, st, wave, lane);
    issue_tile_rows<P, VPR, 8>(rs_do, rb_do, (uint32_t)j * 32 * rb_do, st + DO_OFF, wave, lane);
  };
  // Tiles past the end are requested like the others (every row is out of range: the bounds check zero-fills the stage
  // and nothing reads it), so that the number of DMA instructions in flight behind any tile is a constant, 2 (NST - 2),
  // and no wait depends on how many tiles are left.
  auto wait_tile = [&]() {
    static_assert(NST >= 2 && 2 * (NST - 2) <= 15, "vmcnt immediate");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * (NST - 2)));
  };
  // Work-group barrier with no fence attached: a release fence would make the compiler wait for every outstanding
  // buffer_load ... lds (vmcnt(0)), i.e. for the tiles requested ahead.  This wave's own LDS traffic is waited for here;
  // what a barrier publishes of the DMA data is decided by the explicit wait_tile() in front of it.
  auto bare_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
  // delta = rowsum(dout * o) of the 32 query rows of a tile, by the whole work-group: 16 lanes per row, one 16-byte
  // vector of dout and of o per lane (lanes past the head dim read zeros), summed across the 16 lanes.
  const uint32_t rb_o = (uint32_t)p.st[4][1] * 2;
  // The three loads of a delta request are raw instructions with an explicit wait (delta_wait): loads the compiler tracks
  // would be waited for with vmcnt(0) / vmcnt(1) -- it does not count the tile DMA issued behind them -- i.e. together with
  // the tile requested in the same iteration.  Every lane loads (no divergent branch around a raw load: the compiler could
  // copy the destination register at the join before the data is there); lanes without a row read a clamped address.
  struct DeltaRows { u32x4 d, o; float lse; };
  const u32x4 rsw_do = rows_rsrc_words(reinterpret_cast<const T*>(p.dout) + base(0), rb_do, p.Lq, D * 2);
  const u32x4 rsw_o = rows_rsrc_words(reinterpret_cast<const T*>(p.o) + base(4), rb_o, p.Lq, D * 2);
  auto delta_request = [&](int j) {
    const int qrow = 32 * j + (tid >> 4), cv = tid & 15;
    DeltaRows r;
    const float* lp = p.lse + (int64_t)bh * p.Lq + min(qrow, p.Lq - 1);
    asm volatile("global_load_dword %0, %1, off" : "=v"(r.lse) : "v"(lp));
    const uint32_t vd = cv < VPR ? (uint32_t)qrow * rb_do + cv * 16 : 0x7ffffff0u, vo = cv < VPR ? (uint32_t)qrow * rb_o + cv * 16 : 0x7ffffff0u;
    // (s_nop: a descriptor the compiler has just restored with v_readlane needs five wait states before a vector memory
    //  instruction may read it, and the compiler does not look into the block for that)
    asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %2, %4, 0 offen\n\tbuffer_load_dwordx4 %1, %3, %5, 0 offen"
                 : "=&v"(r.d), "=&v"(r.o)
                 : "v"(vd), "v"(vo), "s"(rsw_do), "s"(rsw_o));
    return r;
  };
  // N = vector-memory instructions issued since the request that may stay in flight
  auto delta_wait = [&](DeltaRows& r, auto nc) {
    asm volatile("s_waitcnt vmcnt(%[n])" : "+v"(r.d), "+v"(r.o), "+v"(r.lse) : [n] "n"(decltype(nc)::value));
  };
  auto delta_finish = [&](int j, const DeltaRows& r) {
    // Packed bf16 dot products with fp32 accumulation: four instructions for the eight products instead of sixteen
    // unpacks and eight multiply-adds (the tile loop is bound by the instructions it issues).  The dot instructions have a
    // longer pipeline than other VALU operations: chained through their accumulator they need no wait, but an ordinary
    // VALU instruction that reads the result needs three wait states, which the compiler does not insert for a block it
    // cannot look into -- hence the s_nop behind it (and one in front, for the accumulator's initial value).
    float s = 0.f;
    asm volatile(
        "s_nop 1\n\t"
        "v_dot2c_f32_bf16 %0, %1, %5\n\t"
        "v_dot2c_f32_bf16 %0, %2, %6\n\t"
        "v_dot2c_f32_bf16 %0, %3, %7\n\t"
        "v_dot2c_f32_bf16 %0, %4, %8\n\t"
        "s_nop 3"
        : "+v"(s)
        : "v"(r.d[0]), "v"(r.d[1]), "v"(r.d[2]), "v"(r.d[3]), "v"(r.o[0]), "v"(r.o[1]), "v"(r.o[2]), "v"(r.o[3]));
    // inclusive sum over the row of 16 lanes (DPP row_shr 1, 2, 4, 8; lanes shifted in from outside read 0): lane 15 holds it
    auto shr = [](float x, auto n) {
      return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0x110 + decltype(n)::value, 0xf, 0xf, true));
    };
    s += shr(s, std::integral_constant<int, 1>{});
    s += shr(s, std::integral_constant<int, 2>{});
    s += shr(s, std::integral_constant<int, 4>{});
    s += shr(s, std::integral_constant<int, 8>{});
    const int qrow = 32 * j + (tid >> 4);
    if ((tid & 15) == 15) {
      const bool qok = qrow < p.Lq;
      if constexpr (SC) {   // rows past the end: P = 0 through a huge "lse"
        // (raw stores: in front of a store it tracks the compiler would wait for the tile DMA in flight)
        const uint32_t row = lds_addr(smem) + FC::QS_OFF + (j % NST) * STAGE + ((tid >> 4) * P + VPR) * 16;
        u32x4 lv = split3_bf16(qok ? -r.lse * kLog2e : -1e30f);
        lv[1] |= 0xF14A0000u;   // fourth pad element: -1e30 (bf16), met by a one only in the K rows of keys past the end
        lds_write128_untracked<0>(row, lv);
        lds_write128_untracked<DO_OFF>(row, split3_bf16(qok ? -s : 0.f));
      } else {
        stat_delta[qrow] = qok ? s : 0.f;
      }
      if (qok) p.delta[(int64_t)bh * p.Lq + qrow] = s;
    }
  };

  if constexpr (!SC) {
    if (tid < 256) stat_lse[tid] = tid < p.Lq ? p.lse[(int64_t)bh * p.Lq + tid] : INFINITY;   // +inf switches padded query rows off (P = 0)
  }
  DeltaRows dr = delta_request(0);
  issue_q(0);
  // ---- this wave's 32 key rows, whole rows by DMA: K straight into its tile of the LDS-resident copy (the phase 2
  //      operand, and where phase 1 takes its register operand from), V into the exchange area, which nobody uses
  //      before the first barrier (rows past Lkv read as zeros)
  issue_rows<P, VPR, 32>(rs_k, rb_k, (uint32_t)(wave * 32) * rb_k, smem + FC::K_OFF + wave * TB, lane);
  issue_rows<P, VPR, 32>(rs_v, rb_v, (uint32_t)(wave * 32) * rb_v, smem + FC::X_OFF + wave * TB, lane);
  for (int j = 1; j < NST - 1; ++j) issue_q(j);
  wait_tile();    // loads complete in order: the key rows, tile 0 and the delta request have landed, the later tiles may still be in flight
  delta_wait(dr, std::integral_constant<int, 2 * (NST - 2)>{});
  // ---- this lane's key row: V stays in registers for the whole kernel, K (times scale*log2e) is re-read from the LDS
  //      copy at the top of every half (so that its registers are free while dQ is formed)
  const int krow = wave * 32 + c32;
  const uint32_t k_row_addr = lds_addr(smem) + FC::K_OFF + (krow * P + g) * 16;   // pad vectors of the K tiles are zero
  u32x4 Kr[NCHUNK], Vr[NCHUNK];
  {
    const uint32_t va = lds_addr(smem) + FC::X_OFF + krow * P * 16;
    static_for<NCHUNK>([&](auto cc) {
      constexpr int c = decltype(cc)::value;
      // (the upper half of the last chunk of a head dim that is not a multiple of 16 does not exist: zeroed below)
      Vr[c] = lds_read128_issue<32 * c>(2 * c + 1 < VPR ? va + g * 16 : va);
    });
    lds_read128_wait<0>(Vr[NCHUNK - 1]);
#pragma unroll
    for (int c = 0; c + 1 < NCHUNK; ++c) asm volatile("" : "+v"(Vr[c]));
    if constexpr (2 * NCHUNK > VPR) {
      if (g == 1) Vr[NCHUNK - 1] = SC ? ones3_bf16() : u32x4{0, 0, 0, 0};
    }
  }
  delta_finish(0, dr);
  const bool kvalid = krow < p.Lkv;

  f32x16 dK[NMT], dV[NMT];
  f32x4 dK16[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}}, dV16[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
#pragma unroll
  for (int t = 0; t < NMT; ++t) {
    dK[t] = f32x16{0};
    dV[t] = f32x16{0};
  }

  // lane addresses (relative to a tile base): row-operand reads, transposed reads, remainder operand
  const uint32_t row_addr = lds_addr(smem) + c32 * STR * 2 + g * 16;
  const uint32_t col_off = ((4 * g + ((lane & 15) >> 2)) * STR + 16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
  const uint32_t tail_off = tail_lane_offset(lane, STR, 32 * NMT) * 2;
  // exchange tiles: [32 keys][32 queries] bf16, pitch 64 bytes
  const uint32_t x_base = lds_addr(smem) + FC::X_OFF;
  // The eight 8-byte pieces (4 queries) of key row k are stored at piece index (piece ^ ((k >> 2) & 7)): without the
  // swizzle the 64 lanes of a store (key = lane % 32, row pitch 64 bytes) fall on 8 of the 32 bank pairs.
  const uint32_t x_swz = (c32 >> 2) & 7;

  for (int half = 0; half * 4 < nqt; ++half) {
    // ================= phase 1: query tiles 4*half .. 4*half+3 against this wave's keys
    const int j_end = min(nqt, 4 * half + 4);
    static_for<NCHUNK>([&](auto cc) { Kr[decltype(cc)::value] = lds_read128_issue<32 * decltype(cc)::value>(k_row_addr); });
    lds_read128_wait<0>(Kr[NCHUNK - 1]);
#pragma unroll
    for (int c = 0; c + 1 < NCHUNK; ++c) asm volatile("" : "+v"(Kr[c]));
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) Kr[c] = scale_bf16x8(Kr[c], p.scale_log2);
    if constexpr (SC) {
      // (keys past the end: a fourth one against the -1e30 that every Q row carries in that slot, so that their P, and
      //  with it their dS, is exactly zero without a select in the tile loop)
      if (g == 1) Kr[NCHUNK - 1] = kvalid ? ones3_bf16() : u32x4{0x3f803f80u, 0x3f803f80u, 0u, 0u};
    }
    for (int j = 4 * half; j < j_end; ++j) {
      if (j == 0 || j != 4 * half) {   // (the first tile of a later half was waited for before the dQ rows were stored)
        wait_tile();      // this wave's share of tile j has landed
        bare_barrier();   // ... and everyone else's; all waves are done with the stage of tile j-1
      }
      dr = delta_request(min(j + 1, nqt - 1));   // (before the tile request: its data is wanted first; behind the last tile: dropped)
      issue_q(j + NST - 1);
      const uint32_t stage_off = FC::QS_OFF + (j % NST) * STAGE;
      const uint32_t ra = row_addr + stage_off, ca = lds_addr(smem) + col_off + stage_off;

      // ---- The four products of a tile are four MFMA runs: S = Q K^T (log2 units) and dP = dout V^T (rows = queries,
      //      in-lane; columns = keys, lanes), then dV^T += dout^T P and dK^T += Q^T dS.  The arithmetic in between is issued
      //      inside the run that does not depend on it -- P = exp2(S - lse*log2e) between the MFMAs of dP, dS = P (dP - delta)
      //      and its hand-over to the exchange array between the MFMAs of dV -- because an MFMA holds the matrix pipe for 32
      //      cycles but the issue port for 4, and a wave issues in order: only interleaved in program order do the two overlap
      //      (left alone the scheduler gathers the MFMAs, hence the pins).  Padded query rows carry lse = +inf (P = 0), padded
      //      keys are switched off where dS is handed over.
      f32x16 S = {0}, dP = {0}, Pm, dS;
      ColOperand pp[2], ds[2];
      const uint32_t xa = x_base + ((j & 3) * 8 + wave) * FC::XTILE + c32 * 64;   // this lane's key row of tile X[j % 4][wave]
      // lse / delta of the slice's four queries: raw reads like the operands, requested one slice ahead (a tracked read
      // would be waited for with lgkmcnt(0), i.e. together with the operand reads just issued behind it)
      //      (With SC both statistics are already inside S and dP and none of this is read.)
      constexpr bool ST = !SC;
      const uint32_t stat_addr = lds_addr(stat_lse) + (j * 32 + 4 * g) * 4;
      u32x4 sl[2], sd[2];
      auto p_slice = [&](auto jc) {   // elements 4jj .. 4jj+3: queries 8jj + 4g .. +3 of the tile
        constexpr int jj = decltype(jc)::value;
        const u32x4 l4 = sl[jj & 1];
#pragma unroll
        for (int e = 0; e < 4; ++e) Pm[4 * jj + e] = fast_exp2(SC ? S[4 * jj + e] : fmaf(__uint_as_float(l4[e]), -kLog2e, S[4 * jj + e]));
        if constexpr (jj & 1) pp[jj >> 1] = acc_operand<T>(Pm, jj >> 1);
      };
      auto ds_slice = [&](auto jc) {
        constexpr int jj = decltype(jc)::value;
        const u32x4 d4 = sd[jj & 1];
#pragma unroll
        for (int e = 0; e < 4; ++e) dS[4 * jj + e] = Pm[4 * jj + e] * (SC ? dP[4 * jj + e] : dP[4 * jj + e] - __uint_as_float(d4[e]));
        if constexpr (jj & 1) {
          ds[jj >> 1] = acc_operand<T>(dS, jj >> 1);
          // dS tile -> X (zeros for keys past the end: their K rows -- not zero-filled when the rows of a broadcast operand
          // alias -- must not reach dQ; with SC their P is zero already, see the K operand above)
          static_for<2>([&](auto hc) {
            constexpr int q4 = jj - 1 + decltype(hc)::value;   // queries 8 q4 + 4g .. +3 of key row c32
            const u32x2 w = SC || kvalid ? u32x2{ds[q4 >> 1].v[2 * (q4 & 1)], ds[q4 >> 1].v[2 * (q4 & 1) + 1]} : u32x2{0, 0};
            lds_write64_untracked<0>(xa + (((2 * q4 + g) ^ x_swz) << 3), w);
          });
        }
      };
      static_assert(NCHUNK >= 4, "the four P slices ride between the first four dP MFMAs");
      {
        // run 1: S.  All of its operands are requested at once (a wave alone on its SIMD would otherwise wait out one LDS
        // latency per MFMA), then the first operand and the first lse slice of the next run.
        u32x4 qc[NCHUNK], oc[2];
        static_for<NCHUNK>([&](auto cc) { qc[decltype(cc)::value] = lds_read128_issue<32 * decltype(cc)::value>(ra); });
        oc[0] = lds_read128_issue<DO_OFF>(ra);
        if constexpr (ST) sl[0] = lds_read128_issue<0>(stat_addr);
        static_for<NCHUNK>([&](auto cc) {
          constexpr int c = decltype(cc)::value;
          lds_read128_wait<NCHUNK - 1 - c + (ST ? 2 : 1)>(qc[c]);
          mma_chunk<T>(S, qc[c], Kr[c]);
        });
        static_for<NCHUNK>([&](auto cc) {   // run 2: dP, P formed meanwhile
          constexpr int c = decltype(cc)::value;
          constexpr bool more = c + 1 < NCHUNK;
          if constexpr (more) oc[(c + 1) & 1] = lds_read128_issue<32 * (c + 1) + DO_OFF>(ra);
          if constexpr (ST && c + 1 < 4) sl[(c + 1) & 1] = lds_read128_issue<32 * (c + 1)>(stat_addr);   // 8 queries = 32 bytes per slice
          // operand c and lse slice c were requested one step ago: leave what has been requested since in flight
          if constexpr (ST && c < 4) lds_read128_wait<(more ? 1 : 0) + (c + 1 < 4 ? 1 : 0)>(oc[c & 1], sl[c & 1]);
          else lds_read128_wait<more ? 1 : 0>(oc[c & 1]);
          DMF_PIN();
          mma_chunk<T>(dP, oc[c & 1], Vr[c]);
          DMF_PIN();
          if constexpr (c < 4) p_slice(cc);
          DMF_PIN();
        });
      }
      {
        constexpr int NG = 2 * NMT, NGT = NG + (TAIL ? 1 : 0);
        static_assert(NGT >= 4, "the four dS slices ride between the first four dV MFMAs");
        TrPair qq[2], oo[2];
        auto lo_off = [](int gi) constexpr { return (16 * (gi / NMT) * STR + 32 * (gi % NMT)) * 2; };
        const uint32_t ta = lds_addr(smem) + tail_off + stage_off;
        oo[0] = lds_tr16_issue<lo_off(0) + DO_OFF, lo_off(0) + 8 * STR * 2 + DO_OFF>(ca);
        if constexpr (ST) sd[0] = lds_read128_issue<1024>(stat_addr);   // stat_delta = stat_lse + 256 floats
        static_for<NGT>([&](auto gc) {   // run 3: dV^T += dout^T P, dS formed and handed over meanwhile
          constexpr int gi = decltype(gc)::value;
          if constexpr (gi + 1 < NG) {
            constexpr int LO = lo_off(gi + 1), HI = LO + 8 * STR * 2;
            oo[(gi + 1) & 1] = lds_tr16_issue<LO + DO_OFF, HI + DO_OFF>(ca);
          } else if constexpr (gi + 1 < NGT) {
            oo[(gi + 1) & 1] = lds_tr16_issue<DO_OFF, 8 * STR * 2 + DO_OFF>(ta);
          } else {
            qq[0] = lds_tr16_issue<lo_off(0), lo_off(0) + 8 * STR * 2>(ca);   // first operand of the next run
          }
          if constexpr (ST && gi + 1 < 4) sd[(gi + 1) & 1] = lds_read128_issue<1024 + 32 * (gi + 1)>(stat_addr);
          if constexpr (ST && gi < 4) {
            asm volatile("s_waitcnt lgkmcnt(%[n])" : "+v"(oo[gi & 1].lo), "+v"(oo[gi & 1].hi), "+v"(sd[gi & 1]) : [n] "n"(gi + 1 < 4 ? 3 : 2));
          } else {
            lds_tr16_wait<2>(oo[gi & 1]);
          }
          DMF_PIN();
          if constexpr (gi < NG) {
            mma_col<T>(dV[gi % NMT], tr_operand(oo[gi & 1]), pp[gi / NMT]);
          } else {
            ColOperand p0, p1;
            tail_operands(pp[0], pp[1], p0, p1);
            mma16(dV16[0], tr_operand(oo[gi & 1]), p0);
            mma16(dV16[1], tr_operand(oo[gi & 1]), p1);
          }
          DMF_PIN();
          if constexpr (gi < 4) ds_slice(gc);
          DMF_PIN();
        });
        static_for<NGT>([&](auto gc) {   // run 4: dK^T += Q^T dS
          constexpr int gi = decltype(gc)::value;
          constexpr bool more = gi + 1 < NGT;
          if constexpr (gi + 1 < NG) {
            constexpr int LO = lo_off(gi + 1), HI = LO + 8 * STR * 2;
            qq[(gi + 1) & 1] = lds_tr16_issue<LO, HI>(ca);
          } else if constexpr (more) {
            qq[(gi + 1) & 1] = lds_tr16_issue<0, 8 * STR * 2>(ta);
          }
          lds_tr16_wait<more ? 2 : 0>(qq[gi & 1]);
          if constexpr (gi < NG) {
            mma_col<T>(dK[gi % NMT], tr_operand(qq[gi & 1]), ds[gi / NMT]);
          } else {
            ColOperand d0, d1;
            tail_operands(ds[0], ds[1], d0, d1);
            mma16(dK16[0], tr_operand(qq[gi & 1]), d0);
            mma16(dK16[1], tr_operand(qq[gi & 1]), d1);
          }
        });
      }
#undef DMF_PIN
      delta_wait(dr, std::integral_constant<int, 2>{});   // (this iteration's tile request may stay in flight)
      if (j + 1 < nqt) delta_finish(j + 1, dr);   // visible to the other waves after the next barrier
    }
    // This wave's dS tiles are in LDS, then everyone's: X holds every dS tile of this half.  A bare barrier: the fenced
    // lds_barrier() would also wait for the Q / dout tile DMA in flight (vmcnt(0): a release fence covers the LDS writes of
    // outstanding buffer_load ... lds instructions), about 2000 cycles per half, and nothing read below comes from a DMA
    // that is still in flight (the K tiles landed before the first tile).
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    // ================= phase 2: dQ^T = K^T dS^T for query tile jq, output tiles of this wave's part
    const int jq = 4 * half + (wave & 3);
    const bool part1 = wave >= 4;
    f32x16 dQ[NT0];
    f32x4 dQ16[2] = {f32x4{0, 0, 0, 0}, f32x4{0, 0, 0, 0}};
#pragma unroll
    for (int t = 0; t < NT0; ++t) dQ[t] = f32x16{0};
    if constexpr (NMT == 2) {
      // Straight-line form (two output tiles, one per part): always all eight key blocks -- the K rows and the dS tiles of
      // keys past the end are zeros -- fully unrolled, every operand read issued as a raw instruction one key block ahead
      // with an explicit lgkmcnt wait, no branch between an issue and its wait.  (Read through the tracked intrinsics the
      // first operand would make the compiler wait for the Q / dout tile DMA in flight, about 2000 cycles per half.)  Both
      // parts run the remainder products; part 1 drops its copy (two 16x16x32 MFMAs per key block) rather than branch.
      if (jq < nqt) {
        const int i16 = lane & 15, piece = 4 * ((lane >> 4) & 1) + (i16 & 3), r0 = 4 * g + (i16 >> 2);
        // lane address inside a swizzled exchange tile: key row r, query piece `piece` (cf. the writer's x_swz)
        auto xoff = [&](int r) { return (uint32_t)(r * 32 + ((piece ^ ((r >> 2) & 7)) << 2)) * 2; };
        const uint32_t xb = x_base + (wave & 3) * 8 * FC::XTILE;
        const uint32_t x00 = xb + xoff(r0), x01 = xb + xoff(r0 + 8), x10 = xb + xoff(r0 + 16), x11 = xb + xoff(r0 + 24);
        const uint32_t ka = lds_addr(smem) + FC::K_OFF + col_off + (part1 ? 64u : 0u);   // part 1: head-dim columns 32 .. 63
        const uint32_t kta = lds_addr(smem) + FC::K_OFF + tail_off;
        struct RawOps { u32x2 b0l, b0h, b1l, b1h; TrPair a0, a1, tl; };
        constexpr int NRD = 8 + (TAIL ? 2 : 0);   // LDS instructions per key block
        RawOps ro[2];
        auto issue_kb = [&](auto kc_) {
          constexpr int kb = decltype(kc_)::value;
          RawOps& o = ro[kb & 1];
          o.b0l = lds_tr16_issue1<kb * FC::XTILE>(x00);
          o.b0h = lds_tr16_issue1<kb * FC::XTILE>(x01);
          o.b1l = lds_tr16_issue1<kb * FC::XTILE>(x10);
          o.b1h = lds_tr16_issue1<kb * FC::XTILE>(x11);
          o.a0 = lds_tr16_issue<kb * TB, kb * TB + 8 * STR * 2>(ka);
          o.a1 = lds_tr16_issue<kb * TB + 16 * STR * 2, kb * TB + 24 * STR * 2>(ka);
          if constexpr (TAIL) o.tl = lds_tr16_issue<kb * TB, kb * TB + 8 * STR * 2>(kta);
        };
        issue_kb(std::integral_constant<int, 0>{});
        static_for<8>([&](auto kc_) {
          constexpr int kb = decltype(kc_)::value;
          if constexpr (kb + 1 < 8) issue_kb(std::integral_constant<int, kb + 1>{});
          RawOps& o = ro[kb & 1];
          if constexpr (TAIL)
            asm volatile("s_waitcnt lgkmcnt(%[n])" : "+v"(o.b0l), "+v"(o.b0h), "+v"(o.b1l), "+v"(o.b1h), "+v"(o.a0.lo), "+v"(o.a0.hi),
                         "+v"(o.a1.lo), "+v"(o.a1.hi), "+v"(o.tl.lo), "+v"(o.tl.hi) : [n] "n"(kb + 1 < 8 ? NRD : 0));
          else
            asm volatile("s_waitcnt lgkmcnt(%[n])" : "+v"(o.b0l), "+v"(o.b0h), "+v"(o.b1l), "+v"(o.b1h), "+v"(o.a0.lo), "+v"(o.a0.hi),
                         "+v"(o.a1.lo), "+v"(o.a1.hi) : [n] "n"(kb + 1 < 8 ? NRD : 0));
          ColOperand b0, b1;
          b0.v = u32x4{o.b0l[0], o.b0l[1], o.b0h[0], o.b0h[1]};
          b1.v = u32x4{o.b1l[0], o.b1l[1], o.b1h[0], o.b1h[1]};
          mma_col<T>(dQ[0], tr_operand(o.a0), b0);
          mma_col<T>(dQ[0], tr_operand(o.a1), b1);
          if constexpr (TAIL) {
            ColOperand d0, d1;
            tail_operands(b0, b1, d0, d1);
            mma16(dQ16[0], tr_operand(o.tl), d0);
            mma16(dQ16[1], tr_operand(o.tl), d1);
          }
        });
      }
    } else if (jq < nqt) {
      // Operands through the tracked LDS-read intrinsics here, not the raw-instruction helpers of phase 1: those are
      // only safe in straight-line code (between the issue and the wait the compiler may copy the destination
      // registers, e.g. at a branch, and would copy stale data), and this loop branches on the wave's part.  The
      // price is that the compiler waits for the tile DMA in flight before the first read, which was requested a
      // whole tile earlier.
      const T* xt = reinterpret_cast<const T*>(smem + FC::X_OFF) + (wave & 3) * 8 * (FC::XTILE / 2);
      // lds_col_operand on a swizzled exchange tile: key rows 16s + 4g + (i >> 2) (+ 8), query piece 4 * half + (i & 3)
      auto x_operand = [&](const T* tile, int st) {
        const int i = lane & 15, piece = 4 * ((lane >> 4) & 1) + (i & 3), r = 16 * st + 4 * g + (i >> 2);
        const T* lo = tile + r * 32 + ((piece ^ ((r >> 2) & 7)) << 2);
        const T* hi = tile + (r + 8) * 32 + ((piece ^ (((r + 8) >> 2) & 7)) << 2);
        const u32x2 a = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, lo)));
        const u32x2 b = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, hi)));
        ColOperand o;
        o.v = u32x4{a[0], a[1], b[0], b[1]};
        return o;
      };
      const T* kt = reinterpret_cast<const T*>(smem + FC::K_OFF);
      constexpr int NT1 = NMT - NT0;
      // Operands of one key block: dS^T of 16 keys each (steps 0, 1) for this wave's 32 queries (B), the K^T tiles of this
      // wave's part (A).  The operands of block kb + 1 are requested before the products of block kb are issued, so
      // that only the first block waits for the LDS.
      struct Ops { ColOperand b0, b1, a0, a1, a2, a3, tail; };   // (plain members: an array member ends up in scratch memory)
      static_assert(NT0 <= 2 && NT1 <= 2, "operand slots for at most two output tiles per part");
      auto load_ops = [&](int kb, Ops& o) {
        const T* x = xt + kb * (FC::XTILE / 2);
        const T* kk = kt + kb * (TB / 2);
        o.b0 = x_operand(x, 0);
        o.b1 = x_operand(x, 1);
        auto tile_ops = [&](int col, ColOperand& s0, ColOperand& s1) {
          s0 = lds_col_operand<T, STR>(kk, 0, col, 0, lane);
          s1 = lds_col_operand<T, STR>(kk, 0, col, 1, lane);
        };
        if (!part1) {
          tile_ops(0, o.a0, o.a1);
          if constexpr (NT0 > 1) tile_ops(32, o.a2, o.a3);
          if constexpr (TAIL) {
            const T* tp = kk + tail_lane_offset(lane, STR, 32 * NMT);
            const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, tp)));
            const u32x2 hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, tp + 8 * STR)));
            o.tail.v = u32x4{lo[0], lo[1], hi[0], hi[1]};
          }
        } else {
          if constexpr (NT1 > 0) tile_ops(32 * NT0, o.a0, o.a1);
          if constexpr (NT1 > 1) tile_ops(32 * (NT0 + 1), o.a2, o.a3);
        }
      };
      auto multiply = [&](const Ops& o) {
        if (!part1) {
          mma_col<T>(dQ[0], o.a0, o.b0);
          mma_col<T>(dQ[0], o.a1, o.b1);
          if constexpr (NT0 > 1) {
            mma_col<T>(dQ[1], o.a2, o.b0);
            mma_col<T>(dQ[1], o.a3, o.b1);
          }
          if constexpr (TAIL) {
            ColOperand d0, d1;
            tail_operands(o.b0, o.b1, d0, d1);
            mma16(dQ16[0], o.tail, d0);
            mma16(dQ16[1], o.tail, d1);
          }
        } else {
          if constexpr (NT1 > 0) {
            mma_col<T>(dQ[0], o.a0, o.b0);
            mma_col<T>(dQ[0], o.a1, o.b1);
          }
          if constexpr (NT1 > 1) {
            mma_col<T>(dQ[1], o.a2, o.b0);
            mma_col<T>(dQ[1], o.a3, o.b1);
          }
        }
      };
      Ops oa, ob;
      if constexpr (NMT <= 2) {
        load_ops(0, oa);
        for (int kb = 0; kb < nkb; kb += 2) {
          if (kb + 1 < nkb) load_ops(kb + 1, ob);
          multiply(oa);
          if (kb + 1 < nkb) {
            if (kb + 2 < nkb) load_ops(kb + 2, oa);
            multiply(ob);
          }
        }
      } else {   // three output tiles: no registers left for a second operand set
        for (int kb = 0; kb < nkb; ++kb) {
          load_ops(kb, oa);
          multiply(oa);
        }
      }
    }
    // The next half's first Q / dout tile was requested a whole tile ago: wait for it here, before the dQ rows are
    // stored, so that the barrier below also publishes it and the next wait for memory comes a tile after the stores.
    wait_tile();
    bare_barrier();  // every wave has read its dS tiles: X becomes the staging area of this half's dQ rows
    {
      using C = Cfg<T, D>;
      T* stage = reinterpret_cast<T*>(smem + FC::X_OFF);
      T* srow = stage + ((wave & 3) * 32 + c32) * C::OSTRIDE;
      constexpr int NT1 = NMT - NT0;
      if (!part1) {
#pragma unroll
        for (int t = 0; t < NT0; ++t)
#pragma unroll
          for (int jj = 0; jj < 4; ++jj)
            store4<T>(srow + t * 32 + jj * 8 + 4 * g, dQ[t][4 * jj] * p.scale, dQ[t][4 * jj + 1] * p.scale, dQ[t][4 * jj + 2] * p.scale,
                      dQ[t][4 * jj + 3] * p.scale);
        if constexpr (TAIL)
          store_tail16<T, D, NMT>(stage + (wave & 3) * 32 * C::OSTRIDE, lane, [&](int hq, int e) { return dQ16[hq][e] * p.scale; });
      } else {
#pragma unroll
        for (int t = 0; t < NT1; ++t)
#pragma unroll
          for (int jj = 0; jj < 4; ++jj)
            store4<T>(srow + (NT0 + t) * 32 + jj * 8 + 4 * g, dQ[t][4 * jj] * p.scale, dQ[t][4 * jj + 1] * p.scale, dQ[t][4 * jj + 2] * p.scale,
                      dQ[t][4 * jj + 3] * p.scale);
      }
      bare_barrier();   // (no fence: tiles of the next half are in flight)
      T* gdq = reinterpret_cast<T*>(p.dq) + base(5);
      for (int v = tid; v < 128 * VPR; v += 512) {
        const int row = v / VPR, cv = v % VPR, qrow = half * 128 + row;
        if (qrow < p.Lq)
          *reinterpret_cast<u32x4*>(gdq + (int64_t)qrow * p.st[5][1] + cv * C::VEC) =
              *reinterpret_cast<const u32x4*>(stage + row * C::OSTRIDE + cv * C::VEC);
      }
      // (the next half's first barrier orders these staging reads before X is written again)
    }
  }

  // ---- dK, dV of this wave's 32 keys
  T* stage = reinterpret_cast<T*>(smem + FC::X_OFF);
  store_rows_transposed<T, D, 8, NMT>(stage, reinterpret_cast<T*>(p.dk) + base(6), p.st[6][1], 0, p.Lkv, tid,
                                      [&](int t, int i) { return dK[t][i] * p.scale; },
                                      [&](void* ws) {
                                        if constexpr (TAIL) store_tail16<T, D, NMT>(ws, lane, [&](int hq, int e) { return dK16[hq][e] * p.scale; });
                                      });
  store_rows_transposed<T, D, 8, NMT>(stage, reinterpret_cast<T*>(p.dv) + base(7), p.st[7][1], 0, p.Lkv, tid,
                                      [&](int t, int i) { return dV[t][i]; },
                                      [&](void* ws) {
                                        if constexpr (TAIL) store_tail16<T, D, NMT>(ws, lane, [&](int hq, int e) { return dV16[hq][e]; });
                                      });
}

template <int D>
static int launch_bwd_fused_t(const BwdParams& p, int BH, hipStream_t stream) {
  auto kern = attn_bwd_fused_bf16_kernel<D>;
  static bool lds_ok[64] = {};
  if (!ensure_dynamic_lds(kern, BwdFusedCfg<D>::LDS_BYTES, lds_ok)) return -7;
  return launch_kernel(kern, dim3((uint32_t)BH), dim3(512), BwdFusedCfg<D>::LDS_BYTES, stream, p);
}

template <int D>
static int launch_bwd_fast_t(const BwdParams& p, int BH, hipStream_t stream) {
  using F = BwdFastCfg<D, true>;
  constexpr int tiles = 2 * (2 * F::TBYTES + F::STAT) + 512;
  constexpr int stage = 128 * Cfg<__bf16, D>::OROWV * 16;
  constexpr int stage2 = 32 * kKvWaves * Cfg<__bf16, D>::OROWV * 16;
  constexpr int smem = tiles > stage2 ? tiles : stage2;
  constexpr int tiles1 = 2 * kDqSub * 2 * F::TBYTES + 512;
  constexpr int smem1 = tiles1 > stage ? tiles1 : stage;
  auto k1 = attn_bwd_dq_bf16_kernel<D, kDqSub>;
  auto k2 = attn_bwd_dkv_bf16_kernel<D, kKvWaves>;
  static bool lds_ok1[64] = {}, lds_ok2[64] = {};
  if (!ensure_dynamic_lds(k1, smem1, lds_ok1) || !ensure_dynamic_lds(k2, smem, lds_ok2)) return -7;
  const uint32_t nqb = (p.Lq + 127) / 128, nkb = (p.Lkv + 32 * kKvWaves - 1) / (32 * kKvWaves);
  if (int rc = launch_kernel(k1, dim3(nqb * (uint32_t)BH), dim3(256), smem1, stream, p)) return rc;
  return launch_kernel(k2, dim3(nkb * (uint32_t)BH), dim3(64 * kKvWaves), smem, stream, p);
}

// Policy: does the single-pass kernel take this case?  Whole (batch, head) units per work-group, every score tile formed
// once: 5 GEMM units where the kernel pair executes 7.  That also decides head dim 64, where the pair (124 / 166 registers,
// four / three work-groups per CU) is the faster schedule -- on all-zero operands B256 H16 N256 0.278 ms against 0.299 -- but
// both run into the package-power limit on data and the one that executes less wins: 0.40 -> 0.35 ms there,
// 0.085 -> 0.071 at B64 H12, 0.045 -> 0.043 at B32 H12, 0.0216 -> 0.0207 at B8 H16.
// (Head dim 128: K, the tile stages and the exchange area exceed the LDS.)
bool bwd_single_pass(int Lq, int Lkv, int D, int /*BH*/) {
  const int Lmax = std::max(Lq, Lkv);
  if (D != 64 && D != 72 && D != 80 && D != 96) return false;
  return Lmax >= kFusedMinRows && Lmax <= kFusedMaxRows;
}

bool plan_bwd_bf16_fast(int Lq, int Lkv, int D, int BH, char* buf, size_t n) {
  if (D != 64 && D != 72 && D != 80 && D != 96 && D != 128) return false;
  if (bwd_single_pass(Lq, Lkv, D, BH)) snprintf(buf, n, "dmf::attn_bwd_fused_bf16_kernel<%d>", D);
  else snprintf(buf, n, "dmf::attn_bwd_dq_bf16_kernel<%d, %d> + dmf::attn_bwd_dkv_bf16_kernel<%d, %d>", D, kDqSub, D, kKvWaves);
  return true;
}

// Returns 1 if there is no tuned kernel for the case (caller uses the generic ones).
int launch_bwd_bf16_fast(const BwdParams& p, int BH, int D, hipStream_t stream) {
  // 32-bit buffer addressing: every (batch, head) slab of rows must span < 2 GiB
  const int64_t max_row = std::max(std::max(std::max(p.st[0][1], p.st[1][1]), std::max(p.st[2][1], p.st[3][1])), p.st[4][1]);
  if (max_row * 2 * (int64_t)(std::max(p.Lq, p.Lkv) + 256) >= (int64_t)1 << 31) return 1;
  if (bwd_single_pass(p.Lq, p.Lkv, D, BH)) {
    switch (D) {
      case 64: return launch_bwd_fused_t<64>(p, BH, stream);
      case 72: return launch_bwd_fused_t<72>(p, BH, stream);
      case 80: return launch_bwd_fused_t<80>(p, BH, stream);
      case 96: return launch_bwd_fused_t<96>(p, BH, stream);
      default: break;
    }
  }
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
