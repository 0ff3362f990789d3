// Fused DiT-block glue kernels with forward-mode tangents (C ABI: include/dmf_block.h).
//
// All of these are single-pass, HBM-bound kernels: every operand is read once
// with 16-byte (bf16) / 2x16-byte (fp32) vector loads, every result is written
// once, arithmetic is fp32 in registers.  Row kernels (LayerNorm, RMSNorm) keep
// a whole row in the registers of one wave (LayerNorm) or of a 16-lane group
// (RMSNorm) so that statistics, primal, tangent and gradient come from one read.
// Reductions over the sequence (gradients of shift / scale / gate / gain) are
// two-stage: per-work-group partial sums in a caller-provided workspace, then a
// small second kernel that adds them in a fixed order.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <type_traits>

#include "../../include/dmf_block.h"
#include "attn_common.h"
#include "attn_kernels.h"

namespace dmf {
namespace blk {

constexpr int kWaves = 4;          // waves per work-group
constexpr int kThreads = 64 * kWaves;
constexpr int kChunkRows = 16;     // rows of one sample handled by one work-group in the reducing backward kernels
constexpr int kMaxC = 2048;        // 4 vectors of 8 per lane
constexpr int kRmsBlocksMax = 1024;

// ---- 8-wide loads / stores with a run-time (wave-uniform) element type -------------------------------------------

__device__ __forceinline__ void zero8(float (&o)[8]) {
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = 0.f;
}

// p == nullptr reads as zeros.  idx is an element index, a multiple of 8.
__device__ __forceinline__ void load8(const void* p, int bf16, int64_t idx, float (&o)[8]) {
  if (p == nullptr) {
    zero8(o);
  } else if (bf16) {
    const u32x4 r = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(p) + idx);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(r[i] << 16);
      o[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
    }
  } else {
    const f32x4* q = reinterpret_cast<const f32x4*>(static_cast<const float*>(p) + idx);
    const f32x4 a = q[0], b = q[1];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[i] = a[i];
      o[4 + i] = b[i];
    }
  }
}

__device__ __forceinline__ void store8(void* p, int bf16, int64_t idx, const float (&v)[8]) {
  if (bf16) {
    *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(p) + idx) =
        u32x4{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7])};
  } else {
    f32x4* q = reinterpret_cast<f32x4*>(static_cast<float*>(p) + idx);
    q[0] = f32x4{v[0], v[1], v[2], v[3]};
    q[1] = f32x4{v[4], v[5], v[6], v[7]};
  }
}

__device__ __forceinline__ float sum8(const float (&v)[8]) {
  return ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
}

// sum over the wave; every lane gets the same bits (no LDS traffic: DPP rotations inside the rows of 16 lanes, then the
// 16- and 32-lane swaps)
__device__ __forceinline__ float wave_sum(float v) {
  v = group16_sum(v);
  float even, odd;
  swap16f(v, even, odd);
  return xhalf_sum(even + odd);
}

// ---- a row of C elements held by one wave: lane owns columns (j*64 + lane)*8 .. +8, j < NV -------------------------

template <int NV>
struct Row {
  float v[NV][8];
};

template <int NV>
__device__ __forceinline__ void load_row(const void* p, int bf16, int64_t base, int C, int lane, Row<NV>& r) {
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int col = (j * 64 + lane) * 8;
    if (col < C) load8(p, bf16, base + col, r.v[j]);
    else zero8(r.v[j]);
  }
}

template <int NV>
__device__ __forceinline__ void store_row(void* p, int bf16, int64_t base, int C, int lane, const Row<NV>& r) {
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int col = (j * 64 + lane) * 8;
    if (col < C) store8(p, bf16, base + col, r.v[j]);
  }
}

template <int NV>
__device__ __forceinline__ float row_sum(const Row<NV>& r) {
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) s += sum8(r.v[j]);
  return wave_sum(s);
}

template <int NV>
__device__ __forceinline__ float row_dot(const Row<NV>& a, const Row<NV>& b) {
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) s = fmaf(a.v[j][e], b.v[j][e], s);
  return wave_sum(s);
}

// In place: x -> xh = (x - mean) * rstd (padding columns stay 0).  Returns rstd.
template <int NV>
__device__ __forceinline__ float normalize_row(Row<NV>& x, int C, int lane, float eps) {
  const float inv_c = 1.f / static_cast<float>(C);
  const float mean = row_sum(x) * inv_c;
  float q = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const bool live = (j * 64 + lane) * 8 < C;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float d = live ? x.v[j][e] - mean : 0.f;
      x.v[j][e] = d;
      q = fmaf(d, d, q);
    }
  }
  const float rstd = 1.f / sqrtf(wave_sum(q) * inv_c + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) x.v[j][e] *= rstd;
  return rstd;
}

// t -> rstd * (t - mean(t) - xh * mean(xh * t)): the tangent (or, with t a cotangent, the gradient) of the
// normalisation through the row statistics.
template <int NV>
__device__ __forceinline__ void project_row(Row<NV>& t, const Row<NV>& xh, float rstd, int C, int lane) {
  const float inv_c = 1.f / static_cast<float>(C);
  const float m1 = row_sum(t) * inv_c;
  const float m2 = row_dot(xh, t) * inv_c;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const bool live = (j * 64 + lane) * 8 < C;
#pragma unroll
    for (int e = 0; e < 8; ++e) t.v[j][e] = live ? rstd * (t.v[j][e] - m1 - xh.v[j][e] * m2) : 0.f;
  }
}

// ---- LayerNorm + modulate -----------------------------------------------------------------------------------------

struct LnFwdParams {
  const void *x, *tx, *shift, *scale, *tshift, *tscale;
  void *y, *ty;
  int64_t rows, ms[4];
  int L, C;
  float eps;
  int xbf, mbf, ybf;
};

template <int NV, bool JVP>
__global__ __launch_bounds__(kThreads) void ln_modulate_fwd_kernel(LnFwdParams p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kWaves + wave;
  if (row >= p.rows) return;  // no work-group barrier in this kernel
  const int64_t b = row / p.L, base = row * p.C;
  Row<NV> xh, t;
  load_row(p.x, p.xbf, base, p.C, lane, xh);
  if (JVP) load_row(p.tx, p.xbf, base, p.C, lane, t);
  const float rstd = normalize_row(xh, p.C, lane, p.eps);
  if (JVP) project_row(t, xh, rstd, p.C, lane);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int col = (j * 64 + lane) * 8;
    if (col >= p.C) continue;
    float sh[8], sc[8], out[8];
    load8(p.shift, p.mbf, b * p.ms[0] + col, sh);
    load8(p.scale, p.mbf, b * p.ms[1] + col, sc);
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = fmaf(xh.v[j][e], 1.f + sc[e], sh[e]);
    store8(p.y, p.ybf, base + col, out);
    if (JVP) {
      float tsh[8], tsc[8];
      load8(p.tshift, p.mbf, b * p.ms[2] + col, tsh);
      load8(p.tscale, p.mbf, b * p.ms[3] + col, tsc);
#pragma unroll
      for (int e = 0; e < 8; ++e) out[e] = fmaf(t.v[j][e], 1.f + sc[e], fmaf(xh.v[j][e], tsc[e], tsh[e]));
      store8(p.ty, p.ybf, base + col, out);
    }
  }
}

// Adds the per-wave column accumulators of a work-group and writes them as one partial-sum row.
// acc[k]: K accumulators; out: partial + k*C; LDS: (kWaves-1) * K * NV * 512 floats.
template <int NV, int K>
__device__ __forceinline__ void reduce_waves_to_partial(Row<NV> (&acc)[K], float* lds, float* out, int C, int lane,
                                                        int wave) {
  constexpr int kRow = NV * 512;
  if (wave > 0) {
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
      for (int j = 0; j < NV; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) lds[((wave - 1) * K + k) * kRow + (j * 64 + lane) * 8 + e] = acc[k].v[j][e];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int col = (j * 64 + lane) * 8;
        if (col >= C) continue;
        float s[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float a = acc[k].v[j][e];
          for (int w = 0; w < kWaves - 1; ++w) a += lds[(w * K + k) * kRow + col + e];
          s[e] = a;
        }
        store8(out + static_cast<int64_t>(k) * C, 0, col, s);
      }
  }
}

struct LnBwdParams {
  const void *gy, *x, *scale, *gres;  // gres: optional gradient reaching x from its other consumers, added to gx
  void* gx;
  float* partial;  // (B, nchunk, 2, C): [0] sum gy, [1] sum gy * xh
  int64_t ss;
  int L, C, nchunk;
  float eps;
  int xbf, mbf, gbf;
};

template <int NV>
__global__ __launch_bounds__(kThreads) void ln_modulate_bwd_kernel(LnBwdParams p) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t b = blockIdx.x / p.nchunk;
  const int chunk = blockIdx.x % p.nchunk;
  const int r1 = min(p.L, (chunk + 1) * kChunkRows);
  Row<NV> one_plus_scale, acc[2];
  load_row(p.scale, p.mbf, b * p.ss, p.C, lane, one_plus_scale);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    zero8(acc[0].v[j]);
    zero8(acc[1].v[j]);
#pragma unroll
    for (int e = 0; e < 8; ++e) one_plus_scale.v[j][e] += 1.f;
  }
  for (int r = chunk * kChunkRows + wave; r < r1; r += kWaves) {
    const int64_t base = (b * p.L + r) * p.C;
    Row<NV> xh, g;
    load_row(p.x, p.xbf, base, p.C, lane, xh);
    load_row(p.gy, p.gbf, base, p.C, lane, g);
    const float rstd = normalize_row(xh, p.C, lane, p.eps);
#pragma unroll
    for (int j = 0; j < NV; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        acc[0].v[j][e] += g.v[j][e];
        acc[1].v[j][e] = fmaf(g.v[j][e], xh.v[j][e], acc[1].v[j][e]);
        g.v[j][e] *= one_plus_scale.v[j][e];
      }
    project_row(g, xh, rstd, p.C, lane);
    if (p.gres != nullptr) {
      load_row(p.gres, p.xbf, base, p.C, lane, xh);
#pragma unroll
      for (int j = 0; j < NV; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) g.v[j][e] += xh.v[j][e];
    }
    store_row(p.gx, p.xbf, base, p.C, lane, g);
  }
  reduce_waves_to_partial<NV, 2>(acc, lds, p.partial + static_cast<int64_t>(blockIdx.x) * 2 * p.C, p.C, lane, wave);
}

// out[k][b][c] = sum_chunk partial[b][chunk][k][c]; out[k] dense (B, C) of the given element type.
struct ReduceParams {
  const float* partial;
  void* out[2];
  int64_t total;  // B * K * C / 8 vectors
  int nchunk, K, C;
  int obf;
};

// Work-group: 64 output vectors (8 columns each); wave w adds chunks w, w+4, ...; the four waves meet in LDS.
__global__ __launch_bounds__(kThreads) void reduce_partials_kernel(ReduceParams p) {
  __shared__ float lds[kWaves - 1][64 * 8];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t v = static_cast<int64_t>(blockIdx.x) * 64 + lane;
  const bool live = v < p.total;
  const int vec_per_row = p.C / 8;
  const int col = static_cast<int>(v % vec_per_row) * 8;
  const int64_t bk = v / vec_per_row;
  const int k = static_cast<int>(bk % p.K);
  const int64_t b = bk / p.K;
  float s[8];
  zero8(s);
  if (live) {
#pragma unroll 4
    for (int c = wave; c < p.nchunk; c += kWaves) {
      float t[8];
      load8(p.partial, 0, ((b * p.nchunk + c) * p.K + k) * p.C + col, t);
#pragma unroll
      for (int e = 0; e < 8; ++e) s[e] += t[e];
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int e = 0; e < 8; ++e) lds[wave - 1][lane * 8 + e] = s[e];
  }
  __syncthreads();
  if (wave == 0 && live) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      for (int w = 0; w < kWaves - 1; ++w) s[e] += lds[w][lane * 8 + e];
    store8(p.out[k], p.obf, b * p.C + col, s);
  }
}

// ---- gated residual -----------------------------------------------------------------------------------------------

struct GateFwdParams {
  const void *x, *tx, *gate, *tgate, *h, *th;
  void *y, *ty;
  int64_t total, gs[2];  // total = B*L*C/8 vectors
  int L, C;
  int xbf, mbf, hbf;
};

template <bool JVP>
__global__ __launch_bounds__(kThreads) void gate_residual_fwd_kernel(GateFwdParams p) {
  const int64_t v = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (v >= p.total) return;
  const int vec_per_row = p.C / 8;
  const int col = static_cast<int>(v % vec_per_row) * 8;
  const int64_t row = v / vec_per_row, b = row / p.L, idx = v * 8;
  float x[8], g[8], h[8], out[8];
  load8(p.x, p.xbf, idx, x);
  load8(p.h, p.hbf, idx, h);
  load8(p.gate, p.mbf, b * p.gs[0] + col, g);
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = fmaf(g[e], h[e], x[e]);
  store8(p.y, p.xbf, idx, out);
  if (JVP) {
    float tx[8], tg[8], th[8];
    load8(p.tx, p.xbf, idx, tx);
    load8(p.th, p.hbf, idx, th);
    load8(p.tgate, p.mbf, b * p.gs[1] + col, tg);
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = fmaf(tg[e], h[e], fmaf(g[e], th[e], tx[e]));
    store8(p.ty, p.xbf, idx, out);
  }
}

struct GateBwdParams {
  const void *gy, *gate, *h;
  void* gh;
  float* partial;  // (B, nchunk, 1, C)
  int64_t gs;
  int L, C, nchunk;
  int gbf, mbf, hbf;
};

template <int NV>
__global__ __launch_bounds__(kThreads) void gate_residual_bwd_kernel(GateBwdParams p) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t b = blockIdx.x / p.nchunk;
  const int chunk = blockIdx.x % p.nchunk;
  const int r1 = min(p.L, (chunk + 1) * kChunkRows);
  Row<NV> gate, acc[1];
  load_row(p.gate, p.mbf, b * p.gs, p.C, lane, gate);
#pragma unroll
  for (int j = 0; j < NV; ++j) zero8(acc[0].v[j]);
  for (int r = chunk * kChunkRows + wave; r < r1; r += kWaves) {
    const int64_t base = (b * p.L + r) * p.C;
    Row<NV> g, h;
    load_row(p.gy, p.gbf, base, p.C, lane, g);
    load_row(p.h, p.hbf, base, p.C, lane, h);
#pragma unroll
    for (int j = 0; j < NV; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        acc[0].v[j][e] = fmaf(g.v[j][e], h.v[j][e], acc[0].v[j][e]);
        g.v[j][e] *= gate.v[j][e];
      }
    store_row(p.gh, p.hbf, base, p.C, lane, g);
  }
  reduce_waves_to_partial<NV, 1>(acc, lds, p.partial + static_cast<int64_t>(blockIdx.x) * p.C, p.C, lane, wave);
}

// ---- gated residual fused with the LayerNorm + modulate that consumes it ---------------------------------------------
// y = x + gate * h;  z = LayerNorm(y) * (1 + scale) + shift  (and tangents): the residual stream is read once and
// written once per half block instead of being re-read by a separate normalisation kernel.

struct ResLnFwdParams {
  const void *x, *tx, *gate, *tgate, *h, *th, *shift, *scale, *tshift, *tscale;
  void *y, *ty, *z, *tz;
  int64_t rows, ms[6];  // batch strides of gate, tgate, shift, scale, tshift, tscale
  int L, C;
  float eps;
  int xbf, mbf, hbf, zbf;
};

template <int NV, bool JVP>
__global__ __launch_bounds__(kThreads) void residual_ln_modulate_fwd_kernel(ResLnFwdParams p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kWaves + wave;
  if (row >= p.rows) return;  // no work-group barrier in this kernel
  const int64_t b = row / p.L, base = row * p.C;
  Row<NV> y, t, h;
  load_row(p.x, p.xbf, base, p.C, lane, y);
  load_row(p.h, p.hbf, base, p.C, lane, h);
  if (JVP) load_row(p.tx, p.xbf, base, p.C, lane, t);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int col = (j * 64 + lane) * 8;
    if (col >= p.C) continue;
    float g[8];
    load8(p.gate, p.mbf, b * p.ms[0] + col, g);
#pragma unroll
    for (int e = 0; e < 8; ++e) y.v[j][e] = fmaf(g[e], h.v[j][e], y.v[j][e]);
    store8(p.y, p.xbf, base + col, y.v[j]);
    if (JVP) {
      float tg[8], th[8];
      load8(p.tgate, p.mbf, b * p.ms[1] + col, tg);
      load8(p.th, p.hbf, base + col, th);
#pragma unroll
      for (int e = 0; e < 8; ++e) t.v[j][e] = fmaf(tg[e], h.v[j][e], fmaf(g[e], th[e], t.v[j][e]));
      store8(p.ty, p.xbf, base + col, t.v[j]);
    }
  }
  const float rstd = normalize_row(y, p.C, lane, p.eps);
  if (JVP) project_row(t, y, rstd, p.C, lane);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int col = (j * 64 + lane) * 8;
    if (col >= p.C) continue;
    float sh[8], sc[8], out[8];
    load8(p.shift, p.mbf, b * p.ms[2] + col, sh);
    load8(p.scale, p.mbf, b * p.ms[3] + col, sc);
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = fmaf(y.v[j][e], 1.f + sc[e], sh[e]);
    store8(p.z, p.zbf, base + col, out);
    if (JVP) {
      float tsh[8], tsc[8];
      load8(p.tshift, p.mbf, b * p.ms[4] + col, tsh);
      load8(p.tscale, p.mbf, b * p.ms[5] + col, tsc);
#pragma unroll
      for (int e = 0; e < 8; ++e) out[e] = fmaf(t.v[j][e], 1.f + sc[e], fmaf(y.v[j][e], tsc[e], tsh[e]));
      store8(p.tz, p.zbf, base + col, out);
    }
  }
}

// ---- pointwise activations: GELU (tanh approximation) and SiLU ------------------------------------------------------

constexpr float kGeluA = 0.7978845608028654f;  // sqrt(2/pi)
constexpr float kGeluB = 0.044715f;
enum { kActGelu = 0, kActSilu = 1 };

// y = act(x), dy = act'(x)
template <int ACT>
__device__ __forceinline__ void act_eval(float x, float& y, float& dy) {
  if (ACT == kActGelu) {
    const float x2 = x * x;
    const float t = tanhf(kGeluA * x * fmaf(kGeluB, x2, 1.f));
    y = 0.5f * x * (1.f + t);
    dy = 0.5f * (1.f + t) + 0.5f * x * (1.f - t * t) * kGeluA * fmaf(3.f * kGeluB, x2, 1.f);
  } else {
    const float sg = 1.f / (1.f + expf(-x));
    y = x * sg;
    dy = sg * fmaf(x, 1.f - sg, 1.f);
  }
}

struct ActParams {
  const void *x, *t;  // t: tangent (forward) or cotangent (backward)
  void *y, *ty;       // backward writes gx to ty
  int64_t total;      // n / 8
  int xbf, ybf;       // element types of x (and tx, gx) and of y (and ty, gy)
};

// MODE 0: y only; 1: y and ty = act'(x) * t; 2: ty = act'(x) * t only (backward, t = gy).
template <int ACT, int MODE>
__global__ __launch_bounds__(kThreads) void act_kernel(ActParams p) {
  const int64_t v = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (v >= p.total) return;
  float x[8], t[8], y[8], d[8];
  load8(p.x, p.xbf, v * 8, x);
  if (MODE) load8(p.t, MODE == 2 ? p.ybf : p.xbf, v * 8, t);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    act_eval<ACT>(x[e], y[e], d[e]);
    if (MODE) d[e] *= t[e];
  }
  if (MODE != 2) store8(p.y, p.ybf, v * 8, y);
  if (MODE) store8(p.ty, MODE == 2 ? p.xbf : p.ybf, v * 8, d);
}

// ---- per-head RMS norm --------------------------------------------------------------------------------------------
// A 16-lane group owns one (b, l, h) row (lane i of the group holds elements 8i..8i+7, lanes past D/8 idle), so a
// wave covers 4 rows and a work-group 16.

struct RmsParams {
  const void *x, *tx, *gain, *gy;
  void *y, *ty;    // backward: y = gx
  float* partial;  // backward: (nblocks, D)
  int64_t rows, sx[3], stx[3];   // element strides {sB, sL, sH} of x and of tx (forward) / gx (backward)
  int L, H, D;
  float eps;
  int bf, gbf;
};

__device__ __forceinline__ int64_t strided_row(int64_t row, int L, int H, const int64_t (&s)[3]) {
  const int64_t h = row % H, bl = row / H;
  return (bl / L) * s[0] + (bl % L) * s[1] + h * s[2];
}

template <bool JVP>
__global__ __launch_bounds__(kThreads) void rmsnorm_fwd_kernel(RmsParams p) {
  const int sub = threadIdx.x & 15;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * (kThreads / 16) + (threadIdx.x >> 4);
  const int col = sub * 8;
  const bool live = row < p.rows && col < p.D;
  // every lane takes part in the group reductions; dead lanes contribute zeros
  float x[8], t[8], g[8], out[8];
  zero8(x);
  zero8(t);
  if (live) {
    load8(p.x, p.bf, strided_row(row, p.L, p.H, p.sx) + col, x);
    if (JVP) load8(p.tx, p.bf, strided_row(row, p.L, p.H, p.stx) + col, t);
  }
  float ss = 0.f, st = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    ss = fmaf(x[e], x[e], ss);
    st = fmaf(x[e], t[e], st);
  }
  const float inv_d = 1.f / static_cast<float>(p.D);
  const float r = 1.f / sqrtf(group16_sum(ss) * inv_d + p.eps);
  float dr = 0.f;
  if (JVP) dr = -r * r * r * group16_sum(st) * inv_d;
  if (!live) return;
  load8(p.gain, p.gbf, col, g);
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = x[e] * r * g[e];
  store8(p.y, p.bf, row * p.D + col, out);
  if (JVP) {
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = fmaf(t[e], r, x[e] * dr) * g[e];
    store8(p.ty, p.bf, row * p.D + col, out);
  }
}

__global__ __launch_bounds__(kThreads) void rmsnorm_bwd_kernel(RmsParams p) {
  __shared__ float lds[kWaves][128];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, sub = threadIdx.x & 15;
  const int col = sub * 8;
  const bool col_live = col < p.D;
  const float inv_d = 1.f / static_cast<float>(p.D);
  float gain[8], acc[8];
  zero8(gain);
  zero8(acc);
  if (col_live) load8(p.gain, p.gbf, col, gain);
  const int64_t rows_per_pass = static_cast<int64_t>(gridDim.x) * (kThreads / 16);
  const int64_t npass = (p.rows + rows_per_pass - 1) / rows_per_pass;  // same trip count for every lane
  for (int64_t it = 0; it < npass; ++it) {
    const int64_t row = it * rows_per_pass + static_cast<int64_t>(blockIdx.x) * (kThreads / 16) + (threadIdx.x >> 4);
    const bool live = row < p.rows && col_live;
    float x[8], g[8];
    zero8(x);
    zero8(g);
    if (live) {
      load8(p.x, p.bf, strided_row(row, p.L, p.H, p.sx) + col, x);
      load8(p.gy, p.bf, row * p.D + col, g);
    }
    float ss = 0.f, sg = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      ss = fmaf(x[e], x[e], ss);
      sg = fmaf(x[e], g[e] * gain[e], sg);
    }
    const float r = 1.f / sqrtf(group16_sum(ss) * inv_d + p.eps);
    const float c = r * r * r * group16_sum(sg) * inv_d;
    if (live) {
      float out[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        acc[e] = fmaf(g[e], x[e] * r, acc[e]);
        out[e] = fmaf(g[e] * gain[e], r, -x[e] * c);
      }
      store8(p.y, p.bf, strided_row(row, p.L, p.H, p.stx) + col, out);   // stx: strides of gx in this kernel
    }
  }
  // the four lane groups of a wave, then the waves of the work-group
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    acc[e] += __shfl_xor(acc[e], 16);
    acc[e] += __shfl_xor(acc[e], 32);
  }
  if (lane < 16) {
#pragma unroll
    for (int e = 0; e < 8; ++e) lds[wave][col + e] = acc[e];
  }
  __syncthreads();
  if (wave == 0 && lane < 16 && col_live) {
    float s[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float a = 0.f;
      for (int w = 0; w < kWaves; ++w) a += lds[w][col + e];
      s[e] = a;
    }
    store8(p.partial, 0, static_cast<int64_t>(blockIdx.x) * p.D + col, s);
  }
}

// ---- column sums of a dense (rows, C) matrix ----------------------------------------------------------------------
// Work-group (x, y): rows [x*kColsumRows, +kColsumRows), 64 vector columns starting at y*64.  Wave w takes rows
// w, w+4, ... of the chunk (four loads in flight per lane), the four waves are added through LDS.

constexpr int kColsumRows = 64;

struct ColsumParams {
  const void* x;
  float* partial;  // (nchunk, C)
  int64_t rows;
  int C;
  int xbf;
};

__global__ __launch_bounds__(kThreads) void colsum_kernel(ColsumParams p) {
  __shared__ float lds[kWaves - 1][64 * 8];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = (blockIdx.y * 64 + lane) * 8;
  const bool live = col < p.C;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * kColsumRows;
  const int64_t r1 = r0 + kColsumRows < p.rows ? r0 + kColsumRows : p.rows;
  float acc[8];
  zero8(acc);
  if (live) {
    int64_t r = r0 + wave;
    for (; r + 3 * kWaves < r1; r += 4 * kWaves) {
      float v[4][8];
#pragma unroll
      for (int u = 0; u < 4; ++u) load8(p.x, p.xbf, (r + u * kWaves) * p.C + col, v[u]);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += (v[0][e] + v[1][e]) + (v[2][e] + v[3][e]);
    }
    for (; r < r1; r += kWaves) {
      float v[8];
      load8(p.x, p.xbf, r * p.C + col, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += v[e];
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int e = 0; e < 8; ++e) lds[wave - 1][lane * 8 + e] = acc[e];
  }
  __syncthreads();
  if (wave == 0 && live) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      for (int w = 0; w < kWaves - 1; ++w) acc[e] += lds[w][lane * 8 + e];
    store8(p.partial, 0, static_cast<int64_t>(blockIdx.x) * p.C + col, acc);
  }
}

// ---- host side ----------------------------------------------------------------------------------------------------

inline bool dtype_ok(int d) { return d == DMF_ATTN_F32 || d == DMF_ATTN_BF16; }
inline int ebytes(int d) { return d == DMF_ATTN_BF16 ? 2 : 4; }
inline bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }
inline int nchunks(int L) { return (L + kChunkRows - 1) / kChunkRows; }


// Shape checks shared by the (B, L, C) entry points.
inline int check_blc(int B, int L, int C) {
  if (B < 1 || L < 1 || C < 8 || C % 8 || C > kMaxC) return DMF_ATTN_ESHAPE;
  if (static_cast<int64_t>(B) * L * (C / 8) / kThreads + 1 > 0x7fffffffLL) return DMF_ATTN_ESHAPE;
  return DMF_ATTN_OK;
}

// A (B, C) modulation operand: pointer alignment and batch stride.
inline int check_mod(const void* p, int64_t stride, int dtype, bool required) {
  if (p == nullptr) return required ? DMF_ATTN_ENULL : DMF_ATTN_OK;
  if (!aligned16(p)) return DMF_ATTN_EALIGN;
  if (stride < 0 || (stride * ebytes(dtype)) % 16) return DMF_ATTN_ESTRIDE;
  return DMF_ATTN_OK;
}

template <typename F>
inline int dispatch_nv(int C, F&& f) {
  switch ((C + 511) / 512) {
    case 1: return f(std::integral_constant<int, 1>{});
    case 2: return f(std::integral_constant<int, 2>{});
    case 3: return f(std::integral_constant<int, 3>{});
    default: return f(std::integral_constant<int, 4>{});
  }
}

inline int reduce_partials(const float* partial, void* out0, void* out1, int B, int nchunk, int K, int C, int obf,
                           hipStream_t s) {
  ReduceParams r{};
  r.partial = partial;
  r.out[0] = out0;
  r.out[1] = out1;
  r.total = static_cast<int64_t>(B) * K * (C / 8);
  r.nchunk = nchunk;
  r.K = K;
  r.C = C;
  r.obf = obf;
  const unsigned grid = static_cast<unsigned>((r.total + 63) / 64);
  return launch_kernel(reduce_partials_kernel, dim3(grid), dim3(kThreads), 0, s, r);
}

template <int ACT>
inline int act_impl(const void* x, const void* t, void* y, void* ty, int64_t n, int x_dtype, int y_dtype, int mode,
                    void* stream) {
  if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return DMF_ATTN_EDTYPE;
  if (n < 8 || n % 8 || n / 8 / kThreads + 1 > 0x7fffffffLL) return DMF_ATTN_ESHAPE;
  if (!x || (mode != 2 && !y) || (mode && (!t || !ty))) return DMF_ATTN_ENULL;
  if (!aligned16(x) || !aligned16(t) || !aligned16(y) || !aligned16(ty)) return DMF_ATTN_EALIGN;
  ActParams p{};
  p.x = x; p.t = t; p.y = y; p.ty = ty; p.total = n / 8;
  p.xbf = x_dtype == DMF_ATTN_BF16; p.ybf = y_dtype == DMF_ATTN_BF16;
  const unsigned grid = static_cast<unsigned>((p.total + kThreads - 1) / kThreads);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (mode == 0) return launch_kernel(act_kernel<ACT, 0>, dim3(grid), dim3(kThreads), 0, s, p);
  if (mode == 1) return launch_kernel(act_kernel<ACT, 1>, dim3(grid), dim3(kThreads), 0, s, p);
  return launch_kernel(act_kernel<ACT, 2>, dim3(grid), dim3(kThreads), 0, s, p);
}

}  // namespace blk
}  // namespace dmf

using namespace dmf::blk;
using dmf::launch_kernel;

extern "C" {

int64_t dmf_block_workspace_floats(int which, int B, int L, int dim) {
  if (B < 1 || L < 1 || dim < 1) return 0;
  switch (which) {
    case 0: return static_cast<int64_t>(B) * nchunks(L) * 2 * dim;
    case 1: return static_cast<int64_t>(B) * nchunks(L) * dim;
    case 2: return static_cast<int64_t>(kRmsBlocksMax) * dim;
    case 3: return ((static_cast<int64_t>(B) * L + kColsumRows - 1) / kColsumRows) * dim;
    default: return 0;
  }
}

int dmf_ln_modulate_fwd(const void* x, const void* tx, const void* shift, const void* scale, const void* tshift,
                        const void* tscale, void* y, void* ty, const int64_t* mod_strides, int B, int L, int C,
                        float eps, int x_dtype, int mod_dtype, int y_dtype, void* stream) {
  if (!dtype_ok(x_dtype) || !dtype_ok(mod_dtype) || !dtype_ok(y_dtype)) return DMF_ATTN_EDTYPE;
  if (int rc = check_blc(B, L, C)) return rc;
  if (!x || !y || !shift || !scale || !mod_strides) return DMF_ATTN_ENULL;
  if (!aligned16(x) || !aligned16(y) || !aligned16(tx) || !aligned16(ty)) return DMF_ATTN_EALIGN;
  const void* mods[4] = {shift, scale, tshift, tscale};
  for (int i = 0; i < 4; ++i)
    if (int rc = check_mod(mods[i], mod_strides[i], mod_dtype, i < 2)) return rc;
  LnFwdParams p{};
  p.x = x; p.tx = tx; p.shift = shift; p.scale = scale; p.tshift = tshift; p.tscale = tscale;
  p.y = y; p.ty = ty;
  p.rows = static_cast<int64_t>(B) * L;
  for (int i = 0; i < 4; ++i) p.ms[i] = mod_strides[i];
  p.L = L; p.C = C; p.eps = eps;
  p.xbf = x_dtype == DMF_ATTN_BF16; p.mbf = mod_dtype == DMF_ATTN_BF16; p.ybf = y_dtype == DMF_ATTN_BF16;
  const unsigned grid = static_cast<unsigned>((p.rows + kWaves - 1) / kWaves);
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dispatch_nv(C, [&](auto nv) {
    constexpr int NV = decltype(nv)::value;
    if (ty) return launch_kernel(ln_modulate_fwd_kernel<NV, true>, dim3(grid), dim3(kThreads), 0, s, p);
    return launch_kernel(ln_modulate_fwd_kernel<NV, false>, dim3(grid), dim3(kThreads), 0, s, p);
  });
}

int dmf_ln_modulate_bwd(const void* gy, const void* x, const void* scale, const void* gres, void* gx, void* gshift,
                        void* gscale, float* workspace, int64_t scale_stride, int B, int L, int C, float eps, int x_dtype,
                        int mod_dtype, int gy_dtype, void* stream) {
  if (!dtype_ok(x_dtype) || !dtype_ok(mod_dtype) || !dtype_ok(gy_dtype)) return DMF_ATTN_EDTYPE;
  if (int rc = check_blc(B, L, C)) return rc;
  if (!gy || !x || !scale || !gx || !gshift || !gscale || !workspace) return DMF_ATTN_ENULL;
  if (!aligned16(gy) || !aligned16(x) || !aligned16(gres) || !aligned16(gx) || !aligned16(gshift) ||
      !aligned16(gscale) || !aligned16(workspace))
    return DMF_ATTN_EALIGN;
  if (int rc = check_mod(scale, scale_stride, mod_dtype, true)) return rc;
  LnBwdParams p{};
  p.gy = gy; p.x = x; p.scale = scale; p.gres = gres; p.gx = gx; p.partial = workspace; p.ss = scale_stride;
  p.L = L; p.C = C; p.nchunk = nchunks(L); p.eps = eps;
  p.xbf = x_dtype == DMF_ATTN_BF16; p.mbf = mod_dtype == DMF_ATTN_BF16; p.gbf = gy_dtype == DMF_ATTN_BF16;
  const unsigned grid = static_cast<unsigned>(B) * p.nchunk;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int rc = dispatch_nv(C, [&](auto nv) {
    constexpr int NV = decltype(nv)::value;
    constexpr size_t lds = (kWaves - 1) * 2 * NV * 512 * sizeof(float);
    return launch_kernel(ln_modulate_bwd_kernel<NV>, dim3(grid), dim3(kThreads), lds, s, p);
  });
  if (rc) return rc;
  return reduce_partials(workspace, gshift, gscale, B, p.nchunk, 2, C, p.mbf, s);
}

int dmf_gate_residual_fwd(const void* x, const void* tx, const void* gate, const void* tgate, const void* h,
                          const void* th, void* y, void* ty, const int64_t* gate_strides, int B, int L, int C,
                          int x_dtype, int mod_dtype, int h_dtype, void* stream) {
  if (!dtype_ok(x_dtype) || !dtype_ok(mod_dtype) || !dtype_ok(h_dtype)) return DMF_ATTN_EDTYPE;
  if (int rc = check_blc(B, L, C)) return rc;
  if (!x || !gate || !h || !y || !gate_strides) return DMF_ATTN_ENULL;
  if (!aligned16(x) || !aligned16(tx) || !aligned16(h) || !aligned16(th) || !aligned16(y) || !aligned16(ty))
    return DMF_ATTN_EALIGN;
  if (int rc = check_mod(gate, gate_strides[0], mod_dtype, true)) return rc;
  if (int rc = check_mod(tgate, gate_strides[1], mod_dtype, false)) return rc;
  GateFwdParams p{};
  p.x = x; p.tx = tx; p.gate = gate; p.tgate = tgate; p.h = h; p.th = th; p.y = y; p.ty = ty;
  p.total = static_cast<int64_t>(B) * L * (C / 8);
  p.gs[0] = gate_strides[0]; p.gs[1] = gate_strides[1];
  p.L = L; p.C = C;
  p.xbf = x_dtype == DMF_ATTN_BF16; p.mbf = mod_dtype == DMF_ATTN_BF16; p.hbf = h_dtype == DMF_ATTN_BF16;
  const unsigned grid = static_cast<unsigned>((p.total + kThreads - 1) / kThreads);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (ty) return launch_kernel(gate_residual_fwd_kernel<true>, dim3(grid), dim3(kThreads), 0, s, p);
  return launch_kernel(gate_residual_fwd_kernel<false>, dim3(grid), dim3(kThreads), 0, s, p);
}

int dmf_gate_residual_bwd(const void* gy, const void* gate, const void* h, void* gh, void* ggate, float* workspace,
                          int64_t gate_stride, int B, int L, int C, int gy_dtype, int mod_dtype, int h_dtype,
                          void* stream) {
  if (!dtype_ok(gy_dtype) || !dtype_ok(mod_dtype) || !dtype_ok(h_dtype)) return DMF_ATTN_EDTYPE;
  if (int rc = check_blc(B, L, C)) return rc;
  if (!gy || !gate || !h || !gh || !ggate || !workspace) return DMF_ATTN_ENULL;
  if (!aligned16(gy) || !aligned16(h) || !aligned16(gh) || !aligned16(ggate) || !aligned16(workspace))
    return DMF_ATTN_EALIGN;
  if (int rc = check_mod(gate, gate_stride, mod_dtype, true)) return rc;
  GateBwdParams p{};
  p.gy = gy; p.gate = gate; p.h = h; p.gh = gh; p.partial = workspace; p.gs = gate_stride;
  p.L = L; p.C = C; p.nchunk = nchunks(L);
  p.gbf = gy_dtype == DMF_ATTN_BF16; p.mbf = mod_dtype == DMF_ATTN_BF16; p.hbf = h_dtype == DMF_ATTN_BF16;
  const unsigned grid = static_cast<unsigned>(B) * p.nchunk;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int rc = dispatch_nv(C, [&](auto nv) {
    constexpr int NV = decltype(nv)::value;
    constexpr size_t lds = (kWaves - 1) * NV * 512 * sizeof(float);
    return launch_kernel(gate_residual_bwd_kernel<NV>, dim3(grid), dim3(kThreads), lds, s, p);
  });
  if (rc) return rc;
  return reduce_partials(workspace, ggate, nullptr, B, p.nchunk, 1, C, p.mbf, s);
}

int dmf_residual_ln_modulate_fwd(const void* x, const void* tx, const void* gate, const void* tgate, const void* h,
                                 const void* th, const void* shift, const void* scale, const void* tshift,
                                 const void* tscale, void* y, void* ty, void* z, void* tz, const int64_t* mod_strides,
                                 int B, int L, int C, float eps, int x_dtype, int mod_dtype, int h_dtype, int z_dtype,
                                 void* stream) {
  if (!dtype_ok(x_dtype) || !dtype_ok(mod_dtype) || !dtype_ok(h_dtype) || !dtype_ok(z_dtype)) return DMF_ATTN_EDTYPE;
  if (int rc = check_blc(B, L, C)) return rc;
  if (!x || !gate || !h || !shift || !scale || !y || !z || !mod_strides) return DMF_ATTN_ENULL;
  const bool jvp = ty != nullptr || tz != nullptr;
  if (jvp && (!ty || !tz)) return DMF_ATTN_ENULL;
  if (!aligned16(x) || !aligned16(tx) || !aligned16(h) || !aligned16(th) || !aligned16(y) || !aligned16(ty) ||
      !aligned16(z) || !aligned16(tz))
    return DMF_ATTN_EALIGN;
  const void* mods[6] = {gate, tgate, shift, scale, tshift, tscale};
  const bool required[6] = {true, false, true, true, false, false};
  for (int i = 0; i < 6; ++i)
    if (int rc = check_mod(mods[i], mod_strides[i], mod_dtype, required[i])) return rc;
  ResLnFwdParams p{};
  p.x = x; p.tx = tx; p.gate = gate; p.tgate = tgate; p.h = h; p.th = th;
  p.shift = shift; p.scale = scale; p.tshift = tshift; p.tscale = tscale;
  p.y = y; p.ty = ty; p.z = z; p.tz = tz;
  p.rows = static_cast<int64_t>(B) * L;
  for (int i = 0; i < 6; ++i) p.ms[i] = mod_strides[i];
  p.L = L; p.C = C; p.eps = eps;
  p.xbf = x_dtype == DMF_ATTN_BF16; p.mbf = mod_dtype == DMF_ATTN_BF16;
  p.hbf = h_dtype == DMF_ATTN_BF16; p.zbf = z_dtype == DMF_ATTN_BF16;
  const unsigned grid = static_cast<unsigned>((p.rows + kWaves - 1) / kWaves);
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dispatch_nv(C, [&](auto nv) {
    constexpr int NV = decltype(nv)::value;
    if (jvp) return launch_kernel(residual_ln_modulate_fwd_kernel<NV, true>, dim3(grid), dim3(kThreads), 0, s, p);
    return launch_kernel(residual_ln_modulate_fwd_kernel<NV, false>, dim3(grid), dim3(kThreads), 0, s, p);
  });
}

int dmf_gelu_tanh_fwd(const void* x, const void* tx, void* y, void* ty, int64_t n, int dtype, void* stream) {
  if (ty && !tx) return DMF_ATTN_ENULL;
  return act_impl<kActGelu>(x, tx, y, ty, n, dtype, dtype, ty ? 1 : 0, stream);
}

int dmf_gelu_tanh_bwd(const void* gy, const void* x, void* gx, int64_t n, int dtype, void* stream) {
  return act_impl<kActGelu>(x, gy, nullptr, gx, n, dtype, dtype, 2, stream);
}

int dmf_silu_fwd(const void* x, const void* tx, void* y, void* ty, int64_t n, int x_dtype, int y_dtype,
                 void* stream) {
  if (ty && !tx) return DMF_ATTN_ENULL;
  return act_impl<kActSilu>(x, tx, y, ty, n, x_dtype, y_dtype, ty ? 1 : 0, stream);
}

int dmf_silu_bwd(const void* gy, const void* x, void* gx, int64_t n, int x_dtype, int gy_dtype, void* stream) {
  return act_impl<kActSilu>(x, gy, nullptr, gx, n, x_dtype, gy_dtype, 2, stream);
}

int dmf_colsum(const void* x, void* out, float* workspace, int64_t rows, int C, int x_dtype, int out_dtype,
               void* stream) {
  if (!dtype_ok(x_dtype) || !dtype_ok(out_dtype)) return DMF_ATTN_EDTYPE;
  if (rows < 1 || C < 8 || C % 8) return DMF_ATTN_ESHAPE;
  const int64_t nchunk = (rows + kColsumRows - 1) / kColsumRows;
  if (nchunk > 0x7fffffffLL || C > 8 * 64 * 65535) return DMF_ATTN_ESHAPE;
  if (!x || !out || !workspace) return DMF_ATTN_ENULL;
  if (!aligned16(x) || !aligned16(out) || !aligned16(workspace)) return DMF_ATTN_EALIGN;
  ColsumParams p{};
  p.x = x; p.partial = workspace; p.rows = rows; p.C = C; p.xbf = x_dtype == DMF_ATTN_BF16;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(nchunk), static_cast<unsigned>((C / 8 + 63) / 64));
  if (int rc = launch_kernel(colsum_kernel, grid, dim3(kThreads), 0, s, p)) return rc;
  return reduce_partials(workspace, out, nullptr, 1, static_cast<int>(nchunk), 1, C, out_dtype == DMF_ATTN_BF16, s);
}

// ---- dmf_colsum for callers that cannot allocate: the partial sums live in library-owned device memory -------------
//
// `colsum_scratch` is the name of a per-device symbol, not a device address: host code may only use the address that
// hipGetSymbolAddress returns for the current device (each GPU holds its own copy of the array at its own address).
constexpr int64_t kColsumStaticFloats = DMF_COLSUM_STATIC_MAX_FLOATS;
static __device__ __align__(256) float colsum_scratch[kColsumStaticFloats];

// Address of this device's copy of the array, looked up once per device (a race between two host threads at worst
// repeats the idempotent lookup).  Returns nullptr if the runtime cannot resolve the symbol.
static float* colsum_scratch_on_current_device() {
  static float* addr[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  if (addr[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(colsum_scratch)) != hipSuccess) return nullptr;
    addr[dev] = static_cast<float*>(p);
  }
  return addr[dev];
}

int dmf_colsum_static(const void* x, void* out, int64_t rows, int C, int x_dtype, int out_dtype, void* stream) {
  // size check first, so that an oversized request is refused whatever else is wrong with it
  if (rows < 1 || C < 8 || C % 8) return DMF_ATTN_ESHAPE;
  const int64_t nchunk = (rows + kColsumRows - 1) / kColsumRows;
  if (nchunk > kColsumStaticFloats / C) return DMF_ATTN_ESCRATCH;
  float* ws = colsum_scratch_on_current_device();
  if (ws == nullptr) return DMF_ATTN_ELAUNCH;
  // Stage one overwrites every partial sum that stage two reads, so nothing has to be cleared between calls.
  return dmf_colsum(x, out, ws, rows, C, x_dtype, out_dtype, stream);
}

// Validates a strided (B, L, H, D) operand and copies {sB, sL, sH}.
static int check_blhd(const void* ptr, const int64_t* st4, int eb, int64_t (&st3)[3]) {
  if (!aligned16(ptr)) return DMF_ATTN_EALIGN;
  if (st4[3] != 1) return DMF_ATTN_ESTRIDE;
  for (int i = 0; i < 3; ++i) {
    if (st4[i] < 0 || (st4[i] * eb) % 16) return DMF_ATTN_ESTRIDE;
    st3[i] = st4[i];
  }
  return DMF_ATTN_OK;
}

static int check_rms(int B, int L, int H, int D, int dtype, int gain_dtype) {
  if (!dtype_ok(dtype) || !dtype_ok(gain_dtype)) return DMF_ATTN_EDTYPE;
  if (D < 8 || D % 8 || D > 128) return DMF_ATTN_EHEADDIM;
  if (B < 1 || L < 1 || H < 1) return DMF_ATTN_ESHAPE;
  if (static_cast<int64_t>(B) * L * H / (kThreads / 16) + 1 > 0x7fffffffLL) return DMF_ATTN_ESHAPE;
  return DMF_ATTN_OK;
}

int dmf_rmsnorm_fwd(const void* x, const void* tx, const void* gain, void* y, void* ty, const int64_t* strides, int B,
                    int L, int H, int D, float eps, int dtype, int gain_dtype, void* stream) {
  if (int rc = check_rms(B, L, H, D, dtype, gain_dtype)) return rc;
  if (!x || !gain || !y || !strides) return DMF_ATTN_ENULL;
  if (!aligned16(gain) || !aligned16(y) || !aligned16(ty)) return DMF_ATTN_EALIGN;
  RmsParams p{};
  if (int rc = check_blhd(x, strides, ebytes(dtype), p.sx)) return rc;
  if (tx)
    if (int rc = check_blhd(tx, strides + 4, ebytes(dtype), p.stx)) return rc;
  p.x = x; p.tx = tx; p.gain = gain; p.y = y; p.ty = ty;
  p.rows = static_cast<int64_t>(B) * L * H;
  p.L = L; p.H = H; p.D = D; p.eps = eps;
  p.bf = dtype == DMF_ATTN_BF16; p.gbf = gain_dtype == DMF_ATTN_BF16;
  const unsigned grid = static_cast<unsigned>((p.rows + kThreads / 16 - 1) / (kThreads / 16));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (ty) return launch_kernel(rmsnorm_fwd_kernel<true>, dim3(grid), dim3(kThreads), 0, s, p);
  return launch_kernel(rmsnorm_fwd_kernel<false>, dim3(grid), dim3(kThreads), 0, s, p);
}

int dmf_rmsnorm_bwd(const void* gy, const void* x, const void* gain, void* gx, void* ggain, float* workspace,
                    const int64_t* strides, int B, int L, int H, int D, float eps, int dtype, int gain_dtype,
                    void* stream) {
  if (int rc = check_rms(B, L, H, D, dtype, gain_dtype)) return rc;
  if (!gy || !x || !gain || !gx || !ggain || !workspace || !strides) return DMF_ATTN_ENULL;
  if (!aligned16(gy) || !aligned16(gain) || !aligned16(ggain) || !aligned16(workspace)) return DMF_ATTN_EALIGN;
  RmsParams p{};
  if (int rc = check_blhd(x, strides, ebytes(dtype), p.sx)) return rc;
  if (int rc = check_blhd(gx, strides + 4, ebytes(dtype), p.stx)) return rc;
  p.x = x; p.gy = gy; p.gain = gain; p.y = gx; p.partial = workspace;
  p.rows = static_cast<int64_t>(B) * L * H;
  p.L = L; p.H = H; p.D = D; p.eps = eps;
  p.bf = dtype == DMF_ATTN_BF16; p.gbf = gain_dtype == DMF_ATTN_BF16;
  const int64_t want = (p.rows + kThreads / 16 - 1) / (kThreads / 16);
  const int nblocks = static_cast<int>(std::min<int64_t>(want, kRmsBlocksMax));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (int rc = launch_kernel(rmsnorm_bwd_kernel, dim3(nblocks), dim3(kThreads), 0, s, p)) return rc;
  return reduce_partials(workspace, ggain, nullptr, 1, nblocks, 1, D, p.gbf, s);
}

}  // extern "C"
