// Measurement aids for bench.py (not part of the attention library or its ABI; built into libbench_probes.so).
//
// dmf_probe_mfma_tflops: sustained rate of v_mfma_f32_32x32x16_bf16 on this
// device from a register-only loop, with constant or with random operand bits.
// With random operands the device runs into its power limit and clocks down,
// which bounds what any bf16 MFMA kernel working on real data can reach.
//
// dmf_probe_rows_stream_tbps: what the memory system delivers for the access
// pattern of the attention operator without any math -- per (batch, head) read
// six and write two tensors of N rows of D bf16 values, rows strided by H*D as
// in a (B, N, H, D) tensor (or contiguous per head).  This is the practical
// HBM ceiling for short sequences, where the operator is bandwidth-bound.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

namespace {

__global__ __launch_bounds__(256) void mfma_loop(float* out, int iters, int random_operands) {
  u32x4 a[4], b[4];
  uint32_t s = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
  for (int j = 0; j < 4; ++j)
    for (int e = 0; e < 4; ++e) {
      // random sign and mantissa, exponent fixed so that values stay in [0.5, 1)
      s = s * 1664525u + 1013904223u;
      a[j][e] = random_operands ? ((s & 0x807f807fu) | 0x3f003f00u) : 0x3f803f80u;
      s = s * 1664525u + 1013904223u;
      b[j][e] = random_operands ? ((s & 0x807f807fu) | 0x3f003f00u) : 0x3f803f80u;
    }
  f32x16 acc[4];
  for (int i = 0; i < 4; ++i) acc[i] = f32x16{0};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[i]), __builtin_bit_cast(bf16x8, b[(i + it) & 3]),
                                                       acc[i], 0, 0, 0);
  }
  float r = 0;
  for (int i = 0; i < 4; ++i)
    for (int e = 0; e < 16; ++e) r += acc[i][e];
  out[blockIdx.x * 256 + threadIdx.x] = r;
}

typedef __attribute__((ext_vector_type(4))) uint32_t vec16;
// One work-group per (batch, head); consecutive heads of a batch element are placed on one XCD (the hardware deals
// work-group ids round robin over the 8 XCDs), so that the cache lines two adjacent 144-byte head rows share are
// fetched into one L2 -- without that the strided pattern streams at 3.7-3.9 TB/s instead of 4.6 -- and every thread
// keeps four rows' worth of loads in flight.
constexpr int kStreamUnroll = 4;
__global__ __launch_bounds__(256) void rows_stream(const vec16* __restrict__ a0, const vec16* __restrict__ a1, const vec16* __restrict__ a2,
                                                   const vec16* __restrict__ a3, const vec16* __restrict__ a4, const vec16* __restrict__ a5,
                                                   vec16* __restrict__ o0, vec16* __restrict__ o1, int H, int N, int vpr, int head_contiguous) {
  const uint32_t total_wgs = gridDim.x;
  const int bh = total_wgs % 8 == 0 ? (blockIdx.x % 8) * (total_wgs / 8) + blockIdx.x / 8 : blockIdx.x;
  const int b = bh / H, h = bh % H, total = N * vpr;
  for (int v0 = threadIdx.x; v0 < total; v0 += 256 * kStreamUnroll) {
    vec16 x[kStreamUnroll][6];
    size_t idx[kStreamUnroll];
#pragma unroll
    for (int u = 0; u < kStreamUnroll; ++u) {
      const int v = v0 + u * 256, n = v / vpr, cv = v % vpr;
      idx[u] = head_contiguous ? (((size_t)b * H + h) * N + n) * vpr + cv : (((size_t)b * N + n) * H + h) * vpr + cv;
      if (v < total) {
        x[u][0] = a0[idx[u]]; x[u][1] = a1[idx[u]]; x[u][2] = a2[idx[u]];
        x[u][3] = a3[idx[u]]; x[u][4] = a4[idx[u]]; x[u][5] = a5[idx[u]];
      }
    }
#pragma unroll
    for (int u = 0; u < kStreamUnroll; ++u)
      if (v0 + u * 256 < total) {
        o0[idx[u]] = x[u][0] ^ x[u][1] ^ x[u][2];
        o1[idx[u]] = x[u][3] ^ x[u][4] ^ x[u][5];
      }
  }
}

}  // namespace

// Returns TB/s moved (8 tensors of B*N*H*D bf16 values per launch), or a negative value on error.  D % 8 == 0.
extern "C" __attribute__((visibility("default"))) float dmf_probe_rows_stream_tbps(int B, int H, int N, int D, int head_contiguous) {
  const int vpr = D / 8;
  const size_t bytes = (size_t)B * N * H * D * 2;
  vec16* buf[8] = {};
  bool ok = true;
  for (int i = 0; i < 8 && ok; ++i) ok = hipMalloc(&buf[i], bytes) == hipSuccess && hipMemset(buf[i], i + 1, bytes) == hipSuccess;
  float ms = 0.f;
  if (ok) {
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    auto launch = [&] {
      hipLaunchKernelGGL(rows_stream, dim3(B * H), dim3(256), 0, 0, buf[0], buf[1], buf[2], buf[3], buf[4], buf[5], buf[6], buf[7], H, N, vpr,
                         head_contiguous);
    };
    for (int i = 0; i < 10; ++i) launch();
    (void)hipEventRecord(e0, 0);
    for (int i = 0; i < 50; ++i) launch();
    (void)hipEventRecord(e1, 0);
    ok = hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
  }
  for (int i = 0; i < 8; ++i)
    if (buf[i]) (void)hipFree(buf[i]);
  if (!ok || ms <= 0.f) return -1.f;
  return (float)(8.0 * bytes * 50 / (ms * 1e-3) / 1e12);
}

// Returns TFLOP/s (dense bf16 MFMA, 2 waves per SIMD), or a negative value on a HIP error.
extern "C" __attribute__((visibility("default"))) float dmf_probe_mfma_tflops(int random_operands, int iters) {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
    return -1.f;
  const int wgs = 2 * cus;   // 4 waves per work-group -> 2 waves per SIMD
  float* out = nullptr;
  if (hipMalloc(&out, (size_t)wgs * 256 * sizeof(float)) != hipSuccess) return -1.f;
  hipEvent_t e0, e1;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  hipLaunchKernelGGL(mfma_loop, dim3(wgs), dim3(256), 0, 0, out, iters, random_operands);   // warm-up, same length: lets clocks settle
  (void)hipEventRecord(e0, 0);
  hipLaunchKernelGGL(mfma_loop, dim3(wgs), dim3(256), 0, 0, out, iters, random_operands);
  (void)hipEventRecord(e1, 0);
  float ms = 0.f;
  const bool ok = hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipFree(out);
  if (!ok || ms <= 0.f) return -1.f;
  const double flops = (double)wgs * 4 /*waves*/ * iters * 4 /*mfma*/ * 32768.0;
  return (float)(flops / (ms * 1e-3) / 1e12);
}
