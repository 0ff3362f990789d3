// Shared device primitives for the gfx950 (MI355X) attention kernels.
//
// Register/lane conventions used everywhere (wave64, MFMA 32x32 tiles):
//   lane = threadIdx.x & 63,  c32 = lane & 31,  g = lane >> 5.
//   A 32x32 fp32 accumulator tile `acc[16]` of a lane holds
//       row(i) = (i/4)*8 + 4*g + (i%4),   col = c32.
//   An MFMA operand "chunk" is one 16-byte vector per lane:
//     bf16: 8 elements = contraction slots of ONE v_mfma_f32_32x32x16_bf16,
//     fp32: 4 elements = the operand of FOUR v_mfma_f32_32x32x2_f32.
//   Both operands of a product always use the same slot->index mapping, so
//   any consistent permutation of the contraction index is legal; the kernels
//   exploit that to feed accumulator tiles straight back in as operands.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <utility>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

namespace dmf {

// Compile-time unrolled loop: f(std::integral_constant<int, 0>{}) ... f(<N-1>).
template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Exchange between lane and lane^32 (the two halves of a 32x32 tile column).
__device__ __forceinline__ float xhalf_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xhalf_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// v + (v rotated right by N lanes within each row of 16 lanes), as one DPP-modified add
template <int N>
__device__ __forceinline__ float row_ror_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x120 + N, 0xf, 0xf, false));
}

// sum over the 16 lanes of an aligned lane group; every lane of the group gets the same bits
__device__ __forceinline__ float group16_sum(float v) {
  v = row_ror_add<8>(v);
  v = row_ror_add<4>(v);
  v = row_ror_add<2>(v);
  return row_ror_add<1>(v);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  f32x2 x = {a, b};
  bf16x2 y = __builtin_convertvector(x, bf16x2);  // v_cvt_pk_bf16_f32, round-to-nearest-even
  return __builtin_bit_cast(uint32_t, y);
}

// x as the sum of three bf16 numbers h + m + l (relative error 2^-24), packed into the first three elements of an
// eight-element bf16 vector; the other five are zero.
__device__ __forceinline__ u32x4 split3_bf16(float x) {
  const uint32_t h = pack_bf16x2(x, 0.f);
  const float r1 = x - __uint_as_float(h << 16);
  const uint32_t m = pack_bf16x2(r1, 0.f);
  const float r2 = r1 - __uint_as_float(m << 16);
  return u32x4{h | (m << 16), pack_bf16x2(r2, 0.f), 0u, 0u};
}

// Static configuration for element type T (float or __bf16) and head dim D.
template <typename T, int D>
struct Cfg {
  static_assert(D % 8 == 0 && D >= 16 && D <= 128, "head dim must be a multiple of 8 in [16,128]");
  static constexpr bool BF = sizeof(T) == 2;
  static constexpr int VEC = 16 / (int)sizeof(T);              // elements per 16-byte vector
  static constexpr int VPR = D / VEC;                          // valid vectors per row
  static constexpr int NCHUNK = BF ? (D + 15) / 16 : D / 8;    // operand chunks over the head dim
  static constexpr int NDT = (D + 31) / 32;                    // 32-wide output tiles over the head dim
  static constexpr int ROWV0 = (2 * NCHUNK > VPR ? 2 * NCHUNK : VPR);
  static constexpr int ROWV = ROWV0 + 1 + (ROWV0 & 1);         // LDS row pitch in vectors, odd => conflict-free b128 reads
  static constexpr int STRIDE = ROWV * VEC;                    // LDS row pitch in elements
  static constexpr int OROWV = NDT * 32 / VEC + 1;             // epilogue staging pitch (vectors, odd)
  static constexpr int OSTRIDE = OROWV * VEC;
  static constexpr int NSUB = BF ? 2 : 1;                      // 32-row sub-tiles per KV tile
  static constexpr int BKV = 32 * NSUB;
  static constexpr int TILE_BYTES = BKV * ROWV * 16;
  static constexpr int PV_STEPS = BF ? 2 : 16;                 // operand steps per 32-row sub-tile in P*V-like products
};

// acc += A_chunk * B_chunk  (one 16-byte operand chunk per lane each).
template <typename T>
__device__ __forceinline__ void mma_chunk(f32x16& acc, const u32x4& a, const u32x4& b) {
  if constexpr (sizeof(T) == 2) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[e]), __uint_as_float(b[e]), acc, 0, 0, 0);
  }
}

// Operand chunk c of row `row` of a row-major LDS tile (contraction along the row).
template <typename T, int STRIDE>
__device__ __forceinline__ u32x4 lds_row_chunk(const T* tile, int row, int c, int g) {
  return *reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(tile) + (size_t)row * STRIDE * sizeof(T) + (2 * c + g) * 16);
}

// "Column" operand for products that contract over the ROWS of a row-major LDS
// tile (P*V-like): the lane's M index is column col0 + c32 and the contraction
// slots follow the accumulator row order of the lane (see header comment), so
// an accumulator tile converted with acc_operand() is the matching B operand.
//   bf16: step s in {0,1} covers rows r0+16s .. r0+16s+15 (two ds_read_b64_tr_b16).
//   fp32: step s in 0..15 covers row r0 + (s/4)*8 + 4g + s%4.
struct ColOperand { u32x4 v; };

template <typename T, int STRIDE>
__device__ __forceinline__ ColOperand lds_col_operand(const T* tile, int r0, int col0, int s, int lane) {
  ColOperand r;
  if constexpr (sizeof(T) == 2) {
    const int g = lane >> 5, i = lane & 15, half = (lane >> 4) & 1;
    // 16 lanes cooperatively fetch a 4(row) x 16(col) block; lane i supplies row i/4, cols 4*(i%4)..+3
    const T* p = tile + (r0 + 16 * s + 4 * g + (i >> 2)) * STRIDE + col0 + 16 * half + 4 * (i & 3);
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(s16x4, p + 8 * STRIDE));
    u32x2 a = __builtin_bit_cast(u32x2, lo), b = __builtin_bit_cast(u32x2, hi);
    r.v = u32x4{a[0], a[1], b[0], b[1]};
  } else {
    const int g = lane >> 5, c32 = lane & 31;
    const int row = r0 + (s >> 2) * 8 + 4 * g + (s & 3);
    r.v = u32x4{__float_as_uint(tile[row * STRIDE + col0 + c32]), 0u, 0u, 0u};
  }
  return r;
}

// bf16 column operands issued as raw instructions that the compiler does not
// model as LDS accesses.  Rationale: in front of the ds_read_b64_tr_b16
// *intrinsic* the compiler places a full `s_waitcnt vmcnt(0)` whenever an
// HBM->LDS DMA load is in flight, which would serialise the tile prefetch with
// the math.  lds_tr16_issue() starts the two transposed reads of one operand
// (rows r..r+3 at byte offset OFF_LO, rows r+8..r+11 at OFF_HI, relative to the
// lane address described at lds_col_operand); lds_tr16_wait() must be applied
// to the results before they are used.  LDS operations complete in order, so
// these untracked reads only ever make the compiler's own lgkmcnt waits more
// conservative.
struct TrPair { u32x2 lo, hi; };

template <int OFF_LO, int OFF_HI>
__device__ __forceinline__ TrPair lds_tr16_issue(uint32_t lane_addr) {
  TrPair r;
  asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
               : "=&v"(r.lo), "=&v"(r.hi)
               : "v"(lane_addr), "n"(OFF_LO), "n"(OFF_HI));
  return r;
}
// Wait until at most N LDS instructions issued after these operands are still
// outstanding (N = number of reads issued since, for software pipelining).
template <int N>
__device__ __forceinline__ void lds_tr16_wait(TrPair& a) {
  asm volatile("s_waitcnt lgkmcnt(%[n])" : "+v"(a.lo), "+v"(a.hi) : [n] "n"(N));
}
template <int N>
__device__ __forceinline__ void lds_tr16_wait(TrPair& a, TrPair& b) {
  asm volatile("s_waitcnt lgkmcnt(%[n])" : "+v"(a.lo), "+v"(a.hi), "+v"(b.lo), "+v"(b.hi) : [n] "n"(N));
}
// Row-operand chunk (16 bytes per lane) issued the same untracked way.
template <int OFF>
__device__ __forceinline__ u32x4 lds_read128_issue(uint32_t lane_addr) {
  u32x4 r;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(lane_addr), "n"(OFF));
  return r;
}
template <int N>
__device__ __forceinline__ void lds_read128_wait(u32x4& a) {
  asm volatile("s_waitcnt lgkmcnt(%[n])" : "+v"(a) : [n] "n"(N));
}
template <int N>
__device__ __forceinline__ void lds_read128_wait(u32x4& a, u32x4& b) {
  asm volatile("s_waitcnt lgkmcnt(%[n])" : "+v"(a), "+v"(b) : [n] "n"(N));
}
template <int N>
__device__ __forceinline__ void lds_read128_wait(u32x4& a, u32x4& b, u32x4& c, u32x4& d) {
  asm volatile("s_waitcnt lgkmcnt(%[n])" : "+v"(a), "+v"(b), "+v"(c), "+v"(d) : [n] "n"(N));
}
__device__ __forceinline__ ColOperand tr_operand(const TrPair& a) {
  ColOperand r;
  r.v = u32x4{a.lo[0], a.lo[1], a.hi[0], a.hi[1]};
  return r;
}
// 16x16x32 bf16 MFMA on the same operand containers (A/B: lane = index % 16,
// contraction slots 8*(lane/16)..+7; C: column = lane % 16, rows 4*(lane/16)..+3).
__device__ __forceinline__ void mma16(f32x4& acc, const ColOperand& a, const ColOperand& b) {
  acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a.v), __builtin_bit_cast(bf16x8, b.v), acc, 0, 0, 0);
}
// v_permlane16_swap: returns {x.row0, y.row0, x.row2, y.row2} and {x.row1, y.row1, x.row3, y.row3}
// (rows = groups of 16 lanes).
__device__ __forceinline__ void swap16(uint32_t x, uint32_t y, uint32_t& even, uint32_t& odd) {
  auto r = __builtin_amdgcn_permlane16_swap(x, y, false, false);
  even = r[0];
  odd = r[1];
}
__device__ __forceinline__ void swap16f(float x, float& even, float& odd) {
  uint32_t a, b;
  swap16(__float_as_uint(x), __float_as_uint(x), a, b);
  even = __uint_as_float(a);
  odd = __uint_as_float(b);
}

// Byte address in LDS of a pointer into the work-group's shared memory.
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
  return (uint32_t)(uintptr_t)LDS_PTR(const char, p);
}

// Matching B operand built from a lane's accumulator tile (already converted to
// the probabilities / weights to be contracted).
template <typename T>
__device__ __forceinline__ ColOperand acc_operand(const f32x16& e, int s) {
  ColOperand r;
  if constexpr (sizeof(T) == 2) {
    r.v = u32x4{pack_bf16x2(e[8 * s + 0], e[8 * s + 1]), pack_bf16x2(e[8 * s + 2], e[8 * s + 3]),
                pack_bf16x2(e[8 * s + 4], e[8 * s + 5]), pack_bf16x2(e[8 * s + 6], e[8 * s + 7])};
  } else {
    r.v = u32x4{__float_as_uint(e[s]), 0u, 0u, 0u};
  }
  return r;
}

template <typename T>
__device__ __forceinline__ void mma_col(f32x16& acc, const ColOperand& a, const ColOperand& b) {
  if constexpr (sizeof(T) == 2) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a.v), __builtin_bit_cast(bf16x8, b.v), acc, 0, 0, 0);
  } else {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.v[0]), __uint_as_float(b.v[0]), acc, 0, 0, 0);
  }
}

// Row index inside a 32-row tile held by accumulator element i of a lane in half g.
__device__ __forceinline__ int acc_row(int i, int g) { return (i >> 2) * 8 + 4 * g + (i & 3); }

// XCD-aware work-group remap: hardware deals consecutive work-group ids round
// robin over the 8 XCDs (each with a private L2).  Give every XCD a contiguous
// range of logical ids so the q-blocks that share one head's K/V hit one L2.
__device__ __forceinline__ uint32_t xcd_remap(uint32_t id, uint32_t total) {
  constexpr uint32_t kXcd = 8;
  if (total % kXcd) return id;
  return (id % kXcd) * (total / kXcd) + id / kXcd;
}

// Work-group barrier that orders LDS traffic only.  __syncthreads() also makes
// prior *global* stores visible, i.e. waits until they are acknowledged -- which
// stalls an epilogue for microseconds when output rows have just been stored.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Convert four consecutive fp32 values to T and store them to LDS.
template <typename T>
__device__ __forceinline__ void store4(T* dst, float a, float b, float c, float d) {
  if constexpr (sizeof(T) == 2) {
    *reinterpret_cast<u32x2*>(dst) = u32x2{pack_bf16x2(a, b), pack_bf16x2(c, d)};
  } else {
    *reinterpret_cast<f32x4*>(dst) = f32x4{a, b, c, d};
  }
}

// Cooperative HBM -> register -> LDS streaming of NT row-major tiles of ROWS
// rows x D elements by a 256-thread work-group.  issue() starts the global
// loads (rows at or past `nrows` read as zero), commit() writes them to LDS.
template <typename T, int D, int ROWS, int NT>
struct TileStream {
  using C = Cfg<T, D>;
  static constexpr int TILE_VECS = ROWS * C::VPR;
  static constexpr int ITERS = (TILE_VECS + 255) / 256;
  u32x4 pre[NT][ITERS];

  __device__ __forceinline__ void issue(const T* const (&src)[NT], const int64_t (&row_stride)[NT], int row0, int nrows, int tid) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int v = tid + it * 256;
        const int row = v / C::VPR, cv = v % C::VPR;
        const bool ok = (v < TILE_VECS) && (row0 + row < nrows);
        pre[t][it] = ok ? *reinterpret_cast<const u32x4*>(src[t] + (int64_t)(row0 + row) * row_stride[t] + cv * C::VEC)
                        : u32x4{0, 0, 0, 0};
      }
    }
  }
  __device__ __forceinline__ void commit(T* const (&dst)[NT], int tid) const {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int v = tid + it * 256;
        const int row = v / C::VPR, cv = v % C::VPR;
        if (v < TILE_VECS) *reinterpret_cast<u32x4*>(dst[t] + row * C::STRIDE + cv * C::VEC) = pre[t][it];
      }
    }
  }
};

// Zero the contraction padding (vectors VPR .. 2*NCHUNK-1 of every row) of an
// LDS tile; tile commits never touch those columns afterwards.
template <typename T, int D, int ROWS>
__device__ __forceinline__ void zero_tile_padding(T* tile, int tid) {
  using C = Cfg<T, D>;
  if constexpr (2 * C::NCHUNK > C::VPR) {
    constexpr int PADV = 2 * C::NCHUNK - C::VPR;
    for (int i = tid; i < ROWS * PADV; i += 256) {
      const int row = i / PADV, cv = C::VPR + i % PADV;
      *reinterpret_cast<u32x4*>(tile + row * C::STRIDE + cv * C::VEC) = u32x4{0, 0, 0, 0};
    }
  }
}

// Epilogue helper: a work-group's NDT transposed accumulator tiles (lane = output
// row wave*32+c32, in-lane = head-dim index) are scaled, transposed through the
// LDS staging area and stored with coalesced 16-byte rows.  Must be called by
// all 64*NW threads of the work-group (NW waves, 32 rows each); `stage` may alias the tile buffers (the leading barrier
// protects them).
//
// NMAIN (default: all NDT tiles) limits `value` to the first NMAIN 32-wide tiles;
// `tail(wave_stage)` may then write the remaining columns itself (wave_stage =
// staging row 0 of this wave, row pitch Cfg::OSTRIDE).
struct NoTail { __device__ __forceinline__ void operator()(void*) const {} };

// Part 1: write the scaled accumulators into the staging rows of this wave (no barrier, no global traffic).
template <typename T, int D, int NMAIN = Cfg<T, D>::NDT, typename F, typename TF = NoTail>
__device__ __forceinline__ void stage_rows(T* stage, int tid, F value, TF tail = TF{}) {
  using C = Cfg<T, D>;
  const int lane = tid & 63, wave = tid >> 6, c32 = lane & 31, g = lane >> 5;
  T* srow = stage + (wave * 32 + c32) * C::OSTRIDE;
#pragma unroll
  for (int t = 0; t < NMAIN; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      store4<T>(srow + t * 32 + j * 8 + 4 * g, value(t, 4 * j), value(t, 4 * j + 1), value(t, 4 * j + 2), value(t, 4 * j + 3));
  tail(stage + wave * 32 * C::OSTRIDE);
}
// Part 2: "round" r of the coalesced copy staging -> global: every thread moves one 16-byte vector.
// Rounds 0 .. store_rounds()-1 cover the 32*NW staged rows.
template <typename T, int D, int NW>
__device__ __forceinline__ constexpr int store_rounds() { return (32 * NW * Cfg<T, D>::VPR + 64 * NW - 1) / (64 * NW); }

template <typename T, int D, int NW>
__device__ __forceinline__ void store_staged_round(const T* stage, T* gdst, int64_t row_stride, int row0, int nrows, int tid, int r) {
  using C = Cfg<T, D>;
  const int v = tid + r * 64 * NW;
  const int row = v / C::VPR, cv = v % C::VPR;
  if (v < 32 * NW * C::VPR && row0 + row < nrows)
    *reinterpret_cast<u32x4*>(gdst + (int64_t)(row0 + row) * row_stride + cv * C::VEC) =
        *reinterpret_cast<const u32x4*>(stage + row * C::OSTRIDE + cv * C::VEC);
}

template <typename T, int D, int NW = 4, int NMAIN = Cfg<T, D>::NDT, typename F, typename TF = NoTail>
__device__ __forceinline__ void store_rows_transposed(T* stage, T* gdst, int64_t row_stride, int row0, int nrows, int tid, F value,
                                                      TF tail = TF{}) {
  lds_barrier();
  stage_rows<T, D, NMAIN>(stage, tid, value, tail);
  lds_barrier();
  for (int r = 0; r < store_rounds<T, D, NW>(); ++r) store_staged_round<T, D, NW>(stage, gdst, row_stride, row0, nrows, tid, r);
}

// Issue the HBM -> LDS loads of one tensor tile (32 rows): wave w of the NW waves
// moves rows (32/NW)*w .. (32/NW)*(w+1)-1.  LDS placement is lane-linear (base + lane*16), which with a
// row-major padded tile means slot = row*PITCH + vector; lanes that fall on
// padding vectors are switched off.  The source is a raw buffer resource that
// covers exactly the Lkv rows of this (batch, head): `soffset` selects the
// tile, and rows past the end read as zeros (hardware bounds check).
template <int PITCH, int VPR, int NW = 4>
__device__ __forceinline__ void issue_tile_rows(__amdgpu_buffer_rsrc_t rsrc, uint32_t row_bytes, uint32_t soffset,
                                                char* lds_tile, int wave, int lane) {
  constexpr int RPW = 32 / NW;          // rows per wave
  constexpr int SLOTS = RPW * PITCH;
#pragma unroll
  for (int i = 0; i < (SLOTS + 63) / 64; ++i) {
    const int slot = 64 * i + lane;
    const int r = slot / PITCH, cv = slot % PITCH;
    if (slot < SLOTS && cv < VPR) {
      const uint32_t voff = (uint32_t)(RPW * wave + r) * row_bytes + cv * 16;
      char* dst = lds_tile + (RPW * wave * PITCH + 64 * i) * 16;   // wave-uniform
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dst, 16, voff, soffset, 0, 0);
    }
  }
}

// HBM -> LDS loads of ROWS whole rows by ONE wave: LDS placement is lane-linear (row pitch PITCH vectors, VPR of them
// valid), lanes that fall on padding vectors are switched off; rows past the end of the resource read as zeros.
template <int PITCH, int VPR, int ROWS>
__device__ __forceinline__ void issue_rows(__amdgpu_buffer_rsrc_t rsrc, uint32_t row_bytes, uint32_t soffset, char* lds_dst, int lane) {
  constexpr int SLOTS = ROWS * PITCH;
#pragma unroll
  for (int i = 0; i < (SLOTS + 63) / 64; ++i) {
    const int slot = 64 * i + lane;
    const int r = slot / PITCH, cv = slot % PITCH;
    if (slot < SLOTS && cv < VPR)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(lds_dst + 64 * i * 16), 16,
                                               (uint32_t)r * row_bytes + cv * 16, soffset, 0, 0);
  }
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rows_rsrc(const void* base, uint32_t row_bytes, int nrows, int row_payload_bytes) {
  // raw buffer, byte-granular bounds: [base, base + (nrows-1)*row_bytes + payload)
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (nrows - 1) * row_bytes + row_payload_bytes, 0x00020000);
}

// The same descriptor as four plain words, for raw buffer instructions in inline assembly ("s" operand).
__device__ __forceinline__ u32x4 rows_rsrc_words(const void* base, uint32_t row_bytes, int nrows, int row_payload_bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(base);
  return u32x4{(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, (uint32_t)((nrows - 1) * row_bytes + row_payload_bytes), 0x00020000u};
}

// Epilogue of the 16-wide remainder tiles (head dims 72, 80): lane (i = lane % 16,
// w = lane / 16) holds head-dim columns 32*NMT + 4w .. +3 of row i (tile 0) and of
// row 16 + i (tile 1) of this wave's 32 rows; value(hq, e) supplies the numbers.
// `ws` = staging row 0 of this wave (see store_rows_transposed).
template <typename T, int D, int NMT, typename VF>
__device__ __forceinline__ void store_tail16(void* ws, int lane, VF value) {
  constexpr int OSTR = Cfg<T, D>::OSTRIDE, TAILW = D - 32 * NMT;
  const int w16 = lane >> 4, i16 = lane & 15;
  if (4 * w16 < TAILW) {
#pragma unroll
    for (int hq = 0; hq < 2; ++hq)
      store4<T>(static_cast<T*>(ws) + (16 * hq + i16) * OSTR + 32 * NMT + 4 * w16, value(hq, 0), value(hq, 1), value(hq, 2), value(hq, 3));
  }
}

// Both B operands (query/key halves 0 and 1) of the 16x16x32 remainder products
// from the two 32x32x16-layout operands of a 32-row tile (steps 0 and 1).
__device__ __forceinline__ void tail_operands(const ColOperand& st0, const ColOperand& st1, ColOperand& half0, ColOperand& half1) {
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    uint32_t ev, od;
    swap16(st0.v[r], st1.v[r], ev, od);
    half0.v[r] = ev;
    half1.v[r] = od;
  }
}

// Lane offset (in elements) for the transposed remainder operand inside a
// row-major 32-row tile of pitch STR: 16-lane row w covers tile rows
// 16*(w%2) + 4*(w/2) + {0..3, 8..11} at columns col0 .. col0+15.
__device__ __forceinline__ int tail_lane_offset(int lane, int STR, int col0) {
  return (16 * ((lane >> 4) & 1) + 4 * (lane >> 5) + ((lane & 15) >> 2)) * STR + col0 + 4 * (lane & 3);
}

// All NCHUNK 16-byte operand chunks of one row (this lane's row, half g) with
// bounds-checked buffer loads issued back to back: rows past the end of the
// resource read as zeros, chunk vectors past the head dim are zeroed here.
template <int NCHUNK, int VPR>
__device__ __forceinline__ void load_row_chunks(__amdgpu_buffer_rsrc_t rsrc, uint32_t row_bytes, int row, int g, u32x4 (&out)[NCHUNK]) {
  // A chunk vector past the head dim gets an out-of-range offset, so the bounds check zero-fills it too and the
  // loaded registers need no fix-up (a fix-up would make the caller wait for the data right here).
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const uint32_t off = (2 * c + g < VPR) ? (uint32_t)row * row_bytes + (2 * c + g) * 16 : 0x7ffffff0u;
    out[c] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0));
  }
}

}  // namespace dmf
