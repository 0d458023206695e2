// Shared definitions of the gfx950 kernels: element types, 16-byte fragments,
// MFMA wrappers for bfloat16 and true float32, wave reductions.
//
// Everything here is written for CDNA4 (gfx950): 64-lane waves, MFMA matrix
// cores. There is no other target.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define TW_DTYPE_F32 0
#define TW_DTYPE_BF16 1

#define TW_ERR_BAD_ARGUMENT 10001   // a launcher refused its arguments (shape, alignment, size)
#define TW_ERR_TOO_LARGE 10002      // an input exceeds the fixed capacity of an entry point that brings its own scratch memory

typedef __bf16 bf16_t;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define TW_WAVE 64

// ---- scalar conversions ---------------------------------------------------
__device__ __forceinline__ float tw_to_float(float v) { return v; }
__device__ __forceinline__ float tw_to_float(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T tw_from_float(float v);
template <> __device__ __forceinline__ float tw_from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t tw_from_float<bf16_t>(float v) { return (bf16_t)v; }  // round to nearest even

// ---- element type traits ----------------------------------------------------
// A "fragment" is 16 bytes per lane: 8 bfloat16 or 4 float32 consecutive along
// the reduction dimension. One fragment pair feeds one bf16 MFMA or four fp32
// MFMAs, so kernels are written once over fragments.
template <typename T> struct Elem;

template <> struct Elem<float> {
  typedef f32x4 Frag;
  static constexpr int kPerFrag = 4;       // elements in 16 bytes
  static constexpr int kId = TW_DTYPE_F32;
  __device__ static __forceinline__ Frag zero() { return Frag{0.f, 0.f, 0.f, 0.f}; }
};

template <> struct Elem<bf16_t> {
  typedef bf16x8 Frag;
  static constexpr int kPerFrag = 8;
  static constexpr int kId = TW_DTYPE_BF16;
  __device__ static __forceinline__ Frag zero() {
    u32x4 z = {0u, 0u, 0u, 0u};
    return __builtin_bit_cast(Frag, z);
  }
};

template <typename T>
__device__ __forceinline__ typename Elem<T>::Frag tw_load_frag(const T* p) {
  return *reinterpret_cast<const typename Elem<T>::Frag*>(p);
}

// For data that a kernel reads once (weights of a decode step, the cache in decode attention): the
// caches are told not to keep it.
template <typename T>
__device__ __forceinline__ typename Elem<T>::Frag tw_load_frag_stream(const T* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const typename Elem<T>::Frag*>(p));
}

// ---- LDS: which lanes a 16-byte read serves together ------------------------------------
// A wave's 16-byte LDS read is served in four passes of 16 lanes, 256 bytes (all 64 banks) a pass, and the
// lanes of a pass are not neighbours: {0-3, 12-15, 20-23, 24-27}, {4-11, 16-19, 28-31}, and the same + 32
// (found with a probe that lets two lanes meet in one bank and reads SQ_LDS_BANK_CONFLICT; 16-byte writes
// go 8 neighbouring lanes a pass). For the 16x16 MFMA's fragments (lane = 16 * piece + row) a pass
// therefore holds all 16 rows, eight of them with piece p and the other eight (rows 4-11, or the rest)
// with piece p + 1. Two layouts put those 16 lanes in 16 different 16-byte columns:
//   rows whose length is 32 bytes more than a multiple of 256 (32 * an odd number), pieces in order;
//   rows of 64 bytes (four pieces) with piece p of row r at p ^ tw_lds_swz4(r).
// (Rows longer by 16 bytes, or p ^ (r / 4 % 4), look right for 16 neighbouring lanes and meet a 2-way
// conflict in every read.)
__device__ __host__ __forceinline__ constexpr int tw_lds_swz4(int row) {
  return (0x78 >> ((row >> 1) & 6)) & 3;                     // 0, 2, 3, 1 for row / 4 % 4 = 0, 1, 2, 3
}

// ---- MFMA: 16x16 tiles --------------------------------------------------------
// Lane l = 16*g + r (g = l / 16, r = l % 16).
//   A operand: row r of the 16-row tile, the fragment chosen by g.
//   B operand: column r of the 16-column tile, the fragment chosen by g.
//   accumulator: 4 floats, element j is D[4*g + j][r].
// Summation over the reduction index is complete once every (g, element) pair
// of A has met the same pair of B; which actual k a pair stands for is free as
// long as A and B agree, so callers lay k out for contiguous memory access.
__device__ __forceinline__ void tw_mma16(f32x4& acc, bf16x8 a, bf16x8 b) {
  acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
}
__device__ __forceinline__ void tw_mma16(f32x4& acc, f32x4 a, f32x4 b) {
  acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[0], b[0], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[1], b[1], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[2], b[2], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[3], b[3], acc, 0, 0, 0);
}

// 16x16 tile with 4 reduction elements per lane (the k index of element j in
// lane group g is 4*g + j): used where the B operand is an accumulator.
__device__ __forceinline__ void tw_mma16_k4(f32x4& acc, bf16x4 a, f32x4 b) {
  bf16x4 bb = {(bf16_t)b[0], (bf16_t)b[1], (bf16_t)b[2], (bf16_t)b[3]};
  acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a),
                                                  __builtin_bit_cast(s16x4, bb), acc, 0, 0, 0);
}
__device__ __forceinline__ void tw_mma16_k4(f32x4& acc, f32x4 a, f32x4 b) {
  acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[0], b[0], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[1], b[1], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[2], b[2], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[3], b[3], acc, 0, 0, 0);
}

// ---- MFMA: 32x32 tiles --------------------------------------------------------
// Lane l = 32*g + r (g = l / 32, r = l % 32).
//   A operand: row r, fragment chosen by g; B operand: column r, fragment by g.
//   accumulator: 16 floats, element j is D[8*(j/4) + 4*g + (j%4)][r].
__device__ __forceinline__ void tw_mma32(f32x16& acc, bf16x8 a, bf16x8 b) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
}
__device__ __forceinline__ void tw_mma32(f32x16& acc, f32x4 a, f32x4 b) {
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b[0], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[1], b[1], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[2], b[2], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[3], b[3], acc, 0, 0, 0);
}

// ---- reductions ------------------------------------------------------------------
__device__ __forceinline__ float tw_wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, TW_WAVE);
  return v;
}
__device__ __forceinline__ float tw_wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, TW_WAVE));
  return v;
}

// A value combined over lanes l, l ^ 16, l ^ 32, l ^ 48 (the four 16-lane rows of a wave) with gfx950's
// lane-swap instructions: two vector instructions per step instead of a round trip through the LDS
// crossbar (ds_bpermute), which sat in the dependent chain of every softmax block.
__device__ __forceinline__ float tw_rows_max(float x) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float tw_rows_sum(float x) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Sum over a block of up to 1024 threads; every thread gets the result. The
// order of additions is fixed by the block size alone.
__device__ __forceinline__ float tw_block_sum(float v, float* lds /* >= 16 floats */) {
  v = tw_wave_sum(v);
  const int wave = threadIdx.x / TW_WAVE, lane = threadIdx.x % TW_WAVE;
  const int waves = (blockDim.x + TW_WAVE - 1) / TW_WAVE;
  __syncthreads();
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += lds[w];
  return total;
}

static inline int tw_div_up(long a, long b) { return (int)((a + b - 1) / b); }

#define TW_REQUIRE(cond)                      \
  do {                                        \
    if (!(cond)) return TW_ERR_BAD_ARGUMENT;  \
  } while (0)

#define TW_LAUNCH_RESULT() ((int)hipGetLastError())
