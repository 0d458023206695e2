// Shared by the two linear-layer sources: gemm.hip (few rows, any K, the C entry points) and
// gemm_tiled.hip (many rows), which are compiled apart because they want different register
// allocation for their MFMA accumulators.
#pragma once
#include "tw_common.h"

__device__ __forceinline__ float tw_silu(float g) { return g / (1.0f + expf(-g)); }

// Sum of split-K partial sums partial[split][M][N], in split order, then bias and residual.
template <typename OutT>
__global__ void splitk_reduce_kernel(const float* __restrict__ partial, int splits,
                                     const float* __restrict__ bias, const float* residual, long ldr,
                                     OutT* C, long ldc, int M, int N) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)M * N) return;
  const int row = (int)(i / N), col = (int)(i % N);
  float v = 0.f;
  for (int s = 0; s < splits; ++s) v += partial[(size_t)s * M * N + i];
  if (bias) v += bias[col];
  if (residual) v += residual[(size_t)row * ldr + col];
  C[(size_t)row * ldc + col] = tw_from_float<OutT>(v);
}

// The tiled kernels (gemm_tiled.hip). shape: 0 = choose, 1 = tiles of 128x128, 2 = 128x256,
// 3 = 256x256 (bfloat16 with shuffled weights only). Returns 0 or an error code.
int tw_tiled_linear(int dtype, int out_f32, int shuffled, int glu, int shape, const void* A, long lda,
                    const void* W, long ldw, const float* bias, const float* residual, long ldr, void* C,
                    long ldc, float* partial, long partial_bytes, int M, int N, int K, hipStream_t stream);
// Bytes of split-K scratch the tiled kernels can use for `rows` rows of an [N, K] weight (0: none).
long tw_tiled_workspace_bytes(int dtype, int rows, int N, int K);
