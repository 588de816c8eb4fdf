// C[M, N] = A[M, K] * W[N, K]^T with float FMA arithmetic (no matrix-core, no reduced precision).
//
// The 32-bit path's matrix product, also the fallback for sizes the MFMA kernels refuse.
// Every output element is one chain of fused multiply-adds over k = 0..K-1 in ascending order,
// so a row's result does not depend on how many other rows are in the batch or where the row
// sits in it.  The grouped form runs E products at once: rows [off[e], off[e+1]) of the
// (expert-sorted) row list use W[e]; A's rows may be gathered through `a_rows`.
#include "common.h"

constexpr int BM = 64, BN = 64, BK = 16;

template <typename T, typename TO>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const T* __restrict__ A, const T* __restrict__ W,
                                                         TO* __restrict__ C, int M, int N, int K,
                                                         const int* __restrict__ a_rows,
                                                         const int* __restrict__ group_offsets) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  int row_begin = 0, row_end = M;
  if (group_offsets) {
    const int e = blockIdx.z;
    row_begin = group_offsets[e];
    row_end = group_offsets[e + 1];
    W += (size_t)e * N * K;
  }
  const int m0 = row_begin + blockIdx.y * BM;
  if (m0 >= row_end) return;
  const int n0 = blockIdx.x * BN;
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  // loader role: row lr of the tile, 4 consecutive k starting at lk
  const int lr = tid >> 2, lk = (tid & 3) * 4;
  const int am = m0 + lr;
  const T* a_src = nullptr;
  if (am < row_end) a_src = A + (size_t)(a_rows ? a_rows[am] : am) * K;
  const int wn = n0 + lr;
  const T* w_src = wn < N ? W + (size_t)wn * K : nullptr;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + lk + j;
      As[lk + j][lr] = (a_src && k < K) ? to_f32<T>(a_src[k]) : 0.f;
      Ws[lk + j][lr] = (w_src && k < K) ? to_f32<T>(w_src[k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= row_end) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) C[(size_t)m * N + n] = from_f32<TO>(acc[i][j]);
    }
  }
}

// dtype: storage of A and W; out_dtype: storage of C.
// groups == 0: plain product of M rows. groups > 0: grouped, M = total rows (upper bound of any group).
SHARPI_EXPORT int sharpi_gemm_tiled(const void* A, const void* W, void* C, int dtype, int out_dtype, int M, int N,
                                    int K, const int* a_rows, const int* group_offsets, int groups,
                                    hipStream_t stream) {
  if (M <= 0) return SHARPI_OK;
  if (N <= 0 || K <= 0 || groups < 0 || groups > 65535) return SHARPI_ERR_ARG;
  if (groups > 0 && group_offsets == nullptr) return SHARPI_ERR_ARG;
  if (ceil_div(M, BM) > 65535) return SHARPI_ERR_ARG;
  dim3 grid(ceil_div(N, BN), ceil_div(M, BM), groups > 0 ? groups : 1), block(256);
  const int* go = groups > 0 ? group_offsets : nullptr;
  if (dtype == DT_F32 && out_dtype == DT_F32)
    gemm_tiled_kernel<float, float><<<grid, block, 0, stream>>>((const float*)A, (const float*)W, (float*)C, M, N,
                                                               K, a_rows, go);
  else if (dtype == DT_BF16 && out_dtype == DT_BF16)
    gemm_tiled_kernel<bf16_t, bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, (bf16_t*)C,
                                                                 M, N, K, a_rows, go);
  else if (dtype == DT_BF16 && out_dtype == DT_F32)
    gemm_tiled_kernel<bf16_t, float><<<grid, block, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, (float*)C, M,
                                                                N, K, a_rows, go);
  else
    return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
