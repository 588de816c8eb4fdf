// The grouped product for many rows with the gated unit in its epilogue (gemm_grouped_kernel.h holds
// the kernel).
#include "gemm_grouped_kernel.h"

// The grouped product with the gated unit in its epilogue: W [>= n_groups, N, K] holds gate rows
// [0, N/2) then up rows of every group; out [n_rows, N/2] bf16 = act(s g) * (s u) with g, u the two
// products rounded to bfloat16, s = act_scale[row] (null: 1) and act the activation's code
// (common.h).  N % 32 == 0; the rest as above.
SHARPI_EXPORT int sharpi_gemm_grouped_swiglu(const void* x, int x_rows, const void* W, void* out, int n_rows, int N,
                                             int K, const int* a_rows, const int* group_offsets, const int* plan,
                                             int n_groups, const float* act_scale, int packed, int act,
                                             int max_blocks, hipStream_t stream) {
  if (n_rows <= 0) return SHARPI_OK;
  if (!act_known(act)) return SHARPI_ERR_ARG;
  if ((N & 31) || !grouped_args_ok(x_rows, n_rows, N, K, n_groups, packed, group_offsets, plan)) return SHARPI_ERR_ARG;
  constexpr int GN = columns_of(kMaxNT);   // the gated form pairs gate tiles with up tiles
  const int nb = ceil_div(N / 2, GN / 2);
  const dim3 grid = grouped_grid(n_rows, n_groups, nb, max_blocks), block(GW * kWave);
  if (packed)
    grouped_gemm_kernel<bf16_t, kMaxNT, true, true><<<grid, block, 0, stream>>>(
        (const bf16_t*)x, (const bf16_t*)W, (bf16_t*)out, N, K, a_rows, act_scale, act, group_offsets, plan, n_groups, nb);
  else
    grouped_gemm_kernel<bf16_t, kMaxNT, false, true><<<grid, block, 0, stream>>>(
        (const bf16_t*)x, (const bf16_t*)W, (bf16_t*)out, N, K, a_rows, act_scale, act, group_offsets, plan, n_groups, nb);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

