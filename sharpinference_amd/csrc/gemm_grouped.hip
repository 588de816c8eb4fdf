// The grouped product for many rows, plain form (gemm_grouped_kernel.h holds the kernel; the gated
// form is compiled in a file of its own so that the two build side by side).
#include "gemm_grouped_kernel.h"

// x [x_rows, K] bf16 (rows gathered through a_rows if given), W [>= n_groups, N, K] bf16, out
// [n_rows, N]; group_offsets [n_groups + 1] and plan (grouped_plan.h) from the routing kernel.
// packed: W is stored tile by tile, [E][N/16][K/128][16 runs of 8 k][16 rows][8] (N % 16 == 0,
// K % 128 == 0).  max_blocks > 0 bounds the blocks launched (they stay until the work is done).
// The plan's ticket counters are used and set back by the launch: two products that read one plan
// must not run at the same time.
SHARPI_EXPORT int sharpi_gemm_grouped(const void* x, int x_rows, const void* W, void* out, int out_dtype, int n_rows,
                                      int N, int K, const int* a_rows, const int* group_offsets, const int* plan,
                                      int n_groups, int packed, int max_blocks, hipStream_t stream) {
  if (n_rows <= 0) return SHARPI_OK;
  if (!grouped_args_ok(x_rows, n_rows, N, K, n_groups, packed, group_offsets, plan)) return SHARPI_ERR_ARG;
  const int nb = ceil_div(N, columns_of(kMaxNT));
  const dim3 grid = grouped_grid(n_rows, n_groups, nb, max_blocks), block(GW * kWave);
#define GG_LAUNCH(TOV, PK)                                                                                             \
  grouped_gemm_kernel<TOV, kMaxNT, PK, false><<<grid, block, 0, stream>>>((const bf16_t*)x, (const bf16_t*)W, (TOV*)out, \
                                                                         N, K, a_rows, nullptr, 0, group_offsets, plan, \
                                                                         n_groups, nb)
  if (out_dtype == DT_BF16) {
    if (packed) GG_LAUNCH(bf16_t, true); else GG_LAUNCH(bf16_t, false);
  } else if (out_dtype == DT_F32) {
    if (packed) GG_LAUNCH(float, true); else GG_LAUNCH(float, false);
  } else {
    return SHARPI_ERR_ARG;
  }
#undef GG_LAUNCH
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

SHARPI_EXPORT int sharpi_gemm_grouped_tile_rows() { return GM; }
