// The few-rows product with SwiGLU in its epilogue: the entry points whose kernels apply the
// activation (the kernel is in gemm_skinny_kernel.h).
#include "gemm_skinny_kernel.h"

// The grouped product with SwiGLU applied in its epilogue: W [groups, N, K] holds gate rows
// [0, N/2) and up rows [N/2, N) of every expert; out [M, N/2] bf16 =
// act(s g) * (s u) with g, u the two products rounded to bfloat16, s = act_scale[row] (null: 1) and
// act the activation's code (common.h).
// Rows are the expert-sorted list (row_blocks * 16 of an expert at a time).  R in {2, 4}, NW in {4, 8};
// packed as above (N % 32 == 0 then).
SHARPI_EXPORT int sharpi_gemm_skinny_swiglu(const void* x, const void* W, void* out, int M, int N, int K,
                                            const int* a_rows, const int* group_offsets, int groups,
                                            const float* act_scale, int R, int NW, int packed, int row_blocks,
                                            int act, hipStream_t stream) {
  if (M <= 0) return SHARPI_OK;
  if (N <= 0 || (N & 7) || K <= 0 || (K & 127) || groups <= 0 || groups > 65535 || !act_known(act)) return SHARPI_ERR_ARG;
  if (group_offsets == nullptr) return SHARPI_ERR_ARG;
  if (packed && (N & 31)) return SHARPI_ERR_ARG;
  const int MB = row_blocks > 0 ? row_blocks : 1;
#define SKA1(RR, WW, MBV, PK) \
  return launch_skinny<RR, MBV, WW, true, PK>(x, W, out, DT_BF16, M, N, K, a_rows, group_offsets, groups, act_scale, stream, Picks{}, act)
#define SKA(RR, WW)                                    \
  if (R == RR && NW == WW) {                           \
    if (MB == 1) { if (packed) SKA1(RR, WW, 1, true); else SKA1(RR, WW, 1, false); }  \
    if (MB == 2) { if (packed) SKA1(RR, WW, 2, true); else SKA1(RR, WW, 2, false); }  \
    if (MB == 4) { if (packed) SKA1(RR, WW, 4, true); else SKA1(RR, WW, 4, false); }  \
    return SHARPI_ERR_ARG;                             \
  }
  SKA(2, 4); SKA(2, 8);
  SKA(4, 4); SKA(4, 8);
#undef SKA
#undef SKA1
  return SHARPI_ERR_ARG;
}

// The picked form's SwiGLU half (see sharpi_gemm_skinny_picked): the arguments are checked there.
int skinny_picked_swiglu(const void* x, const void* W, void* out, int M, int N, int K, const Picks& pk, int groups, int R,
                         int NW, int packed, int act, hipStream_t stream) {
  const int MB = pk.n_pairs <= 16 ? 1 : pk.n_pairs <= 32 ? 2 : 4;
#define SKP1(RR, WW, MBV, PK) \
  return launch_skinny<RR, MBV, WW, true, PK>(x, W, out, DT_BF16, M, N, K, nullptr, pk.ids, groups, nullptr, stream, pk, act)
#define SKP(RR, WW)                                                      \
  if (R == RR && NW == WW) {                                             \
    if (MB == 1) { if (packed) SKP1(RR, WW, 1, true); else SKP1(RR, WW, 1, false); } \
    if (MB == 2) { if (packed) SKP1(RR, WW, 2, true); else SKP1(RR, WW, 2, false); } \
    if (packed) SKP1(RR, WW, 4, true); else SKP1(RR, WW, 4, false);       \
  }
  SKP(2, 4); SKP(2, 8);
  SKP(4, 4); SKP(4, 8);
#undef SKP
#undef SKP1
  return SHARPI_ERR_ARG;
}
