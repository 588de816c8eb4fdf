// The few-rows product's entry points without an activation (the kernel is in gemm_skinny_kernel.h;
// the SwiGLU form is compiled in a file of its own, so that the two halves build side by side).
#include "gemm_skinny_kernel.h"

// defined beside the SwiGLU form's kernels
int skinny_picked_swiglu(const void* x, const void* W, void* out, int M, int N, int K, const Picks& pk, int groups, int R,
                         int NW, int packed, int act, hipStream_t stream);

template <int R, int NW, bool PACKED>
static int dispatch_mb(int MB, const void* x, const void* W, void* out, int out_dtype, int M, int N, int K,
                       const int* a_rows, const int* group_offsets, int groups, hipStream_t stream) {
  if (MB == 1) return launch_skinny<R, 1, NW, false, PACKED>(x, W, out, out_dtype, M, N, K, a_rows, group_offsets, groups, nullptr, stream);
  if (MB == 2) return launch_skinny<R, 2, NW, false, PACKED>(x, W, out, out_dtype, M, N, K, a_rows, group_offsets, groups, nullptr, stream);
  return launch_skinny<R, 4, NW, false, PACKED>(x, W, out, out_dtype, M, N, K, a_rows, group_offsets, groups, nullptr, stream);
}

// x [M, K] bf16 (rows gathered through a_rows if given), W [N, K] or [groups, N, K] bf16,
// out [M, N] (out_dtype float or bf16).  groups == 0: plain.  groups > 0: rows are the
// expert-sorted list, group_offsets [groups + 1].  R in {1, 2, 4}: 16-row weight tiles per block;
// NW in {4, 8, 16}: waves per block splitting K (16 only with R = 1: a block of 1,024 threads has
// 128 registers a lane, which wider tiles do not fit).  packed: W is stored tile by tile,
// [N/16][K/128][16 runs of 8 k][16 rows][8] (N % 16 == 0), instead of row by row.
SHARPI_EXPORT int sharpi_gemm_skinny(const void* x, const void* W, void* out, int out_dtype, int M, int N, int K,
                                     const int* a_rows, const int* group_offsets, int groups, int R, int NW,
                                     int packed, int row_blocks, hipStream_t stream) {
  if (M <= 0) return SHARPI_OK;
  if (N <= 0 || (N & 3) || K <= 0 || (K & 127) || groups < 0 || groups > 65535) return SHARPI_ERR_ARG;
  if (groups == 0 && M > 64) return SHARPI_ERR_ARG;
  if (groups > 0 && group_offsets == nullptr) return SHARPI_ERR_ARG;
  if (out_dtype != DT_F32 && out_dtype != DT_BF16) return SHARPI_ERR_ARG;
  if (packed && (N & 15)) return SHARPI_ERR_ARG;
  // plain: all row blocks at once.  Grouped: row_blocks (1, 2 or 4) blocks of 16 rows of an expert at
  // a time; an expert with more rows is walked in turns, reading its weights again for each
  const int MB = groups > 0 ? (row_blocks > 0 ? row_blocks : 1) : ceil_div(M, 16);
  if (MB < 1 || MB > 4) return SHARPI_ERR_ARG;
#define SK(RR, WW)                                                                                                        \
  if (R == RR && NW == WW)                                                                                                \
  return packed ? dispatch_mb<RR, WW, true>(MB, x, W, out, out_dtype, M, N, K, a_rows, group_offsets, groups, stream)     \
                : dispatch_mb<RR, WW, false>(MB, x, W, out, out_dtype, M, N, K, a_rows, group_offsets, groups, stream)
  SK(1, 4); SK(1, 8); SK(1, 16);
  SK(2, 4); SK(2, 8);
  SK(4, 4); SK(4, 8);
#undef SK
  return SHARPI_ERR_ARG;
}

// The picked form: per-expert products of a few decode tokens straight from the router's picks.
// ids [n_pairs] (pair i = token i / k, pick i % k), W [n_experts (+ 1 if shared), N, K]; out row i is
// pair i, rows n_pairs .. n_pairs + n_pairs / k - 1 are the tokens through expert n_experts (shared != 0).
// gather: x [tokens, K] is read by token; otherwise x rows are in the output's order.  With act != 0
// (an activation's code, common.h) W holds gate then up rows and out [rows, N/2] bf16 =
// act(s g) * (s u), s = w[i] for pair i (w may be null: no scaling) and 1 for the shared rows.  n_pairs and the tokens fit one wave's ballot (<= 64).
SHARPI_EXPORT int sharpi_gemm_skinny_picked(const void* x, const void* W, void* out, int out_dtype, int N, int K,
                                            const int* ids, const float* w, int n_pairs, int k, int n_experts,
                                            int shared, int gather, int act, int R, int NW, int packed,
                                            hipStream_t stream) {
  if (n_pairs <= 0) return SHARPI_OK;
  if (ids == nullptr || k <= 0 || n_pairs % k != 0 || n_pairs > kMaxPicked || n_experts <= 0) return SHARPI_ERR_ARG;
  if (N <= 0 || (N & (act ? 7 : 3)) || K <= 0 || (K & 127)) return SHARPI_ERR_ARG;
  if (packed && (N & (act ? 31 : 15))) return SHARPI_ERR_ARG;
  if (out_dtype != DT_F32 && out_dtype != DT_BF16) return SHARPI_ERR_ARG;
  if (act && (out_dtype != DT_BF16 || !act_known(act))) return SHARPI_ERR_ARG;
  // a group for every expert that can have rows: no more distinct experts than pairs
  const int groups = (n_experts < n_pairs ? n_experts : n_pairs) + (shared ? 1 : 0);
  if (groups > 65535) return SHARPI_ERR_ARG;
  const int M = n_pairs + (shared ? n_pairs / k : 0);
  const Picks pk = {ids, w, n_pairs, k, n_experts, gather, shared ? 1 : 0};
  if (act) return skinny_picked_swiglu(x, W, out, M, N, K, pk, groups, R, NW, packed, act, stream);
  // an expert has at most n_pairs rows: one, two or four blocks of sixteen rows against one stream of its weights
  const int MB = n_pairs <= 16 ? 1 : n_pairs <= 32 ? 2 : 4;
  // group_offsets is not read in this form; the pointer only has to be non-null for the grid's sake
#define SKP1(RR, WW, ACTV, MBV, PK) \
  return launch_skinny<RR, MBV, WW, ACTV, PK>(x, W, out, out_dtype, M, N, K, nullptr, ids, groups, nullptr, stream, pk)
#define SKP(RR, WW, ACTV)                                                      \
  if (R == RR && NW == WW && !ACTV) {                             \
    if (MB == 1) { if (packed) SKP1(RR, WW, ACTV, 1, true); else SKP1(RR, WW, ACTV, 1, false); } \
    if (MB == 2) { if (packed) SKP1(RR, WW, ACTV, 2, true); else SKP1(RR, WW, ACTV, 2, false); } \
    if (packed) SKP1(RR, WW, ACTV, 4, true); else SKP1(RR, WW, ACTV, 4, false); \
  }
  SKP(1, 4, false); SKP(1, 8, false); SKP(1, 16, false);
  SKP(2, 4, false); SKP(2, 8, false);
  SKP(4, 4, false); SKP(4, 8, false);
#undef SKP1
#undef SKP
  return SHARPI_ERR_ARG;
}

SHARPI_EXPORT int sharpi_gemm_skinny_max_picked() { return kMaxPicked; }
