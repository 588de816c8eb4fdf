// Weight-streaming matrix product for few rows (decode): out[M, N] = x[M, K] * W[N, K]^T, bfloat16
// inputs, float accumulation on the matrix cores (v_mfma_f32_16x16x32_bf16); M <= 64, or any number
// of rows in the grouped form as long as an expert has few.
//
// The weights are read from HBM exactly once; everything else is arranged around that.  They are
// read with the streaming hint (nontemporal: a line is not kept in the caches for a second use
// that never comes), which alone is worth a tenth of the bandwidth: 6.3 against 5.7 TB/s for a
// pure read in this kernel's access pattern.
//  * A block owns R tiles of 16 weight rows; its NW waves split K into contiguous slices.  Per
//    128-wide K unit a lane loads 64 contiguous bytes of each of its weight rows and of each of
//    its x rows and feeds 4 MFMAs per (tile, row block): W is the A operand (rows = n), x the
//    B operand.  Both operands take element (group g, index i) of a lane from the same k, so
//    the order of k inside a unit is free: lanes read 64-byte runs, not 16-byte ones.
//  * The waves' partial sums meet in LDS and are added in wave order.  R and NW are chosen from
//    the weight's shape alone and the x rows never mix, so a row's result does not depend on
//    the batch around it.
//  * Grouped form (routed experts): block (tile, expert e) handles rows
//    [offsets[e], offsets[e + 1]) of the expert-sorted row list with W[e], MB blocks of sixteen at
//    a time (an expert with more is walked in turns and its weights read again for each); x rows
//    are gathered through a_rows.  Experts without rows return at once.
//
//  * Picked form (a few decode tokens): instead of a sorted row list the kernel is given the
//    router's picks themselves.  Row i of the output is pair i = (token i / k, its pick i % k), in
//    that order, followed by one row per token for an always-on expert that shares the tensor; a
//    block finds the rows of its expert with one ballot over the picks.  No kernel has to sort
//    the pairs first, and the x rows wait for one index load instead of two.
//
//  * Packed weights (PACKED): the matrix is stored tile by tile instead of row by row, the 4 KB
//    of a (16-row tile, 128-wide K unit) contiguous and in the order the lanes want them, and
//    the K units are dealt to the waves in turn: a block's reads are contiguous runs of NW * 4 KB
//    rather than 256-byte pieces a row apart, worth about a tenth of the bandwidth.
//  * Gated form (ACT): W holds gate rows [0, N/2) and up rows [N/2, N); a block takes R/2 tiles
//    of each at the same columns, and the wave that adds up a gate tile adds up its up tile too,
//    rounds both to bfloat16 (what a separate activation kernel would have read) and stores
//    act(s g) * (s u), s the row's score and act the activation the caller names (SiLU, GELU):
//    out is [M, N/2] and the gate|up rows never go to memory.
//
// Limits (the caller falls back to other kernels otherwise): K % 128 == 0, N % 4 == 0, M <= 64 (plain form).
#pragma once
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

template <typename TO> __device__ __forceinline__ void store4(TO* p, f32x4 v);
template <> __device__ __forceinline__ void store4<float>(float* p, f32x4 v) {
  *reinterpret_cast<f32x4*>(p) = v;
}
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, f32x4 v) {
  uint2 packed;
  packed.x = (uint32_t)f32_to_bf16(v[0]).bits | ((uint32_t)f32_to_bf16(v[1]).bits << 16);
  packed.y = (uint32_t)f32_to_bf16(v[2]).bits | ((uint32_t)f32_to_bf16(v[3]).bits << 16);
  *reinterpret_cast<uint2*>(p) = packed;
}

constexpr int kRedTiles = 2;  // (tile, row block) pairs summed per LDS round
constexpr int kMaxPicked = 64;  // pairs (and tokens) of the picked form: one ballot of a wave

// The picked form's arguments (ids null: the other forms).
struct Picks {
  const int* ids;      // [n_pairs] expert of pair i
  const float* w;      // [n_pairs] its score (the SwiGLU form scales by it), or null
  int n_pairs, k, n_experts;
  int gather;          // x rows are tokens (pair i reads row i / k); otherwise x is in the output's row order
  int shared;          // the tensor holds one more expert (index n_experts) that every token goes through
};

// Forms whose registers hold two K units at once (the loop then requests a unit ahead).
template <int R, int MB> constexpr bool kSkinnyPipelined = MB == 1 && R <= 2;

template <int R, int MB, int NW, typename TO, bool ACT, bool PACKED>
__global__ __launch_bounds__(NW* kWave) void skinny_gemm_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ W, TO* __restrict__ out, int M, int N, int K,
    const int* __restrict__ a_rows, const int* __restrict__ group_offsets, const float* __restrict__ act_scale,
    int act, Picks pk) {
  static_assert(!ACT || R % 2 == 0, "the SwiGLU form pairs gate and up tiles");
  constexpr int RT = ACT ? R : kRedTiles;   // tiles that meet in LDS per round
  constexpr int TG = ACT ? R / 2 : R;       // tiles of distinct output columns per block
  __shared__ f32x4 red[NW][RT][kWave];
  __shared__ int members[kMaxPicked];       // picked form: the output rows of this block's expert
  __shared__ int n_members;
  __shared__ int block_expert;
  const int lane = threadIdx.x & (kWave - 1);
  const int w = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int nb = blockIdx.x;
  const int e = blockIdx.y;
  const bool picked = pk.ids != nullptr;
  int row_begin = 0, row_end = M;
  if (picked) {
    // The grid has a group for every expert that CAN have rows, not for every expert there is
    // (a block that finds no rows still costs a launch slot, and with one token fifteen of
    // seventeen would): the first group is the always-on expert, if there is one; group y after it
    // is the y-th DISTINCT expert among the picks, in the order of its first pick.  The groups
    // that find no expert (fewer distinct experts than pairs) are then the grid's last blocks,
    // where they hold nobody up.
    if (w == 0) {
      const int n_groups = gridDim.y;
      const bool always_on = pk.shared && blockIdx.y == 0;
      const int ordinal_wanted = (int)blockIdx.y - pk.shared;
      const int mine_e = lane < pk.n_pairs ? pk.ids[lane] : -1;
      int expert = -1;                            // the block's expert; -1: there are fewer distinct experts than groups
      if (always_on) {
        expert = pk.n_experts;
      } else if (n_groups - pk.shared == pk.n_experts) {
        expert = ordinal_wanted;                  // as many groups as experts: group y is expert y
      } else {
        bool first = lane < pk.n_pairs;           // no earlier pair picked this lane's expert
        for (int j = 0; j < pk.n_pairs; ++j) {
          const int ej = __shfl(mine_e, j, kWave);
          if (j < lane && ej == mine_e) first = false;
        }
        const unsigned long long firsts = __builtin_amdgcn_ballot_w64(first);
        const int ordinal = __popcll(firsts & ((1ull << lane) - 1ull));
        const unsigned long long chosen = __builtin_amdgcn_ballot_w64(first && ordinal == ordinal_wanted);
        if (chosen) expert = __shfl(mine_e, __ffsll((long long)chosen) - 1, kWave);
      }
      const bool routed = !always_on;
      const bool mine = expert < 0 ? false : routed ? (lane < pk.n_pairs && mine_e == expert) : lane < pk.n_pairs / pk.k;
      const unsigned long long mask = __builtin_amdgcn_ballot_w64(mine);
      if (mine) members[__popcll(mask & ((1ull << lane) - 1ull))] = routed ? lane : pk.n_pairs + lane;
      if (lane == 0) {
        n_members = __popcll(mask);
        block_expert = expert;
      }
    }
    __syncthreads();
    row_end = n_members;
    if (row_end <= 0) return;
    W += (size_t)block_expert * N * K;
  } else if (group_offsets) {
    row_begin = group_offsets[e];
    row_end = group_offsets[e + 1];
    W += (size_t)e * N * K;
  }
  const int n_rows = row_end - row_begin;
  if (n_rows <= 0) return;
  // where row m of the block's list reads x, and where it is stored
  auto out_row = [&](int m) { return picked ? members[m] : m; };
  auto x_row = [&](int m) {
    if (!picked) return a_rows ? a_rows[m] : m;
    const int i = members[m];
    return pk.gather ? (i < pk.n_pairs ? i / pk.k : i - pk.n_pairs) : i;
  };
  const int n_base = nb * 16 * TG;
  const int n_out = ACT ? N / 2 : N;        // output columns

  // this wave's K units
  const int U = K >> 7;
  const int u_begin = (U * w) / NW;
  const int u_end = (U * (w + 1)) / NW;

  // Row layout: lane (row r, group g) reads the 64-byte run k0 + g*32 .. + 32 of its row, 16 bytes
  // per MFMA step j.  Packed layout: the 4 KB of a (16-row tile, 128-wide unit) are contiguous
  // in the order [j][g][r][8 elements], so step j of a wave is one contiguous 1 KB read and the
  // lane's 8 elements are k0 + (4j + g)*8 .. + 8 of row r; x is read at the same k.
  const bf16_t* wrow[R];
#pragma unroll
  for (int t = 0; t < R; ++t) {
    if constexpr (PACKED) {
      int tile = (n_base >> 4) + (t % TG);
      if (tile * 16 >= n_out) tile = (n_out >> 4) - 1;   // loaded, never stored
      if (ACT && t >= TG) tile += n_out >> 4;            // the up tile of the same columns
      wrow[t] = W + (size_t)tile * 16 * K + lane * 8;
    } else {
      int n = n_base + (t % TG) * 16 + r;
      if (n >= n_out) n = n_out - 1;  // loaded, never stored
      if (ACT && t >= TG) n += n_out;  // the up row of the same column
      wrow[t] = W + (size_t)n * K + g * 32;
    }
  }
  constexpr int XG = PACKED ? 8 : 32;    // x: a lane's first k within a unit is g * XG, step j adds XJ
  constexpr int XJ = PACKED ? 32 : 8;

  // this wave's K units: first, first + step, ... (count of them).  Row layout: a wave takes a
  // contiguous slice of K.  Packed layout: units are dealt to the waves in turn, so that the
  // block reads NW * 4 KB of a tile side by side at every step.
  const int u_first = PACKED ? w : u_begin;
  const int u_step = PACKED ? NW : 1;
  const int u_count = PACKED ? (w < U ? (U - w + NW - 1) / NW : 0) : u_end - u_begin;

  for (int rb0 = 0; rb0 * 16 < n_rows; rb0 += MB) {
    // Rows beyond the group's last read its last row again: what they give is never stored (a
    // column of the product depends on its own x row only), and no load sits behind a branch.
    const bf16_t* xrow[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = min(row_begin + (rb0 + mb) * 16 + r, row_end - 1);
      xrow[mb] = x + (size_t)x_row(m) * K + g * XG;
    }
    f32x4 acc[R][MB];
#pragma unroll
    for (int t = 0; t < R; ++t)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[t][mb] = f32x4{0.f, 0.f, 0.f, 0.f};

    struct Unit {
      bf16x8 wf[R][4], xf[MB][4];
    };
    auto load_unit = [&](int u, Unit& un) {
      const int k0 = u << 7;
#pragma unroll
      for (int t = 0; t < R; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          un.wf[t][j] = __builtin_nontemporal_load(
              reinterpret_cast<const bf16x8*>(wrow[t] + (PACKED ? (size_t)u * 2048 + j * 512 : (size_t)k0 + j * 8)));
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        if (mb > 0 && (rb0 + mb) * 16 >= n_rows) continue;   // a row block beyond the group's rows (block-uniform)
#pragma unroll
        for (int j = 0; j < 4; ++j) un.xf[mb][j] = *reinterpret_cast<const bf16x8*>(xrow[mb] + k0 + j * XJ);
      }
    };
    auto use_unit = [&](const Unit& un) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        // a row block beyond the group's rows is not multiplied (the same for every lane of the block)
        if (mb > 0 && (rb0 + mb) * 16 >= n_rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int t = 0; t < R; ++t)
            acc[t][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(un.wf[t][j], un.xf[mb][j], acc[t][mb], 0, 0, 0);
      }
    };
    if constexpr (kSkinnyPipelined<R, MB>) {
      // One row block: the registers hold two units, and the next unit's loads go out before the
      // current one is multiplied (a wave alone then keeps the memory busy while it computes;
      // measured at one row: 12.6 against 15.0 us for the 7,168 x 5,120 projection).
      Unit a, b;
      if (u_count > 0) load_unit(u_first, a);
      int i = 0;
      for (; i + 2 < u_count; i += 2) {
        load_unit(u_first + (i + 1) * u_step, b);
        use_unit(a);
        load_unit(u_first + (i + 2) * u_step, a);
        use_unit(b);
      }
      if (i + 1 < u_count) {          // two units left (a holds the first of them)
        load_unit(u_first + (i + 1) * u_step, b);
        use_unit(a);
        use_unit(b);
      } else if (i < u_count) {
        use_unit(a);
      }
    } else {
      for (int i = 0; i < u_count; ++i) {
        Unit a;
        load_unit(u_first + i * u_step, a);
        use_unit(a);
      }
    }

    if constexpr (ACT) {
      // per row block all tiles meet at once; wave t < TG adds up gate tile t and up tile t + TG in wave order
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        if (mb > 0 && (rb0 + mb) * 16 >= n_rows) continue;   // uniform over the block
        __syncthreads();
#pragma unroll
        for (int t = 0; t < R; ++t) red[w][t][lane] = acc[t][mb];
        __syncthreads();
        if (w < TG) {
          f32x4 gv = red[0][w][lane], uv = red[0][w + TG][lane];
#pragma unroll
          for (int ww = 1; ww < NW; ++ww) {
            gv += red[ww][w][lane];
            uv += red[ww][w + TG][lane];
          }
          const int row = row_begin + (rb0 + mb) * 16 + r;
          const int n = n_base + w * 16 + g * 4;
          if (row < row_end && n < n_out) {
            const int orow = out_row(row);
            float sc = 1.0f;
            bool scaled = act_scale != nullptr;
            if (picked) {            // a pair's score; the always-on expert's rows are not scaled
              scaled = pk.w != nullptr;
              if (scaled) sc = orow < pk.n_pairs ? pk.w[orow] : 1.0f;
            } else if (scaled) {
              sc = act_scale[row];
            }
            f32x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i)
              o[i] = gated_f32(act, bf16_to_f32(f32_to_bf16(gv[i])), bf16_to_f32(f32_to_bf16(uv[i])), sc, scaled);
            store4<TO>(out + (size_t)orow * n_out + n, o);
          }
        }
      }
      continue;
    }
    // add the waves' K slices in wave order, kRedTiles (tile, row block) pairs per round;
    // pair p of a round is summed and stored by wave p
#pragma unroll
    for (int p0 = 0; p0 < R * MB; p0 += kRedTiles) {
      // a round whose pairs all lie in row blocks beyond the group's rows is skipped (uniform over the block)
      bool any = false;
#pragma unroll
      for (int p = 0; p < kRedTiles; ++p) any = any || (p0 + p < R * MB && ((p0 + p) % MB == 0 || (rb0 + (p0 + p) % MB) * 16 < n_rows));
      if (!any) continue;
      __syncthreads();
#pragma unroll
      for (int p = 0; p < kRedTiles; ++p)
        if (p0 + p < R * MB) red[w][p][lane] = acc[(p0 + p) / MB][(p0 + p) % MB];
      __syncthreads();
      if (w < kRedTiles && p0 + w < R * MB) {
        const int t = (p0 + w) / MB, mb = (p0 + w) % MB;
        f32x4 v = red[0][w][lane];
#pragma unroll
        for (int ww = 1; ww < NW; ++ww) v += red[ww][w][lane];
        // lane holds out[row = ... + r][n = n_base + t*16 + g*4 + 0..3]
        const int row = row_begin + (rb0 + mb) * 16 + r;
        const int n = n_base + t * 16 + g * 4;
        if (row < row_end && n < N) store4<TO>(out + (size_t)out_row(row) * N + n, v);
      }
    }
  }
}

template <int R, int MB, int NW, bool ACT, bool PACKED>
static inline int launch_skinny(const void* x, const void* W, void* out, int out_dtype, int M, int N, int K,
                         const int* a_rows, const int* group_offsets, int groups, const float* act_scale,
                         hipStream_t stream, Picks pk = Picks{}, int act = ACT_SILU) {
  dim3 grid(ceil_div(ACT ? N / 2 : N, 16 * (ACT ? R / 2 : R)), groups > 0 ? groups : 1), block(NW * kWave);
  const int* go = groups > 0 ? group_offsets : nullptr;
  if (out_dtype == DT_F32)
    skinny_gemm_kernel<R, MB, NW, float, ACT, PACKED><<<grid, block, 0, stream>>>(
        (const bf16_t*)x, (const bf16_t*)W, (float*)out, M, N, K, a_rows, go, act_scale, act, pk);
  else
    skinny_gemm_kernel<R, MB, NW, bf16_t, ACT, PACKED><<<grid, block, 0, stream>>>(
        (const bf16_t*)x, (const bf16_t*)W, (bf16_t*)out, M, N, K, a_rows, go, act_scale, act, pk);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
