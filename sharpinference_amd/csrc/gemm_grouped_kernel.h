// Grouped matrix product for routed experts with many rows (prefill):
//   out[row, :] = x[a_rows[row], :] * W[e]^T   for the rows of expert e in the expert-sorted list,
// bfloat16 inputs, float accumulation on the matrix cores.
//
// The product is bound by reading the experts' weights while few rows share them, and by the
// matrix cores' operand traffic once many do.  A block takes up to 128 rows of its expert against
// 512 weight rows: an expert's weights are then read once for every 128 of its rows.  An expert
// with more rows is cut into sibling tiles of equal height, and the blocks that multiply the SAME
// weight rows by sibling tiles start side by side on one XCD, so that the weights cross the memory
// interface about once all the same (grouped_plan.h says how the routing kernel lays that out;
// the host never learns the routing).  The tile's work is compiled for every height in steps of
// 32 rows up to 128, and a block takes the smallest that holds its rows: no branch inside a K
// stage, nothing multiplied for 32-row pieces that hold no row (rows are staged in passes of 64).
//  * The blocks are persistent: as many as there are compute units (each holds one), every block
//    taking the next slot of its XCD's walk from a ticket counter until none is left, then slots
//    of other XCDs.  Experts of very different loads, whose tiles take very different times, are
//    so levelled at run time; with blocks dealt out beforehand an XCD that drew a block more than
//    its units can hold at once ran a second round alone.  The caller may bound the number of
//    blocks, to leave compute units to other work that runs beside the product.
//  * Each of the 8 waves owns 64 weight rows (4 MFMA tiles) and reads them straight from global
//    memory into registers, a ring of 64-wide K stages ahead: a weight element is used by one wave
//    only.  An x fragment read from LDS feeds four products (with two tiles a wave and 192-row
//    blocks the LDS reads, one per two products, kept pace with the matrix cores and bounded them
//    at 0.92 PFLOP/s at 8,192 tokens; four tiles reach 1.09).
//  * The x rows (gathered through a_rows) are shared by the waves and staged through LDS, 64
//    columns of K at a time, double-buffered and fetched two stages ahead; the 16-byte chunks of
//    a row are swizzled so that reads and stores are free of bank conflicts.
//  * W is the A operand (rows = n), x the B operand: a lane ends up with 4 consecutive n of one
//    row, stored as one 8-byte write.  Each output is one chain over k in ascending order, so a
//    row's result does not depend on which other rows share its tile, nor on which block took it.
//  * SwiGLU form (ACT): W holds gate rows [0, N/2) and up rows [N/2, N) of every expert; a wave's
//    tiles are two gate tiles and the up tiles of the same 32 columns, so a lane ends up with both
//    products of its outputs, rounds them to bfloat16 (what a separate activation kernel would have
//    read) and stores act(s g) * (s u), s the row's score: out is [rows, N/2] and the gate|up
//    rows never go to memory.
// Limits: K % 64 == 0, N % 4 == 0 (N % 32 == 0 in the SwiGLU form).
#pragma once
#include <type_traits>

#include "common.h"
#include "grouped_plan.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

#ifndef SHARPI_GAHEAD
#define SHARPI_GAHEAD 2
#endif
#ifndef SHARPI_GQ
#define SHARPI_GQ 4
#endif
#ifndef SHARPI_GK
#define SHARPI_GK 64
#endif
constexpr int GM = kPlanTileRows;  // rows per tile
static_assert(GM == kPlanTileRows, "the routing kernel's plan is made for tiles of this height");
constexpr int GMT = GM / 16;  // 16-row groups per tile
#ifndef SHARPI_GW
#define SHARPI_GW 8
#endif
#ifndef SHARPI_GNT
#define SHARPI_GNT 4
#endif
constexpr int GW = SHARPI_GW;   // waves per block
constexpr int kMaxNT = SHARPI_GNT;  // 16-row weight tiles per wave: this many, or a half or a quarter where a slot is cut
constexpr int columns_of(int nt) { return 16 * nt * GW; }   // weight rows (output columns) of a block
constexpr int GK = SHARPI_GK;  // K per LDS stage
constexpr int GPAD = GK;      // LDS row: no pad, the 16-byte chunks of a row are swizzled instead (xs_col)
constexpr int GROWS = GW * 64 / (GK / 8);   // rows staged per pass: GK / 8 threads per row
constexpr int GPASS = GM / GROWS;  // staging passes
constexpr int kXcds = kPlanXcds;   // accelerator dies, each with its own L2
constexpr int kAhead = SHARPI_GAHEAD;  // K stages of weights in flight per wave (2, 3 or 4)
constexpr int GQ = SHARPI_GQ;       // 16-row groups whose LDS reads go out together (divides 4)

// Where column `col` (a multiple of 8 elements = one 16-byte chunk) of LDS row `row` is kept: the
// chunk index is XORed with bits 1..3 of the row.  The LDS serves a 16-byte read of a wave in four
// turns of two octets of lanes, one octet from rows 0..7 and one from rows 8..15 of the operand
// (measured with the bank-conflict counter: rows padded to 144 bytes conflict two ways).  With the
// swizzle the eight chunks an octet reads fall into eight different 16-byte bank groups of its half
// (even rows use one half of the 256-byte bank space, odd rows the other), and the two octets of a
// turn into different ones; an octet of the staging stores fills one whole row, i.e. one half.
static_assert(GK == 64, "the swizzle assumes rows of eight 16-byte chunks");
__device__ __forceinline__ int xs_col(int row, int col) { return col ^ (((row >> 1) & 7) << 3); }

// A weight fragment.  STREAM: with the streaming hint (nontemporal), for a group whose weights no
// other row tile reads: a pure read in this kernel's pattern reaches 6.9 TB/s with the hint and
// 6.2 without.  A group cut into sibling tiles reads them without the hint: what the first
// sibling fetches the others are to find in the L2.
template <bool STREAM> __device__ __forceinline__ bf16x8 load_weights(const bf16_t* p) {
  if constexpr (STREAM) return __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p));
  else return *reinterpret_cast<const bf16x8*>(p);
}

// The work of one tile of MT * 16 rows (the block's rows, rounded up) against 16 * NT * GW weight rows.
template <typename TO, int MT, int NT, bool PACKED, bool ACT, bool STREAM>
__device__ __forceinline__ void grouped_tile(const bf16_t* __restrict__ x, const bf16_t* __restrict__ We,
                                             TO* __restrict__ out, int N, int K, const int* __restrict__ a_rows,
                                             const float* __restrict__ act_scale, int act, int row0, int row_end,
                                             int n_base, bf16_t (*xs)[GM][GPAD]) {
  static_assert(!ACT || NT % 2 == 0, "the SwiGLU form pairs gate tiles with up tiles");
  constexpr int HT = ACT ? NT / 2 : NT;         // tiles of distinct output columns per wave
  const int n_out = ACT ? N / 2 : N;            // output columns
  constexpr int PASS = (MT * 16 + GROWS - 1) / GROWS;   // staging passes
  constexpr int Q = MT % GQ == 0 ? GQ : 2;      // 16-row groups whose LDS reads go out together
  static_assert(MT % Q == 0, "tile heights come in steps of 32 rows");
  const int lane = threadIdx.x & (kWave - 1);
  const int r = lane & 15, g = lane >> 4;

  // 32-bit element offsets from uniform bases (the host checks that they fit): half the address registers
  // Row layout: lane (r, g) reads 16 bytes of row n at k = c*GK + j*32 + g*8.  Packed layout (the
  // matrix stored as [N/16][K/128][16 runs of 8 k][16 rows][8]): the same element sits at
  // tile*16*K + c*GK*16 + j*512 + lane*8, and a wave's load is one contiguous 1 KB.
  constexpr uint32_t kStageStep = PACKED ? GK * 16 : GK;
  constexpr uint32_t kSubStep = PACKED ? 512 : 32;
  static_assert(128 % GK == 0, "a K stage must not straddle a packed 128-wide unit");
  uint32_t woff[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    // ACT: tile 0 is the gate tile of the wave's 16 columns, tile 1 the up tile of the same columns
    if constexpr (PACKED) {
      int n = n_base + (t % HT) * 16;
      if (n >= n_out) n = n_out - 16;  // loaded, never stored
      if (ACT && t >= HT) n += n_out;
      woff[t] = (uint32_t)n * (uint32_t)K + lane * 8;
    } else {
      int n = n_base + (t % HT) * 16 + r;
      if (n >= n_out) n = n_out - 1;  // loaded, never stored
      if (ACT && t >= HT) n += n_out;
      woff[t] = (uint32_t)n * (uint32_t)K + g * 8;
    }
  }
  // staging role: thread loads 16 bytes of row (tid / 8 + GROWS * pass), columns (tid % 8) * 8
  const int srow = threadIdx.x / (GK / 8), scol = (threadIdx.x % (GK / 8)) * 8;
  uint32_t xoff[PASS];
#pragma unroll
  for (int ps = 0; ps < PASS; ++ps) {
    // rows beyond the expert's last read its last row again: every load is unconditional, and what
    // such rows produce is never stored
    const int row = min(row0 + srow + GROWS * ps, row_end - 1);
    xoff[ps] = (uint32_t)(a_rows ? a_rows[row] : row) * (uint32_t)K + scol;
  }

  f32x4 acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int mb = 0; mb < MT; ++mb) acc[t][mb] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int chunks = K / GK;
  // The memory counter retires loads in order, so waiting for one load waits for every load issued
  // before it.  Both streams therefore run the same distance ahead: x rows of stage c + 2 go into
  // one of two register sets while stage c is multiplied (and into LDS one stage later), weights
  // of stage c + kAhead into the ring slot that stage c has just used up.
  u32x4 stage[2][PASS];
  bf16x8 wf[kAhead][GK / 32][NT];   // weight fragments of the next kAhead stages, a ring indexed by stage % kAhead
#pragma unroll
  for (int ps = 0; ps < PASS; ++ps) stage[0][ps] = *reinterpret_cast<const u32x4*>(x + xoff[ps]);
  if (chunks > 1) {
#pragma unroll
    for (int ps = 0; ps < PASS; ++ps) stage[1][ps] = *reinterpret_cast<const u32x4*>(x + xoff[ps] + GK);
  }
  auto fill_ring = [&](auto all_tag) {
#pragma unroll
    for (int a = 0; a < kAhead; ++a)
      if (decltype(all_tag)::value || a < chunks) {
#pragma unroll
        for (int j = 0; j < GK / 32; ++j)
#pragma unroll
          for (int t = 0; t < NT; ++t) wf[a][j][t] = load_weights<STREAM>(We + woff[t] + a * kStageStep + j * kSubStep);
      }
  };
  if (chunks >= kAhead) fill_ring(std::true_type{}); else fill_ring(std::false_type{});
#pragma unroll
  for (int ps = 0; ps < PASS; ++ps) *reinterpret_cast<u32x4*>(&xs[0][srow + GROWS * ps][xs_col(srow + GROWS * ps, scol)]) = stage[0][ps];
  __syncthreads();

  // One K stage; `slot` (the stage's place in the ring) and `par` (its parity) are compile-time
  // constants.  `steady`: every load of the stage is known to be in range, so none sits behind a
  // branch.  The compiler counts outstanding loads statically; a load that may or may not have been
  // issued makes it wait for all of them, and nothing would be hidden.
  auto stage_step = [&](int c, auto slot_tag, auto par_tag, auto steady_tag) {
    constexpr int slot = decltype(slot_tag)::value;
    constexpr int par = decltype(par_tag)::value;
    constexpr bool steady = decltype(steady_tag)::value;
    if (steady || c + 2 < chunks) {   // this stage's register set went to LDS a stage ago
#pragma unroll
      for (int ps = 0; ps < PASS; ++ps) stage[par][ps] = *reinterpret_cast<const u32x4*>(x + xoff[ps] + (c + 2) * GK);
    }
    // the loads above are issued here and waited for a stage later: without the fence the compiler
    // moves each load down to the LDS store that uses it and waits for it at once
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < GK / 32; ++j) {
      // 16-row groups GQ at a time: their LDS reads go out together, then their MFMAs
#pragma unroll
      for (int mq = 0; mq < MT; mq += Q) {
        bf16x8 xf[Q];
#pragma unroll
        for (int i = 0; i < Q; ++i) xf[i] = *reinterpret_cast<const bf16x8*>(&xs[par][(mq + i) * 16 + r][xs_col(r, j * 32 + g * 8)]);
#pragma unroll
        for (int i = 0; i < Q; ++i)
#pragma unroll
          for (int t = 0; t < NT; ++t)
            acc[t][mq + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[slot][j][t], xf[i], acc[t][mq + i], 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (steady || c + kAhead < chunks) {   // this slot's weights are used up: fetch those of kAhead stages on
#pragma unroll
      for (int j = 0; j < GK / 32; ++j)
#pragma unroll
        for (int t = 0; t < NT; ++t)
          wf[slot][j][t] = load_weights<STREAM>(We + woff[t] + (c + kAhead) * kStageStep + j * kSubStep);
    }
    if (steady || c + 1 < chunks) {   // the next stage's x rows, fetched a stage ago
#pragma unroll
      for (int ps = 0; ps < PASS; ++ps) *reinterpret_cast<u32x4*>(&xs[par ^ 1][srow + GROWS * ps][xs_col(srow + GROWS * ps, scol)]) = stage[par ^ 1][ps];
    }
    __syncthreads();
  };
  // stages are unrolled over ring slot x parity, so that both are constants
  constexpr int kUnroll = (kAhead % 2 == 0) ? kAhead : 2 * kAhead;
  auto stage_group = [&](int c, auto steady_tag) {
    auto one = [&](auto i_tag) {
      constexpr int i = decltype(i_tag)::value;
      if (decltype(steady_tag)::value || c + i < chunks)
        stage_step(c + i, std::integral_constant<int, i % kAhead>{}, std::integral_constant<int, i % 2>{}, steady_tag);
    };
    // exactly kUnroll stages: the loops below advance by that many
    one(std::integral_constant<int, 0>{}); one(std::integral_constant<int, 1>{});
    if constexpr (kUnroll > 2) { one(std::integral_constant<int, 2>{}); one(std::integral_constant<int, 3>{}); }
    if constexpr (kUnroll > 4) { one(std::integral_constant<int, 4>{}); one(std::integral_constant<int, 5>{}); }
    static_assert(kUnroll == 2 || kUnroll == 4 || kUnroll == 6, "stage_group lists two, four or six stages");
  };
  int c = 0;
  for (; c + kUnroll + kAhead <= chunks; c += kUnroll) stage_group(c, std::true_type{});   // every fetch is of a stage that exists
  for (; c < chunks; c += kUnroll) stage_group(c, std::false_type{});                      // the last stages check each fetch

  // lane holds out[row0 + mb*16 + r][n_base + t*16 + 4g + 0..3]
  auto store = [&](TO* dst, const f32x4& v) {
    if constexpr (sizeof(TO) == 4) {
      *reinterpret_cast<f32x4*>(dst) = v;
    } else {
      uint2 packed;
      packed.x = (uint32_t)f32_to_bf16(v[0]).bits | ((uint32_t)f32_to_bf16(v[1]).bits << 16);
      packed.y = (uint32_t)f32_to_bf16(v[2]).bits | ((uint32_t)f32_to_bf16(v[3]).bits << 16);
      *reinterpret_cast<uint2*>(dst) = packed;
    }
  };
#pragma unroll
  for (int mb = 0; mb < MT; ++mb) {
    const int row = row0 + mb * 16 + r;
    if (row >= row_end) continue;
    if constexpr (ACT) {
      const float sc = act_scale ? act_scale[row] : 1.0f;
#pragma unroll
      for (int h = 0; h < HT; ++h) {
        const int n = n_base + h * 16 + 4 * g;
        if (n >= n_out) continue;
        f32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          o[i] = gated_f32(act, bf16_to_f32(f32_to_bf16(acc[h][mb][i])), bf16_to_f32(f32_to_bf16(acc[h + HT][mb][i])), sc,
                           act_scale != nullptr);
        store(out + (size_t)row * n_out + n, o);
      }
    } else {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int n = n_base + t * 16 + 4 * g;
        if (n >= N) continue;
        store(out + (size_t)row * N + n, acc[t][mb]);
      }
    }
  }
}

template <typename TO, int NT, bool PACKED, bool ACT>
__global__ __launch_bounds__(GW* kWave, 2) void grouped_gemm_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ W, TO* __restrict__ out, int N, int K,
    const int* __restrict__ a_rows, const float* __restrict__ act_scale, int act,
    const int* __restrict__ group_offsets, const int* __restrict__ plan, int n_groups, int nb) {
  __shared__ __attribute__((aligned(16))) bf16_t xs[2][GM][GPAD];
  __shared__ int s_slot;
  constexpr int GN = columns_of(NT);
  constexpr int kCols = ACT ? GN / 2 : GN;   // output columns of a block
  const int n_out = ACT ? N / 2 : N;
  // The blocks stay (one to a compute unit, as many as there are units) and take work until none is
  // left.  Workgroups go to the 8 XCDs round-robin by their linear id, so this block sits on XCD
  // blockIdx.x % 8 and walks that XCD's units first, slot by slot: a unit's column blocks times its
  // siblings, the siblings of a column block side by side.  The slots of an XCD are handed out by a
  // ticket counter; when its own XCD's are gone a block takes slots of the next XCD's walk.
  //
  // A slot takes a block about as long whatever its rows (it streams the same weights), and a walk
  // is only a few slots per block long: slots that fill no whole round of the XCD's blocks would
  // leave most of them idle for a slot's time at the end.  Those last slots are therefore cut by
  // columns into 2 or 4 narrower ones (2 or 1 weight tiles a wave), as many as spread them over
  // the blocks; a walk of fewer slots than blocks is cut the same way.
  int* counters = const_cast<int*>(plan) + plan_counters_at(n_groups);
  const int home = blockIdx.x % kXcds;
  const int per_xcd = ((int)gridDim.x + kXcds - 1) / kXcds;   // blocks whose first walk is one XCD's
  constexpr int kMaxCut = ACT ? NT / 2 : NT;                  // the gated form keeps a gate and an up tile a wave
  for (int q = 0; q < kXcds; ++q) {
    const int xcd = (home + q) % kXcds;
    const int* px = plan + xcd * plan_stride(n_groups);
    const int n_units = px[0];
    int total = 0;                                 // slots of this walk
    for (int j = 0; j < n_units; ++j) {
      const int* pu = px + 1 + 4 * j;
      total += (plan_part_first(pu[1] + 1, pu[2], nb) - plan_part_first(pu[1], pu[2], nb)) * pu[3];
    }
    const int whole = total / per_xcd * per_xcd;   // slots of whole rounds: taken as they are
    const int rest = total - whole;
    int cut = 1;
    if (rest > 0 && 2 * rest <= per_xcd) cut = (4 * rest <= per_xcd && kMaxCut >= 4) ? 4 : (kMaxCut >= 2 ? 2 : 1);
    const int tickets = whole + rest * cut;
    for (;;) {
      if (threadIdx.x == 0) s_slot = atomicAdd(&counters[xcd], 1);
      __syncthreads();
      const int ticket = s_slot;
      __syncthreads();
      if (ticket >= tickets) break;                // this walk is done
      const int width = ticket < whole ? 1 : cut;  // this slot is 1 / width of a column block
      int slot = ticket < whole ? ticket : whole + (ticket - whole) / width;
      const int piece = ticket < whole ? 0 : (ticket - whole) % width;
      int e = -1, n_sib = 1, col0 = 0;
      for (int j = 0; j < n_units; ++j) {          // (a handful of units per XCD)
        const int* pu = px + 1 + 4 * j;
        const int first = plan_part_first(pu[1], pu[2], nb);
        const int slots = (plan_part_first(pu[1] + 1, pu[2], nb) - first) * pu[3];
        if (slot < slots) {
          e = pu[0];
          n_sib = pu[3];
          col0 = first;
          break;
        }
        slot -= slots;
      }
      if (e < 0) break;                            // (behind the walk's last unit: not reached)
      const int sib = slot % n_sib;
      const int nblock = col0 + slot / n_sib;
      const int col_base = nblock * kCols + piece * (kCols / width);
      if (col_base >= n_out) continue;
      const int first_row = group_offsets[e];
      const int last_row = group_offsets[e + 1];
      const int height = plan_height(last_row - first_row, n_sib);
      const int row0 = first_row + sib * height;
      const int row_end = min(last_row, row0 + height);
      const int n_rows = row_end - row0;
      if (n_rows <= 0) continue;
      const int wave_cols = (ACT ? 8 * NT : 16 * NT) / width;   // output columns of a wave
      const int n_base = col_base + (threadIdx.x >> 6) * wave_cols;
      const bf16_t* We = W + (size_t)e * N * K;
      static_assert(GM == 128, "tile heights are compiled in steps of 32 rows up to 128");
#define GT1(MTV, NTV, ST) grouped_tile<TO, MTV, NTV, PACKED, ACT, ST>(x, We, out, N, K, a_rows, act_scale, act, row0, row_end, n_base, xs)
      // (the hint only for weights stored tile by tile, the order the served model keeps them in)
#define GT2(MTV, NTV)                                \
  do {                                               \
    if (PACKED && n_sib == 1) GT1(MTV, NTV, PACKED); \
    else GT1(MTV, NTV, false);                       \
  } while (0)
#define GT(NTV)                     \
  do {                              \
    if (n_rows <= 32) GT2(2, NTV);  \
    else if (n_rows <= 64) GT2(4, NTV); \
    else if (n_rows <= 96) GT2(6, NTV); \
    else GT2(8, NTV);               \
  } while (0)
      if (width == 1) GT(NT);
      else if constexpr (kMaxCut >= 2) {
        if (width == 2) GT(NT / 2);
        else if constexpr (kMaxCut >= 4) GT(NT / 4);
      }
#undef GT
#undef GT2
#undef GT1
    }
  }
  // the last block to leave sets the counters back for the next product that reads this plan
  if (threadIdx.x == 0) {
    if (atomicAdd(&counters[kXcds], 1) == (int)gridDim.x - 1) {
      for (int i = 0; i <= kXcds; ++i) counters[i] = 0;
    }
  }
}

static bool grouped_args_ok(int x_rows, int n_rows, int N, int K, int n_groups, int packed, const int* group_offsets,
                            const int* plan) {
  if (N <= 0 || (N & 3) || K <= 0 || K % GK != 0 || n_groups <= 0) return false;
  if (packed && ((N & 15) || (K & 127))) return false;
  if (!group_offsets || !plan) return false;
  // the kernel addresses x and one group's weights with 32-bit element offsets
  return (long long)N * K <= 0x7fffffffLL && x_rows > 0 && (long long)x_rows * K <= 0x7fffffffLL;
}

static int compute_units() {
  static int units[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (units[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    units[dev] = n;
  }
  return units[dev];
}

// As many blocks as stay at once (one to a compute unit), fewer if there is less work (a slot may
// be cut in up to four) or if the caller bounds them (max_blocks > 0: the compute units left over
// are for other work).
static dim3 grouped_grid(int n_rows, int n_groups, int nb, int max_blocks) {
  long long blocks = 4LL * kXcds * plan_slots_bound(n_rows, n_groups, nb);
  const long long stay = compute_units();
  if (blocks > stay) blocks = stay;
  if (max_blocks > 0 && blocks > max_blocks) blocks = max_blocks;
  return dim3((unsigned)(blocks < 1 ? 1 : blocks));
}

