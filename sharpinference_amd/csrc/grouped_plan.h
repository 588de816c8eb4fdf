// The plan of the grouped product for many rows (prefill), made on the device by the routing
// kernel and read by the product's blocks; the host never learns the routing.
//
// An expert's rows are cut into as few row tiles of at most kPlanTileRows as hold them, all of
// one height (a multiple of 32): its *siblings*.  A *unit* is (expert, one half of the weight
// rows): the blocks of a unit multiply the same weights by the expert's sibling tiles.  Units are
// dealt to the 8 XCDs (each with an L2 of its own), the ones with most siblings first, and every
// XCD walks its units one after the other; inside a unit the siblings of one column block are
// neighbours.  Blocks go to XCDs round-robin by their linear id, so block b is slot b / 8 of XCD
// b % 8: sibling blocks start together on one XCD and stream the same weight rows at the same
// pace, and what the first fetches from memory the others find in that XCD's L2.  No block is
// launched for a sibling that does not exist, except behind an XCD's last unit.
//
// plan (int32), per XCD x at plan + x * plan_stride(E):
//   [0]                 units of this XCD
//   [1 .. 1 + U]        running sum of the units' sibling counts (U + 1 entries, U = 2 * E)
//   [2 + U + 2j], [+1]  expert and half (0 or 1) of unit j
#pragma once

constexpr int kPlanXcds = 8;
constexpr int kPlanTileRows = 192;
constexpr int kPlanHalves = 2;

__host__ __device__ inline int plan_units_max(int n_experts) { return kPlanHalves * n_experts; }
__host__ __device__ inline int plan_stride(int n_experts) { return 2 + 3 * plan_units_max(n_experts); }
__host__ __device__ inline int plan_ints(int n_experts) { return kPlanXcds * plan_stride(n_experts); }
__host__ __device__ inline int plan_siblings(int rows) { return (rows + kPlanTileRows - 1) / kPlanTileRows; }
__host__ __device__ inline int plan_height(int rows, int n_sib) { return ((rows + n_sib - 1) / n_sib + 31) & ~31; }
// Slots (blocks of one column block) an XCD may have to walk, from what the host knows: n_rows
// rows over n_experts experts.  Siblings in all: at most ceil(n_rows / tile) + n_experts, twice
// that in units' siblings, dealt with a difference of at most one unit between XCDs.
inline int plan_sibling_slots_bound(int n_rows, int n_experts) {
  const int tall = (n_rows + kPlanTileRows - 1) / kPlanTileRows;
  const int all = kPlanHalves * (tall + n_experts);
  return (all + kPlanXcds - 1) / kPlanXcds + tall + 1;
}
