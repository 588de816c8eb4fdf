// The plan of the grouped product for many rows (prefill), made on the device by the routing
// kernel and read by the product's blocks; the host never learns the routing.
//
// A *group* is an expert (or the always-on expert that shares the experts' tensor, or a dense
// matrix taken as a single group).  A group's rows are cut into as few row tiles of at most
// kPlanTileRows as hold them, all of one height (a multiple of 32): its *siblings*.  Its column
// blocks are cut into `parts` ranges, more of them the more siblings it has (plan_parts), and a
// *unit* is (group, part): the blocks of a unit multiply the same weight rows by the group's
// sibling tiles.  Units are dealt to the 8 XCDs (each with an L2 of its own), the heaviest first,
// and every XCD walks its units one after the other; inside a unit the siblings of one column
// block are neighbours.  Blocks go to XCDs round-robin by their linear id, so block b is slot
// b / 8 of XCD b % 8: sibling blocks start together on one XCD and stream the same weight rows at
// the same pace, and what the first fetches from memory the others find in that XCD's L2.
//
// The product's blocks stay on their compute units and take slots until none is left: the slots
// of an XCD's walk are handed out in order by a ticket counter that lies behind the unit lists,
// first to the blocks of that XCD (block b sits on XCD b % 8), then to blocks of other XCDs that
// have run out of their own.  So an uneven load is levelled at run time, while the first round of
// slots, the heaviest units, starts as the plan lays it out.
//
// plan (int32), per XCD x at plan + x * plan_stride(G), G groups:
//   [0]                      units of this XCD
//   [1 + 4j .. 4 + 4j]       unit j: group, part, parts, siblings
#pragma once

constexpr int kPlanXcds = 8;
constexpr int kPlanTileRows = 128;
constexpr int kPlanMaxParts = 16;

__host__ __device__ inline int plan_siblings(int rows) { return (rows + kPlanTileRows - 1) / kPlanTileRows; }
__host__ __device__ inline int plan_height(int rows, int n_sib) { return ((rows + n_sib - 1) / n_sib + 31) & ~31; }
// parts of a group's column blocks: as many as keep a unit's work (siblings x column blocks) about level
__host__ __device__ inline int plan_parts(int n_sib) { return n_sib <= 2 ? 2 : n_sib <= 4 ? 4 : n_sib <= 8 ? 8 : kPlanMaxParts; }
// what a unit weighs when units are dealt to the XCDs: its share of the group's (siblings x column blocks)
__host__ __device__ inline int plan_weight(int n_sib) { return n_sib * (kPlanMaxParts / plan_parts(n_sib)); }
// column blocks [first, first + count) of part `part` of `parts`, of nb column blocks in all
__host__ __device__ inline int plan_part_first(int part, int parts, int nb) { return (int)((long long)part * nb / parts); }
__host__ __device__ inline int plan_units_per_xcd_max(int n_groups) { return (kPlanMaxParts * n_groups + kPlanXcds - 1) / kPlanXcds + 1; }
__host__ __device__ inline int plan_stride(int n_groups) { return 1 + 4 * plan_units_per_xcd_max(n_groups); }
// behind the XCDs' unit lists: one ticket counter per XCD (the next slot of that XCD's walk to hand
// out) and a count of the blocks that have left; the routing kernel zeroes them with the plan, and
// the last block of a product to leave zeroes them again for the next product that reads the plan
constexpr int kPlanCounters = 16;
__host__ __device__ inline int plan_ints(int n_groups) { return kPlanXcds * plan_stride(n_groups) + kPlanCounters; }
__host__ __device__ inline int plan_counters_at(int n_groups) { return kPlanXcds * plan_stride(n_groups); }
// Slots (blocks) an XCD may have to walk, from what the host knows: n_rows rows over n_groups
// groups, nb column blocks.  Siblings in all: at most ceil(n_rows / tile) + n_groups; an XCD gets
// an eighth of the (sibling x column block) pairs, give or take one unit.
inline long long plan_slots_bound(int n_rows, int n_groups, int nb) {
  const long long tall = (n_rows + kPlanTileRows - 1) / kPlanTileRows;
  const long long pairs = (tall + n_groups) * nb;
  const long long unit = tall * ((nb + kPlanMaxParts - 1) / kPlanMaxParts + 1) + nb;
  return (pairs + kPlanXcds - 1) / kPlanXcds + unit + 1;
}
