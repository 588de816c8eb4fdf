// MoE routing on the device: router logits, gate, top-k, and the expert-sorted row list.
//
// router_topk: one block per token, or per four tokens when there are many.
// logits[e] = Wr[e, :] . x[t, :] in float (each wave owns experts e = wave, wave + nwaves, ...;
// lanes stride over the hidden width, so the order of the additions depends on the width only).
// gate 0 = sigmoid over every expert, gate 1 = softmax over every expert.  The k picks scan
// ascending with a strict >, so the lowest index wins a tie; the weight of a pick is its gate
// value; renorm divides the k weights by their sum.
//
// moe_permute: one block. Counts rows per expert, prefix-sums them into offsets[E + 1] and
// writes, in expert order, the token and weight of every (token, pick) pair plus the inverse
// map inv_pos[t * k + j] = row in that order, and the plan that the grouped product of many rows
// walks (grouped_plan.h: units of sibling row tiles dealt to the XCDs).  With shared_group the list gets one
// more group after the experts: every token once, weight 1 (an always-on expert that shares the
// experts' weight tensor); offsets then has n_experts + 2 entries and the row arrays n_tokens more.
#include "common.h"
#include "grouped_plan.h"

constexpr int kMaxExperts = 1024;

// One thread: gate the logits g[0 .. n_experts) in place, pick k of them (ascending scan with a
// strict >, so the lowest index wins a tie) into ids / w.
__device__ void gate_and_pick(float* g, int n_experts, int k, int gate, int renorm, int* ids, float* w,
                              float* gate_out) {
  if (gate == 0) {
    for (int e = 0; e < n_experts; ++e) g[e] = 1.0f / (1.0f + expf(-g[e]));
  } else {
    float mx = g[0];
    for (int e = 1; e < n_experts; ++e) mx = fmaxf(mx, g[e]);
    float sum = 0.f;
    for (int e = 0; e < n_experts; ++e) {
      g[e] = expf(g[e] - mx);
      sum += g[e];
    }
    const float inv = 1.0f / sum;
    for (int e = 0; e < n_experts; ++e) g[e] *= inv;
  }
  if (gate_out)
    for (int e = 0; e < n_experts; ++e) gate_out[e] = g[e];
  float wsum = 0.f;
  for (int j = 0; j < k; ++j) {
    int best = -1;
    float bv = -INFINITY;
    for (int e = 0; e < n_experts; ++e) {
      bool taken = false;
      for (int i = 0; i < j; ++i) taken |= (ids[i] == e);
      if (!taken && (best < 0 || g[e] > bv)) {
        bv = g[e];
        best = e;
      }
    }
    ids[j] = best;
    w[j] = bv;
    wsum += bv;
  }
  if (renorm && k > 1 && wsum > 0.f)
    for (int j = 0; j < k; ++j) w[j] /= wsum;
}

// One wave: s[i] = wrow . xr[i] for TT rows, in float.  Lanes stride over the width in runs of 8
// (one fused multiply-add chain per lane and row, in ascending order), then the lanes are summed:
// the order of the additions depends on the width only, and each row has its own accumulator, so
// a token's logit is the same bits whatever TT is and whichever kernel calls this.
template <typename T, typename TW, int TT>
__device__ __forceinline__ void wave_dot_rows(const T* const (&xr)[TT], const TW* __restrict__ wrow, int hidden,
                                              int lane, float (&out)[TT]) {
  float s[TT];
#pragma unroll
  for (int i = 0; i < TT; ++i) s[i] = 0.f;
  if ((hidden & 7) == 0) {
    // Q runs are fetched before the first is added: a row is a dozen dependent round trips
    // to the cache otherwise, and the kernel is nothing but their latency
    constexpr int Q = TT == 1 ? 4 : 2;
    int c = lane * 8;
    for (; c + (Q - 1) * kWave * 8 < hidden; c += Q * kWave * 8) {
      float a[TT][Q][8], b[Q][8];
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        load8(wrow + c + q * kWave * 8, b[q]);
#pragma unroll
        for (int i = 0; i < TT; ++i) load8(xr[i] + c + q * kWave * 8, a[i][q]);
      }
#pragma unroll
      for (int i = 0; i < TT; ++i)
#pragma unroll
        for (int q = 0; q < Q; ++q)
#pragma unroll
          for (int j = 0; j < 8; ++j) s[i] = fmaf(a[i][q][j], b[q][j], s[i]);
    }
    for (; c < hidden; c += kWave * 8) {
      float b[8];
      load8(wrow + c, b);
#pragma unroll
      for (int i = 0; i < TT; ++i) {
        float a[8];
        load8(xr[i] + c, a);
#pragma unroll
        for (int j = 0; j < 8; ++j) s[i] = fmaf(a[j], b[j], s[i]);
      }
    }
  } else {
    for (int c = lane; c < hidden; c += kWave) {
      const float b = to_f32<TW>(wrow[c]);
#pragma unroll
      for (int i = 0; i < TT; ++i) s[i] = fmaf(to_f32<T>(xr[i][c]), b, s[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < TT; ++i) out[i] = wave_sum(s[i]);
}

template <typename T, typename TW, int TT>
__global__ __launch_bounds__(1024) void router_topk_kernel(const T* __restrict__ x, const TW* __restrict__ wr,
                                                           int* __restrict__ topk_ids,
                                                           float* __restrict__ topk_w,
                                                           float* __restrict__ gate_out, int n_tokens, int hidden,
                                                           int n_experts, int k, int gate, int renorm) {
  // TT tokens per block: a router row is fetched once for all of them.
  __shared__ float g[TT][kMaxExperts];
  const int t0 = blockIdx.x * TT;
  const int lane = threadIdx.x & (kWave - 1);
  const int w = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const T* xr[TT];
#pragma unroll
  for (int i = 0; i < TT; ++i) xr[i] = x + (size_t)min(t0 + i, n_tokens - 1) * hidden;   // beyond the last: computed, not kept
  for (int e = w; e < n_experts; e += nw) {
    float v[TT];
    wave_dot_rows<T, TW, TT>(xr, wr + (size_t)e * hidden, hidden, lane, v);
    if (lane == 0) {
#pragma unroll
      for (int i = 0; i < TT; ++i) g[i][e] = v[i];
    }
  }
  __syncthreads();
  if (threadIdx.x < TT && t0 + threadIdx.x < n_tokens) {
    const int t = t0 + threadIdx.x;
    gate_and_pick(g[threadIdx.x], n_experts, k, gate, renorm, topk_ids + (size_t)t * k, topk_w + (size_t)t * k,
                  gate_out ? gate_out + (size_t)t * n_experts : nullptr);
  }
}

// Residual add + RMSNorm + router in one launch, for a few decode tokens: one block per token
// forms h += delta, normalises it (the arithmetic of the norm kernel: a thread per run of 8, the
// same statistics), stores the normalised row in `out` for the experts and keeps a copy in LDS,
// from which its waves then compute the router's logits (wave_dot_rows over the stored, rounded
// values: the bits of the router kernel) and one thread picks.  hidden % 8 == 0, hidden <= 8192.
constexpr int kFusedMaxHidden = 8192;

template <typename TW, typename TWR>
__global__ __launch_bounds__(1024) void add_rmsnorm_router_kernel(
    float* __restrict__ h, const bf16_t* __restrict__ delta, const TW* __restrict__ w, bf16_t* __restrict__ out,
    int hidden, float eps, const TWR* __restrict__ wr, int* __restrict__ topk_ids, float* __restrict__ topk_w,
    int n_experts, int k, int gate, int renorm) {
  __shared__ float red[16];
  __shared__ float g[1][kMaxExperts];
  __shared__ __attribute__((aligned(16))) bf16_t row[kFusedMaxHidden];
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1);
  const int wv = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  float* hr = h + (size_t)t * hidden;
  const int c = threadIdx.x * 8;
  float x[8], wk[8];
  float ss = 0.f;
  if (c < hidden) {
    load8(hr + c, x);
    if (w) load8(w + c, wk);
    if (delta) {
      float d[8];
      load8(delta + (size_t)t * hidden + c, d);
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] += d[j];
      store8(hr + c, x);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += x[j] * x[j];
  }
  const float total = block_sum(ss, red);
  const float s = 1.0f / sqrtf(total / (float)hidden + eps);
  if (c < hidden) {
    float y[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] = w ? (x[j] * s) * wk[j] : x[j] * s;
    store8(out + (size_t)t * hidden + c, y);
    store8(row + c, y);            // the same rounding: what the router would read back from memory
  }
  __syncthreads();
  const bf16_t* xr[1] = {row};
  for (int e = wv; e < n_experts; e += nw) {
    float v[1];
    wave_dot_rows<bf16_t, TWR, 1>(xr, wr + (size_t)e * hidden, hidden, lane, v);
    if (lane == 0) g[0][e] = v[0];
  }
  __syncthreads();
  if (threadIdx.x == 0)
    gate_and_pick(g[0], n_experts, k, gate, renorm, topk_ids + (size_t)t * k, topk_w + (size_t)t * k, nullptr);
}

// h [T, hidden] float (updated), delta [T, hidden] bf16 or null, w the norm's weights (bf16 or float, or
// null), out [T, hidden] bf16, wr [n_experts, hidden] (bf16 or float): what sharpi_add_rmsnorm then
// sharpi_router_topk give, in one launch.
SHARPI_EXPORT int sharpi_add_rmsnorm_router(float* h, const void* delta, const void* w, int w_dtype, void* out,
                                            int n_tokens, int hidden, float eps, const void* wr, int wr_dtype,
                                            int* topk_ids, float* topk_w, int n_experts, int k, int gate,
                                            int renorm, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (hidden <= 0 || (hidden & 7) || hidden > kFusedMaxHidden || !(eps > 0.f)) return SHARPI_ERR_ARG;
  if (n_experts <= 0 || n_experts > kMaxExperts || k <= 0 || k > n_experts || gate < 0 || gate > 1) return SHARPI_ERR_ARG;
  dim3 grid(n_tokens), block(1024);
#define FUSED_LAUNCH(TWV, TWRV)                                                                                  \
  add_rmsnorm_router_kernel<TWV, TWRV><<<grid, block, 0, stream>>>(h, (const bf16_t*)delta, (const TWV*)w,      \
                                                                   (bf16_t*)out, hidden, eps, (const TWRV*)wr,  \
                                                                   topk_ids, topk_w, n_experts, k, gate, renorm)
  const bool wf = w == nullptr || w_dtype == DT_F32;
  if (!wf && w_dtype != DT_BF16) return SHARPI_ERR_ARG;
  if (wr_dtype == DT_BF16) {
    if (wf) FUSED_LAUNCH(float, bf16_t); else FUSED_LAUNCH(bf16_t, bf16_t);
  } else if (wr_dtype == DT_F32) {
    if (wf) FUSED_LAUNCH(float, float); else FUSED_LAUNCH(bf16_t, float);
  } else {
    return SHARPI_ERR_ARG;
  }
#undef FUSED_LAUNCH
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

SHARPI_EXPORT int sharpi_router_topk(const void* x, int x_dtype, const void* wr, int w_dtype, int* topk_ids,
                                     float* topk_w, float* gate_out, int n_tokens, int hidden, int n_experts,
                                     int k, int gate, int renorm, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (hidden <= 0 || n_experts <= 0 || n_experts > kMaxExperts || k <= 0 || k > n_experts) return SHARPI_ERR_ARG;
  if (gate < 0 || gate > 1) return SHARPI_ERR_ARG;
  // one wave per expert at a time: enough waves for the experts, at most 16; with many tokens four
  // share a block (and each fetch of a router row)
  const int tt = n_tokens >= 64 ? 4 : 1;
  dim3 grid(ceil_div(n_tokens, tt)), block(kWave * (n_experts >= 16 ? 16 : n_experts >= 8 ? 8 : 4));
#define ROUTER_LAUNCH(TX, TWT)                                                                                   \
  do {                                                                                                           \
    if (tt == 4)                                                                                                 \
      router_topk_kernel<TX, TWT, 4><<<grid, block, 0, stream>>>((const TX*)x, (const TWT*)wr, topk_ids, topk_w, \
                                                                 gate_out, n_tokens, hidden, n_experts, k, gate, \
                                                                 renorm);                                        \
    else                                                                                                         \
      router_topk_kernel<TX, TWT, 1><<<grid, block, 0, stream>>>((const TX*)x, (const TWT*)wr, topk_ids, topk_w, \
                                                                 gate_out, n_tokens, hidden, n_experts, k, gate, \
                                                                 renorm);                                        \
  } while (0)
  if (x_dtype == DT_F32 && w_dtype == DT_F32) ROUTER_LAUNCH(float, float);
  else if (x_dtype == DT_BF16 && w_dtype == DT_BF16) ROUTER_LAUNCH(bf16_t, bf16_t);
  else if (x_dtype == DT_BF16 && w_dtype == DT_F32) ROUTER_LAUNCH(bf16_t, float);
  else if (x_dtype == DT_F32 && w_dtype == DT_BF16) ROUTER_LAUNCH(float, bf16_t);
  else return SHARPI_ERR_ARG;
#undef ROUTER_LAUNCH
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// One block: the expert-sorted list of the (token, pick) pairs; count and cursor are LDS of
// n_experts ints.  Every thread of the block calls it; the pairs must be visible to the block.
__device__ void permute_block(const int* __restrict__ topk_ids, const float* __restrict__ topk_w,
                              int* __restrict__ offsets, int* __restrict__ sorted_token,
                              float* __restrict__ sorted_w, int* __restrict__ inv_pos, int* __restrict__ plan,
                              int n_pairs, int k, int n_experts, int shared_group, int* count, int* cursor,
                              int* plan_scratch) {
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) atomicAdd(&count[topk_ids[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < n_experts; ++e) {
      offsets[e] = run;
      cursor[e] = run;
      run += count[e];
    }
    offsets[n_experts] = run;
    // an always-on expert as one more group: every token once, in token order, with weight 1
    if (shared_group) offsets[n_experts + 1] = run + n_pairs / k;
  }
  if (shared_group) {
    for (int t = threadIdx.x; t < n_pairs / k; t += blockDim.x) {
      sorted_token[n_pairs + t] = t;
      sorted_w[n_pairs + t] = 1.0f;
    }
  }
  if (plan) {
    // The plan of the grouped product (grouped_plan.h).  Groups: the experts, and the always-on
    // group (every token once) if there is one.  Every group with rows gives plan_parts units;
    // units in the order of their weight (then of group and part) are dealt to the XCDs row by
    // row, rows alternating in direction so that the XCDs' loads stay level.
    const int n_groups = n_experts + (shared_group ? 1 : 0);
    const int stride = plan_stride(n_groups);
    if (shared_group && threadIdx.x == 0) count[n_experts] = n_pairs / k;
    __syncthreads();
    // unit_base[g]: units of the groups before g (in cursor's place it would clash: a second array)
    int* unit_base = plan_scratch;
    if (threadIdx.x == 0) {
      int run = 0;
      for (int g = 0; g < n_groups; ++g) {
        unit_base[g] = run;
        if (count[g] > 0) run += plan_parts(plan_siblings(count[g]));
      }
      unit_base[n_groups] = run;
    }
    __syncthreads();
    const int units = unit_base[n_groups];
    for (int g = threadIdx.x; g < n_groups; g += blockDim.x) {
      if (count[g] == 0) continue;
      const int sg = plan_siblings(count[g]);
      const int wg = plan_weight(sg), pg = plan_parts(sg);
      // units that come before this group's: of heavier groups all, of equally heavy ones those of lower index
      int before = 0;
      for (int j = 0; j < n_groups; ++j) {
        if (count[j] == 0 || j == g) continue;
        const int sj = plan_siblings(count[j]);
        const int wj = plan_weight(sj);
        if (wj > wg || (wj == wg && j < g)) before += plan_parts(sj);
      }
      for (int part = 0; part < pg; ++part) {
        const int u = before + part;
        const int pos = u / kPlanXcds;
        const int xcd = (pos & 1) ? kPlanXcds - 1 - u % kPlanXcds : u % kPlanXcds;
        int* pu = plan + xcd * stride + 1 + 4 * pos;
        pu[0] = g;
        pu[1] = part;
        pu[2] = pg;
        pu[3] = sg;
      }
    }
    if (threadIdx.x < kPlanXcds) {
      // XCD x holds one unit of every full row of 8, and of the last row the units that exist
      const int x = threadIdx.x;
      int n = 0;
      for (int pos = 0; pos * kPlanXcds < units; ++pos) {
        const int u = pos * kPlanXcds + ((pos & 1) ? kPlanXcds - 1 - x : x);
        if (u < units) ++n;
      }
      plan[x * stride] = n;
    }
    if (threadIdx.x < kPlanCounters) plan[plan_counters_at(n_groups) + threadIdx.x] = 0;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) {
    const int e = topk_ids[i];
    const int r = atomicAdd(&cursor[e], 1);
    sorted_token[r] = i / k;
    sorted_w[r] = topk_w[i];
    inv_pos[i] = r;
  }
}

__global__ __launch_bounds__(1024) void moe_permute_kernel(const int* __restrict__ topk_ids,
                                                           const float* __restrict__ topk_w,
                                                           int* __restrict__ offsets,
                                                           int* __restrict__ sorted_token,
                                                           float* __restrict__ sorted_w,
                                                           int* __restrict__ inv_pos, int* __restrict__ plan,
                                                           int n_pairs, int k, int n_experts, int shared_group) {
  __shared__ int count[kMaxExperts + 1];
  __shared__ int cursor[kMaxExperts];
  __shared__ int plan_scratch[kMaxExperts + 2];
  permute_block(topk_ids, topk_w, offsets, sorted_token, sorted_w, inv_pos, plan, n_pairs, k, n_experts,
                shared_group, count, cursor, plan_scratch);
}

// plan: plan_ints(n_experts + shared_group) ints (grouped_plan.h) for the grouped product of many rows, or null.
SHARPI_EXPORT int sharpi_moe_permute(const int* topk_ids, const float* topk_w, int* offsets, int* sorted_token,
                                     float* sorted_w, int* inv_pos, int* plan, int plan_len, int n_tokens, int k,
                                     int n_experts, int shared_group, hipStream_t stream) {
  if (n_experts <= 0 || n_experts > kMaxExperts || k <= 0) return SHARPI_ERR_ARG;
  if (n_tokens < 0) return SHARPI_ERR_ARG;
  if (plan && plan_len < plan_ints(n_experts + (shared_group ? 1 : 0))) return SHARPI_ERR_ARG;
  moe_permute_kernel<<<1, 1024, 0, stream>>>(topk_ids, topk_w, offsets, sorted_token, sorted_w, inv_pos, plan,
                                             n_tokens * k, k, n_experts, shared_group);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

SHARPI_EXPORT int sharpi_grouped_plan_ints(int n_groups) { return plan_ints(n_groups); }
SHARPI_EXPORT int sharpi_router_max_experts() { return kMaxExperts; }
SHARPI_EXPORT int sharpi_add_rmsnorm_router_max_hidden() { return kFusedMaxHidden; }
