// Token selection from float logits [rows, vocab]: argmax, and temperature sampling with the
// top-k / min-p / top-p filters, one block per row.
//
// argmax: the lowest index among equal maxima wins.
// sample: p = softmax(logits / T); top-k keeps every p >= the k-th largest value and
// renormalises; min-p zeroes p < min_p * max p; top-p keeps every p >= the value at which the
// descending running sum first reaches top_p (equal values at that cut are all kept); after a
// last renormalisation the token is the first index whose ascending running sum reaches u, or
// vocab - 1 if rounding leaves none.  `probs` is a [rows, vocab] float workspace.
#include "common.h"

constexpr int kSampThreads = 1024;

__device__ __forceinline__ float block_max(float v, float* red) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wid = threadIdx.x >> 6;
  const int nw = (blockDim.x + kWave - 1) >> 6;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) red[wid] = v;
  __syncthreads();
  float t = red[0];
  for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
  return t;
}

__global__ __launch_bounds__(kSampThreads) void argmax_rows_kernel(const float* __restrict__ logits,
                                                                  int* __restrict__ out, int vocab) {
  __shared__ float bv[kSampThreads / kWave];
  __shared__ int bi[kSampThreads / kWave];
  const float* x = logits + (size_t)blockIdx.x * vocab;
  float best = -INFINITY;
  int idx = 0x7fffffff;
  int i0 = 0;
  if ((vocab & 3) == 0) {
    // 16-byte loads, two in flight per thread: one block reads a row at a compute unit's full rate.
    // A thread's indices still ascend, so a strict > keeps the lowest index of equal values.
    const int v4 = vocab >> 2;
    const float4* x4 = reinterpret_cast<const float4*>(x);
    int q = threadIdx.x;
    for (; q + (int)blockDim.x < v4; q += 2 * blockDim.x) {
      const float4 a = x4[q], b = x4[q + blockDim.x];
      const float va[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int i = (j < 4 ? q : q + (int)blockDim.x) * 4 + (j & 3);
        if (va[j] > best || idx == 0x7fffffff) {
          best = va[j];
          idx = i;
        }
      }
    }
    for (; q < v4; q += blockDim.x) {
      const float4 a = x4[q];
      const float va[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (va[j] > best || idx == 0x7fffffff) {
          best = va[j];
          idx = q * 4 + j;
        }
    }
    i0 = vocab;
  }
  for (int i = i0 + threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = x[i];
    if (v > best || idx == 0x7fffffff) {  // ascending i per thread: strict > keeps the lowest index
      best = v;
      idx = i;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, kWave);
    const int oi = __shfl_xor(idx, off, kWave);
    if (oi != 0x7fffffff && (idx == 0x7fffffff || ov > best || (ov == best && oi < idx))) {
      best = ov;
      idx = oi;
    }
  }
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x >> 6;
  if (lane == 0) {
    bv[wid] = best;
    bi[wid] = idx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < (int)(blockDim.x >> 6); ++i) {
      if (bi[i] != 0x7fffffff && (idx == 0x7fffffff || bv[i] > best || (bv[i] == best && bi[i] < idx))) {
        best = bv[i];
        idx = bi[i];
      }
    }
    out[blockIdx.x] = idx == 0x7fffffff ? 0 : idx;
  }
}

SHARPI_EXPORT int sharpi_argmax_rows(const float* logits, int* out, int rows, int vocab, hipStream_t stream) {
  if (rows <= 0) return SHARPI_OK;
  if (vocab <= 0) return SHARPI_ERR_ARG;
  argmax_rows_kernel<<<rows, kSampThreads, 0, stream>>>(logits, out, vocab);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// count and sum of the entries of p with bits >= thr_bits (p >= 0, so float order == uint order)
__device__ __forceinline__ void count_sum_ge(const float* p, int vocab, uint32_t thr_bits, float* red,
                                             int* red_i, int& count, float& sum) {
  int c = 0;
  float s = 0.f;
  #pragma unroll 8
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = p[i];
    if (__float_as_uint(v) >= thr_bits) {
      ++c;
      s += v;
    }
  }
  sum = block_sum(s, red);
  // integer block sum
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x >> 6;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off, kWave);
  __syncthreads();
  if (lane == 0) red_i[wid] = c;
  __syncthreads();
  int t = 0;
  for (int i = 0; i < (int)(blockDim.x >> 6); ++i) t += red_i[i];
  count = t;
}

__device__ __forceinline__ void renormalise(float* p, int vocab, float* red) {
  float s = 0.f;
  #pragma unroll 8
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) s += p[i];
  const float total = block_sum(s, red);
  if (total > 0.f && total != 1.0f) {
    const float inv = 1.0f / total;
    #pragma unroll 8
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) p[i] *= inv;
  }
  __syncthreads();
}


// Rows with a small top-k (the usual case: 40 of 200,000) need the whole vocabulary three times
// only: for the maximum, for the softmax sum, and to collect the few entries that can survive.
// Every thread's largest probability is one element, so the k-th largest of those 1,024 values is a
// lower bound of the k-th largest probability: entries at or above it (a few more than k) go to
// LDS, one per thread, and top-k, min-p, top-p, both renormalisations and the inverse CDF run
// there, with the same definitions as the full path below (ties at a cut are all kept; the CDF
// walks ascending indices).  The probabilities have the same bits as the full path's.
// Without a top-k (k = 0) the 256 largest-or-so entries are gathered the same way, and the result
// stands if nothing else can survive: the gathered entries that pass min-p already hold top_p of
// the mass (a peaked distribution), or min-p's cut lies at or above the gathering bound.
// Returns false, with nothing written, if more entries than threads reach the bound or that
// cannot be shown: the caller then takes the full path.  Every thread of the block returns the
// same value.
constexpr int kFastMaxK = 256;

__device__ __forceinline__ bool sample_few_survivors(const float* __restrict__ x, int vocab, float T, int k, float mp,
                                                     float tp, float u, int* __restrict__ out_r, float* red) {
  __shared__ float a_p[kSampThreads];
  __shared__ int a_i[kSampThreads];
  __shared__ float b_p[kSampThreads];
  __shared__ int b_i[kSampThreads];
  __shared__ float s_bound;
  __shared__ int s_count, s_win;
  const int t = threadIdx.x;
  const int nt = blockDim.x;
  const float invT = 1.0f / T;
  const bool scaled = T != 1.0f;

  float vmax = -INFINITY;
  #pragma unroll 8
  for (int i = t; i < vocab; i += nt) vmax = fmaxf(vmax, scaled ? x[i] * invT : x[i]);
  const float mx = block_max(vmax, red);
  float s = 0.f;
  #pragma unroll 8
  for (int i = t; i < vocab; i += nt) s += expf((scaled ? x[i] * invT : x[i]) - mx);
  const float inv_sum = 1.0f / block_sum(s, red);

  // the k-th largest of the threads' largest probabilities (a thread without an element holds -1)
  const float lm = vmax == -INFINITY ? -1.f : expf(vmax - mx) * inv_sum;
  a_p[t] = lm;
  if (t == 0) {
    s_count = 0;
    s_win = 0x7fffffff;
  }
  __syncthreads();
  int rank = 0;
  for (int j = 0; j < nt; ++j) {
    const float o = a_p[j];
    rank += (o > lm || (o == lm && j < t)) ? 1 : 0;
  }
  if (rank == (k > 0 ? k : kFastMaxK) - 1) s_bound = lm;   // ranks are a permutation: one thread has this one
  __syncthreads();
  const float bound = s_bound;
  #pragma unroll 8
  for (int i = t; i < vocab; i += nt) {
    const float p = expf((scaled ? x[i] * invT : x[i]) - mx) * inv_sum;
    if (p >= bound) {
      const int slot = atomicAdd(&s_count, 1);
      if (slot < kSampThreads) {
        b_p[slot] = p;
        b_i[slot] = i;
      }
    }
  }
  __syncthreads();
  const int c = s_count;
  if (c > kSampThreads || c > nt) return false;

  // top-k with ties: an entry stays if fewer than k entries are strictly larger
  const bool have = t < c;
  const float p0 = have ? b_p[t] : -1.f;
  const int idx = have ? b_i[t] : 0x7fffffff;
  int larger = 0;
  for (int j = 0; j < c; ++j) larger += b_p[j] > p0 ? 1 : 0;
  const bool kept = have && (k > 0 ? larger < k : true);
  a_i[t] = kept ? idx : 0x7fffffff;
  __syncthreads();
  // in ascending index order: a_p / a_i [0, n)
  int pos = 0, n = 0;
  for (int j = 0; j < c; ++j) {
    const int o = a_i[j];
    pos += o < idx ? 1 : 0;
    n += o != 0x7fffffff ? 1 : 0;
  }
  __syncthreads();
  if (kept) {
    a_p[pos] = p0;
    a_i[pos] = idx;
  }
  __syncthreads();
  const bool mine = t < n;
  float q = mine ? a_p[t] : 0.f;
  float total = 0.f;
  for (int j = 0; j < n; ++j) total += a_p[j];
  if (k > 0 && total > 0.f && total != 1.0f) q *= 1.0f / total;   // top-k renormalises; without it nothing has gone
  b_p[t] = q;
  __syncthreads();
  float pm = 0.f;
  for (int j = 0; j < n; ++j) pm = fmaxf(pm, b_p[j]);
  if (mp > 0.f) {
    if (q < mp * pm) q = 0.f;
    __syncthreads();
    b_p[t] = q;
    __syncthreads();
  }
  if (k <= 0) {
    // what was not gathered lies below the bound: it is out if min-p cuts there or higher, or if the
    // gathered entries alone reach top_p (then the descending sum stops among them)
    float held = 0.f;
    for (int j = 0; j < n; ++j) held += b_p[j];
    const bool shown = (mp > 0.f && mp * pm >= bound) || (tp > 0.f && tp < 1.0f && held >= tp);
    if (!shown) return false;
  }
  if (tp > 0.f && tp < 1.0f) {
    // the descending running sum reaches top_p at some value: an entry stays if what is strictly
    // larger than it has not reached top_p yet
    float above = 0.f;
    for (int j = 0; j < n; ++j) {
      const float o = b_p[j];
      above += o > q ? o : 0.f;
    }
    if (!(above < tp)) q = 0.f;
    __syncthreads();
    b_p[t] = q;
    __syncthreads();
  }
  total = 0.f;
  for (int j = 0; j < n; ++j) total += b_p[j];
  const float inv = (total > 0.f && total != 1.0f) ? 1.0f / total : 1.0f;
  const bool rescale = total > 0.f && total != 1.0f;
  if (mine) {
    float run = 0.f;
    for (int j = 0; j <= t; ++j) run += rescale ? b_p[j] * inv : b_p[j];
    if (u <= run) atomicMin(&s_win, t);
  }
  __syncthreads();
  // (a uniform of exactly 0 is reached by the running sum at index 0 already, whatever lies there)
  if (t == 0) *out_r = u <= 0.f ? 0 : s_win < n ? a_i[s_win] : vocab - 1;
  return true;
}

// Rows without any filter: token i has probability e_i / S with e_i = exp(v_i - max), so the first
// index whose running sum of e reaches u * S is the one whose running sum of e / S reaches u.
// No probability is written: one pass for the maximum, one in which every thread adds up its
// contiguous piece of the row, and the thread whose piece holds the target walks it once more.
// S is the running sum at the last entry, so the target (u < 1) always lies inside the row.
__device__ __forceinline__ void sample_unfiltered(const float* __restrict__ x, int vocab, float T, float u,
                                                  int* __restrict__ out_r, float* red) {
  __shared__ double piece[kSampThreads];
  const int t = threadIdx.x;
  const int nt = blockDim.x;
  const float invT = 1.0f / T;
  const bool scaled = T != 1.0f;
  float vmax = -INFINITY;
#pragma unroll 8
  for (int i = t; i < vocab; i += nt) vmax = fmaxf(vmax, scaled ? x[i] * invT : x[i]);
  const float mx = block_max(vmax, red);
  const int chunk = (vocab + nt - 1) / nt;
  const int b = min(t * chunk, vocab), e = min(b + chunk, vocab);
  double cs = 0.0;   // the running sums are kept in double: where the target falls is then decided by the
                     // terms themselves, not by the rounding of sums of thousands of them
#pragma unroll 4
  for (int i = b; i < e; ++i) cs += (double)expf((scaled ? x[i] * invT : x[i]) - mx);
  piece[t] = cs;
  __syncthreads();
  // running sums before and after this thread's piece, and the whole, each added up in the same
  // ascending order by every thread that needs them
  double before = 0.0, total = 0.0;
  for (int j = 0; j < nt; ++j) {
    if (j == t) before = total;
    total += piece[j];
  }
  const double target = (double)u * total;
  if (u <= 0.f) {
    if (t == 0) *out_r = 0;   // a uniform of exactly 0 is reached at index 0 already
    return;
  }
  // exactly one piece has before < target <= before + piece (the sums are the same numbers in every thread)
  if (b < e && before < target && target <= before + cs) {
    double run = before;
    int pick = e - 1;
    for (int i = b; i < e; ++i) {
      run += (double)expf((scaled ? x[i] * invT : x[i]) - mx);
      if (target <= run) {
        pick = i;
        break;
      }
    }
    *out_r = pick;
  }
}

__global__ __launch_bounds__(kSampThreads) void sample_rows_kernel(
    const float* __restrict__ logits, float* __restrict__ probs, const float* __restrict__ temperature,
    const float* __restrict__ uniform, const int* __restrict__ top_k, const float* __restrict__ top_p,
    const float* __restrict__ min_p, int* __restrict__ out, int vocab) {
  __shared__ float red[16];
  __shared__ int red_i[16];
  __shared__ float chunk_prefix[kSampThreads];
  __shared__ int winner;
  const int r = blockIdx.x;
  const float* x = logits + (size_t)r * vocab;
  float* p = probs + (size_t)r * vocab;
  const float T = temperature[r];
  const float invT = 1.0f / T;
  const int k = top_k ? top_k[r] : 0;
  const float tp0 = top_p ? top_p[r] : 1.0f, mp0 = min_p ? min_p[r] : 0.f;
  if ((k <= 0 || k >= vocab) && mp0 <= 0.f && !(tp0 > 0.f && tp0 < 1.0f)) {
    sample_unfiltered(x, vocab, T, uniform[r], out + r, red);
    return;
  }
  if ((k > 0 && k <= kFastMaxK && k < vocab) ||
      (k <= 0 && vocab > kFastMaxK && (mp0 > 0.f || (tp0 > 0.f && tp0 < 1.0f)))) {
    if (sample_few_survivors(x, vocab, T, k, min_p ? min_p[r] : 0.f, top_p ? top_p[r] : 1.0f, uniform[r], out + r, red))
      return;
  }

  // softmax(logits / T)
  float mx = -INFINITY;
  #pragma unroll 8
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = (T != 1.0f) ? x[i] * invT : x[i];
    p[i] = v;
    mx = fmaxf(mx, v);
  }
  mx = block_max(mx, red);
  float s = 0.f;
  #pragma unroll 8
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float e = expf(p[i] - mx);
    p[i] = e;
    s += e;
  }
  const float inv_sum = 1.0f / block_sum(s, red);
  #pragma unroll 8
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) p[i] *= inv_sum;
  __syncthreads();

  // top-k: largest threshold whose count of p >= threshold is still >= k
  if (k > 0 && k < vocab) {
    uint32_t lo = 0u, hi = 0x7f800000u;  // invariant: count(>= lo) >= k, count(>= hi + 1) < k
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo + 1) / 2;
      int c;
      float sm;
      count_sum_ge(p, vocab, mid, red, red_i, c, sm);
      if (c >= k) lo = mid; else hi = mid - 1;
    }
    #pragma unroll 8
    for (int i = threadIdx.x; i < vocab; i += blockDim.x)
      if (__float_as_uint(p[i]) < lo) p[i] = 0.f;
    __syncthreads();
    renormalise(p, vocab, red);
  }
  // min-p
  const float mp = min_p ? min_p[r] : 0.f;
  if (mp > 0.f) {
    float pm = 0.f;
    #pragma unroll 8
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) pm = fmaxf(pm, p[i]);
    pm = block_max(pm, red);
    const float thr = mp * pm;
    #pragma unroll 8
    for (int i = threadIdx.x; i < vocab; i += blockDim.x)
      if (p[i] < thr) p[i] = 0.f;
    __syncthreads();
  }
  // top-p: largest threshold whose sum of p >= threshold still reaches top_p
  const float tp = top_p ? top_p[r] : 1.0f;
  if (tp > 0.f && tp < 1.0f) {
    uint32_t lo = 1u, hi = 0x7f800000u;  // bits 1 = smallest positive: keeps every non-zero entry
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo + 1) / 2;
      int c;
      float sm;
      count_sum_ge(p, vocab, mid, red, red_i, c, sm);
      if (sm >= tp) lo = mid; else hi = mid - 1;
    }
    #pragma unroll 8
    for (int i = threadIdx.x; i < vocab; i += blockDim.x)
      if (__float_as_uint(p[i]) < lo) p[i] = 0.f;
    __syncthreads();
  }
  renormalise(p, vocab, red);

  // inverse CDF: contiguous chunk per thread, ascending index
  const int chunk = (vocab + blockDim.x - 1) / blockDim.x;
  const int b = threadIdx.x * chunk;
  const int e = min(b + chunk, vocab);
  float cs = 0.f;
  for (int i = b; i < e; ++i) cs += p[i];
  chunk_prefix[threadIdx.x] = cs;
  if (threadIdx.x == 0) winner = 0x7fffffff;
  __syncthreads();
  if (threadIdx.x == 0) {
    float run = 0.f;
    for (int i = 0; i < (int)blockDim.x; ++i) {
      const float c = chunk_prefix[i];
      chunk_prefix[i] = run;
      run += c;
    }
  }
  __syncthreads();
  const float u = uniform[r];
  float run = chunk_prefix[threadIdx.x];
  for (int i = b; i < e; ++i) {
    run += p[i];
    if (u <= run) {
      atomicMin(&winner, i);
      break;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) out[r] = winner == 0x7fffffff ? vocab - 1 : winner;
}

SHARPI_EXPORT int sharpi_sample_rows(const float* logits, float* probs, const float* temperature,
                                     const float* uniform, const int* top_k, const float* top_p,
                                     const float* min_p, int* out, int rows, int vocab, hipStream_t stream) {
  if (rows <= 0) return SHARPI_OK;
  if (vocab <= 0) return SHARPI_ERR_ARG;
  sample_rows_kernel<<<rows, kSampThreads, 0, stream>>>(logits, probs, temperature, uniform, top_k, top_p, min_p,
                                                        out, vocab);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// Sparse logit edits before sampling (repetition / frequency / presence penalties, additive bias):
// for entry i of row r (entries [row_offsets[r], row_offsets[r+1])): id = ids[i]
//   x = logits[r, id]; if rep != 1: x = x > 0 ? x / rep : x * rep; x -= counts[i] * freq + pres (if count > 0);
//   x += bias[i]
__global__ void edit_logits_kernel(float* __restrict__ logits, const int* __restrict__ row_offsets,
                                   const int* __restrict__ ids, const int* __restrict__ counts,
                                   const float* __restrict__ bias, const float* __restrict__ rep,
                                   const float* __restrict__ freq, const float* __restrict__ pres, int vocab) {
  const int r = blockIdx.x;
  float* x = logits + (size_t)r * vocab;
  for (int i = row_offsets[r] + threadIdx.x; i < row_offsets[r + 1]; i += blockDim.x) {
    const int id = ids[i];
    if (id < 0 || id >= vocab) continue;
    float v = x[id] + bias[i];
    const int c = counts[i];
    if (c > 0) {
      const float rp = rep[r];
      if (rp != 1.0f) v = v > 0.f ? v / rp : v * rp;
      v -= (float)c * freq[r] + pres[r];
    }
    x[id] = v;
  }
}

SHARPI_EXPORT int sharpi_edit_logits(float* logits, const int* row_offsets, const int* ids, const int* counts,
                                     const float* bias, const float* rep, const float* freq, const float* pres,
                                     int rows, int vocab, hipStream_t stream) {
  if (rows <= 0) return SHARPI_OK;
  if (vocab <= 0) return SHARPI_ERR_ARG;
  edit_logits_kernel<<<rows, 256, 0, stream>>>(logits, row_offsets, ids, counts, bias, rep, freq, pres, vocab);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
