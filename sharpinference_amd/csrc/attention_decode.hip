// Attention for single-token entries (decode): split-K flash-decode on the matrix cores.
//
// One block = (a run of SPLIT_KEYS keys, one token, one kv head with up to 16 of its query
// heads).  Everything is computed transposed, so that no operand ever has to be re-laid-out:
//   S^T[key, head] = K[key, :] . Q[head, :]      A = K block (16 keys x 32 d), B = Q^T
//   O^T[d, head]  += V^T[d, key] * P^T[key, head] A = V^T block (16 d x 32 keys), B = P^T
// The S^T accumulator of a lane (4 keys of each of two 16-key blocks, one head) is exactly
// the B operand the second product wants, once exponentiated and split into a bfloat16 pair
// (hi + lo, two products, so the probabilities keep ~16 bits); the
// value cache is stored transposed inside a page for the A operand of the second product.
// Keys are walked in 16-key blocks aligned to absolute positions (a block never straddles a
// page); keys before the window's start or after the query are masked.  The four waves take
// 32-key chunks round-robin and meet in LDS; the block leaves (max, sum, unnormalised O) per
// head, and a second kernel merges the runs of a token.  The run length is fixed, so the sums
// of a query depend on (start, position) only, not on the batch.
#include "common.h"
#include "sharpi_noalloc.h"
#include <mutex>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// the head sizes the kernel is compiled for
#define SHARPI_DECODE_HEAD_SIZES(X) X(32) X(64) X(96) X(128) X(160) X(192) X(224) X(256)

#ifndef SHARPI_DEC_PRE2_MAX_HD
#define SHARPI_DEC_PRE2_MAX_HD 128   // head sizes up to this keep two chunks of a wave's keys in flight
#endif
constexpr int kDecWaves = 4;
constexpr int kSplitBlocks = 16;  // 16-key blocks per run: 256 keys

__device__ __forceinline__ __bf16 to_bf16_rne(float f) {
  bf16_t b = f32_to_bf16(f);
  return __builtin_bit_cast(__bf16, b.bits);
}

template <int HD>
__global__ __launch_bounds__(kDecWaves* kWave) void attn_decode_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_table, const int* __restrict__ entry_of_token,
    const int* __restrict__ positions, const int* __restrict__ token_list, float* __restrict__ part_o,
    float* __restrict__ part_ml, int window_kind, int window, float scale, int nh, int nkv, int page_size,
    int max_blocks, int num_pages, int max_splits) {
  constexpr int NJ = HD / 32;  // 32-wide d chunks of the first product
  constexpr int ND = HD / 16;  // 16-row d tiles of the second product
  __shared__ f32x4 acc_s[kDecWaves][ND][kWave];
  __shared__ float m_s[kDecWaves][16];
  __shared__ float l_s[kDecWaves][kWave];

  const int lane = threadIdx.x & (kWave - 1);
  const int w = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  // Blocks are handed out kv head first, then token, then run: the heads of a (token, run) read
  // neighbouring pieces of the same pages at the same time, and the runs that lie beyond a
  // token's keys (the launch is sized for the longest context it may meet) all come last, where
  // they hold nobody up.
  const int sp = blockIdx.z;
  const int li = blockIdx.y;
  const int t = token_list ? token_list[li] : li;
  const int G = nh / nkv;
  const int hgroups = (G + 15) / 16;
  const int kvh = blockIdx.x / hgroups;
  const int h0 = kvh * G + (blockIdx.x % hgroups) * 16;
  const int hcount = min(16, kvh * G + G - h0);

  const int p = positions[t];
  int start = 0;
  if (window_kind == 1) start = (p / window) * window;
  else if (window_kind == 2) start = p - window + 1 > 0 ? p - window + 1 : 0;
  const int b_first = (start >> 4) + sp * kSplitBlocks;
  const int b_last = min(p >> 4, b_first + kSplitBlocks - 1);
  if (b_first > (p >> 4)) return;  // this run lies beyond the query
  const int* bt = block_table + (size_t)entry_of_token[t] * max_blocks;

  // Q^T fragments: lane (head r, group g) holds q[head][j*32 + g*8 .. +8]
  bf16x8 qf[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    // columns beyond the group's heads repeat its last head; they are never stored
    qf[j] = *reinterpret_cast<const bf16x8*>(q + ((size_t)t * nh + h0 + min(r, hcount - 1)) * HD + j * 32 + g * 8);
  }

  float m = -INFINITY, l = 0.f;   // for head r: m identical in the 4 lanes of a column, l a partial sum
  f32x4 acc[ND];
#pragma unroll
  for (int d = 0; d < ND; ++d) acc[d] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Keys and values are read once per step, so with the streaming hint (nontemporal).
  // A wave's chunks of the run are 2 * kDecWaves blocks apart; PRE of them are requested before
  // anything is computed (all of a 256-key run where the registers allow it: the run is then one
  // round trip to memory, not one per chunk).  Every load is unconditional: a block beyond the
  // run's last is fetched as the last one again and masked, so that the compiler's count of
  // outstanding loads stays exact and the first chunk does not wait for the second.
  constexpr int PRE = HD <= SHARPI_DEC_PRE2_MAX_HD ? 2 : 1;
  for (int b0 = b_first + 2 * w; b0 <= b_last; b0 += 2 * kDecWaves * PRE) {
    bf16x8 kf[PRE][2][NJ];
    bf16x4 vq[PRE][2][ND];
#pragma unroll
    for (int it = 0; it < PRE; ++it) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int bb = min(b0 + it * 2 * kDecWaves + u, b_last);
        const int pi = min((bb << 4) / page_size, max_blocks - 1);
        const int page = min(max(bt[pi], 0), num_pages - 1);   // a table that is wrong reads a wrong page, never outside
        const int off = (bb << 4) % page_size;
        const long long kbase = (((long long)page * nkv + kvh) * page_size + off) * HD;
        const long long vbase = ((long long)page * nkv + kvh) * HD * page_size + off;
#pragma unroll
        for (int j = 0; j < NJ; ++j)
          kf[it][u][j] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(k_cache + kbase + (size_t)r * HD + j * 32 + g * 8));
#pragma unroll
        for (int d = 0; d < ND; ++d)   // V^T fragment: lane (d row r, group g) holds keys 4g..4g+3 of the block
          vq[it][u][d] = __builtin_nontemporal_load(reinterpret_cast<const bf16x4*>(v_cache + vbase + (size_t)(d * 16 + r) * page_size + 4 * g));
      }
    }
#pragma unroll
    for (int it = 0; it < PRE; ++it) {
    const int b = b0 + it * 2 * kDecWaves;
    if (b > b_last) break;   // wave-uniform
    f32x4 s[2];
    bool have[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) have[u] = b + u <= b_last;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      s[u] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < NJ; ++j) s[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[it][u][j], qf[j], s[u], 0, 0, 0);
    }
    // lane holds S^T[key = 16*(b+u) + 4g + i][head r]
    float cm = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = ((b + u) << 4) + 4 * g + i;
        const bool ok = have[u] && key >= start && key <= p;
        s[u][i] = ok ? s[u][i] * scale : -INFINITY;
        cm = fmaxf(cm, s[u][i]);
      }
    cm = fmaxf(cm, __shfl_xor(cm, 16, kWave));
    cm = fmaxf(cm, __shfl_xor(cm, 32, kWave));
    const float m_new = fmaxf(m, cm);
    float corr = 1.0f;
    bf16x8 pf, pf_lo;   // probabilities as a bfloat16 pair hi + lo: ~16 bits survive the product
    if (m_new == -INFINITY) {
      pf = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      pf_lo = pf;
    } else {
      corr = expf(m - m_new);  // m = -inf gives 0
      float ls = 0.f;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float e = expf(s[u][i] - m_new);  // masked: exp(-inf) = 0
          ls += e;
          const bf16_t hi = f32_to_bf16(e);
          pf[u * 4 + i] = __builtin_bit_cast(__bf16, hi.bits);
          pf_lo[u * 4 + i] = to_bf16_rne(e - bf16_to_f32(hi));
        }
      l = l * corr + ls;
      m = m_new;
    }
#pragma unroll
    for (int d = 0; d < ND; ++d) {
      // keys 4g..4g+3 of block b, then of block b + 1
      const bf16x8 vf = __builtin_shufflevector(vq[it][0][d], vq[it][1][d], 0, 1, 2, 3, 4, 5, 6, 7);
      acc[d] *= corr;   // corr belongs to head r = the accumulator's column
      acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, acc[d], 0, 0, 0);
      acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf_lo, acc[d], 0, 0, 0);
    }
    }
  }

  // meet in LDS: per head, the four waves' (m, l, O)
  if (g == 0) m_s[w][r] = m;
  l_s[w][lane] = l;
#pragma unroll
  for (int d = 0; d < ND; ++d) acc_s[w][d][lane] = acc[d];
  __syncthreads();
  if (w != 0) return;
  float M = m_s[0][r];
#pragma unroll
  for (int ww = 1; ww < kDecWaves; ++ww) M = fmaxf(M, m_s[ww][r]);
  float f[kDecWaves];
  float L = 0.f;
#pragma unroll
  for (int ww = 0; ww < kDecWaves; ++ww) {
    f[ww] = m_s[ww][r] == -INFINITY ? 0.f : expf(m_s[ww][r] - M);
    const float lw = l_s[ww][r] + l_s[ww][r + 16] + l_s[ww][r + 32] + l_s[ww][r + 48];
    L += f[ww] * lw;
  }
  if (r >= hcount) return;
  const size_t slot = ((size_t)li * nh + h0 + r) * max_splits + sp;
  if (g == 0) {
    part_ml[slot * 2] = M;
    part_ml[slot * 2 + 1] = L;
  }
#pragma unroll
  for (int d = 0; d < ND; ++d) {
    f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ww = 0; ww < kDecWaves; ++ww) o += acc_s[ww][d][lane] * f[ww];
    // lane holds O^T[d*16 + 4g + i][head r]
    *reinterpret_cast<f32x4*>(part_o + slot * HD + d * 16 + 4 * g) = o;
  }
}

// merge the runs of one (token, head): out = sum_s O_s e^(m_s - M) / sum_s l_s e^(m_s - M).
// A block's threads are (run lane, 4-wide column of d): the run lanes walk the runs side by side
// with independent loads and meet in LDS, in an order that depends on the number of runs only.
constexpr int kMergeThreads = 256;

__global__ __launch_bounds__(kMergeThreads) void attn_decode_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ positions,
    const int* __restrict__ token_list, bf16_t* __restrict__ out, int window_kind, int window, int nh, int hd,
    int max_splits) {
  __shared__ float red_s[kMergeThreads / kWave];
  __shared__ f32x4 o_s[kMergeThreads];
  __shared__ float l_s[kMergeThreads];
  const int li = blockIdx.x;
  const int h = blockIdx.y;
  const int t = token_list ? token_list[li] : li;
  const int p = positions[t];
  int start = 0;
  if (window_kind == 1) start = (p / window) * window;
  else if (window_kind == 2) start = p - window + 1 > 0 ? p - window + 1 : 0;
  // Never beyond the runs the workspace holds, whatever the caller's bound was; but a bound too
  // small for this token (its nearest keys would be dropped without a trace) gives a row of NaN,
  // which no caller can take for attention.
  const int runs_wanted = ((p >> 4) - (start >> 4)) / kSplitBlocks + 1;
  const int n_runs = min(runs_wanted, max_splits);
  const size_t base = ((size_t)li * nh + h) * max_splits;

  float M = -INFINITY;
  for (int s = threadIdx.x; s < n_runs; s += kMergeThreads) M = fmaxf(M, part_ml[(base + s) * 2]);
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o, kWave));
  if ((threadIdx.x & (kWave - 1)) == 0) red_s[threadIdx.x >> 6] = M;
  __syncthreads();
  M = red_s[0];
#pragma unroll
  for (int ww = 1; ww < kMergeThreads / kWave; ++ww) M = fmaxf(M, red_s[ww]);

  const int ncol = hd >> 2;                      // 4-wide columns of a head
  const int lanes = kMergeThreads / ncol;        // run lanes (hd <= 256: at least 4)
  const int col = threadIdx.x % ncol, rl = threadIdx.x / ncol;
  f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
  float L = 0.f;
  if (rl < lanes) {
    for (int s = rl; s < n_runs; s += lanes) {
      const float ms = part_ml[(base + s) * 2];
      const float f = ms == -INFINITY ? 0.f : expf(ms - M);
      const f32x4 po = *reinterpret_cast<const f32x4*>(part_o + (base + s) * hd + col * 4);
      L += part_ml[(base + s) * 2 + 1] * f;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] += f > 0.f ? po[i] * f : 0.f;
    }
  }
  o_s[threadIdx.x] = o;
  l_s[threadIdx.x] = L;
  __syncthreads();
  if (rl != 0) return;
  for (int x = 1; x < lanes; ++x) {
    o += o_s[x * ncol + col];
    L += l_s[x * ncol + col];
  }
  unsigned short b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) b[i] = runs_wanted > max_splits ? (unsigned short)0x7fc0 : f32_to_bf16(L > 0.f ? o[i] / L : 0.f).bits;
  uint2 pk;
  pk.x = b[0] | ((unsigned)b[1] << 16);
  pk.y = b[2] | ((unsigned)b[3] << 16);
  *reinterpret_cast<uint2*>(out + ((size_t)t * nh + h) * hd + col * 4) = pk;
}

template <int HD>
static int launch_decode(const void* q, const void* k_cache, const void* v_cache, const int* block_table,
                         const int* entry_of_token, const int* positions, const int* token_list, float* part_o,
                         float* part_ml, void* out, int window_kind, int window, float scale, int n_list, int nh,
                         int nkv, int page_size, int max_blocks, int num_pages, int max_splits, hipStream_t stream) {
  const int G = nh / nkv;
  dim3 grid(nkv * ((G + 15) / 16), n_list, max_splits), block(kDecWaves * kWave);
  attn_decode_kernel<HD><<<grid, block, 0, stream>>>((const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache,
                                                    block_table, entry_of_token, positions, token_list, part_o,
                                                    part_ml, window_kind, window, scale, nh, nkv, page_size,
                                                    max_blocks, num_pages, max_splits);
  SHARPI_CHECK_LAUNCH();
  dim3 mgrid(n_list, nh), mblock(kMergeThreads);
  attn_decode_merge_kernel<<<mgrid, mblock, 0, stream>>>(part_o, part_ml, positions, token_list, (bf16_t*)out,
                                                         window_kind, window, nh, HD, max_splits);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// q [T, nh, hd] bf16; caches K [pages, nkv, page_size, hd], V [pages, nkv, hd, page_size] bf16;
// token_list [n_list] (or null: tokens 0..n_list-1); part_o float [n_list, nh, max_splits, hd];
// part_ml float [n_list, nh, max_splits, 2]; out [T, nh, hd] bf16 (rows of the listed tokens).
// max_splits must cover every listed token: ((position >> 4) - (first visible key >> 4)) / 16 + 1
// runs of 256 keys (runs are aligned to absolute positions, so a window that starts inside a run
// takes one more than its length suggests); ((context - 1) >> 4) / 16 + 1 covers every window of a
// context.  A token whose runs exceed max_splits gets a row of NaN.
SHARPI_EXPORT int sharpi_attention_decode(const void* q, const void* k_cache, const void* v_cache,
                                          const int* block_table, const int* entry_of_token, const int* positions,
                                          const int* token_list, float* part_o, float* part_ml, void* out,
                                          int window_kind, int window, float scale, int n_list, int nh, int nkv,
                                          int hd, int page_size, int max_blocks, int num_pages, int max_splits,
                                          hipStream_t stream) {
  if (n_list <= 0) return SHARPI_OK;
  if (nh <= 0 || nkv <= 0 || nh % nkv != 0 || nh > 65535 || n_list > 65535) return SHARPI_ERR_ARG;
  if (page_size <= 0 || page_size % 16 != 0 || max_blocks <= 0 || num_pages <= 0 || max_splits <= 0 || max_splits > 65535) return SHARPI_ERR_ARG;
  if (window_kind < 0 || window_kind > 2 || (window_kind != 0 && window <= 0)) return SHARPI_ERR_ARG;
  if (nkv * ((nh / nkv + 15) / 16) > 65535) return SHARPI_ERR_ARG;
#define DEC(HDV)                                                                                                  \
  if (hd == HDV)                                                                                                  \
    return launch_decode<HDV>(q, k_cache, v_cache, block_table, entry_of_token, positions, token_list, part_o,    \
                              part_ml, out, window_kind, window, scale, n_list, nh, nkv, page_size, max_blocks,   \
                              num_pages, max_splits, stream);
  SHARPI_DECODE_HEAD_SIZES(DEC)
#undef DEC
  return SHARPI_ERR_ARG;  // other head sizes go to the generic kernel
}

// 1 if the kernel is compiled for this head size (the caller's choice of kernel asks here).
SHARPI_EXPORT int sharpi_attention_decode_takes(int hd) {
#define DEC(HDV) if (hd == HDV) return 1;
  SHARPI_DECODE_HEAD_SIZES(DEC)
#undef DEC
  return 0;
}

SHARPI_EXPORT int sharpi_attention_decode_split_keys() { return kSplitBlocks * 16; }

// ---------------------------------------------------------------------------------------------
// The same without workspace arguments, for callers that cannot allocate: the partial results go
// to a file-scope device array.  In host code the array's name is only a stand-in for the symbol,
// not a device address; each device's address is looked up once, with that device current, and
// that pointer is what the kernels get.
static __device__ __align__(256) float scratch[SHARPI_NOALLOC_SCRATCH_FLOATS];

constexpr int kMaxDevices = 64;
static float* scratch_of_device[kMaxDevices];   // per device: where its copy of `scratch` lies
static std::mutex scratch_lock;

static int scratch_here(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return SHARPI_ERR_ARG;
  std::lock_guard<std::mutex> guard(scratch_lock);
  if (!scratch_of_device[dev]) {
    float* p = nullptr;
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return SHARPI_ERR_LAUNCH;
    scratch_of_device[dev] = p;
  }
  *out = scratch_of_device[dev];
  return SHARPI_OK;
}

int sharpi_attention_decode_noalloc(const void* q, const void* k_cache, const void* v_cache, const int* block_table,
                                    const int* entry_of_token, const int* positions, const int* token_list, void* out,
                                    int window_kind, int window, float scale, int n_list, int nh, int nkv, int hd,
                                    int page_size, int max_blocks, int num_pages, int max_splits, hipStream_t stream) {
  if (n_list <= 0) return SHARPI_OK;
  if (nh <= 0 || hd <= 0 || max_splits <= 0) return SHARPI_ERR_ARG;
  // part_o [n_list, nh, max_splits, hd] then part_ml [n_list, nh, max_splits, 2]
  const unsigned long long runs = (unsigned long long)n_list * (unsigned long long)nh * (unsigned long long)max_splits;
  if (runs * (unsigned long long)(hd + 2) > (unsigned long long)SHARPI_NOALLOC_SCRATCH_FLOATS) return SHARPI_ERR_ARG;
  float* ws = nullptr;
  const int rc = scratch_here(&ws);
  if (rc != SHARPI_OK) return rc;
  float* part_o = ws;
  float* part_ml = ws + runs * (unsigned long long)hd;   // hd is a multiple of 32: stays 16-byte aligned
  return sharpi_attention_decode(q, k_cache, v_cache, block_table, entry_of_token, positions, token_list, part_o,
                                 part_ml, out, window_kind, window, scale, n_list, nh, nkv, hd, page_size, max_blocks,
                                 num_pages, max_splits, stream);
}
