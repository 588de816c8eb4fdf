// Attention over the paged cache, one block per (token, head), float arithmetic throughout.
//
// This is the reference-grade kernel: it serves the 32-bit path for every size and stands in
// for the tiled kernels on sizes they refuse.  The keys of a query at position p are
// [start, p] with start = 0 (all keys), floor(p / W) * W (chunk-local) or max(0, p - W + 1)
// (sliding).  Keys are visited in blocks of 64 dealt round-robin to the block's four waves, so
// the order of every sum depends on (start, p) alone: not on how the tokens were batched.
// Values may have another width than keys (vd): q and keys are hd wide, values and the output vd.
#include "common.h"

constexpr int kAttnWaves = 4;
constexpr int kAttnMaxHd = 256;

template <typename T>
__global__ __launch_bounds__(kAttnWaves* kWave) void attn_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, const int* __restrict__ entry_of_token,
    const int* __restrict__ positions, T* __restrict__ out, int window_kind, int window, float scale, int nh,
    int nkv, int hd, int vd, int page_size, int max_blocks, int num_pages) {
  __shared__ float qs[kAttnMaxHd];
  __shared__ float pw[kAttnWaves][kWave];
  __shared__ int vrow[kAttnWaves][kWave];
  __shared__ float m_s[kAttnWaves], l_s[kAttnWaves];
  __shared__ float acc_s[kAttnWaves][kAttnMaxHd];

  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x & (kWave - 1);
  const int w = threadIdx.x >> 6;
  const int kvh = h / (nh / nkv);
  const int e = entry_of_token[t];
  const int p = positions[t];
  int start = 0;
  if (window_kind == 1) start = (p / window) * window;
  else if (window_kind == 2) start = p - window + 1 > 0 ? p - window + 1 : 0;
  const int nkeys = p - start + 1;

  const T* qrow = q + ((size_t)t * nh + h) * hd;
  for (int d = threadIdx.x; d < hd; d += blockDim.x) qs[d] = to_f32<T>(qrow[d]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  const int* bt = block_table + (size_t)e * max_blocks;

  for (int kb0 = 0; kb0 * kWave < nkeys; kb0 += kAttnWaves) {
    const int kb = kb0 + w;
    const int key = start + kb * kWave + lane;
    bool valid = key <= p;
    int row = 0;
    float s = -INFINITY;
    if (valid) {
      const int blk = key / page_size;
      const int page = blk < max_blocks ? bt[blk] : -1;
      if (page < 0 || page >= num_pages) {
        valid = false;
      } else {
        row = (page * nkv + kvh) * page_size + (key % page_size);
        const T* kr = k_cache + (size_t)row * hd;
        float dot = 0.f;
        for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], to_f32<T>(kr[d]), dot);
        s = dot * scale;
      }
    }
    const float mb = wave_max(s);
    if (mb > -INFINITY) {  // this wave has at least one key in this round
      const float m_new = fmaxf(m, mb);
      const float pe = valid ? expf(s - m_new) : 0.f;
      const float corr = expf(m - m_new);
      l = l * corr + wave_sum(pe);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] *= corr;
      m = m_new;
      pw[w][lane] = pe;
      vrow[w][lane] = valid ? row : -1;
    } else {
      vrow[w][lane] = -1;
      pw[w][lane] = 0.f;
    }
    __syncthreads();
    if (mb > -INFINITY) {
      for (int j = 0; j < kWave; ++j) {
        const int r = vrow[w][j];
        if (r < 0) continue;
        const float pj = pw[w][j];
        // values are stored transposed inside a page: [page][kv head][vd][page_size]
        const T* vr = v_cache + (size_t)(r / page_size) * vd * page_size + (r % page_size);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int d = lane + i * kWave;
          if (d < vd) acc[i] = fmaf(pj, to_f32<T>(vr[(size_t)d * page_size]), acc[i]);
        }
      }
    }
    __syncthreads();
  }

  if (lane == 0) {
    m_s[w] = m;
    l_s[w] = l;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + i * kWave;
    if (d < vd) acc_s[w][d] = acc[i];
  }
  __syncthreads();
  float M = m_s[0];
  for (int i = 1; i < kAttnWaves; ++i) M = fmaxf(M, m_s[i]);
  float L = 0.f;
  float f[kAttnWaves];
  for (int i = 0; i < kAttnWaves; ++i) {
    f[i] = m_s[i] > -INFINITY ? expf(m_s[i] - M) : 0.f;
    L += l_s[i] * f[i];
  }
  T* orow = out + ((size_t)t * nh + h) * vd;
  for (int d = threadIdx.x; d < vd; d += blockDim.x) {
    float o = 0.f;
    for (int i = 0; i < kAttnWaves; ++i) o += acc_s[i][d] * f[i];
    orow[d] = from_f32<T>(L > 0.f ? o / L : 0.f);
  }
}

SHARPI_EXPORT int sharpi_attention_generic(const void* q, const void* k_cache, const void* v_cache, int dtype,
                                           const int* block_table, const int* entry_of_token,
                                           const int* positions, void* out, int window_kind, int window,
                                           float scale, int n_tokens, int nh, int nkv, int hd, int vd, int page_size,
                                           int max_blocks, int num_pages, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (hd <= 0 || hd > kAttnMaxHd || vd <= 0 || vd > kAttnMaxHd || nh <= 0 || nkv <= 0 || nh % nkv != 0 || nh > 65535) return SHARPI_ERR_ARG;
  if (page_size <= 0 || max_blocks <= 0 || num_pages <= 0) return SHARPI_ERR_ARG;
  if (window_kind < 0 || window_kind > 2 || (window_kind != 0 && window <= 0)) return SHARPI_ERR_ARG;
  dim3 grid(n_tokens, nh), block(kAttnWaves * kWave);
  if (dtype == DT_F32)
    attn_generic_kernel<float><<<grid, block, 0, stream>>>(
        (const float*)q, (const float*)k_cache, (const float*)v_cache, block_table, entry_of_token, positions,
        (float*)out, window_kind, window, scale, nh, nkv, hd, vd, page_size, max_blocks, num_pages);
  else if (dtype == DT_BF16)
    attn_generic_kernel<bf16_t><<<grid, block, 0, stream>>>(
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, entry_of_token, positions,
        (bf16_t*)out, window_kind, window, scale, nh, nkv, hd, vd, page_size, max_blocks, num_pages);
  else
    return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
