// Position encoding, weightless per-head norm, query temperature and the cache write, one kernel.
//
// Input  qkv [T, (nh + nkv) * hd + nkv * vd]: q heads, then k heads (hd wide), then v heads (vd wide,
// usually hd) of each token; an optional bias of the row's width (float) is added to every
// token's row first, in float.
// q head : rotate (if inv_freq) -> norm (if qk_norm) -> * temperature (if temp_tuning) -> q_out
// k head : rotate (if inv_freq) -> norm (if qk_norm) -> cache K at slot_mapping[t]
// v head : cache V at slot_mapping[t]
// Rotation is on the first rotary_dim elements of a head (the rest pass through unrotated), in
// pairs (2i, 2i+1) (interleaved) or (i, i + rotary_dim/2) (half-split), with
// angle = float(pos) * inv_freq[i], i < rotary_dim/2, all in float.  The norm runs over the whole head.
// Cache layout of one layer: keys [page][kv head][page_size][hd], values transposed inside the page,
// [page][kv head][hd][page_size] (so that the matrix-core kernels read runs of keys for one
// value column); slot = page * page_size + offset;
// a negative slot means "do not store" (the layer reads another layer's cache).
#include "common.h"

template <typename T>
__global__ void rope_kv_kernel(const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_cache,
                               T* __restrict__ v_cache, const int* __restrict__ slot_mapping,
                               const int* __restrict__ positions, const float* __restrict__ inv_freq,
                               const float* __restrict__ bias,
                               int qk_norm, float eps, int temp_tuning, float floor_scale, float attn_scale,
                               int nh, int nkv, int hd, int vd, int page_size, int half_split, int rotary_dim) {
  const int t = blockIdx.x;
  const int head = blockIdx.y;            // 0..nh-1 q, nh..nh+nkv-1 k, then v
  const int lane = threadIdx.x;           // one wave
  const int half = hd >> 1;
  const size_t row_width = (size_t)(nh + nkv) * hd + (size_t)nkv * vd;
  const size_t head_at = head < nh + nkv ? (size_t)head * hd : (size_t)(nh + nkv) * hd + (size_t)(head - nh - nkv) * vd;
  const T* src = qkv + (size_t)t * row_width + head_at;
  const float* hb = bias ? bias + head_at : nullptr;
  const int pos = positions[t];
  const bool is_q = head < nh;
  const bool is_k = !is_q && head < nh + nkv;
  const int slot = slot_mapping[t];

  if (!is_q && !is_k) {  // v: plain copy into the cache
    if (slot < 0) return;
    const int kvh = head - nh - nkv;
    T* dst = v_cache + ((size_t)(slot / page_size) * nkv + kvh) * vd * page_size + (slot % page_size);
    for (int d = lane; d < vd; d += kWave)
      dst[(size_t)d * page_size] = hb ? from_f32<T>(to_f32<T>(src[d]) + hb[d]) : src[d];
    return;
  }
  if (is_k && slot < 0) return;

  // pairs handled by this lane: i = lane, lane + 64, ... (hd <= 512).  Pair i < rotary_dim/2 is a
  // rotary pair, at elements (2i, 2i+1) or (i, i + rotary_dim/2); the pairs after them are the
  // neighbouring elements of the unrotated rest.
  const int rot_pairs = rotary_dim >> 1;
  float x0[4], x1[4];
  int e0[4], e1[4];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = lane + j * kWave;
    x0[j] = 0.f;
    x1[j] = 0.f;
    e0[j] = e1[j] = 0;
    if (i < half) {
      if (i >= rot_pairs) {
        e0[j] = 2 * i;
        e1[j] = 2 * i + 1;
      } else if (half_split) {
        e0[j] = i;
        e1[j] = i + rot_pairs;
      } else {
        e0[j] = 2 * i;
        e1[j] = 2 * i + 1;
      }
      float a = to_f32<T>(src[e0[j]]);
      float b = to_f32<T>(src[e1[j]]);
      if (hb) {
        a += hb[e0[j]];
        b += hb[e1[j]];
      }
      if (inv_freq && i < rot_pairs) {
        const float ang = (float)pos * inv_freq[i];
        const float c = cosf(ang);
        const float s = sinf(ang);
        const float ra = a * c - b * s;
        const float rb = a * s + b * c;
        a = ra;
        b = rb;
      }
      x0[j] = a;
      x1[j] = b;
      ss += a * a + b * b;
    }
  }
  float mul = 1.0f;
  if (qk_norm) {
    const float total = wave_sum(ss);
    mul = 1.0f / sqrtf(total / (float)hd + eps);
  }
  float post = 1.0f;
  if (is_q && temp_tuning) {
    post = 1.0f + attn_scale * logf(floorf(((float)pos + 1.0f) / floor_scale) + 1.0f);
  }
  T* dst;
  if (is_q) {
    dst = q_out + ((size_t)t * nh + head) * hd;
  } else {
    const int kvh = head - nh;
    dst = k_cache + (((size_t)(slot / page_size) * nkv + kvh) * page_size + (slot % page_size)) * hd;
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = lane + j * kWave;
    if (i < half) {
      float a = x0[j], b = x1[j];
      if (qk_norm) {
        a *= mul;
        b *= mul;
      }
      if (is_q && temp_tuning) {
        a *= post;
        b *= post;
      }
      dst[e0[j]] = from_f32<T>(a);
      dst[e1[j]] = from_f32<T>(b);
    }
  }
}

// The same for head sizes 32, 64, 128, 256 with interleaved pairs and a rotary width that is a
// multiple of 8 (runs beyond it pass through): a thread per run of 8 elements (4 rotary pairs),
// 16-byte accesses; the hd/8 lanes of a head are neighbours in a wave and sum their squares with
// shuffles.  Blocks (token, y) share a token's heads between them, 256 runs each, so that a
// handful of decode tokens still spreads over many compute units.
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_vec_kernel(
    const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int* __restrict__ slot_mapping, const int* __restrict__ positions, const float* __restrict__ inv_freq,
    const float* __restrict__ bias, int qk_norm, float eps, int temp_tuning, float floor_scale, float attn_scale,
    int nh, int nkv, int hd, int page_size, int rotary_dim) {
  const int t = blockIdx.x;
  const int per_head = hd >> 3;                    // lanes per head: 4, 8, 16 or 32
  const int chunks = (nh + 2 * nkv) * per_head;
  const int pos = positions[t];
  const int slot = slot_mapping[t];
  const T* src = qkv + (size_t)t * (nh + 2 * nkv) * hd;
  float post = 1.0f;
  if (temp_tuning) post = 1.0f + attn_scale * logf(floorf(((float)pos + 1.0f) / floor_scale) + 1.0f);
  // a thread's run within a head is the same in every turn of the loop (the block size is a multiple
  // of the lanes per head), and so are its four angles: their sines and cosines are computed once
  const int run = threadIdx.x % per_head;
  float cs[4], sn[4];
  const bool rotates = inv_freq != nullptr && run * 8 < rotary_dim;
  if (rotates) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float ang = (float)pos * inv_freq[run * 4 + j];
      cs[j] = cosf(ang);
      sn[j] = sinf(ang);
    }
  }
  for (int base = blockIdx.y * blockDim.x; base < chunks; base += gridDim.y * blockDim.x) {
    const int ci = base + threadIdx.x;
    const bool valid = ci < chunks;
    const int head = valid ? ci / per_head : 0;
    const bool is_q = head < nh;
    const bool is_k = !is_q && head < nh + nkv;
    float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (valid) {
      load8(src + (size_t)head * hd + run * 8, x);
      if (bias) {
        float b8[8];
        load8(bias + (size_t)head * hd + run * 8, b8);
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] += b8[j];
      }
    }
    float ss = 0.f;
    if (valid && (is_q || is_k)) {
      if (rotates) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float a = x[2 * j], b = x[2 * j + 1];
          x[2 * j] = a * cs[j] - b * sn[j];
          x[2 * j + 1] = a * sn[j] + b * cs[j];
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += x[j] * x[j];
    }
    if (qk_norm) {   // every lane takes part in the shuffles
      for (int off = per_head >> 1; off > 0; off >>= 1) ss += __shfl_xor(ss, off, kWave);
      const float mul = 1.0f / sqrtf(ss / (float)hd + eps);
      if (is_q || is_k) {
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] *= mul;
      }
    }
    if (!valid) continue;
    if (is_q) {
      if (temp_tuning) {
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] *= post;
      }
      store8(q_out + ((size_t)t * nh + head) * hd + run * 8, x);
    } else if (slot >= 0) {
      const size_t page = (size_t)(slot / page_size);
      const int off = slot % page_size;
      if (is_k) {
        store8(k_cache + ((page * nkv + (head - nh)) * page_size + off) * hd + run * 8, x);
      } else {
        T* dst = v_cache + (page * nkv + (head - nh - nkv)) * hd * page_size + off;
#pragma unroll
        for (int j = 0; j < 8; ++j) dst[(size_t)(run * 8 + j) * page_size] = from_f32<T>(x[j]);
      }
    }
  }
}

SHARPI_EXPORT int sharpi_rope_kv(const void* qkv, void* q_out, void* k_cache, void* v_cache, int dtype,
                                 const int* slot_mapping, const int* positions, const float* inv_freq,
                                 const float* bias, int qk_norm, float eps, int temp_tuning, float floor_scale, float attn_scale,
                                 int n_tokens, int nh, int nkv, int hd, int vd, int page_size, int pair_layout,
                                 int rotary_dim, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  // pair_layout: 0 = pairs (2i, 2i+1), 1 = pairs (i, i + rotary_dim/2); rotary_dim even, <= hd
  if (pair_layout < 0 || pair_layout > 1) return SHARPI_ERR_ARG;
  if (inv_freq == nullptr) rotary_dim = 0;
  else if (rotary_dim <= 0 || (rotary_dim & 1) || rotary_dim > hd) return SHARPI_ERR_ARG;
  if (hd <= 0 || (hd & 1) || hd > 512 || vd <= 0 || nh <= 0 || nkv <= 0 || page_size <= 0) return SHARPI_ERR_ARG;
  if (nh + 2 * nkv > 65535) return SHARPI_ERR_ARG;
  if (temp_tuning && !(floor_scale > 0.f)) return SHARPI_ERR_ARG;
  dim3 grid(n_tokens, nh + 2 * nkv), block(kWave);
  if (dtype != DT_F32 && dtype != DT_BF16) return SHARPI_ERR_ARG;
  if ((hd == 32 || hd == 64 || hd == 128 || hd == 256) && vd == hd && pair_layout == 0 && (rotary_dim & 7) == 0) {
    // a few tokens (decode): a token's heads over several blocks, for the compute units' sake;
    // many tokens: one block per token, which then computes its angles once for all heads
    const dim3 vgrid(n_tokens, n_tokens <= 64 ? ceil_div((nh + 2 * nkv) * (hd >> 3), 256) : 1);
    if (dtype == DT_F32)
      rope_kv_vec_kernel<float><<<vgrid, 256, 0, stream>>>((const float*)qkv, (float*)q_out, (float*)k_cache,
                                                             (float*)v_cache, slot_mapping, positions, inv_freq,
                                                             bias, qk_norm, eps, temp_tuning, floor_scale, attn_scale,
                                                             nh, nkv, hd, page_size, rotary_dim);
    else
      rope_kv_vec_kernel<bf16_t><<<vgrid, 256, 0, stream>>>((const bf16_t*)qkv, (bf16_t*)q_out,
                                                              (bf16_t*)k_cache, (bf16_t*)v_cache, slot_mapping,
                                                              positions, inv_freq, bias, qk_norm, eps, temp_tuning,
                                                              floor_scale, attn_scale, nh, nkv, hd, page_size, rotary_dim);
    SHARPI_CHECK_LAUNCH();
    return SHARPI_OK;
  }
  if (dtype == DT_F32)
    rope_kv_kernel<float><<<grid, block, 0, stream>>>((const float*)qkv, (float*)q_out, (float*)k_cache,
                                                     (float*)v_cache, slot_mapping, positions, inv_freq, bias, qk_norm,
                                                     eps, temp_tuning, floor_scale, attn_scale, nh, nkv, hd, vd,
                                                     page_size, pair_layout, rotary_dim);
  else if (dtype == DT_BF16)
    rope_kv_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)qkv, (bf16_t*)q_out, (bf16_t*)k_cache,
                                                      (bf16_t*)v_cache, slot_mapping, positions, inv_freq, bias,
                                                      qk_norm, eps, temp_tuning, floor_scale, attn_scale, nh, nkv,
                                                      hd, vd, page_size, pair_layout, rotary_dim);
  else
    return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
