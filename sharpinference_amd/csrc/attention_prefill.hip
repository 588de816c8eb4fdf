// Attention for entries of several tokens (prompt portions): flash attention on the matrix cores
// over the paged cache, causal and window masks applied per element.
//
// A wave owns a tile of up to 32 consecutive tokens of one entry and one query head, and walks
// the keys its rows can see in 32-key chunks (two 16-key blocks aligned to absolute positions,
// so a block never straddles a page).  As in the decode kernel everything is transposed:
//   S^T[key, q]  = K[key, :] . Q[q, :]          A = K block, B = Q^T
//   O^T[d, q]   += V^T[d, key] * P^T[key, q]    A = V^T block (values are stored transposed
//                                               inside a page), B = P^T
// and the S^T accumulator of a lane is the B operand of the second product once exponentiated
// and split into a bfloat16 pair hi + lo.  Softmax state (running max and sum per query) is
// float.  The keys of a query are always visited in the same blocks, whatever the portion it
// arrived in, so its sums do not depend on how the prompt was cut.  Waves do not share data:
// there is no LDS and no barrier.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kPreWaves = 4;
constexpr int kQT = 2;            // 16-token column tiles per wave
constexpr int kTileTokens = 16 * kQT;

template <int HD>
__global__ __launch_bounds__(kPreWaves* kWave) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_table, const int* __restrict__ positions, const int* __restrict__ tiles,
    bf16_t* __restrict__ out, int n_tiles, int window_kind, int window, float scale, int nh, int nkv,
    int page_size, int max_blocks, int num_pages) {
  constexpr int NJ = HD / 32;
  constexpr int ND = HD / 16;
  const int lane = threadIdx.x & (kWave - 1);
  const int w = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int ti = blockIdx.x * kPreWaves + w;
  if (ti >= n_tiles) return;
  const int h = blockIdx.y;
  const int kvh = h / (nh / nkv);
  const int entry = tiles[ti * 3], tok0 = tiles[ti * 3 + 1], rows = tiles[ti * 3 + 2];
  const int pos0 = positions[tok0];
  const int* bt = block_table + (size_t)entry * max_blocks;

  // per column tile: this lane's query row, its position and the first key it may see
  int qpos[kQT], qstart[kQT];
  bool qok[kQT];
  bf16x8 qf[kQT][NJ];
#pragma unroll
  for (int c = 0; c < kQT; ++c) {
    const int row = c * 16 + r;
    qok[c] = row < rows;
    qpos[c] = pos0 + row;
    int st = 0;
    if (window_kind == 1) st = (qpos[c] / window) * window;
    else if (window_kind == 2) st = qpos[c] - window + 1 > 0 ? qpos[c] - window + 1 : 0;
    qstart[c] = st;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      if (qok[c]) qf[c][j] = *reinterpret_cast<const bf16x8*>(q + ((size_t)(tok0 + row) * nh + h) * HD + j * 32 + g * 8);
      else qf[c][j] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  int first = pos0;   // the first key of the tile's first row
  if (window_kind == 1) first = (pos0 / window) * window;
  else if (window_kind == 2) first = pos0 - window + 1 > 0 ? pos0 - window + 1 : 0;
  else first = 0;
  const int b_first = first >> 4;
  const int b_last = (pos0 + rows - 1) >> 4;

  float m[kQT], l[kQT];
  f32x4 acc[kQT][ND];
#pragma unroll
  for (int c = 0; c < kQT; ++c) {
    m[c] = -INFINITY;
    l[c] = 0.f;
#pragma unroll
    for (int d = 0; d < ND; ++d) acc[c][d] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  for (int b = b_first; b <= b_last; b += 2) {
    long long kbase[2], vbase[2];
    bool have[2];
    f32x4 s[kQT][2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int bb = b + u;
      have[u] = bb <= b_last;
      int page = -1;
      if (have[u]) {
        const int pi = (bb << 4) / page_size;
        page = pi < max_blocks ? bt[pi] : -1;
        if (page < 0 || page >= num_pages) have[u] = false;
      }
      const int off = (bb << 4) % page_size;
      kbase[u] = have[u] ? (((long long)page * nkv + kvh) * page_size + off) * HD : 0;
      vbase[u] = have[u] ? ((long long)page * nkv + kvh) * HD * page_size + off : 0;
#pragma unroll
      for (int c = 0; c < kQT; ++c) s[c][u] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (have[u]) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          const bf16x8 kf = *reinterpret_cast<const bf16x8*>(k_cache + kbase[u] + (size_t)r * HD + j * 32 + g * 8);
#pragma unroll
          for (int c = 0; c < kQT; ++c) s[c][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[c][j], s[c][u], 0, 0, 0);
        }
      }
    }
    bf16x8 pf[kQT], pf_lo[kQT];
    float corr[kQT];
#pragma unroll
    for (int c = 0; c < kQT; ++c) {
      // lane holds S^T[key = 16*(b+u) + 4g + i][query row c*16 + r]
      float cm = -INFINITY;
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = ((b + u) << 4) + 4 * g + i;
          const bool ok = have[u] && qok[c] && key >= qstart[c] && key <= qpos[c];
          s[c][u][i] = ok ? s[c][u][i] * scale : -INFINITY;
          cm = fmaxf(cm, s[c][u][i]);
        }
      cm = fmaxf(cm, __shfl_xor(cm, 16, kWave));
      cm = fmaxf(cm, __shfl_xor(cm, 32, kWave));
      const float m_new = fmaxf(m[c], cm);
      corr[c] = 1.0f;
      if (m_new == -INFINITY) {
        pf[c] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
        pf_lo[c] = pf[c];
      } else {
        corr[c] = expf(m[c] - m_new);
        float ls = 0.f;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float e = expf(s[c][u][i] - m_new);
            ls += e;
            const bf16_t hi = f32_to_bf16(e);
            pf[c][u * 4 + i] = __builtin_bit_cast(__bf16, hi.bits);
            pf_lo[c][u * 4 + i] = __builtin_bit_cast(__bf16, f32_to_bf16(e - bf16_to_f32(hi)).bits);
          }
        l[c] = l[c] * corr[c] + ls;
        m[c] = m_new;
      }
    }
#pragma unroll
    for (int d = 0; d < ND; ++d) {
      bf16x4 va = bf16x4{0, 0, 0, 0}, vb = bf16x4{0, 0, 0, 0};
      if (have[0]) va = *reinterpret_cast<const bf16x4*>(v_cache + vbase[0] + (size_t)(d * 16 + r) * page_size + 4 * g);
      if (have[1]) vb = *reinterpret_cast<const bf16x4*>(v_cache + vbase[1] + (size_t)(d * 16 + r) * page_size + 4 * g);
      const bf16x8 vf = __builtin_shufflevector(va, vb, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
      for (int c = 0; c < kQT; ++c) {
        acc[c][d] *= corr[c];
        acc[c][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[c], acc[c][d], 0, 0, 0);
        acc[c][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf_lo[c], acc[c][d], 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int c = 0; c < kQT; ++c) {
    float L = l[c];
    L += __shfl_xor(L, 16, kWave);
    L += __shfl_xor(L, 32, kWave);
    if (!qok[c]) continue;
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    bf16_t* orow = out + ((size_t)(tok0 + c * 16 + r) * nh + h) * HD;
#pragma unroll
    for (int d = 0; d < ND; ++d) {
      // lane holds O^T[d*16 + 4g + i][query row]
      const f32x4 o = acc[c][d] * inv;
      uint2 packed;
      packed.x = (uint32_t)f32_to_bf16(o[0]).bits | ((uint32_t)f32_to_bf16(o[1]).bits << 16);
      packed.y = (uint32_t)f32_to_bf16(o[2]).bits | ((uint32_t)f32_to_bf16(o[3]).bits << 16);
      *reinterpret_cast<uint2*>(orow + d * 16 + 4 * g) = packed;
    }
  }
}

// q [T, nh, hd] bf16; caches K [pages, nkv, page_size, hd], V [pages, nkv, hd, page_size] bf16;
// tiles int32 [n_tiles, 3] = (entry, first token, rows <= 32), tokens of a tile consecutive in
// one entry; out [T, nh, hd] bf16 (rows of the listed tiles).
SHARPI_EXPORT int sharpi_attention_prefill(const void* q, const void* k_cache, const void* v_cache,
                                           const int* block_table, const int* positions, const int* tiles,
                                           void* out, int n_tiles, int window_kind, int window, float scale,
                                           int nh, int nkv, int hd, int page_size, int max_blocks, int num_pages,
                                           hipStream_t stream) {
  if (n_tiles <= 0) return SHARPI_OK;
  if (nh <= 0 || nkv <= 0 || nh % nkv != 0 || nh > 65535) return SHARPI_ERR_ARG;
  if (page_size <= 0 || page_size % 16 != 0 || max_blocks <= 0 || num_pages <= 0) return SHARPI_ERR_ARG;
  if (window_kind < 0 || window_kind > 2 || (window_kind != 0 && window <= 0)) return SHARPI_ERR_ARG;
  dim3 grid(ceil_div(n_tiles, kPreWaves), nh), block(kPreWaves * kWave);
#define PRE(HDV)                                                                                              \
  if (hd == HDV) {                                                                                            \
    attn_prefill_kernel<HDV><<<grid, block, 0, stream>>>((const bf16_t*)q, (const bf16_t*)k_cache,            \
                                                        (const bf16_t*)v_cache, block_table, positions, tiles, \
                                                        (bf16_t*)out, n_tiles, window_kind, window, scale, nh, \
                                                        nkv, page_size, max_blocks, num_pages);               \
    SHARPI_CHECK_LAUNCH();                                                                                    \
    return SHARPI_OK;                                                                                         \
  }
  PRE(32) PRE(64) PRE(96) PRE(128) PRE(192) PRE(256)
#undef PRE
  return SHARPI_ERR_ARG;  // head sizes that are no multiple of 32 go to the generic kernel
}

SHARPI_EXPORT int sharpi_attention_prefill_tile_tokens() { return kTileTokens; }
