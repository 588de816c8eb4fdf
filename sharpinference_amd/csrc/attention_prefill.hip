// Attention for entries of several tokens (prompt portions): flash attention on the matrix cores
// over the paged cache, causal and window masks applied per element.
//
// A block owns a tile of up to 128 consecutive tokens of one entry and one query head; each of its
// four waves takes 32 of the tokens (or, for tiles of up to 64 tokens, 16: the keys of a tile are
// walked one chunk after the other, so a short prompt, whose last tiles alone decide how long the
// launch takes, is served faster by twice the blocks of half the rows; a row's sums are the same
// either way).  The block walks the keys its rows can see in 32-key chunks
// (two 16-key blocks aligned to absolute positions, so a block never straddles a page); a chunk's
// keys and values are fetched from the cache once, staged in LDS (double-buffered; two chunks
// are on their way through registers) and read from there by all four waves.  As in the decode kernel everything is transposed:
//   S^T[key, q]  = K[key, :] . Q[q, :]          A = K block, B = Q^T
//   O^T[d, q]   += V^T[d, key] * P^T[key, q]    A = V^T block (values are stored transposed
//                                               inside a page), B = P^T
// and the S^T accumulator of a lane is the B operand of the second product once exponentiated
// and split into a bfloat16 pair hi + lo (two products: the probabilities keep ~16 bits; the row's
// sum is taken from the unrounded values).  In LDS the value columns are permuted so that the
// eight keys a lane needs (4 of each 16-key block) sit side by side; rows and their 16-byte chunks
// are placed so that reads and stores are free of bank conflicts (see the layouts below).  Softmax
// state (a reference maximum and the sum per query) is float, kept in base-2 units (scores times
// log2 e, the hardware's exp2).
// The keys of a query are always visited in the same chunks (pairs of 16-key blocks at absolute
// positions), whatever the portion or tile it arrived in, so its sums do not depend on how the prompt was cut.
#include <type_traits>

#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// the head sizes the kernel is compiled for
#define SHARPI_PREFILL_HEAD_SIZES(X) X(32) X(64) X(96) X(128) X(160) X(192)

#ifndef SHARPI_PREFILL_P_PAIR
// 1: probabilities enter the second product as a bfloat16 pair hi + lo.  0 (hi alone) is 4 % faster at
// 2,048 tokens and 10 % at 8,192, but then rounds every probability to 8 bits, which the comparison
// with a float softmax does not forgive where the softmax is sharp: random mixed traces at a weight
// scale of 0.08 left the derived bfloat16 bound by up to a quarter in 4 of 60, none with the pair.
#define SHARPI_PREFILL_P_PAIR 1
#endif
constexpr int kPreWaves = 4;
constexpr int kMaxQT = 2;                            // most 16-token column tiles per wave
constexpr int kTileTokens = 16 * kMaxQT * kPreWaves; // 128 tokens per block at most (64 with one column tile a wave)
constexpr int kVRow = 32;                            // LDS row of the value tile: 32 keys, no pad (chunks swizzled)

// LDS layouts.  The LDS serves a 16-byte read of a wave in four turns of two octets of lanes: one
// octet holding operand rows 0..7 and one holding rows 8..15 of the neighbouring lane group (measured
// with the bank-conflict counter).  The 16 chunks of 16 bytes that a turn reads must fall into the 16
// different 16-byte groups of the 256-byte bank space; the chunk index is XORed with row bits so that
// they do, for rows of 256 bytes (keys, head size 128), 128 bytes (head size 64) and 64 bytes
// (values: 32 keys, see v_row).  Other head sizes keep key rows padded by 16 bytes (two-way conflicts).
template <int HD> __device__ __forceinline__ constexpr int k_row_elems() { return (HD == 128 || HD == 64) ? HD : HD + 8; }
template <int HD> __device__ __forceinline__ int k_col(int row, int col) {   // col a multiple of 8 elements
  if constexpr (HD == 128) return col ^ ((row & 15) << 3);
  else if constexpr (HD == 64) return col ^ (((row >> 1) & 7) << 3);
  else return col;
}
// values: rows of 64 bytes (32 keys), sixteen to a 1 KB tile.  Within a tile the rows are kept in the
// order 0 1 8 9 | 2 3 10 11 | 4 5 12 13 | 6 7 14 15 (rows 0..7 in one half of the bank space, 8..15 in
// the other) and a row's four chunks are XORed with bits 1..2 of the row: an octet of lanes (rows
// r..r+7 of a tile, one chunk column) then reads eight different 16-byte groups of one half, and
// the stores (a lane per row and half row) are as free of conflicts (both measured with the counter;
// XORing the chunk alone left every read and store two-way conflicted).
__device__ __forceinline__ int v_row(int d) { return (d & ~15) | (d & 1) | (((d >> 3) & 1) << 1) | (((d >> 1) & 3) << 2); }
__device__ __forceinline__ int v_col(int d, int col) { return col ^ (((d >> 1) & 3) << 3); }   // 4 chunks a row
constexpr float kLazyMax = 8.0f;                     // how far the row maximum may outgrow its reference
// the reference before a row has seen a key: finite, so that a masked score (-inf) minus it is
// -inf and its probability 0, and far below any score, so that the first key moves it
constexpr float kNoMax = -1.0e30f;

template <int HD, int kQT>
__global__ __launch_bounds__(kPreWaves* kWave, HD <= 128 ? (kQT == 1 ? 3 : 2) : 1) void attn_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_table, const int* __restrict__ positions, const int* __restrict__ tiles,
    bf16_t* __restrict__ out, int window_kind, int window, float scale, int nh, int nkv, int page_size,
    int max_blocks, int num_pages) {
  constexpr int kWaveTokens = 16 * kQT;
  constexpr int NJ = HD / 32;
  constexpr int ND = HD / 16;
  constexpr int KPAD = k_row_elems<HD>();
  constexpr int PIECES = 4 * HD;                                   // 16-byte pieces of a K (or V) chunk
  constexpr int NST = (PIECES + kPreWaves * kWave - 1) / (kPreWaves * kWave);
  constexpr int VPAIRS = 2 * HD;                                   // (value row, half of its 16 keys per block) pairs of a chunk
  constexpr int NSV = (VPAIRS + kPreWaves * kWave - 1) / (kPreWaves * kWave);
  __shared__ __attribute__((aligned(16))) bf16_t Ks[2][32][KPAD];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[2][HD][kVRow];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int w = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  // heads run fastest and tiles from the last backwards: later tiles of a prompt see more keys, and
  // the longest blocks should start first
  const int ti = gridDim.y - 1 - blockIdx.y;
  const int h = blockIdx.x;
  const int kvh = h / (nh / nkv);
  const int entry = tiles[ti * 3], tok0 = tiles[ti * 3 + 1], rows = tiles[ti * 3 + 2];
  const int pos0 = positions[tok0];
  const int* bt = block_table + (size_t)entry * max_blocks;

  // this wave's 32 tokens: per column tile, the lane's query row, its position, its first key
  const int wrow0 = w * kWaveTokens;
  int qpos[kQT], qstart[kQT];
  bool qok[kQT];
  bf16x8 qf[kQT][NJ];
#pragma unroll
  for (int c = 0; c < kQT; ++c) {
    const int row = wrow0 + c * 16 + r;
    qok[c] = row < rows;
    qpos[c] = pos0 + row;
    int st = 0;
    if (window_kind == 1) st = (qpos[c] / window) * window;
    else if (window_kind == 2) st = qpos[c] - window + 1 > 0 ? qpos[c] - window + 1 : 0;
    qstart[c] = st;
    // rows beyond the tile's last read its last row (every load unconditional, see the note on the
    // chunk loop); their scores are masked and their output is never stored
    const int qrow = min(row, rows - 1);
#pragma unroll
    for (int j = 0; j < NJ; ++j)
      qf[c][j] = *reinterpret_cast<const bf16x8*>(q + ((size_t)(tok0 + qrow) * nh + h) * HD + j * 32 + g * 8);
  }
  const int wave_last = pos0 + min(rows, wrow0 + kWaveTokens) - 1;   // last position of this wave's rows
  const bool wave_has_rows = wrow0 < rows;
  const bool wave_full = wrow0 + kWaveTokens <= rows;                 // all 32 rows exist
  const int wave_first_pos = pos0 + wrow0;
  int wave_last_start = 0;                                            // first key the wave's last row may see
  if (window_kind == 1) wave_last_start = (wave_last / window) * window;
  else if (window_kind == 2) wave_last_start = wave_last - window + 1 > 0 ? wave_last - window + 1 : 0;
  const float scale_log2 = scale * 1.4426950408889634f;               // softmax in base 2: exp(x) = 2^(x log2 e)
  int wave_first = pos0 + wrow0;                                      // first key the wave's first row may see
  if (window_kind == 1) wave_first = (wave_first / window) * window;
  else if (window_kind == 2) wave_first = wave_first - window + 1 > 0 ? wave_first - window + 1 : 0;
  else wave_first = 0;

  int first = 0;   // the first key of the tile's first row
  if (window_kind == 1) first = (pos0 / window) * window;
  else if (window_kind == 2) first = pos0 - window + 1 > 0 ? pos0 - window + 1 : 0;
  // chunks are pairs of 16-key blocks aligned to absolute positions (an even block first): which keys
  // share a chunk does not depend on the tile.  The block before a window's first, if the pair starts
  // there, is masked whole; its page may have been given back (the table's -1 reads page 0: finite
  // values that meet probabilities of zero).
  const int b_first = (first >> 4) & ~1;
  const int b_last = (pos0 + rows - 1) >> 4;

  float m[kQT], l[kQT];
  f32x4 acc[kQT][ND];
#pragma unroll
  for (int c = 0; c < kQT; ++c) {
    m[c] = kNoMax;
    l[c] = 0.f;
#pragma unroll
    for (int d = 0; d < ND; ++d) acc[c][d] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // The block table of the entry, 64 pages at a time, one per lane (and the next 64 behind them):
  // a chunk's pages come out of a register with a uniform lane read, not out of memory, so the
  // address of a chunk's keys does not wait for a load of its own.
  int pv_base = (b_first << 4) / page_size;
  auto load_pages = [&](int base) { return bt[min(base + lane, max_blocks - 1)]; };
  int pv = load_pages(pv_base), pv_next = load_pages(pv_base + kWave);
  auto page_of = [&](int bb) {                               // bb uniform, within the 128 pages held
    const int pi = (bb << 4) / page_size - pv_base;
    const int page = pi < kWave ? __builtin_amdgcn_readlane(pv, pi) : __builtin_amdgcn_readlane(pv_next, pi - kWave);
    return min(max(page, 0), num_pages - 1);                 // a table that is wrong reads a wrong page, never outside
  };

  // staging: fetch the chunk that starts at 16-key block b into registers.  Every load is
  // unconditional: a 16-key block beyond the tile's last is fetched as the last one again (its
  // keys are masked, its values are finite and meet probabilities of zero).  The compiler counts
  // outstanding loads statically; one load behind a branch and every wait in the loop becomes a
  // wait for all loads, the chunk in flight included.
  u32x4 kst[2][NST], vst[2][NSV][2];   // two chunks on their way
  auto fetch = [&](int b, auto set_tag) {
    constexpr int set = decltype(set_tag)::value;
    long long kbase[2], vbase[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int bb = min(b + u, b_last);
      const int page = page_of(bb);
      const int off = (bb << 4) % page_size;
      kbase[u] = (((long long)page * nkv + kvh) * page_size + off) * HD;
      vbase[u] = ((long long)page * nkv + kvh) * HD * page_size + off;
    }
#pragma unroll
    for (int i = 0; i < NST; ++i) {
      const int piece = min(tid + i * kPreWaves * kWave, PIECES - 1);
      const int key = piece / (HD / 8), dcol = (piece % (HD / 8)) * 8;     // K: 32 keys x HD
      kst[set][i] = *reinterpret_cast<const u32x4*>(k_cache + kbase[key >> 4] + (size_t)(key & 15) * HD + dcol);
    }
#pragma unroll
    for (int i = 0; i < NSV; ++i) {
      // V^T: a thread takes keys 8*half .. 8*half+7 of both 16-key blocks for one value row
      const int pair = min(tid + i * kPreWaves * kWave, VPAIRS - 1);
      const int d = pair >> 1, half = pair & 1;
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
        vst[set][i][blk] = *reinterpret_cast<const u32x4*>(v_cache + vbase[blk] + (size_t)d * page_size + half * 8);
    }
  };
  auto stash = [&](auto set_tag) {   // register set `set` goes to LDS buffer `set`
    constexpr int set = decltype(set_tag)::value;
    constexpr int buf = set;
#pragma unroll
    for (int i = 0; i < NST; ++i) {
      const int piece = tid + i * kPreWaves * kWave;
      if (piece < PIECES) {
        const int key = piece / (HD / 8), dcol = (piece % (HD / 8)) * 8;
        *reinterpret_cast<u32x4*>(&Ks[buf][key][k_col<HD>(key, dcol)]) = kst[set][i];
      }
    }
#pragma unroll
    for (int i = 0; i < NSV; ++i) {
      const int pair = tid + i * kPreWaves * kWave;
      if (pair < VPAIRS) {
        // chunk g of a row holds keys 4g .. 4g+3 of the first block, then of the second: what lane
        // group g of the second product wants side by side.  The thread's keys are those of the
        // groups g = 2*half and 2*half + 1.
        const int d = pair >> 1, half = pair & 1;
        const u32x4 a = vst[set][i][0], b = vst[set][i][1];
        *reinterpret_cast<u32x4*>(&Vs[buf][v_row(d)][v_col(d, (2 * half) * 8)]) = u32x4{a[0], a[1], b[0], b[1]};
        *reinterpret_cast<u32x4*>(&Vs[buf][v_row(d)][v_col(d, (2 * half + 1) * 8)]) = u32x4{a[2], a[3], b[2], b[3]};
      }
    }
  };

  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;
  fetch(b_first, Set0{});
  fetch(b_first + 2 <= b_last ? b_first + 2 : b_first, Set1{});
  stash(Set0{});
  __syncthreads();
  // One chunk: the chunk in LDS buffer `par` is multiplied while the chunk after it waits in register set
  // par ^ 1 and the one after that is requested into set par (two chunks on their way: the keys
  // and values of a prompt were just written by another kernel and come from memory, not from cache).
  auto one_chunk = [&](int b, auto par_tag) {
    constexpr int par = decltype(par_tag)::value;
    constexpr int buf = par;
    const int b_fetch = b + 4 <= b_last ? b + 4 : b;            // beyond the last chunk: this one again, unused
    if ((((b_fetch + 1) << 4) / page_size) - pv_base >= 2 * kWave - 1) {   // the pages held run out: move on by 64
      pv = pv_next;
      pv_base += kWave;
      pv_next = load_pages(pv_base + kWave);
    }
    fetch(b_fetch, par_tag);
    __builtin_amdgcn_sched_barrier(0);                       // the loads are issued here, not where they are used
    // does any row of this wave see a key of this chunk?
    const bool active = wave_has_rows && (b << 4) <= wave_last && ((b + 2) << 4) > wave_first;
    if (active) {
      bool have[2];
      f32x4 s[kQT][2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        have[u] = b + u <= b_last;
#pragma unroll
        for (int c = 0; c < kQT; ++c) s[c][u] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (have[u]) {
#pragma unroll
          for (int j = 0; j < NJ; ++j) {
            const bf16x8 kf = *reinterpret_cast<const bf16x8*>(&Ks[buf][u * 16 + r][k_col<HD>(u * 16 + r, j * 32 + g * 8)]);
#pragma unroll
            for (int c = 0; c < kQT; ++c) s[c][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[c][j], s[c][u], 0, 0, 0);
          }
        }
      }
      bf16x8 pf[kQT];
#if SHARPI_PREFILL_P_PAIR
      bf16x8 pf_lo[kQT];
#endif
      // a chunk that every row of the wave sees whole needs no mask
      const bool whole = wave_full && have[1] && ((b + 2) << 4) - 1 <= wave_first_pos && (b << 4) >= wave_last_start;
      // lane holds S^T[key = 16*(b+u) + 4g + i][query row c*16 + r]; scores go to base-2 units
      float lmax[kQT];
      bool grown = false;
#pragma unroll
      for (int c = 0; c < kQT; ++c) {
        float lm = -INFINITY;   // the largest score this lane holds of the row
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float t = s[c][u][i] * scale_log2;
            if (!whole) {
              const int key = ((b + u) << 4) + 4 * g + i;
              const bool ok = have[u] && qok[c] && key >= qstart[c] && key <= qpos[c];
              t = ok ? t : -INFINITY;
            }
            s[c][u][i] = t;
            lm = fmaxf(lm, t);
          }
        lmax[c] = lm;
        grown = grown || lm - m[c] > kLazyMax;
      }
      // m is a reference, not the running maximum: a row moves it only when the chunk's largest
      // score lies more than kLazyMax (base-2 units) above it.  Probabilities then reach 2^kLazyMax
      // at most, which float sums carry easily.  Most chunks move no row of the wave: they need
      // no exchange between lanes and no rescaling.  The rule is the row's own (its four lanes
      // hold the same m and, once exchanged, the same maximum), so what a row ends up with does
      // not depend on the rows it shares a wave with.
      float corr[kQT];
      bool rescale[kQT];
#pragma unroll
      for (int c = 0; c < kQT; ++c) {
        corr[c] = 1.0f;
        rescale[c] = false;
      }
      if (__builtin_amdgcn_ballot_w64(grown) != 0) {   // wave-uniform
#pragma unroll
        for (int c = 0; c < kQT; ++c) {
          float cm = lmax[c];
          cm = fmaxf(cm, __shfl_xor(cm, 16, kWave));
          cm = fmaxf(cm, __shfl_xor(cm, 32, kWave));
          const bool move = cm - m[c] > kLazyMax;
          corr[c] = move ? __builtin_amdgcn_exp2f(m[c] - cm) : 1.0f;
          m[c] = move ? cm : m[c];
          l[c] *= corr[c];
          rescale[c] = __builtin_amdgcn_ballot_w64(move) != 0;
        }
      }
#pragma unroll
      for (int c = 0; c < kQT; ++c) {
        float ls = 0.f;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float e = __builtin_amdgcn_exp2f(s[c][u][i] - m[c]);   // masked: 2^-inf = 0
            ls += e;
            const __bf16 hi = (__bf16)e;                                   // round to nearest even
            pf[c][u * 4 + i] = hi;
#if SHARPI_PREFILL_P_PAIR
            pf_lo[c][u * 4 + i] = (__bf16)(e - (float)hi);
#endif
          }
        l[c] += ls;
      }
#pragma unroll
      for (int d = 0; d < ND; ++d) {
        // lane (d row r, group g): keys 4g..4g+3 of block b, then of block b + 1, side by side in LDS
        const bf16x8 vf = *reinterpret_cast<const bf16x8*>(&Vs[buf][v_row(d * 16 + r)][v_col(d * 16 + r, g * 8)]);
#pragma unroll
        for (int c = 0; c < kQT; ++c) {
          if (rescale[c]) {
            // rare, and to stay a branch: the empty statement keeps the compiler from turning it into
            // a multiplication by one in every chunk
            asm volatile("");
            acc[c][d] *= corr[c];
          }
          acc[c][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[c], acc[c][d], 0, 0, 0);
#if SHARPI_PREFILL_P_PAIR
          acc[c][d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf_lo[c], acc[c][d], 0, 0, 0);
#endif
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    stash(std::integral_constant<int, par ^ 1>{});
    __syncthreads();
  };
  for (int b = b_first; b <= b_last; b += 4) {
    one_chunk(b, Set0{});
    if (b + 2 > b_last) break;
    one_chunk(b + 2, Set1{});
  }

#pragma unroll
  for (int c = 0; c < kQT; ++c) {
    float L = l[c];
    L += __shfl_xor(L, 16, kWave);
    L += __shfl_xor(L, 32, kWave);
    if (!qok[c]) continue;
    const float inv = L > 0.f ? 1.0f / L : 0.f;
    bf16_t* orow = out + ((size_t)(tok0 + wrow0 + c * 16 + r) * nh + h) * HD;
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
// tiles int32 [n_tiles, 3] = (entry, first token, rows <= tile_tokens), tokens of a tile consecutive
// in one entry; tile_tokens 128 or 64 (what the caller cut the tiles to: no tile may hold more);
// out [T, nh, hd] bf16 (rows of the listed tiles).
SHARPI_EXPORT int sharpi_attention_prefill(const void* q, const void* k_cache, const void* v_cache,
                                           const int* block_table, const int* positions, const int* tiles,
                                           void* out, int n_tiles, int tile_tokens, int window_kind, int window,
                                           float scale, int nh, int nkv, int hd, int page_size, int max_blocks,
                                           int num_pages, hipStream_t stream) {
  if (n_tiles <= 0) return SHARPI_OK;
  if (nh <= 0 || nkv <= 0 || nh % nkv != 0 || n_tiles > 65535) return SHARPI_ERR_ARG;
  if (tile_tokens != kTileTokens && tile_tokens != kTileTokens / 2) return SHARPI_ERR_ARG;
  if (page_size <= 0 || page_size % 16 != 0 || max_blocks <= 0 || num_pages <= 0) return SHARPI_ERR_ARG;
  if (window_kind < 0 || window_kind > 2 || (window_kind != 0 && window <= 0)) return SHARPI_ERR_ARG;
  dim3 grid(nh, n_tiles), block(kPreWaves * kWave);
#define PRE_QT(HDV, QTV)                                                                                        \
  attn_prefill_kernel<HDV, QTV><<<grid, block, 0, stream>>>((const bf16_t*)q, (const bf16_t*)k_cache,               \
                                                           (const bf16_t*)v_cache, block_table, positions, tiles,  \
                                                           (bf16_t*)out, window_kind, window, scale, nh, nkv,      \
                                                           page_size, max_blocks, num_pages)
#define PRE(HDV)                                  \
  if (hd == HDV) {                                \
    if (tile_tokens == kTileTokens) PRE_QT(HDV, 2); \
    else PRE_QT(HDV, 1);                          \
    SHARPI_CHECK_LAUNCH();                        \
    return SHARPI_OK;                             \
  }
  SHARPI_PREFILL_HEAD_SIZES(PRE)
#undef PRE
#undef PRE_QT
  return SHARPI_ERR_ARG;  // other head sizes go to the generic kernel
}

// 1 if the kernel is compiled for this head size (the caller's choice of kernel asks here).
SHARPI_EXPORT int sharpi_attention_prefill_takes(int hd) {
#define PRE(HDV) if (hd == HDV) return 1;
  SHARPI_PREFILL_HEAD_SIZES(PRE)
#undef PRE
  return 0;
}

SHARPI_EXPORT int sharpi_attention_prefill_tile_tokens() { return kTileTokens; }
