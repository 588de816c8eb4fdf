// Row-wise kernels: embedding gather, residual add + RMSNorm, SiLU*up, MoE combine, casts.
// All statistics and sums are float; storage may be float or bfloat16.
#include "common.h"

// ---------------------------------------------------------------------------
// embedding gather: out[t, :] = table[ids[t], :] * scale   (out is the float residual stream; the
// product in float; scale 1 leaves the row as it is)
// ---------------------------------------------------------------------------
template <typename T>
__global__ void embed_gather_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                    float* __restrict__ out, int hidden, float scale) {
  const int t = blockIdx.x;
  const T* row = table + (size_t)ids[t] * hidden;
  float* o = out + (size_t)t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = to_f32<T>(row[i]) * scale;
}

SHARPI_EXPORT int sharpi_embed_gather(const int* ids, const void* table, int table_dtype, float* out,
                                      int n_tokens, int hidden, float scale, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (hidden <= 0) return SHARPI_ERR_ARG;
  dim3 grid(n_tokens), block(256);
  if (table_dtype == DT_F32)
    embed_gather_kernel<float><<<grid, block, 0, stream>>>(ids, (const float*)table, out, hidden, scale);
  else if (table_dtype == DT_BF16)
    embed_gather_kernel<bf16_t><<<grid, block, 0, stream>>>(ids, (const bf16_t*)table, out, hidden, scale);
  else
    return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// ---------------------------------------------------------------------------
// residual add + RMSNorm.
//   r = rows ? rows[i] : i
//   x = h[r, :] (+ delta[r, :])           float sum
//   if write_back: h[r, :] = x
//   out[i, :] = (x * rsqrt(mean(x^2) + eps)) * w     (w may be absent)
// One block per output row; the order of the additions depends on `hidden` only.
// ---------------------------------------------------------------------------
template <typename TD, typename TW, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                   const TW* __restrict__ w, TO* __restrict__ out,
                                   const int* __restrict__ rows, int hidden, float eps, int write_back) {
  __shared__ float red[16];
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  float* hr = h + (size_t)r * hidden;
  const TD* dr = delta ? delta + (size_t)r * hidden : nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float x = hr[c];
    if (dr) {
      x += to_f32<TD>(dr[c]);
      if (write_back) hr[c] = x;
    }
    ss += x * x;
  }
  const float total = block_sum(ss, red);
  const float s = 1.0f / sqrtf(total / (float)hidden + eps);
  TO* o = out + (size_t)i * hidden;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float x = hr[c];
    if (dr && !write_back) x += to_f32<TD>(dr[c]);
    float y = x * s;
    if (w) y *= to_f32<TW>(w[c]);
    o[c] = from_f32<TO>(y);
  }
}

// The same with rows a multiple of 8 wide: 16-byte accesses, the row kept in registers between
// the two passes (up to kNormKeep runs of 8 per thread, of up to 1,024 threads; wider rows are read again).
constexpr int kNormKeep = 2;

// delta of row r, columns c .. c + 7, as floats.  Plain: delta[r].  As an expert sum (sum_pos
// given): the rows sum_pos[r*k .. r*k + k) of delta (each times its weight sum_w[r*k + q], if
// weights are given: scores applied to the experts' outputs) plus sum_shared[r], added in that
// order in float and rounded to the storage type, which is what the separate combine kernel
// would have stored for the norm to read.
template <typename TD>
__device__ __forceinline__ void load_delta8(const TD* __restrict__ delta, const int* __restrict__ sum_pos,
                                            const TD* __restrict__ sum_shared, const float* __restrict__ sum_w,
                                            int sum_k, int r, int hidden, int c, float* d) {
  if (!sum_pos) {
    load8(delta + (size_t)r * hidden + c, d);
    return;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) d[j] = 0.f;
  for (int q = 0; q < sum_k; ++q) {
    float v[8];
    load8(delta + (size_t)sum_pos[r * sum_k + q] * hidden + c, v);
    const float wq = sum_w ? sum_w[r * sum_k + q] : 1.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) d[j] += sum_w ? wq * v[j] : v[j];
  }
  if (sum_shared) {
    float v[8];
    load8(sum_shared + (size_t)r * hidden + c, v);
#pragma unroll
    for (int j = 0; j < 8; ++j) d[j] += v[j];
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) d[j] = to_f32<TD>(from_f32<TD>(d[j]));
}

template <typename TD, typename TW, typename TO>
__global__ __launch_bounds__(1024) void add_rmsnorm_vec_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                                               const TW* __restrict__ w, TO* __restrict__ out,
                                                               const int* __restrict__ rows, int hidden, float eps,
                                                               int write_back, const int* __restrict__ sum_pos,
                                                               const TD* __restrict__ sum_shared,
                                                               const float* __restrict__ sum_w, int sum_k) {
  __shared__ float red[16];
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  float* hr = h + (size_t)r * hidden;
  const bool dr = delta != nullptr;
  // A block has a thread per run of 8 where the row allows it (the launch sees to that): the row,
  // its delta and the norm's weights are then requested in one go, the kernel is one trip to
  // memory, the reduction and one store.  With a handful of rows (decode) that latency is all
  // the kernel costs.
  float keep[kNormKeep][8], wk[kNormKeep][8];
  float ss = 0.f;
#pragma unroll
  for (int n = 0; n < kNormKeep; ++n) {
    const int c = (threadIdx.x + n * blockDim.x) * 8;
    if (c < hidden) {
      load8(hr + c, keep[n]);
      if (w) load8(w + c, wk[n]);
    }
  }
#pragma unroll
  for (int n = 0; n < kNormKeep; ++n) {
    const int c = (threadIdx.x + n * blockDim.x) * 8;
    if (c < hidden) {
      if (dr) {
        float d[8];
        load_delta8<TD>(delta, sum_pos, sum_shared, sum_w, sum_k, r, hidden, c, d);
#pragma unroll
        for (int j = 0; j < 8; ++j) keep[n][j] += d[j];
        if (write_back) store8(hr + c, keep[n]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += keep[n][j] * keep[n][j];
    }
  }
  // rows wider than the registers hold: the rest is read again in the second pass
  for (int c = (threadIdx.x + kNormKeep * blockDim.x) * 8; c < hidden; c += blockDim.x * 8) {
    float x[8];
    load8(hr + c, x);
    if (dr) {
      float d[8];
      load_delta8<TD>(delta, sum_pos, sum_shared, sum_w, sum_k, r, hidden, c, d);
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] += d[j];
      if (write_back) store8(hr + c, x);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) ss += x[j] * x[j];
  }
  const float total = block_sum(ss, red);
  const float s = 1.0f / sqrtf(total / (float)hidden + eps);
  TO* o = out + (size_t)i * hidden;
#pragma unroll
  for (int n = 0; n < kNormKeep; ++n) {
    const int c = (threadIdx.x + n * blockDim.x) * 8;
    if (c < hidden) {
      float y[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = w ? (keep[n][j] * s) * wk[n][j] : keep[n][j] * s;
      store8(o + c, y);
    }
  }
  for (int c = (threadIdx.x + kNormKeep * blockDim.x) * 8; c < hidden; c += blockDim.x * 8) {
    float x[8];
    load8(hr + c, x);
    if (dr && !write_back) {
      float d[8];
      load_delta8<TD>(delta, sum_pos, sum_shared, sum_w, sum_k, r, hidden, c, d);
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] += d[j];
    }
    float y[8];
    if (w) {
      float wv[8];
      load8(w + c, wv);
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = (x[j] * s) * wv[j];
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = x[j] * s;
    }
    store8(o + c, y);
  }
}

template <typename TD, typename TW>
static int launch_add_rmsnorm_o(float* h, const void* delta, const void* w, void* out, int out_dtype,
                                const int* rows, int n_out, int hidden, float eps, int write_back,
                                const int* sum_pos, const void* sum_shared, const float* sum_w, int sum_k, hipStream_t stream) {
  dim3 grid(n_out), block(hidden >= 2048 ? 512 : 256);
  if (out_dtype != DT_F32 && out_dtype != DT_BF16) return SHARPI_ERR_ARG;
  if ((hidden & 7) == 0) {
    // a thread per run of 8, in whole waves, up to 1,024: the same for every number of rows, so
    // that a row's statistics are the same sums however many rows share the launch
    dim3 vblock(min(1024, ceil_div(hidden / 8, kWave) * kWave));
    if (out_dtype == DT_F32)
      add_rmsnorm_vec_kernel<TD, TW, float><<<grid, vblock, 0, stream>>>(h, (const TD*)delta, (const TW*)w,
                                                                        (float*)out, rows, hidden, eps, write_back,
                                                                        sum_pos, (const TD*)sum_shared, sum_w, sum_k);
    else
      add_rmsnorm_vec_kernel<TD, TW, bf16_t><<<grid, vblock, 0, stream>>>(h, (const TD*)delta, (const TW*)w,
                                                                         (bf16_t*)out, rows, hidden, eps, write_back,
                                                                         sum_pos, (const TD*)sum_shared, sum_w, sum_k);
  } else if (sum_pos)
    return SHARPI_ERR_ARG;   // an expert sum is folded in by the vector kernel only (width % 8 == 0)
  else if (out_dtype == DT_F32)
    add_rmsnorm_kernel<TD, TW, float><<<grid, block, 0, stream>>>(h, (const TD*)delta, (const TW*)w,
                                                                 (float*)out, rows, hidden, eps, write_back);
  else
    add_rmsnorm_kernel<TD, TW, bf16_t><<<grid, block, 0, stream>>>(h, (const TD*)delta, (const TW*)w,
                                                                  (bf16_t*)out, rows, hidden, eps, write_back);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

template <typename TD>
static int launch_add_rmsnorm_w(float* h, const void* delta, const void* w, int w_dtype, void* out,
                                int out_dtype, const int* rows, int n_out, int hidden, float eps,
                                int write_back, const int* sum_pos, const void* sum_shared, const float* sum_w,
                                int sum_k, hipStream_t stream) {
  if (w_dtype == DT_F32 || w == nullptr)
    return launch_add_rmsnorm_o<TD, float>(h, delta, w, out, out_dtype, rows, n_out, hidden, eps, write_back,
                                           sum_pos, sum_shared, sum_w, sum_k, stream);
  if (w_dtype == DT_BF16)
    return launch_add_rmsnorm_o<TD, bf16_t>(h, delta, w, out, out_dtype, rows, n_out, hidden, eps, write_back,
                                            sum_pos, sum_shared, sum_w, sum_k, stream);
  return SHARPI_ERR_ARG;
}

// h [*, hidden] float; delta the branch output to add first (null: none).  With sum_pos the
// delta is an expert sum: row r = delta[sum_pos[r*sum_k ..]] summed (+ sum_shared[r]), see
// load_delta8; hidden % 8 == 0 then.
SHARPI_EXPORT int sharpi_add_rmsnorm(float* h, const void* delta, int delta_dtype, const void* w, int w_dtype,
                                     void* out, int out_dtype, const int* rows, int n_out, int hidden,
                                     float eps, int write_back, const int* sum_pos, const void* sum_shared,
                                     const float* sum_w, int sum_k, hipStream_t stream) {
  if (n_out <= 0) return SHARPI_OK;
  if (hidden <= 0 || !(eps > 0.f)) return SHARPI_ERR_ARG;
  if (rows && write_back) return SHARPI_ERR_ARG;  // gathered rows never write the stream back
  if (sum_pos && (delta == nullptr || sum_k <= 0)) return SHARPI_ERR_ARG;
  if (delta == nullptr || delta_dtype == DT_F32)
    return launch_add_rmsnorm_w<float>(h, delta, w, w_dtype, out, out_dtype, rows, n_out, hidden, eps, write_back,
                                       sum_pos, sum_shared, sum_w, sum_k, stream);
  if (delta_dtype == DT_BF16)
    return launch_add_rmsnorm_w<bf16_t>(h, delta, w, w_dtype, out, out_dtype, rows, n_out, hidden, eps, write_back,
                                        sum_pos, sum_shared, sum_w, sum_k, stream);
  return SHARPI_ERR_ARG;
}

// ---------------------------------------------------------------------------
// The gated unit on a fused [M, 2*I] buffer (gate columns first, up columns second):
//   out[m, i] = act(s_m * g) * (s_m * u),  s_m = scale ? scale[m] : 1,  act as common.h codes it
// ---------------------------------------------------------------------------
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, const float* __restrict__ scale,
                                T* __restrict__ out, int inter, int act) {
  const int m = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= inter) return;
  const T* row = gu + (size_t)m * 2 * inter;
  const float g = to_f32<T>(row[i]);
  const float u = to_f32<T>(row[inter + i]);
  out[(size_t)m * inter + i] = from_f32<T>(gated_f32(act, g, u, scale ? scale[m] : 1.0f, scale != nullptr));
}

template <typename T>
__global__ void silu_mul_vec_kernel(const T* __restrict__ gu, const float* __restrict__ scale,
                                    T* __restrict__ out, int inter, int act) {
  const int m = blockIdx.x;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= inter) return;
  const T* row = gu + (size_t)m * 2 * inter;
  float g[8], u[8], o[8];
  load8(row + i, g);
  load8(row + inter + i, u);
  const float s = scale ? scale[m] : 1.0f;
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = gated_f32(act, g[j], u[j], s, scale != nullptr);
  store8(out + (size_t)m * inter + i, o);
}

SHARPI_EXPORT int sharpi_silu_mul(const void* gu, const float* scale, void* out, int dtype, int rows, int inter,
                                  int act, hipStream_t stream) {
  if (rows <= 0) return SHARPI_OK;
  if (inter <= 0 || ceil_div(inter, 256) > 65535 || !act_known(act)) return SHARPI_ERR_ARG;
  dim3 block(256), grid(rows, ceil_div(inter, 256));
  if (dtype != DT_F32 && dtype != DT_BF16) return SHARPI_ERR_ARG;
  if ((inter & 7) == 0) {
    dim3 vgrid(rows, ceil_div(inter, 256 * 8));
    if (dtype == DT_F32)
      silu_mul_vec_kernel<float><<<vgrid, block, 0, stream>>>((const float*)gu, scale, (float*)out, inter, act);
    else
      silu_mul_vec_kernel<bf16_t><<<vgrid, block, 0, stream>>>((const bf16_t*)gu, scale, (bf16_t*)out, inter, act);
  } else if (dtype == DT_F32)
    silu_mul_kernel<float><<<grid, block, 0, stream>>>((const float*)gu, scale, (float*)out, inter, act);
  else
    silu_mul_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)gu, scale, (bf16_t*)out, inter, act);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// ---------------------------------------------------------------------------
// MoE combine: out[t, :] = sum_j w[t*k + j] * y[inv_pos[t*k + j], :] (+ shared[t, :]); w null: ones;
// float sums, j ascending.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ y, const int* __restrict__ inv_pos,
                                   const T* __restrict__ shared, const float* __restrict__ w,
                                   T* __restrict__ out, int hidden, int k) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= hidden) return;
  float acc = 0.f;
  for (int j = 0; j < k; ++j) {
    const float v = to_f32<T>(y[(size_t)inv_pos[t * k + j] * hidden + c]);
    acc += w ? w[t * k + j] * v : v;
  }
  if (shared) acc += to_f32<T>(shared[(size_t)t * hidden + c]);
  out[(size_t)t * hidden + c] = from_f32<T>(acc);
}

template <typename T>
__global__ void moe_combine_vec_kernel(const T* __restrict__ y, const int* __restrict__ inv_pos,
                                       const T* __restrict__ shared, const float* __restrict__ w,
                                       T* __restrict__ out, int hidden, int k) {
  const int t = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (c >= hidden) return;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int j = 0; j < k; ++j) {
    float v[8];
    load8(y + (size_t)inv_pos[t * k + j] * hidden + c, v);
    const float wj = w ? w[t * k + j] : 1.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += w ? wj * v[i] : v[i];
  }
  if (shared) {
    float v[8];
    load8(shared + (size_t)t * hidden + c, v);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += v[i];
  }
  store8(out + (size_t)t * hidden + c, acc);
}

SHARPI_EXPORT int sharpi_moe_combine(const void* y, const int* inv_pos, const void* shared, const float* w, void* out, int dtype,
                                     int n_tokens, int hidden, int k, hipStream_t stream) {
  if (n_tokens <= 0) return SHARPI_OK;
  if (hidden <= 0 || k <= 0 || ceil_div(hidden, 256) > 65535) return SHARPI_ERR_ARG;
  dim3 block(256), grid(n_tokens, ceil_div(hidden, 256));
  if (dtype != DT_F32 && dtype != DT_BF16) return SHARPI_ERR_ARG;
  if ((hidden & 7) == 0) {
    dim3 vblock(128), vgrid(n_tokens, ceil_div(hidden, 128 * 8));
    if (dtype == DT_F32)
      moe_combine_vec_kernel<float><<<vgrid, vblock, 0, stream>>>((const float*)y, inv_pos, (const float*)shared, w,
                                                                 (float*)out, hidden, k);
    else
      moe_combine_vec_kernel<bf16_t><<<vgrid, vblock, 0, stream>>>((const bf16_t*)y, inv_pos, (const bf16_t*)shared, w,
                                                                  (bf16_t*)out, hidden, k);
  } else if (dtype == DT_F32)
    moe_combine_kernel<float><<<grid, block, 0, stream>>>((const float*)y, inv_pos, (const float*)shared, w,
                                                         (float*)out, hidden, k);
  else
    moe_combine_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)y, inv_pos, (const bf16_t*)shared, w,
                                                          (bf16_t*)out, hidden, k);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// ---------------------------------------------------------------------------
// casts between the two storage types
// ---------------------------------------------------------------------------
template <typename TI, typename TO>
__global__ void cast_kernel(const TI* __restrict__ in, TO* __restrict__ out, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) out[i] = from_f32<TO>(to_f32<TI>(in[i]));
}

SHARPI_EXPORT int sharpi_cast(const void* in, int in_dtype, void* out, int out_dtype, long long n,
                              hipStream_t stream) {
  if (n <= 0) return SHARPI_OK;
  long long nb = (n + 255) / 256;
  dim3 block(256), grid((unsigned)(nb > 65536 ? 65536 : nb));
  if (in_dtype == DT_F32 && out_dtype == DT_BF16)
    cast_kernel<float, bf16_t><<<grid, block, 0, stream>>>((const float*)in, (bf16_t*)out, (size_t)n);
  else if (in_dtype == DT_BF16 && out_dtype == DT_F32)
    cast_kernel<bf16_t, float><<<grid, block, 0, stream>>>((const bf16_t*)in, (float*)out, (size_t)n);
  else if (in_dtype == DT_F32 && out_dtype == DT_F32)
    cast_kernel<float, float><<<grid, block, 0, stream>>>((const float*)in, (float*)out, (size_t)n);
  else if (in_dtype == DT_BF16 && out_dtype == DT_BF16)
    cast_kernel<bf16_t, bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)in, (bf16_t*)out, (size_t)n);
  else
    return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// ---------------------------------------------------------------------------
// x [T, N] += bias [N] (float), in place; the sum in float, rounded to x's storage.  For the
// projections of architectures that carry biases (the products themselves have no bias term).
// ---------------------------------------------------------------------------
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ x, const float* __restrict__ bias, int n_rows, int N) {
  const size_t total = (size_t)n_rows * N;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
    x[i] = from_f32<T>(to_f32<T>(x[i]) + bias[i % N]);
}

SHARPI_EXPORT int sharpi_add_bias(void* x, int dtype, const float* bias, int n_rows, int N, hipStream_t stream) {
  if (n_rows <= 0) return SHARPI_OK;
  if (N <= 0 || !bias) return SHARPI_ERR_ARG;
  const size_t total = (size_t)n_rows * N;
  const dim3 block(256), grid((unsigned)min((size_t)4096, (total + 255) / 256));
  if (dtype == DT_F32) add_bias_kernel<float><<<grid, block, 0, stream>>>((float*)x, bias, n_rows, N);
  else if (dtype == DT_BF16) add_bias_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)x, bias, n_rows, N);
  else return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// ---------------------------------------------------------------------------
// logits in place: x <- x * scale, then (cap > 0) x <- cap * tanh(x / cap): the head's scale and the
// soft cap of architectures that have them.
// ---------------------------------------------------------------------------
__global__ void scale_softcap_kernel(float* __restrict__ x, size_t n, float scale, float cap) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    float v = x[i] * scale;
    if (cap > 0.f) v = tanhf(v / cap) * cap;
    x[i] = v;
  }
}

SHARPI_EXPORT int sharpi_scale_softcap(float* x, long long n, float scale, float cap, hipStream_t stream) {
  if (n <= 0) return SHARPI_OK;
  if (!(cap >= 0.f)) return SHARPI_ERR_ARG;
  const dim3 block(256), grid((unsigned)min((long long)8192, (n + 255) / 256));
  scale_softcap_kernel<<<grid, block, 0, stream>>>(x, (size_t)n, scale, cap);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
