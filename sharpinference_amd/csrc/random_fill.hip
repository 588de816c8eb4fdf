// Seeded random tensors without a generator state: element i of a tensor is a function of
// (key, i) alone, key = hash of (seed, tensor name) made by the host.  The host has the same
// function (weights/random_fill.py), so a tensor made here equals the one a model file written
// from the same seed holds, bit for bit, and any part of a tensor can be made anywhere, in any order.
//
//   mix(z): z ^= z >> 30; z *= 0xBF58476D1CE4E5B9; z ^= z >> 27; z *= 0x94D049BB133111EB; z ^= z >> 31
//   word(c) = mix(key + (c + 1) * 0x9E3779B97F4A7C15)                       (64-bit wrap-around)
//   normal : S = the twelve 16-bit fields of word(3i), word(3i+1), word(3i+2) added up;
//            value = float(S - 393210) * scale, scale = std / 65536 (a sum of twelve uniforms: mean 0,
//            deviation std, tails to +-6 std); one float product, so host and device agree exactly
//   uniform: u = word(i) >> 40 (24 bits); m = round(lo * 2^24) + ((u * round((hi - lo) * 2^24)) >> 24);
//            value = float(m) * 2^-24  (lo, hi fixed by the host as the two integers)
//   int    : word(i) >> 49 (15 bits)
// No transcendental function and no fused multiply-add is involved anywhere.
#include "common.h"

__device__ __forceinline__ unsigned long long fill_mix(unsigned long long z) {
  z ^= z >> 30;
  z *= 0xBF58476D1CE4E5B9ull;
  z ^= z >> 27;
  z *= 0x94D049BB133111EBull;
  z ^= z >> 31;
  return z;
}
__device__ __forceinline__ unsigned long long fill_word(unsigned long long key, unsigned long long c) {
  return fill_mix(key + (c + 1ull) * 0x9E3779B97F4A7C15ull);
}
__device__ __forceinline__ int fill_fields(unsigned long long w) {
  return (int)(w & 0xffffull) + (int)((w >> 16) & 0xffffull) + (int)((w >> 32) & 0xffffull) + (int)(w >> 48);
}

enum : int { FILL_NORMAL = 0, FILL_UNIFORM = 1, FILL_INT = 2 };

template <typename T>
__global__ void random_fill_kernel(T* __restrict__ out, unsigned long long n, unsigned long long key, int kind,
                                   float scale, int lo_fixed, int span_fixed) {
  unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x;
  const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    float v;
    if (kind == FILL_NORMAL) {
      const int s = fill_fields(fill_word(key, 3 * i)) + fill_fields(fill_word(key, 3 * i + 1)) +
                    fill_fields(fill_word(key, 3 * i + 2));
      v = __fmul_rn((float)(s - 393210), scale);
    } else {
      const unsigned long long u = fill_word(key, i) >> 40;
      const int m = lo_fixed + (int)((u * (unsigned long long)span_fixed) >> 24);
      v = __fmul_rn((float)m, 5.9604644775390625e-08f);   // 2^-24
    }
    out[i] = from_f32<T>(v);
  }
}

__global__ void random_fill_int_kernel(int* __restrict__ out, unsigned long long n, unsigned long long key) {
  unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x;
  const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
  for (; i < n; i += stride) out[i] = (int)(fill_word(key, i) >> 49);
}

// out: n elements of dtype (float32 / bfloat16; kind FILL_INT: int32 whatever dtype says).
// key: the 64 bits that stand for (seed, name).  scale: std / 65536 (normal).  lo_fixed, span_fixed:
// round(lo * 2^24), round((hi - lo) * 2^24) (uniform).
SHARPI_EXPORT int sharpi_random_fill(void* out, int dtype, long long n, unsigned long long key, int kind, float scale,
                                     int lo_fixed, int span_fixed, hipStream_t stream) {
  if (n <= 0) return SHARPI_OK;
  if (kind < FILL_NORMAL || kind > FILL_INT) return SHARPI_ERR_ARG;
  const long long nb = (n + 255) / 256;
  dim3 block(256), grid((unsigned)(nb > 262144 ? 262144 : nb));
  if (kind == FILL_INT)
    random_fill_int_kernel<<<grid, block, 0, stream>>>((int*)out, (unsigned long long)n, key);
  else if (dtype == DT_F32)
    random_fill_kernel<float><<<grid, block, 0, stream>>>((float*)out, (unsigned long long)n, key, kind, scale, lo_fixed,
                                                         span_fixed);
  else if (dtype == DT_BF16)
    random_fill_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)out, (unsigned long long)n, key, kind, scale,
                                                          lo_fixed, span_fixed);
  else
    return SHARPI_ERR_ARG;
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
