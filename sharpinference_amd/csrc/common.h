// Shared device helpers for the gfx950 kernels: storage types, conversions, wave reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define SHARPI_OK 0
#define SHARPI_ERR_ARG 1001   // a size or option the kernel does not take
#define SHARPI_ERR_LAUNCH 1002

#define SHARPI_CHECK_LAUNCH()                                   \
  do {                                                          \
    hipError_t e__ = hipGetLastError();                         \
    if (e__ != hipSuccess) return (int)e__;                     \
  } while (0)

#define SHARPI_EXPORT extern "C" __attribute__((visibility("default")))

constexpr int kWave = 64;

// bfloat16 as raw bits; conversions are round-to-nearest-even, NaN kept quiet.
struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v.bits) << 16);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
  return __uint_as_float(bits16 << 16);
}
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  bf16_t r;
  if ((u & 0x7fffffffu) > 0x7f800000u) {  // NaN
    r.bits = (uint16_t)((u >> 16) | 0x0040u);
    return r;
  }
  u += 0x7fffu + ((u >> 16) & 1u);
  r.bits = (uint16_t)(u >> 16);
  return r;
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return bf16_to_f32(v); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return f32_to_bf16(v); }

// eight consecutive elements as floats (p must be 16-byte aligned for bfloat16, 32 for float)
__device__ __forceinline__ void load8(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float* v) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  v[0] = bf16_bits_to_f32(a.x & 0xffffu); v[1] = bf16_bits_to_f32(a.x >> 16);
  v[2] = bf16_bits_to_f32(a.y & 0xffffu); v[3] = bf16_bits_to_f32(a.y >> 16);
  v[4] = bf16_bits_to_f32(a.z & 0xffffu); v[5] = bf16_bits_to_f32(a.z >> 16);
  v[6] = bf16_bits_to_f32(a.w & 0xffffu); v[7] = bf16_bits_to_f32(a.w >> 16);
}
__device__ __forceinline__ void store8(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8(bf16_t* p, const float* v) {
  uint4 o;
  o.x = (uint32_t)f32_to_bf16(v[0]).bits | ((uint32_t)f32_to_bf16(v[1]).bits << 16);
  o.y = (uint32_t)f32_to_bf16(v[2]).bits | ((uint32_t)f32_to_bf16(v[3]).bits << 16);
  o.z = (uint32_t)f32_to_bf16(v[4]).bits | ((uint32_t)f32_to_bf16(v[5]).bits << 16);
  o.w = (uint32_t)f32_to_bf16(v[6]).bits | ((uint32_t)f32_to_bf16(v[7]).bits << 16);
  *reinterpret_cast<uint4*>(p) = o;
}

// The gated unit of a feed-forward, one element: act(s g) * (s u), with the activation a code that
// the caller passes (shared with the Python side): SiLU x / (1 + exp(-x)), or GELU in its tanh form
// 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))).  One definition for the activation kernel and
// for the products that apply it in their epilogue, so both give the same bits.
enum : int { ACT_SILU = 1, ACT_GELU_TANH = 2 };
static inline __host__ __device__ bool act_known(int act) { return act == ACT_SILU || act == ACT_GELU_TANH; }
__device__ __forceinline__ float gated_f32(int act, float g, float u, float s, bool scaled) {
  if (scaled) {
    g *= s;
    u *= s;
  }
  if (act == ACT_GELU_TANH) {
    const float t = tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g));
    return (0.5f * g * (1.0f + t)) * u;
  }
  return (g / (1.0f + expf(-g))) * u;
}

// dtype codes shared with the Python side
enum : int { DT_F32 = 0, DT_BF16 = 1 };

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Block-wide sum for blocks of up to 1024 threads; `red` is LDS of >= 16 floats.
// The result is the same in every thread; the order of additions is fixed.
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wid = threadIdx.x >> 6;
  const int nw = (blockDim.x + kWave - 1) >> 6;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) red[wid] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += red[i];
  return t;
}

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
