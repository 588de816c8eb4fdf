// Two measuring kernels that say what this GPU gives a kernel of this library at best: a pure
// read of a large buffer (the memory roofline as it can be reached, beside the published one) and
// a loop of matrix-core products on registers (the bfloat16 compute roofline likewise).  The
// benchmark prints both beside the published peaks.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 peak_bf16x8;
typedef __attribute__((ext_vector_type(4))) float peak_f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned peak_u32x4;

// The buffer is read in chunks of 32 KB: a block of eight waves takes chunk (step * blocks + block)
// at every step, a wave 4 KB of it as four loads of 1 KB, all four on their way before any is
// used.  (Measured on MI355X: 6.8 to 7.0 TB/s with 2,048 blocks, whether a block's chunks lie side
// by side or a grid apart; more loads in flight per thread do not read faster.)  What is read
// is folded into one word per thread so that no load can be dropped.
constexpr int kReadBlocks = 2048;
__global__ __launch_bounds__(512) void peak_read_kernel(const peak_u32x4* __restrict__ buf, int steps, unsigned* __restrict__ sink) {
  const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
  unsigned acc = 0;
  for (int s = 0; s < steps; ++s) {
    const peak_u32x4* p = buf + ((size_t)s * gridDim.x + blockIdx.x) * 2048 + w * 256 + lane;
    peak_u32x4 v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = __builtin_nontemporal_load(p + j * 64);
#pragma unroll
    for (int j = 0; j < 4; ++j) acc ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;   // practically never: the store only keeps the loads alive
}

// The first (nbytes rounded down to a multiple of 64 MiB) bytes of buf are read once; the number
// of bytes read is returned through *read_bytes (host memory).  sink: one word of device memory.
SHARPI_EXPORT int sharpi_peak_read(const void* buf, long long nbytes, void* sink, long long* read_bytes, hipStream_t stream) {
  const long long per_step = (long long)kReadBlocks * 32768;
  const int steps = (int)(nbytes / per_step);
  if (steps <= 0 || !read_bytes) return SHARPI_ERR_ARG;
  *read_bytes = steps * per_step;
  peak_read_kernel<<<dim3(kReadBlocks), dim3(512), 0, stream>>>((const peak_u32x4*)buf, steps, (unsigned*)sink);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}

// Every wave issues `iters` rounds of eight independent 16x16x32 bfloat16 products on registers.
__global__ __launch_bounds__(256) void peak_mfma_kernel(float* __restrict__ sink, int iters) {
  peak_bf16x8 a, b;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    a[j] = (__bf16)(0.001f * (float)((threadIdx.x + j) & 7));
    b[j] = (__bf16)(0.002f * (float)((threadIdx.x * 3 + j) & 7));
  }
  peak_f32x4 acc[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) acc[t] = peak_f32x4{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int t = 0; t < 8; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[t], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int t = 0; t < 8; ++t) s += acc[t][0] + acc[t][1] + acc[t][2] + acc[t][3];
  if (s == 12345.678f) sink[0] = s;
}

// blocks of four waves; flops = blocks * 4 * iters * 8 * (2 * 16 * 16 * 32).
SHARPI_EXPORT int sharpi_peak_mfma(void* sink, int blocks, int iters, hipStream_t stream) {
  if (blocks <= 0 || iters <= 0) return SHARPI_ERR_ARG;
  peak_mfma_kernel<<<dim3(blocks), dim3(256), 0, stream>>>((float*)sink, iters);
  SHARPI_CHECK_LAUNCH();
  return SHARPI_OK;
}
