// Two probes of what this GPU delivers, for the benchmark line: the rate at which a kernel can stream
// memory (every compute unit reading 16 bytes per lane back to back) and the rate of the matrix cores on
// the instruction the kernels of this folder use (v_mfma_f32_16x16x32_bf16, operands in registers, four
// independent accumulators per wave). Roofline fractions are quoted against the published peaks; these
// measured figures stand beside them.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 probe_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float probe_f32x4;

__global__ void __launch_bounds__(256) read_probe_kernel(const uint4* __restrict__ src, size_t count, uint32_t* __restrict__ out) {
  uint32_t acc = 0;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
    const uint4 v = stream_load16(src + i);  // non-temporal: the faster way to read memory once (common.h)
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x9e3779b9u) out[0] = acc;  // keeps the loads alive; nearly never true
}

// Reads `bytes` (a multiple of 16) from src once. `out` is one word the kernel may write.
extern "C" int me_probe_read(const void* src, long long bytes, void* out, hipStream_t stream) {
  if (!src || !out || bytes < 16 || bytes % 16) return me_fail("me_probe_read: bytes=%lld", bytes);
  read_probe_kernel<<<256 * 8, 256, 0, stream>>>((const uint4*)src, (size_t)bytes / 16, (uint32_t*)out);
  return me_check_launch("me_probe_read");
}

__global__ void __launch_bounds__(256) mfma_probe_kernel(int iterations, float* __restrict__ out) {
  probe_bf16x8 a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(0.001f * (threadIdx.x + i));
    b[i] = (__bf16)(0.002f * (threadIdx.x - i));
  }
  probe_f32x4 c0 = {0, 0, 0, 0}, c1 = c0, c2 = c0, c3 = c0;
  for (int it = 0; it < iterations; ++it) {
    c0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c3, 0, 0, 0);
  }
  const float s = c0[0] + c1[1] + c2[2] + c3[3];
  if (s == 12345.678f) out[0] = s;
}

// `blocks` blocks of four waves, each wave issuing 4 * iterations products of 16 x 16 x 32: the launch performs
// blocks * 4 * 4 * iterations * 2 * 16 * 16 * 32 floating-point operations.
extern "C" int me_probe_mfma(int blocks, int iterations, void* out, hipStream_t stream) {
  if (!out || blocks < 1 || iterations < 1) return me_fail("me_probe_mfma: blocks=%d iterations=%d", blocks, iterations);
  mfma_probe_kernel<<<blocks, 256, 0, stream>>>(iterations, (float*)out);
  return me_check_launch("me_probe_mfma");
}
