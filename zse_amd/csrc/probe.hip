// Two probes of what the machine gives, for the measurement harness: how fast a kernel can
// stream memory, and how fast the matrix cores multiply bfloat16 when nothing else holds them
// up.  A roofline fraction against these says how far a kernel is from what is reachable;
// the fraction against the published peaks says how far from the data sheet.
#include "common.h"

typedef float f32x4_p __attribute__((ext_vector_type(4)));

// Every thread walks the buffer in 16-byte pieces, a whole grid's stride apart, four loads in
// flight, and folds what it read into one word; the word is stored only if it has a value it
// cannot have, which keeps the loads alive.
__global__ __launch_bounds__(256) void probe_read_kernel(const f32x4_p* __restrict__ src, size_t n16,
                                                        float* __restrict__ sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  f32x4_p a = {0.f, 0.f, 0.f, 0.f}, b = a, c = a, d = a;
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const f32x4_p v0 = __builtin_nontemporal_load(src + i), v1 = __builtin_nontemporal_load(src + i + stride);
    const f32x4_p v2 = __builtin_nontemporal_load(src + i + 2 * stride), v3 = __builtin_nontemporal_load(src + i + 3 * stride);
    a += v0; b += v1; c += v2; d += v3;
  }
  for (; i < n16; i += stride) a += src[i];
  a += b; c += d; a += c;
  const float t = a[0] + a[1] + a[2] + a[3];
  if (t == 1.2345678e-30f) sink[0] = t;
}

extern "C" int zk_probe_read(const void* src, size_t bytes, void* sink, void* stream) {
  ZK_REQUIRE(src != nullptr && sink != nullptr && bytes >= 16 && (uintptr_t)src % 16 == 0,
             "zk_probe_read: needs a 16-byte aligned buffer");
  probe_read_kernel<<<256 * 8, 256, 0, (hipStream_t)stream>>>((const f32x4_p*)src, bytes / 16, (float*)sink);
  return zk_launch_status("zk_probe_read");
}

#if ZSE_ACT_BF16
typedef __bf16 bf16x8_p __attribute__((ext_vector_type(8)));
typedef float f32x16_p __attribute__((ext_vector_type(16)));

// Eight independent chains of 32x32x16 products a wave, operands in registers: nothing but
// the matrix cores' own rate limits it.  2 * 32 * 32 * 16 flops a product.
__global__ __launch_bounds__(256) void probe_mfma_kernel(int iters, float* __restrict__ sink) {
  bf16x8_p x, y;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    x[e] = (__bf16)(float)((threadIdx.x + e) & 3);
    y[e] = (__bf16)(float)((threadIdx.x * 3 + e) & 1);
  }
  f32x16_p acc[8];
#pragma unroll
  for (int j = 0; j < 8; j++)
#pragma unroll
    for (int e = 0; e < 16; e++) acc[j][e] = 0.f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int j = 0; j < 8; j++) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, acc[j], 0, 0, 0);
  }
  float t = 0.f;
#pragma unroll
  for (int j = 0; j < 8; j++)
#pragma unroll
    for (int e = 0; e < 16; e++) t += acc[j][e];
  if (t == 1.2345678e-30f) sink[0] = t;
}

// Returns through *flops the number of floating-point operations the launch performs.
extern "C" int zk_probe_mfma_bf16(int iters, void* sink, double* flops, void* stream) {
  ZK_REQUIRE(iters > 0 && sink != nullptr, "zk_probe_mfma_bf16: bad arguments");
  const int blocks = 256 * 2;
  probe_mfma_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>(iters, (float*)sink);
  if (flops) *flops = (double)blocks * 4.0 * (double)iters * 8.0 * 2.0 * 32.0 * 32.0 * 16.0;
  return zk_launch_status("zk_probe_mfma_bf16");
}
#endif
