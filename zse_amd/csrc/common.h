// Shared by every kernel file.  The library is built twice from the same
// sources: with ZSE_ACT_BF16=1 activations, weights and the cache are
// bfloat16; with ZSE_ACT_BF16=0 they are float and nothing is computed below
// 32 bits.  Residual stream, statistics, scores and logits are float in both.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <string>

#ifndef ZSE_ACT_BF16
#error "build with -DZSE_ACT_BF16=0 or 1"
#endif

#if ZSE_ACT_BF16
typedef __bf16 act_t;
#else
typedef float act_t;
#endif

#define ZSE_WAVE 64

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(__bf16 x) { return (float)x; }
template <typename T>
__device__ __forceinline__ T from_f32(float x);
template <>
__device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <>
__device__ __forceinline__ __bf16 from_f32<__bf16>(float x) { return (__bf16)x; }

// One rotation of a pair by an angle, written so that every kernel that rotates rounds alike
// (a token's values must not depend on how many tokens the step holds or on which kernel took
// it): a product rounded, then one fused multiply-add.
__device__ __forceinline__ void rotate_pair(float a, float b, float sn, float cs, float& ra, float& rb) {
  ra = __fmaf_rn(a, cs, -__fmul_rn(b, sn));
  rb = __fmaf_rn(b, cs, __fmul_rn(a, sn));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = ZSE_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, ZSE_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = ZSE_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, ZSE_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// ``scratch`` holds at least 17 floats of LDS.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (ZSE_WAVE - 1), wave = threadIdx.x / ZSE_WAVE;
  const int nw = (blockDim.x + ZSE_WAVE - 1) / ZSE_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  if (wave == 0) {
    float t = lane < nw ? scratch[lane] : 0.f;
    t = wave_sum(t);
    if (lane == 0) scratch[16] = t;
  }
  __syncthreads();
  return scratch[16];
}

// ---- host side ----
extern thread_local std::string zk_error;
int zk_fail(const char* msg);
int zk_launch_status(const char* what);

#define ZK_REQUIRE(cond, msg) \
  do {                        \
    if (!(cond)) return zk_fail(msg); \
  } while (0)

// The definitions behind the three declarations above and the two functions through which a
// caller asks a library for its last message and its storage type.  Each shared library has
// them once: the kernel libraries in elementwise.hip, a library of a part's own kernels in its
// own source file.
#define ZK_DEFINE_HOST_SIDE                                               \
  thread_local std::string zk_error;                                      \
  int zk_fail(const char* msg) {                                          \
    zk_error = msg;                                                       \
    return -1;                                                            \
  }                                                                       \
  int zk_launch_status(const char* what) {                                \
    hipError_t e = hipGetLastError();                                     \
    if (e != hipSuccess) {                                                \
      zk_error = std::string(what) + ": " + hipGetErrorString(e);         \
      return (int)e;                                                      \
    }                                                                     \
    return 0;                                                             \
  }                                                                       \
  extern "C" const char* zk_last_error() { return zk_error.c_str(); }     \
  extern "C" int zk_act_is_bf16() { return ZSE_ACT_BF16; }
