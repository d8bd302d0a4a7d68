// A toy step between a mixer's q|k|v product and the rotation: every query and key head of
// every token is scaled to unit length, in place (the value heads stay).  One block a token.
#include "common.h"
#include "packed_call.h"

ZK_DEFINE_HOST_SIDE

__global__ __launch_bounds__(64) void toy_head_norm_kernel(act_t* __restrict__ qkv, int width, int heads, int hd) {
  act_t* row = qkv + (size_t)blockIdx.x * width;
  for (int h = 0; h < heads; h++) {
    act_t* v = row + (size_t)h * hd;
    float ss = 0.f;
    for (int d = threadIdx.x; d < hd; d += 64) ss += to_f32(v[d]) * to_f32(v[d]);
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss + 1e-12f);
    for (int d = threadIdx.x; d < hd; d += 64) v[d] = from_f32<act_t>(to_f32(v[d]) * inv);
  }
}

// qkv: [T, width] activations; the first ``heads`` heads of ``hd`` channels of each row are scaled.
extern "C" int zk_toy_head_norm(void* qkv, int T, int width, int heads, int hd, void* stream) {
  ZK_REQUIRE(T >= 0 && heads * hd <= width && hd > 0, "zk_toy_head_norm: heads do not fit the row");
  if (T == 0) return 0;
  toy_head_norm_kernel<<<T, 64, 0, (hipStream_t)stream>>>((act_t*)qkv, width, heads, hd);
  return zk_launch_status("zk_toy_head_norm");
}
ZK_PACKED(zk_toy_head_norm)
