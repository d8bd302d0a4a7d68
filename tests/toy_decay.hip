// The toy mixer's recurrence as a kernel of its own: s = decay * s + x_t over a request's
// tokens of this step, y_t = s, the state kept between steps in the request's slot.  What
// differs from step to step (which rows are whose, which slot is whose) is read from device
// memory, so the launch can be captured and written down.
#include "common.h"
#include "packed_call.h"

ZK_DEFINE_HOST_SIDE

__global__ void toy_decay_kernel(const act_t* __restrict__ x, act_t* __restrict__ y, float* __restrict__ state,
                                 int slot_words, int offset_words, const int* __restrict__ q_start,
                                 const int* __restrict__ slot_of_req, int H, float decay) {
  const int r = blockIdx.x;
  const int t0 = q_start[r], t1 = q_start[r + 1];
  if (t1 <= t0) return;                       // a padding request of a captured step
  float* st = state + (size_t)slot_of_req[r] * slot_words + offset_words;
  for (int d = threadIdx.x; d < H; d += blockDim.x) {
#pragma clang fp contract(off)
    float s = st[d];
    for (int t = t0; t < t1; t++) {
      s = decay * s + to_f32(x[(size_t)t * H + d]);      // a product and a sum, each rounded, as the host does it
      y[(size_t)t * H + d] = from_f32<act_t>(s);
    }
    st[d] = s;
  }
}

extern "C" int zk_toy_decay(const void* x, void* y, float* state, int slot_words, int offset_words,
                            const int* q_start, const int* slot_of_req, int R, int H, float decay, void* stream) {
  ZK_REQUIRE(R >= 0 && H > 0 && slot_words >= offset_words + H, "zk_toy_decay: the state does not fit its slot");
  if (R == 0) return 0;
  toy_decay_kernel<<<R, 256, 0, (hipStream_t)stream>>>((const act_t*)x, (act_t*)y, state, slot_words, offset_words,
                                                       q_start, slot_of_req, H, decay);
  return zk_launch_status("zk_toy_decay");
}
ZK_PACKED(zk_toy_decay)
