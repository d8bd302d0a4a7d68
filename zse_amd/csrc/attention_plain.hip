// Plain paged attention: one wave per (token, query head), every token of the
// step alike, whether it is a decoded token or one of a prompt portion.  Keys
// and values come only from the cache, through the request's block table.
//
//   s_j = softcap((q . k_j) * scale),   j in [lo, pos],  lo = max(0, pos - window + 1)
//   o   = sum_j softmax(s)_j v_j
//
// Keys are visited in tiles of 64 aligned to absolute positions, with a
// running maximum and sum, so the order of every sum depends on the token's
// position alone, not on how the step was cut.  Scores, softmax and the output
// sum are float.  The reference's decode kernel has the same shape of work
// (orchestrator/kernels.py:524-671: one block per (sequence, head), block
// table walk, three passes in shared memory); its prefill kernel reads
// contiguous K/V instead (:859-958) and never applies a window (:883).
#include "common.h"

#define AP_MAX_HD 256

__global__ __launch_bounds__(64) void attention_plain_kernel(
    const act_t* __restrict__ q, int q_stride, const act_t* __restrict__ kcache,
    const act_t* __restrict__ vcache, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ req_of_token, const int* __restrict__ positions,
    act_t* __restrict__ out, int nh, int nkv, int hd, int bs, float scale, float softcap,
    int window, int v_transposed) {
  __shared__ float sq[AP_MAX_HD];
  __shared__ float sp[64];
  __shared__ int spage[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int pos = positions[t];
  act_t* o = out + ((size_t)t * nh + h) * hd;
  if (pos < 0) {  // padding row
    for (int d = lane; d < hd; d += 64) o[d] = from_f32<act_t>(0.f);
    return;
  }
  const int r = req_of_token[t];
  const int kvh = h / (nh / nkv);
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int* table = block_table + (size_t)r * max_blocks;
  const act_t* qr = q + (size_t)t * q_stride + (size_t)h * hd;
  for (int d = lane; d < hd; d += 64) sq[d] = to_f32(qr[d]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[AP_MAX_HD / 64] = {};
  for (int j0 = (lo / 64) * 64; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j >= lo && j <= pos;
    float s = -INFINITY;
    int page = -1;
    if (valid) {
      page = table[j / bs];
      const act_t* kr = kcache + (((size_t)page * nkv + kvh) * bs + (j % bs)) * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; d++) dot = fmaf(sq[d], to_f32(kr[d]), dot);
      s = dot * scale;
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // m = -inf on the first tile: exp(-inf) = 0
    l = l * corr + wave_sum(p);
    m = m_new;
    __syncthreads();
    sp[lane] = p;
    spage[lane] = page;
    __syncthreads();
#pragma unroll
    for (int c = 0; c < AP_MAX_HD / 64; c++) {
      const int d = lane + c * 64;
      if (d < hd) {
        float a = acc[c] * corr;
        for (int jj = 0; jj < 64; jj++) {
          const int pg = spage[jj];
          if (pg < 0) continue;
          const size_t head_base = ((size_t)pg * nkv + kvh) * bs * hd;
          const size_t off = (j0 + jj) % bs;
          const act_t v = v_transposed ? vcache[head_base + (size_t)d * bs + off]
                                       : vcache[head_base + off * hd + d];
          a = fmaf(sp[jj], to_f32(v), a);
        }
        acc[c] = a;
      }
    }
  }
  const float inv = 1.f / l;
#pragma unroll
  for (int c = 0; c < AP_MAX_HD / 64; c++) {
    const int d = lane + c * 64;
    if (d < hd) o[d] = from_f32<act_t>(acc[c] * inv);
  }
}

// softcap <= 0: no cap; window <= 0: every earlier key is visible.  v_transposed: V is
// cached as [page][kv head][hd][bs] instead of [page][kv head][bs][hd].
extern "C" int zk_attention_plain(const void* q, int q_stride, const void* kcache, const void* vcache,
                                  const int* block_table, int max_blocks, const int* req_of_token,
                                  const int* positions, void* out, int T, int nh, int nkv, int hd,
                                  int bs, float scale, float softcap, int window, int v_transposed,
                                  void* stream) {
  ZK_REQUIRE(T >= 0 && nh > 0 && nkv > 0 && hd > 0 && bs > 0 && max_blocks > 0,
             "zk_attention_plain: bad sizes");
  ZK_REQUIRE(nh % nkv == 0, "zk_attention_plain: heads must be a multiple of kv heads");
  ZK_REQUIRE(hd <= AP_MAX_HD, "zk_attention_plain: head_dim above 256 is not supported");
  ZK_REQUIRE(nh <= 65535, "zk_attention_plain: too many heads");
  ZK_REQUIRE(q_stride >= nh * hd, "zk_attention_plain: q row stride too small");
  if (T == 0) return 0;
  dim3 grid(T, nh);
  attention_plain_kernel<<<grid, 64, 0, (hipStream_t)stream>>>(
      (const act_t*)q, q_stride, (const act_t*)kcache, (const act_t*)vcache, block_table, max_blocks,
      req_of_token, positions, (act_t*)out, nh, nkv, hd, bs, scale, softcap, window, v_transposed);
  return zk_launch_status("zk_attention_plain");
}
