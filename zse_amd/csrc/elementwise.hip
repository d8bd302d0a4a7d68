// Row-wise and element-wise kernels: embedding gather, RMS norms joined to the
// residual stream, gated activation, soft cap, rotary encoding with the write
// into the paged cache, dtype conversion and seeded random fill.
//
// Formulas follow the reference's kernels, which are fp16 strings compiled at
// run time (zse-engine/zse_engine/orchestrator/kernels.py): gather to an fp32
// stream :1789-1806, rsqrt(sum/H + eps) :1435-1465, rotate-half pairs
// :264-297, gelu-tanh gate :1678-1697, cap*tanh(x/cap) :1714-1727, the scatter
// of K and V into pages :961-1012.
#include "common.h"

#include <algorithm>

ZK_DEFINE_HOST_SIDE

// ------------------------------------------------------------------ embedding

// strip: the table is in the matrix-core kernels' strip layout (element (n, k) at
// ((n/16 * (H/32) + k/32) * 64 + (k%32)/8 * 16 + n%16) * 8 + k%8) instead of row-major.
template <typename W>
__global__ void embed_kernel(const W* __restrict__ table, const int* __restrict__ tokens,
                             float* __restrict__ out, float scale, int H, int V, int strip) {
  const int t = blockIdx.x;
  int tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= V ? V - 1 : tok);
  float* o = out + (size_t)t * H;
  if (strip) {
    const size_t base = (size_t)(tok >> 4) * (H / 32) * 512 + (tok & 15) * 8;
    for (int i = threadIdx.x; i < H; i += blockDim.x)
      o[i] = to_f32(table[base + (size_t)(i >> 5) * 512 + ((i & 31) >> 3) * 128 + (i & 7)]) * scale;
    return;
  }
  const W* row = table + (size_t)tok * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_f32(row[i]) * scale;
}

// ------------------------------------------------------------------ norms

__device__ __forceinline__ float gain(const float* w, int i, int unit_offset) {
  return unit_offset ? 1.f + w[i] : w[i];
}

// out[r] = N(x[rows ? rows[r] : r])
template <typename TIn>
__global__ void rmsnorm_kernel(const TIn* __restrict__ x, const int* __restrict__ rows,
                               const float* __restrict__ w, act_t* __restrict__ out, float eps,
                               int unit_offset, int H) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  const TIn* xr = x + (size_t)src * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = to_f32(xr[i]);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float rs = rsqrtf(ss / (float)H + eps);
  act_t* o = out + (size_t)r * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    o[i] = from_f32<act_t>(to_f32(xr[i]) * rs * gain(w, i, unit_offset));
}

// One value of the sublayer's output.  parts > 0: it still lies in `parts` float planes of
// [rows, H] partial sums (a matrix product that split K and left the adding up to its reader);
// they are added in order and rounded to the activation type, which is what the product's own
// joining kernel would have stored.
__device__ __forceinline__ float sub_value(const void* __restrict__ sub, int parts, size_t plane, size_t at) {
  if (parts <= 0) return to_f32(((const act_t*)sub)[at]);
  float x = ((const float*)sub)[at];
  for (int p = 1; p < parts; p++) x += ((const float*)sub)[p * plane + at];
  return to_f32(from_f32<act_t>(x));
}

// h += N_post(sub)  (w_post null: h += sub);  then, if w_next: out = N_next(h)
__global__ void norm_add_norm_kernel(const void* __restrict__ sub, int parts, const float* __restrict__ w_post,
                                     float eps_post, int uo_post, float* __restrict__ h,
                                     const float* __restrict__ w_next, float eps_next, int uo_next,
                                     act_t* __restrict__ out, int H) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const size_t plane = (size_t)gridDim.x * H, row = (size_t)r * H;
  float* hr = h + (size_t)r * H;
  float rs = 1.f;
  if (w_post) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      float v = sub_value(sub, parts, plane, row + i);
      ss += v * v;
    }
    ss = block_sum(ss, red);
    rs = rsqrtf(ss / (float)H + eps_post);
  }
  float ss2 = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = sub_value(sub, parts, plane, row + i);
    if (w_post) v = v * rs * gain(w_post, i, uo_post);
    v = hr[i] + v;
    hr[i] = v;
    ss2 += v * v;
  }
  if (!w_next) return;
  ss2 = block_sum(ss2, red);
  const float rs2 = rsqrtf(ss2 / (float)H + eps_next);
  act_t* o = out + (size_t)r * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x)  // each thread re-reads what it wrote
    o[i] = from_f32<act_t>(hr[i] * rs2 * gain(w_next, i, uo_next));
}

// Single-pass variants for rows of up to 8192 values in whole groups of four: a
// thread keeps its part of the row in registers (four values at tid*4 + j*1024), so the
// row is read once and the two block sums are the only synchronisation.
#define NF_MAXV 8

template <typename TIn>
__device__ __forceinline__ void load4(const TIn* p, float v[4]);
template <>
__device__ __forceinline__ void load4<float>(const float* p, float v[4]) {
  const float4 t = *(const float4*)p;
  v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
template <>
__device__ __forceinline__ void load4<__bf16>(const __bf16* p, float v[4]) {
  typedef __bf16 b4 __attribute__((ext_vector_type(4)));
  const b4 t = *(const b4*)p;
#pragma unroll
  for (int i = 0; i < 4; i++) v[i] = (float)t[i];
}
__device__ __forceinline__ void store4(float* p, const float v[4]) {
  *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store4(__bf16* p, const float v[4]) {
  typedef __bf16 b4 __attribute__((ext_vector_type(4)));
  b4 t;
#pragma unroll
  for (int i = 0; i < 4; i++) t[i] = (__bf16)v[i];
  *(b4*)p = t;
}

template <typename TIn>
__global__ __launch_bounds__(256) void rmsnorm_fast_kernel(const TIn* __restrict__ x,
                                                           const int* __restrict__ rows,
                                                           const float* __restrict__ w,
                                                           act_t* __restrict__ out, float eps,
                                                           int unit_offset, int H) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const TIn* xr = x + (size_t)(rows ? rows[r] : r) * H;
  float v[NF_MAXV][4];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NF_MAXV; j++) {
    const int i = threadIdx.x * 4 + j * 1024;
    if (i < H) {
      load4<TIn>(xr + i, v[j]);
#pragma unroll
      for (int e = 0; e < 4; e++) ss += v[j][e] * v[j][e];
    }
  }
  ss = block_sum(ss, red);
  const float rs = rsqrtf(ss / (float)H + eps);
  act_t* o = out + (size_t)r * H;
#pragma unroll
  for (int j = 0; j < NF_MAXV; j++) {
    const int i = threadIdx.x * 4 + j * 1024;
    if (i < H) {
      float g[4], y[4];
      load4<float>(w + i, g);
#pragma unroll
      for (int e = 0; e < 4; e++) y[e] = v[j][e] * rs * (unit_offset ? 1.f + g[e] : g[e]);
      store4(o + i, y);
    }
  }
}

// MAXV: vectors of four a thread holds (4 x 256 x MAXV >= H); small rows take fewer registers
// and more rows share a CU.
template <int MAXV>
__global__ __launch_bounds__(256) void norm_add_norm_fast_kernel(
    const void* __restrict__ sub, int parts, const float* __restrict__ w_post, float eps_post, int uo_post,
    float* __restrict__ h, const float* __restrict__ w_next, float eps_next, int uo_next,
    act_t* __restrict__ out, int H) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const act_t* s = (const act_t*)sub + (size_t)r * H;
  const float* sf = (const float*)sub + (size_t)r * H;      // parts > 0: planes of [rows, H] partial sums
  const size_t plane = (size_t)gridDim.x * H;
  float* hr = h + (size_t)r * H;
  // every load is issued before the first sum is needed: one trip to memory, not three
  float v[MAXV][4], hv[MAXV][4], gp[MAXV][4], gn[MAXV][4];
  float ss = 0.f;
  if constexpr (MAXV <= 3) {
    // narrow rows: a vector's planes are summed where it is loaded (fewer registers; measured
    // faster than the arrangement below at 2,304 columns)
#pragma unroll
    for (int j = 0; j < MAXV; j++) {
      const int i = threadIdx.x * 4 + j * 1024;
      if (i < H) {
        if (parts <= 0) {
          load4<act_t>(s + i, v[j]);
        } else {
          load4<float>(sf + i, v[j]);
          // four planes a turn, their loads issued together; a plane past the last is read from
          // the last and not added
          for (int p0 = 1; p0 < parts; p0 += 4) {
            float t[4][4];
#pragma unroll
            for (int q = 0; q < 4; q++) load4<float>(sf + (size_t)min(p0 + q, parts - 1) * plane + i, t[q]);
#pragma unroll
            for (int q = 0; q < 4; q++)
              if (p0 + q < parts) {
#pragma unroll
                for (int e = 0; e < 4; e++) v[j][e] += t[q][e];
              }
          }
#pragma unroll
          for (int e = 0; e < 4; e++) v[j][e] = to_f32(from_f32<act_t>(v[j][e]));
        }
        load4<float>(hr + i, hv[j]);
        if (w_post) load4<float>(w_post + i, gp[j]);
        if (w_next) load4<float>(w_next + i, gn[j]);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < MAXV; j++) {
      const int i = threadIdx.x * 4 + j * 1024;
      if (i < H) {
        if (parts <= 0) load4<act_t>(s + i, v[j]);
        else load4<float>(sf + i, v[j]);
        load4<float>(hr + i, hv[j]);
        if (w_post) load4<float>(w_post + i, gp[j]);
        if (w_next) load4<float>(w_next + i, gn[j]);
      }
    }
    if (parts > 0) {
      // wide rows: four planes a turn, the loads of the thread's whole share of the row issued
      // together, so that a turn is one trip to memory whatever the width.  A plane past the
      // last is read from the last and not added; the planes are added in their order.
      for (int p0 = 1; p0 < parts; p0 += 4) {
        float t[MAXV][4][4];
#pragma unroll
        for (int j = 0; j < MAXV; j++) {
          const int i = threadIdx.x * 4 + j * 1024;
          if (i < H) {
#pragma unroll
            for (int q = 0; q < 4; q++) load4<float>(sf + (size_t)min(p0 + q, parts - 1) * plane + i, t[j][q]);
          }
        }
#pragma unroll
        for (int j = 0; j < MAXV; j++) {
          const int i = threadIdx.x * 4 + j * 1024;
          if (i < H) {
#pragma unroll
            for (int q = 0; q < 4; q++)
              if (p0 + q < parts) {
#pragma unroll
                for (int e = 0; e < 4; e++) v[j][e] += t[j][q][e];
              }
          }
        }
      }
#pragma unroll
      for (int j = 0; j < MAXV; j++)
        if (threadIdx.x * 4 + j * 1024 < H) {
#pragma unroll
          for (int e = 0; e < 4; e++) v[j][e] = to_f32(from_f32<act_t>(v[j][e]));
        }
    }
  }
#pragma unroll
  for (int j = 0; j < MAXV; j++) {
    const int i = threadIdx.x * 4 + j * 1024;
    if (i < H) {
#pragma unroll
      for (int e = 0; e < 4; e++) ss += v[j][e] * v[j][e];
    }
  }
  float rs = 1.f;
  if (w_post) {
    ss = block_sum(ss, red);
    rs = rsqrtf(ss / (float)H + eps_post);
  }
  float ss2 = 0.f;
#pragma unroll
  for (int j = 0; j < MAXV; j++) {
    const int i = threadIdx.x * 4 + j * 1024;
    if (i < H) {
#pragma unroll
      for (int e = 0; e < 4; e++) {
        float t = v[j][e];
        if (w_post) t = t * rs * (uo_post ? 1.f + gp[j][e] : gp[j][e]);
        t = hv[j][e] + t;
        v[j][e] = t;
        ss2 += t * t;
      }
      store4(hr + i, v[j]);
    }
  }
  if (!w_next) return;
  ss2 = block_sum(ss2, red);
  const float rs2 = rsqrtf(ss2 / (float)H + eps_next);
  act_t* o = out + (size_t)r * H;
#pragma unroll
  for (int j = 0; j < MAXV; j++) {
    const int i = threadIdx.x * 4 + j * 1024;
    if (i < H) {
      float y[4];
#pragma unroll
      for (int e = 0; e < 4; e++) y[e] = v[j][e] * rs2 * (uo_next ? 1.f + gn[j][e] : gn[j][e]);
      store4(o + i, y);
    }
  }
}

// The same for the few rows of a decode step (up to 64 rows of 2,048 to 8,192 values): 1,024
// threads a row instead of 256, so a thread holds one or two vectors (4 x 1024 x MAXV >= H) and can
// ask for all planes of partial sums at once, eight a turn.  With so few rows the kernel's time is
// its trips to memory and its two block sums, not its bytes: 8 rows of 4,608 values that come as
// eight planes (27B shapes) 2.9 us less a launch, a decode step at batch 8 of 2B shapes 2.46 -> 2.42
// ms, of 9B shapes (14 layers) 2.47 -> 2.40 ms, 2B shapes at batch 32 4.51 -> 4.40 ms; with 2,048
// rows it loses (the 2B prefill 12.43 -> 12.75 ms), so more than 64 rows stay with the kernel
// above.  The sums of the planes are the same bits; the two row sums are added up in another
// order than by 256 threads, so which of the two kernels serves a launch depends on the rows and
// the width alone, never on whether planes come.
template <int MAXV>
__global__ __launch_bounds__(1024) void norm_add_norm_wide_kernel(
    const void* __restrict__ sub, int parts, const float* __restrict__ w_post, float eps_post, int uo_post,
    float* __restrict__ h, const float* __restrict__ w_next, float eps_next, int uo_next,
    act_t* __restrict__ out, int H) {
  __shared__ float red[17];
  const int r = blockIdx.x;
  const act_t* s = (const act_t*)sub + (size_t)r * H;
  const float* sf = (const float*)sub + (size_t)r * H;
  const size_t plane = (size_t)gridDim.x * H;
  float* hr = h + (size_t)r * H;
  float v[MAXV][4], hv[MAXV][4], gp[MAXV][4], gn[MAXV][4];
#pragma unroll
  for (int j = 0; j < MAXV; j++) {
    const int i = threadIdx.x * 4 + j * 4096;
    if (i < H) {
      if (parts <= 0) load4<act_t>(s + i, v[j]);
      else load4<float>(sf + i, v[j]);
      load4<float>(hr + i, hv[j]);
      if (w_post) load4<float>(w_post + i, gp[j]);
      if (w_next) load4<float>(w_next + i, gn[j]);
    }
  }
  if (parts > 0) {
    // a plane past the last is read from the last and not added; the planes are added in order
    for (int p0 = 1; p0 < parts; p0 += 8) {
      float t[MAXV][8][4];
#pragma unroll
      for (int j = 0; j < MAXV; j++) {
        const int i = threadIdx.x * 4 + j * 4096;
        if (i < H) {
#pragma unroll
          for (int q = 0; q < 8; q++) load4<float>(sf + (size_t)min(p0 + q, parts - 1) * plane + i, t[j][q]);
        }
      }
#pragma unroll
      for (int j = 0; j < MAXV; j++) {
        if (threadIdx.x * 4 + j * 4096 < H) {
#pragma unroll
          for (int q = 0; q < 8; q++)
            if (p0 + q < parts) {
#pragma unroll
              for (int e = 0; e < 4; e++) v[j][e] += t[j][q][e];
            }
        }
      }
    }
#pragma unroll
    for (int j = 0; j < MAXV; j++)
      if (threadIdx.x * 4 + j * 4096 < H) {
#pragma unroll
        for (int e = 0; e < 4; e++) v[j][e] = to_f32(from_f32<act_t>(v[j][e]));
      }
  }
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < MAXV; j++)
    if (threadIdx.x * 4 + j * 4096 < H) {
#pragma unroll
      for (int e = 0; e < 4; e++) ss += v[j][e] * v[j][e];
    }
  float rs = 1.f;
  if (w_post) {
    ss = block_sum(ss, red);
    rs = rsqrtf(ss / (float)H + eps_post);
  }
  float ss2 = 0.f;
#pragma unroll
  for (int j = 0; j < MAXV; j++) {
    const int i = threadIdx.x * 4 + j * 4096;
    if (i < H) {
#pragma unroll
      for (int e = 0; e < 4; e++) {
        float t = v[j][e];
        if (w_post) t = t * rs * (uo_post ? 1.f + gp[j][e] : gp[j][e]);
        t = hv[j][e] + t;
        v[j][e] = t;
        ss2 += t * t;
      }
      store4(hr + i, v[j]);
    }
  }
  if (!w_next) return;
  ss2 = block_sum(ss2, red);
  const float rs2 = rsqrtf(ss2 / (float)H + eps_next);
  act_t* o = out + (size_t)r * H;
#pragma unroll
  for (int j = 0; j < MAXV; j++) {
    const int i = threadIdx.x * 4 + j * 4096;
    if (i < H) {
      float y[4];
#pragma unroll
      for (int e = 0; e < 4; e++) y[e] = v[j][e] * rs2 * (uo_next ? 1.f + gn[j][e] : gn[j][e]);
      store4(o + i, y);
    }
  }
}

// ------------------------------------------------------------------ gated activation

__device__ __forceinline__ float gelu_tanh(float g) {
  const float k = 0.7978845608028654f;
  return 0.5f * g * (1.0f + tanhf(k * (g + 0.044715f * g * g * g)));
}
__device__ __forceinline__ float silu(float g) { return g / (1.0f + expf(-g)); }

// gu: [T, 2I], gate in columns [0, I), up in [I, 2I)
__global__ void gated_act_kernel(const act_t* __restrict__ gu, act_t* __restrict__ out, int I,
                                 int act) {
  const int t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= I) return;
  const float g = to_f32(gu[(size_t)t * 2 * I + i]);
  const float u = to_f32(gu[(size_t)t * 2 * I + I + i]);
  const float a = act == 0 ? gelu_tanh(g) : silu(g);
  out[(size_t)t * I + i] = from_f32<act_t>(a * u);
}

__global__ void softcap_kernel(float* __restrict__ z, size_t n, float cap) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) z[i] = cap * tanhf(z[i] / cap);
}

// ------------------------------------------------------------------ rotary + cache write

// qkv: [T, (nh + 2 nkv) hd] rows of [q | k | v].  q is rotated in place; k is
// rotated and stored, v is stored, at slot = page * bs + offset of the token
// (slot < 0: nothing stored).  Cache layout per layer: K [page][kv head][bs][hd];
// V the same, or transposed [page][kv head][hd][bs] when v_transposed is set.

// Where the rows come from: the matrix itself, or (sums > 0) that many planes of [T, width]
// float partial sums of a product that split K, added in order and rounded to the activation
// type, which is what the product's own joining kernel would have stored.  q then goes to qkv.
struct QkvSource {
  const act_t* rows;
  const float* planes;
  int sums;
  size_t plane;
  __device__ __forceinline__ float at(size_t i) const {
    if (sums <= 0) return to_f32(rows[i]);
    float x = planes[i];
    for (int p = 1; p < sums; p++) x += planes[p * plane + i];
    return to_f32(from_f32<act_t>(x));
  }
  __device__ __forceinline__ void at4(size_t i, float v[4]) const {
    if (sums <= 0) {
      load4<act_t>(rows + i, v);
      return;
    }
    load4<float>(planes + i, v);
    for (int p = 1; p < sums; p++) {
      float w[4];
      load4<float>(planes + p * plane + i, w);
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] += w[e];
    }
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] = to_f32(from_f32<act_t>(v[e]));
  }
};

__global__ void rope_cache_write_kernel(act_t* __restrict__ qkv, QkvSource from, const int* __restrict__ positions,
                                        const int* __restrict__ slot_map,
                                        const float* __restrict__ inv_freq, int rotary_dim,
                                        act_t* __restrict__ kcache, act_t* __restrict__ vcache,
                                        int nh, int nkv, int hd, int bs, int v_transposed) {
  const int t = blockIdx.x;
  const int head = blockIdx.y;  // [0,nh): q; [nh, nh+nkv): k; [nh+nkv, nh+2nkv): v
  const size_t at = (size_t)t * (nh + 2 * nkv) * hd + (size_t)head * hd;
  act_t* q_out = qkv + at;
  const float pos = (float)positions[t];
  const int half = rotary_dim / 2;
  const int slot = slot_map ? slot_map[t] : -1;
  act_t* dst = nullptr;
  if (head >= nh && slot >= 0) {
    const int kvh = (head - nh) % nkv;
    act_t* base = head < nh + nkv ? kcache : vcache;
    const size_t page = slot / bs, off = slot % bs;
    if (head >= nh + nkv && v_transposed) {
      act_t* vt = vcache + (page * nkv + kvh) * (size_t)hd * bs + off;
      for (int i = threadIdx.x; i < hd; i += blockDim.x) vt[(size_t)i * bs] = from_f32<act_t>(from.at(at + i));
      return;
    }
    dst = base + ((page * nkv + kvh) * bs + off) * hd;
  }
  if (head < nh + nkv) {
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
      const float ang = pos * inv_freq[i];
      float sn, cs;
      sincosf(ang, &sn, &cs);
      const float a = from.at(at + i), b = from.at(at + i + half);
      float fa, fb;
      rotate_pair(a, b, sn, cs, fa, fb);
      const act_t ra = from_f32<act_t>(fa), rb = from_f32<act_t>(fb);
      if (head < nh) {
        q_out[i] = ra;
        q_out[i + half] = rb;
      } else if (dst) {
        dst[i] = ra;
        dst[i + half] = rb;
      }
    }
    if (head < nh) {
      if (from.sums > 0)      // what is not rotated still has to reach qkv
        for (int i = rotary_dim + threadIdx.x; i < hd; i += blockDim.x) q_out[i] = from_f32<act_t>(from.at(at + i));
    } else if (dst) {
      for (int i = rotary_dim + threadIdx.x; i < hd; i += blockDim.x) dst[i] = from_f32<act_t>(from.at(at + i));
    }
  } else if (dst) {
    for (int i = threadIdx.x; i < hd; i += blockDim.x) dst[i] = from_f32<act_t>(from.at(at + i));
  }
}

// The same for the usual case (rotation over the whole head, head_dim a multiple of 8 and at
// most 512): one block a token, the sines and cosines of the token's angles computed once for
// all heads, four values a load.
#define ROPE_MAX_HALF 256
__global__ __launch_bounds__(256) void rope_cache_write_token_kernel(
    act_t* __restrict__ qkv, QkvSource from, const int* __restrict__ positions, const int* __restrict__ slot_map,
    const float* __restrict__ inv_freq, act_t* __restrict__ kcache, act_t* __restrict__ vcache, int nh,
    int nkv, int hd, int bs, int v_transposed) {
  __shared__ float s_sin[ROPE_MAX_HALF], s_cos[ROPE_MAX_HALF];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int half = hd / 2;
  const float pos = (float)positions[t];
  const int slot = slot_map ? slot_map[t] : -1;
  for (int i = tid; i < half; i += 256) sincosf(pos * inv_freq[i], &s_sin[i], &s_cos[i]);
  __syncthreads();
  const size_t width = (size_t)(nh + 2 * nkv) * hd, row_at = (size_t)t * width;
  act_t* row = qkv + row_at;
  const size_t page = slot >= 0 ? slot / bs : 0, off = slot >= 0 ? slot % bs : 0;
  // q and k heads: pieces of four pairs (i, i + half)
  const int ppr = half / 4;
  for (int it = tid; it < (nh + nkv) * ppr; it += 256) {
    const int head = it / ppr, i = (it % ppr) * 4;
    float a[4], b[4], ra[4], rb[4];
    from.at4(row_at + (size_t)head * hd + i, a);
    from.at4(row_at + (size_t)head * hd + i + half, b);
#pragma unroll
    for (int e = 0; e < 4; e++) {
      rotate_pair(a[e], b[e], s_sin[i + e], s_cos[i + e], ra[e], rb[e]);
    }
    if (head < nh) {
      store4(row + (size_t)head * hd + i, ra);
      store4(row + (size_t)head * hd + i + half, rb);
    } else if (slot >= 0) {
      act_t* dst = kcache + ((page * nkv + (head - nh)) * bs + off) * hd;
      store4(dst + i, ra);
      store4(dst + i + half, rb);
    }
  }
  // v heads.  Transposed cache: eight tokens in a row of the step whose slots are eight in a
  // row of one page (a prompt portion) go out together, 8 values of a channel per store, each
  // of the eight blocks an eighth of the channels; other tokens are written value by value.
  if (v_transposed) {
    const int tl = t - t % 8;
    bool together = bs % 8 == 0 && tl + 7 < (int)gridDim.x && slot_map != nullptr;
    int slot0 = -1;
    if (together) {
      slot0 = slot_map[tl];
      together = slot0 >= 0 && slot0 % 8 == 0;
      for (int e = 1; together && e < 8; e++) together = slot_map[tl + e] == slot0 + e;
    }
    if (together) {
      // the eight tokens' blocks share the (kv head, channel) pairs among them, an eighth each
      typedef act_t av8 __attribute__((ext_vector_type(8)));
      const size_t page0 = slot0 / bs, off0 = slot0 % bs;
      const size_t row0 = (size_t)tl * width;
      const int items = nkv * hd, mine = (items + 7) / 8, first = (t - tl) * mine;
      for (int it = first + tid; it < min(first + mine, items); it += 256) {
        const int kvh = it / hd, d = it % hd;
        const size_t src = row0 + (size_t)(nh + nkv + kvh) * hd + d;
        av8 v;
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = from_f32<act_t>(from.at(src + (size_t)e * width));
        *(av8*)(vcache + ((page0 * nkv + kvh) * (size_t)hd + d) * bs + off0) = v;
      }
      return;
    }
  }
  if (slot < 0) return;
  for (int it = tid; it < nkv * (hd / 4); it += 256) {
    const int kvh = it / (hd / 4), d = (it % (hd / 4)) * 4;
    float v[4];
    from.at4(row_at + (size_t)(nh + nkv + kvh) * hd + d, v);
    if (v_transposed) {
      act_t* vt = vcache + ((page * nkv + kvh) * (size_t)hd + d) * bs + off;
#pragma unroll
      for (int e = 0; e < 4; e++) vt[(size_t)e * bs] = from_f32<act_t>(v[e]);
    } else {
      store4(vcache + ((page * nkv + kvh) * bs + off) * hd + d, v);
    }
  }
}

__global__ void feed_tokens_kernel(int* __restrict__ tokens, const int* __restrict__ ids, const int* __restrict__ dst,
                                   const int* __restrict__ src, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) tokens[dst[i]] = ids[src[i]];
}

// ------------------------------------------------------------------ conversion, fill

// src_tag: 0 = float32, 1 = bfloat16, 2 = float16
template <typename D>
__global__ void convert_kernel(const void* __restrict__ src, int src_tag, D* __restrict__ dst,
                               size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float v;
  if (src_tag == 0) v = ((const float*)src)[i];
  else if (src_tag == 1) v = (float)((const __bf16*)src)[i];
  else v = (float)((const _Float16*)src)[i];
  dst[i] = from_f32<D>(v);
}

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// Normal(mean, std) values as a pure function of (seed, stream, element index), by Box-Muller.
// The host can make the very same values (zse_amd/weights/normal.py): logarithm, sine and cosine
// are written out here as short sums of single correctly rounded float operations (no library
// call, no fused multiply-add: contraction is off in these functions), so that NumPy, doing the
// same operations in the same order, gets the same bits.
//
//   r = mix64(mix64(seed ^ stream * C) + pair);  k = (r >> 40) + 1 in [1, 2^24];  j = (r >> 8) & (2^24 - 1)
//   u1 = k / 2^24,  angle = 2 pi j / 2^24
//   element 2 pair = mean + std * sqrt(-2 ln u1) * cos(angle), element 2 pair + 1 the same with sin

// ln(k / 2^24) for an integer k in [1, 2^24]: k = m * 2^e with m in [1/sqrt2, sqrt2),
// ln m = 2 atanh(s) = 2 s (1 + s^2/3 + s^4/5 + s^6/7 + s^8/9), s = (m - 1) / (m + 1).
__device__ __forceinline__ float exact_log_u24(uint32_t k) {
#pragma clang fp contract(off)
  int e = 31 - __clz((int)k);
  float m = (float)k * __int_as_float((127 - e) << 23);       // k / 2^e, exact: k has at most 24 bits
  if (m > 1.41421354f) {
    m = m * 0.5f;
    e += 1;
  }
  const float s = (m - 1.0f) / (m + 1.0f);
  const float s2 = s * s;
  float p = 0.111111112f;
  p = p * s2 + 0.142857149f;
  p = p * s2 + 0.2f;
  p = p * s2 + 0.333333343f;
  p = p * s2 + 1.0f;
  const float lm = (2.0f * s) * p;
  return (float)(e - 24) * 0.693147182f + lm;
}

// sin and cos of 2 pi j / 2^24 for an integer j in [0, 2^24): the quarter turn and the fold to
// [0, pi/4] are integer work, the rest two short polynomials in x = r * (pi / 2^23), r <= 2^21.
__device__ __forceinline__ void exact_sincos_u24(uint32_t j, float& sn, float& cs) {
#pragma clang fp contract(off)
  const uint32_t q = j >> 22;
  uint32_t r = j & 0x3FFFFFu;
  const bool fold = r > 0x200000u;
  if (fold) r = 0x400000u - r;
  const float x = (float)r * 3.74507039e-07f;                 // pi / 2 / 2^22
  const float x2 = x * x;
  float ps = 2.75573188e-06f;                                 // 1/9!
  ps = ps * x2 + -1.98412701e-04f;                            // -1/7!
  ps = ps * x2 + 8.33333377e-03f;                             // 1/5!
  ps = ps * x2 + -1.66666672e-01f;                            // -1/3!
  const float s0 = x + (x * x2) * ps;
  float pc = -2.75573188e-07f;                                // -1/10!
  pc = pc * x2 + 2.48015876e-05f;                             // 1/8!
  pc = pc * x2 + -1.38888892e-03f;                            // -1/6!
  pc = pc * x2 + 4.16666679e-02f;                             // 1/4!
  pc = pc * x2 + -0.5f;
  const float c0 = 1.0f + x2 * pc;
  const float s1 = fold ? c0 : s0, c1 = fold ? s0 : c0;       // sin(pi/2 - x) = cos x
  switch (q) {
    case 0: sn = s1; cs = c1; break;
    case 1: sn = c1; cs = -s1; break;
    case 2: sn = -s1; cs = -c1; break;
    default: sn = -c1; cs = s1; break;
  }
}

template <typename D>
__global__ void fill_normal_kernel(D* __restrict__ dst, size_t n, uint64_t seed, uint64_t stream,
                                   float mean, float std) {
#pragma clang fp contract(off)
  size_t pair = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t i = pair * 2;
  if (i >= n) return;
  uint64_t r = mix64(mix64(seed ^ (stream * 0xD1342543DE82EF95ull)) + pair);
  const uint32_t k = (uint32_t)(r >> 40) + 1u;
  const uint32_t j = (uint32_t)((r >> 8) & 0xFFFFFFu);
  const float rad = sqrtf(-2.0f * exact_log_u24(k));     // correctly rounded, as NumPy's
  float sn, cs;
  exact_sincos_u24(j, sn, cs);
  const float a = std * (rad * cs), b = std * (rad * sn);
  dst[i] = from_f32<D>(mean + a);
  if (i + 1 < n) dst[i + 1] = from_f32<D>(mean + b);
}

__global__ void zero_kernel(uint32_t* __restrict__ p, size_t n_words) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_words) p[i] = 0u;
}

// Clears whole pages in several slabs at once: block (x, y) clears page pages.id[x] of slab y.
// A slab is an array of pages of slab_page_bytes[y] bytes each (a multiple of 16), so a page id
// names the same place in each of them.  The ids come by value with the launch.
#define ZERO_PAGES_MOST 64
struct PageIds {
  int n;
  int id[ZERO_PAGES_MOST];
};
__global__ __launch_bounds__(256) void zero_pages_kernel(void* const* __restrict__ slabs,
                                                         const unsigned long long* __restrict__ slab_page_bytes,
                                                         PageIds pages) {
  const unsigned long long nbytes = slab_page_bytes[blockIdx.y];
  uint4* dst = (uint4*)((char*)slabs[blockIdx.y] + (size_t)pages.id[blockIdx.x] * nbytes);
  const uint4 z = make_uint4(0u, 0u, 0u, 0u);
  for (size_t i = threadIdx.x; i < nbytes / 16; i += 256) dst[i] = z;
}

// ------------------------------------------------------------------ C interface

extern "C" {

int zk_embed(const void* table, const int* tokens, float* out, float scale, int T, int H, int V,
             int strip, void* stream) {
  ZK_REQUIRE(T >= 0 && H > 0 && V > 0, "zk_embed: bad sizes");
  ZK_REQUIRE(!strip || H % 32 == 0, "zk_embed: strip layout needs H % 32 == 0");
  if (T == 0) return 0;
  embed_kernel<act_t><<<T, 256, 0, (hipStream_t)stream>>>((const act_t*)table, tokens, out, scale, H, V, strip);
  return zk_launch_status("zk_embed");
}

// x_is_f32: input rows are the float residual stream, else activations.
int zk_rmsnorm(const void* x, int x_is_f32, const int* rows, const float* w, void* out, float eps,
               int unit_offset, int R, int H, void* stream) {
  ZK_REQUIRE(R >= 0 && H > 0, "zk_rmsnorm: bad sizes");
  if (R == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (H % 4 == 0 && H <= NF_MAXV * 1024) {
    if (x_is_f32)
      rmsnorm_fast_kernel<float><<<R, 256, 0, s>>>((const float*)x, rows, w, (act_t*)out, eps, unit_offset, H);
    else
      rmsnorm_fast_kernel<act_t><<<R, 256, 0, s>>>((const act_t*)x, rows, w, (act_t*)out, eps, unit_offset, H);
    return zk_launch_status("zk_rmsnorm");
  }
  if (x_is_f32)
    rmsnorm_kernel<float><<<R, 256, 0, s>>>((const float*)x, rows, w, (act_t*)out, eps, unit_offset, H);
  else
    rmsnorm_kernel<act_t><<<R, 256, 0, s>>>((const act_t*)x, rows, w, (act_t*)out, eps, unit_offset, H);
  return zk_launch_status("zk_rmsnorm");
}

// sub_parts > 0: sub holds that many float planes of [T, H] partial sums instead of [T, H]
// values of the activation type (see sub_value).
int zk_norm_add_norm(const void* sub, int sub_parts, const float* w_post, float eps_post, int uo_post, float* h,
                     const float* w_next, float eps_next, int uo_next, void* out, int T, int H,
                     void* stream) {
  ZK_REQUIRE(T >= 0 && H > 0 && sub_parts >= 0, "zk_norm_add_norm: bad sizes");
  ZK_REQUIRE(w_next == nullptr || out != nullptr, "zk_norm_add_norm: next norm without output");
  if (T == 0) return 0;
  if (ZSE_ACT_BF16 && T <= 64 && H % 4 == 0 && H >= 2048 && H <= 8192) {
    // few rows of at least 2,048 values (see the kernel): a decode step's norms.  The 32-bit
    // library keeps to one kernel whatever the rows, so that its results stay the same bits
    // however a request's tokens are cut into steps.
    hipStream_t st = (hipStream_t)stream;
    if (H <= 4096)
      norm_add_norm_wide_kernel<1><<<T, 1024, 0, st>>>(sub, sub_parts, w_post, eps_post, uo_post, h, w_next, eps_next,
                                                       uo_next, (act_t*)out, H);
    else
      norm_add_norm_wide_kernel<2><<<T, 1024, 0, st>>>(sub, sub_parts, w_post, eps_post, uo_post, h, w_next, eps_next,
                                                       uo_next, (act_t*)out, H);
    return zk_launch_status("zk_norm_add_norm");
  }
  if (H % 4 == 0 && H <= NF_MAXV * 1024) {
    hipStream_t st = (hipStream_t)stream;
#define ZK_NAN_(V)                                                                                              \
  norm_add_norm_fast_kernel<V><<<T, 256, 0, st>>>(sub, sub_parts, w_post, eps_post, uo_post, h, w_next, eps_next, \
                                                  uo_next, (act_t*)out, H)
    // a thread holds ceil(H / 1024) vectors of four: the narrowest kernel that covers the row
    const int vecs = (H + 1023) / 1024;
    if (vecs <= 3) ZK_NAN_(3);
    else if (vecs == 4) ZK_NAN_(4);
    else if (vecs == 5) ZK_NAN_(5);
    else ZK_NAN_(NF_MAXV);
#undef ZK_NAN_
    return zk_launch_status("zk_norm_add_norm");
  }
  norm_add_norm_kernel<<<T, 256, 0, (hipStream_t)stream>>>(sub, sub_parts, w_post, eps_post, uo_post, h, w_next,
                                                           eps_next, uo_next, (act_t*)out, H);
  return zk_launch_status("zk_norm_add_norm");
}

// act: 0 = gelu_tanh, 1 = silu
int zk_gated_act(const void* gu, void* out, int T, int I, int act, void* stream) {
  ZK_REQUIRE(T >= 0 && I > 0 && (act == 0 || act == 1), "zk_gated_act: bad arguments");
  ZK_REQUIRE(T <= 65535, "zk_gated_act: more than 65535 rows");
  if (T == 0) return 0;
  dim3 grid((I + 255) / 256, T);
  gated_act_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const act_t*)gu, (act_t*)out, I, act);
  return zk_launch_status("zk_gated_act");
}

int zk_softcap(float* z, size_t n, float cap, void* stream) {
  ZK_REQUIRE(cap > 0.f, "zk_softcap: cap must be positive");
  if (n == 0) return 0;
  ZK_REQUIRE((n + 255) / 256 < 2147483647ull, "zk_softcap: too many elements");
  softcap_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(z, n, cap);
  return zk_launch_status("zk_softcap");
}

// sums > 0: the rows are not in qkv yet but come as that many planes of [T, (nh + 2 nkv) hd] float
// partial sums (a product that split K and left the adding up to its reader, see QkvSource).
int zk_rope_cache_write_sums(void* qkv, const float* planes, int sums, const int* positions, const int* slot_map,
                             const float* inv_freq, int rotary_dim, void* kcache, void* vcache, int T, int nh,
                             int nkv, int hd, int bs, int v_transposed, void* stream) {
  ZK_REQUIRE(T >= 0 && nh > 0 && nkv >= 0 && hd > 0 && bs > 0 && sums >= 0, "zk_rope_cache_write: bad sizes");
  ZK_REQUIRE(rotary_dim >= 0 && rotary_dim <= hd && rotary_dim % 2 == 0,
             "zk_rope_cache_write: rotary_dim must be even and at most head_dim");
  ZK_REQUIRE(rotary_dim == 0 || inv_freq != nullptr, "zk_rope_cache_write: no frequency table");
  ZK_REQUIRE(nh + 2 * nkv <= 65535, "zk_rope_cache_write: too many heads");
  ZK_REQUIRE(sums == 0 || (planes != nullptr && (uintptr_t)planes % 16 == 0), "zk_rope_cache_write: partial sums must be 16-byte aligned");
  if (T == 0) return 0;
  const QkvSource from{(const act_t*)qkv, planes, sums, (size_t)T * (nh + 2 * nkv) * hd};
  // a block a token pays off with many tokens (13.6 against 18.6 us at 2048 tokens of 8 + 2 x 4
  // heads of 256); a handful of decoded tokens is quicker spread over a block per (token, head)
  if (T >= 64 && rotary_dim == hd && hd % 8 == 0 && hd / 2 <= ROPE_MAX_HALF) {
    rope_cache_write_token_kernel<<<T, 256, 0, (hipStream_t)stream>>>((act_t*)qkv, from, positions, slot_map, inv_freq,
                                                                     (act_t*)kcache, (act_t*)vcache, nh, nkv,
                                                                     hd, bs, v_transposed);
    return zk_launch_status("zk_rope_cache_write");
  }
  dim3 grid(T, nh + 2 * nkv);
  rope_cache_write_kernel<<<grid, 64, 0, (hipStream_t)stream>>>((act_t*)qkv, from, positions, slot_map, inv_freq,
                                                                rotary_dim, (act_t*)kcache,
                                                                (act_t*)vcache, nh, nkv, hd, bs, v_transposed);
  return zk_launch_status("zk_rope_cache_write");
}

int zk_rope_cache_write(void* qkv, const int* positions, const int* slot_map, const float* inv_freq,
                        int rotary_dim, void* kcache, void* vcache, int T, int nh, int nkv, int hd,
                        int bs, int v_transposed, void* stream) {
  return zk_rope_cache_write_sums(qkv, nullptr, 0, positions, slot_map, inv_freq, rotary_dim, kcache, vcache, T, nh, nkv,
                                  hd, bs, v_transposed, stream);
}

// dst_kind: 0 = float32, 1 = the library's activation type
int zk_convert(const void* src, int src_tag, void* dst, int dst_kind, size_t n, void* stream) {
  ZK_REQUIRE(src_tag >= 0 && src_tag <= 2 && (dst_kind == 0 || dst_kind == 1), "zk_convert: bad tags");
  if (n == 0) return 0;
  ZK_REQUIRE((n + 255) / 256 < 2147483647ull, "zk_convert: too many elements");
  unsigned g = (unsigned)((n + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dst_kind == 0) convert_kernel<float><<<g, 256, 0, s>>>(src, src_tag, (float*)dst, n);
  else convert_kernel<act_t><<<g, 256, 0, s>>>(src, src_tag, (act_t*)dst, n);
  return zk_launch_status("zk_convert");
}

int zk_fill_normal(void* dst, int dst_kind, size_t n, uint64_t seed, uint64_t stream_id, float mean,
                   float std, void* stream) {
  ZK_REQUIRE(dst_kind == 0 || dst_kind == 1, "zk_fill_normal: bad dst kind");
  if (n == 0) return 0;
  size_t pairs = (n + 1) / 2;
  ZK_REQUIRE((pairs + 255) / 256 < 2147483647ull, "zk_fill_normal: too many elements");
  unsigned g = (unsigned)((pairs + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dst_kind == 0) fill_normal_kernel<float><<<g, 256, 0, s>>>((float*)dst, n, seed, stream_id, mean, std);
  else fill_normal_kernel<act_t><<<g, 256, 0, s>>>((act_t*)dst, n, seed, stream_id, mean, std);
  return zk_launch_status("zk_fill_normal");
}

// tokens[dst[i]] = ids[src[i]] for i < n: the ids a step's sampling left on the device become
// the next step's tokens without a trip to the host, for the requests the next step decodes, in
// whatever order it holds them.
int zk_feed_tokens(int* tokens, const int* ids, const int* dst, const int* src, int n, void* stream) {
  ZK_REQUIRE(n >= 0, "zk_feed_tokens: bad count");
  if (n == 0) return 0;
  ZK_REQUIRE(tokens && ids && dst && src, "zk_feed_tokens: null argument");
  feed_tokens_kernel<<<(n + 255) / 256, 256, 0, (hipStream_t)stream>>>(tokens, ids, dst, src, n);
  return zk_launch_status("zk_feed_tokens");
}

// Clears ``nbytes`` (a multiple of 4) with a kernel, so that it may be captured in a graph.
int zk_zero(void* p, size_t nbytes, void* stream) {
  ZK_REQUIRE(nbytes % 4 == 0, "zk_zero: size must be a multiple of 4 bytes");
  if (nbytes == 0) return 0;
  size_t n = nbytes / 4;
  ZK_REQUIRE((n + 255) / 256 < 2147483647ull, "zk_zero: too many bytes");
  zero_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>((uint32_t*)p, n);
  return zk_launch_status("zk_zero");
}

// Clears pages ``pages[0 .. n_pages)`` (host array of ids) of each of ``n_slabs`` slabs, whose
// base addresses and page sizes in bytes lie in device memory.  Launched per 64 ids.
int zk_zero_pages(const void* slabs, const void* slab_page_bytes, int n_slabs, const int* pages, int n_pages,
                  void* stream) {
  ZK_REQUIRE(n_slabs >= 0 && n_slabs <= 65535 && n_pages >= 0, "zk_zero_pages: bad counts");
  if (n_slabs == 0 || n_pages == 0) return 0;
  ZK_REQUIRE(slabs != nullptr && slab_page_bytes != nullptr && pages != nullptr, "zk_zero_pages: null argument");
  for (int at = 0; at < n_pages; at += ZERO_PAGES_MOST) {
    PageIds ids;
    ids.n = std::min(ZERO_PAGES_MOST, n_pages - at);
    for (int i = 0; i < ids.n; i++) {
      ZK_REQUIRE(pages[at + i] >= 0, "zk_zero_pages: negative page id");
      ids.id[i] = pages[at + i];
    }
    zero_pages_kernel<<<dim3(ids.n, n_slabs), 256, 0, (hipStream_t)stream>>>(
        (void* const*)slabs, (const unsigned long long*)slab_page_bytes, ids);
  }
  return zk_launch_status("zk_zero_pages");
}

}  // extern "C"
