// Picking the next token from float logits on the device.
//
// Greedy: the lowest index among the maxima.  The reference's host scan keeps
// the first maximum (orchestrator/sampler.py:135-143) while its device tree
// reduction depends on thread order (orchestrator/kernels.py:2307-2349); here
// ties always go to the lowest index.
// Temperature: inverse CDF over softmax(z / T): the first index whose running
// sum exceeds u (orchestrator/sampler.py:168-173, 205-213), with u given per
// row by the caller so that it never depends on what else is in the batch.
// A row whose ``keep_from`` threshold is set ignores logits below it (top-k /
// top-p cut-offs computed by the caller).
#include "common.h"

// Stage 1: block (slice, row) scans its slice of the row; stage 2: one block a row joins the
// slices.  Larger value wins, equal values go to the lower index, NaNs never win.
#define AM_SLICES 64
__device__ __forceinline__ void argmax_block_reduce(float& best, int& bi, float* sv, int* si) {
  sv[threadIdx.x] = best;
  si[threadIdx.x] = bi;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (threadIdx.x < s) {
      const float ov = sv[threadIdx.x + s];
      const int oi = si[threadIdx.x + s];
      if (ov > sv[threadIdx.x] || (ov == sv[threadIdx.x] && oi < si[threadIdx.x])) {
        sv[threadIdx.x] = ov;
        si[threadIdx.x] = oi;
      }
    }
    __syncthreads();
  }
  best = sv[0];
  bi = si[0];
}

__global__ __launch_bounds__(256) void argmax_slices_kernel(const float* __restrict__ logits, int V,
                                                            float* __restrict__ pv, int* __restrict__ pi) {
  __shared__ float sv[256];
  __shared__ int si[256];
  const int row = blockIdx.y, slice = blockIdx.x;
  const float* z = logits + (size_t)row * V;
  const int per = (V + AM_SLICES - 1) / AM_SLICES;
  const int b = slice * per, e = min(V, b + per);
  float best = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = b + threadIdx.x; i < e; i += 256) {
    const float v = z[i];
    if (v > best || (bi == 0x7fffffff && v == v)) {
      best = v;
      bi = i;
    }
  }
  argmax_block_reduce(best, bi, sv, si);
  if (threadIdx.x == 0) {
    pv[row * AM_SLICES + slice] = best;
    pi[row * AM_SLICES + slice] = bi;
  }
}

__global__ __launch_bounds__(256) void argmax_join_kernel(const float* __restrict__ pv,
                                                          const int* __restrict__ pi,
                                                          int* __restrict__ out) {
  __shared__ float sv[256];
  __shared__ int si[256];
  const int row = blockIdx.x;
  float best = -INFINITY;
  int bi = 0x7fffffff;
  if (threadIdx.x < AM_SLICES) {
    best = pv[row * AM_SLICES + threadIdx.x];
    bi = pi[row * AM_SLICES + threadIdx.x];
  }
  argmax_block_reduce(best, bi, sv, si);
  if (threadIdx.x == 0) out[row] = bi == 0x7fffffff ? 0 : bi;
}

// One block per row.  Thread i owns the contiguous segment [i*seg, (i+1)*seg).
__global__ __launch_bounds__(256) void sample_kernel(const float* __restrict__ logits, int V,
                                                     const float* __restrict__ temperature,
                                                     const double* __restrict__ uniform,
                                                     const float* __restrict__ keep_from,
                                                     int* __restrict__ out) {
  __shared__ float smax[256];
  __shared__ double ssum[256];
  __shared__ int s_owner;
  __shared__ double s_before, s_target;
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* z = logits + (size_t)r * V;
  const float thr = keep_from ? keep_from[r] : -INFINITY;
  const double inv_t = 1.0 / (double)temperature[r];
  float mx = -INFINITY;
  for (int i = tid; i < V; i += 256) {
    const float v = z[i];
    if (v >= thr) mx = fmaxf(mx, v);
  }
  smax[tid] = mx;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (tid < s) smax[tid] = fmaxf(smax[tid], smax[tid + s]);
    __syncthreads();
  }
  mx = smax[0];
  const int seg = (V + 255) / 256;
  const int b = tid * seg, e = min(V, b + seg);
  double part = 0.0;
  for (int i = b; i < e; i++) {
    const float v = z[i];
    if (v >= thr) part += exp((double)(v - mx) * inv_t);
  }
  ssum[tid] = part;
  __syncthreads();
  if (tid == 0) {
    double total = 0.0;
    for (int i = 0; i < 256; i++) total += ssum[i];
    const double target = uniform[r] * total;
    double run = 0.0;
    int owner = -1;
    for (int i = 0; i < 256; i++) {
      if (run + ssum[i] > target) {
        owner = i;
        break;
      }
      run += ssum[i];
    }
    s_owner = owner;
    s_before = run;
    s_target = target;
    if (owner < 0) {  // rounding left the target at or past the total: last kept index
      int last = V - 1;
      while (last > 0 && !(z[last] >= thr)) last--;
      out[r] = last;
    }
  }
  __syncthreads();
  if (tid == s_owner) {
    const double target = s_target;
    double run = s_before;
    int pick = -1, last_kept = -1;
    for (int i = b; i < e; i++) {
      const float v = z[i];
      if (!(v >= thr)) continue;
      last_kept = i;
      run += exp((double)(v - mx) * inv_t);
      if (run > target) {
        pick = i;
        break;
      }
    }
    out[r] = pick >= 0 ? pick : last_kept;
  }
}

extern "C" {

// scratch: room for rows * 64 floats and rows * 64 ints (zk_argmax_scratch_bytes)
size_t zk_argmax_scratch_bytes(int rows) { return (size_t)rows * AM_SLICES * 8; }

int zk_argmax(const float* logits, int* out, int rows, int V, void* scratch, void* stream) {
  ZK_REQUIRE(rows >= 0 && V > 0, "zk_argmax: bad sizes");
  ZK_REQUIRE(rows <= 65535, "zk_argmax: too many rows");
  ZK_REQUIRE(scratch != nullptr, "zk_argmax: no scratch buffer");
  if (rows == 0) return 0;
  float* pv = (float*)scratch;
  int* pi = (int*)scratch + (size_t)rows * AM_SLICES;
  dim3 grid(AM_SLICES, rows);
  argmax_slices_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(logits, V, pv, pi);
  argmax_join_kernel<<<rows, 256, 0, (hipStream_t)stream>>>(pv, pi, out);
  return zk_launch_status("zk_argmax");
}

int zk_sample(const float* logits, const float* temperature, const double* uniform,
              const float* keep_from, int* out, int rows, int V, void* stream) {
  ZK_REQUIRE(rows >= 0 && V > 0, "zk_sample: bad sizes");
  if (rows == 0) return 0;
  sample_kernel<<<rows, 256, 0, (hipStream_t)stream>>>(logits, V, temperature, uniform, keep_from, out);
  return zk_launch_status("zk_sample");
}

}  // extern "C"
