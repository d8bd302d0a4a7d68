// Picking the next token from float logits on the device.
//
// Greedy: the lowest index among the maxima.  The reference's host scan keeps
// the first maximum (orchestrator/sampler.py:135-143) while its device tree
// reduction depends on thread order (orchestrator/kernels.py:2307-2349); here
// ties always go to the lowest index.
// Temperature: inverse CDF over softmax(z / T): the first index whose running
// sum exceeds u (orchestrator/sampler.py:168-173, 205-213), with u given per
// row by the caller so that it never depends on what else is in the batch.
// A row whose ``keep_from`` cut-off is set ignores logits below it (top-k and
// top-p, worked out by sample_cutoff_kernel).
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

// Inverse CDF in three launches, so that one row keeps many CUs busy: the slices' maxima (the
// argmax's first stage), the slices' weights, then one block a row that finds the slice and
// the index the uniform number falls into.
// keep_from / keep_ties (may be null): a row keeps its logits above keep_from[r] and, in the
// order of their indices, the first keep_ties[r] of those equal to it (a negative count: all of
// them), which is what the cut-offs of top-k and top-p come to (sample_cutoff_kernel).
struct KeepRule {
  float thr;
  int ties;
  __device__ __forceinline__ bool keeps(float v, int& seen) const { return v > thr || (v == thr && seen++ < ties); }
};
__device__ __forceinline__ KeepRule keep_rule(const float* keep_from, const int* keep_ties, int r) {
  KeepRule k;
  k.thr = keep_from ? keep_from[r] : -INFINITY;
  k.ties = (keep_from && keep_ties && keep_ties[r] >= 0) ? keep_ties[r] : 0x7fffffff;
  return k;
}
__device__ __forceinline__ float row_max(const float* pv, int r) {
  float mx = -INFINITY;
  for (int i = 0; i < AM_SLICES; i++) mx = fmaxf(mx, pv[r * AM_SLICES + i]);
  return mx;
}

// Block (slice, row): how many logits of the slice equal the cut-off, and (second launch, when
// the ties before the slice are known) the slice's weight.
__global__ __launch_bounds__(256) void sample_slice_ties_kernel(const float* __restrict__ logits, int V,
                                                                const float* __restrict__ keep_from,
                                                                int* __restrict__ pties) {
  __shared__ int red[256];
  const int row = blockIdx.y, slice = blockIdx.x, tid = threadIdx.x;
  const float thr = keep_from[row];
  const float* z = logits + (size_t)row * V;
  const int per = (V + AM_SLICES - 1) / AM_SLICES;
  const int b = slice * per, e = min(V, b + per);
  int n = 0;
  for (int i = b + tid; i < e; i += 256) n += z[i] == thr;
  red[tid] = n;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (tid < s) red[tid] += red[tid + s];
    __syncthreads();
  }
  if (tid == 0) pties[row * AM_SLICES + slice] = red[0];
}

// Thread t of block (slice, row) owns the contiguous piece [b + t seg, b + (t + 1) seg) of the slice.
__global__ __launch_bounds__(256) void sample_slice_sums_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature, const float* __restrict__ pv,
    const float* __restrict__ keep_from, const int* __restrict__ keep_ties, const int* __restrict__ pties,
    double* __restrict__ psum) {
  __shared__ double red[256];
  __shared__ int sties[256];
  const int row = blockIdx.y, slice = blockIdx.x, tid = threadIdx.x;
  const KeepRule keep = keep_rule(keep_from, keep_ties, row);
  const float* z = logits + (size_t)row * V;
  const double inv_t = 1.0 / (double)temperature[row];
  const float mx = row_max(pv, row);
  const int per = (V + AM_SLICES - 1) / AM_SLICES;
  const int b0 = slice * per, e0 = min(V, b0 + per);
  const int seg = (per + 255) / 256;
  const int b = min(e0, b0 + tid * seg), e = min(e0, b + seg);
  int seen = 0;
  if (pties) {                                   // ties before this thread's piece
    for (int q = 0; q < slice; q++) seen += pties[row * AM_SLICES + q];
    int mine = 0;
    for (int i = b; i < e; i++) mine += z[i] == keep.thr;
    sties[tid] = mine;
    __syncthreads();
    for (int q = 0; q < tid; q++) seen += sties[q];
  }
  double part = 0.0;
  for (int i = b; i < e; i++) {
    const float v = z[i];
    if (keep.keeps(v, seen)) part += exp((double)(v - mx) * inv_t);
  }
  red[tid] = part;
  __syncthreads();
  if (tid == 0) {
    double total = 0.0;
    for (int i = 0; i < 256; i++) total += red[i];       // in order: the third launch adds the same way
    psum[row * AM_SLICES + slice] = total;
  }
}

__global__ __launch_bounds__(256) void sample_pick_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature, const double* __restrict__ uniform,
    const float* __restrict__ pv, const float* __restrict__ keep_from, const int* __restrict__ keep_ties,
    const int* __restrict__ pties, const double* __restrict__ psum, int* __restrict__ out) {
  __shared__ double red[256];
  __shared__ int sties[256];
  __shared__ int s_owner;
  __shared__ double s_before;
  const int row = blockIdx.x, tid = threadIdx.x;
  const KeepRule keep = keep_rule(keep_from, keep_ties, row);
  const float* z = logits + (size_t)row * V;
  const double inv_t = 1.0 / (double)temperature[row];
  const float mx = row_max(pv, row);
  // the slice
  double total = 0.0;
  for (int i = 0; i < AM_SLICES; i++) total += psum[row * AM_SLICES + i];
  const double target = uniform[row] * total;
  double before = 0.0;
  int slice = -1;
  for (int i = 0; i < AM_SLICES; i++) {
    const double w = psum[row * AM_SLICES + i];
    if (before + w > target) {
      slice = i;
      break;
    }
    before += w;
  }
  if (slice < 0) {      // rounding left the target at or past the total: the last kept index
    if (tid == 0) {
      int last = V - 1;
      while (last > 0 && !(z[last] > keep.thr)) last--;
      out[row] = last;
    }
    return;
  }
  // the thread's piece of the slice, as in the second launch
  const int per = (V + AM_SLICES - 1) / AM_SLICES;
  const int b0 = slice * per, e0 = min(V, b0 + per);
  const int seg = (per + 255) / 256;
  const int b = min(e0, b0 + tid * seg), e = min(e0, b + seg);
  int seen = 0;
  if (pties) {
    for (int q = 0; q < slice; q++) seen += pties[row * AM_SLICES + q];
    int mine = 0;
    for (int i = b; i < e; i++) mine += z[i] == keep.thr;
    sties[tid] = mine;
    __syncthreads();
    for (int q = 0; q < tid; q++) seen += sties[q];
  }
  const int seen0 = seen;
  double part = 0.0;
  for (int i = b; i < e; i++) {
    const float v = z[i];
    if (keep.keeps(v, seen)) part += exp((double)(v - mx) * inv_t);
  }
  red[tid] = part;
  __syncthreads();
  if (tid == 0) {
    double run = before;
    int owner = -1;
    for (int i = 0; i < 256; i++) {
      if (run + red[i] > target) {
        owner = i;
        break;
      }
      run += red[i];
    }
    s_owner = owner;
    s_before = run;
    if (owner < 0) {    // the slice's pieces fall short of what the slice's sum promised: its last kept index
      int last = e0 - 1;
      while (last > b0 && !(z[last] > keep.thr)) last--;
      out[row] = last;
    }
  }
  __syncthreads();
  if (tid == s_owner) {
    double run = s_before;
    int pick = -1, last_kept = -1;
    seen = seen0;
    for (int i = b; i < e; i++) {
      const float v = z[i];
      if (!keep.keeps(v, seen)) continue;
      last_kept = i;
      run += exp((double)(v - mx) * inv_t);
      if (run > target) {
        pick = i;
        break;
      }
    }
    out[row] = pick >= 0 ? pick : last_kept;
  }
}

// ------------------------------------------------------------------ top-k and top-p cut-offs
// Both come to one value of the row and a number of its ties: top-k keeps everything from the
// k-th largest logit on (all its ties, orchestrator/sampler.py:146-156), top-p then the fewest
// of the largest that hold a share p of what is left, equal ones in the order of their indices
// (:186-203).  The value is found by narrowing a range of keys (the logits' bits, made to sort
// like the numbers) by eight bits a pass: a histogram over the range, by count for top-k, by
// weight exp((z - max) / T) for top-p, walked from the top.  Every wave has a histogram of its
// own in LDS, so that lanes of different waves never meet at one counter.  Weights are added up
// as 64-bit integers (units of 2^-44 of the largest logit's weight): integer additions in LDS
// are one instruction where additions of doubles are a loop, and their sum does not depend on
// the order, so the cut-off is the same on every run.
__device__ __forceinline__ unsigned int key_of(float v) {
  const unsigned int b = __float_as_uint(v);
  return v != v ? 0u : ((b & 0x80000000u) ? ~b : (b | 0x80000000u));
}
__device__ __forceinline__ float value_of(unsigned int k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}
// exp(x) for x <= 0 in units of 2^-44
__device__ __forceinline__ unsigned long long weight_of(float x) {
  return (unsigned long long)((double)__expf(x) * 17592186044416.0);
}

#define SC_WAVES 16
// Every logit of a row through f, four to a load where the row allows it (the block has one CU's
// share of the memory system to itself, so it wants many loads in flight).
template <typename F>
__device__ __forceinline__ void each_logit(const float* __restrict__ z, int V, int tid, F f) {
  if (V % 4 == 0 && (uintptr_t)z % 16 == 0) {
    const float4* z4 = (const float4*)z;
    int i = tid;
    for (; i + 64 * SC_WAVES < V / 4; i += 2 * 64 * SC_WAVES) {
      const float4 a = z4[i], b = z4[i + 64 * SC_WAVES];
      f(a.x); f(a.y); f(a.z); f(a.w);
      f(b.x); f(b.y); f(b.z); f(b.w);
    }
    if (i < V / 4) {
      const float4 a = z4[i];
      f(a.x); f(a.y); f(a.z); f(a.w);
    }
  } else {
    for (int i = tid; i < V; i += 64 * SC_WAVES) f(z[i]);
  }
}

__global__ __launch_bounds__(64 * SC_WAVES) void sample_cutoff_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, float* __restrict__ keep_from, int* __restrict__ keep_ties) {
  __shared__ unsigned int h_cnt[SC_WAVES][256];
  __shared__ unsigned long long h_w[SC_WAVES][256];
  __shared__ unsigned int s_lo, s_hi, s_kmin, s_kmax, s_count;
  __shared__ unsigned long long s_above, s_target;
  __shared__ float s_red[SC_WAVES];
  const int r = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const float* z = logits + (size_t)r * V;
  const int k = top_k ? top_k[r] : 0;
  const float p = top_p ? top_p[r] : 1.f;
  const bool use_k = k > 0 && k < V, use_p = p < 1.f;
  if (!use_k && !use_p) {
    if (tid == 0) {
      keep_from[r] = -INFINITY;
      keep_ties[r] = -1;
    }
    return;
  }
  const float inv_t = 1.f / temperature[r];
  // the row's largest logit and the range of its keys
  float mx = -INFINITY;
  unsigned int kmin = 0xffffffffu, kmax = 0u;
  each_logit(z, V, tid, [&](float v) {
    const unsigned int key = key_of(v);
    mx = fmaxf(mx, v);
    kmin = min(kmin, key);
    kmax = max(kmax, key);
  });
  mx = wave_max(mx);
  for (int o = 32; o > 0; o >>= 1) {
    kmin = min(kmin, (unsigned int)__shfl_xor((int)kmin, o, 64));
    kmax = max(kmax, (unsigned int)__shfl_xor((int)kmax, o, 64));
  }
  if (tid == 0) {
    s_kmin = 0xffffffffu;
    s_kmax = 0u;
  }
  __syncthreads();
  if (lane == 0) {
    s_red[wave] = mx;
    atomicMin(&s_kmin, kmin);
    atomicMax(&s_kmax, kmax);
  }
  __syncthreads();
  mx = s_red[0];
  for (int w = 1; w < SC_WAVES; w++) mx = fmaxf(mx, s_red[w]);
  kmin = s_kmin;
  kmax = s_kmax;
  __syncthreads();

  // Narrows [s_lo, s_hi] to one key: the key at which, walking down from the largest, the
  // count (by_weight false) of the keys >= floor reaches `target`, or their weight the share
  // `share` of its total (which the first pass, over all of them, gives: s_target).  Leaves in
  // s_above what lies above that key and in s_count how many logits have it.
  auto narrow = [&](bool by_weight, unsigned int floor_key, unsigned long long target, float share) {
    if (tid == 0) {
      s_lo = max(kmin, floor_key);
      s_hi = kmax;
      s_above = 0;
      s_count = 0;
      s_target = target;
    }
    __syncthreads();
    bool counted = false;
    while (true) {
      const unsigned int lo = s_lo, hi = s_hi;
      if (lo == hi && counted) break;
      const unsigned int width = hi - lo;                       // inclusive range minus one
      const int shift = width < 256u ? 0 : 32 - __builtin_clz(width) - 8;
      for (int i = lane; i < 256; i += 64) {
        h_cnt[wave][i] = 0;
        h_w[wave][i] = 0;
      }
      __syncthreads();
      each_logit(z, V, tid, [&](float v) {
        const unsigned int key = key_of(v);
        if (key < lo || key > hi) return;
        const unsigned int b = (key - lo) >> shift;
        atomicAdd(&h_cnt[wave][b], 1u);
        if (by_weight) atomicAdd(&h_w[wave][b], weight_of((v - mx) * inv_t));
      });
      __syncthreads();
      for (int i = tid; i < 256; i += 64 * SC_WAVES) {
        unsigned int c = 0;
        unsigned long long w = 0;
        for (int q = 0; q < SC_WAVES; q++) {
          c += h_cnt[q][i];
          w += h_w[q][i];
        }
        h_cnt[0][i] = c;
        h_w[0][i] = w;
      }
      __syncthreads();
      if (tid == 0) {
        if (by_weight && !counted) {
          unsigned long long total = 0;
          for (int b = 0; b < 256; b++) total += h_w[0][b];
          s_target = (unsigned long long)ceil((double)share * (double)total);
        }
        const unsigned long long target = s_target;
        unsigned long long acc = s_above;
        int pick = -1, lowest = -1;
        for (int b = 255; b >= 0; b--) {
          if (h_cnt[0][b] == 0) continue;
          lowest = b;
          const unsigned long long here = by_weight ? h_w[0][b] : (unsigned long long)h_cnt[0][b];
          if (acc + here >= target) {
            pick = b;
            break;
          }
          acc += here;
        }
        if (pick < 0) {           // rounding: the whole range falls short of the target; its lowest keys then
          pick = lowest;
          acc -= by_weight ? h_w[0][pick] : (unsigned long long)h_cnt[0][pick];
        }
        s_above = acc;
        s_count = h_cnt[0][pick];
        const unsigned long long first = (unsigned long long)lo + ((unsigned long long)pick << shift);
        s_lo = (unsigned int)first;
        s_hi = (unsigned int)min((unsigned long long)hi, first + ((1ull << shift) - 1ull));
      }
      __syncthreads();
      counted = true;
    }
  };

  unsigned int floor_key = 0u;
  int ties = -1;
  if (use_k) {
    narrow(false, 0u, (unsigned long long)k, 0.f);
    floor_key = s_lo;
    __syncthreads();
  }
  if (use_p) {
    narrow(true, floor_key, 0, p);
    if (tid == 0) {
      const unsigned long long each = weight_of((value_of(s_lo) - mx) * inv_t);
      const unsigned long long missing = s_target > s_above ? s_target - s_above : 0;
      unsigned long long c = each > 0 ? (missing + each - 1) / each : 1;
      c = max(1ull, min(c, (unsigned long long)s_count));
      ties = (int)c;
    }
    floor_key = s_lo;
  }
  if (tid == 0) {
    keep_from[r] = value_of(floor_key);
    keep_ties[r] = ties;
  }
}

// z[tok] /= s where z[tok] > 0, *= s otherwise, for every (row, token, s) of a list: the
// repetition penalty with the scale worked out by the caller from how often the token has
// appeared (orchestrator/sampler.py:64-74).
__global__ void penalty_kernel(float* __restrict__ logits, int V, const int* __restrict__ rows,
                               const int* __restrict__ tokens, const float* __restrict__ scales, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int t = tokens[i];
  if (t < 0 || t >= V) return;
  float* z = logits + (size_t)rows[i] * V + t;
  const float v = *z, s = scales[i];
  *z = v > 0.f ? v / s : v * s;
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

// scratch: as for zk_argmax plus rows * 64 doubles and rows * 64 ints (zk_sample_scratch_bytes)
size_t zk_sample_scratch_bytes(int rows) { return (size_t)rows * AM_SLICES * (8 + 8 + 4); }

int zk_sample(const float* logits, const float* temperature, const double* uniform,
              const float* keep_from, const int* keep_ties, int* out, int rows, int V, void* scratch,
              void* stream) {
  ZK_REQUIRE(rows >= 0 && V > 0, "zk_sample: bad sizes");
  ZK_REQUIRE(rows <= 65535, "zk_sample: too many rows");
  ZK_REQUIRE(scratch != nullptr && (uintptr_t)scratch % 8 == 0, "zk_sample: no scratch buffer");
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  double* psum = (double*)scratch;
  float* pv = (float*)(psum + (size_t)rows * AM_SLICES);
  int* pi = (int*)(pv + (size_t)rows * AM_SLICES);
  int* pties = keep_from ? pi : nullptr;          // the maxima's indices are not needed here
  dim3 grid(AM_SLICES, rows);
  argmax_slices_kernel<<<grid, 256, 0, s>>>(logits, V, pv, pi);
  if (keep_from) sample_slice_ties_kernel<<<grid, 256, 0, s>>>(logits, V, keep_from, pties);
  sample_slice_sums_kernel<<<grid, 256, 0, s>>>(logits, V, temperature, pv, keep_from, keep_ties, pties, psum);
  sample_pick_kernel<<<rows, 256, 0, s>>>(logits, V, temperature, uniform, pv, keep_from, keep_ties, pties, psum, out);
  return zk_launch_status("zk_sample");
}

// top_k[r] <= 0 or >= V: no top-k; top_p[r] >= 1: no top-p.  Either pointer may be null.
int zk_sample_cutoff(const float* logits, const float* temperature, const int* top_k, const float* top_p,
                     float* keep_from, int* keep_ties, int rows, int V, void* stream) {
  ZK_REQUIRE(rows >= 0 && V > 0, "zk_sample_cutoff: bad sizes");
  ZK_REQUIRE(temperature && keep_from && keep_ties, "zk_sample_cutoff: temperature and outputs are needed");
  if (rows == 0) return 0;
  sample_cutoff_kernel<<<rows, 64 * SC_WAVES, 0, (hipStream_t)stream>>>(logits, V, temperature, top_k, top_p,
                                                                        keep_from, keep_ties);
  return zk_launch_status("zk_sample_cutoff");
}

// Each (rows[i], tokens[i]) pair must be listed once: the kernel reads and writes the logit.
int zk_penalize(float* logits, int V, const int* rows, const int* tokens, const float* scales, int n,
                void* stream) {
  ZK_REQUIRE(n >= 0 && V > 0, "zk_penalize: bad sizes");
  if (n == 0) return 0;
  penalty_kernel<<<(n + 255) / 256, 256, 0, (hipStream_t)stream>>>(logits, V, rows, tokens, scales, n);
  return zk_launch_status("zk_penalize");
}

}  // extern "C"
