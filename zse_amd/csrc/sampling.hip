// Picking the next token from float logits on the device.
//
// Greedy: the lowest index among the maxima.  The reference's host scan keeps
// the first maximum (orchestrator/sampler.py:135-143) while its device tree
// reduction depends on thread order (orchestrator/kernels.py:2307-2349); here
// ties always go to the lowest index.
// Temperature: inverse CDF over softmax(z / T): the first index whose running
// sum exceeds u (orchestrator/sampler.py:168-173, 205-213), with u given per
// row by the caller so that it never depends on what else is in the batch.
// Top-k and top-p: a cut-off value and a number of its ties per row, found and
// applied by the kernels of zk_sample_cut.
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
// the index the uniform number falls into.  (Rows with top-k or top-p are drawn further down.)
// A logit is kept when it is above ``thr`` or is, in the order of the indices, one of the first
// ``ties`` equal to it: what the cut-offs of top-k and top-p come to.
struct KeepRule {
  float thr;
  int ties;
  __device__ __forceinline__ bool keeps(float v, int& seen) const { return v > thr || (v == thr && seen++ < ties); }
};
__device__ __forceinline__ float row_max(const float* pv, int r) {
  float mx = -INFINITY;
  for (int i = 0; i < AM_SLICES; i++) mx = fmaxf(mx, pv[r * AM_SLICES + i]);
  return mx;
}

// Thread t of block (slice, row) owns the contiguous piece [b + t seg, b + (t + 1) seg) of the slice.
__device__ __forceinline__ bool has_cut_offs(const int* top_k, const double* top_p, int row, int V) {
  const int k = top_k ? top_k[row] : 0;
  return (k > 0 && k < V) || (top_p && top_p[row] < 1.0);
}

__global__ __launch_bounds__(256) void sample_slice_sums_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature, const float* __restrict__ pv,
    const int* __restrict__ top_k, const double* __restrict__ top_p, double* __restrict__ psum) {
  __shared__ double red[256];
  const int row = blockIdx.y, slice = blockIdx.x, tid = threadIdx.x;
  if (temperature[row] <= 0.f || has_cut_offs(top_k, top_p, row, V)) return;
  const float* z = logits + (size_t)row * V;
  const double inv_t = 1.0 / (double)temperature[row];
  const float mx = row_max(pv, row);
  const int per = (V + AM_SLICES - 1) / AM_SLICES;
  const int b0 = slice * per, e0 = min(V, b0 + per);
  const int seg = (per + 255) / 256;
  const int b = min(e0, b0 + tid * seg), e = min(e0, b + seg);
  double part = 0.0;
  for (int i = b; i < e; i++) part += exp((double)(z[i] - mx) * inv_t);
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
    const float* __restrict__ pv, const int* __restrict__ top_k, const double* __restrict__ top_p,
    const double* __restrict__ psum, int* __restrict__ out) {
  __shared__ double red[256];
  __shared__ int s_owner;
  __shared__ double s_before;
  const int row = blockIdx.x, tid = threadIdx.x;
  if (temperature[row] <= 0.f || has_cut_offs(top_k, top_p, row, V)) return;
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
  if (slice < 0) {      // rounding left the target at or past the total: the last index that is not minus infinity
    if (tid == 0) {
      int last = V - 1;
      while (last > 0 && !(z[last] > -INFINITY)) last--;
      out[row] = last;
    }
    return;
  }
  // the thread's piece of the slice, as in the second launch
  const int per = (V + AM_SLICES - 1) / AM_SLICES;
  const int b0 = slice * per, e0 = min(V, b0 + per);
  const int seg = (per + 255) / 256;
  const int b = min(e0, b0 + tid * seg), e = min(e0, b + seg);
  double part = 0.0;
  for (int i = b; i < e; i++) part += exp((double)(z[i] - mx) * inv_t);
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
    if (owner < 0) {    // the slice's pieces fall short of what the slice's sum promised: its last index that is not minus infinity
      int last = e0 - 1;
      while (last > b0 && !(z[last] > -INFINITY)) last--;
      out[row] = last;
    }
  }
  __syncthreads();
  if (tid == s_owner) {
    double run = s_before;
    int pick = -1, last_kept = -1;
    for (int i = b; i < e; i++) {
      const float v = z[i];
      if (!(v > -INFINITY)) continue;
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

// ------------------------------------------------------------------ drawing with top-k and top-p
// Both cut-offs come to one value of the row and a number of its ties: top-k keeps everything
// from the k-th largest logit on (all its ties, orchestrator/sampler.py:146-156), top-p then the
// fewest of the largest that hold a share p of what is left, equal ones in the order of their
// indices (:186-203).  Weights exp((z - max) / T) are added up as 64-bit integers (units of 2^-44
// of the largest logit's weight): their sum does not depend on the order, so the cut-off is the
// same on every run and whichever of the ways below finds it.
//
// Five launches for any number of rows: the rows' maxima; a histogram of each row over
// (max - z) / T in steps of 1/32 (counts, and weights where there is no top-k; whatever lies 32
// or more below the maximum weighs nothing and is one bucket); one block a row walks it from
// the top to the bucket that holds the k-th largest logit (or, without top-k, the logit at
// which the share is reached) and chooses the row's way; the logits that way needs are
// gathered; and one block a row finishes:
//   way 1, the rule with a real model's logits or a small k: the logits down to that bucket are
//     few (up to TOP_CAP); the block sorts them, applies both cut-offs and draws among what is
//     left in the order of the indices, all in LDS;
//   way 3, one cut-off and many logits above it (a flat row with top-p, a large k): the bucket
//     alone is gathered and sorted, which with the sums of the buckets above it gives the
//     cut-off, and the draw goes over the whole row;
//   way 2, whatever is left (more equal logits at the cut-off than the block sorts, both
//     cut-offs with many candidates, a k-th largest logit 32 below the maximum): the block
//     narrows a range of keys (the logits' bits, made to sort like the numbers) by eight bits
//     a pass over the whole row, four passes for top-k and four for top-p (fewer from the
//     bucket's own keys on, where the walk found the bucket of a single cut-off), then draws
//     over the row;
// A row without cut-offs (way 0) is left alone: zk_sample draws it.
// (the two zeros are one key: they are equal logits, and which of the equal ones are kept goes
// by their indices)
__device__ __forceinline__ unsigned int key_of(float v) {
  const unsigned int b = v == 0.f ? 0u : __float_as_uint(v);
  return v != v ? 0u : ((b & 0x80000000u) ? ~b : (b | 0x80000000u));
}
__device__ __forceinline__ float value_of(unsigned int k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}
// exp(x) for x <= 0 in units of 2^-44
__device__ __forceinline__ unsigned long long weight_of(float x) {
  return (unsigned long long)((double)__expf(x) * 17592186044416.0);
}

#define TOP_BUCKETS 1024
#define TOP_PER_UNIT 32.f
#define TOP_CAP 2048
#define CUT_THREADS 1024
#define CUT_WAVES (CUT_THREADS / 64)
#define ALL_TIES 0x7fffffff

// Between calls cnt and w hold zero (the last launch leaves them so).
struct TopRow {
  unsigned int cnt[TOP_BUCKETS];
  unsigned long long w[TOP_BUCKETS];
  unsigned long long total;         // the whole row's weight (rows without top-k)
  unsigned long long target;        // the weight at which the share is reached (rows without top-k)
  unsigned long long above_w;       // weight, and
  unsigned int above_cnt;           // number of the logits in the buckets before first_bucket
  unsigned int found;               // candidates gathered so far
  int mode;                         // the row's way
  int first_bucket, last_bucket;    // whose logits are gathered
  int n_cand;
  float mx, inv_t;
};
struct Candidate {
  float z;
  int index;
};

// Falls with z: a larger logit never lies in a later bucket.  NaN and whatever is 32 or more
// below the maximum go to the last one.
__device__ __forceinline__ int top_bucket(float z, float mx, float inv_t) {
  const float x = (mx - z) * inv_t;
  return x < (TOP_BUCKETS - 1) / TOP_PER_UNIT ? (int)(x * TOP_PER_UNIT) : TOP_BUCKETS - 1;
}
__device__ __forceinline__ void cut_kind(const float* temperature, const int* top_k, const double* top_p, int row, int V,
                                         int& k, double& p, bool& by_count, bool& by_weight) {
  k = top_k ? top_k[row] : 0;
  p = top_p ? top_p[row] : 1.0;
  const bool drawn = temperature[row] > 0.f;       // a row that is not drawn has no cut-offs either
  by_count = drawn && k > 0 && k < V;
  by_weight = drawn && p < 1.0;
}

// f(value, index) for every NT-th element of z[b, e) from b + threadIdx.x on.  Eight loads are
// on their way at a time: a loop of one load and one atomic addition a turn waits for memory
// every turn.
template <int NT, typename F>
__device__ __forceinline__ void each_of(const float* __restrict__ z, int b, int e, F f) {
  for (int i0 = b + (int)threadIdx.x; i0 < e; i0 += 8 * NT) {
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = z[min(i0 + j * NT, e - 1)];
#pragma unroll
    for (int j = 0; j < 8; j++)
      if (i0 + j * NT < e) f(v[j], i0 + j * NT);
  }
}

__global__ __launch_bounds__(256) void top_hist_kernel(const float* __restrict__ logits, int V,
                                                       const float* __restrict__ pv,
                                                       const float* __restrict__ temperature,
                                                       const int* __restrict__ top_k, const double* __restrict__ top_p,
                                                       TopRow* __restrict__ rows) {
  __shared__ unsigned int h_cnt[TOP_BUCKETS];
  __shared__ unsigned long long h_w[TOP_BUCKETS];
  const int row = blockIdx.y, slice = blockIdx.x, tid = threadIdx.x;
  int k;
  double p;
  bool by_count, by_weight;
  cut_kind(temperature, top_k, top_p, row, V, k, p, by_count, by_weight);
  if (!by_count && !by_weight) return;
  const bool weigh = !by_count;
  for (int i = tid; i < TOP_BUCKETS; i += 256) {
    h_cnt[i] = 0;
    h_w[i] = 0;
  }
  __syncthreads();
  const float mx = row_max(pv, row), inv_t = 1.f / temperature[row];
  const int per = (V + AM_SLICES - 1) / AM_SLICES;
  const int b = slice * per, e = min(V, b + per);
  unsigned int rest = 0;
  each_of<256>(logits + (size_t)row * V, b, e, [&](float v, int) {
    const int bucket = top_bucket(v, mx, inv_t);
    if (bucket == TOP_BUCKETS - 1) {
      rest++;
      return;
    }
    atomicAdd(&h_cnt[bucket], 1u);
    if (weigh) atomicAdd(&h_w[bucket], weight_of((v - mx) * inv_t));
  });
  if (rest) atomicAdd(&h_cnt[TOP_BUCKETS - 1], rest);
  __syncthreads();
  TopRow& t = rows[row];
  for (int i = tid; i < TOP_BUCKETS; i += 256) {
    if (h_cnt[i]) atomicAdd(&t.cnt[i], h_cnt[i]);
    if (weigh && h_w[i]) atomicAdd(&t.w[i], h_w[i]);
  }
}

// Thread t is bucket t.
__global__ __launch_bounds__(CUT_THREADS) void top_walk_kernel(const float* __restrict__ pv,
                                                               const float* __restrict__ temperature,
                                                               const int* __restrict__ top_k,
                                                               const double* __restrict__ top_p, int V,
                                                               TopRow* __restrict__ rows) {
  __shared__ unsigned int c[TOP_BUCKETS];
  __shared__ unsigned long long w[TOP_BUCKETS];
  static_assert(CUT_THREADS == TOP_BUCKETS, "a thread a bucket");
  const int row = blockIdx.x, t = threadIdx.x;
  TopRow& tr = rows[row];
  int k;
  double p;
  bool by_count, by_weight;
  cut_kind(temperature, top_k, top_p, row, V, k, p, by_count, by_weight);
  if (t == 0) {
    tr.mx = row_max(pv, row);
    tr.inv_t = 1.f / temperature[row];
    tr.found = 0;
    tr.mode = (by_count || by_weight) ? 2 : 0;
    tr.first_bucket = 0;
    tr.last_bucket = -1;
    tr.n_cand = 0;
  }
  if (!by_count && !by_weight) return;
  c[t] = tr.cnt[t];
  w[t] = by_count ? 0ull : tr.w[t];
  __syncthreads();
  for (int off = 1; off < TOP_BUCKETS; off <<= 1) {
    const unsigned int a = t >= off ? c[t - off] : 0u;
    const unsigned long long aw = t >= off ? w[t - off] : 0ull;
    __syncthreads();
    c[t] += a;
    w[t] += aw;
    __syncthreads();
  }
  bool mine;
  unsigned long long target = 0;
  if (by_count) {
    mine = c[t] >= (unsigned int)k && (t == 0 || c[t - 1] < (unsigned int)k);
  } else {
    const unsigned long long total = w[TOP_BUCKETS - 1];
    target = (unsigned long long)ceil(p * (double)total);
    if (t == 0) tr.total = total;
    mine = total > 0 && w[t] >= target && (t == 0 || w[t - 1] < target);
  }
  if (!mine || t == TOP_BUCKETS - 1) return;
  const unsigned int before = t ? c[t - 1] : 0u;
  if (c[t] <= TOP_CAP) {
    tr.mode = 1;
    tr.first_bucket = 0;
    tr.n_cand = (int)c[t];
  } else if (by_count != by_weight && c[t] - before <= TOP_CAP) {
    tr.mode = 3;
    tr.first_bucket = t;
    tr.n_cand = (int)(c[t] - before);
    tr.above_cnt = before;
    tr.above_w = t ? w[t - 1] : 0ull;
    tr.target = target;
  } else if (by_count != by_weight) {     // way 2, but from this bucket on
    tr.first_bucket = t;
    tr.above_cnt = before;
    tr.above_w = t ? w[t - 1] : 0ull;
    tr.target = target;
  } else {
    return;
  }
  tr.last_bucket = t;
}

// The block's candidates wait in LDS until it knows where they go: one addition to the row's
// count a block, not one a candidate (each takes microseconds to come back).
#define GATHER_ROOM 512
__global__ __launch_bounds__(256) void top_gather_kernel(const float* __restrict__ logits, int V,
                                                         TopRow* __restrict__ rows, Candidate* __restrict__ cand) {
  __shared__ Candidate stash[GATHER_ROOM];
  __shared__ unsigned int n_here, base;
  const int row = blockIdx.y, slice = blockIdx.x, tid = threadIdx.x;
  TopRow& t = rows[row];
  if (t.mode != 1 && t.mode != 3) return;
  const float mx = t.mx, inv_t = t.inv_t;
  const int first = t.first_bucket, last = t.last_bucket;
  const int per = (V + AM_SLICES - 1) / AM_SLICES;
  const int b = slice * per, e = min(V, b + per);
  Candidate* mine = cand + (size_t)row * TOP_CAP;
  if (tid == 0) n_here = 0;
  __syncthreads();
  each_of<256>(logits + (size_t)row * V, b, e, [&](float v, int i) {
    const int bucket = top_bucket(v, mx, inv_t);
    if (bucket < first || bucket > last) return;
    const unsigned int at = atomicAdd(&n_here, 1u);
    if (at < GATHER_ROOM) {
      stash[at] = Candidate{v, i};
    } else {                                   // more than the block has room for: straight to the row's list
      const unsigned int to = atomicAdd(&t.found, 1u);
      if (to < TOP_CAP) mine[to] = Candidate{v, i};
    }
  });
  __syncthreads();
  const unsigned int n = min(n_here, (unsigned int)GATHER_ROOM);
  if (n == 0) return;
  if (tid == 0) base = atomicAdd(&t.found, n);
  __syncthreads();
  for (unsigned int i = tid; i < n; i += 256)
    if (base + i < TOP_CAP) mine[base + i] = stash[i];
}

// ---- pieces of the last launch (one block a row; nt: the threads that still run)
// Sorts keys[0, n2) (n2 a power of two) in LDS, largest first: a thread a pair of keys a turn.
__device__ __forceinline__ void sort_down(unsigned long long* keys, int n2, int nt) {
  for (int k2 = 2; k2 <= n2; k2 <<= 1)
    for (int j = k2 >> 1; j > 0; j >>= 1) {
      for (int q = threadIdx.x; q < n2 / 2; q += nt) {
        const int i = ((q & ~(j - 1)) << 1) | (q & (j - 1)), o = i | j;
        const unsigned long long a = keys[i], b = keys[o];
        if ((a < b) == ((i & k2) == 0)) {
          keys[i] = b;
          keys[o] = a;
        }
      }
      __syncthreads();
    }
}
// Running sums in place over s[0, n2), n2 <= 8 nt: afterwards s[i] = s[0] + ... + s[i].
template <typename T>
__device__ __forceinline__ void running_sums(T* s, int n2, int nt) {
  for (int off = 1; off < n2; off <<= 1) {
    T a[8];
#pragma unroll
    for (int q = 0; q < 8; q++) {
      const int i = threadIdx.x + q * nt;
      a[q] = (i < n2 && i >= off) ? s[i - off] : T(0);
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < 8; q++) {
      const int i = threadIdx.x + q * nt;
      if (i < n2) s[i] += a[q];
    }
    __syncthreads();
  }
}
__device__ __forceinline__ int pow2_from(int n) {
  int p = 64;
  while (p < n) p <<= 1;
  return p;
}
// The candidates as keys that sort the largest logit first, equal ones in the order of their indices.
__device__ __forceinline__ void candidate_keys(const Candidate* mine, int n, int n2, unsigned long long* keys, int nt) {
  for (int i = threadIdx.x; i < n2; i += nt)
    keys[i] = i < n ? ((unsigned long long)key_of(mine[i].z) << 32) | (0xffffffffu - (unsigned int)mine[i].index) : 0ull;
  __syncthreads();
  sort_down(keys, n2, nt);
}
__device__ __forceinline__ float key_value(unsigned long long key) { return value_of((unsigned int)(key >> 32)); }

struct CutSearch {
  unsigned int lo, hi, floor_key, count;
  unsigned long long above, target;
  int passes, done;
};

// Way 2 to the cut-off.  hist: CUT_WAVES histograms of 256 counts and 256 weights, sums: one of each.
// ``from``: null, or the row's walk found the bucket of its one cut-off: the search then starts
// from the keys that bucket holds, with what lies above it already counted, and its keys
// spread evenly over the first pass's counters (a search from all keys puts a flat row's
// logits into a handful of them, and the lanes of a wave wait for each other there).
__device__ void search_row(const float* __restrict__ z, int V, float mx, float inv_t, int k, double p, bool by_count,
                           bool by_weight, const TopRow* from, unsigned int* h_cnt, unsigned long long* h_w,
                           unsigned int* cnt, unsigned long long* w, CutSearch* cs, float& keep_from, int& keep_ties) {
  const int tid = threadIdx.x, wave = tid >> 6;
  if (tid == 0) {
    cs->floor_key = 0u;
    cs->lo = 0xffffffffu;
    cs->hi = 0u;
  }
  if (from) {
    __syncthreads();
    const int bucket = from->last_bucket;
    each_of<CUT_THREADS>(z, 0, V, [&](float v, int) {
      if (top_bucket(v, mx, inv_t) != bucket) return;
      atomicMin(&cs->lo, key_of(v));
      atomicMax(&cs->hi, key_of(v));
    });
  }
  for (int stage = 0; stage < 2; stage++) {
    const bool weigh = stage == 1;
    if (weigh ? !by_weight : !by_count) continue;
    __syncthreads();
    if (tid == 0) {
      if (from) {
        cs->above = weigh ? from->above_w : (unsigned long long)from->above_cnt;
        cs->target = weigh ? from->target : (unsigned long long)k;
      } else {
        if (weigh && by_count) cs->floor_key = cs->lo;      // top-k ran: its key is the floor
        cs->lo = weigh ? cs->floor_key : 0u;
        cs->hi = 0xffffffffu;
        cs->above = 0;
        cs->target = weigh ? 0ull : (unsigned long long)k;
      }
      cs->count = 0;
      cs->passes = from ? 1 : 0;
      cs->done = 0;
    }
    __syncthreads();
    for (int pass = 0; pass < 4; pass++) {               // 32 bits of key, eight a pass
      const unsigned int lo = cs->lo, hi = cs->hi;
      if (cs->done) break;
      const unsigned int width = hi - lo;
      const int shift = width < 256u ? 0 : 32 - __builtin_clz(width) - 8;
      for (int i = tid; i < CUT_WAVES * 256; i += CUT_THREADS) {
        h_cnt[i] = 0;
        h_w[i] = 0;
      }
      __syncthreads();
      each_of<CUT_THREADS>(z, 0, V, [&](float v, int) {
        const unsigned int key = key_of(v);
        if (key < lo || key > hi) return;
        const unsigned int bucket = (key - lo) >> shift;
        atomicAdd(&h_cnt[wave * 256 + bucket], 1u);
        if (weigh) atomicAdd(&h_w[wave * 256 + bucket], weight_of((v - mx) * inv_t));
      });
      __syncthreads();
      if (tid < 256) {
        unsigned int n = 0;
        unsigned long long sw = 0;
        for (int q = 0; q < CUT_WAVES; q++) {
          n += h_cnt[q * 256 + tid];
          sw += h_w[q * 256 + tid];
        }
        cnt[tid] = n;
        w[tid] = sw;
      }
      __syncthreads();
      if (tid == 0) {
        if (weigh && cs->passes == 0) {      // the first pass covers everything top-k left: its sum is the whole
          unsigned long long total = 0;
          for (int b = 0; b < 256; b++) total += w[b];
          cs->target = (unsigned long long)ceil(p * (double)total);
        }
        unsigned long long acc = cs->above;
        int pick = -1, lowest = -1;
        for (int b = 255; b >= 0; b--) {
          if (cnt[b] == 0) continue;
          lowest = b;
          const unsigned long long here = weigh ? w[b] : (unsigned long long)cnt[b];
          if (acc + here >= cs->target) {
            pick = b;
            break;
          }
          acc += here;
        }
        if (pick < 0) {       // rounding: the whole range falls short of the target; its lowest keys then
          pick = max(lowest, 0);
          acc -= weigh ? w[pick] : (unsigned long long)cnt[pick];
        }
        const unsigned long long first = (unsigned long long)lo + ((unsigned long long)pick << shift);
        cs->above = acc;
        cs->count = cnt[pick];
        cs->hi = (unsigned int)min((unsigned long long)hi, first + ((1ull << shift) - 1ull));
        cs->lo = (unsigned int)first;
        cs->passes++;
        cs->done = cs->lo == cs->hi;
      }
      __syncthreads();
    }
  }
  __syncthreads();
  if (by_weight) {            // top-p ran: the first few of the ties at its key
    const unsigned long long each = weight_of((value_of(cs->lo) - mx) * inv_t);
    const unsigned long long missing = cs->target > cs->above ? cs->target - cs->above : 0;
    unsigned long long n = each > 0 ? (missing + each - 1) / each : 1;
    n = max(1ull, min(n, (unsigned long long)cs->count));
    keep_from = value_of(cs->lo);
    keep_ties = (int)n;
  } else {                    // top-k alone: all ties of its key
    keep_from = value_of(cs->lo);
    keep_ties = ALL_TIES;
  }
}

// Inverse CDF over a whole row by one block of CUT_THREADS threads.  A logit is kept when it is
// above ``thr`` or is, in the order of the indices, one of the first ``ties`` equal to it.  A wave
// owns a sixteenth of the row and walks it 512 logits a turn, eight that follow each other a
// lane: first (if the ties are limited) to the index of the last tie kept, then to the weight
// of its part; the wave whose part holds the uniform number's place then walks it again.
struct DrawShared {
  double wsum[CUT_WAVES];
  int wties[CUT_WAVES];
  int last_tie, pick;
};
__device__ __forceinline__ void load8(const float* __restrict__ z, int i0, int e, bool whole, float (&v)[8]) {
  if (whole && i0 + 8 <= e) {
    const float4 a = *(const float4*)(z + i0), b = *(const float4*)(z + i0 + 4);
    v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
  } else {
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = z[min(i0 + j, e - 1)];
  }
}
__device__ __forceinline__ int wave_sum_int(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
template <typename T>
__device__ __forceinline__ T wave_running(T v, int lane) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const T o = __shfl_up(v, off, 64);
    if (lane >= off) v += o;
  }
  return v;
}

__device__ int draw_row(const float* __restrict__ z, int V, float mx, double inv_t, double u, float thr, int ties,
                        DrawShared* d) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const bool whole = ((uintptr_t)z & 15) == 0;
  const int turns = ((V + 511) / 512 + CUT_WAVES - 1) / CUT_WAVES;
  const int w_b = min(V, wave * turns * 512), w_e = min(V, w_b + turns * 512);
  float v[8];
  int last_tie = ALL_TIES;
  if (ties != ALL_TIES) {
    int c = 0;
    for (int i0 = w_b + lane * 8; i0 < w_e; i0 += 512) {
      load8(z, i0, w_e, whole, v);
#pragma unroll
      for (int j = 0; j < 8; j++) c += (i0 + j < w_e && v[j] == thr);
    }
    c = wave_sum_int(c);
    if (lane == 0) d->wties[wave] = c;
    if (tid == 0) d->last_tie = ALL_TIES;        // fewer ties than may be kept: all of them
    __syncthreads();
    int before = 0, owner = -1;
    for (int q = 0; q < CUT_WAVES; q++) {
      if (before + d->wties[q] >= ties) {
        owner = q;
        break;
      }
      before += d->wties[q];
    }
    if (owner == wave) {
      int run = before;
      for (int i0 = w_b + lane * 8; run < ties && i0 - lane * 8 < w_e; i0 += 512) {
        load8(z, i0, w_e, whole, v);
        int mine = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) mine += (i0 + j < w_e && v[j] == thr);
        const int incl = wave_running<int>(mine, lane);
        int s = run + incl - mine;
        if (s < ties && s + mine >= ties) {
#pragma unroll
          for (int j = 0; j < 8; j++)
            if (i0 + j < w_e && v[j] == thr && ++s == ties) d->last_tie = i0 + j;
        }
        run += __shfl(incl, 63, 64);
      }
    }
    __syncthreads();
    last_tie = d->last_tie;
  }
  auto kept = [&](float x, int i) { return x > thr || (x == thr && i <= last_tie); };
  double sum = 0.0;
  for (int i0 = w_b + lane * 8; i0 < w_e; i0 += 512) {
    load8(z, i0, w_e, whole, v);
#pragma unroll
    for (int j = 0; j < 8; j++)
      if (i0 + j < w_e && kept(v[j], i0 + j)) sum += exp((double)(v[j] - mx) * inv_t);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
  if (lane == 0) d->wsum[wave] = sum;
  if (tid == 0) d->pick = -1;
  __syncthreads();
  double total = 0.0;
  for (int q = 0; q < CUT_WAVES; q++) total += d->wsum[q];
  const double target = u * total;
  double before = 0.0;
  int owner = -1;
  for (int q = 0; q < CUT_WAVES; q++) {
    if (before + d->wsum[q] > target) {
      owner = q;
      break;
    }
    before += d->wsum[q];
  }
  if (owner == wave) {
    double run = before;
    int last_kept = -1;
    bool done = false;
    for (int i0 = w_b + lane * 8; !done && i0 - lane * 8 < w_e; i0 += 512) {
      load8(z, i0, w_e, whole, v);
      double e8[8], mine = 0.0;
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const bool in = i0 + j < w_e && kept(v[j], i0 + j);
        e8[j] = in ? exp((double)(v[j] - mx) * inv_t) : 0.0;
        mine += e8[j];
        if (in) last_kept = i0 + j;
      }
      const double incl = wave_running<double>(mine, lane);
      const unsigned long long passed = __ballot(mine > 0.0 && run + incl > target);
      if (passed) {
        if (lane == __ffsll((long long)passed) - 1) {
          double r = run + incl - mine;
          int pick = -1, last = -1;
#pragma unroll
          for (int j = 0; j < 8; j++) {
            if (e8[j] > 0.0 && pick < 0) {
              r += e8[j];
              last = i0 + j;
              if (r > target) pick = i0 + j;
            }
          }
          d->pick = pick >= 0 ? pick : last;
        }
        done = true;
      }
      run += __shfl(incl, 63, 64);
    }
    if (!done) {              // rounding left the target at or past the part's weight: its last kept index
      for (int o = 32; o > 0; o >>= 1) last_kept = max(last_kept, __shfl_xor(last_kept, o, 64));
      if (lane == 0) d->pick = last_kept;
    }
  }
  __syncthreads();
  const int pick = d->pick;
  __syncthreads();
  if (pick >= 0) return pick;
  if (tid == 0) {             // rounding left the target at or past the total: the last logit above the cut-off
    int last = V - 1;
    while (last > 0 && !(z[last] > thr)) last--;
    d->pick = last;
  }
  __syncthreads();
  return d->pick;
}

#define CUT_LDS_BYTES (CUT_WAVES * 256 * 12 + 256 * 12 + 64)
__global__ __launch_bounds__(CUT_THREADS) void sample_cut_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature, const double* __restrict__ uniform,
    const int* __restrict__ top_k, const double* __restrict__ top_p, TopRow* __restrict__ rows,
    const Candidate* __restrict__ cand, int* __restrict__ out) {
  // ways 1 and 3: keys [TOP_CAP] and sums [TOP_CAP] of 8 bytes; way 2: the histograms
  __shared__ __attribute__((aligned(16))) unsigned char lds[CUT_LDS_BYTES > TOP_CAP * 16 ? CUT_LDS_BYTES : TOP_CAP * 16];
  __shared__ DrawShared draw;
  __shared__ int s_int[4];
  const int row = blockIdx.x, tid = threadIdx.x;
  TopRow& tr = rows[row];
  int k;
  double p;
  bool by_count, by_weight;
  cut_kind(temperature, top_k, top_p, row, V, k, p, by_count, by_weight);
  const int mode = tr.mode;
  if (mode == 0) return;          // no cut-offs: zk_sample's row
  const float mx = tr.mx, inv_t = tr.inv_t;
  const double inv_td = 1.0 / (double)temperature[row];
  const double u = uniform[row];
  const float* z = logits + (size_t)row * V;
  unsigned long long* keys = (unsigned long long*)lds;
  unsigned long long* sums = keys + TOP_CAP;
  const Candidate* mine = cand + (size_t)row * TOP_CAP;
  int nt = CUT_THREADS;
  if (mode == 1) {
    // a thread a pair of candidates; the waves that have none leave, and a barrier among few
    // waves (among one, up to 128 candidates) costs little
    const int n = tr.n_cand, n2 = pow2_from(n);
    nt = max(64, n2 / 2);
    if (tid >= nt) return;
    candidate_keys(mine, n, n2, keys, nt);
    // top-k: all ties of the k-th largest
    if (tid == 0) s_int[0] = n;
    __syncthreads();
    if (by_count) {
      const unsigned int kth = (unsigned int)(keys[k - 1] >> 32);
      for (int i = tid; i < n; i += nt)
        if ((unsigned int)(keys[i] >> 32) >= kth && (i + 1 == n || (unsigned int)(keys[i + 1] >> 32) < kth)) s_int[0] = i + 1;
      __syncthreads();
    }
    const int n_k = s_int[0];
    // top-p: the fewest of them that hold the share
    if (tid == 0) s_int[1] = n_k;
    if (by_weight) {
      for (int i = tid; i < n2; i += nt) sums[i] = i < n_k ? weight_of((key_value(keys[i]) - mx) * inv_t) : 0ull;
      __syncthreads();
      running_sums<unsigned long long>(sums, n2, nt);
      const unsigned long long total = by_count ? sums[n_k - 1] : tr.total;
      const unsigned long long target = (unsigned long long)ceil(p * (double)total);
      for (int i = tid; i < n_k; i += nt)
        if (sums[i] >= target && (i == 0 || sums[i - 1] < target)) s_int[1] = i + 1;
    }
    __syncthreads();
    const int n_p = s_int[1], m2 = pow2_from(n_p);
    // what is left, in the order of the indices (sorted down by the complement of the index)
    for (int i = tid; i < n2; i += nt) {
      const unsigned long long key = keys[i];
      sums[i] = i < n_p ? ((key & 0xffffffffull) << 32) | (key >> 32) : 0ull;
    }
    __syncthreads();
    sort_down(sums, m2, nt);
    double* run = (double*)keys;
    for (int i = tid; i < m2; i += nt)
      run[i] = i < n_p ? exp((double)(value_of((unsigned int)(sums[i] & 0xffffffffull)) - mx) * inv_td) : 0.0;
    __syncthreads();
    running_sums<double>(run, m2, nt);
    const double target = u * run[m2 - 1];
    if (tid == 0) s_int[2] = n_p - 1;              // rounding left the target at or past the total: the last kept index
    __syncthreads();
    for (int i = tid; i < n_p; i += nt)
      if (run[i] > target && (i == 0 || !(run[i - 1] > target))) s_int[2] = i;
    __syncthreads();
    if (tid == 0) out[row] = (int)(0xffffffffu - (unsigned int)(sums[s_int[2]] >> 32));
  } else {
    float thr = -INFINITY;
    int ties = ALL_TIES;
    if (mode == 3) {
      // the cut-off lies in the gathered bucket; what the buckets above it hold is known
      const int n = tr.n_cand, n2 = pow2_from(n);
      candidate_keys(mine, n, n2, keys, nt);
      if (by_count) {
        thr = key_value(keys[k - (int)tr.above_cnt - 1]);
      } else {
        for (int i = tid; i < n2; i += nt) sums[i] = i < n ? weight_of((key_value(keys[i]) - mx) * inv_t) : 0ull;
        __syncthreads();
        running_sums<unsigned long long>(sums, n2, nt);
        const unsigned long long target = tr.target - tr.above_w;
        if (tid == 0) s_int[0] = n - 1;
        __syncthreads();
        for (int i = tid; i < n; i += nt)
          if (sums[i] >= target && (i == 0 || sums[i - 1] < target)) s_int[0] = i;
        __syncthreads();
        const int at = s_int[0];
        const unsigned int zk = (unsigned int)(keys[at] >> 32);
        for (int i = tid; i <= at; i += nt)
          if ((unsigned int)(keys[i] >> 32) == zk && (i == 0 || (unsigned int)(keys[i - 1] >> 32) != zk)) s_int[1] = i;
        __syncthreads();
        thr = value_of(zk);
        ties = at + 1 - s_int[1];
      }
      __syncthreads();
    } else if (mode == 2) {
      unsigned int* h_cnt = (unsigned int*)lds;
      unsigned long long* h_w = (unsigned long long*)(lds + CUT_WAVES * 256 * 4);
      unsigned long long* w = h_w + CUT_WAVES * 256;
      unsigned int* cnt = (unsigned int*)(w + 256);
      CutSearch* cs = (CutSearch*)(cnt + 256);
      search_row(z, V, mx, inv_t, k, p, by_count, by_weight, tr.last_bucket >= 0 ? &tr : nullptr, h_cnt, h_w, cnt, w,
                 cs, thr, ties);
    }
    const int pick = draw_row(z, V, mx, inv_td, u, thr, ties, &draw);
    if (tid == 0) out[row] = pick;
  }
  // the row's histogram back to zero for the next call
  for (int i = tid; i < TOP_BUCKETS; i += nt) {
    tr.cnt[i] = 0;
    tr.w[i] = 0;
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

// scratch: as for zk_argmax plus rows * 64 doubles (zk_sample_scratch_bytes)
size_t zk_sample_scratch_bytes(int rows) { return (size_t)rows * AM_SLICES * (8 + 8); }

// top_k, top_p (may be null): rows that have cut-offs (as zk_sample_cut reads them) are left alone,
// and so is a row whose temperature is not positive (its caller takes the largest logit: zk_argmax
// into the same ``out`` first serves a batch of both kinds).
int zk_sample(const float* logits, const float* temperature, const double* uniform, const int* top_k,
              const double* top_p, int* out, int rows, int V, void* scratch, void* stream) {
  ZK_REQUIRE(rows >= 0 && V > 0, "zk_sample: bad sizes");
  ZK_REQUIRE(rows <= 65535, "zk_sample: too many rows");
  ZK_REQUIRE(scratch != nullptr && (uintptr_t)scratch % 8 == 0, "zk_sample: no scratch buffer");
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  double* psum = (double*)scratch;
  float* pv = (float*)(psum + (size_t)rows * AM_SLICES);
  int* pi = (int*)(pv + (size_t)rows * AM_SLICES);
  dim3 grid(AM_SLICES, rows);
  argmax_slices_kernel<<<grid, 256, 0, s>>>(logits, V, pv, pi);
  sample_slice_sums_kernel<<<grid, 256, 0, s>>>(logits, V, temperature, pv, top_k, top_p, psum);
  sample_pick_kernel<<<rows, 256, 0, s>>>(logits, V, temperature, uniform, pv, top_k, top_p, psum, out);
  return zk_launch_status("zk_sample");
}

// Draws the rows that have top-k or top-p.  top_k[r] <= 0 or >= V: no top-k; top_p[r] >= 1: no
// top-p; either pointer may be null; out[r] of a row with neither, or whose temperature is not
// positive, is not written.  scratch: zk_sample_cut_scratch_bytes(room) bytes, room >= rows, that
// held zero when they were first handed in and are handed in again, with the same room, as the
// last call left them.
size_t zk_sample_cut_scratch_bytes(int rows) {
  return (size_t)rows * (sizeof(TopRow) + TOP_CAP * sizeof(Candidate) + AM_SLICES * 8) + 64;
}

size_t zk_sample_cut_row_bytes() { return sizeof(TopRow); }
size_t zk_sample_cut_mode_offset() { return offsetof(TopRow, mode); }

int zk_sample_cut(const float* logits, const float* temperature, const double* uniform, const int* top_k,
                  const double* top_p, int* out, int rows, int V, void* scratch, int room, void* stream) {
  ZK_REQUIRE(rows >= 0 && V > 0 && room >= rows, "zk_sample_cut: bad sizes");
  ZK_REQUIRE(rows <= 65535, "zk_sample_cut: too many rows");
  ZK_REQUIRE(temperature && uniform && out, "zk_sample_cut: temperature, uniform numbers and output are needed");
  ZK_REQUIRE(scratch != nullptr && (uintptr_t)scratch % 8 == 0, "zk_sample_cut: no scratch buffer");
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  TopRow* tr = (TopRow*)scratch;
  Candidate* cand = (Candidate*)(tr + room);
  float* pv = (float*)(cand + (size_t)room * TOP_CAP);
  int* pi = (int*)(pv + (size_t)room * AM_SLICES);
  argmax_slices_kernel<<<dim3(AM_SLICES, rows), 256, 0, s>>>(logits, V, pv, pi);
  top_hist_kernel<<<dim3(AM_SLICES, rows), 256, 0, s>>>(logits, V, pv, temperature, top_k, top_p, tr);
  top_walk_kernel<<<rows, CUT_THREADS, 0, s>>>(pv, temperature, top_k, top_p, V, tr);
  top_gather_kernel<<<dim3(AM_SLICES, rows), 256, 0, s>>>(logits, V, tr, cand);
  sample_cut_kernel<<<rows, CUT_THREADS, 0, s>>>(logits, V, temperature, uniform, top_k, top_p, tr, cand, out);
  return zk_launch_status("zk_sample_cut");
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
