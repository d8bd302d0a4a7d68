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
// like the numbers) by eight bits a pass, four passes for each of the two: a histogram over the
// range, by count for top-k, by weight exp((z - max) / T) for top-p, walked from the top.  A
// pass is two launches: 16 blocks a row fill histograms of their slices (each wave one of its
// own in LDS, so that lanes of different waves never meet at one counter), one block a row adds
// them up and walks.  Weights are added up as 64-bit integers (units of 2^-44 of the largest
// logit's weight): integer additions are one instruction where additions of doubles are a loop,
// and their sum does not depend on the order, so the cut-off is the same on every run.
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

#define SC_SLICES 16
struct CutState {
  unsigned int lo, hi;            // the range of keys still in question (inclusive)
  unsigned int floor_key;         // top-p: what top-k left
  unsigned int count;             // logits with the key the range has narrowed to
  unsigned long long above;       // count or weight of the keys above the range
  unsigned long long target;
  float mx, inv_t, share;
  int by_weight, active, passes;
};
struct CutHist {
  unsigned int cnt[256];
  unsigned long long w[256];
};
__device__ __forceinline__ int cut_shift(unsigned int lo, unsigned int hi) {
  const unsigned int width = hi - lo;
  return width < 256u ? 0 : 32 - __builtin_clz(width) - 8;
}

// Starts a row's search: stage 0 = top-k over all keys, stage 1 = top-p over what top-k left.
__global__ void cutoff_begin_kernel(CutState* __restrict__ st, const float* __restrict__ pv,
                                    const float* __restrict__ temperature, const int* __restrict__ top_k,
                                    const float* __restrict__ top_p, int V, int stage, int rows) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  CutState& c = st[r];
  if (stage == 0) {
    const int k = top_k ? top_k[r] : 0;
    c.mx = row_max(pv, r);
    c.inv_t = 1.f / temperature[r];
    c.floor_key = 0u;
    c.lo = 0u;
    c.hi = 0xffffffffu;
    c.above = 0;
    c.count = 0;
    c.target = (unsigned long long)max(k, 0);
    c.by_weight = 0;
    c.passes = 0;
    c.active = k > 0 && k < V;
  } else {
    const float p = top_p ? top_p[r] : 1.f;
    if (c.active) c.floor_key = c.lo;      // top-k ran: its key is the floor
    c.lo = c.floor_key;
    c.hi = 0xffffffffu;
    c.above = 0;
    c.count = 0;
    c.share = p;
    c.by_weight = 1;
    c.passes = 0;
    c.active = p < 1.f;
  }
}

__global__ __launch_bounds__(256) void cutoff_hist_kernel(const float* __restrict__ logits, int V,
                                                          const CutState* __restrict__ st, CutHist* __restrict__ hist) {
  __shared__ unsigned int h_cnt[4][256];
  __shared__ unsigned long long h_w[4][256];
  const int row = blockIdx.y, slice = blockIdx.x, tid = threadIdx.x, wave = tid >> 6;
  const CutState c = st[row];
  if (!c.active || (c.lo == c.hi && c.passes > 0)) return;
  for (int i = tid; i < 4 * 256; i += 256) {
    (&h_cnt[0][0])[i] = 0;
    (&h_w[0][0])[i] = 0;
  }
  __syncthreads();
  const float* z = logits + (size_t)row * V;
  const int per = (V + SC_SLICES - 1) / SC_SLICES;
  const int b = slice * per, e = min(V, b + per);
  const int shift = cut_shift(c.lo, c.hi);
  for (int i = b + tid; i < e; i += 256) {
    const float v = z[i];
    const unsigned int key = key_of(v);
    if (key < c.lo || key > c.hi) continue;
    const unsigned int bucket = (key - c.lo) >> shift;
    atomicAdd(&h_cnt[wave][bucket], 1u);
    if (c.by_weight) atomicAdd(&h_w[wave][bucket], weight_of((v - c.mx) * c.inv_t));
  }
  __syncthreads();
  CutHist& out = hist[(size_t)row * SC_SLICES + slice];
  out.cnt[tid] = h_cnt[0][tid] + h_cnt[1][tid] + h_cnt[2][tid] + h_cnt[3][tid];
  out.w[tid] = h_w[0][tid] + h_w[1][tid] + h_w[2][tid] + h_w[3][tid];
}

// Adds the slices' histograms up and walks them from the top: to the bucket at which the count
// (or the weight) of the keys from the floor on reaches the target; the range becomes that bucket.
__global__ __launch_bounds__(256) void cutoff_walk_kernel(CutState* __restrict__ st, const CutHist* __restrict__ hist) {
  __shared__ unsigned int cnt[256];
  __shared__ unsigned long long w[256];
  const int row = blockIdx.x, tid = threadIdx.x;
  CutState& c = st[row];
  if (!c.active || (c.lo == c.hi && c.passes > 0)) return;
  unsigned int n = 0;
  unsigned long long sw = 0;
  for (int q = 0; q < SC_SLICES; q++) {
    n += hist[(size_t)row * SC_SLICES + q].cnt[tid];
    sw += hist[(size_t)row * SC_SLICES + q].w[tid];
  }
  cnt[tid] = n;
  w[tid] = sw;
  __syncthreads();
  if (tid != 0) return;
  if (c.by_weight && c.passes == 0) {          // the first pass covers everything top-k left: its sum is the whole
    unsigned long long total = 0;
    for (int b = 0; b < 256; b++) total += w[b];
    c.target = (unsigned long long)ceil((double)c.share * (double)total);
  }
  const int shift = cut_shift(c.lo, c.hi);
  unsigned long long acc = c.above;
  int pick = -1, lowest = -1;
  for (int b = 255; b >= 0; b--) {
    if (cnt[b] == 0) continue;
    lowest = b;
    const unsigned long long here = c.by_weight ? w[b] : (unsigned long long)cnt[b];
    if (acc + here >= c.target) {
      pick = b;
      break;
    }
    acc += here;
  }
  if (pick < 0) {             // rounding: the whole range falls short of the target; its lowest keys then
    pick = max(lowest, 0);
    acc -= c.by_weight ? w[pick] : (unsigned long long)cnt[pick];
  }
  const unsigned long long first = (unsigned long long)c.lo + ((unsigned long long)pick << shift);
  c.above = acc;
  c.count = cnt[pick];
  c.hi = (unsigned int)min((unsigned long long)c.hi, first + ((1ull << shift) - 1ull));
  c.lo = (unsigned int)first;
  c.passes++;
}

__global__ void cutoff_end_kernel(const CutState* __restrict__ st, float* __restrict__ keep_from,
                                  int* __restrict__ keep_ties, int rows) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  const CutState& c = st[r];
  if (c.active) {             // top-p ran: the first few of the ties at its key
    const unsigned long long each = weight_of((value_of(c.lo) - c.mx) * c.inv_t);
    const unsigned long long missing = c.target > c.above ? c.target - c.above : 0;
    unsigned long long n = each > 0 ? (missing + each - 1) / each : 1;
    n = max(1ull, min(n, (unsigned long long)c.count));
    keep_from[r] = value_of(c.lo);
    keep_ties[r] = (int)n;
  } else {                    // top-k alone (all ties of its key) or nothing
    keep_from[r] = c.floor_key ? value_of(c.floor_key) : -INFINITY;
    keep_ties[r] = -1;
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
// scratch: zk_sample_cutoff_scratch_bytes(rows).
size_t zk_sample_cutoff_scratch_bytes(int rows) {
  return (size_t)rows * (sizeof(CutState) + SC_SLICES * sizeof(CutHist) + AM_SLICES * 8) + 64;
}

int zk_sample_cutoff(const float* logits, const float* temperature, const int* top_k, const float* top_p,
                     float* keep_from, int* keep_ties, int rows, int V, void* scratch, void* stream) {
  ZK_REQUIRE(rows >= 0 && V > 0, "zk_sample_cutoff: bad sizes");
  ZK_REQUIRE(rows <= 65535, "zk_sample_cutoff: too many rows");
  ZK_REQUIRE(temperature && keep_from && keep_ties, "zk_sample_cutoff: temperature and outputs are needed");
  ZK_REQUIRE(scratch != nullptr && (uintptr_t)scratch % 8 == 0, "zk_sample_cutoff: no scratch buffer");
  if (rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  CutHist* hist = (CutHist*)scratch;
  CutState* st = (CutState*)(hist + (size_t)rows * SC_SLICES);
  float* pv = (float*)(st + rows);
  int* pi = (int*)(pv + (size_t)rows * AM_SLICES);
  argmax_slices_kernel<<<dim3(AM_SLICES, rows), 256, 0, s>>>(logits, V, pv, pi);
  for (int stage = 0; stage < 2; stage++) {
    if (stage == 0 && top_k == nullptr) {
      // no top-k anywhere: the state still has to be set up
    }
    cutoff_begin_kernel<<<(rows + 63) / 64, 64, 0, s>>>(st, pv, temperature, top_k, top_p, V, stage, rows);
    if ((stage == 0 && top_k == nullptr) || (stage == 1 && top_p == nullptr)) continue;
    for (int pass = 0; pass < 4; pass++) {          // 32 bits of key, eight a pass
      cutoff_hist_kernel<<<dim3(SC_SLICES, rows), 256, 0, s>>>(logits, V, st, hist);
      cutoff_walk_kernel<<<rows, 256, 0, s>>>(st, hist);
    }
  }
  cutoff_end_kernel<<<(rows + 63) / 64, 64, 0, s>>>(st, keep_from, keep_ties, rows);
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
