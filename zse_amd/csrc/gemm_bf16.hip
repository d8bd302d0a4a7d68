// bfloat16 matrix products on the matrix cores (MFMA), float accumulation:
//   C[M,N] = A[M,K] * W[N,K]^T        (weights [out, in], both operands K-contiguous)
//
// Three kernels, chosen by M:
//  * skinny (M <= 16, or weights not in strip layout up to 64): the weight matrix is streamed
//    once from HBM.  A block owns a strip of 16 weight rows; its waves split K and each feeds
//    16x16x32 MFMAs straight from global memory: a lane's 16-byte load is exactly its MFMA
//    operand (row = lane % 16, eight k values at 8 * (lane / 16)), so no LDS staging is
//    needed.  Partial sums of the waves meet in LDS.
//  * mid (17 <= M <= 64, strip layout): four strips a block, two waves each, the activations
//    of a k chunk shared through LDS, K split over blocks when N alone gives too few of them.
//  * tile (M > 64, prefill): 256x256x64 (sixteen waves), 128x256x64 (eight) or 128x128x64 (four)
//    block tiles staged through LDS, each wave a 64x64 corner built from 32x32x16 MFMAs.
// Epilogues: plain store (bf16 or float), soft cap on float output (LM head), and
// the gated activation act(gate) * up over a [2I, K] weight whose first I rows are
// the gate (the feed-forward's first product; the [T, 2I] intermediate never
// reaches memory).
//
// The reference's products are scalar-FMA tiles and a one-warp-per-row GEMV
// (orchestrator/kernels.py:1075-1126, 2077-2107), gate and up separate
// (orchestrator/model_runner.py:1270-1275).
#include "common.h"
#include "gemm_bf16_static.h"

#include <mutex>

// Where a product that splits K over blocks leaves its partial sums.  ``strict``: the split is
// chosen as for the standard workspace (so that the bits do not depend on who brought the
// memory) and refused, not narrowed, when ``bytes`` cannot hold it.
#define ZK_GEMM_WORKSPACE_BYTES ((size_t)320 << 20)
struct GemmWorkspace {
  void* ptr;
  size_t bytes;
  bool strict;
  size_t split_bytes() const { return strict ? ZK_GEMM_WORKSPACE_BYTES : bytes; }
  int too_small(size_t need) const {
    static thread_local char msg[200];
    snprintf(msg, sizeof msg, "zk_gemm_bf16_static: this shape's partial sums need %zu bytes, the "
             "static scratch array holds %zu", need, bytes);
    return zk_fail(msg);
  }
};

#if ZSE_ACT_BF16

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// EPI_PICK (the LM head of a step whose next tokens are the largest logits): nothing of C is
// stored; each strip of 16 columns leaves, per row, its largest value after the soft cap (cap
// <= 0: none) and that value's column in ``partials`` [M][strips] as (float, int), larger value
// first, equal values to the lower column, NaN never, which a joining kernel reduces to one
// column a row: the greedy choice without the logits ever reaching memory.
enum { EPI_NONE = 0, EPI_SOFTCAP = 1, EPI_GELU_TANH = 2, EPI_SILU = 3, EPI_PICK = 4 };

struct Pick {
  float value;
  int column;
};

// A lane's four results x[i] at columns n + i of one row, joined with the lanes 16, 32 and 48
// further on (the other columns of the strip); afterwards every one of the four lanes holds
// the strip's pick.
__device__ __forceinline__ Pick pick_of_strip(const float (&x)[4], int n, int N, float cap) {
  Pick p{-INFINITY, 0x7fffffff};
#pragma unroll
  for (int i = 0; i < 4; i++) {
    if (n + i >= N) continue;
    const float v = cap > 0.f ? cap * tanhf(x[i] / cap) : x[i];
    if (v > p.value || (p.column == 0x7fffffff && v == v)) {
      p.value = v;
      p.column = n + i;
    }
  }
#pragma unroll
  for (int off = 16; off <= 32; off *= 2) {
    const float ov = __shfl_xor(p.value, off);
    const int oc = __shfl_xor(p.column, off);
    const bool other_valid = oc != 0x7fffffff, mine_valid = p.column != 0x7fffffff;
    if (other_valid && (!mine_valid || ov > p.value || (ov == p.value && oc < p.column))) {
      p.value = ov;
      p.column = oc;
    }
  }
  return p;
}

// 0.5 g (1 + tanh(u)) = g / (1 + exp(-2 u)): one exponential and one reciprocal instead of the
// library's tanh, which cost a tenth of the prompt's gate|up product; the difference (a few
// units in the last place of a float) vanishes when the result is rounded to 16 bits.
__device__ __forceinline__ float epi_gelu_tanh(float g) {
  const float k = 0.7978845608028654f;
  const float u = k * (g + 0.044715f * g * g * g);
  return g * __builtin_amdgcn_rcpf(1.0f + __expf(-2.0f * u));
}
__device__ __forceinline__ float epi_gate(float g, float u, int epi) {
  return (epi == EPI_GELU_TANH ? epi_gelu_tanh(g) : g / (1.0f + expf(-g))) * u;
}

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; i++) z[i] = (__bf16)0.f;
  return z;
}

// ------------------------------------------------------------------ skinny
// What the q|k|v product of decoded tokens does with its results instead of storing them all:
// q and k heads are rotated (pairs (i, i + hd/2), angle position * inv_freq[i]), q goes to C,
// k and v to the token's place in the paged cache.
struct RopeStore {
  const int* positions;
  const int* slot_map;  // null: nothing is stored in the cache (nkv = 0)
  const float* inv_freq;
  __bf16* kcache;
  __bf16* vcache;
  int nh, nkv, hd, bs, v_transposed;
};

__device__ __forceinline__ void store4(__bf16* dst, const float (&x)[4]) {
  bf16x4 o;
#pragma unroll
  for (int i = 0; i < 4; i++) o[i] = (__bf16)x[i];
  *(bf16x4*)dst = o;
}

// GATED: the block also streams the strip of "up" rows I + n and stores act(g)*u.
// ROPE (M <= 16): W is [(nh + 2 nkv) hd, K]; the block's 16 weight rows are eight places of a
// head's first half and their partners in the rotation, hd/2 rows further on, so that partners
// meet in lanes 32 apart; the results are finished as RopeStore says.  Every result is rounded
// to 16 bits before it is rotated, as the separate product and rotation kernels do, so a
// token's keys are the same bits whichever way it came.
// EXACT (weights in strip layout, so K is a whole number of 32-wide steps): no load is under a
// condition.  A step past the wave's run reads the run's last step again and its weights are
// set to zero afterwards; a row past M reads row M - 1 (its results are never stored).  Only so
// can the compiler count the loads in flight and let a group's products wait for that group
// alone: with loads under per-lane conditions it waits for every load before each group, and
// the next group's loads, just issued, no longer overlap anything (down projection of 2304 x
// 9216 at 8 rows: 14 us against 9).
template <int MT, bool GATED, int NW, bool ROPE = false, bool EXACT = false, bool SPLIT = false>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const __bf16* __restrict__ A, int lda,
                                                          const __bf16* __restrict__ W,
                                                          void* __restrict__ C, int ldc, int c_is_f32,
                                                          int M, int N, int K, int epi, float cap,
                                                          int w_strip, RopeStore rs,
                                                          float* __restrict__ partials = nullptr, int ksplit = 1) {
  static_assert(!ROPE || (MT == 1 && !GATED), "the rotating epilogue takes up to 16 rows");
  constexpr int NS = GATED ? 2 : 1;
  __shared__ f32x4 red[NW - 1][NS][MT][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kq = lane >> 4;
  // the block's strips of 16 weight rows
  const int strip0 = blockIdx.x, strip1 = N / 16 + blockIdx.x;
  const int n0 = strip0 * 16;
  // Row-major weights: a lane reads row n0 + r at 8 * kq, a 32-wide step further on is 32
  // elements away.  Strip layout: the 64 lanes' pieces of one (strip, step) are one
  // contiguous KB, a step further on is 512 elements away, strips follow each other.
  const int wrow = min(n0 + r, N - 1);
  const int ksteps = (K + 31) / 32;
  const size_t wstep = w_strip ? 512 : 32;
  const __bf16* wp[NS];
  wp[0] = w_strip ? W + (size_t)strip0 * ksteps * 512 + lane * 8 : W + (size_t)wrow * K + kq * 8;
  if (GATED)
    wp[NS - 1] = w_strip ? W + (size_t)strip1 * ksteps * 512 + lane * 8
                         : W + (size_t)(N + wrow) * K + kq * 8;
  int head = 0, hpos = 0;  // ROPE: the head and the first of the block's eight places in its first half
  if (ROPE) {
    const int per_head = rs.hd / 16;
    head = blockIdx.x / per_head;
    hpos = (blockIdx.x % per_head) * 8;
    const int row = head * rs.hd + hpos + (r < 8 ? r : rs.hd / 2 + r - 8);
    wp[0] = w_strip ? W + (size_t)(row / 16) * ksteps * 512 + (16 * kq + row % 16) * 8
                    : W + (size_t)row * K + kq * 8;
  }
  const __bf16* ap[MT];
  bool av[MT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
    const int m = mt * 16 + r;
    av[mt] = m < M;
    ap[mt] = A + (size_t)min(m, M - 1) * lda + kq * 8;
  }
  f32x4 acc[NS][MT];
#pragma unroll
  for (int s = 0; s < NS; s++)
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[s][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // the K range is cut into NW equal runs of 32-wide steps, one run a wave.  A wave works in
  // groups of STEPS steps and keeps the next group's loads in flight while it multiplies the
  // current one (two register sets, the loop is unrolled by two to name them).
  constexpr int STEPS = (MT * NS >= 4) ? 4 : 8;
  const int total_steps = (K + 31) / 32;
  const int per_wave = (total_steps + NW - 1) / NW;
  const int s_begin = wave * per_wave, s_end = min(total_steps, s_begin + per_wave);
  // EXACT: whole groups of STEPS steps are shared out among the waves as evenly as they go
  const int total_groups = (total_steps + STEPS - 1) / STEPS;
  const int uwave = __builtin_amdgcn_readfirstlane(wave);      // the same in every lane: loop bounds stay scalar
  // (SPLIT) blockIdx.y takes one of ksplit ranges of the groups, its waves share the range out
  static_assert(!SPLIT || (EXACT && MT == 1 && !GATED && !ROPE), "K is split for plain products of up to 16 rows");
  const int gy0 = SPLIT ? (int)blockIdx.y * total_groups / ksplit : 0;
  const int gy1 = SPLIT ? ((int)blockIdx.y + 1) * total_groups / ksplit : total_groups;
  const int gw0 = gy0 + uwave * (gy1 - gy0) / NW, gw1 = gy0 + (uwave + 1) * (gy1 - gy0) / NW;
  const int run_lo = gw0 * STEPS, run_n = (gw1 - gw0) * STEPS;      // the wave's run of steps
  auto fetch = [&](int s0, bf16x8 (&wf)[NS][STEPS], bf16x8 (&af)[MT][STEPS]) {
    if (EXACT) {
      // A whole group of steps, counted from the start of the wave's run; only the last group
      // of K may hold fewer steps, and then the steps past K read K's last step again and count
      // as zero.
#pragma unroll
      for (int s = 0; s < STEPS; s++) {
        const int step = min(run_lo + s0 + s, total_steps - 1);
#pragma unroll
        for (int mt = 0; mt < MT; mt++) af[mt][s] = *(const bf16x8*)(ap[mt] + step * 32);
#pragma unroll
        for (int g = 0; g < NS; g++) wf[g][s] = *(const bf16x8*)(wp[g] + (size_t)step * wstep);
      }
      if (run_lo + run_n > total_steps) {
#pragma unroll
        for (int s = 0; s < STEPS; s++)
          if (run_lo + s0 + s >= total_steps) {
#pragma unroll
            for (int g = 0; g < NS; g++) wf[g][s] = zero8();
          }
      }
      return;
    }
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
      const int k = (s0 + s) * 32;
      const bool in = (s0 + s < s_end) && (k + kq * 8 < K);
#pragma unroll
      for (int mt = 0; mt < MT; mt++) af[mt][s] = (in && av[mt]) ? *(const bf16x8*)(ap[mt] + k) : zero8();
#pragma unroll
      for (int g = 0; g < NS; g++) wf[g][s] = in ? *(const bf16x8*)(wp[g] + (size_t)(s0 + s) * wstep) : zero8();
    }
  };
  auto multiply = [&](const bf16x8 (&wf)[NS][STEPS], const bf16x8 (&af)[MT][STEPS]) {
#pragma unroll
    for (int s = 0; s < STEPS; s++)
#pragma unroll
      for (int g = 0; g < NS; g++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
          acc[g][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[g][s], af[mt][s], acc[g][mt], 0, 0, 0);
  };
  bf16x8 wf0[NS][STEPS], af0[MT][STEPS], wf1[NS][STEPS], af1[MT][STEPS];
  if (EXACT) {
    if (gw0 < gw1) fetch(0, wf0, af0);
  } else if (s_begin < s_end) {
    fetch(s_begin, wf0, af0);
  }
  // the angles of the lane's four pairs, worked out while the first loads are on their way
  float sn[4], cs[4];
  int slot = -1;
  if (ROPE && wave == 0) {
    if (head >= rs.nh && rs.slot_map) slot = rs.slot_map[min(r, M - 1)];
    if (head < rs.nh + rs.nkv) {
      const float pos = (float)rs.positions[min(r, M - 1)];
#pragma unroll
      for (int i = 0; i < 4; i++) sincosf(pos * rs.inv_freq[hpos + 4 * (kq & 1) + i], &sn[i], &cs[i]);
    }
  }
  if (EXACT) {
    // The wave's run is a whole number of groups [gw0, gw1).  In the loop every product follows
    // a fetch, so the number of loads in flight at each wait is known; the last one or two
    // groups have code of their own.  Nothing is loaded twice.  (The scheduling barriers keep
    // the compiler from moving a group's loads down to their first use, which would put each
    // load right in front of the product that waits for it.)
    if (gw0 < gw1) {
      int g = 0;
      const int gw1 = run_n / STEPS;         // groups of the run, counted from its start
      for (; g + 2 < gw1; g += 2) {
        fetch((g + 1) * STEPS, wf1, af1);
        __builtin_amdgcn_sched_barrier(0);
        multiply(wf0, af0);
        __builtin_amdgcn_sched_barrier(0);
        fetch((g + 2) * STEPS, wf0, af0);
        __builtin_amdgcn_sched_barrier(0);
        multiply(wf1, af1);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (g + 2 == gw1) {
        fetch((g + 1) * STEPS, wf1, af1);
        __builtin_amdgcn_sched_barrier(0);
        multiply(wf0, af0);
        __builtin_amdgcn_sched_barrier(0);
        multiply(wf1, af1);
      } else {
        multiply(wf0, af0);
      }
    }
  } else {
    for (int s0 = s_begin; s0 < s_end; s0 += 2 * STEPS) {
      if (s0 + STEPS < s_end) fetch(s0 + STEPS, wf1, af1);
      multiply(wf0, af0);
      if (s0 + STEPS >= s_end) break;
      if (s0 + 2 * STEPS < s_end) fetch(s0 + 2 * STEPS, wf0, af0);
      multiply(wf1, af1);
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int g = 0; g < NS; g++)
#pragma unroll
      for (int mt = 0; mt < MT; mt++) red[wave - 1][g][mt][lane] = acc[g][mt];
  }
  __syncthreads();
  if (wave > 0) return;
  // lane holds rows n = n0 + 4*kq + i (i = 0..3) of column m = mt*16 + r
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
    const int m = mt * 16 + r;
    f32x4 v[NS];
#pragma unroll
    for (int g = 0; g < NS; g++) {
      v[g] = acc[g][mt];
#pragma unroll
      for (int w = 0; w < NW - 1; w++) v[g] += red[w][g][mt][lane];
    }
    if (SPLIT) {
      // the range's partial sums: plane blockIdx.y of [M, npad] floats, to be added up in the
      // order of the ranges by whoever reads them (zk_norm_add_norm, or the joining kernel)
      if (m < M) {
        const size_t npad = (size_t)gridDim.x * 16;
        *(f32x4*)(partials + ((size_t)blockIdx.y * M + m) * npad + n0 + 4 * kq) = v[0];
      }
      continue;
    }
    if (ROPE) {
      // results 4 kq + i of the block's 16: lanes 0..31 hold places hpos + 4 kq + i of the
      // head's first half, lanes 32..63 their partners in the second
      const bool first = kq < 2;
      const int half = rs.hd / 2, at = hpos + 4 * (kq & 1) + (first ? 0 : half);
      float x[4];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        x[i] = (float)(__bf16)v[0][i];
        const float y = __shfl_xor(x[i], 32);
        if (head < rs.nh + rs.nkv) {
          float ra, rb;
          rotate_pair(first ? x[i] : y, first ? y : x[i], sn[i], cs[i], ra, rb);
          x[i] = first ? ra : rb;
        }
      }
      if (m >= M) continue;
      if (head < rs.nh) {
        store4((__bf16*)C + (size_t)m * ldc + (size_t)head * rs.hd + at, x);
        continue;
      }
      if (slot < 0) continue;
      const int kvh = (head - rs.nh) % rs.nkv;
      const size_t page = slot / rs.bs, off = slot % rs.bs;
      if (head < rs.nh + rs.nkv || !rs.v_transposed) {
        store4((head < rs.nh + rs.nkv ? rs.kcache : rs.vcache) + ((page * rs.nkv + kvh) * rs.bs + off) * rs.hd + at, x);
      } else {
        __bf16* vt = rs.vcache + (page * rs.nkv + kvh) * (size_t)rs.hd * rs.bs + off;
#pragma unroll
        for (int i = 0; i < 4; i++) vt[(size_t)(at + i) * rs.bs] = (__bf16)x[i];
      }
      continue;
    }
    if (!GATED && epi == EPI_PICK) {
      const float x[4] = {v[0][0], v[0][1], v[0][2], v[0][3]};
      const Pick p = pick_of_strip(x, n0 + 4 * kq, N, cap);
      if (kq == 0 && m < M) ((Pick*)partials)[(size_t)m * gridDim.x + blockIdx.x] = p;
      continue;
    }
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int n = n0 + 4 * kq + i;
      if (n >= N) continue;
      float x = v[0][i];
      if (GATED) x = epi_gate(x, v[NS - 1][i], epi);
      else if (epi == EPI_SOFTCAP) x = cap * tanhf(x / cap);
      if (c_is_f32) ((float*)C)[(size_t)m * ldc + n] = x;
      else ((__bf16*)C)[(size_t)m * ldc + n] = (__bf16)x;
    }
  }
}

// ------------------------------------------------------------------ tile
// Block tile (32 WMT NWM) x (64 NWN) x 64 with NWM x NWN waves; a wave owns WMT x 2 MFMA tiles
// of 32 x 32.  The k tiles alternate between two LDS buffers: the loads of the next tile are
// issued before the products of the current one and stored after them, one barrier a tile.
#define GT_BK 64
#define GT_LD (GT_BK + 8)

// Blocks that share a weight tile run on one XCD (ids go round-robin over 8 XCDs).
__device__ __forceinline__ void tile_of_block(int id, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  if (total % 8 == 0) id = (id % 8) * (total / 8) + id / 8;
  tn = id / tiles_m;
  tm = id % tiles_m;
}

// The products are taken as W tile x A tile^T, so that a lane holds neighbouring columns of one
// row of C.  Four results of a lane: row lr of the wave's 32 x 32 tiles (i, 0) and (i, 1),
// columns 8 b + 4 lk + e (e = 0..3); x0 belongs to tile (i, 0), x1 to tile (i, 1) (gate and up
// when GATED).
template <int WMT, int NWN, bool GATED>
__device__ __forceinline__ void tile_store_quad(const f32x4& x0, const f32x4& x1, int i, int b,
                                                void* __restrict__ C, int ldc, int c_is_f32, int M, int N,
                                                int m0, int n0, int wm, int wn, int lane, int epi, float cap) {
  const int lr = lane & 31, lk = lane >> 5;
  const int m = m0 + wm * (32 * WMT) + i * 32 + lr;
  if (m >= M) return;
#pragma unroll
  for (int e = 0; e < 4; e++) {
    const int c = 8 * b + 4 * lk + e;
    if (GATED) {
      const int n = n0 + wn * 32 + c;
      if (n < N) {
        const float x = epi_gate(x0[e], x1[e], epi);
        if (c_is_f32) ((float*)C)[(size_t)m * ldc + n] = x;
        else ((__bf16*)C)[(size_t)m * ldc + n] = (__bf16)x;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const int n = n0 + wn * 64 + j * 32 + c;
        if (n >= N) continue;
        float x = j ? x1[e] : x0[e];
        if (epi == EPI_SOFTCAP) x = cap * tanhf(x / cap);
        if (c_is_f32) ((float*)C)[(size_t)m * ldc + n] = x;
        else ((__bf16*)C)[(size_t)m * ldc + n] = (__bf16)x;
      }
    }
  }
}

template <int WMT, int NWN, bool GATED>
__device__ __forceinline__ void tile_store(const f32x16 (&acc)[WMT][2], void* __restrict__ C, int ldc,
                                           int c_is_f32, int M, int N, int m0, int n0, int wm, int wn,
                                           int lane, int epi, float cap) {
#pragma unroll
  for (int i = 0; i < WMT; i++)
#pragma unroll
    for (int b = 0; b < 4; b++) {
      const f32x4 x0 = {acc[i][0][4 * b], acc[i][0][4 * b + 1], acc[i][0][4 * b + 2], acc[i][0][4 * b + 3]};
      const f32x4 x1 = {acc[i][1][4 * b], acc[i][1][4 * b + 1], acc[i][1][4 * b + 2], acc[i][1][4 * b + 3]};
      tile_store_quad<WMT, NWN, GATED>(x0, x1, i, b, C, ldc, c_is_f32, M, N, m0, n0, wm, wn, lane, epi, cap);
    }
}

// The same for a wave whose tile lies inside a 16-bit C with rows that are whole 16-byte pieces:
// the wave's results go through its own piece of LDS (rows of SLD values) and leave as 16 bytes
// a lane, whole 128- or 64-byte runs of a row, instead of two bytes a lane.
template <int WMT, bool GATED>
__device__ __forceinline__ void tile_store_staged(const f32x16 (&acc)[WMT][2], __bf16* __restrict__ C, int ldc,
                                                  int row0, int col0, int lane, int epi, float cap,
                                                  __bf16* __restrict__ stage) {
  constexpr int COLS = GATED ? 32 : 64, SLD = COLS + 8;
  const int lr = lane & 31, lk = lane >> 5;
#pragma unroll
  for (int i = 0; i < WMT; i++)
#pragma unroll
    for (int b = 0; b < 4; b++) {
      float x[4], y[4];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        x[e] = acc[i][0][4 * b + e];
        y[e] = acc[i][1][4 * b + e];
        if (GATED) x[e] = epi_gate(x[e], y[e], epi);
        else if (epi == EPI_SOFTCAP) {
          x[e] = cap * tanhf(x[e] / cap);
          y[e] = cap * tanhf(y[e] / cap);
        }
      }
      __bf16* dst = stage + (i * 32 + lr) * SLD + 8 * b + 4 * lk;
      store4(dst, x);
      if (!GATED) store4(dst + 32, y);
    }
  // the wave reads what its other lanes wrote: LDS takes a wave's accesses in order
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  constexpr int PPR = COLS / 8, RPI = 64 / PPR;      // pieces a row, rows an instruction
  const int prow = lane / PPR, pcol = (lane % PPR) * 8;
#pragma unroll
  for (int r = 0; r < 32 * WMT; r += RPI)
    *(bf16x8*)(C + (size_t)(row0 + r + prow) * ldc + col0 + pcol) = *(const bf16x8*)(stage + (r + prow) * SLD + pcol);
}

template <int WMT, int NWM, int NWN, bool GATED, bool EXACT>
__global__ __launch_bounds__(64 * NWM * NWN, NWM * NWN <= 4 ? 2 : 1) void gemm_tile_kernel(
    const __bf16* __restrict__ A, int lda, const __bf16* __restrict__ W, void* __restrict__ C, int ldc,
    int c_is_f32, int M, int N, int K_all, int epi, float cap, int tiles_m, int tiles_n, int w_strip,
    f32x16* __restrict__ partials, int ksplit, int tile_base) {
  constexpr int T = 64 * NWM * NWN;
  constexpr int BM = 32 * WMT * NWM, BN = 64 * NWN;
  constexpr int RPP = T / 8;                   // rows one pass of the block's threads covers
  constexpr int APT = BM / RPP, BPT = BN / RPP;   // 16-byte pieces a thread moves per k tile
  static_assert(BM % RPP == 0 && BN % RPP == 0 && (T / 64) % 2 == 0, "tile and thread counts do not fit");
  extern __shared__ __align__(16) unsigned char gt_lds[];
  typedef __bf16 (*tile_t)[GT_LD];
  const tile_t tiles = (tile_t)gt_lds;          // buffer b: A rows, then W rows, from row b (BM + BN)
  int tm, tn;
  tile_of_block(blockIdx.x + tile_base, tiles_m, tiles_n, tm, tn);     // a launch takes tiles [tile_base, tile_base + gridDim.x)
  const int m0 = tm * BM;
  constexpr int NCOLS = GATED ? BN / 2 : BN;         // output columns of the block
  const int n0 = tn * NCOLS;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / NWN, wn = wave % NWN;
  const int lr = lane & 31, lk = lane >> 5;
  // blockIdx.y takes a range of k tiles (the whole of K unless the launch splits it); the
  // operand pointers start at the range, so below K counts from there
  const int ktiles = (K_all + GT_BK - 1) / GT_BK;
  const int kt0 = (int)((long)blockIdx.y * ktiles / ksplit), kt1 = (int)((long)(blockIdx.y + 1) * ktiles / ksplit);
  const int kbase = kt0 * GT_BK;
  const int K = min(K_all, kt1 * GT_BK) - kbase;

  // piece c = tid + T i of a tile: row c / 8, eight k values at (c % 8) * 8
  const int prow = tid >> 3, pcol = (tid & 7) * 8;
  const __bf16* ga[APT];
  const __bf16* gb[BPT];
#pragma unroll
  for (int i = 0; i < APT; i++) ga[i] = A + (size_t)min(m0 + prow + RPP * i, M - 1) * lda + kbase;
  int brow[BPT], bcol;      // where a thread's pieces of the weight tile land in LDS
  if (w_strip) {
    // a wave copies whole KB blocks: block wave + (T / 64) i of the tile's BN / 16 strips x 2
    // steps, lane l its 16 bytes; the k tile advances by two steps = 1024 elements
    const int tstep = wave & 1;
    const int ksteps = (K_all + 31) / 32;
    const int strips = GATED ? 2 * N / 16 : (N + 15) / 16;
    bcol = tstep * 32 + (lane >> 4) * 8;
#pragma unroll
    for (int i = 0; i < BPT; i++) {
      const int sit = (wave + (T / 64) * i) >> 1;            // strip within the tile
      brow[i] = sit * 16 + (lane & 15);
      int gs;
      if (GATED) gs = sit < BN / 32 ? n0 / 16 + sit : N / 16 + n0 / 16 + (sit - BN / 32);
      else gs = n0 / 16 + sit;
      gs = min(gs, strips - 1);
      gb[i] = W + ((size_t)gs * ksteps + 2 * kt0) * 512 + lane * 8;
    }
  } else {
    bcol = pcol;
#pragma unroll
    for (int i = 0; i < BPT; i++) {
      const int row = prow + RPP * i;
      brow[i] = row;
      int bn;
      if (GATED) bn = row < BN / 2 ? min(n0 + row, N - 1) : N + min(n0 + row - BN / 2, N - 1);
      else bn = min(n0 + row, N - 1);
      gb[i] = W + (size_t)bn * K_all + kbase;
    }
  }
  // a piece's offset from its row's (strip's) first element: tile t, then the place in the tile
  const int boff = w_strip ? (wave & 1) * 512 : pcol, bstep = w_strip ? 1024 : GT_BK;
  f32x16 acc[WMT][2];
#pragma unroll
  for (int i = 0; i < WMT; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

  // Two register sets: the loads of tile t + 2 are issued while tile t is multiplied and tile
  // t + 1 waits in the other set, so a load has a whole tile's products to arrive in.
  bf16x8 ra0[APT], rb0[BPT], ra1[APT], rb1[BPT];
  // EXACT (K a multiple of the k tile): no load is under a condition, so that the compiler
  // can count the loads in flight and wait for the older set alone; a tile beyond K is read
  // from the last tile instead and never multiplied.  Otherwise pieces beyond K are zeros.
  auto fetch = [&](int k0, bf16x8 (&ra)[APT], bf16x8 (&rb)[BPT]) {
    if (EXACT) {
      const int kc = min(k0, K - GT_BK);
      const int aoff = kc + pcol, woff = (kc / GT_BK) * bstep + boff;
#pragma unroll
      for (int i = 0; i < APT; i++) ra[i] = *(const bf16x8*)(ga[i] + aoff);
#pragma unroll
      for (int i = 0; i < BPT; i++) rb[i] = *(const bf16x8*)(gb[i] + woff);
    } else {
      const bool in = k0 + pcol < K, inb = k0 + bcol < K;
#pragma unroll
      for (int i = 0; i < APT; i++) ra[i] = in ? *(const bf16x8*)(ga[i] + k0 + pcol) : zero8();
#pragma unroll
      for (int i = 0; i < BPT; i++) rb[i] = inb ? *(const bf16x8*)(gb[i] + (k0 / GT_BK) * bstep + boff) : zero8();
    }
  };
  auto stash = [&](int buf, const bf16x8 (&ra)[APT], const bf16x8 (&rb)[BPT]) {
#pragma unroll
    for (int i = 0; i < APT; i++) *(bf16x8*)(&tiles[buf * (BM + BN) + prow + RPP * i][pcol]) = ra[i];
#pragma unroll
    for (int i = 0; i < BPT; i++) *(bf16x8*)(&tiles[buf * (BM + BN) + BM + brow[i]][bcol]) = rb[i];
  };
  auto multiply = [&](int buf) {
    if constexpr (NWM * NWN > 8) {
      // sixteen waves: 128 registers a wave, no room for a second set of operands
#pragma unroll
      for (int ks = 0; ks < GT_BK / 16; ks++) {
        bf16x8 fa[WMT], fb[2];
#pragma unroll
        for (int i = 0; i < WMT; i++) fa[i] = *(const bf16x8*)(&tiles[buf * (BM + BN) + wm * (32 * WMT) + i * 32 + lr][ks * 16 + lk * 8]);
#pragma unroll
        for (int j = 0; j < 2; j++) {
          const int row = GATED ? j * (BN / 2) + wn * 32 : wn * 64 + j * 32;
          fb[j] = *(const bf16x8*)(&tiles[buf * (BM + BN) + BM + row + lr][ks * 16 + lk * 8]);
        }
#pragma unroll
        for (int i = 0; i < WMT; i++)
#pragma unroll
          for (int j = 0; j < 2; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
      }
      return;
    }
    // the operands of k step ks + 1 are read from LDS while the products of step ks run: two
    // sets of fragments, and a fence that keeps the reads before the products they follow in
    // the source (the compiler would put every read right before its use and wait for it)
    bf16x8 fa[2][WMT], fb[2][2];
    auto read = [&](int ks, bf16x8 (&a)[WMT], bf16x8 (&b)[2]) {
#pragma unroll
      for (int i = 0; i < WMT; i++) a[i] = *(const bf16x8*)(&tiles[buf * (BM + BN) + wm * (32 * WMT) + i * 32 + lr][ks * 16 + lk * 8]);
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const int row = GATED ? j * (BN / 2) + wn * 32 : wn * 64 + j * 32;
        b[j] = *(const bf16x8*)(&tiles[buf * (BM + BN) + BM + row + lr][ks * 16 + lk * 8]);
      }
    };
    read(0, fa[0], fb[0]);
#pragma unroll
    for (int ks = 0; ks < GT_BK / 16; ks++) {
      if (ks + 1 < GT_BK / 16) read(ks + 1, fa[(ks + 1) & 1], fb[(ks + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0x616);
#pragma unroll
      for (int i = 0; i < WMT; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[ks & 1][j], fa[ks & 1][i], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0x616);
    }
  };
  // The loop takes two tiles a turn.  An odd number of tiles: when EXACT the first tile is
  // taken alone before the loop, otherwise the last one is all zeros.
  int kfirst = 0;
  if (EXACT && (K / GT_BK) % 2 == 1) {
    fetch(0, ra0, rb0);
    stash(0, ra0, rb0);
    __syncthreads();
    multiply(0);
    __syncthreads();
    kfirst = GT_BK;
  }
  if (kfirst < K) {
    fetch(kfirst, ra0, rb0);
    stash(0, ra0, rb0);
    fetch(kfirst + GT_BK, ra0, rb0);
    __syncthreads();
  }
  for (int k0 = kfirst; k0 < K; k0 += 2 * GT_BK) {
    // tile k0 is in buffer 0, tile k0 + BK in set 0
    fetch(k0 + 2 * GT_BK, ra1, rb1);
    multiply(0);
    stash(1, ra0, rb0);
    __syncthreads();
    // tile k0 + BK is in buffer 1, tile k0 + 2 BK in set 1
    fetch(k0 + 3 * GT_BK, ra0, rb0);
    multiply(1);
    stash(0, ra1, rb1);
    __syncthreads();
  }
  if (ksplit > 1) {
    // partial sums of this k range, in lane order; the join kernel adds the ranges up
    f32x16* mine = partials + (((size_t)blockIdx.x * ksplit + blockIdx.y) * (NWM * NWN) + wave) * (WMT * 2 * 64) + lane;
#pragma unroll
    for (int i = 0; i < WMT; i++)
#pragma unroll
      for (int j = 0; j < 2; j++) mine[(i * 2 + j) * 64] = acc[i][j];
    return;
  }
  // every wave has passed the loop's last barrier: the tile buffers are free
  if (!c_is_f32 && m0 + BM <= M && n0 + NCOLS <= N && ldc % 8 == 0 && (uintptr_t)C % 16 == 0) {
    constexpr int WCOLS = GATED ? 32 : 64;
    tile_store_staged<WMT, GATED>(acc, (__bf16*)C, ldc, m0 + wm * (32 * WMT), n0 + wn * WCOLS, lane, epi, cap,
                                  (__bf16*)gt_lds + (size_t)wave * (32 * WMT) * (WCOLS + 8));
    return;
  }
  tile_store<WMT, NWN, GATED>(acc, C, ldc, c_is_f32, M, N, m0, n0, wm, wn, lane, epi, cap);
}

// A tile product whose operands are copied from memory straight into LDS (global_load_lds, 16
// bytes a lane): no registers hold a tile on its way and no LDS writes are issued, so a wave
// has room for a second set of operand fragments, and LDS has room for GD_NS stages of 32 k
// values each.  The block meets at a barrier once per stage, and the reads of a wave's operands
// run one k step of 16 ahead of its products across that barrier: when the barrier of stage s
// has shown that stage s + 1 is there, its first operands are read while the second half of
// stage s is multiplied, so the matrix unit does not drain at a stage's end.  For weights in the
// strip layout and K a whole number of 64; the sums and their order are those of
// gemm_tile_kernel, and so are the partial sums of a split K and the results' way out.
// Measured on 2B and 9B layer shapes of 2,048 and 4,096 rows against the 256 x 256 block of
// sixteen waves that stages its tiles through registers: two stages of 64 k with one barrier
// each and 16-byte pieces of sixteen different rows a quarter wave 1.05 of its time; the same
// with 128-byte runs of a row 0.98; four stages of 32 k with the reads running ahead 0.96 (five
// stages 0.97); eight waves of 128 x 64 each instead of sixteen of 64 x 64 0.94.
//
// Such a load puts lane l's 16 bytes at (destination + 16 l).  W: a strip's 1 KB for one k
// step lies in LDS as it lies in memory, [k piece of 8][row 16][8 values]; an operand read
// (row lane % 32, k piece lane / 32) takes whole 256-byte runs.  A: an instruction takes 16
// rows x 32 k, four lanes a row (a 64-byte run of the row); lane c of a row fetches k piece
// c ^ ((row / 4) % 4), so piece q of row R lies at place q ^ ((R / 4) % 4) of the row's 64
// bytes and the sixteen rows a read takes at once lie in different banks.
#define ZK_GLOBAL_AS __attribute__((address_space(1)))
#define ZK_LDS_AS __attribute__((address_space(3)))
#define GD_NS 4
#define GD_BK 32
template <int WMT, int NWM, int NWN, bool GATED>
__global__ __launch_bounds__(64 * NWM * NWN, NWM * NWN <= 4 ? 2 : 1) void gemm_tile_direct_kernel(
    const __bf16* __restrict__ A, int lda, const __bf16* __restrict__ W, void* __restrict__ C, int ldc,
    int c_is_f32, int M, int N, int K_all, int epi, float cap, int tiles_m, int tiles_n, int w_strip,
    f32x16* __restrict__ partials, int ksplit, int tile_base) {
  constexpr int BM = 32 * WMT * NWM, BN = 64 * NWN, NW = NWM * NWN;
  constexpr int LPA = BM / 16 / NW, LPB = BN / 16 / NW;     // row blocks of A, strips of W, a wave copies
  static_assert(LPA * NW * 16 == BM && LPB * NW * 16 == BN, "the waves do not share the copies evenly");
  constexpr int HALF = BM * GD_BK * 2, STAGE = (BM + BN) * GD_BK * 2;      // bytes of a stage's A part, of a stage
  extern __shared__ __align__(16) unsigned char gt_lds[];
  int tm, tn;
  tile_of_block(blockIdx.x + tile_base, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM;
  constexpr int NCOLS = GATED ? BN / 2 : BN;
  const int n0 = tn * NCOLS;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / NWN, wn = wave % NWN;
  const int lr = lane & 31, lk = lane >> 5;
  const int ktiles = K_all / GT_BK;
  const int kt0 = (int)((long)blockIdx.y * ktiles / ksplit), kt1 = (int)((long)(blockIdx.y + 1) * ktiles / ksplit);
  const int ns = 2 * (kt1 - kt0);                       // stages: an even number
  // a wave copies the 16-row blocks wave, wave + NW, .. of A and the same strips of W
  const __bf16* ga[LPA];
  const __bf16* gw[LPB];
  const int ksteps = K_all / 32;
  const int strips = GATED ? 2 * N / 16 : N / 16;
#pragma unroll
  for (int c = 0; c < LPA; c++) {
    const int a_row = (wave + c * NW) * 16 + (lane >> 2);
    ga[c] = A + (size_t)min(m0 + a_row, M - 1) * lda + (size_t)kt0 * GT_BK + (((lane & 3) ^ ((a_row >> 2) & 3)) * 8);
  }
#pragma unroll
  for (int c = 0; c < LPB; c++) {
    const int blk = wave + c * NW;
    int gs;
    if (GATED) gs = blk < BN / 32 ? n0 / 16 + blk : N / 16 + n0 / 16 + (blk - BN / 32);
    else gs = n0 / 16 + blk;
    gs = min(gs, strips - 1);
    gw[c] = W + ((size_t)gs * ksteps + 2 * kt0) * 512 + lane * 8;
  }
  auto issue = [&](int buf, int stage) {
    stage = min(stage, ns - 1);      // past the end: the last stage again, into a buffer nobody reads
    unsigned char* dst = gt_lds + buf * STAGE + wave * 1024;
#pragma unroll
    for (int c = 0; c < LPA; c++)
      __builtin_amdgcn_global_load_lds((const ZK_GLOBAL_AS void*)(ga[c] + (size_t)stage * GD_BK), (ZK_LDS_AS void*)(dst + c * NW * 1024), 16, 0, 0);
#pragma unroll
    for (int c = 0; c < LPB; c++)
      __builtin_amdgcn_global_load_lds((const ZK_GLOBAL_AS void*)(gw[c] + (size_t)stage * 512), (ZK_LDS_AS void*)(dst + HALF + c * NW * 1024), 16, 0, 0);
  };
  // where a lane reads its operand pieces of k step ks (0 or 1) of a stage
  int a_at[2];
#pragma unroll
  for (int ks = 0; ks < 2; ks++) a_at[ks] = (wm * (32 * WMT) + lr) * 64 + (((ks * 2 + lk) ^ ((lr >> 2) & 3)) * 16);   // + i * 2048
  const int w_row = GATED ? wn * 32 : wn * 64;                                    // + j * (GATED ? 128 : 32)
  const int w_at = HALF + (w_row / 16 + (lr >> 4)) * 1024 + lk * 256 + (lr & 15) * 16;   // + ks * 512 + j * W_J
  constexpr int W_J = GATED ? (BN / 32) * 1024 : 2048;
  f32x16 acc[WMT][2];
#pragma unroll
  for (int i = 0; i < WMT; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;
  bf16x8 fa[2][WMT], fb[2][2];
  auto read = [&](int buf, int ks) {
    const unsigned char* base = gt_lds + buf * STAGE;
#pragma unroll
    for (int i = 0; i < WMT; i++) fa[ks][i] = *(const bf16x8*)(base + a_at[ks] + i * 2048);
#pragma unroll
    for (int j = 0; j < 2; j++) fb[ks][j] = *(const bf16x8*)(base + w_at + ks * 512 + j * W_J);
  };
  auto products = [&](int ks) {
    __builtin_amdgcn_sched_barrier(0x616);
#pragma unroll
    for (int i = 0; i < WMT; i++)
#pragma unroll
      for (int j = 0; j < 2; j++)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[ks][j], fa[ks][i], acc[i][j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0x616);
  };
  // Stage s lives in buffer s % GD_NS.  In flight when a step begins: stages s + 1 .. s + GD_NS - 2
  // (LPA + LPB loads a wave each); the wait is for the wave's own loads of stage s + 1, the barrier
  // then says that every wave's are there and that every wave has read stage s - 1 (the products
  // that use its operands were issued before the barrier, so the operands had arrived), whose
  // buffer the next loads go to.
  auto step = [&](int b, int s) {
    read(b, 1);
    products(0);
    // (the barrier as text: before one it knows, the compiler waits for every load in flight)
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((LPA + LPB) * (GD_NS - 3)) : "memory");
    issue((b + GD_NS - 1) % GD_NS, s + GD_NS - 1);
    read((b + 1) % GD_NS, 0);
    products(1);
  };
#pragma unroll
  for (int b = 0; b < GD_NS - 1; b++) issue(b, b);
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((LPA + LPB) * (GD_NS - 2)) : "memory");
  read(0, 0);
  for (int s = 0; s < ns; s += GD_NS) {
#pragma unroll
    for (int b = 0; b < GD_NS; b += 2) {
      if (b > 0 && s + b >= ns) break;
      step(b, s + b);
      step(b + 1, s + b + 1);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();                              // the buffers are free for the results' way out
  if (ksplit > 1) {
    f32x16* mine = partials + (((size_t)blockIdx.x * ksplit + blockIdx.y) * NW + wave) * (WMT * 2 * 64) + lane;
#pragma unroll
    for (int i = 0; i < WMT; i++)
#pragma unroll
      for (int j = 0; j < 2; j++) mine[(i * 2 + j) * 64] = acc[i][j];
    return;
  }
  if (!c_is_f32 && m0 + BM <= M && n0 + NCOLS <= N && ldc % 8 == 0 && (uintptr_t)C % 16 == 0) {
    constexpr int WCOLS = GATED ? 32 : 64;
    tile_store_staged<WMT, GATED>(acc, (__bf16*)C, ldc, m0 + wm * (32 * WMT), n0 + wn * WCOLS, lane, epi, cap,
                                  (__bf16*)gt_lds + (size_t)wave * (32 * WMT) * (WCOLS + 8));
    return;
  }
  tile_store<WMT, NWN, GATED>(acc, C, ldc, c_is_f32, M, N, m0, n0, wm, wn, lane, epi, cap);
}

// Second half of a tile product whose K was split over blocks: the ranges are added in order.
// A thread takes four consecutive floats of a lane's accumulator pair (i, 0), (i, 1), so the
// partial sums are read in 16-byte pieces, neighbours by neighbouring threads.
template <int WMT, int NWM, int NWN, bool GATED>
__global__ __launch_bounds__(256) void gemm_tile_join_kernel(
    const f32x4* __restrict__ partials, int ksplit, void* __restrict__ C, int ldc, int c_is_f32, int M,
    int N, int epi, float cap, int tiles_m, int tiles_n, int tile_base, int tile_count) {
  constexpr int BM = 32 * WMT * NWM, BN = 64 * NWN, NW = NWM * NWN;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  const int b = (int)(idx & 3), lane = (int)((idx >> 2) & 63);
  const int i = (int)((idx >> 8) % WMT), wave = (int)((idx >> 8) / WMT % NW);
  const int tile = (int)((idx >> 8) / (WMT * NW));      // counted from the launch's first tile, as the partial sums are
  if (tile >= tile_count) return;
  int tm, tn;
  tile_of_block(tile + tile_base, tiles_m, tiles_n, tm, tn);
  // float4 index of (tile, range p, wave, pair member j, lane, b): an accumulator is 4 float4
  const size_t per_wave = (size_t)WMT * 2 * 64 * 4;
  if constexpr (!GATED) {
    // A whole tile into a 16-bit C with rows of whole 16-byte pieces: a thread takes the two
    // halves (lanes lr and lr + 32) of eight neighbouring columns of a row, so its store is 16
    // bytes and four threads fill a 64-byte line (the general way below stores two bytes at a
    // time, half a line's bytes from one wave and the other half from another).  The block's
    // 256 threads are (b, lr, j) here; the sums are the same, in the same order.
    const int m0 = tm * BM + (wave / NWN) * (32 * WMT) + i * 32, n0 = tn * BN + (wave % NWN) * 64;
    if (!c_is_f32 && epi == EPI_NONE && ldc % 8 == 0 && (uintptr_t)C % 16 == 0 && m0 + 32 <= M && n0 + 64 <= N) {
      const int lr = lane & 31, j = lane >> 5;
      const f32x4* at = partials + ((size_t)tile * ksplit * NW + wave) * per_wave + ((size_t)(i * 2 + j) * 64 + lr) * 4 + b;
      f32x4 lo = at[0], hi = at[32 * 4];
      for (int p = 1; p < ksplit; p++) {
        lo += at[(size_t)p * NW * per_wave];
        hi += at[(size_t)p * NW * per_wave + 32 * 4];
      }
      bf16x8 out;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        out[e] = (__bf16)lo[e];
        out[4 + e] = (__bf16)hi[e];
      }
      *(bf16x8*)((__bf16*)C + (size_t)(m0 + lr) * ldc + n0 + j * 32 + 8 * b) = out;
      return;
    }
  }
  const f32x4* src = partials + ((size_t)tile * ksplit * NW + wave) * per_wave + ((size_t)(i * 2) * 64 + lane) * 4 + b;
  f32x4 x0 = src[0], x1 = src[64 * 4];
  for (int p = 1; p < ksplit; p++) {
    x0 += src[(size_t)p * NW * per_wave];
    x1 += src[(size_t)p * NW * per_wave + 64 * 4];
  }
  tile_store_quad<WMT, NWN, GATED>(x0, x1, i, b, C, ldc, c_is_f32, M, N, tm * BM, tn * (GATED ? BN / 2 : BN),
                                   wave / NWN, wave % NWN, lane, epi, cap);
}

template <int WMT, int NWM, int NWN, bool GATED, bool EXACT, bool DIRECT = false>
static int launch_tile(const void* A, int lda, const void* W, void* C, int ldc, int c_is_f32, int M, int N,
                       int K, int epi, float cap, int w_strip, const GemmWorkspace& wsp, int ksplit,
                       int tail_split, hipStream_t s) {
  constexpr int BM = 32 * WMT * NWM, BN = 64 * NWN;
  constexpr int ncols = GATED ? BN / 2 : BN;
  constexpr size_t lds_staged = (size_t)2 * (BM + BN) * GT_LD * sizeof(__bf16);
  constexpr size_t lds = DIRECT && (size_t)GD_NS * (BM + BN) * GD_BK * 2 > lds_staged ? (size_t)GD_NS * (BM + BN) * GD_BK * 2 : lds_staged;
  auto kernel = gemm_tile_kernel<WMT, NWM, NWN, GATED, EXACT>;
  if constexpr (DIRECT) kernel = gemm_tile_direct_kernel<WMT, NWM, NWN, GATED>;
  static bool prepared = false;
  if (!prepared) {
    if (lds > 64 * 1024 &&
        hipFuncSetAttribute((const void*)kernel,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return zk_fail("zk_gemm_bf16: the tile kernel's LDS buffers were refused");
    prepared = true;
  }
  const int tiles_n = (N + ncols - 1) / ncols, tiles_m = (M + BM - 1) / BM;
  ZK_REQUIRE((long long)tiles_m * tiles_n < 2147483647LL, "zk_gemm_bf16: too many tiles");
  // K split over blockIdx.y only as far as the partial sums fit the workspace
  const size_t per_range = (size_t)tiles_m * tiles_n * BM * BN * sizeof(float);
  void* ws = wsp.ptr;
  if (ws == nullptr || (uintptr_t)ws % 64 != 0) ksplit = 1;
  while (ksplit > 1 && per_range * ksplit > wsp.split_bytes()) ksplit--;
  if (ksplit > 1 && per_range * ksplit > wsp.bytes) return wsp.too_small(per_range * ksplit);
  const int tiles = tiles_m * tiles_n;
  // The tail.  The CUs take the tiles in rounds (256 a round for the blocks of eight and sixteen
  // waves, 512 for those of four, two of which share a CU), and a last round with few tiles
  // costs a whole round's time.  Where the caller's model of the times says it pays (a long K:
  // the partial sums of about 256 tile ranges, 16 to 67 MB, cost the same whatever K is), such
  // a last round goes into a launch of its own that splits K into ``tail_split`` ranges, and a
  // join of those tiles alone.
  constexpr int round_blocks = 256 * (NWM * NWN <= 4 ? 2 : 1);
  const int tail = tiles % round_blocks;
  if (ksplit > 1 || tail == 0 || tiles <= round_blocks || ws == nullptr || (uintptr_t)ws % 64 != 0) tail_split = 1;
  if (tail_split > 1 && (size_t)tail * tail_split * BM * BN * sizeof(float) > wsp.split_bytes()) tail_split = 1;
  if (tail_split > 1 && (size_t)tail * tail_split * BM * BN * sizeof(float) > wsp.bytes)
    return wsp.too_small((size_t)tail * tail_split * BM * BN * sizeof(float));
  const int whole = tail_split > 1 ? tiles - tail : tiles;
  kernel<<<dim3(whole, ksplit), 64 * NWM * NWN, lds, s>>>(
      (const __bf16*)A, lda, (const __bf16*)W, C, ldc, c_is_f32, M, N, K, epi, cap, tiles_m, tiles_n, w_strip,
      (f32x16*)ws, ksplit, 0);
  if (ksplit > 1)
    gemm_tile_join_kernel<WMT, NWM, NWN, GATED><<<dim3(tiles * WMT * NWM * NWN), 256, 0, s>>>(
        (const f32x4*)ws, ksplit, C, ldc, c_is_f32, M, N, epi, cap, tiles_m, tiles_n, 0, tiles);
  if (tail_split > 1) {
    kernel<<<dim3(tail, tail_split), 64 * NWM * NWN, lds, s>>>(
        (const __bf16*)A, lda, (const __bf16*)W, C, ldc, c_is_f32, M, N, K, epi, cap, tiles_m, tiles_n, w_strip,
        (f32x16*)ws, tail_split, whole);
    gemm_tile_join_kernel<WMT, NWM, NWN, GATED><<<dim3(tail * WMT * NWM * NWN), 256, 0, s>>>(
        (const f32x4*)ws, tail_split, C, ldc, c_is_f32, M, N, epi, cap, tiles_m, tiles_n, whole, tail);
  }
  return zk_launch_status("zk_gemm_bf16 (tile)");
}

// A caller that passes `parts` takes the partial sums of a split product as they are: planes of
// [M, N] floats at the start of the workspace, nothing in C.  That fits a plain product into a
// 16-bit C whose rows are N long, N a whole number of strips.
static bool joinable_by_reader(int N, int ldc, int c_is_f32, int epi) {
  return N % 16 == 0 && ldc == N && !c_is_f32 && epi == EPI_NONE;
}

// ------------------------------------------------------------------ mid (16 < M <= 64)
// With more than one column tile the activations weigh more than the weights on the way
// from L2 to the CUs when every 16-row strip fetches them again (64 rows of A per 16 rows
// of W).  Here a block owns four strips, a pair of waves each, all walk K together, and the
// activations of the current 256-wide k chunk wait in LDS for all of them: 64 rows of A per
// 64 rows of W.  Weights come straight from global memory in strip layout, the loads of the
// next two chunks are in flight while the current one is multiplied.
//
// Few column blocks (N of a few thousand) cannot fill 256 CUs, so blockIdx.y splits K into
// `ksplit` ranges.  Then each block leaves its partial sums in the workspace and a second,
// small kernel adds them in the order of the ranges and applies the epilogue.  (One kernel
// with a ticket per column block, the last block adding up, was measured three times slower:
// the device-wide fences it needs write back and invalidate the L2 of every XCD.)
#define GM_STEPS 8
#define GM_LD (GM_STEPS * 32 + 16)

// A lane's results of one strip: rows n = 16 * strip + 4 * kq + i of W, column m = 16 * mt + r of A.
template <int MT, bool GATED>
__device__ __forceinline__ void mid_store(const f32x4 (&acc)[GATED ? 2 : 1][MT], void* __restrict__ C, int ldc,
                                          int c_is_f32, int M, int N, int strip, int lane, int epi, float cap,
                                          float* __restrict__ picks, int nstrips) {
  const int r = lane & 15, kq = lane >> 4;
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
    const int m = mt * 16 + r;
    if (!GATED && epi == EPI_PICK) {
      const float x[4] = {acc[0][mt][0], acc[0][mt][1], acc[0][mt][2], acc[0][mt][3]};
      const Pick p = pick_of_strip(x, strip * 16 + 4 * kq, N, cap);
      if (kq == 0 && m < M) ((Pick*)picks)[(size_t)m * nstrips + strip] = p;
      continue;
    }
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int n = strip * 16 + 4 * kq + i;
      if (n >= N) continue;
      float x = acc[0][mt][i];
      if (GATED) x = epi_gate(x, acc[GATED ? 1 : 0][mt][i], epi);
      else if (epi == EPI_SOFTCAP) x = cap * tanhf(x / cap);
      if (c_is_f32) ((float*)C)[(size_t)m * ldc + n] = x;
      else ((__bf16*)C)[(size_t)m * ldc + n] = (__bf16)x;
    }
  }
}

// Eight waves a block, two for each of its four strips: waves 0..3 take the first half of a
// chunk's steps, waves 4..7 the second, and the second wave's sums reach the first through LDS
// at the end.  A wave holds three chunks' weights in registers (one being multiplied, two on
// their way) and the activations have three buffers in LDS: a chunk's products take less time
// than a load (at 64 rows with a gate about 1.2 us against 2 us), so with one chunk on its way
// every chunk waited for its loads, and where the column blocks are too few for a second block
// on the CU (N = 9216 with a gate: 144 blocks) nothing filled the wait.  Against four waves with
// one chunk ahead: 5 to 17 % less time at 24 to 64 rows on the layer shapes of the 2B, 9B and
// 27B models (2B down at 64 rows 15.4 -> 13.1 us, 9B down at 32 rows 25.0 -> 21.2 us); two waves
// a strip alone, without the second chunk ahead, gave 0 to 3 %.
template <int MT, bool GATED>
__global__ __launch_bounds__(512) void gemm_mid_kernel(const __bf16* __restrict__ A, int lda,
                                                        const __bf16* __restrict__ W,
                                                        void* __restrict__ C, int ldc, int c_is_f32,
                                                        int M, int N, int K, int epi, float cap,
                                                        float* __restrict__ partials, int ksplit, int spb) {
  constexpr int NS = GATED ? 2 : 1;
  constexpr int WSTEPS = GM_STEPS / 2;                  // steps of a chunk a wave multiplies
  __shared__ __bf16 sA[3][MT * 16][GM_LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = (tid >> 6) & 3, khalf = tid >> 8;
  const int r = lane & 15, kq = lane >> 4;
  const int ksteps = K / 32;
  const int s_begin = (int)((long)blockIdx.y * ksteps / ksplit);
  const int s_end = (int)((long)(blockIdx.y + 1) * ksteps / ksplit);
  const int nstrips = (N + 15) / 16;
  // spb strips a block (3 where that spreads the strips more evenly over the CUs).  The waves of
  // the fourth place then do the first place's work over again and store nothing: their loads
  // hit what the first place's waves have just fetched, and a branch around loads would make
  // the compiler wait for every load in flight.
  const int strip = blockIdx.x * spb + (wave < spb ? wave : 0);
  const bool strip_ok = wave < spb && strip < nstrips;
  const int strip_read = strip < nstrips ? strip : 0;
  const __bf16* wp[NS];
  wp[0] = W + (size_t)strip_read * ksteps * 512 + lane * 8;
  if (GATED) wp[NS - 1] = W + ((size_t)(N / 16) + strip_read) * ksteps * 512 + lane * 8;
  // A pieces of a chunk: MT*16 rows x 32 pieces of 16 bytes, 16 rows a pass of the 512 threads
  constexpr int APT = MT * 16 * 32 / 512;
  const int a_piece = tid & 31, a_row0 = tid >> 5;
  f32x4 acc[NS][MT];
#pragma unroll
  for (int g = 0; g < NS; g++)
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[g][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Every load is issued, none under a condition: a step past the range reads the range's last
  // step again, a row past M row M - 1; activations outside are set to zero afterwards, which
  // makes the product nothing whatever the weights.
  auto fetch_a = [&](int s0, bf16x8 (&ra)[APT]) {
#pragma unroll
    for (int j = 0; j < APT; j++) {
      const int row = a_row0 + 16 * j;
      const bool in = row < M && s0 + a_piece / 4 < s_end;
      const int step = min(s0 + a_piece / 4, s_end - 1);
      const bf16x8 v = *(const bf16x8*)(A + (size_t)min(row, M - 1) * lda + step * 32 + (a_piece % 4) * 8);
      ra[j] = in ? v : zero8();
    }
  };
  auto stash_a = [&](int buf, const bf16x8 (&ra)[APT]) {
#pragma unroll
    for (int j = 0; j < APT; j++) *(bf16x8*)(&sA[buf][a_row0 + 16 * j][a_piece * 8]) = ra[j];
  };
  auto fetch_w = [&](int s0, bf16x8 (&wf)[NS][WSTEPS]) {
#pragma unroll
    for (int s = 0; s < WSTEPS; s++)
#pragma unroll
      for (int g = 0; g < NS; g++)
        wf[g][s] = *(const bf16x8*)(wp[g] + (size_t)min(s0 + khalf * WSTEPS + s, s_end - 1) * 512);
  };
  auto multiply = [&](int buf, const bf16x8 (&wf)[NS][WSTEPS]) {
#pragma unroll
    for (int s = 0; s < WSTEPS; s++)
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        const bf16x8 af = *(const bf16x8*)(&sA[buf][mt * 16 + r][(khalf * WSTEPS + s) * 32 + kq * 8]);
#pragma unroll
        for (int g = 0; g < NS; g++)
          acc[g][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[g][s], af, acc[g][mt], 0, 0, 0);
      }
  };

  // Chunk c: its activations wait in LDS buffer c % 3, its weights in register set c % 3; the
  // activations of chunk c + 1 are in register set (c + 1) % 2 on their way to LDS.  A turn
  // asks for chunk c + 2, multiplies chunk c, puts chunk c + 1's activations into LDS.
  bf16x8 ra0[APT], ra1[APT], w0[NS][WSTEPS], w1[NS][WSTEPS], w2[NS][WSTEPS];
  fetch_a(s_begin, ra0);
  fetch_w(s_begin, w0);
  fetch_a(s_begin + GM_STEPS, ra1);
  fetch_w(s_begin + GM_STEPS, w1);
  stash_a(0, ra0);
  __syncthreads();
#define ZK_MID8_TURN(BUF, WCUR, WNEXT2, RA_NEXT2, RA_NEXT1)   \
  fetch_a(s0 + 2 * GM_STEPS, RA_NEXT2);                       \
  fetch_w(s0 + 2 * GM_STEPS, WNEXT2);                         \
  multiply(BUF, WCUR);                                        \
  s0 += GM_STEPS;                                             \
  if (s0 >= s_end) break;                                     \
  stash_a((BUF + 1) % 3, RA_NEXT1);                           \
  __syncthreads();
  for (int s0 = s_begin;;) {
    ZK_MID8_TURN(0, w0, w2, ra0, ra1)
    ZK_MID8_TURN(1, w1, w0, ra1, ra0)
    ZK_MID8_TURN(2, w2, w1, ra0, ra1)
    ZK_MID8_TURN(0, w0, w2, ra1, ra0)
    ZK_MID8_TURN(1, w1, w0, ra0, ra1)
    ZK_MID8_TURN(2, w2, w1, ra1, ra0)
  }
#undef ZK_MID8_TURN
  // the second wave of each strip hands its sums over (the activation buffers are free once
  // every wave has left the loop); first half + second half, in that order
  __syncthreads();
  static_assert(sizeof(sA) >= (size_t)4 * NS * MT * 64 * sizeof(f32x4), "no room to hand the sums over");
  f32x4* hand = (f32x4*)&sA[0][0][0] + ((size_t)wave * NS * MT) * 64 + lane;
  if (khalf == 1) {
#pragma unroll
    for (int g = 0; g < NS; g++)
#pragma unroll
      for (int mt = 0; mt < MT; mt++) hand[(g * MT + mt) * 64] = acc[g][mt];
  }
  __syncthreads();
  if (khalf == 1) return;
#pragma unroll
  for (int g = 0; g < NS; g++)
#pragma unroll
    for (int mt = 0; mt < MT; mt++) acc[g][mt] += hand[(g * MT + mt) * 64];
  if (ksplit > 1) {
    // the range's partial sums: plane (range, g) of [M, npad] floats
    if (!strip_ok) return;
    const size_t npad = (size_t)nstrips * 16;
    float* planes = partials + (size_t)blockIdx.y * NS * M * npad + strip * 16 + 4 * kq;
#pragma unroll
    for (int g = 0; g < NS; g++)
#pragma unroll
      for (int mt = 0; mt < MT; mt++)
        if (mt * 16 + r < M) *(f32x4*)(planes + ((size_t)g * M + mt * 16 + r) * npad) = acc[g][mt];
    return;
  }
  if (strip_ok) mid_store<MT, GATED>(acc, C, ldc, c_is_f32, M, N, strip, lane, epi, cap, partials, nstrips);
}

// Second half of a mid product whose K was split over blocks: `ksplit`
// ranges of one ([M, npad] floats) or, GATED, two planes each; a thread adds four neighbouring
// columns of a row in the order of the ranges and applies the epilogue.  A reader that adds the
// planes up itself in the same order (zk_norm_add_norm) makes this launch unnecessary.
template <bool GATED>
__global__ __launch_bounds__(256) void gemm_join_kernel(const float* __restrict__ partials, int ksplit,
                                                        void* __restrict__ C, int ldc, int c_is_f32, int M,
                                                        int N, int npad, int epi, float cap) {
  constexpr int NS = GATED ? 2 : 1;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  const int m = (int)(idx / (npad / 4)), n = (int)(idx % (npad / 4)) * 4;
  if (m >= M) return;
  const size_t plane = (size_t)M * npad;
  const float* at = partials + (size_t)m * npad + n;
  f32x4 x = *(const f32x4*)at, y = x;
  if (GATED) y = *(const f32x4*)(at + plane);
  for (int p = 1; p < ksplit; p++) {
    x += *(const f32x4*)(at + (size_t)p * NS * plane);
    if (GATED) y += *(const f32x4*)(at + ((size_t)p * NS + 1) * plane);
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    if (n + i >= N) continue;
    float v = x[i];
    if (GATED) v = epi_gate(v, y[i], epi);
    else if (epi == EPI_SOFTCAP) v = cap * tanhf(v / cap);
    if (c_is_f32) ((float*)C)[(size_t)m * ldc + n + i] = v;
    else ((__bf16*)C)[(size_t)m * ldc + n + i] = (__bf16)v;
  }
}


template <bool GATED>
static int launch_mid(const void* A, int lda, const void* W, void* C, int ldc, int c_is_f32, int M, int N,
                      int K, int epi, float cap, const GemmWorkspace& wsp, int* parts, hipStream_t s) {
  const int mt = (M + 15) / 16;
  const int npad = (N + 15) / 16 * 16;
  const int nstrips = (N + 15) / 16;
  // Strips a block: four, or three where the blocks of four fill the CUs unevenly and K is not
  // split anyway (N = 9216 with a gate is 576 strips: 144 blocks of four leave 112 CUs idle, 192
  // blocks of three give every busy CU a quarter less to read: 28.0 -> 24.6 us at 64 rows;
  // 2304 strips: three rounds of blocks either way, 157 -> 146 us).  What counts is the most
  // strips a CU gets, rounds of 256 blocks times the strips of a block.
  int spb = 4;
  {
    auto most = [&](int b) { return (long)(((nstrips + b - 1) / b + 255) / 256) * b; };
    if ((nstrips + 3) / 4 > 128 && most(3) * 10 <= most(4) * 9) spb = 3;
  }
  const int cblocks = (nstrips + spb - 1) / spb;
  // Split K until every CU has a block, a range no shorter than a chunk of GM_STEPS steps; two
  // blocks a CU where ranges stay long (16 chunks or more: the blocks of a CU then cover each
  // other's waits).  More ranges than that cost more in partial sums than they gain.  The
  // longest range sets the time, so of the splits with that longest range the one with the
  // fewest ranges is taken (8 chunks: 4 ranges of 2 instead of 7 of 1 or 2; measured at the
  // shapes of the 2B, 9B and 27B layers with 24 to 64 rows).
  const int chunks = max(1, K / 32 / GM_STEPS);
  int ksplit = max(1, min(256 / cblocks, chunks));
  if (chunks / max(1, 512 / cblocks) >= 16) ksplit = max(1, min(512 / cblocks, chunks));
  {
    const int longest = (chunks + ksplit - 1) / ksplit;
    ksplit = (chunks + longest - 1) / longest;
  }
  const size_t per_range = (size_t)(GATED ? 2 : 1) * M * npad * sizeof(float);
  void* ws = wsp.ptr;
  if (ws == nullptr || (uintptr_t)ws % 16 != 0 || epi == EPI_PICK) ksplit = 1;      // picks are taken from whole sums
  while (ksplit > 1 && ksplit * per_range > wsp.split_bytes()) ksplit--;
  if (ksplit > 1 && ksplit * per_range > wsp.bytes) return wsp.too_small(ksplit * per_range);
  float* partials = (float*)ws;
  dim3 grid(cblocks, ksplit);
#define ZK_MID(MT_)                                                                                   \
  gemm_mid_kernel<MT_, GATED><<<grid, 512, 0, s>>>((const __bf16*)A, lda, (const __bf16*)W, C, ldc, c_is_f32, \
                                                   M, N, K, epi, cap, partials, ksplit, spb)
  if (mt == 2) { ZK_MID(2); }
  else if (mt == 3) { ZK_MID(3); }
  else { ZK_MID(4); }
#undef ZK_MID
  if (ksplit > 1) {
    if (parts && joinable_by_reader(N, ldc, c_is_f32, epi)) {
      *parts = ksplit;
      return zk_launch_status("zk_gemm_bf16 (mid)");
    }
    const size_t quads = (size_t)M * (npad / 4);
    gemm_join_kernel<GATED><<<(unsigned)((quads + 255) / 256), 256, 0, s>>>(partials, ksplit, C, ldc, c_is_f32, M, N,
                                                                          npad, epi, cap);
  }
  return zk_launch_status("zk_gemm_bf16 (mid)");
}

template <bool GATED>
static int launch_skinny(const void* A, int lda, const void* W, void* C, int ldc, int c_is_f32, int M,
                         int N, int K, int epi, float cap, int w_strip, const GemmWorkspace& wsp, int* parts,
                         hipStream_t s) {
  const int mt = (M + 15) / 16;
  dim3 grid((N + 15) / 16);
  // A strip is a block, and the blocks of a CU share its way to memory: the kernel takes as
  // long as the CU with the most blocks.  288 strips (N = 4608) leave 32 of the 256 CUs with two
  // blocks and the rest with one, twice the time of an even spread; 144 strips leave 112 CUs
  // idle.  Splitting K into ks ranges makes ks times the blocks of 1/ks the length, and the time
  // of the fullest CU goes with ceil(strips ks / 256) / ks.  That pays where strips are more
  // than the CUs and spread unevenly (N = 4608 with K = 36864 at 8 rows: 87 -> 50 us with eight
  // ranges); with fewer strips than CUs it was measured three times and lost each time (144
  // strips, two and eight ranges: the product then goes as fast as memory gives to this pattern
  // of reads whatever the number of CUs, and the shorter blocks only add their start-up).
  // Only where the reader adds up the partial sums itself (the norm kernel, through `parts`):
  // a joining launch would cost what the split gains.
  int ksplit = 1;
  float* partials = (float*)wsp.ptr;
  const size_t npad = (size_t)grid.x * 16;
  if (!GATED && mt == 1 && w_strip && grid.x > 256 && parts != nullptr && partials != nullptr &&
      (uintptr_t)partials % 16 == 0 && joinable_by_reader(N, ldc, c_is_f32, epi)) {
    auto longest = [&](int ks) { return (double)(((long)grid.x * ks + 255) / 256) / ks; };
    double best = longest(1);
    for (int ks = 2; ks <= 8; ks *= 2) {
      if (K / ks < 1024 || (size_t)ks * M * npad * sizeof(float) > wsp.split_bytes()) break;
      if (longest(ks) < 0.97 * best && longest(ks) <= 0.85 * longest(1)) {
        best = longest(ks);
        ksplit = ks;
      }
    }
    if (ksplit > 1 && (size_t)ksplit * M * npad * sizeof(float) > wsp.bytes)
      return wsp.too_small((size_t)ksplit * M * npad * sizeof(float));
    grid.y = ksplit;
  }
  // few strips: eight waves a strip keep enough loads in flight
  const bool wide = (long)grid.x * ksplit < 512 && K / ksplit >= 2048 && mt <= 2;
#define ZK_SKINNY(MT_, NW_)                                                                           \
  do {                                                                                                \
    if (w_strip)                                                                                      \
      gemm_skinny_kernel<MT_, GATED, NW_, false, true><<<grid, NW_ * 64, 0, s>>>(                     \
          (const __bf16*)A, lda, (const __bf16*)W, C, ldc, c_is_f32, M, N, K, epi, cap, w_strip, RopeStore{}, \
          partials, 1);                                                                               \
    else                                                                                              \
      gemm_skinny_kernel<MT_, GATED, NW_><<<grid, NW_ * 64, 0, s>>>(                                  \
          (const __bf16*)A, lda, (const __bf16*)W, C, ldc, c_is_f32, M, N, K, epi, cap, w_strip, RopeStore{}, \
          partials, 1);                                                                               \
  } while (0)
  if (ksplit > 1) {
    if constexpr (!GATED) {
      if (wide)
        gemm_skinny_kernel<1, false, 8, false, true, true><<<grid, 8 * 64, 0, s>>>(
            (const __bf16*)A, lda, (const __bf16*)W, C, ldc, c_is_f32, M, N, K, epi, cap, w_strip, RopeStore{},
            partials, ksplit);
      else
        gemm_skinny_kernel<1, false, 4, false, true, true><<<grid, 4 * 64, 0, s>>>(
            (const __bf16*)A, lda, (const __bf16*)W, C, ldc, c_is_f32, M, N, K, epi, cap, w_strip, RopeStore{},
            partials, ksplit);
    }
  } else if (mt == 1) { if (wide) ZK_SKINNY(1, 8); else ZK_SKINNY(1, 4); }
  else if (mt == 2) { if (wide) ZK_SKINNY(2, 8); else ZK_SKINNY(2, 4); }
  else if (mt == 3) ZK_SKINNY(3, 4);
  else ZK_SKINNY(4, 4);
#undef ZK_SKINNY
  if (ksplit > 1) *parts = ksplit;
  return zk_launch_status("zk_gemm_bf16 (skinny)");
}

// The q|k|v product of up to 16 decoded tokens with the rotation and the cache store as its
// epilogue: W [(nh + 2 nkv) hd, K] (row-major or strip layout), q rotated into Q [M, ldq] at
// columns [0, nh hd), k rotated and v as it is into the cache at slot_map[m] (a negative slot
// stores nothing).  The same bits as zk_gemm_bf16 followed by zk_rope_cache_write.  nkv may be 0
// (a mixer that reads another's cache); then slot_map and the caches are not used.
extern "C" int zk_qkv_rope_bf16_supports(int M, int K, int hd, int rotary_dim) {
  return M >= 1 && M <= 16 && K % 8 == 0 && hd % 16 == 0 && rotary_dim == hd;
}

extern "C" int zk_qkv_rope_bf16(const void* A, int lda, const void* W, void* Q, int ldq, int M, int K,
                                int w_strip, const int* positions, const int* slot_map,
                                const float* inv_freq, void* kcache, void* vcache, int nh, int nkv, int hd,
                                int bs, int v_transposed, void* stream) {
  ZK_REQUIRE(M >= 1 && M <= 16 && K > 0 && K % 8 == 0 && lda % 8 == 0 && lda >= K,
             "zk_qkv_rope_bf16: 1 to 16 rows, K and lda multiples of 8");
  ZK_REQUIRE(nh > 0 && nkv >= 0 && hd > 0 && hd % 16 == 0, "zk_qkv_rope_bf16: head_dim must be a multiple of 16");
  ZK_REQUIRE(ldq >= nh * hd && ldq % 4 == 0, "zk_qkv_rope_bf16: ldq too small or not a multiple of 4");
  ZK_REQUIRE(!w_strip || K % 32 == 0, "zk_qkv_rope_bf16: strip layout needs K % 32 == 0");
  ZK_REQUIRE(positions && inv_freq, "zk_qkv_rope_bf16: positions and inv_freq are needed");
  ZK_REQUIRE(nkv == 0 || (slot_map && kcache && vcache && bs > 0), "zk_qkv_rope_bf16: the cache is needed");
  ZK_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0) && ((uintptr_t)Q % 8 == 0),
             "zk_qkv_rope_bf16: operands must be 16-byte aligned");
  const int N = (nh + 2 * nkv) * hd;
  RopeStore rs{positions, nkv ? slot_map : nullptr, inv_freq, (__bf16*)kcache, (__bf16*)vcache, nh, nkv, hd, bs,
               v_transposed};
  dim3 grid(N / 16);
  hipStream_t s = (hipStream_t)stream;
#define ZK_QKV(NW_, EX_)                                                                                  \
  gemm_skinny_kernel<1, false, NW_, true, EX_><<<grid, NW_ * 64, 0, s>>>((const __bf16*)A, lda, (const __bf16*)W, Q, \
                                                                         ldq, 0, M, N, K, EPI_NONE, 0.f, w_strip, rs)
  if (grid.x < 512 && K >= 2048) {
    if (w_strip) ZK_QKV(8, true); else ZK_QKV(8, false);
  } else {
    if (w_strip) ZK_QKV(4, true); else ZK_QKV(4, false);
  }
#undef ZK_QKV
  return zk_launch_status("zk_qkv_rope_bf16");
}

// Strip layout of a [N, K] weight matrix, K % 32 == 0: rows in strips of 16 (the last strip
// padded with zeros), each (strip, 32-wide k step) one KB in which lane l = 16 * kq + r holds
// W[16 * strip + r][32 * step + 8 * kq .. + 8], i.e. exactly what the 64 lanes of a wave load
// for one 16x16x32 MFMA; steps follow each other, then strips.  A wave that streams its run
// of steps reads contiguous memory instead of sixteen rows K elements apart, which keeps
// every memory channel busy whatever K is (row strides of 4096 or 18432 bytes do not).
__global__ void strip_layout_kernel(const __bf16* __restrict__ src, __bf16* __restrict__ dst, int N, int K,
                                    size_t pieces) {
  const size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= pieces) return;
  const int ksteps = K / 32;
  const size_t block = q >> 6;
  const int l = (int)(q & 63);
  const int n = (int)(block / ksteps) * 16 + (l & 15);
  const int k = (int)(block % ksteps) * 32 + (l >> 4) * 8;
  *(bf16x8*)(dst + q * 8) = n < N ? *(const bf16x8*)(src + (size_t)n * K + k) : zero8();
}

// dst holds ceil(N / 16) * 16 rows of K elements.
extern "C" int zk_strip_layout(const void* src, void* dst, int N, int K, void* stream) {
  ZK_REQUIRE(N > 0 && K > 0 && K % 32 == 0, "zk_strip_layout: K must be a positive multiple of 32");
  const size_t pieces = (size_t)((N + 15) / 16) * 16 * K / 8;
  ZK_REQUIRE((pieces + 255) / 256 < 2147483647ull, "zk_strip_layout: matrix too large");
  strip_layout_kernel<<<(unsigned)((pieces + 255) / 256), 256, 0, (hipStream_t)stream>>>(
      (const __bf16*)src, (__bf16*)dst, N, K, pieces);
  return zk_launch_status("zk_strip_layout");
}

// epi: 0 none, 1 soft cap (cap > 0), 2 gelu_tanh gate, 3 silu gate.  For the gated
// epilogues W is [2N, K] (gate rows, then up rows) and C is [M, N].
// w_strip: W is in strip layout (zk_strip_layout), which needs K % 32 == 0 and, for the
// gated epilogues, N % 16 == 0.
// The workspace may be null; then K is never split over blocks.  It serves one launch at a time.
// parts (may be null): a caller whose next kernel can add partial sums up itself passes a place
// for their number.  0 comes back when the result is in C as usual; P > 0 when C was not
// written and the workspace starts with P planes of [M, N] floats, to be added in order and
// rounded to 16 bits (zk_norm_add_norm reads them so), before the next product overwrites them.
extern "C" size_t zk_gemm_bf16_workspace() { return ZK_GEMM_WORKSPACE_BYTES; }

// A tile variant (0: 128 x 128 blocks of four waves, 1: 64 x 128, 2: 128 x 256 of eight,
// 3: 256 x 256 of sixteen) with K split into ks ranges, and a model of its time in microseconds:
// the CU with the most blocks works through them one after the other, a block costs a start-up
// and a time per 64-wide k tile, a lone block a CU differs from one of several by a factor,
// and a split adds a joining kernel that moves the partial sums.  The constants are fitted to
// measurements (see where it is used).
struct TileChoice { int v, ks; };
static double tile_cost(TileChoice c, int M, int N, int K, bool gated, size_t room, int* tail_split = nullptr) {
  if (tail_split) *tail_split = 1;
  static const int BM[4] = {128, 64, 128, 256}, BN[4] = {128, 128, 256, 256};
  static const double start[4] = {0.0, 0.0, 0.974, 4.75}, per_ktile[4] = {0.522, 0.344, 0.881, 1.48},
                      lone[4] = {1.274, 1.432, 0.994, 0.903};
  const double launch = 3.774, join_start = 4.183, join_per_mb = 0.553;
  const int ncols = gated ? BN[c.v] / 2 : BN[c.v];
  const long tiles = (long)((M + BM[c.v] - 1) / BM[c.v]) * ((N + ncols - 1) / ncols);
  const double range_bytes = (double)tiles * BM[c.v] * BN[c.v] * 4.0;
  int ks = c.ks;
  while (ks > 1 && range_bytes * ks > (double)room) ks--;     // as the launcher will clamp it
  if (ks != c.ks) return 1e30;                                  // priced under the split it becomes
  if (ks > 1 && (K + GT_BK - 1) / GT_BK < 2 * ks) return 1e30;  // no ranges of less than two k tiles
  const int ktiles_all = (K + GT_BK - 1) / GT_BK;
  const int ktiles = (ktiles_all + ks - 1) / ks;
  const long per_cu = (tiles * ks + 255) / 256;
  double t = launch + per_cu * (start[c.v] + ktiles * per_ktile[c.v]) * (per_cu == 1 ? lone[c.v] : 1.0);
  if (ks > 1) t += join_start + ks * range_bytes / 1e6 * join_per_mb;
  // a last round of few tiles is launched apart with K in ranges (launch_tile has the rule)
  const long round_blocks = c.v <= 1 ? 512 : 256, tail = tiles % round_blocks;
  if (ks == 1 && tiles > round_blocks && tail > 0 && 2 * tail <= round_blocks && room > 0) {
    const double tile_bytes = (double)BM[c.v] * BN[c.v] * 4.0;
    int ts = (int)(round_blocks / tail < 8 ? round_blocks / tail : 8);
    while (ts > 1 && (ktiles_all / ts < 4 || tail * ts * tile_bytes > (double)room)) ts--;
    if (ts > 1) {
      const long tail_per_cu = (tail * ts + 255) / 256;
      const double apart =
          launch + (double)((tiles - tail) / 256) * (start[c.v] + ktiles_all * per_ktile[c.v]) + 3.0 +
          tail_per_cu * (start[c.v] + (ktiles_all + ts - 1) / ts * per_ktile[c.v]) * (tail_per_cu == 1 ? lone[c.v] : 1.0) +
          join_start + ts * tail * tile_bytes / 1e6 * join_per_mb;
      if (apart < 0.95 * t) {
        t = apart;
        if (tail_split) *tail_split = ts;
      }
    }
  }
  // No faster than memory delivers: the blocks of a weight tile's column walk through all of
  // the activations, which come from memory once per column when they are too many to stay in
  // the memory-side cache (4096 rows of K = 36864: 302 MB, 36 columns of 128: 11 GB).
  const double a_mb = (double)M * K * 2.0 / 1e6, w_mb = (gated ? 2.0 : 1.0) * N * K * 2.0 / 1e6;
  const double traffic_mb = w_mb + a_mb * (a_mb > 128.0 ? (double)((N + ncols - 1) / ncols) : 1.0);
  const double memory = traffic_mb / 6.0;          // 6 TB/s
  return t > memory ? t : memory;
}

static int gemm_bf16_run(const void* A, int lda, const void* W, void* C, int ldc, int c_is_f32,
                         int M, int N, int K, int epi, float cap, int w_strip, const GemmWorkspace& wsp,
                         int* parts, void* stream) {
  ZK_REQUIRE(M >= 0 && N > 0 && K > 0, "zk_gemm_bf16: bad sizes");
  ZK_REQUIRE(K % 8 == 0 && lda % 8 == 0, "zk_gemm_bf16: K and lda must be multiples of 8");
  ZK_REQUIRE(lda >= K && ldc >= N, "zk_gemm_bf16: leading dimensions too small");
  ZK_REQUIRE(epi >= 0 && epi <= EPI_PICK, "zk_gemm_bf16: unknown epilogue");
  ZK_REQUIRE(epi != EPI_SOFTCAP || cap > 0.f, "zk_gemm_bf16: soft cap must be positive");
  ZK_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "zk_gemm_bf16: operands must be 16-byte aligned");
  const bool gated = epi == EPI_GELU_TANH || epi == EPI_SILU;
  ZK_REQUIRE(!w_strip || (K % 32 == 0 && (!gated || N % 16 == 0)), "zk_gemm_bf16: strip layout needs K % 32 == 0 (and N % 16 == 0 when gated)");
  if (parts) *parts = 0;
  if (M == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (M > 16 && M <= 64 && w_strip) {
    return gated ? launch_mid<true>(A, lda, W, C, ldc, c_is_f32, M, N, K, epi, cap, wsp, parts, s)
                 : launch_mid<false>(A, lda, W, C, ldc, c_is_f32, M, N, K, epi, cap, wsp, parts, s);
  }
  if (M <= 64) {
    return gated ? launch_skinny<true>(A, lda, W, C, ldc, c_is_f32, M, N, K, epi, cap, w_strip, wsp, parts, s)
                 : launch_skinny<false>(A, lda, W, C, ldc, c_is_f32, M, N, K, epi, cap, w_strip, wsp, parts, s);
  }
  // 128 x 128 blocks of four waves (two share a CU) or 128 x 256 blocks of eight (one a CU,
  // about 1.2 times the rate).  What counts is the CU with the most blocks; a lone small block
  // runs at about 0.8 of the rate of two.  The constants are measured (M = 512 and 2048 with
  // N = 2304 to 18432): the rule picked the faster of the two in each of those.
  const int tiles_m = (M + 127) / 128;
  const long nb_small = (long)tiles_m * ((N + (gated ? 64 : 128) - 1) / (gated ? 64 : 128));
  const long nb_wide = (long)tiles_m * ((N + (gated ? 128 : 256) - 1) / (gated ? 128 : 256));
  const long per_cu_small = (nb_small + 255) / 256, per_cu_wide = (nb_wide + 255) / 256;
  const double cost_small = per_cu_small * 16384.0 / (per_cu_small == 1 ? 0.8 : 1.0);
  const double cost_wide = per_cu_wide * 32768.0 / 1.2;
  const bool wide = cost_wide < cost_small;
  const bool exact = K % GT_BK == 0;
  // Few small blocks: split K over blocks until about 320 blocks exist, a range no shorter than
  // 8 k tiles, and the partial sums (4 M N bytes a range, written and read) no more than W.
  auto ranges = [&](long blocks) {
    int ks = (int)(320 / blocks);
    ks = min(ks, (K + GT_BK - 1) / GT_BK / 8);
    ks = min(ks, K / (4 * M));
    return max(ks, 1);
  };
  int ksplit = (!wide && nb_small < 160) ? ranges(nb_small) : 1;
  // few rows and a K too short to split: 128 x 128 tiles leave half of the CUs or more without
  // a block; 64-row tiles make twice as many (they lose to a split of K where K allows one)
  const bool low = !wide && M > 64 && nb_small * ksplit <= 128;
  if (low) ksplit = ranges((long)((M + 63) / 64) * (nb_small / tiles_m));
#define ZK_TILE_(W_, M_, N_, G_, E_) \
  launch_tile<W_, M_, N_, G_, E_>(A, lda, W, C, ldc, c_is_f32, M, N, K, epi, cap, w_strip, wsp, ksplit, tail_split, s)
#define ZK_TILE(W_, M_, N_)                                                                            \
  (gated ? (exact ? ZK_TILE_(W_, M_, N_, true, true) : ZK_TILE_(W_, M_, N_, true, false))             \
         : (exact ? ZK_TILE_(W_, M_, N_, false, true) : ZK_TILE_(W_, M_, N_, false, false)))
  // 256 x 256 blocks of sixteen waves where there are tiles enough.  The tile product is bound
  // by what L2 delivers to a CU (a 128 x 256 x 64 step moves 48 KB for 4.2 MFLOP: at the 10 TB/s
  // all CUs get together that is 0.9 PFLOP/s, which is what the 128 x 256 blocks reach); a
  // 256 x 256 block moves a third fewer bytes per flop.  Measured against 128 x 256: 0.88 of its
  // time with many rounds of tiles (4096 x 36864 x 4608 gated), 0.91 at 2048 x 9216 x 2304 gated
  // (2.25 rounds), 1.4 at 2048 x 4096 x 2304 (half a round: half of the CUs idle).  The rule:
  // time = (rounds, at least one, + 0.15) x time of a tile.
  int variant = wide ? 2 : low ? 1 : 0;       // 128 x 128, 64 x 128, 128 x 256, 256 x 256
  if (wide && exact) {
    const long nb_big = (long)((M + 255) / 256) * ((N + (gated ? 128 : 256) - 1) / (gated ? 128 : 256));
    auto rounds_cost = [](long nb, double unit) { return ((nb > 256 ? nb / 256.0 : 1.0) + 0.15) * unit; };
    if (rounds_cost(nb_big, 2.0 * 0.8836 * 32768.0 / 1.2) < rounds_cost(nb_wide, 32768.0 / 1.2)) variant = 3;
  }
  // The rules above are right for the shapes they were made on and miss elsewhere: long K with
  // few hundred rows wants more ranges of K than they allow, narrow products of thousands of
  // rows (N = 2304 to 4608) the 256 x 256 blocks.  So every variant and split is priced by a
  // model of its time fitted to a sweep of 1339 measured (rows, shape, variant, split)
  // combinations (2B, 9B and 27B layer shapes, 96 to 4096 rows; 10 % rms error), and the model's
  // choice replaces the rules' when it promises at least 12 % (with that margin it was never
  // more than 3 % slower than the rules on the sweep, and 5 % faster in the sum).
  {
    const TileChoice rule{variant, ksplit};
    const size_t room = (wsp.ptr != nullptr && (uintptr_t)wsp.ptr % 64 == 0) ? wsp.split_bytes() : 0;
    const double rule_cost = tile_cost(rule, M, N, K, gated, room);
    TileChoice best = rule;
    double best_cost = rule_cost;
    static const int splits[] = {1, 2, 3, 4, 6, 8};
    for (int v = 0; v < (exact ? 4 : 3); v++)
      for (int ks : splits) {
        const TileChoice c{v, ks};
        const double t = tile_cost(c, M, N, K, gated, room);
        if (t < best_cost) { best = c; best_cost = t; }
      }
    if (best_cost * 1.12 < rule_cost) { variant = best.v; ksplit = best.ks; }
  }
  int tail_split = 1;
  {
    const size_t room = (wsp.ptr != nullptr && (uintptr_t)wsp.ptr % 64 == 0) ? wsp.split_bytes() : 0;
    tile_cost(TileChoice{variant, ksplit}, M, N, K, gated, room, &tail_split);
  }
  // The two wide blocks have a form that copies its operands straight into LDS (weights in the
  // strip layout, K a whole number of tiles): 3 to 6 % less time from about 200 rows on, the
  // same sums in the same order.  (The 128 x 128 and 64 x 128 blocks gained nothing from it
  // where K is split and lost where it is short.)
#define ZK_DIRECT(W_, M_, N_)                                                                                              \
  (gated ? launch_tile<W_, M_, N_, true, true, true>(A, lda, W, C, ldc, c_is_f32, M, N, K, epi, cap, w_strip, wsp, ksplit, tail_split, s) \
         : launch_tile<W_, M_, N_, false, true, true>(A, lda, W, C, ldc, c_is_f32, M, N, K, epi, cap, w_strip, wsp, ksplit, tail_split, s))
  if (w_strip && K % GT_BK == 0 && N % 16 == 0) {
    if (variant == 3) return ZK_DIRECT(4, 2, 4);
    if (variant == 2) return ZK_DIRECT(2, 2, 4);
  }
#undef ZK_DIRECT
  if (variant == 3) return gated ? ZK_TILE_(2, 4, 4, true, true) : ZK_TILE_(2, 4, 4, false, true);
  if (variant == 2) return ZK_TILE(2, 2, 4);
  if (variant == 1) return ZK_TILE(1, 2, 2);
  return ZK_TILE(2, 2, 2);
#undef ZK_TILE
#undef ZK_TILE_
}

extern "C" int zk_gemm_bf16(const void* A, int lda, const void* W, void* C, int ldc, int c_is_f32,
                            int M, int N, int K, int epi, float cap, int w_strip, void* ws,
                            size_t ws_bytes, int* parts, void* stream) {
  ZK_REQUIRE(epi != EPI_PICK, "zk_gemm_bf16: the picking epilogue belongs to zk_head_pick_bf16");
  return gemm_bf16_run(A, lda, W, C, ldc, c_is_f32, M, N, K, epi, cap, w_strip, GemmWorkspace{ws, ws_bytes, false},
                       parts, stream);
}

// ---- the LM head of a greedy step: the largest logit's column of every row, no logits stored
//
// One block a row joins the strips' picks: larger value first, equal values to the lower
// column, NaN never; a row without any valid value gets column 0 (as zk_argmax does).
__global__ __launch_bounds__(1024) void pick_join_kernel(const Pick* __restrict__ picks, int nstrips,
                                                         int* __restrict__ ids) {
  __shared__ float sv[16];
  __shared__ int sc[16];
  const Pick* row = picks + (size_t)blockIdx.x * nstrips;
  Pick best{-INFINITY, 0x7fffffff};
  auto better = [](const Pick& a, const Pick& b) {       // a before b
    if (a.column == 0x7fffffff) return false;
    return b.column == 0x7fffffff || a.value > b.value || (a.value == b.value && a.column < b.column);
  };
  // eight loads of a thread on their way at a time (a place past the end reads the last pick
  // again, which changes nothing): with one block a row the time is the trips to memory
  for (int i0 = threadIdx.x; i0 < nstrips; i0 += 8 * 1024) {
    Pick p[8];
#pragma unroll
    for (int j = 0; j < 8; j++) p[j] = row[min(i0 + j * 1024, nstrips - 1)];
#pragma unroll
    for (int j = 0; j < 8; j++)
      if (better(p[j], best)) best = p[j];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const Pick o{__shfl_xor(best.value, off), __shfl_xor(best.column, off)};
    if (better(o, best)) best = o;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    sv[wave] = best.value;
    sc[wave] = best.column;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 16; w++) {
      const Pick o{sv[w], sc[w]};
      if (better(o, best)) best = o;
    }
    ids[blockIdx.x] = best.column == 0x7fffffff ? 0 : best.column;
  }
}

extern "C" size_t zk_head_pick_bf16_workspace(int M, int N) {
  return (size_t)(M > 0 ? M : 0) * (size_t)((N + 15) / 16) * sizeof(Pick);
}

// ids[m] = the column of the largest value of row m of A W^T after the soft cap (cap <= 0: no
// cap): what zk_gemm_bf16 with the soft-cap epilogue followed by zk_argmax gives, bit for bit,
// without the [M, N] logits.  1 to 64 rows; more than 16 need W in strip layout.  ``picks``:
// zk_head_pick_bf16_workspace(M, N) bytes of scratch, 16-byte aligned.
extern "C" int zk_head_pick_bf16(const void* A, int lda, const void* W, int M, int N, int K, float cap, int w_strip,
                                 void* picks, size_t picks_bytes, void* ids, void* stream) {
  ZK_REQUIRE(M >= 1 && M <= 64, "zk_head_pick_bf16: 1 to 64 rows");
  ZK_REQUIRE(M <= 16 || w_strip, "zk_head_pick_bf16: more than 16 rows need the weights in strip layout");
  ZK_REQUIRE(picks != nullptr && (uintptr_t)picks % 16 == 0 && ids != nullptr, "zk_head_pick_bf16: no scratch or no result");
  ZK_REQUIRE(picks_bytes >= zk_head_pick_bf16_workspace(M, N), "zk_head_pick_bf16: scratch too small");
  if (int rc = gemm_bf16_run(A, lda, W, nullptr, N, 1, M, N, K, EPI_PICK, cap, w_strip,
                             GemmWorkspace{picks, picks_bytes, false}, nullptr, stream))
    return rc;
  pick_join_kernel<<<M, 1024, 0, (hipStream_t)stream>>>((const Pick*)picks, (N + 15) / 16, (int*)ids);
  return zk_launch_status("zk_head_pick_bf16");
}

// ---- the same product for callers that cannot allocate (declared in gemm_bf16_static.h)
//
// The partial sums of a product that splits K go to a statically allocated array instead of a
// workspace the caller brings.  Every GPU holds its own copy of the array at its own address;
// host code never uses the array's name as an address, only the pointer that
// hipGetSymbolAddress gave for the device that is current.
static __device__ __align__(256) unsigned char scratch[ZK_GEMM_STATIC_SCRATCH_BYTES];

#define ZK_MAX_DEVICES 64
static void* scratch_of_device[ZK_MAX_DEVICES];     // null until the device's set-up has run
static std::mutex scratch_mutex;

// The array's address on the current device, asked for once per device.
static int static_scratch(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return zk_fail("zk_gemm_bf16_static: no current device");
  ZK_REQUIRE(dev >= 0 && dev < ZK_MAX_DEVICES, "zk_gemm_bf16_static: device index out of range");
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_of_device[dev] == nullptr) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();
      return zk_fail("zk_gemm_bf16_static: hipGetSymbolAddress of the scratch array failed");
    }
    scratch_of_device[dev] = ptr;
  }
  *out = scratch_of_device[dev];
  return 0;
}

extern "C" size_t zk_gemm_bf16_static_bytes() { return ZK_GEMM_STATIC_SCRATCH_BYTES; }

extern "C" int zk_gemm_bf16_static_init() {
  void* ptr = nullptr;
  return static_scratch(&ptr);
}

extern "C" int zk_gemm_bf16_static(const void* A, int lda, const void* W, void* C, int ldc, int c_is_f32,
                                   int M, int N, int K, int epi, float cap, int w_strip, void* stream) {
  void* ptr = nullptr;
  if (int rc = static_scratch(&ptr)) return rc;
  // strict: K is split exactly as zk_gemm_bf16 splits it with its standard workspace, so the
  // results have the same bits; a split whose partial sums do not fit the array is refused.
  // Nothing in the array has to start at zero: each range's plane is written in full by the
  // product kernel before the joining kernel of the same call reads it.
  ZK_REQUIRE(epi != EPI_PICK, "zk_gemm_bf16_static: the picking epilogue belongs to zk_head_pick_bf16");
  return gemm_bf16_run(A, lda, W, C, ldc, c_is_f32, M, N, K, epi, cap, w_strip,
                       GemmWorkspace{ptr, ZK_GEMM_STATIC_SCRATCH_BYTES, true}, nullptr, stream);
}

#endif  // ZSE_ACT_BF16
