// Paged attention on the matrix cores, bfloat16 in, float softmax.
//
// A wave owns up to 32 query rows: TPW consecutive tokens of one request times the g = nh / nkv
// query heads that share a KV head, so every K and V tile it loads serves the
// whole group (the reference's paged_attention_v2 stages a K/V tile once for
// the heads of a group too, orchestrator/kernels.py:687-854, but is never
// launched; the launched kernels read K and V once per query head and hold one
// score per cached token in shared memory, :524-671, :859-958).
//
// Per tile of 32 keys:
//   S^T[key, row]  = K[key, :] . Q[row, :]        32x32x16 MFMA, hd/16 steps
//   scale, soft cap, mask (key <= pos, pos - key < window), running max / sum
//   O^T[d, row]   += V^T[d, key] * P^T[key, row]  32x32x16 MFMA, 2 per 32 channels
// S^T and O^T both keep a query row in a fixed lane (column = lane % 32), so the
// running maximum, sum and rescale are per-lane scalars, and the probabilities
// a lane holds after the first product are exactly its operand for the second:
// the contraction order over keys is permuted to match (slots e < 4 of lane half
// h are keys 4h + e, slots e >= 4 are keys 8 + 4h + e - 4), and V is read with
// the same permutation.  V is therefore cached transposed, [page][kv head][hd][bs],
// so that four consecutive keys of a channel are one 8-byte load.
//
// Portions have three kernels, chosen by the launch's sizes (zk_attention_bf16): a group of 32
// rows a block, its four waves sharing out the keys (attn_mfma_kernel: few groups); four or
// eight consecutive groups a block with every tile of keys and values fetched once into LDS for
// all of them (attn_shared_kernel: many groups); and the latter with the keys of a block of rows
// cut into ranges over several blocks, joined by attn_portion_join_kernel (few groups with long
// contexts: a portion of a prompt behind thousands of tokens).
//
// Decoded tokens use a split variant: the keys are cut into chunks of 64 (or 32, as
// the caller says) aligned to absolute positions, one wave per chunk writes (max, sum, O)
// and a second kernel joins the chunks in order; the cut is the caller's choice and never
// follows from the batch, so a request's result is the same whoever shares its step.  With
// at most 16 heads a KV head the chunks run on 16x16x32 MFMAs (attn_decode_kernel):
// a single query token fills only g of a tile's columns, and the narrower tile
// halves both the accumulator registers and the wasted work, so two waves fit a SIMD.
#include "common.h"

#include <algorithm>

#if ZSE_ACT_BF16

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define ATT_CHUNK 64
#define ATT_MOST_RANGES 8      // ranges of keys a block of rows of a portion is cut into, at most

struct AttnParams {
  const __bf16* q;
  int q_stride;
  const __bf16* kcache;   // [page][nkv][bs][hd]
  const __bf16* vcache;   // [page][nkv][hd][bs]
  const int* block_table;
  int max_blocks;
  const int* q_start;     // [R + 1]
  const int* ctx_len;     // [R]
  __bf16* out;            // [T][nh][hd]
  float* part_o;          // split: [slot][hd]
  float* part_ml;         // split: [slot][2]
  int nh, nkv, hd, bs;
  int bs_shift;           // page size is 1 << bs_shift in the tuned kernels
  float scale, softcap;
  // scores in the log2 domain: with a cap c,  s2 = c2 * tanh(k2 * dot / 2)  computed as
  // c2 * (1 - 2 / (exp2(k2 * dot) + 1)),  k2 = 2 * scale / c * log2(e),  c2 = c * log2(e);
  // without a cap  s2 = k1 * dot,  k1 = scale * log2(e).  Probabilities are exp2(s2 - m2).
  float k1, k2, c2;
  int window;
  int tpw;                // tokens a wave owns
  int r_begin;            // first request of this launch
  int nchunks;            // split: chunks the grid covers
  int from_window;        // decode: block 0 of a request is the one its window begins in
  int chunk;              // decoded tokens on 16-wide tiles: keys a wave takes, 32 or 64
};

__device__ __forceinline__ float score_log2(const AttnParams& p, float dot) {
  if (p.softcap > 0.f) {
    const float e = __builtin_amdgcn_exp2f(p.k2 * dot);
    return p.c2 * (1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f));
  }
  return p.k1 * dot;
}

// Portions: which (group, KV head) a block takes.  Blocks go to the 8 XCDs in turn by their
// number, and every XCD has an L2 of its own; blocks that read the same keys and values (those
// of one KV head) are therefore given to as few XCDs as possible, so that what one of them has
// fetched is in the L2 for the others instead of crossing from the memory side once per block.
__device__ __forceinline__ void portion_block(int& bx, int& by) {
  const int gx = gridDim.x, gy = gridDim.y;
  bx = blockIdx.x;
  by = blockIdx.y;
  const int total = gx * gy;
  if (total % 8) return;
  const int lin = blockIdx.x + gx * blockIdx.y, xcd = lin & 7, slot = lin >> 3;
  if (gy <= 8 && 8 % gy == 0) {            // 8 / gy XCDs a head
    const int per = 8 / gy;
    by = xcd % gy;
    bx = slot * per + xcd / gy;
  } else if (gy % 8 == 0) {                // gy / 8 heads an XCD
    const int heads = gy / 8;
    by = xcd + 8 * (slot % heads);
    bx = slot / heads;
  }
}

template <int HD16, bool SPLIT, bool PAIR>
__global__ __launch_bounds__(256, (HD16 <= 8 && !PAIR) ? 2 : 1) void attn_mfma_kernel(AttnParams p) {
  constexpr int DT = (HD16 + 1) / 2;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lr = lane & 31, lk = lane >> 5;
  const int r = p.r_begin + blockIdx.z;
  int block_x = blockIdx.x, kvh = blockIdx.y;
  if (!SPLIT) portion_block(block_x, kvh);
  const int qs = p.q_start[r], n = p.q_start[r + 1] - qs;
  if (n <= 0) return;
  const int start = p.ctx_len[r] - n;
  // portions: a block owns one group of rows and its four waves take every fourth tile of
  // keys (their results are joined at the end).  Or (PAIR, for portions whose groups would
  // need a second, half-empty round of blocks) two groups: one from the end of the portion,
  // which sees many keys, and its mirror from the start, which sees few, so that every block
  // has about the same work; the four waves are shared out between the two by their numbers
  // of key tiles (3 + 1, 2 + 2 or 1 + 3), a group's waves taking its tiles in turn.
  // Decoded tokens: a wave owns one chunk of keys.
  int gi = 0, phase = wave, nphase = 4, first_wave = 0;        // group, and the wave's place among its waves
  int na_block = 4;                                            // waves of the block's first group
  // single groups: the last group of a portion sees the most keys and goes first, so that the
  // blocks still running at the end are the short ones
  if (!SPLIT && !PAIR) gi = (n + p.tpw - 1) / p.tpw - 1 - block_x;
  if (PAIR) {
    const int groups = (n + p.tpw - 1) / p.tpw;
    if (block_x >= (groups + 1) / 2) return;           // the whole block is past the portion
    const int ga = groups - 1 - block_x, gb = block_x;
    if (ga != gb) {
      auto tiles_of = [&](int gr) {
        const int lo = start + gr * p.tpw, hi = start + min(n, (gr + 1) * p.tpw) - 1;
        const int klo = p.window > 0 ? max(0, lo - p.window + 1) : 0;
        return hi / 32 - klo / 32 + 1;
      };
      const int ta = tiles_of(ga), tb = tiles_of(gb);
      const int na = min(3, max(1, (4 * ta + (ta + tb) / 2) / (ta + tb)));
      na_block = na;
      if (wave < na) { gi = ga; phase = wave; nphase = na; }
      else { gi = gb; phase = wave - na; nphase = 4 - na; first_wave = na; }
    } else {
      gi = ga;
    }
  }
  const int chunk = SPLIT ? block_x * 4 + wave : 0;
  const int t0 = gi * p.tpw;
  if (!PAIR && (gi < 0 || t0 >= n)) return;
  const int g = p.nh / p.nkv;
  const int tok = lr / g, hq = lr - tok * g;
  const int ntok = min(p.tpw, n - t0);
  const bool row_ok = tok < ntok;
  const int trow = qs + t0 + (row_ok ? tok : 0);
  const int pos = start + t0 + (row_ok ? tok : 0);
  const int head = kvh * g + (row_ok ? hq : 0);
  const int pos_lo = start + t0, pos_hi = start + t0 + ntok - 1;
  int key_lo = p.window > 0 ? max(0, pos_lo - p.window + 1) : 0;
  int key_hi = pos_hi;
  if (SPLIT) {
    key_lo = max(key_lo, chunk * ATT_CHUNK);
    key_hi = min(key_hi, chunk * ATT_CHUNK + ATT_CHUNK - 1);
  }
  if (SPLIT && key_lo > key_hi) return;
  const int row_lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
  const int* table = p.block_table + (size_t)r * p.max_blocks;
  const int hd = p.hd, bsh = p.bs_shift, bmask = p.bs - 1, nkv = p.nkv;

  bf16x8 qf[HD16];
  {
    const __bf16* qr = p.q + (size_t)trow * p.q_stride + (size_t)head * hd + lk * 8;
#pragma unroll
    for (int ks = 0; ks < HD16; ks++) {
      if (row_ok) qf[ks] = *(const bf16x8*)(qr + ks * 16);
      else
#pragma unroll
        for (int e = 0; e < 8; e++) qf[ks][e] = (__bf16)0.f;
    }
  }
  f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int e = 0; e < 16; e++) o[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  // where the lane's channels dt * 32 + lr lie in a (page, kv head) block of the transposed V cache
  int vrow[DT];
#pragma unroll
  for (int dt = 0; dt < DT; dt++) vrow[dt] = min(dt * 32 + lr, hd - 1) << bsh;
  const bool capped = p.softcap > 0.f;
  // keys every row of the group sees (none beyond the first row's position, none before the
  // last row's window; no range at all unless every lane holds a row): tiles inside this range
  // need no mask
  const int all_hi = ntok * g == 32 ? pos_lo : -1;
  const int all_lo = p.window > 0 ? max(0, pos_hi - p.window + 1) : 0;

  // The pages of a tile are looked up a tile ahead as well, so that no load waits for a table
  // entry: the lane's key row, and the four places its V pieces come from.
  struct TilePages { int k, va[2], vb[2]; };
  auto look_up = [&](int key0, TilePages& pg) {
    pg.k = table[min(key0 + lr, key_hi) >> bsh];
#pragma unroll
    for (int h = 0; h < 2; h++) {
      pg.va[h] = table[min(key0 + h * 16 + 4 * lk, key_hi & ~3) >> bsh];
      pg.vb[h] = table[min(key0 + h * 16 + 8 + 4 * lk, key_hi & ~3) >> bsh];
    }
  };
  auto load_k = [&](int key0, int page, bf16x8 (&kf)[HD16]) {
    const int kk = min(key0 + lr, key_hi);
    const __bf16* kr = p.kcache + ((((size_t)max(page, 0) * nkv + kvh) << bsh) + (kk & bmask)) * hd + lk * 8;
#pragma unroll
    for (int ks = 0; ks < HD16; ks++) kf[ks] = *(const bf16x8*)(kr + ks * 16);
  };
  auto tile = [&](int key0, const TilePages& pg, int knext, TilePages& pn) {
    bf16x8 kf[HD16];
    load_k(key0, pg.k, kf);
    look_up(knext, pn);
    // ---- S^T = K Q^T
    f32x16 s;
#pragma unroll
    for (int e = 0; e < 16; e++) s[e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < HD16; ks++) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks], qf[ks], s, 0, 0, 0);
    // ---- V^T pieces for this tile (issued early; used after the softmax)
    bf16x8 vf[DT][2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const int ka = min(key0 + h * 16 + 4 * lk, key_hi & ~3), kb = min(key0 + h * 16 + 8 + 4 * lk, key_hi & ~3);
      const int pa = max(pg.va[h], 0), pb = max(pg.vb[h], 0);
      const __bf16* vpa = p.vcache + ((((size_t)pa * nkv + kvh) * hd) << bsh) + (ka & bmask);
      const __bf16* vpb = p.vcache + ((((size_t)pb * nkv + kvh) * hd) << bsh) + (kb & bmask);
#pragma unroll
      for (int dt = 0; dt < DT; dt++) {
        const bf16x4 va = *(const bf16x4*)(vpa + vrow[dt]);
        const bf16x4 vb = *(const bf16x4*)(vpb + vrow[dt]);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          vf[dt][h][e] = va[e];
          vf[dt][h][4 + e] = vb[e];
        }
      }
    }
    // ---- scale, cap, mask, running softmax (one query row per lane)
    float mt = -INFINITY;
    if (capped) {
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const float ex = __builtin_amdgcn_exp2f(p.k2 * s[e]);
        s[e] = p.c2 * (1.f - 2.f * __builtin_amdgcn_rcpf(ex + 1.f));
      }
    } else {
#pragma unroll
      for (int e = 0; e < 16; e++) s[e] *= p.k1;
    }
    if (key0 < all_lo || key0 + 31 > all_hi || key0 < key_lo || key0 + 31 > key_hi) {
#pragma unroll
      for (int j = 0; j < 4; j++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int key = key0 + 8 * j + 4 * lk + i;
          const bool ok = row_ok && key >= row_lo && key <= pos && key >= key_lo && key <= key_hi;
          s[4 * j + i] = ok ? s[4 * j + i] : -INFINITY;
        }
    }
#pragma unroll
    for (int e = 0; e < 16; e++) mt = fmaxf(mt, s[e]);
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float m_new = mt > m_run + 8.f ? mt : m_run;      // the reference follows the maximum lazily
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const bool moved = m_new > m_run;
    const float corr = moved ? __builtin_amdgcn_exp2f(m_run - m_use) : 1.f;
    float rs = 0.f;
#pragma unroll
    for (int e = 0; e < 16; e++) {
      const float pe = __builtin_amdgcn_exp2f(s[e] - m_use);
      s[e] = pe;
      rs += pe;
    }
    rs += __shfl_xor(rs, 32, 64);
    l_run = l_run * corr + rs;
    m_run = m_new;
    bf16x8 pb[2];
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
      for (int e = 0; e < 8; e++) pb[h][e] = (__bf16)s[8 * h + e];
    // ---- O^T = corr * O^T + V^T P^T  (the maximum rarely rises by the threshold after a
    // row's first tiles; said so, the compiler keeps the accumulators where the products
    // want them instead of moving all of them on every tile)
    if (__builtin_expect(__any(moved), 0)) {
      // in the accumulation registers, where the products keep them: written so, the compiler
      // does not copy all of them to ordinary registers on every tile for this rare path
#pragma unroll
      for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int e = 0; e < 16; e++) {
          float t;
          asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 %0, %1"
                       : "+a"(o[dt][e]), "=&v"(t)
                       : "v"(corr));
        }
    }
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
      o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[dt][0], pb[0], o[dt], 0, 0, 0);
      o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[dt][1], pb[1], o[dt], 0, 0, 0);
    }
  
  };
  {
    const int kstep = SPLIT ? 32 : 32 * nphase;
    int key0 = (key_lo / 32) * 32 + (SPLIT ? 0 : phase * 32);
    TilePages p0, p1;
    if (key0 <= key_hi) look_up(key0, p0);
    for (; key0 <= key_hi; key0 += 2 * kstep) {
      tile(key0, p0, key0 + kstep, p1);
      if (key0 + kstep > key_hi) break;
      tile(key0 + kstep, p1, key0 + 2 * kstep, p0);
    }
  }
  if (SPLIT) {
    if (!row_ok) return;
    const size_t slot = ((size_t)(r - p.r_begin) * p.nh + head) * p.nchunks + chunk;
    if (lk == 0) {
      p.part_ml[slot * 2] = m_run;
      p.part_ml[slot * 2 + 1] = l_run;
    }
    float* po = p.part_o + slot * hd;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int d = dt * 32 + 8 * j + 4 * lk;
        if (d < hd) *(f32x4*)(po + d) = f32x4{o[dt][4 * j], o[dt][4 * j + 1], o[dt][4 * j + 2], o[dt][4 * j + 3]};
      }
  } else {
    // join a group's waves: common maximum and sum per row, then the accumulators of the
    // group's other waves reach its first wave through LDS, one wave a round (a slot a group)
    extern __shared__ float dyn[];
    float* sm_ml = dyn;                          // [4][32][2]
    float* sm_o = dyn + 4 * 32 * 2;              // [2][DT * 16][64]
    if (lk == 0) {
      sm_ml[(wave * 32 + lr) * 2] = m_run;
      sm_ml[(wave * 32 + lr) * 2 + 1] = l_run;
    }
    __syncthreads();
    float m_all = -INFINITY;
    for (int w = first_wave; w < first_wave + nphase; w++) m_all = fmaxf(m_all, sm_ml[(w * 32 + lr) * 2]);
    float l_all = 0.f;
    for (int w = first_wave; w < first_wave + nphase; w++) {
      const float mw = sm_ml[(w * 32 + lr) * 2];
      l_all += mw == -INFINITY ? 0.f : sm_ml[(w * 32 + lr) * 2 + 1] * __builtin_amdgcn_exp2f(mw - m_all);
    }
    const float f = m_run == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run - m_all);
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int e = 0; e < 16; e++) o[dt][e] *= f;
    float* slot = sm_o + (size_t)(first_wave ? 1 : 0) * DT * 16 * 64;
    const int rounds = max(na_block, 4 - na_block) - 1;
    for (int step = 1; step <= rounds; step++) {
      if (phase == step) {
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
          for (int e = 0; e < 16; e++) slot[(dt * 16 + e) * 64 + lane] = o[dt][e];
      }
      __syncthreads();
      if (phase == 0 && step < nphase) {
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
          for (int e = 0; e < 16; e++) o[dt][e] += slot[(dt * 16 + e) * 64 + lane];
      }
      __syncthreads();
    }
    if (phase != 0 || !row_ok) return;
    const float inv = 1.f / l_all;
    __bf16* orow = p.out + ((size_t)trow * p.nh + head) * hd;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int d = dt * 32 + 8 * j + 4 * lk;
        if (d < hd) {
          bf16x4 w;
#pragma unroll
          for (int i = 0; i < 4; i++) w[i] = (__bf16)(o[dt][4 * j + i] * inv);
          *(bf16x4*)(orow + d) = w;
        }
      }
  }
}

// Long portions.  A block of NW waves owns NW groups of rows that follow each other in one
// request (NW * tpw tokens times the g heads of a KV head), every wave one group, and all of
// them walk the same keys: a tile of 32 keys and its values come from the cache once a block,
// wait in LDS and serve every wave (attn_mfma_kernel fetches them once a group of 32 rows:
// with many groups the way from L2 to the CUs then sets the time).  No join: a wave sees all
// the keys of its rows.  Two buffers: the loads of the next tile are in flight while the
// current one is multiplied, and one barrier a tile suffices.
//   sK [2][32 keys][hd + 8]       a lane's piece for the first product is 16 bytes of a key's row
//   sV [2][hd][32 + 8]            a channel's 32 keys in the order the second product wants:
//                                 piece 2h + lk = keys 16h + 4lk + (0..3), 16h + 8 + 4lk + (0..3)
// The padding of 16 bytes a row keeps the 16-byte reads of 16 lanes on different banks.
// Pages of at least 8 keys (a 16-byte piece of the transposed V holds 8 keys of one page).
//
// SPLIT: a launch of few blocks with many keys each (a prompt of a few thousand tokens and few
// heads) cuts the keys of a block of rows into ranges of p.chunk tiles, counted from the
// block's first tile; blockIdx.x is (block of rows) * p.nchunks + range.  A block then leaves
// (max, sum, O) of its range for every row, as the chunks of a decoded token do, and
// attn_portion_join_kernel joins a row's ranges in their order.
template <int HD16, int NW, bool SPLIT>
__global__ __launch_bounds__(NW * 64, (HD16 <= 8 && NW <= 4) ? 2 : 1) void attn_shared_kernel(AttnParams p) {
  constexpr int HD = HD16 * 16, DT = (HD16 + 1) / 2;
  constexpr int KLD = HD + 8, VLD = 32 + 8;
  constexpr int NT = NW * 64;
  constexpr int PIECES = 4 * HD;                        // 16-byte pieces of a K tile, and of a V tile
  constexpr int PPT = (PIECES + NT - 1) / NT;           // pieces of each a thread moves
  constexpr int CPK = HD / 8;                           // pieces of a key's row
  extern __shared__ __attribute__((aligned(16))) unsigned char shared_raw[];
  __bf16* sK = (__bf16*)shared_raw;                     // [2][32][KLD]
  __bf16* sV = sK + 2 * 32 * KLD;                       // [2][HD][VLD]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 31, lk = lane >> 5;
  const int r = p.r_begin + blockIdx.z;
  int block_x, kvh;
  portion_block(block_x, kvh);
  const int qs = p.q_start[r], n = p.q_start[r + 1] - qs;
  if (n <= 0) return;
  const int start = p.ctx_len[r] - n;
  const int per_block = NW * p.tpw;
  // the last rows of a portion see the most keys and go first
  const int rows_x = SPLIT ? block_x / p.nchunks : block_x;
  const int range = SPLIT ? block_x - rows_x * p.nchunks : 0;
  const int bi = (n + per_block - 1) / per_block - 1 - rows_x;
  if (bi < 0) return;
  const int g = p.nh / p.nkv;
  // the block's keys: from the window of its first row to its last row
  const int blk_lo = start + bi * per_block, blk_hi = start + min(n, (bi + 1) * per_block) - 1;
  int key_lo = p.window > 0 ? max(0, blk_lo - p.window + 1) : 0;
  int key_hi = blk_hi;
  if (SPLIT) {
    const int first_tile = key_lo / 32 + range * p.chunk;
    if (first_tile * 32 > key_hi) return;              // the block of rows has fewer ranges
    key_lo = max(key_lo, first_tile * 32);
    key_hi = min(key_hi, (first_tile + p.chunk) * 32 - 1);
  }
  // the wave's rows
  const int t0 = bi * per_block + wave * p.tpw;
  const int ntok = max(0, min(p.tpw, n - t0));
  const int tok = lr / g, hq = lr - tok * g;
  const bool row_ok = tok < ntok;
  const int trow = qs + (row_ok ? t0 + tok : 0);
  const int pos = start + (row_ok ? t0 + tok : 0);
  const int head = kvh * g + (row_ok ? hq : 0);
  const int pos_lo = start + t0, pos_hi = start + t0 + ntok - 1;          // ntok == 0: no keys at all
  const int row_lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
  const int all_hi = ntok * g == 32 ? pos_lo : -1;
  const int all_lo = p.window > 0 ? max(0, pos_hi - p.window + 1) : 0;
  const int* table = p.block_table + (size_t)r * p.max_blocks;
  const int bsh = p.bs_shift, bmask = p.bs - 1, nkv = p.nkv;

  bf16x8 qf[HD16];
  {
    const __bf16* qr = p.q + (size_t)trow * p.q_stride + (size_t)head * HD + lk * 8;
#pragma unroll
    for (int ks = 0; ks < HD16; ks++) {
      if (row_ok) qf[ks] = *(const bf16x8*)(qr + ks * 16);
      else
#pragma unroll
        for (int e = 0; e < 8; e++) qf[ks][e] = (__bf16)0.f;
    }
  }
  f32x16 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int e = 0; e < 16; e++) o[dt][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // The thread's pieces of a tile.  K: piece q is 8 channels (q % CPK) of key q / CPK.  V: the
  // pieces of a page's part of the tile lie one behind the other in the cache, channel by
  // channel: with tk = min(page size, 32) keys of a page in the tile, piece q is the keys
  // [8c, 8c + 8) of channel d in part q / (HD tk / 8), d = (q / (tk / 8)) % HD, c = q % (tk / 8).
  const int tk_shift = min(bsh, 5);                     // log2 of a page's keys in a tile
  const int cpp_shift = tk_shift - 3;                   // log2 of the pieces of a channel in a page's part
  // What does not change from tile to tile is worked out here, per piece: its place in the page
  // table relative to the tile's first entry, its offset inside a page's block of the cache (the
  // KV head, the key's place in the page, the channels) and its place in LDS.  A tile then costs
  // a piece one table entry and one multiply-add.  (Tiles start at multiples of 32 keys: with
  // pages of up to 32 keys a key's place in its page does not depend on the tile, with larger
  // pages the whole tile lies in one page and the tile's offset in it is the same for all.)
  int k_idx[PPT], v_idx[PPT], k_lds[PPT], v_lds[PPT];
  unsigned k_off[PPT], v_off[PPT];
#pragma unroll
  for (int j = 0; j < PPT; j++) {
    const int q = min(tid + j * NT, PIECES - 1);
    const int kk = q / CPK, col = (q % CPK) * 8;
    const int part = q / (HD << cpp_shift), rem = q - part * (HD << cpp_shift);
    const int d = rem >> cpp_shift;
    const int vk = (part << tk_shift) + ((rem & ((1 << cpp_shift) - 1)) << 3);
    k_idx[j] = kk >> bsh;
    k_off[j] = (unsigned)(((kvh << bsh) + (kk & bmask)) * HD + col);
    k_lds[j] = kk * KLD + col;
    v_idx[j] = vk >> bsh;
    v_off[j] = (unsigned)(((kvh * HD + d) << bsh) + (vk & bmask));
    // keys 8c + (0..3) go to piece 2h of the channel, keys 8c + 4 + (0..3) to piece 2h + 1,
    // both at slot 4 (c % 2), with h = c / 2
    const int c = vk >> 3;
    v_lds[j] = d * VLD + (c >> 1) * 16 + (c & 1) * 4;
  }
  const size_t page_elems = ((size_t)nkv * HD) << bsh;        // of a page of K, and of a page of V
  const int last_entry = p.max_blocks - 1;
  struct Pages { int k[PPT], v[PPT]; };
  struct Stage { bf16x8 k[PPT], v[PPT]; };
  // A key past the request's last (in its last tile, or in the tile fetched after the last) is
  // read from wherever its table entry points, page 0 where there is none.  It is masked, but
  // its value still meets a weight of 0 in the second product, and 0 x NaN is NaN: the caller
  // keeps page 0 cleared and clears a page before a request first writes to part of it, so
  // what is read here is the request's own or zero, never what another request left.
  auto look_up = [&](int key0, Pages& pg) {
    const int first = key0 >> bsh;
#pragma unroll
    for (int j = 0; j < PPT; j++) {
      pg.k[j] = table[min(first + k_idx[j], last_entry)];
      pg.v[j] = table[min(first + v_idx[j], last_entry)];
    }
  };
  auto fetch = [&](int key0, const Pages& pg, Stage& st) {
    const unsigned in_page = (unsigned)(key0 & bmask);
#pragma unroll
    for (int j = 0; j < PPT; j++) {
      st.k[j] = *(const bf16x8*)(p.kcache + ((size_t)max(pg.k[j], 0) * page_elems + (k_off[j] + in_page * HD)));
      st.v[j] = *(const bf16x8*)(p.vcache + ((size_t)max(pg.v[j], 0) * page_elems + (v_off[j] + in_page)));
    }
  };
  auto stash = [&](int buf, const Stage& st) {
    __bf16* kb = sK + buf * 32 * KLD;
    __bf16* vb = sV + buf * HD * VLD;
#pragma unroll
    for (int j = 0; j < PPT; j++) {
      if (PIECES % NT == 0 || tid + j * NT < PIECES) {
        *(bf16x8*)(kb + k_lds[j]) = st.k[j];
        __bf16* vrow = vb + v_lds[j];
        bf16x4 lo4, hi4;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          lo4[e] = st.v[j][e];
          hi4[e] = st.v[j][4 + e];
        }
        *(bf16x4*)vrow = lo4;
        *(bf16x4*)(vrow + 8) = hi4;
      }
    }
  };
  const bool capped = p.softcap > 0.f;
  auto tile = [&](int buf, int key0) {
    const __bf16* kb = sK + buf * 32 * KLD + lr * KLD + lk * 8;
    const __bf16* vb = sV + buf * HD * VLD + lk * 8;
    // ---- S^T = K Q^T
    f32x16 s;
#pragma unroll
    for (int e = 0; e < 16; e++) s[e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < HD16; ks++)
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)(kb + ks * 16), qf[ks], s, 0, 0, 0);
    // ---- scale, cap, mask, running softmax (one query row per lane)
    float mt = -INFINITY;
    if (capped) {
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const float ex = __builtin_amdgcn_exp2f(p.k2 * s[e]);
        s[e] = p.c2 * (1.f - 2.f * __builtin_amdgcn_rcpf(ex + 1.f));
      }
    } else {
#pragma unroll
      for (int e = 0; e < 16; e++) s[e] *= p.k1;
    }
    if (key0 < all_lo || key0 + 31 > all_hi) {
#pragma unroll
      for (int j = 0; j < 4; j++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int key = key0 + 8 * j + 4 * lk + i;
          const bool ok = row_ok && key >= row_lo && key <= pos;
          s[4 * j + i] = ok ? s[4 * j + i] : -INFINITY;
        }
    }
#pragma unroll
    for (int e = 0; e < 16; e++) mt = fmaxf(mt, s[e]);
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float m_new = mt > m_run + 8.f ? mt : m_run;      // the maximum is followed lazily
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const bool moved = m_new > m_run;
    const float corr = moved ? __builtin_amdgcn_exp2f(m_run - m_use) : 1.f;
    float rs = 0.f;
#pragma unroll
    for (int e = 0; e < 16; e++) {
      const float pe = __builtin_amdgcn_exp2f(s[e] - m_use);
      s[e] = pe;
      rs += pe;
    }
    rs += __shfl_xor(rs, 32, 64);
    l_run = l_run * corr + rs;
    m_run = m_new;
    bf16x8 pb[2];
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
      for (int e = 0; e < 8; e++) pb[h][e] = (__bf16)s[8 * h + e];
    // ---- O^T = corr O^T + V^T P^T
    if (__builtin_expect(__any(moved), 0)) {
      // in the accumulation registers, where the products keep them
#pragma unroll
      for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int e = 0; e < 16; e++) {
          float t;
          asm volatile("v_accvgpr_read_b32 %1, %0\n\tv_mul_f32 %1, %1, %2\n\ts_nop 0\n\tv_accvgpr_write_b32 %0, %1"
                       : "+a"(o[dt][e]), "=&v"(t)
                       : "v"(corr));
        }
    }
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
      const __bf16* vr = vb + min(dt * 32 + lr, HD - 1) * VLD;
      o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)vr, pb[0], o[dt], 0, 0, 0);
      o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)(vr + 16), pb[1], o[dt], 0, 0, 0);
    }
  };

  // Every wave takes every tile of the block, also the few near the diagonal (or before its
  // window) that none of its rows sees: masked, such a tile adds nothing, and a loop without a
  // branch around the products lets the compiler leave the accumulators where they are (with
  // the branch it copied all of them to ordinary registers on every turn: 852 instead of 1,135 us
  // at 16 heads of 256).  The turn after the last tile fetches that tile again and leaves it
  // unused.
  {
    int key0 = (key_lo / 32) * 32;
    Pages pg, pn;
    Stage st;
    look_up(key0, pg);
    fetch(key0, pg, st);
    look_up(key0 + 32, pn);
    stash(0, st);
    __syncthreads();
    for (int buf = 0; key0 <= key_hi; key0 += 32, buf ^= 1) {
      fetch(key0 + 32, pn, st);
      look_up(key0 + 64, pn);
      tile(buf, key0);
      stash(buf ^ 1, st);
      __syncthreads();
    }
  }
  if (!SPLIT && !row_ok) return;
  if (SPLIT) {
    // A wave's results of its range, as they lie in its registers: 16 bytes a lane, a wave's 64
    // lanes one contiguous KB per (dt, j), so every store is whole lines.  The joining kernel
    // reads them back with the same lanes.  Every lane stores, rows or not.
    const size_t slot = ((((size_t)blockIdx.z * p.nkv + kvh) * (gridDim.x / p.nchunks) + rows_x) * p.nchunks + range) * NW + wave;
    p.part_ml[slot * 128 + lane] = lk == 0 ? m_run : l_run;
    f32x4* po = (f32x4*)p.part_o + slot * (DT * 4 * 64) + lane;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int j = 0; j < 4; j++)
        po[(dt * 4 + j) * 64] = f32x4{o[dt][4 * j], o[dt][4 * j + 1], o[dt][4 * j + 2], o[dt][4 * j + 3]};
    return;
  }
  const float inv = 1.f / l_run;
  __bf16* orow = p.out + ((size_t)trow * p.nh + head) * HD;
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int d = dt * 32 + 8 * j + 4 * lk;
      if (d < HD) {
        bf16x4 w;
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (__bf16)(o[dt][4 * j + i] * inv);
        *(bf16x4*)(orow + d) = w;
      }
    }
}

// Joins the ranges of keys of a portion's rows (attn_shared_kernel, SPLIT), in their order: a
// block of 64 threads per (32 channels of a wave of a block of rows, KV head, request), every
// lane the row and the channels it had in the kernel that wrote the partial results.  The ranges a block of rows
// has follow from its first and last key as there; a range that a row does not see at all (one
// past its position, in a block of rows on the diagonal) has the maximum -inf and weighs nothing.
__global__ __launch_bounds__(64) void attn_portion_join_kernel(AttnParams p, int per_block, int row_blocks, int dts) {
  const int r = p.r_begin + blockIdx.z, kvh = blockIdx.y;
  const int dt = blockIdx.x % dts, ww = blockIdx.x / dts;      // 32 channels of a wave's rows a block
  const int rows_x = ww >> 2, wave = ww & 3;
  const int lane = threadIdx.x, lr = lane & 31, lk = lane >> 5;
  const int qs = p.q_start[r], n = p.q_start[r + 1] - qs;
  if (n <= 0) return;
  const int start = p.ctx_len[r] - n;
  const int bi = (n + per_block - 1) / per_block - 1 - rows_x;
  if (bi < 0) return;
  const int g = p.nh / p.nkv;
  const int t0 = bi * per_block + wave * p.tpw;
  const int ntok = max(0, min(p.tpw, n - t0));
  const int tok = lr / g, hq = lr - tok * g;
  if (tok >= ntok) return;
  const int blk_lo = start + bi * per_block, blk_hi = start + min(n, (bi + 1) * per_block) - 1;
  const int key_lo = p.window > 0 ? max(0, blk_lo - p.window + 1) : 0;
  const int ranges = (blk_hi / 32 - key_lo / 32) / p.chunk + 1;
  const size_t slot0 = ((((size_t)blockIdx.z * p.nkv + kvh) * row_blocks + rows_x) * p.nchunks) * 4 + wave;
  float m = -INFINITY;
  for (int c = 0; c < ranges; c++) m = fmaxf(m, p.part_ml[(slot0 + (size_t)c * 4) * 128 + lr]);
  f32x4 acc[4];
#pragma unroll
  for (int j = 0; j < 4; j++) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  float l = 0.f;
  for (int c = 0; c < ranges; c++) {
    const size_t slot = slot0 + (size_t)c * 4;
    const float mc = p.part_ml[slot * 128 + lr];
    const float w = mc == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mc - m);
    l += w * p.part_ml[slot * 128 + 32 + lr];
    const f32x4* po = (const f32x4*)p.part_o + slot * ((size_t)dts * 4 * 64) + (size_t)dt * 4 * 64 + lane;
#pragma unroll
    for (int j = 0; j < 4; j++) acc[j] += w * po[j * 64];
  }
  const float inv = 1.f / l;
  __bf16* orow = p.out + ((size_t)(qs + t0 + tok) * p.nh + kvh * g + hq) * p.hd;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int d = dt * 32 + 8 * j + 4 * lk;
    if (d < p.hd) {
      bf16x4 w4;
#pragma unroll
      for (int i = 0; i < 4; i++) w4[i] = (__bf16)(acc[j][i] * inv);
      *(bf16x4*)(orow + d) = w4;
    }
  }
}

// One wave per (request, KV head, chunk of 64 keys) for requests that bring one token.
// Columns of every tile are the g query heads of the KV head (col = lane % 16), rows are
// keys (first product) or channels (second product).
template <int HD32>
__global__ __launch_bounds__(256, 2) void attn_decode_kernel(AttnParams p) {
  constexpr int KS = HD32;       // 32-wide steps over head_dim
  constexpr int DT = HD32 * 2;   // 16-channel output tiles
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, kq = lane >> 4;
  const int r = p.r_begin + blockIdx.z;
  const int kvh = blockIdx.y;
  // Where the window is much shorter than the longest context, the grid covers a window's
  // blocks only and counts them from the block the request's window begins in.
  int block_x = blockIdx.x;
  if (p.from_window) block_x += max(0, p.ctx_len[r] - p.window) / (4 * p.chunk);
  const int chunk = block_x * 4 + wave;
  const int* table = p.block_table + (size_t)r * p.max_blocks;
  const int hd = p.hd, bsh = p.bs_shift, bmask = p.bs - 1, nkv = p.nkv;
  // The pages of the chunk's (up to two) tiles are asked for before the request's length is
  // known, beside it: where a key lies follows from the chunk alone.  A key past the context is
  // masked below; a hole in the table reads page 0, which the caller keeps cleared, and the
  // places of a request's last page behind its last token are cleared too (a masked value
  // still meets a weight of 0 in the second product, and 0 x NaN is NaN).
  int kpage[2][2], vpage[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int k0 = chunk * p.chunk + 32 * i;
#pragma unroll
    for (int t = 0; t < 2; t++) {
      kpage[i][t] = table[min((k0 + 16 * t + col) >> bsh, p.max_blocks - 1)];
      vpage[i][t] = table[min((k0 + 16 * t + 4 * kq) >> bsh, p.max_blocks - 1)];
    }
  }
  const int n = p.q_start[r + 1] - p.q_start[r];
  if (n <= 0) return;
  const int pos = p.ctx_len[r] - 1;
  const int row_lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
  // a block whose four chunks all lie past the context or before the window ends here, all
  // its waves alike: the grid is sized for the longest context the caller allows
  const int first_chunk = block_x * 4;
  if (first_chunk * p.chunk > pos || first_chunk * p.chunk + 4 * p.chunk - 1 < row_lo) return;
  const int key_lo = max(row_lo, chunk * p.chunk);
  const int key_hi = min(pos, chunk * p.chunk + p.chunk - 1);
  const bool active = key_lo <= key_hi;          // a wave without keys still meets the others at the barrier
  const int g = p.nh / p.nkv;
  const bool col_ok = col < g;
  const int head = kvh * g + (col_ok ? col : 0);
  const int trow = p.q_start[r];

  // the query operand waits in LDS (one 16-byte piece per lane and step), not in registers
  __shared__ bf16x8 sq[4][KS][64];
  {
    const __bf16* qr = p.q + (size_t)trow * p.q_stride + (size_t)head * hd + kq * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      bf16x8 t;
      if (col_ok) t = *(const bf16x8*)(qr + ks * 32);
      else
#pragma unroll
        for (int e = 0; e < 8; e++) t[e] = (__bf16)0.f;
      sq[wave][ks][lane] = t;
    }
  }
  f32x4 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; dt++) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;

#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int key0 = chunk * p.chunk + 32 * i;
    if (!active || 32 * i >= p.chunk || key0 > key_hi || key0 + 31 < key_lo) continue;
    bf16x8 kf[2][KS];
#pragma unroll
    for (int t = 0; t < 2; t++) {
      const int kk = key0 + 16 * t + col;
      const int page = max(kpage[i][t], 0);
      const __bf16* kr = p.kcache + ((((size_t)page * nkv + kvh) << bsh) + (kk & bmask)) * hd + kq * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) kf[t][ks] = *(const bf16x8*)(kr + ks * 32);
    }
    bf16x8 vf[DT];
    {
      const int ka = key0 + 4 * kq, kb = key0 + 16 + 4 * kq;
      const int pa = max(vpage[i][0], 0), pb = max(vpage[i][1], 0);
      const __bf16* va_base = p.vcache + ((((size_t)pa * nkv + kvh) * hd) << bsh) + (ka & bmask);
      const __bf16* vb_base = p.vcache + ((((size_t)pb * nkv + kvh) * hd) << bsh) + (kb & bmask);
#pragma unroll
      for (int dt = 0; dt < DT; dt++) {
        const int d = dt * 16 + col;
        const bf16x4 va = *(const bf16x4*)(va_base + ((size_t)d << bsh));
        const bf16x4 vb = *(const bf16x4*)(vb_base + ((size_t)d << bsh));
#pragma unroll
        for (int e = 0; e < 4; e++) {
          vf[dt][e] = va[e];
          vf[dt][4 + e] = vb[e];
        }
      }
    }
    f32x4 s[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
      s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ks++) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][ks], sq[wave][ks][lane], s[t], 0, 0, 0);
    }
    float mt = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int key = key0 + 16 * t + 4 * kq + i;
        float v = score_log2(p, s[t][i]);
        v = (col_ok && key >= key_lo && key <= key_hi) ? v : -INFINITY;
        s[t][i] = v;
        mt = fmaxf(mt, v);
      }
    mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
    mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
    const float m_new = fmaxf(m_run, mt);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float corr = __builtin_amdgcn_exp2f(m_run - m_use);
    float rs = 0.f;
    bf16x8 pb8;
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const float pe = __builtin_amdgcn_exp2f(s[t][i] - m_use);
        rs += pe;
        pb8[4 * t + i] = (__bf16)pe;
      }
    rs += __shfl_xor(rs, 16, 64);
    rs += __shfl_xor(rs, 32, 64);
    l_run = l_run * corr + rs;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
      o[dt] *= corr;
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pb8, o[dt], 0, 0, 0);
    }
  }
  // the block's four chunks are joined here, in chunk order: one partial result per 256 keys
  extern __shared__ float dyn[];
  float* sm_ml = dyn;                 // [4][16][2]
  float* sm_o = dyn + 4 * 16 * 2;     // [4][g][hd]
  if (col_ok) {
    if (kq == 0) {
      sm_ml[(wave * 16 + col) * 2] = m_run;
      sm_ml[(wave * 16 + col) * 2 + 1] = l_run;
    }
    float* so = sm_o + ((size_t)wave * g + col) * hd;
#pragma unroll
    for (int dt = 0; dt < DT; dt++) *(f32x4*)(so + dt * 16 + 4 * kq) = o[dt];
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < g * hd; idx += 256) {
    const int c = idx / hd, d = idx - c * hd;
    float mw[4], m = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; w++) {
      mw[w] = sm_ml[(w * 16 + c) * 2];
      m = fmaxf(m, mw[w]);
    }
    float acc = 0.f, l = 0.f;
#pragma unroll
    for (int w = 0; w < 4; w++) {
      const float e = mw[w] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw[w] - m);
      acc += e * sm_o[((size_t)w * g + c) * hd + d];
      l += e * sm_ml[(w * 16 + c) * 2 + 1];
    }
    const size_t slot = ((size_t)(r - p.r_begin) * p.nh + kvh * g + c) * p.nchunks + block_x;
    p.part_o[slot * hd + d] = acc;
    if (d == 0) {
      p.part_ml[slot * 2] = m;
      p.part_ml[slot * 2 + 1] = l;
    }
  }
}

// Joins the chunks of a decoded token's attention, in chunk order: a block per
// (request, head), a thread per channel; the chunks' weights exp(m_c - m) are computed once.
#define ATT_MAX_CHUNKS 1024
__global__ __launch_bounds__(256) void attn_combine_kernel(const float* __restrict__ part_o,
                                                           const float* __restrict__ part_ml,
                                                           const int* __restrict__ q_start,
                                                           const int* __restrict__ ctx_len,
                                                           __bf16* __restrict__ out, int nh, int hd,
                                                           int window, int r_begin, int nchunks, int span) {
  __shared__ float wgt[ATT_MAX_CHUNKS];
  __shared__ float red[17];
  const int rr = blockIdx.x, head = blockIdx.y;
  const int r = r_begin + rr;
  const int n = q_start[r + 1] - q_start[r];
  if (n <= 0) return;
  const int pos = ctx_len[r] - 1;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int c0 = lo / span, c1 = pos / span;
  const size_t base = ((size_t)rr * nh + head) * nchunks;
  const int np = c1 - c0 + 1;
  // the first partial results of the thread's channel are asked for now: they come in while
  // the weights are worked out (a part past the last is read from the last and not used)
  constexpr int PF = 16;
  const int d0 = min((int)threadIdx.x, hd - 1);
  float pf[PF];
  {
    const float* po = part_o + (base + c0) * hd + d0;
#pragma unroll
    for (int c = 0; c < PF; c++) pf[c] = po[(size_t)min(c, np - 1) * hd];
  }
  float m = -INFINITY;
  for (int c = c0 + threadIdx.x; c <= c1; c += 256) m = fmaxf(m, part_ml[(base + c) * 2]);
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float l = 0.f;
  for (int c = c0 + threadIdx.x; c <= c1; c += 256) {
    const float w = __builtin_amdgcn_exp2f(part_ml[(base + c) * 2] - m);
    wgt[c - c0] = w;
    l += part_ml[(base + c) * 2 + 1] * w;
  }
  l = block_sum(l, red);
  const float inv = 1.f / l;
  __bf16* orow = out + ((size_t)q_start[r] * nh + head) * hd;
  for (int d = threadIdx.x; d < hd; d += 256) {
    const float* po = part_o + (base + c0) * hd + d;
    float acc = 0.f;
    int c = 0;
    if (d == d0) {                      // the channel whose first parts are here already
#pragma unroll
      for (int q = 0; q < PF; q++)
        if (q < np) acc += pf[q] * wgt[q];
      c = min(np, PF);
    }
    for (; c + 4 <= np; c += 4) {       // four loads in flight, summed in part order
      const float v0 = po[(size_t)c * hd], v1 = po[(size_t)(c + 1) * hd];
      const float v2 = po[(size_t)(c + 2) * hd], v3 = po[(size_t)(c + 3) * hd];
      acc += v0 * wgt[c];
      acc += v1 * wgt[c + 1];
      acc += v2 * wgt[c + 2];
      acc += v3 * wgt[c + 3];
    }
    for (; c < np; c++) acc += po[(size_t)c * hd] * wgt[c];
    orow[d] = (__bf16)(acc * inv);
  }
}

template <bool SPLIT, bool PAIR>
static int launch_attn(const AttnParams& p, dim3 grid, hipStream_t s) {
  // the join of a portion's four waves needs [4][32][2] + [2][ceil(hd/32) * 16][64] floats of LDS
  const size_t lds = SPLIT ? 0 : (4 * 32 * 2 + (size_t)2 * ((p.hd + 31) / 32) * 16 * 64) * sizeof(float);
  switch (p.hd / 16) {
    case 1: attn_mfma_kernel<1, SPLIT, PAIR><<<grid, 256, lds, s>>>(p); break;
    case 2: attn_mfma_kernel<2, SPLIT, PAIR><<<grid, 256, lds, s>>>(p); break;
    case 4: attn_mfma_kernel<4, SPLIT, PAIR><<<grid, 256, lds, s>>>(p); break;
    case 8: attn_mfma_kernel<8, SPLIT, PAIR><<<grid, 256, lds, s>>>(p); break;
    case 16: attn_mfma_kernel<16, SPLIT, PAIR><<<grid, 256, lds, s>>>(p); break;
    default: return zk_fail("zk_attention_bf16: head_dim must be 16, 32, 64, 128 or 256");
  }
  return zk_launch_status("zk_attention_bf16");
}

template <int HD16, int NW, bool SPLIT>
static int launch_shared_one(const AttnParams& p, dim3 grid, hipStream_t s) {
  constexpr int HD = HD16 * 16;
  constexpr size_t lds = ((size_t)2 * 32 * (HD + 8) + (size_t)2 * HD * (32 + 8)) * sizeof(__bf16);
  static bool prepared = false;
  if (!prepared) {
    if (lds > 64 * 1024 && hipFuncSetAttribute((const void*)attn_shared_kernel<HD16, NW, SPLIT>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return zk_fail("zk_attention_bf16: the shared-tile kernel's LDS buffers were refused");
    prepared = true;
  }
  attn_shared_kernel<HD16, NW, SPLIT><<<grid, NW * 64, lds, s>>>(p);
  return zk_launch_status("zk_attention_bf16 (shared tiles)");
}

template <int NW, bool SPLIT>
static int launch_shared(const AttnParams& p, dim3 grid, hipStream_t s) {
  switch (p.hd / 16) {
    case 1: return launch_shared_one<1, NW, SPLIT>(p, grid, s);
    case 2: return launch_shared_one<2, NW, SPLIT>(p, grid, s);
    case 4: return launch_shared_one<4, NW, SPLIT>(p, grid, s);
    case 8: return launch_shared_one<8, NW, SPLIT>(p, grid, s);
    case 16:
      if constexpr (NW <= 4) return launch_shared_one<16, NW, SPLIT>(p, grid, s);
      else return zk_fail("zk_attention_bf16: eight waves a block take head sizes up to 128");
    default: return zk_fail("zk_attention_bf16: head_dim must be 16, 32, 64, 128 or 256");
  }
}

// Bytes the portions' split variant needs behind the decoded tokens' part of the workspace.
// Per (request, KV head, block of rows, range, wave): the wave's accumulators as they lie in
// its registers (ceil(hd / 32) x 16 floats a lane) and 128 floats of maxima and sums.
static size_t portion_split_bytes(long row_blocks, int nkv, int hd, int ranges) {
  const size_t dt = (size_t)(hd + 31) / 32;
  return (size_t)row_blocks * nkv * ranges * 4 * (dt * 16 * 64 + 128) * sizeof(float);
}

// The ranges of keys for a launch of few blocks of rows: tiles a range (0: do not split) and the
// most ranges a block of rows can have.  Priced for one causal request of max_q_len rows ending
// at max_ctx, window or not: blocks(ct) = sum over the blocks of rows of ceil(tiles / ct), and
// the time goes with ceil(blocks / 256) * ct; of equal times the longer range (fewer partial
// results).  No split unless it at least halves the longest block's tiles; at most
// ATT_MOST_RANGES ranges for the longest block of rows the caller's limits allow (bound_tiles),
// which bounds the workspace.
static int portion_ranges(int max_q_len, int max_ctx, int window, int per_block, int nkv, int r_prefill,
                          int bound_tiles) {
  const int row_blocks = (max_q_len + per_block - 1) / per_block;
  auto tiles_of = [&](int bi) {
    const int lo = max_ctx - max_q_len + bi * per_block, hi = std::min(max_ctx, lo + per_block) - 1;
    const int klo = window > 0 ? std::max(0, lo - window + 1) : 0;
    return hi / 32 - klo / 32 + 1;
  };
  int longest = 0;
  for (int bi = 0; bi < row_blocks; bi++) longest = std::max(longest, tiles_of(bi));
  static const int cands[] = {32, 24, 16, 12, 10, 8, 6, 4};
  int best = 0;
  long best_cost = (long)((long)row_blocks * nkv * r_prefill + 255) / 256 * (longest + 10);
  for (int ct : cands) {
    if (2 * ct > longest || (bound_tiles + ct - 1) / ct > ATT_MOST_RANGES) continue;
    long blocks = 0;
    for (int bi = 0; bi < row_blocks; bi++) blocks += (tiles_of(bi) + ct - 1) / ct;
    blocks *= (long)nkv * r_prefill;
    const long cost = (blocks + 255) / 256 * (ct + 10) + 6;   // a block's start and end, the joining launch: in tiles' worth
    if (cost < best_cost) { best = ct; best_cost = cost; }
  }
  return best;
}

// 0: the portion kernel is chosen by the sizes; 1: a group of rows a block; 4, 8: shared
// tiles with that many waves a block; 5: shared tiles, four waves, the keys in ranges (as far as
// the workspace allows).  For tests and measurements (process-wide).
static int portion_kernel_mode = 0;

extern "C" {

int zk_attention_bf16_portion_kernel(int mode) {
  const int before = portion_kernel_mode;
  if (mode == 0 || mode == 1 || mode == 4 || mode == 5 || mode == 8) portion_kernel_mode = mode;
  return before;
}

// 1 if the matrix-core kernel takes these sizes, else 0 (the caller then uses the plain kernel).
int zk_attention_bf16_supports(int nh, int nkv, int hd, int bs) {
  if (nkv <= 0 || nh % nkv) return 0;
  const int g = nh / nkv;
  const bool hd_ok = hd == 16 || hd == 32 || hd == 64 || hd == 128 || hd == 256;
  return hd_ok && g <= 32 && bs >= 4 && (bs & (bs - 1)) == 0;
}

// Bytes of workspace the split variant needs for ``n_decode`` single-token requests.
size_t zk_attention_bf16_workspace(int n_decode, int nh, int hd, int max_ctx) {
  const size_t nchunks = ((size_t)max_ctx + ATT_CHUNK - 1) / ATT_CHUNK;      // an upper bound for both variants
  return (size_t)n_decode * nh * nchunks * (hd + 2) * sizeof(float);
}

// Bytes of workspace that let portions of up to ``max_rows`` rows in all split their keys into
// ranges (a launch of few blocks of rows with long contexts), on top of the decoded tokens'
// part.  A caller that brings less gets the kernels that need none.
size_t zk_attention_bf16_portion_workspace(int max_rows, int nh, int nkv, int hd) {
  if (max_rows <= 0 || nkv <= 0 || nh % nkv || hd <= 0) return 0;
  const int per_block = 4 * std::max(1, 32 / (nh / nkv));
  return portion_split_bytes((max_rows + per_block - 1) / per_block, nkv, hd, ATT_MOST_RANGES) + 256;
}

// Whether decoded tokens of these sizes run on the 16-wide tiles (partial results joined four
// chunks at a time inside a block) or on the 32-wide ones (one partial result a chunk).
static bool decode_on_narrow_tiles(int nh, int nkv, int hd) { return nh / nkv <= 16 && hd % 32 == 0; }

// The longest context the split variant takes for decoded tokens (the joining kernel keeps one
// weight per partial result in LDS).  ``decode_chunk`` as in zk_attention_bf16.
long long zk_attention_bf16_max_context(int nh, int nkv, int hd, int decode_chunk) {
  if (nkv <= 0 || nh % nkv) return 0;
  const int chunk = decode_chunk == 32 ? 32 : ATT_CHUNK;
  const long long span = decode_on_narrow_tiles(nh, nkv, hd) ? 4LL * chunk : ATT_CHUNK;
  return span * ATT_MAX_CHUNKS;
}

// Requests [0, r_prefill) hold portions of more than one token (max_q_len the longest);
// requests [r_prefill, R) hold one token each and use the split variant over max_ctx keys.
// decode_chunk: keys a wave of the split variant takes on the 16-wide tiles, 32 or 64 (0: 64).
// It fixes where the sums over keys are cut, and so the bits of the result: a caller that wants
// a request's result not to depend on the rest of the batch passes the same value in every
// step.  32 gives twice the waves, each with one load from memory in its chain instead of
// two: better for few requests with short contexts, worse for many.
int zk_attention_bf16(const void* q, int q_stride, const void* kcache, const void* vcache_t,
                      const int* block_table, int max_blocks, const int* q_start, const int* ctx_len,
                      void* out, int R, int r_prefill, int max_q_len, int max_ctx, int nh, int nkv,
                      int hd, int bs, float scale, float softcap, int window, int decode_chunk,
                      void* workspace, size_t workspace_bytes, void* stream) {
  ZK_REQUIRE(R >= 0 && r_prefill >= 0 && r_prefill <= R, "zk_attention_bf16: bad request counts");
  ZK_REQUIRE(zk_attention_bf16_supports(nh, nkv, hd, bs), "zk_attention_bf16: sizes not supported "
             "(head_dim 16/32/64/128/256, at most 32 heads a KV head, page size a power of two from 4)");
  ZK_REQUIRE(q_stride >= nh * hd && q_stride % 8 == 0 && ((uintptr_t)q % 16 == 0),
             "zk_attention_bf16: q rows must be 16-byte aligned");
  ZK_REQUIRE(max_blocks > 0 && nkv <= 65535 && R <= 65535, "zk_attention_bf16: grid too large");
  ZK_REQUIRE(decode_chunk == 0 || decode_chunk == 32 || decode_chunk == 64,
             "zk_attention_bf16: decode_chunk must be 32 or 64");
  if (R == 0) return 0;
  // everything that can refuse is checked before the first launch
  if (R - r_prefill > 0) {
    ZK_REQUIRE(max_ctx > 0, "zk_attention_bf16: max_ctx must be positive");
    ZK_REQUIRE(max_ctx <= zk_attention_bf16_max_context(nh, nkv, hd, decode_chunk),
               "zk_attention_bf16: context too long for the split variant");
    ZK_REQUIRE(zk_attention_bf16_workspace(R - r_prefill, nh, hd, max_ctx) <= workspace_bytes,
               "zk_attention_bf16: workspace too small for the split partial results");
  }
  if (r_prefill > 0) ZK_REQUIRE(max_q_len > 0, "zk_attention_bf16: max_q_len must be positive");
  hipStream_t s = (hipStream_t)stream;
  AttnParams p;
  p.q = (const __bf16*)q; p.q_stride = q_stride;
  p.kcache = (const __bf16*)kcache; p.vcache = (const __bf16*)vcache_t;
  p.block_table = block_table; p.max_blocks = max_blocks;
  p.q_start = q_start; p.ctx_len = ctx_len; p.out = (__bf16*)out;
  p.nh = nh; p.nkv = nkv; p.hd = hd; p.bs = bs;
  p.scale = scale; p.softcap = softcap; p.window = window;
  p.from_window = 0;
  p.bs_shift = 0;
  while ((1 << p.bs_shift) < bs) p.bs_shift++;
  const float log2e = 1.4426950408889634f;
  p.k1 = scale * log2e;
  p.k2 = softcap > 0.f ? 2.f * scale / softcap * log2e : 0.f;
  p.c2 = softcap * log2e;
  const int g = nh / nkv;
  if (r_prefill > 0) {
    p.tpw = 32 / g; p.r_begin = 0; p.nchunks = 1; p.part_o = nullptr; p.part_ml = nullptr;
    const int groups = (max_q_len + p.tpw - 1) / p.tpw;
    // one block a group; two groups a block when that lets every block run at once (256 CUs,
    // one block each) where single groups would need a second round
    const long long single = (long long)groups * nkv * r_prefill, paired = (long long)((groups + 1) / 2) * nkv * r_prefill;
    int rc;
    // Many groups: tiles shared by the four or eight groups of a block, where that still gives
    // every CU a block (four) or two (eight; head sizes up to 128, whose registers let two
    // waves share a SIMD).  Measured at 8 to 32 heads of 128 and 256 with 512 to 8,192 rows:
    // with fewer than about 768 groups the kernel of one group a block is faster (2,048 rows of
    // 8 heads of 256, 512 groups: 75 us against 111; 768 groups: a tie), with more the shared
    // tiles are (8 portions of 512 rows behind 7,680 tokens, 32 heads of 128: 1,630 -> 780 us;
    // 16 heads of 256: 1,560 -> 845 us; 8,192 rows of 8 heads of 256: 877 -> 463 us).
    int shared_waves = 0;
    if (bs >= 8 && portion_kernel_mode != 1) {
      if (portion_kernel_mode > 1) shared_waves = portion_kernel_mode;
      else if (single >= 4096 && hd <= 128) shared_waves = 8;
      else if (single >= 768) shared_waves = 4;
      if (shared_waves == 8 && hd > 128) shared_waves = 4;       // no room for two waves a SIMD
    }
    // Few blocks of rows with many keys each (a portion of a few hundred rows behind thousands of
    // tokens): four groups a block and the keys in ranges, where the workspace behind the decoded
    // tokens' part holds the ranges' partial results.  512 rows behind 3,584 tokens, 8 heads of
    // 256: 111 -> 52 us; behind 7,680: 209 -> 79 us; 16 heads of 256: 118 -> 76 us; 32 heads of
    // 128: 100 -> 73 us.  A whole prompt from its first token, 8 heads of 256: 2,048 rows 74 -> 62
    // us, 1,024 rows the same time either way (its blocks of rows are many and short already).
    int range_tiles = 0, most_ranges = 0;
    size_t split_at = 0;
    if (bs >= 8 && (portion_kernel_mode == 5 || (portion_kernel_mode == 0 && !shared_waves))) {
      const int per_block = 4 * p.tpw;
      // no block of rows has more tiles than this, whatever its request's length
      int bound = (max_ctx + 31) / 32;
      if (window > 0) bound = std::min(bound, (window + per_block + 31) / 32 + 1);
      range_tiles = portion_ranges(max_q_len, max_ctx, window, per_block, nkv, r_prefill, bound);
      if (range_tiles) {
        most_ranges = (bound + range_tiles - 1) / range_tiles;
        if (R - r_prefill > 0) split_at = (zk_attention_bf16_workspace(R - r_prefill, nh, hd, max_ctx) + 255) / 256 * 256;
        const size_t need = portion_split_bytes((long)r_prefill * ((max_q_len + per_block - 1) / per_block), nkv, hd,
                                                most_ranges);
        if (workspace == nullptr || (uintptr_t)workspace % 16 != 0 || split_at + need > workspace_bytes)
          range_tiles = 0;
      }
    }
    if (range_tiles) {
      const int per_block = 4 * p.tpw;
      AttnParams ps = p;
      ps.chunk = range_tiles;
      ps.nchunks = most_ranges;
      const int row_blocks = (max_q_len + per_block - 1) / per_block;
      const size_t slots = (size_t)r_prefill * nkv * row_blocks * most_ranges * 4;
      const int dts = (hd + 31) / 32;
      ps.part_o = (float*)((char*)workspace + split_at);
      ps.part_ml = ps.part_o + slots * dts * 16 * 64;
      dim3 grid(row_blocks * most_ranges, nkv, r_prefill);
      rc = launch_shared<4, true>(ps, grid, s);
      if (rc) return rc;
      attn_portion_join_kernel<<<dim3(row_blocks * 4 * dts, nkv, r_prefill), 64, 0, s>>>(ps, per_block, row_blocks, dts);
      rc = zk_launch_status("zk_attention_bf16 (join of the portions' ranges)");
    } else if (shared_waves) {
      if (shared_waves == 5) shared_waves = 4;
      dim3 grid((groups + shared_waves - 1) / shared_waves, nkv, r_prefill);
      rc = shared_waves == 4 ? launch_shared<4, false>(p, grid, s) : launch_shared<8, false>(p, grid, s);
    } else if (single > 256 && paired <= 256) rc = launch_attn<false, true>(p, dim3((groups + 1) / 2, nkv, r_prefill), s);
    else rc = launch_attn<false, false>(p, dim3(groups, nkv, r_prefill), s);
    if (rc) return rc;
  }
  const int n_dec = R - r_prefill;
  if (n_dec > 0) {
    const int nchunks = (max_ctx + ATT_CHUNK - 1) / ATT_CHUNK;
    p.tpw = 1; p.r_begin = r_prefill; p.nchunks = nchunks;
    p.part_o = (float*)workspace;
    p.part_ml = (float*)workspace + (size_t)n_dec * nh * nchunks * hd;
    dim3 grid((nchunks + 3) / 4, nkv, n_dec);
    int rc = 0;
    int span = ATT_CHUNK;        // keys one partial result covers
    p.chunk = ATT_CHUNK;
    if (decode_on_narrow_tiles(nh, nkv, hd)) {
      if (decode_chunk == 32) {
        p.chunk = ATT_CHUNK / 2;
        grid.x = (2 * nchunks + 3) / 4;
      }
      // the block joins its four chunks: one partial result per 4 chunks of keys
      span = 4 * p.chunk;
      p.nchunks = grid.x;
      // a window covers at most ceil(window / span) + 1 blocks of span keys
      const int window_blocks = window > 0 ? (window + span - 1) / span + 1 : 0;
      if (window > 0 && window_blocks < (int)grid.x) {
        p.from_window = 1;
        grid.x = window_blocks;
      }
      p.part_ml = (float*)workspace + (size_t)n_dec * nh * p.nchunks * hd;
      const size_t lds = (4 * 16 * 2 + (size_t)4 * g * hd) * sizeof(float);
      switch (hd / 32) {
        case 1: attn_decode_kernel<1><<<grid, 256, lds, s>>>(p); break;
        case 2: attn_decode_kernel<2><<<grid, 256, lds, s>>>(p); break;
        case 4: attn_decode_kernel<4><<<grid, 256, lds, s>>>(p); break;
        default: attn_decode_kernel<8><<<grid, 256, lds, s>>>(p); break;
      }
      rc = zk_launch_status("zk_attention_bf16 (decode)");
    } else {
      rc = launch_attn<true, false>(p, grid, s);
    }
    if (rc) return rc;
    dim3 cgrid(n_dec, nh);
    attn_combine_kernel<<<cgrid, 256, 0, s>>>(p.part_o, p.part_ml, q_start, ctx_len, (__bf16*)out, nh, hd,
                                              window, r_prefill, p.nchunks, span);
    return zk_launch_status("zk_attention_bf16 (combine)");
  }
  return 0;
}

}  // extern "C"

#endif  // ZSE_ACT_BF16
