// The launch sequence of a step, kept on the native side.
//
// A step of the model is a few hundred kernel launches whose arguments depend only on the
// step's shape (how many tokens, requests and wanted rows, how long the longest portion and
// context are): device addresses come from a bump allocator that hands out the same
// addresses for the same sequence of sizes, and what differs between steps of one shape
// (tokens, positions, block tables) is read by the kernels from device memory.  The first
// step of a shape runs from Python, call by call, and every call is also written down here;
// later steps of that shape are one call into zk_steplist_run, which launches the whole
// sequence from C++.  The reference drives each launch from Python (it measured about 7 us a
// launch, orchestrator/hip_graph.py:3-5) and has a C dispatch table for single launches that
// is switched off (orchestrator/fast_dispatch.py:151-337).
#include "common.h"

#include <cstring>
#include <vector>

extern "C" {
int zk_embed(const void* table, const int* tokens, float* out, float scale, int T, int H, int V, int strip,
             void* stream);
int zk_rmsnorm(const void* x, int x_is_f32, const int* rows, const float* w, void* out, float eps, int unit_offset,
               int n_rows, int H, void* stream);
int zk_norm_add_norm(const void* sub, int sub_parts, const float* w_post, float eps_post, int uo_post, float* h,
                     const float* w_next, float eps_next, int uo_next, void* out, int T, int H, void* stream);
int zk_gated_act(const void* gu, void* out, int T, int I, int act, void* stream);
int zk_softcap(float* z, size_t n, float cap, void* stream);
int zk_rope_cache_write(void* qkv, const int* positions, const int* slot_map, const float* inv_freq, int rotary_dim,
                        void* kcache, void* vcache, int T, int nh, int nkv, int hd, int bs, int v_transposed,
                        void* stream);
int zk_zero(void* p, size_t nbytes, void* stream);
int zk_gemm_plain(const void* A, int lda, const void* W, void* C, int ldc, int c_is_f32, int M, int N, int K,
                  void* stream);
int zk_attention_plain(const void* q, int q_stride, const void* kcache, const void* vcache, const int* block_table,
                       int max_blocks, const int* req_of_token, const int* positions, void* out, int T, int nh,
                       int nkv, int hd, int bs, float scale, float softcap, int window, int v_transposed,
                       void* stream);
#if ZSE_ACT_BF16
int zk_gemm_bf16(const void* A, int lda, const void* W, void* C, int ldc, int c_is_f32, int M, int N, int K, int epi,
                 float cap, int w_strip, void* ws, size_t ws_bytes, int* parts, void* stream);
int zk_qkv_rope_bf16(const void* A, int lda, const void* W, void* Q, int ldq, int M, int K, int w_strip,
                     const int* positions, const int* slot_map, const float* inv_freq, void* kcache, void* vcache,
                     int nh, int nkv, int hd, int bs, int v_transposed, void* stream);
int zk_attention_bf16(const void* q, int q_stride, const void* kcache, const void* vcache_t, const int* block_table,
                      int max_blocks, const int* q_start, const int* ctx_len, void* out, int R, int r_prefill,
                      int max_q_len, int max_ctx, int nh, int nkv, int hd, int bs, float scale, float softcap,
                      int window, int decode_chunk, void* workspace, size_t workspace_bytes, void* stream);
#endif
}

namespace {

// One written-down call: which entry point, and its arguments as 64-bit words in the order
// of the C signature (a pointer or size as it is, an int sign-extended, a float as its bits).
// The last argument of every entry point is the stream; a run puts its own there.
struct StepCall {
  int op;
  int n;
  uint64_t a[24];
};

struct StepList {
  std::vector<StepCall> calls;
};

inline void* P(uint64_t w) { return (void*)(uintptr_t)w; }
inline int I(uint64_t w) { return (int)(int64_t)w; }
inline size_t Z(uint64_t w) { return (size_t)w; }
inline float F(uint64_t w) {
  const uint32_t b = (uint32_t)w;
  float f;
  memcpy(&f, &b, 4);
  return f;
}

struct OpInfo {
  const char* name;
  int nargs;
};

enum {
  OP_EMBED, OP_RMSNORM, OP_NORM_ADD_NORM, OP_GATED_ACT, OP_SOFTCAP, OP_ROPE_CACHE_WRITE, OP_ZERO, OP_GEMM_PLAIN,
  OP_ATTENTION_PLAIN, OP_GEMM_BF16, OP_QKV_ROPE_BF16, OP_ATTENTION_BF16, OP_COUNT
};

const OpInfo OPS[OP_COUNT] = {
    {"zk_embed", 9},        {"zk_rmsnorm", 10},   {"zk_norm_add_norm", 13},    {"zk_gated_act", 6},
    {"zk_softcap", 4},      {"zk_rope_cache_write", 14}, {"zk_zero", 3},        {"zk_gemm_plain", 10},
    {"zk_attention_plain", 19}, {"zk_gemm_bf16", 16}, {"zk_qkv_rope_bf16", 19}, {"zk_attention_bf16", 24},
};

int run_call(const StepCall& c, void* s) {
  const uint64_t* a = c.a;
  switch (c.op) {
    case OP_EMBED:
      return zk_embed(P(a[0]), (const int*)P(a[1]), (float*)P(a[2]), F(a[3]), I(a[4]), I(a[5]), I(a[6]), I(a[7]), s);
    case OP_RMSNORM:
      return zk_rmsnorm(P(a[0]), I(a[1]), (const int*)P(a[2]), (const float*)P(a[3]), P(a[4]), F(a[5]), I(a[6]),
                        I(a[7]), I(a[8]), s);
    case OP_NORM_ADD_NORM:
      return zk_norm_add_norm(P(a[0]), I(a[1]), (const float*)P(a[2]), F(a[3]), I(a[4]), (float*)P(a[5]),
                              (const float*)P(a[6]), F(a[7]), I(a[8]), P(a[9]), I(a[10]), I(a[11]), s);
    case OP_GATED_ACT:
      return zk_gated_act(P(a[0]), P(a[1]), I(a[2]), I(a[3]), I(a[4]), s);
    case OP_SOFTCAP:
      return zk_softcap((float*)P(a[0]), Z(a[1]), F(a[2]), s);
    case OP_ROPE_CACHE_WRITE:
      return zk_rope_cache_write(P(a[0]), (const int*)P(a[1]), (const int*)P(a[2]), (const float*)P(a[3]), I(a[4]),
                                 P(a[5]), P(a[6]), I(a[7]), I(a[8]), I(a[9]), I(a[10]), I(a[11]), I(a[12]), s);
    case OP_ZERO:
      return zk_zero(P(a[0]), Z(a[1]), s);
    case OP_GEMM_PLAIN:
      return zk_gemm_plain(P(a[0]), I(a[1]), P(a[2]), P(a[3]), I(a[4]), I(a[5]), I(a[6]), I(a[7]), I(a[8]), s);
    case OP_ATTENTION_PLAIN:
      return zk_attention_plain(P(a[0]), I(a[1]), P(a[2]), P(a[3]), (const int*)P(a[4]), I(a[5]), (const int*)P(a[6]),
                                (const int*)P(a[7]), P(a[8]), I(a[9]), I(a[10]), I(a[11]), I(a[12]), I(a[13]),
                                F(a[14]), F(a[15]), I(a[16]), I(a[17]), s);
#if ZSE_ACT_BF16
    case OP_GEMM_BF16: {
      // the number of partial-sum planes follows from the shape: the Python side read it when
      // the call was written down and laid the next call out accordingly; here it is dropped
      int parts = 0;
      return zk_gemm_bf16(P(a[0]), I(a[1]), P(a[2]), P(a[3]), I(a[4]), I(a[5]), I(a[6]), I(a[7]), I(a[8]), I(a[9]),
                          F(a[10]), I(a[11]), P(a[12]), Z(a[13]), a[14] ? &parts : nullptr, s);
    }
    case OP_QKV_ROPE_BF16:
      return zk_qkv_rope_bf16(P(a[0]), I(a[1]), P(a[2]), P(a[3]), I(a[4]), I(a[5]), I(a[6]), I(a[7]),
                              (const int*)P(a[8]), (const int*)P(a[9]), (const float*)P(a[10]), P(a[11]), P(a[12]),
                              I(a[13]), I(a[14]), I(a[15]), I(a[16]), I(a[17]), s);
    case OP_ATTENTION_BF16:
      return zk_attention_bf16(P(a[0]), I(a[1]), P(a[2]), P(a[3]), (const int*)P(a[4]), I(a[5]), (const int*)P(a[6]),
                               (const int*)P(a[7]), P(a[8]), I(a[9]), I(a[10]), I(a[11]), I(a[12]), I(a[13]), I(a[14]),
                               I(a[15]), I(a[16]), F(a[17]), F(a[18]), I(a[19]), I(a[20]), P(a[21]), Z(a[22]), s);
#endif
    default:
      return zk_fail("zk_steplist_run: unknown entry point");
  }
}

}  // namespace

extern "C" {

// The number of an entry point that can be written down, or -1.
int zk_steplist_op(const char* name) {
  for (int i = 0; i < OP_COUNT; i++) {
#if !ZSE_ACT_BF16
    if (i >= OP_GEMM_BF16) break;
#endif
    if (strcmp(OPS[i].name, name) == 0) return i;
  }
  return -1;
}

void* zk_steplist_create() { return new StepList(); }

void zk_steplist_destroy(void* list) { delete (StepList*)list; }

int zk_steplist_size(void* list) { return list ? (int)((StepList*)list)->calls.size() : 0; }

// Appends a call: ``args`` holds the entry point's arguments as 64-bit words, stream included.
int zk_steplist_add(void* list, int op, const uint64_t* args, int nargs) {
  ZK_REQUIRE(list != nullptr && args != nullptr, "zk_steplist_add: no list");
  ZK_REQUIRE(op >= 0 && op < OP_COUNT && nargs == OPS[op].nargs, "zk_steplist_add: wrong number of arguments");
  StepCall c;
  c.op = op;
  c.n = nargs;
  memcpy(c.a, args, sizeof(uint64_t) * nargs);
  ((StepList*)list)->calls.push_back(c);
  return 0;
}

// Launches every call of the list, in order, on ``stream``.  Stops at the first entry point
// that refuses: its status comes back, ``*failed_at`` is its index, zk_last_error() its message.
int zk_steplist_run(void* list, void* stream, int* failed_at) {
  ZK_REQUIRE(list != nullptr, "zk_steplist_run: no list");
  const std::vector<StepCall>& calls = ((StepList*)list)->calls;
  for (size_t i = 0; i < calls.size(); i++) {
    const int rc = run_call(calls[i], stream);
    if (rc != 0) {
      if (failed_at) *failed_at = (int)i;
      return rc;
    }
  }
  return 0;
}

// The name of the entry point of call ``index`` (for error messages).
const char* zk_steplist_name(void* list, int index) {
  if (!list || index < 0 || index >= (int)((StepList*)list)->calls.size()) return "";
  return OPS[((StepList*)list)->calls[index].op].name;
}

}  // extern "C"
