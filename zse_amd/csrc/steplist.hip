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
//
// The entry points are a table, not a list of names known here: a row holds a name, the
// number of arguments and a function that calls the entry point from its arguments as words
// (packed_call.h).  This library's own entry points enter the table when it is loaded; a
// library of a part's own kernels adds its rows with zk_steplist_register.
#include "common.h"
#include "packed_call.h"

#include <cstring>
#include <mutex>
#include <string>
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
int zk_rope_cache_write_sums(void* qkv, const float* planes, int sums, const int* positions, const int* slot_map,
                             const float* inv_freq, int rotary_dim, void* kcache, void* vcache, int T, int nh,
                             int nkv, int hd, int bs, int v_transposed, void* stream);
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
int zk_head_pick_bf16(const void* A, int lda, const void* W, int M, int N, int K, float cap, int w_strip,
                      void* picks, size_t picks_bytes, void* ids, void* stream);
int zk_attention_bf16(const void* q, int q_stride, const void* kcache, const void* vcache_t, const int* block_table,
                      int max_blocks, const int* q_start, const int* ctx_len, void* out, int R, int r_prefill,
                      int max_q_len, int max_ctx, int nh, int nkv, int hd, int bs, float scale, float softcap,
                      int window, int decode_chunk, void* workspace, size_t workspace_bytes, void* stream);
#endif
}

namespace {

constexpr int MOST_ARGS = 24;

// One written-down call: a row of the table, and the entry point's arguments as 64-bit words
// in the order of its C signature.  The last argument of every entry point is the stream; a
// run puts its own there.
struct StepCall {
  int op;
  uint64_t a[MOST_ARGS];
};

struct StepList {
  std::vector<StepCall> calls;
};

struct Op {
  std::string name;
  int nargs;
  zk_packed_fn fn;
};

std::mutex table_lock;

// Room for every row is set aside once, so a row never moves: a list may be launched (rows
// read without the lock) while another thread adds a row.
constexpr size_t MOST_OPS = 1024;

std::vector<Op>& table() {
  static std::vector<Op> ops = []() {
    std::vector<Op> v;
    v.reserve(MOST_OPS);
    return v;
  }();
  return ops;
}

int enter(const char* name, int nargs, zk_packed_fn fn) {
  if (!name || !fn || nargs < 1 || nargs > MOST_ARGS) return -1;
  std::lock_guard<std::mutex> hold(table_lock);
  std::vector<Op>& ops = table();
  for (size_t i = 0; i < ops.size(); i++)
    if (ops[i].name == name) {          // entered again (a library loaded a second time): the newer function
      if (ops[i].nargs != nargs) return -1;
      ops[i].fn = fn;
      return (int)i;
    }
  if (ops.size() >= MOST_OPS) return -1;
  ops.push_back(Op{name, nargs, fn});
  return (int)ops.size() - 1;
}

// zk_gemm_bf16 tells the caller by reference into how many planes of partial sums it split K.
// That number follows from the shape: the Python side read it when the call was written down
// and laid the next call out accordingly; a repeated call gets a throw-away int (packed_call.h).
#define OWN(fn) enter(#fn, zk_packed::Call<fn>::nargs, zk_packed::Call<fn>::call)
const int entered_at_load = []() {
  OWN(zk_embed);
  OWN(zk_rmsnorm);
  OWN(zk_norm_add_norm);
  OWN(zk_gated_act);
  OWN(zk_softcap);
  OWN(zk_rope_cache_write);
  OWN(zk_rope_cache_write_sums);
  OWN(zk_zero);
  OWN(zk_gemm_plain);
  OWN(zk_attention_plain);
#if ZSE_ACT_BF16
  OWN(zk_gemm_bf16);
  OWN(zk_qkv_rope_bf16);
  OWN(zk_attention_bf16);
  OWN(zk_head_pick_bf16);
#endif
  return 0;
}();
#undef OWN

}  // namespace

extern "C" {

// Adds an entry point to the table: ``fn`` calls it from ``nargs`` argument words, the stream
// last (the *_packed function that ZK_PACKED defines).  Returns its number, the one
// zk_steplist_op gives for the name from now on; -1 for a bad argument.
int zk_steplist_register(const char* name, int nargs, void* fn) { return enter(name, nargs, (zk_packed_fn)fn); }

// The number of an entry point that can be written down, or -1.
int zk_steplist_op(const char* name) {
  if (!name) return -1;
  std::lock_guard<std::mutex> hold(table_lock);
  const std::vector<Op>& ops = table();
  for (size_t i = 0; i < ops.size(); i++)
    if (ops[i].name == name) return (int)i;
  return -1;
}

void* zk_steplist_create() { return new StepList(); }

void zk_steplist_destroy(void* list) { delete (StepList*)list; }

int zk_steplist_size(void* list) { return list ? (int)((StepList*)list)->calls.size() : 0; }

// Appends a call: ``args`` holds the entry point's arguments as 64-bit words, stream included.
int zk_steplist_add(void* list, int op, const uint64_t* args, int nargs) {
  ZK_REQUIRE(list != nullptr && args != nullptr, "zk_steplist_add: no list");
  {
    std::lock_guard<std::mutex> hold(table_lock);
    const std::vector<Op>& ops = table();
    ZK_REQUIRE(op >= 0 && op < (int)ops.size() && nargs == ops[op].nargs, "zk_steplist_add: wrong number of arguments");
  }
  StepCall c;
  c.op = op;
  memcpy(c.a, args, sizeof(uint64_t) * nargs);
  ((StepList*)list)->calls.push_back(c);
  return 0;
}

// Launches every call of the list, in order, on ``stream``.  Stops at the first entry point
// that refuses: its status comes back, ``*failed_at`` is its index; its message is with the
// library the entry point belongs to.
int zk_steplist_run(void* list, void* stream, int* failed_at) {
  ZK_REQUIRE(list != nullptr, "zk_steplist_run: no list");
  const std::vector<StepCall>& calls = ((StepList*)list)->calls;
  // rows are only ever added and never move: no lock while launching
  const std::vector<Op>& ops = table();
  for (size_t i = 0; i < calls.size(); i++) {
    const int rc = ops[calls[i].op].fn(calls[i].a, stream);
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
  return table()[((StepList*)list)->calls[index].op].name.c_str();
}

}  // extern "C"
