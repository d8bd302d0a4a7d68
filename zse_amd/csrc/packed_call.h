// Calling an entry point from its arguments written down as 64-bit words.
//
// Every entry point of the kernel libraries has the shape
//     extern "C" int zk_name(<pointers, ints, floats, sizes...>, void* stream);
// A launch list (steplist.hip) keeps a call as the entry point's number and its arguments as
// words: a pointer or size as it is, an int sign-extended, a float as its bits.  ZK_PACKED(zk_name)
// defines, beside the entry point,
//     int zk_name_packed(const uint64_t* words, void* stream)   which unpacks and calls it, and
//     int zk_name_nargs()                                       the number of arguments, stream included,
// so that a table of such functions can repeat any call.  A library of a part's own kernels
// uses the same macro and hands the two functions to zk_steplist_register; nothing in the
// launch lists knows the entry points by name.
//
// An argument of type ``int*`` (not const) is a result the host reads by reference; a call
// repeated from a list gets a throw-away int there when the word is not 0.  Device memory is
// passed as ``void*`` or as a pointer to const.
#pragma once
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <utility>

typedef int (*zk_packed_fn)(const uint64_t* words, void* stream);

namespace zk_packed {

template <typename T>
struct Arg;
template <typename T>
struct Arg<T*> {
  static T* get(uint64_t w) { return (T*)(uintptr_t)w; }
};
template <>
struct Arg<int*> {
  static int* get(uint64_t w) {
    static thread_local int thrown_away;
    return w ? &thrown_away : nullptr;
  }
};
template <>
struct Arg<int> {
  static int get(uint64_t w) { return (int)(int64_t)w; }
};
template <>
struct Arg<unsigned long> {
  static unsigned long get(uint64_t w) { return (unsigned long)w; }
};
template <>
struct Arg<unsigned long long> {
  static unsigned long long get(uint64_t w) { return (unsigned long long)w; }
};
template <>
struct Arg<float> {
  static float get(uint64_t w) {
    const uint32_t b = (uint32_t)w;
    float f;
    memcpy(&f, &b, 4);
    return f;
  }
};

template <auto F>
struct Call;
template <typename... A, int (*F)(A...)>
struct Call<F> {
  static constexpr int nargs = (int)sizeof...(A);
  // the last argument is the stream: the caller's, not the one that was written down
  template <size_t... I>
  static int go(const uint64_t* w, void* stream, std::index_sequence<I...>) {
    return F(Arg<A>::get(I + 1 == sizeof...(A) ? (uint64_t)(uintptr_t)stream : w[I])...);
  }
  static int call(const uint64_t* w, void* stream) { return go(w, stream, std::index_sequence_for<A...>{}); }
};

}  // namespace zk_packed

#define ZK_PACKED(fn)                                                                                  \
  extern "C" int fn##_packed(const uint64_t* words, void* stream) { return zk_packed::Call<fn>::call(words, stream); } \
  extern "C" int fn##_nargs() { return zk_packed::Call<fn>::nargs; }
