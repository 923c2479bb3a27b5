// Launch functions that a step program can record and replay (program.hip).
//
// A launch function is any `int f(..., hipStream_t stream)` whose other arguments are pointers, int,
// long or float.  `FL_RECORDABLE(f)` beside its definition makes it known to the recorder under its
// own name: a static object registers a trampoline that unpacks recorded arguments and calls `f`
// with the replay's stream.  Nothing else has to be edited when a kernel is added.  A launch function
// of another shared library joins the same way, or by calling fl_program_register itself.
#pragma once
#include <type_traits>
#include <utility>
#include "api.h"

namespace fl_rec {

template <typename T>
inline T arg_as(const FlArg& a) {
    if constexpr (std::is_pointer<T>::value) return (T)a.p;
    else if constexpr (std::is_same<T, float>::value) return a.f;
    else if constexpr (std::is_same<T, long>::value) return a.l;
    else {
        static_assert(std::is_same<T, int>::value, "launch functions take pointers, int, long and float");
        return a.i;
    }
}

// argument I of N: the recorded value, or the replay's stream for the last one
template <typename T, size_t I, size_t N>
inline T pick(const FlArg* a, hipStream_t stream) {
    if constexpr (I + 1 == N) {
        static_assert(std::is_same<T, hipStream_t>::value, "the stream is the last argument of every launch function");
        return stream;
    } else {
        return arg_as<T>(a[I]);
    }
}

template <typename... A, size_t... I>
inline int invoke(int (*fn)(A...), const FlArg* a, hipStream_t stream, std::index_sequence<I...>) {
    return fn(pick<A, I, sizeof...(A)>(a, stream)...);
}

template <auto Fn>
struct Tramp {
    template <typename... A>
    static constexpr int count(int (*)(A...)) { return (int)sizeof...(A); }
    template <typename... A>
    static int run(int (*fn)(A...), const FlArg* a, hipStream_t s) { return invoke(fn, a, s, std::index_sequence_for<A...>{}); }
    static int call(const FlArg* a, hipStream_t s) { return run(Fn, a, s); }
    static constexpr int n_args = count(Fn);
};

struct Registrar {
    Registrar(const char* name, FlTrampoline call, int n_args) { fl_program_register(name, call, n_args); }
};

}  // namespace fl_rec

#define FL_RECORDABLE(f) \
    static const fl_rec::Registrar fl_rec_registrar_##f(#f, &fl_rec::Tramp<&f>::call, fl_rec::Tramp<&f>::n_args);
