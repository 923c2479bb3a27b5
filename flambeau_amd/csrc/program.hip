// Step programs: a recorded list of calls of this library's launch functions, replayed with ONE
// call from the host language.
//
// The step function of the engine is driven from Python: a forward pass of a 7B model is some 230
// launches, each a Python call, an argument check and a foreign-function call (3 to 4 ms of host
// time per step).  While a step runs for the first time, every launch is also appended here with
// the values of its arguments; a later step of the same shape (same numbers of rows, same kernel
// choices, same buffers) replays the list from C++, which costs the launches alone.  Arguments are
// kept as they were given: device pointers must still be valid and mean the same (the caller keys
// its programs by everything that decides them and drops them when a buffer moves).  The stream is
// not recorded: every function of the interface takes it last, and the replay passes its own.
//
// The reference keeps its whole step on the native side (crates/forward/src/runtime/mod.rs:185-264);
// this is the part of that which a host language cannot do quickly.
#include <string.h>
#include <type_traits>
#include <utility>
#include <vector>
#include "common.h"
#include "api.h"

namespace {

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

typedef int (*Trampoline)(const FlArg*, hipStream_t);

template <auto Fn>
struct Tramp {
    template <typename... A>
    static constexpr int count(int (*)(A...)) { return (int)sizeof...(A); }
    template <typename... A>
    static int run(int (*fn)(A...), const FlArg* a, hipStream_t s) { return invoke(fn, a, s, std::index_sequence_for<A...>{}); }
    static int call(const FlArg* a, hipStream_t s) { return run(Fn, a, s); }
    static constexpr int n_args = count(Fn);
};

struct Known {
    const char* name;
    Trampoline call;
    int n_args;
};

#define FL_KNOWN(f) {#f, &Tramp<&f>::call, Tramp<&f>::n_args}
const Known g_known[] = {
    FL_KNOWN(fl_embed), FL_KNOWN(fl_rmsnorm), FL_KNOWN(fl_add_inplace), FL_KNOWN(fl_gemm_plain), FL_KNOWN(fl_rope_kv_write),
    FL_KNOWN(fl_rope_table), FL_KNOWN(fl_attn_plain), FL_KNOWN(fl_silu_mul), FL_KNOWN(fl_feed_tokens), FL_KNOWN(fl_argmax),
    FL_KNOWN(fl_sample), FL_KNOWN(fl_gemm_skinny), FL_KNOWN(fl_gemm_skinny_fused), FL_KNOWN(fl_gemm_mid),
    FL_KNOWN(fl_gemm_mid_scaled), FL_KNOWN(fl_gemm_mid_residual), FL_KNOWN(fl_gemm_mid_partials), FL_KNOWN(fl_reduce_residual),
    FL_KNOWN(fl_gemm_tiled), FL_KNOWN(fl_gemm_skinny_rope), FL_KNOWN(fl_gemm_tiled_rope), FL_KNOWN(fl_gemm_tiled_scaled),
    FL_KNOWN(fl_gemm_tiled_residual), FL_KNOWN(fl_attn_decode), FL_KNOWN(fl_attn_decode_static), FL_KNOWN(fl_attn_prefill),
    FL_KNOWN(fl_gemm_mid_ex), FL_KNOWN(fl_gemm_tiled_ex), FL_KNOWN(fl_gemm_tiled_residual_ex), FL_KNOWN(fl_gemm_tiled_rope_ex), FL_KNOWN(fl_attn_decode_items),
    FL_KNOWN(fl_gemm_tiled_partials),
};
#undef FL_KNOWN

struct Entry {
    const Known* what;
    size_t first_arg;
};

struct Program {
    std::vector<Entry> entries;
    std::vector<FlArg> args;
};

}  // namespace

extern "C" void* fl_program_new(void) { return new Program(); }

extern "C" void fl_program_free(void* program) { delete (Program*)program; }

extern "C" int fl_program_size(const void* program) { return program ? (int)((const Program*)program)->entries.size() : 0; }

// Append one call: `name` is the launch function's name, args[0 .. n_args - 1] its arguments with the
// stream left out or in (n_args may count it or not; its value is ignored).
extern "C" int fl_program_append(void* program, const char* name, const FlArg* args, int n_args) {
    FL_CHECK(program && name && (args || n_args == 0), "program_append: needs a program, a name and arguments");
    Program* p = (Program*)program;
    for (const Known& k : g_known) {
        if (strcmp(k.name, name) != 0) continue;
        FL_CHECK(n_args == k.n_args || n_args == k.n_args - 1, "program_append: %s takes %d arguments, %d given", name,
                 k.n_args, n_args);
        p->entries.push_back(Entry{&k, p->args.size()});
        for (int i = 0; i < k.n_args; ++i) {
            FlArg a;
            a.l = 0;
            if (i < n_args) a = args[i];
            p->args.push_back(a);
        }
        return 0;
    }
    fl_set_error("program_append: '%s' is no launch function of this library", name);
    return -1;
}

// Run every recorded call in order on `stream`.  Stops at the first call that fails: its index goes to
// *failed_at (if given), its code is returned, and fl_last_error() says why.
extern "C" int fl_program_run(const void* program, hipStream_t stream, int* failed_at) {
    FL_CHECK(program, "program_run: no program");
    const Program* p = (const Program*)program;
    const FlArg* args = p->args.data();
    const size_t n = p->entries.size();
    for (size_t i = 0; i < n; ++i) {
        const Entry& e = p->entries[i];
        const int rc = e.what->call(args + e.first_arg, stream);
        if (rc != 0) {
            if (failed_at) *failed_at = (int)i;
            return rc;
        }
    }
    return 0;
}
