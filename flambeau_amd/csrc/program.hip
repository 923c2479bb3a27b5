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
#include <string>
#include <vector>
#include "common.h"
#include "api.h"

namespace {

struct Known {
    std::string name;
    FlTrampoline call;
    int n_args;
};

// Filled by the static registrars of FL_RECORDABLE (recordable.h) while the library is loaded, and by
// fl_program_register afterwards; made at first use, so the order in which files initialise does not
// matter.  Entries are never removed: a program keeps indices into it.
std::vector<Known>& known() {
    static std::vector<Known> v;
    return v;
}

int find_known(const char* name) {
    const std::vector<Known>& v = known();
    for (size_t i = 0; i < v.size(); ++i)
        if (v[i].name == name) return (int)i;
    return -1;
}

struct Entry {
    int what;           // index into known()
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
    const int at = find_known(name);
    FL_CHECK(at >= 0, "program_append: '%s' is no launch function known to the recorder (FL_RECORDABLE or fl_program_register)", name);
    const int want = known()[at].n_args;
    FL_CHECK(n_args == want || n_args == want - 1, "program_append: %s takes %d arguments, %d given", name, want, n_args);
    p->entries.push_back(Entry{at, p->args.size()});
    for (int i = 0; i < want; ++i) {
        FlArg a;
        a.l = 0;
        if (i < n_args) a = args[i];
        p->args.push_back(a);
    }
    return 0;
}

// Make a launch function known to the recorder: `call` unpacks n_args recorded arguments (the last is
// the stream's place) and calls it.  Registering a name again replaces its trampoline.
extern "C" int fl_program_register(const char* name, FlTrampoline call, int n_args) {
    FL_CHECK(name && *name && call && n_args >= 1, "program_register: needs a name, a trampoline and the number of arguments");
    const int at = find_known(name);
    if (at >= 0) {
        known()[at].call = call;
        known()[at].n_args = n_args;
    } else {
        known().push_back(Known{name, call, n_args});
    }
    return 0;
}

// Arguments of a recordable launch function (the stream included), or -1 if the name is unknown.
extern "C" int fl_program_knows(const char* name) {
    const int at = name ? find_known(name) : -1;
    return at < 0 ? -1 : known()[at].n_args;
}

// Run every recorded call in order on `stream`.  Stops at the first call that fails: its index goes to
// *failed_at (if given), its code is returned, and fl_last_error() says why.
extern "C" int fl_program_run(const void* program, hipStream_t stream, int* failed_at) {
    FL_CHECK(program, "program_run: no program");
    const Program* p = (const Program*)program;
    const FlArg* args = p->args.data();
    const Known* calls = known().data();
    const size_t n = p->entries.size();
    for (size_t i = 0; i < n; ++i) {
        const Entry& e = p->entries[i];
        const int rc = calls[e.what].call(args + e.first_arg, stream);
        if (rc != 0) {
            if (failed_at) *failed_at = (int)i;
            return rc;
        }
    }
    return 0;
}
