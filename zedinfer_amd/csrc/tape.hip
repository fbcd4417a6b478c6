// The step tape: the launches of one step, recorded once as (entry point, arguments) and run again
// with one call.  A step whose shape recurs (the same numbers of tokens and entries, the same
// buffers) makes the same calls into this library with the same arguments; only the contents of the
// device memory they point to change.  Replaying the list from here costs the host the launches
// alone, a few microseconds each, where the interpreter needs about twenty for each call it makes.
// (The reference keeps its whole step in native code for the same reason:
// src/frontend/models/transformer_forward.cpp:60-150.)
//
// Arguments are recorded as 64-bit words: integers and pointers by value, float and double parameters
// as the bits of a double.  The caller knows each entry point's parameter kinds; the number of
// arguments is checked against the declaration in zi_api.h.  A tape holds pointers: it is valid as long
// as the memory they name is, which is the recorder's business, and it must be run on the device and
// stream it was recorded on.  Nothing here touches the device.
#include "zi_api.h"
#include "zi_common.h"
#include <string.h>
#include <type_traits>
#include <utility>
#include <vector>

namespace {

template <typename T>
T tape_arg(int64_t bits) {
    if constexpr (std::is_pointer_v<T>) {
        return reinterpret_cast<T>(static_cast<uintptr_t>(bits));
    } else if constexpr (std::is_floating_point_v<T>) {
        double d;
        memcpy(&d, &bits, sizeof(d));
        return static_cast<T>(d);
    } else {
        return static_cast<T>(bits);
    }
}

typedef int (*TapeThunk)(const int64_t* args);

template <auto F>
struct Thunk;
template <typename... A, int (*F)(A...)>
struct Thunk<F> {
    static constexpr int count = sizeof...(A);
    template <size_t... I>
    static int go(const int64_t* a, std::index_sequence<I...>) {
        return F(tape_arg<A>(a[I])...);
    }
    static int call(const int64_t* a) { return go(a, std::index_sequence_for<A...>{}); }
};

struct TapeEntryPoint {
    const char* name;
    TapeThunk thunk;
    int count;
};

#define ZI_TAPE_ENTRY(f) {#f, &Thunk<&f>::call, Thunk<&f>::count},
const TapeEntryPoint tape_entry_points[] = {ZI_STREAM_ENTRY_POINTS(ZI_TAPE_ENTRY)};

struct TapeCall {
    const TapeEntryPoint* entry;
    size_t first;      // of its arguments in `words`
};

struct Tape {
    std::vector<TapeCall> calls;
    std::vector<int64_t> words;
};

}  // namespace

extern "C" void* zi_tape_new() { return new Tape(); }

extern "C" void zi_tape_free(void* tape) { delete static_cast<Tape*>(tape); }

extern "C" int zi_tape_length(const void* tape) { return tape ? (int)static_cast<const Tape*>(tape)->calls.size() : 0; }

// Append a call of the entry point `name` with `count` argument words.
extern "C" int zi_tape_record(void* tape, const char* name, const int64_t* words, int count) {
    ZI_REQUIRE(tape && name && (words || count == 0), "tape_record: null argument");
    for (const TapeEntryPoint& e : tape_entry_points) {
        if (strcmp(e.name, name) != 0) continue;
        ZI_REQUIRE(count == e.count, "tape_record: %s takes %d arguments, %d were recorded", name, e.count, count);
        Tape* t = static_cast<Tape*>(tape);
        t->calls.push_back(TapeCall{&e, t->words.size()});
        t->words.insert(t->words.end(), words, words + count);
        return 0;
    }
    return zi_fail("tape_record: %s is not an entry point that a tape can hold", name);
}

// Append `calls` calls at once: their names one after the other, each ended by a zero byte; counts[i] argument
// words of call i, all words in one row.  Nothing is appended when one of them is refused.
extern "C" int zi_tape_record_many(void* tape, const char* names, const int* counts, const int64_t* words, int calls) {
    ZI_REQUIRE(tape && names && counts && (words || calls == 0) && calls >= 0, "tape_record_many: null argument");
    Tape* t = static_cast<Tape*>(tape);
    const size_t had_calls = t->calls.size(), had_words = t->words.size();
    for (int i = 0; i < calls; ++i) {
        if (zi_tape_record(tape, names, words, counts[i]) != 0) {
            t->calls.resize(had_calls);
            t->words.resize(had_words);
            return 1;
        }
        names += strlen(names) + 1;
        words += counts[i];
    }
    return 0;
}

// Make every recorded call again, in order.  Stops at the first that fails and returns what it returned
// (its message is the one zi_last_error() gives); `done`, when not null, receives the number of calls made.
extern "C" int zi_tape_run(const void* tape, int* done) {
    ZI_REQUIRE(tape, "tape_run: null tape");
    const Tape* t = static_cast<const Tape*>(tape);
    int made = 0, rc = 0;
    for (const TapeCall& c : t->calls) {
        rc = c.entry->thunk(t->words.data() + c.first);
        if (rc != 0) break;
        ++made;
    }
    if (done) *done = made;
    return rc;
}
