// Replays the recorded launches of one layer for another layer like it.
//
// A step walks layers that differ in nothing but their tensors: the same kernels, grids and sizes, other
// weights and other cache pages.  The bindings record the launches of the first such layer (entry point and
// arguments, `GbTapeEntry`), and this runner makes them again for every later one with the pointers that lay
// inside the recorded layer's tensors moved into the tensors of the layer at hand.  A replayed launch costs
// what the device runtime's launch costs and nothing of the interpreter.
//
// The recorded entry points are those that GB_TAPED (hip/common.h) gives: `int entry_taped(const uint64* slots)`.
#include <cstdint>

namespace {

constexpr int kMaxArgs = 32;

struct GbTapeEntry {
  uint64_t entry;     // address of the `_taped` form of the entry point
  uint64_t pointers;  // bit i: argument i is a pointer
  uint32_t n_args;
  uint32_t reserved;
  uint64_t args[kMaxArgs];
};
static_assert(sizeof(GbTapeEntry) == 24 + 8 * kMaxArgs, "the bindings pack entries of this size");

typedef int (*TapedEntry)(const unsigned long long*);

}  // namespace

extern "C" {

int gbh_tape_entry_bytes() { return (int)sizeof(GbTapeEntry); }
int gbh_tape_max_args() { return kMaxArgs; }

// Makes the `n` recorded launches again.  A pointer argument p with from[r] <= p < from[r] + bytes[r] for some
// range r (the first that holds it) becomes to[r] + (p - from[r]); every other argument is passed as recorded.
// Returns 0, or 1 + the index of the first launch whose entry point refused (its library holds the message):
// launches before it have been made, none after it.
int gbh_tape_run(const void* entries, int n, const uint64_t* from, const uint64_t* bytes, const uint64_t* to,
                 int n_ranges) {
  const GbTapeEntry* tape = (const GbTapeEntry*)entries;
  unsigned long long args[kMaxArgs];
  for (int e = 0; e < n; ++e) {
    const GbTapeEntry& t = tape[e];
    if (t.n_args > (uint32_t)kMaxArgs) return 1 + e;
    for (uint32_t i = 0; i < t.n_args; ++i) {
      uint64_t v = t.args[i];
      if ((t.pointers >> i & 1) && v != 0) {
        for (int r = 0; r < n_ranges; ++r) {
          if (v >= from[r] && v - from[r] < bytes[r]) {
            v = to[r] + (v - from[r]);
            break;
          }
        }
      }
      args[i] = v;
    }
    if (((TapedEntry)(uintptr_t)t.entry)(args) != 0) return 1 + e;
  }
  return 0;
}

}  // extern "C"
