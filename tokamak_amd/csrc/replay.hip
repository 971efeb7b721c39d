// Host code: issue a recorded list of kernel launches with other addresses put in.
//
// A step that is not replayed from a HIP graph records the launches of the first layer of a
// kind and launches the other layers of that kind from the list (engine/layer_replay.py).
// Each entry is an entry point in its slot form (slots.h) and its arguments as slots; a
// patch names a slot that holds an address inside one of the layer's own tensors, the
// tensor's place in `addresses`, and the offset inside it.  One call from the host language
// issues the whole layer.
#include <cstdint>

typedef int (*slots_fn)(const unsigned long long*);

// Returns -1 when every call returned the status it returned when it was recorded; else the
// index of the first call that did not (its status in *got), after which nothing is issued.
extern "C" __attribute__((visibility("default"))) int tk_replay_calls(
    int ncalls, const void* const* fns, const int* first_slot, unsigned long long* slots, int npatches,
    const int* patch_slot, const int* patch_key, const long long* patch_offset,
    const unsigned long long* addresses, const int* expected, int* got) {
  for (int p = 0; p < npatches; ++p)
    slots[patch_slot[p]] = addresses[patch_key[p]] + (unsigned long long)patch_offset[p];
  for (int c = 0; c < ncalls; ++c) {
    const int status = reinterpret_cast<slots_fn>(const_cast<void*>(fns[c]))(slots + first_slot[c]);
    if (status != expected[c]) {
      *got = status;
      return c;
    }
  }
  return -1;
}
