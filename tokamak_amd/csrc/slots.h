// Every entry point that a layer's recorded launch list may hold also exists in a form with
// one signature, int f(const unsigned long long* slots): argument i is slot i, an integer or
// a pointer as it is, a float by its bits in the slot's low half.  A list of such calls is
// issued by one call from the host language (replay.hip) instead of one foreign call each.
#pragma once

#include <cstdint>
#include <cstring>
#include <utility>

namespace tk {

template <typename T>
inline T from_slot(uint64_t slot) {
  static_assert(sizeof(T) <= sizeof(uint64_t), "an argument fits a slot");
  T value;
  std::memcpy(&value, &slot, sizeof(T));  // little-endian: the low bytes
  return value;
}

template <typename... A, size_t... I>
inline int call_slots(int (*fn)(A...), const uint64_t* slots, std::index_sequence<I...>) {
  return fn(from_slot<A>(slots[I])...);
}

template <typename... A>
inline int call_slots(int (*fn)(A...), const uint64_t* slots) {
  return call_slots(fn, slots, std::index_sequence_for<A...>{});
}

}  // namespace tk

#define TK_SLOTS(name)                                                                       \
  extern "C" __attribute__((visibility("default"))) int name##_slots(const unsigned long long* slots) { \
    return tk::call_slots(&name, reinterpret_cast<const uint64_t*>(slots));                  \
  }
