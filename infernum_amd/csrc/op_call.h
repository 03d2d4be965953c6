// One calling convention for every launcher of the kernel libraries, so that a program of launches can be data.
//
// A launcher `int ia_xyz(typed arguments..., hipStream_t)` gets a twin `int ia_op_ia_xyz(const uint64_t* slots,
// int n)` that takes its arguments as n slots of 8 bytes: a pointer or an integer of any width as its value, a
// float as the bits of a double.  The interpreter of a step's program (step_program.cpp) fills the slots from the
// program's constants, the step's numbers and the step's arrays and calls the twin through a function pointer; it
// knows no launcher by name.  The twin checks the number of slots against the launcher's own parameter list, so a
// program written for another version of a launcher is refused instead of run.
#pragma once
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <utility>

namespace ia_op {

enum { ERR_SLOTS = 10001 };      // IA_ERR_BAD_ARG of common.h

template <class T>
struct Slot {                    // integers of any width, enums
  static T get(uint64_t s) { return static_cast<T>(static_cast<int64_t>(s)); }
};
template <class T>
struct Slot<T*> {
  static T* get(uint64_t s) { return reinterpret_cast<T*>(static_cast<uintptr_t>(s)); }
};
template <>
struct Slot<float> {
  static float get(uint64_t s) {
    double d;
    std::memcpy(&d, &s, sizeof d);
    return static_cast<float>(d);
  }
};
template <>
struct Slot<double> {
  static double get(uint64_t s) {
    double d;
    std::memcpy(&d, &s, sizeof d);
    return d;
  }
};

template <class... A, std::size_t... I>
int call(int (*fn)(A...), const uint64_t* slots, std::index_sequence<I...>) {
  return fn(Slot<A>::get(slots[I])...);
}

template <class... A>
int invoke(int (*fn)(A...), const uint64_t* slots, int n) {
  if (slots == nullptr || n != static_cast<int>(sizeof...(A))) return ERR_SLOTS;
  return call(fn, slots, std::index_sequence_for<A...>{});
}

}  // namespace ia_op

// after the launcher's definition:  IA_OP(ia_embed)  defines  ia_op_ia_embed
#define IA_OP(fn) \
  extern "C" int ia_op_##fn(const uint64_t* slots, int n) { return ia_op::invoke(&fn, slots, n); }
