// mgpu for AMD CDNA4: the small value types host and device code share --
// the error type, a register array, index ranges.  Names and members are the
// public ones of src/moderngpu/types.hxx:9-145; only what the
// load-balancing-search / segmented-reduce path uses is here.
#pragma once
#include <exception>
#include "meta.hxx"
#include "operators.hxx"

BEGIN_MGPU_NAMESPACE

////////////////////////////////////////////////////////////////////////////////
// Failure of a runtime call (allocation, launch, copy).  Thrown by context_t,
// mem_t and the launch front ends; carries the hipError_t it came from.

struct cuda_exception_t : std::exception {
  hipError_t result;
  explicit cuda_exception_t(hipError_t code) : result(code) { }
  const char* what() const noexcept override {
    return hipGetErrorString(result);
  }
};

// Which of two equal keys a search or merge takes first.
enum bounds_t { bounds_lower, bounds_upper };

////////////////////////////////////////////////////////////////////////////////
// `size` values a thread keeps in registers.  Index it with constants
// (iterate<size>(...), fully unrolled loops): a run-time index sends the whole
// array to scratch memory.

template<typename type_t, int size>
struct array_t {
  type_t data[size];

  array_t() = default;
  // Every element set to x.
  MGPU_HOST_DEVICE array_t(type_t x) {
    PRAGMA_UNROLL
    for(int i = 0; i < size; ++i) data[i] = x;
  }

  MGPU_HOST_DEVICE type_t& operator[](int i) { return data[i]; }
  MGPU_HOST_DEVICE type_t operator[](int i) const { return data[i]; }
};

// Nothing to hold (vt == 0 instantiations must still compile).
template<typename type_t>
struct array_t<type_t, 0> {
  MGPU_HOST_DEVICE type_t& operator[](int) { return *(type_t*)nullptr; }
  MGPU_HOST_DEVICE type_t operator[](int) const { return type_t(); }
};

////////////////////////////////////////////////////////////////////////////////
// Half-open index ranges.

struct MGPU_ALIGN(8) range_t {
  int begin, end;
  MGPU_HOST_DEVICE int count() const { return end - begin; }
  MGPU_HOST_DEVICE int size() const { return end - begin; }
  MGPU_HOST_DEVICE bool valid() const { return begin < end; }
};

// Items [nv * cta, nv * (cta + 1)) of `count`, clipped at the end.
MGPU_HOST_DEVICE range_t get_tile(int cta, int nv, int count) {
  int first = nv * cta;
  int left = count - first;                 // first + nv may not fit an int
  return range_t { first, first + (left < nv ? left : nv) };
}

// A tile of a two-input merge: items (A) and segment starts (B).
struct MGPU_ALIGN(16) merge_range_t {
  int a_begin, a_end, b_begin, b_end;

  MGPU_HOST_DEVICE int a_count() const { return a_end - a_begin; }
  MGPU_HOST_DEVICE int b_count() const { return b_end - b_begin; }
  MGPU_HOST_DEVICE int total() const { return a_count() + b_count(); }
  MGPU_HOST_DEVICE range_t a_range() const { return { a_begin, a_end }; }
  MGPU_HOST_DEVICE range_t b_range() const { return { b_begin, b_end }; }
  MGPU_HOST_DEVICE bool a_valid() const { return a_begin < a_end; }
  MGPU_HOST_DEVICE bool b_valid() const { return b_begin < b_end; }

  // The same two ranges laid out back to back from zero (A, then B): their
  // positions in an LDS array that holds the tile's keys.
  MGPU_HOST_DEVICE merge_range_t to_local() const {
    int na = a_count();
    return { 0, na, na, na + b_count() };
  }
  // What is left behind the split mp0 of cross-diagonal diag ...
  MGPU_HOST_DEVICE merge_range_t partition(int mp0, int diag) const {
    return { a_begin + mp0, a_end, b_begin + (diag - mp0), b_end };
  }
  // ... and what lies between the splits of two diagonals.
  MGPU_HOST_DEVICE merge_range_t partition(int mp0, int diag0, int mp1,
    int diag1) const {
    return { a_begin + mp0, a_begin + mp1, b_begin + (diag0 - mp0),
      b_begin + (diag1 - mp1) };
  }
};

// Register arrays handed between the steps of a merge: keys with values, and
// keys with the positions they came from.
template<typename key_t, typename val_t, int size>
struct kv_array_t {
  array_t<key_t, size> keys;
  array_t<val_t, size> vals;
};
template<typename type_t, int size>
struct merge_pair_t {
  array_t<type_t, size> keys;
  array_t<int, size> indices;
};

END_MGPU_NAMESPACE
