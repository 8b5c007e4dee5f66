// mgpu for AMD CDNA4: function objects and index->value iterators that appear
// in the signatures of segreduce / transform_lbs / spmv callers.
// Names and call shapes follow moderngpu's operators.hxx
// (src/moderngpu/operators.hxx:34-343).
#pragma once
#include "meta.hxx"

BEGIN_MGPU_NAMESPACE

// Read-only load.  On CDNA every global load of const data already goes
// through the vector L1/L2 path; there is no separate texture path to select,
// so this is a plain dereference (reference: operators.hxx:34-38 uses __ldg).
template<typename it_t>
MGPU_HOST_DEVICE typename std::iterator_traits<it_t>::value_type
ldg(it_t it) {
  return *it;
}

template<typename real_t>
MGPU_HOST_DEVICE real_t sq(real_t x) { return x * x; }

template<typename type_t>
MGPU_HOST_DEVICE void swap(type_t& a, type_t& b) {
  type_t c = a; a = b; b = c;
}

////////////////////////////////////////////////////////////////////////////////
// Comparison and arithmetic function objects.

#define MGPU_DEF_BINARY(name, ret_t, expr)                                    \
  template<typename type_t>                                                   \
  struct name {                                                               \
    MGPU_HOST_DEVICE ret_t operator()(type_t a, type_t b) const {             \
      return expr;                                                            \
    }                                                                         \
  };

MGPU_DEF_BINARY(less_t, bool, a < b)
MGPU_DEF_BINARY(less_equal_t, bool, a <= b)
MGPU_DEF_BINARY(greater_t, bool, a > b)
MGPU_DEF_BINARY(greater_equal_t, bool, a >= b)
MGPU_DEF_BINARY(equal_to_t, bool, a == b)
MGPU_DEF_BINARY(not_equal_to_t, bool, a != b)

MGPU_DEF_BINARY(plus_t, type_t, a + b)
MGPU_DEF_BINARY(minus_t, type_t, a - b)
MGPU_DEF_BINARY(multiplies_t, type_t, a * b)
// max/min resolve to mgpu::max/min: ties return the left operand.
MGPU_DEF_BINARY(maximum_t, type_t, mgpu::max(a, b))
MGPU_DEF_BINARY(minimum_t, type_t, mgpu::min(a, b))

#undef MGPU_DEF_BINARY

////////////////////////////////////////////////////////////////////////////////
// Iterators that compute their values from an index instead of reading memory.
// They offer what the library's kernels use of a random-access iterator:
// it[i], *it, it + n, it - n, it += n, it -= n and the iterator_traits types.

// The four offset operators for a class self_t whose position is `member`.
#define MGPU_ITERATOR_OFFSETS(self_t, int_t, member)                          \
  MGPU_HOST_DEVICE self_t& operator+=(int_t n) {                              \
    member += n; return static_cast<self_t&>(*this);                          \
  }                                                                           \
  MGPU_HOST_DEVICE self_t& operator-=(int_t n) {                              \
    member -= n; return static_cast<self_t&>(*this);                          \
  }                                                                           \
  MGPU_HOST_DEVICE self_t operator+(int_t n) const {                          \
    self_t moved = static_cast<const self_t&>(*this);                         \
    moved.member += n; return moved;                                          \
  }                                                                           \
  MGPU_HOST_DEVICE self_t operator-(int_t n) const {                          \
    self_t moved = static_cast<const self_t&>(*this);                         \
    moved.member -= n; return moved;                                          \
  }

// The member types std::iterator_traits looks for, as those of a pointer to
// const.  They are spelled out instead of inherited from
// std::iterator_traits<const value_type*>: a base class from namespace std
// would make std an associated namespace of every iterator here, and an
// unqualified make_tuple(...) or get<0>(...) on them ambiguous with the
// standard library's.
template<typename value_t>
struct iterator_types_t {
  typedef value_t value_type;
  typedef std::ptrdiff_t difference_type;
  typedef const value_t* pointer;
  typedef const value_t& reference;
  typedef std::random_access_iterator_tag iterator_category;
};

// CRTP base: a position and the offset operators.
template<typename outer_t, typename int_t, typename value_type>
struct iterator_t : iterator_types_t<value_type> {
  int_t index;
  iterator_t() = default;
  MGPU_HOST_DEVICE iterator_t(int_t i) : index(i) { }
  MGPU_ITERATOR_OFFSETS(outer_t, int_t, index)
};

// CRTP base of the read-only ones: outer_t::operator()(position) is the value.
template<typename outer_t, typename int_t, typename value_type>
struct const_iterator_t : iterator_t<outer_t, int_t, value_type> {
  const_iterator_t() = default;
  MGPU_HOST_DEVICE const_iterator_t(int_t i) :
    iterator_t<outer_t, int_t, value_type>(i) { }

  MGPU_HOST_DEVICE value_type operator[](int_t n) const {
    return static_cast<const outer_t&>(*this)(this->index + n);
  }
  MGPU_HOST_DEVICE value_type operator*() const { return (*this)[0]; }
};

// Accepts any store and keeps nothing (an unwanted output of a function that
// produces several).
template<typename value_type>
struct discard_iterator_t :
  iterator_t<discard_iterator_t<value_type>, int, value_type> {
  struct assign_t {
    MGPU_HOST_DEVICE value_type operator=(value_type) { return value_type(); }
  };
  MGPU_HOST_DEVICE assign_t operator[](int) const { return assign_t(); }
  MGPU_HOST_DEVICE assign_t operator*() const { return assign_t(); }
};

// it[i] is (type_t)(start + i): the item indices that
// load_balance_partitions merges with the segment starts
// (src/moderngpu/search.hxx:35).
template<typename type_t, typename int_t = int>
struct counting_iterator_t :
  const_iterator_t<counting_iterator_t<type_t>, int_t, type_t> {
  typedef const_iterator_t<counting_iterator_t<type_t>, int_t, type_t> base_t;
  counting_iterator_t() = default;
  MGPU_HOST_DEVICE counting_iterator_t(type_t start) : base_t(start) { }
  MGPU_HOST_DEVICE type_t operator()(int_t at) const { return (type_t)at; }
};

// it[i] is offset + i * stride.
template<typename type_t, typename int_t = int>
struct strided_iterator_t :
  const_iterator_t<strided_iterator_t<type_t>, int_t, int> {
  typedef const_iterator_t<strided_iterator_t<type_t>, int_t, int> base_t;
  type_t offset, stride;
  strided_iterator_t() = default;
  MGPU_HOST_DEVICE strided_iterator_t(type_t offset_, type_t stride_) :
    base_t(0), offset(offset_), stride(stride_) { }
  MGPU_HOST_DEVICE type_t operator()(int_t at) const {
    return offset + at * stride;
  }
};

// it[i] is value for every i.
template<typename type_t>
struct constant_iterator_t :
  const_iterator_t<constant_iterator_t<type_t>, int, type_t> {
  typedef const_iterator_t<constant_iterator_t<type_t>, int, type_t> base_t;
  type_t value;
  MGPU_HOST_DEVICE constant_iterator_t(type_t value_) :
    base_t(0), value(value_) { }
  MGPU_HOST_DEVICE type_t operator()(int) const { return value; }
};

////////////////////////////////////////////////////////////////////////////////
// lambda_iterator_t: it[i] calls load(i) when read and store(x, i) when
// assigned to.  Either functor may be empty_t, which makes that direction a
// compile-time error.  transform_segreduce and transform_scan feed their
// kernels through make_load_iterator (src/moderngpu/kernel_segreduce.hxx:278).

template<typename load_t, typename store_t, typename value_type, typename int_t>
struct lambda_iterator_t : iterator_types_t<value_type> {
  enum {
    can_load = !std::is_same<load_t, empty_t>::value,
    can_store = !std::is_same<store_t, empty_t>::value
  };

  load_t load;
  store_t store;
  int_t base;

  lambda_iterator_t(load_t load_, store_t store_, int_t base_) :
    load(load_), store(store_), base(base_) { }

  // What it[i] returns: reads as the value, takes an assignment.
  struct assign_t {
    load_t load;
    store_t store;
    int_t index;

    MGPU_LAMBDA operator value_type() const {
      static_assert(can_load, "store_iterator is being loaded from.");
      return load(index);
    }
    MGPU_LAMBDA assign_t& operator=(value_type x) {
      static_assert(can_store, "load_iterator is being stored to.");
      store(x, index);
      return *this;
    }
  };

  MGPU_LAMBDA assign_t operator[](int_t n) const {
    return assign_t { load, store, base + n };
  }
  MGPU_LAMBDA assign_t operator*() const { return (*this)[0]; }

  MGPU_ITERATOR_OFFSETS(lambda_iterator_t, int_t, base)
};
#undef MGPU_ITERATOR_OFFSETS

// Placeholders for a direction that is not used but must exist.
template<typename value_type>
struct trivial_load_functor {
  template<typename int_t>
  MGPU_HOST_DEVICE value_type operator()(int_t) const { return value_type(); }
};
template<typename value_type>
struct trivial_store_functor {
  template<typename int_t>
  MGPU_HOST_DEVICE void operator()(value_type, int_t) const { }
};

template<typename value_type, typename int_t = int, typename load_t,
  typename store_t>
auto make_load_store_iterator(load_t load, store_t store, int_t base = 0) {
  return lambda_iterator_t<load_t, store_t, value_type, int_t>(
    load, store, base);
}
template<typename value_type, typename int_t = int, typename load_t>
auto make_load_iterator(load_t load, int_t base = 0) {
  return lambda_iterator_t<load_t, empty_t, value_type, int_t>(
    load, empty_t(), base);
}
template<typename value_type, typename int_t = int, typename store_t>
auto make_store_iterator(store_t store, int_t base = 0) {
  return lambda_iterator_t<empty_t, store_t, value_type, int_t>(
    empty_t(), store, base);
}

END_MGPU_NAMESPACE
