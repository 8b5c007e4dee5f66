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
// CRTP bases for index-addressed iterators.  outer_t supplies
// value_type operator()(int_t index).

template<typename outer_t, typename int_t, typename value_type>
struct iterator_t : public std::iterator_traits<const value_type*> {
  int_t index;

  iterator_t() = default;
  MGPU_HOST_DEVICE iterator_t(int_t i) : index(i) { }

  MGPU_HOST_DEVICE outer_t& operator+=(int_t diff) {
    index += diff;
    return *static_cast<outer_t*>(this);
  }
  MGPU_HOST_DEVICE outer_t& operator-=(int_t diff) {
    index -= diff;
    return *static_cast<outer_t*>(this);
  }
  MGPU_HOST_DEVICE outer_t operator+(int_t diff) const {
    outer_t cp = *static_cast<const outer_t*>(this);
    cp.index += diff;
    return cp;
  }
  MGPU_HOST_DEVICE outer_t operator-(int_t diff) const {
    outer_t cp = *static_cast<const outer_t*>(this);
    cp.index -= diff;
    return cp;
  }
};

template<typename outer_t, typename int_t, typename value_type>
struct const_iterator_t : public iterator_t<outer_t, int_t, value_type> {
  typedef iterator_t<outer_t, int_t, value_type> base_t;

  const_iterator_t() = default;
  MGPU_HOST_DEVICE const_iterator_t(int_t i) : base_t(i) { }

  MGPU_HOST_DEVICE value_type operator[](int_t diff) const {
    return static_cast<const outer_t&>(*this)(base_t::index + diff);
  }
  MGPU_HOST_DEVICE value_type operator*() const {
    return (*this)[0];
  }
};

// Store iterator that drops what is written to it.
template<typename value_type>
struct discard_iterator_t :
  iterator_t<discard_iterator_t<value_type>, int, value_type> {

  struct assign_t {
    MGPU_HOST_DEVICE value_type operator=(value_type) {
      return value_type();
    }
  };
  MGPU_HOST_DEVICE assign_t operator[](int) const { return assign_t(); }
  MGPU_HOST_DEVICE assign_t operator*() const { return assign_t(); }
};

// it[i] == (type_t)(base + i).  load_balance_partitions merges this against
// the segment starts (reference search.hxx:35).
template<typename type_t, typename int_t = int>
struct counting_iterator_t :
  const_iterator_t<counting_iterator_t<type_t>, int_t, type_t> {

  counting_iterator_t() = default;
  MGPU_HOST_DEVICE counting_iterator_t(type_t i) :
    const_iterator_t<counting_iterator_t, int_t, type_t>(i) { }

  MGPU_HOST_DEVICE type_t operator()(int_t index) const {
    return (type_t)index;
  }
};

// it[i] == offset + i * stride.
template<typename type_t, typename int_t = int>
struct strided_iterator_t :
  const_iterator_t<strided_iterator_t<type_t>, int_t, int> {

  type_t offset, stride;

  strided_iterator_t() = default;
  MGPU_HOST_DEVICE strided_iterator_t(type_t offset_, type_t stride_) :
    const_iterator_t<strided_iterator_t, int_t, type_t>(0),
    offset(offset_), stride(stride_) { }

  MGPU_HOST_DEVICE type_t operator()(int_t index) const {
    return offset + index * stride;
  }
};

// it[i] == value.
template<typename type_t>
struct constant_iterator_t :
  const_iterator_t<constant_iterator_t<type_t>, int, type_t> {

  type_t value;

  MGPU_HOST_DEVICE constant_iterator_t(type_t value_) :
    const_iterator_t<constant_iterator_t, int, type_t>(0), value(value_) { }

  MGPU_HOST_DEVICE type_t operator()(int) const { return value; }
};

////////////////////////////////////////////////////////////////////////////////
// lambda_iterator_t wraps a load functor f(index)->value and/or a store
// functor g(value, index).  transform_segreduce feeds segreduce through
// make_load_iterator (reference kernel_segreduce.hxx:278).

template<typename load_t, typename store_t, typename value_type, typename int_t>
struct lambda_iterator_t : std::iterator_traits<const value_type*> {
  load_t load;
  store_t store;
  int_t base;

  lambda_iterator_t(load_t load_, store_t store_, int_t base_) :
    load(load_), store(store_), base(base_) { }

  // Proxy returned by operator[]: converts to the value (load) or accepts an
  // assignment (store).
  struct assign_t {
    load_t load;
    store_t store;
    int_t index;

    MGPU_LAMBDA assign_t& operator=(value_type rhs) {
      static_assert(!std::is_same<store_t, empty_t>::value,
        "load_iterator is being stored to.");
      store(rhs, index);
      return *this;
    }
    MGPU_LAMBDA operator value_type() const {
      static_assert(!std::is_same<load_t, empty_t>::value,
        "store_iterator is being loaded from.");
      return load(index);
    }
  };

  MGPU_LAMBDA assign_t operator[](int_t index) const {
    return assign_t { load, store, base + index };
  }
  MGPU_LAMBDA assign_t operator*() const {
    return assign_t { load, store, base };
  }

  MGPU_HOST_DEVICE lambda_iterator_t& operator+=(int_t offset) {
    base += offset;
    return *this;
  }
  MGPU_HOST_DEVICE lambda_iterator_t& operator-=(int_t offset) {
    base -= offset;
    return *this;
  }
  MGPU_HOST_DEVICE lambda_iterator_t operator+(int_t offset) const {
    lambda_iterator_t cp = *this;
    cp.base += offset;
    return cp;
  }
  MGPU_HOST_DEVICE lambda_iterator_t operator-(int_t offset) const {
    lambda_iterator_t cp = *this;
    cp.base -= offset;
    return cp;
  }
};

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
lambda_iterator_t<load_t, store_t, value_type, int_t>
make_load_store_iterator(load_t load, store_t store, int_t base = 0) {
  return lambda_iterator_t<load_t, store_t, value_type, int_t>(
    load, store, base);
}

template<typename value_type, typename int_t = int, typename load_t>
lambda_iterator_t<load_t, empty_t, value_type, int_t>
make_load_iterator(load_t load, int_t base = 0) {
  return make_load_store_iterator<value_type>(load, empty_t(), base);
}

template<typename value_type, typename int_t = int, typename store_t>
lambda_iterator_t<empty_t, store_t, value_type, int_t>
make_store_iterator(store_t store, int_t base = 0) {
  return make_load_store_iterator<value_type>(empty_t(), store, base);
}

END_MGPU_NAMESPACE
