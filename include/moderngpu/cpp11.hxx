// mgpu for AMD CDNA4: helpers over tuples of iterators -- the "caching
// iterators" argument of transform_lbs is a tuple of pointers whose values are
// loaded once per segment (API after src/moderngpu/cpp11.hxx:10-59,128-150).
#pragma once
#include "tuple.hxx"

BEGIN_MGPU_NAMESPACE

// tuple<const int*, const float*>  ->  tuple<int, float>
template<typename tpl_t>
struct tuple_iterator_value;

template<typename... args_t>
struct tuple_iterator_value<tuple<args_t...> > {
  typedef tuple<typename std::iterator_traits<args_t>::value_type...> type;
};

template<typename tpl_t>
using tuple_iterator_value_t = typename tuple_iterator_value<tpl_t>::type;

namespace detail {

template<typename int_t, typename... pointers_t, size_t... seq_i>
MGPU_HOST_DEVICE auto deref_all(tuple<pointers_t...> pointers,
  index_sequence<seq_i...>, int_t index) ->
  decltype(forward_as_tuple(get<seq_i>(pointers)[0]...)) {
  return forward_as_tuple(get<seq_i>(pointers)[index]...);
}

template<typename int_t, typename... pointers_t, size_t... seq_i>
MGPU_HOST_DEVICE tuple_iterator_value_t<tuple<pointers_t...> >
load_all(tuple<pointers_t...> pointers, index_sequence<seq_i...>,
  int_t index) {
  typedef tuple_iterator_value_t<tuple<pointers_t...> > value_t;
  return value_t(get<seq_i>(pointers)[index]...);
}

template<typename int_t, typename... pointers_t, size_t... seq_i>
MGPU_HOST_DEVICE void store_all(tuple<pointers_t...> pointers,
  const tuple_iterator_value_t<tuple<pointers_t...> >& values,
  index_sequence<seq_i...>, int_t index) {
  swallow((get<seq_i>(pointers)[index] = get<seq_i>(values), 0)...);
}

} // namespace detail

// Tuple of lvalue references to element `index` of every pointer.
template<typename int_t, typename... pointers_t>
MGPU_HOST_DEVICE auto dereference(tuple<pointers_t...> pointers,
  int_t index) -> decltype(detail::deref_all(pointers,
    make_index_sequence<sizeof...(pointers_t)>(), index)) {
  return detail::deref_all(pointers,
    make_index_sequence<sizeof...(pointers_t)>(), index);
}

template<typename int_t, typename... pointers_t>
MGPU_HOST_DEVICE tuple_iterator_value_t<tuple<pointers_t...> >
load(tuple<pointers_t...> pointers, int_t index) {
  return detail::load_all(pointers,
    make_index_sequence<sizeof...(pointers_t)>(), index);
}

template<typename int_t, typename... pointers_t>
MGPU_HOST_DEVICE void store(tuple<pointers_t...> pointers,
  tuple_iterator_value_t<tuple<pointers_t...> > values, int_t index) {
  detail::store_all(pointers, values,
    make_index_sequence<sizeof...(pointers_t)>(), index);
}

namespace detail {
template<size_t i, size_t count>
struct tuple_compare_t {
  template<typename tpl_t>
  MGPU_HOST_DEVICE static bool eq(const tpl_t& a, const tpl_t& b) {
    return get<i>(a) == get<i>(b) && tuple_compare_t<i + 1, count>::eq(a, b);
  }
  template<typename tpl_t>
  MGPU_HOST_DEVICE static bool less(const tpl_t& a, const tpl_t& b) {
    if(get<i>(a) < get<i>(b)) return true;
    if(get<i>(b) < get<i>(a)) return false;
    return tuple_compare_t<i + 1, count>::less(a, b);
  }
};
template<size_t count>
struct tuple_compare_t<count, count> {
  template<typename tpl_t>
  MGPU_HOST_DEVICE static bool eq(const tpl_t&, const tpl_t&) { return true; }
  template<typename tpl_t>
  MGPU_HOST_DEVICE static bool less(const tpl_t&, const tpl_t&) {
    return false;
  }
};
} // namespace detail

template<size_t... values> struct var_max;
template<size_t v, size_t... rest>
struct var_max<v, rest...> {
  constexpr static size_t value =
    v > var_max<rest...>::value ? v : var_max<rest...>::value;
};
template<> struct var_max<> { constexpr static size_t value = 0; };

template<typename tpl_t> struct tuple_union_size;
template<typename... args_t>
struct tuple_union_size<tuple<args_t...> > {
  constexpr static size_t value = var_max<sizeof(args_t)...>::value;
};

END_MGPU_NAMESPACE

// Lexicographic comparison, visible through argument-dependent lookup.
template<typename... args_t>
MGPU_HOST_DEVICE bool operator<(const mgpu::tuple<args_t...>& a,
  const mgpu::tuple<args_t...>& b) {
  return mgpu::detail::tuple_compare_t<0, sizeof...(args_t)>::less(a, b);
}
template<typename... args_t>
MGPU_HOST_DEVICE bool operator>(const mgpu::tuple<args_t...>& a,
  const mgpu::tuple<args_t...>& b) { return b < a; }
template<typename... args_t>
MGPU_HOST_DEVICE bool operator<=(const mgpu::tuple<args_t...>& a,
  const mgpu::tuple<args_t...>& b) { return !(b < a); }
template<typename... args_t>
MGPU_HOST_DEVICE bool operator>=(const mgpu::tuple<args_t...>& a,
  const mgpu::tuple<args_t...>& b) { return !(a < b); }
template<typename... args_t>
MGPU_HOST_DEVICE bool operator==(const mgpu::tuple<args_t...>& a,
  const mgpu::tuple<args_t...>& b) {
  return mgpu::detail::tuple_compare_t<0, sizeof...(args_t)>::eq(a, b);
}
template<typename... args_t>
MGPU_HOST_DEVICE bool operator!=(const mgpu::tuple<args_t...>& a,
  const mgpu::tuple<args_t...>& b) { return !(a == b); }
