// mgpu for AMD CDNA4: tuples of iterators.  The "caching iterators" argument
// of transform_lbs / lbs_segreduce / interval_* is a tuple of iterators indexed
// by segment; these helpers read or write one element of every iterator at
// once and compare tuples (names after src/moderngpu/cpp11.hxx:10-59,128-150).
#pragma once
#include "tuple.hxx"

BEGIN_MGPU_NAMESPACE

// tuple<const int*, const float*>  ->  tuple<int, float>
template<typename pointers_t>
struct tuple_iterator_value;
template<typename... its_t>
struct tuple_iterator_value<tuple<its_t...> > {
  typedef tuple<typename std::iterator_traits<its_t>::value_type...> type;
};
template<typename pointers_t>
using tuple_iterator_value_t = typename tuple_iterator_value<pointers_t>::type;

namespace detail {

template<typename... its_t, typename int_t, size_t... at>
MGPU_HOST_DEVICE tuple_iterator_value_t<tuple<its_t...> >
load_each(const tuple<its_t...>& its, int_t index, index_sequence<at...>) {
  return tuple_iterator_value_t<tuple<its_t...> >(get<at>(its)[index]...);
}

template<typename... its_t, typename int_t, size_t... at>
MGPU_HOST_DEVICE void store_each(const tuple<its_t...>& its,
  const tuple_iterator_value_t<tuple<its_t...> >& values, int_t index,
  index_sequence<at...>) {
  ((get<at>(its)[index] = get<at>(values)), ...);
}

template<typename... its_t, typename int_t, size_t... at>
MGPU_HOST_DEVICE auto refer_each(const tuple<its_t...>& its, int_t index,
  index_sequence<at...>) -> decltype(forward_as_tuple(get<at>(its)[index]...)) {
  return forward_as_tuple(get<at>(its)[index]...);
}

// Lexicographic order and equality, element by element from position `at`.
template<size_t at, typename... args_t>
MGPU_HOST_DEVICE bool tuple_less(const tuple<args_t...>& a,
  const tuple<args_t...>& b) {
  if constexpr(at == sizeof...(args_t)) return false;
  else return get<at>(a) < get<at>(b) ||
    (!(get<at>(b) < get<at>(a)) && tuple_less<at + 1>(a, b));
}
template<size_t at, typename... args_t>
MGPU_HOST_DEVICE bool tuple_equal(const tuple<args_t...>& a,
  const tuple<args_t...>& b) {
  if constexpr(at == sizeof...(args_t)) return true;
  else return get<at>(a) == get<at>(b) && tuple_equal<at + 1>(a, b);
}

} // namespace detail

// The values at `index` of every iterator, as a tuple.
template<typename int_t, typename... its_t>
MGPU_HOST_DEVICE tuple_iterator_value_t<tuple<its_t...> >
load(tuple<its_t...> its, int_t index) {
  return detail::load_each(its, index,
    make_index_sequence<sizeof...(its_t)>());
}

// its[k][index] = k-th value, for every k.
template<typename int_t, typename... its_t>
MGPU_HOST_DEVICE void store(tuple<its_t...> its,
  tuple_iterator_value_t<tuple<its_t...> > values, int_t index) {
  detail::store_each(its, values, index,
    make_index_sequence<sizeof...(its_t)>());
}

// A tuple of references to element `index` of every iterator.
template<typename int_t, typename... its_t>
MGPU_HOST_DEVICE auto dereference(tuple<its_t...> its, int_t index) ->
  decltype(detail::refer_each(its, index,
    make_index_sequence<sizeof...(its_t)>())) {
  return detail::refer_each(its, index,
    make_index_sequence<sizeof...(its_t)>());
}

// var_max<a, b, ...>::value: the largest of the arguments, 0 for none.
template<size_t... values>
struct var_max {
  constexpr static size_t value = 0;
};
template<size_t first, size_t... rest>
struct var_max<first, rest...> {
  constexpr static size_t value = first < var_max<rest...>::value ?
    var_max<rest...>::value : first;
};

// Size of the largest element type: what a union of them needs.
template<typename tpl_t>
struct tuple_union_size;
template<typename... args_t>
struct tuple_union_size<tuple<args_t...> > {
  static constexpr size_t pick(size_t a, size_t b) { return a < b ? b : a; }
  template<typename... sizes_t>
  static constexpr size_t largest(size_t first, sizes_t... rest) {
    if constexpr(0 == sizeof...(rest)) return first;
    else return pick(first, largest(rest...));
  }
  constexpr static size_t value = largest((size_t)0, sizeof(args_t)...);
};

END_MGPU_NAMESPACE

// Comparisons live in the global namespace and are found through the tuple
// arguments.
#define MGPU_TUPLE_COMPARE(op, expr)                                          \
  template<typename... args_t>                                                \
  MGPU_HOST_DEVICE bool operator op(const mgpu::tuple<args_t...>& a,          \
    const mgpu::tuple<args_t...>& b) { return expr; }
MGPU_TUPLE_COMPARE(<, mgpu::detail::tuple_less<0>(a, b))
MGPU_TUPLE_COMPARE(>, mgpu::detail::tuple_less<0>(b, a))
MGPU_TUPLE_COMPARE(<=, !mgpu::detail::tuple_less<0>(b, a))
MGPU_TUPLE_COMPARE(>=, !mgpu::detail::tuple_less<0>(a, b))
MGPU_TUPLE_COMPARE(==, mgpu::detail::tuple_equal<0>(a, b))
MGPU_TUPLE_COMPARE(!=, !mgpu::detail::tuple_equal<0>(a, b))
#undef MGPU_TUPLE_COMPARE
