// mgpu for AMD CDNA4: a small tuple usable in device code.  transform_lbs
// exposes mgpu::tuple in its functor signature (the per-segment cached
// values), so callers need tuple / get / make_tuple / tie with the names
// moderngpu uses (src/moderngpu/tuple.hxx:85-391).
//
// Layout: tuple<A, B, C> is a value of A followed by tuple<B, C> (recursive
// aggregate), which keeps it trivially copyable for kernel arguments.  The
// empty tuple at the end takes no room (sizeof(tuple<int>) == 4, not 8): the
// kernels keep one tuple of cached values per segment in LDS.
#pragma once
#include <utility>
#include "meta.hxx"

BEGIN_MGPU_NAMESPACE

template<typename type_t>
using decay_t = typename std::decay<type_t>::type;

template<size_t... int_s>
using index_sequence = std::index_sequence<int_s...>;
template<size_t count>
using make_index_sequence = std::make_index_sequence<count>;

template<bool... args_b> struct var_and;
template<bool a, bool... b> struct var_and<a, b...> {
  enum { value = a && var_and<b...>::value };
};
template<> struct var_and<> { enum { value = true }; };

template<bool... args_b> struct var_or;
template<bool a, bool... b> struct var_or<a, b...> {
  enum { value = a || var_or<b...>::value };
};
template<> struct var_or<> { enum { value = false }; };

template<typename... args_t> struct tuple;

template<size_t i, typename tpl_t> struct tuple_element;
template<size_t i, typename arg_t, typename... args_t>
struct tuple_element<i, tuple<arg_t, args_t...> > :
  tuple_element<i - 1, tuple<args_t...> > { };
template<typename arg_t, typename... args_t>
struct tuple_element<0, tuple<arg_t, args_t...> > { typedef arg_t type; };
template<size_t i, typename tpl_t>
using tuple_element_t = typename tuple_element<i, tpl_t>::type;

template<typename tpl_t> struct tuple_size;
template<typename... args_t>
struct tuple_size<tuple<args_t...> > {
  enum { value = sizeof...(args_t) };
};
template<typename tpl_t>
struct tuple_size<const tpl_t> : tuple_size<tpl_t> { };
template<typename tpl_t>
struct tuple_size<tpl_t&> : tuple_size<tpl_t> { };

template<> struct tuple<> {
  MGPU_HOST_DEVICE tuple() { }
  template<typename... other_t>
  MGPU_HOST_DEVICE tuple(const tuple<other_t...>&) { }
};

template<typename arg_t, typename... args_t>
struct tuple<arg_t, args_t...> {
  typedef tuple<args_t...> tail_t;
  arg_t head;
#if defined(__clang__)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wc++20-extensions"
#endif
  [[no_unique_address]] tail_t tail;
#if defined(__clang__)
#pragma clang diagnostic pop
#endif

  tuple() = default;
  tuple(const tuple&) = default;

  MGPU_HOST_DEVICE tuple(arg_t head_, args_t... tail_) :
    head(static_cast<arg_t&&>(head_)),
    tail(static_cast<args_t&&>(tail_)...) { }

  // Converting copy, e.g. tuple<int&, float&> -> tuple<int, float>.
  template<typename arg2_t, typename... args2_t,
    typename = enable_if_t<sizeof...(args2_t) == sizeof...(args_t)> >
  MGPU_HOST_DEVICE tuple(const tuple<arg2_t, args2_t...>& rhs) :
    head(rhs.head), tail(rhs.tail) { }

  MGPU_HOST_DEVICE tuple& operator=(const tuple& rhs) {
    head = rhs.head;
    tail = rhs.tail;
    return *this;
  }
  template<typename arg2_t, typename... args2_t,
    typename = enable_if_t<sizeof...(args2_t) == sizeof...(args_t)> >
  MGPU_HOST_DEVICE tuple& operator=(const tuple<arg2_t, args2_t...>& rhs) {
    head = rhs.head;
    tail = rhs.tail;
    return *this;
  }
};

namespace detail {
template<size_t i>
struct tuple_get_t {
  template<typename tpl_t>
  MGPU_HOST_DEVICE static auto get(tpl_t& t) ->
    decltype(tuple_get_t<i - 1>::get(t.tail)) {
    return tuple_get_t<i - 1>::get(t.tail);
  }
};
template<>
struct tuple_get_t<0> {
  template<typename tpl_t>
  MGPU_HOST_DEVICE static auto get(tpl_t& t) -> decltype((t.head)) {
    return t.head;
  }
};
} // namespace detail

template<size_t i, typename... args_t>
MGPU_HOST_DEVICE tuple_element_t<i, tuple<args_t...> >&
get(tuple<args_t...>& t) {
  return detail::tuple_get_t<i>::get(t);
}
template<size_t i, typename... args_t>
MGPU_HOST_DEVICE const tuple_element_t<i, tuple<args_t...> >&
get(const tuple<args_t...>& t) {
  return detail::tuple_get_t<i>::get(t);
}
template<size_t i, typename... args_t>
MGPU_HOST_DEVICE tuple_element_t<i, tuple<args_t...> >&&
get(tuple<args_t...>&& t) {
  return static_cast<tuple_element_t<i, tuple<args_t...> >&&>(
    detail::tuple_get_t<i>::get(t));
}

template<typename... args_t>
MGPU_HOST_DEVICE tuple<decay_t<args_t>...> make_tuple(args_t&&... args) {
  return tuple<decay_t<args_t>...>(std::forward<args_t>(args)...);
}

template<typename... args_t>
MGPU_HOST_DEVICE tuple<args_t&&...> forward_as_tuple(args_t&&... args) {
  return tuple<args_t&&...>(std::forward<args_t>(args)...);
}

template<typename... args_t>
MGPU_HOST_DEVICE tuple<args_t&...> tie(args_t&... args) {
  return tuple<args_t&...>(args...);
}

namespace detail {
template<typename tpl1_t, typename tpl2_t> struct tuple_cat_type;
template<typename... a_t, typename... b_t>
struct tuple_cat_type<tuple<a_t...>, tuple<b_t...> > {
  typedef tuple<a_t..., b_t...> type;
};
template<typename... a_t, typename... b_t, size_t... ai, size_t... bi>
MGPU_HOST_DEVICE tuple<a_t..., b_t...> tuple_cat2(const tuple<a_t...>& a,
  const tuple<b_t...>& b, index_sequence<ai...>, index_sequence<bi...>) {
  return tuple<a_t..., b_t...>(get<ai>(a)..., get<bi>(b)...);
}
} // namespace detail

template<typename... a_t>
MGPU_HOST_DEVICE tuple<a_t...> tuple_cat(const tuple<a_t...>& a) { return a; }

template<typename... a_t, typename... b_t>
MGPU_HOST_DEVICE tuple<a_t..., b_t...> tuple_cat(const tuple<a_t...>& a,
  const tuple<b_t...>& b) {
  return detail::tuple_cat2(a, b, make_index_sequence<sizeof...(a_t)>(),
    make_index_sequence<sizeof...(b_t)>());
}

template<typename... a_t, typename... b_t, typename c_t, typename... rest_t>
MGPU_HOST_DEVICE auto tuple_cat(const tuple<a_t...>& a,
  const tuple<b_t...>& b, const c_t& c, const rest_t&... rest) ->
  decltype(tuple_cat(tuple_cat(a, b), c, rest...)) {
  return tuple_cat(tuple_cat(a, b), c, rest...);
}

END_MGPU_NAMESPACE
