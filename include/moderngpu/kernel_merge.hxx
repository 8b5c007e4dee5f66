// mgpu for AMD CDNA4: merge of two sorted sequences, keys alone or keys with
// values (interface after src/moderngpu/kernel_merge.hxx:8-84).  Equal keys
// keep their order and those of `a` go first.
//
// Not part of the load-balancing-search / segmented-reduce path: it is here
// because it is nothing but the CTA-level blocks of cta_merge.hxx put
// together -- merge_path_partitions cuts the merge into tiles, a tile stages
// its parts of both inputs in LDS, every thread finds its cross-diagonal and
// merges vt keys, keys go out through LDS in coalesced order and values are
// gathered by the positions the keys came from.  The sorts that the CUDA
// library builds on top of it are not provided.
#pragma once
#include "cta_merge.hxx"
#include "search.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

typedef launch_box_t<arch_gfx950_cta<256, 8> > merge_launch_default_t;

template<typename launch_t, typename a_keys_it, typename a_vals_it,
  typename b_keys_it, typename b_vals_it, typename c_keys_it,
  typename c_vals_it, typename comp_t>
struct merge_tile_f {
  typedef typename std::iterator_traits<a_keys_it>::value_type key_t;
  typedef typename std::iterator_traits<a_vals_it>::value_type val_t;
  enum { has_values = !std::is_same<val_t, empty_t>::value };

  a_keys_it a_keys; a_vals_it a_vals; int a_count;
  b_keys_it b_keys; b_vals_it b_vals; int b_count;
  c_keys_it c_keys; c_vals_it c_vals;
  comp_t comp;
  const int* splits;

  MGPU_DEVICE void operator()(int tid, int cta) const {
    typedef typename launch_t::sm_ptx params_t;
    enum { nt = params_t::nt, vt = params_t::vt, nv = nt * vt };
    __shared__ union {
      key_t keys[nv + 1];
      int positions[nv];
    } shared;

    merge_range_t range = compute_merge_range(a_count, b_count, cta, nv,
      splits[cta], splits[cta + 1]);
    merge_pair_t<key_t, vt> merged = cta_merge_from_mem<bounds_lower, nt, vt>(
      a_keys, b_keys, range, tid, comp, shared.keys);

    int dest = nv * cta;
    reg_to_mem_thread<nt>(merged.keys, tid, range.total(), c_keys + dest,
      shared.keys);
    if constexpr(has_values) {
      array_t<int, vt> positions = reg_thread_to_strided<nt>(merged.indices,
        tid, shared.positions);
      transfer_two_streams_strided<nt>(a_vals + range.a_begin,
        range.a_count(), b_vals + range.b_begin, range.b_count(), positions,
        tid, c_vals + dest);
    }
  }
};

} // namespace detail

template<typename launch_arg_t = empty_t, typename a_keys_it,
  typename a_vals_it, typename b_keys_it, typename b_vals_it,
  typename c_keys_it, typename c_vals_it, typename comp_t>
void merge(a_keys_it a_keys, a_vals_it a_vals, int a_count, b_keys_it b_keys,
  b_vals_it b_vals, int b_count, c_keys_it c_keys, c_vals_it c_vals,
  comp_t comp, context_t& context) {

  typedef typename conditional_typedef_t<launch_arg_t,
    detail::merge_launch_default_t>::type_t launch_t;
  if(a_count + b_count <= 0) return;
  int nv = launch_t::nv(context);
  mem_t<int> splits = merge_path_partitions<bounds_lower>(a_keys, a_count,
    b_keys, b_count, nv, comp, context);
  detail::merge_tile_f<launch_t, a_keys_it, a_vals_it, b_keys_it, b_vals_it,
    c_keys_it, c_vals_it, comp_t> k { a_keys, a_vals, a_count, b_keys,
      b_vals, b_count, c_keys, c_vals, comp, splits.data() };
  cta_launch<launch_t>(k, div_up(a_count + b_count, nv), context);
}

// Keys only.
template<typename launch_arg_t = empty_t, typename a_keys_it,
  typename b_keys_it, typename c_keys_it, typename comp_t>
void merge(a_keys_it a_keys, int a_count, b_keys_it b_keys, int b_count,
  c_keys_it c_keys, comp_t comp, context_t& context) {
  merge<launch_arg_t>(a_keys, (const empty_t*)nullptr, a_count, b_keys,
    (const empty_t*)nullptr, b_count, c_keys, (empty_t*)nullptr, comp,
    context);
}

END_MGPU_NAMESPACE
