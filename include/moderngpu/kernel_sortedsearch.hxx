// mgpu for AMD CDNA4: vectorized sorted search.  Both inputs are sorted;
// indices[i] = lower (or upper) bound of needles[i] in the haystack.
// Interface after src/moderngpu/kernel_sortedsearch.hxx:7-73.
//
// The merge of needles and haystack is cut into tiles of nv elements with
// merge_path_partitions<bounds>.  With that tie rule (bounds_lower: a needle
// goes in front of equal haystack keys; bounds_upper: behind them) the haystack
// keys in front of a needle in merged order are exactly the keys its bound
// counts, so the bound of every needle of a tile lies inside the tile's own
// haystack range.  The reference merges the tile serially per thread to find
// it; here the tile's haystack keys are staged in LDS and every needle runs a
// branch-free binary search over them -- vt independent searches per thread,
// a fixed number of rounds, every round's LDS reads in flight together.
#pragma once
#include "search.hxx"
#include "cta_load_balance.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

typedef launch_box_t<arch_gfx950_cta<256, 12, 12> >
  sorted_search_launch_default_t;

template<bounds_t bounds, typename launch_t, typename needles_it,
  typename haystack_it, typename indices_it, typename comp_t>
struct sorted_search_f {
  typedef typename std::iterator_traits<needles_it>::value_type type_t;
  needles_it needles;
  int num_needles;
  haystack_it haystack;
  int num_haystack;
  indices_it indices;
  comp_t comp;
  const int* mp_data;
  int num_tiles;

  MGPU_DEVICE void operator()(int tid, int cta) const {
    typedef typename launch_t::sm_ptx params_t;
    enum { nt = params_t::nt, vt = params_t::vt, nv = nt * vt };
    int tile = xcd_tile(cta, num_tiles);
    if(tile >= num_tiles) return;
    __shared__ type_t keys[nv];

    // tile_range() keeps a tile within nv elements and inside both arrays
    // whatever the splits say.
    merge_range_t range = tile_range(num_needles, num_haystack, tile, nv,
      mp_data[tile], mp_data[tile + 1]);
    int a_count = range.a_count(), b_count = range.b_count();

    for(int j = tid; j < b_count; j += nt)
      keys[j] = haystack[range.b_begin + j];
    type_t needle[vt];
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i)
      if(nt * i + tid < a_count)
        needle[i] = needles[range.a_begin + nt * i + tid];
    __syncthreads();

    // found[i] = number of the tile's haystack keys that lie in front of
    // needle i.  `step` runs over the powers of two below the first one that
    // exceeds nv, so found + step never skips a key.
    int found[vt];
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i) found[i] = 0;
    PRAGMA_UNROLL
    for(int step = 1 << s_log2((int)nv); step >= 1; step >>= 1) {
      PRAGMA_UNROLL
      for(int i = 0; i < vt; ++i) {
        int probe = found[i] + step;
        if(probe <= b_count) {
          type_t key = keys[probe - 1];
          bool in_front = (bounds_upper == bounds) ?
            !comp(needle[i], key) : comp(key, needle[i]);
          if(in_front) found[i] = probe;
        }
      }
    }
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i)
      if(nt * i + tid < a_count)
        indices[range.a_begin + nt * i + tid] = range.b_begin + found[i];
  }
};

// Splits in caller-provided device memory: div_up(num_needles +
// num_haystack, nv) + 1 ints.
template<bounds_t bounds, typename launch_t, typename needles_it,
  typename haystack_it, typename indices_it, typename comp_t>
void sorted_search_launch(needles_it needles, int num_needles,
  haystack_it haystack, int num_haystack, indices_it indices, comp_t comp,
  int* mp_data, context_t& context) {
  int64_t total = (int64_t)num_needles + num_haystack;
  if(total >= ((int64_t)1 << 31)) throw cuda_exception_t(hipErrorInvalidValue);
  if(!num_needles) return;
  int nv = launch_t::nv(context);
  int num_tiles = div_up((int)total, nv);
  merge_path_partitions_into<bounds>(needles, (int64_t)num_needles, haystack,
    (int64_t)num_haystack, (int64_t)nv, comp, mp_data, context);
  sorted_search_f<bounds, launch_t, needles_it, haystack_it, indices_it,
    comp_t> k { needles, num_needles, haystack, num_haystack, indices, comp,
      mp_data, num_tiles };
  cta_launch<launch_t>(k, xcd_grid(num_tiles), context);
}

} // namespace detail

template<bounds_t bounds, typename launch_arg_t = empty_t,
  typename needles_it, typename haystack_it, typename indices_it,
  typename comp_it>
void sorted_search(needles_it needles, int num_needles, haystack_it haystack,
  int num_haystack, indices_it indices, comp_it comp, context_t& context) {
  typedef typename conditional_typedef_t<launch_arg_t,
    detail::sorted_search_launch_default_t>::type_t launch_t;
  if(num_needles <= 0) return;
  int64_t total = (int64_t)num_needles + num_haystack;
  mem_t<int> partitions((size_t)div_up(total, (int64_t)launch_t::nv(context))
    + 1, context);
  detail::sorted_search_launch<bounds, launch_t>(needles, num_needles,
    haystack, num_haystack, indices, comp, partitions.data(), context);
}

END_MGPU_NAMESPACE
