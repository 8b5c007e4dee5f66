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
// branch-free binary search over them: a fixed number of rounds, an add, a
// compare, a select and one LDS read per round, two needles side by side.
// (A search with a bounds test per probe, or with every row of needles
// searched whether the tile has that many or not, is bound by instruction
// issue, not by memory: 239 us against 148 us for 2^26 needles in 2^26 keys.)
#pragma once
#include "search.hxx"
#include "cta_load_balance.hxx"
#include "cta_reduce.hxx"
#include "launcher.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

typedef launch_box_t<arch_gfx950_cta<256, 12, 12> >
  sorted_search_launch_default_t;

// with_counts (bounds_lower only): the kernel also writes, for every needle,
// how many haystack keys are equivalent to it -- upper bound minus lower
// bound, what a join needs -- from a second search over the same LDS keys.
// The run of equivalent keys may go on behind the tile's haystack range, so
// up to `beyond` further keys are staged with it; a needle whose run
// outlasts those too finishes its search in global memory.  When totals is
// not null the counts are also added up by blocks of totals_nv needles
// (totals[k] += the counts of needles [totals_nv k, totals_nv (k + 1)); the
// caller has zeroed them), which is what the upsweep of a scan over the
// counts would compute by reading them again.  totals_nv is at least nv, so
// a tile's needles lie in two blocks at most.
template<bounds_t bounds, typename launch_t, typename needles_it,
  typename haystack_it, typename indices_it, typename comp_t,
  bool with_counts = false>
struct sorted_search_f {
  typedef typename std::iterator_traits<needles_it>::value_type type_t;
  static_assert(!with_counts || bounds_lower == bounds,
    "match counts go with lower bounds");
  needles_it needles;
  int num_needles;
  haystack_it haystack;
  int num_haystack;
  indices_it indices;
  comp_t comp;
  const int* mp_data;
  int num_tiles;
  int* counts;
  int* totals;
  int totals_nv;

  MGPU_DEVICE void operator()(int tid, int cta) const {
    typedef typename launch_t::sm_ptx params_t;
    enum {
      nt = params_t::nt, vt = params_t::vt, nv = nt * vt,
      beyond = with_counts ? 64 : 0,
      // LDS keys: the first power of two that holds a tile (and the keys
      // staged behind it).
      room = nv + beyond,
      padded = (room & (room - 1)) ? (2 << s_log2((int)room)) : room,
      lanes = 2,                    // searches a thread runs side by side
      // keys looked at from the lower bound on for the upper bound, less one;
      // the LDS array goes on that far behind its padded size
      window = with_counts ? 8 : 0
    };
    static_assert(beyond <= nt, "one more key per thread at most");
    int tile = xcd_tile(cta, num_tiles);
    if(tile >= num_tiles) return;
    __shared__ type_t keys[padded + window];
    typedef unsigned long long pair_t;      // two 32-bit sums side by side
    typedef cta_reduce_t<nt, pair_t> reduce_t;
    __shared__ typename reduce_t::storage_t reduce_storage;

    // tile_range() keeps a tile within nv elements and inside both arrays
    // whatever the splits say.
    merge_range_t range = tile_range(num_needles, num_haystack, tile, nv,
      mp_data[tile], mp_data[tile + 1]);
    int a_count = range.a_count(), b_count = range.b_count();
    if(!a_count) return;            // b_count <= nv - 1 from here on

    // All global loads of the thread are issued before the first of them is
    // used.  Behind the staged haystack keys the LDS array repeats the last
    // of them up to its padded size: a probe past the end then answers like
    // the last key, the search needs no bounds test, and what it finds is
    // clipped to b_count afterwards.
    // staged = haystack keys in LDS: the tile's own and up to `beyond` more.
    int staged = min(b_count + (int)beyond, num_haystack - range.b_begin);
    type_t hay[vt], needle[vt], hay_beyond;
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i)
      if(nt * i + tid < b_count)
        hay[i] = haystack[range.b_begin + nt * i + tid];
    if(with_counts && b_count + tid < staged)
      hay_beyond = haystack[range.b_begin + b_count + tid];
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i)
      if(nt * i + tid < a_count)
        needle[i] = needles[range.a_begin + nt * i + tid];
    if(staged) {
      type_t filler = haystack[range.b_begin + staged - 1];
      if(with_counts && b_count + tid < staged)
        keys[b_count + tid] = hay_beyond;
      for(int j = staged + tid; j < padded + window; j += nt)
        keys[j] = filler;
    }
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i)
      if(nt * i + tid < b_count) keys[nt * i + tid] = hay[i];
    __syncthreads();

    // Needle nt * i + tid is row i.  Rows past a_count are skipped (the test
    // is the same in every thread); `lanes` rows are searched side by side.
    // at = byte offset behind the keys known to lie in front of the needle;
    // every round tries to move it on by a power of two.
    int rows = div_up(a_count, (int)nt);
    // The tile's needles from `second` on (counted from the tile's first)
    // belong to its second block of totals.
    int second = 0;
    pair_t counted = 0;
    if constexpr(with_counts)
      if(totals) second = totals_nv - range.a_begin % totals_nv;
    PRAGMA_UNROLL
    for(int i0 = 0; i0 < vt; i0 += lanes) {
      if(i0 >= rows) break;
      unsigned at[lanes];
      PRAGMA_UNROLL
      for(int l = 0; l < lanes; ++l) at[l] = 0;
      PRAGMA_UNROLL
      for(int step = padded / 2; step >= 1; step >>= 1) {
        type_t key[lanes];
        PRAGMA_UNROLL
        for(int l = 0; l < lanes; ++l)
          key[l] = *(const type_t*)((const char*)keys + at[l] +
            (step - 1) * sizeof(type_t));
        PRAGMA_UNROLL
        for(int l = 0; l < lanes; ++l) {
          const type_t& mine = needle[i0 + l < vt ? i0 + l : vt - 1];
          bool in_front = (bounds_upper == bounds) ?
            !comp(mine, key[l]) : comp(key[l], mine);
          if(in_front) at[l] += step * sizeof(type_t);
        }
      }
      // The same over "keys not behind the needle": the upper bound.  Runs
      // of equivalent keys are mostly short, so the search first looks at
      // the `window` - 1 keys from the lower bound on (three rounds for a
      // window of eight); only a needle whose run fills that window searches
      // all the keys again.
      unsigned up[lanes];
      if constexpr(with_counts) {
        PRAGMA_UNROLL
        for(int l = 0; l < lanes; ++l) up[l] = at[l];
        PRAGMA_UNROLL
        for(int step = window / 2; step >= 1; step >>= 1) {
          type_t key[lanes];
          PRAGMA_UNROLL
          for(int l = 0; l < lanes; ++l)
            key[l] = *(const type_t*)((const char*)keys + up[l] +
              (step - 1) * sizeof(type_t));
          PRAGMA_UNROLL
          for(int l = 0; l < lanes; ++l) {
            const type_t& mine = needle[i0 + l < vt ? i0 + l : vt - 1];
            if(!comp(mine, key[l])) up[l] += step * sizeof(type_t);
          }
        }
        bool longer = false;
        PRAGMA_UNROLL
        for(int l = 0; l < lanes; ++l)
          longer |= up[l] - at[l] == (window - 1) * sizeof(type_t);
        if(longer) {
          PRAGMA_UNROLL
          for(int l = 0; l < lanes; ++l) up[l] = 0;
          PRAGMA_UNROLL
          for(int step = padded / 2; step >= 1; step >>= 1) {
                type_t key[lanes];
            PRAGMA_UNROLL
            for(int l = 0; l < lanes; ++l)
              key[l] = *(const type_t*)((const char*)keys + up[l] +
                (step - 1) * sizeof(type_t));
            PRAGMA_UNROLL
            for(int l = 0; l < lanes; ++l) {
              const type_t& mine = needle[i0 + l < vt ? i0 + l : vt - 1];
              if(!comp(mine, key[l])) up[l] += step * sizeof(type_t);
            }
          }
        }
      }
      PRAGMA_UNROLL
      for(int l = 0; l < lanes; ++l) {
        int p = nt * (i0 + l) + tid;
        if(i0 + l < vt && p < a_count) {
          int lower = min((int)(at[l] / sizeof(type_t)), b_count);
          indices[range.a_begin + p] = range.b_begin + lower;
          if constexpr(with_counts) {
            int upper = range.b_begin + (int)(up[l] / sizeof(type_t));
            if(upper >= range.b_begin + staged) {
              // Every staged key is equivalent to the needle or in front of
              // it: the run ends somewhere behind them.
              const type_t& mine = needle[i0 + l < vt ? i0 + l : vt - 1];
              int lo = range.b_begin + staged, hi = num_haystack;
              while(lo < hi) {
                int mid = (int)(((unsigned)lo + (unsigned)hi) / 2);
                if(!comp(mine, haystack[mid])) lo = mid + 1;
                else hi = mid;
              }
              upper = lo;
            }
            int found = upper - (range.b_begin + lower);
            counts[range.a_begin + p] = found;
            counted += (pair_t)(unsigned)found <<
              (p >= second ? 32 : 0);
          }
        }
      }
    }
    if constexpr(with_counts) {
      if(totals) {                  // the same in all threads
        pair_t sum = reduce_t().reduce(tid, counted, reduce_storage, nt,
          plus_t<pair_t>(), false);
        if(!tid) {
          int block = range.a_begin / totals_nv;
          if((unsigned)sum) atomicAdd(totals + block, (int)(unsigned)sum);
          if(sum >> 32) atomicAdd(totals + block + 1, (int)(sum >> 32));
        }
      }
    }
  }
};

// The tile splits of a large search, found in two steps.  A scalar binary
// search per split over 2^26 + 2^26 keys is 27 dependent pairs of scattered
// reads, of which the first ten or so find their cache lines in the L2 (every
// split's search starts at the same places) and the rest do not: 48 us for
// 43,700 splits, a quarter of the whole call, with the device all but idle.
// Here every search_sample-th key of both inputs is first copied into two
// small arrays (2 x 64 K keys for 2^26: they stay in the L2), the search
// runs over those as far as they go -- needle positions g k + g - 1 pair
// with haystack positions that are multiples of g when the cross-diagonal
// is one, which the diagonals of the tiles are -- and only the last
// log2(search_sample) steps touch the inputs themselves, within one window of
// search_sample keys of each.
#ifndef MGPU_SEARCH_SAMPLE
#define MGPU_SEARCH_SAMPLE 1024
#endif
enum { search_sample = MGPU_SEARCH_SAMPLE, search_sample_min_total = 1 << 22 };

// Keys of sample storage sorted_search_launch needs (0: no sampling).
MGPU_HOST_DEVICE size_t sorted_search_sample_count(int64_t num_needles,
  int64_t num_haystack, int nv) {
  if(nv % search_sample || num_needles + num_haystack <
    search_sample_min_total) return 0;
  return (size_t)(num_needles / search_sample +
    div_up(num_haystack, (int64_t)search_sample));
}

// Also clears zero[0 .. zero_count), the totals the search kernel will add
// its counts to, which saves a launch.
template<typename needles_it, typename haystack_it, typename type_t>
struct search_sample_f {
  needles_it needles; haystack_it haystack;
  int needle_samples, num_samples;
  type_t* samples;              // needle samples, then haystack samples
  int* zero; int zero_count;
  MGPU_DEVICE void operator()(int index) const {
    enum { g = search_sample };
    if(index < zero_count) zero[index] = 0;
    if(index < num_samples)
      samples[index] = index < needle_samples ?
        (type_t)needles[g * index + g - 1] :
        (type_t)haystack[g * (index - needle_samples)];
  }
};

struct search_clear_f {
  int* zero;
  MGPU_DEVICE void operator()(int index) const { zero[index] = 0; }
};

template<bounds_t bounds, typename needles_it, typename haystack_it,
  typename type_t, typename comp_t>
struct sampled_partition_f {
  needles_it needles; haystack_it haystack;
  int num_needles, num_haystack, nv;
  comp_t comp;
  const type_t* samples;
  int needle_samples;
  int* p;

  MGPU_DEVICE bool takes_needle(const type_t& a_key,
    const type_t& b_key) const {
    return (bounds_upper == bounds) ? comp(a_key, b_key) :
      !comp(b_key, a_key);
  }

  MGPU_DEVICE void operator()(int index) const {
    enum { g = search_sample };
    int64_t total = (int64_t)num_needles + num_haystack;
    int64_t d = (int64_t)nv * index;
    int diag = (int)(d < total ? d : total);
    int begin = max(0, diag - num_haystack);
    int end = min(diag, num_needles);

    if(0 == diag % g) {
      // Needle positions g k + g - 1 inside [begin, end): k in [k0, k1).
      int k0 = begin <= g - 1 ? 0 : div_up(begin - (g - 1), (int)g);
      int k1 = end >= g ? (end - g) / g + 1 : 0;
      int lo = k0, hi = max(k0, k1);
      const type_t* hay_samples = samples + needle_samples;
      while(lo < hi) {
        int k = (int)(((unsigned)lo + (unsigned)hi) / 2);
        if(takes_needle(samples[k], hay_samples[diag / g - k - 1]))
          lo = k + 1;
        else hi = k;
      }
      // Position g (lo - 1) + g - 1 takes a needle, g lo + g - 1 does not.
      if(lo > k0) begin = max(begin, g * lo);
      if(lo < k1) end = min(end, g * lo + g - 1);
    }
    while(begin < end) {
      int mid = (int)(((unsigned)begin + (unsigned)end) / 2);
      if(takes_needle(needles[mid], haystack[diag - 1 - mid]))
        begin = mid + 1;
      else end = mid;
    }
    p[index] = begin;
  }
};

// Splits in caller-provided device memory: div_up(num_needles +
// num_haystack, nv) + 1 ints, and sorted_search_sample_count() keys (or
// null: the splits are then found by plain binary searches).
// counts: null, or (bounds_lower) where the number of haystack keys
// equivalent to each needle goes; totals: null, or div_up(num_needles,
// totals_nv) ints that receive the sums of the counts by blocks of totals_nv
// needles (totals_nv >= nv).
template<bounds_t bounds, typename launch_t, typename needles_it,
  typename haystack_it, typename indices_it, typename comp_t>
void sorted_search_launch(needles_it needles, int num_needles,
  haystack_it haystack, int num_haystack, indices_it indices, comp_t comp,
  int* mp_data,
  typename std::iterator_traits<needles_it>::value_type* samples,
  context_t& context, int* counts = nullptr, int* totals = nullptr,
  int totals_nv = 0) {
  typedef typename std::iterator_traits<needles_it>::value_type type_t;
  int64_t total = (int64_t)num_needles + num_haystack;
  if(total >= ((int64_t)1 << 31)) throw cuda_exception_t(hipErrorInvalidValue);
  if(!num_needles) return;
  int nv = launch_t::nv(context);
  int num_tiles = div_up((int)total, nv);
  size_t num_samples = sorted_search_sample_count(num_needles, num_haystack,
    nv);
  if(totals && (!counts || totals_nv < nv))
    throw cuda_exception_t(hipErrorInvalidValue);
  int num_totals = totals ? div_up(num_needles, totals_nv) : 0;
  if(samples && num_samples) {
    int needle_samples = num_needles / search_sample;
    search_sample_f<needles_it, haystack_it, type_t>
      sample { needles, haystack, needle_samples, (int)num_samples, samples,
        totals, num_totals };
    transform<256>(sample, std::max(num_samples, (size_t)num_totals),
      context);
    sampled_partition_f<bounds, needles_it, haystack_it, type_t, comp_t>
      split { needles, haystack, num_needles, num_haystack, nv, comp,
        samples, needle_samples, mp_data };
    transform<256>(split, (size_t)num_tiles + 1, context);
  } else {
    if(num_totals)
      transform<256>(search_clear_f { totals }, (size_t)num_totals, context);
    merge_path_partitions_into<bounds>(needles, (int64_t)num_needles,
      haystack, (int64_t)num_haystack, (int64_t)nv, comp, mp_data, context);
  }
  if constexpr(bounds_lower == bounds) {
    if(counts) {
      sorted_search_f<bounds, launch_t, needles_it, haystack_it, indices_it,
        comp_t, true> k { needles, num_needles, haystack, num_haystack,
          indices, comp, mp_data, num_tiles, counts, totals, totals_nv };
      cta_launch<launch_t>(k, xcd_grid(num_tiles), context);
      return;
    }
  }
  sorted_search_f<bounds, launch_t, needles_it, haystack_it, indices_it,
    comp_t> k { needles, num_needles, haystack, num_haystack, indices, comp,
      mp_data, num_tiles, nullptr, nullptr, 0 };
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
  if(detail::launcher_sorted_search<launch_arg_t>(bounds_upper == bounds,
    needles, num_needles, haystack, num_haystack, indices, comp, context))
    return;
  int64_t total = (int64_t)num_needles + num_haystack;
  typedef typename std::iterator_traits<needles_it>::value_type type_t;
  int nv = launch_t::nv(context);
  mem_t<int> partitions((size_t)div_up(total, (int64_t)nv) + 1, context);
  mem_t<type_t> samples(detail::sorted_search_sample_count(num_needles,
    num_haystack, nv), context);
  detail::sorted_search_launch<bounds, launch_t>(needles, num_needles,
    haystack, num_haystack, indices, comp, partitions.data(), samples.data(),
    context);
}

END_MGPU_NAMESPACE
