// mgpu for AMD CDNA4: load-balancing search over device-wide inputs.
//
//   transform_lbs(f, count, segments, num_segments, [cached iterators,]
//                 context, args...)
// calls f(index, seg, rank, [tuple of cached values,] args...) once for every
// work-item index in [0, count), where seg is the last segment whose start is
// <= index and rank = index - segments[seg].  Work is cut into tiles of equal
// size in (items + segments), so the cost per CTA does not depend on how the
// segment lengths are distributed.
//
// Interface after src/moderngpu/kernel_load_balance.hxx:8-86.
#pragma once
#include "cta_load_balance.hxx"
#include "search.hxx"
#include "launcher.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

// Default tiles for the search on gfx950: 512 threads (two wavefronts per
// SIMD) x 16 items, with or without per-segment cached values.  On 2^28 items
// in 2^24 segments: the search 204 us against 216 us with 512 x 12 (fewer
// tiles, so fewer reads of a tile's segment starts in between the stores);
// interval_expand 228 against 245 us in its tile kernel.  (Tiles of 512 x 16
// begin up to 873 segments on that input; while at most 512 segments' values
// could be staged in LDS a third of the tiles fell back to gathering a value
// per item and this shape measured 322 us.)
typedef launch_box_t<arch_gfx950_cta<512, 16, 16> > lbs_launch_default_t;
typedef launch_box_t<arch_gfx950_cta<512, 16, 16> > lbs_launch_plain_t;
template<typename pointers_t>
struct lbs_launch_select_t {
  typedef typename std::conditional<0 == tuple_size<pointers_t>::value,
    lbs_launch_plain_t, lbs_launch_default_t>::type type_t;
};

// A functor may take W consecutive work-items per call instead of one:
//   typedef void chunk_functor_tag;
//   template<int W, typename value_t, typename... args_t>
//   void chunk(int index, const int (&seg)[W], const int (&rank)[W],
//     const value_t (&cached)[W], args_t...) const;
// next to the per-item operator() (still used at the ragged end of a tile).
// The library's own load_balance_search / interval_expand functors do, so
// that each lane issues 16-byte stores.
template<typename func_t, typename enable_t = void>
struct is_chunk_functor_t : std::false_type { };
template<typename func_t>
struct is_chunk_functor_t<func_t,
  typename std::conditional<false, typename func_t::chunk_functor_tag,
    void>::type> : std::true_type { };

// A functor may also ask for CTAs that decode several consecutive tiles:
//   enum { lbs_tiles_per_cta = 2 };
// Such a CTA issues the reads of every tile's segment starts and cached
// values before it works on the first tile, so that the later tiles' have
// landed when their turn comes.  That pays where a tile is nothing but its
// reads followed by a stream of stores -- interval_expand: 240 -> 228 us in
// the tile kernel on 2^28 items in 2^24 segments, the search over coarse
// splits 217 -> 201 us -- and not where the functor reads or writes scattered
// memory of its own (interval_scatter 806 -> 823 us, interval_move 643 ->
// 685 us), so the default is one tile per CTA.
template<typename func_t, typename enable_t = void>
struct lbs_tiles_per_cta_t {
  enum { value = 1 };
};
template<typename func_t>
struct lbs_tiles_per_cta_t<func_t,
  typename std::enable_if<(func_t::lbs_tiles_per_cta > 0)>::type> {
  enum { value = func_t::lbs_tiles_per_cta };
};

// own_splits: the kernel is launched without a partition array and finds the
// splits at the ends of its tiles itself (calls of few tiles, see
// transform_lbs_launch).  A separate instantiation: the search in front
// costs the kernel of large calls registers, and with them a resident CTA
// per compute unit, when it is only branched around.
template<typename launch_t, typename func_t, typename segments_it,
  typename pointers_t, typename int_t, bool own_splits = false>
struct transform_lbs_f {
  func_t f;
  int count;
  segments_it segments;
  int num_segments;
  pointers_t caching_iterators;
  const int_t* mp_data;
  int num_tiles;

  // A CTA decodes this many consecutive tiles (see lbs_tiles_per_cta_t).
  enum { tiles_per_cta = lbs_tiles_per_cta_t<func_t>::value };
  MGPU_HOST_DEVICE static int num_ctas(int num_tiles) {
    return div_up(num_tiles, (int)tiles_per_cta);
  }

  template<typename... args_t>
  MGPU_DEVICE void operator()(int tid, int cta, args_t... args) const {
    int num_groups = num_ctas(num_tiles);
    int group = xcd_tile(cta, num_groups);
    if(group >= num_groups) return;
    typedef typename launch_t::sm_ptx params_t;
    enum { nt = params_t::nt, vt = params_t::vt };
    typedef cta_load_balance_t<nt, vt> load_balance_t;
    typedef typename load_balance_t::layout_t layout_t;
    typedef cached_segment_load_t<nt, pointers_t> cached_load_t;
    typedef typename cached_load_t::value_t value_t;
    enum { W = load_balance_t::W, chunks = vt / W };

    __shared__ struct {
      typename load_balance_t::compact_storage_t lbs;
      typename cached_load_t::storage_t cached;
    } shared;

    // Tile ranges, and the reads of every tile's segment starts and cached
    // values (those of segments [b_begin - 1, b_end): each is read once and
    // fanned out through LDS when they fit), all issued before anything waits.
    // Without a partition array the CTA first finds the splits at the ends
    // of its tiles, one wavefront per split; they are not moved onto cache
    // lines of the output.
    __shared__ int own_pairs[own_splits ? 2 * (tiles_per_cta + 1) : 1];
    const int_t* pairs = own_pairs;
    if constexpr(!own_splits) pairs = mp_data + 2 * tiles_per_cta * group;
    else {
      int total = count + num_segments;
      int spacing = lbs_tile_spacing(load_balance_t::nv);
      for(int e = tid / warp_size; e <= tiles_per_cta; e += nt / warp_size) {
        int diag = (int)min((int64_t)spacing * (tiles_per_cta * group + e),
          (int64_t)total);
        int a = merge_path_wave<bounds_upper>(counting_iterator_t<int>(0),
          count, segments, num_segments, diag, less_t<int>(),
          tid % warp_size);
        if(0 == tid % warp_size) {
          own_pairs[2 * e] = a;
          own_pairs[2 * e + 1] = diag - a;
        }
      }
      __syncthreads();
    }

    merge_range_t ranges[tiles_per_cta];
    typename load_balance_t::prefetch_t ahead[tiles_per_cta];
    typename cached_load_t::fetched_t fetched[tiles_per_cta];
    bool staged[tiles_per_cta];
    PRAGMA_UNROLL
    for(int g = 0; g < tiles_per_cta; ++g) {
      int tile = tiles_per_cta * group + g;
      if(tile < num_tiles) {
        ranges[g] = paired_tile_range(count, num_segments, g,
          load_balance_t::nv, pairs);
        ahead[g] = load_balance_t::prefetch(ranges[g], segments, tid);
        staged[g] = cached_load_t::fetch(tid, ranges[g].b_begin - 1,
          ranges[g].b_count() + 1, caching_iterators, fetched[g]);
      }
    }

    PRAGMA_UNROLL
    for(int g = 0; g < tiles_per_cta; ++g) {
      if(tiles_per_cta * group + g >= num_tiles) break;
      if(g) __syncthreads();            // the previous tile is done with LDS

      // After fill_compact(), LDS slot p holds (segment of tile item p) -
      // seg_base, and tile.rank(p, that) is the item's rank in its segment.
      merge_range_t range = ranges[g];
      int a_count = range.a_count();
      int seg_base = range.b_begin - 1;
      typename load_balance_t::compact_tile_t tile =
        load_balance_t().fill_compact(range, segments, tid, shared.lbs,
          ahead[g]);
      cached_load_t::commit(tid, seg_base, range.b_count() + 1, fetched[g],
        shared.cached, caching_iterators);
      const typename load_balance_t::slot_t* slots = tile.slots;

      // The emission loop exists twice -- cached values staged in LDS, or
      // gathered from global memory -- so that each copy is straight-line code.
      auto emit_all = [&](auto staged_tag) {
        constexpr bool in_lds = decltype(staged_tag)::value;
        if constexpr(is_chunk_functor_t<func_t>::value) {
          // The functor consumes W consecutive items at a time (one 16-byte
          // store per chunk for 4-byte results).  Chunk nt * i + tid in step i:
          // consecutive lanes own consecutive chunks.
          // All LDS reads of the thread's chunks come first and none of
          // them sits behind a branch (a slot past the tile's items reads
          // something that is never used, clamped so that what is looked up
          // with it stays inside its array): the compiler issues them back
          // to back, and only the stores are conditional.
          typename load_balance_t::slot_t raw[chunks][W];
          PRAGMA_UNROLL
          for(int i = 0; i < chunks; ++i)
            lds_load_chunk<W>(slots + layout_t::index(W * (nt * i + tid)),
              raw[i]);
          int b_count = range.b_count();
          PRAGMA_UNROLL
          for(int i = 0; i < chunks; ++i) {
            int p = W * (nt * i + tid);
            int index = range.a_begin + p;
            int rel[W], seg[W], rank[W];
            value_t cached[W];
            PRAGMA_UNROLL
            for(int e = 0; e < W; ++e) {
              rel[e] = min((int)raw[i][e], b_count);
              seg[e] = seg_base + rel[e];
              rank[e] = tile.rank(p + e, rel[e]);
              if constexpr(in_lds)
                cached[e] = cached_load_t::get(true, rel[e], seg[e],
                  shared.cached, caching_iterators);
            }
            if(p + W <= a_count) {
              if constexpr(!in_lds) {
                PRAGMA_UNROLL
                for(int e = 0; e < W; ++e)
                  cached[e] = cached_load_t::get(false, rel[e], seg[e],
                    shared.cached, caching_iterators);
              }
              f.template chunk<W>(index, seg, rank, cached, args...);
            } else {
              PRAGMA_UNROLL
              for(int e = 0; e < W; ++e) {
                if(p + e < a_count)
                  f(index + e, seg[e], rank[e],
                    cached_load_t::get(in_lds, rel[e], seg[e], shared.cached,
                      caching_iterators), args...);
              }
            }
          }
        } else {
          // One item per call, item nt * i + tid in step i: whatever the
          // functor stores per item is coalesced across the wavefront.
          PRAGMA_UNROLL
          for(int i = 0; i < vt; ++i) {
            int p = nt * i + tid;
            if(p < a_count) {
              int rel = slots[layout_t::index(p)];
              int seg = seg_base + rel;
              int index = range.a_begin + p;
              f(index, seg, tile.rank(p, rel),
                cached_load_t::get(in_lds, rel, seg, shared.cached,
                  caching_iterators), args...);
            }
          }
        }
      };
      if(staged[g]) emit_all(std::true_type());
      else emit_all(std::false_type());
    }
  }
};

// The tile kernel over coarse splits (load_balance_block_partitions), for
// functors without cached values: mp_data[tile] is the block of lbs_block
// segment starts in which the tile's first split falls.  The tile reads the
// starts of its two blocks and of what lies between them and finds its exact
// (and snapped) splits itself (cta_load_balance_t::fill_blocks), so the
// partition kernel reads one start in lbs_block instead of all of them: 6
// instead of 24 us for 2^24 starts.  The starts a tile reads beyond its own
// (up to a block at either end) mostly come from the L2: the tiles next to
// it, which own them, run on the same XCD.
template<typename launch_t, typename func_t, typename segments_it,
  typename int_t>
struct transform_lbs_blocks_f {
  func_t f;
  int count;
  segments_it segments;
  int num_segments;
  const int_t* mp_data;
  int num_tiles;

  // A CTA decodes this many consecutive tiles (see lbs_tiles_per_cta_t).
  enum { tiles_per_cta = lbs_tiles_per_cta_t<func_t>::value };
  MGPU_HOST_DEVICE static int num_ctas(int num_tiles) {
    return div_up(num_tiles, (int)tiles_per_cta);
  }

  template<typename... args_t>
  MGPU_DEVICE void operator()(int tid, int cta, args_t... args) const {
    int num_groups = num_ctas(num_tiles);
    int group = xcd_tile(cta, num_groups);
    if(group >= num_groups) return;
    typedef typename launch_t::sm_ptx params_t;
    enum { nt = params_t::nt, vt = params_t::vt };
    typedef cta_load_balance_t<nt, vt> load_balance_t;
    typedef typename load_balance_t::layout_t layout_t;
    enum { W = load_balance_t::W, chunks = vt / W };
    constexpr int spacing = lbs_tile_spacing(load_balance_t::nv);
    constexpr bool snap = spacing < load_balance_t::nv;

    __shared__ typename load_balance_t::block_storage_t shared;

    // Which starts each tile has to load (its own and up to a block at either
    // end, see cta_load_balance_t::fill_blocks), with the reads issued before
    // anything waits.
    typename load_balance_t::block_tile_t ahead[tiles_per_cta];
    PRAGMA_UNROLL
    for(int g = 0; g < tiles_per_cta; ++g) {
      int tile = tiles_per_cta * group + g;
      if(tile < num_tiles)
        ahead[g] = load_balance_t::block_prefetch(count, num_segments, tile,
          spacing, mp_data, segments, tid);
    }

    PRAGMA_UNROLL
    for(int g = 0; g < tiles_per_cta; ++g) {
      if(tiles_per_cta * group + g >= num_tiles) break;
      if(g) __syncthreads();            // the previous tile is done with LDS

      // After fill_blocks(), LDS slot p holds (segment of tile item p) -
      // seg_base and starts[rel] is the start of segment seg_base + rel.
      const int* starts;
      merge_range_t range = load_balance_t::fill_blocks(ahead[g], count,
        num_segments, segments, snap, tid, shared, starts);
      int a_count = range.a_count();
      int seg_base = range.b_begin - 1;
      const int* slots = shared.indices;

      if constexpr(is_chunk_functor_t<func_t>::value) {
        // The functor consumes W consecutive items at a time (one 16-byte
        // store per chunk for 4-byte results).  Chunk nt * i + tid in step i:
        // consecutive lanes own consecutive chunks.
        PRAGMA_UNROLL
        for(int i = 0; i < chunks; ++i) {
          int p = W * (nt * i + tid);
          int index = range.a_begin + p;
          if(p + W <= a_count) {
            int rel[W], seg[W], rank[W];
            tuple<> cached[W];
            lds_load_chunk<W>(slots + layout_t::index(p), rel);
            PRAGMA_UNROLL
            for(int e = 0; e < W; ++e) {
              seg[e] = seg_base + rel[e];
              rank[e] = index + e - starts[rel[e]];
            }
            f.template chunk<W>(index, seg, rank, cached, args...);
          } else {
            PRAGMA_UNROLL
            for(int e = 0; e < W; ++e) {
              if(p + e < a_count) {
                int rel = slots[layout_t::index(p + e)];
                f(index + e, seg_base + rel, index + e - starts[rel],
                  tuple<>(), args...);
              }
            }
          }
        }
      } else {
        // One item per call, item nt * i + tid in step i: whatever the
        // functor stores per item is coalesced across the wavefront.
        PRAGMA_UNROLL
        for(int i = 0; i < vt; ++i) {
          int p = nt * i + tid;
          if(p < a_count) {
            int rel = slots[layout_t::index(p)];
            int index = range.a_begin + p;
            f(index, seg_base + rel, index - starts[rel], tuple<>(), args...);
          }
        }
      }
    }
  }
};

} // namespace detail

namespace detail {

// Which of the two tile kernels a call uses.  Without cached values the tiles
// work from coarse splits (2^28 items in 2^24 segments: 210 against 233 us
// for the call).  With cached values they keep exact splits: a tile that
// works from coarse splits can only ask for its segments' values once it has
// counted its exact splits, and its 32-bit slots and staged starts leave room
// for fewer CTAs beside the staged values, so the tile kernel loses more than
// the cheaper partition saves (interval_expand 275 against 256 us as a call,
// its tile kernel 255 against 228 us; interval_gather 615 against 557 us,
// interval_move 662 against 635 us; only inner_join's pair step, one item
// per segment, gained: 159 against 162 us).
template<typename pointers_t>
struct lbs_coarse_splits_t {
  enum { value = 0 == tuple_size<pointers_t>::value };
};

// count + num_segments as the 32-bit total the kernels index with; throws
// instead of wrapping when the sum does not fit.
inline int lbs_total(int count, int num_segments) {
  int64_t total = (int64_t)count + num_segments;
  if(count < 0 || num_segments < 0 || total >= ((int64_t)1 << 31))
    throw cuda_exception_t(hipErrorInvalidValue);
  return (int)total;
}

enum {
  lbs_phase_partition = 1, lbs_phase_tiles = 2, lbs_phase_all = 3,
  // The partition kernel runs whatever the size of the call.
  lbs_phase_partition_always = 8
};

// Ints of partition storage for `total` merged elements cut into tiles of nv:
// one (items, starts) pair per split.
MGPU_HOST_DEVICE size_t lbs_partition_ints(int total, int nv) {
  return 2 * ((size_t)div_up(total, lbs_tile_spacing(nv)) + 1);
}

// Cuts the merge of `count` items with the segment starts into tiles of at
// most nv elements and writes the splits as pairs (lbs_partition_ints ints).
// Returns the number of tiles.
template<typename segments_it>
int lbs_partition_tiles(int count, segments_it segments, int num_segments,
  int nv, int* pairs, context_t& context) {
  int spacing = lbs_tile_spacing(nv);
  // A tile too small to give up lbs_snap_slack elements is cut at every nv
  // exactly and its splits stay where they fall.
  if(spacing < nv)
    load_balance_partitions_snapped<lbs_snap_items, lbs_snap_window>(count,
      segments, num_segments, spacing, pairs, context);
  else
    load_balance_partitions_snapped<1, 1>(count, segments, num_segments,
      spacing, pairs, context);
  return div_up(lbs_total(count, num_segments), spacing);
}

// Partition + tile kernels with the partition array in caller-provided
// device memory: lbs_partition_ints(count + num_segments, nv) ints.
template<typename launch_t, typename func_t, typename segments_it,
  typename pointers_t, typename... args_t>
void transform_lbs_launch(func_t f, int count, segments_it segments,
  int num_segments, pointers_t caching_iterators, int* mp_data, int phases,
  context_t& context, args_t... args) {

  int total = lbs_total(count, num_segments);
  if(!total) return;
  int nv = launch_t::nv(context);
  int num_tiles = div_up(total, lbs_tile_spacing(nv));

  enum { own_splits_max_tiles = 1536 };
  if(num_tiles <= own_splits_max_tiles &&
    !(phases & lbs_phase_partition_always)) {
    // A call of few tiles is bound by its launches: the tile kernel finds
    // its own splits and no partition kernel runs.  load_balance_search over
    // segments of 16 items: 5.6 against 7.4 us for 2^14 items, 7.0 against
    // 8.8 us for 2^20, 12.4 against 14.0 us for 2^23 (1,096 tiles), 19.8
    // against 19.2 us for 2^24.
    if(phases & lbs_phase_tiles) {
      transform_lbs_f<launch_t, func_t, segments_it, pointers_t, int, true>
        k { f, count, segments, num_segments, caching_iterators, nullptr,
          num_tiles };
      cta_launch<launch_t>(k, xcd_grid(k.num_ctas(num_tiles)), context,
        args...);
    }
  } else if constexpr(lbs_coarse_splits_t<pointers_t>::value) {
    if(phases & lbs_phase_partition)
      load_balance_block_partitions(count, segments, num_segments,
        lbs_tile_spacing(nv), mp_data, context);
    if(phases & lbs_phase_tiles) {
      transform_lbs_blocks_f<launch_t, func_t, segments_it, int>
        k { f, count, segments, num_segments, mp_data, num_tiles };
      cta_launch<launch_t>(k, xcd_grid(k.num_ctas(num_tiles)), context,
        args...);
    }
  } else {
    if(phases & lbs_phase_partition)
      lbs_partition_tiles(count, segments, num_segments, nv, mp_data, context);
    if(phases & lbs_phase_tiles) {
      transform_lbs_f<launch_t, func_t, segments_it, pointers_t, int>
        k { f, count, segments, num_segments, caching_iterators, mp_data,
          num_tiles };
      cta_launch<launch_t>(k, xcd_grid(k.num_ctas(num_tiles)), context,
        args...);
    }
  }
}

} // namespace detail

template<typename launch_arg_t = empty_t, typename func_t,
  typename segments_it, typename pointers_t, typename... args_t>
void transform_lbs(func_t f, int count, segments_it segments,
  int num_segments, pointers_t caching_iterators, context_t& context,
  args_t... args) {

  typedef typename conditional_typedef_t<launch_arg_t,
    typename detail::lbs_launch_select_t<pointers_t>::type_t>::type_t launch_t;

  int total = detail::lbs_total(count, num_segments);
  if(!total) return;
  mem_t<int> mp(detail::lbs_partition_ints(total, launch_t::nv(context)),
    context);
  detail::transform_lbs_launch<launch_t>(f, count, segments, num_segments,
    caching_iterators, mp.data(), detail::lbs_phase_all, context, args...);
}

// Without cached values: f(index, seg, rank, args...).
template<typename launch_arg_t = empty_t, typename func_t,
  typename segments_it, typename... args_t>
void transform_lbs(func_t f, int count, segments_it segments,
  int num_segments, context_t& context, args_t... args) {

  transform_lbs<launch_arg_t>(
    [=]MGPU_DEVICE(int index, int seg, int rank, tuple<>, args_t... args) {
      f(index, seg, rank, args...);
    },
    count, segments, num_segments, tuple<>(), context, args...
  );
}

namespace detail {
// output[index] = seg, for any output iterator ...
template<typename output_it>
struct lbs_store_seg_f {
  output_it output;
  MGPU_DEVICE void operator()(int index, int seg, int, tuple<>) const {
    output[index] = seg;
  }
};
// ... and, for int pointers, W segments per 16-byte store.
template<>
struct lbs_store_seg_f<int*> {
  typedef void chunk_functor_tag;
  enum { lbs_tiles_per_cta = 2 };
  int* output;
  MGPU_DEVICE void operator()(int index, int seg, int, tuple<>) const {
    output[index] = seg;
  }
  template<int W>
  MGPU_DEVICE void chunk(int index, const int (&seg)[W], const int (&)[W],
    const tuple<> (&)[W]) const {
    store_consecutive<W>(output + index, seg);
  }
};
} // namespace detail

// output[index] = segment of work-item index.
template<typename launch_arg_t = empty_t, typename segments_it,
  typename output_it>
void load_balance_search(int count, segments_it segments,
  int num_segments, output_it output, context_t& context) {
  if(detail::launcher_load_balance_search<launch_arg_t>(count, segments,
    num_segments, output, context)) return;
  transform_lbs<launch_arg_t>(detail::lbs_store_seg_f<output_it> { output },
    count, segments, num_segments, tuple<>(), context);
}

END_MGPU_NAMESPACE
