// mgpu for AMD CDNA4: dynamic work creation on top of the load-balancing
// search.  Every work-item of a segmented workload may create a segment of
// new work-items for the next pass (a vertex reached by a frontier edge
// creates one work-item per outgoing edge, say):
//
//   auto engine = expt::lbs_workcreate(count, segments, num_segments, context);
//   auto sizes = engine.upsweep(f, cached);    f(index, seg, rank, tuple)
//   mem_t<int> next = engine.downsweep(g, cached, args...);
//                                    g(dest_seg, index, seg, rank, tuple, args...)
//
// upsweep calls f once per work-item; an item that returns n > 0 creates a
// segment of n new work-items.  It returns how many segments and work-items
// the next pass has, so the caller can allocate per-segment outputs.
// downsweep calls g once per creating item, in item order, with the number of
// the segment it creates; g returns the same count f did and may store
// whatever describes the new segment.  The result holds the start offsets of
// the new segments.  Interface after
// src/moderngpu/kernel_workcreate.hxx:14-268.
//
// Both sweeps decode the same tiles (the engine owns the partition).  Between
// them a thread keeps one bit per item it looked at.  The downsweep finds the
// position of a creating item among the tile's creating items from wavefront
// ballots -- in a row of nt consecutive items each wavefront owns 64
// consecutive ones, so popcounts per (row, wavefront), scanned over the tile,
// plus the popcount of the lower lanes give it -- and gathers the creating
// items in that order, so the calls run with all lanes busy and what they
// store per new segment is contiguous.  The start offsets come from the same
// table scheme over wave-level prefix sums of the counts.
#pragma once

#include "kernel_load_balance.hxx"
#include "kernel_scan.hxx"
#include "cta_reduce.hxx"

BEGIN_MGPU_NAMESPACE

namespace expt {

namespace detail {

using namespace mgpu::detail;

// 256 threads x 12 items: the callbacks gather from global memory, so more
// resident CTAs per CU matter more here than the longest possible tile.
typedef launch_box_t<arch_gfx950_cta<256, 12, 12> > workcreate_launch_default_t;

// An upsweep functor that looks at nothing but the item's index may say so:
//   typedef void index_only_tag;
// Its tiles are then not decoded in the upsweep (segment, rank and cached
// values of its calls are meaningless): 2^26 items 67 -> 62 us.
template<typename func_t, typename enable_t = void>
struct is_index_only_t : std::false_type { };
template<typename func_t>
struct is_index_only_t<func_t,
  typename std::conditional<false, typename func_t::index_only_tag,
    void>::type> : std::true_type { };

template<typename arg_t>
struct is_tuple_t : std::false_type { };
template<typename... args_t>
struct is_tuple_t<tuple<args_t...> > : std::true_type { };

// Totals of a tile, and after the scan its offsets, as one 64-bit sum:
// creating items in the low word, created work-items in the high word.
// Neither total reaches 2^31, so the low word never carries into the high.
typedef unsigned long long tile_total_t;
MGPU_HOST_DEVICE tile_total_t pack_total(int creators, int work) {
  return (tile_total_t)(unsigned)work << 32 | (unsigned)creators;
}
MGPU_HOST_DEVICE int total_creators(tile_total_t x) {
  return (int)(unsigned)x;
}
MGPU_HOST_DEVICE int total_work(tile_total_t x) { return (int)(x >> 32); }

// What the two kernels share: tile decode and per-item (seg, rank, cached).
template<typename launch_t, typename segments_it, typename pointers_t>
struct workcreate_tile_t {
  typedef typename launch_t::sm_ptx params_t;
  enum {
    nt = params_t::nt, vt = params_t::vt, num_waves = nt / warp_size,
    table_size = vt * num_waves
  };
  static_assert(0 == nt % warp_size, "whole wavefronts only");
  static_assert(vt <= 32, "one bit per item in a 32-bit word");
  static_assert(table_size <= nt, "the per-row table is scanned by one CTA scan");

  typedef cta_load_balance_t<nt, vt> load_balance_t;
  typedef typename load_balance_t::layout_t layout_t;
  typedef cached_segment_load_t<nt, pointers_t> cached_load_t;
  typedef typename cached_load_t::value_t value_t;
  typedef cta_scan_t<nt, int> scan_t;
  typedef cta_reduce_t<nt, tile_total_t> reduce_t;
  typedef typename std::conditional<(nt * vt <= 65536), unsigned short,
    int>::type target_t;

  struct storage_t {
    typename load_balance_t::storage_t lbs;
    typename cached_load_t::storage_t cached;
    union {
      typename scan_t::storage_t scan;
      typename reduce_t::storage_t reduce;
    };
    int table[table_size];
    MGPU_DEVICE storage_t() { }
  };

  int count;
  segments_it segments;
  int num_segments;
  pointers_t caching_iterators;
  const int* pairs;
  int num_tiles;

  struct decoded_t {
    merge_range_t range;
    bool staged;
  };
  MGPU_DEVICE decoded_t decode(int tid, int tile, storage_t& shared) const {
    merge_range_t range = paired_tile_range(count, num_segments, tile,
      load_balance_t::nv, pairs);
    // The reads of the tile's starts and cached values are issued before
    // anything waits and land while the tile is decoded.
    typename load_balance_t::prefetch_t ahead =
      load_balance_t::prefetch(range, segments, tid);
    typename cached_load_t::fetched_t fetched;
    bool staged = cached_load_t::fetch(tid, range.b_begin - 1,
      range.b_count() + 1, caching_iterators, fetched);
    load_balance_t().fill(range, segments, tid, shared.lbs, ahead);
    cached_load_t::commit(tid, range.b_begin - 1, range.b_count() + 1,
      fetched, shared.cached, caching_iterators);
    return decoded_t { range, staged };
  }

  // Segment, rank and cached values of the thread's items, item nt * i + tid
  // in position i.  Every LDS read is issued for every position, wanted or
  // not, so that none of them waits behind a branch; a position outside
  // `wanted` (bit i) gets the tile's first segment and values that mean
  // nothing.  Cached values that are not staged in LDS are gathered from
  // global memory for the wanted positions only.
  struct items_t {
    int seg[vt];
    int rank[vt];
    value_t cached[vt];
  };
  MGPU_DEVICE void items(int tid, const decoded_t& tile,
    const storage_t& shared, unsigned wanted, items_t& x) const {
    int a_count = tile.range.a_count();
    int seg_base = tile.range.b_begin - 1;
    const int* slots = shared.lbs.indices;
    const int* starts = slots + load_balance_t::starts_offset(a_count);
    int rel[vt];
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i) {
      int p = nt * i + tid;
      rel[i] = slots[layout_t::index(min(p, nt * vt - 1))];
      if(p >= a_count) rel[i] = 0;
    }
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i) {
      x.seg[i] = seg_base + rel[i];
      x.rank[i] = tile.range.a_begin + nt * i + tid - starts[rel[i]];
    }
    if(tile.staged) {
      PRAGMA_UNROLL
      for(int i = 0; i < vt; ++i)
        x.cached[i] = cached_load_t::get(true, rel[i], x.seg[i],
          shared.cached, caching_iterators);
    } else {
      PRAGMA_UNROLL
      for(int i = 0; i < vt; ++i)
        if(wanted & (1u << i))
          x.cached[i] = cached_load_t::get(false, rel[i], x.seg[i],
            shared.cached, caching_iterators);
    }
  }

  // The same for the one item at tile position p < a_count:
  // call(index, seg, rank, cached).
  template<typename call_t>
  MGPU_DEVICE void item(int p, const decoded_t& tile,
    const storage_t& shared, call_t call) const {
    const int* slots = shared.lbs.indices;
    const int* starts = slots +
      load_balance_t::starts_offset(tile.range.a_count());
    int rel = slots[layout_t::index(p)];
    int seg = tile.range.b_begin - 1 + rel;
    int index = tile.range.a_begin + p;
    call(index, seg, index - starts[rel], cached_load_t::get(tile.staged,
      rel, seg, shared.cached, caching_iterators));
  }

  // Exclusive scan of table[0 .. table_size) in place; entry
  // num_waves * i + wave belongs to row i of wavefront `wave`, so the scan
  // runs in item order.  Returns the total.
  MGPU_DEVICE int scan_table(int tid, storage_t& shared) const {
    __syncthreads();
    int x = tid < table_size ? shared.table[tid] : 0;
    scan_result_t<int> result = scan_t().scan(tid, x, shared.scan);
    if(tid < table_size) shared.table[tid] = result.scan;
    __syncthreads();
    return result.reduction;
  }
};

template<typename launch_t, typename func_t, typename segments_it,
  typename pointers_t>
struct workcreate_upsweep_f {
  typedef workcreate_tile_t<launch_t, segments_it, pointers_t> tile_t;
  typedef typename tile_t::value_t value_t;
  enum { nt = tile_t::nt, vt = tile_t::vt };

  tile_t tiles;
  func_t f;
  unsigned* bits_data;            // nt words per tile
  tile_total_t* totals_data;      // one per tile

  MGPU_DEVICE void operator()(int tid, int cta) const {
    int tile = xcd_tile(cta, tiles.num_tiles);
    if(tile >= tiles.num_tiles) return;
    __shared__ typename tile_t::storage_t shared;
    typename tile_t::decoded_t decoded;
    if constexpr(is_index_only_t<func_t>::value)
      decoded.range = paired_tile_range(tiles.count, tiles.num_segments, tile,
        tile_t::load_balance_t::nv, tiles.pairs);
    else
      decoded = tiles.decode(tid, tile, shared);

    // Bit i: item nt * i + tid exists.
    int a_count = decoded.range.a_count();
    unsigned valid = 0;
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i)
      valid |= (unsigned)(nt * i + tid < a_count) << i;
    typename tile_t::items_t x;
    if constexpr(is_index_only_t<func_t>::value) {
      PRAGMA_UNROLL
      for(int i = 0; i < vt; ++i) {
        x.seg[i] = 0; x.rank[i] = 0; x.cached[i] = value_t();
      }
    } else
      tiles.items(tid, decoded, shared, valid, x);

    // All calls first, their results -- which usually come from memory --
    // are only looked at afterwards, so the loads of all calls overlap.
    int created[vt];
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i) {
      created[i] = 0;
      if(valid & (1u << i))
        created[i] = f(decoded.range.a_begin + nt * i + tid, x.seg[i],
          x.rank[i], x.cached[i]);
    }
    unsigned bits = 0;
    int work = 0;
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i) {
      if(created[i] > 0) {
        bits |= 1u << i;
        work += created[i];
      }
    }
    bits_data[nt * tile + tid] = bits;

    tile_total_t total = typename tile_t::reduce_t().reduce(tid,
      pack_total(popc(bits), work), shared.reduce, nt,
      plus_t<tile_total_t>(), false);
    if(!tid) totals_data[tile] = total;
  }
};

template<typename launch_t, typename func_t, typename segments_it,
  typename pointers_t>
struct workcreate_downsweep_f {
  typedef workcreate_tile_t<launch_t, segments_it, pointers_t> tile_t;
  typedef typename tile_t::value_t value_t;
  enum { nt = tile_t::nt, vt = tile_t::vt, num_waves = tile_t::num_waves };

  tile_t tiles;
  func_t f;
  const unsigned* bits_data;
  const tile_total_t* offsets_data;   // exclusive scan of the tile totals
  int* segments_output;

  template<typename... args_t>
  MGPU_DEVICE void operator()(int tid, int cta, args_t... args) const {
    int tile = xcd_tile(cta, tiles.num_tiles);
    if(tile >= tiles.num_tiles) return;
    __shared__ typename tile_t::storage_t shared;
    // Tile positions of the creating items, in item order.
    __shared__ typename tile_t::target_t targets[nt * vt];

    int lane = tid % warp_size, wave = tid / warp_size;
    unsigned bits = bits_data[nt * tile + tid];
    tile_total_t offset = offsets_data[tile];

    // Position of every creating item among the tile's creating items; the
    // items are gathered in that order into targets.
    int below[vt];
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i) {
      lanemask_t creators = ballot(0 != (bits & (1u << i)));
      below[i] = popc(creators & lanemask_lt(lane));
      if(!lane) shared.table[num_waves * i + wave] = popc(creators);
    }
    int num_creators = tiles.scan_table(tid, shared);
    // Tiles without a creating item have nothing to do.  (The branch is
    // uniform: every thread has the same num_creators.)
    if(!num_creators) return;
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i) {
      if(bits & (1u << i))
        targets[shared.table[num_waves * i + wave] + below[i]] =
          (typename tile_t::target_t)(nt * i + tid);
    }
    // (decode() has barriers of its own before anything reads the targets.)
    typename tile_t::decoded_t decoded = tiles.decode(tid, tile, shared);

    // Creating item nt * r + tid in round r: every lane of a round has work,
    // and what the callback stores under dest_seg is contiguous across the
    // CTA.  What the calls return is only looked at after the last call.
    int rounds = div_up(num_creators, (int)nt);
    int dest_base = total_creators(offset);
    int created[vt];
    PRAGMA_UNROLL
    for(int r = 0; r < vt; ++r) {
      created[r] = 0;
      int j = nt * r + tid;
      if(r < rounds && j < num_creators)
        tiles.item(targets[j], decoded, shared,
          [&](int index, int seg, int rank, value_t cached) {
            created[r] = f(dest_base + j, index, seg, rank, cached, args...);
          });
    }

    // Start of every new segment: work-items created in front of it.
    int before[vt];
    PRAGMA_UNROLL
    for(int r = 0; r < vt; ++r) {
      if(r < rounds) {
        created[r] = max(created[r], 0);
        int inclusive = wave_scan(created[r], plus_t<int>(), lane);
        before[r] = inclusive - created[r];
        if(warp_size - 1 == lane)
          shared.table[num_waves * r + wave] = inclusive;
      } else if(warp_size - 1 == lane)
        shared.table[num_waves * r + wave] = 0;
    }
    tiles.scan_table(tid, shared);
    PRAGMA_UNROLL
    for(int r = 0; r < vt; ++r) {
      int j = nt * r + tid;
      if(r < rounds && j < num_creators)
        segments_output[dest_base + j] = total_work(offset) +
          shared.table[num_waves * r + wave] + before[r];
    }
  }
};

// The two kernels over caller-provided arrays: pairs = splits from
// lbs_partition_tiles, bits = nt words per tile, totals / offsets = one
// tile_total_t per tile (offsets is the exclusive scan of totals).
template<typename launch_t, typename func_t, typename segments_it,
  typename pointers_t>
void workcreate_upsweep_launch(func_t f, pointers_t caching_iterators,
  int count, segments_it segments, int num_segments, const int* pairs,
  int num_tiles, unsigned* bits, tile_total_t* totals, context_t& context) {
  typedef workcreate_tile_t<launch_t, segments_it, pointers_t> tile_t;
  workcreate_upsweep_f<launch_t, func_t, segments_it, pointers_t> k {
    tile_t { count, segments, num_segments, caching_iterators, pairs,
      num_tiles }, f, bits, totals };
  cta_launch<launch_t>(k, xcd_grid(num_tiles), context);
}

template<typename launch_t, typename func_t, typename segments_it,
  typename pointers_t, typename... args_t>
void workcreate_downsweep_launch(func_t f, pointers_t caching_iterators,
  int count, segments_it segments, int num_segments, const int* pairs,
  int num_tiles, const unsigned* bits, const tile_total_t* offsets,
  int* segments_output, context_t& context, args_t... args) {
  typedef workcreate_tile_t<launch_t, segments_it, pointers_t> tile_t;
  workcreate_downsweep_f<launch_t, func_t, segments_it, pointers_t> k {
    tile_t { count, segments, num_segments, caching_iterators, pairs,
      num_tiles }, f, bits, offsets, segments_output };
  cta_launch<launch_t>(k, xcd_grid(num_tiles), context, args...);
}

} // namespace detail

template<typename launch_arg_t, typename segments_it>
struct workcreate_t {
  typedef typename conditional_typedef_t<launch_arg_t,
    detail::workcreate_launch_default_t>::type_t launch_t;
  typedef detail::tile_total_t tile_total_t;

  int count;
  segments_it segments;
  int num_segments;
  context_t& context;

  cta_dim_t cta_dim;
  int num_tiles;

  mem_t<int> pairs;               // splits, (items, starts) per tile end
  mem_t<unsigned> bits;           // per thread and tile: who creates work
  mem_t<tile_total_t> offsets;    // per tile: creators and work in front
  tile_total_t total;

  // Sizes of the next pass.
  struct count_t {
    int count;                    // work-items created
    int num_segments;             // items that created any
  };

  workcreate_t(int count_, segments_it segments_, int num_segments_,
    context_t& context_) : count(count_), segments(segments_),
    num_segments(num_segments_), context(context_), total(0) {

    cta_dim = launch_t::cta_dim(context);
    int nv = cta_dim.nv();
    int64_t merged = (int64_t)count + num_segments;
    if(count < 0 || num_segments < 0 || merged >= ((int64_t)1 << 31))
      throw cuda_exception_t(hipErrorInvalidValue);
    num_tiles = 0;
    if(!merged) return;

    pairs = mem_t<int>(mgpu::detail::lbs_partition_ints((int)merged, nv),
      context);
    num_tiles = mgpu::detail::lbs_partition_tiles(count, segments,
      num_segments, nv, pairs.data(), context);
    bits = mem_t<unsigned>((size_t)num_tiles * cta_dim.nt, context);
    offsets = mem_t<tile_total_t>(num_tiles, context);
  }

  // f(int index, int seg, int rank, tuple<...> cached) returns the number of
  // work-items the item creates; zero or less creates nothing.  Waits for
  // the device: the totals come back to the host.
  template<typename func_t, typename pointers_t>
  count_t upsweep(func_t f, pointers_t caching_iterators) {
    if(!num_tiles) return count_t { 0, 0 };

    mem_t<tile_total_t> totals(num_tiles, context);
    detail::workcreate_upsweep_launch<launch_t>(f, caching_iterators, count,
      segments, num_segments, pairs.data(), num_tiles, bits.data(),
      totals.data(), context);

    // Offsets of every tile; the grand total goes to pinned host memory and
    // is there once the event has passed.
    mem_t<tile_total_t> total_host(1, context, memory_space_host);
    scan_event(totals.data(), num_tiles, offsets.data(),
      plus_t<tile_total_t>(), total_host.data(), context, context.event());
    hipError_t status = hipEventSynchronize(context.event());
    if(hipSuccess != status) throw cuda_exception_t(status);

    total = total_host.data()[0];
    return count_t { detail::total_work(total),
      detail::total_creators(total) };
  }

  // f(int index, int seg, int rank).
  template<typename func_t>
  count_t upsweep(func_t f) {
    return upsweep([=]MGPU_DEVICE(int index, int seg, int rank, tuple<>) {
      return f(index, seg, rank);
    }, tuple<>());
  }

  // f(int dest_seg, int index, int seg, int rank, tuple<...> cached, args...)
  // for every item that created work in the upsweep; dest_seg counts those
  // items in item order.  f returns the count it returned in the upsweep.
  // The result has one start offset per new segment.
  template<typename func_t, typename pointers_t, typename... args_t,
    typename = enable_if_t<detail::is_tuple_t<pointers_t>::value> >
  mem_t<int> downsweep(func_t f, pointers_t caching_iterators,
    args_t... args) {
    int num_dest_segments = detail::total_creators(total);
    mem_t<int> result(num_dest_segments, context);
    if(!num_tiles || !num_dest_segments) return result;

    detail::workcreate_downsweep_launch<launch_t>(f, caching_iterators,
      count, segments, num_segments, pairs.data(), num_tiles, bits.data(),
      offsets.data(), result.data(), context, args...);
    return result;
  }

  // f(int dest_seg, int index, int seg, int rank, args...).
  template<typename func_t, typename... args_t>
  mem_t<int> downsweep(func_t f, args_t... args) {
    return downsweep(
      [=]MGPU_DEVICE(int dest_seg, int index, int seg, int rank, tuple<>,
        args_t... args) {
        return f(dest_seg, index, seg, rank, args...);
      }, tuple<>(), args...);
  }
};

// One engine per pass: construct it, call upsweep, then downsweep.
template<typename launch_arg_t = empty_t, typename segments_it>
workcreate_t<launch_arg_t, segments_it>
lbs_workcreate(int count, segments_it segments, int num_segments,
  context_t& context) {
  return workcreate_t<launch_arg_t, segments_it>(count, segments,
    num_segments, context);
}

} // namespace expt

END_MGPU_NAMESPACE
