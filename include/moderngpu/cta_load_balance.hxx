// mgpu for AMD CDNA4: the CTA-level load-balancing search.
//
// A tile is nv = nt * vt consecutive elements of the merge of work-item
// indices (A) with segment starts (B); the partition kernel supplies the
// split, so a tile holds a_count items and b_count segment starts with
// a_count + b_count <= nv, whatever the skew of the segment lengths.
//
// How the tile is decoded here differs from the CUDA library this API
// mirrors (src/moderngpu/cta_load_balance.hxx:16-184).  That code gives each
// thread one cross-diagonal, finds it with a binary search in shared memory
// and then walks vt + 1 dependent shared-memory compares.  On CDNA that chain
// of dependent LDS reads is latency bound, so this implementation does:
//   1. zero an int marker per item slot in LDS (16-byte stores);
//   2. every segment that owns at least one item of the tile writes
//      (its index in the tile + 1) at the slot of its first item -- one plain
//      LDS store per segment, no atomics, because among equal starts only the
//      last one owns items;
//   3. each thread max-scans vt consecutive slots in registers (independent
//      16-byte LDS reads), one cta_scan_t<max> over the thread totals carries
//      the running segment across threads, and the result is written back;
//   4. the slots are read back in strided order, which is the coalesced order
//      for whatever the caller stores per item.
// The LDS layout pads one 16-byte chunk after every eight so that both the
// strided and the thread-order 16-byte accesses spread over all banks.
#pragma once
#include "cta_merge.hxx"
#include "cta_scan.hxx"
#include "operators.hxx"
#include "cpp11.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

////////////////////////////////////////////////////////////////////////////////
// 16-byte vectors of W elements; the _u form may sit at any element-aligned
// address in global memory (global_load/store_dwordx4 only need dword
// alignment).

template<typename type_t, int W>
struct vec_t {
  typedef type_t type __attribute__((ext_vector_type(W)));
  typedef type_t type_u __attribute__((ext_vector_type(W),
    aligned(sizeof(type_t))));
};

// Tile element p lives at LDS element index(p).  W = elements per 16-byte
// chunk (1 disables chunking and padding).  One spare chunk follows every
// MGPU_TILE_PAD_CHUNKS chunks.
#ifndef MGPU_TILE_PAD_CHUNKS
#define MGPU_TILE_PAD_CHUNKS 8
#endif
template<int W>
struct tile_layout_t {
  MGPU_HOST_DEVICE static constexpr int index(int p) {
    return W > 1 ? p + (p / (MGPU_TILE_PAD_CHUNKS * W)) * W : p;
  }
  MGPU_HOST_DEVICE static constexpr int capacity(int n) {
    return index(n) + 2 * W;
  }
};

// Elements per 16-byte chunk when the tile of vt values per thread can be
// moved in whole chunks, else 1.
template<typename type_t, int vt>
struct chunk_width_t {
  enum {
    can = std::is_arithmetic<type_t>::value &&
      (sizeof(type_t) == 4 || sizeof(type_t) == 8) &&
      0 == vt % (16 / sizeof(type_t)),
    value = can ? 16 / sizeof(type_t) : 1
  };
};

// Which tile a CTA works on.  The hardware hands consecutive workgroups of a
// grid to the 8 accelerator dies (XCDs) of the package in turn, and each XCD
// has its own L2.  With tile == blockIdx.x, neighbouring tiles -- which share
// the cache line where one tile's data ends and the next begins -- always sit
// on different XCDs: the line is fetched twice, or written back partially by
// two L2s.  xcd_tile() gives each XCD runs of xcd_run consecutive tiles, and
// the runs of the 8 XCDs interleave, so the set of tiles in flight stays one
// compact window of memory.  xcd_tile_eighths() gives each XCD one contiguous
// eighth of all tiles.  That is the fastest layout for a kernel that only
// stores (1 GiB in ragged tiles of about 30 KB: 171 us against 190-200 us
// with runs or with tile == blockIdx.x), but as soon as each tile also reads
// a couple of KB that miss the L2 the advantage is gone (all three layouts
// 195-205 us), and the search kernels measured slower with it (216 against
// 195 us); the segmented reduce, which reads far more than it writes, takes
// the same time in its tile kernel and 1.1 us less as a whole call on 2^26
// floats (49.2 against 50.3 us), so that kernel uses eighths and the others
// runs.  The grid must be xcd_grid(num_tiles) for either; CTAs whose tile is
// >= num_tiles have nothing to do.
enum { num_xcds = 8, xcd_run = 16 };
MGPU_HOST_DEVICE int xcd_grid(int num_tiles) {
  return div_up(num_tiles, (int)(num_xcds * xcd_run)) * (num_xcds * xcd_run);
}
MGPU_DEVICE inline int xcd_tile(int cta, int) {
  int xcd = cta % num_xcds, local = cta / num_xcds;
  return ((local / xcd_run) * num_xcds + xcd) * xcd_run + local % xcd_run;
}
MGPU_DEVICE inline int xcd_tile_eighths(int cta, int num_tiles) {
  int xcd = cta % num_xcds, local = cta / num_xcds;
  int per = (num_tiles + num_xcds - 1) / num_xcds;
  return local < per ? xcd * per + local : num_tiles;
}

// The tile's item and segment ranges from the two splits at its ends, forced
// to be consistent: each split inside what its cross-diagonal allows, ends not
// before begins, at most nv elements.  For well-formed input (ascending
// starts) this changes nothing; for malformed input it keeps every LDS and
// global access of the tile kernels inside its array (results are then
// meaningless, but nothing faults).
MGPU_DEVICE inline merge_range_t tile_range(int count, int num_segments,
  int cta, int nv, int mp0, int mp1) {
  int total = count + num_segments;
  int diag0 = nv * cta;
  int diag1 = diag0 + min(nv, total - diag0);      // no overflow near 2^31
  mp0 = min(max(mp0, max(0, diag0 - num_segments)), min(diag0, count));
  mp1 = min(max(mp1, max(0, diag1 - num_segments)), min(diag1, count));
  mp1 = mp0 + min(max(mp1 - mp0, 0), nv);
  merge_range_t r { mp0, mp1, diag0 - mp0, diag1 - mp1 };
  r.b_end = r.b_begin +
    min(max(r.b_end - r.b_begin, 0), nv - (mp1 - mp0));
  return r;
}

// Tile ends moved onto 128-byte lines of a 4-byte output.
//
// With splits taken exactly on the cross-diagonals, a tile's items begin and
// end anywhere, so the first and last cache line of what a CTA stores per item
// are shared with its neighbours and every 16-byte store straddles two
// 16-byte slots.  A split (a, b) may however be moved back along the merge
// path to any earlier point of the path without changing any result; the
// partition kernel of the search (load_balance_partitions_snapped) moves it
// to the last point whose item index is a multiple of lbs_snap_items, unless
// lbs_snap_window or more segment starts would have to move with it.  A moved
// split retreats by at most (lbs_snap_items - 1) + (lbs_snap_window - 1)
// merged elements, so tiles cut at multiples of lbs_tile_spacing(nv) =
// nv - lbs_snap_slack never exceed nv elements.
enum { lbs_snap_items = 32, lbs_snap_window = 32, lbs_snap_slack = 64 };

// Segment starts per block of the coarse partition (lbs_block_partition_f in
// search.hxx, cta_load_balance_t::fill_blocks below).
enum { lbs_block = 256 };

MGPU_HOST_DEVICE constexpr int lbs_tile_spacing(int nv) {
  return nv >= 8 * lbs_snap_slack ? nv - lbs_snap_slack : nv;
}

// Range of a tile from the snapped splits at its two ends, pairs[2 * i] =
// items and pairs[2 * i + 1] = starts in front of split i, made consistent
// the way tile_range() does (this only matters for malformed input).
MGPU_DEVICE inline merge_range_t paired_tile_range(int count,
  int num_segments, int tile, int nv, const int* pairs) {
  int a0 = pairs[2 * tile], b0 = pairs[2 * tile + 1];
  int a1 = pairs[2 * tile + 2], b1 = pairs[2 * tile + 3];
  a0 = min(max(a0, 0), count);
  b0 = min(max(b0, 0), num_segments);
  // (unsigned: a0 + nv may pass 2^31 when count is close to the index limit)
  a1 = (int)min(min((unsigned)max(a1, a0), (unsigned)a0 + (unsigned)nv),
    (unsigned)count);
  b1 = (int)min(min((unsigned)max(b1, b0),
    (unsigned)b0 + (unsigned)(nv - (a1 - a0))), (unsigned)num_segments);
  return merge_range_t { a0, a1, b0, b1 };
}

// Read W consecutive LDS elements starting at an index that is a multiple
// of W.
template<int W, typename type_t>
MGPU_DEVICE inline void lds_load_chunk(const type_t* p, type_t (&x)[W]) {
  if constexpr(W > 1) {
    typedef typename vec_t<type_t, W>::type v_t;
    v_t v = *(const v_t*)p;
    PRAGMA_UNROLL
    for(int e = 0; e < W; ++e) x[e] = v[e];
  } else
    x[0] = p[0];
}
template<int W, typename type_t>
MGPU_DEVICE inline void lds_store_chunk(type_t* p, const type_t (&x)[W]) {
  if constexpr(W > 1) {
    typedef typename vec_t<type_t, W>::type v_t;
    v_t v;
    PRAGMA_UNROLL
    for(int e = 0; e < W; ++e) v[e] = x[e];
    *(v_t*)p = v;
  } else
    p[0] = x[0];
}

// Loading W consecutive tile items.  Raw pointers to 4/8-byte arithmetic
// types use one (possibly unaligned) 16-byte global load; anything else is
// element-wise through operator[].

// load(input, base, offset, x) reads items base + offset + [0, W); base is
// the same in all threads of the CTA and offset is not negative, which lets
// a pointer input be addressed as (scalar base address, 32-bit lane offset).
template<typename input_it, typename type_t, int W>
struct tile_loader_t {
  MGPU_DEVICE static void load(input_it input, int base, unsigned offset,
    type_t (&x)[W]) {
    PRAGMA_UNROLL
    for(int e = 0; e < W; ++e) x[e] = input[base + (int)offset + e];
  }
};

template<typename type_t, int W>
struct pointer_loader_t {
  MGPU_DEVICE static void load(const type_t* input, int base,
    unsigned offset, type_t (&x)[W]) {
    const type_t* tile = input + base;
    if constexpr(W > 1) {
      typedef typename vec_t<type_t, W>::type_u v_t;
      // What a tile kernel streams in is read once.  Marking the load
      // non-temporal keeps it from displacing other lines in the caches and
      // is worth 8-15 % of the time of the streaming kernels on this part
      // (segmented reduce 49 -> 43 us for 2^26 floats, scan 157 -> 134 us).
      v_t v = __builtin_nontemporal_load((const v_t*)(tile + offset));
      PRAGMA_UNROLL
      for(int e = 0; e < W; ++e) x[e] = v[e];
    } else
      x[0] = tile[offset];
  }
};
template<typename type_t, int W>
struct tile_loader_t<const type_t*, type_t, W> : pointer_loader_t<type_t, W> { };
template<typename type_t, int W>
struct tile_loader_t<type_t*, type_t, W> : pointer_loader_t<type_t, W> { };

// Stores W consecutive elements.  Element types whose size is a multiple of
// four bytes go out as 16-byte stores (global_store_dwordx4 only needs dword
// alignment); smaller ones element by element.
template<int W, typename type_t>
MGPU_DEVICE inline void store_consecutive(type_t* dest,
  const type_t (&x)[W]) {
  if constexpr(0 == sizeof(type_t) % 4 && W * sizeof(type_t) <= 64) {
    enum { words = W * sizeof(type_t) / 4 };
    typedef unsigned v_t __attribute__((ext_vector_type(words), aligned(4)));
    v_t v;
    __builtin_memcpy(&v, x, sizeof(v));
    *(v_t*)dest = v;
  } else {
    PRAGMA_UNROLL
    for(int e = 0; e < W; ++e) dest[e] = x[e];
  }
}

// The loading counterpart: W consecutive elements of any trivially copyable
// type from an element-aligned address.
template<int W, typename type_t>
MGPU_DEVICE inline void load_consecutive(const type_t* source,
  type_t (&x)[W]) {
  if constexpr(0 == sizeof(type_t) % 4 && W * sizeof(type_t) <= 64) {
    enum { words = W * sizeof(type_t) / 4 };
    typedef unsigned v_t __attribute__((ext_vector_type(words), aligned(4)));
    v_t v = *(const v_t*)source;
    __builtin_memcpy(x, &v, sizeof(v));
  } else {
    PRAGMA_UNROLL
    for(int e = 0; e < W; ++e) x[e] = source[e];
  }
}

} // namespace detail

////////////////////////////////////////////////////////////////////////////////

// Where a thread's slice of the tile's merge begins (interface after
// src/moderngpu/cta_load_balance.hxx:9-65).  `range` is the range of the
// starts that were loaded: the tile's own, one more in front when there is
// one (the segment that is open when the tile begins) and one more behind
// when items remain past the tile.
struct lbs_placement_t {
  merge_range_t range;
  int a_index;            // first item the thread merges
  int b_index;            // segment that item belongs to
};

// Loads the tile's segment starts into b_shared (behind them, up to slot
// nv + 1, `count` as a sentinel) and finds by a merge-path search in LDS
// where thread tid's slice of vt merged elements begins.  b_shared must hold
// nt * vt + 2 - range.a_count() ints.  Two barriers.
template<int nt, int vt, typename segments_it>
MGPU_DEVICE lbs_placement_t cta_load_balance_place(int tid,
  merge_range_t range, int count, segments_it segments, int num_segments,
  int* b_shared) {

  int preceding = range.b_begin > 0;
  range.b_begin -= preceding;
  if(range.b_end < num_segments && range.a_end < count) ++range.b_end;

  int loaded = range.b_count();
  int sentinels = nt * vt + 1 + preceding - loaded - range.a_count();
  for(int i = tid; i < loaded; i += nt)
    b_shared[i] = segments[range.b_begin + i];
  for(int i = tid; i < sentinels; i += nt)
    b_shared[loaded + i] = count;
  __syncthreads();

  // The preceding start has been consumed before the tile begins: skip it.
  int diag = vt * tid + preceding;
  int mp = merge_path<bounds_upper>(counting_iterator_t<int>(range.a_begin),
    range.a_count(), b_shared, loaded + sentinels, diag, less_t<int>());
  __syncthreads();

  // diag - mp starts lie in front of the slice; the last of them is the
  // segment of the slice's first item.
  return lbs_placement_t { range, range.a_begin + mp,
    range.b_begin + (diag - mp) - 1 };
}

// What cta_load_balance_fill leaves behind: shared[i] = segment of tile item
// i for i in [0, range.a_count()), and the start of segment s at
// shared[b_offset + s] (interface after cta_load_balance.hxx:67-105).
struct lbs_fill_t {
  merge_range_t range;
  int b_offset;
};

template<int nt, int vt, typename segments_it, typename partition_it>
MGPU_DEVICE lbs_fill_t cta_load_balance_fill(int count, segments_it segments,
  int num_segments, int tid, int cta, partition_it partitions, int* shared) {

  merge_range_t range = detail::tile_range(count, num_segments, cta, nt * vt,
    partitions[cta], partitions[cta + 1]);
  int* a_shared = shared - range.a_begin;
  int* b_shared = shared + range.a_count();
  lbs_placement_t placement = cta_load_balance_place<nt, vt>(tid, range,
    count, segments, num_segments, b_shared);
  b_shared -= placement.range.b_begin;

  int item = placement.a_index, segment = placement.b_index;
  iterate<vt>([&](int) {
    if(item < b_shared[segment + 1]) a_shared[item++] = segment;
    else ++segment;
  });
  __syncthreads();
  return lbs_fill_t { range, range.a_count() - placement.range.b_begin };
}

template<int nt, int vt>
struct cta_load_balance_t {
  enum {
    nv = nt * vt,
    W = detail::chunk_width_t<int, vt>::value,
    chunks = vt / W
  };
  typedef detail::tile_layout_t<W> layout_t;
  typedef cta_scan_t<nt, int> scan_t;

  struct storage_t {
    // Item slots (padded layout), then the tile's segment starts:
    // starts[0] belongs to the segment that is open when the tile begins,
    // starts[1 + j] to segment b_begin + j.
    alignas(16) int indices[layout_t::capacity(nv) + 4];
    typename scan_t::storage_t scan;
  };

  struct result_t {
    lbs_placement_t placement;
    merge_range_t merge_range;
    int merge_flags;                // thread order: bit i of the serial merge

    // Strided order: element i is tile item nt * i + tid.
    array_t<int, vt> indices;       // global item index
    array_t<int, vt> segments;      // segment of the item
    array_t<int, vt> ranks;         // item index - start of its segment
  };

  // Index of the first start slot for a tile with a_count items.
  MGPU_DEVICE static int starts_offset(int a_count) {
    return layout_t::index((a_count + W - 1) / W * W) + W;
  }

  // Decodes the tile and leaves, for every item slot p in [0, a_count),
  // (segment of item - (b_begin - 1)) in storage.indices[index(p)], and the
  // segment starts behind them.  Ends with a barrier.
  template<typename segments_it, typename partition_it>
  MGPU_DEVICE merge_range_t fill(int count, segments_it segments,
    int num_segments, int tid, int cta, partition_it partitions,
    storage_t& storage) const {

    merge_range_t range = detail::tile_range(count, num_segments, cta, nv,
      partitions[cta], partitions[cta + 1]);
    fill(range, segments, tid, storage);
    return range;
  }

  // The segment starts of a tile read ahead of time into registers (a CTA
  // that decodes several tiles issues the reads for all of them before it
  // works on the first).  Tiles with more than prefetch_rows * nt starts are
  // not read ahead; fill() then reads them itself.
  enum { prefetch_rows = 2 };
  struct prefetch_t {
    int starts[prefetch_rows];
    int preceding;          // start of the segment open at the tile's begin
    bool valid;
  };

  template<typename segments_it>
  MGPU_DEVICE static prefetch_t prefetch(merge_range_t range,
    segments_it segments, int tid) {
    prefetch_t ahead = prefetch_t();
    int b_count = range.b_count();
    ahead.valid = b_count <= prefetch_rows * nt;
    if(ahead.valid) {
      PRAGMA_UNROLL
      for(int r = 0; r < prefetch_rows; ++r)
        if(nt * r + tid < b_count)
          ahead.starts[r] = segments[range.b_begin + nt * r + tid];
      // The start in front of the tile's own is read by the last thread: a
      // read by thread 0 alone becomes a scalar load that the first wavefront
      // waits for on the spot.
      if(nt - 1 == tid && range.b_begin)
        ahead.preceding = segments[range.b_begin - 1];
    }
    return ahead;
  }

  // Same for a tile whose range the caller has worked out.
  template<typename segments_it>
  MGPU_DEVICE void fill(merge_range_t range, segments_it segments, int tid,
    storage_t& storage) const {
    fill(range, segments, tid, storage, prefetch_t());
  }

  // ... and whose starts the caller may have read ahead with prefetch().
  template<typename segments_it>
  MGPU_DEVICE void fill(merge_range_t range, segments_it segments, int tid,
    storage_t& storage, prefetch_t ahead) const {

    int a_count = range.a_count();
    int b_count = range.b_count();
    int* slots = storage.indices;
    int* starts = storage.indices + starts_offset(a_count);

    // 1. clear the item slots.
    int zero[W];
    PRAGMA_UNROLL
    for(int e = 0; e < W; ++e) zero[e] = 0;
    PRAGMA_UNROLL
    for(int i = 0; i < chunks; ++i) {
      int p = W * (nt * i + tid);
      if(p < a_count)
        detail::lds_store_chunk<W>(slots + layout_t::index(p), zero);
    }

    // 2. stage the segment starts of the tile.
    if(ahead.valid) {
      PRAGMA_UNROLL
      for(int r = 0; r < prefetch_rows; ++r)
        if(nt * r + tid < b_count) starts[1 + nt * r + tid] = ahead.starts[r];
      if(nt - 1 == tid) starts[0] = ahead.preceding;
    } else {
      for(int j = tid; j < b_count; j += nt)
        starts[1 + j] = segments[range.b_begin + j];
      if(!tid) starts[0] = range.b_begin ? segments[range.b_begin - 1] : 0;
    }
    __syncthreads();

    // 3. one marker per segment that owns items here.  Starts ascend, so
    // among equal starts only the last segment is non-empty; a start at or
    // past a_end owns nothing in this tile.
    for(int j = tid; j < b_count; j += nt) {
      int s0 = starts[1 + j];
      int s1 = (j + 1 < b_count) ? starts[2 + j] : 0x7fffffff;
      int p = s0 - range.a_begin;
      if(s0 != s1 && p >= 0 && p < a_count)
        slots[layout_t::index(p)] = j + 1;
    }
    __syncthreads();

    // 4. running maximum along the items.
    scan_slots(tid, a_count, slots, storage.scan);
  }

  // Running maximum along the item slots: vt slots per thread in registers,
  // one exclusive max-scan over the thread totals.  Ends with a barrier.
  MGPU_DEVICE static void scan_slots(int tid, int a_count, int* slots,
    typename scan_t::storage_t& scan_storage) {
    scan_slots(tid, a_count, slots, scan_storage, []MGPU_DEVICE() { });
  }
  // before_barrier() is called ahead of the final barrier: LDS writes the
  // caller wants covered by it.
  template<typename before_barrier_t>
  MGPU_DEVICE static void scan_slots(int tid, int a_count, int* slots,
    typename scan_t::storage_t& scan_storage,
    before_barrier_t before_barrier) {
    int x[vt];
    PRAGMA_UNROLL
    for(int c = 0; c < chunks; ++c) {
      int chunk[W];
      detail::lds_load_chunk<W>(
        slots + layout_t::index(vt * tid + W * c), chunk);
      PRAGMA_UNROLL
      for(int e = 0; e < W; ++e) x[W * c + e] = chunk[e];
    }
    PRAGMA_UNROLL
    for(int i = 1; i < vt; ++i) x[i] = max(x[i - 1], x[i]);

    scan_result_t<int> carry = scan_t().scan(tid, x[vt - 1], scan_storage,
      nt, maximum_t<int>(), 0, scan_type_exc);

    PRAGMA_UNROLL
    for(int c = 0; c < chunks; ++c) {
      int chunk[W];
      PRAGMA_UNROLL
      for(int e = 0; e < W; ++e) chunk[e] = max(carry.scan, x[W * c + e]);
      // Slots at or past a_count belong to the segment starts: leave them.
      if(vt * tid + W * c < a_count)
        detail::lds_store_chunk<W>(
          slots + layout_t::index(vt * tid + W * c), chunk);
    }
    before_barrier();
    __syncthreads();
  }

  //////////////////////////////////////////////////////////////////////////////
  // The same decode in half the LDS: 16-bit slots.  A tile has fewer than
  // 2^16 elements, so (segment - first segment + 1) fits 16 bits, and so does
  // the start of every segment that begins inside the tile when it is kept
  // relative to the tile's first item.  Only the start of the segment that is
  // open when the tile begins may lie anywhere in front; it is kept apart, as
  // a 32-bit difference.  With 512 x 12 tiles this is 14 KB instead of 28 KB
  // per CTA, with 512 x 16 tiles 19 KB instead of 37 KB.

  typedef unsigned short slot_t;

  struct compact_storage_t {
    // Item slots (padded layout), then the relative starts: entry 0 is zero
    // and stands for the open segment, entry 1 + j belongs to segment
    // b_begin + j.
    alignas(16) slot_t slots[layout_t::capacity(nv) + 8];
    int open_offset;
    typename scan_t::storage_t scan;
  };

  // What fill_compact() leaves: slot p holds (segment of tile item p) -
  // (b_begin - 1), and the rank of item p in that segment is rank(p, rel).
  struct compact_tile_t {
    const slot_t* slots;
    const slot_t* starts;
    int open_offset;        // first item of the tile - start of open segment
    MGPU_DEVICE int rank(int p, int rel) const {
      return p - (int)starts[rel] + (rel ? 0 : open_offset);
    }
  };

  template<typename segments_it>
  MGPU_DEVICE compact_tile_t fill_compact(merge_range_t range,
    segments_it segments, int tid, compact_storage_t& storage,
    prefetch_t ahead) const {
    static_assert(nv + 2 < 65536, "16-bit tile slots need tiles below 2^16");

    int a_count = range.a_count();
    int b_count = range.b_count();
    slot_t* slots = storage.slots;
    slot_t* starts = storage.slots + starts_offset(a_count);

    // 1. clear the item slots.
    slot_t zero[W];
    PRAGMA_UNROLL
    for(int e = 0; e < W; ++e) zero[e] = 0;
    PRAGMA_UNROLL
    for(int i = 0; i < chunks; ++i) {
      int p = W * (nt * i + tid);
      if(p < a_count)
        detail::lds_store_chunk<W>(slots + layout_t::index(p), zero);
    }

    // 2. stage the segment starts of the tile, relative to its first item
    // (a start of well-formed input lies in [a_begin, a_end]; the clamp is
    // for anything else).
    auto relative = [&](int start) {
      return (slot_t)min(max(start - range.a_begin, 0), 65535);
    };
    int preceding = 0;
    if(ahead.valid) {
      PRAGMA_UNROLL
      for(int r = 0; r < prefetch_rows; ++r)
        if(nt * r + tid < b_count)
          starts[1 + nt * r + tid] = relative(ahead.starts[r]);
      preceding = ahead.preceding;
    } else {
      for(int j = tid; j < b_count; j += nt)
        starts[1 + j] = relative((int)segments[range.b_begin + j]);
      if(nt - 1 == tid && range.b_begin)
        preceding = (int)segments[range.b_begin - 1];
    }
    if(nt - 1 == tid) {
      starts[0] = 0;
      storage.open_offset = range.b_begin ? range.a_begin - preceding : 0;
    }
    __syncthreads();
    int open_offset = storage.open_offset;

    // 3. one marker per segment that owns items here (see fill()).
    for(int j = tid; j < b_count; j += nt) {
      int s0 = starts[1 + j];
      int s1 = (j + 1 < b_count) ? (int)starts[2 + j] : 0x10000;
      if(s0 != s1 && s0 < a_count)
        slots[layout_t::index(s0)] = (slot_t)(j + 1);
    }
    __syncthreads();

    // 4. running maximum along the items.
    scan_compact(tid, a_count, slots, storage.scan);
    return compact_tile_t { slots, starts, open_offset };
  }

  MGPU_DEVICE static void scan_compact(int tid, int a_count, slot_t* slots,
    typename scan_t::storage_t& scan_storage) {
    int x[vt];
    PRAGMA_UNROLL
    for(int c = 0; c < chunks; ++c) {
      slot_t chunk[W];
      detail::lds_load_chunk<W>(
        slots + layout_t::index(vt * tid + W * c), chunk);
      PRAGMA_UNROLL
      for(int e = 0; e < W; ++e) x[W * c + e] = chunk[e];
    }
    PRAGMA_UNROLL
    for(int i = 1; i < vt; ++i) x[i] = max(x[i - 1], x[i]);

    scan_result_t<int> carry = scan_t().scan(tid, x[vt - 1], scan_storage,
      nt, maximum_t<int>(), 0, scan_type_exc);

    PRAGMA_UNROLL
    for(int c = 0; c < chunks; ++c) {
      slot_t chunk[W];
      PRAGMA_UNROLL
      for(int e = 0; e < W; ++e)
        chunk[e] = (slot_t)max(carry.scan, x[W * c + e]);
      // Slots at or past a_count belong to the segment starts: leave them.
      if(vt * tid + W * c < a_count)
        detail::lds_store_chunk<W>(
          slots + layout_t::index(vt * tid + W * c), chunk);
    }
    __syncthreads();
  }

  //////////////////////////////////////////////////////////////////////////////
  // Decoding a tile from coarse splits (detail::lbs_block_partition_f): the
  // partition kernel only says in which block of lbs_block starts each of the
  // tile's two splits lies.  The tile loads the starts of those blocks and of
  // everything between them -- its own starts plus at most a block at either
  // end, as aligned 16-byte loads -- and counts the exact splits itself:
  // the split of cross-diagonal d has as many starts in front of it as there
  // are j with segments[j] + j < d.  It then moves both splits back onto a
  // multiple of lbs_snap_items items where fewer than lbs_snap_window starts
  // have to move along (see lbs_tile_spacing), which the last lbs_snap_window
  // starts in front of each split decide; they are among the loaded ones.

  enum {
    block = detail::lbs_block,
    lookback = detail::lbs_snap_window,
    // Starts a tile may load beyond its own: a block at either end, the
    // look-back, what snapping hands to the tile in front, rounding.
    block_margin = 2 * block + 2 * lookback - 2,
    block_extra = block_margin + 10,
    block_ints = layout_t::capacity(nv) + block_extra,
    // Rows of nt 16-byte loads held in registers ahead of time.
    block_rows = (1024 + 4 * nt - 1) / (4 * nt),
    num_waves = nt / warp_size
  };

  struct block_storage_t {
    // Item slots from the bottom (padded layout), the loaded starts at the
    // top: start j at indices[block_ints - round_up(je - jb, 4) + j - jb].
    alignas(16) int indices[block_ints];
    alignas(16) int below[2 * num_waves];   // per wavefront: starts in front
                                            // of the tile's two diagonals
    typename scan_t::storage_t scan;
  };

  struct block_tile_t {
    int tile;
    int d0, d1;             // cross-diagonals at the tile's two ends
    int jb, je;             // starts [jb, je) are loaded
    bool ahead;             // ... into these registers, ahead of time
    int starts[block_rows][4];
  };

  // Loads starts j .. j + 3 (those below end).
  template<typename segments_it>
  MGPU_DEVICE static void load_starts(segments_it segments, int j, int end,
    int (&x)[4]) {
    if constexpr(std::is_same<segments_it, const int*>::value ||
      std::is_same<segments_it, int*>::value) {
      if(j + 4 <= end) {
        typedef int v4_t __attribute__((ext_vector_type(4), aligned(4)));
        v4_t v = *(const v4_t*)(segments + j);
        x[0] = v[0]; x[1] = v[1]; x[2] = v[2]; x[3] = v[3];
        return;
      }
    }
    PRAGMA_UNROLL
    for(int e = 0; e < 4; ++e)
      if(j + e < end) x[e] = (int)segments[j + e];
  }

  // What a tile has to load, with the loads issued when they fit the
  // registers set aside for them.
  template<typename segments_it>
  MGPU_DEVICE static block_tile_t block_prefetch(int count, int num_segments,
    int tile, int spacing, const int* blocks, segments_it segments,
    int tid) {
    block_tile_t info;
    int total = count + num_segments;
    int last_block = max((num_segments + block - 1) / block - 1, 0);
    info.tile = tile;
    info.d0 = spacing * tile;
    info.d1 = info.d0 + min(spacing, total - info.d0);
    // The clamps only matter for malformed (unsorted) input, which may leave
    // entries of blocks[] unwritten.
    int k0 = min(max(blocks[tile], 0), last_block);
    int k1 = min(max(blocks[tile + 1], k0), last_block);
    info.jb = max(block * k0 - lookback, 0);
    info.je = min(min(block * (k1 + 1), num_segments),
      info.jb + spacing + block_margin + 2);
    info.ahead = info.je - info.jb <= 4 * nt * block_rows;
    if(info.ahead) {
      PRAGMA_UNROLL
      for(int r = 0; r < block_rows; ++r) {
        int j = info.jb + 4 * (nt * r + tid);
        if(j < info.je) load_starts(segments, j, info.je, info.starts[r]);
      }
    }
    return info;
  }

  // Decodes the tile: leaves, for every item slot p in [0, a_count),
  // (segment of item - (b_begin - 1)) in storage.indices[index(p)] and returns
  // the tile's range; starts[rel] is then the start of segment b_begin - 1 +
  // rel.  snap: whether splits are moved onto multiples of lbs_snap_items
  // (the tiles must then be cut every nv - lbs_snap_slack).  Ends with a
  // barrier.
  template<typename segments_it>
  MGPU_DEVICE static merge_range_t fill_blocks(const block_tile_t& info,
    int count, int num_segments, segments_it segments, bool snap, int tid,
    block_storage_t& storage, const int*& starts) {
    return fill_blocks(info, count, num_segments, segments, snap, tid,
      storage, starts, []MGPU_DEVICE() { });
  }
  // before_barrier(): see scan_slots().
  template<typename segments_it, typename before_barrier_t>
  MGPU_DEVICE static merge_range_t fill_blocks(const block_tile_t& info,
    int count, int num_segments, segments_it segments, bool snap, int tid,
    block_storage_t& storage, const int*& starts,
    before_barrier_t before_barrier) {

    int jb = info.jb, je = info.je;
    int loaded = je - jb;
    int* slots = storage.indices;
    int* staged = storage.indices + (block_ints - ((loaded + 3) & ~3));
    // The tile's own starts are all but block_margin of the loaded ones at
    // least, which bounds its items.
    int a_max = max(nv - max(0, loaded - block_margin), 0);

    // 1. clear the item slots.
    int zero[W];
    PRAGMA_UNROLL
    for(int e = 0; e < W; ++e) zero[e] = 0;
    PRAGMA_UNROLL
    for(int i = 0; i < chunks; ++i) {
      int p = W * (nt * i + tid);
      if(p < a_max)
        detail::lds_store_chunk<W>(slots + layout_t::index(p), zero);
    }

    // 2. stage the starts and count those in front of the two diagonals
    // (start j sits at merged position segments[j] + j).
    int below0 = 0, below1 = 0;
    auto stage = [&](int q, const int (&x)[4]) {
      int j = jb + 4 * q;
      detail::lds_store_chunk<4>(staged + 4 * q, x);
      PRAGMA_UNROLL
      for(int e = 0; e < 4; ++e) {
        bool valid = j + e < je;
        below0 += popc(ballot(valid && x[e] < info.d0 - (j + e)));
        below1 += popc(ballot(valid && x[e] < info.d1 - (j + e)));
      }
    };
    if(info.ahead) {
      PRAGMA_UNROLL
      for(int r = 0; r < block_rows; ++r) {
        int q = nt * r + tid;
        if(4 * q < loaded) stage(q, info.starts[r]);
      }
    } else {
      // A tile of many starts: three rows of loads in flight at a time.
      for(int q = tid; 4 * q < loaded; q += 3 * nt) {
        int x[3][4] = { { 0, 0, 0, 0 }, { 0, 0, 0, 0 }, { 0, 0, 0, 0 } };
        PRAGMA_UNROLL
        for(int r = 0; r < 3; ++r)
          if(4 * (q + nt * r) < loaded)
            load_starts(segments, jb + 4 * (q + nt * r), je, x[r]);
        PRAGMA_UNROLL
        for(int r = 0; r < 3; ++r)
          if(4 * (q + nt * r) < loaded) stage(q + nt * r, x[r]);
      }
    }
    if(0 == tid % warp_size) {
      storage.below[2 * (tid / warp_size)] = below0;
      storage.below[2 * (tid / warp_size) + 1] = below1;
    }
    __syncthreads();

    // 3. the exact splits, then the snapped ones.  Lanes 0-31 look at the
    // last starts in front of the first split, lanes 32-63 at those in front
    // of the second; every wavefront does the same.
    int b0 = jb, b1 = jb;
    PRAGMA_UNROLL
    for(int w = 0; w < num_waves; ++w) {
      b0 += storage.below[2 * w];
      b1 += storage.below[2 * w + 1];
    }
    int a0 = info.d0 - b0, a1 = info.d1 - b1;
    if(snap) {
      int lane = tid % warp_size;
      bool second = lane >= warp_size / 2;
      int a_snap = second ? a1 - a1 % detail::lbs_snap_items :
        a0 - a0 % detail::lbs_snap_items;
      int j = (second ? b1 : b0) - 1 - lane % (warp_size / 2);
      bool above = j >= jb && j < je && staged[j - jb] > a_snap;
      lanemask_t mask = ballot(above);
      int back0 = popc((unsigned)mask);
      int back1 = popc((unsigned)(mask >> 32));
      if(info.d0 > 0 && back0 < lookback) {
        a0 -= a0 % detail::lbs_snap_items;
        b0 -= back0;
      }
      if(info.d1 < count + num_segments && back1 < lookback) {
        a1 -= a1 % detail::lbs_snap_items;
        b1 -= back1;
      }
    }
    // For well-formed input these change nothing.
    a0 = min(max(a0, 0), count);
    a1 = min(max(a1, a0), min(count, a0 + a_max));
    b0 = min(max(b0, jb), je);
    b1 = min(max(b1, b0), je);
    merge_range_t range { a0, a1, b0, b1 };
    int a_count = a1 - a0;

    // 4. one marker per segment that owns items here (see fill()).
    for(int j = b0 + tid; j < b1; j += nt) {
      int s0 = staged[j - jb];
      int s1 = (j + 1 < b1) ? staged[j + 1 - jb] : 0x7fffffff;
      int p = s0 - a0;
      if(s0 != s1 && p >= 0 && p < a_count)
        slots[layout_t::index(p)] = j - b0 + 1;
    }
    __syncthreads();

    // 5. running maximum along the items.
    scan_slots(tid, a_count, slots, storage.scan, before_barrier);
    starts = staged + (b0 - 1 - jb);
    return range;
  }

  // The CTA-level search with everything the reference's returns
  // (cta_load_balance.hxx:107-184): the thread's placement, the bits of its
  // serial merge (bit i set: step i of the vt + 1 steps took an item, clear:
  // it moved on to the next segment), and per item in strided order the global
  // index, its segment and its rank; items past the end of the tile get
  // segment b_begin and rank -1.  This is the thread-per-diagonal form --
  // a merge-path search and vt + 1 dependent LDS reads per thread -- for
  // callers that need placement or merge bits; the library's own kernels
  // decode tiles with fill() above, which has neither.
  template<typename segments_it, typename partition_it>
  MGPU_DEVICE result_t load_balance(int count, segments_it segments,
    int num_segments, int tid, int cta, partition_it partitions,
    storage_t& storage) const {

    merge_range_t range = detail::tile_range(count, num_segments, cta, nv,
      partitions[cta], partitions[cta + 1]);
    int* a_shared = storage.indices - range.a_begin;
    int* b_shared = storage.indices + range.a_count();
    lbs_placement_t placement = cta_load_balance_place<nt, vt>(tid, range,
      count, segments, num_segments, b_shared);
    b_shared -= placement.range.b_begin;

    int item = placement.a_index, segment = placement.b_index;
    int merge_flags = 0;
    iterate<vt + 1>([&](int i) {
      bool take = item < b_shared[segment + 1];
      if(take && i < vt) a_shared[item++] = segment;
      else ++segment;
      merge_flags |= (int)take << i;
    });
    __syncthreads();

    result_t result;
    result.placement = placement;
    result.merge_range = range;
    result.merge_flags = merge_flags;
    iterate<vt>([&](int i) {
      int j = nt * i + tid;
      result.indices[i] = range.a_begin + j;
      if(j < range.a_count()) {
        result.segments[i] = storage.indices[j];
        result.ranks[i] = result.indices[i] - b_shared[result.segments[i]];
      } else {
        result.segments[i] = range.b_begin;
        result.ranks[i] = -1;
      }
    });
    __syncthreads();
    return result;
  }
};

namespace detail {

////////////////////////////////////////////////////////////////////////////////
// Per-segment values ("caching iterators") for the items of a tile.  When the
// tile touches at most nt segments each value is read from global memory once
// and fanned out through LDS; otherwise every item gathers its own
// (interface after src/moderngpu/cta_load_balance.hxx:189-259).

template<int nt, typename pointers_t>
struct cached_segment_load_t {
  enum { size = tuple_size<pointers_t>::value };
  typedef tuple_iterator_value_t<pointers_t> value_t;

  // Values of up to 16 bytes are staged for up to 2 * nt - 32 segments (two
  // reads per thread), wider ones for up to nt: a tile of 512 x 16 elements
  // can begin 873 segments on the 2^24-segment benchmark input, and a tile
  // with more segments than are staged has every item gather its own value
  // from global memory, which costs several times what staging does.
  // Values of up to 8 bytes are all read ahead by fetch(); of wider ones
  // only the first row is (registers), and commit() reads the second.
  enum {
    staged_rows = sizeof(value_t) <= 16 ? 2 : 1,
    rows = sizeof(value_t) <= 8 ? staged_rows : 1,
    capacity = staged_rows * nt - (staged_rows > 1 ? 32 : 0)
  };
  struct storage_t {
    value_t data[capacity];
  };
  // What fetch() leaves in registers for commit().
  struct fetched_t {
    value_t x[rows];
  };

  // Stages the values of segments [begin, begin + count) in LDS if they fit
  // (one coalesced global read per segment); ends with a barrier then.
  // `count` must be the same in every thread.
  MGPU_DEVICE static bool stage(int tid, int begin, int count,
    storage_t& storage, pointers_t iterators) {
    fetched_t x;
    bool fits = fetch(tid, begin, count, iterators, x);
    commit(tid, begin, count, x, storage, iterators);
    return fits;
  }
  // The same in two steps, so that the global read can be in flight while
  // the caller does something else (decodes the tile, say): fetch() issues
  // the reads into registers, commit() puts them into LDS and ends with a
  // barrier if the values fit.
  MGPU_DEVICE static bool fetch(int tid, int begin, int count,
    pointers_t iterators, fetched_t& fetched) {
    if(count > capacity) return false;
    PRAGMA_UNROLL
    for(int r = 0; r < rows; ++r) {
      int at = nt * r + tid;
      if(at < count && begin + at >= 0)
        fetched.x[r] = mgpu::load(iterators, begin + at);
    }
    return true;
  }
  MGPU_DEVICE static void commit(int tid, int begin, int count,
    const fetched_t& fetched, storage_t& storage, pointers_t iterators) {
    if(count > capacity) return;
    // Rows that fetch() has not read ahead.
    value_t late[staged_rows - rows + 1];
    PRAGMA_UNROLL
    for(int r = rows; r < staged_rows; ++r) {
      int at = nt * r + tid;
      if(at < count && begin + at >= 0)
        late[r - rows] = mgpu::load(iterators, begin + at);
    }
    PRAGMA_UNROLL
    for(int r = 0; r < staged_rows; ++r) {
      int at = nt * r + tid;
      if(at < count && begin + at >= 0)
        storage.data[at] = r < rows ? fetched.x[r < rows ? r : 0] :
          late[r < rows ? 0 : r - rows];
    }
    __syncthreads();
  }
  // Value of segment seg = begin + rel.
  MGPU_DEVICE static value_t get(bool staged, int rel, int seg,
    const storage_t& storage, pointers_t iterators) {
    return staged ? storage.data[rel] : mgpu::load(iterators, max(seg, 0));
  }

  // range = segments the tile's items can belong to.
  template<int vt0, int vt>
  MGPU_DEVICE static array_t<value_t, vt> load(int tid, int count,
    range_t range, array_t<int, vt> segments, storage_t& storage,
    pointers_t iterators) {

    array_t<value_t, vt> loaded;
    if(range.count() <= nt) {
      if(tid < range.count() && range.begin + tid >= 0)
        storage.data[tid] = mgpu::load(iterators, range.begin + tid);
      __syncthreads();
      strided_iterate<nt, vt, vt0>([&](int i, int) {
        loaded[i] = storage.data[segments[i] - range.begin];
      }, tid, count);
      __syncthreads();
    } else {
      strided_iterate<nt, vt, vt0>([&](int i, int) {
        loaded[i] = mgpu::load(iterators, max(segments[i], 0));
      }, tid, count);
    }
    return loaded;
  }
};

template<int nt>
struct cached_segment_load_t<nt, tuple<> > {
  typedef empty_t storage_t;
  typedef tuple<> value_t;
  typedef empty_t fetched_t;

  MGPU_DEVICE static bool stage(int, int, int, storage_t&, tuple<>) {
    return false;
  }
  MGPU_DEVICE static bool fetch(int, int, int, tuple<>, fetched_t&) {
    return false;
  }
  MGPU_DEVICE static void commit(int, int, int, const fetched_t&,
    storage_t&, tuple<>) {
  }
  MGPU_DEVICE static value_t get(bool, int, int, const storage_t&, tuple<>) {
    return value_t();
  }
  template<int vt0, int vt>
  MGPU_DEVICE static array_t<value_t, vt> load(int, int, range_t,
    array_t<int, vt>, storage_t&, tuple<>) {
    return array_t<value_t, vt>();
  }
};

} // namespace detail

END_MGPU_NAMESPACE
