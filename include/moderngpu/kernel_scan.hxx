// mgpu for AMD CDNA4: device-wide prefix sum.
//
//   scan<scan_type>(input, count, output, op, reduction, context)
// writes, for an exclusive scan, output[0] = type_t() and output[i] =
// input[0] op ... op input[i - 1]; for an inclusive scan output[i] =
// input[0] op ... op input[i].  The fold of all items goes to *reduction
// (device or host-mapped memory, or a discard_iterator_t).  type_t() is only
// placed, never folded into anything.  op must be associative; it need not be
// commutative.
//
// Three launches for more than a few tiles: one partial per tile (upsweep),
// an exclusive scan of the partials by one CTA (spine), and the per-tile scan
// with the tile's partial as carry-in (downsweep).  Tiles are moved with
// 16-byte global loads and stores in strided order and turned into thread
// order through a padded LDS layout, as in the segmented-reduce tile kernel.
// Interface after src/moderngpu/kernel_scan.hxx:11-196 (whose upsweep folds in
// strided order and so silently needs a commutative op; here both sweeps fold
// left to right).
#pragma once
#include "cta_load_balance.hxx"
#include "cta_reduce.hxx"
#include "cta_scan.hxx"
#include "memory.hxx"
#include "operators.hxx"
#include "transform.hxx"
#include "launcher.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

// Default tile on gfx950: 256 threads x 16 values for types up to 8 bytes;
// wider types get fewer values per thread so the tile stays under 64 KB.
template<typename type_t>
struct scan_launch_default_t {
  enum {
    vt = sizeof(type_t) <= 8 ? 16 :
      (128 / sizeof(type_t) > 1 ? 128 / sizeof(type_t) : 1)
  };
  typedef launch_box_t<arch_gfx950_cta<256, vt> > type_t_;
};

// The tile in thread order: x[i] = item vt * tid + i of the tile (undefined
// past tile_count), staged through `values`.  Ends with every thread holding
// its items; the caller may reuse `values` after its next barrier.
template<int nt, int vt, typename input_it, typename type_t>
MGPU_DEVICE void scan_load_tile(input_it input, int begin, int tile_count,
  bool interior, int tid, type_t* values, type_t (&x)[vt]) {
  enum { W = chunk_width_t<type_t, vt>::value, chunks = vt / W };
  typedef tile_layout_t<W> layout_t;
  typedef tile_loader_t<input_it, type_t, W> loader_t;

  type_t r[chunks][W];
  if(interior) {
    PRAGMA_UNROLL
    for(int i = 0; i < chunks; ++i)
      loader_t::load(input, begin, (unsigned)(W * (nt * i + tid)), r[i]);
  } else {
    PRAGMA_UNROLL
    for(int i = 0; i < chunks; ++i) {
      int p = W * (nt * i + tid);
      if(p + W <= tile_count)
        loader_t::load(input, begin, (unsigned)p, r[i]);
      else {
        PRAGMA_UNROLL
        for(int e = 0; e < W; ++e)
          if(p + e < tile_count) r[i][e] = input[begin + p + e];
      }
    }
  }
  PRAGMA_UNROLL
  for(int i = 0; i < chunks; ++i) {
    int p = W * (nt * i + tid);
    if(interior || p < tile_count)
      lds_store_chunk<W>(values + layout_t::index(p), r[i]);
  }
  __syncthreads();
  PRAGMA_UNROLL
  for(int c = 0; c < chunks; ++c) {
    type_t chunk[W];
    lds_load_chunk<W>(values + layout_t::index(vt * tid + W * c), chunk);
    PRAGMA_UNROLL
    for(int e = 0; e < W; ++e) x[W * c + e] = chunk[e];
  }
}

// The reverse: y[i] = item vt * tid + i goes to output[begin + ...] with
// 16-byte stores in strided order.  Each thread first overwrites the LDS slots
// it read in scan_load_tile, so no barrier is needed in between.
template<int nt, int vt, typename output_it, typename type_t>
MGPU_DEVICE void scan_store_tile(const array_t<type_t, vt>& y,
  output_it output, int begin, int tile_count, bool interior, int tid,
  type_t* values) {
  enum { W = chunk_width_t<type_t, vt>::value, chunks = vt / W };
  typedef tile_layout_t<W> layout_t;
  PRAGMA_UNROLL
  for(int c = 0; c < chunks; ++c) {
    type_t chunk[W];
    PRAGMA_UNROLL
    for(int e = 0; e < W; ++e) chunk[e] = y[W * c + e];
    lds_store_chunk<W>(values + layout_t::index(vt * tid + W * c), chunk);
  }
  __syncthreads();

  PRAGMA_UNROLL
  for(int i = 0; i < chunks; ++i) {
    int p = W * (nt * i + tid);
    if(interior || p + W <= tile_count) {
      type_t chunk[W];
      lds_load_chunk<W>(values + layout_t::index(p), chunk);
      if constexpr(std::is_pointer<output_it>::value)
        store_consecutive<W>(output + begin + p, chunk);
      else {
        PRAGMA_UNROLL
        for(int e = 0; e < W; ++e) output[begin + p + e] = chunk[e];
      }
    } else {
      PRAGMA_UNROLL
      for(int e = 0; e < W; ++e)
        if(p + e < tile_count)
          output[begin + p + e] = values[layout_t::index(p + e)];
    }
  }
}

// Upsweep: partials[tile] = fold of the tile's items, left to right.
template<typename launch_t, typename input_it, typename type_t,
  typename op_t>
struct scan_upsweep_f {
  input_it input;
  int count;
  op_t op;
  type_t* partials;
  int num_tiles;

  MGPU_DEVICE void operator()(int tid, int cta) const {
    typedef typename launch_t::sm_ptx params_t;
    enum { nt = params_t::nt, vt = params_t::vt, nv = nt * vt,
      W = chunk_width_t<type_t, vt>::value };
    typedef tile_layout_t<W> layout_t;
    typedef cta_reduce_t<nt, type_t> reduce_t;
    int tile = xcd_tile(cta, num_tiles);
    if(tile >= num_tiles) return;

    __shared__ struct {
      alignas(16) type_t values[layout_t::capacity(nv)];
      typename reduce_t::storage_t reduce;
    } shared;

    range_t range = get_tile(tile, nv, count);
    int tile_count = range.count();
    type_t x[vt];
    scan_load_tile<nt, vt>(input, range.begin, tile_count, nv == tile_count,
      tid, shared.values, x);

    // Fold of the thread's items that exist; threads past the end of the
    // last tile stay out of the CTA-wide fold.
    int mine = min(max(tile_count - vt * tid, 0), (int)vt);
    type_t scalar = x[0];
    PRAGMA_UNROLL
    for(int i = 1; i < vt; ++i)
      if(i < mine) scalar = op(scalar, x[i]);
    type_t total = reduce_t().reduce(tid, scalar, shared.reduce,
      div_up(tile_count, (int)vt), op, false);
    if(!tid) partials[tile] = total;
  }
};

// Spine: exclusive scan of the partials in place by one CTA, total to
// *reduction.  Also the whole scan for inputs of a few tiles.
template<scan_type_t scan_type, int nt, int vt, typename input_it,
  typename output_it, typename type_t, typename op_t, typename reduction_it>
struct scan_spine_f {
  input_it input;
  int count;
  output_it output;
  op_t op;
  reduction_it reduction;

  MGPU_DEVICE void operator()(int tid, int) const {
    enum { nv = nt * vt, W = chunk_width_t<type_t, vt>::value };
    typedef tile_layout_t<W> layout_t;
    typedef cta_scan_t<nt, type_t> scan_t;
    __shared__ struct {
      alignas(16) type_t values[layout_t::capacity(nv)];
      typename scan_t::storage_t scan;
    } shared;

    type_t carry = type_t();
    for(int cur = 0; cur < count; cur += nv) {
      int n = min(count - cur, (int)nv);
      array_t<type_t, vt> x;
      scan_load_tile<nt, vt>(input, cur, n, nv == n, tid, shared.values,
        x.data);
      scan_result_t<type_t, vt> result = scan_t().template scan<vt>(tid, x,
        shared.scan, carry, cur > 0, n, op, type_t(), scan_type);
      scan_store_tile<nt, vt>(result.scan, output, cur, n, nv == n, tid,
        shared.values);
      carry = result.reduction;
      __syncthreads();
    }
    if(!tid) *reduction = carry;
  }
};

// Downsweep: scan of one tile with the fold of everything in front of it
// (carries[tile], not used for tile 0) carried in.
template<scan_type_t scan_type, typename launch_t, typename input_it,
  typename output_it, typename type_t, typename op_t>
struct scan_downsweep_f {
  input_it input;
  int count;
  output_it output;
  op_t op;
  const type_t* carries;
  int num_tiles;

  MGPU_DEVICE void operator()(int tid, int cta) const {
    typedef typename launch_t::sm_ptx params_t;
    enum { nt = params_t::nt, vt = params_t::vt, nv = nt * vt,
      W = chunk_width_t<type_t, vt>::value, chunks = vt / W };
    typedef tile_layout_t<W> layout_t;
    typedef cta_scan_t<nt, type_t> scan_t;
    int tile = xcd_tile(cta, num_tiles);
    if(tile >= num_tiles) return;

    __shared__ struct {
      alignas(16) type_t values[layout_t::capacity(nv)];
      typename scan_t::storage_t scan;
    } shared;

    range_t range = get_tile(tile, nv, count);
    int tile_count = range.count();
    bool interior = nv == tile_count;
    type_t carry_in = tile ? carries[tile] : type_t();

    array_t<type_t, vt> x;
    scan_load_tile<nt, vt>(input, range.begin, tile_count, interior, tid,
      shared.values, x.data);

    array_t<type_t, vt> y = scan_t().template scan<vt>(tid, x, shared.scan,
      carry_in, tile > 0, tile_count, op, type_t(), scan_type).scan;

    scan_store_tile<nt, vt>(y, output, range.begin, tile_count, interior,
      tid, shared.values);
  }
};

// Values per thread of the one-CTA kernels (the spine, and the last step of
// reduce): 8 for types of up to 8 bytes, fewer for wider ones so that the
// 1,024-thread tile stays at 64 KB of LDS.
template<typename type_t>
struct spine_vt_t {
  enum {
    value = sizeof(type_t) <= 8 ? 8 :
      (64 / sizeof(type_t) > 1 ? 64 / sizeof(type_t) : 1)
  };
};

enum {
  scan_spine_nt = 1024, scan_spine_vt = 8,
  // At most this many items are scanned by the spine CTA alone, and at most
  // this many partials before the partials get a scan of their own.
  scan_small_count = 2 * scan_spine_nt * scan_spine_vt,
  scan_spine_limit = 32 * scan_spine_nt * scan_spine_vt
};

// Partials needed for `count` items cut into tiles of nv, over all levels.
MGPU_HOST_DEVICE size_t scan_partials_count(int64_t count, int nv) {
  size_t total = 0;
  while(count > scan_small_count) {
    count = div_up(count, (int64_t)nv);
    total += (size_t)(count + 63) / 64 * 64;
    if(count <= scan_spine_limit) break;
  }
  return total;
}

inline void scan_record(hipEvent_t event, context_t& context) {
  hipError_t result = hipEventRecord(event, context.stream());
  if(hipSuccess != result) throw cuda_exception_t(result);
}

// What a scan of more than scan_small_count items does once partials[tile]
// holds the fold of every tile of nv items: the scan of the partials, the
// total to *reduction, the downsweep.
template<scan_type_t scan_type, typename launch_t, typename input_it,
  typename output_it, typename type_t, typename op_t, typename reduction_it>
void scan_finish(input_it input, int count, output_it output, op_t op,
  reduction_it reduction, type_t* partials, context_t& context,
  hipEvent_t event = nullptr);

// The scan with its temporaries in caller-provided device memory:
// scan_partials_count(count, nv) values of type_t.
// The event, when not null, is recorded as soon as the reduction has been
// written.
template<scan_type_t scan_type, typename launch_t, typename input_it,
  typename output_it, typename type_t, typename op_t, typename reduction_it>
void scan_launch(input_it input, int count, output_it output, op_t op,
  reduction_it reduction, type_t* partials, context_t& context,
  hipEvent_t event = nullptr) {

  int nv = launch_t::nv(context);
  if(count <= scan_small_count) {
    // Few items (or none: the reduction is type_t()): one CTA does it all.
    scan_spine_f<scan_type, scan_spine_nt, spine_vt_t<type_t>::value,
      input_it, output_it, type_t, op_t, reduction_it>
      k { input, count, output, op, reduction };
    cta_launch<scan_spine_nt>(k, 1, context);
    if(event) scan_record(event, context);
    return;
  }

  int num_tiles = div_up(count, nv);
  scan_upsweep_f<launch_t, input_it, type_t, op_t>
    up { input, count, op, partials, num_tiles };
  cta_launch<launch_t>(up, xcd_grid(num_tiles), context);
  scan_finish<scan_type, launch_t>(input, count, output, op, reduction,
    partials, context, event);
}

template<scan_type_t scan_type, typename launch_t, typename input_it,
  typename output_it, typename type_t, typename op_t, typename reduction_it>
void scan_finish(input_it input, int count, output_it output, op_t op,
  reduction_it reduction, type_t* partials, context_t& context,
  hipEvent_t event) {

  int nv = launch_t::nv(context);
  int num_tiles = div_up(count, nv);
  if(num_tiles <= scan_spine_limit) {
    scan_spine_f<scan_type_exc, scan_spine_nt, spine_vt_t<type_t>::value,
      const type_t*, type_t*, type_t, op_t, reduction_it>
      k { partials, num_tiles, partials, op, reduction };
    cta_launch<scan_spine_nt>(k, 1, context);
  } else {
    scan_launch<scan_type_exc, launch_t>((const type_t*)partials, num_tiles,
      partials, op, reduction, partials + (num_tiles + 63) / 64 * 64,
      context);
  }
  if(event) scan_record(event, context);

  scan_downsweep_f<scan_type, launch_t, input_it, output_it, type_t, op_t>
    down { input, count, output, op, partials, num_tiles };
  cta_launch<launch_t>(down, xcd_grid(num_tiles), context);
}

} // namespace detail

// The event, when not null, is recorded once the reduction has been written
// (before the downsweep), so that a caller who only needs the total -- to
// size its next allocation, say -- can wait for that alone.
template<scan_type_t scan_type = scan_type_exc,
  typename launch_arg_t = empty_t, typename input_it,
  typename output_it, typename op_t, typename reduction_it>
void scan_event(input_it input, int count, output_it output, op_t op,
  reduction_it reduction, context_t& context, hipEvent_t event) {

  if(detail::launcher_scan<launch_arg_t>(scan_type_inc == scan_type, input,
    count, output, op, reduction, context, event)) return;
  typedef typename std::iterator_traits<input_it>::value_type type_t;
  typedef typename conditional_typedef_t<launch_arg_t,
    typename detail::scan_launch_default_t<type_t>::type_t_>::type_t launch_t;

  mem_t<type_t> partials(detail::scan_partials_count(count,
    launch_t::nv(context)), context);
  detail::scan_launch<scan_type, launch_t>(input, count, output, op,
    reduction, partials.data(), context, event);
}

template<scan_type_t scan_type = scan_type_exc,
  typename launch_arg_t = empty_t, typename input_it,
  typename output_it, typename op_t, typename reduction_it>
void scan(input_it input, int count, output_it output, op_t op,
  reduction_it reduction, context_t& context) {
  scan_event<scan_type, launch_arg_t>(input, count, output, op, reduction,
    context, (hipEvent_t)nullptr);
}

// Sum scan without a reduction output.
template<scan_type_t scan_type = scan_type_exc,
  typename launch_arg_t = empty_t, typename input_it, typename output_it>
void scan(input_it input, int count, output_it output, context_t& context) {
  typedef typename std::iterator_traits<input_it>::value_type type_t;
  scan<scan_type, launch_arg_t>(input, count, output, plus_t<type_t>(),
    discard_iterator_t<type_t>(), context);
}

// Scan of f(index), index in [0, count).
template<typename type_t, scan_type_t scan_type = scan_type_exc,
  typename launch_arg_t = empty_t, typename func_t, typename output_it,
  typename op_t, typename reduction_it>
void transform_scan_event(func_t f, int count, output_it output, op_t op,
  reduction_it reduction, context_t& context, hipEvent_t event) {
  scan_event<scan_type, launch_arg_t>(make_load_iterator<type_t>(f), count,
    output, op, reduction, context, event);
}

template<typename type_t, scan_type_t scan_type = scan_type_exc,
  typename launch_arg_t = empty_t, typename func_t, typename output_it,
  typename op_t, typename reduction_it>
void transform_scan(func_t f, int count, output_it output, op_t op,
  reduction_it reduction, context_t& context) {
  transform_scan_event<type_t, scan_type, launch_arg_t>(f, count, output, op,
    reduction, context, (hipEvent_t)nullptr);
}

END_MGPU_NAMESPACE
