// mgpu for AMD CDNA4: segmented reduction, transform_segreduce and CSR spmv.
//
//   output[s] = input[segments[s]] op ... op input[segments[s + 1] - 1]
// (the last segment ends at count); an empty segment yields init and init is
// not folded into non-empty ones.  segments[0] must be 0, starts ascend.
// Public interface after src/moderngpu/kernel_segreduce.hxx:193-298.
//
// Structure (three kinds of kernel on the context's stream):
//   K1  load_balance_partitions cuts the merge of items and segment starts
//       into tiles of nv merged elements (search.hxx).  Not launched for a
//       call of up to 4,096 tiles: each tile then finds its two splits itself
//       with a 64-ary search by one wavefront per split.
//   K2  segreduce_tile_f: one CTA per tile.
//         - the tile's items are fetched with 16-byte loads in strided order
//           (unaligned starts are fine for global_load_dwordx4) and written
//           to LDS in a padded thread-order layout;
//         - meanwhile the tile's segment starts set one bit per start in an
//           LDS bitmask (ds_or_b32);
//         - each thread runs a flag-driven inclusive segmented scan over its
//           vt consecutive items in registers and writes the scanned values
//           back in place, so LDS slot e now holds the fold of its segment
//           from max(segment start, thread start) to e;
//         - one cta_segscan_t over the thread totals gives every thread the
//           fold that flows into it;
//         - one thread per segment start then picks the slot where its
//           segment ends in the tile, adds the flow into that slot's thread if
//           the segment began in an earlier thread, and stores output[s].
//       The segment that was already open when the tile began is reported as
//       a (segment, partial) carry for the spine.
//   K3  segreduce_spine_f folds the per-tile carries of segments that span
//       tiles into output[] in one launch (256 carries per CTA; a run of
//       carries that crosses CTAs is finished by the CTA it ends in).
// The CUDA reference instead walks vt + 1 merged elements per thread through
// dependent shared-memory reads and runs a recursive fix-up, one launch per
// level.
#pragma once
#include "search.hxx"
#include "cta_load_balance.hxx"
#include "cta_segscan.hxx"
#include "cta_segreduce.hxx"
#include "launcher.hxx"
#include "cta_reduce.hxx"
#include "transform.hxx"
#include "memory.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

////////////////////////////////////////////////////////////////////////////////
// The fused spmv load: matrix[k] * vector[columns[k]], with the matrix values
// and column indices of W consecutive nonzeros fetched as 16-byte loads.
template<typename type_t>
struct spmv_input_t {
  typedef type_t value_type;
  const type_t* matrix;
  const int* columns;
  const type_t* vector;
  MGPU_DEVICE type_t operator[](int k) const {
    return matrix[k] * vector[columns[k]];
  }
};
template<typename type_t, int W>
struct tile_loader_t<spmv_input_t<type_t>, type_t, W> {
  MGPU_DEVICE static void load(spmv_input_t<type_t> in, int base,
    unsigned offset, type_t (&x)[W]) {
    type_t a[W];
    int c[W];
    pointer_loader_t<type_t, W>::load(in.matrix, base, offset, a);
    // Columns are 4-byte: W of them are 16 bytes or less.
    if constexpr(W > 1) {
      typedef typename vec_t<int, W>::type_u v_t;
      v_t v = *(const v_t*)(in.columns + base + offset);
      PRAGMA_UNROLL
      for(int e = 0; e < W; ++e) c[e] = v[e];
    } else
      c[0] = in.columns[base + offset];
    PRAGMA_UNROLL
    for(int e = 0; e < W; ++e) x[e] = a[e] * in.vector[c[e]];
  }
};

////////////////////////////////////////////////////////////////////////////////
// One step of the thread-serial segmented scan: the running fold `prev`
// continues into `cur` unless bit i of `bits` marks a segment start at this
// item.  The generic form is a compare and a select around op().  For the
// built-in operators on 4/8-byte arithmetic types the select is done with bit
// arithmetic on a mask spread from the flag bit (one v_bfe_i32; written as
// inline assembly because the compiler otherwise turns the mask back into a
// compare, a lane mask in SGPRs and a select):
//   plus:     cur + (prev & keep), keep = all ones unless a segment starts
//   max/min:  op(start ? cur : prev, cur) with one bitfield-insert per 32-bit
//             word for the choice; op(cur, cur) == cur.
// For floating-point plus a segment made only of -0.0 sums to +0.0; sums are
// compared with a tolerance, and max/min stay bit-exact.

template<typename op_t, typename type_t, typename enable_t = void>
struct segscan_step_t {
  // nbits = complement of the start bits.
  template<int i>
  MGPU_DEVICE static type_t step(type_t prev, type_t cur, unsigned nbits,
    op_t op) {
    return ((nbits >> i) & 1) ? op(prev, cur) : cur;
  }
};

template<typename type_t>
struct bitwise_word_t {
  typedef typename std::conditional<sizeof(type_t) == 8, unsigned long long,
    unsigned>::type type;
  MGPU_DEVICE static type to(type_t x) {
    type y; __builtin_memcpy(&y, &x, sizeof(y)); return y;
  }
  MGPU_DEVICE static type_t from(type y) {
    type_t x; __builtin_memcpy(&x, &y, sizeof(x)); return x;
  }
  // All ones if bit i of bits is set, else zero.
  template<int i>
  MGPU_DEVICE static type spread(unsigned bits) {
    int m;
    asm("v_bfe_i32 %0, %1, %2, 1" : "=v"(m) : "v"(bits), "n"(i));
    return (type)(long long)m;
  }
};

template<typename type_t>
struct is_word_arithmetic_t {
  enum { value = std::is_arithmetic<type_t>::value &&
    (sizeof(type_t) == 4 || sizeof(type_t) == 8) };
};

template<typename type_t>
struct segscan_step_t<plus_t<type_t>, type_t,
  enable_if_t<is_word_arithmetic_t<type_t>::value> > {
  template<int i>
  MGPU_DEVICE static type_t step(type_t prev, type_t cur, unsigned nbits,
    plus_t<type_t>) {
    typedef bitwise_word_t<type_t> w;
    return w::from(w::to(prev) & w::template spread<i>(nbits)) + cur;
  }
};

template<typename op_t, typename type_t>
struct segscan_select_step_t {
  template<int i>
  MGPU_DEVICE static type_t step(type_t prev, type_t cur, unsigned nbits,
    op_t op) {
    typedef bitwise_word_t<type_t> w;
    typename w::type keep = w::template spread<i>(nbits);
    return op(w::from((keep & w::to(prev)) | (~keep & w::to(cur))), cur);
  }
};
template<typename type_t>
struct segscan_step_t<maximum_t<type_t>, type_t,
  enable_if_t<is_word_arithmetic_t<type_t>::value> > :
  segscan_select_step_t<maximum_t<type_t>, type_t> { };
template<typename type_t>
struct segscan_step_t<minimum_t<type_t>, type_t,
  enable_if_t<is_word_arithmetic_t<type_t>::value> > :
  segscan_select_step_t<minimum_t<type_t>, type_t> { };

// x[i] = step<i>(x[i - 1], x[i]) for i = first .. vt - 1.
template<int i, int vt>
struct segscan_thread_t {
  template<typename op_t, typename type_t>
  MGPU_DEVICE static void run(type_t (&x)[vt], unsigned nbits, op_t op) {
    x[i] = segscan_step_t<op_t, type_t>::template step<i>(x[i - 1], x[i],
      nbits, op);
    segscan_thread_t<i + 1, vt>::run(x, nbits, op);
  }
};
template<int vt>
struct segscan_thread_t<vt, vt> {
  template<typename op_t, typename type_t>
  MGPU_DEVICE static void run(type_t (&)[vt], unsigned, op_t) { }
};

////////////////////////////////////////////////////////////////////////////////
// Default tiles on gfx950: 16 values per thread, 256 threads for 4-byte values
// and 128 for 8-byte ones (16 KB of values in LDS either way); wider value
// types get fewer values per thread so that the tile stays under the 64 KB a
// workgroup may declare.

template<typename type_t>
struct segreduce_launch_default_t {
  enum {
    vt = sizeof(type_t) <= 8 ? 16 :
      (128 / sizeof(type_t) > 1 ? 128 / sizeof(type_t) : 1)
  };
  // 8-byte values: half the threads for the same bytes per tile.
  typedef launch_box_t<arch_gfx950_cta<(sizeof(type_t) == 8 ? 128 : 256),
    vt> > type_t_;
};

////////////////////////////////////////////////////////////////////////////////
// What a tile (or a spine CTA) passes on: the segment its leading partial
// belongs to, and whether output[segment] still has to be created ("fresh")
// rather than combined with.  seg >= 0: combine; ~seg (negative): fresh;
// none: nothing to pass on.

struct carry_code_t {
  enum : int { none = (int)0x80000000 };
  MGPU_HOST_DEVICE static int make(int seg, bool fresh) {
    return fresh ? ~seg : seg;
  }
  MGPU_HOST_DEVICE static int seg(int code) {      // -1 for none
    return none == code ? -1 : (code < 0 ? ~code : code);
  }
  MGPU_HOST_DEVICE static bool fresh(int code) { return code < 0; }
};

////////////////////////////////////////////////////////////////////////////////
// Items that are not read but computed per (index, segment, rank): the input
// of lbs_segreduce.  The tile kernel runs the load-balancing search of the
// tile first -- its LDS is handed back before the reduction needs any -- and
// calls f(index, seg, rank, cached values, args...) for every item of the
// tile.

template<typename func_t, typename pointers_t, typename type_t>
struct lbs_input_t {
  typedef type_t value_type;
  func_t f;
  pointers_t caching_iterators;
};

template<typename input_it>
struct is_lbs_input_t : std::false_type { };
template<typename func_t, typename pointers_t, typename type_t>
struct is_lbs_input_t<lbs_input_t<func_t, pointers_t, type_t> > :
  std::true_type { };

// LDS the item source needs while it produces a tile's items.
template<typename input_it, int nt, int vt>
struct tile_source_storage_t {
  typedef empty_t type;
};
template<typename func_t, typename pointers_t, typename type_t, int nt,
  int vt>
struct tile_source_storage_t<lbs_input_t<func_t, pointers_t, type_t>, nt,
  vt> {
  struct type {
    typename cta_load_balance_t<nt, vt>::storage_t lbs;
    typename cached_segment_load_t<nt, pointers_t>::storage_t cached;
  };
};

////////////////////////////////////////////////////////////////////////////////
// K2

// own_splits: launched without a partition array, the tile finds its two
// splits itself (calls of few tiles, see segreduce_launch).  A separate
// instantiation, because the search in front costs the kernel of large
// calls time even when it is only branched around (2^26 floats: 49.8
// against 49.2 us per call).
template<typename launch_t, typename input_it, typename segments_it,
  typename output_it, typename op_t, typename type_t, bool own_splits = false>
struct segreduce_tile_f {
  input_it input;
  int count;
  segments_it segments;
  int num_segments;
  output_it output;
  op_t op;
  type_t init;
  const int* mp_data;
  type_t* carry_values;
  int* carry_codes;
  int num_tiles;

  typedef typename launch_t::sm_ptx params_t;
  enum {
    nt = params_t::nt, vt = params_t::vt, nv = nt * vt,
    W = chunk_width_t<type_t, vt>::value,
    chunks = vt / W,
    flag_words = nv / 32 + 2
  };
  static_assert(vt <= 32, "segreduce tiles hold at most 32 values/thread");
  enum {
    // dense_tile() keeps the tile's starts in the part of the values' LDS
    // that the items leave free, which they do for values of 4 bytes or more
    // (a_count + b_count <= nv) that are aligned like an int.
    can_stage_starts = sizeof(type_t) >= sizeof(int) &&
      0 == alignof(type_t) % alignof(int),
    // Rows of nt 16-byte loads that cover the b_count + 1 <= nv + 1 starts.
    start_rows = (nv + 4 * nt) / (4 * nt),
    // Longest run of items a single thread folds by itself there.
    fold_max = 32,
    // Starts (and the start after each) that a thread of an ordinary tile
    // reads ahead into registers; tiles with more than start_regs * nt starts
    // go to dense_tile().  Four for values of up to 4 bytes; wider values
    // have fewer registers to spare (2^27 doubles in four long segments: 186-
    // 188 us with three or four against 184-185 us with two).
#ifdef MGPU_SEGREDUCE_START_REGS
    start_regs = MGPU_SEGREDUCE_START_REGS
#else
    start_regs = sizeof(type_t) <= 4 ? 4 : 2
#endif
  };
  typedef tile_layout_t<W> layout_t;
  typedef cta_segscan_t<nt, type_t> segscan_t;
  typedef tile_loader_t<input_it, type_t, W> loader_t;

  struct work_storage_t {
    alignas(16) type_t values[layout_t::capacity(nv)];
    type_t flow[nt];              // fold flowing into each thread
    unsigned flags[flag_words];   // bit p: a segment starts at tile item p
    typename segscan_t::storage_t segscan;
  };
  // What produces the items may use the same LDS before the reduction does.
  union storage_t {
    work_storage_t work;
    typename tile_source_storage_t<input_it, nt, vt>::type source;
    MGPU_DEVICE storage_t() { }     // members may have constructors
  };

  template<typename... args_t>
  MGPU_DEVICE void operator()(int tid, int cta, args_t... args) const {
    // Neighbouring tiles run on the same XCD (see xcd_tile_eighths).
    cta = xcd_tile_eighths(cta, num_tiles);
    if(cta >= num_tiles) return;
    __shared__ storage_t shared;

    int mp0, mp1;
    if constexpr(!own_splits) {
      mp0 = mp_data[cta];
      mp1 = mp_data[cta + 1];
    } else {
      // No partition kernel has run: one wavefront per end of the tile
      // finds the split.
      __shared__ int own[2];
      int total = count + num_segments;
      for(int end = tid / warp_size; end < 2; end += nt / warp_size) {
        int diag = (int)min((int64_t)nv * (cta + end), (int64_t)total);
        int split = merge_path_wave<bounds_upper>(
          counting_iterator_t<int>(0), count, segments, num_segments, diag,
          less_t<int>(), tid % warp_size);
        if(0 == tid % warp_size) own[end] = split;
      }
      __syncthreads();
      mp0 = own[0];
      mp1 = own[1];
    }
    merge_range_t range = tile_range(count, num_segments, cta, nv, mp0, mp1);
    // A tile that lies nv items or more in front of the end of the input
    // reads nv items whatever its a_count is: what it reads past its own
    // last item belongs to the next tile and is never looked at, and no
    // load or LDS store needs a per-lane bounds check.  The kernel body
    // exists once for such tiles and once with the checks.
    // Computed items exist for the tile's own index range only.
    // A tile with more segment starts than threads goes another way
    // (dense_tile).
    if constexpr(can_stage_starts) {
      if(range.b_count() > start_regs * nt) {
        dense_tile(tid, cta, range, shared, args...);
        return;
      }
    }
    if(!is_lbs_input_t<input_it>::value && range.a_begin <= count - nv)
      tile(std::true_type(), tid, cta, range, shared, args...);
    else
      tile(std::false_type(), tid, cta, range, shared, args...);
  }

  // The items of a tile computed from its load-balancing search, in the
  // strided chunk order the reduction expects.
  template<typename... args_t>
  MGPU_DEVICE void compute_items(merge_range_t range, int tid,
    type_t (&r)[chunks][W], storage_t& shared, args_t... args) const {
    if constexpr(is_lbs_input_t<input_it>::value) {
      typedef cta_load_balance_t<nt, vt> load_balance_t;
      typedef typename load_balance_t::layout_t slot_layout_t;
      typedef decltype(input.caching_iterators) pointers_t;
      typedef cached_segment_load_t<nt, pointers_t> cached_load_t;
      int a_count = range.a_count();
      int seg_base = range.b_begin - 1;
      // The cached values' read is in flight while the tile is decoded.
      typename cached_load_t::fetched_t fetched;
      bool staged = cached_load_t::fetch(tid, seg_base, range.b_count() + 1,
        input.caching_iterators, fetched);
      load_balance_t().fill(range, segments, tid, shared.source.lbs);
      cached_load_t::commit(tid, seg_base, range.b_count() + 1, fetched,
        shared.source.cached, input.caching_iterators);
      const int* slots = shared.source.lbs.indices;
      const int* starts = slots + load_balance_t::starts_offset(a_count);
      PRAGMA_UNROLL
      for(int i = 0; i < chunks; ++i) {
        PRAGMA_UNROLL
        for(int e = 0; e < W; ++e) {
          int p = W * (nt * i + tid) + e;
          if(p < a_count) {
            int rel = slots[slot_layout_t::index(p)];
            int seg = seg_base + rel;
            int index = range.a_begin + p;
            r[i][e] = input.f(index, seg, index - starts[rel],
              cached_load_t::get(staged, rel, seg, shared.source.cached,
                input.caching_iterators), args...);
          }
        }
      }
      // The search's LDS is about to hold the values.
      __syncthreads();
    }
  }

  // Steps 3 to 5 of the tile: the items are in LDS (padded layout) and the
  // start bits in shared.flags; afterwards LDS slot e holds the fold of its
  // segment from max(segment start, start of e's thread) to e, and
  // shared.flow[t] the fold that flows into thread t.  Ends with a barrier.
  template<typename interior_t>
  MGPU_DEVICE void scan_items(interior_t, int tid, int a_count,
    work_storage_t& shared) const {
    enum { interior = interior_t::value };
    // Thread order: items [vt * tid, vt * tid + vt) and their start bits.
    type_t x[vt];
    PRAGMA_UNROLL
    for(int c = 0; c < chunks; ++c) {
      type_t chunk[W];
      lds_load_chunk<W>(shared.values + layout_t::index(vt * tid + W * c),
        chunk);
      PRAGMA_UNROLL
      for(int e = 0; e < W; ++e) x[W * c + e] = chunk[e];
    }
    unsigned bits;
    {
      int pos = vt * tid;
      unsigned long long two = shared.flags[pos >> 5] |
        ((unsigned long long)shared.flags[(pos >> 5) + 1] << 32);
      bits = (unsigned)(two >> (pos & 31));
      if(vt < 32) bits &= (1u << vt) - 1;
    }

    // Inclusive segmented scan of the thread's items, left to right.
    segscan_thread_t<1, vt>::run(x, ~bits, op);

    PRAGMA_UNROLL
    for(int c = 0; c < chunks; ++c) {
      type_t chunk[W];
      PRAGMA_UNROLL
      for(int e = 0; e < W; ++e) chunk[e] = x[W * c + e];
      if(interior || vt * tid + W * c < a_count)
        lds_store_chunk<W>(shared.values + layout_t::index(vt * tid + W * c),
          chunk);
    }

    segscan_result_t<type_t> flow = segscan_t().segscan(tid, 0 != bits, true,
      x[vt - 1], shared.segscan, init, op);
    shared.flow[tid] = flow.scan;
    __syncthreads();

  }

  // Fold of tile items [p .. e] after scan_items(), where no segment starts
  // inside (p, e].
  MGPU_DEVICE type_t fold_to(const work_storage_t& shared, int p, int e) const {
    int te = e / vt;
    type_t v = shared.values[layout_t::index(e)];
    // thread 0 has nothing flowing in; p may be negative for the segment
    // that was open when the tile began.
    if(te && p < te * vt) v = op(shared.flow[te], v);
    return v;
  }

  // Fold of the tile's items [p, e), e > p, as they were loaded (before any
  // scan), left to right by one thread.  (Reading two or four items ahead
  // made tiles of 3- and 8-item segments 5 to 15 % slower.)
  MGPU_DEVICE type_t fold_items(const work_storage_t& shared, int p,
    int e) const {
    type_t v = shared.values[layout_t::index(p)];
    for(int q = p + 1; q < e; ++q)
      v = op(v, shared.values[layout_t::index(q)]);
    return v;
  }

  // The segment that was open when the tile began owns items [0, f), whose
  // fold is `partial`.  Its code tells the spine which segment to fold the
  // partial into, and whether that segment already has a value in output[]:
  // it does unless its start was the very last merged element of its own tile
  // (then that tile held none of its items and wrote nothing).  open_start is
  // the start of that segment.  Called by one thread.
  MGPU_DEVICE void emit_carry(int cta, merge_range_t range, int f,
    int open_start, type_t partial) const {
    if(f > 0 && range.b_begin > 0) {
      int seg = range.b_begin - 1;
      int node = open_start + seg;              // merged position of start
      bool fresh = 0 == (node + 1) % nv;
      carry_values[cta] = partial;
      carry_codes[cta] = carry_code_t::make(seg, fresh);
    } else {
      carry_values[cta] = init;
      carry_codes[cta] = carry_code_t::none;
    }
  }

  template<typename interior_t, typename... args_t>
  MGPU_DEVICE void tile(interior_t, int tid, int cta, merge_range_t range,
    storage_t& storage, args_t... args) const {
    enum { interior = interior_t::value };
    work_storage_t& shared = storage.work;
    int a_count = range.a_count();
    int b_count = range.b_count();

    // Everything the tile needs from segments[] is fetched first, ahead of
    // the item loads, so that the start bits can be set while the items are
    // still in flight and no global load sits on the critical path after
    // the scan: this thread's start, the start after it, and (thread 0) the
    // start of the segment that is open when the tile begins.
    int first_start = 0, first_next = 0, open_start = 0;
    if(tid < b_count) {
      int seg = range.b_begin + tid;
      first_start = segments[seg];
      first_next = (seg + 1 < num_segments) ? (int)segments[seg + 1] : count;
    }
    // ... and the same for further starts of the thread, nt apart (tiles of
    // up to start_regs * nt starts come this way).
    int more_start[start_regs - 1 > 0 ? start_regs - 1 : 1];
    int more_next[start_regs - 1 > 0 ? start_regs - 1 : 1];
    PRAGMA_UNROLL
    for(int k = 1; k < start_regs; ++k) {
      more_start[k - 1] = more_next[k - 1] = 0;
      if(nt * k + tid < b_count) {
        int seg = range.b_begin + nt * k + tid;
        more_start[k - 1] = segments[seg];
        more_next[k - 1] = (seg + 1 < num_segments) ? (int)segments[seg + 1] :
          count;
      }
    }
    if(!tid && range.b_begin > 0) open_start = segments[range.b_begin - 1];
    // The item loads; they are consumed after the flag setup.
    type_t r[chunks][W];
    if constexpr(is_lbs_input_t<input_it>::value) {
      compute_items(range, tid, r, storage, args...);
    } else if constexpr(interior) {
      PRAGMA_UNROLL
      for(int i = 0; i < chunks; ++i)
        loader_t::load(input, range.a_begin, (unsigned)(W * (nt * i + tid)),
          r[i]);
    } else {
      PRAGMA_UNROLL
      for(int i = 0; i < chunks; ++i) {
        int p = W * (nt * i + tid);
        if(p + W <= a_count)
          loader_t::load(input, range.a_begin, (unsigned)p, r[i]);
        else {
          PRAGMA_UNROLL
          for(int e = 0; e < W; ++e)
            if(p + e < a_count) r[i][e] = input[range.a_begin + p + e];
        }
      }
    }

    for(int w = tid; w < flag_words; w += nt) shared.flags[w] = 0;
    __syncthreads();

    // One bit per segment start.  Starts of this tile lie in
    // [a_begin, a_end]; the clamp only guards against malformed input.
    for(int j = tid; j < b_count; j += nt) {
      int s = first_start;
      if(j != tid) {
        int k = (j - tid) / nt;
        s = 0;
        bool held = false;
        PRAGMA_UNROLL
        for(int q = 1; q < start_regs; ++q)
          if(q == k) { s = more_start[q - 1]; held = true; }
        if(!held) s = (int)segments[range.b_begin + j];
      }
      int p = min(max(s - range.a_begin, 0), a_count);
      atomicOr(&shared.flags[p >> 5], 1u << (p & 31));
    }

    PRAGMA_UNROLL
    for(int i = 0; i < chunks; ++i) {
      int p = W * (nt * i + tid);
      if(interior || p < a_count)
        lds_store_chunk<W>(shared.values + layout_t::index(p), r[i]);
    }
    __syncthreads();

    scan_items(interior_t(), tid, a_count, shared);

    // One thread per segment start of the tile.
    for(int j = tid; j < b_count; j += nt) {
      int seg = range.b_begin + j;
      int s = first_start, next = first_next;
      if(j != tid) {
        int k = (j - tid) / nt;
        bool held = false;
        PRAGMA_UNROLL
        for(int q = 1; q < start_regs; ++q)
          if(q == k) { s = more_start[q - 1]; next = more_next[q - 1]; held = true; }
        if(!held) {
          s = segments[seg];
          next = (seg + 1 < num_segments) ? (int)segments[seg + 1] : count;
        }
      }
      int p = s - range.a_begin;
      if(next <= s) output[seg] = init;                  // empty segment
      else if(p >= 0 && p < a_count) {
        int e = min(next, range.a_end) - range.a_begin - 1;
        output[seg] = fold_to(shared, p, e);
      }
      // else: the segment's first item is in the next tile; the spine
      // writes it.
    }

    if(!tid) {
      int f = a_count;
      if(b_count) f = min(max(first_start - range.a_begin, 0), a_count);
      emit_carry(cta, range, f, open_start,
        f > 0 ? fold_to(shared, -1, f - 1) : init);
    }
  }

  // A tile with more segment starts than threads (segments of fewer than
  // vt items on average).  What the ordinary path does per start -- an LDS
  // atomic for its bit, a read of the start and of the one after it from
  // global memory by whichever thread gets to write the segment's result --
  // is most of the work of such a tile, so here the starts are read once,
  // with 16-byte loads issued up front, and kept in LDS: in the part of the
  // values' array that the items leave free (a_count + b_count <= nv).  If no
  // segment has more than fold_max items inside the tile, the flag bits, the
  // segmented scan and the CTA scan are left out altogether: one thread per
  // start folds its segment's items straight from LDS, left to right, and
  // stores the result.  Otherwise the tile continues as the ordinary path
  // does, with its starts coming from LDS.
  template<typename... args_t>
  MGPU_DEVICE void dense_tile(int tid, int cta, merge_range_t range,
    storage_t& storage, args_t... args) const {
    work_storage_t& shared = storage.work;
    int a_count = range.a_count();
    int b_count = range.b_count();
    // st[j] = start of segment b_begin + j for j in [0, b_count]; the start
    // "after the last segment" is count.
    int* st = (int*)(shared.values + layout_t::capacity(nv)) - (b_count + 1);
    int open_start = 0;
    if(!tid && range.b_begin > 0) open_start = segments[range.b_begin - 1];

    // Computed items need the LDS for themselves first.
    type_t r[chunks][W];
    if constexpr(is_lbs_input_t<input_it>::value)
      compute_items(range, tid, r, storage, args...);

    int fetched[start_rows][4];
    int available = min(b_count + 1, num_segments - range.b_begin);
    PRAGMA_UNROLL
    for(int row = 0; row < start_rows; ++row) {
      int j = 4 * (nt * row + tid);
      if(j < available)
        cta_load_balance_t<nt, vt>::load_starts(segments, range.b_begin + j,
          range.b_begin + available, fetched[row]);
    }
    if constexpr(!is_lbs_input_t<input_it>::value) {
      PRAGMA_UNROLL
      for(int i = 0; i < chunks; ++i) {
        int p = W * (nt * i + tid);
        if(p + W <= a_count)
          loader_t::load(input, range.a_begin, (unsigned)p, r[i]);
        else {
          PRAGMA_UNROLL
          for(int e = 0; e < W; ++e)
            if(p + e < a_count) r[i][e] = input[range.a_begin + p + e];
        }
      }
    }
    for(int w = tid; w < flag_words; w += nt) shared.flags[w] = 0;
    PRAGMA_UNROLL
    for(int row = 0; row < start_rows; ++row) {
      int j = 4 * (nt * row + tid);
      PRAGMA_UNROLL
      for(int e = 0; e < 4; ++e)
        if(j + e <= b_count)
          st[j + e] = (j + e < available) ? fetched[row][e] : count;
    }
    PRAGMA_UNROLL
    for(int i = 0; i < chunks; ++i) {
      int p = W * (nt * i + tid);
      if(p < a_count)
        lds_store_chunk<W>(shared.values + layout_t::index(p), r[i]);
    }
    __syncthreads();

    // Items [0, f) belong to the segment that was open when the tile began.
    int f = min(max(st[0] - range.a_begin, 0), a_count);
    // The item ranges the starts own inside the tile: [p, e) for start j,
    // empty for an empty segment.  (The clamps only matter for malformed
    // input.)
    auto owned = [&](int j, int& p, int& e) {
      int s = st[j], next = st[j + 1];
      p = min(max(s - range.a_begin, 0), a_count);
      e = min(max(next - range.a_begin, p), a_count);
      return next > s;
    };
    bool longer = !tid && f > fold_max;
    for(int j = tid; j < b_count; j += nt) {
      int p, e;
      owned(j, p, e);
      longer |= e - p > fold_max;
    }

    if(!__syncthreads_or(longer)) {
      for(int j = tid; j < b_count; j += nt) {
        int p, e;
        bool filled = owned(j, p, e);
        if(!filled) output[range.b_begin + j] = init;
        else if(e > p) output[range.b_begin + j] = fold_items(shared, p, e);
        // else: the segment's first item is in the next tile; the spine
        // writes it.
      }
      if(!tid)
        emit_carry(cta, range, f, open_start,
          f > 0 ? fold_items(shared, 0, f) : init);
      return;
    }

    // Some segment is long: bits, scan and flow as in the ordinary path.
    for(int j = tid; j < b_count; j += nt) {
      int p = min(max(st[j] - range.a_begin, 0), a_count);
      atomicOr(&shared.flags[p >> 5], 1u << (p & 31));
    }
    __syncthreads();
    scan_items(std::false_type(), tid, a_count, shared);
    for(int j = tid; j < b_count; j += nt) {
      int p, e;
      bool filled = owned(j, p, e);
      if(!filled) output[range.b_begin + j] = init;
      else if(e > p) output[range.b_begin + j] = fold_to(shared, p, e - 1);
    }
    if(!tid)
      emit_carry(cta, range, f, open_start,
        f > 0 ? fold_to(shared, -1, f - 1) : init);
  }
};

////////////////////////////////////////////////////////////////////////////////
// K3: fold carries into the output, one launch.  codes[i] says which segment
// tile i carried into (carry_code_t); carries of one segment are consecutive
// ("a run").  A CTA looks at nt carries.  One segmented scan gives every run
// that ends among them its fold back to the run's first carry or to the
// CTA's first carry, whichever comes later.  A run that was already open at
// the CTA's first carry is completed by the CTA in which it ENDS: its start
// is known in closed form (the tile after the one that holds the segment's
// start, at merged position segments[seg] + seg), so that CTA folds the
// carries in front of its own range cooperatively, in order, straight from
// global memory.  No CTA ever waits for another and nothing is handed to a
// second level.

template<int nt, typename output_it, typename segments_it, typename op_t,
  typename type_t>
struct segreduce_spine_f {
  output_it output;
  const type_t* values;
  const int* codes;
  int n;
  segments_it segments;
  int nv;
  op_t op;
  type_t init;

  MGPU_DEVICE void operator()(int tid, int cta) const {
    typedef cta_segscan_t<nt, type_t> segscan_t;
    __shared__ union {
      typename segscan_t::storage_t segscan;
      struct {
        type_t totals[nt / warp_size];
        bool have[nt / warp_size];
      } fold;
    } shared;
    __shared__ int open_first;

    int base = nt * cta;
    int gid = base + tid;
    int code = (gid < n) ? codes[gid] : (int)carry_code_t::none;
    int seg = carry_code_t::seg(code);
    int prev = (gid > 0 && gid - 1 < n) ?
      carry_code_t::seg(codes[gid - 1]) : -1;
    int next = (gid + 1 < n) ? carry_code_t::seg(codes[gid + 1]) : -1;
    type_t value = (gid < n) ? values[gid] : init;

    bool head = seg != prev || -1 == seg;
    bool carry_out = -1 != seg && seg == next;
    bool run_end = -1 != seg && !carry_out;
    // Fetch the value to combine with while the scan runs.
    bool combine = run_end && !carry_code_t::fresh(code);
    type_t old = init;
    if(combine) old = output[seg];
    if(!tid) open_first = -1;

    segscan_result_t<type_t> result = segscan_t().segscan(tid, head,
      carry_out, value, shared.segscan, init, op);
    if(run_end && result.has_carry_in) value = op(result.scan, value);

    // At most one run is open at `base`; if it ends here, its end thread
    // publishes where it began.
    bool open_run = run_end && !result.has_left_head;
    if(open_run) {
      int node = segments[seg] + seg;
      open_first = min(max(node / nv + 1, 0), base);
    }
    __syncthreads();

    int first = open_first;
    if(first >= 0 && first < base) {
      // Ordered fold of carries [first, base).  A lane takes vt consecutive
      // carries (32 bytes), a wavefront row 64 such chunks; a row is read
      // with full-width loads, folded per lane and then across the lanes in
      // order.  A wavefront takes a contiguous block of rows, a batch of
      // them in flight at a time, and folds their totals in order; thread 0
      // folds the wavefronts' results in order.
      enum {
        num_waves = nt / warp_size,
        vt = sizeof(type_t) <= 16 ? 32 / sizeof(type_t) : 1,
        batch = sizeof(type_t) <= 32 ? 8 : 4
      };
      int lane = tid % warp_size, wave = tid / warp_size;
      int len = base - first;
      int chunks = div_up(len, (int)vt);
      int rows = div_up(chunks, (int)warp_size);
      int rows_per_wave = div_up(rows, (int)num_waves);
      int row0 = rows_per_wave * wave;
      int row1 = min(row0 + rows_per_wave, rows);
      type_t x = init;
      bool have = false;
      for(int r0 = row0; r0 < row1; r0 += batch) {
        // Every load is issued before the first row is folded.  A chunk past
        // the end repeats the last one; the last chunk is moved back to end
        // at `base` (base >= nt > vt, so it stays inside the array) and the
        // skip carries in front of its own part are left out of the fold.
        type_t y[batch][vt];
        int skip[batch];
        PRAGMA_UNROLL
        for(int k = 0; k < batch; ++k) {
          int at = vt * min(warp_size * (r0 + k) + lane, chunks - 1);
          int from = min(at, len - vt);
          skip[k] = at - from;
          PRAGMA_UNROLL
          for(int j = 0; j < vt; ++j)
            y[k][j] = values[first + from + j];
        }
        PRAGMA_UNROLL
        for(int k = 0; k < batch; ++k)
          detail::needed_here(y[k][0]);
        PRAGMA_UNROLL
        for(int k = 0; k < batch; ++k) {
          type_t folded = y[k][0];
          PRAGMA_UNROLL
          for(int j = 1; j < vt; ++j)
            folded = (j <= skip[k]) ? y[k][j] : op(folded, y[k][j]);
          int valid = min(chunks - warp_size * (r0 + k), (int)warp_size);
          type_t total = detail::readlane(wave_scan(folded, op, lane),
            max(valid, 1) - 1);
          if(r0 + k < row1) {
            x = have ? op(x, total) : total;
            have = true;
          }
        }
      }
      if(!lane) {
        shared.fold.totals[wave] = x;
        shared.fold.have[wave] = have;
      }
      __syncthreads();
      if(open_run) {
        type_t front = init;
        bool any = false;
        PRAGMA_UNROLL
        for(int w = 0; w < num_waves; ++w)
          if(shared.fold.have[w]) {
            front = any ? op(front, shared.fold.totals[w]) :
              shared.fold.totals[w];
            any = true;
          }
        value = op(front, value);
      }
    }

    if(run_end) output[seg] = combine ? op(old, value) : value;
  }
};

////////////////////////////////////////////////////////////////////////////////
// Workspace layout for one segreduce call (device memory, 256-byte aligned
// pieces): partitions, then one (code, value) carry per tile.

struct segreduce_workspace_t {
  enum { spine_nt = 256 };
  int num_ctas, num_partitions;
  size_t mp_offset, codes_offset, values_offset, bytes;

  static size_t align(size_t x) { return (x + 255) & ~(size_t)255; }

  segreduce_workspace_t(int count, int num_segments, int nv,
    size_t value_size) {
    int64_t total = (int64_t)count + num_segments;
    num_ctas = (int)((total + nv - 1) / nv);
    num_partitions = num_ctas + 1;
    size_t at = 0;
    mp_offset = at; at = align(at + sizeof(int) * num_partitions);
    codes_offset = at; at = align(at + sizeof(int) * num_ctas);
    values_offset = at; at = align(at + value_size * num_ctas);
    bytes = at;
  }
};

enum {
  phase_partition = 1,    // K1
  phase_tiles = 2,        // K2
  phase_spine = 4,        // K3
  phase_all = 7,
  // With this bit the partition kernel runs whatever the size of the call
  // (tests and measurements of that path on small inputs).
  phase_partition_always = 8
};

// Launches K1, K2 and the spine into caller-provided workspace.  `phases`
// selects a subset for measurement; a later phase then relies on what an
// earlier full call left in the workspace.  (A call of few tiles has no K1:
// its split search is part of the tile phase.)
template<typename launch_t, typename input_it, typename segments_it,
  typename output_it, typename op_t, typename type_t, typename... args_t>
void segreduce_launch(input_it input, int count, segments_it segments,
  int num_segments, output_it output, op_t op, type_t init, void* workspace,
  const segreduce_workspace_t& ws, context_t& context,
  int phases = phase_all, args_t... args) {

  if(!ws.num_ctas) return;
  cta_dim_t cta_dim = launch_t::cta_dim(context);
  char* base = (char*)workspace;
  int* mp_data = (int*)(base + ws.mp_offset);

  // A call of few tiles is bound by its launches, not by its tiles: the
  // tiles then search their own two splits (a few dependent reads that hit
  // the L2) and the partition kernel is not launched.  Measured on 2^14 to
  // 2^26 floats in segments of 64: 6.5 against 10.0 us up to 2^18, 19.4
  // against 20.4 us at 2^24 (4,160 tiles), 32.9 against 30.1 us at 2^25.
  enum { own_splits_max_tiles = 4096 };
  bool own_splits = ws.num_ctas <= own_splits_max_tiles &&
    !(phases & phase_partition_always);
  if(!own_splits && (phases & phase_partition))
    load_balance_partitions_into((int64_t)count, segments, num_segments,
      cta_dim.nv(), mp_data, context);

  type_t* carry_values = (type_t*)(base + ws.values_offset);
  int* carry_codes = (int*)(base + ws.codes_offset);
  if((phases & phase_tiles) && own_splits) {
    segreduce_tile_f<launch_t, input_it, segments_it, output_it, op_t, type_t,
      true> k_reduce { input, count, segments, num_segments, output, op,
        init, nullptr, carry_values, carry_codes, ws.num_ctas };
    cta_launch<launch_t>(k_reduce, xcd_grid(ws.num_ctas), context, args...);
  } else if(phases & phase_tiles) {
    segreduce_tile_f<launch_t, input_it, segments_it, output_it, op_t, type_t>
      k_reduce { input, count, segments, num_segments, output, op, init,
        mp_data, carry_values, carry_codes, ws.num_ctas };
    cta_launch<launch_t>(k_reduce, xcd_grid(ws.num_ctas), context, args...);
  }

  if((phases & phase_spine) && ws.num_ctas > 1) {
    enum { spine_nt = segreduce_workspace_t::spine_nt };
    segreduce_spine_f<spine_nt, output_it, segments_it, op_t, type_t>
      k_spine { output, carry_values, carry_codes, ws.num_ctas, segments,
        cta_dim.nv(), op, init };
    cta_launch<spine_nt>(k_spine, div_up(ws.num_ctas, (int)spine_nt), context);
  }
}

} // namespace detail

////////////////////////////////////////////////////////////////////////////////

template<typename launch_arg_t = empty_t, typename input_it,
  typename segments_it, typename output_it, typename op_t, typename type_t>
void segreduce(input_it input, int count, segments_it segments,
  int num_segments, output_it output, op_t op, type_t init,
  context_t& context);

template<typename launch_arg_t = empty_t, typename func_t,
  typename segments_it, typename output_it, typename op_t, typename type_t>
void transform_segreduce(func_t f, int count, segments_it segments,
  int num_segments, output_it output, op_t op, type_t init,
  context_t& context);

namespace detail {

// Generic iterators: the product is formed element by element.
template<typename matrix_it, typename columns_it, typename vector_it,
  typename segments_it, typename output_it, typename launch_arg_t>
void spmv_dispatch(matrix_it matrix, columns_it columns, vector_it vector,
  int count, segments_it segments, int num_segments, output_it output,
  context_t& context, launch_arg_t) {
  typedef typename std::iterator_traits<matrix_it>::value_type type_t;
  transform_segreduce<launch_arg_t>([=]MGPU_DEVICE(int index) {
    return matrix[index] * ldg(vector + columns[index]);
  }, count, segments, num_segments, output, plus_t<type_t>(),
    (type_t)0, context);
}

// Raw pointers: matrix values and column indices come in as 16-byte loads.
template<typename type_t, typename segments_it, typename output_it,
  typename launch_arg_t>
void spmv_dispatch(const type_t* matrix, const int* columns,
  const type_t* vector, int count, segments_it segments, int num_segments,
  output_it output, context_t& context, launch_arg_t) {
  segreduce<launch_arg_t>(spmv_input_t<type_t> { matrix, columns, vector },
    count, segments, num_segments, output, plus_t<type_t>(), (type_t)0,
    context);
}
template<typename type_t, typename segments_it, typename output_it,
  typename launch_arg_t>
void spmv_dispatch(type_t* matrix, int* columns, type_t* vector, int count,
  segments_it segments, int num_segments, output_it output,
  context_t& context, launch_arg_t) {
  spmv_dispatch((const type_t*)matrix, (const int*)columns,
    (const type_t*)vector, count, segments, num_segments, output, context,
    launch_arg_t());
}

} // namespace detail

template<typename launch_arg_t, typename input_it,
  typename segments_it, typename output_it, typename op_t, typename type_t>
void segreduce(input_it input, int count, segments_it segments,
  int num_segments, output_it output, op_t op, type_t init,
  context_t& context) {

  if(detail::launcher_segreduce<launch_arg_t>(input, count, segments,
    num_segments, output, op, init, context)) return;

  typedef typename conditional_typedef_t<launch_arg_t,
    typename detail::segreduce_launch_default_t<type_t>::type_t_
  >::type_t launch_t;

  cta_dim_t cta_dim = launch_t::cta_dim(context);
  detail::segreduce_workspace_t ws(count, num_segments, cta_dim.nv(),
    sizeof(type_t));
  if(!ws.num_ctas) return;

  mem_t<char> workspace(ws.bytes, context);
  detail::segreduce_launch<launch_t>(input, count, segments, num_segments,
    output, op, init, workspace.data(), ws, context);
}

// segreduce over values generated on the fly: input[i] = f(i).
template<typename launch_arg_t, typename func_t,
  typename segments_it, typename output_it, typename op_t, typename type_t>
void transform_segreduce(func_t f, int count, segments_it segments,
  int num_segments, output_it output, op_t op, type_t init,
  context_t& context) {

  segreduce<launch_arg_t>(make_load_iterator<type_t>(f), count, segments,
    num_segments, output, op, init, context);
}

// Segmented reduction over computed items: output[s] = fold over the items i
// of segment s of f(i, s, i - segments[s], cached values of s, args...);
// empty segments get init.  caching_iterators is a tuple of iterators indexed
// by segment, dereferenced once per segment and tile rather than per item
// (interface after src/moderngpu/kernel_segreduce.hxx:303-404).
template<typename launch_arg_t = empty_t, typename func_t,
  typename segments_it, typename pointers_t, typename output_it,
  typename op_t, typename type_t, typename... args_t>
void lbs_segreduce(func_t f, int count, segments_it segments,
  int num_segments, pointers_t caching_iterators, output_it output, op_t op,
  type_t init, context_t& context, args_t... args) {

  typedef typename conditional_typedef_t<launch_arg_t,
    typename detail::segreduce_launch_default_t<type_t>::type_t_
  >::type_t launch_t;

  cta_dim_t cta_dim = launch_t::cta_dim(context);
  detail::segreduce_workspace_t ws(count, num_segments, cta_dim.nv(),
    sizeof(type_t));
  if(!ws.num_ctas) return;

  mem_t<char> workspace(ws.bytes, context);
  detail::lbs_input_t<func_t, pointers_t, type_t>
    input { f, caching_iterators };
  detail::segreduce_launch<launch_t>(input, count, segments, num_segments,
    output, op, init, workspace.data(), ws, context, detail::phase_all,
    args...);
}

// Without cached values: f(index, seg, rank, args...).
template<typename launch_arg_t = empty_t, typename func_t,
  typename segments_it, typename output_it, typename op_t, typename type_t,
  typename... args_t>
void lbs_segreduce(func_t f, int count, segments_it segments,
  int num_segments, output_it output, op_t op, type_t init,
  context_t& context, args_t... args) {

  lbs_segreduce<launch_arg_t>(
    [=]MGPU_DEVICE(int index, int seg, int rank, tuple<>, args_t... args) {
      return f(index, seg, rank, args...);
    },
    count, segments, num_segments, tuple<>(), output, op, init, context,
    args...
  );
}

// CSR sparse matrix * dense vector.  segments = row starts (num_segments
// entries, no trailing nnz), count = number of nonzeros.
template<typename launch_arg_t = empty_t, typename matrix_it,
  typename columns_it, typename vector_it, typename segments_it,
  typename output_it>
void spmv(matrix_it matrix, columns_it columns, vector_it vector,
  int count, segments_it segments, int num_segments, output_it output,
  context_t& context) {

  if(detail::launcher_spmv<launch_arg_t>(matrix, columns, vector, count,
    segments, num_segments, output, context)) return;
  detail::spmv_dispatch(matrix, columns, vector, count, segments,
    num_segments, output, context, launch_arg_t());
}

END_MGPU_NAMESPACE
