// mgpu for AMD CDNA4: partition kernels.  One search per tile boundary cuts a
// merge (or a load-balancing search) into tiles of `spacing` merged elements;
// the tile kernels then run independently.  Interface after
// src/moderngpu/search.hxx:12-51.
#pragma once

#include "loadstore.hxx"
#include "operators.hxx"
#include "cta_search.hxx"
#include "cta_load_balance.hxx"
#include "memory.hxx"
#include "context.hxx"
#include "launcher.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

// One wavefront finds one merge-path split with a 64-ary search: every round
// the 64 lanes probe 64 evenly spaced cross-diagonal positions at once, a
// ballot counts how many probes still take from A, and the range shrinks by
// 64x.  A scalar binary search needs log2(n) dependent global loads (20 for
// 2^20 segments, each an L2 or HBM round trip); this needs ceil(log64(n)),
// which is what makes the partition kernel cheap next to the tile kernels.
// Must be called by all 64 lanes of a wavefront with the same arguments.
template<bounds_t bounds, typename a_keys_it, typename b_keys_it,
  typename int_t, typename comp_t>
MGPU_DEVICE int_t merge_path_wave(a_keys_it a_keys, int_t a_count,
  b_keys_it b_keys, int_t b_count, int_t diag, comp_t comp, int lane) {

  typedef typename std::iterator_traits<a_keys_it>::value_type type_t;
  int_t lo = (diag > b_count) ? (int_t)(diag - b_count) : (int_t)0;
  int_t hi = (diag < a_count) ? diag : a_count;

  // Invariant: the answer (first position whose probe takes from B) lies in
  // [lo, hi]; probes at positions >= hi are never taken from A.
  while(lo < hi) {
    int_t n = hi - lo;
    int_t stride = (n + 63) / 64;
    int_t mid = lo + (int_t)(lane + 1) * stride - 1;
    bool take_a = false;
    if(mid < hi) {
      type_t a_key = a_keys[mid];
      type_t b_key = b_keys[diag - 1 - mid];
      take_a = (bounds_upper == bounds) ?
        comp(a_key, b_key) : !comp(b_key, a_key);
    }
    int k = popc(ballot(take_a));     // probes [0, k) take from A
    int_t new_lo = lo + (int_t)k * stride;
    int_t new_hi = lo + (int_t)(k + 1) * stride - 1;
    lo = new_lo;
    if(new_hi < hi) hi = new_hi;
  }
  return lo;
}

// Kernel body of merge_path_partitions: one scalar binary search per split,
// p[i] = merge-path split of cross-diagonal min(spacing * i, total).
template<bounds_t bounds, typename int_t, typename a_keys_it,
  typename b_keys_it, typename comp_t>
struct merge_path_partition_f {
  a_keys_it a; b_keys_it b;
  int64_t a_count, b_count, spacing;
  comp_t comp;
  int_t* p;

  MGPU_DEVICE void operator()(int index) const {
    int64_t total = a_count + b_count;
    int64_t d = spacing * index;
    int_t diag = (int_t)(d < total ? d : total);
    p[index] = merge_path<bounds>(a, (int_t)a_count, b, (int_t)b_count,
      diag, comp);
  }
};

// Division of a non-negative int by a fixed positive divisor without the
// integer-division sequence: a shift for powers of two, else one 32x32->64
// multiply by magic = floor(2^(31 + s) / d) + 1 with s = ceil(log2 d), which
// gives the exact quotient for every dividend below 2^31.
struct int_divider_t {
  unsigned magic;       // 0: divisor is a power of two
  int shift;

  static int_divider_t make(int d) {
    int s = 0;
    while(((int64_t)1 << s) < d) ++s;
    if(((int64_t)1 << s) == d) return int_divider_t { 0u, s };
    uint64_t m = (((uint64_t)1 << (31 + s)) / (uint64_t)d) + 1;
    return int_divider_t { (unsigned)m, s - 1 };
  }
  MGPU_HOST_DEVICE int div(int n) const {
    return magic ?
      (int)((unsigned)(((uint64_t)(unsigned)n * magic) >> 32) >> shift) :
      (n >> shift);
  }
};

// Kernel body of load_balance_partitions.  The merge of item indices with
// segment starts has a closed form: the start of segment j sits at merged
// position m_j = segments[j] + j (all items before it plus all starts before
// it), so the split of cross-diagonal d is d - #{j : m_j < d}.  Instead of
// one binary search per split (log2(num_segments) dependent, scattered
// loads each) every thread reads vt consecutive segment starts -- 16-byte
// loads, nothing dependent -- and writes the splits of the tile
// boundaries that fall between a start and the next one: none for most
// segments, one for a segment that straddles a boundary, many for a segment
// that spans tiles (long runs are written by the whole wavefront).
//
// With snap > 0 the kernel writes pairs (a, b) = (items, starts) in front of
// each split instead of a alone, and moves every split except the first and
// the last back along the merge path to the nearest earlier point whose item
// index is a multiple of snap -- the tile kernels of the load-balancing
// search then store whole cache lines.  Moving from a to a' = a - a % snap
// also hands back the starts in (a', a]; if there are `window` or more of
// them the split stays where it is.  A moved split retreats by at most
// (snap - 1) + (window - 1) merged elements.
template<int nt, typename int_t, typename segments_it, int snap = 0,
  int window = 32, int vt_ = 8>
struct lbs_partition_scatter_f {
  // A segment with up to `direct` splits inside has them written by its own
  // thread, one with more by a whole wavefront.
  enum { vt = vt_, direct = 64 };
  static_assert(0 == vt % 4, "segments are read four at a time");
  segments_it segments;
  int num_segments;
  int count;
  int spacing;
  int_divider_t by_spacing;
  int_t* p;
  // The grid holds `replicas` copies of the CTAs that cover the starts.
  // Every copy reads the same starts; the first one writes the splits that
  // a thread writes by itself, and the segments that span many tiles are
  // dealt out over the copies -- whole segments when a wavefront has many
  // of them, slices of one segment's splits when it has few -- otherwise a
  // few long segments leave all their splits to one wavefront.
  int base_ctas, replicas;

  MGPU_DEVICE int tile_of(int merged) const {
    return by_spacing.div(merged);
  }

  // Split `boundary` with `before` starts in front of it, where the last of
  // those starts (segment before - 1) is known not to lie behind the snapped
  // item index.
  MGPU_DEVICE void write_inside(int boundary, int before) const {
    int a = boundary * spacing - before;
    if constexpr(snap > 0) {
      if(boundary * spacing < count + num_segments) a -= a % snap;
      p[2 * boundary] = (int_t)a;
      p[2 * boundary + 1] = (int_t)before;
    } else
      p[boundary] = (int_t)a;
  }

  MGPU_DEVICE void write_pair(int boundary, int a, int before) const {
    p[2 * boundary] = (int_t)a;
    p[2 * boundary + 1] = (int_t)before;
  }

  MGPU_DEVICE void operator()(int tid, int cta) const {
    int total = count + num_segments;
    int replica = cta / base_ctas;
    cta -= replica * base_ctas;
    int j0 = vt * (nt * cta + tid);

    // starts[e] for segments j0 + e, e in [0, vt]; the start "after the last
    // segment" is count, which puts its merged position at total.
    int starts[vt + 1];
    if(j0 + vt < num_segments) {
      if constexpr(std::is_pointer<segments_it>::value) {
        typedef int v4_t __attribute__((ext_vector_type(4), aligned(4)));
        PRAGMA_UNROLL
        for(int q = 0; q < vt / 4; ++q) {
          v4_t v = *(const v4_t*)(segments + j0 + 4 * q);
          starts[4 * q] = v[0]; starts[4 * q + 1] = v[1];
          starts[4 * q + 2] = v[2]; starts[4 * q + 3] = v[3];
        }
      } else {
        PRAGMA_UNROLL
        for(int e = 0; e < vt; ++e) starts[e] = segments[j0 + e];
      }
      starts[vt] = segments[j0 + vt];
    } else {
      PRAGMA_UNROLL
      for(int e = 0; e <= vt; ++e)
        starts[e] = (j0 + e < num_segments) ? (int)segments[j0 + e] : count;
    }

    // Boundaries b with m_j < spacing * b <= m_{j+1} have exactly j + 1
    // starts in front of them.  The clamps keep malformed (unsorted) input
    // from writing outside p.  Only the first of them can be closer than
    // `snap` items to the start of segment j.
    int lane = tid % warp_size;
    // tile_at[e] = tile holding merged position m_{j0 + e}.
    int tile_at[vt + 1];
    PRAGMA_UNROLL
    for(int e = 0; e <= vt; ++e)
      tile_at[e] = tile_of(min(max(starts[e] + min(j0 + e, num_segments), 0),
        total));

    // Few segments have a split behind them (one in spacing / mean segment
    // length), so everything but the test for it sits inside the branch.
    PRAGMA_UNROLL
    for(int e = 0; e < vt; ++e) {
      int j = j0 + e;
      int first = tile_at[e] + 1;
      int n = (j < num_segments) ? tile_at[e + 1] - tile_at[e] : 0;

      if(n > 0 && !replica) {
        if constexpr(snap > 0) {
          // First split: the snapped item index may lie in front of the
          // start of segment j and of starts before it.  The thread counts
          // them, eight starts a step, all of a step's loads in flight
          // together; one step is enough for most splits.
          int a = first * spacing - (j + 1);
          int a_snap = a - a % snap;
          bool inner = first * spacing < total;
          int back = 0;
          if(inner && starts[e] > a_snap) {
            back = 1;
            bool more = true;
            while(more && back < window && j - back >= 0) {
              int top = j - back;             // nearest start not yet seen
              int v[8];
              PRAGMA_UNROLL
              for(int q = 0; q < 8; ++q)
                v[q] = segments[max(top - q, 0)];
              PRAGMA_UNROLL
              for(int q = 0; q < 8; ++q) {
                if(more && top - q >= 0 && v[q] > a_snap) ++back;
                else more = false;
              }
            }
          }
          if(inner && back < window) write_pair(first, a_snap, j + 1 - back);
          else write_pair(first, a, j + 1);
        } else
          write_inside(first, j + 1);
      }

      // The other splits inside segment j: written by the thread itself when
      // there are few, by the whole wavefront when the segment spans many
      // tiles.
      if(n > 1 && n <= direct && !replica)
        for(int k = 1; k < n; ++k) write_inside(first + k, j + 1);
      lanemask_t spanning = ballot(n > direct);
      // owners copies take turns with the wavefront's spanning segments;
      // `slices` copies share each segment.
      int spanning_count = popc(spanning);
      int owners = min(max(spanning_count, 1), replicas);
      int slices = max(replicas / owners, 1);
      int slice = replica / owners;
      int ordinal = 0;
      while(spanning) {
        int src = (int)__builtin_ctzll(spanning);
        spanning &= spanning - 1;
        bool mine = (ordinal++ % owners) == (replica % owners) &&
          slice < slices;
        if(!mine) continue;
        int src_first = readlane(first, src);
        int src_n = readlane(n, src);
        int src_before = readlane(j, src) + 1;
        if constexpr(snap == 0 && std::is_same<int_t, int>::value) {
          // four consecutive splits per lane and 16-byte store.
          typedef int v4_t __attribute__((ext_vector_type(4), aligned(4)));
          for(int k = 1 + 4 * (lane + warp_size * slice); k < src_n;
            k += 4 * warp_size * slices) {
            int base = (src_first + k) * spacing - src_before;
            if(k + 4 <= src_n) {
              v4_t v = { base, base + spacing, base + 2 * spacing,
                base + 3 * spacing };
              *(v4_t*)(p + src_first + k) = v;
            } else
              for(int i = 0; k + i < src_n; ++i)
                p[src_first + k + i] = base + i * spacing;
          }
        } else
          for(int k = 1 + lane + warp_size * slice; k < src_n;
            k += warp_size * slices)
            write_inside(src_first + k, src_before);
      }
    }

    if(!cta && !tid && !replica) {
      int last = div_up(total, spacing);
      if constexpr(snap > 0) {
        p[0] = 0; p[1] = 0;
        p[2 * last] = (int_t)count; p[2 * last + 1] = (int_t)num_segments;
      } else {
        p[0] = 0;
        p[last] = (int_t)count;
      }
    }
  }
};

// The same splits, one thread per split: a binary search over the merged
// positions m_j = segments[j] + j of the starts (the split of cross-diagonal d
// is d - #{j : m_j < d}), and for snapped pairs the look-back over the last
// starts.  Where segments are few and long -- several tiles each -- the
// scatter kernel above leaves most of the work to the few threads that hold
// a start while this one has a thread per split and a search that stays in
// the L2.  2^26 items cut into 16,400 tiles: 4.6-4.9 us whatever the number
// of segments, against 6.6 / 21.7 / 16.7 / 7.2 / 5.1 / 4.6 us for the scatter
// kernel on 16 / 128 / 1,024 / 4,096 / 8,192 / 16,384 segments.  It is used
// from two splits per segment on.
template<typename int_t, typename segments_it, int snap = 0, int window = 32>
struct lbs_partition_search_f {
  segments_it segments;
  int num_segments;
  int count;
  int spacing;
  int_t* p;

  MGPU_DEVICE void operator()(int index) const {
    int total = count + num_segments;
    int64_t d = (int64_t)spacing * index;
    int diag = (int)(d < total ? d : total);
    // First j with segments[j] + j >= diag.  The range is cut into quarters
    // (MGPU_LBS_SEARCH_ARITY parts) a step: the probes of a step are loaded
    // together, so there are half as many dependent reads as in a binary
    // search (35,000 splits over 2^24 starts, with the look-back below: 18.7 us
    // in halves, 17.4-17.9 us in quarters, 20.0 us in eighths, 21.9 us in
    // sixteenths -- from there on the number of scattered loads counts).
#ifndef MGPU_LBS_SEARCH_ARITY
#define MGPU_LBS_SEARCH_ARITY 4
#endif
    enum { arity = MGPU_LBS_SEARCH_ARITY };
    int lo = 0, hi = num_segments;
    while(hi - lo >= arity) {
      int n = hi - lo;
      int at[arity - 1], key[arity - 1];
      PRAGMA_UNROLL
      for(int q = 0; q < arity - 1; ++q) {
        at[q] = lo + (int)(((int64_t)n * (q + 1)) / arity);
        key[q] = segments[at[q]];
      }
      // probes are ascending: the first one that is not below diag bounds
      // the answer from above, the last one below it from below
      int new_lo = lo, new_hi = hi;
      PRAGMA_UNROLL
      for(int q = arity - 2; q >= 0; --q)
        if((int64_t)key[q] + at[q] >= diag) new_hi = at[q];
      PRAGMA_UNROLL
      for(int q = 0; q < arity - 1; ++q)
        if((int64_t)key[q] + at[q] < diag) new_lo = at[q] + 1;
      lo = new_lo; hi = new_hi;
    }
    while(lo < hi) {
      int mid = (int)(((unsigned)lo + (unsigned)hi) / 2);
      if((int64_t)segments[mid] + mid < diag) lo = mid + 1;
      else hi = mid;
    }
    int b = lo, a = min(max(diag - b, 0), count);
    if constexpr(snap > 0) {
      if(index > 0 && d < total) {
        // Starts in front of the split that lie behind the snapped item
        // index: counted eight a step, a step's loads in flight together
        // (one dependent read per start took the kernel from 18 to 23 us on
        // 2^24 Zipf-distributed segments, where up to 31 starts lie there).
        int a_snap = a - a % snap;
        int back = 0;
        bool more = true;
        while(more && back < window && b - 1 - back >= 0) {
          int top = b - 1 - back;           // nearest start not yet seen
          int v[8];
          PRAGMA_UNROLL
          for(int q = 0; q < 8; ++q) v[q] = segments[max(top - q, 0)];
          PRAGMA_UNROLL
          for(int q = 0; q < 8; ++q) {
            if(more && top - q >= 0 && v[q] > a_snap) ++back;
            else more = false;
          }
        }
        if(back < window) { a = a_snap; b -= back; }
      }
      p[2 * index] = (int_t)a;
      p[2 * index + 1] = (int_t)b;
    } else
      p[index] = (int_t)a;
  }
};

// It is also used from 2^24 segments on, whatever the number of splits: the
// scatter kernel reads every start (2^26 of them: 65 us, 2^24: 24 us, 22 M:
// 17 us), the searches read some 40 starts per split, the first levels of
// which stay in the L2 (14, 17.5 and 12 us).
#ifndef MGPU_LBS_SEARCH_FROM_SEGMENTS
#define MGPU_LBS_SEARCH_FROM_SEGMENTS (1 << 24)
#endif
inline bool lbs_partition_by_search(int num_segments, int num_partitions) {
  return (int64_t)num_partitions >= 2 * (int64_t)num_segments ||
    num_segments >= MGPU_LBS_SEARCH_FROM_SEGMENTS;
}

// Copies of the scatter kernel's CTAs (see lbs_partition_scatter_f): one,
// unless there are far more splits to write than CTAs reading starts -- few
// segments, many tiles -- in which case the splits inside long segments are
// spread over up to 64 copies.  (2^18 segments of which four span 16,400
// tiles each: 9.6 us with one copy, 5.6 us with four, 6.0 us with sixteen.)
inline int lbs_partition_replicas(int base_ctas, int num_partitions) {
  int splits_per_cta = num_partitions / max(base_ctas, 1);
  return min(max(splits_per_cta / 128, 1), 64);
}

// Coarse splits for the load-balancing search.  The segment starts are looked
// at in blocks of lbs_block: only the first start of every block is read
// (one 4-byte load per lbs_block * 4 bytes of starts, so this kernel moves a
// few per cent of what one pass over the starts would), and for every tile
// boundary B the kernel records the block in which the boundary's split falls:
//   blocks[B] = k  <=>  the number c of starts in front of cross-diagonal
//   spacing * B lies in [lbs_block * k + 1, lbs_block * (k + 1)],
// (blocks[0] = 0, where c = 0).  The tile kernel reads the starts of its two
// blocks anyway -- they are its own starts plus at most a block at either end
// -- and counts its exact splits from them (cta_load_balance_t::fill_blocks).
// Same scatter idea as above: merged position of block k's first start is
// s_k = segments[lbs_block * k] + lbs_block * k, and boundary B belongs to
// block k iff s_k < spacing * B <= s_{k + 1}.
template<int nt, typename segments_it>
struct lbs_block_partition_f {
  enum { direct = 8 };
  segments_it segments;
  int num_segments;
  int count;
  int spacing;
  int_divider_t by_spacing;
  int* blocks;

  MGPU_DEVICE int sample(int k) const {
    int total = count + num_segments;
    int j = lbs_block * k;
    // The clamp keeps malformed input from writing outside blocks[].
    return j < num_segments ? min(max((int)segments[j] + j, 0), total) : total;
  }

  MGPU_DEVICE void operator()(int tid, int cta) const {
    int total = count + num_segments;
    int num_blocks = div_up(num_segments, (int)lbs_block);
    int k = nt * cta + tid;
    int first = 0, n = 0;
    if(k < num_blocks) {
      int t0 = by_spacing.div(sample(k));
      int t1 = by_spacing.div(sample(k + 1));
      first = t0 + 1;
      n = t1 - t0;
    }
    // Boundaries first .. first + n - 1 lie in block k: written by the thread
    // when there are few, by the whole wavefront when a segment of the block
    // spans many tiles.
    if(n > 0 && n <= direct)
      for(int i = 0; i < n; ++i) blocks[first + i] = k;
    int lane = tid % warp_size;
    lanemask_t spanning = ballot(n > direct);
    while(spanning) {
      int src = (int)__builtin_ctzll(spanning);
      spanning &= spanning - 1;
      int src_first = readlane(first, src);
      int src_n = readlane(n, src);
      int src_k = readlane(k, src);
      for(int i = lane; i < src_n; i += warp_size)
        blocks[src_first + i] = src_k;
    }
    if(!cta && !tid) {
      blocks[0] = 0;
      // The last boundary is the end of the merge whether or not it is a
      // multiple of the spacing: every start lies in front of it.
      blocks[div_up(total, spacing)] = max(num_blocks - 1, 0);
    }
  }
};

} // namespace detail

// Writes div_up(a_count + b_count, spacing) + 1 splits into p (device
// memory) on the context's stream.  Returns the number of splits.
template<bounds_t bounds, typename a_keys_it, typename b_keys_it,
  typename comp_t, typename int_t>
int merge_path_partitions_into(a_keys_it a, int64_t a_count, b_keys_it b,
  int64_t b_count, int64_t spacing, comp_t comp, int_t* p,
  context_t& context) {
  int num_partitions = (int)div_up(a_count + b_count, spacing) + 1;
  detail::merge_path_partition_f<bounds, int_t, a_keys_it, b_keys_it, comp_t>
    f { a, b, a_count, b_count, spacing, comp, p };
  transform<256>(f, num_partitions, context);
  return num_partitions;
}

// Splits for the load-balancing search (items [0, count) merged with segment
// starts, bounds_upper) written into p; same result as
// merge_path_partitions_into with a counting iterator, computed by the
// scatter kernel above.
template<typename segments_it, typename int_t>
int load_balance_partitions_into(int64_t count, segments_it segments,
  int num_segments, int spacing, int_t* p, context_t& context) {
  enum { nt = 256, vt = 8 };
  int num_partitions = (int)div_up(count + num_segments, (int64_t)spacing) + 1;
  if(count + num_segments >= ((int64_t)1 << 31))
    throw cuda_exception_t(hipErrorInvalidValue);
  if(!num_segments)     // nothing to scatter from: every split is its diagonal
    return merge_path_partitions_into<bounds_upper>(
      counting_iterator_t<int_t>(0), count, segments, (int64_t)0,
      (int64_t)spacing, less_t<int_t>(), p, context);
  if(detail::lbs_partition_by_search(num_segments, num_partitions)) {
    detail::lbs_partition_search_f<int_t, segments_it> f { segments,
      num_segments, (int)count, spacing, p };
    transform<256>(f, num_partitions, context);
    return num_partitions;
  }
  int base_ctas = div_up(num_segments, nt * vt);
  int replicas = detail::lbs_partition_replicas(base_ctas, num_partitions);
  detail::lbs_partition_scatter_f<nt, int_t, segments_it, 0, 32, vt>
    f { segments, num_segments, (int)count, spacing,
      detail::int_divider_t::make(spacing), p, base_ctas, replicas };
  cta_launch<nt>(f, base_ctas * replicas, context);
  return num_partitions;
}

// Same splits as pairs p[2 * i] = items, p[2 * i + 1] = segment starts in
// front of split i, every inner split moved back to an item index that is a
// multiple of `snap` where fewer than `window` starts have to move with it
// (see lbs_partition_scatter_f).  2 * (div_up(count + num_segments, spacing)
// + 1) ints.  Tiles cut this way hold at most spacing + snap + window - 2
// merged elements.
template<int snap, int window, typename segments_it>
int load_balance_partitions_snapped(int count, segments_it segments,
  int num_segments, int spacing, int* p, context_t& context) {
  enum { nt = 256, vt = 8 };
  int64_t total = (int64_t)count + num_segments;
  int num_partitions = (int)div_up(total, (int64_t)spacing) + 1;
  if(total >= ((int64_t)1 << 31))
    throw cuda_exception_t(hipErrorInvalidValue);
  if(!num_segments) {
    // no starts: split i is (min(spacing * i, count) rounded down, 0).
    transform<256>([=]MGPU_DEVICE(int index) {
      int64_t d = (int64_t)spacing * index;
      int a = d < count ? (int)(d - d % snap) : count;
      p[2 * index] = a;
      p[2 * index + 1] = 0;
    }, num_partitions, context);
    return num_partitions;
  }
  if(detail::lbs_partition_by_search(num_segments, num_partitions)) {
    detail::lbs_partition_search_f<int, segments_it, snap, window> f {
      segments, num_segments, count, spacing, p };
    transform<256>(f, num_partitions, context);
    return num_partitions;
  }
  int base_ctas = div_up(num_segments, nt * vt);
  int replicas = detail::lbs_partition_replicas(base_ctas, num_partitions);
  detail::lbs_partition_scatter_f<nt, int, segments_it, snap, window, vt>
    f { segments, num_segments, count, spacing,
      detail::int_divider_t::make(spacing), p, base_ctas, replicas };
  cta_launch<nt>(f, base_ctas * replicas, context);
  return num_partitions;
}

// The coarse splits of lbs_block_partition_f: div_up(count + num_segments,
// spacing) + 1 ints.
template<typename segments_it>
int load_balance_block_partitions(int count, segments_it segments,
  int num_segments, int spacing, int* blocks, context_t& context) {
  enum { nt = 256 };
  int64_t total = (int64_t)count + num_segments;
  if(total >= ((int64_t)1 << 31))
    throw cuda_exception_t(hipErrorInvalidValue);
  int num_partitions = (int)div_up(total, (int64_t)spacing) + 1;
  if(!num_segments) {
    transform<256>([=]MGPU_DEVICE(int index) { blocks[index] = 0; },
      num_partitions, context);
    return num_partitions;
  }
  detail::lbs_block_partition_f<nt, segments_it> f { segments, num_segments,
    count, spacing, detail::int_divider_t::make(spacing), blocks };
  cta_launch<nt>(f, div_up(div_up(num_segments, (int)detail::lbs_block),
    (int)nt), context);
  return num_partitions;
}

template<bounds_t bounds, typename a_keys_it, typename b_keys_it,
  typename comp_t>
mem_t<typename std::iterator_traits<a_keys_it>::value_type>
merge_path_partitions(a_keys_it a, int64_t a_count, b_keys_it b,
  int64_t b_count, int64_t spacing, comp_t comp, context_t& context) {

  typedef typename std::iterator_traits<a_keys_it>::value_type int_t;
  int num_partitions = (int)div_up(a_count + b_count, spacing) + 1;
  mem_t<int_t> mem(num_partitions, context);
  merge_path_partitions_into<bounds>(a, a_count, b, b_count, spacing, comp,
    mem.data(), context);
  return mem;
}

// Splits of the merge of work-item indices [0, dest_count) with the segment
// starts: tile i owns items [mp[i], mp[i + 1]) and the segments whose start
// falls between the two cross-diagonals.
template<typename segments_it>
auto load_balance_partitions(int64_t dest_count, segments_it segments,
  int num_segments, int spacing, context_t& context) ->
  mem_t<typename std::iterator_traits<segments_it>::value_type> {

  typedef typename std::iterator_traits<segments_it>::value_type int_t;
  int num_partitions = (int)div_up(dest_count + num_segments,
    (int64_t)spacing) + 1;
  mem_t<int_t> mem(num_partitions, context);
  if constexpr(std::is_same<int_t, int>::value) {
    if(detail::launcher_load_balance_partitions(dest_count, segments,
      num_segments, spacing, mem.data(), context)) return mem;
  }
  load_balance_partitions_into(dest_count, segments, num_segments, spacing,
    mem.data(), context);
  return mem;
}

// p[i] = lower/upper bound of min(spacing * i, count) in keys[0, num_items).
template<bounds_t bounds, typename keys_it>
mem_t<int> binary_search_partitions(keys_it keys, int count, int num_items,
  int spacing, context_t& context) {

  int num_partitions = div_up(count, spacing) + 1;
  mem_t<int> mem(num_partitions, context);
  int* p = mem.data();
  transform<256>([=]MGPU_DEVICE(int index) {
    int key = (int)min((int64_t)spacing * index, (int64_t)count);
    p[index] = binary_search<bounds>(keys, num_items, key, less_t<int>());
  }, num_partitions, context);
  return mem;
}

END_MGPU_NAMESPACE
