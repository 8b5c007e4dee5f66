// mgpu for AMD CDNA4: partition kernels.  One search per tile boundary cuts a
// merge (or a load-balancing search) into tiles of `spacing` merged elements;
// the tile kernels then run independently.  Interface after
// src/moderngpu/search.hxx:12-51.
#pragma once

#include "loadstore.hxx"
#include "operators.hxx"
#include "cta_search.hxx"
#include "memory.hxx"
#include "context.hxx"

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

// Kernel body of load_balance_partitions.  The merge of item indices with
// segment starts has a closed form: the start of segment j sits at merged
// position m_j = segments[j] + j (all items before it plus all starts before
// it), so the split of cross-diagonal d is d - #{j : m_j < d}.  Instead of
// one binary search per split (log2(num_segments) dependent, scattered
// loads each) every thread reads four consecutive segment starts -- one
// 16-byte load, nothing dependent -- and writes the splits of the tile
// boundaries that fall between a start and the next one: none for most
// segments, one for a segment that straddles a boundary, many for a segment
// that spans tiles (long runs are queued in LDS and written by the whole CTA).
template<int nt, typename int_t, typename segments_it>
struct lbs_partition_scatter_f {
  enum { vt = 4, direct = 8 };
  segments_it segments;
  int num_segments;
  int count;
  int spacing;
  int shift;            // log2(spacing) if it is a power of two, else -1
  int_t* p;

  MGPU_DEVICE int tile_of(int merged) const {
    return shift >= 0 ? (merged >> shift) : merged / spacing;
  }

  MGPU_DEVICE void operator()(int tid, int cta) const {
    __shared__ int queue_size;
    __shared__ int queue[nt * vt][3];     // first boundary, how many, j + 1
    if(!tid) queue_size = 0;
    __syncthreads();

    int total = count + num_segments;
    int j0 = vt * (nt * cta + tid);

    // starts[e] for segments j0 + e, e in [0, vt]; the start "after the last
    // segment" is count, which puts its merged position at total.
    int starts[vt + 1];
    if(j0 + vt < num_segments) {
      if constexpr(std::is_pointer<segments_it>::value) {
        typedef int v4_t __attribute__((ext_vector_type(4), aligned(4)));
        v4_t v = *(const v4_t*)(segments + j0);
        starts[0] = v[0]; starts[1] = v[1]; starts[2] = v[2]; starts[3] = v[3];
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
    // from writing outside p.
    PRAGMA_UNROLL
    for(int e = 0; e < vt; ++e) {
      int j = j0 + e;
      if(j >= num_segments) break;
      int m0 = min(max(starts[e] + j, 0), total);
      int m1 = min(max(starts[e + 1] + j + 1, 0), total);
      int first = tile_of(m0) + 1;
      int n = tile_of(m1) - first + 1;
      if(n <= 0) continue;
      if(n <= direct) {
        for(int k = 0; k < n; ++k)
          p[first + k] = (int_t)((first + k) * spacing - (j + 1));
      } else {
        int slot = atomicAdd(&queue_size, 1);
        queue[slot][0] = first;
        queue[slot][1] = n;
        queue[slot][2] = j + 1;
      }
    }
    __syncthreads();

    int queued = queue_size;
    for(int q = 0; q < queued; ++q) {
      int first = queue[q][0], n = queue[q][1], before = queue[q][2];
      for(int k = tid; k < n; k += nt)
        p[first + k] = (int_t)((first + k) * spacing - before);
    }

    if(!cta && !tid) {
      p[0] = 0;
      p[div_up(total, spacing)] = (int_t)count;
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
  enum { nt = 256, vt = 4 };
  int num_partitions = (int)div_up(count + num_segments, (int64_t)spacing) + 1;
  if(count + num_segments >= ((int64_t)1 << 31))
    throw cuda_exception_t(hipErrorInvalidValue);
  if(!num_segments)     // nothing to scatter from: every split is its diagonal
    return merge_path_partitions_into<bounds_upper>(
      counting_iterator_t<int_t>(0), count, segments, (int64_t)0,
      (int64_t)spacing, less_t<int_t>(), p, context);
  int shift = is_pow2(spacing) ? s_log2(spacing) : -1;
  detail::lbs_partition_scatter_f<nt, int_t, segments_it>
    f { segments, num_segments, (int)count, spacing, shift, p };
  cta_launch<nt>(f, div_up(num_segments, nt * vt), context);
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
