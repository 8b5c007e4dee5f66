// mgpu for AMD CDNA4: the CTA-level segmented reduction and the carry fix-up
// with the interface that kernels written against the reference's
// detail::cta_segreduce_t and detail::segreduce_fixup expect
// (src/moderngpu/kernel_segreduce.hxx:17-100 and :105-186).  segreduce(),
// transform_segreduce(), lbs_segreduce() and spmv() of this library do not use
// them: their tile kernel decodes a tile from a bitmask of segment starts and
// folds all carries in one launch.  These two are for callers who built their
// own tile kernel from cta_load_balance_place(), the merge bits and this
// struct.
//
// A tile is a slice of the merge of item indices and segment starts, vt + 1
// merged elements per thread: bit i of the thread's merge bits says that
// element i is an item (it belongs to the segment that is open at that point),
// a clear bit that it is a segment start (the open segment ends, the next one
// begins).  A tile reports
//   output[s]             for every segment s that starts in the tile: the
//                         fold of its items that lie in the tile, `init` if it
//                         has none there;
//   carry_out_values[cta] the fold of the items in front of the tile's first
//                         segment start (they belong to a segment that began
//                         in an earlier tile), with
//   carry_out_codes[cta]  = 2 * (that segment) + tail bit, with -1 for the
//                         segment if the tile begins with a segment start.
// The tail bit is set when the tile's last element is a segment start whose
// items begin in the next tile: output[] holds only `init` for it, and the
// fix-up must not fold that in.
#pragma once
#include "cta_load_balance.hxx"
#include "cta_segscan.hxx"
#include "kernel_scan.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

template<int nt, int vt, typename type_t>
struct cta_segreduce_t {
  typedef cta_segscan_t<nt, type_t> segscan_t;

  union storage_t {
    typename segscan_t::storage_t segscan;
    type_t values[nt * vt + 1];
  };

  // On entry storage.values[i] is item merge_range.a_begin + i of the input.
  // `placement` is what cta_load_balance_place() returned for this thread and
  // p its vt + 1 merge bits.
  template<typename op_t, typename output_it>
  MGPU_DEVICE void segreduce(merge_range_t merge_range,
    lbs_placement_t placement, array_t<bool, vt + 1> p, int tid, int cta,
    type_t init, op_t op, output_it output, type_t* carry_out_values,
    int* carry_out_codes, storage_t& storage) {

    // The last thread ends whatever is open when the tile ends.
    bool at_end = nt - 1 == tid;
    bool tail = at_end && !p[vt - 1] && p[vt];
    if(at_end) p[vt] = false;

    // fold[i]: fold of the open segment's items among elements 0 ... i of the
    // thread (init right after a segment start).  open[i]: that segment.
    const type_t* items = storage.values - merge_range.a_begin;
    int item = placement.a_index;
    int open_first = placement.b_index;
    type_t fold[vt];
    int open[vt];
    int segment = open_first;
    bool running = false;
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i) {
      if(p[i]) {
        type_t x = items[item++];
        fold[i] = running ? op(fold[i ? i - 1 : 0], x) : x;
      } else {
        fold[i] = init;
        ++segment;
      }
      running = p[i];
      open[i] = segment;
    }
    // Every thread has read its items: the array is free for the results.
    bool any_tail = __syncthreads_or(tail);

    // What flows into the thread from the threads on its left applies to the
    // segment open at its first element, if that element is an item.
    bool has_start = open_first < segment;
    segscan_result_t<type_t> flow = segscan_t().segscan(tid, has_start,
      p[vt - 1], fold[vt - 1], storage.segscan, init, op);
    bool pending = flow.has_carry_in && p[0];

    // A segment ends behind element i when element i + 1 is a segment start.
    type_t* results = storage.values - placement.range.b_begin;
    PRAGMA_UNROLL
    for(int i = 0; i < vt; ++i) {
      if(!p[i + 1]) {
        results[open[i]] = pending ? op(flow.scan, fold[i]) : fold[i];
        pending = false;
      }
    }
    __syncthreads();

    for(int s = merge_range.b_begin + tid; s < merge_range.b_end; s += nt)
      output[s] = results[s];

    if(!tid) {
      // Thread 0's first element is an item of the segment that was open when
      // the tile began, or a segment start (then nothing is carried).
      bool carries = p[0] && open_first < merge_range.b_begin;
      carry_out_values[cta] = carries ? results[open_first] : init;
      carry_out_codes[cta] = 2 * (carries ? open_first : -1) + (int)any_tail;
    }
  }
};

////////////////////////////////////////////////////////////////////////////////
// Folds the tiles' carries into output[].  Carries of one segment are
// neighbours; their fold goes to output[segment], combined with what is
// there unless the tile in front of the run had its tail bit set.  Operands
// stay in tile order.  One segmented scan over (value, flags) elements with
// the library's scan, so any number of tiles takes the same three launches.

template<typename type_t>
struct carry_element_t {
  type_t value;
  int flags;              // bit 0: first carry of its segment; bit 1: the
                          // tile in front of that one had its tail bit set
};

template<typename type_t, typename op_t>
struct carry_fold_t {
  op_t op;
  MGPU_HOST_DEVICE carry_element_t<type_t> operator()(
    carry_element_t<type_t> a, carry_element_t<type_t> b) const {
    if(b.flags & 1) return b;
    return carry_element_t<type_t> { op(a.value, b.value), a.flags };
  }
};

template<typename output_it, typename type_t, typename op_t>
void segreduce_fixup(output_it output, const type_t* values,
  const int* codes, int count, op_t op, type_t init, context_t& context) {
  if(count <= 0) return;
  typedef carry_element_t<type_t> element_t;
  mem_t<element_t> folded(count, context);
  element_t* folded_data = folded.data();

  auto element = [=]MGPU_DEVICE(int i) {
    int seg = codes[i] >> 1;
    int left = i ? codes[i - 1] : -2;        // -2: no segment, no tail bit
    bool first = -1 == seg || (left >> 1) != seg;
    return element_t { values[i], (int)first | ((left & 1) << 1) };
  };
  transform_scan<element_t, scan_type_inc>(element, count, folded_data,
    carry_fold_t<type_t, op_t> { op }, discard_iterator_t<element_t>(),
    context);

  transform([=]MGPU_DEVICE(int i) {
    int seg = codes[i] >> 1;
    int next = (i + 1 < count) ? (codes[i + 1] >> 1) : -1;
    if(-1 == seg || seg == next) return;
    element_t e = folded_data[i];
    output[seg] = (e.flags & 2) ? e.value : op(output[seg], e.value);
  }, count, context);
}

} // namespace detail

END_MGPU_NAMESPACE
