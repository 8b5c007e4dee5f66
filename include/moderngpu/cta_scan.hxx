// mgpu for AMD CDNA4: CTA-wide scan on 64-lane wavefronts.
//
// Per wavefront: six DPP steps (row_shr 1/2/4/8, row_bcast:15, row_bcast:31)
// give the inclusive scan in registers; wavefront totals go through LDS and
// each thread folds the totals of the wavefronts below it (<= 15 values).
// Interface after src/moderngpu/cta_scan.hxx:8-229.
#pragma once
#include "loadstore.hxx"
#include "intrinsics.hxx"

BEGIN_MGPU_NAMESPACE

enum scan_type_t {
  scan_type_exc,
  scan_type_inc
};

template<typename type_t, int vt = 0, bool is_array = (vt > 0)>
struct scan_result_t {
  type_t scan;
  type_t reduction;
};

template<typename type_t, int vt>
struct scan_result_t<type_t, vt, true> {
  array_t<type_t, vt> scan;
  type_t reduction;
};

////////////////////////////////////////////////////////////////////////////////

template<int nt, typename type_t>
struct cta_scan_t {
  static_assert(0 == nt % warp_size,
    "cta_scan_t requires a multiple of 64 threads");
  enum { num_warps = nt / warp_size };

  struct storage_t {
    type_t warps[num_warps];
  };

  // Scan of one value per thread over threads [0, count).  Exclusive scans
  // return init in thread 0; init is not folded into the other results.
  // Threads at or beyond count receive the reduction.
  template<typename op_t = plus_t<type_t> >
  MGPU_DEVICE scan_result_t<type_t>
  scan(int tid, type_t x, storage_t& storage, int count = nt,
    op_t op = op_t(), type_t init = type_t(),
    scan_type_t type = scan_type_exc) const {

    int lane = tid % warp_size;
    int wave = tid / warp_size;

    type_t inc = wave_scan(x, op, lane);

    // Last in-range lane of each wavefront publishes the wavefront total.
    int last = min(warp_size * (wave + 1), count) - 1;
    if(tid == last) storage.warps[wave] = inc;
    __syncthreads();

    int valid_waves = min(div_up(max(count, 1), (int)warp_size),
      (int)num_warps);
    type_t reduction = storage.warps[0];
    type_t below = reduction;            // fold of wavefronts [0, wave)
    for(int w = 1; w < valid_waves; ++w) {
      reduction = op(reduction, storage.warps[w]);
      if(w < wave) below = reduction;
    }

    type_t scan;
    if(scan_type_inc == type) {
      scan = wave ? op(below, inc) : inc;
    } else {
      type_t prev = wave_shift_up1(inc);   // inclusive value of lane - 1
      if(!lane) scan = wave ? below : init;
      else scan = wave ? op(below, prev) : prev;
    }
    __syncthreads();

    return scan_result_t<type_t> { tid < count ? scan : reduction, reduction };
  }

  // vt values per thread in thread order (element vt * tid + i) over the
  // first `count` elements; optional carry_in folded in front of everything.
  template<int vt, typename op_t = plus_t<type_t> >
  MGPU_DEVICE scan_result_t<type_t, vt>
  scan(int tid, array_t<type_t, vt> x, storage_t& storage,
    type_t carry_in = type_t(), bool use_carry_in = false,
    int count = nt * vt, op_t op = op_t(), type_t init = type_t(),
    scan_type_t type = scan_type_exc) const {

    // Thread-serial inclusive scan; out-of-range slots repeat the last
    // in-range value so x[vt - 1] is the thread's total.
    int base = vt * tid;
    iterate<vt>([&](int i) {
      bool in_range = base + i < count;
      if(i) x[i] = in_range ? op(x[i - 1], x[i]) : x[i - 1];
      else if(!in_range) x[i] = init;
    });

    // Carry-in per thread: exclusive scan of the thread totals.
    scan_result_t<type_t> result = scan(tid, x[vt - 1], storage,
      div_up(count, vt), op, init, scan_type_exc);

    if(use_carry_in) {
      result.reduction = op(carry_in, result.reduction);
      result.scan = tid ? op(carry_in, result.scan) : carry_in;
    } else
      use_carry_in = tid > 0;

    array_t<type_t, vt> y;
    iterate<vt>([&](int i) {
      if(scan_type_exc == type) {
        y[i] = i ? x[i - 1] : result.scan;
        if(use_carry_in && i > 0) y[i] = op(result.scan, y[i]);
      } else {
        y[i] = use_carry_in ? op(result.scan, x[i]) : x[i];
      }
    });
    return scan_result_t<type_t, vt> { y, result.reduction };
  }
};

////////////////////////////////////////////////////////////////////////////////
// Scan of predicates: 64-bit ballot + popcount.

template<int nt>
struct cta_scan_t<nt, bool> {
  static_assert(0 == nt % warp_size,
    "cta_scan_t requires a multiple of 64 threads");
  enum { num_warps = nt / warp_size };

  struct storage_t {
    int warps[num_warps];
  };

  // Exclusive count of true predicates below each thread, and the total.
  MGPU_DEVICE scan_result_t<int> scan(int tid, bool x,
    storage_t& storage) const {
    int lane = tid % warp_size;
    int wave = tid / warp_size;

    lanemask_t bits = ballot(x);
    if(!lane) storage.warps[wave] = popc(bits);
    __syncthreads();

    int below = 0, reduction = 0;
    PRAGMA_UNROLL
    for(int w = 0; w < num_warps; ++w) {
      if(w == wave) below = reduction;
      reduction += storage.warps[w];
    }
    int scan = below + popc(bits & lanemask_lt(lane));
    __syncthreads();
    return scan_result_t<int> { scan, reduction };
  }
};

END_MGPU_NAMESPACE
