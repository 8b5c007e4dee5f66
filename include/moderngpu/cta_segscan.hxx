// mgpu for AMD CDNA4: CTA-wide segmented scan on 64-lane wavefronts.
//
// Contract (after src/moderngpu/cta_segscan.hxx:8-103): every thread brings
// one partial x, a flag has_head_flag ("a segment starts inside this
// thread", so x covers only the part after that start) and a flag
// has_carry_out ("x continues into the next thread").  Each thread gets back
// the fold of the partials that flow into it from the left
// (segscan_result_t::scan, valid when has_carry_in), nothing when the thread
// on its left has no carry-out.
//
// Implementation: the reference finds each thread's left boundary with
// 32-bit ballots staged through shared memory and then runs log2(nt)
// Hillis-Steele passes through shared memory with a barrier each.  Here the
// boundary comes from one 64-bit ballot and a count-leading-zeros, the scan
// inside a wavefront is six guarded DPP steps in registers (wave_segscan),
// and only one summary per wavefront crosses LDS, with a single barrier.
#pragma once
#include "cta_scan.hxx"

BEGIN_MGPU_NAMESPACE

template<typename type_t>
struct segscan_result_t {
  type_t scan;          // fold of everything carried into this thread
  type_t reduction;     // inclusive fold at the last thread of the CTA
  bool has_carry_in;
  int left_lane;        // nearest thread at or below tid that starts a run;
                        // 0 if there is none
  bool has_left_head;   // false if no thread at or below tid starts a run
};

template<int nt, typename type_t>
struct cta_segscan_t {
  static_assert(0 == nt % warp_size,
    "cta_segscan_t requires a multiple of 64 threads");
  enum { num_waves = nt / warp_size };

  struct storage_t {
    type_t totals[num_waves];   // inclusive value of lane 63
    int last_start[num_waves];  // thread index of the last run start, or -1
    int carry_out[num_waves];   // lane 63's has_carry_out
  };

  template<typename op_t = plus_t<type_t> >
  MGPU_DEVICE segscan_result_t<type_t> segscan(int tid, bool has_head_flag,
    bool has_carry_out, type_t x, storage_t& storage,
    type_t init = type_t(), op_t op = op_t()) const {

    int lane = tid % warp_size;
    int wave = tid / warp_size;

    // A run of partials starts at a thread that holds a segment start, and
    // also right after a thread that carries nothing out.  Threads without
    // carry-out feed nobody, so their own value never matters.  Whether lane
    // 0 follows such a thread is only known after the wavefront summaries
    // are exchanged; inside the wavefront it is treated as continuing.
    lanemask_t heads = ballot(has_head_flag);
    lanemask_t carries = ballot(has_carry_out);
    lanemask_t starts = ((heads | ~(carries << 1)) & ~1ull) | (heads & 1);

    int left = 63 - clz(starts & lanemask_le(lane));   // -1 if none
    int dist = lane - left;                            // lane + 1 if none

    // inc = fold of x over [max(left, wavefront begin) .. lane].
    type_t inc = wave_segscan(x, dist, op, lane);

    if(warp_size - 1 == lane) {
      storage.totals[wave] = inc;
      storage.carry_out[wave] = (int)has_carry_out;
    }
    if(!lane)
      storage.last_start[wave] = starts ?
        warp_size * wave + (63 - clz(starts)) : -1;
    __syncthreads();

    // Walk the wavefront summaries left to right.  g is the fully extended
    // inclusive value of a wavefront's lane 63, g_start the thread where its
    // run starts (-1: the run reaches back to the beginning of the CTA
    // without meeting a start).
    type_t g = storage.totals[0];
    int g_start = storage.last_start[0];
    type_t wave_in = init;          // value flowing into this wavefront
    int wave_in_start = -1;
    bool wave_carry_in = false;
    PRAGMA_UNROLL
    for(int w = 1; w < num_waves; ++w) {
      bool cin = 0 != storage.carry_out[w - 1];
      if(w == wave) {
        wave_in = g;
        wave_in_start = g_start;
        wave_carry_in = cin;
      }
      type_t t = storage.totals[w];
      int s = storage.last_start[w];
      if(s >= 0) { g = t; g_start = s; }
      else if(cin) { g = op(g, t); }
      else { g = t; g_start = warp_size * w; }
    }
    type_t reduction = g;

    // Exclusive value = extended inclusive value of the thread below.
    type_t prev = wave_shift_up1(inc);
    bool has_carry_in = lane ? (0 != ((carries >> (lane - 1)) & 1)) :
      wave_carry_in;
    bool start_below = 0 != (starts & lanemask_lt(lane));

    type_t scan = init;
    if(has_carry_in) {
      if(!lane) scan = wave_in;
      else scan = (!start_below && wave_carry_in) ? op(wave_in, prev) : prev;
    }

    // Nearest run start at or below this thread.
    int left_lane;
    if(left >= 0) left_lane = warp_size * wave + left;
    else if(wave && !wave_carry_in) left_lane = warp_size * wave;
    else left_lane = wave ? wave_in_start : -1;
    __syncthreads();

    return segscan_result_t<type_t> {
      scan, reduction, has_carry_in, left_lane < 0 ? 0 : left_lane,
      left_lane >= 0
    };
  }
};

END_MGPU_NAMESPACE
