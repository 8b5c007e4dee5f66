// mgpu for AMD CDNA4: CTA-wide reduction on 64-lane wavefronts.
//
// Each wavefront reduces in registers (DPP quad permutes, ds_swizzle
// butterflies, v_readlane -- see wave_allreduce), one value per wavefront
// goes through LDS, and every thread folds those <= 16 values.  Operand order
// is preserved (x[0] op x[1] op ...), so non-commutative operators work.
// Interface after src/moderngpu/cta_reduce.hxx:11-132, which stages all nt
// values in shared memory and finishes with 32-lane shuffles.
#pragma once
#include "loadstore.hxx"
#include "intrinsics.hxx"

BEGIN_MGPU_NAMESPACE

// Reduction inside one wavefront over the first `count` lanes (count >= 1).
// Returned in every lane.
template<typename type_t, int group_size = warp_size>
struct shfl_reduce_t {
  static_assert(group_size == warp_size,
    "shfl_reduce_t reduces one full 64-lane wavefront");

  template<typename op_t = plus_t<type_t> >
  MGPU_DEVICE type_t reduce(int lane, type_t x, int count,
    op_t op = op_t()) {
    if(count >= group_size) return wave_allreduce(x, op, lane);
    // Partial: an inclusive scan leaves the wanted fold in lane count - 1.
    x = wave_scan(x, op, lane);
    return detail::readlane(x, count - 1);
  }
};

template<int nt, typename type_t>
struct cta_reduce_t {
  static_assert(0 == nt % warp_size,
    "cta_reduce_t requires a multiple of 64 threads");
  enum { num_waves = nt / warp_size };

  struct storage_t {
    type_t waves[num_waves];
  };

  // Reduces x over threads [0, count).  The result is valid in every thread
  // when all_return is set, else in thread 0 only.  All nt threads must call.
  template<typename op_t = plus_t<type_t> >
  MGPU_DEVICE type_t reduce(int tid, type_t x, storage_t& storage,
    int count = nt, op_t op = op_t(), bool all_return = true) const {

    int lane = tid % warp_size;
    int wave = tid / warp_size;
    int wave_count = min(max(count - warp_size * wave, 0), (int)warp_size);

    type_t partial = x;
    if(count >= nt) partial = wave_allreduce(x, op, lane);
    else if(wave_count > 0) {
      // wave-uniform branch: whole wavefront takes it together.
      partial = wave_scan(x, op, lane);
      partial = detail::readlane(partial, wave_count - 1);
    }
    if(1 == num_waves) return partial;

    if(!lane) storage.waves[wave] = partial;
    __syncthreads();

    int valid_waves = min(div_up(max(count, 1), (int)warp_size),
      (int)num_waves);
    if(all_return || !tid) {
      x = storage.waves[0];
      for(int w = 1; w < valid_waves; ++w)
        x = op(x, storage.waves[w]);
    }
    __syncthreads();
    return x;
  }
};

END_MGPU_NAMESPACE
