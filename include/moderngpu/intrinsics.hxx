// mgpu for AMD CDNA4 (gfx950): bit utilities and the 64-lane cross-lane layer.
//
// The CUDA library this API mirrors (src/moderngpu/intrinsics.hxx:25-359)
// builds everything on 32-lane __shfl and inline PTX.  Here the wavefront is
// 64 lanes and the cheap cross-lane paths are
//   * DPP modifiers on VALU moves (row_shr:n inside a 16-lane row,
//     row_bcast:15 / row_bcast:31 to carry a row/half total forward,
//     wave_shr:1, quad_perm) -- no LDS traffic, full rate;
//   * ds_swizzle (the LDS crossbar without touching LDS memory) for
//     xor-butterflies of 4, 8 and 16 lanes;
//   * v_readlane for wave-uniform broadcasts.
// ds_bpermute (HIP's __shfl*) remains the fallback for arbitrary offsets.
//
// All wave_* functions must be called with all 64 lanes of the wavefront
// active (wave-uniform control flow).
#pragma once
#include "operators.hxx"

BEGIN_MGPU_NAMESPACE

typedef unsigned long long lanemask_t;

////////////////////////////////////////////////////////////////////////////////
// Bit utilities, host and device.

MGPU_HOST_DEVICE int popc(unsigned x) { return __builtin_popcount(x); }
MGPU_HOST_DEVICE int popc(int x) { return __builtin_popcount((unsigned)x); }
MGPU_HOST_DEVICE int popc(lanemask_t x) { return __builtin_popcountll(x); }

// Count of leading zero bits; 32 (or 64) for x == 0.
MGPU_HOST_DEVICE int clz(unsigned x) { return x ? __builtin_clz(x) : 32; }
MGPU_HOST_DEVICE int clz(int x) { return clz((unsigned)x); }
MGPU_HOST_DEVICE int clz(lanemask_t x) { return x ? __builtin_clzll(x) : 64; }

// 1-based index of the least significant set bit; 0 for x == 0.
MGPU_HOST_DEVICE int ffs(unsigned x) { return __builtin_ffs((int)x); }
MGPU_HOST_DEVICE int ffs(int x) { return __builtin_ffs(x); }
MGPU_HOST_DEVICE int ffs(lanemask_t x) { return __builtin_ffsll((long long)x); }

// Extract num_bits starting at bit.
MGPU_HOST_DEVICE unsigned bfe(unsigned x, unsigned bit, unsigned num_bits) {
  return num_bits >= 32 ? (x >> bit) : ((x >> bit) & ((1u << num_bits) - 1));
}
// Insert the low num_bits of x into y at bit.
MGPU_HOST_DEVICE unsigned bfi(unsigned x, unsigned y, unsigned bit,
  unsigned num_bits) {
  unsigned mask = (num_bits >= 32 ? ~0u : ((1u << num_bits) - 1)) << bit;
  return (y & ~mask) | ((x << bit) & mask);
}
// Byte permute of the 8 bytes {b:a}; each selector nibble picks one byte.
MGPU_HOST_DEVICE unsigned prmt(unsigned a, unsigned b, unsigned index) {
  unsigned long long both = ((unsigned long long)b << 32) | a;
  unsigned result = 0;
  for(int i = 0; i < 4; ++i) {
    unsigned sel = (index >> (4 * i)) & 7;
    result |= (unsigned)((both >> (8 * sel)) & 0xff) << (8 * i);
  }
  return result;
}

// Bits of x in reverse order.
MGPU_HOST_DEVICE unsigned brev(unsigned x) { return __builtin_bitreverse32(x); }

// floor(log2(x)), or ceil(log2(x)) with round_up; x > 0.
MGPU_HOST_DEVICE int find_log2(int x, bool round_up = false) {
  int floor_log = 31 - clz(x);
  return floor_log + (round_up && (x & (x - 1)) ? 1 : 0);
}

// Upper 32 bits of the 64-bit product.
MGPU_HOST_DEVICE int mulhi(int a, int b) {
  return (int)(((long long)a * b) >> 32);
}
MGPU_HOST_DEVICE unsigned umulhi(unsigned a, unsigned b) {
  return (unsigned)(((unsigned long long)a * b) >> 32);
}

////////////////////////////////////////////////////////////////////////////////
// Wavefront queries.

// Lane index inside the 64-lane wavefront.
MGPU_DEVICE inline int lane_id() {
  return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// 64-bit mask of the lanes whose predicate is true.
MGPU_DEVICE inline lanemask_t ballot(bool predicate) {
  return __ballot(predicate);
}

// Bits at and below `lane`, and strictly below.
MGPU_HOST_DEVICE lanemask_t lanemask_le(int lane) {
  return ~0ull >> (63 - lane);
}
MGPU_HOST_DEVICE lanemask_t lanemask_lt(int lane) {
  return (1ull << lane) - 1;
}

////////////////////////////////////////////////////////////////////////////////
// DPP / swizzle / readlane on arbitrary 4-byte-multiple PODs.

namespace detail {

enum {
  dpp_quad_xor1 = 0xB1,        // quad_perm:[1,0,3,2]
  dpp_quad_xor2 = 0x4E,        // quad_perm:[2,3,0,1]
  dpp_row_shr = 0x110,         // + n, 1 <= n <= 15
  dpp_wave_shr1 = 0x138,
  dpp_row_bcast15 = 0x142,
  dpp_row_bcast31 = 0x143
};

template<typename type_t>
struct lane_words_t {
  enum { words = (sizeof(type_t) + 3) / 4 };
  int w[words];
  MGPU_DEVICE lane_words_t(const type_t& x) {
    for(int i = 0; i < words; ++i) w[i] = 0;
    __builtin_memcpy(w, &x, sizeof(type_t));
  }
  MGPU_DEVICE type_t get() const {
    type_t x;
    __builtin_memcpy(&x, w, sizeof(type_t));
    return x;
  }
};

// v_mov_b32_dpp per 32-bit word.  Lanes with no source (outside the row for
// row_shr, outside row_mask for the broadcasts) keep `old` -- and so does a
// lane whose source lane is switched off.  Every cross-lane helper below
// therefore has to be called by all lanes whose values may be read: never
// behind a lane-dependent branch, and not on the right of `||`, `&&` or `?:`
// either (`!lane || wave_shift_up1(x) != x` runs the shift with lane 0 off,
// and lane 1 then compares x with itself).
template<int ctrl, int row_mask = 0xf, int bank_mask = 0xf, typename type_t>
MGPU_DEVICE inline type_t dpp_move(type_t old, type_t src) {
  lane_words_t<type_t> o(old), s(src);
  PRAGMA_UNROLL
  for(int i = 0; i < lane_words_t<type_t>::words; ++i)
    s.w[i] = __builtin_amdgcn_update_dpp(o.w[i], s.w[i], ctrl, row_mask,
      bank_mask, false);
  return s.get();
}

// ds_swizzle in bit mode: source lane = ((lane & and_mask) | or_mask) ^
// xor_mask inside each group of 32 lanes.
template<int and_mask, int or_mask, int xor_mask, typename type_t>
MGPU_DEVICE inline type_t swizzle(type_t x) {
  lane_words_t<type_t> s(x);
  PRAGMA_UNROLL
  for(int i = 0; i < lane_words_t<type_t>::words; ++i)
    s.w[i] = __builtin_amdgcn_ds_swizzle(s.w[i],
      (xor_mask << 10) | (or_mask << 5) | and_mask);
  return s.get();
}

template<typename type_t>
MGPU_DEVICE inline type_t readlane(type_t x, int lane) {
  lane_words_t<type_t> s(x);
  PRAGMA_UNROLL
  for(int i = 0; i < lane_words_t<type_t>::words; ++i)
    s.w[i] = __builtin_amdgcn_readlane(s.w[i], lane);
  return s.get();
}

// Pins the point at which x has to be in registers: the compiler may not
// move the load that produces x below this call (it otherwise sinks a load
// into the branch that uses it, behind the wait for everything else).
template<typename type_t>
MGPU_DEVICE inline void needed_here(const type_t& x) {
  lane_words_t<type_t> s(x);
  asm volatile("" :: "v"(s.w[0]));
}

template<typename type_t>
MGPU_DEVICE inline type_t bpermute(type_t x, int src_lane) {
  lane_words_t<type_t> s(x);
  PRAGMA_UNROLL
  for(int i = 0; i < lane_words_t<type_t>::words; ++i)
    s.w[i] = __builtin_amdgcn_ds_bpermute(4 * src_lane, s.w[i]);
  return s.get();
}

} // namespace detail

////////////////////////////////////////////////////////////////////////////////
// Wave-wide inclusive scan, lanes 0..63, operand order preserved
// (result[i] = x[0] op x[1] op ... op x[i]).  Six DPP steps: four row_shr
// inside each 16-lane row, then row_bcast:15 folds the preceding row's total
// into rows 1 and 3, then row_bcast:31 folds lane 31's total into the upper
// half.

template<typename type_t, typename op_t>
MGPU_DEVICE inline type_t wave_scan(type_t x, op_t op, int lane) {
  using namespace detail;
  int r = lane & 15;
  type_t y;
  y = dpp_move<dpp_row_shr + 1>(x, x); if(r >= 1) x = op(y, x);
  y = dpp_move<dpp_row_shr + 2>(x, x); if(r >= 2) x = op(y, x);
  y = dpp_move<dpp_row_shr + 4>(x, x); if(r >= 4) x = op(y, x);
  y = dpp_move<dpp_row_shr + 8>(x, x); if(r >= 8) x = op(y, x);
  y = dpp_move<dpp_row_bcast15, 0xa>(x, x); if(lane & 16) x = op(y, x);
  y = dpp_move<dpp_row_bcast31, 0xc>(x, x); if(lane & 32) x = op(y, x);
  return x;
}

// Segmented form.  dist = number of lanes between this lane and the nearest
// lane at or below it that starts a segment (0 if this lane starts one;
// lane + 1 if no lane at or below starts one).  A step that reaches back
// `n` lanes is applied only when dist >= n, so nothing crosses a segment
// start.  After the row steps lane i holds the fold of
// [max(start, row begin) .. i]; the two broadcast steps extend it to
// [start .. i] because the broadcast lane (15/47, then 31) has the same
// segment start whenever that start lies at or below it.
template<typename type_t, typename op_t>
MGPU_DEVICE inline type_t wave_segscan(type_t x, int dist, op_t op, int lane) {
  using namespace detail;
  int r = lane & 15;
  int reach = min(r, dist);
  type_t y;
  y = dpp_move<dpp_row_shr + 1>(x, x); if(reach >= 1) x = op(y, x);
  y = dpp_move<dpp_row_shr + 2>(x, x); if(reach >= 2) x = op(y, x);
  y = dpp_move<dpp_row_shr + 4>(x, x); if(reach >= 4) x = op(y, x);
  y = dpp_move<dpp_row_shr + 8>(x, x); if(reach >= 8) x = op(y, x);
  y = dpp_move<dpp_row_bcast15, 0xa>(x, x);
  if((lane & 16) && dist > r) x = op(y, x);
  y = dpp_move<dpp_row_bcast31, 0xc>(x, x);
  if((lane & 32) && dist > (lane & 31)) x = op(y, x);
  return x;
}

// Value of the lane below (lane 0 keeps its own value).
template<typename type_t>
MGPU_DEVICE inline type_t wave_shift_up1(type_t x) {
  return detail::dpp_move<detail::dpp_wave_shr1>(x, x);
}

// Order-preserving all-reduce: every lane returns x[0] op ... op x[63].
// xor-butterfly: quad_perm DPP for 1 and 2, ds_swizzle for 4, 8 and 16,
// v_readlane to join the two 32-lane halves.
template<typename type_t, typename op_t>
MGPU_DEVICE inline type_t wave_allreduce(type_t x, op_t op, int lane) {
  using namespace detail;
  type_t y;
  y = dpp_move<dpp_quad_xor1>(x, x); x = (lane & 1) ? op(y, x) : op(x, y);
  y = dpp_move<dpp_quad_xor2>(x, x); x = (lane & 2) ? op(y, x) : op(x, y);
  y = swizzle<0x1f, 0, 4>(x);        x = (lane & 4) ? op(y, x) : op(x, y);
  y = swizzle<0x1f, 0, 8>(x);        x = (lane & 8) ? op(y, x) : op(x, y);
  y = swizzle<0x1f, 0, 16>(x);       x = (lane & 16) ? op(y, x) : op(x, y);
  return op(readlane(x, 0), readlane(x, 32));
}

////////////////////////////////////////////////////////////////////////////////
// Shuffle API with moderngpu's names (intrinsics.hxx:167-229 of the
// reference).  width is a power of two <= 64; lanes that would read outside
// their width-sized group keep their own value.

template<typename type_t>
MGPU_DEVICE inline type_t shfl_up(type_t x, int offset,
  int width = warp_size) {
  int lane = lane_id();
  int src = lane - offset;
  type_t y = detail::bpermute(x, src);
  return ((lane & (width - 1)) >= offset) ? y : x;
}

template<typename type_t>
MGPU_DEVICE inline type_t shfl_down(type_t x, int offset,
  int width = warp_size) {
  int lane = lane_id();
  int src = lane + offset;
  type_t y = detail::bpermute(x, src);
  return ((lane & (width - 1)) + offset < width) ? y : x;
}

// x = op(value from `offset` lanes below, x) where that lane is inside the
// group; unchanged elsewhere.
template<typename type_t, typename op_t>
MGPU_DEVICE inline type_t shfl_up_op(type_t x, int offset, op_t op,
  int width = warp_size) {
  int lane = lane_id();
  type_t y = detail::bpermute(x, lane - offset);
  if((lane & (width - 1)) >= offset) x = op(y, x);
  return x;
}

template<typename type_t, typename op_t>
MGPU_DEVICE inline type_t shfl_down_op(type_t x, int offset, op_t op,
  int width = warp_size) {
  int lane = lane_id();
  type_t y = detail::bpermute(x, lane + offset);
  if((lane & (width - 1)) + offset < width) x = op(x, y);
  return x;
}

END_MGPU_NAMESPACE
