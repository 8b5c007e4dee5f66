// mgpu for AMD CDNA4: tile movement between global memory, LDS and registers
// for CTA-level user code.  A tile is nt * vt elements; a thread holds vt of
// them in one of two orders:
//   strided  element nt * i + tid   (what a wavefront touches together is
//                                    contiguous: the coalesced order)
//   thread   element vt * tid + i   (a contiguous run per lane, for serial
//                                    work such as scans and merges)
// The function names and argument orders are those of
// src/moderngpu/loadstore.hxx:12-186.  Everything is built on one routine,
// tile_slots(), that visits a thread's vt slots in either order; a bounded
// visit (count < nt * vt) skips the slots past the end.
//
// The hot kernels of this library (segreduce / transform_lbs / scan tiles) do
// not go through these element-wise helpers: they move 16-byte chunks per lane
// and use a padded LDS layout (detail::tile_layout_t in cta_load_balance.hxx).
#pragma once
#include "types.hxx"
#include "intrinsics.hxx"

BEGIN_MGPU_NAMESPACE

namespace detail {

enum tile_order_t { order_strided, order_thread };

// visit(i, slot) for the thread's slots i = 0 .. vt - 1 with slot < count.
// The first vt0 strided slots are known to be in range for every thread of a
// tile with count >= nt * vt0 and go unchecked then.
template<tile_order_t order, int nt, int vt, int vt0 = vt, typename visit_t>
MGPU_HOST_DEVICE void tile_slots(int tid, int count, visit_t visit) {
  bool guaranteed = order_strided == order && vt0 > 0 && count >= nt * vt0;
  PRAGMA_UNROLL
  for(int i = 0; i < vt; ++i) {
    int slot = order_strided == order ? nt * i + tid : vt * tid + i;
    if((guaranteed && i < vt0) || slot < count) visit(i, slot);
  }
}

// The same with no bound at all.
template<tile_order_t order, int nt, int vt, typename visit_t>
MGPU_HOST_DEVICE void tile_slots(int tid, visit_t visit) {
  PRAGMA_UNROLL
  for(int i = 0; i < vt; ++i)
    visit(i, order_strided == order ? nt * i + tid : vt * tid + i);
}

// registers -> LDS and back, in `order`.
template<tile_order_t order, int nt, int vt, typename type_t>
MGPU_DEVICE void stash(const array_t<type_t, vt>& x, int tid, type_t* shared,
  bool sync) {
  tile_slots<order, nt, vt>(tid, [&](int i, int slot) { shared[slot] = x[i]; });
  if(sync) __syncthreads();
}
template<tile_order_t order, int nt, int vt, typename type_t>
MGPU_DEVICE array_t<type_t, vt> fetch(const type_t* shared, int tid,
  bool sync) {
  array_t<type_t, vt> x;
  tile_slots<order, nt, vt>(tid, [&](int i, int slot) { x[i] = shared[slot]; });
  if(sync) __syncthreads();
  return x;
}

} // namespace detail

////////////////////////////////////////////////////////////////////////////////
// registers <-> LDS.  The LDS array must hold the whole tile.

#define MGPU_TILE_FITS(shared_size)                                           \
  static_assert(shared_size >= nt * vt, "LDS array smaller than the tile")

template<int nt, int vt, typename type_t, int shared_size>
MGPU_DEVICE void reg_to_shared_thread(array_t<type_t, vt> x, int tid,
  type_t (&shared)[shared_size], bool sync = true) {
  MGPU_TILE_FITS(shared_size);
  detail::stash<detail::order_thread, nt, vt>(x, tid, shared, sync);
}

template<int nt, int vt, typename type_t, int shared_size>
MGPU_DEVICE void reg_to_shared_strided(array_t<type_t, vt> x, int tid,
  type_t (&shared)[shared_size], bool sync = true) {
  MGPU_TILE_FITS(shared_size);
  detail::stash<detail::order_strided, nt, vt>(x, tid, shared, sync);
}

template<int nt, int vt, typename type_t, int shared_size>
MGPU_DEVICE array_t<type_t, vt> shared_to_reg_thread(
  const type_t (&shared)[shared_size], int tid, bool sync = true) {
  MGPU_TILE_FITS(shared_size);
  return detail::fetch<detail::order_thread, nt, vt>(shared, tid, sync);
}

template<int nt, int vt, typename type_t, int shared_size>
MGPU_DEVICE array_t<type_t, vt> shared_to_reg_strided(
  const type_t (&shared)[shared_size], int tid, bool sync = true) {
  MGPU_TILE_FITS(shared_size);
  return detail::fetch<detail::order_strided, nt, vt>(shared, tid, sync);
}

// x[i] = data[indices[i]].
template<int nt, int vt, typename type_t, int shared_size>
MGPU_DEVICE array_t<type_t, vt> shared_gather(
  const type_t (&data)[shared_size], array_t<int, vt> indices,
  bool sync = true) {
  MGPU_TILE_FITS(shared_size);
  array_t<type_t, vt> x;
  PRAGMA_UNROLL
  for(int i = 0; i < vt; ++i) x[i] = data[indices[i]];
  if(sync) __syncthreads();
  return x;
}

// Order changes: out through LDS in one order, back in the other.
template<int nt, int vt, typename type_t, int shared_size>
MGPU_DEVICE array_t<type_t, vt> reg_thread_to_strided(array_t<type_t, vt> x,
  int tid, type_t (&shared)[shared_size]) {
  MGPU_TILE_FITS(shared_size);
  detail::stash<detail::order_thread, nt, vt>(x, tid, shared, true);
  return detail::fetch<detail::order_strided, nt, vt>(shared, tid, true);
}

template<int nt, int vt, typename type_t, int shared_size>
MGPU_DEVICE array_t<type_t, vt> reg_strided_to_thread(array_t<type_t, vt> x,
  int tid, type_t (&shared)[shared_size]) {
  MGPU_TILE_FITS(shared_size);
  detail::stash<detail::order_strided, nt, vt>(x, tid, shared, true);
  return detail::fetch<detail::order_thread, nt, vt>(shared, tid, true);
}

template<int nt, int vt, typename type_t, int shared_size>
MGPU_DEVICE array_t<type_t, vt> thread_to_strided(array_t<type_t, vt> x,
  int tid, type_t (&shared)[shared_size]) {
  return reg_thread_to_strided<nt, vt>(x, tid, shared);
}

////////////////////////////////////////////////////////////////////////////////
// registers <-> global memory; `mem` points at the tile, `count` elements of
// it exist.

template<int nt, int vt, int vt0 = vt, typename it_t>
MGPU_DEVICE array_t<typename std::iterator_traits<it_t>::value_type, vt>
mem_to_reg_strided(it_t mem, int tid, int count) {
  array_t<typename std::iterator_traits<it_t>::value_type, vt> x;
  detail::tile_slots<detail::order_strided, nt, vt, vt0>(tid, count,
    [&](int i, int slot) { x[i] = mem[slot]; });
  return x;
}

template<int nt, int vt, int vt0 = vt, typename type_t, typename it_t>
MGPU_DEVICE void reg_to_mem_strided(array_t<type_t, vt> x, int tid,
  int count, it_t mem) {
  detail::tile_slots<detail::order_strided, nt, vt, vt0>(tid, count,
    [&](int i, int slot) { mem[slot] = x[i]; });
}

// Thread order in registers, coalesced in memory: the transposition goes
// through `shared`.
template<int nt, int vt, int vt0 = vt, typename type_t, typename it_t,
  int shared_size>
MGPU_DEVICE array_t<type_t, vt> mem_to_reg_thread(it_t mem, int tid,
  int count, type_t (&shared)[shared_size]) {
  return reg_strided_to_thread<nt, vt>(
    mem_to_reg_strided<nt, vt, vt0>(mem, tid, count), tid, shared);
}

template<int nt, int vt, int vt0 = vt, typename type_t, typename it_t,
  int shared_size>
MGPU_DEVICE void reg_to_mem_thread(array_t<type_t, vt> x, int tid,
  int count, it_t mem, type_t (&shared)[shared_size]) {
  reg_to_mem_strided<nt, vt, vt0>(
    reg_thread_to_strided<nt, vt>(x, tid, shared), tid, count, mem);
}

template<int nt, int vt, int vt0 = vt, typename input_it, typename output_it>
MGPU_DEVICE void mem_to_mem(input_it input, int tid, int count,
  output_it output) {
  reg_to_mem_strided<nt, vt, vt0>(
    mem_to_reg_strided<nt, vt, vt0>(input, tid, count), tid, count, output);
}

////////////////////////////////////////////////////////////////////////////////
// global memory <-> LDS, element `slot` of the tile to shared[slot].

template<int nt, int vt, int vt0 = vt, typename type_t, typename it_t>
MGPU_DEVICE void mem_to_shared(it_t mem, int tid, int count, type_t* shared,
  bool sync = true) {
  // all loads first, then the LDS stores
  array_t<type_t, vt> x = mem_to_reg_strided<nt, vt, vt0>(mem, tid, count);
  detail::tile_slots<detail::order_strided, nt, vt, vt0>(tid, count,
    [&](int i, int slot) { shared[slot] = x[i]; });
  if(sync) __syncthreads();
}

template<int nt, int vt, typename type_t, typename it_t>
MGPU_DEVICE void shared_to_mem(const type_t* shared, int tid, int count,
  it_t mem, bool sync = true) {
  detail::tile_slots<detail::order_strided, nt, vt>(tid, count,
    [&](int, int slot) { mem[slot] = shared[slot]; });
  if(sync) __syncthreads();
}

#undef MGPU_TILE_FITS

END_MGPU_NAMESPACE
