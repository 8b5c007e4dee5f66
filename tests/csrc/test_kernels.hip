// Test-only kernels that expose the CTA-level primitives (cta_scan_t,
// cta_reduce_t, cta_segscan_t, the wave-level helpers) through a small C ABI
// so the Python tests can compare them with serial host scans.
// Built into tests/csrc/libmgpu_test_kernels.so; not part of the product.
#include <moderngpu/cta_reduce.hxx>
#include <moderngpu/cta_scan.hxx>
#include <moderngpu/cta_segscan.hxx>
#include <moderngpu/cta_load_balance.hxx>
#include <moderngpu/search.hxx>
#include <moderngpu/transform.hxx>

using namespace mgpu;

namespace {

class bare_context_t : public context_t {
  hipDeviceProp_t _props;
public:
  bare_context_t() { memset(&_props, 0, sizeof(_props)); }
  virtual const hipDeviceProp_t& props() const { return _props; }
  virtual int ptx_version() const { return arch_version_gfx950; }
  virtual hipStream_t stream() { return 0; }
  virtual void* alloc(size_t, memory_space_t) { return nullptr; }
  virtual void free(void*, memory_space_t) { }
  virtual void synchronize() { }
  virtual hipEvent_t event() { return nullptr; }
  virtual void timer_begin() { }
  virtual double timer_end() { return 0; }
};

template<typename type_t>
struct op_any_t {
  int op;   // 0 plus, 1 max, 2 min, 3 left projection (associative, not
            // commutative: exposes swapped operands)
  MGPU_DEVICE type_t operator()(type_t a, type_t b) const {
    switch(op) {
      case 0: return a + b;
      case 1: return mgpu::max(a, b);
      case 2: return mgpu::min(a, b);
      default: return a;
    }
  }
};

template<int nt, typename type_t>
void run_scan(const type_t* in, int count, type_t* out, type_t* red, int op,
  type_t init, int inclusive) {
  bare_context_t context;
  cta_launch<nt>([=]MGPU_DEVICE(int tid, int) {
    typedef cta_scan_t<nt, type_t> scan_t;
    __shared__ typename scan_t::storage_t storage;
    scan_result_t<type_t> r = scan_t().scan(tid, in[tid], storage, count,
      op_any_t<type_t> { op }, init,
      inclusive ? scan_type_inc : scan_type_exc);
    out[tid] = r.scan;
    if(!tid) *red = r.reduction;
  }, 1, context);
}

template<int nt, int vt, typename type_t>
void run_scan_vt(const type_t* in, int count, type_t* out, type_t* red,
  int op, type_t init, int inclusive, type_t carry_in, int use_carry) {
  bare_context_t context;
  cta_launch<nt>([=]MGPU_DEVICE(int tid, int) {
    typedef cta_scan_t<nt, type_t> scan_t;
    __shared__ typename scan_t::storage_t storage;
    array_t<type_t, vt> x;
    iterate<vt>([&](int i) { x[i] = in[vt * tid + i]; });
    scan_result_t<type_t, vt> r = scan_t().template scan<vt>(tid, x, storage,
      carry_in, 0 != use_carry, count, op_any_t<type_t> { op }, init,
      inclusive ? scan_type_inc : scan_type_exc);
    iterate<vt>([&](int i) { out[vt * tid + i] = r.scan[i]; });
    if(!tid) *red = r.reduction;
  }, 1, context);
}

template<int nt, typename type_t>
void run_reduce(const type_t* in, int count, type_t* out, int op,
  int all_return) {
  bare_context_t context;
  cta_launch<nt>([=]MGPU_DEVICE(int tid, int) {
    typedef cta_reduce_t<nt, type_t> reduce_t;
    __shared__ typename reduce_t::storage_t storage;
    type_t r = reduce_t().reduce(tid, in[tid], storage, count,
      op_any_t<type_t> { op }, 0 != all_return);
    out[tid] = r;
  }, 1, context);
}

template<int nt, typename type_t>
void run_segscan(const type_t* in, const int* heads, const int* carries,
  type_t* scan_out, int* carry_in_out, int* left_out, int* has_left_out,
  type_t* red, int op, type_t init) {
  bare_context_t context;
  cta_launch<nt>([=]MGPU_DEVICE(int tid, int) {
    typedef cta_segscan_t<nt, type_t> segscan_t;
    __shared__ typename segscan_t::storage_t storage;
    segscan_result_t<type_t> r = segscan_t().segscan(tid, 0 != heads[tid],
      0 != carries[tid], in[tid], storage, init, op_any_t<type_t> { op });
    scan_out[tid] = r.scan;
    carry_in_out[tid] = r.has_carry_in;
    left_out[tid] = r.left_lane;
    has_left_out[tid] = r.has_left_head;
    if(!tid) *red = r.reduction;
  }, 1, context);
}

template<int nt>
void run_scan_bool(const int* in, int* out, int* red) {
  bare_context_t context;
  cta_launch<nt>([=]MGPU_DEVICE(int tid, int) {
    typedef cta_scan_t<nt, bool> scan_t;
    __shared__ typename scan_t::storage_t storage;
    scan_result_t<int> r = scan_t().scan(tid, 0 != in[tid], storage);
    out[tid] = r.scan;
    if(!tid) *red = r.reduction;
  }, 1, context);
}

// shfl_up / shfl_down / shfl_up_op / shfl_down_op / wave_allreduce on one
// wavefront.  mode selects the function.
void run_shfl(const int* in, int* out, int mode, int offset, int width) {
  bare_context_t context;
  cta_launch<64>([=]MGPU_DEVICE(int tid, int) {
    int x = in[tid];
    int y = 0;
    switch(mode) {
      case 0: y = shfl_up(x, offset, width); break;
      case 1: y = shfl_down(x, offset, width); break;
      case 2: y = shfl_up_op(x, offset, plus_t<int>(), width); break;
      case 3: y = shfl_down_op(x, offset, plus_t<int>(), width); break;
      case 4: y = wave_allreduce(x, op_any_t<int> { 3 }, tid); break;
      case 5: y = lane_id(); break;
      case 6: y = (int)popc(ballot(x & 1)); break;
    }
    out[tid] = y;
  }, 1, context);
}

// One CTA per tile runs cta_load_balance_t::load_balance (splits from
// load_balance_partitions with spacing nv) and dumps everything it returns;
// with fill_mode, cta_load_balance_fill instead: the segment of every tile item
// and (through b_offset) the rank.
template<int nt, int vt>
void run_load_balance(int count, const int* segments, int num_segments,
  int* partitions, int* a_index, int* b_index, int* merge_flags, int* indices,
  int* segs, int* ranks, int* ranges, int fill_mode) {
  bare_context_t context;
  enum { nv = nt * vt };
  int num_tiles = div_up(count + num_segments, (int)nv);
  load_balance_partitions_into((int64_t)count, segments, num_segments, nv,
    partitions, context);
  cta_launch<nt>([=]MGPU_DEVICE(int tid, int cta) {
    typedef cta_load_balance_t<nt, vt> lbs_t;
    __shared__ typename lbs_t::storage_t storage;
    size_t thread = (size_t)cta * nt + tid;
    if(fill_mode) {
      lbs_fill_t fill = cta_load_balance_fill<nt, vt>(count, segments,
        num_segments, tid, cta, partitions, storage.indices);
      for(int i = 0; i < vt; ++i) {
        int j = nt * i + tid;
        size_t at = thread * vt + i;
        indices[at] = fill.range.a_begin + j;
        if(j < fill.range.a_count()) {
          segs[at] = storage.indices[j];
          ranks[at] = indices[at] - storage.indices[fill.b_offset + segs[at]];
        } else { segs[at] = fill.range.b_begin; ranks[at] = -1; }
      }
      return;
    }
    typename lbs_t::result_t r = lbs_t().load_balance(count, segments,
      num_segments, tid, cta, partitions, storage);
    a_index[thread] = r.placement.a_index;
    b_index[thread] = r.placement.b_index;
    merge_flags[thread] = r.merge_flags;
    for(int i = 0; i < vt; ++i) {
      indices[thread * vt + i] = r.indices[i];
      segs[thread * vt + i] = r.segments[i];
      ranks[thread * vt + i] = r.ranks[i];
    }
    if(!tid) {
      ranges[4 * cta + 0] = r.placement.range.a_begin;
      ranges[4 * cta + 1] = r.placement.range.a_end;
      ranges[4 * cta + 2] = r.placement.range.b_begin;
      ranges[4 * cta + 3] = r.placement.range.b_end;
    }
  }, num_tiles, context);
}

#define BY_NT(fn, ...)                                                        \
  switch(nt) {                                                                \
    case 64: fn<64>(__VA_ARGS__); break;                                      \
    case 128: fn<128>(__VA_ARGS__); break;                                    \
    case 256: fn<256>(__VA_ARGS__); break;                                    \
    case 512: fn<512>(__VA_ARGS__); break;                                    \
    case 1024: fn<1024>(__VA_ARGS__); break;                                  \
    default: return -1;                                                       \
  }

#define BY_NT_T(fn, T, ...)                                                   \
  switch(nt) {                                                                \
    case 64: fn<64, T>(__VA_ARGS__); break;                                   \
    case 128: fn<128, T>(__VA_ARGS__); break;                                 \
    case 256: fn<256, T>(__VA_ARGS__); break;                                 \
    case 512: fn<512, T>(__VA_ARGS__); break;                                 \
    case 1024: fn<1024, T>(__VA_ARGS__); break;                               \
    default: return -1;                                                       \
  }

int finish() {
  hipError_t e = hipDeviceSynchronize();
  return (int)(e != hipSuccess ? e : hipGetLastError());
}

} // namespace

#define API extern "C" __attribute__((visibility("default")))

API int tk_scan_i32(int nt, const int* in, int count, int* out, int* red,
  int op, int init, int inclusive) {
  BY_NT_T(run_scan, int, in, count, out, red, op, init, inclusive)
  return finish();
}
API int tk_scan_i64(int nt, const long long* in, int count, long long* out,
  long long* red, int op, long long init, int inclusive) {
  BY_NT_T(run_scan, long long, in, count, out, red, op, init, inclusive)
  return finish();
}
API int tk_scan_f64(int nt, const double* in, int count, double* out,
  double* red, int op, double init, int inclusive) {
  BY_NT_T(run_scan, double, in, count, out, red, op, init, inclusive)
  return finish();
}
API int tk_scan_vt_i32(int nt, int vt, const int* in, int count, int* out,
  int* red, int op, int init, int inclusive, int carry_in, int use_carry) {
  if(nt == 128 && vt == 7)
    run_scan_vt<128, 7, int>(in, count, out, red, op, init, inclusive, carry_in, use_carry);
  else if(nt == 256 && vt == 4)
    run_scan_vt<256, 4, int>(in, count, out, red, op, init, inclusive, carry_in, use_carry);
  else if(nt == 64 && vt == 3)
    run_scan_vt<64, 3, int>(in, count, out, red, op, init, inclusive, carry_in, use_carry);
  else return -1;
  return finish();
}
API int tk_reduce_i32(int nt, const int* in, int count, int* out, int op,
  int all_return) {
  BY_NT_T(run_reduce, int, in, count, out, op, all_return)
  return finish();
}
API int tk_reduce_f64(int nt, const double* in, int count, double* out,
  int op, int all_return) {
  BY_NT_T(run_reduce, double, in, count, out, op, all_return)
  return finish();
}
API int tk_segscan_i32(int nt, const int* in, const int* heads,
  const int* carries, int* scan_out, int* carry_in_out, int* left_out,
  int* has_left_out, int* red, int op, int init) {
  BY_NT_T(run_segscan, int, in, heads, carries, scan_out, carry_in_out,
    left_out, has_left_out, red, op, init)
  return finish();
}
API int tk_segscan_i64(int nt, const long long* in, const int* heads,
  const int* carries, long long* scan_out, int* carry_in_out, int* left_out,
  int* has_left_out, long long* red, int op, long long init) {
  BY_NT_T(run_segscan, long long, in, heads, carries, scan_out, carry_in_out,
    left_out, has_left_out, red, op, init)
  return finish();
}
API int tk_scan_bool(int nt, const int* in, int* out, int* red) {
  BY_NT(run_scan_bool, in, out, red)
  return finish();
}
API int tk_shfl(const int* in, int* out, int mode, int offset, int width) {
  run_shfl(in, out, mode, offset, width);
  return finish();
}

// The coarse partition of the load-balancing search: the block of starts in
// which each tile boundary's split falls.
API int tk_lbs_block_partitions(int count, const int* segments,
  int num_segments, int spacing, int* blocks) {
  bare_context_t context;
  load_balance_block_partitions(count, segments, num_segments, spacing,
    blocks, context);
  return finish();
}
API int tk_lbs_block(void) { return (int)detail::lbs_block; }

API int tk_load_balance(int nt, int vt, int count, const int* segments,
  int num_segments, int* partitions, int* a_index, int* b_index,
  int* merge_flags, int* indices, int* segs, int* ranks, int* ranges,
  int fill_mode) {
#define LB(NT, VT) if(NT == nt && VT == vt) { run_load_balance<NT, VT>(count,  \
  segments, num_segments, partitions, a_index, b_index, merge_flags, indices, \
  segs, ranks, ranges, fill_mode); return finish(); }
  LB(64, 3) LB(128, 7) LB(128, 11) LB(256, 4) LB(256, 16) LB(512, 12)
#undef LB
  return -1;
}

////////////////////////////////////////////////////////////////////////////////
// A yardstick for the kernels that are streams of stores (the load-balancing
// search family): CTA `tile` stores the ints [begins[tile], begins[tile + 1])
// with 16-byte stores, after reading read_ints ints of `source` (from
// read_ints * tile on; read_ints <= 1024) that the stored values depend on.
// mapping: 0 tile = blockIdx, 1 runs of 16 tiles per XCD (xcd_tile),
// 2 one contiguous eighth of the tiles per XCD (xcd_tile_eighths).
// The grid is xcd_grid(num_tiles).  Launches on `stream` and does not wait.

namespace {
template<int mapping>
__global__ __launch_bounds__(512) void store_probe_k(int* out,
  const int* begins, int num_tiles, int read_ints, const int* source) {
  int tile = 0 == mapping ? (int)blockIdx.x :
    1 == mapping ? detail::xcd_tile(blockIdx.x, num_tiles) :
    detail::xcd_tile_eighths(blockIdx.x, num_tiles);
  if(tile >= num_tiles) return;
  __shared__ int exchange[512];
  int tid = threadIdx.x;
  int x = tid < read_ints ? source[(size_t)read_ints * tile + tid] : 0;
  if(512 + tid < read_ints) x ^= source[(size_t)read_ints * tile + 512 + tid];
  exchange[tid] = x;
  __syncthreads();
  x = exchange[(tid + 1) % 512];
  int begin = begins[tile], n = begins[tile + 1] - begin;
  typedef int v4_t __attribute__((ext_vector_type(4), aligned(4)));
  for(int q = 4 * tid; q < n; q += 4 * 512) {
    if(q + 4 <= n) {
      v4_t v = { q, x, 2, 3 };
      *(v4_t*)(out + begin + q) = v;
    } else
      for(int e = 0; e < 4; ++e)
        if(q + e < n) out[begin + q + e] = x;
  }
}
} // namespace

API int tk_store_probe(int* out, const int* begins, int num_tiles,
  int mapping, int read_ints, const int* source, void* stream) {
  if(num_tiles <= 0 || read_ints < 0 || read_ints > 1024 ||
    mapping < 0 || mapping > 2)
    return (int)hipErrorInvalidValue;
  int grid = detail::xcd_grid(num_tiles);
  hipStream_t s = (hipStream_t)stream;
  switch(mapping) {
    case 0: hipLaunchKernelGGL(store_probe_k<0>, dim3(grid), dim3(512), 0, s,
      out, begins, num_tiles, read_ints, source); break;
    case 1: hipLaunchKernelGGL(store_probe_k<1>, dim3(grid), dim3(512), 0, s,
      out, begins, num_tiles, read_ints, source); break;
    default: hipLaunchKernelGGL(store_probe_k<2>, dim3(grid), dim3(512), 0, s,
      out, begins, num_tiles, read_ints, source); break;
  }
  return (int)hipGetLastError();
}

////////////////////////////////////////////////////////////////////////////////
// A yardstick for the kernels that are streams of loads (segreduce, reduce):
// CTAs of 256 threads read 16 KB each with 16-byte loads, non-temporal or
// ordinary, and store nothing (a store guarded by a value the data never
// folds to keeps the loads alive).  Launches on `stream` and does not wait.

namespace {
template<bool nontemporal>
__global__ __launch_bounds__(256) void read_probe_k(const int* in,
  size_t chunks, int* sink) {
  typedef int v4_t __attribute__((ext_vector_type(4)));
  const v4_t* p = (const v4_t*)in;
  size_t base = (size_t)blockIdx.x * 1024 + threadIdx.x;
  v4_t x[4];
  PRAGMA_UNROLL
  for(int i = 0; i < 4; ++i) {
    size_t at = base + 256 * i;
    if(at >= chunks) at = chunks - 1;
    x[i] = nontemporal ? __builtin_nontemporal_load(p + at) : p[at];
  }
  int acc = 0;
  PRAGMA_UNROLL
  for(int i = 0; i < 4; ++i) acc ^= x[i].x ^ x[i].y ^ x[i].z ^ x[i].w;
  if(0x5bd1e995 == acc && sink) sink[0] = acc;
}
} // namespace

API int tk_read_probe(const int* in, size_t bytes, int nontemporal,
  int* sink, void* stream) {
  size_t chunks = bytes / 16;
  if(!chunks || chunks > ((size_t)1 << 40)) return (int)hipErrorInvalidValue;
  int grid = (int)((chunks + 1023) / 1024);
  hipStream_t s = (hipStream_t)stream;
  if(nontemporal)
    hipLaunchKernelGGL(read_probe_k<true>, dim3(grid), dim3(256), 0, s, in,
      chunks, sink);
  else
    hipLaunchKernelGGL(read_probe_k<false>, dim3(grid), dim3(256), 0, s, in,
      chunks, sink);
  return (int)hipGetLastError();
}
