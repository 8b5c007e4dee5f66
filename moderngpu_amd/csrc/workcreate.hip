// libmgpu_hip: expt::lbs_workcreate with the counts taken from an array
// (f(index, seg, rank) = created[index]) and a downsweep that stores what it
// is called with.
#include "launcher_common.hxx"
#include <moderngpu/kernel_workcreate.hxx>

using namespace mgpu;
using namespace mgpu_hip;

namespace {

typedef expt::detail::workcreate_launch_default_t launch_t;
typedef expt::detail::tile_total_t tile_total_t;
typedef detail::scan_launch_default_t<tile_total_t>::type_t_ scan_launch_t;

// Where each temporary lives in the caller's workspace.
struct workspace_t {
  int num_tiles;
  int* pairs;
  unsigned* bits;
  tile_total_t* totals;
  tile_total_t* offsets;
  tile_total_t* partials;
  size_t bytes;

  workspace_t(int count, int num_segments, void* base) {
    int nt = launch_t::sm_ptx::nt, nv = nt * launch_t::sm_ptx::vt;
    int merged = count + num_segments;
    num_tiles = div_up(merged, detail::lbs_tile_spacing(nv));
    int scan_nv = scan_launch_t::sm_ptx::nt * scan_launch_t::sm_ptx::vt;
    char* at = (char*)base;
    auto take = [&](size_t size) {
      char* p = at;
      at += (size + 255) & ~(size_t)255;
      return p;
    };
    // 8-byte arrays first.
    totals = (tile_total_t*)take(sizeof(tile_total_t) * num_tiles);
    offsets = (tile_total_t*)take(sizeof(tile_total_t) * num_tiles);
    partials = (tile_total_t*)take(sizeof(tile_total_t) *
      detail::scan_partials_count(num_tiles, scan_nv));
    pairs = (int*)take(sizeof(int) * detail::lbs_partition_ints(merged, nv));
    bits = (unsigned*)take(sizeof(unsigned) * (size_t)num_tiles * nt);
    bytes = (size_t)(at - (char*)base);
  }
};

struct created_f {
  typedef void index_only_tag;      // the upsweep need not decode its tiles
  const int* created;
  // The counts are streamed once per sweep: non-temporal loads (2^26 items:
  // whole call 230 -> 219 us).
  MGPU_DEVICE int operator()(int index, int, int, tuple<>) const {
    return __builtin_nontemporal_load(created + index);
  }
};

// Stores the arguments of every downsweep call; null outputs are skipped.
struct record_f {
  const int* created;
  int* source_index;
  int* source_seg;
  int* source_rank;
  MGPU_DEVICE int operator()(int dest_seg, int index, int seg, int rank,
    tuple<>) const {
    if(source_index) source_index[dest_seg] = index;
    if(source_seg) source_seg[dest_seg] = seg;
    if(source_rank) source_rank[dest_seg] = rank;
    return __builtin_nontemporal_load(created + index);
  }
};

} // namespace

extern "C" {

size_t mgpu_hip_workcreate_workspace_bytes(int count, int num_segments) {
  if(!sizes_ok(count, num_segments)) return 0;
  return workspace_t(count, num_segments, nullptr).bytes;
}

int mgpu_hip_workcreate_upsweep(const int* created, int count,
  const int* segments, int num_segments, int* sizes, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream) {
  if(!sizes_ok(count, num_segments) || !sizes || ((uintptr_t)sizes & 7) ||
    (count && !created) || (num_segments && !segments))
    return (int)hipErrorInvalidValue;
  workspace_t ws(count, num_segments, workspace);
  if(ws.bytes && (!workspace || workspace_bytes < ws.bytes))
    return (int)hipErrorInvalidValue;
  return guarded(stream, [&](context_t& context) {
    if(ws.num_tiles) {
      detail::lbs_partition_tiles(count, segments, num_segments,
        launch_t::nv(context), ws.pairs, context);
      expt::detail::workcreate_upsweep_launch<launch_t>(
        created_f { created }, tuple<>(), count, segments, num_segments,
        ws.pairs, ws.num_tiles, ws.bits, ws.totals, context);
    }
    // With no tiles the scan of nothing still stores a zero total.
    detail::scan_launch<scan_type_exc, scan_launch_t>(ws.totals,
      ws.num_tiles, ws.offsets, plus_t<tile_total_t>(),
      (tile_total_t*)sizes, ws.partials, context);
  });
}

int mgpu_hip_workcreate_downsweep(const int* created, int count,
  const int* segments, int num_segments, int* new_segments,
  int* source_index, int* source_seg, int* source_rank, void* workspace,
  size_t workspace_bytes, mgpu_stream_t stream) {
  if(!sizes_ok(count, num_segments) || (count && !created) ||
    (num_segments && !segments))
    return (int)hipErrorInvalidValue;
  workspace_t ws(count, num_segments, workspace);
  if(ws.bytes && (!workspace || workspace_bytes < ws.bytes))
    return (int)hipErrorInvalidValue;
  if(!ws.num_tiles) return (int)hipSuccess;
  if(!new_segments) return (int)hipErrorInvalidValue;
  return guarded(stream, [&](context_t& context) {
    expt::detail::workcreate_downsweep_launch<launch_t>(
      record_f { created, source_index, source_seg, source_rank }, tuple<>(),
      count, segments, num_segments, ws.pairs, ws.num_tiles, ws.bits,
      ws.offsets, new_segments, context);
  });
}

} // extern "C"
