// mgpu for AMD CDNA4: launch_box_t resolves a list of per-architecture
// launch parameters to the gfx950 column.
//
// Resolution order keeps moderngpu's inheritance edges
// (src/moderngpu/launch_box.hxx:31-45: 21<-20, 30<-21, 32<-30, 35<-30,
// 37<-35, 50<-35, 52<-50, 53<-50, 60<-53, 61<-60, 62<-60, 70<-62, 75<-70,
// 80<-75, 86<-80) and appends gfx950<-86, so a box tuned for CUDA parts picks
// the same entry a current NVIDIA part would, unless it names
// arch_gfx950[_cta] explicitly.
#pragma once
#include "context.hxx"

BEGIN_MGPU_NAMESPACE

struct launch_box_default_t {
  typedef launch_cta_t<0, 0, 0> sm_00;
  typedef empty_t sm_20, sm_21, sm_30, sm_32, sm_35, sm_37, sm_50, sm_52,
    sm_53, sm_60, sm_61, sm_62, sm_70, sm_75, sm_80, sm_86, sm_gfx950;

  template<typename new_base_t>
  using rebind = launch_box_default_t;
};

template<typename... params_v>
struct launch_box_t : inherit_t<params_v..., launch_box_default_t> {
  typedef inherit_t<params_v..., launch_box_default_t> base_t;

  template<typename mine_t, typename parent_t>
  using pick_t = typename conditional_typedef_t<mine_t, parent_t>::type_t;

  typedef pick_t<typename base_t::sm_20, typename base_t::sm_00> sm_20;
  typedef pick_t<typename base_t::sm_21, sm_20> sm_21;
  typedef pick_t<typename base_t::sm_30, sm_21> sm_30;
  typedef pick_t<typename base_t::sm_32, sm_30> sm_32;
  typedef pick_t<typename base_t::sm_35, sm_30> sm_35;
  typedef pick_t<typename base_t::sm_37, sm_35> sm_37;
  typedef pick_t<typename base_t::sm_50, sm_35> sm_50;
  typedef pick_t<typename base_t::sm_52, sm_50> sm_52;
  typedef pick_t<typename base_t::sm_53, sm_50> sm_53;
  typedef pick_t<typename base_t::sm_60, sm_53> sm_60;
  typedef pick_t<typename base_t::sm_61, sm_60> sm_61;
  typedef pick_t<typename base_t::sm_62, sm_60> sm_62;
  typedef pick_t<typename base_t::sm_70, sm_62> sm_70;
  typedef pick_t<typename base_t::sm_75, sm_70> sm_75;
  typedef pick_t<typename base_t::sm_80, sm_75> sm_80;
  typedef pick_t<typename base_t::sm_86, sm_80> sm_86;
  typedef pick_t<typename base_t::sm_gfx950, sm_86> sm_gfx950;

  typedef sm_gfx950 sm_00;
  typedef MGPU_LAUNCH_PARAMS(launch_box_t) sm_ptx;

  // ptx_version is what context_t::ptx_version() returns; this library only
  // ever runs on gfx950, so every valid version selects that column.
  static cta_dim_t cta_dim(int ptx_version) {
    if(ptx_version < 20) return cta_dim_t { -1, 0 };
    return cta_dim_t { sm_gfx950::nt, sm_gfx950::vt };
  }
  static cta_dim_t cta_dim(const context_t& context) {
    return cta_dim(context.ptx_version());
  }
  static int nv(const context_t& context) {
    return cta_dim(context.ptx_version()).nv();
  }
};

// Number of CTAs of this kernel that can be resident on the whole device.
template<typename launch_box, typename func_t, typename... args_t>
int occupancy(func_t, const context_t& context, args_t...) {
  int num_blocks = 0;
  int nt = launch_box::cta_dim(context).nt;
  hipError_t result = hipOccupancyMaxActiveBlocksPerMultiprocessor(
    &num_blocks, launch_box_cta_k<launch_box, func_t, args_t...>, nt,
    (size_t)0);
  if(hipSuccess != result) throw cuda_exception_t(result);
  return context.props().multiProcessorCount * num_blocks;
}

END_MGPU_NAMESPACE
