// mgpu for AMD CDNA4: the compile-time launch-parameter vocabulary.
//
// moderngpu keys a (threads, values-per-thread, unguarded-iterations,
// occupancy) tuple on the CUDA arch through a chain of sm_XX typedefs
// (src/moderngpu/launch_params.hxx:7-156, launch_box.hxx:9-80).  This build
// has one target, gfx950, whose tag `sm_gfx950` sits at the end of that chain:
// a box written as launch_box_t<arch_35_cta<...>, arch_52_cta<...>> still
// resolves (gfx950 inherits the newest entry it names), and
// arch_gfx950_cta<nt, vt, vt0> overrides it for CDNA4.
#pragma once
#include "meta.hxx"
#include "tuple.hxx"

// One target: host and device passes select the same column.
#define MGPU_SM_TAG sm_gfx950

#define MGPU_LAUNCH_PARAMS(launch_box) \
  typename launch_box::MGPU_SM_TAG
// The fourth launch parameter (occ) is the minimum number of wavefronts per
// SIMD the kernel should stay resident with (0: no constraint); the register
// allocator is told to stay within that budget.  CUDA boxes written with
// "min blocks per SM" in that slot reach gfx950 only through inheritance;
// arch_gfx950_cta<nt, vt, vt0, occ> states it in CDNA terms.
#define MGPU_LAUNCH_BOUNDS(launch_box) \
  __launch_bounds__(launch_box::sm_ptx::nt) \
  __attribute__((amdgpu_waves_per_eu(launch_box::sm_ptx::occ > 8 ? 0 : \
    launch_box::sm_ptx::occ)))

BEGIN_MGPU_NAMESPACE

// Value ptx_version() reports for gfx950.  Any value >= 900 selects the
// sm_gfx950 column on the host.
enum { arch_version_gfx950 = 950 };

struct MGPU_ALIGN(8) cta_dim_t {
  int nt, vt;
  int nv() const { return nt * vt; }
  int num_ctas(int count) const { return div_up(count, nv()); }
};

// Generic CTA kernel: f(tid, cta, args...).
template<typename launch_box, typename func_t, typename... args_t>
__global__ MGPU_LAUNCH_BOUNDS(launch_box)
void launch_box_cta_k(func_t f, int num_ctas, args_t... args) {
  typedef typename launch_box::sm_ptx params_t;
  int tid = (int)(threadIdx.x % (unsigned)params_t::nt);
  int cta = blockIdx.x;
  (void)num_ctas;
  f(tid, cta, make_restrict(args)...);
}

// Empty kernel; the reference queries its PTX version, we keep it so code
// that names it still links.
template<int dummy_arg>
__global__ void dummy_k() { }

template<int nt_, int vt_ = 1, int vt0_ = vt_, int occ_ = 0>
struct launch_cta_t {
  enum { nt = nt_, vt = vt_, vt0 = vt0_, occ = occ_ };
};

#define MGPU_DEF_ARCH_STRUCT(ver)                                             \
  template<typename params_t, typename base_t = empty_t>                      \
  struct arch_##ver : base_t {                                                \
    typedef params_t sm_##ver;                                                \
    template<typename new_base_t>                                             \
    using rebind = arch_##ver<params_t, new_base_t>;                          \
  };                                                                          \
  template<int nt, int vt = 1, int vt0 = vt, int occ = 0>                     \
  using arch_##ver##_cta = arch_##ver<launch_cta_t<nt, vt, vt0, occ> >;

MGPU_DEF_ARCH_STRUCT(20)
MGPU_DEF_ARCH_STRUCT(21)
MGPU_DEF_ARCH_STRUCT(30)
MGPU_DEF_ARCH_STRUCT(32)
MGPU_DEF_ARCH_STRUCT(35)
MGPU_DEF_ARCH_STRUCT(37)
MGPU_DEF_ARCH_STRUCT(50)
MGPU_DEF_ARCH_STRUCT(52)
MGPU_DEF_ARCH_STRUCT(53)
MGPU_DEF_ARCH_STRUCT(60)
MGPU_DEF_ARCH_STRUCT(61)
MGPU_DEF_ARCH_STRUCT(62)
MGPU_DEF_ARCH_STRUCT(70)
MGPU_DEF_ARCH_STRUCT(75)
MGPU_DEF_ARCH_STRUCT(80)
MGPU_DEF_ARCH_STRUCT(86)
MGPU_DEF_ARCH_STRUCT(gfx950)

#undef MGPU_DEF_ARCH_STRUCT

struct context_t;

// Launch parameters that do not depend on the architecture.
template<int nt, int vt, int vt0 = vt, int occ = 0>
struct launch_params_t : launch_cta_t<nt, vt, vt0, occ> {
  typedef launch_params_t sm_ptx;

  static cta_dim_t cta_dim() { return cta_dim_t { nt, vt }; }
  static cta_dim_t cta_dim(int) { return cta_dim(); }
  static cta_dim_t cta_dim(const context_t&) { return cta_dim(); }
  static int nv(const context_t&) { return cta_dim().nv(); }
};

END_MGPU_NAMESPACE
