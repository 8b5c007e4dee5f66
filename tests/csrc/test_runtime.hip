// The small pieces user kernels are written with: launch front ends
// (transform, cta_transform, cta_launch incl. the device-side tile count),
// tile movement between memory, LDS and registers in both orders, mem_t and
// its factories, tuples of iterators, compile-time helpers.  Each is checked
// against a host computation.  Exit status 1 on the first mismatch.
#include <moderngpu/transform.hxx>
#include <moderngpu/memory.hxx>
#include <moderngpu/loadstore.hxx>
#include <moderngpu/cpp11.hxx>
#include <moderngpu/kernel_load_balance.hxx>
#include <cstdio>

using namespace mgpu;

#define CHECK(cond) do { if(!(cond)) { \
  printf("%s:%d: CHECK(%s) failed\n", __FILE__, __LINE__, #cond); return 1; \
} } while(0)

static_assert(div_up(10, 3) == 4 && div_up((int64_t)1 << 40, (int64_t)3) > 0, "");
static_assert(div_up(2147483647, 4096) == 524288, "no overflow at the top");
static_assert(s_log2(1) == 0 && s_log2(4096) == 12 && s_log2(4097) == 12, "");
static_assert(is_pow2(64) && !is_pow2(96), "");
static_assert(mgpu::max(3, 3) == 3 && mgpu::min(2, 5) == 2, "");
static_assert(tuple_union_size<tuple<char, double, int> >::value == 8, "");

static int check_launches(context_t& context) {
  int count = 100003;
  mem_t<int> out = fill<int>(-1, count, context);
  int* p = out.data();
  // transform with pass-through arguments
  transform([]MGPU_DEVICE(int index, int* dest, int scale) {
    dest[index] = scale * index;
  }, count, context, p, 3);
  std::vector<int> host = from_mem(out);
  for(int i = 0; i < count; ++i) CHECK(host[i] == 3 * i);

  // cta_transform: one CTA per nv items, every thread sees (tid, cta)
  enum { nt = 128, vt = 5 };
  cta_transform<nt, vt>([=]MGPU_DEVICE(int tid, int cta) {
    strided_iterate<nt, vt>([=](int, int j) { p[nt * vt * cta + j] = cta; },
      tid, count - nt * vt * cta);
  }, count, context);
  host = from_mem(out);
  for(int i = 0; i < count; ++i) CHECK(host[i] == i / (nt * vt));

  // cta_launch with the tile count in device memory
  int tiles = 777;
  mem_t<int> num_tiles = to_mem(std::vector<int> { tiles }, context);
  mem_t<int> hits = fill<int>(0, 1000, context);
  int* h = hits.data();
  cta_launch<launch_params_t<64, 1> >([=]MGPU_DEVICE(int tid, int tile) {
    if(!tid) atomicAdd(h + tile, 1);
  }, num_tiles.data(), context);
  host = from_mem(hits);
  for(int i = 0; i < 1000; ++i) CHECK(host[i] == (i < tiles ? 1 : 0));

  // nothing is launched for zero work
  cta_launch<nt>([=]MGPU_DEVICE(int, int) { p[0] = 12345; }, 0, context);
  transform([=]MGPU_DEVICE(int) { p[0] = 12345; }, 0, context);
  CHECK(from_mem(out)[0] == 0);
  return 0;
}

static int check_tile_movement(context_t& context) {
  enum { nt = 128, vt = 7, nv = nt * vt };
  int count = 5 * nv + 333;                 // last tile partial
  int num_ctas = div_up(count, (int)nv);
  std::vector<int> in_host(count);
  for(int i = 0; i < count; ++i) in_host[i] = 10 * i + 1;
  mem_t<int> in = to_mem(in_host, context);
  mem_t<int> a(count, context), b(count, context), c(count, context),
    d(count, context);
  const int* src = in.data();
  int *pa = a.data(), *pb = b.data(), *pc = c.data(), *pd = d.data();

  cta_launch<nt>([=]MGPU_DEVICE(int tid, int cta) {
    __shared__ int shared[nv];
    int base = nv * cta;
    int n = min((int)nv, count - base);

    // strided load -> thread order -> add the position in thread order ->
    // back to strided -> store
    array_t<int, vt> x = mem_to_reg_strided<nt, vt>(src + base, tid, n);
    array_t<int, vt> y = reg_strided_to_thread<nt, vt>(x, tid, shared);
    iterate<vt>([&](int i) { y[i] += vt * tid + i; });
    x = reg_thread_to_strided<nt, vt>(y, tid, shared);
    reg_to_mem_strided<nt, vt>(x, tid, n, pa + base);

    // thread-order load and store through LDS
    array_t<int, vt> z = mem_to_reg_thread<nt, vt>(src + base, tid, n, shared);
    iterate<vt>([&](int i) { z[i] = 2 * z[i]; });
    reg_to_mem_thread<nt, vt>(z, tid, n, pb + base, shared);

    // memory -> LDS -> gather reversed within the tile -> memory
    mem_to_shared<nt, vt>(src + base, tid, n, shared);
    array_t<int, vt> indices;
    iterate<vt>([&](int i) {
      int j = nt * i + tid;
      indices[i] = j < n ? n - 1 - j : 0;
    });
    array_t<int, vt> g = shared_gather<nt, vt>(shared, indices);
    reg_to_mem_strided<nt, vt>(g, tid, n, pc + base);

    // straight copy
    mem_to_mem<nt, vt>(src + base, tid, n, pd + base);
  }, num_ctas, context);

  std::vector<int> ha = from_mem(a), hb = from_mem(b), hc = from_mem(c),
    hd = from_mem(d);
  for(int i = 0; i < count; ++i) {
    int base = i / nv * nv, n = std::min((int)nv, count - base);
    CHECK(ha[i] == in_host[i] + (i - base));
    CHECK(hb[i] == 2 * in_host[i]);
    CHECK(hc[i] == in_host[base + n - 1 - (i - base)]);
    CHECK(hd[i] == in_host[i]);
  }
  return 0;
}

static int check_memory(context_t& context) {
  int count = 4099;
  mem_t<double> halves = fill_function<double>(
    []MGPU_DEVICE(int i) { return 0.5 * i; }, count, context);
  mem_t<double> copy = halves.clone();
  CHECK(copy.data() != halves.data() && copy.size() == halves.size());
  std::vector<double> h = from_mem(copy);
  for(int i = 0; i < count; ++i) CHECK(h[i] == 0.5 * i);

  mem_t<int64_t> counted = copy_to_mem(counting_iterator_t<int64_t>(7), count,
    context);
  std::vector<int64_t> c = from_mem(counted);
  for(int i = 0; i < count; ++i) CHECK(c[i] == 7 + i);

  mem_t<int64_t> second(count, context);
  CHECK(hipSuccess == dtod(second.data(), counted.data(), count));
  std::vector<int64_t> back(3);
  CHECK(hipSuccess == dtoh(back, second.data() + 10, 3));
  CHECK(back.size() == 3 && back[0] == 17 && back[2] == 19);
  std::vector<int64_t> elsewhere(3);
  CHECK(hipSuccess == htoh(elsewhere.data(), back.data(), 3));
  CHECK(elsewhere == back);
  CHECK(hipSuccess == htod(second.data(), elsewhere));
  CHECK(from_mem(second)[1] == 18);

  // the same copies on the context's stream
  mem_t<int64_t> third(count, context);
  CHECK(hipSuccess == dtod(third.data(), counted.data(), count, context));
  std::vector<int64_t> again;
  CHECK(hipSuccess == dtoh(again, third.data() + 20, 3, context));
  CHECK(again.size() == 3 && again[0] == 27 && again[2] == 29);
  CHECK(hipSuccess == htod(third.data(), again, context));
  CHECK(hipSuccess == htod(third.data() + 3, again.data(), 2, context));
  std::vector<int64_t> t5 = from_mem(third);
  CHECK(t5[0] == 27 && t5[2] == 29 && t5[3] == 27 && t5[4] == 28 && t5[5] == 12);

  // pinned host memory, move semantics
  mem_t<int> pinned(16, context, memory_space_host);
  CHECK(memory_space_host == pinned.space());
  pinned.data()[3] = 42;
  mem_t<int> moved = std::move(pinned);
  CHECK(moved.data()[3] == 42 && pinned.data() == nullptr);
  // A small pinned block that is released comes back for the next request of
  // its size (totals travel to the host in such blocks, call after call); a
  // large one goes back to the driver.
  {
    int* first = nullptr;
    {
      mem_t<int> word(2, context, memory_space_host);
      first = word.data();
      first[0] = 7;
    }
    mem_t<int> word(2, context, memory_space_host);
    CHECK(word.data() == first);
    mem_t<char> large((size_t)1 << 20, context, memory_space_host);
    large.data()[(1 << 20) - 1] = 1;
  }

  mem_t<int> sorted = fill_random(0, 1000, 5000, true, context);
  std::vector<int> s = from_mem(sorted);
  CHECK(std::is_sorted(s.begin(), s.end()) && s.front() >= 0 && s.back() <= 1000);
  return 0;
}

static int check_tuples(context_t& context) {
  // host side
  tuple<int, double, char> t = make_tuple(3, 2.5, 'x');
  CHECK(get<0>(t) == 3 && get<1>(t) == 2.5 && get<2>(t) == 'x');
  CHECK(make_tuple(1, 2) < make_tuple(1, 3) && make_tuple(2, 0) > make_tuple(1, 9));
  CHECK(make_tuple(4, 4) == make_tuple(4, 4) && make_tuple(4, 4) != make_tuple(4, 5));
  CHECK(make_tuple(1, 2) <= make_tuple(1, 2) && make_tuple(1, 2) >= make_tuple(1, 2));

  // device side: tuples of iterators read and written as one
  int count = 3001;
  mem_t<int> a(count, context);
  mem_t<float> b(count, context);
  mem_t<int> sum(count, context);
  auto outputs = make_tuple(a.data(), b.data());
  int* s = sum.data();
  transform([=]MGPU_DEVICE(int i) {
    store(outputs, make_tuple(i, 0.25f * i), i);
  }, count, context);
  transform([=]MGPU_DEVICE(int i) {
    tuple<int, float> v = load(outputs, i);
    get<0>(dereference(outputs, i)) += 1;         // a reference into a[]
    s[i] = get<0>(v) + (int)(4 * get<1>(v));
  }, count, context);
  std::vector<int> ha = from_mem(a), hs = from_mem(sum);
  std::vector<float> hb = from_mem(b);
  for(int i = 0; i < count; ++i)
    CHECK(ha[i] == i + 1 && hb[i] == 0.25f * i && hs[i] == 2 * i);
  return 0;
}

// The bit helpers on host and device against plain loops.
static int check_bit_helpers(context_t& context) {
  static_assert(var_max<3, 9, 4>::value == 9 && var_max<>::value == 0, "");
  swallow(1, 2.0, "three");
  {
    int small[5];
    mgpu::fill(small, 7);
    small[2] = -3;
    CHECK(mgpu::reduce(small) == 25);
    kv_array_t<int, float, 3> kv; kv.keys[1] = 4; kv.vals[1] = 0.5f;
    merge_pair_t<short, 2> pair; pair.keys[0] = 9; pair.indices[0] = 1;
    CHECK(kv.keys[1] == 4 && kv.vals[1] == 0.5f && pair.keys[0] == 9 &&
      pair.indices[0] == 1 && M_PI > 3.14);
  }
  const int count = 4096;
  mem_t<unsigned> out(6 * count, context);
  unsigned* p = out.data();
  transform([=]MGPU_DEVICE(int i) {
    unsigned x = 2654435761u * (unsigned)(i + 1);
    p[6 * i + 0] = brev(x);
    p[6 * i + 1] = (unsigned)find_log2((int)(x >> 1) | 1);
    p[6 * i + 2] = (unsigned)find_log2((int)(x >> 1) | 1, true);
    p[6 * i + 3] = (unsigned)mulhi((int)x, (int)(x * 7u + 3u));
    p[6 * i + 4] = umulhi(x, x * 7u + 3u);
    p[6 * i + 5] = bfi(x, ~x, 5, 9) ^ bfe(x, 7, 11) ^ prmt(x, ~x, 0x5140) ^
      (unsigned)popc(x) ^ (unsigned)clz(x) ^ (unsigned)ffs(x);
  }, count, context);
  std::vector<unsigned> got = from_mem(out);
  for(int i = 0; i < count; ++i) {
    unsigned x = 2654435761u * (unsigned)(i + 1);
    unsigned rev = 0;
    for(int b = 0; b < 32; ++b) rev |= ((x >> b) & 1) << (31 - b);
    int v = (int)(x >> 1) | 1, lg = 0;
    while((1ll << (lg + 1)) <= v) ++lg;
    int lg_up = lg + (((1ll << lg) != v) ? 1 : 0);
    unsigned y = x * 7u + 3u;
    CHECK(got[6 * i + 0] == rev && brev(x) == rev);
    CHECK(got[6 * i + 1] == (unsigned)lg && find_log2(v) == lg);
    CHECK(got[6 * i + 2] == (unsigned)lg_up && find_log2(v, true) == lg_up);
    CHECK(got[6 * i + 3] == (unsigned)(int)(((long long)(int)x * (int)y) >> 32));
    CHECK(got[6 * i + 4] == (unsigned)(((unsigned long long)x * y) >> 32));
    CHECK(got[6 * i + 5] == (bfi(x, ~x, 5, 9) ^ bfe(x, 7, 11) ^
      prmt(x, ~x, 0x5140) ^ (unsigned)popc(x) ^ (unsigned)clz(x) ^
      (unsigned)ffs(x)));
  }
  // Hand values.
  CHECK(brev(1u) == 0x80000000u && find_log2(1) == 0 && find_log2(5, true) == 3);
  CHECK(mulhi(-1, 1) == -1 && umulhi(0xffffffffu, 0xffffffffu) == 0xfffffffeu);
  CHECK(bfe(0xabcd1234u, 8, 8) == 0x12u && bfi(0xffu, 0u, 4, 4) == 0xf0u);
  CHECK(prmt(0x33221100u, 0x77665544u, 0x7531) == 0x77553311u);
  return 0;
}

// A context on a stream the null stream does not wait for: blocks released
// while a kernel that writes them is still queued come back from the
// context's cache at once, and whatever fills them next has to be ordered
// behind that kernel.
static int check_nonblocking_stream() {
  hipStream_t stream;
  CHECK(hipSuccess == hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
  {
    standard_context_t context(false, stream);
    int count = 1 << 22;
    std::vector<int> host(count);
    int recycled = 0;
    for(int round = 0; round < 6; ++round) {
      int* first = nullptr;
      {
        mem_t<int> junk = fill<int>(-1, count, context);
        first = junk.data();
      }                                   // released, fill may still run
      for(int i = 0; i < count; ++i) host[i] = i ^ round;
      mem_t<int> mem = to_mem(host, context);
      recycled += mem.data() == first;    // the block just released
      CHECK(from_mem(mem) == host);
      mem_t<int> copy = mem.clone();
      CHECK(from_mem(copy) == host);
    }
    CHECK(recycled > 0);
  }
  CHECK(hipSuccess == hipStreamDestroy(stream));
  return 0;
}

// A context that leaves its device properties empty (as one that only wraps a
// caller's stream may): the launch with a device-side tile count still finds
// the number of compute units.
struct bare_props_context_t : standard_context_t {
  hipDeviceProp_t empty;
  bare_props_context_t() : standard_context_t(false) {
    memset(&empty, 0, sizeof(empty));
  }
  const hipDeviceProp_t& props() const override { return empty; }
};
static int check_launch_without_props() {
  bare_props_context_t context;
  int tiles = 3001;
  mem_t<int> num_tiles = to_mem(std::vector<int> { tiles }, context);
  mem_t<int> hits = fill<int>(0, 4000, context);
  int* h = hits.data();
  cta_launch<launch_params_t<64, 1> >([=]MGPU_DEVICE(int tid, int tile) {
    if(!tid) atomicAdd(h + tile, 1);
  }, num_tiles.data(), context);
  std::vector<int> host = from_mem(hits);
  for(int i = 0; i < 4000; ++i) CHECK(host[i] == (i < tiles ? 1 : 0));
  return 0;
}

// count + num_segments has to fit 31 bits; the call throws instead of
// wrapping round (nothing is launched, the pointers are never read).
static int check_index_limit(context_t& context) {
  bool thrown = false;
  try {
    load_balance_search(2147483647, (const int*)nullptr, 10, (int*)nullptr,
      context);
  } catch(cuda_exception_t& e) {
    thrown = hipErrorInvalidValue == e.result;
  }
  CHECK(thrown);
  thrown = false;
  try {
    transform_lbs([]MGPU_DEVICE(int, int, int) { }, 2000000000,
      (const int*)nullptr, 200000000, context);
  } catch(cuda_exception_t& e) {
    thrown = hipErrorInvalidValue == e.result;
  }
  CHECK(thrown);
  return 0;
}

int main() {
  standard_context_t context(false);
  CHECK(0 == check_bit_helpers(context));
  CHECK(0 == check_launches(context));
  CHECK(0 == check_tile_movement(context));
  CHECK(0 == check_memory(context));
  CHECK(0 == check_tuples(context));
  CHECK(0 == check_nonblocking_stream());
  CHECK(0 == check_launch_without_props());
  CHECK(0 == check_index_limit(context));
  printf("runtime: all passed\n");
  return 0;
}
