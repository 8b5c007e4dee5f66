// The public templates compiled with MGPU_HIP_LAUNCHER: calls with raw
// pointers, built-in value types and operators go to the prebuilt kernels of
// libmgpu_hip.so through the extern "C" layer, everything else instantiates in
// place.  Checks which way each call went (detail::launcher_calls()) and the
// results against host loops.  Exit status 1 on the first mismatch.
#ifndef MGPU_HIP_LAUNCHER
#error "build with -DMGPU_HIP_LAUNCHER"
#endif
#include <moderngpu/kernel_segreduce.hxx>
#include <moderngpu/kernel_intervalmove.hxx>
#include <moderngpu/kernel_reduce.hxx>
#include <moderngpu/kernel_sortedsearch.hxx>
#include <algorithm>
#include <climits>
#include <cstdio>
#include <random>
#include <vector>

using namespace mgpu;

#define CHECK(cond) do { if(!(cond)) { \
  printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); return 1; } } while(0)

static std::vector<int> random_segments(int count, int num_segments, int seed) {
  std::mt19937 mt(seed);
  std::uniform_int_distribution<int> dist(0, count);
  std::vector<int> s(num_segments);
  s[0] = 0;
  for(int i = 1; i < num_segments; ++i) s[i] = dist(mt);
  std::sort(s.begin() + 1, s.end());
  return s;
}

template<typename type_t, typename op_t>
static std::vector<type_t> host_segreduce(const std::vector<type_t>& v,
  const std::vector<int>& segs, op_t op, type_t init) {
  int count = (int)v.size(), n = (int)segs.size();
  std::vector<type_t> out(n);
  for(int s = 0; s < n; ++s) {
    int b = segs[s], e = s + 1 < n ? segs[s + 1] : count;
    type_t x = init;
    for(int i = b; i < e; ++i) x = (i == b) ? v[i] : op(x, v[i]);
    out[s] = x;
  }
  return out;
}

struct absmax_t {     // a user operator: not one the library is built for
  MGPU_HOST_DEVICE int operator()(int a, int b) const {
    int x = a < 0 ? -a : a, y = b < 0 ? -b : b;
    return x < y ? b : a;
  }
};
struct alignas(16) wide_t { int a, b, c, d; };
struct odd_t { int a, b, c; };

template<typename type_t, typename op_t>
static int check_segreduce(op_t op, type_t init, bool expect_call,
  context_t& context) {
  int count = 300000, num_segments = 4000;
  std::vector<int> segs = random_segments(count, num_segments, 7);
  std::vector<type_t> v(count);
  std::mt19937 mt(9);
  for(type_t& x : v) x = (type_t)((int)(mt() % 2001) - 1000);
  mem_t<type_t> in = to_mem(v, context), out(num_segments, context);
  mem_t<int> s = to_mem(segs, context);
  long before = detail::launcher_calls();
  segreduce((const type_t*)in.data(), count, s.data(), num_segments,
    out.data(), op, init, context);
  CHECK((detail::launcher_calls() - before == 1) == expect_call);
  std::vector<type_t> got = from_mem(out), want = host_segreduce(v, segs, op, init);
  for(int i = 0; i < num_segments; ++i) CHECK(got[i] == want[i]);
  return 0;
}

int main() {
  standard_context_t context(false);
  long calls;

  // segreduce: built-in type and operator -> library; anything else -> here.
  CHECK(0 == check_segreduce<int>(plus_t<int>(), -1, true, context));
  CHECK(0 == check_segreduce<float>(maximum_t<float>(), 0.0f, true, context));
  CHECK(0 == check_segreduce<long long>(minimum_t<long long>(), 5ll, true, context));
  CHECK(0 == check_segreduce<unsigned>(plus_t<unsigned>(), 0u, true, context));
  CHECK(0 == check_segreduce<double>(plus_t<double>(), 0.0, true, context));
  CHECK(0 == check_segreduce<int>(absmax_t(), 0, false, context));
  CHECK(0 == check_segreduce<short>(plus_t<short>(), (short)0, false, context));

  int count = 250000, num_segments = 3000;
  std::vector<int> segs = random_segments(count, num_segments, 11);
  mem_t<int> s = to_mem(segs, context);
  std::vector<int> owner(count);
  for(int seg = 0; seg < num_segments; ++seg) {
    int b = segs[seg], e = seg + 1 < num_segments ? segs[seg + 1] : count;
    for(int i = b; i < e; ++i) owner[i] = seg;
  }

  {
    // An explicit launch box, a computed input and an iterator output all
    // stay with the templates.
    mem_t<int> out(num_segments, context);
    calls = detail::launcher_calls();
    mem_t<int> ones = fill<int>(1, count, context);
    segreduce<launch_params_t<128, 7> >((const int*)ones.data(), count,
      s.data(), num_segments, out.data(), plus_t<int>(), 0, context);
    transform_segreduce([]MGPU_DEVICE(int i) { return 1; }, count, s.data(),
      num_segments, out.data(), plus_t<int>(), 0, context);
    CHECK(detail::launcher_calls() == calls);
    std::vector<int> got = from_mem(out);
    for(int seg = 0; seg < num_segments; ++seg) {
      int e = seg + 1 < num_segments ? segs[seg + 1] : count;
      CHECK(got[seg] == e - segs[seg]);
    }
  }
  {
    // load_balance_search.
    mem_t<int> out(count, context);
    calls = detail::launcher_calls();
    load_balance_search(count, s.data(), num_segments, out.data(), context);
    CHECK(detail::launcher_calls() == calls + 1);
    CHECK(from_mem(out) == owner);
    mem_t<short> narrow(count, context);       // not an int output
    load_balance_search(count, s.data(), num_segments, narrow.data(), context);
    CHECK(detail::launcher_calls() == calls + 1);
    std::vector<short> got = from_mem(narrow);
    for(int i = 0; i < count; ++i) CHECK(got[i] == (short)owner[i]);
  }
  {
    // interval_expand for 1, 4, 8 and 16-byte elements -> library; 12 bytes
    // -> templates.
    std::vector<double> hv(num_segments);
    std::vector<char> hc(num_segments);
    std::vector<wide_t> hw(num_segments);
    std::vector<odd_t> ho(num_segments);
    for(int i = 0; i < num_segments; ++i) {
      hv[i] = 0.5 * i; hc[i] = (char)(i * 7);
      hw[i] = wide_t { i, -i, 2 * i, 3 }; ho[i] = odd_t { i, i + 1, i + 2 };
    }
    mem_t<double> dv = to_mem(hv, context), ov(count, context);
    mem_t<char> dc = to_mem(hc, context), oc(count, context);
    mem_t<wide_t> dw = to_mem(hw, context), ow(count, context);
    mem_t<odd_t> d_odd = to_mem(ho, context), o_odd(count, context);
    calls = detail::launcher_calls();
    interval_expand((const double*)dv.data(), count, s.data(), num_segments, ov.data(), context);
    interval_expand(dc.data(), count, s.data(), num_segments, oc.data(), context);
    interval_expand((const wide_t*)dw.data(), count, s.data(), num_segments, ow.data(), context);
    CHECK(detail::launcher_calls() == calls + 3);
    interval_expand(d_odd.data(), count, s.data(), num_segments, o_odd.data(), context);
    CHECK(detail::launcher_calls() == calls + 3);
    std::vector<double> gv = from_mem(ov);
    std::vector<char> gc = from_mem(oc);
    std::vector<wide_t> gw = from_mem(ow);
    std::vector<odd_t> go = from_mem(o_odd);
    for(int i = 0; i < count; ++i) {
      int seg = owner[i];
      CHECK(gv[i] == hv[seg] && gc[i] == hc[seg]);
      CHECK(gw[i].a == seg && gw[i].b == -seg && gw[i].c == 2 * seg && gw[i].d == 3);
      CHECK(go[i].a == seg && go[i].b == seg + 1 && go[i].c == seg + 2);
    }
  }
  {
    // interval_gather / scatter / move with a shuffled layout of the segments.
    std::vector<int> order(num_segments), base(num_segments);
    for(int i = 0; i < num_segments; ++i) order[i] = i;
    std::shuffle(order.begin(), order.end(), std::mt19937(3));
    int at = 0;
    for(int k = 0; k < num_segments; ++k) {
      int seg = order[k];
      int e = seg + 1 < num_segments ? segs[seg + 1] : count;
      base[seg] = at; at += e - segs[seg];
    }
    std::vector<int> hin(count);
    for(int i = 0; i < count; ++i) hin[i] = i * 3 + 1;
    mem_t<int> in = to_mem(hin, context), b = to_mem(base, context);
    mem_t<int> gathered(count, context), scattered(count, context), moved(count, context);
    calls = detail::launcher_calls();
    interval_scatter((const int*)in.data(), count, s.data(), num_segments, (const int*)b.data(), scattered.data(), context);
    interval_gather((const int*)scattered.data(), count, s.data(), num_segments, (const int*)b.data(), gathered.data(), context);
    interval_move((const int*)scattered.data(), count, s.data(), num_segments, (const int*)s.data(), (const int*)b.data(), moved.data(), context);
    CHECK(detail::launcher_calls() == calls + 3);
    std::vector<int> hs = from_mem(scattered);
    for(int i = 0; i < count; ++i)
      CHECK(hs[base[owner[i]] + (i - segs[owner[i]])] == hin[i]);
    CHECK(from_mem(gathered) == hin);
    CHECK(from_mem(moved) == hin);
  }
  {
    // spmv, float: rows = the segments above, x of 1000 entries.
    int cols = 1000;
    std::vector<float> a(count), x(cols);
    std::vector<int> c(count);
    std::mt19937 mt(5);
    for(int i = 0; i < count; ++i) { a[i] = (float)(mt() % 64) / 8; c[i] = mt() % cols; }
    for(int i = 0; i < cols; ++i) x[i] = (float)(mt() % 32) / 4;
    mem_t<float> da = to_mem(a, context), dx = to_mem(x, context), y(num_segments, context);
    mem_t<int> dc = to_mem(c, context);
    calls = detail::launcher_calls();
    spmv(da.data(), dc.data(), dx.data(), count, s.data(), num_segments, y.data(), context);
    CHECK(detail::launcher_calls() == calls + 1);
    std::vector<float> got = from_mem(y);
    for(int seg = 0; seg < num_segments; ++seg) {
      int e = seg + 1 < num_segments ? segs[seg + 1] : count;
      double want = 0, norm = 0;
      for(int i = segs[seg]; i < e; ++i) { want += (double)a[i] * x[c[i]]; norm += (double)a[i] * x[c[i]]; }
      CHECK(std::abs(got[seg] - want) <= 1e-5 * norm + 1e-30);
    }
  }
  {
    // scan and reduce on pointers -> library (not when an event is to be
    // recorded mid-call, and not for computed inputs).
    int n = 1 << 20;
    std::vector<int> hv(n);
    std::mt19937 mt(17);
    for(int& x : hv) x = (int)(mt() % 200) - 100;
    mem_t<int> v = to_mem(hv, context), scanned(n, context), total(1, context);
    calls = detail::launcher_calls();
    scan((const int*)v.data(), n, scanned.data(), plus_t<int>(), total.data(), context);
    CHECK(detail::launcher_calls() == calls + 1);
    std::vector<int> got = from_mem(scanned);
    int run = 0;
    for(int i = 0; i < n; ++i) { CHECK(got[i] == run); run += hv[i]; }
    CHECK(from_mem(total)[0] == run);

    scan<scan_type_inc>(v.data(), n, scanned.data(), maximum_t<int>(),
      discard_iterator_t<int>(), context);
    CHECK(detail::launcher_calls() == calls + 2);
    got = from_mem(scanned);
    int best = hv[0];
    for(int i = 0; i < n; ++i) { best = std::max(best, hv[i]); CHECK(got[i] == best); }

    reduce((const int*)v.data(), n, total.data(), plus_t<int>(), context);
    CHECK(detail::launcher_calls() == calls + 3);
    CHECK(from_mem(total)[0] == run);

    hipEvent_t event;
    CHECK(hipSuccess == hipEventCreate(&event));
    scan_event(v.data(), n, scanned.data(), plus_t<int>(), total.data(), context, event);
    const int* data = v.data();
    transform_reduce([=]MGPU_DEVICE(int i) { return data[i]; }, n, total.data(),
      plus_t<int>(), context);
    CHECK(detail::launcher_calls() == calls + 3);
    CHECK(from_mem(total)[0] == run);
    CHECK(hipSuccess == hipEventDestroy(event));
  }
  {
    // sorted_search on int keys with less_t and load_balance_partitions.
    int n = 200000, h = 150000;
    mem_t<int> needles = fill_random(0, 1 << 20, n, true, context);
    mem_t<int> hay = fill_random(0, 1 << 20, h, true, context);
    mem_t<int> found(n, context);
    calls = detail::launcher_calls();
    sorted_search<bounds_upper>((const int*)needles.data(), n,
      (const int*)hay.data(), h, found.data(), less_t<int>(), context);
    CHECK(detail::launcher_calls() == calls + 1);
    std::vector<int> hn = from_mem(needles), hh = from_mem(hay), got = from_mem(found);
    for(int i = 0; i < n; ++i)
      CHECK(got[i] == (int)(std::upper_bound(hh.begin(), hh.end(), hn[i]) - hh.begin()));
    sorted_search<bounds_lower>(needles.data(), n, hay.data(), h, found.data(),
      [=]MGPU_DEVICE(int a, int b) { return a < b; }, context);   // a lambda: stays here
    CHECK(detail::launcher_calls() == calls + 1);
    got = from_mem(found);
    for(int i = 0; i < n; ++i)
      CHECK(got[i] == (int)(std::lower_bound(hh.begin(), hh.end(), hn[i]) - hh.begin()));

    mem_t<int> mp = load_balance_partitions(count, s.data(), num_segments, 1000, context);
    CHECK(detail::launcher_calls() == calls + 2);
    std::vector<int> hmp = from_mem(mp);
    CHECK((int)hmp.size() == div_up(count + num_segments, 1000) + 1);
    for(size_t i = 0; i < hmp.size(); ++i) {
      int diag = std::min((int)(1000 * i), count + num_segments);
      CHECK(hmp[i] == merge_path<bounds_upper>(counting_iterator_t<int>(0), count,
        segs.data(), num_segments, diag, less_t<int>()));
    }
  }
  {
    // An error from the layer comes back as the library's exception.
    bool thrown = false;
    try {
      segreduce((const int*)nullptr, INT_MAX, (const int*)nullptr, 10,
        (int*)nullptr, plus_t<int>(), 0, context);
    } catch(cuda_exception_t& e) {
      thrown = hipErrorInvalidValue == e.result;
    }
    CHECK(thrown);
  }
  printf("launcher: all passed\n");
  return 0;
}
