// Instantiates the public templates with argument types the other callers do
// not use -- iterators instead of pointers, 64-bit and user-defined key and
// value types, several cached iterators of different types -- and checks each
// result against a host loop.  Exit status 1 on the first mismatch.
#include <moderngpu/kernel_segreduce.hxx>
#include <moderngpu/kernel_intervalmove.hxx>
#include <moderngpu/kernel_scan.hxx>
#include <moderngpu/kernel_reduce.hxx>
#include <moderngpu/kernel_join.hxx>
#include <moderngpu/kernel_workcreate.hxx>
#include <cstdio>
#include <cmath>

using namespace mgpu;

#define CHECK(cond) do { if(!(cond)) { \
  printf("%s:%d: CHECK(%s) failed\n", __FILE__, __LINE__, #cond); return 1; \
} } while(0)

static std::vector<int> make_segments(int count, int num_segments, int seed) {
  std::mt19937 mt(seed);
  std::uniform_int_distribution<int> dist(0, count);
  std::vector<int> s(num_segments, 0);
  for(int i = 1; i < num_segments; ++i) s[i] = dist(mt);
  std::sort(s.begin() + 1, s.end());
  return s;
}

// A 16-byte value with a non-commutative operator: 2x2 integer matrices mod
// 2^32 under multiplication.
struct mat_t {
  unsigned a, b, c, d;
  MGPU_HOST_DEVICE bool operator==(const mat_t& r) const {
    return a == r.a && b == r.b && c == r.c && d == r.d;
  }
};
struct mat_mul_t {
  MGPU_HOST_DEVICE mat_t operator()(mat_t x, mat_t y) const {
    return mat_t { x.a * y.a + x.b * y.c, x.a * y.b + x.b * y.d,
      x.c * y.a + x.d * y.c, x.c * y.b + x.d * y.d };
  }
};
MGPU_HOST_DEVICE mat_t mat_of(int i) {
  return mat_t { 1u + (unsigned)i % 3, (unsigned)i % 5, (unsigned)i % 7, 1u };
}

static int check_wide_values(context_t& context) {
  int count = 150007, num_segments = 1234;
  std::vector<int> seg_host = make_segments(count, num_segments, 41);
  mem_t<int> segments = to_mem(seg_host, context);
  mem_t<mat_t> results(num_segments, context);
  mat_t init = { 9, 9, 9, 9 };
  transform_segreduce([]MGPU_DEVICE(int i) { return mat_of(i); }, count,
    segments.data(), num_segments, results.data(), mat_mul_t(), init, context);
  std::vector<mat_t> got = from_mem(results);
  for(int s = 0; s < num_segments; ++s) {
    int b = seg_host[s], e = s + 1 < num_segments ? seg_host[s + 1] : count;
    mat_t want = init;
    for(int i = b; i < e; ++i) want = (i == b) ? mat_of(i) : mat_mul_t()(want, mat_of(i));
    CHECK(got[s] == want);
  }

  // The same values through scan (inclusive) and reduce.
  int n = 70001;
  mem_t<mat_t> scanned(n, context), total(1, context);
  transform_scan<mat_t, scan_type_inc>([]MGPU_DEVICE(int i) { return mat_of(i); },
    n, scanned.data(), mat_mul_t(), total.data(), context);
  std::vector<mat_t> sc = from_mem(scanned);
  mat_t run = mat_of(0);
  for(int i = 0; i < n; ++i) {
    if(i) run = mat_mul_t()(run, mat_of(i));
    CHECK(sc[i] == run);
  }
  CHECK(from_mem(total)[0] == run);
  mem_t<mat_t> folded(1, context);
  transform_reduce([]MGPU_DEVICE(int i) { return mat_of(i); }, n, folded.data(),
    mat_mul_t(), context);
  CHECK(from_mem(folded)[0] == run);
  return 0;
}

static int check_lbs_with_mixed_cache(context_t& context) {
  int count = 220003, num_segments = 7000;
  std::vector<int> seg_host = make_segments(count, num_segments, 43);
  mem_t<int> segments = to_mem(seg_host, context);
  std::vector<double> weight_host(num_segments);
  for(int s = 0; s < num_segments; ++s) weight_host[s] = 0.5 * s - 3;
  mem_t<double> weights = to_mem(weight_host, context);
  const int* seg_data = segments.data();
  auto seg_it = make_load_iterator<int>([=]MGPU_DEVICE(int i) { return seg_data[i]; });

  // Three cached iterators: a pointer to doubles, a counting iterator, the
  // starts themselves through a load iterator.
  mem_t<double> out(count, context);
  transform_lbs([]MGPU_DEVICE(int index, int seg, int rank,
    tuple<double, int64_t, int> cached, double* out) {
      bool ok = get<1>(cached) == 100 + seg && get<2>(cached) + rank == index;
      out[index] = ok ? get<0>(cached) + rank : -1e30;
    }, count, seg_it, num_segments,
    make_tuple(weights.data(), counting_iterator_t<int64_t>(100), seg_it),
    context, out.data());
  std::vector<double> got = from_mem(out);
  int seg = -1;
  for(int i = 0; i < count; ++i) {
    while(seg + 1 < num_segments && seg_host[seg + 1] <= i) ++seg;
    CHECK(got[i] == weight_host[seg] + (i - seg_host[seg]));
  }

  // lbs_segreduce over the same iterators, double maximum.
  mem_t<double> best(num_segments, context);
  lbs_segreduce([]MGPU_DEVICE(int index, int seg, int rank,
    tuple<double> w) { return get<0>(w) * ((index * 7) % 11) - rank; },
    count, seg_it, num_segments, make_tuple(weights.data()), best.data(),
    maximum_t<double>(), -1e300, context);
  std::vector<double> b = from_mem(best);
  for(int s = 0; s < num_segments; ++s) {
    int lo = seg_host[s], hi = s + 1 < num_segments ? seg_host[s + 1] : count;
    double want = -1e300;
    for(int i = lo; i < hi; ++i) {
      double y = weight_host[s] * ((i * 7) % 11) - (i - lo);
      want = (i == lo) ? y : max(want, y);
    }
    CHECK(b[s] == want);
  }

  // Work creation with the starts through the iterator.
  auto engine = expt::lbs_workcreate(count, seg_it, num_segments, context);
  auto sizes = engine.upsweep([]MGPU_DEVICE(int index, int, int) {
    return index % 5 ? 0 : 2;
  });
  CHECK(sizes.num_segments == (count + 4) / 5 && sizes.count == 2 * sizes.num_segments);
  mem_t<int> next = engine.downsweep([]MGPU_DEVICE(int, int, int, int) { return 2; });
  std::vector<int> nx = from_mem(next);
  for(size_t k = 0; k < nx.size(); ++k) CHECK(nx[k] == 2 * (int)k);
  return 0;
}

static int check_wide_keys(context_t& context) {
  // 64-bit keys, and doubles, in sorted_search and inner_join.
  int na = 90001, nb = 120001;
  std::mt19937_64 mt(47);
  std::vector<int64_t> a(na), b(nb);
  for(auto& x : a) x = (int64_t)(mt() % 50000) << 33;
  for(auto& x : b) x = (int64_t)(mt() % 50000) << 33;
  std::sort(a.begin(), a.end()); std::sort(b.begin(), b.end());
  mem_t<int64_t> da = to_mem(a, context), db = to_mem(b, context);
  mem_t<int> found(na, context);
  sorted_search<bounds_upper>(da.data(), na, db.data(), nb, found.data(),
    less_t<int64_t>(), context);
  std::vector<int> f = from_mem(found);
  for(int i = 0; i < na; ++i)
    CHECK(f[i] == (int)(std::upper_bound(b.begin(), b.end(), a[i]) - b.begin()));

  mem_t<int2> joined = inner_join(da.data(), na, db.data(), nb,
    less_t<int64_t>(), context);
  std::vector<int2> pairs = from_mem(joined);
  size_t k = 0;
  for(int i = 0; i < na; ++i) {
    auto range = std::equal_range(b.begin(), b.end(), a[i]);
    for(auto it = range.first; it != range.second; ++it, ++k) {
      CHECK(k < pairs.size());
      CHECK(pairs[k].x == i && pairs[k].y == (int)(it - b.begin()));
    }
  }
  CHECK(k == pairs.size());

  // Needles from a counting iterator (0, 1, 2, ...) in a haystack of doubles.
  std::vector<double> h(40000);
  for(size_t i = 0; i < h.size(); ++i) h[i] = 1.5 * (double)(i / 3);
  mem_t<double> dh = to_mem(h, context);
  int needles = 50000;
  mem_t<int> lower(needles, context);
  sorted_search<bounds_lower>(counting_iterator_t<double>(0), needles,
    dh.data(), (int)h.size(), lower.data(), less_t<double>(), context);
  std::vector<int> lo = from_mem(lower);
  for(int i = 0; i < needles; ++i)
    CHECK(lo[i] == (int)(std::lower_bound(h.begin(), h.end(), (double)i) - h.begin()));
  return 0;
}

static int check_scans(context_t& context) {
  int n = 300007;
  std::vector<double> v(n);
  std::mt19937 mt(53);
  for(double& x : v) x = (double)((int)(mt() % 2001) - 1000);
  mem_t<double> dv = to_mem(v, context);
  mem_t<double> out(n, context), red(1, context);
  scan<scan_type_inc>(dv.data(), n, out.data(), maximum_t<double>(), red.data(),
    context);
  std::vector<double> got = from_mem(out);
  double run = v[0];
  for(int i = 0; i < n; ++i) { run = i ? max(run, v[i]) : v[0]; CHECK(got[i] == run); }
  CHECK(from_mem(red)[0] == run);

  mem_t<int64_t> sums(n, context);
  scan(counting_iterator_t<int64_t>(1), n, sums.data(), context);   // exclusive plus
  std::vector<int64_t> s = from_mem(sums);
  for(int i = 0; i < n; ++i) CHECK(s[i] == (int64_t)i * (i + 1) / 2);
  return 0;
}

// Every algorithm under a caller's launch box, from one wavefront with one
// item per thread to 1,024 threads.
template<typename box_t>
static int check_box(context_t& context) {
  int count = 70003, num_segments = 900;
  std::vector<int> seg_host = make_segments(count, num_segments, 61);
  mem_t<int> segments = to_mem(seg_host, context);
  std::vector<int> v(count);
  std::mt19937 mt(62);
  for(int& x : v) x = (int)(mt() % 2001) - 1000;
  mem_t<int> values = to_mem(v, context);

  mem_t<int> scanned(count, context), total(1, context);
  scan<scan_type_exc, box_t>(values.data(), count, scanned.data(), plus_t<int>(),
    total.data(), context);
  std::vector<int> sc = from_mem(scanned);
  int run = 0;
  for(int i = 0; i < count; ++i) { CHECK(sc[i] == run); run += v[i]; }
  CHECK(from_mem(total)[0] == run);

  mem_t<int> folded(1, context);
  reduce<box_t>(values.data(), count, folded.data(), maximum_t<int>(), context);
  CHECK(from_mem(folded)[0] == *std::max_element(v.begin(), v.end()));

  mem_t<int> sums(num_segments, context);
  lbs_segreduce<box_t>([]MGPU_DEVICE(int index, int seg, int rank,
    tuple<int> start, const int* values) {
      return values[index] + (get<0>(start) + rank - index);
    }, count, segments.data(), num_segments, make_tuple(segments.data()),
    sums.data(), plus_t<int>(), -1, context, values.data());
  std::vector<int> got = from_mem(sums);
  for(int s = 0; s < num_segments; ++s) {
    int b = seg_host[s], e = s + 1 < num_segments ? seg_host[s + 1] : count;
    int want = -1;
    for(int i = b; i < e; ++i) want = (i == b) ? v[i] : want + v[i];
    CHECK(got[s] == want);
  }

  // gather each segment from where a reversed layout of the segments put it
  std::vector<int> base(num_segments);
  int at = 0;
  for(int s = num_segments - 1; s >= 0; --s) {
    base[s] = at;
    at += (s + 1 < num_segments ? seg_host[s + 1] : count) - seg_host[s];
  }
  mem_t<int> bases = to_mem(base, context);
  mem_t<int> gathered(count, context), moved(count, context);
  interval_gather<box_t>(values.data(), count, segments.data(), num_segments,
    bases.data(), gathered.data(), context);
  interval_move<box_t>(gathered.data(), count, segments.data(), num_segments,
    bases.data(), segments.data(), moved.data(), context);
  std::vector<int> g = from_mem(gathered), mv = from_mem(moved);
  int seg = -1;
  for(int i = 0; i < count; ++i) {
    while(seg + 1 < num_segments && seg_host[seg + 1] <= i) ++seg;
    int rank = i - seg_host[seg];
    CHECK(g[i] == v[base[seg] + rank]);
    CHECK(mv[base[seg] + rank] == g[i]);
  }
  return 0;
}

// Segments that span hundreds of tiles under operators that do not commute:
// the carries of such a segment are folded by the spine in a loop of its own
// (rows of consecutive carries per wavefront, several wavefronts), and any
// carry taken out of order shows.  Affine maps x -> a x + b composed left to
// right, packed in 4 bytes (mod 2^16) and in 8 bytes (mod 2^32), and the
// 16-byte matrices above.
struct affine16_mul_t {
  MGPU_HOST_DEVICE unsigned operator()(unsigned f, unsigned g) const {
    unsigned fa = f >> 16, fb = f & 0xffff, ga = g >> 16, gb = g & 0xffff;
    return ((fa * ga) & 0xffff) << 16 | ((ga * fb + gb) & 0xffff);
  }
};
struct affine32_t {
  unsigned a, b;
  MGPU_HOST_DEVICE bool operator==(const affine32_t& r) const {
    return a == r.a && b == r.b;
  }
};
struct affine32_mul_t {
  MGPU_HOST_DEVICE affine32_t operator()(affine32_t f, affine32_t g) const {
    return affine32_t { f.a * g.a, g.a * f.b + g.b };
  }
};

template<typename type_t, typename op_t, typename make_t>
static int check_long_runs_of(make_t make, op_t op, type_t init,
  context_t& context) {
  const int counts[] = { 9000001, 2000003, 777777 };
  const int begins[] = { 5, 4099, 70001 };
  for(int count : counts) for(int begin : begins) {
    // An empty segment, a short one, the long one, a short tail.
    std::vector<int> seg_host = { 0, 0, begin, count - 7 };
    int num_segments = (int)seg_host.size();
    mem_t<int> segments = to_mem(seg_host, context);
    mem_t<type_t> results(num_segments, context);
    transform_segreduce(make, count, segments.data(), num_segments,
      results.data(), op, init, context);
    std::vector<type_t> got = from_mem(results);
    for(int s = 0; s < num_segments; ++s) {
      int b = seg_host[s], e = s + 1 < num_segments ? seg_host[s + 1] : count;
      type_t want = init;
      for(int i = b; i < e; ++i) want = (i == b) ? make(i) : op(want, make(i));
      CHECK(got[s] == want);
    }
  }
  return 0;
}

static int check_long_runs(context_t& context) {
  CHECK(0 == check_long_runs_of<unsigned>([] __host__ __device__ (int i) {
    return (unsigned)((1 + 2 * (i % 7)) << 16 | (i % 11));
  }, affine16_mul_t(), 0x10000u, context));
  CHECK(0 == check_long_runs_of<affine32_t>([] __host__ __device__ (int i) {
    return affine32_t { 1u + 2 * ((unsigned)i % 5), (unsigned)i % 13 };
  }, affine32_mul_t(), affine32_t { 1, 0 }, context));
  CHECK(0 == check_long_runs_of<mat_t>([] __host__ __device__ (int i) {
    return mat_of(i);
  }, mat_mul_t(), mat_t { 9, 9, 9, 9 }, context));
  return 0;
}

int main() {
  standard_context_t context(false);
  CHECK(0 == check_long_runs(context));
  CHECK(0 == (check_box<launch_params_t<64, 1> >(context)));
  CHECK(0 == (check_box<launch_params_t<64, 3> >(context)));
  CHECK(0 == (check_box<launch_params_t<128, 7> >(context)));
  CHECK(0 == (check_box<launch_params_t<256, 4> >(context)));
  CHECK(0 == (check_box<launch_params_t<512, 2> >(context)));
  CHECK(0 == (check_box<launch_params_t<1024, 1> >(context)));
  CHECK(0 == (check_box<launch_params_t<1024, 8> >(context)));
  CHECK(0 == check_wide_values(context));
  CHECK(0 == check_lbs_with_mixed_cache(context));
  CHECK(0 == check_wide_keys(context));
  CHECK(0 == check_scans(context));
  printf("api surface: all passed\n");
  return 0;
}
