// Exercises the template paths that have no extern "C" counterpart: user
// functors, user value types and operators, custom launch boxes (including a
// box written for CUDA architectures only), interval_expand and spmv through
// the mgpu:: API, and the context's allocator hooks.  Non-zero exit on error.
#include <moderngpu/kernel_segreduce.hxx>
#include <moderngpu/kernel_intervalmove.hxx>
#include <moderngpu/kernel_scan.hxx>
#include <cstdio>
#include <cmath>

using namespace mgpu;

#define CHECK(cond) do { if(!(cond)) { \
  printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); return 1; } } while(0)

// A user value type: running (min distance, index) pair.
struct best_t {
  float distance;
  int index;
};
struct best_min_t {
  MGPU_HOST_DEVICE best_t operator()(best_t a, best_t b) const {
    return (b.distance < a.distance) ? b : a;
  }
};

// A context that counts allocations: the documented extension point.
struct counting_context_t : standard_context_t {
  int allocs = 0, frees = 0;
  counting_context_t() : standard_context_t(false) { }
  virtual void* alloc(size_t size, memory_space_t space) {
    ++allocs;
    return standard_context_t::alloc(size, space);
  }
  virtual void free(void* p, memory_space_t space) {
    ++frees;
    standard_context_t::free(p, space);
  }
};

static std::vector<int> make_segments(int count, int num_segments, int seed) {
  std::mt19937 mt(seed);
  std::uniform_int_distribution<int> dist(0, count);
  std::vector<int> s(num_segments);
  s[0] = 0;
  for(int i = 1; i < num_segments; ++i) s[i] = dist(mt);
  std::sort(s.begin() + 1, s.end());
  return s;
}

template<typename launch_t>
static int run_boxed(context_t& context) {
  int count = 300000, num_segments = 2000;
  std::vector<int> seg_host = make_segments(count, num_segments, 7);
  mem_t<int> segments = to_mem(seg_host, context);
  mem_t<int64_t> results(num_segments, context);
  transform_segreduce<launch_t>([]MGPU_DEVICE(int index) {
    return (int64_t)index * 3;
  }, count, segments.data(), num_segments, results.data(),
    plus_t<int64_t>(), (int64_t)-9, context);
  std::vector<int64_t> got = from_mem(results);
  for(int s = 0; s < num_segments; ++s) {
    int64_t b = seg_host[s], e = s + 1 < num_segments ? seg_host[s + 1] : count;
    int64_t want = e > b ? 3 * ((e - 1) * e / 2 - (b - 1) * b / 2) : -9;
    CHECK(got[s] == want);
  }
  return 0;
}

// load_balance_search under a caller's launch box, against the host merge.
// Mean segment length 8: most tile boundaries have starts close behind them.
template<typename launch_t>
static int run_boxed_lbs(context_t& context) {
  int count = 200003, num_segments = 25000;
  std::vector<int> seg_host = make_segments(count, num_segments, 19);
  mem_t<int> segments = to_mem(seg_host, context);
  mem_t<int> found(count, context);
  load_balance_search<launch_t>(count, segments.data(), num_segments,
    found.data(), context);
  std::vector<int> got = from_mem(found);
  int seg = -1;
  for(int i = 0; i < count; ++i) {
    while(seg + 1 < num_segments && seg_host[seg + 1] <= i) ++seg;
    CHECK(got[i] == seg);
  }
  return 0;
}

int main() {
  counting_context_t context;

  // 1. launch boxes: gfx950-specific, CUDA-only (resolves through the
  // inheritance chain), odd vt (scalar path), fixed launch_params_t.
  typedef launch_box_t<arch_gfx950_cta<128, 8> > box_gfx_t;
  typedef launch_box_t<arch_20_cta<128, 11, 8>, arch_35_cta<128, 7, 5>,
    arch_52_cta<128, 11, 8> > box_cuda_t;
  static_assert(box_cuda_t::sm_ptx::vt == 7, "gfx950 inherits 35 -> ... -> 86");
  static_assert(box_gfx_t::sm_ptx::nt == 128 && box_gfx_t::sm_ptx::vt == 8, "");
  CHECK(0 == run_boxed<box_gfx_t>(context));
  CHECK(0 == run_boxed<box_cuda_t>(context));
  CHECK(0 == (run_boxed<launch_params_t<64, 5> >(context)));
  CHECK(0 == run_boxed<empty_t>(context));
  // The search with tiles from 64 to 896 elements.
  CHECK(0 == run_boxed_lbs<box_cuda_t>(context));
  CHECK(0 == (run_boxed_lbs<launch_params_t<64, 1> >(context)));
  CHECK(0 == (run_boxed_lbs<launch_params_t<64, 4> >(context)));
  CHECK(0 == (run_boxed_lbs<launch_params_t<64, 5> >(context)));
  CHECK(0 == (run_boxed_lbs<launch_params_t<128, 3> >(context)));
  CHECK(0 == (run_boxed_lbs<launch_params_t<256, 2> >(context)));
  CHECK(context.allocs > 0 && context.frees > 0);

  // 2. user value type + user operator through segreduce.
  {
    int count = 100000, num_segments = 777;
    std::vector<int> seg_host = make_segments(count, num_segments, 3);
    std::vector<float> dist_host(count);
    std::mt19937 mt(5);
    for(float& d : dist_host) d = (float)(mt() % 100000) / 7.0f;
    mem_t<int> segments = to_mem(seg_host, context);
    mem_t<float> dist = to_mem(dist_host, context);
    mem_t<best_t> results(num_segments, context);
    const float* d = dist.data();
    best_t init = { -1.0f, -1 };
    transform_segreduce([=]MGPU_DEVICE(int index) {
      return best_t { d[index], index };
    }, count, segments.data(), num_segments, results.data(), best_min_t(),
      init, context);
    std::vector<best_t> got = from_mem(results);
    for(int s = 0; s < num_segments; ++s) {
      int b = seg_host[s], e = s + 1 < num_segments ? seg_host[s + 1] : count;
      best_t want = init;
      for(int i = b; i < e; ++i) {
        best_t y = { dist_host[i], i };
        want = (i == b) ? y : best_min_t()(want, y);
      }
      CHECK(got[s].index == want.index && got[s].distance == want.distance);
    }
  }

  // 3. segreduce on raw pointers with the built-in operators (the path that
  // the C launcher also instantiates), float max.
  {
    int count = 123457, num_segments = 900;
    std::vector<int> seg_host = make_segments(count, num_segments, 11);
    std::vector<float> v(count);
    std::mt19937 mt(6);
    for(float& x : v) x = (float)((int)(mt() % 2001) - 1000);
    mem_t<int> segments = to_mem(seg_host, context);
    mem_t<float> values = to_mem(v, context);
    mem_t<float> results(num_segments, context);
    segreduce(values.data(), count, segments.data(), num_segments,
      results.data(), maximum_t<float>(), -5000.0f, context);
    std::vector<float> got = from_mem(results);
    for(int s = 0; s < num_segments; ++s) {
      int b = seg_host[s], e = s + 1 < num_segments ? seg_host[s + 1] : count;
      float want = -5000.0f;
      for(int i = b; i < e; ++i) want = (i == b) ? v[i] : mgpu::max(want, v[i]);
      CHECK(got[s] == want);
    }
  }

  // 4. interval_expand + transform_lbs with a cached tuple and extra args.
  {
    int count = 250000, num_segments = 5000;
    std::vector<int> seg_host = make_segments(count, num_segments, 13);
    std::vector<float> val_host(num_segments);
    for(int i = 0; i < num_segments; ++i) val_host[i] = 0.5f * i;
    mem_t<int> segments = to_mem(seg_host, context);
    mem_t<float> vals = to_mem(val_host, context);
    mem_t<float> expanded(count, context);
    interval_expand(vals.data(), count, segments.data(), num_segments,
      expanded.data(), context);
    mem_t<int> ranks(count, context);
    mem_t<int> segs(count, context);
    transform_lbs([]MGPU_DEVICE(int index, int seg, int rank,
      tuple<int, float> cached, int* ranks, int* segs) {
      ranks[index] = rank + (get<0>(cached) - get<0>(cached));
      segs[index] = seg;
    }, count, segments.data(), num_segments,
      make_tuple(segments.data(), vals.data()), context, ranks.data(),
      segs.data());
    std::vector<float> e_host = from_mem(expanded);
    std::vector<int> r_host = from_mem(ranks), s_host = from_mem(segs);
    int seg = -1;
    for(int i = 0; i < count; ++i) {
      while(seg + 1 < num_segments && seg_host[seg + 1] <= i) ++seg;
      CHECK(s_host[i] == seg);
      CHECK(r_host[i] == i - seg_host[seg]);
      CHECK(e_host[i] == val_host[seg]);
    }
  }

  // 5. spmv through the template (double), against the textbook loop.
  {
    int rows = 4000;
    std::mt19937 mt(17);
    std::vector<int> row_host(rows), col_host;
    std::vector<double> a_host, x_host(rows);
    for(double& x : x_host) x = (double)(mt() % 1000) / 500.0 - 1.0;
    for(int r = 0; r < rows; ++r) {
      row_host[r] = (int)col_host.size();
      int nnz = mt() % 40;
      for(int k = 0; k < nnz; ++k) {
        col_host.push_back(mt() % rows);
        a_host.push_back((double)(mt() % 1000) / 500.0 - 1.0);
      }
    }
    int nnz = (int)col_host.size();
    mem_t<int> row = to_mem(row_host, context), col = to_mem(col_host, context);
    mem_t<double> a = to_mem(a_host, context), x = to_mem(x_host, context);
    mem_t<double> y(rows, context);
    spmv(a.data(), col.data(), x.data(), nnz, row.data(), rows, y.data(),
      context);
    std::vector<double> y_host = from_mem(y);
    for(int r = 0; r < rows; ++r) {
      int b = row_host[r], e = r + 1 < rows ? row_host[r + 1] : nnz;
      double want = 0, norm = 0;
      for(int k = b; k < e; ++k) {
        want += a_host[k] * x_host[col_host[k]];
        norm += fabs(a_host[k] * x_host[col_host[k]]);
      }
      CHECK(fabs(y_host[r] - want) <= 1e-12 * norm + 1e-300);
    }
  }

  // 6. zero sizes launch nothing and allocate null.
  {
    mem_t<int> nothing(0, context);
    CHECK(nothing.data() == nullptr);
    mem_t<int> segments = to_mem(std::vector<int> { 0 }, context);
    mem_t<int> out(1, context);
    load_balance_search(0, segments.data(), 0, out.data(), context);
    context.synchronize();
  }

  // 7. iterators that are not pointers on every side: segment starts through
  // a load iterator, values from a counting iterator, results through a
  // load/store iterator; the search stored through a store iterator; scan
  // into a store iterator.
  {
    int count = 180001, num_segments = 3000;
    std::vector<int> seg_host = make_segments(count, num_segments, 23);
    mem_t<int> segments = to_mem(seg_host, context);
    const int* seg_data = segments.data();
    auto seg_it = make_load_iterator<int>(
      [=]MGPU_DEVICE(int i) { return seg_data[i]; });

    mem_t<int64_t> results(num_segments, context);
    int64_t* res_data = results.data();
    auto res_it = make_load_store_iterator<int64_t>(
      [=]MGPU_DEVICE(int i) { return res_data[i] - 5; },
      [=]MGPU_DEVICE(int64_t x, int i) { res_data[i] = x + 5; });
    segreduce(counting_iterator_t<int64_t>(0), count, seg_it, num_segments,
      res_it, plus_t<int64_t>(), (int64_t)-9, context);
    std::vector<int64_t> got = from_mem(results);
    for(int s = 0; s < num_segments; ++s) {
      int64_t b = seg_host[s], e = s + 1 < num_segments ? seg_host[s + 1] : count;
      int64_t want = e > b ? (e - 1) * e / 2 - (b - 1) * b / 2 : -9;
      CHECK(got[s] == want + 5);
    }

    mem_t<int> found(count, context);
    int* found_data = found.data();
    load_balance_search(count, seg_it, num_segments, make_store_iterator<int>(
      [=]MGPU_DEVICE(int seg, int i) { found_data[i] = 2 * seg + 1; }), context);
    std::vector<int> f = from_mem(found);
    int seg = -1;
    for(int i = 0; i < count; ++i) {
      while(seg + 1 < num_segments && seg_host[seg + 1] <= i) ++seg;
      CHECK(f[i] == 2 * seg + 1);
    }

    mem_t<float> expanded(count, context);
    interval_expand(strided_iterator_t<int>(7, 3), count, seg_it,
      num_segments, expanded.data(), context);
    std::vector<float> ex = from_mem(expanded);
    seg = -1;
    for(int i = 0; i < count; ++i) {
      while(seg + 1 < num_segments && seg_host[seg + 1] <= i) ++seg;
      CHECK(ex[i] == (float)(7 + 3 * seg));
    }

    mem_t<int> scanned(count, context);
    int* scanned_data = scanned.data();
    mem_t<int> total(1, context);
    scan(counting_iterator_t<int>(0), count, make_store_iterator<int>(
      [=]MGPU_DEVICE(int x, int i) { scanned_data[i] = x ^ 1; }),
      plus_t<int>(), total.data(), context);
    std::vector<int> sc = from_mem(scanned);
    for(int i = 0; i < count; ++i)
      CHECK(sc[i] == ((int)((int64_t)i * (i - 1) / 2) ^ 1));
    CHECK(from_mem(total)[0] == (int)((int64_t)count * (count - 1) / 2));
  }

  // 8. timer and properties.
  context.timer_begin();
  double seconds = context.timer_end();
  CHECK(seconds >= 0);
  CHECK(context.props().multiProcessorCount > 0);
  CHECK(context.ptx_version() >= 900);

  printf("templates: all passed\n");
  return 0;
}
