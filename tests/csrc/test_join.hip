// C++ callers of sorted_search and inner_join.
//  - the reference's sorted-search test (moderngpu tests/test_sortedsearch.cu:
//    1000 sorted needles and 1000 sorted haystack keys drawn from [0, 10000],
//    bounds_lower, each index bracketed by its neighbours) at that size and at
//    larger ones, for both bounds and several launch boxes, float keys with a
//    user comparator included;
//  - the reference's join test (tests/test_join.cu: two empty inputs) and
//    joins of random keys checked pair by pair against a host loop.
// Exit status 1 on the first mismatch.
#include <moderngpu/kernel_join.hxx>
#include <algorithm>
#include <cstdio>
#include <functional>

using namespace mgpu;

#define CHECK(cond) do { if(!(cond)) { \
  printf("%s:%d: CHECK(%s) failed\n", __FILE__, __LINE__, #cond); return 1; \
} } while(0)

template<typename launch_t>
static int check_search(int num_needles, int num_haystack, int max_key,
  context_t& context) {
  mem_t<int> needles = fill_random(0, max_key, num_needles, true, context);
  mem_t<int> haystack = fill_random(0, max_key, num_haystack, true, context);
  std::vector<int> n = from_mem(needles), h = from_mem(haystack);

  mem_t<int> lower(num_needles, context), upper(num_needles, context);
  sorted_search<bounds_lower, launch_t>(needles.data(), num_needles,
    haystack.data(), num_haystack, lower.data(), less_t<int>(), context);
  sorted_search<bounds_upper, launch_t>(needles.data(), num_needles,
    haystack.data(), num_haystack, upper.data(), less_t<int>(), context);
  std::vector<int> lo = from_mem(lower), up = from_mem(upper);
  for(int i = 0; i < num_needles; ++i) {
    // everything in front of the lower bound is smaller, nothing at it is
    CHECK(lo[i] >= 0 && lo[i] <= num_haystack);
    CHECK(lo[i] <= 0 || n[i] > h[lo[i] - 1]);
    CHECK(lo[i] >= num_haystack || n[i] <= h[lo[i]]);
    // everything in front of the upper bound is not greater, what is at it is
    CHECK(up[i] >= lo[i] && up[i] <= num_haystack);
    CHECK(up[i] <= 0 || n[i] >= h[up[i] - 1]);
    CHECK(up[i] >= num_haystack || n[i] < h[up[i]]);
  }
  return 0;
}

// Descending float keys under greater_t.
static int check_search_descending(context_t& context) {
  int count = 70001;
  std::vector<float> n(count), h(count / 2);
  for(int i = 0; i < count; ++i) n[i] = (float)((count - i) / 3) * 0.5f;
  for(size_t i = 0; i < h.size(); ++i) h[i] = (float)((h.size() - i) / 2) * 0.75f;
  mem_t<float> needles = to_mem(n, context), haystack = to_mem(h, context);
  mem_t<int> found(count, context);
  sorted_search<bounds_lower>(needles.data(), count, haystack.data(),
    (int)h.size(), found.data(), greater_t<float>(), context);
  std::vector<int> got = from_mem(found);
  for(int i = 0; i < count; ++i) {
    int want = (int)(std::lower_bound(h.begin(), h.end(), n[i],
      std::greater<float>()) - h.begin());
    CHECK(got[i] == want);
  }
  return 0;
}

template<typename launch_t>
static int check_join(int a_count, int b_count, int max_key,
  context_t& context) {
  mem_t<int> a = fill_random(0, max_key, a_count, true, context);
  mem_t<int> b = fill_random(0, max_key, b_count, true, context);
  std::vector<int> ah = from_mem(a), bh = from_mem(b);
  mem_t<int2> joined = inner_join<launch_t>(a.data(), a_count, b.data(),
    b_count, less_t<int>(), context);
  std::vector<int2> got = from_mem(joined);

  size_t k = 0;
  int lo = 0;
  for(int i = 0; i < a_count; ++i) {
    while(lo < b_count && bh[lo] < ah[i]) ++lo;
    for(int j = lo; j < b_count && bh[j] == ah[i]; ++j, ++k) {
      CHECK(k < got.size());
      if(got[k].x != i || got[k].y != j) {
        printf("pair %d is (%d, %d), expected (%d, %d)\n", (int)k, got[k].x,
          got[k].y, i, j);
        return 1;
      }
    }
  }
  CHECK(k == got.size());
  return 0;
}

int main() {
  standard_context_t context(false);
  typedef launch_box_t<arch_20_cta<128, 15>, arch_35_cta<128, 11>,
    arch_52_cta<128, 15> > box_cuda_t;        // the reference's default
  CHECK(0 == check_search<empty_t>(1000, 1000, 10000, context));
  CHECK(0 == check_search<empty_t>(500000, 300000, 1000, context));     // long equal runs
  CHECK(0 == check_search<empty_t>(300000, 500000, 1 << 30, context));  // mostly distinct
  CHECK(0 == check_search<box_cuda_t>(100000, 100000, 100000, context));
  CHECK(0 == (check_search<launch_params_t<64, 3> >(30000, 20000, 5000, context)));
  CHECK(0 == check_search<empty_t>(5, 0, 10, context));
  CHECK(0 == check_search<empty_t>(0, 5, 10, context));
  CHECK(0 == check_search_descending(context));

  mem_t<int2> none = inner_join((int*)nullptr, 0, (int*)nullptr, 0,
    less_t<int>(), context);
  CHECK(0 == none.size());
  CHECK(0 == check_join<empty_t>(1000, 1000, 10000, context));
  CHECK(0 == check_join<empty_t>(200000, 100000, 30000, context));
  CHECK(0 == check_join<empty_t>(3000, 2000, 3, context));     // ~1.5M pairs from 4 keys
  CHECK(0 == check_join<box_cuda_t>(50000, 60000, 100000, context));
  CHECK(0 == check_join<empty_t>(100, 0, 10, context));
  printf("join: all passed\n");
  return 0;
}
