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
#include <moderngpu/kernel_merge.hxx>
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

// serial_search: a CTA holds both key arrays in LDS, every thread merges vt
// keys from its merge-path split and reports key, position, source and match
// bits; the host merges the same arrays with std::merge's tie rules and looks
// the keys up in the other array.
template<bounds_t bounds>
static int check_serial_search(int na, int nb, int max_key, context_t& context) {
  enum { nt = 128, vt = 5, nv = nt * vt };
  CHECK(na + nb <= nv);
  mem_t<int> a = fill_random(0, max_key, na, true, context);
  mem_t<int> b = fill_random(0, max_key, nb, true, context);
  mem_t<int> keys(nv, context), where(nv, context), flags(3 * nt, context);
  const int* a_data = a.data(); const int* b_data = b.data();
  int* keys_data = keys.data(); int* where_data = where.data();
  int* flags_data = flags.data();
  cta_launch<nt>([=]MGPU_DEVICE(int tid, int) {
    __shared__ int shared[nv + 1];
    for(int i = tid; i < na; i += nt) shared[i] = a_data[i];
    for(int i = tid; i < nb; i += nt) shared[na + i] = b_data[i];
    __syncthreads();
    merge_range_t tile { 0, na, 0, nb };
    merge_range_t local = tile.to_local();
    int diag = min(vt * tid, na + nb);
    int mp = merge_path<bounds>(shared, local, diag, less_t<int>());
    merge_range_t mine = local.partition(mp, diag);
    search_result_t<int, vt> r = serial_search<vt, bounds, true>(shared, mine,
      0, -na, less_t<int>());
    for(int i = 0; i < vt; ++i) {
      keys_data[vt * tid + i] = r.keys[i];
      where_data[vt * tid + i] = r.indices[i];
    }
    flags_data[3 * tid + 0] = r.decisions;
    flags_data[3 * tid + 1] = r.matches_a;
    flags_data[3 * tid + 2] = r.matches_b;
  }, 1, context);

  std::vector<int> ha = from_mem(a), hb = from_mem(b), hk = from_mem(keys),
    hw = from_mem(where), hf = from_mem(flags);
  int ia = 0, ib = 0;
  for(int p = 0; p < na + nb; ++p) {
    bool take_a;
    if(ia >= na) take_a = false;
    else if(ib >= nb) take_a = true;
    else take_a = (bounds_upper == bounds) ? ha[ia] < hb[ib] : !(hb[ib] < ha[ia]);
    int key = take_a ? ha[ia] : hb[ib];
    int at = take_a ? ia : ib;
    bool match = take_a ? std::binary_search(hb.begin(), hb.end(), key) :
      std::binary_search(ha.begin(), ha.end(), key);
    int tid = p / vt, i = p % vt;
    CHECK(hk[p] == key && hw[p] == at);
    CHECK(((hf[3 * tid + 0] >> i) & 1) == (int)take_a);
    CHECK(((hf[3 * tid + 1] >> i) & 1) == (int)(take_a && match));
    CHECK(((hf[3 * tid + 2] >> i) & 1) == (int)(!take_a && match));
    if(take_a) ++ia; else ++ib;
  }
  return 0;
}

// A key/value merge assembled from cta_merge_from_mem (which stands on
// load_two_streams_shared, merge_path and serial_merge) and
// transfer_two_streams_strided, with merge_path_partitions for the tiles --
// the way a merge kernel is put together from the CTA-level blocks (moderngpu
// src/moderngpu/kernel_merge.hxx:30-71).  Values identify where a key came
// from (a: its index, b: -1 - index), so the order of equal keys is checked
// too: a stable merge takes equal keys from a first.
template<int nt, int vt>
static int check_cta_merge(int na, int nb, int max_key, context_t& context) {
  enum { nv = nt * vt };
  mem_t<int> a = fill_random(0, max_key, na, true, context);
  mem_t<int> b = fill_random(0, max_key, nb, true, context);
  mem_t<int> a_vals(na, context), b_vals(nb, context);
  mem_t<int> keys(na + nb, context), vals(na + nb, context);
  int* av = a_vals.data(); int* bv = b_vals.data();
  transform([=]MGPU_DEVICE(int i) { av[i] = i; }, na, context);
  transform([=]MGPU_DEVICE(int i) { bv[i] = -1 - i; }, nb, context);
  mem_t<int> mp = merge_path_partitions<bounds_lower>(a.data(), na, b.data(),
    nb, nv, less_t<int>(), context);
  const int* a_keys = a.data(); const int* b_keys = b.data();
  const int* mp_data = mp.data();
  int* c_keys = keys.data(); int* c_vals = vals.data();
  int num_ctas = div_up(na + nb, (int)nv);
  cta_launch<nt>([=]MGPU_DEVICE(int tid, int cta) {
    __shared__ union { int keys[nv + 1]; int indices[nv]; } shared;
    merge_range_t range = compute_merge_range(na, nb, cta, nv, mp_data[cta],
      mp_data[cta + 1]);
    merge_pair_t<int, vt> merged = cta_merge_from_mem<bounds_lower, nt, vt>(
      a_keys, b_keys, range, tid, less_t<int>(), shared.keys);
    reg_to_mem_thread<nt>(merged.keys, tid, range.total(), c_keys + nv * cta,
      shared.keys);
    array_t<int, vt> where = reg_thread_to_strided<nt>(merged.indices, tid,
      shared.indices);
    transfer_two_streams_strided<nt>(av + range.a_begin, range.a_count(),
      bv + range.b_begin, range.b_count(), where, tid, c_vals + nv * cta);
  }, num_ctas, context);

  std::vector<int> ha = from_mem(a), hb = from_mem(b), hk = from_mem(keys),
    hv = from_mem(vals);
  int ia = 0, ib = 0;
  for(int p = 0; p < na + nb; ++p) {
    bool take_a = ia < na && (ib >= nb || !(hb[ib] < ha[ia]));
    CHECK(hk[p] == (take_a ? ha[ia] : hb[ib]));
    CHECK(hv[p] == (take_a ? ia : -1 - ib));
    if(take_a) ++ia; else ++ib;
  }
  return 0;
}

// merge(): keys with values and keys alone, against a host merge.
template<typename launch_t>
static int check_merge(int na, int nb, int max_key, context_t& context) {
  mem_t<int> a = fill_random(0, max_key, na, true, context);
  mem_t<int> b = fill_random(0, max_key, nb, true, context);
  mem_t<int> a_vals(na, context), b_vals(nb, context);
  int* av = a_vals.data(); int* bv = b_vals.data();
  transform([=]MGPU_DEVICE(int i) { av[i] = i; }, na, context);
  transform([=]MGPU_DEVICE(int i) { bv[i] = -1 - i; }, nb, context);
  mem_t<int> keys(na + nb, context), vals(na + nb, context), only(na + nb, context);
  merge<launch_t>(a.data(), a_vals.data(), na, b.data(), b_vals.data(), nb,
    keys.data(), vals.data(), less_t<int>(), context);
  merge<launch_t>(a.data(), na, b.data(), nb, only.data(), less_t<int>(), context);
  std::vector<int> ha = from_mem(a), hb = from_mem(b), hk = from_mem(keys),
    hv = from_mem(vals), ho = from_mem(only);
  int ia = 0, ib = 0;
  for(int p = 0; p < na + nb; ++p) {
    bool take_a = ia < na && (ib >= nb || !(hb[ib] < ha[ia]));
    int key = take_a ? ha[ia] : hb[ib];
    CHECK(hk[p] == key && ho[p] == key);
    CHECK(hv[p] == (take_a ? ia : -1 - ib));
    if(take_a) ++ia; else ++ib;
  }
  return 0;
}

int main() {
  standard_context_t context(false);
  CHECK(0 == check_merge<empty_t>(1000000, 700000, 1 << 20, context));
  CHECK(0 == check_merge<empty_t>(5000, 300000, 50, context));
  CHECK(0 == (check_merge<launch_params_t<128, 7> >(100000, 99999, 1000, context)));
  CHECK(0 == check_merge<empty_t>(0, 4096, 100, context));
  CHECK(0 == check_merge<empty_t>(1, 0, 100, context));
  CHECK(0 == (check_cta_merge<128, 7>(100000, 130000, 5000, context)));
  CHECK(0 == (check_cta_merge<64, 4>(3000, 50, 40, context)));
  CHECK(0 == (check_cta_merge<256, 3>(1, 70000, 1 << 30, context)));
  CHECK(0 == (check_cta_merge<128, 7>(896 * 5, 896 * 3, 100, context)));
  CHECK(0 == (check_cta_merge<128, 5>(0, 1000, 100, context)));
  CHECK(0 == check_serial_search<bounds_lower>(300, 340, 200, context));
  CHECK(0 == check_serial_search<bounds_upper>(300, 340, 200, context));
  CHECK(0 == check_serial_search<bounds_lower>(100, 500, 10000, context));
  CHECK(0 == check_serial_search<bounds_upper>(520, 17, 30, context));
  CHECK(0 == check_serial_search<bounds_lower>(0, 64, 30, context));
  CHECK(0 == check_serial_search<bounds_upper>(64, 0, 30, context));
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
