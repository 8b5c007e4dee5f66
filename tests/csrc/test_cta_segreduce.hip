// A segmented reduction assembled by the caller from the building blocks the
// reference's own kernel uses (moderngpu src/moderngpu/kernel_segreduce.hxx:
// 219-271): load_balance_partitions, compute_merge_range, mem_to_shared,
// cta_load_balance_place, the thread's merge bits, detail::cta_segreduce_t
// and detail::segreduce_fixup.  Checked against a host loop for several tile
// shapes, segment shapes (many short, few long, empty ones, a segment start
// as the last element of a tile) and a non-commutative operator.
// Exit status 1 on the first mismatch.
#include <moderngpu/kernel_segreduce.hxx>
#include <algorithm>
#include <cstdio>
#include <random>
#include <vector>

using namespace mgpu;

#define CHECK(cond) do { if(!(cond)) { \
  printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); return 1; } } while(0)

// x -> a * x + b over the integers mod 2^32, folded left to right:
// associative, not commutative.
struct affine_t {
  unsigned a, b;
};
struct compose_t {
  MGPU_HOST_DEVICE affine_t operator()(affine_t f, affine_t g) const {
    return affine_t { f.a * g.a, g.a * f.b + g.b };   // g after f
  }
};
static bool same(int x, int y) { return x == y; }
static bool same(affine_t x, affine_t y) { return x.a == y.a && x.b == y.b; }

template<int nt, int vt, typename type_t, typename op_t, typename make_t>
static int run(const std::vector<int>& seg_host, int count, type_t init,
  op_t op, make_t make, context_t& context) {
  enum { nv = nt * vt };
  int num_segments = (int)seg_host.size();
  std::vector<type_t> in_host(count);
  for(int i = 0; i < count; ++i) in_host[i] = make(i);
  mem_t<type_t> input = to_mem(in_host, context);
  mem_t<int> segments = to_mem(seg_host, context);
  mem_t<type_t> output(num_segments, context);

  int num_ctas = div_up(count + num_segments, (int)nv);
  mem_t<type_t> carry_values(num_ctas, context);
  mem_t<int> carry_codes(num_ctas, context);
  mem_t<int> mp = load_balance_partitions(count, segments.data(),
    num_segments, nv, context);

  const type_t* in = input.data();
  const int* segs = segments.data();
  const int* mp_data = mp.data();
  type_t* out = output.data();
  type_t* values = carry_values.data();
  int* codes = carry_codes.data();

  cta_launch<nt>([=]MGPU_DEVICE(int tid, int cta) {
    typedef detail::cta_segreduce_t<nt, vt, type_t> segreduce_t;
    __shared__ union {
      typename segreduce_t::storage_t segreduce;
      type_t room[nv + 2];        // items and starts of a tile: nv + 2 slots
    } shared;

    merge_range_t range = compute_merge_range(count, num_segments, cta, nv,
      mp_data[cta], mp_data[cta + 1]);
    mem_to_shared<nt, vt>(in + range.a_begin, tid, range.a_count(),
      shared.segreduce.values);

    int* starts = (int*)(shared.segreduce.values + range.a_count());
    lbs_placement_t placement = cta_load_balance_place<nt, vt>(tid, range,
      count, segs, num_segments, starts);
    starts -= placement.range.b_begin;

    int item = placement.a_index, segment = placement.b_index;
    array_t<bool, vt + 1> bits;
    iterate<vt + 1>([&](int i) {
      bool is_item = item < starts[segment + 1];
      if(is_item) ++item; else ++segment;
      bits[i] = is_item;
    });

    segreduce_t().segreduce(range, placement, bits, tid, cta, init, op, out,
      values, codes, shared.segreduce);
  }, num_ctas, context);

  if(num_ctas > 1)
    detail::segreduce_fixup(out, values, codes, num_ctas, op, init, context);

  std::vector<type_t> got = from_mem(output);
  for(int s = 0; s < num_segments; ++s) {
    int begin = seg_host[s];
    int end = s + 1 < num_segments ? seg_host[s + 1] : count;
    type_t x = init;
    for(int i = begin; i < end; ++i) x = (i == begin) ? in_host[i] : op(x, in_host[i]);
    if(!same(got[s], x)) {
      printf("nt=%d vt=%d count=%d segments=%d: segment %d [%d, %d) differs\n",
        nt, vt, count, num_segments, s, begin, end);
      return 1;
    }
  }
  return 0;
}

static std::vector<int> random_segments(int count, int num_segments, int seed) {
  std::mt19937 mt(seed);
  std::uniform_int_distribution<int> dist(0, count);
  std::vector<int> s(num_segments);
  s[0] = 0;
  for(int i = 1; i < num_segments; ++i) s[i] = dist(mt);
  std::sort(s.begin() + 1, s.end());
  return s;
}

template<int nt, int vt>
static int shapes(context_t& context) {
  enum { nv = nt * vt };
  auto ints = [](int i) { return (i * 2654435761u >> 20) % 1000 - 300; };
  auto maps = [](int i) { return affine_t { 2u * i + 1, 7u * i + 3 }; };
  affine_t identity = { 1, 0 };

  // Many short segments, a few long ones, lots of empty ones.
  CHECK(0 == (run<nt, vt>(random_segments(200000, 30000, 1), 200000, -1,
    plus_t<int>(), ints, context)));
  CHECK(0 == (run<nt, vt>(random_segments(300000, 5, 2), 300000, 0,
    maximum_t<int>(), ints, context)));
  CHECK(0 == (run<nt, vt>(random_segments(1000, 50000, 3), 1000, 17,
    plus_t<int>(), ints, context)));
  CHECK(0 == (run<nt, vt>(random_segments(150000, 4000, 4), 150000, identity,
    compose_t(), maps, context)));
  CHECK(0 == (run<nt, vt>(random_segments(250000, 3, 5), 250000, identity,
    compose_t(), maps, context)));

  // Segment k starts at item k * (nv - 1): start k is merged element
  // k * nv + ... so that starts fall on the last and first slots of tiles.
  for(int shift = 0; shift < 3; ++shift) {
    int num_segments = 40, count = 40 * nv;
    std::vector<int> s(num_segments);
    for(int k = 0; k < num_segments; ++k)
      s[k] = k ? std::min(count, k * (nv - 1) + shift - 1) : 0;
    CHECK(0 == (run<nt, vt>(s, count, -5, plus_t<int>(), ints, context)));
    CHECK(0 == (run<nt, vt>(s, count, identity, compose_t(), maps, context)));
  }
  // One segment over everything; no items at all; one tile only.
  CHECK(0 == (run<nt, vt>(std::vector<int>(1, 0), 100000, 0, plus_t<int>(),
    ints, context)));
  CHECK(0 == (run<nt, vt>(std::vector<int>(300, 0), 0, 9, plus_t<int>(),
    ints, context)));
  CHECK(0 == (run<nt, vt>(random_segments(nv / 2, nv / 4, 6), nv / 2, 0,
    plus_t<int>(), ints, context)));
  return 0;
}

int main() {
  standard_context_t context(false);
  CHECK(0 == (shapes<128, 7>(context)));
  CHECK(0 == (shapes<64, 3>(context)));
  CHECK(0 == (shapes<256, 4>(context)));
  printf("cta_segreduce: all passed\n");
  return 0;
}
