// The nearest-cities pipeline of the reference's demo (moderngpu
// demo/cities.cu:140-222, everything in front of its segmented sort) on a
// sample of the demo's own data file: for every city the three closest cities
// of the same state.
//   1. scan of the cities per state                  -> state segments
//   2. interval_expand of the state segments         -> first city of each city's state
//   3. transform_lbs with the state sizes cached     -> comparisons per city
//   4. scan of those                                 -> one segment per city
//   5. lbs_segreduce over all (city, other city) pairs with a 24-byte value
//      type, a merge-of-sorted-triples operator, two cached iterators and an
//      explicit 128 x 3 launch box.
// Checked against a host loop over all pairs with the same operator; distances
// are formed with the same roundings on both sides, so the comparison is exact.
// usage: test_cities <statecity_sample.csv>
#include <moderngpu/kernel_segreduce.hxx>
#include <moderngpu/kernel_intervalmove.hxx>
#include <moderngpu/kernel_scan.hxx>
#include <cfloat>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

using namespace mgpu;

#define CHECK(cond) do { if(!(cond)) { \
  printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); return 1; } } while(0)

enum { closest = 3 };
struct near_t {
  float score[closest];
  int city[closest];
};
MGPU_HOST_DEVICE near_t one_city(float score, int city) {
  near_t x;
  for(int i = 0; i < closest; ++i) { x.score[i] = FLT_MAX; x.city[i] = -1; }
  x.score[0] = score; x.city[0] = city;
  return x;
}
// The closest three of two ascending triples; on equal scores the left
// operand's entry goes first.
struct closer_t {
  MGPU_HOST_DEVICE near_t operator()(near_t a, near_t b) const {
    near_t c;
    int ia = 0, ib = 0;
    for(int i = 0; i < closest; ++i) {
      bool take_a = !(b.score[ib] < a.score[ia]);
      c.score[i] = take_a ? a.score[ia] : b.score[ib];
      c.city[i] = take_a ? a.city[ia] : b.city[ib];
      if(take_a) ++ia; else ++ib;
    }
    return c;
  }
};
// The same two roundings on host and device: dy * dy, then one fused
// multiply-add (which both compute exactly rounded), whatever the compiler's
// contraction setting.
MGPU_HOST_DEVICE float squared_distance(float2 p, float2 q) {
#pragma clang fp contract(off)
  float dx = p.x - q.x, dy = p.y - q.y;
  float yy = dy * dy;
  return fmaf(dx, dx, yy);
}

int main(int argc, char** argv) {
  CHECK(argc > 1);
  FILE* f = fopen(argv[1], "r");
  CHECK(f);
  std::vector<int> per_state;
  std::vector<float2> pos;
  char line[256], state[8], last[8] = "";
  CHECK(fgets(line, sizeof(line), f));            // header
  while(fgets(line, sizeof(line), f)) {
    float lat, lon;
    CHECK(3 == sscanf(line, "%7[^,],%f,%f", state, &lat, &lon));
    if(strcmp(state, last)) { per_state.push_back(0); strcpy(last, state); }
    ++per_state.back();
    pos.push_back(make_float2(lon, lat));
  }
  fclose(f);
  int num_states = (int)per_state.size(), num_cities = (int)pos.size();
  CHECK(num_states >= 10 && num_cities > 2000);

  standard_context_t context(false);
  mem_t<int> counts = to_mem(per_state, context);
  mem_t<float2> city_pos = to_mem(pos, context);

  mem_t<int> state_segments(num_states, context);
  scan(counts.data(), num_states, state_segments.data(), context);

  mem_t<int> first_city(num_cities, context);
  interval_expand(state_segments.data(), num_cities, state_segments.data(),
    num_states, first_city.data(), context);

  mem_t<int> pair_segments(num_cities, context);
  int* pair_data = pair_segments.data();
  transform_lbs([=]MGPU_DEVICE(int index, int, int, tuple<int> size) {
    pair_data[index] = get<0>(size) - 1;
  }, num_cities, state_segments.data(), num_states,
    make_tuple(counts.data()), context);
  scan(pair_segments.data(), num_cities, pair_segments.data(), context);

  int num_pairs = 0;
  for(int c : per_state) num_pairs += c * (c - 1);

  const float2* where = city_pos.data();
  mem_t<near_t> nearest(num_cities, context);
  near_t init;
  for(int i = 0; i < closest; ++i) { init.score[i] = 0; init.city[i] = -1; }
  lbs_segreduce<launch_params_t<128, 3> >(
    [=]MGPU_DEVICE(int, int city, int rank, tuple<int, float2> cached) {
      int other = get<0>(cached) + rank;
      if(other >= city) ++other;                  // skip the city itself
      return one_city(squared_distance(get<1>(cached), where[other]), other);
    }, num_pairs, pair_segments.data(), num_cities,
    make_tuple(first_city.data(), city_pos.data()), nearest.data(),
    closer_t(), init, context);

  // Host: the same fold, pair by pair.
  std::vector<near_t> got = from_mem(nearest);
  std::vector<int> got_first = from_mem(first_city);
  int begin = 0, singles = 0;
  for(int s = 0; s < num_states; ++s) {
    int end = begin + per_state[s];
    for(int i = begin; i < end; ++i) {
      CHECK(got_first[i] == begin);
      near_t want = init;
      bool any = false;
      for(int j = begin; j < end; ++j) {
        if(j == i) continue;
        near_t y = one_city(squared_distance(pos[i], pos[j]), j);
        want = any ? closer_t()(want, y) : y;
        any = true;
      }
      singles += !any;
      for(int k = 0; k < closest; ++k) {
        if(got[i].city[k] != want.city[k] || got[i].score[k] != want.score[k]) {
          printf("city %d (state %d) entry %d: got (%.9g, %d) want (%.9g, %d)\n",
            i, s, k, got[i].score[k], got[i].city[k], want.score[k],
            want.city[k]);
          return 1;
        }
      }
    }
    begin = end;
  }
  CHECK(singles >= 1);      // a state with one city: an empty segment -> init
  printf("cities: %d cities in %d states, %d pairs: all passed\n", num_cities,
    num_states, num_pairs);
  return 0;
}
