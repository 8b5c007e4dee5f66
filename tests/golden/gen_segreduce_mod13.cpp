// Writes tests/golden/segreduce_mod13.json.
//
// Inputs: segment starts produced the way the reference's own segreduce test
// produces them (moderngpu tests/test_segreduce.cu:16-22): segments[0] = 0,
// the rest drawn from std::uniform_int_distribution<int>(0, count) on a
// std::mt19937 seeded with the test number, then sorted.  The reference runs
// count = 1e8 with 100 segments; the cases here keep its seeds and shrink
// count so the fixture stays small, and add cases with many segments.
//
// Expected outputs: NOT the reference's loop but the closed form of
//   sum_{i in [b, e)} (i % 13)  =  S(e) - S(b),
//   S(n) = 78 * (n / 13) + r * (r - 1) / 2,  r = n % 13,
// with init (-1, as in the reference test) for empty segments.  A checker
// that folds init into non-empty segments, mishandles empties or is off by one
// at a boundary disagrees with these numbers.
//
// Build and run:  g++ -O2 -o /tmp/gen gen_segreduce_mod13.cpp && /tmp/gen > segreduce_mod13.json
#include <algorithm>
#include <cstdio>
#include <random>
#include <vector>

static long long prefix_mod13(long long n) {
  long long r = n % 13;
  return 78 * (n / 13) + r * (r - 1) / 2;
}

int main() {
  struct case_t { int count, num_segments, seed; };
  const case_t cases[] = {
    { 100000, 100, 0 }, { 100000, 100, 1 }, { 100000, 100, 2 },
    { 1000, 10, 3 }, { 5000, 300, 4 }, { 4096, 4096, 5 }, { 20000, 7, 6 },
    { 50, 64, 7 }, { 1, 3, 8 }, { 262144, 512, 9 }
  };
  const int init = -1;
  printf("{\"init\": %d, \"cases\": [\n", init);
  bool first_case = true;
  for(const case_t& c : cases) {
    std::mt19937 mt19937(c.seed);
    std::uniform_int_distribution<int> dist(0, c.count);
    std::vector<int> segments(c.num_segments);
    segments[0] = 0;
    for(int i = 1; i < c.num_segments; ++i) segments[i] = dist(mt19937);
    std::sort(segments.begin() + 1, segments.end());

    printf("%s{\"count\": %d, \"num_segments\": %d, \"seed\": %d,\n \"segments\": [",
      first_case ? "" : ",\n", c.count, c.num_segments, c.seed);
    for(int i = 0; i < c.num_segments; ++i)
      printf("%s%d", i ? "," : "", segments[i]);
    printf("],\n \"expected\": [");
    for(int i = 0; i < c.num_segments; ++i) {
      long long b = segments[i];
      long long e = (i + 1 < c.num_segments) ? segments[i + 1] : c.count;
      long long x = (e > b) ? prefix_mod13(e) - prefix_mod13(b) : init;
      printf("%s%lld", i ? "," : "", x);
    }
    printf("]}");
    first_case = false;
  }
  printf("\n]}\n");
  return 0;
}
