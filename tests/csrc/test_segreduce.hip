// A C++ caller of transform_segreduce shaped like the reference's own test
// (moderngpu tests/test_segreduce.cu): segment starts drawn uniformly from
// [0, count] and sorted (so empty segments and repeated starts occur), the
// value of item i is i % 13, the operator is plus_t<int> and init is -1.
// The expected sums come from a prefix table of i % 13, which has a closed
// form, instead of a loop per segment.
// usage: test_segreduce [count [items per segment [number of seeds]]]
// Exit status 1 on the first mismatch.
#include <moderngpu/kernel_segreduce.hxx>
#include <cstdio>
#include <cstdlib>

// sum of (i % 13) for i in [0, n)
static long long prefix_mod13(long long n) {
  long long full = n / 13, rest = n % 13;
  return full * 78 + rest * (rest - 1) / 2;
}

static std::vector<int> random_starts(int count, int num_segments, int seed) {
  std::mt19937 generator(seed);
  std::uniform_int_distribution<int> draw(0, count);
  std::vector<int> starts(num_segments, 0);
  for(int s = 1; s < num_segments; ++s) starts[s] = draw(generator);
  std::sort(starts.begin() + 1, starts.end());
  return starts;
}

static bool run_seed(int count, int num_segments, int seed,
  mgpu::context_t& context) {
  const int init = -1;
  std::vector<int> starts = random_starts(count, num_segments, seed);
  mgpu::mem_t<int> segments = mgpu::to_mem(starts, context);
  mgpu::mem_t<int> sums(num_segments, context);

  auto value_of = []MGPU_DEVICE(int index) { return index % 13; };
  mgpu::transform_segreduce(value_of, count, segments.data(), num_segments,
    sums.data(), mgpu::plus_t<int>(), init, context);

  std::vector<int> got = mgpu::from_mem(sums);
  for(int s = 0; s < num_segments; ++s) {
    int first = starts[s];
    int last = s + 1 < num_segments ? starts[s + 1] : count;
    int want = first == last ? init :
      (int)(prefix_mod13(last) - prefix_mod13(first));
    if(got[s] != want) {
      printf("seed %d, segment %d = [%d, %d): got %d, want %d\n", seed, s,
        first, last, got[s], want);
      return false;
    }
  }
  return true;
}

int main(int argc, char** argv) {
  int count = argc > 1 ? atoi(argv[1]) : 10000000;
  int per_segment = argc > 2 ? atoi(argv[2]) : 100000;
  int num_seeds = argc > 3 ? atoi(argv[3]) : 10;

  mgpu::standard_context_t context(false);
  int num_segments = mgpu::div_up(count, per_segment);
  for(int seed = 0; seed < num_seeds; ++seed)
    if(!run_seed(count, num_segments, seed, context)) {
      printf("FAILED\n");
      return 1;
    }
  printf("segreduce: %d tests of %d items passed\n", num_seeds, count);
  return 0;
}
