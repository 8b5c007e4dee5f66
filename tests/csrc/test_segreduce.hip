// Caller written against the mgpu:: template API the way the reference's own
// segreduce test is (moderngpu tests/test_segreduce.cu): random sorted segment
// starts from std::mt19937, transform_segreduce of (index % 13) with
// plus_t<int> and init = -1, compared with the host loop.  Sizes are an
// argument so the harness can keep the run short.  Exit status is non-zero on
// any mismatch.
#include <moderngpu/kernel_segreduce.hxx>
#include <cstdio>
#include <cstdlib>

using namespace mgpu;

static int test_segreduce(int count, int num_segments, int seed,
  context_t& context) {
  std::mt19937 mt19937(seed);
  std::uniform_int_distribution<int> dist(0, count);
  std::vector<int> segments_host(num_segments);
  segments_host[0] = 0;
  for(int i = 1; i < num_segments; ++i)
    segments_host[i] = dist(mt19937);
  std::sort(segments_host.begin() + 1, segments_host.end());

  mem_t<int> segments = to_mem(segments_host, context);
  mem_t<int> results(num_segments, context);

  int init = -1;
  transform_segreduce([]MGPU_DEVICE(int index) {
    return index % 13;
  }, count, segments.data(), num_segments, results.data(),
    plus_t<int>(), init, context);

  std::vector<int> results_host = from_mem(results);
  for(int seg = 0; seg < num_segments; ++seg) {
    int begin = segments_host[seg];
    int end = (seg + 1 < num_segments) ? segments_host[seg + 1] : count;
    int x = init;
    for(int rank = 0; rank < end - begin; ++rank) {
      int y = (begin + rank) % 13;
      x = rank ? x + y : y;
    }
    if(x != results_host[seg]) {
      printf("seed %d: segment %d [%d, %d): device %d host %d\n", seed, seg,
        begin, end, results_host[seg], x);
      return 1;
    }
  }
  return 0;
}

int main(int argc, char** argv) {
  int count = argc > 1 ? atoi(argv[1]) : 10000000;
  int seg_size = argc > 2 ? atoi(argv[2]) : 100000;
  int num_tests = argc > 3 ? atoi(argv[3]) : 10;
  standard_context_t context(false);
  for(int test = 0; test < num_tests; ++test) {
    if(test_segreduce(count, div_up(count, seg_size), test, context)) {
      printf("FAILED\n");
      return 1;
    }
  }
  printf("segreduce: %d tests of %d items passed\n", num_tests, count);
  return 0;
}
