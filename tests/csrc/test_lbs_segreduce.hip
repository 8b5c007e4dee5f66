// Callers of mgpu::lbs_segreduce: the functor of the reference's own test
// (moderngpu tests/test_segreduce.cu:11-13 and :29-30, f = seg + rank, plus,
// init = -1) on that test's segment generator, then cached iterators, extra
// arguments, a user value type with a non-commutative operator and an
// explicit launch box, the way demo/cities.cu:186-222 calls it.  Exit status
// is non-zero on any mismatch.
#include <moderngpu/kernel_segreduce.hxx>
#include <cstdio>
#include <cstdlib>

using namespace mgpu;

#define CHECK(cond, ...) do { if(!(cond)) { printf("FAILED %s:%d: ", __FILE__, __LINE__); printf(__VA_ARGS__); printf("\n"); return 1; } } while(0)

static std::vector<int> make_segments(int count, int num_segments, int seed) {
  std::mt19937 mt19937(seed);
  std::uniform_int_distribution<int> dist(0, count);
  std::vector<int> segments_host(num_segments);
  segments_host[0] = 0;
  for(int i = 1; i < num_segments; ++i) segments_host[i] = dist(mt19937);
  std::sort(segments_host.begin() + 1, segments_host.end());
  return segments_host;
}

static int test_seg_plus_rank(int count, int num_segments, int seed,
  context_t& context) {
  auto f = [=]MGPU_DEVICE(int index, int seg, int rank) {
    return seg + rank;
  };
  std::vector<int> segments_host = make_segments(count, num_segments, seed);
  mem_t<int> segments = to_mem(segments_host, context);
  mem_t<int> results(num_segments, context);
  int init = -1;
  lbs_segreduce(f, count, segments.data(), num_segments, results.data(),
    plus_t<int>(), init, context);
  std::vector<int> results_host = from_mem(results);
  for(int seg = 0; seg < num_segments; ++seg) {
    int begin = segments_host[seg];
    int end = (seg + 1 < num_segments) ? segments_host[seg + 1] : count;
    int x = init;
    for(int rank = 0; rank < end - begin; ++rank)
      x = rank ? (int)((unsigned)x + (unsigned)(seg + rank)) : seg + rank;   // wraps like the device sum
    CHECK(x == results_host[seg], "seed %d segment %d [%d, %d): device %d host %d",
      seed, seg, begin, end, results_host[seg], x);
  }
  return 0;
}

// Keeps the smallest score, and of equal scores the earlier one.
struct best_t { float score; int index; };
struct pick_best_t {
  MGPU_HOST_DEVICE best_t operator()(best_t a, best_t b) const {
    return (b.score < a.score) ? b : a;
  }
};

static int test_cached_and_args(int count, int num_segments, int seed,
  context_t& context) {
  std::vector<int> segments_host = make_segments(count, num_segments, seed);
  std::vector<int> offset_host(num_segments);
  std::vector<float> scale_host(num_segments);
  for(int s = 0; s < num_segments; ++s) {
    offset_host[s] = (s * 37) % 1000;
    scale_host[s] = 1.0f + (s % 5);
  }
  std::vector<float> table_host(1000 + count);
  for(size_t i = 0; i < table_host.size(); ++i)
    table_host[i] = (float)((i * 2654435761u) % 10007) / 16.0f;

  mem_t<int> segments = to_mem(segments_host, context);
  mem_t<int> offset = to_mem(offset_host, context);
  mem_t<float> scale = to_mem(scale_host, context);
  mem_t<float> table = to_mem(table_host, context);
  mem_t<best_t> results(num_segments, context);

  best_t init = { -1.0f, -1 };
  // score = scale[seg] * table[offset[seg] + rank] + bias; offset and scale
  // are cached per segment, the table pointer and the bias are passed along.
  auto f = []MGPU_DEVICE(int index, int seg, int rank, tuple<int, float> desc,
    const float* table, float bias) {
    float score = get<1>(desc) * table[get<0>(desc) + rank] + bias;
    return best_t { score, index };
  };
  typedef launch_params_t<128, 4> launch_t;
  lbs_segreduce<launch_t>(f, count, segments.data(), num_segments,
    make_tuple(offset.data(), scale.data()), results.data(), pick_best_t(),
    init, context, (const float*)table.data(), 0.5f);

  std::vector<best_t> results_host = from_mem(results);
  for(int seg = 0; seg < num_segments; ++seg) {
    int begin = segments_host[seg];
    int end = (seg + 1 < num_segments) ? segments_host[seg + 1] : count;
    best_t x = init;
    for(int rank = 0; rank < end - begin; ++rank) {
      best_t y = { scale_host[seg] * table_host[offset_host[seg] + rank] + 0.5f,
        begin + rank };
      x = rank ? pick_best_t()(x, y) : y;
    }
    CHECK(x.score == results_host[seg].score && x.index == results_host[seg].index,
      "seed %d segment %d [%d, %d): device (%g, %d) host (%g, %d)", seed, seg,
      begin, end, results_host[seg].score, results_host[seg].index, x.score, x.index);
  }
  return 0;
}

int main(int argc, char** argv) {
  int count = argc > 1 ? atoi(argv[1]) : 10000000;
  int seg_size = argc > 2 ? atoi(argv[2]) : 100000;
  standard_context_t context(false);
  for(int test = 0; test < 4; ++test)
    if(test_seg_plus_rank(count, div_up(count, seg_size), test, context)) return 1;
  for(int test = 0; test < 3; ++test) {
    if(test_seg_plus_rank(count / 7, div_up(count, 50), test, context)) return 1;  // short, many empty
    if(test_cached_and_args(count / 3, div_up(count / 3, 300), test, context)) return 1;
    if(test_cached_and_args(50000, 90000, test, context)) return 1;       // mostly empty
  }
  printf("lbs_segreduce: all passed\n");
  return 0;
}
