// Callers of mgpu::scan / transform_scan / reduce / transform_reduce written
// the way the reference's own tests use them (moderngpu tests/test_scan.cu:
// exclusive scan of a constant iterator into device memory with the total in
// host memory; tests/test_reduce.cu: reduce and transform_reduce of an array
// of ones with an explicit launch box over a sweep of sizes), plus a
// non-commutative operator and a user value type.  Exit status is non-zero on
// any mismatch.
#include <moderngpu/kernel_scan.hxx>
#include <moderngpu/kernel_reduce.hxx>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <numeric>

using namespace mgpu;

#define CHECK(cond, ...) do { if(!(cond)) { printf("FAILED %s:%d: ", __FILE__, __LINE__); printf(__VA_ARGS__); printf("\n"); return 1; } } while(0)

// Keeps the left operand's tag and the right operand's count sum: associative,
// not commutative.
struct tagged_t { int tag; int sum; };
struct keep_left_t {
  MGPU_HOST_DEVICE tagged_t operator()(tagged_t a, tagged_t b) const {
    return tagged_t { a.tag, a.sum + b.sum };
  }
};

static int test_scan_constant(context_t& context) {
  typedef double type_t;
  int count = 50000;
  mem_t<type_t> output(count, context);
  mem_t<type_t> total(1, context, memory_space_host);
  scan<scan_type_exc>(constant_iterator_t<type_t>(1.01), count, output.data(),
    plus_t<type_t>(), total.data(), context);
  context.synchronize();
  std::vector<type_t> y = from_mem(output);
  for(int i = 0; i < count; ++i) {
    double want = 1.01 * i;
    CHECK(std::fabs(y[i] - want) <= 1e-12 * (want + 1), "scan[%d] = %.17g want %.17g", i, y[i], want);
  }
  double want = 1.01 * count;
  CHECK(std::fabs(total.data()[0] - want) <= 1e-12 * want, "total %.17g", total.data()[0]);
  return 0;
}

static int test_scan_sizes(context_t& context) {
  for(int count : { 1, 100, 16384, 16385, 70001, 3000017 }) {
    // transform_scan of f(i) = i % 7, inclusive, with an event.
    mem_t<int> output(count, context);
    mem_t<int> total(1, context);
    hipEvent_t event; if(hipEventCreate(&event) != hipSuccess) return 1;
    transform_scan_event<int, scan_type_inc>([]MGPU_DEVICE(int i) { return i % 7; },
      count, output.data(), plus_t<int>(), total.data(), context, event);
    if(hipEventSynchronize(event) != hipSuccess) return 1;
    int total_host = from_mem(total)[0];
    context.synchronize();
    (void)hipEventDestroy(event);
    std::vector<int> y = from_mem(output);
    int x = 0;
    for(int i = 0; i < count; ++i) {
      x += i % 7;
      CHECK(y[i] == x, "count %d: scan[%d] = %d want %d", count, i, y[i], x);
    }
    CHECK(total_host == x, "count %d: total %d want %d", count, total_host, x);

    // user type, non-commutative op, exclusive.
    std::vector<tagged_t> host(count);
    for(int i = 0; i < count; ++i) host[i] = tagged_t { i, 1 };
    mem_t<tagged_t> in = to_mem(host, context);
    mem_t<tagged_t> out(count, context), red(1, context);
    scan<scan_type_exc>(in.data(), count, out.data(), keep_left_t(), red.data(), context);
    std::vector<tagged_t> z = from_mem(out);
    CHECK(z[0].tag == 0 && z[0].sum == 0, "count %d: exclusive[0] is not type_t()", count);
    for(int i = 1; i < count; ++i)
      CHECK(z[i].tag == 0 && z[i].sum == i, "count %d: tagged scan[%d] = (%d, %d)", count, i, z[i].tag, z[i].sum);
    tagged_t r = from_mem(red)[0];
    CHECK(r.tag == 0 && r.sum == count, "count %d: tagged total (%d, %d)", count, r.tag, r.sum);
  }
  return 0;
}

// Tiny tiles make the number of partials exceed what one spine CTA takes, so
// the partials get an upsweep/spine/downsweep of their own.
static int test_scan_two_levels(context_t& context) {
  typedef launch_params_t<64, 4> launch_t;
  int count = 256 * 262144 + 12345;
  mem_t<int> output(count, context);
  mem_t<int> total(1, context);
  transform_scan<int, scan_type_exc, launch_t>(
    []MGPU_DEVICE(int i) { return (i & 3) + 1; }, count, output.data(),
    plus_t<int>(), total.data(), context);
  std::vector<int> y = from_mem(output);
  int x = 0;
  for(int i = 0; i < count; ++i) {
    CHECK(y[i] == x, "two-level scan[%d] = %d want %d", i, y[i], x);
    x += (i & 3) + 1;
  }
  CHECK(from_mem(total)[0] == x, "two-level total");

  // The same with a value type that takes the three-launch path, enough
  // tiles that the partials need a second level.
  int count2 = 256 * 16500 + 77;
  std::vector<tagged_t> host(count2);
  for(int i = 0; i < count2; ++i) host[i] = tagged_t { i, 1 };
  mem_t<tagged_t> in = to_mem(host, context);
  mem_t<tagged_t> out(count2, context), red(1, context);
  scan<scan_type_inc, launch_t>(in.data(), count2, out.data(), keep_left_t(),
    red.data(), context);
  std::vector<tagged_t> z = from_mem(out);
  for(int i = 0; i < count2; ++i)
    CHECK(z[i].tag == 0 && z[i].sum == i + 1, "two-level tagged scan[%d] = (%d, %d)", i, z[i].tag, z[i].sum);
  tagged_t r = from_mem(red)[0];
  CHECK(r.tag == 0 && r.sum == count2, "two-level tagged total (%d, %d)", r.tag, r.sum);
  return 0;
}

static int test_reduce_sweep(context_t& context) {
  typedef launch_params_t<64 * 3, 11> launch_t;
  for(int count = 1000; count < 23456789; count += count / 3) {
    mem_t<int> input = fill(1, count, context);
    const int* input_data = input.data();
    mem_t<int> reduction(1, context);
    reduce<launch_t>(input_data, count, reduction.data(), plus_t<int>(), context);
    int result1 = from_mem(reduction)[0];
    auto f = [=]MGPU_DEVICE(int index) { return input_data[index]; };
    transform_reduce(f, count, reduction.data(), plus_t<int>(), context);
    int result2 = from_mem(reduction)[0];
    CHECK(result1 == count && result2 == count, "count %d: reduce %d transform_reduce %d", count, result1, result2);

    std::vector<tagged_t> host(count);
    for(int i = 0; i < count; ++i) host[i] = tagged_t { i + 5, 2 };
    mem_t<tagged_t> in = to_mem(host, context);
    mem_t<tagged_t> red(1, context);
    reduce(in.data(), count, red.data(), keep_left_t(), context);
    tagged_t r = from_mem(red)[0];
    CHECK(r.tag == 5 && r.sum == 2 * count, "count %d: tagged reduce (%d, %d)", count, r.tag, r.sum);
  }
  return 0;
}

// A 32-byte value type with a non-commutative operator (first tag wins, the
// four sums add): scan and reduce with the default launch boxes, at a size of
// one CTA, of a few tiles and of thousands of tiles.
struct wide_t { int64_t tag; int64_t sum[3]; };
struct wide_left_t {
  MGPU_HOST_DEVICE wide_t operator()(wide_t a, wide_t b) const {
    return wide_t { a.tag, { a.sum[0] + b.sum[0], a.sum[1] + b.sum[1],
      a.sum[2] + b.sum[2] } };
  }
};
static int test_wide_type(context_t& context) {
  static_assert(32 == sizeof(wide_t), "");
  for(int count : { 1, 999, 16384, 16385, 300000, 5000011 }) {
    std::vector<wide_t> host(count);
    for(int i = 0; i < count; ++i)
      host[i] = wide_t { i + 3, { 1, i, -2 } };
    mem_t<wide_t> in = to_mem(host, context);
    mem_t<wide_t> out(count, context), red(1, context);
    scan<scan_type_inc>(in.data(), count, out.data(), wide_left_t(),
      red.data(), context);
    std::vector<wide_t> z = from_mem(out);
    for(int i = 0; i < count; ++i) {
      int64_t tri = (int64_t)i * (i + 1) / 2;
      CHECK(z[i].tag == 3 && z[i].sum[0] == i + 1 && z[i].sum[1] == tri &&
        z[i].sum[2] == -2 * (int64_t)(i + 1), "wide scan, count %d, at %d", count, i);
    }
    wide_t r = from_mem(red)[0];
    CHECK(r.tag == 3 && r.sum[0] == count, "wide scan total, count %d", count);
    reduce(in.data(), count, red.data(), wide_left_t(), context);
    r = from_mem(red)[0];
    CHECK(r.tag == 3 && r.sum[0] == count &&
      r.sum[1] == (int64_t)count * (count - 1) / 2, "wide reduce, count %d", count);
  }
  return 0;
}

int main() {
  standard_context_t context(false);
  if(test_scan_constant(context) || test_scan_sizes(context) ||
    test_scan_two_levels(context) || test_reduce_sweep(context) ||
    test_wide_type(context))
    return 1;
  printf("scan/reduce: all passed\n");
  return 0;
}
