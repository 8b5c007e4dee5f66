// A C++ caller of load_balance_search with the reference's own test shape
// (moderngpu tests/test_load_balance.cu: 200030 items, a segment start every
// 100 items) plus a few more (count, spacing) pairs around tile edges.
// Expected segment of item i is floor(i / spacing), checked here with a
// running counter rather than a division.  Exit status 1 on the first
// mismatch.
#include <moderngpu/kernel_load_balance.hxx>
#include <cstdio>

static bool check_even_segments(int count, int spacing,
  mgpu::context_t& context) {
  int num_segments = mgpu::div_up(count, spacing);
  std::vector<int> starts;
  for(int s = 0; s < num_segments; ++s) starts.push_back(s * spacing);

  mgpu::mem_t<int> segments = mgpu::to_mem(starts, context);
  mgpu::mem_t<int> found(count, context);
  mgpu::load_balance_search(count, segments.data(), num_segments,
    found.data(), context);

  std::vector<int> host = mgpu::from_mem(found);
  int expected = 0, left = spacing;
  for(int i = 0; i < count; ++i, --left) {
    if(!left) { ++expected; left = spacing; }
    if(host[i] != expected) {
      printf("count %d spacing %d: item %d in segment %d, expected %d\n",
        count, spacing, i, host[i], expected);
      return false;
    }
  }
  return true;
}

int main() {
  mgpu::standard_context_t context(false);
  const int cases[][2] = {
    { 200030, 100 }, { 200030, 1 }, { 6144, 6144 }, { 6145, 7 },
    { 1000003, 4099 }
  };
  int items = 0;
  for(const int (&c)[2] : cases) {
    if(!check_even_segments(c[0], c[1], context)) return 1;
    items += c[0];
  }
  printf("load_balance_search: %d items passed\n", items);
  return 0;
}
