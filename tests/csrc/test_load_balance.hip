// Caller shaped like the reference's load-balancing-search test (moderngpu
// tests/test_load_balance.cu): segment starts every `spacing` items,
// load_balance_search, expect lbs[i] == i / spacing.  Non-zero exit on error.
#include <moderngpu/kernel_load_balance.hxx>
#include <cstdio>

using namespace mgpu;

int main() {
  standard_context_t context(false);

  int count = 200030;
  int spacing = 100;
  int num_segments = div_up(count, spacing);
  std::vector<int> segments_host(num_segments);
  for(int i = 0; i < num_segments; ++i) segments_host[i] = i * spacing;
  mem_t<int> segments = to_mem(segments_host, context);

  mem_t<int> lbs(count, context);
  load_balance_search(count, segments.data(), num_segments, lbs.data(),
    context);

  std::vector<int> lbs_host = from_mem(lbs);
  for(size_t i = 0; i < lbs_host.size(); ++i) {
    if(lbs_host[i] != (int)i / spacing) {
      printf("ERROR AT %d: %d\n", (int)i, lbs_host[i]);
      return 1;
    }
  }
  printf("load_balance_search: %d items passed\n", count);
  return 0;
}
