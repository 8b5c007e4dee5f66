// C++ callers of expt::lbs_workcreate.
//
// 1. A functor whose count per item is a pure function of the item: the
//    sizes upsweep returns, the segment starts downsweep returns and the
//    (dest_seg, index, seg, rank, cached) tuples the downsweep functor sees
//    are compared with a host loop, for several launch boxes and segment
//    shapes (including no segments, no items, and nothing created).
// 2. Breadth-first search on synthetic graphs, written the way the reference's
//    demos are (demo/bfs.cu: scan + transform_lbs over all vertices per level;
//    demo/bfs2.cu: a frontier that lbs_workcreate rebuilds per level), against
//    a host queue BFS: vertex levels must agree, and so must the number of
//    vertices and edges of every frontier.  (Which edge discovers a vertex is
//    a race, so the order of a frontier's segments is not compared.)
// Exit status 1 on the first mismatch.
#include <moderngpu/kernel_workcreate.hxx>
#include <cstdio>
#include <cstdlib>
#include <queue>

using namespace mgpu;

#define CHECK(cond) do { if(!(cond)) { \
  printf("%s:%d: CHECK(%s) failed\n", __FILE__, __LINE__, #cond); return 1; \
} } while(0)

// Work-items item `index` creates: none for most, up to 6 for the rest.
MGPU_HOST_DEVICE int created_by(int index, int keep_one_in) {
  unsigned h = (unsigned)index * 2654435761u;
  h ^= h >> 15;
  if(h % (unsigned)keep_one_in) return 0;
  return 1 + (int)((h >> 8) % 6);
}

static std::vector<int> random_starts(int count, int num_segments, int seed) {
  std::mt19937 generator(seed);
  std::uniform_int_distribution<int> draw(0, count);
  std::vector<int> starts(num_segments, 0);
  for(int s = 1; s < num_segments; ++s) starts[s] = draw(generator);
  if(num_segments) std::sort(starts.begin() + 1, starts.end());
  return starts;
}

template<typename launch_t>
static int check_engine(int count, int num_segments, int keep_one_in,
  int seed, context_t& context) {
  std::vector<int> starts = random_starts(count, num_segments, seed);
  mem_t<int> segments = to_mem(starts, context);

  auto engine = expt::lbs_workcreate<launch_t>(count, segments.data(),
    num_segments, context);

  // The cached tuple carries the segment's start: rank must be index - start.
  mem_t<int> bad = fill<int>(0, 1, context);
  int* bad_data = bad.data();
  auto sizes = engine.upsweep(
    [=]MGPU_DEVICE(int index, int seg, int rank, tuple<int> cached) {
      if(get<0>(cached) + rank != index || seg < 0 || seg >= num_segments)
        atomicAdd(bad_data, 1);
      return created_by(index, keep_one_in);
    }, make_tuple(segments.data()));

  // Host: creating items in item order and the starts of what they create.
  std::vector<int> want_index, want_start;
  int work = 0;
  for(int i = 0; i < count; ++i) {
    int n = created_by(i, keep_one_in);
    if(n > 0) { want_index.push_back(i); want_start.push_back(work); work += n; }
  }
  CHECK(sizes.count == work);
  CHECK(sizes.num_segments == (int)want_index.size());

  mem_t<int> from_index(sizes.num_segments, context);
  mem_t<int> from_seg(sizes.num_segments, context);
  mem_t<int> from_rank(sizes.num_segments, context);
  mem_t<int> next = engine.downsweep(
    [=]MGPU_DEVICE(int dest_seg, int index, int seg, int rank,
      tuple<int> cached, int* from_index, int* from_seg, int* from_rank) {
      if(get<0>(cached) + rank != index) atomicAdd(bad_data, 1);
      from_index[dest_seg] = index;
      from_seg[dest_seg] = seg;
      from_rank[dest_seg] = rank;
      return created_by(index, keep_one_in);
    }, make_tuple(segments.data()), from_index.data(), from_seg.data(),
    from_rank.data());
  CHECK((int)next.size() == sizes.num_segments);
  CHECK(0 == from_mem(bad)[0]);

  std::vector<int> got_start = from_mem(next), got_index = from_mem(from_index),
    got_seg = from_mem(from_seg), got_rank = from_mem(from_rank);
  int seg = -1;
  for(size_t k = 0; k < want_index.size(); ++k) {
    int i = want_index[k];
    while(seg + 1 < num_segments && starts[seg + 1] <= i) ++seg;
    if(got_start[k] != want_start[k] || got_index[k] != i ||
      got_seg[k] != seg || got_rank[k] != i - starts[seg]) {
      printf("count %d segments %d: new segment %d is (start %d, item %d, "
        "seg %d, rank %d), expected (%d, %d, %d, %d)\n", count, num_segments,
        (int)k, got_start[k], got_index[k], got_seg[k], got_rank[k],
        want_start[k], i, seg, i - starts[seg]);
      return 1;
    }
  }

  // The forms without a cached tuple.
  auto engine2 = expt::lbs_workcreate<launch_t>(count, segments.data(),
    num_segments, context);
  auto sizes2 = engine2.upsweep([=]MGPU_DEVICE(int index, int, int) {
    return created_by(index, keep_one_in);
  });
  CHECK(sizes2.count == work && sizes2.num_segments == sizes.num_segments);
  mem_t<int> next2 = engine2.downsweep(
    [=]MGPU_DEVICE(int dest_seg, int index, int, int, int* from_index) {
      from_index[dest_seg] = index + 1;
      return created_by(index, keep_one_in);
    }, from_index.data());
  CHECK(from_mem(next2) == want_start);
  got_index = from_mem(from_index);
  for(size_t k = 0; k < want_index.size(); ++k)
    CHECK(got_index[k] == want_index[k] + 1);
  return 0;
}

template<typename launch_t>
static int check_shapes(context_t& context) {
  CHECK(0 == check_engine<launch_t>(300007, 4000, 3, 1, context));
  CHECK(0 == check_engine<launch_t>(200000, 60000, 2, 2, context));   // short segments, empties
  CHECK(0 == check_engine<launch_t>(150001, 1, 1, 3, context));       // one segment, all create
  CHECK(0 == check_engine<launch_t>(100000, 7, 1000003, 4, context)); // item 0 alone creates
  CHECK(0 == check_engine<launch_t>(50, 3, 2, 5, context));
  CHECK(0 == check_engine<launch_t>(0, 5, 2, 6, context));            // no items
  CHECK(0 == check_engine<launch_t>(0, 0, 2, 7, context));
  return 0;
}

////////////////////////////////////////////////////////////////////////////////
// BFS.

struct graph_t {
  int num_vertices;
  std::vector<int> row_starts;    // num_vertices + 1
  std::vector<int> neighbors;
};

// Undirected: a ring lattice (so the graph is deep) plus random chords (so
// frontiers get wide) plus a few hubs (so segment lengths are skewed); the
// last tenth of the vertices is left isolated.
static graph_t make_graph(int num_vertices, int chords, int seed) {
  std::mt19937 generator(seed);
  int live = num_vertices - num_vertices / 10;
  std::vector<std::pair<int, int> > edges;
  for(int v = 0; v < live; ++v) edges.push_back({ v, (v + 1) % live });
  std::uniform_int_distribution<int> pick(0, live - 1);
  for(int e = 0; e < chords; ++e) edges.push_back({ pick(generator), pick(generator) });
  for(int hub = 0; hub < 4; ++hub)
    for(int e = 0; e < live / 50; ++e) edges.push_back({ hub * 7, pick(generator) });

  graph_t g;
  g.num_vertices = num_vertices;
  g.row_starts.assign(num_vertices + 1, 0);
  for(auto& e : edges) { ++g.row_starts[e.first + 1]; ++g.row_starts[e.second + 1]; }
  for(int v = 0; v < num_vertices; ++v) g.row_starts[v + 1] += g.row_starts[v];
  g.neighbors.resize(g.row_starts[num_vertices]);
  std::vector<int> at(g.row_starts.begin(), g.row_starts.end() - 1);
  for(auto& e : edges) {
    g.neighbors[at[e.first]++] = e.second;
    g.neighbors[at[e.second]++] = e.first;
  }
  return g;
}

struct frontier_size_t {
  int vertices, edges;
  bool operator==(const frontier_size_t& rhs) const {
    return vertices == rhs.vertices && edges == rhs.edges;
  }
};

static std::vector<int> host_bfs(const graph_t& g, int source,
  std::vector<frontier_size_t>& fronts) {
  std::vector<int> level(g.num_vertices, -1);
  std::vector<int> frontier { source };
  level[source] = 0;
  for(int depth = 0; !frontier.empty(); ++depth) {
    std::vector<int> next;
    int edges = 0;
    for(int v : frontier)
      for(int k = g.row_starts[v]; k < g.row_starts[v + 1]; ++k) {
        int w = g.neighbors[k];
        if(-1 == level[w]) {
          level[w] = depth + 1;
          next.push_back(w);
          edges += g.row_starts[w + 1] - g.row_starts[w];
        }
      }
    fronts.push_back({ (int)next.size(), edges });
    frontier.swap(next);
  }
  return level;
}

// Every level scans all vertices for the frontier's edge counts, then visits
// the frontier's edges with transform_lbs.
static int bfs_by_scan(const graph_t& g, int source, context_t& context,
  std::vector<int>& level_out, std::vector<int>& edges_per_level) {
  int num_vertices = g.num_vertices;
  mem_t<int> row_starts = to_mem(g.row_starts, context);
  mem_t<int> neighbors = to_mem(g.neighbors, context);
  std::vector<int> level_host(num_vertices, -1);
  level_host[source] = 0;
  mem_t<int> level = to_mem(level_host, context);
  mem_t<int> segments(num_vertices, context);
  mem_t<int> total(1, context);

  const int* rows = row_starts.data();
  const int* adjacent = neighbors.data();
  int* levels = level.data();
  for(int depth = 0; ; ++depth) {
    transform_scan<int>([=]MGPU_DEVICE(int v) {
      return levels[v] == depth ? rows[v + 1] - rows[v] : 0;
    }, num_vertices, segments.data(), plus_t<int>(), total.data(), context);
    int front = from_mem(total)[0];
    edges_per_level.push_back(front);
    if(!front) break;
    transform_lbs([=]MGPU_DEVICE(int, int, int rank, tuple<int> row) {
      atomicCAS(levels + adjacent[get<0>(row) + rank], -1, depth + 1);
    }, front, segments.data(), num_vertices, make_tuple(rows), context);
  }
  level_out = from_mem(level);
  return 0;
}

// The frontier is a workload of (segment starts, first edge of each segment);
// each level's engine builds the next one.
template<typename launch_t>
static int bfs_by_workcreate(const graph_t& g, int source, context_t& context,
  std::vector<int>& level_out, std::vector<frontier_size_t>& fronts) {
  mem_t<int> row_starts = to_mem(g.row_starts, context);
  mem_t<int> neighbors = to_mem(g.neighbors, context);
  std::vector<int> level_host(g.num_vertices, -1);
  level_host[source] = 0;
  mem_t<int> level = to_mem(level_host, context);

  const int* rows = row_starts.data();
  const int* adjacent = neighbors.data();
  int* levels = level.data();

  int count = g.row_starts[source + 1] - g.row_starts[source];
  int num_segments = 1;
  mem_t<int> segments = fill<int>(0, 1, context);
  mem_t<int> first_edge = fill<int>(g.row_starts[source], 1, context);

  for(int depth = 0; num_segments; ++depth) {
    auto engine = expt::lbs_workcreate<launch_t>(count, segments.data(),
      num_segments, context);
    auto sizes = engine.upsweep(
      [=]MGPU_DEVICE(int, int, int rank, tuple<int> first) {
        int w = adjacent[get<0>(first) + rank];
        return -1 == atomicCAS(levels + w, -1, depth + 1) ?
          rows[w + 1] - rows[w] : 0;
      }, make_tuple(first_edge.data()));

    // A vertex without edges is discovered but creates nothing, so the
    // frontier the workload describes leaves it out; count those separately.
    mem_t<int> next_first(sizes.num_segments, context);
    mem_t<int> next_segments = engine.downsweep(
      [=]MGPU_DEVICE(int dest_seg, int, int, int rank, tuple<int> first,
        int* next_first) {
        int w = adjacent[get<0>(first) + rank];
        next_first[dest_seg] = rows[w];
        return rows[w + 1] - rows[w];
      }, make_tuple(first_edge.data()), next_first.data());

    fronts.push_back({ sizes.num_segments, sizes.count });
    count = sizes.count;
    num_segments = sizes.num_segments;
    segments = std::move(next_segments);
    first_edge = std::move(next_first);
  }
  level_out = from_mem(level);
  return 0;
}

template<typename launch_t>
static int check_bfs(int num_vertices, int chords, int seed,
  context_t& context) {
  graph_t g = make_graph(num_vertices, chords, seed);
  int source = 23;
  std::vector<frontier_size_t> want_fronts;
  std::vector<int> want = host_bfs(g, source, want_fronts);

  std::vector<int> got_scan, edges_per_level;
  CHECK(0 == bfs_by_scan(g, source, context, got_scan, edges_per_level));
  CHECK(got_scan == want);
  // Level d's edge count is that of the frontier found at level d - 1.
  CHECK(edges_per_level.size() == want_fronts.size() + 1);
  for(size_t d = 0; d < want_fronts.size(); ++d)
    CHECK(edges_per_level[d + 1] == want_fronts[d].edges);

  std::vector<int> got_create;
  std::vector<frontier_size_t> got_fronts;
  CHECK(0 == bfs_by_workcreate<launch_t>(g, source, context, got_create,
    got_fronts));
  CHECK(got_create == want);
  CHECK(got_fronts.size() == want_fronts.size());
  for(size_t d = 0; d < want_fronts.size(); ++d) {
    // Every vertex of this graph that can be reached has edges.
    CHECK(got_fronts[d] == want_fronts[d]);
  }
  printf("bfs: %d vertices, %d edges, %d levels\n", g.num_vertices,
    (int)g.neighbors.size(), (int)want_fronts.size());
  return 0;
}

int main(int argc, char** argv) {
  int num_vertices = argc > 1 ? atoi(argv[1]) : 400000;
  standard_context_t context(false);

  typedef launch_box_t<arch_gfx950_cta<512, 12, 12> > box_wide_t;
  typedef launch_box_t<arch_20_cta<128, 11, 8>, arch_35_cta<128, 7, 5>,
    arch_52_cta<128, 11, 8> > box_cuda_t;           // the reference's default
  CHECK(0 == check_shapes<empty_t>(context));
  CHECK(0 == check_shapes<box_wide_t>(context));
  CHECK(0 == check_shapes<box_cuda_t>(context));
  CHECK(0 == (check_shapes<launch_params_t<64, 4> >(context)));

  CHECK(0 == check_bfs<empty_t>(num_vertices, num_vertices, 31, context));
  CHECK(0 == check_bfs<box_cuda_t>(num_vertices / 4, num_vertices / 16, 32,
    context));
  printf("workcreate: all passed\n");
  return 0;
}
