// Host-side graph ingest and seeded synthetic graphs (see nd_graph.hpp).
#include "nd_graph.hpp"

#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <functional>
#include <thread>
#include <unordered_map>
#include <vector>

namespace nd {
namespace {

int worker_count() {
  unsigned hw = std::thread::hardware_concurrency();
  if (hw == 0) hw = 4;
  if (const char* env = getenv("ND_HOST_THREADS")) {
    int v = atoi(env);
    if (v > 0) return v;
  }
  return (int)std::min(hw, 16u);
}

// Runs fn(begin, end) over [0, n) split into contiguous blocks handed out dynamically.
void parallel_blocks(size_t n, size_t block, const std::function<void(size_t, size_t)>& fn) {
  if (n == 0) return;
  const int workers = worker_count();
  if (workers <= 1 || n <= block) {
    fn(0, n);
    return;
  }
  std::atomic<size_t> next(0);
  std::vector<std::thread> pool;
  for (int t = 0; t < workers; ++t) {
    pool.emplace_back([&]() {
      for (;;) {
        const size_t b = next.fetch_add(block);
        if (b >= n) return;
        fn(b, std::min(n, b + block));
      }
    });
  }
  for (auto& th : pool) th.join();
}

uint32_t float_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, sizeof(u));
  return u;
}

// Ordering key of an edge inside an adjacency: (destination, weight) ascending, as
// std::sort of std::pair<int, float> gives it.  Monotone map of float to uint32.
uint64_t edge_sort_key(int32_t dst, float w) {
  uint32_t b = float_bits(w);
  b = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
  return ((uint64_t)(uint32_t)dst << 32) | b;
}

void finish_csr(CSR& out) {
  const size_t V = out.row_ptr.size() - 1;
  out.max_weight.assign(V, 0.0f);
  parallel_blocks(V, 4096, [&](size_t b, size_t e) {
    std::vector<uint64_t> keys;
    std::vector<float> ws;
    for (size_t v = b; v < e; ++v) {
      const size_t lo = (size_t)out.row_ptr[v], hi = (size_t)out.row_ptr[v + 1];
      float mw = 0.0f;
      for (size_t i = lo; i < hi; ++i) mw = std::max(mw, out.weight[i]);
      out.max_weight[v] = mw;
      if (hi - lo > 1) {
        // sort (dst, weight) pairs; weights travel with their key
        keys.resize(hi - lo);
        for (size_t i = lo; i < hi; ++i) keys[i - lo] = edge_sort_key(out.col[i], out.weight[i]);
        bool sorted = true;
        for (size_t i = 1; i < keys.size() && sorted; ++i) sorted = keys[i - 1] <= keys[i];
        if (!sorted) {
          std::vector<uint32_t> order(hi - lo);
          for (size_t i = 0; i < order.size(); ++i) order[i] = (uint32_t)i;
          std::sort(order.begin(), order.end(), [&](uint32_t x, uint32_t y) { return keys[x] < keys[y]; });
          ws.resize(hi - lo);
          std::vector<int32_t> cs(hi - lo);
          for (size_t i = 0; i < order.size(); ++i) {
            cs[i] = out.col[lo + order[i]];
            ws[i] = out.weight[lo + order[i]];
          }
          for (size_t i = 0; i < order.size(); ++i) {
            out.col[lo + i] = cs[i];
            out.weight[lo + i] = ws[i];
          }
        }
      }
    }
  });
}

}  // namespace

int csr_from_edges(CSR& out, int32_t n_vertices, size_t n, const int32_t* src, const int32_t* dst, const float* w,
                   std::string* error) {
  int64_t max_id = -1;
  for (size_t i = 0; i < n; ++i) {
    if (src[i] < 0 || dst[i] < 0) {
      if (error) *error = "negative vertex id in edge list";
      return -1;
    }
    max_id = std::max<int64_t>(max_id, std::max(src[i], dst[i]));
  }
  int64_t V = n_vertices > 0 ? n_vertices : max_id + 1;
  if (max_id >= V) {
    if (error) *error = "vertex id exceeds the vertex count";
    return -1;
  }
  if (V <= 0 || V >= INT32_MAX || n >= (size_t)INT32_MAX) {
    if (error) *error = "graph is empty or too large for int32 ids";
    return -1;
  }
  out.row_ptr.assign((size_t)V + 1, 0);
  for (size_t i = 0; i < n; ++i) out.row_ptr[(size_t)src[i] + 1]++;
  for (size_t v = 0; v < (size_t)V; ++v) out.row_ptr[v + 1] += out.row_ptr[v];
  out.col.resize(n);
  out.weight.resize(n);
  std::vector<EdgePos_t> cursor(out.row_ptr.begin(), out.row_ptr.end() - 1);
  for (size_t i = 0; i < n; ++i) {
    const size_t p = (size_t)cursor[src[i]]++;
    out.col[p] = dst[i];
    out.weight[p] = w ? w[i] : 1.0f;
  }
  finish_csr(out);
  return 0;
}

int csr_from_arrays(CSR& out, int32_t n_vertices, int64_t n_edges, const int32_t* row_ptr, const int32_t* col,
                    const float* weight, std::string* error) {
  if (n_vertices <= 0 || n_edges < 0 || n_edges >= INT32_MAX) {
    if (error) *error = "bad graph size";
    return -1;
  }
  if (row_ptr[0] != 0 || row_ptr[n_vertices] != n_edges) {
    if (error) *error = "row_ptr does not span [0, n_edges]";
    return -1;
  }
  for (int32_t v = 0; v < n_vertices; ++v)
    if (row_ptr[v + 1] < row_ptr[v]) {
      if (error) *error = "row_ptr is not monotone";
      return -1;
    }
  for (int64_t i = 0; i < n_edges; ++i)
    if (col[i] < 0 || col[i] >= n_vertices) {
      if (error) *error = "column index out of range";
      return -1;
    }
  out.row_ptr.assign(row_ptr, row_ptr + n_vertices + 1);
  out.col.assign(col, col + n_edges);
  if (weight) out.weight.assign(weight, weight + n_edges);
  else out.weight.assign((size_t)n_edges, 1.0f);
  finish_csr(out);  // sorts any adjacency that is not sorted yet
  return 0;
}

int load_graph_file(CSR& out, const char* path, const char* graph_type, const char* graph_format,
                    std::string* error) {
  auto fail = [&](const std::string& msg) {
    if (error) *error = msg;
    return -1;
  };
  if (!path || !graph_type || !graph_format) return fail("null argument");
  const bool edge_list = strcmp(graph_type, "edge-list") == 0;
  const bool adj_list = strcmp(graph_type, "adj-list") == 0;
  const bool binary = strcmp(graph_format, "binary") == 0;
  const bool text = strcmp(graph_format, "text") == 0;
  if (!edge_list && !adj_list) return fail(std::string("Incorrect graph file type '") + graph_type + "'");
  if ((adj_list && !text) || (edge_list && !binary && !text))
    return fail(std::string("graph_format '") + graph_format + "' not supported for graph_type '" + graph_type + "'");

  FILE* fp = fopen(path, binary ? "rb" : "r");
  if (!fp) return fail(std::string("File '") + path + "' not found");
  std::vector<int32_t> src, dst;
  std::vector<float> w;
  if (binary) {
    fseek(fp, 0, SEEK_END);
    const long size = ftell(fp);
    fseek(fp, 0, SEEK_SET);
    const size_t n = (size_t)size / 12;
    src.resize(n); dst.resize(n); w.resize(n);
    std::vector<unsigned char> buf(1 << 20);
    size_t i = 0;
    const size_t per_read = buf.size() / 12;
    while (i < n) {
      const size_t want = std::min(per_read, n - i);
      if (fread(buf.data(), 12, want, fp) != want) { fclose(fp); return fail("short read"); }
      for (size_t k = 0; k < want; ++k, ++i) {
        memcpy(&src[i], &buf[12 * k], 4);
        memcpy(&dst[i], &buf[12 * k + 4], 4);
        memcpy(&w[i], &buf[12 * k + 8], 4);
      }
    }
  } else if (edge_list) {
    // "src dst [weight]" per line; '#' starts a comment line
    char line[4096];
    while (fgets(line, sizeof(line), fp)) {
      if (line[0] == '#' || line[0] == '%') continue;
      long a, b;
      float weight = 1.0f;
      const int got = sscanf(line, "%ld %ld %f", &a, &b, &weight);
      if (got < 2) continue;
      src.push_back((int32_t)a); dst.push_back((int32_t)b); w.push_back(got == 3 ? weight : 1.0f);
    }
  } else {
    // "v n1 w1 n2 w2 ..." per line (src/graph.hpp:256-326); vertices are renumbered in
    // order of appearance
    std::vector<char> line(1 << 20);
    std::unordered_map<long, int32_t> rename;
    std::vector<long> raw_src, raw_dst;
    while (fgets(line.data(), (int)line.size(), fp)) {
      char* cur = line.data();
      int used = 0;
      long id;
      if (sscanf(cur, "%ld%n", &id, &used) != 1) continue;
      cur += used;
      rename.emplace(id, (int32_t)rename.size());
      long nb;
      float weight;
      while (sscanf(cur, "%ld %f%n", &nb, &weight, &used) == 2) {
        raw_src.push_back(id); raw_dst.push_back(nb); w.push_back(weight);
        cur += used;
      }
    }
    src.resize(raw_src.size()); dst.resize(raw_src.size());
    for (size_t i = 0; i < raw_src.size(); ++i) {
      auto it = rename.find(raw_dst[i]);
      if (it == rename.end()) { fclose(fp); return fail("adjacency list names a vertex that has no line"); }
      src[i] = rename[raw_src[i]];
      dst[i] = it->second;
    }
    fclose(fp);
    return csr_from_edges(out, (int32_t)rename.size(), src.size(), src.data(), dst.data(), w.data(), error);
  }
  fclose(fp);
  return csr_from_edges(out, 0, src.size(), src.data(), dst.data(), w.data(), error);
}

namespace {
constexpr uint32_t kStreamRmat = 0x524D4154u;     // "RMAT"
constexpr uint32_t kStreamEndpoint = 0x434C5545u; // "CLUE"
constexpr uint32_t kStreamWeight = 0x57454947u;   // "WEIG"

float edge_weight_for(uint64_t seed, uint64_t edge) {
  return 1.0f + 4.0f * uniform_at(seed, edge, kStreamWeight, 0);  // [1, 5)
}
}  // namespace

int generate_rmat(CSR& out, int scale, int edge_factor, double a, double b, double c, uint64_t seed,
                  bool symmetrise, std::string* error) {
  if (scale < 1 || scale > 30 || edge_factor < 1) {
    if (error) *error = "bad R-MAT size";
    return -1;
  }
  const size_t V = (size_t)1 << scale;
  const size_t generated = V * (size_t)edge_factor;
  const size_t total = symmetrise ? 2 * generated : generated;
  if (total >= (size_t)INT32_MAX) {
    if (error) *error = "R-MAT edge count does not fit int32 edge positions";
    return -1;
  }
  std::vector<int32_t> src(total), dst(total);
  std::vector<float> w(total);
  const float ta = (float)a, tab = (float)(a + b), tabc = (float)(a + b + c);
  parallel_blocks(generated, 1 << 16, [&](size_t lo, size_t hi) {
    for (size_t e = lo; e < hi; ++e) {
      uint32_t s = 0, d = 0;
      RandState rng;
      rng.reset(seed, e, kStreamRmat);
      for (int level = 0; level < scale; ++level) {
        const float u = rng.next_uniform();
        const uint32_t quadrant = u < ta ? 0u : (u < tab ? 1u : (u < tabc ? 2u : 3u));
        s = (s << 1) | (quadrant >> 1);
        d = (d << 1) | (quadrant & 1u);
      }
      const float weight = edge_weight_for(seed, e);
      src[e] = (int32_t)s; dst[e] = (int32_t)d; w[e] = weight;
      if (symmetrise) {
        src[generated + e] = (int32_t)d; dst[generated + e] = (int32_t)s; w[generated + e] = weight;
      }
    }
  });
  return csr_from_edges(out, (int32_t)V, total, src.data(), dst.data(), w.data(), error);
}

int generate_chung_lu(CSR& out, int32_t n_vertices, int64_t n_edges, double exponent, uint64_t seed,
                      std::string* error) {
  if (n_vertices < 1 || n_edges < 0 || n_edges >= INT32_MAX || exponent <= 1.0) {
    if (error) *error = "bad Chung-Lu parameters";
    return -1;
  }
  const size_t V = (size_t)n_vertices;
  std::vector<double> cdf(V);
  const double power = -1.0 / (exponent - 1.0);
  double acc = 0.0;
  for (size_t i = 0; i < V; ++i) {
    acc += std::pow((double)(i + 1), power);
    cdf[i] = acc;
  }
  const double total_weight = acc;
  std::vector<int32_t> src((size_t)n_edges), dst((size_t)n_edges);
  std::vector<float> w((size_t)n_edges);
  auto pick = [&](double u01) {
    const double target = u01 * total_weight;
    size_t idx = (size_t)(std::upper_bound(cdf.begin(), cdf.end(), target) - cdf.begin());
    return (int32_t)std::min(idx, V - 1);
  };
  parallel_blocks((size_t)n_edges, 1 << 16, [&](size_t lo, size_t hi) {
    for (size_t e = lo; e < hi; ++e) {
      const PhiloxBlock blk = philox4x32_10((uint32_t)e, (uint32_t)(e >> 32), kStreamEndpoint, 0, (uint32_t)seed,
                                            (uint32_t)(seed >> 32));
      // 53-bit uniforms from two words each
      const double u_src = (double)((((uint64_t)blk.w[0] << 32) | blk.w[1]) >> 11) * (1.0 / 9007199254740992.0);
      const double u_dst = (double)((((uint64_t)blk.w[2] << 32) | blk.w[3]) >> 11) * (1.0 / 9007199254740992.0);
      src[e] = pick(u_src);
      dst[e] = pick(u_dst);
      w[e] = edge_weight_for(seed, e);
    }
  });
  return csr_from_edges(out, n_vertices, (size_t)n_edges, src.data(), dst.data(), w.data(), error);
}

}  // namespace nd
