// Host-side validation of sampling results (rules: src/check_results.cu:46-299).
#include "nd_check.hpp"

#include <algorithm>
#include <atomic>
#include <mutex>
#include <sstream>
#include <thread>

namespace nd {
namespace {

bool adjacent(const CSR& g, int32_t from, int32_t to) {
  if (!g.has_vertex(from)) return false;
  const int32_t* first = g.col.data() + g.row_ptr[from];
  const int32_t* last = g.col.data() + g.row_ptr[from + 1];
  return std::binary_search(first, last, to);
}

// The first violation found by any thread; later ones are dropped.
class Verdict {
 public:
  bool failed() const { return failed_.load(std::memory_order_relaxed); }
  void fail(const std::string& what) {
    std::lock_guard<std::mutex> lock(mutex_);
    if (!failed_.load()) {
      report_ = what;
      failed_.store(true);
    }
  }
  const std::string& report() const { return report_; }

 private:
  std::atomic<bool> failed_{false};
  std::mutex mutex_;
  std::string report_;
};

template <class Fn>
void for_each_sample(int64_t n_samples, Verdict& verdict, Fn fn) {
  unsigned workers = std::min(std::thread::hardware_concurrency(), 16u);
  if (workers == 0) workers = 4;
  const int64_t block = 256;
  if (n_samples <= block) workers = 1;
  std::atomic<int64_t> next(0);
  auto work = [&]() {
    for (;;) {
      const int64_t begin = next.fetch_add(block);
      if (begin >= n_samples || verdict.failed()) return;
      const int64_t end = std::min(n_samples, begin + block);
      for (int64_t s = begin; s < end; ++s) fn(s);
    }
  };
  if (workers == 1) {
    work();
    return;
  }
  std::vector<std::thread> pool;
  for (unsigned t = 0; t < workers; ++t) pool.emplace_back(work);
  for (auto& th : pool) th.join();
}

struct StepLayout {
  int64_t transits;  // T_k
  int64_t outputs;   // entries of the step's segment
  int64_t base;      // offset of the segment inside a sample's row
};

std::vector<StepLayout> layout_of(const SampleShape& shape, int64_t* final_size) {
  std::vector<StepLayout> steps(shape.step_size.size());
  int64_t transits = shape.initial_size, base = 0;
  for (size_t k = 0; k < steps.size(); ++k) {
    const int64_t m = shape.step_size[k];
    steps[k].transits = transits;
    steps[k].outputs = shape.collective ? m : transits * m;
    steps[k].base = base;
    base += steps[k].outputs;
    transits = steps[k].outputs;
  }
  *final_size = base;
  return steps;
}

}  // namespace

bool check_sampled_vertices(const CSR& graph, const SampleShape& shape, int64_t n_samples, const int32_t* initial,
                            const int32_t* final_samples, int32_t invalid, std::string* report) {
  int64_t final_size = 0;
  const std::vector<StepLayout> steps = layout_of(shape, &final_size);
  Verdict verdict;
  for_each_sample(n_samples, verdict, [&](int64_t s) {
    const int32_t* row = final_samples + s * final_size;
    for (size_t k = 0; k < steps.size(); ++k) {
      const StepLayout& at = steps[k];
      const int32_t* transits = k == 0 ? initial + s * shape.initial_size : row + steps[k - 1].base;
      const int64_t m = shape.step_size[k];
      int64_t sampled = 0;
      for (int64_t o = 0; o < at.outputs; ++o) {
        const int32_t v = row[at.base + o];
        if (v == invalid) continue;
        ++sampled;
        bool found = false;
        if (v >= 0 && v < graph.get_n_vertices()) {
          // the transit the engine drew this output for, then (apps that choose their own
          // transits) any vertex of the previous step
          if (!shape.collective) {
            const int32_t own = transits[o / m];
            found = own != invalid && adjacent(graph, own, v);
          }
          for (int64_t t = 0; t < at.transits && !found; ++t)
            found = transits[t] != invalid && adjacent(graph, transits[t], v);
        }
        if (!found) {
          std::ostringstream msg;
          msg << "Invalid '" << v << "' in Sample '" << s << "' at Step '" << k << "'";
          verdict.fail(msg.str());
          return;
        }
      }
      if (sampled == 0 && !shape.collective) {
        int64_t edges_before = 0;
        for (int64_t t = 0; t < at.transits; ++t)
          if (transits[t] != invalid && graph.has_vertex(transits[t])) edges_before += graph.n_edges_for_vertex(transits[t]);
        if (edges_before > 0) {
          std::ostringstream msg;
          msg << "Step " << k << ": no vertex sampled for sample '" << s << "' but the vertices of the previous step have "
              << edges_before << " edges";
          verdict.fail(msg.str());
          return;
        }
      }
    }
  });
  if (verdict.failed() && report) *report = verdict.report();
  return !verdict.failed();
}

bool check_layer_adjacency_matrix(const CSR& graph, const SampleShape& shape, int64_t n_samples,
                                  const int32_t* initial, const int32_t* final_samples, const int32_t* rows,
                                  const int32_t* cols, size_t state_stride, int32_t invalid, std::string* report) {
  int64_t final_size = 0;
  const std::vector<StepLayout> steps = layout_of(shape, &final_size);
  Verdict verdict;
  for_each_sample(n_samples, verdict, [&](int64_t s) {
    const int32_t* row = final_samples + s * final_size;
    for (size_t k = 0; k < steps.size(); ++k) {
      const int64_t batch = shape.step_size[k];
      const int64_t n_transits = k == 0 ? shape.initial_size : shape.step_size[k - 1];
      const int32_t* transits = k == 0 ? initial + s * shape.initial_size : row + steps[k - 1].base;
      const int32_t* layer = row + steps[k].base;
      const int32_t* r = rows + s * state_stride + k * batch * batch;
      const int32_t* c = cols + s * state_stride + k * batch * batch;
      for (int64_t i = 0; i < n_transits; ++i) {
        for (int64_t nbr = 0; nbr < batch; ++nbr) {
          const int64_t at = i * batch + nbr;
          const bool recorded = !(r[at] == -1 && c[at] == -1);
          if (recorded && (r[at] != i || c[at] != nbr)) {
            std::ostringstream msg;
            msg << "Sample '" << s << "' step " << k << ": entry " << at << " holds (" << r[at] << ", " << c[at] << ")";
            verdict.fail(msg.str());
            return;
          }
          const int32_t from = transits[i], to = layer[nbr];
          const bool edge = from != invalid && to != invalid && adjacent(graph, from, to);
          if (recorded != edge) {
            std::ostringstream msg;
            if (recorded) msg << "Invalid '" << to << "' in Sample '" << s << "' for previous step vertex '" << from << "' Step '" << k << "'";
            else msg << "Edge '" << from << "'->'" << to << "' exists in Graph but not in sample " << s << " at step " << k;
            verdict.fail(msg.str());
            return;
          }
        }
      }
    }
  });
  if (verdict.failed() && report) *report = verdict.report();
  return !verdict.failed();
}

bool check_subgraph_edge_lists(const CSR& graph, int64_t n_samples, int vertices_per_sample, const int32_t* vertices,
                               const uint32_t* list_start, const int32_t* rows, const int32_t* cols,
                               std::string* report) {
  Verdict verdict;
  for_each_sample(n_samples, verdict, [&](int64_t s) {
    const uint32_t begin = list_start[s], end = list_start[s + 1];
    for (uint32_t e = begin; e < end; ++e) {
      if (!adjacent(graph, rows[e], cols[e])) {
        std::ostringstream msg;
        msg << "Sample '" << s << "': no edge '" << rows[e] << "' -> '" << cols[e] << "' in graph";
        verdict.fail(msg.str());
        return;
      }
    }
    const int32_t* mine = vertices + s * vertices_per_sample;
    for (int a = 0; a < vertices_per_sample; ++a) {
      for (int b = 0; b < vertices_per_sample; ++b) {
        const int32_t v1 = mine[a], v2 = mine[b];
        if (v1 == v2 || !adjacent(graph, v1, v2)) continue;
        bool listed = false;
        for (uint32_t e = begin; e < end && !listed; ++e) listed = rows[e] == v1 && cols[e] == v2;
        if (!listed) {
          std::ostringstream msg;
          msg << "Sample '" << s << "': Edge '" << v1 << "'->'" << v2 << "' exists in graph but not in sample of length '"
              << (end - begin) << "'";
          verdict.fail(msg.str());
          return;
        }
      }
    }
  });
  if (verdict.failed() && report) *report = verdict.report();
  return !verdict.failed();
}

}  // namespace nd
