// Several engines, each sampling a contiguous range of the app's samples on its own stream.
//
// Samples are independent, and an engine given a range uses the sample indices, roots and
// random streams of the whole run (Engine::alloc_range), so the ranges put together are the
// bytes a single engine produces.  This is how the path shards over devices (the reference
// splits samples the same way, src/nextdoor.cu:1902-1909, 2024-2025): one engine per device,
// the graph replicated, nothing exchanged between steps.
//
// On ONE device two ranges of a large walk can run out of phase and fill each other's gaps
// (the inversion's passes are short and latency bound, the step kernel long and bandwidth
// bound), but the smaller launches lose as much as the overlap gains (4.2 M weighted node2vec
// walks: 43.6 ms per pass as one range, 44.8 ms as two), so one range is the default and
// ND_SAMPLE_RANGES=2 is there for tests and comparisons.
//
// With profiling on, the ranges run one after the other so that the per-phase times are
// those of undisturbed kernels.
#pragma once

#include "nd_engine.hpp"

namespace nd {

template <class SampleType, class App>
class ShardedEngine : public EngineBase {
  typedef Engine<SampleType, App> Part;

 public:
  explicit ShardedEngine(const char* name) : name_(name) { parts_.emplace_back(new Part(name)); }

  const char* app_name() const override { return name_; }
  int64_t num_samples() const override {
    int64_t n = 0;
    for (const auto& p : parts_) n += p->num_samples();
    return n;
  }
  int final_sample_size() const override { return parts_[0]->final_sample_size(); }
  int steps() const override { return parts_[0]->steps(); }
  int step_size(int k) const override { return parts_[0]->step_size(k); }
  int initial_sample_size() const override { return parts_[0]->initial_sample_size(); }
  int sampling_type() const override { return parts_[0]->sampling_type(); }
  bool has_explicit_transits() const override { return parts_[0]->has_explicit_transits(); }
  int32_t invalid_vertex() const override { return parts_[0]->invalid_vertex(); }
  int max_bits() const override { return parts_[0]->max_bits(); }
  size_t sample_state_bytes() const override {
    size_t n = 0;
    for (const auto& p : parts_) n += p->sample_state_bytes();
    return n;
  }

  int set_graph(const CSR* graph) override {
    graph_ = nullptr;
    parts_.resize(1);
    if (parts_[0]->set_graph(graph) != 0) return fail(0);
    graph_ = graph;
    return 0;
  }

  int alloc(uint64_t seed) override {
    if (!graph_) { last_error = "alloc before set_graph"; return -1; }
    parts_.resize(1);
    App app;
    const int64_t n = app.numSamples(const_cast<CSR*>(graph_));
    bool walk = app.initialSampleSize(const_cast<CSR*>(graph_)) == 1 && app.steps() > 1;
    for (int k = 0; k < app.steps(); ++k) walk = walk && app.stepSize(k) == 1;
    int n_parts = 1;
    if (const char* env = getenv("ND_SAMPLE_RANGES")) {  // 2: walks are sampled as two ranges
      if (atoi(env) == 2 && walk && n >= 2) n_parts = 2;
    }
    while ((int)parts_.size() < n_parts) {
      parts_.emplace_back(new Part(name_));
      parts_.back()->share_graph(*parts_[0]);
    }
    initialContents.clear();
    int64_t first = 0;
    for (int i = 0; i < n_parts; ++i) {
      const int64_t count = (n - first) / (n_parts - i);
      const int rc = parts_[i]->alloc_range(seed, first, count, /*host_rows=*/false);  // the rows come home through ours
      if (rc != 0) return fail(i, rc);
      initialContents.insert(initialContents.end(), parts_[i]->initialContents.begin(),
                             parts_[i]->initialContents.end());
      first += count;
    }
    hFinalSamples.assign((size_t)n * (size_t)final_sample_size(), invalid_vertex());
    return 0;
  }

  int sample(int mode) override {
    for (auto& p : parts_) {
      p->inversion_period = inversion_period;
      p->launch_graph = launch_graph;
      p->profiling = profiling;
    }
    times = PhaseTimes();
    const auto t0 = std::chrono::steady_clock::now();
    std::vector<int> rc(parts_.size(), 0);
    if (parts_.size() == 1 || profiling) {
      for (size_t i = 0; i < parts_.size(); ++i) rc[i] = parts_[i]->sample(mode);
    } else {
      // one host thread per range: each enqueues its own chain of launches and waits for it
      std::vector<std::thread> threads;
      for (size_t i = 0; i < parts_.size(); ++i)
        threads.emplace_back([this, &rc, i, mode] { rc[i] = parts_[i]->sample(mode); });
      for (auto& t : threads) t.join();
    }
    const auto t1 = std::chrono::steady_clock::now();
    for (size_t i = 0; i < parts_.size(); ++i)
      if (rc[i] != 0) return fail((int)i, rc[i]);
    for (const auto& p : parts_) {
      const PhaseTimes& t = p->times;
      times.inversion += t.inversion;
      times.load_balancing += t.load_balancing;
      times.flat_kernel += t.flat_kernel;
      times.workgroup_kernel += t.workgroup_kernel;
      times.assemble += t.assemble;
      times.flat_launches += t.flat_launches;
      times.workgroup_launches += t.workgroup_launches;
      times.sort_launches += t.sort_launches;
    }
    times.end_to_end = parts_.size() == 1 ? parts_[0]->times.end_to_end
                                          : std::chrono::duration<float, std::milli>(t1 - t0).count();
    return 0;
  }

  int fetch_final_samples() override {
    size_t at = 0;
    for (size_t i = 0; i < parts_.size(); ++i) {
      if (parts_[i]->fetch_final_samples_into(hFinalSamples.data() + at) != 0) return fail((int)i);
      at += (size_t)parts_[i]->num_samples() * (size_t)final_sample_size();
    }
    return 0;
  }

  int fetch_sample_states(void* dst, size_t bytes) override {
    if (bytes != sample_state_bytes() || bytes == 0) { last_error = "sample state size mismatch"; return -1; }
    char* out = (char*)dst;
    for (size_t i = 0; i < parts_.size(); ++i) {
      const size_t n = parts_[i]->sample_state_bytes();
      if (parts_[i]->fetch_sample_states(out, n) != 0) return fail((int)i);
      out += n;
    }
    return 0;
  }

  int distinct() override {
    hDistinctCounts.clear();
    times.distinct = 0;
    for (size_t i = 0; i < parts_.size(); ++i) {
      const int rc = parts_[i]->distinct();
      if (rc != 0) return fail((int)i, rc);
      times.distinct += parts_[i]->times.distinct;
      hDistinctCounts.insert(hDistinctCounts.end(), parts_[i]->hDistinctCounts.begin(),
                             parts_[i]->hDistinctCounts.end());
    }
    return 0;
  }

  int64_t counter(int which) const override {
    int64_t n = 0;
    for (const auto& p : parts_) n += p->counter(which);
    return n;
  }

  void free_device() override {
    for (auto& p : parts_) p->free_device();
    graph_ = nullptr;
  }

 private:
  int fail(int part, int rc = -1) {
    last_error = parts_[(size_t)part]->last_error;
    return rc;
  }

  const char* name_;
  const CSR* graph_ = nullptr;
  std::vector<std::unique_ptr<Part>> parts_;
};

}  // namespace nd
