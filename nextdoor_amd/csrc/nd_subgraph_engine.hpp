// Engine for IndividualNeighborhood apps whose output format is AdjacencyMatrix: the samples'
// results are edge lists (row, col) in storage shared by all samples (the reference's MVS and
// ClusterGCN apps, src/apps/mvs/mvsSampling.cu and src/apps/clustergcn/clusterGCNSampling.cu,
// whose next() appends to per-sample lists with atomics).
//
// Schedule.  The (transit, neighbour slot) lanes of a sample and step, in slot order, are cut
// into units of 64; one wavefront runs one unit, so a sample with many lanes (or with a hub
// among its transits) is spread over many wavefronts.  Every step runs twice:
//   count pass  next() runs with a sink that only counts the emit() calls; the wave stores the
//               unit's total and writes the step's sampled vertices into the sample's result
//               row (they are the next step's transits);
//   write pass  the lengths of the lists (the units of a sample added up) have been scanned
//               over the samples, which fixes where every list starts; next() runs again, and a
//               unit's edges go to: start of the list + the units of the sample before this
//               one (earlier steps first).
// The lists are therefore packed back to back in sample order; inside a list the edges are
// ordered by step, then by unit, and inside a unit the lanes' edges are interleaved (every
// lane's first edge in lane order, then every lane's second edge, ...).
// No atomics, no dependence on the schedule.  Random draws are keyed by the output slot, as in
// the other engines, so both passes see the same numbers.
#pragma once

#include "nd_device_scan.hpp"
#include "nd_engine.hpp"

namespace nd {

struct CountingSink {
  uint32_t n = 0;
  __device__ __forceinline__ void put(VertexID_t, VertexID_t) { ++n; }
};

// Where the edges of a unit go.  Inside a unit the lanes' edges are interleaved: first every
// lane's first edge, in lane order, then every lane's second edge, and so on.  Lanes that run
// in step then write neighbouring entries (a lane that copies thousands of edges of a hub into
// a stretch of its own walks one page per lane instead, and the address translation of 64
// pages per store took 7 us per round: 77 ms for one 320 K-edge hub).  The place of a lane's
// i-th edge depends on the lanes' counts alone, which the count run has fixed:
//   edges of all lanes with index < i, plus the lanes below it that have an i-th edge.
// `order` lists the unit's lanes by ascending count, so a lane keeps the set of lanes that
// still have an i-th edge up to date by retiring entries as i grows.
struct WritingSink {
  typedef const __attribute__((address_space(3))) uint64_t* OrderPointer;
  // nothing the app reads lives in the lists: loads may be moved ahead of these stores
  VertexID_t* __restrict__ rows;  // start of the unit's stretch
  VertexID_t* __restrict__ cols;
  OrderPointer order;             // 64 entries (count << 8 | lane), ascending; unused when no lane has more than kEarly edges
  uint32_t early_at;              // where the lane's next edge of index < kEarly goes: known before next() runs
  uint32_t early_steps;           // then 8 bits each: from edge 0 to edge 1, 1 to 2, 2 to 3 (one running value:
                                  // a choice among four members would keep the whole object in memory)
  uint64_t with_edge = ~0ull;     // from index kEarly on: lanes that have an edge of index n
  uint64_t below_me;
  uint32_t before = 0;            // from index kEarly on: edges of the unit with index < n
  uint32_t retired = 0;           // entries of `order` already taken out of with_edge
  uint32_t n = 0;
  static constexpr uint32_t kEarly = 4;
  __device__ __forceinline__ void put(VertexID_t row, VertexID_t col) {
    uint32_t at;
    if (n < kEarly) {
      // most lanes list a few edges: no trip to the table for those (a lane used to walk the
      // table entry by entry, one LDS latency each, past every lane without edges)
      at = early_at;
      early_at += early_steps & 0xFFu;
      early_steps >>= 8;
    } else {
      while (retired < 64) {
        const uint64_t entry = order[retired];
        if ((uint32_t)(entry >> 8) > n) break;
        with_edge &= ~(1ull << (entry & 63u));
        ++retired;
      }
      at = before + (uint32_t)__popcll(with_edge & below_me);
      before += (uint32_t)__popcll(with_edge);
    }
    rows[at] = row;
    cols[at] = col;
    ++n;
  }
};

// What next() of an AdjacencyMatrix app sees as its sample: the stored state, read only, and
// the lane's sink for edges.
template <class Stored, class Sink>
class EmittingSample {
 public:
  __device__ EmittingSample(const Stored* stored, const Sink& sink) : stored_(stored), sink_(sink) {}
  __device__ __forceinline__ const Stored& state() const { return *stored_; }
  __device__ __forceinline__ void emit(VertexID_t row, VertexID_t col) { sink_.put(row, col); }
  __device__ __forceinline__ uint32_t emitted() const { return sink_.n; }

 private:
  const Stored* stored_;
  Sink sink_;
};

struct SubgraphStepParams {
  CSRPartition csr;
  int step;
  uint32_t step_size;            // m_k
  uint32_t transits_per_sample;  // T_k
  const VertexID_t* transits;    // transit j of sample s: transits[s * transit_pitch + j]
  uint32_t transit_pitch;
  VertexID_t* final_rows;        // [n_samples][final_size]
  uint32_t final_size;
  uint32_t seg_base;             // offset of the step's segment inside a result row
  int32_t invalid;
  uint64_t seed;
  uint64_t first_sample;
  uint32_t n_samples;
  // Apps with explicit transits: what App::stepTransits returned for every output of the step,
  // at the output's place in a second set of rows (the transits of the next step); else nullptr
  VertexID_t* next_transit_rows;
  int is_last;
  const void* stored;            // SampleType[n_samples]
  uint32_t units_per_step;       // units (64 lanes) of this step per sample
  uint32_t units_before_step;    // units of the earlier steps per sample
  uint32_t units_per_sample;     // all steps
  uint32_t* unit_counts;         // [n_samples][units_per_sample] edges emitted by every unit
  const uint32_t* list_start;    // write pass: start of the sample's list in rows / cols
  VertexID_t* rows;
  VertexID_t* cols;
};

constexpr int kSubgraphThreads = 256;  // four units per workgroup

template <class Stored, class App, bool kWrite>
__global__ __launch_bounds__(kSubgraphThreads) void subgraph_step_kernel(SubgraphStepParams P) {
  __shared__ uint64_t s_order[kSubgraphThreads / 64][64];
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = threadIdx.x >> 6;
  const uint64_t unit = (uint64_t)blockIdx.x * (kSubgraphThreads / 64) + wave;
  // wavefronts past the last unit touch nothing
  const bool live = unit < (uint64_t)P.n_samples * P.units_per_step;
  const uint32_t s = live ? (uint32_t)(unit / P.units_per_step) : 0u;
  const uint32_t unit_in_step = live ? (uint32_t)(unit - (uint64_t)s * P.units_per_step) : 0u;
  const uint32_t unit_in_sample = P.units_before_step + unit_in_step;
  const Stored* stored = (const Stored*)P.stored + s;
  const uint32_t lanes_of_sample = P.transits_per_sample * P.step_size;
  CSRPartition csr = P.csr;

  uint32_t* counts_of_sample = P.unit_counts + (size_t)s * P.units_per_sample;
  // write pass: a unit that emitted nothing has nothing to do (the count pass knows)
  if (kWrite && (!live || counts_of_sample[unit_in_sample] == 0)) return;
  const uint32_t l = unit_in_step * 64u + lane;
  const bool has_lane = live && l < lanes_of_sample;
  uint32_t count = 0;
  VertexID neighbor = P.invalid;
  VertexID transit = P.invalid;
  uint32_t nbr = 0;
  EdgePos_t begin = 0, n_edges = 0;
  float max_weight = 0.0f;
  if (has_lane) {
    const uint32_t j = l / P.step_size;
    nbr = l - j * P.step_size;
    transit = P.transits[(size_t)s * P.transit_pitch + j];
    if (transit != P.invalid) {
      begin = csr.row_ptr[transit];
      n_edges = csr.row_ptr[transit + 1] - begin;
      max_weight = csr.max_weights[transit];
    }
  }
  const bool runs = transit != P.invalid && n_edges != 0;  // as src/nextdoor.cu:250-262
  const VertexID* edges = csr.edges + begin;
  const float* weights = csr.weights + begin;
  const uint64_t out_slot = (P.first_sample + s) * (uint64_t)lanes_of_sample + l;
  // explicit transits (src/nextdoor.cu:279-289): after next(), with the same random state, the
  // app names the transit this output stands for at the next step; only the counting run does it
  const bool chooses_transit = !kWrite && App().hasExplicitTransits() && !P.is_last && transit != P.invalid;
  VertexID next_transit = P.invalid;
  if (runs || chooses_transit) {
    curandState rng;
    rng.reset(P.seed, out_slot, (uint32_t)P.step);
    EmittingSample<Stored, CountingSink> view(stored, CountingSink());
    if (runs) {
      const VertexID r = App().template next<EmittingSample<Stored, CountingSink>, const VertexID*, const float*>(
          P.step, &csr, &transit, (VertexID)(P.first_sample + s), &view, max_weight, edges, weights, n_edges,
          (VertexID_t)nbr, &rng);
      neighbor = r == -1 ? P.invalid : r;
      count = view.emitted();
    }
    if (chooses_transit) {
      // the index the reference hands over: its thread number modulo the step's transits per sample
      const VertexID_t t = App().stepTransits(P.step + 1, (VertexID)(P.first_sample + s), view,
                                              (int)(l % P.transits_per_sample), &rng);
      next_transit = t == -1 ? P.invalid : t;
    }
  }
  if (!kWrite) {
    const uint32_t through_me = wave_inclusive_scan(count);
    if (has_lane) P.final_rows[(size_t)s * P.final_size + P.seg_base + l] = neighbor;
    if (has_lane && P.next_transit_rows) P.next_transit_rows[(size_t)s * P.final_size + P.seg_base + l] = next_transit;
    if (live && lane == 63) counts_of_sample[unit_in_sample] = through_me;
    return;
  }
  // edges of the sample's units before this one
  uint32_t before = 0;
  if (live)
    for (uint32_t u = lane; u < unit_in_sample; u += 64) before += counts_of_sample[u];
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) before += __shfl_xor(before, d, 64);
  WritingSink sink;
  uint32_t first_edge = live ? P.list_start[s] + before : 0u;  // of the unit
  {
    const uint64_t below = (1ull << lane) - 1ull;
    const uint64_t have0 = __ballot(count > 0), have1 = __ballot(count > 1), have2 = __ballot(count > 2),
                   have3 = __ballot(count > 3);
    uint32_t through = (uint32_t)__popcll(have0);
    const uint32_t at0 = (uint32_t)__popcll(have0 & below);
    const uint32_t at1 = through + (uint32_t)__popcll(have1 & below);
    through += (uint32_t)__popcll(have1);
    const uint32_t at2 = through + (uint32_t)__popcll(have2 & below);
    through += (uint32_t)__popcll(have2);
    const uint32_t at3 = through + (uint32_t)__popcll(have3 & below);
    sink.early_at = at0;
    sink.early_steps = (at1 - at0) | ((at2 - at1) << 8) | ((at3 - at2) << 16);  // each at most 128
    sink.before = through + (uint32_t)__popcll(have3);
  }
  if (__ballot(count > WritingSink::kEarly) == 0) {
    sink.order = nullptr;  // never read
  } else {
    // the unit's lanes by ascending (count, lane): a lane's place is the number of lanes
    // before it.  Only this wavefront reads its table, and a wavefront's LDS accesses are
    // served in order.
    uint32_t place = 0;
    for (int other = 0; other < 64; ++other) {
      const uint32_t c = __shfl(count, other, 64);
      place += (c < count || (c == count && (uint32_t)other < lane)) ? 1u : 0u;
    }
    s_order[wave][place] = ((uint64_t)count << 8) | lane;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    sink.order = (WritingSink::OrderPointer)s_order[wave];
  }
  if (count != 0) {
    curandState rng;
    rng.reset(P.seed, out_slot, (uint32_t)P.step);
    sink.rows = P.rows + first_edge;
    sink.cols = P.cols + first_edge;
    sink.below_me = (1ull << lane) - 1ull;
    EmittingSample<Stored, WritingSink> view(stored, sink);
    (void)App().template next<EmittingSample<Stored, WritingSink>, const VertexID*, const float*>(
        P.step, &csr, &transit, (VertexID)(P.first_sample + s), &view, max_weight, edges, weights, n_edges,
        (VertexID_t)nbr, &rng);
  }
}

// lengths[s] = sum of the sample's unit counts; lengths[n_samples] = 0
__global__ __launch_bounds__(256) void subgraph_list_lengths(const uint32_t* __restrict__ unit_counts,
                                                             uint32_t units_per_sample, uint32_t n_samples,
                                                             uint32_t* __restrict__ lengths) {
  const uint32_t s = blockIdx.x * 256 + threadIdx.x;
  if (s > n_samples) return;
  uint32_t total = 0;
  if (s < n_samples)
    for (uint32_t u = 0; u < units_per_sample; ++u) total += unit_counts[(size_t)s * units_per_sample + u];
  lengths[s] = total;
}

// total += sum of in[0..n), 64-bit (the lengths are 32-bit; their sum may not be)
__global__ __launch_bounds__(256) void sum_lengths(const uint32_t* __restrict__ in, size_t n,
                                                   unsigned long long* __restrict__ total) {
  __shared__ unsigned long long s_part[4];
  unsigned long long acc = 0;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) acc += in[i];
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) acc += __shfl_down(acc, d, 64);
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) atomicAdd(total, s_part[0] + s_part[1] + s_part[2] + s_part[3]);
}

template <class SampleType, class App>
class SubgraphEngine : public EngineBase {
 public:
  explicit SubgraphEngine(const char* name) : name_(name) {}
  ~SubgraphEngine() override { free_device(); }

  const char* app_name() const override { return name_; }
  int64_t num_samples() const override { return n_samples_; }
  // Every output slot of every step has its place in the result row: sum over the steps of
  // initialSampleSize * stepSize(0) * ... * stepSize(k).  (The reference's getFinalSampleSize,
  // src/nextdoor.cu:1913-1929, leaves the initial size out - 32 and 33 entries for its MVS and
  // ClusterGCN, fewer than the slots their steps have; both apps ignore the result row.)
  int final_sample_size() const override {
    App app;
    int64_t total = 0, per_step = app.initialSampleSize(nullptr);
    for (int k = 0; k < app.steps(); ++k) {
      per_step *= app.stepSize(k);
      total += per_step;
    }
    return (int)total;
  }
  int steps() const override { return App().steps(); }
  int step_size(int k) const override { return App().stepSize(k); }
  int initial_sample_size() const override { return App().initialSampleSize(nullptr); }
  int sampling_type() const override { return App().samplingType(); }
  int32_t invalid_vertex() const override { return invalid_; }
  int max_bits() const override { return max_bits_; }
  size_t sample_state_bytes() const override { return sizeof(SampleType) * (size_t)n_samples_; }

  int set_graph(const CSR* graph) override {
    free_run_buffers();  // sized against the previous graph: alloc() is due again
    graph_ = nullptr;
    if (!dgraph_.upload(graph, false, false, &last_error)) return -1;
    graph_ = graph;
    return 0;
  }

  int alloc(uint64_t seed) override {
    if (!graph_) { last_error = "alloc before set_graph"; return -1; }
    free_run_buffers();
    seed_ = seed;
    CSR* csr = const_cast<CSR*>(graph_);
    App app;
    if (is_collective<App>() || app.outputFormat() != AdjacencyMatrix) {
      last_error = "not an IndividualNeighborhood app with AdjacencyMatrix output";
      return -2;
    }
    const int n_steps = app.steps();
    if (n_steps < 1 || n_steps > kMaxSteps) { last_error = "steps() must be in [1, 128]"; return -2; }
    n_samples_ = app.numSamples(csr);
    init_size_ = app.initialSampleSize(csr);
    if (n_samples_ <= 0 || init_size_ <= 0) { last_error = "app yields no samples"; return -2; }
    if (n_samples_ >= (1ll << 31)) { last_error = "too many samples"; return -2; }
    layout_ = StepLayout();
    uint64_t transits = (uint64_t)init_size_, base = 0;
    for (int k = 0; k < n_steps; ++k) {
      if (app.stepSize(k) <= 0) { last_error = "stepSize must be positive"; return -2; }
      const uint64_t outputs = transits * (uint64_t)app.stepSize(k);
      if (base + outputs >= (1ull << 31)) { last_error = "final sample too large"; return -2; }
      layout_.seg_base[k] = (uint32_t)base;
      layout_.seg_len[k] = (uint32_t)outputs;
      base += outputs;
      transits = outputs;
    }
    invalid_ = graph_->get_n_vertices();
    max_bits_ = 0;
    while ((invalid_ >> max_bits_) != 0) max_bits_++;

    std::vector<SampleType> stored;
    stored.reserve((size_t)n_samples_);
    initialContents.clear();
    for (int64_t s = 0; s < n_samples_; ++s) {
      stored.push_back(app.template initializeSample<SampleType>(csr, (VertexID_t)s));
      std::vector<VertexID_t> roots = app.initialSample((int)s, csr, stored.back());
      if ((EdgePos_t)roots.size() != init_size_) {
        last_error = "initialSample size differs from initialSampleSize";
        return -2;
      }
      if (!roots_are_vertices(roots, graph_->get_n_vertices())) {
        last_error = "initialSample returned a root that is not a vertex of the graph";
        return -2;
      }
      initialContents.insert(initialContents.end(), roots.begin(), roots.end());
    }
    const size_t F = (size_t)final_sample_size();
    hFinalSamples.assign((size_t)n_samples_ * F, invalid_);

    ND_HIP_TRY(hipStreamCreate(&stream_));
    ND_HIP_TRY(hipEventCreate(&ev_begin_));
    ND_HIP_TRY(hipEventCreate(&ev_end_));
    allocated_ = true;
    const size_t per_sample = sizeof(uint32_t) * ((size_t)n_samples_ + 1);
    ND_HIP_TRY(hipMalloc(&d_initial_, sizeof(VertexID_t) * initialContents.size()));
    ND_HIP_TRY(hipMemcpy(d_initial_, initialContents.data(), sizeof(VertexID_t) * initialContents.size(),
                         hipMemcpyHostToDevice));
    ND_HIP_TRY(hipMalloc(&d_stored_, sizeof(SampleType) * (size_t)n_samples_));
    ND_HIP_TRY(hipMemcpy(d_stored_, stored.data(), sizeof(SampleType) * (size_t)n_samples_, hipMemcpyHostToDevice));
    ND_HIP_TRY(hipMalloc(&d_final_, sizeof(VertexID_t) * (size_t)n_samples_ * F));
    if (app.hasExplicitTransits() && n_steps > 1)
      ND_HIP_TRY(hipMalloc(&d_next_transits_, sizeof(VertexID_t) * (size_t)n_samples_ * F));
    ND_HIP_TRY(hipMalloc(&d_lengths_, per_sample));
    ND_HIP_TRY(hipMalloc(&d_list_start_, per_sample));
    units_per_sample_ = 0;
    for (int k = 0; k < n_steps; ++k) {
      units_before_[k] = units_per_sample_;
      units_per_sample_ += (layout_.seg_len[k] + 63u) / 64u;
    }
    ND_HIP_TRY(hipMalloc(&d_unit_counts_, sizeof(uint32_t) * (size_t)n_samples_ * units_per_sample_));
    ND_HIP_TRY(hipMalloc(&d_scan_scratch_, sizeof(uint32_t) * scan_scratch_elems((size_t)n_samples_ + 1)));
    ND_HIP_TRY(hipMalloc(&d_total_, sizeof(unsigned long long)));
    return 0;
  }

  // One schedule for every kernel mode: the lists do not depend on it.
  int sample(int) override {
    if (!allocated_) { last_error = "sample before alloc"; return -1; }
    App app;
    const int n_steps = app.steps();
    times = PhaseTimes();
    ND_HIP_TRY(hipStreamSynchronize(stream_));
    ND_HIP_TRY(hipEventRecord(ev_begin_, stream_));
    ND_HIP_TRY(hipMemsetAsync(d_total_, 0, sizeof(unsigned long long), stream_));
    for (int step = 0; step < n_steps; ++step) {
      subgraph_step_kernel<SampleType, App, false><<<dim3(grid_for(step)), dim3(kSubgraphThreads), 0, stream_>>>(
          params_for(step));
      times.flat_launches++;
    }
    subgraph_list_lengths<<<dim3((unsigned)((n_samples_ + 256) / 256)), dim3(256), 0, stream_>>>(
        d_unit_counts_, units_per_sample_, (uint32_t)n_samples_, d_lengths_);
    ND_HIP_TRY(hipGetLastError());
    // where every list starts, and how much room all of them need
    ND_HIP_TRY(exclusive_scan_u32(d_lengths_, d_list_start_, (size_t)n_samples_ + 1, d_scan_scratch_, stream_));
    sum_lengths<<<dim3(256), dim3(256), 0, stream_>>>(d_lengths_, (size_t)n_samples_, d_total_);
    ND_HIP_TRY(hipGetLastError());
    unsigned long long total = 0;
    ND_HIP_TRY(hipMemcpyAsync(&total, d_total_, sizeof(total), hipMemcpyDeviceToHost, stream_));
    ND_HIP_TRY(hipStreamSynchronize(stream_));
    if (total >= (1ull << 31)) {
      last_error = "the edge lists of all samples hold " + std::to_string(total) + " edges; list positions are 32-bit";
      return -3;
    }
    n_edges_listed_ = (int64_t)total;
    if (total > list_capacity_) {
      release(d_rows_);
      release(d_cols_);
      list_capacity_ = 0;
      ND_HIP_TRY(hipMalloc(&d_rows_, sizeof(VertexID_t) * (size_t)total));
      ND_HIP_TRY(hipMalloc(&d_cols_, sizeof(VertexID_t) * (size_t)total));
      list_capacity_ = total;
    }
    if (total > 0) {
      for (int step = 0; step < n_steps; ++step) {
        subgraph_step_kernel<SampleType, App, true><<<dim3(grid_for(step)), dim3(kSubgraphThreads), 0, stream_>>>(
            params_for(step));
        times.flat_launches++;
      }
      ND_HIP_TRY(hipGetLastError());
    }
    ND_HIP_TRY(hipEventRecord(ev_end_, stream_));
    ND_HIP_TRY(hipStreamSynchronize(stream_));
    ND_HIP_TRY(hipEventElapsedTime(&times.end_to_end, ev_begin_, ev_end_));
    times.flat_kernel = times.end_to_end;
    return 0;
  }

  int fetch_final_samples() override {
    if (!allocated_) { last_error = "no device data"; return -1; }
    ND_HIP_TRY(hipMemcpy(hFinalSamples.data(), d_final_, sizeof(VertexID_t) * hFinalSamples.size(),
                         hipMemcpyDeviceToHost));
    return 0;
  }

  int fetch_sample_states(void* dst, size_t bytes) override {
    if (!allocated_) { last_error = "no device data"; return -1; }
    if (bytes != sample_state_bytes()) { last_error = "sample state buffer has the wrong size"; return -2; }
    ND_HIP_TRY(hipMemcpy(dst, d_stored_, bytes, hipMemcpyDeviceToHost));
    return 0;
  }

  bool lists_edges() const override { return true; }

  int fetch_adjacency() override {
    if (!allocated_) { last_error = "no device data"; return -1; }
    hListStart.resize((size_t)n_samples_ + 1);
    hListRows.resize((size_t)n_edges_listed_);
    hListCols.resize((size_t)n_edges_listed_);
    ND_HIP_TRY(hipMemcpy(hListStart.data(), d_list_start_, sizeof(uint32_t) * hListStart.size(), hipMemcpyDeviceToHost));
    if (n_edges_listed_ > 0) {
      ND_HIP_TRY(hipMemcpy(hListRows.data(), d_rows_, sizeof(VertexID_t) * hListRows.size(), hipMemcpyDeviceToHost));
      ND_HIP_TRY(hipMemcpy(hListCols.data(), d_cols_, sizeof(VertexID_t) * hListCols.size(), hipMemcpyDeviceToHost));
    }
    return 0;
  }

  int distinct() override {
    last_error = "distinct applies to SampledVertices results";
    return -2;
  }

  // 0: edges in the lists of all samples after the last run
  int64_t counter(int which) const override { return which == 0 ? n_edges_listed_ : 0; }

  void free_device() override {
    free_run_buffers();
    dgraph_.release();
    graph_ = nullptr;
  }

 private:
  SubgraphStepParams params_for(int step) const {
    App app;
    SubgraphStepParams P;
    P.csr = dgraph_.view;
    P.step = step;
    P.step_size = (uint32_t)app.stepSize(step);
    P.transits_per_sample = layout_.seg_len[step] / P.step_size;
    P.final_size = (uint32_t)final_sample_size();
    if (step == 0) {
      P.transits = d_initial_;
      P.transit_pitch = (uint32_t)init_size_;
    } else {
      // the previous step's outputs, or what stepTransits made of them
      P.transits = (d_next_transits_ ? d_next_transits_ : d_final_) + layout_.seg_base[step - 1];
      P.transit_pitch = P.final_size;
    }
    P.next_transit_rows = d_next_transits_;
    P.is_last = step == app.steps() - 1;
    P.final_rows = d_final_;
    P.seg_base = layout_.seg_base[step];
    P.invalid = invalid_;
    P.seed = seed_;
    P.first_sample = 0;
    P.n_samples = (uint32_t)n_samples_;
    P.stored = d_stored_;
    P.units_per_step = (layout_.seg_len[step] + 63u) / 64u;
    P.units_before_step = units_before_[step];
    P.units_per_sample = units_per_sample_;
    P.unit_counts = d_unit_counts_;
    P.list_start = d_list_start_;
    P.rows = d_rows_;
    P.cols = d_cols_;
    return P;
  }

  unsigned grid_for(int step) const {
    const uint64_t units = (uint64_t)n_samples_ * ((layout_.seg_len[step] + 63u) / 64u);
    return (unsigned)((units + kSubgraphThreads / 64 - 1) / (kSubgraphThreads / 64));
  }

  template <class T>
  void release(T*& p) {
    if (p) (void)hipFree(p);
    p = nullptr;
  }

  void free_run_buffers() {
    // whatever exists, also after an alloc that failed half way
    if (stream_) (void)hipStreamSynchronize(stream_);
    release(d_initial_);
    release(d_stored_);
    release(d_final_);
    release(d_next_transits_);
    release(d_lengths_);
    release(d_list_start_);
    release(d_unit_counts_);
    release(d_scan_scratch_);
    release(d_total_);
    release(d_rows_);
    release(d_cols_);
    list_capacity_ = 0;
    for (hipEvent_t* ev : {&ev_begin_, &ev_end_}) {
      if (*ev) (void)hipEventDestroy(*ev);
      *ev = nullptr;
    }
    if (stream_) (void)hipStreamDestroy(stream_);
    stream_ = nullptr;
    allocated_ = false;
  }

  const char* name_;
  const CSR* graph_ = nullptr;
  DeviceGraph dgraph_;
  bool allocated_ = false;
  uint64_t seed_ = 0;
  int64_t n_samples_ = 0;
  EdgePos_t init_size_ = 0;
  int32_t invalid_ = 0;
  int max_bits_ = 0;
  StepLayout layout_;
  int64_t n_edges_listed_ = 0;
  unsigned long long list_capacity_ = 0;
  hipStream_t stream_ = nullptr;
  hipEvent_t ev_begin_ = nullptr, ev_end_ = nullptr;
  VertexID_t* d_initial_ = nullptr;
  SampleType* d_stored_ = nullptr;
  VertexID_t* d_final_ = nullptr;
  VertexID_t* d_next_transits_ = nullptr;  // rows of the transits App::stepTransits chose (explicit transits)
  uint32_t* d_lengths_ = nullptr;
  uint32_t* d_list_start_ = nullptr;
  uint32_t* d_unit_counts_ = nullptr;
  uint32_t units_per_sample_ = 0;
  uint32_t units_before_[kMaxSteps] = {};
  uint32_t* d_scan_scratch_ = nullptr;
  unsigned long long* d_total_ = nullptr;
  VertexID_t* d_rows_ = nullptr;
  VertexID_t* d_cols_ = nullptr;
};

}  // namespace nd
