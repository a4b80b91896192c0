// C ABI of the sampling engine (declarations and reference citations: include/nextdoor_amd.h).
#include "../../include/nextdoor_amd.h"

#include <string.h>

#include <deque>
#include <exception>
#include <memory>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "nd_apps_khop.hpp"
#include "nd_apps_multirw.hpp"
#include "nd_apps_subgraph.hpp"
#include "nd_apps_layer.hpp"
#include "nd_apps_walks.hpp"
#include "nd_app_registry.hpp"
#include "nd_graph.hpp"
#include "nd_check.hpp"


struct nd_sampler {
  std::unique_ptr<nd::EngineBase> engine;
  const nd_graph* graph = nullptr;
};

namespace {

thread_local std::string g_error;

int fail(const std::string& msg, int code = -1) {
  g_error = msg;
  return code;
}

// No exception leaves the library: a body that throws (host memory, a container's range
// check) reports through the error text like any other failure.
template <class Body>
int guarded(Body body) {
  try {
    return body();
  } catch (const std::bad_alloc&) {
    return fail("out of host memory");
  } catch (const std::exception& e) {
    return fail(std::string("internal error: ") + e.what());
  } catch (...) {
    return fail("internal error");
  }
}

struct AppEntry {
  const char* name;
  void* (*make)(const char*);
};

template <class SampleType, class App>
void* make_engine(const char* name) {
  return nd::make_app_engine<SampleType, App>(name);
}
template <class SampleType, class App>
void* make_subgraph_engine(const char* name) {
  return nd::make_app_engine<SampleType, App>(name);
}
template <class SampleType, class App>
void* make_layer_engine(const char* name) {
  return nd::make_app_engine<SampleType, App>(name);
}

// name -> instantiation.  The first block carries the reference's app names and sizes.
const AppEntry kApps[] = {
    {"UniformRandomWalk", make_engine<UniformRandomWalkSample, UniformRandomWalkApp>},
    {"DeepWalk", make_engine<DummySample, DeepWalkApp>},
    {"PPR", make_engine<DummySample, PPRApp>},
    {"Node2Vec", make_engine<Node2VecSample, Node2VecApp>},
    {"KHop", make_engine<KHopSample, KHopApp>},
    // one walk per vertex (benchmark configurations) and the weighted second-order walk
    {"DeepWalkPerVertex", make_engine<DummySample, DeepWalkPerVertexApp>},
    {"PPRPerVertex", make_engine<DummySample, PPRPerVertexApp>},
    {"Node2VecPerVertex", make_engine<Node2VecSample, Node2VecPerVertexApp>},
    {"WeightedNode2Vec", make_engine<Node2VecSample, WeightedNode2VecApp>},
    // four weighted second-order walks per vertex
    {"WeightedNode2Vec4PerVertex",
     make_engine<Node2VecSample, WeightedNode2VecAppT<100, 2, 1, 1, 2, nd::apps::WalksPerVertex<100, 4>>>},
    // short variants for quick checks
    {"UniformRandomWalk8", make_engine<UniformRandomWalkSample, UniformRandomWalkAppT<8>>},
    {"WeightedNode2Vec8", make_engine<Node2VecSample, WeightedNode2VecAppT<8>>},
    // the same walk with p = 4, q = 0.5 and with p = 0.5, q = 4: the three biases p, 1/q and 1 all differ
    {"WeightedNode2Vec8P4Q05", make_engine<Node2VecSample, WeightedNode2VecAppT<8, 4, 1, 1, 2>>},
    {"WeightedNode2Vec8P05Q4", make_engine<Node2VecSample, WeightedNode2VecAppT<8, 1, 2, 4, 1>>},
    {"KHop3x2", make_engine<KHopSample, KHopAppT<3, 2>>},
    {"KHop4x3x2", make_engine<KHopSample, KHopAppT<4, 3, 2>>},
    {"KHop40x30", make_engine<KHopSample, KHopAppT<40, 30>>},
    {"KHop10x10", make_engine<KHopSample, KHopAppT<10, 10>>},
    // the reference's LayerSamplingApp (src/apps/layer/layerSampling.cu: k-hop with fan-outs 10, 25)
    // and its multi-dimensional random walk (explicit transits), with a short variant
    {"Layer", make_engine<LayerSample, LayerSamplingApp>},
    {"MultiRW", make_engine<MultiRWSample, MultiRWApp>},
    {"MultiRW4x6", make_engine<MultiRWSampleT<4>, MultiRWAppT<4, 6>>},
    // edge-list results: the reference's MVS (batches of 32 vertices) and ClusterGCN (two clusters
    // of 16), and small variants
    {"MVS", make_subgraph_engine<MVSSample, MVSSamplingApp>},
    {"ClusterGCN", make_subgraph_engine<SubGraphSample, SubGraphSamplingAppI>},
    {"MVS5", make_subgraph_engine<SubgraphSampleT<5>, MVSSamplingAppT<5>>},
    {"ClusterGCN3x2", make_subgraph_engine<SubgraphSampleT<6>, SubGraphSamplingAppT<3, 2>>},
    // layer-wise apps: the reference's FastGCN / LADIES (5 layers of 64, 10000 samples) ...
    {"FastGCN", make_layer_engine<FastGCNSample, FastGCNSamplingApp>},
    {"LADIES", make_layer_engine<ImportanceSample, ImportanceSampleApp>},
    {"LayerLiteral2x8", make_layer_engine<LayerSampleT<2, 8>, LayerSamplingAppT<2, 8, 50>>},
    {"LayerLiteral3x16", make_layer_engine<LayerSampleT<3, 16>, LayerSamplingAppT<3, 16, 200>>},
    // ... and importance sampling over the union neighbourhood
    {"FastGCNImportance", make_layer_engine<LayerNoState, FastGCNImportanceAppT<2, 64, 4096>>},
    {"FastGCNImportance2x8", make_layer_engine<LayerNoState, FastGCNImportanceAppT<2, 8, 100>>},
    {"FastGCNImportance3x16", make_layer_engine<LayerNoState, FastGCNImportanceAppT<3, 16, 300>>},
    {"LADIESImportance", make_layer_engine<LayerNoState, LadiesImportanceAppT<2, 512, 1024>>},
    // the same samplers with fewer batches per launch (quick checks on the full-size graphs)
    {"FastGCNImportanceB128", make_layer_engine<LayerNoState, FastGCNImportanceAppT<2, 64, 128>>},
    {"LADIESImportanceB8", make_layer_engine<LayerNoState, LadiesImportanceAppT<2, 512, 8>>},
    {"LADIESImportance2x8", make_layer_engine<LayerNoState, LadiesImportanceAppT<2, 8, 100>>},
    {"LADIESImportance3x16", make_layer_engine<LayerNoState, LadiesImportanceAppT<3, 16, 300>>},
};
constexpr int kNumBuiltInApps = (int)(sizeof(kApps) / sizeof(kApps[0]));

// Applications added with nd_register_app, after the built-in ones.  A function-local static:
// registrations run from the static initialisers of other shared objects, in no set order.
struct RegisteredApp {
  std::string name;
  void* (*make)(const char*);
};
std::deque<RegisteredApp>& registered_apps() {
  static std::deque<RegisteredApp> apps;  // deque: names handed out stay where they are
  return apps;
}
std::mutex& registry_mutex() {
  static std::mutex m;
  return m;
}

bool find_app(const char* name, AppEntry* out) {
  for (int i = 0; i < kNumBuiltInApps; ++i)
    if (strcmp(kApps[i].name, name) == 0) { *out = kApps[i]; return true; }
  std::lock_guard<std::mutex> lock(registry_mutex());
  for (const RegisteredApp& a : registered_apps())
    if (a.name == name) { *out = AppEntry{a.name.c_str(), a.make}; return true; }
  return false;
}

nd_sampler* g_module_sampler = nullptr;
nd_graph* g_module_graph = nullptr;

struct DeviceBuffer {
  void* p = nullptr;
  ~DeviceBuffer() { if (p) (void)hipFree(p); }
  hipError_t alloc(size_t bytes) { return hipMalloc(&p, bytes ? bytes : 4); }
  template <class T> T* as() { return (T*)p; }
};

__global__ void philox_fill_kernel(uint64_t seed, uint32_t step, uint64_t first_slot, size_t n_slots,
                                   int draws_per_slot, int grouped, float* out) {
  const size_t slot = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (slot >= n_slots) return;
  nd::RandState rng;
  if (grouped) rng.reset_grouped(seed, first_slot + slot, step);
  else rng.reset(seed, first_slot + slot, step);
  for (int d = 0; d < draws_per_slot; ++d) out[slot * draws_per_slot + d] = rng.next_uniform();
}

__device__ __forceinline__ uint32_t probe_mix(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

// Every lane reads `reads` 8-byte words at hashed positions of a table of (mask + 1) words,
// kInFlight of them issued before any is used.
template <int kInFlight>
__global__ __launch_bounds__(256) void gather_rate_kernel(const uint2* __restrict__ table, uint32_t mask,
                                                         uint32_t rounds, uint32_t* sink) {
  const uint32_t lane = blockIdx.x * blockDim.x + threadIdx.x;
  uint32_t acc = 0, at = probe_mix(lane * 2654435761u + 1u);
  for (uint32_t r = 0; r < rounds; ++r) {
    uint2 got[kInFlight];
#pragma unroll
    for (int k = 0; k < kInFlight; ++k) {
      at = probe_mix(at + (uint32_t)k + r);
      got[k] = table[at & mask];
    }
#pragma unroll
    for (int k = 0; k < kInFlight; ++k) acc += got[k].x ^ got[k].y;
    at ^= acc & 1u;
  }
  sink[lane] = acc;
}

__global__ void run_counts_kernel(const uint32_t* run_start, const nd::RunsMeta* meta, uint32_t* counts) {
  const uint32_t r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r < meta->n_runs) counts[r] = run_start[r + 1] - run_start[r];
}

// Working memory of nd_sort_pairs_noalloc: one ping-pong side of the sort (keys, values), the
// digit table and the digit totals, for at most ND_SORT_PAIRS_NOALLOC_MAX pairs.  Every GPU the
// library runs on holds its own copy of the array, at its own address, until the process ends.
constexpr size_t kNoAllocMaxPairs = ND_SORT_PAIRS_NOALLOC_MAX;
constexpr size_t kNoAllocTiles = (kNoAllocMaxPairs + (size_t)nd::kSortThreads * nd::kSortItemsSmall - 1) /
                                 ((size_t)nd::kSortThreads * nd::kSortItemsSmall);
constexpr size_t kNoAllocKeysAt = 0;
constexpr size_t kNoAllocValsAt = kNoAllocKeysAt + kNoAllocMaxPairs;
constexpr size_t kNoAllocHistAt = kNoAllocValsAt + kNoAllocMaxPairs;
constexpr size_t kNoAllocTotalsAt = kNoAllocHistAt + (size_t)nd::kRadix * kNoAllocTiles;
constexpr size_t kNoAllocWords = kNoAllocTotalsAt + nd::kRadix;
static_assert(kNoAllocMaxPairs < nd::kSortLargeFrom, "the digit table is sized for the small sort tile");

static __device__ __align__(256) uint32_t scratch[kNoAllocWords];

// Address of `scratch` on each device.  In host code the array's name is only a stand-in for
// the symbol, not a device address: the address is asked for once per device, with that device
// current, and everything below uses the pointer.
constexpr int kMaxDevices = 64;
uint32_t* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

hipError_t scratch_on_current_device(uint32_t** out) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_scratch_ptr[device] = (uint32_t*)p;
  }
  *out = g_scratch_ptr[device];
  return hipSuccess;
}

#define CAPI_HIP(expr)                                                                        \
  do {                                                                                        \
    hipError_t e_ = (expr);                                                                   \
    if (e_ != hipSuccess) return fail(std::string(#expr) + ": " + hipGetErrorString(e_));     \
  } while (0)

}  // namespace

extern "C" {

const char* nd_last_error(void) { return g_error.c_str(); }

int nd_num_apps(void) {
  std::lock_guard<std::mutex> lock(registry_mutex());
  return kNumBuiltInApps + (int)registered_apps().size();
}
const char* nd_app_name(int index) {
  if (index >= 0 && index < kNumBuiltInApps) return kApps[index].name;
  std::lock_guard<std::mutex> lock(registry_mutex());
  const int i = index - kNumBuiltInApps;
  return i >= 0 && i < (int)registered_apps().size() ? registered_apps()[(size_t)i].name.c_str() : nullptr;
}

int nd_engine_abi(void) { return nd::engine_abi(); }

int nd_register_app(const char* name, void* (*make)(const char* name), int engine_abi) {
  return guarded([&]() -> int {
    if (!name || !*name || !make) return fail("null argument");
    if (engine_abi != nd::engine_abi())
      return fail(std::string("app '") + name + "' was built against engine ABI " + std::to_string(engine_abi) +
                  ", the library has " + std::to_string(nd::engine_abi()), -2);
    // one lock over the look-up and the insertion: two shared objects loading at the same time
    // cannot both find the name free
    std::lock_guard<std::mutex> lock(registry_mutex());
    bool taken = false;
    for (int i = 0; i < kNumBuiltInApps; ++i) taken = taken || strcmp(kApps[i].name, name) == 0;
    for (const RegisteredApp& a : registered_apps()) taken = taken || a.name == name;
    if (taken) return fail(std::string("an app named '") + name + "' is already registered", -3);
    registered_apps().push_back(RegisteredApp{name, make});
    return 0;
  });
}

// ---- graphs ---------------------------------------------------------------------------

int nd_graph_load(const char* path, const char* graph_type, const char* graph_format, nd_graph** out) {
  return guarded([&]() -> int {
    if (!out) return fail("null out");
    std::unique_ptr<nd_graph> g(new nd_graph);
    std::string err;
    if (nd::load_graph_file(*g, path, graph_type, graph_format, &err) != 0) return fail(err);
    *out = g.release();
    return 0;
  });
}

int nd_graph_from_edges(int32_t n_vertices, int64_t n_edges, const int32_t* src, const int32_t* dst,
                        const float* weight, nd_graph** out) {
  return guarded([&]() -> int {
    if (!out || n_edges < 0 || (n_edges > 0 && (!src || !dst))) return fail("bad argument");
    std::unique_ptr<nd_graph> g(new nd_graph);
    std::string err;
    if (nd::csr_from_edges(*g, n_vertices, (size_t)n_edges, src, dst, weight, &err) != 0) return fail(err);
    *out = g.release();
    return 0;
  });
}

int nd_graph_from_csr(int32_t n_vertices, int64_t n_edges, const int32_t* row_ptr, const int32_t* col,
                      const float* weight, nd_graph** out) {
  return guarded([&]() -> int {
    if (!out || !row_ptr || (n_edges > 0 && !col)) return fail("bad argument");
    std::unique_ptr<nd_graph> g(new nd_graph);
    std::string err;
    if (nd::csr_from_arrays(*g, n_vertices, n_edges, row_ptr, col, weight, &err) != 0) return fail(err);
    *out = g.release();
    return 0;
  });
}

int nd_graph_rmat(int scale, int edge_factor, double a, double b, double c, uint64_t seed, int symmetrise,
                  nd_graph** out) {
  return guarded([&]() -> int {
    if (!out) return fail("null out");
    std::unique_ptr<nd_graph> g(new nd_graph);
    std::string err;
    if (nd::generate_rmat(*g, scale, edge_factor, a, b, c, seed, symmetrise != 0, &err) != 0) return fail(err);
    *out = g.release();
    return 0;
  });
}

int nd_graph_chung_lu(int32_t n_vertices, int64_t n_edges, double exponent, uint64_t seed, nd_graph** out) {
  return guarded([&]() -> int {
    if (!out) return fail("null out");
    std::unique_ptr<nd_graph> g(new nd_graph);
    std::string err;
    if (nd::generate_chung_lu(*g, n_vertices, n_edges, exponent, seed, &err) != 0) return fail(err);
    *out = g.release();
    return 0;
  });
}

int32_t nd_graph_num_vertices(const nd_graph* g) { return g ? g->get_n_vertices() : 0; }
int64_t nd_graph_num_edges(const nd_graph* g) { return g ? (int64_t)g->col.size() : 0; }
const int32_t* nd_graph_row_ptr(const nd_graph* g) { return g ? g->row_ptr.data() : nullptr; }
const int32_t* nd_graph_col(const nd_graph* g) { return g ? g->col.data() : nullptr; }
const float* nd_graph_weight(const nd_graph* g) { return g ? g->weight.data() : nullptr; }
const float* nd_graph_max_weight(const nd_graph* g) { return g ? g->max_weight.data() : nullptr; }
void nd_graph_free(nd_graph* g) { delete g; }

// ---- sampler --------------------------------------------------------------------------

int nd_sampler_create(const char* app_name, nd_sampler** out) {
  return guarded([&]() -> int {
    if (!app_name || !out) return fail("null argument");
    AppEntry app;
    if (!find_app(app_name, &app)) return fail(std::string("unknown app '") + app_name + "'");
    std::unique_ptr<nd_sampler> s(new nd_sampler);
    s->engine.reset((nd::EngineBase*)app.make(app.name));
    if (!s->engine) return fail(std::string("the factory of app '") + app_name + "' returned no engine");
    *out = s.release();
    return 0;
  });
}

int nd_sampler_set_graph(nd_sampler* s, const nd_graph* g) {
  return guarded([&]() -> int {
    if (!s || !g) return fail("null argument");
    int n_devices = 0;
    if (hipGetDeviceCount(&n_devices) != hipSuccess || n_devices < 1) return fail("no HIP device available");
    s->graph = g;
    {
      // the address of nd_sort_pairs_noalloc's working array on this device, asked for here so
      // that a later first call of it under graph capture has nothing left to set up
      uint32_t* unused = nullptr;
      (void)scratch_on_current_device(&unused);
    }
    const int rc = s->engine->set_graph(g);
    return rc == 0 ? 0 : fail(s->engine->last_error, rc);
  });
}

int nd_sampler_alloc(nd_sampler* s, uint64_t seed) {
  return guarded([&]() -> int {
    if (!s) return fail("null sampler");
    const int rc = s->engine->alloc(seed);
    return rc == 0 ? 0 : fail(s->engine->last_error, rc);
  });
}

int nd_sampler_do_transit_parallel(nd_sampler* s, int enable_load_balancing) {
  return guarded([&]() -> int {
    if (!s) return fail("null sampler");
    const int rc = s->engine->sample(enable_load_balancing ? nd::kTransitParallelLoadBalanced : nd::kTransitParallel);
    return rc == 0 ? 0 : fail(s->engine->last_error, rc);
  });
}

int nd_sampler_do_sample_parallel(nd_sampler* s) {
  return guarded([&]() -> int {
    if (!s) return fail("null sampler");
    const int rc = s->engine->sample(nd::kSampleParallel);
    return rc == 0 ? 0 : fail(s->engine->last_error, rc);
  });
}

int nd_sampler_get_final_samples(nd_sampler* s, const int32_t** data, int64_t* length) {
  return guarded([&]() -> int {
    if (!s || !data || !length) return fail("null argument");
    const int rc = s->engine->fetch_final_samples();
    if (rc != 0) return fail(s->engine->last_error, rc);
    *data = s->engine->hFinalSamples.data();
    *length = (int64_t)s->engine->hFinalSamples.size();
    return 0;
  });
}

int nd_sampler_final_sample_size(const nd_sampler* s) { return s ? s->engine->final_sample_size() : -1; }
int64_t nd_sampler_num_samples(const nd_sampler* s) { return s ? s->engine->num_samples() : -1; }

int nd_sampler_initial_contents(const nd_sampler* s, const int32_t** data, int64_t* length) {
  if (!s || !data || !length) return fail("null argument");
  *data = s->engine->initialContents.data();
  *length = (int64_t)s->engine->initialContents.size();
  return 0;
}

int32_t nd_sampler_invalid_vertex(const nd_sampler* s) { return s ? s->engine->invalid_vertex() : -1; }
int nd_sampler_max_bits(const nd_sampler* s) { return s ? s->engine->max_bits() : -1; }
int nd_sampler_steps(const nd_sampler* s) { return s ? s->engine->steps() : -1; }
int nd_sampler_step_size(const nd_sampler* s, int step) {
  return s && step >= 0 && step < s->engine->steps() ? s->engine->step_size(step) : -1;
}
int nd_sampler_initial_sample_size(const nd_sampler* s) { return s ? s->engine->initial_sample_size() : -1; }
int nd_sampler_sampling_type(const nd_sampler* s) { return s ? s->engine->sampling_type() : -1; }

int64_t nd_sampler_sample_state_bytes(const nd_sampler* s) { return s ? (int64_t)s->engine->sample_state_bytes() : -1; }

int nd_sampler_get_sample_states(nd_sampler* s, void* dst, int64_t bytes) {
  return guarded([&]() -> int {
    if (!s || !dst) return fail("null argument");
    const int rc = s->engine->fetch_sample_states(dst, (size_t)bytes);
    return rc == 0 ? 0 : fail(s->engine->last_error, rc);
  });
}

int nd_sampler_set_inversion_period(nd_sampler* s, int period) {
  if (!s) return fail("null sampler");
  if (period < 0) return fail("the inversion period is 0 (engine decides) or positive");
  s->engine->inversion_period = period;
  return 0;
}

int nd_sampler_set_launch_graph(nd_sampler* s, int mode) {
  if (!s) return fail("null sampler");
  if (mode != 0 && mode != 1) return fail("launch graph mode is 0 (off) or 1 (on)");
  s->engine->launch_graph = mode;
  return 0;
}

int nd_sampler_set_profiling(nd_sampler* s, int on) {
  if (!s) return fail("null sampler");
  s->engine->profiling = on != 0;
  return 0;
}

int nd_sampler_phase_times(const nd_sampler* s, float out[12]) {
  if (!s || !out) return fail("null argument");
  const nd::PhaseTimes& t = s->engine->times;
  out[0] = t.end_to_end; out[1] = t.inversion; out[2] = t.load_balancing; out[3] = t.flat_kernel;
  out[4] = t.workgroup_kernel; out[5] = (float)t.flat_launches; out[6] = (float)t.workgroup_launches;
  out[7] = (float)t.sort_launches;
  out[8] = t.assemble;
  out[9] = t.distinct;
  out[10] = t.neighborhood;
  out[11] = (float)t.neighborhood_launches;
  return 0;
}

int nd_sampler_get_adjacency(nd_sampler* s, const int32_t** rows, const int32_t** cols, int64_t* n_edges,
                             const uint32_t** list_start, int64_t* n_samples) {
  return guarded([&]() -> int {
    if (!s || !rows || !cols || !n_edges || !list_start || !n_samples) return fail("null argument");
    const int rc = s->engine->fetch_adjacency();
    if (rc != 0) return fail(s->engine->last_error, rc);
    *rows = s->engine->hListRows.data();
    *cols = s->engine->hListCols.data();
    *n_edges = (int64_t)s->engine->hListRows.size();
    *list_start = s->engine->hListStart.data();
    *n_samples = s->engine->num_samples();
    return 0;
  });
}

int nd_sampler_distinct(nd_sampler* s) {
  return guarded([&]() -> int {
    if (!s) return fail("null sampler");
    const int rc = s->engine->distinct();
    return rc == 0 ? 0 : fail(s->engine->last_error, rc);
  });
}

int nd_sampler_get_distinct_counts(const nd_sampler* s, const int32_t** data, int64_t* length) {
  if (!s || !data || !length) return fail("null argument");
  *data = s->engine->hDistinctCounts.data();
  *length = (int64_t)s->engine->hDistinctCounts.size();
  return 0;
}

int64_t nd_sampler_counter(const nd_sampler* s, int which) { return s ? s->engine->counter(which) : 0; }

int nd_check_sampled_vertices(const nd_graph* g, int n_steps, const int32_t* step_sizes, int initial_size,
                              int collective, int64_t n_samples, const int32_t* initial,
                              const int32_t* final_samples, int32_t invalid) {
  return guarded([&]() -> int {
    if (!g || !step_sizes || n_steps < 1 || initial_size < 1 || n_samples < 0 ||
        (n_samples > 0 && (!initial || !final_samples)))
      return fail("bad argument");
    nd::SampleShape shape;
    shape.step_size.assign(step_sizes, step_sizes + n_steps);
    shape.initial_size = initial_size;
    shape.collective = collective != 0;
    std::string report;
    if (nd::check_sampled_vertices(*g, shape, n_samples, initial, final_samples, invalid, &report)) return 1;
    g_error = report;
    return 0;
  });
}

int nd_sampler_check_results(nd_sampler* s, int* ok) {
  return guarded([&]() -> int {
    if (!s || !ok) return fail("null argument");
    if (!s->graph) return fail("no graph set");
    nd::EngineBase& e = *s->engine;
    // the rule "adjacent to a vertex of the previous step" presumes that the previous step's
    // samples are the transits (the reference checks its MultiRW app with a rule of its own,
    // src/tests/multiGPU/multirw.cu:12-137, against the walkers left in the sample state)
    if (e.has_explicit_transits()) return fail("no validator for apps that choose their own transits");
    const int rc = e.fetch_final_samples();
    if (rc != 0) return fail(e.last_error, rc);
    nd::SampleShape shape;
    for (int k = 0; k < e.steps(); ++k) shape.step_size.push_back(e.step_size(k));
    shape.initial_size = e.initial_sample_size();
    shape.collective = e.sampling_type() == SamplingType::CollectiveNeighborhood;
    std::string report;
    bool pass;
    // a layer-wise app whose sample state is the per-layer adjacency matrix
    // {len[L], row[L][B*B], col[L][B*B], val[L][B*B]} records edges instead of sampling along them
    if (e.lists_edges()) {
      const int rc2 = e.fetch_adjacency();
      if (rc2 != 0) return fail(e.last_error, rc2);
      pass = nd::check_subgraph_edge_lists(*s->graph, e.num_samples(), shape.initial_size, e.initialContents.data(),
                                           e.hListStart.data(), e.hListRows.data(), e.hListCols.data(), &report);
      *ok = pass ? 1 : 0;
      if (!pass) g_error = report;
      return 0;
    }
    const size_t layers = shape.step_size.size(), cells = (size_t)shape.step_size[0] * shape.step_size[0];
    const size_t matrix_ints = layers + 3 * layers * cells;
    if (shape.collective && e.sample_state_bytes() == sizeof(int32_t) * matrix_ints * (size_t)e.num_samples()) {
      std::vector<int32_t> states((size_t)e.num_samples() * matrix_ints);
      const int rc2 = e.fetch_sample_states(states.data(), states.size() * sizeof(int32_t));
      if (rc2 != 0) return fail(e.last_error, rc2);
      pass = nd::check_layer_adjacency_matrix(*s->graph, shape, e.num_samples(), e.initialContents.data(),
                                              e.hFinalSamples.data(), states.data() + layers,
                                              states.data() + layers + layers * cells, matrix_ints, e.invalid_vertex(),
                                              &report);
    } else {
      pass = nd::check_sampled_vertices(*s->graph, shape, e.num_samples(), e.initialContents.data(),
                                        e.hFinalSamples.data(), e.invalid_vertex(), &report);
    }
    *ok = pass ? 1 : 0;
    if (!pass) g_error = report;
    return 0;
  });
}

void nd_sampler_free_device(nd_sampler* s) {
  if (s) s->engine->free_device();
}

void nd_sampler_destroy(nd_sampler* s) { delete s; }

// ---- module-level functions ---------------------------------------------------------------

void nd_free_device_memory(void) {
  if (g_module_sampler) nd_sampler_destroy(g_module_sampler);
  g_module_sampler = nullptr;
  if (g_module_graph) nd_graph_free(g_module_graph);
  g_module_graph = nullptr;
}

int nd_init_sampling(const char* app_name, const char* graph_path, uint64_t seed) {
  return guarded([&]() -> int {
    nd_free_device_memory();
    int rc = nd_graph_load(graph_path, "edge-list", "binary", &g_module_graph);
    if (rc != 0) return rc;
    rc = nd_sampler_create(app_name, &g_module_sampler);
    if (rc == 0) rc = nd_sampler_set_graph(g_module_sampler, g_module_graph);
    if (rc == 0) rc = nd_sampler_alloc(g_module_sampler, seed);
    if (rc != 0) {
      const std::string keep = g_error;
      nd_free_device_memory();
      g_error = keep;
    }
    return rc;
  });
}

int nd_init_sampling_from_csr(const char* app_name, int32_t n_vertices, int64_t n_edges, const int32_t* row_ptr,
                              const int32_t* col, const float* weight, uint64_t seed) {
  return guarded([&]() -> int {
    nd_free_device_memory();
    int rc = nd_graph_from_csr(n_vertices, n_edges, row_ptr, col, weight, &g_module_graph);
    if (rc != 0) return rc;
    rc = nd_sampler_create(app_name, &g_module_sampler);
    if (rc == 0) rc = nd_sampler_set_graph(g_module_sampler, g_module_graph);
    if (rc == 0) rc = nd_sampler_alloc(g_module_sampler, seed);
    if (rc != 0) {
      const std::string keep = g_error;
      nd_free_device_memory();
      g_error = keep;
    }
    return rc;
  });
}

int nd_sample(void) {
  if (!g_module_sampler) return fail("sample() before initSampling()");
  return nd_sampler_do_transit_parallel(g_module_sampler, 1);
}

int64_t nd_final_sample_length(void) {
  return g_module_sampler ? (int64_t)g_module_sampler->engine->hFinalSamples.size() : 0;
}

const int32_t* nd_final_samples_array(void) {
  if (!g_module_sampler) { fail("finalSamplesArray() before initSampling()"); return nullptr; }
  const int32_t* data = nullptr;
  int64_t len = 0;
  if (nd_sampler_get_final_samples(g_module_sampler, &data, &len) != 0) return nullptr;
  return data;
}

// ---- building blocks ------------------------------------------------------------------------

int nd_philox_fill_uniform(uint64_t seed, uint32_t step, uint64_t first_slot, int64_t n_slots, int draws_per_slot,
                           float* out) {
  return nd_philox_fill_step(seed, step, 1, first_slot, n_slots, draws_per_slot, out);
}

int nd_philox_fill_step(uint64_t seed, uint32_t step, int step_size, uint64_t first_slot, int64_t n_slots,
                        int draws_per_slot, float* out) {
  return guarded([&]() -> int {
    if (step_size < 1) return fail("bad argument");
    if (n_slots < 0 || draws_per_slot < 1 || (n_slots > 0 && !out)) return fail("bad argument");
    if (n_slots == 0) return 0;
    DeviceBuffer d;
    const size_t bytes = sizeof(float) * (size_t)n_slots * draws_per_slot;
    CAPI_HIP(d.alloc(bytes));
    philox_fill_kernel<<<dim3((unsigned)((n_slots + 255) / 256)), dim3(256), 0, 0>>>(seed, step, first_slot,
                                                                                    (size_t)n_slots, draws_per_slot,
                                                                                    step_size > 1 ? 1 : 0, d.as<float>());
    CAPI_HIP(hipGetLastError());
    CAPI_HIP(hipMemcpy(out, d.p, bytes, hipMemcpyDeviceToHost));
    return 0;
  });
}

int nd_sort_pairs(const int32_t* keys, const int32_t* vals, int64_t n, int key_bits, int32_t* keys_out,
                  int32_t* vals_out) {
  return guarded([&]() -> int {
    if (n < 0 || key_bits < 1 || key_bits > 32 || (n > 0 && (!keys || !keys_out || !vals_out)))
      return fail("bad argument");
    if (n == 0) return 0;
    if (n >= (int64_t)1 << 31) return fail("too many pairs");
    const nd::SortPlan plan = nd::make_sort_plan((size_t)n, key_bits);
    DeviceBuffer k_in, v_in, k_a, v_a, k_b, v_b, hist, totals;
    const size_t bytes = sizeof(uint32_t) * (size_t)n;
    CAPI_HIP(k_in.alloc(bytes));
    CAPI_HIP(k_a.alloc(bytes));
    CAPI_HIP(v_a.alloc(bytes));
    CAPI_HIP(k_b.alloc(bytes));
    CAPI_HIP(v_b.alloc(bytes));
    CAPI_HIP(hist.alloc(sizeof(uint32_t) * plan.hist_elems));
    CAPI_HIP(totals.alloc(sizeof(uint32_t) * plan.scratch_elems));
    CAPI_HIP(hipMemcpy(k_in.p, keys, bytes, hipMemcpyHostToDevice));
    if (vals) {
      CAPI_HIP(v_in.alloc(bytes));
      CAPI_HIP(hipMemcpy(v_in.p, vals, bytes, hipMemcpyHostToDevice));
    }
    uint32_t *k_sorted = nullptr, *v_sorted = nullptr;
    CAPI_HIP(nd::radix_sort_pairs(plan, k_in.as<uint32_t>(), vals ? v_in.as<uint32_t>() : nullptr, k_a.as<uint32_t>(),
                                  v_a.as<uint32_t>(), k_b.as<uint32_t>(), v_b.as<uint32_t>(), hist.as<uint32_t>(),
                                  totals.as<uint32_t>(), 0, &k_sorted, &v_sorted));
    CAPI_HIP(hipDeviceSynchronize());
    CAPI_HIP(hipMemcpy(keys_out, k_sorted, bytes, hipMemcpyDeviceToHost));
    CAPI_HIP(hipMemcpy(vals_out, v_sorted, bytes, hipMemcpyDeviceToHost));
    return 0;
  });
}

int nd_sort_pairs_noalloc(const int32_t* d_keys, const int32_t* d_vals, int64_t n, int key_bits, int32_t* d_keys_out,
                          int32_t* d_vals_out, void* stream) {
  return guarded([&]() -> int {
    if (n < 0 || key_bits < 1 || key_bits > 32 || (n > 0 && (!d_keys || !d_keys_out || !d_vals_out)))
      return fail("bad argument");
    if ((uint64_t)n > kNoAllocMaxPairs)
      return fail("nd_sort_pairs_noalloc sorts at most " + std::to_string(kNoAllocMaxPairs) + " pairs, " +
                  std::to_string(n) + " given (use nd_sort_pairs)", -2);
    if (n == 0) return 0;
    {
      // no array of the call may share a byte with another one it is written while read:
      // the outputs with each other and with the inputs
      const size_t bytes = sizeof(int32_t) * (size_t)n;
      auto overlap = [bytes](const void* a, const void* b) {
        const uintptr_t x = (uintptr_t)a, y = (uintptr_t)b;
        return a && b && x < y + bytes && y < x + bytes;
      };
      if (overlap(d_keys_out, d_vals_out) || overlap(d_keys_out, d_keys) || overlap(d_keys_out, d_vals) ||
          overlap(d_vals_out, d_keys) || overlap(d_vals_out, d_vals))
        return fail("the sort is not in place: input and output arrays must not overlap", -3);
    }
    uint32_t* work = nullptr;
    CAPI_HIP(scratch_on_current_device(&work));
    const nd::SortPlan plan = nd::make_sort_plan((size_t)n, key_bits);
    // the digit passes alternate between the caller's output arrays and the scratch side, in
    // the order that makes the last pass land in the output arrays
    const bool first_to_out = plan.passes % 2 == 1;
    nd::SortJob job;
    job.keys_in = (const uint32_t*)d_keys;
    job.vals_in = (const uint32_t*)d_vals;
    job.keys_a = first_to_out ? (uint32_t*)d_keys_out : work + kNoAllocKeysAt;
    job.vals_a = first_to_out ? (uint32_t*)d_vals_out : work + kNoAllocValsAt;
    job.keys_b = first_to_out ? work + kNoAllocKeysAt : (uint32_t*)d_keys_out;
    job.vals_b = first_to_out ? work + kNoAllocValsAt : (uint32_t*)d_vals_out;
    // every word of the digit table and the totals that a pass reads, the pass has written
    // before: nothing of the previous call's contents is used and nothing needs clearing
    job.hist = work + kNoAllocHistAt;
    job.scratch = work + kNoAllocTotalsAt;
    CAPI_HIP(nd::radix_sort(plan, job, (hipStream_t)stream));
    if (job.keys_sorted != (uint32_t*)d_keys_out) return fail("internal error: result outside the output arrays");
    return 0;
  });
}

int nd_load_balancing_thresholds(int32_t out[3]) {
  if (!out) return fail("null argument");
  out[0] = (int32_t)nd::kWorkgroupWork;
  out[1] = (int32_t)nd::kChunkOutputs;
  out[2] = (int32_t)nd::kCacheEdges;
  return 0;
}

// ---- measurement: what the memory system gives independent random 8-byte reads --------------

int nd_measure_gather_rate_shaped(int64_t table_bytes, int reads_in_flight, int workgroup_lanes,
                                  double* requests_per_s) {
  return guarded([&]() -> int {
    if (!requests_per_s || table_bytes < 4096 || table_bytes > (1ll << 35) || (table_bytes & (table_bytes - 1)))
      return fail("table_bytes must be a power of two between 4 KiB and 32 GiB");
    if (reads_in_flight != 1 && reads_in_flight != 2 && reads_in_flight != 4 && reads_in_flight != 8)
      return fail("reads_in_flight must be 1, 2, 4 or 8");
    if (workgroup_lanes != 64 && workgroup_lanes != 256) return fail("workgroup_lanes must be 64 or 256");
    constexpr uint32_t kLanes = 1u << 22;
    const uint32_t rounds = 16u / (uint32_t)reads_in_flight < 2u ? 2u : 16u / (uint32_t)reads_in_flight;  // 16 reads per lane
    DeviceBuffer table, sink;
    CAPI_HIP(table.alloc((size_t)table_bytes));
    CAPI_HIP(sink.alloc(sizeof(uint32_t) * kLanes));
    CAPI_HIP(hipMemset(table.p, 1, (size_t)table_bytes));
    hipEvent_t begin = nullptr, end = nullptr;
    CAPI_HIP(hipEventCreate(&begin));
    hipError_t e = hipEventCreate(&end);
    float best_ms = 0.0f;
    const dim3 grid(kLanes / (uint32_t)workgroup_lanes), block((uint32_t)workgroup_lanes);
    const uint32_t mask = (uint32_t)(table_bytes / 8 - 1);
    for (int rep = 0; e == hipSuccess && rep < 3; ++rep) {  // the first launch warms the translation caches
      e = hipEventRecord(begin, nullptr);
      switch (reads_in_flight) {
        case 1: gather_rate_kernel<1><<<grid, block>>>(table.as<uint2>(), mask, rounds, sink.as<uint32_t>()); break;
        case 2: gather_rate_kernel<2><<<grid, block>>>(table.as<uint2>(), mask, rounds, sink.as<uint32_t>()); break;
        case 4: gather_rate_kernel<4><<<grid, block>>>(table.as<uint2>(), mask, rounds, sink.as<uint32_t>()); break;
        default: gather_rate_kernel<8><<<grid, block>>>(table.as<uint2>(), mask, rounds, sink.as<uint32_t>()); break;
      }
      if (e == hipSuccess) e = hipGetLastError();
      if (e == hipSuccess) e = hipEventRecord(end, nullptr);
      if (e == hipSuccess) e = hipEventSynchronize(end);
      float ms = 0.0f;
      if (e == hipSuccess) e = hipEventElapsedTime(&ms, begin, end);
      if (rep > 0 && (best_ms == 0.0f || ms < best_ms)) best_ms = ms;
    }
    (void)hipEventDestroy(begin);
    if (end) (void)hipEventDestroy(end);
    CAPI_HIP(e);
    *requests_per_s = (double)kLanes * rounds * reads_in_flight / ((double)best_ms / 1000.0);
    return 0;
  });
}

int nd_measure_gather_rate(int64_t table_bytes, double* requests_per_s) {
  return nd_measure_gather_rate_shaped(table_bytes, 2, 256, requests_per_s);
}

int nd_classify_runs(const int32_t* sorted_keys, int64_t n, const int32_t* degrees, int32_t n_vertices, int step_size,
                     int pairs_per_lane, int32_t* items, int64_t capacity, int64_t* n_items, uint8_t* taken,
                     int64_t counters[5]) {
  return guarded([&]() -> int {
    if (n < 0 || n_vertices < 1 || step_size < 1 || capacity < 1 || !degrees || !items || !n_items || !taken ||
        !counters || (n > 0 && !sorted_keys) || n >= (1ll << 31) || capacity >= (1ll << 31) ||
        (pairs_per_lane != 1 && pairs_per_lane != nd::kClassifyItemsLarge))
      return fail("bad argument");
    for (int64_t i = 0; i < n; ++i)
      if (sorted_keys[i] < 0 || sorted_keys[i] >= n_vertices || (i > 0 && sorted_keys[i] < sorted_keys[i - 1]))
        return fail("keys must be vertices in ascending order");
    std::vector<EdgePos_t> row_ptr((size_t)n_vertices + 1, 0);
    for (int32_t v = 0; v < n_vertices; ++v) {
      if (degrees[v] < 0) return fail("negative degree");
      row_ptr[(size_t)v + 1] = row_ptr[v] + degrees[v];
    }
    *n_items = 0;
    for (int i = 0; i < 5; ++i) counters[i] = 0;
    memset(taken, 0, (size_t)n_vertices);
    if (n == 0) return 0;
    DeviceBuffer d_keys, d_n, d_meta, d_rows, d_items, d_taken, d_balance;
    constexpr size_t kFoundWords = nd::kMaxSteps + 2;
    CAPI_HIP(d_keys.alloc(sizeof(uint32_t) * (size_t)n));
    CAPI_HIP(d_n.alloc(sizeof(uint32_t)));
    CAPI_HIP(d_meta.alloc(sizeof(nd::RunsMeta) * 2));
    CAPI_HIP(d_rows.alloc(sizeof(EdgePos_t) * row_ptr.size()));
    CAPI_HIP(d_items.alloc(sizeof(nd::WorkItem) * (size_t)capacity));
    CAPI_HIP(d_taken.alloc(sizeof(uint32_t) * (size_t)n_vertices));
    constexpr size_t kCounterBytes = sizeof(nd::ClassCounters) * nd::kCounterCopies;
    CAPI_HIP(d_balance.alloc(sizeof(uint32_t) * kFoundWords + kCounterBytes));
    const uint32_t n32 = (uint32_t)n;
    CAPI_HIP(hipMemcpy(d_keys.p, sorted_keys, sizeof(uint32_t) * (size_t)n, hipMemcpyHostToDevice));
    CAPI_HIP(hipMemcpy(d_n.p, &n32, sizeof(n32), hipMemcpyHostToDevice));
    CAPI_HIP(hipMemcpy(d_rows.p, row_ptr.data(), sizeof(EdgePos_t) * row_ptr.size(), hipMemcpyHostToDevice));
    nd::RunsMeta fresh[2] = {};
    fresh[0].stamp = 1;  // the stamp that marks the transits taken at this (the only) step
    CAPI_HIP(hipMemcpy(d_meta.p, fresh, sizeof(fresh), hipMemcpyHostToDevice));
    CAPI_HIP(hipMemset(d_taken.p, 0, sizeof(uint32_t) * (size_t)n_vertices));
    CAPI_HIP(hipMemset(d_balance.p, 0, sizeof(uint32_t) * kFoundWords + kCounterBytes));
    nd::RunsMeta* meta = d_meta.as<nd::RunsMeta>();
    nd::ClassCounters* d_counters = (nd::ClassCounters*)(d_balance.as<uint32_t>() + kFoundWords);
    if (pairs_per_lane == 1) {
      nd::classify_run_tails<1><<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, 0>>>(
          d_keys.as<uint32_t>(), d_n.as<uint32_t>(), meta, meta + 1, d_rows.as<EdgePos_t>(), (uint32_t)step_size,
          d_items.as<nd::WorkItem>(), (uint32_t)capacity, d_taken.as<uint32_t>(), d_counters, d_balance.as<uint32_t>(), 1u);
    } else {
      const int64_t per_block = nd::kClassifyThreadsLarge * nd::kClassifyItemsLarge;
      nd::classify_run_tails<nd::kClassifyItemsLarge, nd::kClassifyThreadsLarge>
          <<<dim3((unsigned)((n + per_block - 1) / per_block)), dim3(nd::kClassifyThreadsLarge), 0, 0>>>(
          d_keys.as<uint32_t>(), d_n.as<uint32_t>(), meta, meta + 1, d_rows.as<EdgePos_t>(), (uint32_t)step_size,
          d_items.as<nd::WorkItem>(), (uint32_t)capacity, d_taken.as<uint32_t>(), d_counters, d_balance.as<uint32_t>(), 1u);
    }
    CAPI_HIP(hipGetLastError());
    CAPI_HIP(hipDeviceSynchronize());
    nd::RunsMeta h;
    nd::ClassCounters copies[nd::kCounterCopies], c = nd::ClassCounters();
    CAPI_HIP(hipMemcpy(&h, meta, sizeof(h), hipMemcpyDeviceToHost));
    CAPI_HIP(hipMemcpy(copies, d_counters, sizeof(copies), hipMemcpyDeviceToHost));
    for (const nd::ClassCounters& one : copies) {
      c.sorted_pairs += one.sorted_pairs;
      c.workgroup_pairs += one.workgroup_pairs;
      c.split_pairs += one.split_pairs;
      c.refused_pairs += one.refused_pairs;
      c.work_items += one.work_items;
    }
    // the kernel counts every item it wants; those beyond the capacity were not written
    *n_items = h.n_chunks;
    const int64_t written = h.n_chunks < capacity ? (int64_t)h.n_chunks : capacity;
    std::vector<nd::WorkItem> records((size_t)written);
    CAPI_HIP(hipMemcpy(records.data(), d_items.p, sizeof(nd::WorkItem) * (size_t)written, hipMemcpyDeviceToHost));
    for (int64_t i = 0; i < written; ++i) {
      const nd::WorkItem& r = records[(size_t)i];
      // what the item says of its transit is what the caller's arrays say
      if (r.transit != sorted_keys[r.first_pair] || r.begin != row_ptr[(size_t)r.transit] || r.n_edges != degrees[r.transit])
        return fail("internal error: a work item does not describe its transit");
      items[2 * i] = (int32_t)r.first_pair;
      items[2 * i + 1] = (int32_t)r.n_pairs;
    }
    std::vector<uint32_t> stamps((size_t)n_vertices);
    CAPI_HIP(hipMemcpy(stamps.data(), d_taken.p, sizeof(uint32_t) * stamps.size(), hipMemcpyDeviceToHost));
    for (int32_t v = 0; v < n_vertices; ++v) taken[v] = stamps[(size_t)v] == fresh[0].stamp ? 1 : 0;
    counters[0] = (int64_t)c.sorted_pairs;
    counters[1] = (int64_t)c.workgroup_pairs;
    counters[2] = (int64_t)c.split_pairs;
    counters[3] = (int64_t)c.refused_pairs;
    counters[4] = (int64_t)c.work_items;
    return 0;
  });
}

int nd_unique_transits(const int32_t* sorted_keys, int64_t n, int32_t invalid, int32_t* uniq, int32_t* counts,
                       int32_t* offsets, int64_t* n_runs, int64_t* n_valid) {
  return guarded([&]() -> int {
    if (n < 0 || !n_runs || !n_valid || (n > 0 && (!sorted_keys || !uniq || !counts || !offsets)))
      return fail("bad argument");
    *n_runs = 0;
    *n_valid = 0;
    if (n == 0) return 0;
    const size_t bytes = sizeof(uint32_t) * (size_t)n;
    DeviceBuffer keys, run_key, run_start, run_count, meta, scan_tmp;
    CAPI_HIP(keys.alloc(bytes));
    CAPI_HIP(run_key.alloc(bytes));
    CAPI_HIP(run_start.alloc(bytes + sizeof(uint32_t)));
    CAPI_HIP(run_count.alloc(bytes));
    CAPI_HIP(meta.alloc(sizeof(nd::RunsMeta)));
    CAPI_HIP(scan_tmp.alloc(sizeof(uint32_t) * nd::runs_scratch_elems((size_t)n)));
    CAPI_HIP(hipMemcpy(keys.p, sorted_keys, bytes, hipMemcpyHostToDevice));
    CAPI_HIP(nd::find_transit_runs(keys.as<uint32_t>(), (size_t)n, (uint32_t)invalid, run_key.as<uint32_t>(),
                                   run_start.as<uint32_t>(), meta.as<nd::RunsMeta>(), scan_tmp.as<uint32_t>(), 0));
    run_counts_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, 0>>>(run_start.as<uint32_t>(),
                                                                             meta.as<nd::RunsMeta>(),
                                                                             run_count.as<uint32_t>());
    CAPI_HIP(hipGetLastError());
    nd::RunsMeta h;
    CAPI_HIP(hipMemcpy(&h, meta.p, sizeof(h), hipMemcpyDeviceToHost));
    *n_runs = h.n_runs;
    *n_valid = h.n_valid;
    if (h.n_runs) {
      CAPI_HIP(hipMemcpy(uniq, run_key.p, sizeof(uint32_t) * h.n_runs, hipMemcpyDeviceToHost));
      CAPI_HIP(hipMemcpy(counts, run_count.p, sizeof(uint32_t) * h.n_runs, hipMemcpyDeviceToHost));
      CAPI_HIP(hipMemcpy(offsets, run_start.p, sizeof(uint32_t) * h.n_runs, hipMemcpyDeviceToHost));
    }
    return 0;
  });
}

int nd_collective_neighborhood(const nd_graph* g, const int32_t* transits, int64_t n_samples,
                               int32_t transits_per_sample, int32_t invalid, int32_t* sizes, int32_t* offsets,
                               int32_t* cols, float* weights, int64_t capacity, int32_t* row_offsets) {
  return guarded([&]() -> int {
    if (!g || !transits || n_samples < 1 || transits_per_sample < 1 || !sizes || !offsets || !cols || !weights ||
        !row_offsets || (uint32_t)transits_per_sample > nd::kMaxLayerTransits || n_samples >= (1ll << 31))
      return fail("bad argument");
    const uint32_t S = (uint32_t)n_samples;
    const size_t n_tr = (size_t)S * transits_per_sample;
    // the kernels index the row extents with every transit that is not a "no vertex" value
    uint64_t entries = 0;
    for (size_t i = 0; i < n_tr; ++i) {
      const int32_t t = transits[i];
      if (t == invalid || t == -1) continue;
      if (!g->has_vertex(t)) return fail("transit " + std::to_string(t) + " is not a vertex of the graph");
      entries += (uint64_t)g->n_edges_for_vertex(t);
    }
    if (entries >= (1ull << 31)) return fail("collective neighbourhoods of more than 2^31 entries");
    if ((int64_t)entries > capacity) return fail("collective neighbourhood larger than the capacity given");
    nd::DeviceGraph dg;
    std::string err;
    if (!dg.upload(g, false, false, &err)) return fail(err);
    DeviceBuffer d_tr, d_sizes, d_offsets, d_scratch, d_cols, d_weights, d_rows;
    CAPI_HIP(d_tr.alloc(sizeof(int32_t) * n_tr));
    CAPI_HIP(d_sizes.alloc(sizeof(uint32_t) * ((size_t)S + 1)));
    CAPI_HIP(d_offsets.alloc(sizeof(uint32_t) * ((size_t)S + 1)));
    CAPI_HIP(d_scratch.alloc(sizeof(uint32_t) * nd::scan_scratch_elems((size_t)S + 1)));
    CAPI_HIP(d_rows.alloc(sizeof(uint32_t) * n_tr));
    CAPI_HIP(hipMemcpy(d_tr.p, transits, sizeof(int32_t) * n_tr, hipMemcpyHostToDevice));
    CAPI_HIP(hipMemset(d_sizes.p, 0, sizeof(uint32_t) * ((size_t)S + 1)));
    nd::TransitView tv{d_tr.as<int32_t>(), (uint32_t)transits_per_sample, (uint32_t)transits_per_sample};
    nd::collective_sizes<<<dim3((S + 3) / 4), dim3(256), 0, 0>>>(dg.view, tv, S, invalid, d_sizes.as<uint32_t>());
    CAPI_HIP(nd::exclusive_scan_u32(d_sizes.as<uint32_t>(), d_offsets.as<uint32_t>(), (size_t)S + 1,
                                    d_scratch.as<uint32_t>(), 0));
    CAPI_HIP(hipMemcpy(sizes, d_sizes.p, sizeof(uint32_t) * S, hipMemcpyDeviceToHost));
    CAPI_HIP(hipMemcpy(offsets, d_offsets.p, sizeof(uint32_t) * ((size_t)S + 1), hipMemcpyDeviceToHost));
    const int64_t total = offsets[S];
    if (total > capacity) return fail("collective neighbourhood larger than the capacity given");
    CAPI_HIP(d_cols.alloc(sizeof(int32_t) * (size_t)total));
    CAPI_HIP(d_weights.alloc(sizeof(float) * (size_t)total));
    DeviceBuffer d_item_count, d_item_start;
    CAPI_HIP(d_item_count.alloc(sizeof(uint32_t) * ((size_t)S + 1)));
    CAPI_HIP(d_item_start.alloc(sizeof(uint32_t) * ((size_t)S + 1)));
    uint64_t n_items = 0;
    for (uint32_t i = 0; i < S; ++i) {
      const uint64_t items = ((uint64_t)(uint32_t)sizes[i] + nd::kBuildItemEntries - 1) / nd::kBuildItemEntries;
      n_items += items ? items : 1;
    }
    nd::build_item_counts<<<dim3((S + 1 + 255) / 256), dim3(256), 0, 0>>>(d_sizes.as<uint32_t>(), S,
                                                                         d_item_count.as<uint32_t>());
    CAPI_HIP(nd::exclusive_scan_u32(d_item_count.as<uint32_t>(), d_item_start.as<uint32_t>(), (size_t)S + 1,
                                    d_scratch.as<uint32_t>(), 0));
    nd::collective_build<<<dim3((unsigned)n_items), dim3(256), 0, 0>>>(
        dg.view, tv, invalid, d_offsets.as<uint32_t>(), d_item_start.as<uint32_t>(), S, d_cols.as<int32_t>(),
        d_weights.as<float>(), d_rows.as<uint32_t>());
    CAPI_HIP(hipGetLastError());
    CAPI_HIP(hipMemcpy(cols, d_cols.p, sizeof(int32_t) * (size_t)total, hipMemcpyDeviceToHost));
    CAPI_HIP(hipMemcpy(weights, d_weights.p, sizeof(float) * (size_t)total, hipMemcpyDeviceToHost));
    CAPI_HIP(hipMemcpy(row_offsets, d_rows.p, sizeof(uint32_t) * n_tr, hipMemcpyDeviceToHost));
    return 0;
  });
}

}  // extern "C"
