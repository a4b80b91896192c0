// C++ host API over the C ABI of libnextdoor_amd.so, under the names and template spellings of
// the reference's host API (src/libNextDoor.hpp:13-50; definitions in src/nextdoor.cu, the
// command line of src/main.cu).  Header only; link with -lnextdoor_amd.
//
//   NextDoorData<SampleType, App>, loadGraph(Graph&, file, type, format),
//   allocNextDoorDataOnGPU<SampleType, App>(csr, data), transferCSRToGPUs(data, csr),
//   doTransitParallelSampling<SampleType, App>(csr, data, lb), doSampleParallelSampling(csr, data),
//   getFinalSamples(data), getFinalSampleSize<App>(), freeDeviceData(data),
//   nextdoor<SampleType, App>(file, type, format, nruns, chk, print, kernelType, lb, checker),
//   appMain<SampleType, App>(argc, argv, checker), checkSampledVerticesResult<SampleType, App>.
//
// A caller written for the reference (src/tests/testBase.h:14-24, src/apps/khop/main.cu:23-27)
// compiles against this header.  How <SampleType, App> reaches an engine:
//   * an application compiled into the library is found by its registry name
//     (NextDoorAppName<App>, declared next to the App in the nd_apps_*.hpp headers, which
//     nextdoor_amd_apps.hpp includes): this works in a host-only translation unit (g++);
//   * any other App - the caller's own struct on the App contract - is instantiated on the
//     engine right here and registered on first use (nd_app_registry.hpp); that needs a device
//     compiler, i.e. the translation unit is built with hipcc, as the reference's are with nvcc.
// Failures return false / nullptr and leave the reason in nd_last_error(); nothing aborts.
#ifndef LIBNEXTDOOR_AMD_HPP
#define LIBNEXTDOOR_AMD_HPP

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <typeinfo>
#include <vector>

#include "nextdoor_amd.h"
#include "../nextdoor_amd/csrc/nd_contract.hpp"  // VertexID_t, EdgePos_t, CSR, NextDoorAppName; nd_graph is a CSR
#if defined(__HIPCC__) && !defined(ND_HOST_API_ONLY)
#include "../nextdoor_amd/csrc/nd_app_registry.hpp"
#endif

// What loadGraph fills besides returning the CSR (the reference keeps the vertex and edge
// lists here, src/graph.hpp:14-104; callers only ask for the counts, src/nextdoor.cu:3255-3256).
class Graph {
 public:
  struct Vertices {
    size_t count;
    size_t size() const { return count; }
  };
  EdgePos_t get_n_edges() const { return n_edges_; }
  Vertices get_vertices() const { return Vertices{n_vertices_}; }
  void set_counts(size_t n_vertices, EdgePos_t n_edges) {
    n_vertices_ = n_vertices;
    n_edges_ = n_edges;
  }

 private:
  size_t n_vertices_ = 0;
  EdgePos_t n_edges_ = 0;
};

struct GPUCSRPartition {  // src/csr.hpp:387-397: one per device; this build runs on one
  int device = 0;
};

// The host-visible members of NextDoorData a caller of the reference reads (src/libNextDoor.hpp:13-37),
// plus the sampler handle.  The per-device buffers of the reference live inside the library.
struct NextDoorDataByName {
  explicit NextDoorDataByName(const char* app, uint64_t seed = 42) : appName(app ? app : ""), seed(seed) {}
  ~NextDoorDataByName() {
    if (sampler) nd_sampler_destroy(sampler);
  }
  NextDoorDataByName(const NextDoorDataByName&) = delete;
  NextDoorDataByName& operator=(const NextDoorDataByName&) = delete;

  std::string appName;
  uint64_t seed;
  nd_sampler* sampler = nullptr;
  CSR* csr = nullptr;                       // the caller's graph; stays set after freeDeviceData
  bool graphOnDevice = false;
  std::vector<VertexID_t> hFinalSamples;    // libNextDoor.hpp:17
  std::vector<VertexID_t> initialContents;  // libNextDoor.hpp:18
  std::vector<int> devices;                 // libNextDoor.hpp:20
  std::vector<GPUCSRPartition> gpuCSRPartitions;  // libNextDoor.hpp:36
  VertexID_t INVALID_VERTEX = 0;            // libNextDoor.hpp:34
  int maxBits = 0;                          // libNextDoor.hpp:35
};

// Registry name of <SampleType, App>: the name the App carries when it is compiled into the
// library; else, under hipcc, the name under which this translation unit registers its own
// instantiation of the engine (once); else nullptr.
template <class SampleType, class App>
inline const char* nextDoorRegistryName() {
  if (NextDoorAppName<App>::name() != nullptr) return NextDoorAppName<App>::name();
#if defined(__HIPCC__) && !defined(ND_HOST_API_ONLY)
  static const std::string name = [] {
    std::string n = std::string("app:") + typeid(App).name() + ":" + typeid(SampleType).name();
    if (nd_register_app(n.c_str(), &nd::make_app_engine<SampleType, App>, nd::engine_abi()) != 0)
      fprintf(stderr, "nextdoor: %s\n", nd_last_error());
    return n;
  }();
  return name.c_str();
#else
  return nullptr;
#endif
}

template <class SampleType, typename App>
struct NextDoorData : NextDoorDataByName {
  NextDoorData() : NextDoorDataByName(nextDoorRegistryName<SampleType, App>()) {}
  // libNextDoor.hpp:16: one SampleType per sample.  After allocNextDoorDataOnGPU what
  // initializeSample / initialSample left in it (src/nextdoor.cu:1955-1963), after
  // getFinalSamples the state the sampling left on the device (src/nextdoor.cu:3226-3227);
  // the reference's checkers read it (src/check_results.cu:55, src/tests/singleGPU/multirw.cu:21).
  std::vector<SampleType> samples;
};

// Device -> data.samples.  False when the engine keeps a state of another size than
// sizeof(SampleType) per sample (the caller's SampleType is not the engine's).
template <class SampleType, typename App>
inline bool fetchSampleStates(NextDoorData<SampleType, App>& data) {
  if (!data.sampler) return false;
  const int64_t n = nd_sampler_num_samples(data.sampler);
  const int64_t bytes = nd_sampler_sample_state_bytes(data.sampler);
  data.samples.assign((size_t)(n > 0 ? n : 0), SampleType());
  if (bytes == 0) return true;  // a SampleType without members: nothing is kept on the device
  if (bytes != (int64_t)sizeof(SampleType) * n) return false;
  return nd_sampler_get_sample_states(data.sampler, (void*)data.samples.data(), bytes) == 0;
}

// loadGraph(graph, file, type, format), src/nextdoor.cu:1845-1891: nullptr on failure.
inline CSR* loadGraph(Graph& graph, const char* graph_file, const char* graph_type, const char* graph_format) {
  nd_graph* g = nullptr;
  if (nd_graph_load(graph_file, graph_type, graph_format, &g) != 0) {
    fprintf(stderr, "loadGraph: %s\n", nd_last_error());
    return nullptr;
  }
  graph.set_counts((size_t)nd_graph_num_vertices(g), (EdgePos_t)nd_graph_num_edges(g));
  return g;
}
inline CSR* loadGraph(const char* graph_file, const char* graph_type, const char* graph_format) {
  Graph graph;
  return loadGraph(graph, graph_file, graph_type, graph_format);
}
// The CSR* of this API is always a graph of the library's (loadGraph made it).
inline void freeGraph(CSR* csr) { nd_graph_free(static_cast<nd_graph*>(csr)); }

// transferCSRToGPUs(data, csr), src/nextdoor.cu:1893-1911.
inline std::vector<GPUCSRPartition> transferCSRToGPUs(NextDoorDataByName& data, CSR* csr) {
  std::vector<GPUCSRPartition> none;
  if (data.graphOnDevice && data.csr == csr) return std::vector<GPUCSRPartition>(1);
  if (data.appName.empty()) {
    fprintf(stderr, "nextdoor: this App is not compiled into libnextdoor_amd.so; build the caller with hipcc so that "
                    "the engine is instantiated for it\n");
    return none;
  }
  if (!data.sampler && nd_sampler_create(data.appName.c_str(), &data.sampler) != 0) return none;
  if (nd_sampler_set_graph(data.sampler, static_cast<nd_graph*>(csr)) != 0) return none;
  data.csr = csr;
  data.graphOnDevice = true;
  data.devices.assign(1, 0);
  return std::vector<GPUCSRPartition>(1);
}

// allocNextDoorDataOnGPU(csr, data), src/nextdoor.cu:1931-2086.  The reference allocates before
// it transfers the graph (src/nextdoor.cu:3262-3264); here the per-run buffers are sized against
// the graph on the device, so the graph is transferred first when the caller has not done so.
inline bool allocNextDoorDataOnGPU(CSR* csr, NextDoorDataByName& data) {
  if ((data.csr != csr || !data.graphOnDevice) && transferCSRToGPUs(data, csr).empty()) return false;
  if (nd_sampler_alloc(data.sampler, data.seed) != 0) return false;
  const VertexID_t* roots = nullptr;
  int64_t n = 0;
  if (nd_sampler_initial_contents(data.sampler, &roots, &n) != 0) return false;
  data.initialContents.assign(roots, roots + n);
  data.INVALID_VERTEX = nd_sampler_invalid_vertex(data.sampler);
  data.maxBits = nd_sampler_max_bits(data.sampler);
  return true;
}
template <class SampleType, typename App>
inline bool allocNextDoorDataOnGPU(CSR* csr, NextDoorData<SampleType, App>& data) {
  return allocNextDoorDataOnGPU(csr, static_cast<NextDoorDataByName&>(data)) && fetchSampleStates(data);
}

// doTransitParallelSampling(csr, data, enableLoadBalancing), src/nextdoor.cu:2191-3006: the
// sample -> transit map is inverted before every step.
inline bool doTransitParallelSampling(CSR*, NextDoorDataByName& data, bool enableLoadBalancing) {
  return data.sampler && nd_sampler_set_inversion_period(data.sampler, 1) == 0 &&
         nd_sampler_do_transit_parallel(data.sampler, enableLoadBalancing ? 1 : 0) == 0;
}
template <class SampleType, typename App>
inline bool doTransitParallelSampling(CSR* csr, NextDoorData<SampleType, App>& data, bool enableLoadBalancing) {
  return doTransitParallelSampling(csr, static_cast<NextDoorDataByName&>(data), enableLoadBalancing);
}

// doSampleParallelSampling(csr, data), src/nextdoor.cu:3009-3209: the reference's baseline
// mode, every sample's work in sample order: the engine never brings the pairs into transit
// order (it only drops the dead ones) and does no load balancing.  The samples are the same
// bytes either way.
inline bool doSampleParallelSampling(CSR*, NextDoorDataByName& data) {
  return data.sampler && nd_sampler_do_sample_parallel(data.sampler) == 0;
}
template <class SampleType, typename App>
inline bool doSampleParallelSampling(CSR* csr, NextDoorData<SampleType, App>& data) {
  return doSampleParallelSampling(csr, static_cast<NextDoorDataByName&>(data));
}

// getFinalSamples(data), src/nextdoor.cu:3211-3237.
inline std::vector<VertexID_t>& getFinalSamples(NextDoorDataByName& data) {
  const VertexID_t* p = nullptr;
  int64_t n = 0;
  if (data.sampler && nd_sampler_get_final_samples(data.sampler, &p, &n) == 0) data.hFinalSamples.assign(p, p + n);
  return data.hFinalSamples;
}

// ... and, with the template spelling, data.samples (src/nextdoor.cu:3226-3227).
template <class SampleType, typename App>
inline std::vector<VertexID_t>& getFinalSamples(NextDoorData<SampleType, App>& data) {
  getFinalSamples(static_cast<NextDoorDataByName&>(data));
  if (!fetchSampleStates(data)) fprintf(stderr, "getFinalSamples: %s\n", nd_last_error());
  return data.hFinalSamples;
}

// getFinalSampleSize<App>(), src/nextdoor.cu:1913-1929; by the data block, or by the App alone.
inline int getFinalSampleSize(const NextDoorDataByName& data) {
  return data.sampler ? nd_sampler_final_sample_size(data.sampler) : 0;
}
template <class App>
inline int getFinalSampleSize() {
  // the shape algebra of the App itself where the App is a complete type with steps() ...
  // ... every output slot of every step: an individual app's steps start from its
  // initialSampleSize transits (one for the reference's walk and k-hop apps)
  App app;
  const bool collective = app.samplingType() == CollectiveNeighborhood;
  long total = 0, per_step = collective ? 1 : (long)app.initialSampleSize(nullptr);
  for (int k = 0; k < app.steps(); ++k) {
    if (collective) per_step = app.stepSize(k); else per_step *= app.stepSize(k);
    total += per_step;
  }
  return (int)total;
}

// freeDeviceData(data), src/nextdoor.cu:2088-2115.
inline void freeDeviceData(NextDoorDataByName& data) {
  if (data.sampler) nd_sampler_free_device(data.sampler);
  data.graphOnDevice = false;
}

// checkSampledVerticesResult<SampleType, App>(data), src/check_results.cu:162-299: the checker
// the reference's per-transit apps hand to nextdoor().  Works on the host copies
// (data.hFinalSamples, data.initialContents, data.csr), so also after freeDeviceData.
inline bool checkSampledVerticesResult(NextDoorDataByName& data) {
  if (!data.sampler || !data.csr) return false;
  const int steps = nd_sampler_steps(data.sampler);
  std::vector<int32_t> sizes((size_t)(steps > 0 ? steps : 0));
  for (int k = 0; k < steps; ++k) sizes[(size_t)k] = nd_sampler_step_size(data.sampler, k);
  const int initial = nd_sampler_initial_sample_size(data.sampler);
  const int64_t n_samples = initial > 0 ? (int64_t)data.initialContents.size() / initial : 0;
  const int verdict = nd_check_sampled_vertices(static_cast<nd_graph*>(data.csr), steps, sizes.data(), initial,
                                                nd_sampler_sampling_type(data.sampler) == 1, n_samples,
                                                data.initialContents.data(), data.hFinalSamples.data(),
                                                data.INVALID_VERTEX);
  if (verdict != 1) fprintf(stderr, "%s\n", nd_last_error());
  return verdict == 1;
}
template <class SampleType, typename App>
inline bool checkSampledVerticesResult(NextDoorData<SampleType, App>& data) {
  return checkSampledVerticesResult(static_cast<NextDoorDataByName&>(data));
}

// The edge lists of the apps whose outputFormat() is AdjacencyMatrix on per-transit sampling
// (MVS, ClusterGCN; the reference reads dRowStorage / dColStorage at sample.posInStorage):
// sample i owns rows/cols[list_start[i] .. list_start[i + 1]).
inline bool getAdjacency(NextDoorDataByName& data, std::vector<VertexID_t>& rows, std::vector<VertexID_t>& cols,
                         std::vector<uint32_t>& list_start) {
  const int32_t *r = nullptr, *c = nullptr;
  const uint32_t* start = nullptr;
  int64_t n_edges = 0, n_samples = 0;
  if (!data.sampler || nd_sampler_get_adjacency(data.sampler, &r, &c, &n_edges, &start, &n_samples) != 0) return false;
  rows.assign(r, r + n_edges);
  cols.assign(c, c + n_edges);
  list_start.assign(start, start + n_samples + 1);
  return true;
}

// The body of nextdoor<>() (src/nextdoor.cu:3239-3306): load, allocate, sample nruns times,
// fetch, count the sampled (non-INVALID) vertices, free, then run the caller's check on the
// final samples.  kernelType: "TransitParallel" or "SampleParallel" (src/main.cu:19-21).
template <class Data, class CheckFn>
inline bool nextdoorRun(Data& data, const char* graph_file, const char* graph_type, const char* graph_format,
                        int nruns, bool chk_results, bool print_samples, const char* kernelType,
                        bool enableLoadBalancing, CheckFn checkResultsFunc) {
  Graph graph;
  CSR* csr = loadGraph(graph, graph_file, graph_type, graph_format);
  if (!csr) return false;
  printf("Graph has %d edges and %zu vertices \n", graph.get_n_edges(), graph.get_vertices().size());
  const bool transit_parallel = kernelType && strcmp(kernelType, "TransitParallel") == 0;
  const bool sample_parallel = kernelType && strcmp(kernelType, "SampleParallel") == 0;
  bool ok = transit_parallel || sample_parallel;  // the reference aborts on any other kernel type
  if (!ok) fprintf(stderr, "nextdoor: kernel type must be TransitParallel or SampleParallel\n");
  data.csr = csr;
  ok = ok && allocNextDoorDataOnGPU(csr, data);
  if (ok) data.gpuCSRPartitions = transferCSRToGPUs(data, csr);
  for (int run = 0; ok && run < nruns; ++run)
    ok = sample_parallel ? doSampleParallelSampling(csr, data) : doTransitParallelSampling(csr, data, enableLoadBalancing);
  if (ok) {
    std::vector<VertexID_t>& final_samples = getFinalSamples(data);
    const size_t final_size = (size_t)getFinalSampleSize(data);
    size_t total_sampled = 0;
    for (VertexID_t v : final_samples) total_sampled += v != data.INVALID_VERTEX;
    if (print_samples) {
      for (size_t s = 0; final_size && s < final_samples.size(); s += final_size) {
        printf("Contents of sample %zu [", s / final_size);
        for (size_t v = s; v < s + final_size; ++v) printf("%d, ", final_samples[v]);
        printf("]\n");
      }
    }
    printf("totalSampledVertices %zu\n", total_sampled);
    freeDeviceData(data);
    if (chk_results) ok = checkResultsFunc(data);
  } else {
    fprintf(stderr, "nextdoor: %s\n", nd_last_error());
  }
  // the data block is done with the graph before the graph goes
  if (data.sampler) {
    nd_sampler_destroy(data.sampler);
    data.sampler = nullptr;
  }
  data.csr = nullptr;
  freeGraph(csr);
  return ok;
}

// nextdoor<SampleType, App>(file, type, format, nruns, chk, print, kernelType, lb, checker),
// src/nextdoor.cu:3239-3306, with the checker as the function pointer the reference takes.
template <class SampleType, typename App>
inline bool nextdoor(const char* graph_file, const char* graph_type, const char* graph_format, const int nruns,
                     const bool chk_results, const bool print_samples, const char* kernelType,
                     const bool enableLoadBalancing, bool (*checkResultsFunc)(NextDoorData<SampleType, App>&)) {
  NextDoorData<SampleType, App> nextDoorData;
  auto check = [&](NextDoorData<SampleType, App>& d) { return checkResultsFunc ? checkResultsFunc(d) : true; };
  return nextdoorRun(nextDoorData, graph_file, graph_type, graph_format, nruns, chk_results && checkResultsFunc,
                     print_samples, kernelType, enableLoadBalancing, check);
}

// The same for an app picked by its registry name, with any callable as the checker.
template <class CheckFn>
inline bool nextdoor(const char* app, const char* graph_file, const char* graph_type, const char* graph_format,
                     int nruns, bool chk_results, bool print_samples, const char* kernelType,
                     bool enableLoadBalancing, CheckFn checkResultsFunc) {
  NextDoorDataByName data(app);
  return nextdoorRun(data, graph_file, graph_type, graph_format, nruns, chk_results, print_samples, kernelType,
                     enableLoadBalancing, checkResultsFunc);
}

// appMain<SampleType, App>(argc, argv, checker), src/main.cu:5-55: the command line of every
// app binary of the reference.  -g graph file, -t adj-list | edge-list, -f binary | text,
// -n runs, -c check results, -p print samples, -k SampleParallel | TransitParallel, -l load
// balancing (long forms as in src/main.cu:11-29).
template <class SampleType, typename App>
inline int appMain(int argc, char* argv[], bool (*checkResults)(NextDoorData<SampleType, App>& nextDoorData)) {
  const char *graph_file = nullptr, *graph_type = nullptr, *graph_format = nullptr, *kernel = "TransitParallel";
  int nruns = 1;
  bool check = false, print = false, balance = false;
  auto is = [](const char* a, const char* s, const char* l) { return strcmp(a, s) == 0 || strcmp(a, l) == 0; };
  for (int i = 1; i < argc; ++i) {
    const char* a = argv[i];
    const char* value = i + 1 < argc ? argv[i + 1] : nullptr;
    if (is(a, "-g", "--graph-file") && value) graph_file = argv[++i];
    else if (is(a, "-t", "--graph-type") && value) graph_type = argv[++i];
    else if (is(a, "-f", "--format") && value) graph_format = argv[++i];
    else if (is(a, "-n", "--nruns") && value) nruns = atoi(argv[++i]);
    else if (is(a, "-k", "--kernel-type") && value) kernel = argv[++i];
    else if (is(a, "-c", "--check-results")) check = true;
    else if (is(a, "-p", "--print-samples")) print = true;
    else if (is(a, "-l", "--load-balancing")) balance = true;
  }
  if (!graph_file || !graph_type || !graph_format) {
    printf("usage: \n\n-h --help              Prints this help\n-g --graph-file        File containing graph\n"
           "-t --graph-type <type> Format of graph file: 'adj-list' or 'edge-list'\n"
           "-f --format <format>   Format of graph file: 'binary' or 'text'\n-n --nruns             Number of runs\n"
           "-c --check-results     Check results using an algorithm\n-p --print-samples     Print Samples\n"
           "-k --kernel-type       Type of Kernel: 'SampleParallel' or 'TransitParallel'\n"
           "-l --load-balancing    Enable Load Balancing\n");
    return 0;
  }
  nextdoor<SampleType, App>(graph_file, graph_type, graph_format, nruns, check, print, kernel, balance, checkResults);
  return 0;
}

#endif  // LIBNEXTDOOR_AMD_HPP
