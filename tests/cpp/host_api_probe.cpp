// Compiles the C++ host API header against the library and exercises what runs without a
// GPU: the app registry, graph ingest through loadGraph, and the error path of a sampler
// whose app does not exist.  With "gpu" as the third argument it also runs the whole
// nextdoor<>() sequence and checks the shape of the result.
#include <string.h>

#include <libNextDoor_amd.hpp>
#include <nextdoor_amd_apps.hpp>

// A test written as the reference writes them (src/tests/testBase.h:14-24 and
// src/tests/singleGPU/khop.cu:9-11), for an App that is compiled into the library; this file is
// host-only C++ (g++), so the App is found by its registry name.
#define APP_TEST_BINARY(SampleClass, AppName, App, Graph, Path, Runs, CheckResults, chkResultsFunc, KernelType, \
                        LoadBalancing)                                                                           \
  static bool AppName##_##Graph(const char* Path) {                                                              \
    bool b = nextdoor<SampleClass, App>(Path, "edge-list", "text", Runs, CheckResults, false, KernelType,        \
                                        LoadBalancing, chkResultsFunc);                                          \
    return b;                                                                                                    \
  }
#define COMMA ,
APP_TEST_BINARY(KHopSample, KHop, KHopApp, RingLB, path, 1, true, checkSampledVerticesResult<KHopSample COMMA KHopApp>,
                "TransitParallel", true)
APP_TEST_BINARY(DummySample, DeepWalk, DeepWalkApp, RingTP, path, 2, true,
                checkSampledVerticesResult<DummySample COMMA DeepWalkApp>, "TransitParallel", false)

int main(int argc, char** argv) {
  if (argc < 2) return 2;
  const char* graph_file = argv[1];
  const bool gpu = argc > 2 && strcmp(argv[2], "gpu") == 0;
  if (nd_num_apps() < 5) return 3;
  Graph graph;
  CSR* csr = loadGraph(graph, graph_file, "edge-list", "text");
  if (!csr) return 4;
  printf("vertices %zu edges %lld\n", graph.get_vertices().size(), (long long)graph.get_n_edges());
  {
    NextDoorDataByName bogus("NoSuchApp");
    if (!transferCSRToGPUs(bogus, csr).empty()) return 5;  // unknown app: false, message, no abort
    printf("error %s\n", nd_last_error());
  }
  if (loadGraph("/nonexistent/graph", "edge-list", "text") != nullptr) return 6;
  freeGraph(csr);
  // the template spellings resolve the library's apps by type, and the shape algebra runs on the host
  if (getFinalSampleSize<KHopApp>() != 275 || getFinalSampleSize<DeepWalkApp>() != 100) return 14;
  if (strcmp(NextDoorAppName<KHopApp>::name(), "KHop") != 0) return 15;
  if (!gpu) return 0;
  if (!KHop_RingLB(graph_file) || !DeepWalk_RingTP(graph_file)) return 16;
  printf("reference-style tests pass\n");
  int final_size = 0;
  size_t n_values = 0;
  const bool ok = nextdoor("UniformRandomWalk8", graph_file, "edge-list", "text", 2, true, false, "TransitParallel", true,
                           [&](NextDoorDataByName& data) {
                             final_size = getFinalSampleSize(data);
                             n_values = data.hFinalSamples.size();
                             // the library's validator, on the host copies after freeDeviceData
                             return final_size == 8 && n_values == data.initialContents.size() * 8 &&
                                    checkSampledVerticesResult(data);
                           });
  printf("final_size %d values %zu\n", final_size, n_values);
  if (!ok) return 7;
  // the reference's other kernel type gives the same samples
  std::vector<VertexID_t> transit_parallel, sample_parallel;
  for (int mode = 0; mode < 2; ++mode) {
    CSR* g = loadGraph(graph_file, "edge-list", "text");
    NextDoorDataByName data("UniformRandomWalk8");
    if (!g || !allocNextDoorDataOnGPU(g, data)) return 8;
    if (!(mode == 0 ? doTransitParallelSampling(g, data, true) : doSampleParallelSampling(g, data))) return 9;
    (mode == 0 ? transit_parallel : sample_parallel) = getFinalSamples(data);
    freeDeviceData(data);
    freeGraph(g);
  }
  if (transit_parallel.empty() || transit_parallel != sample_parallel) return 10;
  printf("kernel types agree\n");
  {  // an edge-list app: every listed edge leaves a vertex of its sample
    CSR* g = loadGraph(graph_file, "edge-list", "text");
    NextDoorDataByName data("MVS5");
    std::vector<VertexID_t> rows, cols;
    std::vector<uint32_t> start;
    if (!g || !allocNextDoorDataOnGPU(g, data) || !doTransitParallelSampling(g, data, true)) return 11;
    if (!getAdjacency(data, rows, cols, start) || rows.size() != cols.size() || start.empty() ||
        start.back() != rows.size())
      return 12;
    for (size_t s = 0; s + 1 < start.size(); ++s)
      for (uint32_t e = start[s]; e < start[s + 1]; ++e) {
        bool mine = false;
        for (int i = 0; i < 5; ++i) mine = mine || data.initialContents[s * 5 + (size_t)i] == rows[e];
        if (!mine) return 13;
      }
    printf("edge lists %zu\n", rows.size());
    freeDeviceData(data);
    freeGraph(g);
  }
  return 0;
}
