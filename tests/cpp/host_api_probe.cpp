// Compiles the C++ host API header against the library and exercises what runs without a
// GPU: the app registry, graph ingest through loadGraph, and the error path of a sampler
// whose app does not exist.  With "gpu" as the third argument it also runs the whole
// nextdoor<>() sequence and checks the shape of the result.
#include <string.h>

#include <libNextDoor_amd.hpp>

int main(int argc, char** argv) {
  if (argc < 2) return 2;
  const char* graph_file = argv[1];
  const bool gpu = argc > 2 && strcmp(argv[2], "gpu") == 0;
  if (nd_num_apps() < 5) return 3;
  CSR* csr = loadGraph(graph_file, "edge-list", "text");
  if (!csr) return 4;
  printf("vertices %d edges %lld\n", nd_graph_num_vertices(csr), (long long)nd_graph_num_edges(csr));
  {
    NextDoorData bogus("NoSuchApp");
    if (transferCSRToGPUs(bogus, csr)) return 5;  // unknown app: false, message, no abort
    printf("error %s\n", nd_last_error());
  }
  if (loadGraph("/nonexistent/graph", "edge-list", "text") != nullptr) return 6;
  nd_graph_free(csr);
  if (!gpu) return 0;
  int final_size = 0;
  size_t n_values = 0;
  const bool ok = nextdoor("UniformRandomWalk8", graph_file, "edge-list", "text", 2, true, false, "TransitParallel", true,
                           [&](NextDoorData& data) {
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
    NextDoorData data("UniformRandomWalk8");
    if (!g || !allocNextDoorDataOnGPU(g, data)) return 8;
    if (!(mode == 0 ? doTransitParallelSampling(g, data, true) : doSampleParallelSampling(g, data))) return 9;
    (mode == 0 ? transit_parallel : sample_parallel) = getFinalSamples(data);
    freeDeviceData(data);
    nd_graph_free(g);
  }
  if (transit_parallel.empty() || transit_parallel != sample_parallel) return 10;
  printf("kernel types agree\n");
  {  // an edge-list app: every listed edge leaves a vertex of its sample
    CSR* g = loadGraph(graph_file, "edge-list", "text");
    NextDoorData data("MVS5");
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
    nd_graph_free(g);
  }
  return 0;
}
