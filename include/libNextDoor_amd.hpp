// C++ host API over the C ABI of libnextdoor_amd.so, under the names of the reference's
// host API (src/libNextDoor.hpp:39-50; definitions in src/nextdoor.cu).  Header only; link
// with -lnextdoor_amd.
//
// The reference's functions are templates over <SampleType, App> and take
// NextDoorData<SampleType, App>&.  Here the app is compiled into the library and picked by
// its registry name, so NextDoorData carries the name instead of template parameters;
// everything else (call order, bool results, the host vectors a caller reads) is the same.
// Failures return false / nullptr and leave the reason in nd_last_error(); nothing aborts.
#ifndef LIBNEXTDOOR_AMD_HPP
#define LIBNEXTDOOR_AMD_HPP

#include <stdint.h>
#include <stdio.h>

#include <vector>

#include "nextdoor_amd.h"

typedef int32_t VertexID_t;

// The reference's CSR* as returned by loadGraph: an opaque host graph.
typedef nd_graph CSR;

// NextDoorData<SampleType, App> (src/libNextDoor.hpp:13-37): the host-visible members a
// caller of the reference reads, plus the sampler handle.
struct NextDoorData {
  explicit NextDoorData(const char* app, uint64_t seed = 42) : appName(app), seed(seed) {}
  ~NextDoorData() {
    if (sampler) nd_sampler_destroy(sampler);
  }
  NextDoorData(const NextDoorData&) = delete;
  NextDoorData& operator=(const NextDoorData&) = delete;

  const char* appName;
  uint64_t seed;
  nd_sampler* sampler = nullptr;
  CSR* csr = nullptr;                       // the caller's graph; stays set after freeDeviceData
  bool graphOnDevice = false;
  std::vector<VertexID_t> hFinalSamples;    // libNextDoor.hpp:17
  std::vector<VertexID_t> initialContents;  // libNextDoor.hpp:18
  VertexID_t INVALID_VERTEX = 0;            // libNextDoor.hpp:35
  int maxBits = 0;                          // libNextDoor.hpp:36
};

// loadGraph(graph, file, type, format), src/nextdoor.cu:1845-1891: nullptr on failure.
inline CSR* loadGraph(const char* graph_file, const char* graph_type, const char* graph_format) {
  CSR* csr = nullptr;
  if (nd_graph_load(graph_file, graph_type, graph_format, &csr) != 0) {
    fprintf(stderr, "loadGraph: %s\n", nd_last_error());
    return nullptr;
  }
  return csr;
}

// transferCSRToGPUs(data, csr), src/nextdoor.cu:1893-1911.
inline bool transferCSRToGPUs(NextDoorData& data, CSR* csr) {
  if (!data.sampler && nd_sampler_create(data.appName, &data.sampler) != 0) return false;
  if (nd_sampler_set_graph(data.sampler, csr) != 0) return false;
  data.csr = csr;
  data.graphOnDevice = true;
  return true;
}

// allocNextDoorDataOnGPU(csr, data), src/nextdoor.cu:1931-2086.  Transfers the graph first
// when the caller has not done so.
inline bool allocNextDoorDataOnGPU(CSR* csr, NextDoorData& data) {
  if ((data.csr != csr || !data.graphOnDevice) && !transferCSRToGPUs(data, csr)) return false;
  if (nd_sampler_alloc(data.sampler, data.seed) != 0) return false;
  const VertexID_t* roots = nullptr;
  int64_t n = 0;
  if (nd_sampler_initial_contents(data.sampler, &roots, &n) != 0) return false;
  data.initialContents.assign(roots, roots + n);
  data.INVALID_VERTEX = nd_sampler_invalid_vertex(data.sampler);
  data.maxBits = nd_sampler_max_bits(data.sampler);
  return true;
}

// doTransitParallelSampling(csr, data, enableLoadBalancing), src/nextdoor.cu:2191-3006: the
// sample -> transit map is inverted before every step.
inline bool doTransitParallelSampling(CSR*, NextDoorData& data, bool enableLoadBalancing) {
  return data.sampler && nd_sampler_set_inversion_period(data.sampler, 1) == 0 &&
         nd_sampler_do_transit_parallel(data.sampler, enableLoadBalancing ? 1 : 0) == 0;
}

// doSampleParallelSampling(csr, data), src/nextdoor.cu:3009-3209: the reference's baseline
// mode, every sample's work in sample order: the engine never brings the pairs into transit
// order (it only drops the dead ones) and does no load balancing.  The samples are the same
// bytes either way.
inline bool doSampleParallelSampling(CSR*, NextDoorData& data) {
  return data.sampler && nd_sampler_do_sample_parallel(data.sampler) == 0;
}

// getFinalSamples(data), src/nextdoor.cu:3211-3237.
inline std::vector<VertexID_t>& getFinalSamples(NextDoorData& data) {
  const VertexID_t* p = nullptr;
  int64_t n = 0;
  if (data.sampler && nd_sampler_get_final_samples(data.sampler, &p, &n) == 0) data.hFinalSamples.assign(p, p + n);
  return data.hFinalSamples;
}

// getFinalSampleSize<App>(), src/nextdoor.cu:1913-1929.
inline int getFinalSampleSize(const NextDoorData& data) {
  return data.sampler ? nd_sampler_final_sample_size(data.sampler) : 0;
}

// freeDeviceData(data), src/nextdoor.cu:2088-2115.
inline void freeDeviceData(NextDoorData& data) {
  if (data.sampler) nd_sampler_free_device(data.sampler);
  data.graphOnDevice = false;
}

// checkSampledVerticesResult<SampleType, App>(data), src/check_results.cu:162-299: the checker
// the reference's per-transit apps hand to nextdoor().  Works on the host copies
// (data.hFinalSamples, data.initialContents, data.csr), so also after freeDeviceData.
inline bool checkSampledVerticesResult(NextDoorData& data) {
  if (!data.sampler || !data.csr) return false;
  const int steps = nd_sampler_steps(data.sampler);
  std::vector<int32_t> sizes((size_t)(steps > 0 ? steps : 0));
  for (int k = 0; k < steps; ++k) sizes[(size_t)k] = nd_sampler_step_size(data.sampler, k);
  const int initial = nd_sampler_initial_sample_size(data.sampler);
  const int64_t n_samples = initial > 0 ? (int64_t)data.initialContents.size() / initial : 0;
  const int verdict = nd_check_sampled_vertices(data.csr, steps, sizes.data(), initial,
                                                nd_sampler_sampling_type(data.sampler) == 1, n_samples,
                                                data.initialContents.data(), data.hFinalSamples.data(),
                                                data.INVALID_VERTEX);
  if (verdict != 1) fprintf(stderr, "%s\n", nd_last_error());
  return verdict == 1;
}

// The edge lists of the apps whose outputFormat() is AdjacencyMatrix on per-transit sampling
// (MVS, ClusterGCN; the reference reads dRowStorage / dColStorage at sample.posInStorage):
// sample i owns rows/cols[list_start[i] .. list_start[i + 1]).
inline bool getAdjacency(NextDoorData& data, std::vector<VertexID_t>& rows, std::vector<VertexID_t>& cols,
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

// nextdoor<SampleType, App>(file, type, format, nruns, chk, print, kernelType, lb, checker),
// src/nextdoor.cu:3239-3306: load, allocate, sample nruns times, fetch, count the sampled
// (non-INVALID) vertices, free, then run the caller's check on the final samples.
// kernelType: "TransitParallel" or "SampleParallel" (src/main.cu:19-21).
template <class CheckFn>
inline bool nextdoor(const char* app, const char* graph_file, const char* graph_type, const char* graph_format,
                     int nruns, bool chk_results, bool print_samples, const char* kernelType,
                     bool enableLoadBalancing, CheckFn checkResultsFunc) {
  CSR* csr = loadGraph(graph_file, graph_type, graph_format);
  if (!csr) return false;
  bool ok = false;
  {
    NextDoorData data(app);
    const bool sample_parallel = kernelType && kernelType[0] == 'S';
    ok = allocNextDoorDataOnGPU(csr, data);
    for (int run = 0; ok && run < nruns; ++run)
      ok = sample_parallel ? doSampleParallelSampling(csr, data) : doTransitParallelSampling(csr, data, enableLoadBalancing);
    if (ok) {
      std::vector<VertexID_t>& final_samples = getFinalSamples(data);
      size_t total_sampled = 0;
      for (VertexID_t v : final_samples) total_sampled += v != data.INVALID_VERTEX;
      printf("totalSampledVertices %zu\n", total_sampled);
      if (print_samples) {
        const int len = getFinalSampleSize(data);
        for (size_t i = 0; i < final_samples.size(); ++i)
          printf("%d%c", final_samples[i], (i + 1) % (size_t)len == 0 ? '\n' : ' ');
      }
      freeDeviceData(data);
      if (chk_results) ok = checkResultsFunc(data);
    } else {
      fprintf(stderr, "nextdoor: %s\n", nd_last_error());
    }
  }
  nd_graph_free(csr);
  return ok;
}

#endif  // LIBNEXTDOOR_AMD_HPP
