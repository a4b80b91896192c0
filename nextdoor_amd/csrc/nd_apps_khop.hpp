// k-hop neighbourhood sampling (GraphSAGE style) on the App contract.
//
// Reference: src/apps/khop/khop.cu:1-81 (two hops, fan-outs 25 and 10, one root per
// sample, every draw uniform WITH replacement from the transit's adjacency) and
// src/apps/layer/layerSampling.cu (same sampler with other fan-outs).
#pragma once

#include "nd_contract.hpp"

class KHopSample {};

// Fan-outs are template parameters so other sizes instantiate the same code;
// kFanout2 == 0 means a single hop.
template <int kFanout0, int kFanout1, int kFanout2 = 0>
struct KHopAppT {
  __host__ __device__ int steps() { return kFanout2 > 0 ? 3 : 2; }
  __host__ __device__ int stepSize(int k) { return k == 0 ? kFanout0 : (k == 1 ? kFanout1 : kFanout2); }

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int, CSRPartition*, const VertexID*, const VertexID, SampleType*, const float,
                                  EdgeArray& transitEdges, WeightArray&, const EdgePos_t numEdges, const VertexID_t,
                                  curandState* state) {
    if (numEdges == 0) return -1;
    return transitEdges[RandNumGen::rand_int(state, numEdges)];
  }

  __host__ __device__ int samplingType() { return SamplingType::IndividualNeighborhood; }
  __host__ __device__ OutputFormat outputFormat() { return SampledVertices; }
  __host__ __device__ EdgePos_t numSamples(CSR* graph) { return graph->get_n_vertices(); }
  __host__ __device__ EdgePos_t initialSampleSize(CSR*) { return 1; }
  __host__ __device__ bool hasExplicitTransits() { return false; }

  template <class SampleType>
  __host__ std::vector<VertexID_t> initialSample(int sampleIdx, CSR*, SampleType&) {
    return std::vector<VertexID_t>(1, sampleIdx);
  }

  template <class SampleType>
  __host__ __device__ VertexID_t stepTransits(int, const VertexID_t, SampleType&, int, curandState*) {
    return -1;
  }

  template <class SampleType>
  __host__ SampleType initializeSample(CSR*, const VertexID_t) {
    return SampleType();
  }
};

typedef KHopAppT<25, 10> KHopApp;
// src/apps/layer/layerSampling.cu:1-81: the same sampler with fan-outs 10 and 25
class LayerSample {};
typedef KHopAppT<10, 25> LayerSamplingApp;

ND_APP_REGISTERED_AS(KHopApp, "KHop")
ND_APP_REGISTERED_AS(LayerSamplingApp, "Layer")
typedef KHopAppT<3, 2> KHop3x2App;
ND_APP_REGISTERED_AS(KHop3x2App, "KHop3x2")
