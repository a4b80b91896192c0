// Multi-dimensional random walk on the App contract: the reference's one app with
// explicit transits (src/apps/multiRW/multiRW.cu:1-108).
//
// A sample owns kRoots walkers.  Every step advances one of them: the walker is the step's
// transit, next() draws one of its neighbours uniformly, returns it and (after step 0)
// puts it in the walker's place; stepTransits() then draws the walker of the following
// step.  The engine calls stepTransits(step + 1, ...) right after next(), with the same
// random state, as the reference's step kernels do (src/nextdoor.cu:279-289).
//
// Where this differs from the reference: the walkers' start vertices come from a fixed
// Philox stream instead of rand() (multiRW.cu:95-106), so runs are reproducible, and
// lastRootIdx starts at 0 instead of being left uninitialised.
#pragma once

#include "nd_contract.hpp"

template <int kRoots>
class MultiRWSampleT {
 public:
  int rootVertices[kRoots];
  int lastRootIdx;
};

template <int kRoots, int kSteps>
struct MultiRWAppT {
  static constexpr uint64_t kRootSeed = 0x4D525752ull;  // "MRWR"
  static constexpr uint32_t kRootStream = 0x524F4F54u;  // "ROOT"

  __host__ __device__ int steps() { return kSteps; }
  __host__ __device__ int stepSize(int) { return 1; }

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int step, CSRPartition*, const VertexID*, const VertexID, SampleType* sample,
                                  const float, EdgeArray& transitEdges, WeightArray&, const EdgePos_t numEdges,
                                  const VertexID_t, curandState* state) {
    if (numEdges == 0) return -1;
    const VertexID_t v = numEdges == 1 ? transitEdges[0] : transitEdges[RandNumGen::rand_int(state, numEdges)];
    if (step > 0) sample->rootVertices[sample->lastRootIdx] = v;
    return v;
  }

  __host__ __device__ int samplingType() { return SamplingType::IndividualNeighborhood; }
  __host__ __device__ OutputFormat outputFormat() { return SampledVertices; }
  __host__ __device__ EdgePos_t numSamples(CSR* graph) { return graph->get_n_vertices(); }
  __host__ __device__ EdgePos_t initialSampleSize(CSR*) { return 1; }
  __host__ __device__ bool hasExplicitTransits() { return true; }

  template <class SampleType>
  __host__ std::vector<VertexID_t> initialSample(int, CSR*, SampleType& sample) {
    return std::vector<VertexID_t>(1, sample.rootVertices[0]);
  }

  // the walker of the coming step: uniform over the walkers (multiRW.cu:84-92)
  template <class SampleType>
  __device__ VertexID_t stepTransits(int, const VertexID_t, SampleType& sample, int, curandState* randState) {
    const int x = RandNumGen::rand_int(randState, kRoots);
    sample.lastRootIdx = x;
    return sample.rootVertices[x];
  }

  template <class SampleType>
  __host__ SampleType initializeSample(CSR* graph, const VertexID_t sampleID) {
    SampleType sample;
    for (int i = 0; i < kRoots; i++) {
      const float u = nd::uniform_at(kRootSeed, (uint64_t)sampleID, kRootStream, (uint32_t)i);
      sample.rootVertices[i] = nd::rand_int_from_uniform(u, graph->get_n_vertices());
    }
    sample.lastRootIdx = 0;
    return sample;
  }
};

// The reference's sizes: 100 walkers, 100 steps (multiRW.cu:3, 14).
typedef MultiRWSampleT<100> MultiRWSample;
typedef MultiRWAppT<100, 100> MultiRWApp;

ND_APP_REGISTERED_AS(MultiRWApp, "MultiRW")
