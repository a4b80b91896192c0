// Two applications of a user's own, written on the App contract in the style of the reference's
// apps (plain structs, sizes as literals: src/apps/khop/khop.cu, src/apps/randomwalks/randomWalks.cu),
// that are NOT compiled into libnextdoor_amd.so.  This file is built by hipcc into a shared
// object of its own (tests/cpp/libuser_apps.so); loading it registers them with the library.
#include "../../nextdoor_amd/csrc/nd_app_registry.hpp"

class UserHopSample {};

// three hops with fan-outs 5, 3, 2, uniform with replacement, one sample per vertex
struct UserThreeHopApp {
  __host__ __device__ int steps() { return 3; }
  __host__ __device__ int stepSize(int k) { return k == 0 ? 5 : (k == 1 ? 3 : 2); }

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int step, CSRPartition* csr, const VertexID* transit, const VertexID sampleIdx,
                                  SampleType* sample, const float max_weight, EdgeArray& transitEdges,
                                  WeightArray& transitEdgeWeights, const EdgePos_t numEdges,
                                  const VertexID_t neighbrID, curandState* state) {
    if (numEdges == 0) return -1;
    EdgePos_t id = RandNumGen::rand_int(state, numEdges);
    return transitEdges[id];
  }

  __host__ __device__ int samplingType() { return SamplingType::IndividualNeighborhood; }
  __host__ __device__ OutputFormat outputFormat() { return SampledVertices; }
  __host__ __device__ EdgePos_t numSamples(CSR* graph) { return graph->get_n_vertices(); }

  template <class SampleType>
  __host__ std::vector<VertexID_t> initialSample(int sampleIdx, CSR* graph, SampleType& sample) {
    std::vector<VertexID_t> initialValue;
    initialValue.push_back(sampleIdx);
    return initialValue;
  }

  __host__ __device__ EdgePos_t initialSampleSize(CSR* graph) { return 1; }
  __host__ __device__ bool hasExplicitTransits() { return false; }

  template <class SampleType>
  __host__ __device__ VertexID_t stepTransits(int step, const VertexID_t sampleID, SampleType& sample,
                                              int transitIdx, curandState* randState) {
    return -1;
  }

  template <class SampleType>
  __host__ SampleType initializeSample(CSR* graph, const VertexID_t sampleID) {
    SampleType sample;
    return sample;
  }
};

class UserWalkSample {};

// walks of 7 steps, three per vertex, each step drawn by edge weight with rejection against the
// vertex's largest weight (the rule of the reference's DeepWalkApp, randomWalks.cu:65-91)
struct UserShortDeepWalkApp {
  __host__ __device__ int steps() { return 7; }
  __host__ __device__ int stepSize(int k) { return 1; }

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int step, CSRPartition* csr, const VertexID* transit, const VertexID sampleIdx,
                                  SampleType* sample, const float max_weight, EdgeArray& transitEdges,
                                  WeightArray& transitEdgeWeights, const EdgePos_t numEdges,
                                  const VertexID_t neighbrID, curandState* state) {
    if (numEdges == 0) return -1;
    if (numEdges == 1) return transitEdges[0];
    EdgePos_t x = RandNumGen::rand_int(state, numEdges);
    float y = curand_uniform(state) * max_weight;
    while (y > transitEdgeWeights[x]) {
      x = RandNumGen::rand_int(state, numEdges);
      y = curand_uniform(state) * max_weight;
    }
    return transitEdges[x];
  }

  __host__ __device__ int samplingType() { return SamplingType::IndividualNeighborhood; }
  __host__ __device__ OutputFormat outputFormat() { return SampledVertices; }
  __host__ __device__ EdgePos_t numSamples(CSR* graph) { return 3 * graph->get_n_vertices(); }

  template <class SampleType>
  __host__ std::vector<VertexID_t> initialSample(int sampleIdx, CSR* graph, SampleType& sample) {
    std::vector<VertexID_t> initialValue;
    initialValue.push_back(sampleIdx % graph->get_n_vertices());
    return initialValue;
  }

  __host__ __device__ EdgePos_t initialSampleSize(CSR* graph) { return 1; }
  __host__ __device__ bool hasExplicitTransits() { return false; }

  template <class SampleType>
  __host__ __device__ VertexID_t stepTransits(int step, const VertexID_t sampleID, SampleType& sample,
                                              int transitIdx, curandState* randState) {
    return -1;
  }

  template <class SampleType>
  __host__ SampleType initializeSample(CSR* graph, const VertexID_t sampleID) {
    SampleType sample = SampleType();
    return sample;
  }
};

// An app that chooses its transits itself and has several per sample: a sample holds four
// "anchor" vertices; every step samples a neighbour of each transit (the k-hop rule), and
// stepTransits sends each output back to one of the anchors for the next step, or nowhere.
struct UserAnchorSample {
  VertexID_t anchors[4];
};

struct UserAnchorHopApp {
  __host__ __device__ int steps() { return 3; }
  __host__ __device__ int stepSize(int k) { return k == 1 ? 3 : 2; }

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int step, CSRPartition* csr, const VertexID* transit, const VertexID sampleIdx,
                                  SampleType* sample, const float max_weight, EdgeArray& transitEdges,
                                  WeightArray& transitEdgeWeights, const EdgePos_t numEdges,
                                  const VertexID_t neighbrID, curandState* state) {
    if (numEdges == 0) return -1;
    EdgePos_t x = RandNumGen::rand_int(state, numEdges);
    return transitEdges[x];
  }

  __host__ __device__ int samplingType() { return SamplingType::IndividualNeighborhood; }
  __host__ __device__ OutputFormat outputFormat() { return SampledVertices; }
  __host__ __device__ EdgePos_t numSamples(CSR* graph) { return graph->get_n_vertices(); }

  template <class SampleType>
  __host__ std::vector<VertexID_t> initialSample(int sampleIdx, CSR* graph, SampleType& sample) {
    std::vector<VertexID_t> initialValue;
    for (int i = 0; i < 4; i++) {
      sample.anchors[i] = (VertexID_t)(((int64_t)sampleIdx * 7 + i * 13) % graph->get_n_vertices());
      initialValue.push_back(sample.anchors[i]);
    }
    return initialValue;
  }

  __host__ __device__ EdgePos_t initialSampleSize(CSR* graph) { return 4; }
  __host__ __device__ bool hasExplicitTransits() { return true; }

  template <class SampleType>
  __host__ __device__ VertexID_t stepTransits(int step, const VertexID_t sampleID, SampleType& sample,
                                              int transitIdx, curandState* randState) {
    EdgePos_t x = RandNumGen::rand_int(randState, 5);
    if (x == 4) return -1;
    return sample.anchors[(transitIdx + x) % 4];
  }

  template <class SampleType>
  __host__ SampleType initializeSample(CSR* graph, const VertexID_t sampleID) {
    SampleType sample = SampleType();
    return sample;
  }
};

ND_REGISTER_APP("UserAnchorHop", UserAnchorSample, UserAnchorHopApp)
ND_REGISTER_APP("UserThreeHop", UserHopSample, UserThreeHopApp)
ND_REGISTER_APP("UserShortDeepWalk", UserWalkSample, UserShortDeepWalkApp)
