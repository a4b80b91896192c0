// Random-walk applications on the App contract (see nd_contract.hpp).
//
// Semantics follow the reference's apps; file:line below are in the reference tree:
//   UniformRandomWalkApp    example/uniformRandWalk.cu:15-93
//   DeepWalkApp             src/apps/randomwalks/randomWalks.cu:3-91
//   PPRApp                  src/apps/randomwalks/randomWalks.cu:93-125
//   Node2VecApp             src/apps/randomwalks/randomWalks.cu:132-178 (literal, including
//                           the comparison of an edge index with a vertex id at :159)
//   WeightedNode2VecApp     not in the reference: second-order bias times edge weight,
//                           rejected against max_weight * max(p, 1/q, 1)
// Every walk samples one neighbour per step (stepSize 1) from the individual
// neighbourhood of its single transit; a return of -1 ends the walk.
#pragma once

#include "nd_contract.hpp"

struct UniformRandomWalkSample {};
class DummySample {};

class Node2VecSample {
 public:
  VertexID t;  // vertex visited before the current transit
};

namespace nd {
namespace apps {

// Members shared by all walks.  kWalkLength steps, one root per sample.
template <int kWalkLength>
struct WalkCommon {
  __host__ __device__ int steps() { return kWalkLength; }
  __host__ __device__ int stepSize(int) { return 1; }
  __host__ __device__ int samplingType() { return SamplingType::IndividualNeighborhood; }
  __host__ __device__ OutputFormat outputFormat() { return SampledVertices; }
  __host__ __device__ EdgePos_t initialSampleSize(CSR*) { return 1; }
  __host__ __device__ bool hasExplicitTransits() { return false; }

  template <class SampleType>
  __host__ __device__ VertexID_t stepTransits(int, const VertexID_t, SampleType&, int, curandState*) {
    return -1;
  }

  template <class SampleType>
  __host__ SampleType initializeSample(CSR*, const VertexID_t) {
    return SampleType();
  }
};

// One walk rooted at every vertex: sample i starts at vertex i.
template <int kWalkLength>
struct OneWalkPerVertex : WalkCommon<kWalkLength> {
  __host__ __device__ EdgePos_t numSamples(CSR* graph) { return graph->get_n_vertices(); }

  template <class SampleType>
  __host__ std::vector<VertexID_t> initialSample(int sampleIdx, CSR*, SampleType&) {
    return std::vector<VertexID_t>(1, sampleIdx);
  }
};

// Several walks rooted at every vertex: sample i starts at vertex i mod |V|.
template <int kWalkLength, int kWalksPerVertex>
struct WalksPerVertex : WalkCommon<kWalkLength> {
  __host__ __device__ EdgePos_t numSamples(CSR* graph) { return kWalksPerVertex * graph->get_n_vertices(); }

  template <class SampleType>
  __host__ std::vector<VertexID_t> initialSample(int sampleIdx, CSR* graph, SampleType&) {
    return std::vector<VertexID_t>(1, sampleIdx % graph->get_n_vertices());
  }
};

// The reference's RandomWalkApp sizing (randomWalks.cu:23-37): small graphs get 100
// walks per vertex, roots wrap around the vertex range.
template <int kWalkLength>
struct HundredWalksOnSmallGraphs : WalkCommon<kWalkLength> {
  __host__ __device__ EdgePos_t numSamples(CSR* graph) {
    const VertexID n = graph->get_n_vertices();
    return n < 256 * 1024 ? 100 * n : n;
  }

  template <class SampleType>
  __host__ std::vector<VertexID_t> initialSample(int sampleIdx, CSR* graph, SampleType&) {
    return std::vector<VertexID_t>(1, sampleIdx % graph->get_n_vertices());
  }
};

// Rejection sampling of an edge proportionally to its weight, against the largest
// weight of the transit (randomWalks.cu:81-88).  Returns the accepted edge index.
// Candidate i consumes draws 2i (edge index) and 2i+1 (height).
template <typename WeightArray>
__device__ __forceinline__ EdgePos_t weighted_edge_by_rejection(const WeightArray& w, EdgePos_t n, float max_weight,
                                                                curandState* state) {
  EdgePos_t x = RandNumGen::rand_int(state, n);
  float y = curand_uniform(state) * max_weight;
  while (y > w[x]) {
    x = RandNumGen::rand_int(state, n);
    y = curand_uniform(state) * max_weight;
  }
  return x;
}

}  // namespace apps
}  // namespace nd

template <int kWalkLength>
struct UniformRandomWalkAppT : nd::apps::OneWalkPerVertex<kWalkLength> {
  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int, CSRPartition*, const VertexID*, const VertexID, SampleType*, const float,
                                  EdgeArray& transitEdges, WeightArray&, const EdgePos_t numEdges, const VertexID_t,
                                  curandState* state) {
    return transitEdges[RandNumGen::rand_int(state, numEdges)];
  }
};

template <class Sizing>
struct DeepWalkAppT : Sizing {
  static constexpr bool kUsesEdgeWeights = true;

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int, CSRPartition*, const VertexID*, const VertexID, SampleType*,
                                  const float max_weight, EdgeArray& transitEdges, WeightArray& transitEdgeWeights,
                                  const EdgePos_t numEdges, const VertexID_t, curandState* state) {
    if (numEdges == 0) return -1;
    if (numEdges == 1) return transitEdges[0];
    return transitEdges[nd::apps::weighted_edge_by_rejection(transitEdgeWeights, numEdges, max_weight, state)];
  }
};

template <class Sizing>
struct PPRAppT : Sizing {
  static constexpr bool kUsesEdgeWeights = true;

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int, CSRPartition*, const VertexID*, const VertexID, SampleType*,
                                  const float max_weight, EdgeArray& transitEdges, WeightArray& transitEdgeWeights,
                                  const EdgePos_t numEdges, const VertexID_t, curandState* state) {
    if (numEdges == 0) return -1;
    // the walk ends with probability 0.01 at every step (randomWalks.cu:105-109)
    if (curand_uniform(state) < 0.01f) return -1;
    if (numEdges == 1) return transitEdges[0];
    return transitEdges[nd::apps::weighted_edge_by_rejection(transitEdgeWeights, numEdges, max_weight, state)];
  }
};

template <class Sizing>
struct Node2VecAppT : Sizing {
  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int step, CSRPartition* csr, const VertexID* transits, const VertexID,
                                  SampleType* sample, const float, EdgeArray& transitEdges, WeightArray&,
                                  const EdgePos_t numEdges, const VertexID_t, curandState* state) {
    if (numEdges == 0) return -1;
    if (numEdges == 1 || step == 0) {
      sample->t = *transits;
      return transitEdges[0];
    }
    const float p = 2.0f, q = 0.5f;
    const float envelope = fmaxf(fmaxf(p, 1 / q), 1.0f);
    for (;;) {
      const EdgePos_t x = RandNumGen::rand_int(state, numEdges);
      const VertexID v = transitEdges[x];
      const float y = curand_uniform(state) * envelope;
      const VertexID prev = sample->t;
      const CSR::Edge* prevEdges = csr->get_edges(prev);
      const EdgePos_t prevDegree = csr->get_n_edges_for_vertex(prev);
      float h = 1.0f;
      if (x == prev) h = p;  // as in the reference: edge index against vertex id
      else if (utils::binarySearch(prevEdges, v, prevDegree)) h = 1 / q;
      if (y < h) {
        sample->t = *transits;
        return v;
      }
    }
  }
};

// Weighted second-order walk, p = kPNum / kPDen and q = kQNum / kQDen (default p = 2,
// q = 0.5).  Bias of candidate v reached over edge x from transit u, with t the vertex
// visited before u:
//   h = p if v == t, 1/q if v is adjacent to t, else 1   (h = 1 at step 0: no t yet)
// accepted when uniform * max_weight(u) * max(p, 1/q, 1) < h * weight(x).
template <int kWalkLength, int kPNum = 2, int kPDen = 1, int kQNum = 1, int kQDen = 2,
          class Sizing = nd::apps::OneWalkPerVertex<kWalkLength>>
struct WeightedNode2VecAppT : Sizing {
  static constexpr bool kUsesEdgeWeights = true;
  static constexpr bool kUsesEdgeLookup = true;

  __host__ __device__ static float return_bias() { return (float)kPNum / (float)kPDen; }        // p
  __host__ __device__ static float adjacent_bias() { return 1 / ((float)kQNum / (float)kQDen); }  // 1/q
  __host__ __device__ static float largest_bias() { return fmaxf(fmaxf(return_bias(), adjacent_bias()), 1.0f); }
  __host__ __device__ static float smallest_bias() { return fminf(fminf(return_bias(), adjacent_bias()), 1.0f); }

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int step, CSRPartition* csr, const VertexID* transits, const VertexID,
                                  SampleType* sample, const float max_weight, EdgeArray& transitEdges,
                                  WeightArray& transitEdgeWeights, const EdgePos_t numEdges, const VertexID_t,
                                  curandState* state) {
    if (numEdges == 0) return -1;
    if (numEdges == 1) {
      sample->t = *transits;
      return transitEdges[0];
    }
    const float envelope = max_weight * largest_bias();
    VertexID prev = -1;  // read from the sample only when a decision depends on it
    // candidate i consumes draws 2i (edge index) and 2i+1 (height)
    for (;;) {
      const EdgePos_t x = RandNumGen::rand_int(state, numEdges);
      const float y = curand_uniform(state) * envelope;
      const VertexID v = transitEdges[x];
      const float wx = transitEdgeWeights[x];
      bool accepted;
      if (step == 0) {
        accepted = y < wx;  // no previous vertex yet: bias 1
      } else if (y < smallest_bias() * wx) {
        accepted = true;    // the bias is one of {p, 1/q, 1}: below the smallest, accepted whatever it is
      } else if (!(y < largest_bias() * wx)) {
        accepted = false;   // not below the largest: rejected whatever it is
      } else {
        // only in the band between does the candidate's relation to the previous vertex matter
        if (prev < 0) prev = sample->t;
        float h = 1.0f;
        if (v == prev) h = return_bias();
        else if (csr->has_edge_logn(prev, v)) h = adjacent_bias();
        accepted = y < h * wx;
      }
      if (accepted) {
        sample->t = *transits;
        return v;
      }
    }
  }
};

// Names and sizes of the reference's apps.
typedef UniformRandomWalkAppT<100> UniformRandomWalkApp;
typedef nd::apps::HundredWalksOnSmallGraphs<100> RandomWalkApp;
typedef DeepWalkAppT<RandomWalkApp> DeepWalkApp;
typedef PPRAppT<RandomWalkApp> PPRApp;
typedef Node2VecAppT<RandomWalkApp> Node2VecApp;
typedef WeightedNode2VecAppT<100> WeightedNode2VecApp;
// One-walk-per-vertex sizings of the same samplers.
typedef DeepWalkAppT<nd::apps::OneWalkPerVertex<100>> DeepWalkPerVertexApp;
typedef Node2VecAppT<nd::apps::OneWalkPerVertex<100>> Node2VecPerVertexApp;
typedef PPRAppT<nd::apps::OneWalkPerVertex<100>> PPRPerVertexApp;

ND_APP_REGISTERED_AS(UniformRandomWalkApp, "UniformRandomWalk")
ND_APP_REGISTERED_AS(DeepWalkApp, "DeepWalk")
ND_APP_REGISTERED_AS(PPRApp, "PPR")
ND_APP_REGISTERED_AS(Node2VecApp, "Node2Vec")
ND_APP_REGISTERED_AS(WeightedNode2VecApp, "WeightedNode2Vec")
ND_APP_REGISTERED_AS(DeepWalkPerVertexApp, "DeepWalkPerVertex")
ND_APP_REGISTERED_AS(Node2VecPerVertexApp, "Node2VecPerVertex")
ND_APP_REGISTERED_AS(PPRPerVertexApp, "PPRPerVertex")
ND_APP_REGISTERED_AS(UniformRandomWalkAppT<8>, "UniformRandomWalk8")
