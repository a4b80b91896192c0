// Layer-wise (CollectiveNeighborhood) applications on the App contract.
//
//   LayerSamplingAppT       the reference's FastGCNSamplingApp and ImportanceSampleApp (LADIES),
//                           src/apps/fastgcn/fastgcnSampling.cu:1-100 and
//                           src/apps/ladies/ladiessampling.cu:1-100: identical bodies that draw
//                           every layer vertex uniformly from ALL vertices and record which
//                           transits it is adjacent to.  Sizes are template parameters where
//                           the reference has macros (NUM_LAYERS 5, 64 x 64, NUM_SAMPLES 10000).
//   FastGCNImportanceAppT   not in the reference: draws from the distinct vertices of the
//                           union neighbourhood with probability proportional to degree^2.
#pragma once

#include "nd_contract.hpp"

// Adjacency-matrix scratch of one sample, laid out as the reference's FastGCNSample /
// ImportanceSample (fastgcnSampling.cu:6-13): entry [step][i * kBatch + nbr] describes the
// pair (transit i, sampled vertex nbr) of that step.
template <int kLayers, int kBatch>
class LayerSampleT {
 public:
  int adjacencyMatrixLen[kLayers];
  int adjacencyMatrixRow[kLayers][kBatch * kBatch];
  int adjacencyMatrixCol[kLayers][kBatch * kBatch];
  int adjacencyMatrixVal[kLayers][kBatch * kBatch];
};

namespace nd {
namespace apps {

// What the engine hands a CollectiveNeighborhood app's next() as transitEdges /
// transitEdgeWeights / numEdges:
//   kConcatenated  the adjacencies of the sample's transits, concatenated (ids, float weights)
//   kDistinctByDegreeSquared  transitEdges is a view of the distinct ids of that neighbourhood
//                  weighted by degree(id)^2: total() is the sum of the weights and
//                  first_exceeding(t) the smallest id whose running sum (ids ascending) exceeds t;
//                  numEdges = how many distinct ids there are; no weight array
//   kRankedByLadiesImportance  the distinct ids ordered by descending Efraimidis-Spirakis key
//                  for the LADIES importance (squared column norm of the row-normalised
//                  adjacency restricted to the transits); no weights
enum NeighborhoodForm { kConcatenated = 0, kDistinctByDegreeSquared = 1, kRankedByLadiesImportance = 2 };

// The form an App's next() takes the collective neighbourhood in: App::kNeighborhoodForm, or the
// concatenation for an App that does not say (the reference's layer-wise apps, whose next() is
// handed the concatenated adjacencies and never looks at them: fastgcnSampling.cu:23-47).
template <class App, class = void>
struct neighborhood_form_of { static constexpr int value = kConcatenated; };
template <class App>
struct neighborhood_form_of<App, decltype((void)App::kNeighborhoodForm)> { static constexpr int value = App::kNeighborhoodForm; };

template <int kLayers, int kBatch, int kNumSamples>
struct LayerCommon {
  __host__ __device__ int steps() { return kLayers; }
  __host__ __device__ int stepSize(int) { return kBatch; }
  __host__ __device__ int samplingType() { return SamplingType::CollectiveNeighborhood; }
  __host__ __device__ OutputFormat outputFormat() { return AdjacencyMatrix; }
  __host__ EdgePos_t numSamples(CSR*) { return kNumSamples; }
  __host__ __device__ EdgePos_t initialSampleSize(CSR*) { return kBatch; }
  __host__ __device__ bool hasExplicitTransits() { return false; }

  template <class SampleType>
  __device__ VertexID_t stepTransits(int, const VertexID_t, SampleType&, int, curandState*) {
    return -1;
  }
};

}  // namespace apps
}  // namespace nd

template <int kLayers, int kBatch, int kNumSamples>
struct LayerSamplingAppT : nd::apps::LayerCommon<kLayers, kBatch, kNumSamples> {
  static constexpr bool kUsesEdgeLookup = true;
  static constexpr int kNeighborhoodForm = nd::apps::kConcatenated;

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int step, CSRPartition* csr, const VertexID* transits, const VertexID,
                                  SampleType* sample, const float, EdgeArray&, WeightArray&, const EdgePos_t,
                                  const VertexID_t neighbrID, curandState* state) {
    const VertexID id = RandNumGen::rand_int(state, csr->get_n_vertices());
    for (int i = 0; i < kBatch; i++) {
      const bool adjacent = csr->has_edge_logn(transits[i], id);
      const int at = i * kBatch + neighbrID;
      sample->adjacencyMatrixRow[step][at] = adjacent ? i : -1;
      sample->adjacencyMatrixCol[step][at] = adjacent ? neighbrID : -1;
    }
    return id;
  }

  // roots of sample s: kBatch consecutive vertex ids, wrapping around (fastgcnSampling.cu:75-85)
  template <class SampleType>
  __host__ std::vector<VertexID_t> initialSample(int sampleIdx, CSR* graph, SampleType&) {
    std::vector<VertexID_t> roots(kBatch);
    for (int i = 0; i < kBatch; i++) roots[i] = (VertexID_t)(((int64_t)sampleIdx * kBatch + i) % graph->get_n_vertices());
    return roots;
  }

  template <class SampleType>
  __host__ SampleType initializeSample(CSR*, const VertexID_t) {
    return SampleType();  // all zero: adjacencyMatrixLen[] = 0 as in fastgcnSampling.cu:87-95
  }
};

// FastGCN-style importance sampling: every layer draws kBatch vertices, independently and
// with replacement, from the distinct vertices D of the union neighbourhood of the previous
// layer, vertex v with probability degree(v)^2 / sum_{D} degree^2 (the squared degree
// normalised over D).  Exact integer inverse CDF: r = top 24 bits of the slot's first
// Philox word, target = (r * total) >> 24, pick the first id (ascending) whose running sum
// exceeds it.
// Roots of a batch are drawn uniformly from all vertices from a fixed Philox stream.
template <int kLayers, int kBatch, int kNumSamples>
struct FastGCNImportanceAppT : nd::apps::LayerCommon<kLayers, kBatch, kNumSamples> {
  static constexpr int kNeighborhoodForm = nd::apps::kDistinctByDegreeSquared;
  static constexpr uint64_t kRootSeed = 0x46475243ull;  // "FGRC"
  static constexpr uint32_t kRootStream = 0x524F4F54u;  // "ROOT"

  __host__ __device__ OutputFormat outputFormat() { return SampledVertices; }

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int, CSRPartition*, const VertexID*, const VertexID, SampleType*, const float,
                                  EdgeArray& distinctByDegreeSquared, WeightArray&, const EdgePos_t numDistinct,
                                  const VertexID_t, curandState* state) {
    if (numDistinct == 0) return -1;
    const uint64_t total = distinctByDegreeSquared.total();
    if (total == 0) return -1;
    const uint64_t r = state->next_word() >> 8;
    // (r * total) >> 24 with the 88-bit product held as (hi, lo)
    const uint64_t lo = r * total;
    const uint64_t hi = __umul64hi(r, total);
    const uint64_t target = (hi << 40) | (lo >> 24);
    return distinctByDegreeSquared.first_exceeding(target);
  }

  template <class SampleType>
  __host__ std::vector<VertexID_t> initialSample(int sampleIdx, CSR* graph, SampleType&) {
    std::vector<VertexID_t> roots(kBatch);
    for (int i = 0; i < kBatch; i++) {
      const float u = nd::uniform_at(kRootSeed, (uint64_t)sampleIdx * kBatch + i, kRootStream, 0);
      roots[i] = nd::rand_int_from_uniform(u, graph->get_n_vertices());
    }
    return roots;
  }

  template <class SampleType>
  __host__ SampleType initializeSample(CSR*, const VertexID_t) {
    return SampleType();
  }
};

// LADIES-style layer-dependent importance sampling WITHOUT replacement.  With U the
// previous layer, importance(v) = sum over edges u -> v, u in U, of (w_uv * (1 / rowsum(u)))^2 (the inverse rounded to float once per row).
// The engine computes it over the collective neighbourhood, draws one Efraimidis-Spirakis
// key log2(uniform) / importance per distinct vertex (uniform from Philox, four consecutive
// vertices of a sample to a block) and hands next() the vertices in descending key order: the first
// stepSize(k) of them are a weighted sample without replacement, in selection order.
template <int kLayers, int kBatch, int kNumSamples>
struct LadiesImportanceAppT : FastGCNImportanceAppT<kLayers, kBatch, kNumSamples> {
  static constexpr int kNeighborhoodForm = nd::apps::kRankedByLadiesImportance;

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ inline VertexID next(int, CSRPartition*, const VertexID*, const VertexID, SampleType*, const float,
                                  EdgeArray& rankedIds, WeightArray&, const EdgePos_t numDistinct,
                                  const VertexID_t neighbrID, curandState*) {
    return neighbrID < numDistinct ? rankedIds[neighbrID] : -1;
  }
};

class LayerNoState {};

// The reference's names and sizes (left out with ND_NO_REFERENCE_APP_NAMES, for a translation
// unit that brings the reference's own structs of these names).
#ifndef ND_NO_REFERENCE_APP_NAMES
typedef LayerSampleT<5, 64> FastGCNSample;
typedef LayerSamplingAppT<5, 64, 10000> FastGCNSamplingApp;
typedef LayerSampleT<5, 64> ImportanceSample;
typedef LayerSamplingAppT<5, 64, 10000> ImportanceSampleApp;

// FastGCNSamplingApp and ImportanceSampleApp are one type, as the reference's two apps are one text
ND_APP_REGISTERED_AS(FastGCNSamplingApp, "FastGCN")
#endif
