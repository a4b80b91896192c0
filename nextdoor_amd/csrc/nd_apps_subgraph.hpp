// Subgraph-extraction applications on the App contract: samples whose result is a list of
// edges (row, col) in storage shared by all samples, not a row of sampled vertices.
//
//   MVSSamplingAppT       src/apps/mvs/mvsSampling.cu:1-103: a sample is a batch of 32
//                         consecutive vertices; its edge list is every edge leaving the batch.
//   SubGraphSamplingAppT  src/apps/clustergcn/clusterGCNSampling.cu:1-128 (ClusterGCN): a sample is
//                         two clusters of 16 consecutive vertices; its edge list is the
//                         subgraph the 32 vertices induce.
//
// The reference's next() appends to the sample's list with atomicAdd(&sample->length, 1), so
// the order inside a list depends on the schedule, and it reserves the list's room by host
// arithmetic (MVS) or a global atomic (ClusterGCN).  Here next() hands every edge to
// sample->emit(row, col) and the engine (nd_subgraph_engine.hpp) runs next() twice - once to
// count, once to write at offsets from a prefix sum - so a list is packed, starts where the
// lists of the samples before it end, and has a fixed order (by step, then by groups of 64
// consecutive (transit, neighbour slot) lanes, the lanes' edges interleaved inside a group):
// the same bytes whatever the schedule.  `sample` is the engine's
// per-lane view: sample->state() is the stored SampleType (the sample's vertices).
#pragma once

#include <algorithm>

#include "nd_contract.hpp"

// The stored state of a sample: its vertices (MVSSample::vertices, SubGraphSample::vertices).
// Position and length of its edge list are kept by the engine, not in the state.
template <int kVertices>
class SubgraphSampleT {
 public:
  VertexID_t vertices[kVertices];
};

namespace nd {
namespace apps {

template <int kVertices>
struct SubgraphCommon {
  static constexpr bool kListsEdges = true;  // next() hands edges to sample->emit: the edge-list engine
  __host__ __device__ int samplingType() { return SamplingType::IndividualNeighborhood; }
  __host__ __device__ OutputFormat outputFormat() { return AdjacencyMatrix; }
  __host__ __device__ EdgePos_t initialSampleSize(CSR*) { return kVertices; }
  __host__ __device__ bool hasExplicitTransits() { return false; }

  // the reference's sample counts (mvsSampling.cu:57-60, clusterGCNSampling.cu:84-87): eight
  // samples' worth of vertices per vertex of the graph, capped
  __host__ static EdgePos_t samples_for(CSR* graph, int64_t cap) {
    if (graph->get_n_edges() > 100000000) return 800000;
    const int64_t wanted = ((int64_t)graph->get_n_vertices() * 8 + kVertices - 1) / kVertices;
    return (EdgePos_t)std::min<int64_t>(cap, wanted);
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

}  // namespace apps
}  // namespace nd

// MVS: one step; lane `neighbrID` of transit v copies the edges neighbrID, neighbrID + 32, ...
// of v (mvsSampling.cu:36-43).  No vertex is sampled: every final-sample entry stays INVALID.
template <int kBatch>
struct MVSSamplingAppT : nd::apps::SubgraphCommon<kBatch> {
  __host__ __device__ int steps() { return 1; }
  __host__ __device__ int stepSize(int) { return kBatch; }

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ __forceinline__ VertexID next(int, CSRPartition*, const VertexID* transits, const VertexID, SampleType* sample,
                                  const float, EdgeArray& transitEdges, WeightArray&, const EdgePos_t numEdges,
                                  const VertexID_t neighbrID, curandState*) {
    const VertexID_t row = transits[0];
    EdgePos_t e = neighbrID;
    // a hub keeps its lanes busy for thousands of rounds: fetch eight edges before handing
    // them over, so that eight loads are under way instead of one
    for (; e + 7 * kBatch < numEdges; e += 8 * kBatch) {
      VertexID_t ahead[8];
#pragma unroll
      for (int i = 0; i < 8; i++) ahead[i] = transitEdges[e + i * kBatch];
#pragma unroll
      for (int i = 0; i < 8; i++) sample->emit(row, ahead[i]);
    }
    for (; e < numEdges; e += kBatch) sample->emit(row, transitEdges[e]);
    return -1;
  }

  __host__ EdgePos_t numSamples(CSR* graph) { return this->samples_for(graph, 1500000); }

  // batch s = vertices s * 32 ... s * 32 + 31, wrapping around (mvsSampling.cu:74-94)
  template <class SampleType>
  __host__ std::vector<VertexID_t> initialSample(int sampleIdx, CSR* graph, SampleType& sample) {
    std::vector<VertexID_t> batch(kBatch);
    for (int i = 0; i < kBatch; i++) {
      batch[i] = (VertexID_t)(((int64_t)sampleIdx * kBatch + i) % graph->get_n_vertices());
      sample.vertices[i] = batch[i];
    }
    return batch;
  }
};

// ClusterGCN: an app with explicit transits, as in the reference: the transits of step 1 are
// the sample's vertices, named by stepTransits (clusterGCNSampling.cu:89-104), whatever step 0
// returned (the reference uses step 0 to add up the room its list may need; here it returns the
// vertex).  At step 1 lane `neighbrID` of transit v1 tests the edge v1 -> vertices[neighbrID]
// with a binary search of v1's adjacency (clusterGCNSampling.cu:46-67).  The final sample holds
// the 32 vertices (those with edges), then INVALID.
template <int kClusterVertices, int kClusters>
struct SubGraphSamplingAppT : nd::apps::SubgraphCommon<kClusterVertices * kClusters> {
  static constexpr int kVertices = kClusterVertices * kClusters;

  __host__ __device__ int steps() { return 2; }
  __host__ __device__ int stepSize(int k) { return k == 0 ? 1 : kVertices; }

  template <typename SampleType, typename EdgeArray, typename WeightArray>
  __device__ __forceinline__ VertexID next(int step, CSRPartition*, const VertexID* transits, const VertexID,
                                  SampleType* sample, const float, EdgeArray& transitEdges, WeightArray&,
                                  const EdgePos_t numEdges, const VertexID_t neighbrID, curandState*) {
    const VertexID_t v1 = transits[0];
    if (step == 0) return v1;
    const VertexID_t v2 = sample->state().vertices[neighbrID];
    if (utils::binarySearch(transitEdges, v2, numEdges)) sample->emit(v1, v2);
    return -1;
  }

  __host__ __device__ bool hasExplicitTransits() { return true; }

  // clusterGCNSampling.cu:95-104, without the global atomic that reserves the list's room
  template <class SampleType>
  __device__ VertexID_t stepTransits(int, const VertexID_t, SampleType& sample, int transitIdx, curandState*) {
    return sample.state().vertices[transitIdx];
  }

  // clusters are runs of 16 consecutive vertex ids (the reference's foo(),
  // clusterGCNSampling.cu:166-172); a graph smaller than one cluster yields no samples
  __host__ EdgePos_t numSamples(CSR* graph) {
    return graph->get_n_vertices() < kClusterVertices ? 0 : this->samples_for(graph, 2000000);
  }

  // sample s = clusters 2s and 2s + 1, wrapping around (clusterGCNSampling.cu:107-122)
  template <class SampleType>
  __host__ std::vector<VertexID_t> initialSample(int sampleIdx, CSR* graph, SampleType& sample) {
    const int64_t n_clusters = graph->get_n_vertices() / kClusterVertices;
    std::vector<VertexID_t> members;
    for (int i = 0; i < kClusters; i++) {
      const int64_t cluster = ((int64_t)sampleIdx * kClusters + i) % n_clusters;
      for (int v = 0; v < kClusterVertices; v++) {
        sample.vertices[members.size()] = (VertexID_t)(cluster * kClusterVertices + v);
        members.push_back((VertexID_t)(cluster * kClusterVertices + v));
      }
    }
    return members;
  }
};

typedef SubgraphSampleT<32> MVSSample;
typedef MVSSamplingAppT<32> MVSSamplingApp;
typedef SubgraphSampleT<32> SubGraphSample;
typedef SubGraphSamplingAppT<16, 2> SubGraphSamplingAppI;

ND_APP_REGISTERED_AS(MVSSamplingApp, "MVS")
ND_APP_REGISTERED_AS(SubGraphSamplingAppI, "ClusterGCN")
