// The compile-time App contract of the sampling engine, for gfx950.
//
// An application is a stateless struct (the engine constructs it on the fly as App())
// with the member functions of the reference's apps (example/uniformRandWalk.cu:15-93):
//   steps(), stepSize(k), next(...), samplingType(), outputFormat(), numSamples(CSR*),
//   initialSample(idx, CSR*, SampleType&), initialSampleSize(CSR*), hasExplicitTransits(),
//   stepTransits(...), initializeSample(CSR*, id).
// This header supplies, in the global namespace and under the spellings those app sources
// use, every type and helper they refer to: VertexID / VertexID_t / EdgePos_t, CSR and
// CSRPartition, SamplingType / OutputFormat, RandNumGen::rand_int, utils::binarySearch and
// the random-state handle.  The handle is the engine's own Philox cursor (nd::RandState);
// it only carries the name the app signature spells.  No vendor RNG library is involved.
//
// Device translation units (hipcc) see the real qualifiers.  A host-only translation unit
// (g++: the host API header, checkers that call an App's next() in a plain CPU loop) sees
// __host__ / __device__ / __forceinline__ as empty words, so the same App source compiles as
// ordinary C++.
#pragma once

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#else
#include <math.h>
#ifndef __host__
#define __host__
#endif
#ifndef __device__
#define __device__
#endif
#ifndef __forceinline__
#define __forceinline__ inline
#endif
#endif
#include <stdint.h>

#include <algorithm>
#include <vector>

#include "nd_philox.hpp"

typedef int32_t VertexID;
typedef int32_t EdgePos_t;
typedef VertexID VertexID_t;

// src/nextdoor.cu:62-71
enum SamplingType { IndividualNeighborhood, CollectiveNeighborhood };
enum OutputFormat { SampledVertices, AdjacencyMatrix };
// src/nextdoor.cu:48
constexpr int ALL_NEIGHBORS = -1;

// Host-side graph in CSR form.  Plays the role of the reference's CSR class
// (src/csr.hpp:46-196) for the host members of an App (numSamples, initialSample ...).
// Stored as structure-of-arrays: row_ptr[V+1], col[E], weight[E], max_weight[V];
// the adjacency of every vertex is sorted ascending by (destination, weight) with
// duplicates kept (src/graph.hpp:38,156) and max_weight[v] = max(0, weights of v)
// (src/graph.hpp:71-80).
class CSR {
 public:
  typedef VertexID Edge;

  std::vector<EdgePos_t> row_ptr;
  std::vector<Edge> col;
  std::vector<float> weight;
  std::vector<float> max_weight;

  VertexID get_n_vertices() const { return row_ptr.empty() ? 0 : (VertexID)(row_ptr.size() - 1); }
  EdgePos_t get_n_edges() const { return (EdgePos_t)col.size(); }
  bool has_vertex(VertexID v) const { return 0 <= v && v < get_n_vertices(); }
  EdgePos_t n_edges_for_vertex(VertexID v) const { return row_ptr[v + 1] - row_ptr[v]; }
  EdgePos_t get_start_edge_idx(VertexID v) const { return row_ptr[v]; }
  // inclusive end, -1 for a vertex without edges (src/csr.hpp:75-77, 413-416)
  EdgePos_t get_end_edge_idx(VertexID v) const { return n_edges_for_vertex(v) == 0 ? -1 : row_ptr[v + 1] - 1; }
  const Edge* get_edges() const { return col.data(); }
  const float* get_weights() const { return weight.data(); }
};

// Device view of the graph, handed to App::next as `CSRPartition* csr`
// (accessor names of src/csr.hpp:198-385).  Lives in kernel arguments, not in
// constant memory.
class CSRPartition {
 public:
  const EdgePos_t* row_ptr;
  const CSR::Edge* edges;
  const float* weights;
  const float* max_weights;
  VertexID n_vertices;
  EdgePos_t n_edges;

  __host__ __device__ __forceinline__ VertexID get_n_vertices() const { return n_vertices; }
  __host__ __device__ __forceinline__ EdgePos_t get_n_edges() const { return n_edges; }
  __host__ __device__ __forceinline__ bool has_vertex(int v) const { return v >= 0 && v < n_vertices; }
  __host__ __device__ __forceinline__ EdgePos_t get_start_edge_idx(int v) const { return row_ptr[v]; }
  __host__ __device__ __forceinline__ EdgePos_t get_end_edge_idx(int v) const {
    const EdgePos_t b = row_ptr[v], e = row_ptr[v + 1];
    return e == b ? -1 : e - 1;
  }
  __host__ __device__ __forceinline__ EdgePos_t get_n_edges_for_vertex(VertexID v) const {
    return row_ptr[v + 1] - row_ptr[v];
  }
  __host__ __device__ __forceinline__ float get_max_weight(int v) const { return max_weights[v]; }
  __host__ __device__ __forceinline__ CSR::Edge get_edge(EdgePos_t idx) const { return edges[idx]; }
  __host__ __device__ __forceinline__ float get_weight(EdgePos_t idx) const { return weights[idx]; }
  __host__ __device__ __forceinline__ const CSR::Edge* get_edges() const { return edges; }
  __host__ __device__ __forceinline__ const float* get_weights() const { return weights; }
  __host__ __device__ __forceinline__ const CSR::Edge* get_edges(VertexID v) const { return edges + row_ptr[v]; }
  __host__ __device__ __forceinline__ const float* get_weights(VertexID v) const { return weights + row_ptr[v]; }

  // Optional exact edge index over all edges, built by the engine for apps that declare
  // kUsesEdgeLookup; nullptr otherwise.  Keys are (src << 32 | dst), empty slots all-ones.
  // The table is made of buckets of kEdgeBucket consecutive keys (32 bytes, aligned: one
  // bucket is fetched with two 16-byte loads, i.e. one memory round trip); a key lives in the
  // first bucket, counted from the one its hash names, that had room when it was inserted, and
  // a bucket fills from its first slot on.  With at most a quarter of the slots in use a
  // bucket holds one key on average and overflows into its neighbour for one key in some
  // hundreds: the answer nearly always takes ONE round trip, found or not.  (A table of
  // single keys, half full, needs 1.5 dependent round trips for a key that is there and 2.5
  // for one that is not - and a wavefront waits for its slowest lane.)
  static constexpr uint32_t kEdgeBucket = 4;
  struct alignas(16) EdgeKeyPair {  // half a bucket: one 16-byte load
    unsigned long long x, y;
  };
  const unsigned long long* edge_table;
  uint32_t edge_table_mask;  // number of buckets - 1 (a power of two)

  __host__ __device__ __forceinline__ static uint32_t edge_hash(uint32_t src, uint32_t dst) {
    uint32_t h = src * 0x9E3779B1u ^ dst * 0x85EBCA77u;
    h ^= h >> 15;
    h *= 0x2C1B3C6Du;
    h ^= h >> 12;
    h *= 0x297A2D39u;
    h ^= h >> 15;
    return h;
  }

  // Is dst in the adjacency of src?  The reference answers with a binary search of the
  // sorted adjacency (src/csr.hpp:342-359); with the edge index present the same answer
  // comes from the key's bucket instead of log2(degree) dependent loads.
  __host__ __device__ __forceinline__ bool has_edge_logn(VertexID src, VertexID dst) const {
    if (edge_table != nullptr) {
      const unsigned long long key = ((unsigned long long)(uint32_t)src << 32) | (uint32_t)dst;
      uint32_t bucket = edge_hash((uint32_t)src, (uint32_t)dst) & edge_table_mask;
      for (;;) {
        const EdgeKeyPair* keys = (const EdgeKeyPair*)(edge_table + (size_t)bucket * kEdgeBucket);
        // a bucket fills from its first slot on and holds one key on average: the first half
        // decides 9 tests in 10, and the second half is then in the cache the first came through
        const EdgeKeyPair first = keys[0];
        if (first.x == key || first.y == key) return true;
        if (first.y == ~0ull) return false;
        const EdgeKeyPair second = keys[1];
        if (second.x == key || second.y == key) return true;
        if (second.y == ~0ull) return false;  // the bucket has room: the key was never pushed past it
        bucket = (bucket + 1) & edge_table_mask;
      }
    }
    EdgePos_t l = row_ptr[src];
    EdgePos_t r = row_ptr[src + 1] - 1;
    while (l <= r) {
      const EdgePos_t m = l + (r - l) / 2;
      const CSR::Edge e = edges[m];
      if (e == dst) return true;
      if (e < dst) l = m + 1; else r = m - 1;
    }
    return false;
  }
};

// The random-state handle named in App::next / App::stepTransits.
typedef nd::RandState curandState;

// Uniform variate in [0, 1) from the engine's Philox cursor.
__host__ __device__ __forceinline__ float curand_uniform(curandState* state) { return state->next_uniform(); }

// src/rand_num_gen.cuh:117-122
struct RandNumGen {
  __host__ __device__ __forceinline__ static EdgePos_t rand_int(curandState* state, const EdgePos_t n) {
    return nd::rand_int_from_uniform(state->next_uniform(), n);
  }
};

namespace utils {
// src/utils.hpp:30-48
template <typename F, typename T>
__host__ __device__ __forceinline__ bool binarySearch(F& array, T x, int size) {
  EdgePos_t l = 0;
  EdgePos_t r = size - 1;
  while (l <= r) {
    const EdgePos_t m = l + (r - l) / 2;
    const auto probe = array[m];
    if (probe == x) return true;
    if (probe < x) l = m + 1; else r = m - 1;
  }
  return false;
}
}  // namespace utils

namespace nd {

// Adjacency of the current transit staged in LDS, all of it (a transit whose adjacency does
// not fit is not given to the workgroup class).  One of the EdgeArray / WeightArray types an
// App::next is instantiated with (the other is a plain pointer); only operator[] is required
// (the reference's CachedArray, src/nextdoor.cu:76-124, plays this role).  The array is held
// as a pointer in the LDS address space, so reads of it are plain LDS loads: no generic-pointer
// test, and no branch to a copy in memory whose possible load every LDS read would wait for.
#if defined(__HIPCC__)
template <typename T>
struct LdsArray {
  typedef const __attribute__((address_space(3))) T* LdsPointer;
  LdsPointer lds;
  __device__ __forceinline__ explicit LdsArray(const T* lds_array) : lds((LdsPointer)lds_array) {}
  __device__ __forceinline__ T operator[](EdgePos_t i) const { return lds[i]; }
};
#endif

// Optional compile-time hints an App may carry; absent members mean `false`.
//   static constexpr bool kUsesEdgeWeights = true;  -> next() reads transitEdgeWeights: the
//        engine keeps an interleaved (destination, weight) copy of the edges so that one
//        8-byte record serves both arrays, and stages weights in LDS as well
//   static constexpr bool kUsesEdgeLookup = true;   -> next() calls csr->has_edge_logn: the
//        engine builds the exact edge index behind it
template <typename App, typename = void>
struct app_uses_weights { static constexpr bool value = false; };
template <typename App>
struct app_uses_weights<App, decltype((void)App::kUsesEdgeWeights)> { static constexpr bool value = App::kUsesEdgeWeights; };
template <typename App, typename = void>
struct app_uses_edge_lookup { static constexpr bool value = false; };
template <typename App>
struct app_uses_edge_lookup<App, decltype((void)App::kUsesEdgeLookup)> { static constexpr bool value = App::kUsesEdgeLookup; };

// Interleaved edge record and the two array views over it: transitEdges[x] and
// transitEdgeWeights[x] read the two halves of one 8-byte record, i.e. one memory line
// instead of one line in each of two arrays.
struct EdgeRecord {
  VertexID dst;
  float weight;
};

struct PairedEdgeIds {
  const EdgeRecord* base;
  __device__ __forceinline__ VertexID operator[](EdgePos_t i) const { return base[i].dst; }
};

struct PairedEdgeWeights {
  const EdgeRecord* base;
  __device__ __forceinline__ float operator[](EdgePos_t i) const { return base[i].weight; }
};

}  // namespace nd

// Registry name of an App that is compiled into libnextdoor_amd.so (nullptr: it is not): how
// the template spellings of the host API (include/libNextDoor_amd.hpp) find the library's
// instantiation for an App type.  Declared next to the App with ND_APP_REGISTERED_AS.
template <class App>
struct NextDoorAppName {
  static const char* name() { return nullptr; }
};
#define ND_APP_REGISTERED_AS(App, literal)             \
  template <>                                           \
  struct NextDoorAppName<App> {                         \
    static const char* name() { return literal; }       \
  };

// The opaque graph handle of the C ABI (include/nextdoor_amd.h) is the host CSR above: C++
// callers may use an nd_graph* as the CSR* the reference's host functions pass around
// (loadGraph returns it, App::numSamples / initialSample receive it).
struct nd_graph : CSR {};
