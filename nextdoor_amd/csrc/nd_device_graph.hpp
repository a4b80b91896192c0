// The graph as the device sees it: CSR arrays plus the derived structures an app asks for.
//
// Stands for transferCSRToGPUs / copyPartitionToGPU of the reference
// (src/nextdoor.cu:1893-1911, src/utils.hpp:378-395): the whole graph is resident on the
// one device.  Structure of arrays instead of the reference's 16-byte vertex record
// (src/csr.hpp:49-79).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

#include "nd_contract.hpp"

namespace nd {

__device__ __forceinline__ VertexID source_of_edge(const EdgePos_t* row_ptr, VertexID n_vertices, EdgePos_t e) {
  // largest v with row_ptr[v] <= e
  VertexID lo = 0, hi = n_vertices;
  while (hi - lo > 1) {
    const VertexID mid = lo + (hi - lo) / 2;
    if (row_ptr[mid] <= e) lo = mid; else hi = mid;
  }
  return lo;
}

// One lane per edge: the key goes into the first free slot of the first bucket with room,
// counted from the bucket its hash names.  Slots of a bucket are tried in order, so a bucket
// fills from its first slot on; a duplicate edge finds its key on the way and stops.
__global__ void build_edge_table(CSRPartition csr, unsigned long long* table, uint32_t bucket_mask) {
  const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= (size_t)csr.n_edges) return;
  const VertexID src = source_of_edge(csr.row_ptr, csr.n_vertices, (EdgePos_t)e);
  const VertexID dst = csr.edges[e];
  const unsigned long long key = ((unsigned long long)(uint32_t)src << 32) | (uint32_t)dst;
  uint32_t bucket = CSRPartition::edge_hash((uint32_t)src, (uint32_t)dst) & bucket_mask;
  for (;;) {
    unsigned long long* slots = table + (size_t)bucket * CSRPartition::kEdgeBucket;
    for (uint32_t i = 0; i < CSRPartition::kEdgeBucket; ++i) {
      const unsigned long long seen = atomicCAS(&slots[i], ~0ull, key);
      if (seen == ~0ull || seen == key) return;  // inserted, or a duplicate edge already there
    }
    bucket = (bucket + 1) & bucket_mask;
  }
}

__global__ void build_paired_edges(const CSR::Edge* col, const float* weight, size_t n, EdgeRecord* out) {
  const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e < n) out[e] = EdgeRecord{col[e], weight[e]};
}

class DeviceGraph {
 public:
  CSRPartition view{};
  EdgeRecord* paired = nullptr;  // interleaved (dst, weight) copy, when asked for

  ~DeviceGraph() { release(); }

  // Uploads the graph.  want_paired: also keep the interleaved edge records;
  // want_edge_table: also build the exact edge index behind CSRPartition::has_edge_logn.
  // Returns false and sets *error on failure.
  bool upload(const CSR* graph, bool want_paired, bool want_edge_table, std::string* error) {
    release();
    const size_t V = (size_t)graph->get_n_vertices();
    const size_t E = graph->col.size();
    if (V == 0) return fail(error, "graph has no vertices");
    if (E >= (size_t)INT32_MAX) return fail(error, "edge count does not fit int32 edge positions");
#define ND_GRAPH_TRY(expr)                                                              \
  do {                                                                                  \
    hipError_t e_ = (expr);                                                             \
    if (e_ != hipSuccess) return fail(error, std::string(#expr) + ": " + hipGetErrorString(e_)); \
  } while (0)
    ND_GRAPH_TRY(hipMalloc(&row_ptr_, sizeof(EdgePos_t) * (V + 1)));
    ND_GRAPH_TRY(hipMalloc(&col_, sizeof(VertexID) * (E ? E : 1)));
    ND_GRAPH_TRY(hipMalloc(&weight_, sizeof(float) * (E ? E : 1)));
    ND_GRAPH_TRY(hipMalloc(&max_weight_, sizeof(float) * V));
    ND_GRAPH_TRY(hipMemcpy(row_ptr_, graph->row_ptr.data(), sizeof(EdgePos_t) * (V + 1), hipMemcpyHostToDevice));
    if (E) {
      ND_GRAPH_TRY(hipMemcpy(col_, graph->col.data(), sizeof(VertexID) * E, hipMemcpyHostToDevice));
      ND_GRAPH_TRY(hipMemcpy(weight_, graph->weight.data(), sizeof(float) * E, hipMemcpyHostToDevice));
    }
    ND_GRAPH_TRY(hipMemcpy(max_weight_, graph->max_weight.data(), sizeof(float) * V, hipMemcpyHostToDevice));
    view.row_ptr = row_ptr_;
    view.edges = col_;
    view.weights = weight_;
    view.max_weights = max_weight_;
    view.n_vertices = (VertexID)V;
    view.n_edges = (EdgePos_t)E;
    view.edge_table = nullptr;
    view.edge_table_mask = 0;
    if (want_paired) {
      ND_GRAPH_TRY(hipMalloc(&paired, sizeof(EdgeRecord) * (E ? E : 1)));
      if (E) build_paired_edges<<<dim3((unsigned)((E + 255) / 256)), dim3(256)>>>(col_, weight_, E, paired);
      ND_GRAPH_TRY(hipGetLastError());
    }
    if (want_edge_table) {
      size_t slots = 16;  // power of two, at most a quarter full
      while (slots < 4 * E) slots <<= 1;
      const size_t buckets = slots / CSRPartition::kEdgeBucket;
      ND_GRAPH_TRY(hipMalloc(&edge_table_, sizeof(unsigned long long) * slots));
      ND_GRAPH_TRY(hipMemset(edge_table_, 0xFF, sizeof(unsigned long long) * slots));
      if (E) build_edge_table<<<dim3((unsigned)((E + 255) / 256)), dim3(256)>>>(view, edge_table_, (uint32_t)(buckets - 1));
      ND_GRAPH_TRY(hipGetLastError());
      view.edge_table = edge_table_;
      view.edge_table_mask = (uint32_t)(buckets - 1);
    }
    ND_GRAPH_TRY(hipDeviceSynchronize());
#undef ND_GRAPH_TRY
    return true;
  }

  void release() {
    free_one(row_ptr_);
    free_one(col_);
    free_one(weight_);
    free_one(max_weight_);
    free_one(paired);
    free_one(edge_table_);
    view = CSRPartition{};
  }

  const EdgePos_t* row_ptr() const { return row_ptr_; }

 private:
  static bool fail(std::string* error, const std::string& msg) {
    if (error) *error = msg;
    return false;
  }
  template <class T>
  static void free_one(T*& p) {
    if (p) (void)hipFree(p);
    p = nullptr;
  }

  EdgePos_t* row_ptr_ = nullptr;
  VertexID* col_ = nullptr;
  float* weight_ = nullptr;
  float* max_weight_ = nullptr;
  unsigned long long* edge_table_ = nullptr;
};

}  // namespace nd
