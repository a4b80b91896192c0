// Host-side validation of sampling results against the graph (the library's `-c` option).
//
// Follows the rules of the reference's validators, src/check_results.cu:
//   checkSampledVerticesResult (162-299): a vertex sampled at step k must be adjacent to a
//     valid vertex the sample held at step k-1 (the roots for k = 0), and a step may come out
//     empty only when the vertices of step k-1 have no edges at all;
//   checkAdjacencyMatrixResult (46-160): for the layer-wise apps that record an adjacency
//     matrix per layer, every recorded (row, col) is an edge of the graph and every edge of the
//     graph between two consecutive layers is recorded.
// Differences: all steps are checked (the reference stops after four), adjacency is tested by
// binary search in the CSR rows instead of one hash set per vertex, and the first violation is
// reported as text instead of printed.
#pragma once

#include <stdint.h>

#include <string>
#include <vector>

#include "nd_contract.hpp"

namespace nd {

struct SampleShape {
  std::vector<int> step_size;  // m_k for every step
  int initial_size = 1;        // roots per sample
  bool collective = false;     // CollectiveNeighborhood: step k holds m_k vertices, else T_k * m_k
};

// final_samples: [n_samples][F] in the engine's layout; initial: [n_samples][initial_size].
// Returns true when every sample passes; else false with *report naming the first violation.
bool check_sampled_vertices(const CSR& graph, const SampleShape& shape, int64_t n_samples, const int32_t* initial,
                            const int32_t* final_samples, int32_t invalid, std::string* report);

// rows / cols of sample s and layer k start at rows[s * state_stride + k * B * B] (B = step
// size = roots per sample); entry [i * B + nbr] is (i, nbr) when transit i of the layer is
// adjacent to the layer's nbr-th vertex, else (-1, -1).
bool check_layer_adjacency_matrix(const CSR& graph, const SampleShape& shape, int64_t n_samples,
                                  const int32_t* initial, const int32_t* final_samples, const int32_t* rows,
                                  const int32_t* cols, size_t state_stride, int32_t invalid, std::string* report);

// checkMVSResult / checkSubGraphResult (src/tests/multiGPU/mvs.cu:12-101,
// src/tests/multiGPU/clustergcn.cu:10-93): sample s owns entries [list_start[s], list_start[s+1])
// of rows / cols and the vertices[s * vertices_per_sample ...] it was built from.  Every listed
// (row, col) must be an edge of the graph, and every edge of the graph between two different
// vertices of the sample must be listed.
bool check_subgraph_edge_lists(const CSR& graph, int64_t n_samples, int vertices_per_sample, const int32_t* vertices,
                               const uint32_t* list_start, const int32_t* rows, const int32_t* cols,
                               std::string* report);

}  // namespace nd
