// Host-side graph ingest and seeded synthetic graphs for the sampling engine.
//
// CSR construction follows the reference's loaders and csr_from_graph
// (src/graph.hpp:106-159, src/csr.hpp:399-424): the adjacency of every vertex is sorted
// ascending by (destination, weight), duplicate edges are kept, vertex count is the
// largest id seen plus one, and max_weight[v] = max(0, weights of v) (src/graph.hpp:71-80).
// The binary edge list is a sequence of 12-byte records {int32 src, int32 dst, float32 w}.
#pragma once

#include <stdint.h>

#include <string>

#include "nd_contract.hpp"

namespace nd {

// Builds `out` from n edges (src[i] -> dst[i], weight w[i]).  n_vertices <= 0: use the
// largest id + 1.  Returns 0, or a negative value with *error set.
int csr_from_edges(CSR& out, int32_t n_vertices, size_t n, const int32_t* src, const int32_t* dst, const float* w,
                   std::string* error);

// Builds `out` from caller-supplied CSR arrays (adjacency must already be sorted per
// vertex); computes max_weight.  weight == nullptr: all ones.
int csr_from_arrays(CSR& out, int32_t n_vertices, int64_t n_edges, const int32_t* row_ptr, const int32_t* col,
                    const float* weight, std::string* error);

// loadGraph (src/nextdoor.cu:1845-1891): graph_type "edge-list" with format "binary" or
// "text" ("src dst [weight]" per line), or "adj-list" with "text" ("v n1 n2 ..." per line).
int load_graph_file(CSR& out, const char* path, const char* graph_type, const char* graph_format,
                    std::string* error);

// R-MAT (Chakrabarti et al.): 2^scale vertices, edge_factor * 2^scale generated edges,
// quadrant probabilities a, b, c (d = 1 - a - b - c), one Philox uniform per level keyed
// by (seed, edge index).  Weights are uniform in [1, 5).  symmetrise adds the reverse of
// every edge with the same weight.
int generate_rmat(CSR& out, int scale, int edge_factor, double a, double b, double c, uint64_t seed,
                  bool symmetrise, std::string* error);

// Chung-Lu style power-law graph: n_edges directed edges whose endpoints are drawn
// independently with probability proportional to (i + 1)^(-1 / (exponent - 1)).
// Weights are uniform in [1, 5).
int generate_chung_lu(CSR& out, int32_t n_vertices, int64_t n_edges, double exponent, uint64_t seed,
                      std::string* error);

}  // namespace nd
