// TEST INFRASTRUCTURE ONLY.  The reference's own application sources, compiled from where they
// lie under the reference tree (REFERENCE_ROOT, given by oracle/Makefile; nothing is copied into
// this repository) as ordinary host C++ against the App contract header, and run in a plain
// CPU loop: sample after sample, transit after transit, one App::next() call per output slot
// with the output's own Philox stream.  What comes out is what the reference's functor code
// itself computes for those draws; tests/test_reference_apps_host.py holds the oracle's
// restatement (oracle/nd_oracle.c) against it, byte for byte.
//
// The loop, the slot layout and the random streams are this repository's (the reference's are
// not reproducible: src/nextdoor.cu:229, 304, 473); the functors are the reference's, unchanged:
//   src/apps/khop/khop.cu               KHopApp, KHopSample
//   src/apps/randomwalks/randomWalks.cu DeepWalkApp, PPRApp, Node2VecApp, DummySample, Node2VecSample
//   src/apps/fastgcn/fastgcnSampling.cu FastGCNSamplingApp, FastGCNSample (5 layers of 64)
//   src/apps/ladies/ladiessampling.cu   ImportanceSampleApp, ImportanceSample (the same text under other names)
//   src/apps/layer/layerSampling.cu     LayerSamplingApp, LayerSample (k-hop with fan-outs 10, 25)
//   src/apps/multiRW/multiRW.cu         MultiRWApp, MultiRWSample (explicit transits: stepTransits)
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <vector>

#include "../nextdoor_amd/csrc/nd_contract.hpp"

using std::max;  // the app sources call max(float, float) unqualified, as CUDA lets them
using std::min;

#include REFERENCE_KHOP
#include REFERENCE_RANDOM_WALKS
#undef VERTICES_PER_SAMPLE  // each app source sets its own (1 for the walks and k-hop, 64 for FastGCN)
#include REFERENCE_FASTGCN
#include REFERENCE_LADIES  // the same four sizes again, with the same values
#undef VERTICES_PER_SAMPLE
#include REFERENCE_LAYER
#include REFERENCE_MULTIRW
#undef VERTICES_PER_SAMPLE
#define VERTICES_PER_SAMPLE 64  // for the loops below: the layer-wise apps' batch

namespace {

struct HostGraph {
  CSR csr;
  CSRPartition view;
};

template <class SampleType, class App>
int sample_individual(HostGraph& g, uint64_t seed, int64_t n_samples, const int32_t* initial, int32_t* final_samples,
                      int32_t* state_t) {
  App app;
  const int32_t invalid = g.csr.get_n_vertices();
  const int init = app.initialSampleSize(&g.csr);
  int64_t F = 0, per = init;
  for (int k = 0; k < app.steps(); ++k) { per *= app.stepSize(k); F += per; }
  for (int64_t s = 0; s < n_samples; ++s) {
    SampleType sample = app.template initializeSample<SampleType>(&g.csr, (VertexID_t)s);
    int32_t* out = final_samples + s * F;
    const int32_t* prev = initial + s * init;
    int64_t T = init, seg_base = 0;
    for (int k = 0; k < app.steps(); ++k) {
      const int m = app.stepSize(k);
      int32_t* seg = out + seg_base;
      for (int64_t j = 0; j < T; ++j) {
        const VertexID transit = prev[j];
        for (int nbr = 0; nbr < m; ++nbr) {
          int32_t neighbor = invalid;
          // next() only runs for a real transit that has edges (src/nextdoor.cu:250-262)
          if (transit != invalid && transit != -1 && g.view.get_n_edges_for_vertex(transit) != 0) {
            curandState rng;
            // steps that draw several outputs per transit use the grouped form of the stream
            if (m > 1) rng.reset_grouped(seed, (uint64_t)((s * T + j) * m + nbr), (uint32_t)k);
            else rng.reset(seed, (uint64_t)((s * T + j) * m + nbr), (uint32_t)k);
            const CSR::Edge* edges = g.view.get_edges(transit);
            const float* weights = g.view.get_weights(transit);
            const VertexID r = app.template next<SampleType, const CSR::Edge*, const float*>(
                k, &g.view, &transit, (VertexID)s, &sample, g.view.get_max_weight(transit), edges, weights,
                g.view.get_n_edges_for_vertex(transit), (VertexID_t)nbr, &rng);
            neighbor = r == -1 ? invalid : r;  // src/nextdoor.cu:288
          }
          seg[j * m + nbr] = neighbor;
        }
      }
      prev = seg;
      seg_base += T * m;
      T *= m;
    }
    if (state_t) {
      int32_t t = -1;
      if (sizeof(SampleType) >= sizeof(int32_t)) memcpy(&t, &sample, sizeof(int32_t));
      state_t[s] = t;
    }
  }
  return 0;
}

// The layer-wise apps of the reference (fastgcnSampling.cu, ladiessampling.cu: 5 layers of 64 from 64
// roots), sample by sample: next() for every slot of every layer with the slot's own stream.
template <class LayerSampleType, class LayerApp>
int sample_layers(int32_t n_vertices, int64_t n_edges, const int32_t* row_ptr, const int32_t* col, uint64_t seed,
                  int64_t n_samples, const int32_t* initial, int32_t* final_samples, int32_t* rows, int32_t* cols) {
  CSR csr;
  csr.row_ptr.assign(row_ptr, row_ptr + n_vertices + 1);
  csr.col.assign(col, col + n_edges);
  CSRPartition view = CSRPartition();
  view.row_ptr = csr.row_ptr.data();
  view.edges = csr.col.data();
  view.n_vertices = n_vertices;
  view.n_edges = (EdgePos_t)n_edges;
  view.edge_table = nullptr;
  LayerApp app;
  const int32_t invalid = n_vertices;
  const int layers = app.steps(), B = VERTICES_PER_SAMPLE;
  int F = 0;
  for (int k = 0; k < layers; ++k) F += app.stepSize(k);
  std::vector<LayerSampleType> one(1);
  for (int64_t s = 0; s < n_samples; ++s) {
    LayerSampleType& sample = one[0];
    memset(&sample, 0xFF, sizeof(sample));  // -1 everywhere: nothing recorded yet
    int32_t* row = final_samples + s * F;
    int base = 0;
    for (int k = 0; k < layers; ++k) {
      const int m = app.stepSize(k);
      // transits of a layer: the roots, then the layer before (src/nextdoor.cu:1402-1411)
      const VertexID* transits = k == 0 ? initial + s * B : row + base - app.stepSize(k - 1);
      for (int nbr = 0; nbr < m; ++nbr) {
        int32_t neighbor = invalid;
        if (transits[0] != invalid && transits[0] != -1) {  // src/nextdoor.cu:1421
          curandState rng;
          rng.reset(seed, (uint64_t)(s * m + nbr), (uint32_t)k);
          const CSR::Edge* no_edges = nullptr;
          const float* no_weights = nullptr;
          const VertexID r = app.template next<LayerSampleType, const CSR::Edge*, const float*>(
              k, &view, transits, (VertexID)s, &sample, 0.0f, no_edges, no_weights, 0, (VertexID_t)nbr, &rng);
          neighbor = r == -1 ? invalid : r;
        }
        row[base + nbr] = neighbor;
      }
      base += m;
    }
    memcpy(rows + s * layers * B * B, sample.adjacencyMatrixRow, sizeof(int32_t) * layers * B * B);
    memcpy(cols + s * layers * B * B, sample.adjacencyMatrixCol, sizeof(int32_t) * layers * B * B);
  }
  return 0;
}

}  // namespace

extern "C" {

enum { REF_KHOP = 0, REF_DEEPWALK = 1, REF_PPR = 2, REF_NODE2VEC = 3, REF_LAYER = 4 };

// steps, step sizes and samples of the reference app itself
int ref_app_shape(int app, int32_t n_vertices, int32_t* steps, int32_t* step_sizes, int64_t* n_samples) {
  CSR probe;
  probe.row_ptr.assign((size_t)n_vertices + 1, 0);
  auto fill = [&](auto a) {
    *steps = a.steps();
    for (int k = 0; k < a.steps(); ++k) step_sizes[k] = a.stepSize(k);
    *n_samples = a.numSamples(&probe);
    return 0;
  };
  switch (app) {
    case REF_KHOP: return fill(KHopApp());
    case REF_DEEPWALK: return fill(DeepWalkApp());
    case REF_PPR: return fill(PPRApp());
    case REF_NODE2VEC: return fill(Node2VecApp());
    case REF_LAYER: return fill(LayerSamplingApp());
    default: return -1;
  }
}

// final_samples[n_samples][F]; state_t (nullable): the first int of the sample state (Node2VecSample::t)
int ref_sample_individual(int app, int32_t n_vertices, int64_t n_edges, const int32_t* row_ptr, const int32_t* col,
                          const float* weight, const float* max_weight, uint64_t seed, int64_t n_samples,
                          const int32_t* initial, int32_t* final_samples, int32_t* state_t) {
  HostGraph g;
  g.csr.row_ptr.assign(row_ptr, row_ptr + n_vertices + 1);
  g.csr.col.assign(col, col + n_edges);
  g.csr.weight.assign(weight, weight + n_edges);
  g.csr.max_weight.assign(max_weight, max_weight + n_vertices);
  g.view = CSRPartition();
  g.view.row_ptr = g.csr.row_ptr.data();
  g.view.edges = g.csr.col.data();
  g.view.weights = g.csr.weight.data();
  g.view.max_weights = g.csr.max_weight.data();
  g.view.n_vertices = n_vertices;
  g.view.n_edges = (EdgePos_t)n_edges;
  g.view.edge_table = nullptr;
  switch (app) {
    case REF_KHOP: return sample_individual<KHopSample, KHopApp>(g, seed, n_samples, initial, final_samples, nullptr);
    case REF_DEEPWALK: return sample_individual<DummySample, DeepWalkApp>(g, seed, n_samples, initial, final_samples, nullptr);
    case REF_PPR: return sample_individual<DummySample, PPRApp>(g, seed, n_samples, initial, final_samples, nullptr);
    case REF_NODE2VEC: return sample_individual<Node2VecSample, Node2VecApp>(g, seed, n_samples, initial, final_samples, state_t);
    case REF_LAYER: return sample_individual<LayerSample, LayerSamplingApp>(g, seed, n_samples, initial, final_samples, nullptr);
    default: return -1;
  }
}

// The reference's FastGCN app (5 layers of 64 from 64 roots): final_samples[n_samples][320],
// rows / cols [n_samples][5][64 * 64] = adjacencyMatrixRow / adjacencyMatrixCol of the sample state.
int ref_sample_fastgcn(int32_t n_vertices, int64_t n_edges, const int32_t* row_ptr, const int32_t* col, uint64_t seed,
                       int64_t n_samples, const int32_t* initial, int32_t* final_samples, int32_t* rows, int32_t* cols) {
  return sample_layers<FastGCNSample, FastGCNSamplingApp>(n_vertices, n_edges, row_ptr, col, seed, n_samples, initial,
                                                          final_samples, rows, cols);
}

// ... and its LADIES app (src/apps/ladies/ladiessampling.cu), the same loop on ImportanceSampleApp.
int ref_sample_ladies(int32_t n_vertices, int64_t n_edges, const int32_t* row_ptr, const int32_t* col, uint64_t seed,
                      int64_t n_samples, const int32_t* initial, int32_t* final_samples, int32_t* rows, int32_t* cols) {
  return sample_layers<ImportanceSample, ImportanceSampleApp>(n_vertices, n_edges, row_ptr, col, seed, n_samples, initial,
                                                              final_samples, rows, cols);
}

// The reference's multi-dimensional random walk (src/apps/multiRW/multiRW.cu): NUM_ROOT_VERTICES
// walkers per sample, given in walkers[n_samples][NUM_ROOT_VERTICES] (in: where they start; out:
// where they are after the last step; the reference draws the starts with rand()).  Every step
// calls next() for the walker that is the transit and then, unless it is the last step,
// stepTransits(step + 1) with the same random state (src/nextdoor.cu:279-289).
// final_samples[n_samples][steps], last_root_idx[n_samples] = MultiRWSample::lastRootIdx.
int ref_multirw_shape(int32_t* n_roots, int32_t* steps) {
  *n_roots = NUM_ROOT_VERTICES;
  *steps = MultiRWApp().steps();
  return 0;
}

int ref_sample_multirw(int32_t n_vertices, int64_t n_edges, const int32_t* row_ptr, const int32_t* col, uint64_t seed,
                       int64_t n_samples, int32_t* walkers, int32_t* last_root_idx, int32_t* final_samples) {
  CSR csr;
  csr.row_ptr.assign(row_ptr, row_ptr + n_vertices + 1);
  csr.col.assign(col, col + n_edges);
  CSRPartition view = CSRPartition();
  view.row_ptr = csr.row_ptr.data();
  view.edges = csr.col.data();
  view.n_vertices = n_vertices;
  view.n_edges = (EdgePos_t)n_edges;
  view.edge_table = nullptr;
  MultiRWApp app;
  const int32_t invalid = n_vertices;
  const int steps = app.steps();
  for (int64_t s = 0; s < n_samples; ++s) {
    MultiRWSample sample;
    memcpy(sample.rootVertices, walkers + s * NUM_ROOT_VERTICES, sizeof(sample.rootVertices));
    sample.lastRootIdx = 0;
    VertexID transit = app.initialSample((int)s, &csr, sample)[0];
    for (int k = 0; k < steps; ++k) {
      int32_t neighbor = invalid;
      curandState rng;
      rng.reset(seed, (uint64_t)s, (uint32_t)k);
      if (transit != invalid && view.get_n_edges_for_vertex(transit) != 0) {
        const CSR::Edge* edges = view.get_edges(transit);
        const float* no_weights = nullptr;
        const VertexID r = app.template next<MultiRWSample, const CSR::Edge*, const float*>(
            k, &view, &transit, (VertexID)s, &sample, 0.0f, edges, no_weights, view.get_n_edges_for_vertex(transit), 0,
            &rng);
        neighbor = r == -1 ? invalid : r;
      }
      final_samples[s * steps + k] = neighbor;
      if (k != steps - 1 && transit != invalid) {
        const VertexID_t t = app.stepTransits(k + 1, (VertexID_t)s, sample, 0, &rng);
        transit = t == -1 ? invalid : t;
      }
    }
    memcpy(walkers + s * NUM_ROOT_VERTICES, sample.rootVertices, sizeof(sample.rootVertices));
    last_root_idx[s] = sample.lastRootIdx;
  }
  return 0;
}

}  // extern "C"
