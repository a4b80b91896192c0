/*
 * CPU oracle for the transit-parallel sampling path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the sampler semantics of plasma-umass/NextDoor
 * (file:line citations are relative to the reference checkout) evaluated the
 * obvious way: one sample after the other, one transit after the other.  It is
 * the checker for the HIP engine; nothing that ships may link, import or call it.
 * Only tests, the smoke check and the cpu_baseline leg of the benchmark use it.
 *
 * Parity status of each function is stated next to its declaration:
 *   "pinned by ..."     - an independent check exists in tests/ (KAT, closed form,
 *                         brute force, special case reducing to a library routine)
 *   "parity unpinned"   - no independent check pins the function.
 * A sampler that is this repository's own definition (the reference has no such app) says
 * so; what pins it is then its stated mathematical definition: a draw-by-draw evaluation
 * written apart from this file, and the distribution it must produce.
 */
#ifndef ND_ORACLE_H
#define ND_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NDO_MAX_STEPS 128

/* App identifiers (the structs under src/apps and example/ of the reference). */
enum ndo_app_kind {
  NDO_UNIFORM_WALK = 0,      /* example/uniformRandWalk.cu:27-37            */
  NDO_DEEPWALK = 1,          /* src/apps/randomwalks/randomWalks.cu:65-91   */
  NDO_PPR = 2,               /* src/apps/randomwalks/randomWalks.cu:93-125  */
  NDO_NODE2VEC = 3,          /* src/apps/randomwalks/randomWalks.cu:132-173 */
  NDO_WEIGHTED_NODE2VEC = 4, /* this repo's weighted variant (no counterpart in the reference);
                                pinned by a draw-by-draw trace and chi-square over all three biases */
  NDO_KHOP = 5,              /* src/apps/khop/khop.cu:10-23                 */
  NDO_LAYER_LITERAL = 6,     /* src/apps/fastgcn/fastgcnSampling.cu:23-47 and
                                src/apps/ladies/ladiessampling.cu:23-47 (identical bodies) */
  NDO_FASTGCN_IMPORTANCE = 7,/* this repo's degree^2 importance sampler; parity unpinned */
  NDO_LADIES_IMPORTANCE = 8  /* this repo's column-norm^2 sampler; parity unpinned */
};

typedef struct {
  int32_t n_vertices;
  int64_t n_edges;
  const int32_t* row_ptr;    /* [n_vertices+1]; adjacency of v is col[row_ptr[v] .. row_ptr[v+1]) */
  const int32_t* col;        /* sorted ascending by (dst, weight) per vertex, duplicates kept (graph.hpp:38,156) */
  const float* weight;
  const float* max_weight;   /* [n_vertices]; max(0, weights of v) (graph.hpp:71-80) */
} ndo_graph;

typedef struct {
  int kind;                       /* enum ndo_app_kind */
  int steps;                      /* App::steps() */
  int step_size[NDO_MAX_STEPS];   /* App::stepSize(k) */
  int initial_size;               /* App::initialSampleSize() */
  float p, q;                     /* node2vec parameters (reference hard-codes 2.0 / 0.5) */
} ndo_app_desc;

typedef struct {
  int64_t next_calls;     /* times the app's next() ran */
  int64_t draws;          /* uniform variates consumed */
  int64_t search_probes;  /* binary-search loop iterations */
  int64_t valid_outputs;  /* output slots != INVALID (reference: totalSampledVertices, nextdoor.cu:3284-3299) */
  int64_t edge_reads;     /* neighbour-id loads */
  int64_t weight_reads;   /* edge-weight loads */
  int64_t band_tests;     /* weighted node2vec: candidates whose acceptance depends on the bias, i.e.
                             min(p, 1/q, 1) * w <= height < max(p, 1/q, 1) * w at a step after the first:
                             the adjacency tests a sampler needs that only tests when the answer matters */
} ndo_stats;

/* ---- random numbers (replaces cuRAND XORWOW; rand_num_gen.cuh:117-122) ---- */

/* Philox4x32-10 block function (Salmon et al., SC'11; Random123 1.09).
 * pinned by the Random123 known-answer vectors in tests/test_oracle_philox.py. */
void ndo_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);

/* The draw-th uniform of (slot, step): word (draw & 3) of the block with counter
 * (slot_lo, slot_hi, step, draw >> 2) and key (seed_lo, seed_hi), mapped to [0,1) as
 * (word >> 8) * 2^-24.  pinned by KAT + range/closed-form tests. */
float ndo_uniform(uint64_t seed, uint64_t slot, uint32_t step, uint32_t draw);
/* The form of the stream at steps whose stepSize is > 1 (one draw per output, a uniform pick):
 * draw 0 of four consecutive slots comes from one block,
 *   draw 0 = ndo_uniform(seed, slot >> 2, step | 2^31, slot & 3),  draw d >= 1 = ndo_uniform(seed, slot, step, d - 1).
 * The engine's definition (nd_philox.hpp), like the plain form; the block function under both is
 * pinned by the Random123 vectors. */
float ndo_uniform_grouped(uint64_t seed, uint64_t slot, uint32_t step, uint32_t draw);

/* RandNumGen::rand_int (rand_num_gen.cuh:117-122): min((int)(u*n), n-1) in float.
 * pinned by closed-form cases incl. the u*n == n rounding case. */
int32_t ndo_rand_int(float u, int32_t n);

/* ---- shape algebra (nextdoor.cu:126-197, 1913-1929) ---- */
int64_t ndo_step_size_at_step(const ndo_app_desc* app, int step);    /* stepSizeAtStep   */
int64_t ndo_number_of_transits(const ndo_app_desc* app, int step);   /* numberOfTransits */
int64_t ndo_sub_warp_size_at_step(const ndo_app_desc* app, int step);/* subWarpSizeAtStep */
int64_t ndo_final_sample_size(const ndo_app_desc* app);              /* getFinalSampleSize */
int ndo_is_collective(const ndo_app_desc* app);
int ndo_max_bits(int32_t n_vertices);                                /* nextdoor.cu:1993-1999 */

/* ---- IndividualNeighborhood sampling (walks, k-hop) ----
 * Step semantics: samplingKernel nextdoor.cu:212-336; output layout: step-k segment
 * starts at sum_{i<k} (outputs of step i per sample); inside it slot j*m_k + nbr holds
 * the nbr-th neighbour drawn for the j-th transit (the j-th entry of the step k-1
 * segment; roots for k = 0).  The reference places entries inside a segment with an
 * atomic cursor (nextdoor.cu:304,473), i.e. in no fixed order; this canonical order
 * is one of the orders it can produce.  RNG slot of that output:
 * ((first_sample + s) * T_k + j) * m_k + nbr.
 * final[n_samples * F] is fully written (INVALID = n_vertices where nothing was sampled).
 * state_t (may be NULL): Node2VecSample::t per sample after the last step.
 * Uniform/k-hop: pinned by closed forms on path/star/complete graphs;
 * DeepWalk: pinned by equal-weight reduction + chi-square; Node2Vec literal: pinned by
 * hand-traced cases; weighted node2vec (own definition): pinned by a draw-by-draw trace at
 * (p, q) = (4, 0.5), (0.5, 4), (2, 0.5) that visits the return, adjacent and far branch, and by
 * chi-square against bias * weight where p, 1/q and 1 all differ. */
int ndo_sample_individual(const ndo_graph* g, const ndo_app_desc* app, uint64_t seed,
                          int64_t n_samples, int64_t first_sample,
                          const int32_t* initial, int32_t* final_samples,
                          int32_t* state_t, ndo_stats* stats, int n_threads);

/* ---- multi-dimensional random walk (src/apps/multiRW/multiRW.cu:13-106) ----
 * A sample owns n_roots walkers.  Step k: the transit is one of the walkers (step 0: walker
 * 0); next() moves it to a uniformly drawn neighbour v, which is the step's output, and for
 * k > 0 stores v in the walker's place (multiRW.cu:27-49; a walker without edges yields
 * INVALID and stays).  Then, unless k is the last step, stepTransits(k + 1) draws the walker
 * of the next step uniformly (multiRW.cu:84-92) from the SAME random state next() used, as
 * the reference's step kernel does (nextdoor.cu:279-289): the draw after next()'s, i.e. draw
 * 1 if next() drew (degree > 1), else draw 0, of the stream of output slot
 * (first_sample + s) at step k.
 * Walker start vertices: ndo_multirw_root.  The reference fills them with rand()
 * (multiRW.cu:95-106); here they are Philox draws, so they are reproducible.
 * roots[n_samples * n_roots] in/out (the walkers after the last step), last_root_idx[n_samples]
 * out (0 if never drawn).  Pinned by a hand trace on a small graph and by the invariant that
 * every output is adjacent to the walker that was the transit (tests); the sampled values
 * themselves are parity unpinned by the reference, whose random numbers differ. */
int32_t ndo_multirw_root(int64_t sample, int root_index, int32_t n_vertices);
int ndo_sample_multirw(const ndo_graph* g, uint64_t seed, int64_t n_samples, int64_t first_sample, int n_roots,
                       int steps, int32_t* roots, int32_t* last_root_idx, int32_t* final_samples,
                       int32_t* transits_out);

/* An app with explicit transits and SEVERAL transits per sample (the reference's contract allows
 * it, nextdoor.cu:279-289; of its own apps only ClusterGCN has both, clusterGCNSampling.cu:89-104).
 * The test application "anchor hop" (tests/cpp/user_apps.hip): a sample holds n_anchors vertices,
 * which are its initial transits; next() is the k-hop rule (khop.cu:18-22); stepTransits(k + 1),
 * called after next() with the same random state for every output whose transit is a vertex,
 * draws x uniformly from [0, n_anchors] and names anchors[(index + x) % n_anchors] as the transit
 * the output stands for at the next step, or none (x == n_anchors: that branch of the sample ends).
 * index is what the reference passes: (thread number) % (transits per sample at step k), i.e.
 * (j * stepSize(k) + nbr) % T_k for neighbour slot nbr of transit j.  Outputs are laid out as
 * for every per-transit app; transits_out (nullable, same layout) gets, at the first output slot
 * of every transit, the transit itself.  Pinned by tests that evaluate the rule draw by draw
 * with ndo_uniform / ndo_rand_int and by adjacency to the named anchors; the values are parity
 * unpinned by the reference, like every other app's. */
int ndo_sample_anchor_hop(const ndo_graph* g, uint64_t seed, int64_t n_samples, int64_t first_sample,
                          int n_anchors, const int32_t* anchors, int steps, const int* step_size,
                          int32_t* final_samples, int32_t* transits_out);

/* ---- inversion, run-length encode, scan, binning (nextdoor.cu:2924-2939, 2529-2572,
 *      1520-1802; utils.hpp:491-497) ---- */

/* Stable sort of (key, value) pairs by key (cub::DeviceRadixSort::SortPairs semantics).
 * pinned by comparison with numpy's stable argsort in tests. */
void ndo_sort_pairs(const int32_t* keys_in, const int32_t* vals_in, int64_t n,
                    int32_t* keys_out, int32_t* vals_out);

/* Unique keys of the sorted prefix whose keys != invalid, their counts and start
 * offsets (RLE + exclusive sum).  Returns the number of runs.
 * pinned by numpy.unique in tests. */
int64_t ndo_unique_transits(const int32_t* sorted_keys, int64_t n, int32_t invalid,
                            int32_t* uniq, int32_t* counts, int32_t* offsets,
                            int64_t* n_valid);

/* Kernel class of a transit that count samples sit on, sub-warp size W:
 * count*W >= 256 -> 1 (grid), >= 32 -> 2 (block), >= 8 -> 3 (sub-warp), else 4 (identity)
 * (utils.hpp:491-497, nextdoor.cu:55-61, 1560-1600). pinned by threshold table test. */
int ndo_kernel_class(int64_t count, int64_t sub_warp_size);

/* ---- distinct post-pass for k-hop (behavioural hint: src/distinct.cuh:1-111) ----
 * Per sample, per hop segment: ascending unique valid ids packed left, rest = invalid;
 * counts[s*steps + k] = number kept.  Own definition: parity unpinned by the reference;
 * pinned by sort+unique brute force and idempotence. */
void ndo_distinct(const ndo_app_desc* app, int64_t n_samples, int32_t invalid,
                  int32_t* final_samples, int32_t* counts);

/* ---- validators (src/check_results.cu) ---- */

/* checkSampledVerticesResult (check_results.cu:162-299) as written: first 4 steps,
 * "adjacent to some valid vertex of the previous step's segment", and "segment all
 * INVALID only if the previous segment has no edges".  Returns 1 when it passes. */
int ndo_check_sampled_vertices(const ndo_graph* g, const ndo_app_desc* app,
                               int64_t n_samples, const int32_t* initial,
                               const int32_t* final_samples, int32_t invalid, int n_threads);

/* Stronger check used by this repo's tests: all steps, and each output must be a
 * neighbour of exactly the transit it was drawn for (canonical layout). */
int ndo_check_exact_transits(const ndo_graph* g, const ndo_app_desc* app,
                             int64_t n_samples, const int32_t* initial,
                             const int32_t* final_samples, int32_t invalid);

/* CSRPartition::has_edge_logn (csr.hpp:342-359). */
int ndo_has_edge(const ndo_graph* g, int32_t src, int32_t dst);

/* ---- CollectiveNeighborhood sampling (layer-wise: FastGCN, LADIES) ----
 * Transits of sample s at step k (sampleParallelKernel, nextdoor.cu:1394-1411): the
 * initial vertices for k = 0, else the step k-1 segment of its result row,
 * final[s*F + stepSizeAtStep(k-2) ...].  Output nbr of step k goes to
 * final[s*F + stepSizeAtStep(k-1) + nbr] (nextdoor.cu:1485-1487); its RNG slot is
 * (first_sample + s) * m_k + nbr. */

/* Collective neighbourhood of one sample (collectiveNeighbrsSize nextdoor.cu:1206-1246,
 * collectiveNeighborhood 1248-1283): the adjacencies of its valid transits concatenated in
 * transit order.  row_offsets[i] = start of transit i's adjacency inside the concatenation
 * (INVALID transits contribute nothing).  cols / weights may be NULL (size only).
 * pinned by a numpy concatenation in tests. */
int64_t ndo_collective_neighborhood(const ndo_graph* g, const int32_t* transits, int n_transits,
                                    int32_t invalid, int32_t* cols, float* weights, int32_t* row_offsets);

/* The reference's FastGCN / LADIES apps as written (identical bodies,
 * fastgcnSampling.cu:23-47, ladiessampling.cu:23-47): the vertex is drawn uniformly from
 * ALL vertices, and for every transit i the pair (i, nbr) is recorded at
 * [step][i*B + nbr] when the graph has the edge transit_i -> vertex, else (-1, -1).
 * rows / cols: [n_samples][steps][B*B] (adjacencyMatrixRow / adjacencyMatrixCol).
 * pinned by closed form (draw 0 of the slot) and brute-force adjacency on small graphs. */
int ndo_sample_layer_literal(const ndo_graph* g, const ndo_app_desc* app, uint64_t seed,
                             int64_t n_samples, int64_t first_sample, const int32_t* initial,
                             int32_t* final_samples, int32_t* rows, int32_t* cols, int n_threads);

/* checkAdjacencyMatrixResult (check_results.cu:46-160) as written: every recorded
 * (row, col) is a graph edge, and every graph edge between consecutive layers is recorded. */
int ndo_check_adjacency_matrix(const ndo_graph* g, const ndo_app_desc* app, int64_t n_samples,
                               const int32_t* initial, const int32_t* final_samples,
                               const int32_t* rows, const int32_t* cols, int32_t invalid);

/* FastGCN-style importance sampling over the union neighbourhood (own definition; the
 * reference's app ignores the neighbourhood, see above): D = ascending distinct vertices
 * of the collective neighbourhood; weight(v) = degree(v)^2 (the squared degree normalised
 * over D, up to the common factor); m_k independent draws WITH replacement by inverse CDF
 * in exact integer arithmetic: r = top 24 bits of draw 0 of the slot,
 * target = (r * total) >> 24, result = D[first i with prefix_i > target].
 * Empty neighbourhood or total 0 -> INVALID.  parity unpinned by the reference; pinned by
 * brute-force probability vectors and chi-square tests. */
int ndo_sample_fastgcn_importance(const ndo_graph* g, const ndo_app_desc* app, uint64_t seed,
                                  int64_t n_samples, int64_t first_sample, const int32_t* initial,
                                  int32_t* final_samples, ndo_stats* stats, int n_threads);

/* LADIES-style layer-dependent importance sampling (own definition; parity unpinned by
 * the reference, whose LADIES app is the literal one above).  For a layer with frontier
 * (transits) U: every occurrence (u, x) of an edge u -> v = col[x], u a valid transit, in
 * contributes term = (w_x * (1 / rowsum_u))^2 (float; the inverse rounded once per row),
 * rowsum_u = the weights of u summed in edge order (float, sequential).  importance(v) = the terms of v's occurrences, each truncated
 * to a 2^53 fixed-point integer and summed exactly (so the sum does not depend on the order
 * of the additions), converted to float: the squared column norm of the row-normalised
 * adjacency restricted to the frontier, times 2^53.  m_k vertices are drawn WITHOUT replacement with probability
 * proportional to importance by Efraimidis-Spirakis keys: key(v) = log2(u_v) / importance(v),
 * u_v = ((word >> 8) + 0.5) * 2^-24, word = word (P & 3) of the Philox block with counter
 * (P >> 2, layer k, 0), P = (first_sample + s) * (|V| rounded up to a multiple of 4) + v (four
 * consecutive vertices of a sample share a block);
 * log2 is ndo_det_log2 (single IEEE operations only, so the GPU reproduces it bit for bit).
 * The result is the m_k largest keys in descending key order, ties by ascending vertex id;
 * fewer than m_k distinct vertices leave INVALID.  pinned by brute-force probability
 * vectors on tiny graphs and inclusion-frequency tests. */
int ndo_sample_ladies_importance(const ndo_graph* g, const ndo_app_desc* app, uint64_t seed,
                                 int64_t n_samples, int64_t first_sample, const int32_t* initial,
                                 int32_t* final_samples, ndo_stats* stats, int n_threads);

/* ---- edge-list apps: MVS and ClusterGCN ----
 * Both leave, per sample, a list of edges (row, col).  The reference appends to the list with
 * atomicAdd(&sample->length, 1) (mvsSampling.cu:36-39, clusterGCNSampling.cu:52-57), so only
 * the CONTENT of a list is fixed by it; the order used here is this repo's definition: the
 * slots l = j * stepSize + nbr (transit index j, neighbour slot nbr) are taken in groups of 64
 * consecutive l, and inside a group the appends are interleaved: the first append of every
 * slot in slot order, then the second append of every slot, ...  (With at most one append per
 * slot, as in ClusterGCN, that is plain slot order.)  Lists are packed in sample order: list_start[s] = edges of the samples before s,
 * list_start[n_samples] = total.  rows / cols may be NULL (sizes only).  Return the total. */

/* numSamples of both apps (mvsSampling.cu:57-60 cap 1500000, clusterGCNSampling.cu:84-87 cap
 * 2000000): 800000 for graphs of more than 1e8 edges, else min(cap, ceil(8 V / vertices)). */
int64_t ndo_subgraph_num_samples(const ndo_graph* g, int vertices_per_sample, int64_t cap);

/* initialSample of MVS (mvsSampling.cu:74-94): vertex i of sample s = (s * batch + i) mod V. */
void ndo_mvs_vertices(const ndo_graph* g, int64_t n_samples, int batch, int32_t* vertices);

/* initialSample of ClusterGCN (clusterGCNSampling.cu:107-122, clusters built at 166-172):
 * cluster c = vertices c*cluster_size .. +cluster_size-1, V / cluster_size clusters; sample s
 * = clusters (s * n_clusters_per_sample + i) mod #clusters. */
void ndo_clustergcn_vertices(const ndo_graph* g, int64_t n_samples, int cluster_size, int clusters_per_sample,
                             int32_t* vertices);

/* MVSSamplingApp::next (mvsSampling.cu:27-46): one step of `batch` slots per transit; slot nbr
 * of transit v appends (v, adj(v)[e]) for e = nbr, nbr + batch, ...
 * pinned by: the multiset of a sample's list equals the concatenated adjacencies of its
 * vertices (numpy), and the reference's checkMVSResult rules (src/tests/multiGPU/mvs.cu:12-101). */
int64_t ndo_sample_mvs(const ndo_graph* g, int64_t n_samples, int batch, const int32_t* vertices,
                       uint32_t* list_start, int32_t* rows, int32_t* cols);

/* SubGraphSamplingAppI::next (clusterGCNSampling.cu:32-73): step 0 returns the transit
 * (an isolated vertex never reaches next(): INVALID, nextdoor.cu:250-262); step 1, slot nbr of
 * transit v1 appends (v1, vertices[nbr]) when v1's adjacency holds vertices[nbr].
 * final_samples: [n_samples][n + n*n], n = vertices per sample: the step-0 outputs, then
 * INVALID (next returns -1 at step 1).
 * pinned by: a dense adjacency-matrix brute force on small graphs (numpy) and the reference's
 * checkSubGraphResult rules (src/tests/multiGPU/clustergcn.cu:10-93). */
int64_t ndo_sample_clustergcn(const ndo_graph* g, int64_t n_samples, int vertices_per_sample,
                              const int32_t* vertices, int32_t* final_samples, uint32_t* list_start,
                              int32_t* rows, int32_t* cols);

/* log2 of a positive normal float from exponent extraction and an atanh series; every step
 * is one IEEE single-precision operation.  pinned against libm (absolute error < 2e-6). */
float ndo_det_log2(float x);

#ifdef __cplusplus
}
#endif
#endif
