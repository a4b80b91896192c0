/*
 * C ABI of the MI355X transit-parallel sampling engine (libnextdoor_amd.so).
 *
 * Plain pointers and sizes only.  Every function that can fail returns 0 on success and
 * a negative value on failure; nd_last_error() then describes the failure (per thread).
 * Nothing here aborts the process.  The library owns every buffer it returns a pointer
 * to; such pointers stay valid until the owning object is freed or the call that
 * produced them is repeated.  One caller at a time per sampler (the reference's
 * single-host-thread contract); all device work of a sampler runs on its private stream.
 *
 * Citations (file:line) name the reference interface each entry point stands for;
 * paths are relative to the plasma-umass/NextDoor tree.
 */
#ifndef NEXTDOOR_AMD_H
#define NEXTDOOR_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct nd_graph nd_graph;     /* host CSR: the reference's CSR* (src/csr.hpp:46-196) */
typedef struct nd_sampler nd_sampler; /* NextDoorData<SampleType, App> + engine state (src/libNextDoor.hpp:13-37) */

const char* nd_last_error(void);

/* Apps compiled into the library (the reference builds one binary per app; here one
 * library holds all of them and the app is chosen by name, e.g. "DeepWalk", "KHop"). */
int nd_num_apps(void);
const char* nd_app_name(int index);

/* Adds an application to the registry, so that nd_sampler_create(name) finds it.  The reference
 * has no registry: every application is a translation unit that instantiates the engine on its
 * <SampleType, App> (src/apps/khop/main.cu:1-21, src/tests/testBase.h:14-24).  Here such a
 * translation unit - the App struct, nd_app_registry.hpp and ND_REGISTER_APP - is compiled with
 * hipcc into a shared object of its own, and loading it calls this.  make(name) returns a new
 * nd::EngineBase* (nd_engine.hpp) for the application; engine_abi must be nd::engine_abi()
 * (nd_app_registry.hpp) of the headers the caller was built from: ND_ENGINE_ABI, raised by hand
 * with every change of the engine's interface, combined with the sizes of the structs the two
 * sides share, so that a forgotten raise is caught as well.  nd_engine_abi() is the library's own
 * value.  Returns 0, or a negative value (-2 ABI mismatch, -3 name taken). */
#define ND_ENGINE_ABI 3
int nd_engine_abi(void);
int nd_register_app(const char* name, void* (*make)(const char* name), int engine_abi);

/* ---- graphs ------------------------------------------------------------------------ */

/* loadGraph(graph, file, type, format), src/nextdoor.cu:1845-1891.
 * type: "edge-list" | "adj-list"; format: "binary" | "text". */
int nd_graph_load(const char* path, const char* graph_type, const char* graph_format, nd_graph** out);
/* csr_from_graph, src/csr.hpp:399-424, from in-memory edges (sorted per vertex by
 * (dst, weight), duplicates kept).  n_vertices <= 0: largest id + 1.  weight may be NULL. */
int nd_graph_from_edges(int32_t n_vertices, int64_t n_edges, const int32_t* src, const int32_t* dst,
                        const float* weight, nd_graph** out);
/* Same from CSR arrays (row_ptr[n_vertices + 1], col[n_edges], weight[n_edges] or NULL). */
int nd_graph_from_csr(int32_t n_vertices, int64_t n_edges, const int32_t* row_ptr, const int32_t* col,
                      const float* weight, nd_graph** out);
/* Seeded synthetic graphs used by the benchmark configurations (no counterpart in the
 * reference, which downloads its datasets: downloadDataset.sh:1). */
int nd_graph_rmat(int scale, int edge_factor, double a, double b, double c, uint64_t seed, int symmetrise,
                  nd_graph** out);
int nd_graph_chung_lu(int32_t n_vertices, int64_t n_edges, double exponent, uint64_t seed, nd_graph** out);
int32_t nd_graph_num_vertices(const nd_graph* g);
int64_t nd_graph_num_edges(const nd_graph* g);
const int32_t* nd_graph_row_ptr(const nd_graph* g);
const int32_t* nd_graph_col(const nd_graph* g);
const float* nd_graph_weight(const nd_graph* g);
const float* nd_graph_max_weight(const nd_graph* g); /* src/graph.hpp:71-80 */
void nd_graph_free(nd_graph* g);

/* ---- sampler: the libNextDoor.hpp host API ------------------------------------------ */

int nd_sampler_create(const char* app_name, nd_sampler** out);
/* transferCSRToGPUs(data, csr), src/nextdoor.cu:1893-1911.  The graph must outlive the sampler. */
int nd_sampler_set_graph(nd_sampler* s, const nd_graph* g);
/* allocNextDoorDataOnGPU(csr, data), src/nextdoor.cu:1931-2086.  seed keys the Philox
 * stream that replaces init_curand_states (src/nextdoor.cu:1838-1843). */
int nd_sampler_alloc(nd_sampler* s, uint64_t seed);
/* doTransitParallelSampling(csr, data, enableLoadBalancing), src/nextdoor.cu:2191-3006. */
int nd_sampler_do_transit_parallel(nd_sampler* s, int enable_load_balancing);
/* doSampleParallelSampling(csr, data), src/nextdoor.cu:3009-3209: the reference's baseline
 * mode.  The (sample -> transit) map is never sorted by transit: before a step the pairs whose
 * transit is INVALID are dropped (one stable compaction, sample order kept) and every remaining
 * pair gets its lanes; no load balancing.  Walks advance several steps per launch between
 * compactions.  Layer-wise apps have one schedule only and run it.  Same samples, byte for
 * byte, as the transit-parallel modes. */
int nd_sampler_do_sample_parallel(nd_sampler* s);
/* How often walks re-invert the (sample -> transit) map.  The reference inverts before every
 * step (src/nextdoor.cu:2924-2939), which is period 1 and the default.  period p > 1: the walks
 * are not brought into transit order (no load balancing); before step 1 and then every p-th
 * step the walks that have ended are dropped from the list, in between the list is walked as
 * it stands.  period 0: the engine decides from the walks-per-vertex ratio.
 * The samples do not depend on the period.  Apps other than walks always invert. */
int nd_sampler_set_inversion_period(nd_sampler* s, int period);
/* getFinalSamples(data), src/nextdoor.cu:3211-3237: copies device -> host and returns the
 * host array (num_samples * final_sample_size int32, INVALID = n_vertices).  The array is
 * page-locked memory of the library's (the copy runs at the bus rate: 57 GB/s measured for
 * 1.68 GB, against 18 GB/s into pageable memory). */
int nd_sampler_get_final_samples(nd_sampler* s, const int32_t** data, int64_t* length);
/* getFinalSampleSize<App>(), src/nextdoor.cu:1913-1929. */
int nd_sampler_final_sample_size(const nd_sampler* s);
/* App::numSamples(csr) as fixed by alloc. */
int64_t nd_sampler_num_samples(const nd_sampler* s);
/* NextDoorData::initialContents (src/libNextDoor.hpp:18): the roots of every sample. */
int nd_sampler_initial_contents(const nd_sampler* s, const int32_t** data, int64_t* length);
/* NextDoorData::INVALID_VERTEX and ::maxBits (src/libNextDoor.hpp:35-36). */
int32_t nd_sampler_invalid_vertex(const nd_sampler* s);
int nd_sampler_max_bits(const nd_sampler* s);
/* App().steps(), App().stepSize(k), App().initialSampleSize(), App().samplingType(). */
int nd_sampler_steps(const nd_sampler* s);
int nd_sampler_step_size(const nd_sampler* s, int step);
int nd_sampler_initial_sample_size(const nd_sampler* s);
int nd_sampler_sampling_type(const nd_sampler* s);
/* NextDoorData::dOutputSamples (src/libNextDoor.hpp:23) copied to the host: num_samples
 * SampleType structs.  nd_sampler_sample_state_bytes is 0 for an empty SampleType. */
int64_t nd_sampler_sample_state_bytes(const nd_sampler* s);
int nd_sampler_get_sample_states(nd_sampler* s, void* dst, int64_t bytes);
/* No counterpart in the reference (whose step loop waits for the host several times per step,
 * src/nextdoor.cu:2498-2636).  A pass here is a fixed sequence of launches with all varying
 * sizes in device memory, so it can be recorded once as a HIP graph and replayed: mode 1 on,
 * 0 off (default: measured, the replay gains nothing here).  Samples are the same bytes either
 * way; per-phase profiling runs eagerly. */
int nd_sampler_set_launch_graph(nd_sampler* s, int mode);
/* The per-phase wall-clock breakdown the reference prints (src/nextdoor.cu:2963-2966),
 * measured with events on the sampler's stream when profiling is on.
 * out[0] end to end, [1] inversion, [2] load balancing, [3] flat (identity / sub-wavefront)
 * kernel, [4] workgroup + grid-wide kernel, [8] final-row assembly, [9] the last distinct pass, all in
 * milliseconds; [5] flat launches, [6] workgroup launches, [7] sort passes; layer-wise apps:
 * [10] milliseconds in the kernel that walks the collective neighbourhoods, [11] its launches. */
int nd_sampler_set_profiling(nd_sampler* s, int on);
int nd_sampler_phase_times(const nd_sampler* s, float out[12]);
/* Apps whose outputFormat() is AdjacencyMatrix on per-transit sampling (MVS, ClusterGCN:
 * src/apps/mvs/mvsSampling.cu, src/apps/clustergcn/clusterGCNSampling.cu) leave one edge list
 * per sample.  The reference keeps them in dRowStorage / dColStorage at
 * sample.posInStorage / adjMatrixPos with sample.length / adjacencyMatrixLen entries, in the
 * order its atomics happened to run.  Here the lists are packed back to back in sample order:
 * sample i owns entries [list_start[i], list_start[i + 1]) of rows / cols (list_start has
 * n_samples + 1 entries), ordered by step, transit index, neighbour slot and emit order.
 * Borrowed host pointers, valid until the next call.  Other apps: error. */
int nd_sampler_get_adjacency(nd_sampler* s, const int32_t** rows, const int32_t** cols, int64_t* n_edges,
                             const uint32_t** list_start, int64_t* n_samples);
/* Distinct post-pass for SampledVertices results (GraphSAGE: draw with replacement, then
 * distinct): every hop segment of every sample is replaced, on the device, by its ascending
 * unique valid ids packed left and INVALID-padded; counts[sample * steps + hop] = ids kept.
 * The reference's k-hop app does not deduplicate; the behaviour follows its unused helper
 * remove_duplicates_in_hop_per_block, src/distinct.cuh:1-111.  Call after
 * nd_sampler_do_transit_parallel; nd_sampler_get_final_samples then returns the packed rows. */
int nd_sampler_distinct(nd_sampler* s);
int nd_sampler_get_distinct_counts(const nd_sampler* s, const int32_t** data, int64_t* length);
/* Sizes the last run worked on.  Layer-wise apps: which 0 = entries of all collective
 * neighbourhoods built, 1 = distinct (sample, vertex) pairs found, 2 = chunks of samples
 * processed, 3 = ready-made stretch bitmaps of the graph's hubs (built by nd_sampler_set_graph for
 * the FastGCN importance form).  Per-transit apps, after a load-balanced pass, the pairs per
 * kernel class summed over its steps (what the reference's printKernelTypes shows,
 * src/nextdoor.cu:2117-2189): 0 = pairs the classifications looked at, 1 = of these, pairs on
 * transits the workgroup kernel served as one work item, 2 = pairs on transits split over several
 * work items (grid-wide), 3 = pairs in runs long enough for the workgroup kernel that stayed with
 * the flat kernel because of the transit's degree, 4 = work items; the flat kernel served
 * 0 minus 1 minus 2.  Edge-list apps: 0 = edges listed. */
int64_t nd_sampler_counter(const nd_sampler* s, int which);
/* The validators the reference's apps pass to nextdoor() as checkResultsFunc
 * (src/check_results.cu): checkSampledVerticesResult (162-299) for the per-transit apps and
 * importance samplers, checkAdjacencyMatrixResult (46-160) for the layer-wise apps that record
 * an adjacency matrix.  Runs on the host over the fetched final samples (and sample states).
 * *ok = 1 when the samples pass; 0 with the first violation in nd_last_error(). */
int nd_sampler_check_results(nd_sampler* s, int* ok);
/* The same rule over caller-supplied arrays (no device needed): final_samples is
 * [n_samples][F], initial [n_samples][initial_size]; collective != 0: step k holds
 * step_sizes[k] vertices (CollectiveNeighborhood layout), else T_k * step_sizes[k].
 * Returns 1 (pass), 0 (violation, text in nd_last_error()) or a negative error. */
int nd_check_sampled_vertices(const nd_graph* g, int n_steps, const int32_t* step_sizes, int initial_size,
                              int collective, int64_t n_samples, const int32_t* initial,
                              const int32_t* final_samples, int32_t invalid);
/* freeDeviceData(data), src/nextdoor.cu:2088-2115. */
void nd_sampler_free_device(nd_sampler* s);
void nd_sampler_destroy(nd_sampler* s);

/* ---- module-level functions (src/nextDoorPythonModule.cu:40-102) --------------------- */
/* One process-wide sampler, as the reference's static NextDoorData per module. */

/* initSampling(graph): binary edge-list path (nextDoorPythonModule.cu:40-52).  The
 * reference compiles one module per app; here the app is named.  seed as above. */
int nd_init_sampling(const char* app_name, const char* graph_path, uint64_t seed);
/* The same for a graph the caller already holds as CSR arrays (copied; sorted rows as in
 * nd_graph_from_csr; weight == NULL: all 1).  No counterpart in the reference, whose module
 * only reads files. */
int nd_init_sampling_from_csr(const char* app_name, int32_t n_vertices, int64_t n_edges, const int32_t* row_ptr,
                              const int32_t* col, const float* weight, uint64_t seed);
/* sample() (nextDoorPythonModule.cu:54-58); runs the load-balanced transit-parallel engine. */
int nd_sample(void);
/* finalSampleLength() (nextDoorPythonModule.cu:75-81): total length of the final-samples vector. */
int64_t nd_final_sample_length(void);
/* finalSamplesArray() (nextDoorPythonModule.cu:90-94): borrowed pointer into the host vector. */
const int32_t* nd_final_samples_array(void);
/* freeDeviceMemory() (nextDoorPythonModule.cu:83-87). */
void nd_free_device_memory(void);

/* ---- building blocks, exposed for parity tests ---------------------------------------- */
/* All take HOST buffers, run the device kernel the engine uses, and copy the result back. */

/* The random-number buffer of one step: out[slot * draws_per_slot + d] = uniform draw d of
 * output slot (first_slot + slot) at `step` (replaces curand_uniform over per-thread
 * states, src/rand_num_gen.cuh:117-122). */
int nd_philox_fill_uniform(uint64_t seed, uint32_t step, uint64_t first_slot, int64_t n_slots,
                           int draws_per_slot, float* out);
/* The same for a step of the given stepSize: steps that draw several outputs per transit
 * (step_size > 1) use the grouped form of the stream, in which the first draw of four consecutive
 * output slots comes from one Philox block (nd_philox.hpp); step_size 1 is nd_philox_fill_uniform. */
int nd_philox_fill_step(uint64_t seed, uint32_t step, int step_size, uint64_t first_slot, int64_t n_slots,
                        int draws_per_slot, float* out);
/* cub::DeviceRadixSort::SortPairs as called at src/nextdoor.cu:2930-2933: stable sort of
 * (key, value) by the low key_bits bits.  vals == NULL: value = index. */
int nd_sort_pairs(const int32_t* keys, const int32_t* vals, int64_t n, int key_bits, int32_t* keys_out,
                  int32_t* vals_out);
/* No counterpart in the reference.  For callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): nd_sort_pairs on
 * DEVICE arrays, enqueued on `stream` (a hipStream_t; NULL = the default stream) without
 * waiting for it, with all working memory in a fixed array inside the library
 * (ND_SORT_PAIRS_NOALLOC_MAX pairs at most: 8.4 MiB per GPU, held until the process ends).
 * Calls no hipMalloc / hipFree / memset.  d_vals == NULL: value = index.  No output array may
 * overlap an input array or the other output array (returns -3).  The first call on a device asks
 * the runtime for the address of the working array (hipGetSymbolAddress, which may load the
 * library's code object): make that call outside graph capture; nd_sampler_set_graph on the
 * device does it as well.  More than ND_SORT_PAIRS_NOALLOC_MAX pairs: returns -2.  All
 * calls on one GPU share the working array: calls that overlap on one GPU (two streams, two
 * host threads) race; calls on one stream are ordered by the stream. */
#define ND_SORT_PAIRS_NOALLOC_MAX 1048576
int nd_sort_pairs_noalloc(const int32_t* d_keys, const int32_t* d_vals, int64_t n, int key_bits, int32_t* d_keys_out,
                          int32_t* d_vals_out, void* stream);
/* invalidVertexStartPos + DeviceRunLengthEncode::Encode + DeviceScan::ExclusiveSum
 * (src/nextdoor.cu:1804-1836, 2535-2545, 2560-2567) over a sorted key array.  Stand-alone: the
 * sampling pass classifies runs at their last pair (nd_classify_runs) and never lists them. */
int nd_unique_transits(const int32_t* sorted_keys, int64_t n, int32_t invalid, int32_t* uniq, int32_t* counts,
                       int32_t* offsets, int64_t* n_runs, int64_t* n_valid);

/* partitionTransitsInKernels with its thresholds (src/nextdoor.cu:1520-1802, src/utils.hpp:491-497)
 * over a sorted key array, as the engine runs it between the inversion and the step kernels:
 * degrees[v] = edges of vertex v; a run of `count` equal keys goes to the workgroup kernel when
 * count * step_size >= thresholds[0], the transit has edges and staging its adjacency pays (at
 * most thresholds[2] edges, and no more than 32 staged edges per output); such a run is cut
 * into work items of at most thresholds[1] / step_size pairs: items[2 i] = first pair,
 * items[2 i + 1] = pairs, in no particular order; taken[v] = 1 for the transits so served (the flat
 * kernel skips their pairs).  *n_items = items wanted (those beyond `capacity` are not written and
 * their transit is then not marked).  counters: 0 pairs looked at, 1 pairs in single-item runs,
 * 2 pairs in runs cut into several items (grid-wide), 3 pairs in runs long enough but refused for
 * their degree, 4 items.  pairs_per_lane: 1 or 16, the two launch shapes the engine uses. */
int nd_load_balancing_thresholds(int32_t thresholds[3]);
int nd_classify_runs(const int32_t* sorted_keys, int64_t n, const int32_t* degrees, int32_t n_vertices, int step_size,
                     int pairs_per_lane, int32_t* items, int64_t capacity, int64_t* n_items, uint8_t* taken,
                     int64_t counters[5]);

/* Measurement, no counterpart in the reference: the rate (requests per second) at which this GPU
 * serves independent random 8-byte reads over a table of table_bytes (a power of two, 4 KiB to
 * 32 GiB; allocated and freed inside): 4 M lanes, 16 reads each, two in flight per lane.  The
 * ceiling a gather-bound step kernel is priced against next to the HBM byte peak. */
int nd_measure_gather_rate(int64_t table_bytes, double* requests_per_s);
/* The same with the shape of the probe chosen: reads_in_flight (1, 2, 4 or 8) independent reads
 * issued per lane before any is used, in workgroups of workgroup_lanes (64 or 256) lanes; 16
 * reads per lane in all.  nd_measure_gather_rate is (2, 256).  The ceiling of the path is the
 * largest rate over the shapes. */
int nd_measure_gather_rate_shaped(int64_t table_bytes, int reads_in_flight, int workgroup_lanes,
                                  double* requests_per_s);

/* collectiveNeighbrsSize + collectiveNeighborhood (src/nextdoor.cu:1206-1283) for n_samples
 * samples of transits_per_sample transits each (transits[s * transits_per_sample + i]):
 * sizes[s] = sum of the degrees of the valid transits, offsets = their exclusive scan
 * (offsets[n_samples] = total), cols / weights = the adjacencies concatenated in transit
 * order at offsets[s], row_offsets[s * transits_per_sample + i] = start of transit i inside
 * its sample's concatenation.  Fails when the total exceeds capacity. */
int nd_collective_neighborhood(const nd_graph* g, const int32_t* transits, int64_t n_samples,
                               int32_t transits_per_sample, int32_t invalid, int32_t* sizes, int32_t* offsets,
                               int32_t* cols, float* weights, int64_t capacity, int32_t* row_offsets);

#ifdef __cplusplus
}
#endif
#endif
