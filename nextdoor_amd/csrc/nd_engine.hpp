// Transit-parallel sampling engine for one MI355X (gfx950, wave64).
//
// What this implements, against the reference (file:line in the reference tree):
//   allocNextDoorDataOnGPU     src/nextdoor.cu:1931-2086   -> Engine::alloc
//   transferCSRToGPUs          src/nextdoor.cu:1893-1911   -> Engine::set_graph
//   doTransitParallelSampling  src/nextdoor.cu:2191-3006   -> Engine::sample
//   getFinalSamples            src/nextdoor.cu:3211-3237   -> Engine::final_samples
//   freeDeviceData             src/nextdoor.cu:2088-2115   -> Engine::free_device
//   samplingKernel / identityKernel / gridKernel  212-336 / 338-504 / 976-1204
//                                                      -> step_flat_kernel / step_workgroup_kernel
//   partitionTransitsInKernels 1520-1802               -> classify_run_tails
//
// Differences that are deliberate:
//  * The (sample -> transit) map stores only the transit; the map index IS the slot
//    (sample * transitsPerSample + j).  The inversion sorts (transit, slot) and the step
//    kernels write output (slot * stepSize + nbr) of sample slot / transitsPerSample at a
//    fixed place: final[sample * F + segBase + j * stepSize + nbr].  The reference places
//    k-hop outputs with an atomic cursor per sample (nextdoor.cu:304, 473), i.e. in no
//    fixed order; this order is one it can produce, and it never changes between runs or
//    kernel classes.
//  * Random numbers are Philox draws keyed by the output slot and the step (nd_philox.hpp),
//    so load balancing on/off, kernel class and lane assignment cannot change a result.
//  * No host round trip inside the step loop: run counts, work lists and the
//    valid-prefix length stay in device memory; kernels whose work size is only known on
//    the device are launched with a fixed grid and stride over the device-side count.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <chrono>
#include <memory>
#include <string>
#include <thread>
#include <type_traits>
#include <vector>

#include "nd_contract.hpp"
#include "nd_device_graph.hpp"
#include "nd_distinct.hpp"
#include "nd_radix_sort.hpp"
#include "nd_transit_runs.hpp"

namespace nd {

// ---------------------------------------------------------------------------------------
// Host-visible, app-independent interface (what the C ABI talks to)
// ---------------------------------------------------------------------------------------

// kSampleParallel: the reference's baseline (src/nextdoor.cu:3009-3209), every sample's work in
// sample order: the (sample -> transit) map is never sorted by transit, the pairs whose transit
// is INVALID are only dropped (one stable compaction), and there is no load balancing.
enum KernelMode { kTransitParallel = 0, kTransitParallelLoadBalanced = 1, kSampleParallel = 2 };

struct PhaseTimes {  // milliseconds, accumulated over one sample() call when profiling is on
  float end_to_end = 0, inversion = 0, load_balancing = 0, flat_kernel = 0, workgroup_kernel = 0, assemble = 0, distinct = 0;
  int flat_launches = 0, workgroup_launches = 0, sort_launches = 0;
  // layer-wise apps: the kernel that walks the collective neighbourhoods (marking / building)
  float neighborhood = 0;
  int neighborhood_launches = 0;
};

// Host array the device copies results into.  Page-locked (hipHostMalloc) when a device is
// there: the copy of 1.68 GB of walks takes 94 ms into pageable memory (17.8 GB/s) and about a
// third of that into page-locked memory.  Falls back to ordinary memory (no device, or the
// driver refuses).
template <class T>
class HostArray {
 public:
  HostArray() = default;
  HostArray(const HostArray&) = delete;
  HostArray& operator=(const HostArray&) = delete;
  ~HostArray() { clear(); }
  T* data() { return data_; }
  const T* data() const { return data_; }
  size_t size() const { return size_; }
  bool empty() const { return size_ == 0; }
  // n elements, every one `value`
  void assign(size_t n, T value) {
    if (n != size_) {
      clear();
      if (n) {
        void* p = nullptr;
        if (hipHostMalloc(&p, n * sizeof(T), hipHostMallocDefault) == hipSuccess && p) {
          pinned_ = true;
        } else {
          (void)hipGetLastError();  // the refusal is not an error of a later call
          p = malloc(n * sizeof(T));
          pinned_ = false;
        }
        data_ = (T*)p;
        size_ = data_ ? n : 0;
      }
    }
    std::fill_n(data_, size_, value);
  }
  void clear() {
    if (data_) {
      if (pinned_) (void)hipHostFree(data_); else free(data_);
    }
    data_ = nullptr;
    size_ = 0;
  }

 private:
  T* data_ = nullptr;
  size_t size_ = 0;
  bool pinned_ = false;
};

// Roots index the row extents in the kernels: each must be a vertex, or the "no vertex" value
// (the number of vertices).  The reference does not check (a root outside the graph reads past
// its arrays there).
inline bool roots_are_vertices(const std::vector<VertexID_t>& roots, int32_t n_vertices) {
  for (VertexID_t r : roots)
    if (r < 0 || r > n_vertices) return false;
  return true;
}

class EngineBase {
 public:
  virtual ~EngineBase() {}
  virtual const char* app_name() const = 0;
  virtual int set_graph(const CSR* graph) = 0;
  virtual int alloc(uint64_t seed) = 0;
  virtual int sample(int mode) = 0;
  // Walks: how often the (sample -> transit) map is inverted.  1: before every step, as the
  // reference does.  p > 1: the walks are not brought into transit order at all; before step
  // 1 and then every p-th step the walks that have ended are dropped from the list (a stable
  // compaction in slot order), and there is no load balancing.  0: the engine decides from
  // the walks-per-vertex ratio.  Results do not depend on it.  Other apps always invert.
  int inversion_period = 1;
  // 1: replay a pass as a recorded HIP graph instead of enqueueing its launches one by one;
  // 0 (default): enqueue.  Layer-wise and edge-list apps have few, long launches and ignore it.
  int launch_graph = 0;
  virtual int fetch_final_samples() = 0;
  virtual void free_device() = 0;
  virtual int64_t num_samples() const = 0;
  virtual int final_sample_size() const = 0;
  virtual int steps() const = 0;
  virtual int step_size(int k) const = 0;
  virtual int initial_sample_size() const = 0;
  virtual int sampling_type() const = 0;
  virtual int32_t invalid_vertex() const = 0;
  virtual int max_bits() const = 0;
  virtual size_t sample_state_bytes() const = 0;
  virtual int fetch_sample_states(void* dst, size_t bytes) = 0;
  virtual int distinct() = 0;
  // engine-specific sizes of the last run (layer engine: 0 = entries of all collective
  // neighbourhoods, 1 = distinct (sample, vertex) pairs, 2 = chunks); 0 where not applicable
  virtual int64_t counter(int) const { return 0; }
  // Apps with AdjacencyMatrix output on the per-transit engine (MVS, ClusterGCN): device ->
  // hListStart / hListRows / hListCols
  virtual bool lists_edges() const { return false; }
  // App::hasExplicitTransits(): the transits of a step are not the previous step's samples
  virtual bool has_explicit_transits() const { return false; }
  virtual int fetch_adjacency() {
    last_error = "this app does not produce edge lists";
    return -2;
  }

  HostArray<VertexID_t> hFinalSamples;         // as NextDoorData::hFinalSamples (libNextDoor.hpp:17)
  std::vector<VertexID_t> initialContents;     // as NextDoorData::initialContents (libNextDoor.hpp:18)
  std::vector<int32_t> hDistinctCounts;        // [num_samples * steps] ids kept by distinct()
  // edge lists of all samples, packed in sample order: sample s owns entries
  // [hListStart[s], hListStart[s + 1]) of hListRows / hListCols
  std::vector<uint32_t> hListStart;
  std::vector<VertexID_t> hListRows, hListCols;
  std::string last_error;
  bool profiling = false;
  PhaseTimes times;
};

#define ND_HIP_TRY(expr)                                                                  \
  do {                                                                                    \
    hipError_t nd_e_ = (expr);                                                            \
    if (nd_e_ != hipSuccess) {                                                            \
      last_error = std::string(#expr) + ": " + hipGetErrorString(nd_e_);                  \
      return -1;                                                                          \
    }                                                                                     \
  } while (0)

// ---------------------------------------------------------------------------------------
// Step kernels
// ---------------------------------------------------------------------------------------

// Steps an app may have for its INVALID outputs to be written by the step kernels instead of
// a fill of the whole result.
constexpr int kMaxFillLevels = 8;

struct StepParams {
  CSRPartition csr;
  int step;
  uint32_t step_size;            // m_k
  uint32_t lanes_shift;          // flat kernel: 2^lanes_shift lanes share the outputs of a pair
  uint32_t groups_per_pair;      // step_size > 1: the groups of four consecutive output slots (one
                                 // Philox block each for the first draw, nd_philox.hpp) the outputs
                                 // of a pair can touch at most; a lane works through whole groups
  uint32_t transits_per_sample;  // T_k
  uint32_t seg_base;             // offset of this step's segment inside a final sample
  uint32_t final_size;           // F
  int32_t invalid;
  int is_last;
  uint64_t seed;
  uint64_t first_slot;           // RNG slot of local output 0 (first sample of this device)
  uint32_t first_sample;
  uint32_t n_pairs;              // S * T_k
  const uint32_t* live_pairs;    // device count of pairs in pair_keys (sorted map: pairs with a real transit); nullptr: n_pairs
  const uint32_t* pair_keys;     // transit of each pair (sorted, or the raw map at step 0)
  const uint32_t* pair_slots;    // slot of each pair; nullptr: slot == index
  int32_t* step_out;             // outputs of this step: output slot o of sample s sits at
                                 // step_out[s * out_pitch + (o - s * T_k * m_k)].  Either an
                                 // array of its own (out_pitch = T_k * m_k: indexed by o),
                                 // regrouped per sample at the end, or the step's segment
                                 // inside the rows of the result (out_pitch = F).  It is also
                                 // the (sample -> transit) map of step k+1.
  uint32_t out_pitch;
  // Walks whose transit is the previous step's result: the results of steps 2j and 2j + 1 of
  // sample s share one 8-byte cell, pair_cells[(j * pair_cell_samples + s) * 2 + (step & 1)],
  // and the odd step writes both at once (it knows the even step's result: it is its transit) -
  // one scattered store per two steps instead of two.  nullptr: step_out as described above.
  int32_t* pair_cells;
  uint32_t pair_cell_samples;
  // With the cells: walk_cells[s] = how many cells of walk s hold results, written once per pass
  // by the step at which the walk ends (its result is INVALID, or it is the last step).  The
  // regrouping reads only those cells, so nothing fills the cells before a pass.
  uint32_t* walk_cells;
  void* samples;                 // SampleType[S] or nullptr
  // Apps with explicit transits that are not walks: the (sample -> transit) map of step k+1,
  // indexed like step_out's own array form (output slot o of this step is pair o of the next):
  // what App::stepTransits returned for the output.  nullptr: the step's outputs are the map.
  int32_t* explicit_out;
  // Results written straight into the rows, with nothing filled in beforehand: an output that
  // is INVALID (and a pair with no transit or no edges, for all its outputs) leads nowhere at
  // the later steps, whose pairs the inversion drops - no kernel ever reaches the slots that
  // descend from it, so whoever writes the INVALID writes them too.  Level 0 is this step
  // (offset 0, one slot per output), level l the l-th step after it: output q of a sample owns
  // slots [q * fill_mult[l], (q + 1) * fill_mult[l]) at step_out + fill_off[l] of its row.
  // fill_levels == 0: the result was filled before the pass, nothing of this is done.
  uint32_t fill_levels;
  uint32_t fill_off[kMaxFillLevels];
  uint32_t fill_mult[kMaxFillLevels];
  const EdgeRecord* paired_edges; // interleaved (dst, weight) copy of the edges, or nullptr
  // Walks (one transit per sample, stepSize 1 everywhere): the step kernels also emit the
  // next step's pairs in THIS step's pair order - coalesced, and without the pairs the
  // inversion dropped - and a 4-byte SampleType travels with its pair instead of being
  // gathered from samples[] by every next() (nullptr: not in use).
  int state_travels;             // the state is read from pair_state (samples[] at step 0) and
                                 // goes back to samples[] only when its walk ends
  const uint32_t* pair_state;    // state of each pair entering the step; nullptr: samples[sample]
  uint32_t* emit_keys;           // next transit of each pair; nullptr: nothing is emitted
  uint32_t* emit_slots;          // its slot
  uint32_t* emit_state;          // its state after next()
  // Small maps (see small_map_scan): a pair that goes on also takes its place among the pairs
  // that will share its next transit - emit_ranks[pair] = its number among them, counted in
  // emit_counts[next transit] - so that the next inversion needs no sort (nullptr: not in use).
  // Transit v counts in the counters [emit_counter_base[v], emit_counter_base[v + 1]), a power
  // of two of them, a pair counting in copy (its index & (copies - 1)): atomics on one address
  // are served tens of nanoseconds apart, and a hub that takes thousands of walks per step would
  // otherwise hold the step kernel up.  Most vertices have one counter.
  uint32_t* emit_counts;
  uint32_t* emit_ranks;
  const uint32_t* emit_counter_base;
  // Small maps placed as they are emitted (nullptr: not in use): counter c owns the places
  // [emit_place_start[c], emit_place_start[c + 1]) of the next step's pair arrays - room for
  // about twice the walks it expects - and a pair whose rank fits goes straight there; the few
  // that do not fit take a place past emit_spill_first, handed out by the counter *emit_spill.
  // The next step's lanes walk ALL places, the empty ones hold INVALID: the map is inverted, with
  // gaps, by the kernel that produced it, and a step is one launch.
  const uint32_t* emit_place_start;
  uint32_t* emit_spill;
  uint32_t emit_spill_first;
  // ... and the other side of it: the lane that takes a pair from such an array marks its place
  // empty again, and the first lanes clear the counters the pairs were placed by, so that the
  // arrays and counters are ready when they are written the step after next (two sets alternate).
  uint32_t* taken_keys;       // == pair_keys, writable; nullptr: the pairs are a dense list
  uint32_t* taken_counts;     // the counters behind pair_keys, the spill counter after the last
  uint32_t taken_n_counts;
};

// A SampleType small enough to travel with its pair through the inversion.
template <class SampleType>
struct state_fits_pair {
  static constexpr bool value = !std::is_empty<SampleType>::value && sizeof(SampleType) == sizeof(uint32_t) &&
                                std::is_trivially_copyable<SampleType>::value;
};

constexpr int kStepThreads = 256;
// Workgroup size of the flat kernel: one wavefront.  A workgroup keeps its slot until its
// slowest wave is done and rejection loops make wave run times very uneven, so single-wave
// workgroups keep more waves in flight (256 -> 64 threads: 34.6 -> 32.8 ms per pass).
#ifndef ND_CHUNK_OUTPUTS
#define ND_CHUNK_OUTPUTS 2048
#endif
#ifndef ND_FLAT_THREADS
#define ND_FLAT_THREADS 64
#endif
constexpr int kFlatThreads = ND_FLAT_THREADS;
// LDS adjacency cache of the workgroup kernel, in edges (k-hop pass with 8192 / 6144 / 4096: 3.58 / 3.75 /
// 3.87 ms - a smaller cache lets more workgroups share a compute unit, but hands the flat kernel
// more of the hubs than that wins).
#ifndef ND_CACHE_EDGES
#define ND_CACHE_EDGES 8192
#endif
constexpr int kCacheEdges = ND_CACHE_EDGES;
// A transit goes to the workgroup kernel when at least this many outputs are drawn from it.
constexpr uint32_t kWorkgroupWork = 256;
// Outputs one work item of the workgroup kernel covers at most; larger runs are split
// over several workgroups (the grid-wide case).
constexpr uint32_t kChunkOutputs = ND_CHUNK_OUTPUTS;

// next() for one output and, for apps with explicit transits, stepTransits() for the step
// after it (nextdoor.cu:279-289: the random state is the one next() used).  Returns the
// sampled vertex; *next_transit is the transit the pair has at the next step.
// grouped: the step draws several outputs per transit, and first_word is the output's word of
// its group's shared block (the grouped form of the stream, nd_philox.hpp).
template <class SampleType, class App, class EdgeArray, class WeightArray>
__device__ __forceinline__ VertexID run_app(const StepParams& P, CSRPartition& csr, VertexID transit, uint32_t sample,
                                            uint32_t transit_index, uint64_t out_slot, uint32_t nbr,
                                            EdgePos_t n_edges, float max_weight, EdgeArray& edges,
                                            WeightArray& weights, SampleType* state, VertexID* next_transit,
                                            bool grouped, uint32_t first_word) {
  const VertexID sample_id = (VertexID)(P.first_sample + sample);
  const bool runs = transit != P.invalid && n_edges != 0;  // next() only runs for a real transit
                                                           // that has edges (nextdoor.cu:250-262)
  const bool explicit_transits = App().hasExplicitTransits();
  curandState rng;
  // a pair whose transit is no vertex is dead, with or without explicit transits
  const bool chooses_transit = explicit_transits && !P.is_last && transit != P.invalid;
  if (runs || chooses_transit) {
    if (grouped) rng.reset_with_first(P.seed, P.first_slot + out_slot, (uint32_t)P.step, first_word);
    else rng.reset(P.seed, P.first_slot + out_slot, (uint32_t)P.step);
  }
  VertexID neighbor = P.invalid;
  if (runs) {
    const VertexID r = App().template next<SampleType, EdgeArray, WeightArray>(
        P.step, &csr, &transit, sample_id, state, max_weight, edges, weights, n_edges, (VertexID_t)nbr, &rng);
    neighbor = r == -1 ? P.invalid : r;  // nextdoor.cu:288
  }
  *next_transit = neighbor;
  if (chooses_transit) {
    // the index the reference hands over is its thread number modulo the step's transits per
    // sample (nextdoor.cu:282: threadId % numTransits): the transit's own index where the step
    // size is 1 (walks: 0; ClusterGCN's step 0: the vertex's place in the sample)
    const uint32_t index = (transit_index * P.step_size + nbr) % P.transits_per_sample;
    const VertexID_t t = App().stepTransits(P.step + 1, sample_id, *state, (int)index, &rng);
    *next_transit = t == -1 ? P.invalid : t;
  }
  return neighbor;
}

// The result of a walk's step into the cells two steps share (StepParams::pair_cells).  An even
// step leaves its result to the odd step that follows - a walk that ends at the even step has
// INVALID there, which the cell holds already - unless it is the last step of all.
// Cells of a walk that hold results when the walk ends at `step`: an odd step has just written
// cell (step - 1) / 2; an even step writes its cell only when it is the last step of all.
__device__ __forceinline__ uint32_t walk_cells_at_end(int step, bool last_of_all) {
  return (step & 1) ? (uint32_t)(step + 1) / 2u : (uint32_t)step / 2u + (last_of_all ? 1u : 0u);
}

__device__ __forceinline__ void store_walk_result(const StepParams& P, uint32_t sample, VertexID transit,
                                                  VertexID neighbor, int step) {
  int32_t* cell = P.pair_cells + ((size_t)(step >> 1) * P.pair_cell_samples + sample) * 2;
  if (step & 1) {
    *reinterpret_cast<int2*>(cell) = make_int2(transit, neighbor);
  } else if (P.is_last) {
    cell[0] = neighbor;
  }
  if (P.walk_cells && (P.is_last || neighbor == P.invalid)) P.walk_cells[sample] = walk_cells_at_end(step, P.is_last);
}
__device__ __forceinline__ void store_walk_result(const StepParams& P, uint32_t sample, VertexID transit,
                                                  VertexID neighbor) {
  store_walk_result(P, sample, transit, neighbor, P.step);
}

// pair: index of the pair in the order the step kernels walk them (sorted by transit, or
// the raw map at step 0).
// First half: next() (and stepTransits) for the output; nothing of the step's results is stored.
// kStateOut: the state that travels with the pair is handed to the caller, who knows where the
// pair goes (store_output<true>), instead of being written next to the pair's index.
template <class SampleType, class App, class EdgeArray, class WeightArray, bool kStateOut = false>
__device__ __forceinline__ void compute_output(const StepParams& P, CSRPartition& csr, VertexID transit, uint32_t pair,
                                               uint32_t pair_slot, uint32_t sample, uint32_t nbr, EdgePos_t n_edges,
                                               float max_weight, EdgeArray& edges, WeightArray& weights, bool grouped,
                                               uint32_t first_word, VertexID* neighbor_out, VertexID* next_transit_out,
                                               uint32_t* state_out = nullptr) {
  const uint64_t out_slot = (uint64_t)pair_slot * P.step_size + nbr;
  const uint32_t transit_index = pair_slot - sample * P.transits_per_sample;
  VertexID neighbor = P.invalid, next_transit = P.invalid;
  bool travelled = false;
  if constexpr (state_fits_pair<SampleType>::value) {
    if (P.state_travels) {
      // the state travels with the pair: a register copy
      SampleType state;
      uint32_t bits = P.pair_state ? P.pair_state[pair] : ((const uint32_t*)P.samples)[sample];
      __builtin_memcpy(&state, &bits, sizeof(uint32_t));
      neighbor = run_app<SampleType, App>(P, csr, transit, sample, transit_index, out_slot, nbr, n_edges, max_weight,
                                          edges, weights, &state, &next_transit, grouped, first_word);
      __builtin_memcpy(&bits, &state, sizeof(uint32_t));
      if (kStateOut) *state_out = bits;
      else if (P.emit_state) P.emit_state[pair] = bits;
      // a walk that ends here leaves the stream of pairs: its state goes home
      if (P.is_last || next_transit == P.invalid) ((uint32_t*)P.samples)[sample] = bits;
      travelled = true;
    }
  }
  if (!travelled) {
    if constexpr (std::is_empty<SampleType>::value) {
      SampleType no_state;
      neighbor = run_app<SampleType, App>(P, csr, transit, sample, transit_index, out_slot, nbr, n_edges, max_weight,
                                          edges, weights, &no_state, &next_transit, grouped, first_word);
    } else {
      neighbor = run_app<SampleType, App>(P, csr, transit, sample, transit_index, out_slot, nbr, n_edges, max_weight,
                                          edges, weights, (SampleType*)P.samples + sample, &next_transit, grouped,
                                          first_word);
    }
  }
  *neighbor_out = neighbor;
  *next_transit_out = next_transit;
}

// Four consecutive ids of a result, at an address that is a multiple of four bytes only.
struct __attribute__((packed, aligned(4))) FourIds {
  VertexID a, b, c, d;
};

// Output q (index inside the sample's segment of this step) is INVALID: so is everything the
// later steps would have drawn from it (StepParams::fill_levels).
// (Inlined although it is rare and repeated at every store: a call from a step kernel costs the
// kernel its register allocation - the k-hop pass took 9.9 ms instead of 3.5 with this out of line.)
__device__ __forceinline__ void fill_below(const StepParams& P, uint32_t sample, uint32_t q) {
  int32_t* row = P.step_out + (size_t)sample * P.out_pitch;
#pragma unroll
  for (int l = 1; l < kMaxFillLevels; ++l) {
    if ((uint32_t)l < P.fill_levels) {
      int32_t* dst = row + P.fill_off[l] + (size_t)q * P.fill_mult[l];
      for (uint32_t x = 0; x < P.fill_mult[l]; ++x) dst[x] = P.invalid;
    }
  }
}

// All outputs of a pair (slot pair_slot) are INVALID - it has no transit, or the transit has no
// edge: its m outputs and what descends from them are contiguous stretches of the sample's row,
// written by the lanes of the wavefront that are still at work: `helper` is the lane's number
// among them, `helpers` how many they are.
__device__ __forceinline__ void fill_dead_pair(const StepParams& P, uint32_t pair_slot, uint32_t helper,
                                               uint32_t helpers) {
  const uint32_t sample = P.transits_per_sample == 1 ? pair_slot : pair_slot / P.transits_per_sample;
  const uint32_t q0 = (pair_slot - sample * P.transits_per_sample) * P.step_size;
  int32_t* row = P.step_out + (size_t)sample * P.out_pitch;
#pragma unroll
  for (int l = 0; l < kMaxFillLevels; ++l) {
    if ((uint32_t)l < P.fill_levels) {
      int32_t* dst = row + P.fill_off[l] + (size_t)q0 * P.fill_mult[l];
      const uint32_t n = P.step_size * P.fill_mult[l];
      // 16 bytes per lane and store (the address is a multiple of four bytes only), then the rest
      const uint32_t fours = n / 4u;
      for (uint32_t x = helper; x < fours; x += helpers)
        *reinterpret_cast<FourIds*>(dst + 4u * x) = FourIds{P.invalid, P.invalid, P.invalid, P.invalid};
      for (uint32_t x = 4u * fours + helper; x < n; x += helpers) dst[x] = P.invalid;
    }
  }
}

// Second half: the output goes to its place in the step's results, and what the next step
// needs of it to the next step's map.
// kPlaces: the flat kernel of walks over small maps (flat_lane's kPlaces), whose lanes place the
// pair for the next step themselves (StepParams::emit_place_start) and then also store its
// travelling state.
// kWalkStep: the step may be a walk's (one output per pair); cells shared by two steps and
// emitted pairs exist only there, and the code of steps that draw several outputs per pair is
// compiled without them (the k-hop kernels are slower by a tenth with that code merely present).
template <bool kPlaces = false, bool kWalkStep = true>
__device__ __forceinline__ void store_output(const StepParams& P, VertexID transit, uint32_t pair, uint32_t pair_slot,
                                             uint32_t sample, uint32_t nbr, VertexID neighbor, VertexID next_transit,
                                             uint32_t state_bits = 0, bool chooses_transits = true) {
  const uint64_t out_slot = (uint64_t)pair_slot * P.step_size + nbr;
  if (kWalkStep && P.pair_cells) {
    store_walk_result(P, sample, transit, neighbor);
  } else {
    const uint32_t per_sample = P.transits_per_sample * P.step_size;
    const uint32_t q = (uint32_t)(out_slot - (uint64_t)sample * per_sample);
    P.step_out[(size_t)sample * P.out_pitch + q] = neighbor;
    if (P.fill_levels > 1 && neighbor == P.invalid) fill_below(P, sample, q);
  }
  // (chooses_transits: App::hasExplicitTransits(), where the caller knows the app)
  if (chooses_transits && P.explicit_out) P.explicit_out[out_slot] = next_transit;
  if (kWalkStep && P.emit_keys) {
    uint32_t at = pair;
    if (P.emit_counts && next_transit != P.invalid) {
      const uint32_t first = P.emit_counter_base[next_transit];
      const uint32_t copies = P.emit_counter_base[next_transit + 1] - first;
      const uint32_t counter = first + (pair & (copies - 1u));
      const uint32_t rank = atomicAdd(&P.emit_counts[counter], 1u);
      if (kPlaces && P.emit_place_start) {
        const uint32_t place = P.emit_place_start[counter];
        at = place + rank < P.emit_place_start[counter + 1] ? place + rank : P.emit_spill_first + atomicAdd(P.emit_spill, 1u);
      } else {
        P.emit_ranks[pair] = rank;
      }
    }
    // placed pairs: a walk that has ended takes no place (the empty places hold INVALID already)
    if (!(kPlaces && P.emit_place_start) || next_transit != P.invalid) {
      P.emit_keys[at] = (uint32_t)next_transit;
      P.emit_slots[at] = pair_slot;
      if (kPlaces && P.emit_state) P.emit_state[at] = state_bits;
    }
  }
}

template <class SampleType, class App, class EdgeArray, class WeightArray, bool kPlaces = false>
__device__ __forceinline__ void produce_output(const StepParams& P, CSRPartition& csr, VertexID transit, uint32_t pair,
                                               uint32_t pair_slot, uint32_t nbr, EdgePos_t n_edges, float max_weight,
                                               EdgeArray& edges, WeightArray& weights) {
  const uint32_t sample = P.transits_per_sample == 1 ? pair_slot : pair_slot / P.transits_per_sample;
  VertexID neighbor, next_transit;
  uint32_t state_bits = 0;
  compute_output<SampleType, App, EdgeArray, WeightArray, kPlaces>(P, csr, transit, pair, pair_slot, sample, nbr,
                                                                   n_edges, max_weight, edges, weights, false, 0u,
                                                                   &neighbor, &next_transit, &state_bits);
  store_output<kPlaces>(P, transit, pair, pair_slot, sample, nbr, neighbor, next_transit, state_bits);
}

// The outputs of a pair that fall into group `gi` of the pair's groups of four consecutive
// (global) output slots: one shared Philox block, then up to four outputs.  For steps with
// step_size > 1.  In two halves, so that a lane that works through several groups can have
// the gathers of the next group under way while the results of this one are stored.
struct GroupOutputs {
  uint64_t first;     // global slot of the pair's output 0
  uint64_t base;      // global slot of the group's word 0 (a multiple of four)
  uint32_t from, to;  // the words [from, to) of the group belong to the pair
  uint32_t sample;
  VertexID neighbor[4], next_transit[4];  // by word
};

template <class SampleType, class App, class EdgeArray, class WeightArray>
__device__ __forceinline__ void compute_group(const StepParams& P, CSRPartition& csr, VertexID transit, uint32_t pair,
                                              uint32_t pair_slot, uint32_t gi, EdgePos_t n_edges, float max_weight,
                                              EdgeArray& edges, WeightArray& weights, GroupOutputs* out) {
  const uint64_t first = P.first_slot + (uint64_t)pair_slot * P.step_size;  // global slot of the pair's output 0
  const uint64_t group = (first >> 2) + gi;
  const uint64_t base = group * 4;
  const uint64_t end = first + P.step_size;
  out->first = first;
  out->base = base;
  out->from = base < first ? (uint32_t)(first - base) : 0u;
  out->to = base + 4 <= end ? 4u : (end > base ? (uint32_t)(end - base) : 0u);
  if (out->from >= out->to) return;
  PhiloxBlock block = PhiloxBlock();
  // next() draws for a real transit with edges; stepTransits for any real transit (run_app)
  if (transit != P.invalid && (n_edges != 0 || (App().hasExplicitTransits() && !P.is_last)))
    block = grouped_first_block_scalar_seed(P.seed, group, (uint32_t)P.step);
  out->sample = P.transits_per_sample == 1 ? pair_slot : pair_slot / P.transits_per_sample;
  // all draws of the group before any store: its up to four gathers are under way together.
  // Word w of the block belongs to slot base + w: which word an output takes is known when
  // the loop is unrolled, nothing is selected at run time.
  if (std::is_empty<SampleType>::value && !App().hasExplicitTransits()) {
    // An app without sample state draws nothing but its result: all four words are drawn, whether
    // the pair owns them or not, and those it does not own are dropped afterwards.  Without a
    // branch around each draw the four gathers are issued one after the other and waited for
    // once; with it, each waited for its own (and for the stores of the group before).
    // (Looking at what next() returned only after the stores of the lane's previous group have
    // been issued, so that the gathers do not queue behind those stores: no gain, 1.26 against
    // 1.24 ms for the k-hop flat launches.)
    VertexID drawn[4] = {P.invalid, P.invalid, P.invalid, P.invalid};
    if (transit != P.invalid && n_edges != 0) {  // next() only runs for a real transit that has edges (run_app)
      const VertexID sample_id = (VertexID)(P.first_sample + out->sample);
      VertexID at = transit;
      SampleType no_state;
      VertexID r[4];
#pragma unroll
      for (uint32_t w = 0; w < 4; ++w) {
        const bool owned = w >= out->from && w < out->to;
        curandState rng;
        rng.reset_with_first(P.seed, base + w, (uint32_t)P.step, block.w[w]);
        r[w] = App().template next<SampleType, EdgeArray, WeightArray>(
            P.step, &csr, &at, sample_id, &no_state, max_weight, edges, weights, n_edges,
            (VertexID_t)(owned ? (uint32_t)(base + w - first) : 0u), &rng);
      }
#pragma unroll
      for (uint32_t w = 0; w < 4; ++w) drawn[w] = r[w] == -1 ? P.invalid : r[w];  // nextdoor.cu:288
    }
#pragma unroll
    for (uint32_t w = 0; w < 4; ++w) {
      const bool owned = w >= out->from && w < out->to;
      out->neighbor[w] = out->next_transit[w] = owned ? drawn[w] : P.invalid;
    }
    return;
  }
#pragma unroll
  for (uint32_t w = 0; w < 4; ++w) {
    out->neighbor[w] = out->next_transit[w] = P.invalid;
    if (w >= out->from && w < out->to)
      compute_output<SampleType, App, EdgeArray, WeightArray>(P, csr, transit, pair, pair_slot, out->sample,
                                                              (uint32_t)(base + w - first), n_edges, max_weight, edges,
                                                              weights, true, block.w[w], &out->neighbor[w],
                                                              &out->next_transit[w]);
  }
}

template <class App>
__device__ __forceinline__ void store_group(const StepParams& P, VertexID transit, uint32_t pair, uint32_t pair_slot,
                                            const GroupOutputs& g) {
  if (g.from >= g.to) return;
  const bool chooses_transits = App().hasExplicitTransits();  // a constant of the app
  if (g.from == 0 && g.to == 4 && !(chooses_transits && P.explicit_out)) {
    // a whole group whose outputs are all there is to store: the four ids are neighbours in
    // the step's results (word aligned, not more), and go out as one 16-byte store
    const uint32_t per_sample = P.transits_per_sample * P.step_size;
    const uint64_t out_slot = (uint64_t)pair_slot * P.step_size + (g.base - g.first);
    const uint32_t q = (uint32_t)(out_slot - (uint64_t)g.sample * per_sample);
    FourIds* dst = reinterpret_cast<FourIds*>(P.step_out + (size_t)g.sample * P.out_pitch + q);
    *dst = FourIds{g.neighbor[0], g.neighbor[1], g.neighbor[2], g.neighbor[3]};
    if (P.fill_levels > 1) {
#pragma unroll
      for (uint32_t x = 0; x < 4; ++x)
        if (g.neighbor[x] == P.invalid) fill_below(P, g.sample, q + x);
    }
    return;
  }
#pragma unroll
  for (uint32_t w = 0; w < 4; ++w)
    if (w >= g.from && w < g.to)
      store_output<false, false>(P, transit, pair, pair_slot, g.sample, (uint32_t)(g.base + w - g.first), g.neighbor[w],
                                 g.next_transit[w], 0u, chooses_transits);
}

// The groups first, first + stride, ... of a pair, the draws of a group made before the
// results of the group before it are stored.
template <class SampleType, class App, class EdgeArray, class WeightArray>
__device__ __forceinline__ void produce_groups(const StepParams& P, CSRPartition& csr, VertexID transit, uint32_t pair,
                                               uint32_t pair_slot, uint32_t first_group, uint32_t stride,
                                               EdgePos_t n_edges, float max_weight, EdgeArray& edges,
                                               WeightArray& weights) {
  GroupOutputs held;
  held.first = held.base = 0;
  held.from = held.to = 0;  // nothing held yet
  for (uint32_t gi = first_group; gi < P.groups_per_pair; gi += stride) {
    GroupOutputs now;
    compute_group<SampleType, App, EdgeArray, WeightArray>(P, csr, transit, pair, pair_slot, gi, n_edges, max_weight,
                                                           edges, weights, &now);
    store_group<App>(P, transit, pair, pair_slot, held);
    held = now;
  }
  store_group<App>(P, transit, pair, pair_slot, held);
}

// The same without holding a group back: for the workgroup class, whose draws come from LDS
// and have no memory latency to hide behind the stores of the group before.
template <class SampleType, class App, class EdgeArray, class WeightArray>
__device__ __forceinline__ void produce_groups_in_turn(const StepParams& P, CSRPartition& csr, VertexID transit,
                                                       uint32_t pair, uint32_t pair_slot, uint32_t first_group,
                                                       uint32_t stride, EdgePos_t n_edges, float max_weight,
                                                       EdgeArray& edges, WeightArray& weights) {
  for (uint32_t gi = first_group; gi < P.groups_per_pair; gi += stride) {
    GroupOutputs now;
    compute_group<SampleType, App, EdgeArray, WeightArray>(P, csr, transit, pair, pair_slot, gi, n_edges, max_weight,
                                                           edges, weights, &now);
    store_group<App>(P, transit, pair, pair_slot, now);
  }
}

// inversion_period == 0: walks are inverted before every step when there are at least this
// many walks per vertex, else every kSparseInversionPeriod steps (measured on 4.2 M weighted
// node2vec walks over 4.2 M vertices: 45.3 ms per 100 steps inverting every step, 38.0 every
// 4th, 35.5 only once; the sorted order saves 3.4 ms in the step kernels and costs 13.7).
constexpr double kWalksPerVertexForInversion = 4.0;
constexpr int kSparseInversionPeriod = 32;

// Lanes the flat kernel wants before it gives a lane all the outputs of a pair: enough to fill
// the machine where the map is sorted by transit (neighbouring lanes then share their transit's
// lines, and what a lane fetches once per pair - transit, slot, row extent - is spread over all
// the pair's outputs), many more at step 0, where the roots come in sample order, every lane's
// gathers miss the caches and a lane that draws all 25 outputs of a root keeps its wavefront
// alive seven round trips long.  Measured on the two hops of 2.1 M k-hop samples (flat launches,
// ms): 2^20 at both steps 1.26; roots 2^23 (4 lanes per root) 1.12; roots 2^25 (8 lanes) 1.08;
// 2^26 at both steps (2 lanes per pair at the second hop) 1.21; 2^27 (4 lanes) 1.52.
constexpr uint64_t kFlatLanesWanted = 1ull << 20;
constexpr uint64_t kFlatLanesWantedForRoots = 1ull << 25;

constexpr uint32_t kXcds = 8;
// Consecutive workgroups (in sorted-pair order) one XCD handles before the next XCD takes over.
#ifndef ND_XCD_RUN
#define ND_XCD_RUN 64
#endif
constexpr uint32_t kXcdRun = ND_XCD_RUN;

// Workgroups are handed to the 8 XCDs round-robin (workgroup b runs on XCD b % 8), each XCD
// with its own L2.  The pairs are sorted by transit, so an XCD is given runs of kXcdRun
// CONSECUTIVE workgroups' worth of pairs: samples of one hot transit then mostly share one
// L2, while the runs still interleave finely enough that all XCDs get equal shares of the
// live prefix and of the INVALID tail of the sorted map.
__device__ __forceinline__ uint32_t flat_block_index() {
  const uint32_t xcd = blockIdx.x % kXcds;
  const uint32_t turn = blockIdx.x / kXcds;  // how many workgroups this XCD has started before
  return (turn / kXcdRun) * (kXcds * kXcdRun) + xcd * kXcdRun + turn % kXcdRun;
}

// 2^lanes_shift lanes per pair: lane i serves pair i >> lanes_shift and draws the
// neighbours sub, sub + L, ... (sub = i mod L, L = 2^lanes_shift) of it.  One lane per pair
// (L = 1) when there are enough pairs to fill the machine: the pair, its row extent and the
// marker are then fetched once for all stepSize draws, whose gathers are independent and
// overlap; several lanes per pair when pairs are few.  With the map sorted by transit,
// neighbouring lanes share row extents and adjacency lines.
// taken_stamp (nullable): per-vertex marker of the transits that work items cover at this
// step - those whose entry equals `stamp` (RunsMeta::stamp of the step).
// kSingleOutput: stepSize is 1 (walks); the loop over neighbours is compiled away.
// kPlaces: a walk over a small map whose pairs are placed as they are emitted
// (StepParams::emit_place_start, taken_keys); a kernel of its own, so that the others are
// compiled without it.
template <class SampleType, class App, bool kSingleOutput, bool kPlaces = false>
__device__ __forceinline__ void flat_lane(StepParams& P, uint64_t i, const uint32_t* __restrict__ taken_stamp,
                                          uint32_t stamp) {
  if (kSingleOutput) {
    P.lanes_shift = 0;
    P.step_size = 1;
  }
  if (kPlaces && P.taken_keys) {
    // pairs placed as they were emitted: nobody reads their counters during this step
    if (i < P.taken_n_counts) P.taken_counts[i] = 0;
  }
  const uint64_t total = (uint64_t)(P.live_pairs ? *P.live_pairs : P.n_pairs) << P.lanes_shift;
  if (i >= total) return;
  CSRPartition csr = P.csr;
  const uint32_t pair = (uint32_t)(i >> P.lanes_shift);
  const uint32_t first_nbr = (uint32_t)i & ((1u << P.lanes_shift) - 1u);
  const uint32_t nbr_stride = 1u << P.lanes_shift;
  VertexID transit;
  if (kPlaces && P.taken_keys) {
    transit = (VertexID)P.taken_keys[pair];
    if (transit == P.invalid) return;  // an empty place
    P.taken_keys[pair] = (uint32_t)P.invalid;
  } else {
    transit = (VertexID)P.pair_keys[pair];
  }
  const uint32_t slot = P.pair_slots ? P.pair_slots[pair] : pair;
  EdgePos_t n_edges = 0, begin = 0;
  float max_weight = 0.0f;
  if (transit != P.invalid) {
    // the marker, the row extent and the largest weight are fetched together
    const uint32_t mark = taken_stamp ? taken_stamp[transit] : 0u;
    begin = csr.row_ptr[transit];
    n_edges = csr.row_ptr[transit + 1] - begin;
    max_weight = csr.max_weights[transit];
    if (taken_stamp && mark == stamp) return;
  }
  if (P.fill_levels != 0) {
    // pairs all of whose outputs are INVALID: no draw, the wavefront writes their stretches
    const bool dead = transit == P.invalid || n_edges == 0;
    uint64_t todo = __ballot(dead && first_nbr == 0);
    if (todo) {
      // lanes past the last pair, or whose transit a work item covers, have left already
      const uint64_t at_work = __ballot(1);
      const uint32_t helper = (uint32_t)__popcll(at_work & ((1ull << (threadIdx.x & (kWave - 1))) - 1ull));
      const uint32_t helpers = (uint32_t)__popcll(at_work);
      while (todo) {
        const int src = __ffsll((unsigned long long)todo) - 1;
        todo &= todo - 1;
        fill_dead_pair(P, __shfl(slot, src, kWave), helper, helpers);
      }
    }
    if (dead) return;
  }
  // one output (walks), or the pair's groups of four output slots first_nbr, first_nbr + stride, ...
  if (app_uses_weights<App>::value) {
    PairedEdgeIds edges{P.paired_edges + begin};
    PairedEdgeWeights weights{P.paired_edges + begin};
    if (kSingleOutput) {
      produce_output<SampleType, App, PairedEdgeIds, PairedEdgeWeights, kPlaces>(P, csr, transit, pair, slot, 0, n_edges,
                                                                                 max_weight, edges, weights);
    } else {
      produce_groups<SampleType, App, PairedEdgeIds, PairedEdgeWeights>(P, csr, transit, pair, slot, first_nbr,
                                                                        nbr_stride, n_edges, max_weight, edges, weights);
    }
  } else {
    const CSR::Edge* edges = csr.edges + begin;
    const float* weights = csr.weights + begin;
    if (kSingleOutput) {
      produce_output<SampleType, App, const CSR::Edge*, const float*, kPlaces>(P, csr, transit, pair, slot, 0, n_edges,
                                                                              max_weight, edges, weights);
    } else {
      produce_groups<SampleType, App, const CSR::Edge*, const float*>(P, csr, transit, pair, slot, first_nbr,
                                                                     nbr_stride, n_edges, max_weight, edges, weights);
    }
  }
}

// meta (with taken_stamp): the step's bookkeeping, whose stamp marks the taken transits.
template <class SampleType, class App, bool kSingleOutput, bool kPlaces = false>
__global__ __launch_bounds__(kFlatThreads) void step_flat_kernel(StepParams P,
                                                                 const uint32_t* __restrict__ taken_stamp,
                                                                 const RunsMeta* __restrict__ meta) {
  const uint32_t stamp = taken_stamp ? meta->stamp : 0u;
  flat_lane<SampleType, App, kSingleOutput, kPlaces>(P, (uint64_t)flat_block_index() * kFlatThreads + threadIdx.x,
                                                     taken_stamp, stamp);
}

// Walks that are not re-inverted for a while: one lane keeps its walk for a whole stretch of
// steps, with the current vertex and the sample state in registers.  Besides saving the
// reads and writes of the pair list between steps, this evens out the rejection loops: a
// wavefront waits for the SUM of its lanes' rounds over the stretch, not for the slowest
// lane of every single step.  Step k of the stretch writes step_out[k * out_stride + slot].
template <class SampleType, class App>
__global__ __launch_bounds__(kFlatThreads) void walk_stretch_kernel(StepParams P, int stretch_steps, int last_step,
                                                                    size_t out_stride) {
  const uint32_t total = P.live_pairs ? *P.live_pairs : P.n_pairs;
  const uint32_t i = blockIdx.x * kFlatThreads + threadIdx.x;
  if (i >= total) return;
  CSRPartition csr = P.csr;
  VertexID transit = (VertexID)P.pair_keys[i];
  const uint32_t slot = P.pair_slots ? P.pair_slots[i] : i;  // == the sample: one transit per sample
  constexpr bool kTravels = state_fits_pair<SampleType>::value;
  SampleType local_state;
  SampleType* state = &local_state;
  if constexpr (kTravels) {
    const uint32_t bits = P.pair_state ? P.pair_state[i] : ((const uint32_t*)P.samples)[slot];
    __builtin_memcpy(&local_state, &bits, sizeof(uint32_t));
  } else if (!std::is_empty<SampleType>::value) {
    state = (SampleType*)P.samples + slot;
  }
  const bool explicit_transits = App().hasExplicitTransits();
  int step = P.step;
  for (int k = 0; k < stretch_steps && transit != P.invalid; ++k, ++step) {
    const EdgePos_t begin = csr.row_ptr[transit];
    const EdgePos_t n_edges = csr.row_ptr[transit + 1] - begin;
    VertexID neighbor = P.invalid;
    curandState rng;
    if (n_edges != 0) {  // next() only runs for a transit that has edges (nextdoor.cu:250-262)
      const float max_weight = csr.max_weights[transit];
      rng.reset(P.seed, P.first_slot + slot, (uint32_t)step);
      VertexID r;
      if (app_uses_weights<App>::value) {
        PairedEdgeIds edges{P.paired_edges + begin};
        PairedEdgeWeights weights{P.paired_edges + begin};
        r = App().template next<SampleType, PairedEdgeIds, PairedEdgeWeights>(
            step, &csr, &transit, (VertexID)(P.first_sample + slot), state, max_weight, edges, weights, n_edges, 0, &rng);
      } else {
        const CSR::Edge* edges = csr.edges + begin;
        const float* weights = csr.weights + begin;
        r = App().template next<SampleType, const CSR::Edge*, const float*>(
            step, &csr, &transit, (VertexID)(P.first_sample + slot), state, max_weight, edges, weights, n_edges, 0, &rng);
      }
      neighbor = r == -1 ? P.invalid : r;  // nextdoor.cu:288
    }
    if (P.pair_cells) {
      // the last step of all, or of this walk, or of the stretch may be an even one
      int32_t* cell = P.pair_cells + ((size_t)(step >> 1) * P.pair_cell_samples + slot) * 2;
      if (step & 1) *reinterpret_cast<int2*>(cell) = make_int2(transit, neighbor);
      else if (step == last_step) cell[0] = neighbor;
      if (P.walk_cells && (step == last_step || neighbor == P.invalid))
        P.walk_cells[slot] = walk_cells_at_end(step, step == last_step);
    } else {
      P.step_out[(size_t)k * out_stride + slot] = neighbor;
    }
    transit = neighbor;
    if (explicit_transits && step != last_step) {
      if (n_edges == 0) rng.reset(P.seed, P.first_slot + slot, (uint32_t)step);
      const VertexID_t t = App().stepTransits(step + 1, (VertexID)(P.first_sample + slot), *state, 0, &rng);
      transit = t == -1 ? P.invalid : t;
    }
  }
  // the walk as it stands after the stretch (INVALID: it has ended and the next compaction drops it)
  const bool pass_over = step > last_step;
  if (P.emit_keys && !pass_over) {
    P.emit_keys[i] = (uint32_t)transit;
    P.emit_slots[i] = slot;
  }
  if constexpr (kTravels) {
    uint32_t bits;
    __builtin_memcpy(&bits, &local_state, sizeof(uint32_t));
    if (P.emit_state && !pass_over) P.emit_state[i] = bits;
    if (pass_over || transit == P.invalid) ((uint32_t*)P.samples)[slot] = bits;  // the state goes home
  }
}

// A work item of the workgroup class: a stretch of pairs on one transit, with what the
// classification knew of the transit, so that the workgroup that takes the item goes from this
// one record straight to the adjacency (one 32-byte fetch instead of a chain of three
// dependent ones: item, transit of its first pair, row extent).
struct alignas(16) WorkItem {
  uint32_t first_pair, n_pairs;
  int32_t transit;
  EdgePos_t begin, n_edges;  // the transit's row extent
  uint32_t unused[3];
};

// The first `count` (at most kCacheEdges) words of `src` into LDS by the whole workgroup.  A
// lane takes four consecutive words per round (one 16-byte load from a word-aligned address)
// and has the loads of ALL its rounds under way before it writes the first to LDS: a loop of
// "load one word, wait, write it" costs a memory round trip per 256 words - for a
// 2000-edge adjacency eight trips one after the other, and the workgroup class spent most of
// its time there.  (Holding the words of the NEXT work item in registers while the workgroup
// draws from this one's adjacency was measured too: 31 more registers per lane, four wavefronts
// per SIMD instead of five, and the k-hop launch 9 % slower.)
template <class T>
__device__ __forceinline__ void stage_into_lds(const T* __restrict__ src, T* lds, EdgePos_t count) {
  static_assert(sizeof(T) == 4, "32-bit words");
  struct __attribute__((packed, aligned(4))) FourWords { uint32_t a, b, c, d; };
  constexpr int kRounds = kCacheEdges / (kStepThreads * 4);
  FourWords held[kRounds];
#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
    const EdgePos_t e = (EdgePos_t)(r * kStepThreads + threadIdx.x) * 4;
    if (e + 4 <= count) held[r] = *reinterpret_cast<const FourWords*>(src + e);
  }
  // the up to three words after the last whole four
  const EdgePos_t rest = count & ~(EdgePos_t)3;
  T last = T();
  if ((EdgePos_t)threadIdx.x < count - rest) last = src[rest + threadIdx.x];
#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
    const EdgePos_t e = (EdgePos_t)(r * kStepThreads + threadIdx.x) * 4;
    if (e + 4 <= count) *reinterpret_cast<uint4*>(lds + e) = make_uint4(held[r].a, held[r].b, held[r].c, held[r].d);
  }
  if ((EdgePos_t)threadIdx.x < count - rest) lds[rest + threadIdx.x] = last;
}

// One workgroup per work item = a stretch of pairs that sit on the SAME transit.  The
// transit's adjacency (and weights, when the app draws by weight) is staged once into LDS
// with coalesced reads and every draw of the stretch gathers from LDS.  The workgroup takes
// the items first_item, first_item + item_stride, ...
// kSingleOutput: the step draws one output per pair; each form is compiled without the other.
template <class SampleType, class App, bool kSingleOutput>
__device__ __forceinline__ void workgroup_items(StepParams& P, const WorkItem* __restrict__ chunks, uint32_t n_chunks,
                                                uint32_t first_item, uint32_t item_stride, CSR::Edge* s_edges,
                                                float* s_weights) {
  constexpr bool kWeights = app_uses_weights<App>::value;
  CSRPartition csr = P.csr;
  // the five words of an item that are used, as scalars (the same for every lane)
  uint32_t first_pair = 0, n_pairs = 0;
  VertexID transit = 0;
  EdgePos_t begin = 0, n_edges = 0;
  auto fetch = [&](uint32_t c, uint32_t* fp, uint32_t* np, VertexID* t, EdgePos_t* b, EdgePos_t* ne) {
    *fp = chunks[c].first_pair;
    *np = chunks[c].n_pairs;
    *t = (VertexID)chunks[c].transit;
    *b = chunks[c].begin;
    *ne = chunks[c].n_edges;
  };
  if (first_item < n_chunks) fetch(first_item, &first_pair, &n_pairs, &transit, &begin, &n_edges);
  for (uint32_t c = first_item; c < n_chunks; c += item_stride) {
    // the record of the item after this one is fetched while this one is worked on
    uint32_t coming_first_pair = 0, coming_n_pairs = 0;
    VertexID coming_transit = 0;
    EdgePos_t coming_begin = 0, coming_n_edges = 0;
    if (c + item_stride < n_chunks)
      fetch(c + item_stride, &coming_first_pair, &coming_n_pairs, &coming_transit, &coming_begin, &coming_n_edges);
    const float max_weight = csr.max_weights[transit];  // every next() is handed it, hint or no hint
    const EdgePos_t cached = n_edges < kCacheEdges ? n_edges : kCacheEdges;
    // Lanes per pair: one, or the power of two (at most the groups of four output slots a pair
    // has) that the item's pairs leave room for in the workgroup; lane `sub` of a pair takes the
    // pair's groups sub, sub + L, ...  (Dealing the (pair, group) tasks of an item to the lanes
    // one by one keeps more lanes busy - 94 instead of 59 % for 100 pairs of three groups - and
    // was slower: 1.23 against 1.17 ms for the k-hop launch, which does not wait for its lanes.)
    // The slot of a lane's first pair is fetched together with the adjacency, not after it.
    uint32_t lanes_shift = 0;
    if (!kSingleOutput)
      while ((1u << lanes_shift) < P.groups_per_pair && (n_pairs << (lanes_shift + 1)) <= (uint32_t)kStepThreads) lanes_shift++;
    const uint32_t lanes = n_pairs << lanes_shift;
    uint32_t slot = threadIdx.x < lanes ? P.pair_slots[first_pair + (threadIdx.x >> lanes_shift)] : 0u;
    __syncthreads();  // the previous work item is done with the cache
    stage_into_lds(csr.edges + begin, s_edges, cached);
    if (kWeights) stage_into_lds(csr.weights + begin, s_weights, cached);
    __syncthreads();
    // the classification hands over no transit whose adjacency exceeds the cache
    LdsArray<CSR::Edge> edges{s_edges};
    typedef typename std::conditional<kWeights, LdsArray<float>, const float*>::type Weights;
    Weights weights_of_transit = [&]() {
      if constexpr (kWeights) return LdsArray<float>{s_weights};
      else return csr.weights + begin;
    }();
    for (uint32_t t = threadIdx.x; t < lanes; t += kStepThreads) {
      const uint32_t p = t >> lanes_shift;
      if (t != threadIdx.x) slot = P.pair_slots[first_pair + p];
      if (kSingleOutput) {
        produce_output<SampleType, App, LdsArray<CSR::Edge>, Weights>(P, csr, transit, first_pair + p, slot, 0, n_edges,
                                                                      max_weight, edges, weights_of_transit);
      } else {
        produce_groups_in_turn<SampleType, App, LdsArray<CSR::Edge>, Weights>(P, csr, transit, first_pair + p, slot,
                                                                      t & ((1u << lanes_shift) - 1u), 1u << lanes_shift,
                                                                      n_edges, max_weight, edges, weights_of_transit);
      }
    }
    first_pair = coming_first_pair;
    n_pairs = coming_n_pairs;
    transit = coming_transit;
    begin = coming_begin;
    n_edges = coming_n_edges;
  }
}

template <class SampleType, class App, bool kSingleOutput>
__global__ __launch_bounds__(kStepThreads) void step_workgroup_kernel(StepParams P,
                                                                      const WorkItem* __restrict__ chunks,
                                                                      const RunsMeta* __restrict__ meta,
                                                                      uint32_t chunk_capacity) {
  __shared__ __align__(16) CSR::Edge s_edges[kCacheEdges];  // filled with 16-byte stores
  __shared__ __align__(16) float s_weights[app_uses_weights<App>::value ? kCacheEdges : 4];
  const uint32_t n_chunks = meta->n_chunks < chunk_capacity ? meta->n_chunks : chunk_capacity;
  workgroup_items<SampleType, App, kSingleOutput>(P, chunks, n_chunks, blockIdx.x, gridDim.x, s_edges, s_weights);
}

// Both classes of a load-balanced step in ONE launch: the flat lanes and the work items touch
// disjoint pairs (a transit belongs to the work items exactly when its marker carries the step's
// stamp, and nobody clears a marker), so nothing orders them.  The grid is made of groups of
// kBalancedFlatBlocks flat workgroups followed by wg_per_group work-item workgroups, so that
// both kinds start side by side from the first moment on; inside the flat part a workgroup
// finds its pairs as in step_flat_kernel (runs of consecutive workgroups per XCD: a group is a
// whole number of such runs for all XCDs, and wg_per_group is a multiple of the XCD count).
// Every workgroup reserves the LDS of the adjacency cache, whichever kind it is: this launch
// is for maps where the number of launches matters more than the flat lanes' occupancy.
constexpr uint32_t kBalancedFlatBlocks = kXcds * kXcdRun;

template <class SampleType, class App, bool kSingleOutput>
__global__ __launch_bounds__(kStepThreads) void step_balanced_kernel(StepParams P,
                                                                     const uint32_t* __restrict__ taken_stamp,
                                                                     const RunsMeta* __restrict__ meta,
                                                                     const WorkItem* __restrict__ chunks,
                                                                     uint32_t chunk_capacity, uint32_t wg_per_group) {
  __shared__ __align__(16) CSR::Edge s_edges[kCacheEdges];  // filled with 16-byte stores
  __shared__ __align__(16) float s_weights[app_uses_weights<App>::value ? kCacheEdges : 4];
  const uint32_t per_group = kBalancedFlatBlocks + wg_per_group;
  const uint32_t group = blockIdx.x / per_group;
  const uint32_t local = blockIdx.x - group * per_group;
  if (local < kBalancedFlatBlocks) {
    // the XCD this workgroup runs on is blockIdx.x % kXcds == local % kXcds
    const uint32_t xcd = local % kXcds, turn = local / kXcds;  // turn < kXcdRun
    const uint32_t block = group * kBalancedFlatBlocks + xcd * kXcdRun + turn;
    flat_lane<SampleType, App, kSingleOutput>(P, (uint64_t)block * kStepThreads + threadIdx.x, taken_stamp,
                                              meta->stamp);
  } else {
    const uint32_t n_groups = gridDim.x / per_group;
    const uint32_t n_chunks = meta->n_chunks < chunk_capacity ? meta->n_chunks : chunk_capacity;
    workgroup_items<SampleType, App, kSingleOutput>(P, chunks, n_chunks,
                                                    group * wg_per_group + (local - kBalancedFlatBlocks),
                                                    n_groups * wg_per_group, s_edges, s_weights);
  }
}

// Load balancing without a scan or a run-length encode: the pairs are sorted by transit, so
// the last pair of a run finds the run's start by looking back.  Only runs long enough for
// the workgroup kernel matter, so the tail first looks one threshold back (a single read
// that rules out nearly every run) and only then gallops to the start.  One launch,
// classify_run_tails, where the reference has a boundary search, a run-length encode, a
// scan, a partition kernel and three blocking copies (src/nextdoor.cu:2498-2636).
//
// Classes by neighbour-work (outputs drawn from the transit = count * stepSize):
//   work <  kWorkgroupWork                      -> flat kernel (sub-wavefront: the lanes of a
//                                                  wave that share the transit share its lines)
//   work >= kWorkgroupWork, one work item       -> workgroup kernel
//   work >  kChunkOutputs, several work items   -> grid-wide: the transit is split over workgroups
// A transit whose adjacency does not fit the LDS cache, or is much longer than the number
// of draws taken from it, is cheaper to gather directly and stays with the flat kernel.

// First index of the run of `transit` that ends at i (keys sorted, keys[i] == transit).
__device__ __forceinline__ uint32_t run_start(const uint32_t* __restrict__ keys, uint32_t i, uint32_t transit) {
  // gallop back while the key still matches ...
  uint32_t hi = i, step = 1;
  while (hi >= step && keys[hi - step] == transit) {
    hi -= step;
    step <<= 1;
  }
  // ... the start is in (hi - step, hi] (or [0, hi] when the gallop ran off the front)
  uint32_t lo = hi >= step ? hi - step + 1 : 0;
  while (lo < hi) {
    const uint32_t mid = lo + (hi - lo) / 2;
    if (keys[mid] == transit) hi = mid; else lo = mid + 1;
  }
  return lo;
}

// The stamp after `stamp`: 1, 2, ..., 2^32 - 1, 1, ... (0 is what a cleared marker holds).
__device__ __forceinline__ uint32_t next_stamp(uint32_t stamp) { return stamp + 1u == 0u ? 1u : stamp + 1u; }

// Pairs per kernel class, summed over the load-balanced steps of a pass (what the reference's
// printKernelTypes shows per step, src/nextdoor.cu:2117-2189).
struct ClassCounters {
  unsigned long long sorted_pairs;     // pairs the inversions kept and the classification looked at
  unsigned long long workgroup_pairs;  // on transits served by the workgroup kernel as one work item
  unsigned long long split_pairs;      // on transits split over several work items (grid-wide)
  unsigned long long refused_pairs;    // in runs long enough for the workgroup kernel that stay with the flat
                                       // kernel because of the transit's degree
  unsigned long long work_items;       // work items handed to the workgroup kernel
};
// The counters are kept in kCounterCopies copies, a wavefront adding to copy (its number mod
// kCounterCopies), and summed on the host: atomics on one address are served one after the
// other, and a k-hop step has more than 10^5 qualifying runs.
constexpr uint32_t kCounterCopies = 64;

constexpr uint32_t kDirectSegment = 16;  // ids: segments this long are written straight into the result rows
// Consecutive pairs per lane of classify_run_tails: many for large maps (fewer atomics),
// one for small ones (the launch is latency bound: 3.4 vs 1.8 ms over the 99 steps of 4.2 M walks).
constexpr int kClassifyItemsLarge = 16;
// (workgroups of 1024 lanes, for a quarter of the atomics that claim work items: 0.34 ms
// against 0.24 on 5.2e7 pairs - the launch waits for its slowest lanes, not for the atomics)
constexpr int kClassifyThreadsLarge = 256;
constexpr uint32_t kClassifyLargeFrom = 16u << 20;  // pairs

// A run of `count` pairs on `transit` that starts at pair `start`: should the workgroup kernel
// take it?  Gives the run and the number of work items it needs.  refused_out (nullable): set to
// the run's length when the run is long enough but stays with the flat kernel because of the degree.
__device__ __forceinline__ bool workgroup_takes_run(uint32_t transit, uint32_t start, uint32_t count,
                                                    const EdgePos_t* __restrict__ row_ptr, uint32_t step_size,
                                                    uint32_t* transit_out, uint32_t* start_out, uint32_t* count_out,
                                                    uint32_t* n_items_out, uint32_t* refused_out = nullptr,
                                                    EdgePos_t* begin_out = nullptr, EdgePos_t* degree_out = nullptr) {
  const uint64_t work = (uint64_t)count * step_size;
  if (work < kWorkgroupWork) return false;
  const EdgePos_t begin = row_ptr[transit];
  const uint32_t degree = (uint32_t)(row_ptr[transit + 1] - begin);
  if (degree == 0) return false;
  if (degree > (uint32_t)kCacheEdges || (uint64_t)degree > 32ull * work) {
    if (refused_out) *refused_out = count;
    return false;
  }
  if (begin_out) *begin_out = begin;
  if (degree_out) *degree_out = (EdgePos_t)degree;
  uint32_t pairs_per_chunk = kChunkOutputs / step_size;
  if (pairs_per_chunk == 0) pairs_per_chunk = 1;
  *transit_out = transit;
  *start_out = start;
  *count_out = count;
  *n_items_out = (count + pairs_per_chunk - 1) / pairs_per_chunk;
  return true;
}

// Pair i, on `transit`, is the last of its run, whose start is not known: the same question.
__device__ __forceinline__ bool workgroup_run_of_tail(const uint32_t* __restrict__ keys, uint32_t i, uint32_t transit,
                                                      const EdgePos_t* __restrict__ row_ptr, uint32_t step_size,
                                                      uint32_t* transit_out, uint32_t* start_out,
                                                      uint32_t* count_out, uint32_t* n_items_out,
                                                      uint32_t* refused_out = nullptr, EdgePos_t* begin_out = nullptr,
                                                      EdgePos_t* degree_out = nullptr) {
  // pairs a run needs for the workgroup kernel; a shorter run is ruled out with one read
  const uint32_t needed = (kWorkgroupWork + step_size - 1) / step_size;
  if (i + 1 < needed || keys[i + 1 - needed] != transit) return false;
  const uint32_t start = run_start(keys, i + 1 - needed, transit);
  return workgroup_takes_run(transit, start, i + 1 - start, row_ptr, step_size, transit_out, start_out, count_out,
                             n_items_out, refused_out, begin_out, degree_out);
}

// Every lane looks at kClassifyItems consecutive pairs.  The work items of a workgroup's
// runs are claimed with ONE atomic per workgroup or wavefront (atomics on a single counter are served
// one after the other, ~10 ns each: one per run cost 3 ms on 1.5e5 qualifying runs); their
// order in the list is irrelevant to the results.  The list is sized so that every claim
// fits (see Engine::alloc); should one not fit, the transit is left to the flat kernel and
// the entries that did fit are processed twice with identical results.
// When the classifications of the two steps before found nothing for the workgroup kernel (or did
// not look; two, because walks on a bipartite graph meet its hubs every other step), this one
// only looks every kQuietLookEvery-th step: on a map where no transit carries
// enough pairs, as with one walk per vertex of a large graph, most launches end at once.
// found_by_step[k] != 0: step k's classification found a run; cleared before every pass.  What
// a step's classification decides never changes a result, only which kernel draws it.
constexpr uint32_t kQuietLookEvery = 4;

template <int kClassifyItems, int kThreads = 256>
__global__ __launch_bounds__(kThreads) void classify_run_tails(const uint32_t* __restrict__ keys,
                                                          const uint32_t* __restrict__ n_dev, RunsMeta* meta,
                                                          RunsMeta* meta_of_next_step,
                                                          const EdgePos_t* __restrict__ row_ptr, uint32_t step_size,
                                                          WorkItem* __restrict__ chunks, uint32_t chunk_capacity,
                                                          uint32_t* __restrict__ taken_stamp,
                                                          ClassCounters* __restrict__ counters,
                                                          uint32_t* __restrict__ found_by_step, uint32_t step) {
  __shared__ uint32_t s_wave[kThreads / kWave];
  __shared__ uint32_t s_base;
  const uint32_t n = *n_dev;
  const uint32_t stamp = meta->stamp;
  // the work-item counters alternate between steps: this launch clears the one the next
  // step will count into (its last reader, the previous step's workgroup kernel, is done)
  // and hands the next step its stamp
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    meta_of_next_step->n_chunks = 0;
    meta_of_next_step->stamp = next_stamp(stamp);
  }
  if (step > 2 && found_by_step[step - 1] == 0 && found_by_step[step - 2] == 0 && step % kQuietLookEvery != 0) return;
  if (blockIdx.x == 0 && threadIdx.x == 0) atomicAdd(&counters->sorted_pairs, (unsigned long long)n);
  const uint64_t first = ((uint64_t)blockIdx.x * kThreads + threadIdx.x) * kClassifyItems;
  uint32_t transit, start, count, n_items;
  EdgePos_t begin = 0, degree = 0;
  // the first run the lane found stays in registers for the second sweep (few lanes find two)
  int kept_k = -1;
  uint32_t kept_transit = 0, kept_start = 0, kept_count = 0, kept_items = 0;
  EdgePos_t kept_begin = 0, kept_degree = 0;
  uint32_t mine = 0;
  uint32_t single_pairs = 0, split_pairs = 0, refused_pairs = 0;
  // the lane's keys and the one after them, fetched together (16 bytes at a time where the lane
  // has a multiple of four keys and all of them exist): only the last pair of a run reads more
  uint32_t held[kClassifyItems + 1];
  if (kClassifyItems % 4 == 0 && first + kClassifyItems < n && (reinterpret_cast<uintptr_t>(keys) & 15u) == 0) {
#pragma unroll
    for (int k = 0; k < kClassifyItems; k += 4) {
      const uint4 four = *reinterpret_cast<const uint4*>(keys + first + k);
      held[k] = four.x;
      held[k + 1] = four.y;
      held[k + 2] = four.z;
      held[k + 3] = four.w;
    }
    held[kClassifyItems] = keys[first + kClassifyItems];
  } else {
#pragma unroll
    for (int k = 0; k <= kClassifyItems; ++k) held[k] = first + k < n ? keys[first + k] : 0u;
  }
  uint32_t tails = 0;  // bit k: pair first + k is the last of its run
#pragma unroll
  for (int k = 0; k < kClassifyItems; ++k) {
    const uint64_t i = first + k;
    if (i < n && (i + 1 == n || held[k + 1] != held[k])) tails |= 1u << k;
  }
  // Where the run that a lane's first tail closes starts: after the last tail of the lanes
  // before it in the wavefront (their keys are the ones just before the lane's own).  Only a
  // run that began before the wavefront's first key is searched for in memory.
  uint32_t start_known;  // 0: not known; else the start of the run the next tail closes
  {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    uint32_t after_last = tails ? (uint32_t)first + (31u - (uint32_t)__clz(tails)) + 1u : 0u;
    for (int d = 1; d < kWave; d <<= 1) {
      const uint32_t other = __shfl_up(after_last, d, kWave);
      if (lane >= (uint32_t)d && other > after_last) after_last = other;
    }
    start_known = __shfl_up(after_last, 1, kWave);
    if (lane == 0) start_known = 0;
  }
#pragma unroll
  for (int k = 0; k < kClassifyItems; ++k) {
    uint32_t refused = 0;
    if (((tails >> k) & 1u) == 0) continue;
    const uint32_t i = (uint32_t)(first + k);
    const bool takes = start_known != 0
                           ? workgroup_takes_run(held[k], start_known, i + 1 - start_known, row_ptr, step_size,
                                                 &transit, &start, &count, &n_items, &refused, &begin, &degree)
                           : workgroup_run_of_tail(keys, i, held[k], row_ptr, step_size, &transit, &start, &count,
                                                   &n_items, &refused, &begin, &degree);
    start_known = i + 1;
    if (takes) {
      if (kept_k < 0) {
        kept_k = k;
        kept_transit = transit;
        kept_start = start;
        kept_count = count;
        kept_items = n_items;
        kept_begin = begin;
        kept_degree = degree;
      }
      mine += n_items;
      if (n_items > 1) split_pairs += count; else single_pairs += count;
    }
    refused_pairs += refused;
  }
  {
    // the wavefront's counts, added by one lane to the wavefront's copy of the counters
    uint32_t items = mine;
    for (int d = 1; d < kWave; d <<= 1) {
      single_pairs += __shfl_xor(single_pairs, d, kWave);
      split_pairs += __shfl_xor(split_pairs, d, kWave);
      refused_pairs += __shfl_xor(refused_pairs, d, kWave);
      items += __shfl_xor(items, d, kWave);
    }
    if ((threadIdx.x & (kWave - 1)) == 0) {
      ClassCounters* mine_c = counters + ((blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave) % kCounterCopies);
      if (single_pairs) atomicAdd(&mine_c->workgroup_pairs, (unsigned long long)single_pairs);
      if (split_pairs) atomicAdd(&mine_c->split_pairs, (unsigned long long)split_pairs);
      if (refused_pairs) atomicAdd(&mine_c->refused_pairs, (unsigned long long)refused_pairs);
      if (items) atomicAdd(&mine_c->work_items, (unsigned long long)items);
    }
  }
  uint32_t base;
  if (kClassifyItems == 1) {
    // small maps: one atomic per wavefront, no barrier
    const uint32_t incl = wave_inclusive_scan(mine);
    const uint32_t wave_total = __shfl(incl, kWave - 1, kWave);
    if (wave_total == 0) return;  // the same for every lane of the wavefront
    uint32_t wave_base = 0;
    if ((threadIdx.x & (kWave - 1)) == kWave - 1) wave_base = atomicAdd(&meta->n_chunks, wave_total);
    base = __shfl(wave_base, kWave - 1, kWave) + incl - mine;
  } else {
    uint32_t block_total;
    base = block_exclusive_scan<kThreads>(mine, s_wave, &block_total);
    if (block_total == 0) return;  // the same for every lane of the workgroup
    if (threadIdx.x == 0) s_base = atomicAdd(&meta->n_chunks, block_total);
    __syncthreads();
    base += s_base;
  }
  if (mine == 0) return;
  uint32_t pairs_per_chunk = kChunkOutputs / step_size;
  if (pairs_per_chunk == 0) pairs_per_chunk = 1;
  for (int k = 0; k < kClassifyItems; ++k) {
    const uint64_t i = first + k;
    // one pair per lane: the run found above is still in the registers
    if (kClassifyItems > 1) {
      if (k == kept_k) {
        transit = kept_transit;
        start = kept_start;
        count = kept_count;
        n_items = kept_items;
        begin = kept_begin;
        degree = kept_degree;
      } else if (!(k > kept_k && ((tails >> k) & 1u) != 0 &&
                   workgroup_run_of_tail(keys, (uint32_t)i, keys[i], row_ptr, step_size, &transit, &start, &count,
                                         &n_items, nullptr, &begin, &degree))) {
        continue;
      }
    }
    const bool fits = base + n_items <= chunk_capacity;
    for (uint32_t g = 0; g < n_items && base + g < chunk_capacity; ++g) {
      const uint32_t off = g * pairs_per_chunk;
      WorkItem item = WorkItem();
      item.first_pair = start + off;
      item.n_pairs = count - off < pairs_per_chunk ? count - off : pairs_per_chunk;
      item.transit = (int32_t)transit;
      item.begin = begin;
      item.n_edges = degree;
      chunks[base + g] = item;
    }
    if (fits) {
      taken_stamp[transit] = stamp;
      found_by_step[step] = 1;  // the next step looks again
    }
    base += n_items;
  }
}

// ---------------------------------------------------------------------------------------
// Inversion of a small map without a sort
// ---------------------------------------------------------------------------------------
// A digit pass of the radix sort is three dependent launches, and on a map of a few ten thousand
// pairs every launch is a handful of microseconds of latency whatever it does: 57 K walks spend
// 3.5 of their 4.8 ms per pass there.  For walks over at most kSmallMapPairs pairs and
// kSmallMapVertices vertices the step kernels count, as they emit a pair, how many pairs went to
// the same next transit before it (emit_ranks, emit_counts); two launches then place every pair:
// small_map_scan turns the counts into starts inside chunks of 1024 counters and chunk totals;
// small_map_place scans the (at most 1024) chunk totals once per workgroup in LDS - cheaper than
// a third launch or a ticket that every chunk takes with an atomic on one address - and writes
// pair i to start[transit] + rank and lets the pair with rank 0 classify
// its run for the load-balancing classes, as classify_run_tails does from the run's tail.  The
// order inside a run is the order the atomics were served in; results do not depend on it
// (randomness is keyed by the slot).  The counters of a transit (StepParams::emit_counter_base)
// are consecutive, so its run is still one stretch of the placed pairs.
//
// Where the places are not many times the pairs, the two placing launches go too: every counter
// owns a fixed stretch of the next step's pair arrays, with room for twice the walks it expects
// from its share of the edge ends, and the emitting lane writes its pair straight to stretch
// start + rank (StepParams::emit_place_start; the few pairs whose rank does not fit take a place
// after all stretches).  The next step's launch has a lane for every place and skips the empty
// ones; the lane that takes a pair marks its place empty again and the first lanes clear the
// counters, so two sets of arrays alternate without a launch of their own.  A step is then one
// launch (8.4 us on 56,944 walks, against 18.2 us for the three launches of count, place and
// step); every pair goes to the flat lanes - the transits many walks share keep their adjacency
// in the caches of a map this small - so nothing is classified.  ND_SMALL_MAP=1 keeps the two
// placing launches, ND_SMALL_MAP=0 the sort.
constexpr uint32_t kSmallMapPairs = 1u << 17;
constexpr uint32_t kSmallMapCounters = 1u << 20;  // counters of all vertices at most
constexpr uint32_t kSmallMapWalksPerCounter = 16;   // a vertex expected to take more walks per step gets copies
constexpr uint32_t kSmallMapMaxCopies = 256;
constexpr uint32_t kSmallMapChunk = 1024;  // counters per workgroup of small_map_scan; at most 1024 chunks
constexpr uint32_t kSmallMapSparePlaces = 4;    // places of a counter beyond twice the walks it expects
constexpr size_t kSmallMapPlacesPerPair = 12;   // placing at emission: places of all counters per pair at most

__global__ __launch_bounds__(256) void small_map_scan(uint32_t* __restrict__ counts, uint32_t n_counters,
                                                      uint32_t* __restrict__ local_start,
                                                      uint32_t* __restrict__ chunk_total) {
  __shared__ uint32_t s_wave[kScanThreads / kWave];
  const uint32_t first = blockIdx.x * kSmallMapChunk + threadIdx.x * 4u;
  uint32_t c[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) c[k] = first + k < n_counters ? counts[first + k] : 0u;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if (c[k]) counts[first + k] = 0;  // ready for the pairs the coming step emits
  }
  uint32_t block_total;
  uint32_t before = block_exclusive_scan_256(c[0] + c[1] + c[2] + c[3], s_wave, &block_total);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if (first + k < n_counters) local_start[first + k] = before;
    before += c[k];
  }
  if (threadIdx.x == 0) chunk_total[blockIdx.x] = block_total;
}

__global__ __launch_bounds__(256) void small_map_place(
    const uint32_t* __restrict__ emit_keys, const uint32_t* __restrict__ emit_slots,
    const uint32_t* __restrict__ emit_state, const uint32_t* __restrict__ emit_ranks, const uint32_t* __restrict__ n_in_dev,
    uint32_t n_in_host, uint32_t invalid, const uint32_t* __restrict__ counter_base, const uint32_t* __restrict__ local_start,
    const uint32_t* __restrict__ chunk_total, uint32_t n_chunks, uint32_t* __restrict__ live_out,
    uint32_t* __restrict__ keys_out, uint32_t* __restrict__ slots_out,
    uint32_t* __restrict__ state_out,
    // load balancing (classify == 0: none of it)
    uint32_t classify, RunsMeta* meta, RunsMeta* meta_of_next_step, const EdgePos_t* __restrict__ row_ptr,
    uint32_t step_size, WorkItem* __restrict__ chunks, uint32_t chunk_capacity, uint32_t* __restrict__ taken_stamp,
    ClassCounters* __restrict__ counters) {
  __shared__ uint32_t s_wave[kScanThreads / kWave];
  __shared__ uint32_t chunk_base[1024];
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  // the pair's own words do not wait for the chunk scan; n_in_host bounds the arrays
  uint32_t transit = invalid, rank = 0, slot = 0, state = 0;
  if (i < n_in_host) {
    transit = emit_keys[i];
    rank = emit_ranks[i];
    slot = emit_slots[i];
    if (state_out) state = emit_state[i];
  }
  const uint32_t n_in = n_in_dev ? *n_in_dev : n_in_host;
  if (i >= n_in) transit = invalid;
  {
    // where every chunk starts among the placed pairs
    uint32_t t[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) t[k] = threadIdx.x * 4u + k < n_chunks ? chunk_total[threadIdx.x * 4u + k] : 0u;
    uint32_t total;
    uint32_t base = block_exclusive_scan_256(t[0] + t[1] + t[2] + t[3], s_wave, &total);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      chunk_base[threadIdx.x * 4u + k] = base;
      base += t[k];
    }
    __syncthreads();
    if (i == 0) {
      *live_out = total;  // pairs that go on: what the step kernels of this step walk
      if (classify) {
        meta_of_next_step->n_chunks = 0;  // see classify_run_tails
        meta_of_next_step->stamp = next_stamp(meta->stamp);
        atomicAdd(&counters->sorted_pairs, (unsigned long long)total);
      }
    }
  }
  uint32_t start = 0, count = 0, n_items = 0, refused = 0;
  bool head = false;
  {
    if (transit != invalid) {
      const uint32_t first_copy = counter_base[transit];
      const uint32_t beyond = counter_base[transit + 1];  // the counter after the last one exists
      const uint32_t mine = first_copy + (i & (beyond - first_copy - 1u));
      const uint32_t pos = chunk_base[mine / kSmallMapChunk] + local_start[mine] + rank;
      keys_out[pos] = transit;
      slots_out[pos] = slot;
      if (state_out) state_out[pos] = state;
      if (rank == 0) {
        // the first pair of the first copy that counted any is the first pair of the run
        const uint32_t run_start = chunk_base[first_copy / kSmallMapChunk] + local_start[first_copy];
        if (pos == run_start) {
          head = true;
          start = pos;
          count = chunk_base[beyond / kSmallMapChunk] + local_start[beyond] - run_start;
        }
      }
    }
  }
  if (!classify) return;
  // the run's class, decided by its first pair (rules of workgroup_run_of_tail)
  EdgePos_t begin = 0;
  uint32_t degree = 0;
  if (head) {
    const uint64_t work = (uint64_t)count * step_size;
    begin = row_ptr[transit];
    degree = (uint32_t)(row_ptr[transit + 1] - begin);
    if (work >= kWorkgroupWork && degree != 0) {
      if (degree > (uint32_t)kCacheEdges || (uint64_t)degree > 32ull * work) {
        refused = count;
      } else {
        uint32_t pairs_per_chunk = kChunkOutputs / step_size;
        if (pairs_per_chunk == 0) pairs_per_chunk = 1;
        n_items = (count + pairs_per_chunk - 1) / pairs_per_chunk;
      }
    }
  }
  uint32_t single_pairs = n_items == 1 ? count : 0, split_pairs = n_items > 1 ? count : 0, items = n_items;
  for (int d = 1; d < kWave; d <<= 1) {
    single_pairs += __shfl_xor(single_pairs, d, kWave);
    split_pairs += __shfl_xor(split_pairs, d, kWave);
    refused += __shfl_xor(refused, d, kWave);
    items += __shfl_xor(items, d, kWave);
  }
  if ((threadIdx.x & (kWave - 1)) == 0) {
    ClassCounters* mine_c = counters + ((blockIdx.x * (256 / kWave) + threadIdx.x / kWave) % kCounterCopies);
    if (single_pairs) atomicAdd(&mine_c->workgroup_pairs, (unsigned long long)single_pairs);
    if (split_pairs) atomicAdd(&mine_c->split_pairs, (unsigned long long)split_pairs);
    if (refused) atomicAdd(&mine_c->refused_pairs, (unsigned long long)refused);
    if (items) atomicAdd(&mine_c->work_items, (unsigned long long)items);
  }
  if (items == 0) return;  // the same for every lane of the wavefront
  const uint32_t incl = wave_inclusive_scan(n_items);
  uint32_t wave_base = 0;
  if ((threadIdx.x & (kWave - 1)) == kWave - 1) wave_base = atomicAdd(&meta->n_chunks, incl);
  const uint32_t base = __shfl(wave_base, kWave - 1, kWave) + incl - n_items;
  if (n_items == 0) return;
  uint32_t pairs_per_chunk = kChunkOutputs / step_size;
  if (pairs_per_chunk == 0) pairs_per_chunk = 1;
  for (uint32_t g = 0; g < n_items && base + g < chunk_capacity; ++g) {
    const uint32_t off = g * pairs_per_chunk;
    WorkItem item = WorkItem();
    item.first_pair = start + off;
    item.n_pairs = count - off < pairs_per_chunk ? count - off : pairs_per_chunk;
    item.transit = (int32_t)transit;
    item.begin = begin;
    item.n_edges = (EdgePos_t)degree;
    chunks[base + g] = item;
  }
  if (base + n_items <= chunk_capacity) taken_stamp[transit] = meta->stamp;
}

__global__ void fill_i32(int32_t* dst, size_t n, int32_t value) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = value;
}

// ---------------------------------------------------------------------------------------
// Final-sample assembly
// ---------------------------------------------------------------------------------------

constexpr int kMaxSteps = 128;
#ifndef ND_ASSEMBLE_ROWS
#define ND_ASSEMBLE_ROWS 64
#endif
constexpr uint32_t kAssembleRows = ND_ASSEMBLE_ROWS;  // rows a workgroup of the final assembly stages at most

struct StepLayout {
  int n_steps;
  uint32_t seg_base[kMaxSteps];  // offset of the step's segment inside a final sample
  uint32_t seg_len[kMaxSteps];   // outputs of the step per sample
};

// The step kernels leave step k's outputs in one array per step, grouped by sample
// (step_out_k[s * len_k + j]).  The result layout is one row per sample
// (final[s * F + base_k + j], getFinalSamples: src/nextdoor.cu:3211-3237).  A workgroup
// stages the rows of a block of samples in LDS (row pitch padded to an odd word count) and
// writes them out as whole contiguous lines, so HBM sees each result byte written once.
__global__ __launch_bounds__(256) void assemble_final_rows(const int32_t* __restrict__ step_out,
                                                           int32_t* __restrict__ final_samples, uint32_t n_samples,
                                                           uint32_t final_size, uint32_t row_pitch,
                                                           uint32_t samples_per_block, StepLayout layout) {
  extern __shared__ int32_t s_rows[];
  const uint32_t s0 = blockIdx.x * samples_per_block;
  const uint32_t nb = n_samples - s0 < samples_per_block ? n_samples - s0 : samples_per_block;
  // Steps whose slice of this block is narrower than the workgroup (walks: one entry per
  // sample and step) are read several steps at a time, so that all lanes have a load in
  // flight; wider slices one step at a time.
  int k = 0;
  while (k < layout.n_steps) {
    const uint32_t len = layout.seg_len[k];
    const uint32_t slice = nb * len;
    uint32_t group = slice >= 256 ? 1u : 256u / slice;
    uint32_t same = 1;  // consecutive steps with the same segment length
    while (same < group && k + (int)same < layout.n_steps && layout.seg_len[k + same] == len) ++same;
    group = same;
    for (uint32_t e = threadIdx.x; e < slice * group; e += 256) {
      const uint32_t g = e / slice;
      const uint32_t within = e - g * slice;
      const uint32_t s = len == 1 ? within : within / len;
      const uint32_t j = within - s * len;
      const uint32_t base = layout.seg_base[k + g];
      s_rows[s * row_pitch + base + j] = step_out[(size_t)n_samples * base + (size_t)s0 * len + within];
    }
    k += (int)group;
  }
  __syncthreads();
  int32_t* dst = final_samples + (size_t)s0 * final_size;
  for (uint32_t e = threadIdx.x; e < nb * final_size; e += 256) {
    const uint32_t s = e / final_size;
    dst[e] = s_rows[s * row_pitch + (e - s * final_size)];
  }
}

// The same for walks (every step contributes one id per sample: step_out[k * n_samples + s], or,
// paired != 0, the 8-byte cells two steps share, see StepParams::pair_cells),
// without the index arithmetic of the general case: a wavefront reads 64 consecutive samples
// of one step, and the rows are written out with running (row, column) counters.
__global__ __launch_bounds__(256) void assemble_walk_rows(const int32_t* __restrict__ step_out,
                                                          int32_t* __restrict__ final_samples, uint32_t n_samples,
                                                          uint32_t n_steps, uint32_t row_pitch,
                                                          uint32_t samples_per_block, uint32_t paired,
                                                          const uint32_t* __restrict__ walk_cells, int32_t invalid) {
  extern __shared__ int32_t s_rows[];
  const uint32_t s0 = blockIdx.x * samples_per_block;
  const uint32_t nb = n_samples - s0 < samples_per_block ? n_samples - s0 : samples_per_block;
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  for (uint32_t first = 0; first < nb; first += 64u) {
    const uint32_t s = first + lane;
    if (s >= nb) continue;
    if (paired) {
      const int2* cells = reinterpret_cast<const int2*>(step_out);
      // (walk_cells: the cells beyond the walk's last one were never written)
      const uint32_t written = walk_cells ? walk_cells[s0 + s] : ~0u;
      for (uint32_t j = wave; 2u * j < n_steps; j += 4u) {
        const int2 c = j < written ? cells[(size_t)j * n_samples + s0 + s] : make_int2(invalid, invalid);
        s_rows[s * row_pitch + 2u * j] = c.x;
        if (2u * j + 1u < n_steps) s_rows[s * row_pitch + 2u * j + 1u] = c.y;
      }
    } else {
      for (uint32_t k = wave; k < n_steps; k += 4u) s_rows[s * row_pitch + k] = step_out[(size_t)k * n_samples + s0 + s];
    }
  }
  __syncthreads();
  int32_t* dst = final_samples + (size_t)s0 * n_steps;
  const uint32_t total = nb * n_steps;
  uint32_t row = threadIdx.x / n_steps, col = threadIdx.x - row * n_steps;
  const uint32_t row_step = 256u / n_steps, col_step = 256u - row_step * n_steps;
  for (uint32_t e = threadIdx.x; e < total; e += 256u) {
    dst[e] = s_rows[row * row_pitch + col];
    row += row_step;
    col += col_step;
    if (col >= n_steps) {
      col -= n_steps;
      row++;
    }
  }
}

// Fallback for rows too long to stage: one launch per step, straight copy.
__global__ void assemble_final_step(const int32_t* __restrict__ src, int32_t* __restrict__ final_samples,
                                    size_t n_elems, uint32_t len, uint32_t final_size, uint32_t seg_base) {
  const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n_elems) return;
  const size_t s = e / len;
  final_samples[s * final_size + seg_base + (e - s * len)] = src[e];
}

// ---------------------------------------------------------------------------------------
// Shape algebra (nextdoor.cu:126-197, 1913-1929)
// ---------------------------------------------------------------------------------------

template <class App>
inline bool is_collective() { return App().samplingType() == CollectiveNeighborhood; }

template <class App>
inline int64_t step_size_at_step(int step) {
  if (step == -1) return 0;
  int64_t n = is_collective<App>() ? 0 : (int64_t)App().initialSampleSize(nullptr);
  for (int i = 0; i <= step; ++i) {
    if (is_collective<App>()) n += App().stepSize(i); else n *= App().stepSize(i);
  }
  return n;
}

// Individual apps: every output slot of every step has its place in the result row, so the
// row holds initialSampleSize * stepSize(0) * ... * stepSize(k) entries for step k.  (The
// reference's getFinalSampleSize, nextdoor.cu:1913-1929, starts the product at 1; that is the
// same for its apps with one root per sample, and too short for the slots of the others.)
template <class App>
inline int final_sample_size() {
  int64_t total = 0, per_step = is_collective<App>() ? 1 : (int64_t)App().initialSampleSize(nullptr);
  for (int k = 0; k < App().steps(); ++k) {
    if (is_collective<App>()) per_step = App().stepSize(k); else per_step *= App().stepSize(k);
    total += per_step;
  }
  return (int)total;
}

// ---------------------------------------------------------------------------------------
// Engine
// ---------------------------------------------------------------------------------------

template <class SampleType, class App>
class Engine : public EngineBase {
 public:
  explicit Engine(const char* name) : name_(name) {}
  ~Engine() override { free_device(); }

  const char* app_name() const override { return name_; }
  int64_t num_samples() const override { return n_samples_; }
  int final_sample_size() const override { return nd::final_sample_size<App>(); }
  bool has_explicit_transits() const override { return App().hasExplicitTransits(); }
  int steps() const override { return App().steps(); }
  int step_size(int k) const override { return App().stepSize(k); }
  int initial_sample_size() const override { return App().initialSampleSize(nullptr); }
  int sampling_type() const override { return App().samplingType(); }
  int32_t invalid_vertex() const override { return invalid_; }
  int max_bits() const override { return max_bits_; }
  size_t sample_state_bytes() const override {
    return std::is_empty<SampleType>::value ? 0 : sizeof(SampleType) * (size_t)n_samples_;
  }

  // transferCSRToGPUs: the whole graph is resident on the device, plus the derived
  // structures the app asks for (interleaved edges, edge index).
  int set_graph(const CSR* graph) override {
    free_run_buffers();  // sized against the previous graph: alloc() is due again
    graph_ = nullptr;
    dgraph_ = std::make_shared<DeviceGraph>();
    if (!dgraph_->upload(graph, app_uses_weights<App>::value, app_uses_edge_lookup<App>::value, &last_error)) return -1;
    graph_ = graph;
    view_ = dgraph_->view;
    return 0;
  }

  // The device graph another engine of the same app has uploaded (engines that each sample
  // a range of the samples share one copy).
  void share_graph(const Engine& other) {
    dgraph_ = other.dgraph_;
    graph_ = other.graph_;
    view_ = other.view_;
  }

  int alloc(uint64_t seed) override { return alloc_range(seed, 0, -1); }

  // allocNextDoorDataOnGPU: run the host half of the App (numSamples, initializeSample,
  // initialSample) and allocate every per-run buffer once.
  // Allocates for samples [first, first + count) of the app's samples (count < 0: all).
  // Sample indices, roots and random streams are those of the whole run, so the ranges of
  // several engines put together are the bytes one engine produces for everything.
  // host_rows false: the caller fetches the rows into memory of its own (fetch_final_samples_into).
  int alloc_range(uint64_t seed, int64_t first, int64_t count, bool host_rows = true) {
    if (!graph_) { last_error = "alloc before set_graph"; return -1; }
    free_run_buffers();
    seed_ = seed;
    CSR* csr = const_cast<CSR*>(graph_);
    App app;
    if (is_collective<App>()) { last_error = "collective apps need the layer engine"; return -2; }
    const int n_steps = app.steps();
    if (n_steps < 1 || n_steps > kMaxSteps) { last_error = "steps() must be in [1, 128]"; return -2; }
    for (int k = 0; k < n_steps; ++k)
      if (app.stepSize(k) <= 0) { last_error = "stepSize must be positive (ALL_NEIGHBORS is not supported)"; return -2; }
    const int64_t all_samples = app.numSamples(csr);
    if (first < 0 || first > all_samples || (count >= 0 && first + count > all_samples)) {
      last_error = "sample range outside the app's samples";
      return -2;
    }
    first_sample_ = first;
    n_samples_ = count < 0 ? all_samples - first : count;
    init_size_ = app.initialSampleSize(csr);
    if (n_samples_ <= 0 || init_size_ <= 0) { last_error = "app yields no samples"; return -2; }
    invalid_ = graph_->get_n_vertices();  // nextdoor.cu:1993
    max_bits_ = 0;
    while ((invalid_ >> max_bits_) != 0) max_bits_++;

    samples_.clear();
    initialContents.clear();
    samples_.reserve((size_t)n_samples_);
    initialContents.reserve((size_t)n_samples_ * init_size_);
    for (int64_t s = 0; s < n_samples_; ++s) {
      samples_.push_back(app.template initializeSample<SampleType>(csr, (VertexID_t)(first_sample_ + s)));
      std::vector<VertexID_t> roots = app.initialSample((int)(first_sample_ + s), csr, samples_.back());
      if ((EdgePos_t)roots.size() != init_size_) {
        last_error = "initialSample size differs from initialSampleSize";  // nextdoor.cu:1964-1969
        return -2;
      }
      if (!roots_are_vertices(roots, graph_->get_n_vertices())) {
        last_error = "initialSample returned a root that is not a vertex of the graph";
        return -2;
      }
      initialContents.insert(initialContents.end(), roots.begin(), roots.end());
    }

    // shape of every step
    layout_.n_steps = n_steps;
    uint64_t pairs = (uint64_t)n_samples_ * init_size_, max_pairs = 0, max_outputs = 0, chunk_cap = 0;
    uint64_t per_sample = (uint64_t)init_size_, base = 0;
    for (int k = 0; k < n_steps; ++k) {
      const uint64_t mk = (uint64_t)app.stepSize(k);
      if (k > 0 && pairs > max_pairs) max_pairs = pairs;  // step 0 is not sorted
      // work-item list: a run of `count` pairs emits ceil(count / pairsPerChunk) items and at
      // most outputs / kWorkgroupWork runs qualify, so this bound holds at every step
      uint64_t per_chunk = kChunkOutputs / mk;
      if (per_chunk == 0) per_chunk = 1;
      const uint64_t need = pairs / per_chunk + pairs * mk / kWorkgroupWork + 2;
      if (need > chunk_cap) chunk_cap = need;
      pairs *= mk;
      per_sample *= mk;
      if (pairs > max_outputs) max_outputs = pairs;
      layout_.seg_base[k] = (uint32_t)base;
      layout_.seg_len[k] = (uint32_t)per_sample;
      base += per_sample;
    }
    if (max_outputs >= (1ull << 32) || max_pairs >= (1ull << 31)) {
      last_error = "a step has 2^32 or more outputs; split the samples over several runs";
      return -2;
    }
    if (max_pairs == 0) max_pairs = 1;
    max_pairs_ = (size_t)max_pairs;
    chunk_capacity_ = (uint32_t)chunk_cap;
    const size_t F = (size_t)final_sample_size();
    if (base != F) { last_error = "the steps' segments do not add up to the final sample size"; return -2; }
    if (host_rows) hFinalSamples.assign((size_t)n_samples_ * F, invalid_); else hFinalSamples.clear();

    ND_HIP_TRY(hipStreamCreate(&stream_));
    ND_HIP_TRY(hipMalloc(&d_initial_, sizeof(VertexID_t) * initialContents.size()));
    ND_HIP_TRY(hipMemcpy(d_initial_, initialContents.data(), sizeof(VertexID_t) * initialContents.size(),
                         hipMemcpyHostToDevice));
    if (!std::is_empty<SampleType>::value) {
      // the states initializeSample produced stay on the device; every run starts from a copy
      ND_HIP_TRY(hipMalloc(&d_samples_, sizeof(SampleType) * (size_t)n_samples_));
      ND_HIP_TRY(hipMalloc(&d_samples_init_, sizeof(SampleType) * (size_t)n_samples_));
      ND_HIP_TRY(hipMemcpy(d_samples_init_, samples_.data(), sizeof(SampleType) * (size_t)n_samples_,
                           hipMemcpyHostToDevice));
      // what fetch_sample_states gives before the first run
      ND_HIP_TRY(hipMemcpy(d_samples_, d_samples_init_, sizeof(SampleType) * (size_t)n_samples_,
                           hipMemcpyDeviceToDevice));
    }
    ND_HIP_TRY(hipMalloc(&d_final_, sizeof(VertexID_t) * (size_t)n_samples_ * F));
    // Steps whose segment of a result row is at least a memory line long write straight
    // into the rows; short segments (walks: one id per step) would touch a separate line of
    // the result per output, so they go to one array per step and are regrouped at the end.
    rows_direct_ = true;
    for (int k = 0; k < n_steps; ++k) rows_direct_ = rows_direct_ && layout_.seg_len[k] >= kDirectSegment;
    // (one more column where the steps of a walk are odd in number: its results go in cells of two)
    if (!rows_direct_) ND_HIP_TRY(hipMalloc(&d_step_out_, sizeof(VertexID_t) * (size_t)n_samples_ * (F + 1)));
    ND_HIP_TRY(hipMalloc(&d_keys_a_, sizeof(uint32_t) * max_pairs_));
    ND_HIP_TRY(hipMalloc(&d_vals_a_, sizeof(uint32_t) * max_pairs_));
    ND_HIP_TRY(hipMalloc(&d_keys_b_, sizeof(uint32_t) * max_pairs_));
    ND_HIP_TRY(hipMalloc(&d_vals_b_, sizeof(uint32_t) * max_pairs_));
    const SortPlan plan = make_sort_plan(max_pairs_, max_bits_);
    ND_HIP_TRY(hipMalloc(&d_hist_, sizeof(uint32_t) * sort_hist_capacity(max_pairs_)));
    ND_HIP_TRY(hipMalloc(&d_scratch_, sizeof(uint32_t) * plan.scratch_elems));
    ND_HIP_TRY(hipMalloc(&d_live_, sizeof(uint32_t) * 2));
    // walks: every step has one pair per sample and one output per pair
    walk_mode_ = init_size_ == 1 && n_steps > 1;
    for (int k = 0; k < n_steps; ++k) walk_mode_ = walk_mode_ && app.stepSize(k) == 1;
    state_travels_ = walk_mode_ && state_fits_pair<SampleType>::value;
    // apps that choose their transits themselves and are not walks: the next step's map is an
    // array of its own, written next to the step's outputs
    explicit_map_ = app.hasExplicitTransits() && !walk_mode_;
    if (explicit_map_) ND_HIP_TRY(hipMalloc(&d_explicit_, sizeof(VertexID_t) * max_pairs_));
    if (walk_mode_) {
      ND_HIP_TRY(hipMalloc(&d_emit_keys_, sizeof(uint32_t) * max_pairs_));
      ND_HIP_TRY(hipMalloc(&d_emit_slots_, sizeof(uint32_t) * max_pairs_));
    }
    // Counters per vertex for the small-map inversion: the walks that step onto a vertex are
    // about its share of the edge ends; one counter per kSmallMapWalksPerCounter of them.
    small_map_ = false;
    if (walk_mode_ && max_pairs_ <= kSmallMapPairs && (uint64_t)invalid_ < kSmallMapCounters &&
        !(getenv("ND_SMALL_MAP") && atoi(getenv("ND_SMALL_MAP")) == 0)) {
      const size_t V = (size_t)graph_->get_n_vertices();
      const double per_edge = graph_->col.empty() ? 0.0 : (double)max_pairs_ / (double)graph_->col.size();
      std::vector<uint32_t> base(V + 1), edges_into(V, 0), place_start(1, 0u);
      for (const CSR::Edge dst : graph_->col) edges_into[(size_t)dst]++;
      uint64_t at = 0;
      for (size_t v = 0; v < V; ++v) {
        base[v] = (uint32_t)at;
        const double walks = per_edge * (double)edges_into[v];
        uint32_t copies = 1;
        while (copies < kSmallMapMaxCopies && (double)(copies * kSmallMapWalksPerCounter) < walks) copies <<= 1;
        at += copies;
        // places of each of its counters when the pairs are placed as they are emitted: twice
        // the walks it expects and a few more
        const uint32_t places = (uint32_t)(2.0 * walks / copies) + kSmallMapSparePlaces;
        for (uint32_t c = 0; c < copies; ++c) place_start.push_back(place_start.back() + places);
      }
      base[V] = (uint32_t)at;
      small_counters_ = (size_t)at + 1;  // one more, so that every run has an end to read
      place_start.push_back(place_start.back());  // ... which owns no place
      small_map_ = small_counters_ < kSmallMapCounters;
      if (small_map_) {
        ND_HIP_TRY(hipMalloc(&d_counter_base_, sizeof(uint32_t) * base.size()));
        ND_HIP_TRY(hipMemcpy(d_counter_base_, base.data(), sizeof(uint32_t) * base.size(), hipMemcpyHostToDevice));
      }
      // Placing at emission walks every place at every step: only where the places are not many
      // times the pairs (ND_SMALL_MAP=1 keeps the two placing launches).
      small_placed_ = small_map_ && (size_t)place_start.back() <= kSmallMapPlacesPerPair * max_pairs_ &&
                      !(getenv("ND_SMALL_MAP") && atoi(getenv("ND_SMALL_MAP")) == 1);
      if (small_placed_) {
        placed_spill_first_ = place_start.back();
        placed_places_ = (size_t)placed_spill_first_ + max_pairs_;  // every pair could spill
        ND_HIP_TRY(hipMalloc(&d_place_start_, sizeof(uint32_t) * place_start.size()));
        ND_HIP_TRY(hipMemcpy(d_place_start_, place_start.data(), sizeof(uint32_t) * place_start.size(),
                             hipMemcpyHostToDevice));
        for (int b = 0; b < 2; ++b) {
          ND_HIP_TRY(hipMalloc(&d_placed_keys_[b], sizeof(uint32_t) * placed_places_));
          ND_HIP_TRY(hipMalloc(&d_placed_slots_[b], sizeof(uint32_t) * placed_places_));
          ND_HIP_TRY(hipMemset(d_placed_slots_[b], 0, sizeof(uint32_t) * placed_places_));
          if (state_fits_pair<SampleType>::value) {
            ND_HIP_TRY(hipMalloc(&d_placed_state_[b], sizeof(uint32_t) * placed_places_));
            ND_HIP_TRY(hipMemset(d_placed_state_[b], 0, sizeof(uint32_t) * placed_places_));
          }
          ND_HIP_TRY(hipMalloc(&d_placed_counts_[b], sizeof(uint32_t) * (small_counters_ + 1)));
        }
        placed_dirty_ = true;  // cleared by the first pass that uses them
      }
    }
    if (small_map_) {
      // counters, their starts inside a chunk, chunk totals
      const size_t counters = small_counters_, chunks = (counters + kSmallMapChunk - 1) / kSmallMapChunk;
      ND_HIP_TRY(hipMalloc(&d_small_, sizeof(uint32_t) * (2 * counters + chunks)));
      ND_HIP_TRY(hipMemset(d_small_, 0, sizeof(uint32_t) * (2 * counters + chunks)));
      ND_HIP_TRY(hipMalloc(&d_emit_ranks_, sizeof(uint32_t) * max_pairs_));
    }
    if (state_travels_) {
      ND_HIP_TRY(hipMalloc(&d_emit_state_, sizeof(uint32_t) * max_pairs_));
      ND_HIP_TRY(hipMalloc(&d_aux_a_, sizeof(uint32_t) * max_pairs_));
      ND_HIP_TRY(hipMalloc(&d_aux_b_, sizeof(uint32_t) * max_pairs_));
    }
    ND_HIP_TRY(hipMalloc(&d_meta_, sizeof(RunsMeta) * 2));
    {
      RunsMeta fresh[2] = {};
      fresh[0].stamp = 1;  // the first load-balanced step; every classification hands the next one its stamp
      ND_HIP_TRY(hipMemcpy(d_meta_, fresh, sizeof(fresh), hipMemcpyHostToDevice));
    }
    ND_HIP_TRY(hipMalloc(&d_balance_, sizeof(uint32_t) * kBalanceWords));
    ND_HIP_TRY(hipMemset(d_balance_, 0, sizeof(uint32_t) * kBalanceWords));
    class_counters_ = ClassCounters();
    idle_passes_ = 0;
    balanced_steps_ = 0;
    markers_cleared_at_ = 0;
    schedule_counts_ = ScheduleCounts();
    items_seen_ = false;
    ND_HIP_TRY(hipMalloc(&d_chunks_, sizeof(WorkItem) * (size_t)chunk_capacity_));
    ND_HIP_TRY(hipMalloc(&d_taken_stamp_, sizeof(uint32_t) * ((size_t)invalid_ + 1)));
    ND_HIP_TRY(hipMemset(d_taken_stamp_, 0, sizeof(uint32_t) * ((size_t)invalid_ + 1)));
    ND_HIP_TRY(hipStreamCreate(&side_stream_));
    ND_HIP_TRY(hipEventCreate(&ev_a_));
    ND_HIP_TRY(hipEventCreate(&ev_b_));
    ND_HIP_TRY(hipEventCreate(&ev_begin_));
    ND_HIP_TRY(hipEventCreate(&ev_end_));
    ND_HIP_TRY(hipEventCreateWithFlags(&ev_fork_, hipEventDisableTiming));
    ND_HIP_TRY(hipEventCreateWithFlags(&ev_join_, hipEventDisableTiming));
    forced_schedule_ = kScheduleAuto;
    if (const char* env = getenv("ND_STEP_SCHEDULE")) {
      if (strcmp(env, "serial") == 0) forced_schedule_ = kScheduleSerial;
      else if (strcmp(env, "merged") == 0) forced_schedule_ = kScheduleMerged;
      else if (strcmp(env, "forked") == 0) forced_schedule_ = kScheduleForked;
    }
    // ND_MARK_UNWRITTEN=1: a pass whose kernels write every slot of the result themselves first
    // sets the result to a value that is neither a vertex nor INVALID, so that a slot no kernel
    // wrote shows in the result instead of keeping what an earlier pass left there (for tests)
    mark_unwritten_ = false;
    if (const char* env = getenv("ND_MARK_UNWRITTEN")) mark_unwritten_ = strcmp(env, "1") == 0;

    // rows staged per workgroup by the final assembly: as many as fit 64 KiB of LDS
    row_pitch_ = (uint32_t)(F | 1);
    rows_per_block_ = (uint32_t)(65536 / (row_pitch_ * sizeof(int32_t)));
    if (rows_per_block_ > kAssembleRows) rows_per_block_ = kAssembleRows;
    if (rows_per_block_ > 0) {
      ND_HIP_TRY(hipFuncSetAttribute((const void*)assemble_final_rows, hipFuncAttributeMaxDynamicSharedMemorySize,
                                     65536));
      ND_HIP_TRY(hipFuncSetAttribute((const void*)assemble_walk_rows, hipFuncAttributeMaxDynamicSharedMemorySize,
                                     65536));
    }
    paired_results_ = walk_mode_ && !rows_direct_ && rows_per_block_ > 0 && !App().hasExplicitTransits() &&
                      !(getenv("ND_PAIRED_RESULTS") && atoi(getenv("ND_PAIRED_RESULTS")) == 0);
    if (paired_results_) ND_HIP_TRY(hipMalloc(&d_walk_cells_, sizeof(uint32_t) * (size_t)n_samples_));
    allocated_ = true;
    return 0;
  }

  // doTransitParallelSampling: the step loop.  Everything is enqueued on one stream;
  // the only host wait is at the end.
  int sample(int mode) override {
    if (!allocated_) { last_error = "sample before alloc"; return -1; }
    times = PhaseTimes();
    if (!std::is_empty<SampleType>::value) {
      ND_HIP_TRY(hipMemcpyAsync(d_samples_, d_samples_init_, sizeof(SampleType) * (size_t)n_samples_,
                                hipMemcpyDeviceToDevice, stream_));
    }
    if (balanced_steps_ - markers_cleared_at_ >= (1ull << 31)) {
      // a marker is only ever compared with the stamp of the step that reads it; stamps repeat
      // after 2^32 - 1 load-balanced steps, so the markers are wiped long before one can be
      // mistaken for a fresh one
      const size_t n = (size_t)invalid_ + 1;
      fill_i32<<<dim3((unsigned)((n + 1023) / 1024)), dim3(1024), 0, stream_>>>((int32_t*)d_taken_stamp_, n, 0);
      markers_cleared_at_ = balanced_steps_;
    }
    ND_HIP_TRY(hipStreamSynchronize(stream_));
    ND_HIP_TRY(hipEventRecord(ev_begin_, stream_));
    const int rc = wants_launch_graph() ? replay_pass(mode) : enqueue_pass(mode);
    if (rc != 0) return rc;
    ND_HIP_TRY(hipEventRecord(ev_end_, stream_));
    ND_HIP_TRY(hipStreamSynchronize(stream_));
    ND_HIP_TRY(hipEventElapsedTime(&times.end_to_end, ev_begin_, ev_end_));
    schedule_counts_.passes++;
    if (balanced_this_pass_) {
      schedule_counts_.classified_passes++;
      // after the pass and outside its timed region: what the classifications counted
      ClassCounters copies[kCounterCopies];
      ND_HIP_TRY(hipMemcpy(copies, counters_dev(), sizeof(copies), hipMemcpyDeviceToHost));
      class_counters_ = ClassCounters();
      for (const ClassCounters& c : copies) {
        class_counters_.sorted_pairs += c.sorted_pairs;
        class_counters_.workgroup_pairs += c.workgroup_pairs;
        class_counters_.split_pairs += c.split_pairs;
        class_counters_.refused_pairs += c.refused_pairs;
        class_counters_.work_items += c.work_items;
      }
      idle_passes_ = class_counters_.work_items == 0 && class_counters_.sorted_pairs != 0 ? 1 : 0;
      items_seen_ = class_counters_.work_items != 0;
    }
    return 0;
  }

  // Per-transit apps: 0 = pairs the classifications of the last load-balanced pass looked at,
  // 1 = of these, pairs on transits the workgroup kernel served as one work item, 2 = pairs on
  // transits split over several work items (grid-wide), 3 = pairs in runs long enough for the
  // workgroup kernel that stayed with the flat kernel because of the transit's degree,
  // 4 = work items; the flat kernel served 0 minus 1 minus 2.
  // Since the buffers were allocated: 5 = passes, 6 = passes whose steps were classified (a
  // pass after one that found nothing for the workgroup class is not), 7 = load-balanced steps
  // whose two classes ran as one launch, 8 = as two launches side by side on two streams,
  // 9 = one after the other.
  int64_t counter(int which) const override {
    switch (which) {
      case 0: return (int64_t)class_counters_.sorted_pairs;
      case 1: return (int64_t)class_counters_.workgroup_pairs;
      case 2: return (int64_t)class_counters_.split_pairs;
      case 3: return (int64_t)class_counters_.refused_pairs;
      case 4: return (int64_t)class_counters_.work_items;
      case 5: return (int64_t)schedule_counts_.passes;
      case 6: return (int64_t)schedule_counts_.classified_passes;
      case 7: return (int64_t)schedule_counts_.merged_steps;
      case 8: return (int64_t)schedule_counts_.forked_steps;
      case 9: return (int64_t)schedule_counts_.serial_steps;
      default: return 0;
    }
  }

  // Every launch of one pass, in order, on stream_; no host wait in between.
  int enqueue_pass(int mode) {
    App app;
    const int n_steps = app.steps();
    const size_t F = (size_t)final_sample_size();
    // With few walks per vertex hardly any two walks share a transit: the sorted order then
    // saves less in the step kernels (shared lines) than the inversion costs.
    int sort_period = inversion_period;
    if (sort_period <= 0)
      sort_period = (double)n_samples_ < kWalksPerVertexForInversion * (double)invalid_ ? kSparseInversionPeriod : 1;
    const bool sample_parallel = mode == kSampleParallel;
    if (sample_parallel && sort_period <= 1) sort_period = kSparseInversionPeriod;
    // A pass whose classifications found nothing at all for the workgroup kernel is followed by
    // passes that do not classify (nor launch the workgroup kernel); every kIdleLookEvery-th
    // pass looks again.  Results do not depend on it.
    bool balance = mode == kTransitParallelLoadBalanced && n_steps > 1 && !(walk_mode_ && sort_period > 1);
    // small maps inverted at every step, the pairs placed by the kernel that emits them: one launch
    // per step, every pair with the flat lanes (what a hub's adjacency is, is in the caches)
    const bool placed = small_placed_ && sort_period == 1 && !sample_parallel;
    if (placed) {
      balance = false;
      if (placed_dirty_) {
        // a pass that did not get to its end left pairs or counts behind
        for (int b = 0; b < 2; ++b) {
          fill_i32<<<dim3((unsigned)((placed_places_ + 1023) / 1024)), dim3(1024), 0, stream_>>>(
              (int32_t*)d_placed_keys_[b], placed_places_, invalid_);
          fill_i32<<<dim3((unsigned)((small_counters_ + 1 + 1023) / 1024)), dim3(1024), 0, stream_>>>(
              (int32_t*)d_placed_counts_[b], small_counters_ + 1, 0);
        }
      }
      placed_dirty_ = true;
    }
    if (balance && !wants_launch_graph() && idle_passes_ > 0 && idle_passes_ % kIdleLookEvery != 0) {
      balance = false;
      idle_passes_++;
    }
    balanced_this_pass_ = balance;
    if (balance)
      fill_i32<<<dim3((kBalanceWords + 255) / 256), dim3(256), 0, stream_>>>((int32_t*)d_balance_, kBalanceWords, 0);
    // pairs whose transit is INVALID are dropped by the inversion and never reach a step
    // kernel: their outputs keep this fill - unless the step kernels write the rows themselves
    // and, with every INVALID, what descends from it (StepParams::fill_levels)
    const bool kernels_fill = rows_direct_ && !explicit_map_ && !walk_mode_ && n_steps <= kMaxFillLevels;
    // walks whose results go into cells of two steps: the regrouping reads only the cells a walk
    // has written (StepParams::walk_cells)
    const bool no_fill = kernels_fill || paired_results();
    if (!no_fill || mark_unwritten_) {
      const int32_t value = no_fill ? invalid_ + 1 : invalid_;
      const size_t n_out = (size_t)n_samples_ * (paired_results() ? (F + 1) / 2 * 2 : F);
      fill_i32<<<dim3((unsigned)((n_out + 1023) / 1024)), dim3(1024), 0, stream_>>>(
          rows_direct_ ? d_final_ : d_step_out_, n_out, value);
    }

    uint32_t transits_per_sample = (uint32_t)init_size_;
    const uint32_t* live_last = nullptr;  // pairs the last inversion kept (device count)
    int sorts_done = 0;
    const int32_t* transits = d_initial_;  // (sample -> transit) map entering the step
    KeyLayout transits_layout;             // and how it is laid out
    for (int step = 0; step < n_steps; ++step) {
      const uint32_t m = (uint32_t)app.stepSize(step);
      const uint32_t n_pairs = (uint32_t)((uint64_t)n_samples_ * transits_per_sample);
      StepParams P;
      P.csr = view_;
      P.step = step;
      P.step_size = m;
      P.transits_per_sample = transits_per_sample;
      P.seg_base = layout_.seg_base[step];
      P.final_size = (uint32_t)F;
      P.invalid = invalid_;
      P.is_last = step == n_steps - 1;
      P.seed = seed_;
      P.first_slot = (uint64_t)first_sample_ * transits_per_sample * m;  // outputs of the samples before ours
      P.first_sample = (uint32_t)first_sample_;
      P.n_pairs = n_pairs;
      P.live_pairs = nullptr;
      if (rows_direct_) {
        P.step_out = d_final_ + layout_.seg_base[step];
        P.out_pitch = (uint32_t)F;
      } else {
        P.step_out = d_step_out_ + (size_t)n_samples_ * layout_.seg_base[step];
        P.out_pitch = layout_.seg_len[step];
      }
      P.pair_cells = paired_results() ? d_step_out_ : nullptr;
      P.pair_cell_samples = (uint32_t)n_samples_;
      P.walk_cells = paired_results() ? d_walk_cells_ : nullptr;
      P.samples = d_samples_;
      P.explicit_out = explicit_map_ && step + 1 < n_steps ? d_explicit_ : nullptr;
      P.fill_levels = 0;
      if (kernels_fill) {
        uint32_t mult = 1;
        for (int later = step; later < n_steps; ++later) {
          if (later > step) mult *= (uint32_t)app.stepSize(later);
          P.fill_off[P.fill_levels] = layout_.seg_base[later] - layout_.seg_base[step];
          P.fill_mult[P.fill_levels] = mult;
          P.fill_levels++;
        }
      }
      P.paired_edges = dgraph_->paired;
      const bool emits = walk_mode_ && step + 1 < n_steps;
      P.state_travels = state_travels_;
      P.pair_state = nullptr;
      P.emit_keys = emits ? d_emit_keys_ : nullptr;
      P.emit_slots = emits ? d_emit_slots_ : nullptr;
      P.emit_state = emits && state_travels_ ? d_emit_state_ : nullptr;
      // small maps inverted at every step: the emitting kernels count the pairs per next transit
      const bool counted = small_map_ && sort_period == 1 && !sample_parallel;
      P.emit_counts = emits && counted ? d_small_ : nullptr;
      P.emit_ranks = emits && counted ? d_emit_ranks_ : nullptr;
      P.emit_counter_base = d_counter_base_;
      P.emit_place_start = nullptr;
      P.emit_spill = nullptr;
      P.emit_spill_first = 0;
      P.taken_keys = nullptr;
      P.taken_counts = nullptr;
      P.taken_n_counts = 0;
      if (placed && emits) {
        const int to = step & 1;  // step k writes set k % 2 and reads the other
        P.emit_keys = d_placed_keys_[to];
        P.emit_slots = d_placed_slots_[to];
        P.emit_state = state_travels_ ? d_placed_state_[to] : nullptr;
        P.emit_counts = d_placed_counts_[to];
        P.emit_ranks = nullptr;
        P.emit_place_start = d_place_start_;
        P.emit_spill = d_placed_counts_[to] + small_counters_;
        P.emit_spill_first = placed_spill_first_;
      }
      uint32_t* live_now = d_live_ + (sorts_done & 1);  // pairs the inversion of this step keeps
      // lanes of the flat kernel per pair: one when the pairs alone fill the machine, else
      // the power of two (at most the step size, rounded up) that brings the lanes to ~2^20
      // groups of four consecutive output slots a pair's outputs can touch: the pair's first
      // slot is a multiple of m, so its place in its group is one of (i * m) % 4
      P.groups_per_pair = 0;
      if (m > 1)
        for (uint32_t i = 0; i < 4; ++i) {
          const uint32_t groups = ((i * m) % 4 + m - 1) / 4 + 1;
          if (groups > P.groups_per_pair) P.groups_per_pair = groups;
        }
      P.lanes_shift = 0;
      const uint64_t lanes_wanted = step == 0 ? kFlatLanesWantedForRoots : kFlatLanesWanted;
      while ((1u << P.lanes_shift) < P.groups_per_pair && ((uint64_t)n_pairs << P.lanes_shift) < lanes_wanted)
        P.lanes_shift++;
      const uint64_t flat_lanes = (uint64_t)n_pairs << P.lanes_shift;

      if (step == 0) {
        // roots are used in sample order (the reference also feeds step 0 an unsorted map
        // when there is more than one step, nextdoor.cu:2400 and the FIXME at 2372)
        P.pair_keys = (const uint32_t*)transits;
        P.pair_slots = nullptr;
        if (launch_step(P, flat_lanes, false, nullptr) != 0) return -1;
      } else {
        // inversion: sort (transit, slot) by transit.  Walks sort the pairs the previous
        // step emitted (only those still alive); other apps sort the previous step's
        // output array, whose index is the slot.
        // Walks that invert only now and then gain nothing from the transit order (few of them
        // share a transit, and the order is stale one step later): they only drop the walks
        // that have ended, keeping slot order, in which the writes of a step's results coalesce.
        if (placed) {
          // small map, placed by the previous step's kernel: every place is a lane
          const int from = (step - 1) & 1;
          P.pair_keys = d_placed_keys_[from];
          P.pair_slots = d_placed_slots_[from];
          P.pair_state = state_travels_ ? d_placed_state_[from] : nullptr;
          P.n_pairs = (uint32_t)placed_places_;
          P.taken_keys = d_placed_keys_[from];
          P.taken_counts = d_placed_counts_[from];
          P.taken_n_counts = (uint32_t)small_counters_ + 1;
          const uint64_t lanes = placed_places_ > small_counters_ + 1 ? placed_places_ : small_counters_ + 1;
          if (launch_step(P, lanes, false, nullptr) != 0) return -1;
        } else if (counted) {
          // small map: the previous step's kernels have counted the pairs per transit
          const uint32_t n_keys = (uint32_t)small_counters_;
          const uint32_t n_chunks = (n_keys + kSmallMapChunk - 1) / kSmallMapChunk;
          uint32_t* counts = d_small_;
          uint32_t* local_start = counts + n_keys;
          uint32_t* chunk_total = local_start + n_keys;
          RunsMeta* meta = d_meta_ + (balanced_steps_ & 1);
          RunsMeta* meta_next = d_meta_ + ((balanced_steps_ + 1) & 1);
          if (balance) balanced_steps_++;
          tick();
          small_map_scan<<<dim3(n_chunks), dim3(256), 0, stream_>>>(counts, n_keys, local_start, chunk_total);
          small_map_place<<<dim3((n_pairs + 255) / 256), dim3(256), 0, stream_>>>(
              d_emit_keys_, d_emit_slots_, state_travels_ ? d_emit_state_ : nullptr, d_emit_ranks_, live_last, n_pairs,
              (uint32_t)invalid_, d_counter_base_, local_start, chunk_total, n_chunks, live_now,
              d_keys_a_, d_vals_a_,
              state_travels_ ? d_aux_a_ : nullptr, balance ? 1u : 0u, meta, meta_next, dgraph_->row_ptr(), m, d_chunks_,
              chunk_capacity_, d_taken_stamp_, counters_dev());
          tock(&times.inversion);
          times.sort_launches += 1;
          P.pair_keys = d_keys_a_;
          P.pair_slots = d_vals_a_;
          P.pair_state = state_travels_ ? d_aux_a_ : nullptr;
          P.live_pairs = live_now;
          live_last = live_now;
          sorts_done++;
          if (launch_step(P, flat_lanes, balance, meta) != 0) return -1;
        } else {
          const bool compact_only = sample_parallel || (walk_mode_ && sort_period > 1);
          const SortPlan plan = make_sort_plan(n_pairs, compact_only ? 0 : max_bits_);
          SortJob job;
          if (walk_mode_) {
            job.keys_in = d_emit_keys_;
            job.vals_in = d_emit_slots_;
            job.aux_in = state_travels_ ? d_emit_state_ : nullptr;
            job.n_in_dev = live_last;
          } else {
            job.keys_in = (const uint32_t*)transits;
            job.keys_in_layout = transits_layout;
          }
          job.keys_a = d_keys_a_;
          job.vals_a = d_vals_a_;
          job.aux_a = d_aux_a_;
          job.keys_b = d_keys_b_;
          job.vals_b = d_vals_b_;
          job.aux_b = d_aux_b_;
          job.hist = d_hist_;
          job.scratch = d_scratch_;
          job.drop_key = (uint32_t)invalid_;
          job.kept_dev = live_now;
          tick();
          ND_HIP_TRY(radix_sort(plan, job, stream_));
          tock(&times.inversion);
          times.sort_launches += plan.passes;
          uint32_t* sorted_keys = job.keys_sorted;
          P.pair_keys = sorted_keys;
          P.pair_slots = job.vals_sorted;
          P.pair_state = state_travels_ ? job.aux_sorted : nullptr;
          P.live_pairs = live_now;
          live_last = live_now;
          sorts_done++;
          if (compact_only && walk_mode_) {
            // the walks keep their lanes until the next compaction
            const int stretch = n_steps - step < sort_period ? n_steps - step : sort_period;
            P.emit_keys = d_emit_keys_;
            P.emit_slots = d_emit_slots_;
            P.emit_state = state_travels_ ? d_emit_state_ : nullptr;
            tick();
            walk_stretch_kernel<SampleType, App><<<dim3((n_pairs + kFlatThreads - 1) / kFlatThreads), dim3(kFlatThreads), 0,
                                                   stream_>>>(P, stretch, n_steps - 1, (size_t)n_samples_);
            tock(&times.flat_kernel);
            times.flat_launches++;
            step += stretch - 1;
          } else if (!balance || compact_only) {
            if (launch_step(P, flat_lanes, false, nullptr) != 0) return -1;
          } else {
            tick();
            const unsigned pair_blocks = (n_pairs + 255) / 256;
            RunsMeta* meta = d_meta_ + (balanced_steps_ & 1);
            RunsMeta* meta_next = d_meta_ + ((balanced_steps_ + 1) & 1);
            balanced_steps_++;
            if (n_pairs >= kClassifyLargeFrom) {
              const unsigned per_block = kClassifyThreadsLarge * kClassifyItemsLarge;
              const unsigned tail_blocks = (n_pairs + per_block - 1) / per_block;
              classify_run_tails<kClassifyItemsLarge, kClassifyThreadsLarge>
                  <<<dim3(tail_blocks), dim3(kClassifyThreadsLarge), 0, stream_>>>(
                  sorted_keys, live_now, meta, meta_next, dgraph_->row_ptr(), m, d_chunks_, chunk_capacity_,
                  d_taken_stamp_, counters_dev(), d_balance_, (uint32_t)step);
            } else {
              classify_run_tails<1><<<dim3(pair_blocks), dim3(256), 0, stream_>>>(
                  sorted_keys, live_now, meta, meta_next, dgraph_->row_ptr(), m, d_chunks_, chunk_capacity_,
                  d_taken_stamp_, counters_dev(), d_balance_, (uint32_t)step);
            }
            tock(&times.load_balancing);
            if (launch_step(P, flat_lanes, true, meta) != 0) return -1;
          }
        }
      }
      ND_HIP_TRY(hipGetLastError());
      transits = P.step_out;
      if (explicit_map_) {
        transits = d_explicit_;  // one entry per output slot, no rows
      } else if (rows_direct_) {
        // (A second, contiguous copy of the first step's outputs for this inversion to read its
        // keys from, written by the step-0 kernel in whole lines: inversion 0.89 -> 0.79 ms on the
        // k-hop pass, the step-0 launch 0.16 ms longer - it is bound by its write requests.  The
        // contiguous array alone, copied into the rows by the inversion's first pass: step-0 launch
        // 0.045 ms shorter, inversion 0.04 ms longer - the pieces of rows cost the same whoever
        // writes them.)
        transits_layout.rows(layout_.seg_len[step], (uint32_t)F);
      }
      transits_per_sample *= m;
    }

    // regroup the per-step arrays into one row per sample
    tick();
    if (rows_direct_) {
      // the step kernels wrote the rows themselves
    } else if (walk_mode_ && rows_per_block_ > 0) {
      const unsigned blocks = (unsigned)((n_samples_ + rows_per_block_ - 1) / rows_per_block_);
      const size_t lds = (size_t)rows_per_block_ * row_pitch_ * sizeof(int32_t);
      assemble_walk_rows<<<dim3(blocks), dim3(256), lds, stream_>>>(d_step_out_, d_final_, (uint32_t)n_samples_,
                                                                    (uint32_t)n_steps, row_pitch_, rows_per_block_,
                                                                    paired_results() ? 1u : 0u,
                                                                    paired_results() ? d_walk_cells_ : nullptr, invalid_);
    } else if (rows_per_block_ > 0) {
      const unsigned blocks = (unsigned)((n_samples_ + rows_per_block_ - 1) / rows_per_block_);
      const size_t lds = (size_t)rows_per_block_ * row_pitch_ * sizeof(int32_t);
      assemble_final_rows<<<dim3(blocks), dim3(256), lds, stream_>>>(d_step_out_, d_final_, (uint32_t)n_samples_,
                                                                     (uint32_t)F, row_pitch_, rows_per_block_, layout_);
    } else {
      for (int k = 0; k < n_steps; ++k) {
        const size_t n = (size_t)n_samples_ * layout_.seg_len[k];
        assemble_final_step<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream_>>>(
            d_step_out_ + (size_t)n_samples_ * layout_.seg_base[k], d_final_, n, layout_.seg_len[k], (uint32_t)F,
            layout_.seg_base[k]);
      }
    }
    tock(&times.assemble);
    ND_HIP_TRY(hipGetLastError());
    if (placed) placed_dirty_ = false;  // the last step has taken every pair and cleared the counters behind it
    return 0;
  }

  // A pass can be recorded once as a HIP graph and replayed: nothing in it depends on the host
  // (sizes that change from step to step live in device memory), so the graph of one pass is
  // the graph of every pass with the same mode, inversion period and load-balancing parity.
  // No memset nodes: buffers are cleared by fill kernels.  Off by default: on the pass it was
  // meant for (56,944 walks, ~1300 launches of 3-9 us each) the replay takes 4.72 ms against
  // 4.8 ms enqueued one by one - the kernels' own durations add up to the pass, not the gaps.
  bool wants_launch_graph() const { return launch_graph == 1 && !profiling; }

  int replay_pass(int mode) {
    const int parity = balanced_steps_ & 1;
    RecordedPass* pass = nullptr;
    for (RecordedPass& r : recorded_)
      if (r.mode == mode && r.inversion_period == inversion_period && r.parity == parity && r.items_seen == items_seen_)
        pass = &r;
    if (!pass) {
      RecordedPass r;
      r.mode = mode;
      r.inversion_period = inversion_period;
      r.parity = parity;
      r.items_seen = items_seen_;  // decides how the two classes of a step are launched
      const uint64_t before = balanced_steps_;
      const ScheduleCounts counts_before = schedule_counts_;
      ND_HIP_TRY(hipStreamBeginCapture(stream_, hipStreamCaptureModeThreadLocal));
      const int rc = enqueue_pass(mode);
      hipGraph_t graph = nullptr;
      const hipError_t ended = hipStreamEndCapture(stream_, &graph);
      r.balanced_steps = balanced_steps_ - before;
      r.balanced = balanced_this_pass_;
      r.merged_steps = schedule_counts_.merged_steps - counts_before.merged_steps;
      r.forked_steps = schedule_counts_.forked_steps - counts_before.forked_steps;
      r.serial_steps = schedule_counts_.serial_steps - counts_before.serial_steps;
      balanced_steps_ = before;  // advanced below, as for every replay
      schedule_counts_ = counts_before;
      if (rc != 0 || ended != hipSuccess) {
        if (graph) (void)hipGraphDestroy(graph);
        if (rc == 0) last_error = std::string("hipStreamEndCapture: ") + hipGetErrorString(ended);
        return rc != 0 ? rc : -1;
      }
      const hipError_t made = hipGraphInstantiate(&r.exec, graph, nullptr, nullptr, 0);
      (void)hipGraphDestroy(graph);
      if (made != hipSuccess) {
        last_error = std::string("hipGraphInstantiate: ") + hipGetErrorString(made);
        return -1;
      }
      r.counts = times;
      recorded_.push_back(r);
      pass = &recorded_.back();
    }
    times = pass->counts;  // launch counts of the recorded pass; durations stay zero
    balanced_steps_ += pass->balanced_steps;
    balanced_this_pass_ = pass->balanced;  // the replayed pass's, not the last recorded one's
    schedule_counts_.merged_steps += pass->merged_steps;
    schedule_counts_.forked_steps += pass->forked_steps;
    schedule_counts_.serial_steps += pass->serial_steps;
    ND_HIP_TRY(hipGraphLaunch(pass->exec, stream_));
    return 0;
  }

  void drop_recorded_passes() {
    for (RecordedPass& r : recorded_)
      if (r.exec) (void)hipGraphExecDestroy(r.exec);
    recorded_.clear();
  }

  // getFinalSamples: device -> hFinalSamples
  int fetch_final_samples() override { return fetch_final_samples_into(hFinalSamples.data()); }

  int fetch_final_samples_into(VertexID_t* dst) {
    if (!allocated_) { last_error = "no device data"; return -1; }
    ND_HIP_TRY(hipMemcpy(dst, d_final_, sizeof(VertexID_t) * (size_t)n_samples_ * (size_t)final_sample_size(),
                         hipMemcpyDeviceToHost));
    return 0;
  }

  bool is_walk() const { return walk_mode_; }

  int fetch_sample_states(void* dst, size_t bytes) override {
    if (!allocated_ || std::is_empty<SampleType>::value) { last_error = "no sample state"; return -1; }
    if (bytes != sample_state_bytes()) { last_error = "sample state size mismatch"; return -1; }
    ND_HIP_TRY(hipMemcpy(dst, d_samples_, bytes, hipMemcpyDeviceToHost));
    return 0;
  }

  // Distinct post-pass over the device-resident result rows (see nd_distinct.hpp): every
  // hop segment of every sample becomes its ascending unique valid ids, INVALID-padded.
  int distinct() override {
    if (!allocated_) { last_error = "distinct before alloc"; return -1; }
    App app;
    if (app.outputFormat() != SampledVertices) { last_error = "distinct needs SampledVertices output"; return -2; }
    const int n_steps = app.steps();
    if (!d_distinct_counts_) {
      ND_HIP_TRY(hipMalloc(&d_distinct_counts_, sizeof(int32_t) * (size_t)n_samples_ * n_steps));
    }
    times.distinct = 0;
    ND_HIP_TRY(hipEventRecord(ev_begin_, stream_));
    const bool rows_at_once = launch_distinct_rows(d_final_, d_distinct_counts_, (uint32_t)n_samples_,
                                                   (uint32_t)final_sample_size(), layout_.seg_base, layout_.seg_len,
                                                   (uint32_t)n_steps, invalid_, !app.hasExplicitTransits(), stream_);
    for (int k = 0; k < n_steps && !rows_at_once; ++k) {
      if (!launch_distinct_segment(d_final_, d_distinct_counts_, (uint32_t)n_samples_, (uint32_t)final_sample_size(),
                                   layout_.seg_base[k], layout_.seg_len[k], invalid_, (uint32_t)n_steps, (uint32_t)k,
                                   stream_)) {
        last_error = "a hop segment is longer than 4096 ids";
        return -2;
      }
    }
    ND_HIP_TRY(hipGetLastError());
    ND_HIP_TRY(hipEventRecord(ev_end_, stream_));
    ND_HIP_TRY(hipStreamSynchronize(stream_));
    ND_HIP_TRY(hipEventElapsedTime(&times.distinct, ev_begin_, ev_end_));
    hDistinctCounts.resize((size_t)n_samples_ * n_steps);
    ND_HIP_TRY(hipMemcpy(hDistinctCounts.data(), d_distinct_counts_, sizeof(int32_t) * hDistinctCounts.size(),
                         hipMemcpyDeviceToHost));
    return 0;
  }

  void free_device() override {
    free_run_buffers();
    free_graph();
  }

 private:
  // d_balance_: found_by_step[kMaxSteps + 1], then the ClassCounters (8-byte aligned)
  static constexpr int kBalanceWords =
      kMaxSteps + 2 + (int)(kCounterCopies * sizeof(ClassCounters) / sizeof(uint32_t));
  static constexpr int kIdleLookEvery = 8;
  ClassCounters* counters_dev() const { return (ClassCounters*)(d_balance_ + kMaxSteps + 2); }
  // Walks write their results in cells of two steps (StepParams::pair_cells) where a step's
  // transit is the previous step's result and the rows are regrouped by assemble_walk_rows.
  bool paired_results() const { return paired_results_; }

  void launch_workgroup(const StepParams& P, unsigned grid, const RunsMeta* meta) {
    if (P.step_size == 1)
      step_workgroup_kernel<SampleType, App, true><<<dim3(grid), dim3(kStepThreads), 0, stream_>>>(P, d_chunks_, meta,
                                                                                                   chunk_capacity_);
    else
      step_workgroup_kernel<SampleType, App, false><<<dim3(grid), dim3(kStepThreads), 0, stream_>>>(P, d_chunks_, meta,
                                                                                                    chunk_capacity_);
  }

  void launch_flat(const StepParams& P, uint64_t lanes, const uint32_t* taken_stamp, const RunsMeta* meta) {
    const unsigned grid = flat_grid_for(lanes);
    if (P.emit_place_start || P.taken_keys)
      step_flat_kernel<SampleType, App, true, true><<<dim3(grid), dim3(kFlatThreads), 0, stream_>>>(P, taken_stamp, meta);
    else if (P.step_size == 1)
      step_flat_kernel<SampleType, App, true><<<dim3(grid), dim3(kFlatThreads), 0, stream_>>>(P, taken_stamp, meta);
    else
      step_flat_kernel<SampleType, App, false><<<dim3(grid), dim3(kFlatThreads), 0, stream_>>>(P, taken_stamp, meta);
  }

  // How the two classes of a load-balanced step are launched.
  //   serial  flat kernel, then workgroup kernel, on the one stream
  //   merged  one launch (step_balanced_kernel): for maps so small that a launch costs more
  //           than what it computes
  //   forked  the workgroup kernel on a second stream beside the flat kernel: for large maps,
  //           where each keeps the occupancy of its own launch
  // Auto: serial until a classified pass has found work items at all (a pass over a map where
  // no transit gathers enough pairs should not pay for the second class), then by the size of
  // the step.  ND_STEP_SCHEDULE=serial|merged|forked forces one (read when the buffers are
  // allocated).  Results do not depend on it.
  enum { kScheduleAuto = -1, kScheduleSerial = 0, kScheduleMerged = 1, kScheduleForked = 2 };
  static constexpr uint64_t kMergedLanesAtMost = 1ull << 19;
  static constexpr uint32_t kMergedWorkgroupBlocks = 16384;

  int schedule_for(uint64_t lanes) const {
    if (forced_schedule_ != kScheduleAuto) return forced_schedule_;
    if (!items_seen_) return kScheduleSerial;
    return lanes <= kMergedLanesAtMost ? kScheduleMerged : kScheduleForked;
  }

  // The kernels of one step over the pairs P describes.  balance: the step was classified
  // (meta: its bookkeeping), and the transits its work items cover carry its stamp.
  int launch_step(const StepParams& P, uint64_t lanes, bool balance, const RunsMeta* meta) {
    if (P.explicit_out) {
      // the outputs of the pairs that never reach a kernel (no transit) lead nowhere
      const size_t n = (size_t)P.n_pairs * P.step_size;
      fill_i32<<<dim3((unsigned)((n + 1023) / 1024)), dim3(1024), 0, stream_>>>(P.explicit_out, n, P.invalid);
    }
    if (!balance) {
      tick();
      launch_flat(P, lanes, nullptr, nullptr);
      tock(&times.flat_kernel);
      times.flat_launches++;
      return 0;
    }
    // The workgroups of the work-item kernel take the items in turn.  Many more workgroups than
    // the device holds at once: the ones that end early make room for others, which evens out the
    // items' sizes (k-hop launch with 1280 workgroups - what fits - 1.35 ms; 4096: 1.10; 16384: 1.07;
    // 65536: 1.07).
    const unsigned wg_grid = chunk_capacity_ < 16384u ? chunk_capacity_ : 16384u;
    const int schedule = schedule_for(lanes);
    if (schedule == kScheduleMerged) {
      const uint64_t flat_blocks = (lanes + kStepThreads - 1) / kStepThreads;
      uint64_t groups = (flat_blocks + kBalancedFlatBlocks - 1) / kBalancedFlatBlocks;
      if (groups == 0) groups = 1;
      const uint64_t wanted = chunk_capacity_ < kMergedWorkgroupBlocks ? chunk_capacity_ : kMergedWorkgroupBlocks;
      uint32_t wg_per_group = (uint32_t)(((wanted + groups - 1) / groups + kXcds - 1) / kXcds * kXcds);
      if (wg_per_group < kXcds) wg_per_group = kXcds;
      const unsigned grid = (unsigned)(groups * (kBalancedFlatBlocks + wg_per_group));
      tick();
      if (P.step_size == 1)
        step_balanced_kernel<SampleType, App, true><<<dim3(grid), dim3(kStepThreads), 0, stream_>>>(
            P, d_taken_stamp_, meta, d_chunks_, chunk_capacity_, wg_per_group);
      else
        step_balanced_kernel<SampleType, App, false><<<dim3(grid), dim3(kStepThreads), 0, stream_>>>(
            P, d_taken_stamp_, meta, d_chunks_, chunk_capacity_, wg_per_group);
      tock(&times.flat_kernel);
      times.flat_launches++;
      schedule_counts_.merged_steps++;
    } else if (schedule == kScheduleForked && !profiling) {
      // (with per-phase events the two run one after the other, each timed undisturbed)
      // The work items start at once on the main stream; the flat kernel, whose single-wave
      // workgroups would fill every free slot of the machine, follows on the side stream and
      // takes what the work items leave.
      ND_HIP_TRY(hipEventRecord(ev_fork_, stream_));
      ND_HIP_TRY(hipStreamWaitEvent(side_stream_, ev_fork_, 0));
      launch_workgroup(P, wg_grid, meta);
      {
        const unsigned grid = flat_grid_for(lanes);
        if (P.step_size == 1)
          step_flat_kernel<SampleType, App, true><<<dim3(grid), dim3(kFlatThreads), 0, side_stream_>>>(P, d_taken_stamp_, meta);
        else
          step_flat_kernel<SampleType, App, false><<<dim3(grid), dim3(kFlatThreads), 0, side_stream_>>>(P, d_taken_stamp_, meta);
      }
      ND_HIP_TRY(hipEventRecord(ev_join_, side_stream_));
      ND_HIP_TRY(hipStreamWaitEvent(stream_, ev_join_, 0));
      times.flat_launches++;
      times.workgroup_launches++;
      schedule_counts_.forked_steps++;
    } else {
      tick();
      launch_flat(P, lanes, d_taken_stamp_, meta);
      tock(&times.flat_kernel);
      times.flat_launches++;
      tick();
      launch_workgroup(P, wg_grid, meta);
      tock(&times.workgroup_kernel);
      times.workgroup_launches++;
      if (schedule == kScheduleForked) schedule_counts_.forked_steps++; else schedule_counts_.serial_steps++;
    }
    return 0;
  }

  // workgroups of the flat kernel for this many outputs: whole groups of kXcds * kXcdRun, so
  // that flat_block_index is a bijection
  static unsigned flat_grid_for(uint64_t outputs) {
    const uint64_t blocks = (outputs + kFlatThreads - 1) / kFlatThreads;
    return (unsigned)((blocks + kXcds * kXcdRun - 1) / (kXcds * kXcdRun) * (kXcds * kXcdRun));
  }

  void tick() {
    if (profiling) (void)hipEventRecord(ev_a_, stream_);
  }
  void tock(float* acc) {
    if (!profiling) return;
    (void)hipEventRecord(ev_b_, stream_);
    (void)hipEventSynchronize(ev_b_);
    float ms = 0;
    (void)hipEventElapsedTime(&ms, ev_a_, ev_b_);
    *acc += ms;
  }

  template <class T>
  static void release(T*& p) {
    if (p) (void)hipFree(p);
    p = nullptr;
  }

  void free_graph() {
    dgraph_.reset();
    graph_ = nullptr;
  }

  void free_run_buffers() {
    drop_recorded_passes();
    release(d_initial_);
    release(d_samples_);
    release(d_samples_init_);
    release(d_final_);
    release(d_step_out_);
    release(d_walk_cells_);
    release(d_keys_a_);
    release(d_vals_a_);
    release(d_keys_b_);
    release(d_vals_b_);
    release(d_hist_);
    release(d_scratch_);
    release(d_live_);
    release(d_emit_keys_);
    release(d_emit_slots_);
    release(d_emit_ranks_);
    release(d_place_start_);
    for (int b = 0; b < 2; ++b) {
      release(d_placed_keys_[b]);
      release(d_placed_slots_[b]);
      release(d_placed_state_[b]);
      release(d_placed_counts_[b]);
    }
    small_placed_ = false;
    release(d_small_);
    release(d_counter_base_);
    release(d_emit_state_);
    release(d_aux_a_);
    release(d_aux_b_);
    release(d_meta_);
    release(d_balance_);
    release(d_chunks_);
    release(d_taken_stamp_);
    release(d_explicit_);
    release(d_distinct_counts_);
    // whatever exists, also after an alloc that failed half way
    for (hipEvent_t* ev : {&ev_a_, &ev_b_, &ev_begin_, &ev_end_, &ev_fork_, &ev_join_}) {
      if (*ev) (void)hipEventDestroy(*ev);
      *ev = nullptr;
    }
    if (side_stream_) (void)hipStreamDestroy(side_stream_);
    side_stream_ = nullptr;
    if (stream_) (void)hipStreamDestroy(stream_);
    stream_ = nullptr;
    allocated_ = false;
  }

  const char* name_;
  const CSR* graph_ = nullptr;
  CSRPartition view_{};
  std::shared_ptr<DeviceGraph> dgraph_;
  int64_t first_sample_ = 0;  // index of our first sample among the app's samples

  std::vector<SampleType> samples_;
  int64_t n_samples_ = 0;
  int init_size_ = 0;
  int32_t invalid_ = 0;
  int max_bits_ = 0;
  uint64_t seed_ = 0;
  size_t max_pairs_ = 0;
  uint32_t chunk_capacity_ = 0;
  uint32_t row_pitch_ = 0, rows_per_block_ = 0;
  bool paired_results_ = false;
  StepLayout layout_{};
  bool allocated_ = false;

  hipStream_t stream_ = nullptr;
  hipStream_t side_stream_ = nullptr;  // the workgroup kernel of a forked step
  hipEvent_t ev_a_ = nullptr, ev_b_ = nullptr, ev_begin_ = nullptr, ev_end_ = nullptr;
  hipEvent_t ev_fork_ = nullptr, ev_join_ = nullptr;
  VertexID_t* d_initial_ = nullptr;
  SampleType* d_samples_ = nullptr;
  SampleType* d_samples_init_ = nullptr;
  VertexID_t* d_final_ = nullptr;
  VertexID_t* d_step_out_ = nullptr;
  uint32_t* d_walk_cells_ = nullptr;  // cells of every walk that hold results (StepParams::walk_cells)
  uint32_t *d_keys_a_ = nullptr, *d_vals_a_ = nullptr, *d_keys_b_ = nullptr, *d_vals_b_ = nullptr;
  uint32_t* d_hist_ = nullptr;
  uint32_t* d_scratch_ = nullptr;
  uint32_t* d_live_ = nullptr;          // pairs the inversion kept (real transits); two words, alternating by step
  bool walk_mode_ = false, state_travels_ = false, rows_direct_ = false, mark_unwritten_ = false;
  bool explicit_map_ = false;           // App::stepTransits fills the next step's map (apps that are not walks)
  VertexID_t* d_explicit_ = nullptr;    // that map: the transit of every pair of the coming step
  uint32_t *d_emit_keys_ = nullptr, *d_emit_slots_ = nullptr, *d_emit_state_ = nullptr;  // next step's pairs
  // small maps: the inversion without a sort (small_map_scan, small_map_place)
  bool small_map_ = false;
  size_t small_counters_ = 0;
  uint32_t* d_counter_base_ = nullptr;  // first counter of every vertex
  uint32_t* d_emit_ranks_ = nullptr;
  uint32_t* d_small_ = nullptr;  // counters, their starts inside a chunk, chunk totals
  // small maps whose pairs are placed as they are emitted (StepParams::emit_place_start): two
  // sets of pair arrays with gaps and of counters, one written while the other is read
  bool small_placed_ = false, placed_dirty_ = false;
  uint32_t placed_spill_first_ = 0;
  size_t placed_places_ = 0;
  uint32_t* d_place_start_ = nullptr;
  uint32_t *d_placed_keys_[2] = {nullptr, nullptr}, *d_placed_slots_[2] = {nullptr, nullptr};
  uint32_t *d_placed_state_[2] = {nullptr, nullptr}, *d_placed_counts_[2] = {nullptr, nullptr};
  uint32_t *d_aux_a_ = nullptr, *d_aux_b_ = nullptr;  // ping-pong of the travelling state
  RunsMeta* d_meta_ = nullptr;          // two work-item counters, alternating between load-balanced steps
  uint32_t* d_balance_ = nullptr;       // which steps' classifications found a run; the pass's ClassCounters
  ClassCounters class_counters_{};      // of the last load-balanced pass
  int idle_passes_ = 0;                 // passes since one whose classifications found nothing (0: none)
  bool balanced_this_pass_ = false;
  struct RecordedPass {
    int mode = 0, inversion_period = 0, parity = 0;
    bool items_seen = false, balanced = false;
    uint64_t merged_steps = 0, forked_steps = 0, serial_steps = 0;
    uint64_t balanced_steps = 0;  // load-balanced steps of the pass
    PhaseTimes counts;            // its launch counts
    hipGraphExec_t exec = nullptr;
  };
  std::vector<RecordedPass> recorded_;
  uint64_t balanced_steps_ = 0;        // ... counted over the life of the buffers, so the parity never repeats
  WorkItem* d_chunks_ = nullptr;
  uint32_t* d_taken_stamp_ = nullptr;  // per vertex: the stamp of the last step whose work items covered it
  uint64_t markers_cleared_at_ = 0;    // balanced_steps_ when the markers were last wiped
  struct ScheduleCounts {
    uint64_t passes = 0, classified_passes = 0, merged_steps = 0, forked_steps = 0, serial_steps = 0;
  };
  ScheduleCounts schedule_counts_;
  bool items_seen_ = false;            // the last classified pass found work items
  int forced_schedule_ = kScheduleAuto;
  int32_t* d_distinct_counts_ = nullptr;
};

}  // namespace nd
