// Layer-wise (CollectiveNeighborhood) sampling engine for one MI355X (gfx950, wave64).
//
// Reference behaviour this covers (file:line in the reference tree):
//   collective branch of doTransitParallelSampling   src/nextdoor.cu:2402-2453, 2475-2496, 2900-2923
//   collectiveNeighbrsSize                           src/nextdoor.cu:1206-1246  -> collective_sizes
//   collectiveNeighborhood                           src/nextdoor.cu:1248-1283  -> collective_build
//   sampleParallelKernel, Collective branch          src/nextdoor.cu:1394-1446, 1485-1487 -> layer_execute_kernel
//
// Per layer k, for every sample s: its transits are the initial vertices (k = 0) or the
// layer k-1 segment of its result row; the collective neighbourhood is the concatenation
// of the transits' adjacencies; next() runs once per (sample, nbr < stepSize(k)) and its
// result goes to final[s * F + stepSizeAtStep(k-1) + nbr].
//
// Differences that are deliberate:
//  * The reference sizes the neighbourhood with a global atomic (offsets in arrival order),
//    cudaMallocs it inside the step loop and never hands it to next() (transitEdges is
//    nullptr, nextdoor.cu:1441-1446).  Here offsets are an exclusive scan over samples
//    (deterministic), the buffers are grown once and reused, and next() receives the
//    neighbourhood in the form the app declares (nd::apps::NeighborhoodForm).
//  * For kDistinctByDegreeSquared the concatenation is never stored, nor a list of its distinct
//    vertices: every entry marks its vertex in a per-sample bitmap, built stretch by stretch
//    in LDS; degree^2 of the marked vertices is summed over groups and parts of the bitmap,
//    and a draw searches those sums.
//  * For kRankedByLadiesImportance each entry also carries (weight * (1 / rowsum(transit)))^2;
//    the terms of a vertex are summed as 2^53 fixed-point integers (in LDS) into one sum per
//    (sample, vertex), its Efraimidis-Spirakis key is formed from the sum as it leaves LDS (the
//    only thing stored per sample and vertex), a radix select keeps
//    the few entries that can be among a sample's first picks, and stable sorts order those by
//    descending key.
//  * Samples are processed in chunks whose concatenated neighbourhoods fit a fixed budget
//    of entries, so a layer whose frontier sits on hubs cannot outgrow memory.
//  * Random numbers: Philox keyed by the output slot s * stepSize(k) + nbr and the layer.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <string>
#include <type_traits>
#include <vector>

#include "nd_apps_layer.hpp"
#include "nd_contract.hpp"
#include "nd_device_graph.hpp"
#include "nd_engine.hpp"
#include "nd_radix_sort.hpp"

namespace nd {

constexpr uint32_t kMaxLayerTransits = 1024;  // transits of one sample the build kernel stages in LDS

// transits of sample s: base[s * stride + i], i < count
struct TransitView {
  const int32_t* base;
  uint32_t stride;
  uint32_t count;
};

// One wave per sample: sum of the degrees of its valid transits.
__global__ __launch_bounds__(256) void collective_sizes(CSRPartition csr, TransitView tv, uint32_t n_samples,
                                                        int32_t invalid, uint32_t* __restrict__ sizes) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t s = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (s >= n_samples) return;
  const int32_t* transits = tv.base + (size_t)s * tv.stride;
  uint64_t sum = 0;
  for (uint32_t i = lane; i < tv.count; i += 64u) {
    const int32_t t = transits[i];
    if (t != invalid && t != -1) sum += (uint64_t)(csr.row_ptr[t + 1] - csr.row_ptr[t]);
  }
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) {
    const uint32_t lo = __shfl_down((uint32_t)sum, d, 64);
    const uint32_t hi = __shfl_down((uint32_t)(sum >> 32), d, 64);
    sum += ((uint64_t)hi << 32) | lo;
  }
  // sizes are 32-bit; a neighbourhood that does not fit saturates and the host refuses it
  if (lane == 0) sizes[s] = sum > 0xFFFFFFFFull ? 0xFFFFFFFFu : (uint32_t)sum;
}

// Entries of a sample's concatenation one workgroup of collective_build copies; samples
// with longer neighbourhoods are spread over several workgroups.
constexpr uint32_t kBuildItemEntries = 8192;

// Copies the adjacencies of every sample's transits, in transit order, to
// cols[offsets[s] ...] (and weights).
// Work items: item_start[s] = number of items of the samples before s (exclusive scan of
// ceil(size_s / kBuildItemEntries), with the total at [n_samples]); workgroup b serves the
// sample whose item range holds b and the b - item_start[s]-th stretch of its entries.
__global__ __launch_bounds__(256) void collective_build(CSRPartition csr, TransitView tv, int32_t invalid,
                                                        const uint32_t* __restrict__ offsets,
                                                        const uint32_t* __restrict__ item_start, uint32_t n_samples,
                                                        int32_t* __restrict__ cols, float* __restrict__ weights,
                                                        uint32_t* __restrict__ row_offsets) {
  __shared__ uint32_t s_start[kMaxLayerTransits + 1];  // start of transit i inside the sample's concatenation
  __shared__ uint32_t s_scan_tmp[4];
  // sample of this work item: last s with item_start[s] <= blockIdx.x
  uint32_t lo_s = 0, hi_s = n_samples;
  while (hi_s - lo_s > 1) {
    const uint32_t mid = lo_s + (hi_s - lo_s) / 2;
    if (item_start[mid] <= blockIdx.x) lo_s = mid; else hi_s = mid;
  }
  const uint32_t s = lo_s;
  const uint32_t item = blockIdx.x - item_start[s];
  const int32_t* transits = tv.base + (size_t)s * tv.stride;
  uint32_t carry = 0;
  for (uint32_t chunk = 0; chunk < tv.count; chunk += 256) {
    const uint32_t i = chunk + threadIdx.x;
    uint32_t deg = 0;
    if (i < tv.count) {
      const int32_t t = transits[i];
      if (t != invalid && t != -1) deg = (uint32_t)(csr.row_ptr[t + 1] - csr.row_ptr[t]);
    }
    uint32_t total;
    const uint32_t excl = block_exclusive_scan_256(deg, s_scan_tmp, &total);
    if (i < tv.count) s_start[i] = carry + excl;
    carry += total;
  }
  if (threadIdx.x == 0) s_start[tv.count] = carry;
  __syncthreads();
  const uint32_t base = offsets[s];
  const uint32_t size = s_start[tv.count];
  if (row_offsets && item == 0)
    for (uint32_t i = threadIdx.x; i < tv.count; i += 256) row_offsets[(size_t)s * tv.count + i] = s_start[i];
  const uint32_t first = item * kBuildItemEntries;
  const uint32_t last = first + kBuildItemEntries < size ? first + kBuildItemEntries : size;
  uint32_t cur = 0;  // transit of the previous entry this lane copied: the next one is usually the same
  for (uint32_t e = first + threadIdx.x; e < last; e += 256) {
    if (!(s_start[cur] <= e && e < s_start[cur + 1])) {
      // transit whose range holds e: last i with s_start[i] <= e
      uint32_t lo = 0, hi = tv.count;
      while (hi - lo > 1) {
        const uint32_t mid = lo + (hi - lo) / 2;
        if (s_start[mid] <= e) lo = mid; else hi = mid;
      }
      cur = lo;
    }
    const int32_t t = transits[cur];
    const EdgePos_t src = csr.row_ptr[t] + (EdgePos_t)(e - s_start[cur]);
    cols[base + e] = csr.edges[src];
    if (weights) weights[base + e] = csr.weights[src];
  }
}

// (weight * (1 / rowsum))^2 as a 2^53 fixed-point integer, truncated: sums of up to 1024 of
// them fit 64 bits and, unlike float sums, do not depend on the order of the additions.
// A float in (0, 1) is (2^23 + m) * 2^(e - 150) with exponent field e and mantissa m, so the
// product with 2^53 is the 24-bit mantissa shifted by e - 97; the same integer as
// (unsigned long long)(term * 2^53f), without a float -> 64-bit conversion.
__host__ __device__ __forceinline__ unsigned long long importance_term_fixed(float term) {
  uint32_t bits;
  __builtin_memcpy(&bits, &term, sizeof(bits));
  if ((int32_t)bits <= 0) return 0ull;  // zero or negative
  if (bits >= 0x3F800000u) return bits > 0x7F800000u ? 0ull : 1ull << 53;  // >= 1 (NaN: 0)
  const uint32_t e = bits >> 23;
  const uint32_t mantissa = (bits & 0x7FFFFFu) | (e ? 0x800000u : 0u);
  const int shift = (int)e - 97;
  if (shift >= 0) return (unsigned long long)mantissa << shift;
  return shift > -24 ? (unsigned long long)(mantissa >> -shift) : 0ull;
}

// ---- the distinct vertices of a collective neighbourhood, marked stretch by stretch ----
//
// collective_mark_binned walks the neighbourhood as collective_build does, but instead of
// copying an entry it marks the entry's vertex; nothing of the concatenation is stored.  A
// neighbourhood that sits on hubs repeats its vertices many times over (3.8e10 entries hold
// 2.0e9 distinct pairs at FastGCN's full size).  FastGCN form: the result is a bitmap per
// sample (words_per_sample 32-bit words, a multiple of the tile below).  LADIES form
// (kWithImportance): every entry also adds (weight * inverse_row_sum[transit])^2, as a 2^53
// fixed-point integer, to the 64-bit sum of (sample, vertex) in LDS; the result is the sampling
// key formed from that sum for every vertex of every sample, kAbsentKey where the sample's
// neighbourhood does not hold the vertex.
constexpr uint32_t kBitmapTileWords = 2048;  // bitmaps are padded to whole tiles of 65536 vertices (4 parts)

// log2 of a positive normal float from exponent extraction and an atanh series; every step
// is a single IEEE operation so that host and device agree bit for bit.
__host__ __device__ __forceinline__ float det_log2(float x) {
  uint32_t bits;
#if defined(__HIP_DEVICE_COMPILE__)
  bits = __float_as_uint(x);
#else
  memcpy(&bits, &x, sizeof(bits));
#endif
  int e = (int)(bits >> 23) - 127;
  const uint32_t mbits = (bits & 0x7FFFFFu) | 0x3F800000u;
  float m;
#if defined(__HIP_DEVICE_COMPILE__)
  m = __uint_as_float(mbits);
#else
  memcpy(&m, &mbits, sizeof(m));
#endif
  if (m > 1.41421354f) { m = m * 0.5f; e += 1; }
  const float z = (m - 1.0f) / (m + 1.0f);
  const float z2 = z * z;
  float poly = z2 * 0.142857149f;
  poly = poly + 0.2f;
  poly = poly * z2;
  poly = poly + 0.333333343f;
  poly = poly * z2;
  poly = poly + 1.0f;
  float ln_m = z * poly;
  ln_m = ln_m * 2.0f;
  return (float)e + ln_m * 1.44269502f;
}

// Efraimidis-Spirakis key of (sample, vertex): log2(u) / importance, importance the fixed-point
// sum of the vertex's terms (the common 2^53 scale does not change the order of the keys), u
// from Philox: the pair's index is P = sample * (|V| rounded up to a multiple of 4) + vertex,
// its uniform comes from word P & 3 of the block with counter P >> 2 - four consecutive
// vertices of a sample share a block, so a lane that handles four of them pays for one (the
// ten rounds of multiplications are what the key pass of a dense layer is bound by).  As
// sortable bits, inverted so that an ascending sort yields descending keys.  No key is
// 0xFFFFFFFF (it would be a negative NaN): kAbsentKey marks the vertices a sample's
// neighbourhood does not hold.
constexpr uint32_t kAbsentKey = 0xFFFFFFFFu;
// importance sums stay below 2^63 (at most 1024 transits, each adding at most 2^53)
constexpr unsigned long long kAbsentSum = ~0ull;
__host__ __device__ __forceinline__ uint64_t ladies_pair_index(uint64_t sample, uint32_t n_vertices, uint32_t v) {
  return sample * (uint64_t)((n_vertices + 3u) & ~3u) + v;
}
__device__ __forceinline__ PhiloxBlock ladies_block(uint64_t pair, uint32_t step, uint64_t seed) {
  const uint64_t block = pair >> 2;
  return philox4x32_10((uint32_t)block, (uint32_t)(block >> 32), step, 0, (uint32_t)seed, (uint32_t)(seed >> 32));
}
__device__ __forceinline__ uint32_t ladies_key_from_word(unsigned long long importance_fixed, uint32_t word) {
  const float importance = (float)importance_fixed;
  const float u = ((float)(word >> 8) + 0.5f) * 5.9604644775390625e-08f;
  float key = -__builtin_inff();
  if (importance > 0.0f) key = det_log2(u) / importance;
  uint32_t b = __float_as_uint(key);
  b = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
  return ~b;
}
// one pair on its own
__device__ __forceinline__ uint32_t ladies_key_bits(unsigned long long importance_fixed, uint64_t pair, uint32_t step,
                                                    uint64_t seed) {
  const PhiloxBlock blk = ladies_block(pair, step, seed);
  const uint32_t which = (uint32_t)pair & 3u;
  uint32_t word = blk.w[0];
  word = which == 1 ? blk.w[1] : word;
  word = which == 2 ? blk.w[2] : word;
  word = which == 3 ? blk.w[3] : word;
  return ladies_key_from_word(importance_fixed, word);
}

// ---- wave-wide data movement on the VALU (DPP), no LDS traffic ----
// The value of the lane `shift` below inside the lane's row of 16; lanes without one get `fill`.
template <int kShift>
__device__ __forceinline__ uint32_t row_shift_up(uint32_t fill, uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)fill, (int)x, 0x110 | kShift, 0xF, 0xF, false);
}
// The value of lane - 1 / lane + 1 across the whole wavefront; the end lanes get `fill`.
__device__ __forceinline__ uint32_t wave_from_below(uint32_t fill, uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)fill, (int)x, 0x138, 0xF, 0xF, false);  // wave_shr:1
}
__device__ __forceinline__ uint32_t wave_from_above(uint32_t fill, uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)fill, (int)x, 0x130, 0xF, 0xF, false);  // wave_shl:1
}

// One step of a segmented inclusive sum along a row of 16 lanes: (closed, term) of this lane
// takes in (up_closed, up_term) of a lane further down.  A lane is closed once its sum has
// reached the start of its segment.
__device__ __forceinline__ void take_in(uint32_t up_closed, uint32_t up_lo, uint32_t up_hi, uint32_t& closed,
                                        unsigned long long& term) {
  if (!closed) term += ((unsigned long long)up_hi << 32) | up_lo;
  closed |= up_closed;
}

template <int kShift>
__device__ __forceinline__ void segmented_row_step(uint32_t& closed, unsigned long long& term) {
  // lanes without a source take in the neutral element (open, 0)
  const uint32_t c = row_shift_up<kShift>(0u, closed);
  const uint32_t lo = row_shift_up<kShift>(0u, (uint32_t)term);
  const uint32_t hi = row_shift_up<kShift>(0u, (uint32_t)(term >> 32));
  take_in(c, lo, hi, closed, term);
}

// The same marking with the presence map (and the importance sums) of one stretch of the vertex
// range held in LDS: one workgroup per (sample, stretch).  Adjacencies are sorted by
// destination, so the part of a transit's adjacency that falls into the stretch is one
// sub-range, found by two binary searches; the workgroup streams the sub-ranges of all the
// sample's transits, marks and adds in LDS, and writes the stretch out once - plain stores
// that cover the whole map, so nothing is cleared beforehand and no atomic reaches memory
// (global atomics stop at ~24 G/s on this part; the LADIES form needs 4.2e9 of them).
// The LDS pipeline is what this kernel runs out of (counters: a wavefront waits for LDS a
// third of its time), so it is kept for the map itself: every wavefront walks a contiguous
// part of the stretch's entries, which lets a lane step from one sub-range to the next instead
// of searching the table for every entry, and the sums along the wavefront move through DPP.
constexpr uint32_t kBinThreads = 1024;
constexpr uint32_t kBinWaves = kBinThreads / 64;
constexpr uint32_t kBinAhead = 4;             // entries a lane fetches before it works on the first
constexpr EdgePos_t kShortRest = 16;          // edges left of an adjacency that are stepped through one by one
// consecutive stretches of a sample one workgroup takes (FastGCN form: few, large stretches per
// sample, and the low ones hold most entries; LADIES form: hundreds of small ones)
constexpr uint32_t kBinsPerGroupBits = 8;
constexpr uint32_t kBinsPerGroupSums = 16;
constexpr uint32_t kBinWordsBits = 2048;      // FastGCN form: 65,536 vertices, one byte each in LDS (64 KB)
constexpr uint32_t kBinVerticesSums = 7168;   // LADIES form: 56 KB of 64-bit sums + 896 B of bits

// Dense pieces.  What a hub contributes to a stretch can be thousands of entries (a layer
// drawn by degree^2 sits on the hubs: 144 K entries per transit at FastGCN's full size), and
// it is the same for every sample that holds the hub.  Where a vertex has kDensePieceEntries
// (LADIES form: kDensePieceEntriesSums) or more edges into one stretch, the stretch's piece of
// that vertex is built once per graph - FastGCN form: its bitmap (2048 words); LADIES form:
// the importance sum of every vertex of the stretch (7168 64-bit integers, kAbsentSum where
// there is no edge; the sums are integers, so adding a piece gives the bits that adding its
// edges one by one gives) - and a sample ORs / adds the piece on the stretch's way out of LDS
// instead of going through the entries.  hub_row[v] = row of v in piece_of or -1;
// piece_of[row * stretches + stretch] = piece index or kNoPiece.
constexpr uint32_t kDensePieceEntries = 1024;
constexpr uint32_t kDensePieceEntriesSums = 2048;  // LADIES form: a piece is 7168 64-bit sums
constexpr size_t kDensePieceBudgetBytes = (size_t)2 << 30;
constexpr uint32_t kNoPiece = 0xFFFFFFFFu;
struct DensePieces {
  const int32_t* hub_row = nullptr;  // nullptr: the graph has none
  const uint32_t* piece_of = nullptr;
  const uint32_t* words = nullptr;            // FastGCN form: 2048 words of bits per piece
  const unsigned long long* sums = nullptr;  // LADIES form: 7168 importance sums per piece (kAbsentSum: no edge)
};

// LADIES form: the marking kernel turns the importance sums into sampling keys itself where a
// stretch leaves LDS (a lane takes four consecutive vertices and pays for one Philox block) and
// writes those, 4 bytes per vertex and sample.  Writing the sums instead and forming the keys in
// the selection's pass cost 8 + 8 + 4 bytes per vertex and sample of traffic, and 3.4 ms more
// per pass at full size.
struct KeysOnTheWayOut {
  uint32_t* keys = nullptr;
  uint64_t seed = 0;
  uint64_t first_sample = 0;
  uint32_t step = 0;
  uint32_t n_vertices = 0;
};

// 32-bit words of one sample's presence map: a bit per vertex, padded to whole tiles.
inline uint32_t bitmap_words_for(uint32_t n_vertices) {
  return ((n_vertices + 31u) / 32u + kBitmapTileWords - 1) / kBitmapTileWords * kBitmapTileWords;
}

// First edge of the sorted adjacency [from, end) whose destination is >= v_hi, given that the
// destination of `from` is below it; *next = that edge's destination (0xFFFFFFFF: none left).
// A workgroup waits for the slowest of these searches and each probe is a trip to the caches:
// a short rest is stepped through edge by edge, a long one galloped and bisected.
__device__ __forceinline__ EdgePos_t first_edge_at_or_above(const VertexID* __restrict__ edges, EdgePos_t from,
                                                            EdgePos_t end, uint32_t v_hi, uint32_t* next) {
  EdgePos_t lo = from;
  if (end - from <= kShortRest) {
    uint32_t dst;
    do {
      ++lo;
      dst = lo < end ? (uint32_t)edges[lo] : 0xFFFFFFFFu;
    } while (dst < v_hi);
    *next = dst;
    return lo;
  }
  EdgePos_t width = 64;
  while (lo < end) {
    const EdgePos_t probe = lo + width < end ? lo + width : end;
    if ((uint32_t)edges[probe - 1] >= v_hi) break;
    lo = probe;
    width <<= 1;
  }
  EdgePos_t hi = lo + width < end ? lo + width : end;
  while (lo < hi) {
    const EdgePos_t mid = lo + (hi - lo) / 2;
    if ((uint32_t)edges[mid] < v_hi) lo = mid + 1; else hi = mid;
  }
  *next = lo < end ? (uint32_t)edges[lo] : 0xFFFFFFFFu;
  return lo;
}

// One wavefront: drops the empty sub-ranges of the per-transit tables (length, first edge,
// row sum) and turns lengths into starts: starts[k] = first entry of kept sub-range k,
// starts[kept] = all entries; *ranges = kept.  A length with kPieceFlag set stands for a
// transit whose entries reach the stretch as a ready-made piece: no sub-range, and the piece
// index joins the list that takes the place of the lengths, *pieces = how many.  The tables
// are rewritten in place: an entry moves down or stays, and a round only writes below what it
// has read.
constexpr uint32_t kPieceFlag = 0x80000000u;
template <bool kWithImportance>
__device__ __forceinline__ void keep_filled_subranges(uint32_t n_transits, uint32_t lane, uint32_t* lengths,
                                                      EdgePos_t* edge, float* row_sum, uint32_t* starts,
                                                      uint32_t* ranges, uint32_t* pieces) {
  uint32_t kept = 0, entries = 0, listed = 0;
  for (uint32_t c = 0; c < n_transits; c += 64) {
    const uint32_t i = c + lane;
    const uint32_t raw = i < n_transits ? lengths[i] : 0u;
    const bool is_piece = (raw & kPieceFlag) != 0;
    const uint32_t len = is_piece ? 0u : raw;
    const EdgePos_t first = i < n_transits ? edge[i] : 0;
    const float sum = kWithImportance && i < n_transits ? row_sum[i] : 1.0f;
    const uint64_t holds = __ballot(len != 0), ready = __ballot(is_piece);
    const uint64_t below = (1ull << lane) - 1ull;
    const uint32_t through = wave_inclusive_scan(len);
    if (len != 0) {
      const uint32_t k = kept + (uint32_t)__popcll(holds & below);
      starts[k] = entries + through - len;
      edge[k] = first;
      if (kWithImportance) row_sum[k] = sum;
    }
    if (is_piece) lengths[listed + (uint32_t)__popcll(ready & below)] = raw & ~kPieceFlag;
    kept += (uint32_t)__popcll(holds);
    listed += (uint32_t)__popcll(ready);
    entries += __shfl(through, 63, kWave);
  }
  if (lane == 0) {
    starts[kept] = entries;
    *ranges = kept;
    *pieces = listed;
  }
}

// A sample without hubs among its transits and with at most this many entries in a
// workgroup's stretches (a layer whose transits are drawn uniformly) marks them all at once.
constexpr uint32_t kSparseGroupEntries = 32768;
constexpr uint32_t kSparseGroupEntriesSums = 2048;  // LADIES form: sums in an LDS table of twice as many slots

// Two workgroups of 16 wavefronts share a compute unit only at 8 wavefronts per SIMD, which the
// kernel's attributes ask the compiler for.  Measured without them: 63 (LADIES form) and 66
// registers per lane, 7 wavefronts per SIMD, one workgroup resident, and the LADIES form takes
// 1.6 times as long; the LDS size (tried: 62 to 70 KB) makes no difference.
template <bool kWithImportance>
__global__ __launch_bounds__(kBinThreads, 8) __attribute__((amdgpu_num_vgpr(56))) void collective_mark_binned(
    CSRPartition csr, TransitView tv, int32_t invalid, uint32_t n_samples, uint32_t bins_per_sample,
    uint32_t* __restrict__ bitmap,
    uint32_t words_per_sample, const float* __restrict__ inverse_row_sums,
    uint32_t keys_per_sample, DensePieces dense, KeysOnTheWayOut keys_out) {
  constexpr uint32_t kBinWords = kWithImportance ? kBinVerticesSums / 32u : kBinWordsBits;
  constexpr uint32_t kBinVertices = kBinWords * 32u;
  // FastGCN form: a byte per vertex, set with plain LDS stores (every writer stores 1) and
  // packed into bits on the way out; LADIES form: bits and 64-bit sums, LDS atomics
  __shared__ __align__(16) uint32_t s_bits[kWithImportance ? kBinWords : kBinVertices / 4u];
  __shared__ __align__(16) unsigned long long s_acc[kWithImportance ? kBinVerticesSums : 1];
  uint8_t* s_bytes = (uint8_t*)s_bits;
  // the sub-ranges that hold entries, in transit order
  __shared__ uint32_t s_start[kMaxLayerTransits + 1];  // first entry of sub-range k among the stretch's entries
  __shared__ EdgePos_t s_edge[kMaxLayerTransits];      // its first edge
  __shared__ float s_row_sum[kWithImportance ? kMaxLayerTransits : 1];  // 1 / (the weights of its transit added up)
  __shared__ uint32_t s_length[kMaxLayerTransits];     // length of every transit's sub-range, then the stretch's dense pieces
  __shared__ uint32_t s_ranges;                        // sub-ranges kept
  __shared__ uint32_t s_pieces;                        // dense pieces listed
  // A workgroup takes kBinsPerGroup consecutive stretches of one sample, one after the other:
  // where a transit's sub-range ends in one stretch it begins in the next, and the end is
  // then only a short gallop away instead of a search of the whole adjacency.
  constexpr uint32_t kBinsPerGroup = kWithImportance ? kBinsPerGroupSums : kBinsPerGroupBits;
  // the low stretches hold the hubs and take longest: all samples' first groups start first
  const uint32_t group = blockIdx.x / n_samples;
  const uint32_t s = blockIdx.x - group * n_samples;
  const uint32_t first_bin = group * kBinsPerGroup;
  const int32_t* transits = tv.base + (size_t)s * tv.stride;
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = threadIdx.x >> 6;
  // tv.count <= kBinThreads: lane i keeps transit i's adjacency and how far the stretches
  // before this one reach into it
  EdgePos_t my_end = 0, my_reach = 0;
  uint32_t my_next = 0xFFFFFFFFu;  // destination of edge my_reach; none left: above every vertex
  float my_row_sum = 1.0f;
  int32_t my_hub = -1;
  int32_t my_transit = -1;
  if (threadIdx.x < tv.count) {
    my_transit = transits[threadIdx.x];
    if (my_transit == invalid) my_transit = -1;
    if (my_transit != -1 && dense.hub_row) my_hub = dense.hub_row[my_transit];
  }
  bool hubs_among_transits = false;
  if (!kWithImportance) {
    // the byte map starts out clear and every stretch leaves it clear: what it reads on the
    // way out it sets back to zero, so no stretch spends a pass on clearing
    for (uint32_t i = threadIdx.x; i < kBinVertices / 4u; i += kBinThreads) s_bits[i] = 0;
    if (threadIdx.x < tv.count) s_start[threadIdx.x] = (uint32_t)my_transit;  // the table is free until the first stretch
    hubs_among_transits = __syncthreads_or(my_hub >= 0) != 0;
    // A vertex marks the same bits however often it is among the transits, and a layer drawn
    // with replacement by degree^2 repeats its hubs: 29 distinct transits of 64 at full size,
    // four fifths of all entries belong to repeats.  Only a vertex's first occurrence counts.
    if (my_transit != -1) {
      bool repeated = false;
      for (uint32_t j = 0; j < threadIdx.x; ++j) repeated |= s_start[j] == (uint32_t)my_transit;
      if (repeated) {
        my_transit = -1;
        my_hub = -1;
      }
    }
    __syncthreads();  // the table is written next
  } else {
    hubs_among_transits = __syncthreads_or(my_hub >= 0) != 0;
  }
  if (threadIdx.x < tv.count) {
    const int32_t t = my_transit;
    if (t != -1) {
      my_end = csr.row_ptr[t + 1];
      EdgePos_t lo = csr.row_ptr[t], hi = my_end;  // first edge whose destination is in the first stretch or above
      const uint32_t v_first = first_bin * kBinVertices;
      while (lo < hi) {
        const EdgePos_t mid = lo + (hi - lo) / 2;
        if ((uint32_t)csr.edges[mid] < v_first) lo = mid + 1; else hi = mid;
      }
      my_reach = lo;
      if (lo < my_end) my_next = (uint32_t)csr.edges[lo];
      if (kWithImportance) my_row_sum = inverse_row_sums[t];
    }
  }
  if (kWithImportance && !hubs_among_transits) {
    // LADIES form, a sample without hubs: the stretches of the workgroup as one.  At most kSparseGroupEntriesSums entries: their sums are
    // gathered in an LDS table hashed by vertex (in the room of the per-vertex sums), the
    // keys of the whole range are written as absent, and the table's vertices then get theirs.
    // Stretch by stretch, 16 chains of searches, tables and barriers cost a workgroup 130 us
    // for a few hundred entries.
    const uint32_t group_bins = first_bin + kBinsPerGroup < bins_per_sample ? kBinsPerGroup : bins_per_sample - first_bin;
    const uint32_t v_lo = first_bin * kBinVertices, v_hi = v_lo + group_bins * kBinVertices;
    if (threadIdx.x < tv.count) {
      uint32_t unused;
      const EdgePos_t stop =
          my_next < v_hi ? first_edge_at_or_above(csr.edges, my_reach, my_end, v_hi, &unused) : my_reach;
      s_length[threadIdx.x] = (uint32_t)(stop - my_reach);
      s_edge[threadIdx.x] = my_reach;
      s_row_sum[threadIdx.x] = my_row_sum;
    }
    __syncthreads();
    if (wave == 0) keep_filled_subranges<true>(tv.count, lane, s_length, s_edge, s_row_sum, s_start, &s_ranges, &s_pieces);
    __syncthreads();
    const uint32_t ranges = s_ranges;
    const uint32_t size = s_start[ranges];
    if (size <= kSparseGroupEntriesSums) {
      constexpr uint32_t kSlots = 2u * kSparseGroupEntriesSums;  // a power of two
      unsigned long long* slot_sum = s_acc;
      uint32_t* slot_vertex = (uint32_t*)(s_acc + kSlots);
      for (uint32_t i = threadIdx.x; i < kSlots; i += kBinThreads) {
        slot_vertex[i] = 0xFFFFFFFFu;
        slot_sum[i] = 0;
      }
      uint32_t* out_keys = keys_out.keys + (size_t)s * keys_per_sample + v_lo;
      for (uint32_t i = threadIdx.x; i < group_bins * kBinVertices; i += kBinThreads) out_keys[i] = kAbsentKey;
      __syncthreads();
      for (uint32_t e = threadIdx.x; e < size; e += kBinThreads) {
        uint32_t lo = 0, hi = ranges;  // the sub-range that holds entry e
        while (hi - lo > 1) {
          const uint32_t mid = lo + (hi - lo) / 2;
          if (s_start[mid] <= e) lo = mid; else hi = mid;
        }
        const EdgePos_t src = s_edge[lo] + (EdgePos_t)(e - s_start[lo]);
        const uint32_t local = (uint32_t)csr.edges[src] - v_lo;
        const float p = csr.weights[src] * s_row_sum[lo];
        const unsigned long long term = importance_term_fixed(p * p);
        uint32_t slot = (local * 2654435761u) >> 20 & (kSlots - 1u);
        for (;;) {  // at most half of the slots are ever taken
          const uint32_t before = atomicCAS(&slot_vertex[slot], 0xFFFFFFFFu, local);
          if (before == 0xFFFFFFFFu || before == local) break;
          slot = (slot + 1u) & (kSlots - 1u);
        }
        if (term != 0) atomicAdd(&slot_sum[slot], term);
      }
      __syncthreads();  // the table is complete, and the absent keys have been written
      for (uint32_t i = threadIdx.x; i < kSlots; i += kBinThreads) {
        const uint32_t local = slot_vertex[i];
        if (local == 0xFFFFFFFFu) continue;
        const uint32_t v = v_lo + local;
        out_keys[local] = ladies_key_bits(slot_sum[i], ladies_pair_index(keys_out.first_sample + s, keys_out.n_vertices, v),
                                          keys_out.step, keys_out.seed);
      }
      return;
    }
    // too many entries for that: stretch by stretch (the tables are next written after every
    // lane has read the size above)
  }
  if (!kWithImportance && !hubs_among_transits) {
    // The stretches of the workgroup as one: a bit per vertex fits the same LDS, and the few
    // entries can afford LDS atomics.  Per stretch, the searches, the table and the way out
    // are chains of dependent trips (to the caches, to LDS, through barriers) that cost the
    // same however few entries there are: 3.5 ms a layer at full size for 2 K entries a sample.
    const uint32_t group_bins = first_bin + kBinsPerGroup < bins_per_sample ? kBinsPerGroup : bins_per_sample - first_bin;
    const uint32_t v_lo = first_bin * kBinVertices, v_hi = v_lo + group_bins * kBinVertices;
    if (threadIdx.x < tv.count) {
      uint32_t unused;
      const EdgePos_t stop =
          my_next < v_hi ? first_edge_at_or_above(csr.edges, my_reach, my_end, v_hi, &unused) : my_reach;
      s_length[threadIdx.x] = (uint32_t)(stop - my_reach);
      s_edge[threadIdx.x] = my_reach;
    }
    __syncthreads();
    if (wave == 0) keep_filled_subranges<false>(tv.count, lane, s_length, s_edge, nullptr, s_start, &s_ranges, &s_pieces);
    __syncthreads();
    const uint32_t ranges = s_ranges;
    const uint32_t size = s_start[ranges];
    if (size <= kSparseGroupEntries) {
      for (uint32_t e = threadIdx.x; e < size; e += kBinThreads) {
        uint32_t lo = 0, hi = ranges;  // the sub-range that holds entry e
        while (hi - lo > 1) {
          const uint32_t mid = lo + (hi - lo) / 2;
          if (s_start[mid] <= e) lo = mid; else hi = mid;
        }
        const uint32_t local = (uint32_t)csr.edges[s_edge[lo] + (EdgePos_t)(e - s_start[lo])] - v_lo;
        atomicOr(&s_bits[local >> 5], 1u << (local & 31u));
      }
      __syncthreads();
      const uint32_t first_word = first_bin * kBinWords;
      uint32_t* out = bitmap + (size_t)s * words_per_sample + first_word;
      for (uint32_t i = threadIdx.x; i < group_bins * kBinWords && first_word + i < words_per_sample; i += kBinThreads)
        out[i] = s_bits[i];
      return;
    }
    // too many entries for that: stretch by stretch (nothing has been marked, and the tables
    // are next written after every lane has read the size above)
  }
  for (uint32_t bin = first_bin; bin < first_bin + kBinsPerGroup && bin < bins_per_sample; ++bin) {
  const uint32_t v_lo = bin * kBinVertices;
  if (kWithImportance) {
    for (uint32_t i = threadIdx.x; i < kBinWords; i += kBinThreads) s_bits[i] = 0;
    for (uint32_t i = threadIdx.x; i < kBinVerticesSums; i += kBinThreads) s_acc[i] = 0;
  }
  if (threadIdx.x < tv.count) {
    const EdgePos_t my_from = my_reach;
    const uint32_t v_hi = v_lo + kBinVertices;
    // nothing is fetched where the next edge already lies beyond the stretch (a short
    // adjacency misses most stretches)
    if (my_next < v_hi) my_reach = first_edge_at_or_above(csr.edges, my_from, my_end, v_hi, &my_next);
    uint32_t length = (uint32_t)(my_reach - my_from);
    if (my_hub >= 0 && length != 0) {
      const uint32_t piece = dense.piece_of[(size_t)my_hub * bins_per_sample + bin];
      if (piece != kNoPiece) length = kPieceFlag | piece;  // these entries reach the stretch ready-made
    }
    s_length[threadIdx.x] = length;
    s_edge[threadIdx.x] = my_from;  // by transit for now
    if (kWithImportance) s_row_sum[threadIdx.x] = my_row_sum;
  }
  __syncthreads();
  if (wave == 0)
    keep_filled_subranges<kWithImportance>(tv.count, lane, s_length, s_edge, s_row_sum, s_start, &s_ranges, &s_pieces);
  __syncthreads();
  const uint32_t ranges = s_ranges;
  const uint32_t size = s_start[ranges];
  // every wavefront walks a contiguous part of the entries, 64 * kBinAhead per round
  constexpr uint32_t kRound = 64u * kBinAhead;
  const uint32_t part = (size + kBinWaves * kRound - 1) / (kBinWaves * kRound) * kRound;
  const uint32_t part_begin = wave * part;
  const uint32_t part_end = part_begin + part < size ? part_begin + part : size;
  uint32_t cur = 0, cur_begin = 0, cur_end = 0;
  EdgePos_t cur_edges = 0;
  float cur_row_sum = 1.0f;
  if (part_begin + lane < part_end) {  // the sub-range of the lane's first entry
    const uint32_t e = part_begin + lane;
    uint32_t lo = 0, hi = ranges;
    while (hi - lo > 1) {
      const uint32_t mid = lo + (hi - lo) / 2;
      if (s_start[mid] <= e) lo = mid; else hi = mid;
    }
    cur = lo;
    cur_begin = s_start[lo];
    cur_end = s_start[lo + 1];
    cur_edges = s_edge[lo];
    if (kWithImportance) cur_row_sum = s_row_sum[lo];
  }
  if (!kWithImportance) {
    // FastGCN form: nothing is shared between neighbouring entries, so a lane takes four
    // consecutive entries per round - one 16-byte load and one round of index arithmetic for
    // four marks (the kernel is bound by instruction issue: its edge stream comes from the
    // caches) - unless its four entries straddle the end of a sub-range or of the part.
    struct __attribute__((packed, aligned(4))) FourIds { uint32_t id[4]; };
    for (uint32_t e0 = part_begin; e0 < part_end; e0 += kRound) {
      const uint32_t e = e0 + lane * kBinAhead;
      if (e >= part_end) continue;
      if (e >= cur_end) {
        do {
          ++cur;
          cur_begin = cur_end;
          cur_end = s_start[cur + 1];
        } while (e >= cur_end);
        cur_edges = s_edge[cur];
      }
      if (e + kBinAhead <= cur_end && e + kBinAhead <= part_end) {
        FourIds four;
        __builtin_memcpy(&four, csr.edges + cur_edges + (EdgePos_t)(e - cur_begin), sizeof(four));
#pragma unroll
        for (uint32_t a = 0; a < kBinAhead; ++a) s_bytes[four.id[a] - v_lo] = 1;
      } else {
        for (uint32_t a = 0; a < kBinAhead && e + a < part_end; ++a) {
          while (e + a >= cur_end) {
            ++cur;
            cur_begin = cur_end;
            cur_end = s_start[cur + 1];
            cur_edges = s_edge[cur];
          }
          s_bytes[(uint32_t)csr.edges[cur_edges + (EdgePos_t)(e + a - cur_begin)] - v_lo] = 1;
        }
      }
    }
  }
  for (uint32_t e0 = part_begin; kWithImportance && e0 < part_end; e0 += kRound) {  // the same trip count for every lane of a wave
    uint32_t locals[kBinAhead];  // vertex - v_lo
    float weights[kBinAhead], sums_of_row[kBinAhead];
#pragma unroll
    for (uint32_t a = 0; a < kBinAhead; ++a) {
      const uint32_t e = e0 + a * 64u + lane;
      locals[a] = 0xFFFFFFFFu;
      weights[a] = 0.0f;
      sums_of_row[a] = 1.0f;
      if (e < part_end) {
        if (e >= cur_end) {
          do {  // no sub-range is empty: at most a few steps
            ++cur;
            cur_begin = cur_end;
            cur_end = s_start[cur + 1];
          } while (e >= cur_end);
          cur_edges = s_edge[cur];
          if (kWithImportance) cur_row_sum = s_row_sum[cur];
        }
        const EdgePos_t src = cur_edges + (EdgePos_t)(e - cur_begin);
        locals[a] = (uint32_t)csr.edges[src] - v_lo;
        if (kWithImportance) {
          weights[a] = csr.weights[src];
          sums_of_row[a] = cur_row_sum;
        }
      }
    }
#pragma unroll
    for (uint32_t a = 0; a < kBinAhead; ++a) {
      const uint32_t local = locals[a];
      if (kWithImportance) {
        unsigned long long term = 0;
        if (local != 0xFFFFFFFFu) {
          const float p = weights[a] * sums_of_row[a];
          term = importance_term_fixed(p * p);
        }
        // Parallel edges sit in neighbouring lanes.  A few of them may as well hit the same
        // LDS word one after the other; a run of four or more somewhere in the wave (hub pairs
        // are joined by thousands of edges) is added up first, inside the rows of 16 lanes.
        // 0xFFFFFFFE: no lane holds it, so lane 0 always starts a segment.
        const uint32_t left = wave_from_below(0xFFFFFFFEu, local);
        uint32_t closed = (left != local || (lane & 15u) == 0) ? 1u : 0u;
        const uint64_t repeats = __ballot(left == local && local != 0xFFFFFFFFu);
        bool adds = true;  // this lane adds its term to the vertex's sum
        if ((repeats & (repeats >> 1) & (repeats >> 2)) != 0) {
          segmented_row_step<1>(closed, term);
          segmented_row_step<2>(closed, term);
          segmented_row_step<4>(closed, term);
          segmented_row_step<8>(closed, term);
          const uint32_t right = wave_from_above(0xFFFFFFFEu, local);
          adds = right != local || (lane & 15u) == 15u;
        }
        if (local != 0xFFFFFFFFu && adds) {
          if (term != 0) atomicAdd(&s_acc[local], term);
          atomicOr(&s_bits[local >> 5], 1u << (local & 31u));
        }
      } else if (local != 0xFFFFFFFFu) {
        s_bytes[local] = 1;
      }
    }
  }
  __syncthreads();
  if (kWithImportance) {
    // LADIES form: what leaves the workgroup is the sampling key of every vertex of the
    // stretch (kAbsentKey where the neighbourhood does not hold the vertex); no bitmap.
    // A lane takes four consecutive vertices: 16-byte accesses to LDS, to the pieces and to
    // the output, and one Philox block where it forms keys.
    const uint32_t n_pieces = s_pieces;
    for (uint32_t q = threadIdx.x; q < kBinVerticesSums / 4u; q += kBinThreads) {
      const uint32_t i = 4u * q;
      const uint32_t bits = (s_bits[i >> 5] >> (i & 31u)) & 15u;
      const ulonglong2 low = ((const ulonglong2*)s_acc)[2u * q], high = ((const ulonglong2*)s_acc)[2u * q + 1u];
      unsigned long long sum[4] = {low.x, low.y, high.x, high.y};  // 0 where nothing was added
      bool present[4] = {(bits & 1u) != 0, (bits & 2u) != 0, (bits & 4u) != 0, (bits & 8u) != 0};
#pragma unroll 4
      for (uint32_t p = 0; p < n_pieces; ++p) {  // integer sums: the order of the additions does not matter
        const ulonglong2* piece = (const ulonglong2*)(dense.sums + (size_t)s_length[p] * kBinVerticesSums + i);
        const ulonglong2 a = piece[0], b = piece[1];
        const unsigned long long ready[4] = {a.x, a.y, b.x, b.y};
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k)
          if (ready[k] != kAbsentSum) {
            sum[k] += ready[k];
            present[k] = true;
          }
      }
      uint32_t key[4] = {kAbsentKey, kAbsentKey, kAbsentKey, kAbsentKey};
      if (present[0] || present[1] || present[2] || present[3]) {
        const PhiloxBlock blk = ladies_block(ladies_pair_index(keys_out.first_sample + s, keys_out.n_vertices, v_lo + i),
                                             keys_out.step, keys_out.seed);
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k)
          if (present[k]) key[k] = ladies_key_from_word(sum[k], blk.w[k]);
      }
      *(uint4*)(keys_out.keys + (size_t)s * keys_per_sample + v_lo + i) = make_uint4(key[0], key[1], key[2], key[3]);
    }
  } else {
    const uint32_t first_word = bin * kBinWords;
    uint32_t* out = bitmap + (size_t)s * words_per_sample + first_word;
    const uint32_t n_pieces = s_pieces;
    // two words per lane (stretches and bitmaps hold even numbers of words): eight bytes per
    // load of a piece, several pieces under way
    const uint32_t i = 2u * threadIdx.x;
    if (i < kBinWords && first_word + i < words_per_sample) {
      uint2 words = make_uint2(0u, 0u);
      if (size != 0) {  // 2 x 32 bytes, each 0 or 1 -> 2 x 32 bits
        uint4* bytes = (uint4*)s_bits + i * 2u;
        const uint4 q0 = bytes[0], q1 = bytes[1], q2 = bytes[2], q3 = bytes[3];
        const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
        bytes[0] = zero;
        bytes[1] = zero;
        bytes[2] = zero;
        bytes[3] = zero;
        const uint32_t low[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
        const uint32_t high[8] = {q2.x, q2.y, q2.z, q2.w, q3.x, q3.y, q3.z, q3.w};
#pragma unroll
        for (uint32_t q = 0; q < 8; ++q) {
          const uint32_t four = low[q], next_four = high[q];
          words.x |= ((four & 1u) | ((four >> 7) & 2u) | ((four >> 14) & 4u) | ((four >> 21) & 8u)) << (4u * q);
          words.y |= ((next_four & 1u) | ((next_four >> 7) & 2u) | ((next_four >> 14) & 4u) | ((next_four >> 21) & 8u))
                     << (4u * q);
        }
      }
#pragma unroll 8
      for (uint32_t p = 0; p < n_pieces; ++p) {
        const uint2 piece = *(const uint2*)(dense.words + (size_t)s_length[p] * kBinWords + i);
        words.x |= piece.x;
        words.y |= piece.y;
      }
      *(uint2*)(out + i) = words;
    }
  }
  __syncthreads();  // the next stretch clears what this one has just read
  }
}

// ---- FastGCN form: the marked vertices of a sample weighted by degree^2, without a list ----
//
// The app draws "the first marked vertex, ascending, whose running sum of degree^2 exceeds a
// target".  Listing the marked vertices with their running sums costs 20 bytes for each of
// the 2.0e9 distinct pairs of a full-size pass; instead the bitmap is kept and summed at two
// levels - groups of 256 vertices (8 words) and parts of 64 groups - so that a draw searches
// the parts of its sample, then the groups of one part, then walks one group's set bits.
constexpr uint32_t kGroupWords = 8;
constexpr uint32_t kGroupsPerPart = 64;
constexpr uint32_t kPartWords = kGroupWords * kGroupsPerPart;  // 16384 vertices

// The degrees of a part's 16,384 vertices do not depend on the sample, so a workgroup keeps
// them in LDS and runs its samples past them: fetching the row extents of every marked vertex
// of every sample from the caches instead (2.0e9 gathers a pass at full size, a lane waiting
// for each) took as long as the marking itself.
constexpr uint32_t kSumThreads = 1024;
constexpr uint32_t kSumSamplesPerBlock = 128;
constexpr uint32_t kGroupVertices = kGroupWords * 32u;
constexpr uint32_t kGroupPitch = kGroupVertices + 1u;  // lanes walk different groups: the odd pitch spreads them over the banks

// One workgroup per (part, block of 128 samples), a wavefront per sample, a lane per group:
// group_through[(s * parts + part) * 64 + g] = degree^2 of the marked vertices of groups 0..g
// of the part; part_total[s * parts + part]; marked[s] += marked vertices.  Workgroups of the
// low parts (where the hubs of a skewed graph sit, marked in nearly every sample) come first.
__global__ __launch_bounds__(kSumThreads) void bitmap_group_sums(const uint32_t* __restrict__ bitmap,
                                                                 uint32_t words_per_sample, uint32_t n_samples,
                                                                 uint32_t n_vertices,
                                                                 const EdgePos_t* __restrict__ row_ptr,
                                                                 uint64_t* __restrict__ group_through,
                                                                 uint64_t* __restrict__ part_total,
                                                                 uint32_t* __restrict__ marked) {
  __shared__ uint32_t s_degree[kGroupsPerPart * kGroupPitch];
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t parts_per_sample = words_per_sample / kPartWords;
  const uint32_t sample_blocks = (n_samples + kSumSamplesPerBlock - 1) / kSumSamplesPerBlock;
  const uint32_t part = blockIdx.x / sample_blocks;
  const uint32_t first_sample = (blockIdx.x - part * sample_blocks) * kSumSamplesPerBlock;
  const uint32_t first_vertex = part * (kPartWords * 32u);
  for (uint32_t i = threadIdx.x; i < kPartWords * 32u; i += kSumThreads) {
    const uint32_t v = first_vertex + i;
    s_degree[(i / kGroupVertices) * kGroupPitch + i % kGroupVertices] =
        v < n_vertices ? (uint32_t)(row_ptr[v + 1] - row_ptr[v]) : 0u;
  }
  __syncthreads();
  const uint32_t end_sample = first_sample + kSumSamplesPerBlock < n_samples ? first_sample + kSumSamplesPerBlock : n_samples;
  const uint32_t* mine = s_degree + lane * kGroupPitch;
  for (uint32_t s = first_sample + wave; s < end_sample; s += kSumThreads / kWave) {
    const uint4* words = (const uint4*)(bitmap + (size_t)s * words_per_sample + (size_t)part * kPartWords + lane * kGroupWords);
    const uint4 a = words[0], b = words[1];
    // word by word: finding and clearing the lowest set bit of a 32-bit word is three vector
    // instructions, of a 64-bit one eight, and the launch is bound by instruction issue
    const uint32_t w[kGroupWords] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    uint64_t sum = 0;
    uint32_t count = 0;
#pragma unroll
    for (uint32_t k = 0; k < kGroupWords; ++k) {
      uint32_t bits = w[k];
      count += (uint32_t)__popc(bits);
      const uint32_t* from = mine + k * 32u;
      while (bits) {
        const uint32_t i0 = (uint32_t)__ffs((int)bits) - 1u;
        bits &= bits - 1u;
        const uint64_t d0 = from[i0];
        sum += d0 * d0;
      }
    }
    const uint64_t through = wave_inclusive_scan_u64(sum);
    const size_t at = (size_t)s * parts_per_sample + part;
    group_through[at * kGroupsPerPart + lane] = through;
    if (lane == 63) part_total[at] = through;
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) count += __shfl_xor(count, d, kWave);
    if (lane == 0 && count) atomicAdd(&marked[s], count);
  }
}

// One wavefront per sample: part_before[s * (parts + 1) + p] = degree^2 of the marked vertices
// of the sample's parts before p; entry `parts` is the sample's total.
__global__ __launch_bounds__(64) void sample_part_sums(const uint64_t* __restrict__ part_total, uint32_t parts,
                                                       uint64_t* __restrict__ part_before) {
  const uint32_t s = blockIdx.x, lane = threadIdx.x;
  uint64_t carry = 0;
  for (uint32_t p0 = 0; p0 < parts; p0 += 64) {
    const uint32_t p = p0 + lane;
    const uint64_t mine = p < parts ? part_total[(size_t)s * parts + p] : 0ull;
    const uint64_t through = wave_inclusive_scan_u64(mine);
    if (p < parts) part_before[(size_t)s * (parts + 1) + p] = carry + through - mine;
    const uint32_t lo = __shfl((uint32_t)through, 63, kWave), hi = __shfl((uint32_t)(through >> 32), 63, kWave);
    carry += ((uint64_t)hi << 32) | lo;
  }
  if (lane == 0) part_before[(size_t)s * (parts + 1) + parts] = carry;
}

// What next() of a kDistinctByDegreeSquared app receives as transitEdges.
struct DistinctByDegreeSquared {
  const uint32_t* bits;           // the sample's bitmap
  const uint64_t* part_before;    // the sample's parts + 1 entries
  const uint64_t* group_through;  // the sample's parts * 64 entries
  const EdgePos_t* row_ptr;
  uint32_t parts;

  __device__ __forceinline__ uint64_t total() const { return part_before[parts]; }

  // the smallest marked vertex whose running sum of degree^2 (marked vertices ascending)
  // exceeds target; target < total()
  __device__ inline VertexID first_exceeding(uint64_t target) const {
    uint32_t lo = 0, hi = parts;  // last part whose sum-before is <= target
    while (hi - lo > 1) {
      const uint32_t mid = lo + (hi - lo) / 2;
      if (part_before[mid] <= target) lo = mid; else hi = mid;
    }
    const uint32_t part = lo;
    target -= part_before[part];
    const uint64_t* through = group_through + (size_t)part * kGroupsPerPart;
    uint32_t first = 0, last = kGroupsPerPart - 1;  // first group whose sum-through exceeds target
    while (first < last) {
      const uint32_t mid = first + (last - first) / 2;
      if (through[mid] > target) last = mid; else first = mid + 1;
    }
    if (first) target -= through[first - 1];
    const uint32_t first_word = part * kPartWords + first * kGroupWords;
    uint64_t running = 0;
    VertexID found = -1;
    for (uint32_t k = 0; k < kGroupWords && found < 0; ++k) {
      uint32_t word = bits[first_word + k];
      while (word) {
        const uint32_t v = (first_word + k) * 32u + (uint32_t)__ffs((int)word) - 1u;
        const uint64_t d = (uint64_t)(row_ptr[v + 1] - row_ptr[v]);
        running += d * d;
        if (running > target) { found = (VertexID)v; break; }
        word &= word - 1u;
      }
    }
    return found;
  }
};

// item_count[s] = work items of sample s (at least one, so that row offsets get written)
__global__ void build_item_counts(const uint32_t* __restrict__ sizes, uint32_t n, uint32_t* __restrict__ item_count) {
  const uint32_t s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s < n) {
    const uint32_t items = (sizes[s] + kBuildItemEntries - 1) / kBuildItemEntries;
    item_count[s] = items ? items : 1u;
  } else if (s == n) {
    item_count[s] = 0;
  }
}

__global__ void gather_u32(const uint32_t* __restrict__ table, const uint32_t* __restrict__ index, size_t n,
                           uint32_t* __restrict__ out, uint32_t* __restrict__ index_copy) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint32_t p = index[i];
  out[i] = table[p];
  if (index_copy) index_copy[i] = p;
}

__global__ void fill_u32(uint32_t* dst, size_t n, uint32_t value) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = value;
}

// ---- the best m keys of every sample, without sorting everything ----
//
// Only the first stepSize ranked vertices of a sample are ever read, out of up to millions of
// distinct ones.  A radix select on the upper 14 bits of the sort key finds, per sample, the
// smallest prefix T such that at least m keys have a prefix <= T; the entries with a prefix
// <= T (m and some more) are copied out and only those are sorted.
// The keys of a chunk are dense: keys[s * keys_per_sample + v] for every vertex v (kAbsentKey
// where sample s does not hold v), so position tells sample and vertex and no list of the
// distinct pairs is ever written.

// One workgroup per sample, one pass over its keys: counts the present ones by their upper
// kSelectBits bits in an LDS
// histogram and picks the bin that holds the wanted-th smallest key: threshold[s] = that bin,
// kept[s] = keys up to and including it (a sample with fewer keys than wanted keeps them all),
// present[s] = all its keys.  A sample's whole histogram stays in the workgroup: no atomic
// reaches memory, and no second pass over the keys refines the threshold (two levels of 8 bits,
// counted by a workgroup per tile of 8192 keys, read every key twice).
constexpr uint32_t kSelectBits = 14;
constexpr uint32_t kSelectBins = 1u << kSelectBits;
constexpr uint32_t kSelectThreads = 1024;
// The pass also notes, for every stretch of 256 consecutive keys (what a wavefront handles at a
// time, four keys per lane), the smallest prefix in it: the copying of the kept entries then
// reads only the stretches that hold one (a few hundred of a sample's 12,000).
constexpr uint32_t kCollectStretch = 256;
__device__ __forceinline__ void note_best_of_stretch(const uint32_t (&key)[4], uint32_t quad, uint32_t lane,
                                                     uint16_t* __restrict__ best_of) {
  uint32_t a = key[0] < key[1] ? key[0] : key[1], b = key[2] < key[3] ? key[2] : key[3];
  uint32_t best = (a < b ? a : b) >> (32u - kSelectBits);  // kAbsentKey: the largest prefix
  // minimum of the wavefront into lane 63, on the VALU (DPP): along the rows of 16 lanes, then
  // the last lane of a row into the next row, then lane 31 into the upper half
  const uint32_t none = 0xFFFFFFFFu;
  uint32_t other = row_shift_up<1>(none, best);
  best = other < best ? other : best;
  other = row_shift_up<2>(none, best);
  best = other < best ? other : best;
  other = row_shift_up<4>(none, best);
  best = other < best ? other : best;
  other = row_shift_up<8>(none, best);
  best = other < best ? other : best;
  other = (uint32_t)__builtin_amdgcn_update_dpp((int)none, (int)best, 0x142, 0xA, 0xF, false);  // row_bcast:15
  best = other < best ? other : best;
  other = (uint32_t)__builtin_amdgcn_update_dpp((int)none, (int)best, 0x143, 0xC, 0xF, false);  // row_bcast:31
  best = other < best ? other : best;
  if (lane == 63) best_of[quad / 64u] = (uint16_t)best;
}
__global__ __launch_bounds__(kSelectThreads, 8) __attribute__((amdgpu_num_vgpr(56))) void select_threshold(
    const uint32_t* __restrict__ keys, uint32_t keys_per_sample, uint32_t wanted,
    uint32_t* __restrict__ threshold, uint32_t* __restrict__ kept, uint32_t* __restrict__ present,
    uint16_t* __restrict__ stretch_best) {
  __shared__ uint32_t s_hist[kSelectBins];
  __shared__ uint32_t s_wave_total[kSelectThreads / 64];
  const uint32_t s = blockIdx.x;
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  for (uint32_t i = threadIdx.x; i < kSelectBins; i += kSelectThreads) s_hist[i] = 0;
  __syncthreads();
  const uint32_t* mine = keys + (size_t)s * keys_per_sample;
  uint16_t* my_best = stretch_best + (size_t)s * (keys_per_sample / kCollectStretch);
  {
    const uint4* my_keys = (const uint4*)mine;
    for (uint32_t q0 = 0; q0 < keys_per_sample / 4u; q0 += 4 * kSelectThreads) {
      uint4 batch[4];
#pragma unroll
      for (uint32_t k = 0; k < 4; ++k) {
        const uint32_t q = q0 + k * kSelectThreads + threadIdx.x;
        batch[k] = q < keys_per_sample / 4u ? my_keys[q] : make_uint4(kAbsentKey, kAbsentKey, kAbsentKey, kAbsentKey);
      }
#pragma unroll
      for (uint32_t k = 0; k < 4; ++k) {
        const uint32_t q = q0 + k * kSelectThreads + threadIdx.x;
        if (q >= keys_per_sample / 4u) continue;  // whole wavefronts: the sample holds a multiple of 256 keys
        const uint32_t key[4] = {batch[k].x, batch[k].y, batch[k].z, batch[k].w};
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i)
          if (key[i] != kAbsentKey) atomicAdd(&s_hist[key[i] >> (32u - kSelectBits)], 1u);
        note_best_of_stretch(key, q, lane, my_best);
      }
    }
  }
  __syncthreads();
  // lane t owns bins [16 t, 16 t + 16): the bin in which the running count reaches `wanted`
  constexpr uint32_t kOwn = kSelectBins / kSelectThreads;
  uint32_t own = 0;
#pragma unroll
  for (uint32_t b = 0; b < kOwn; ++b) own += s_hist[threadIdx.x * kOwn + b];
  const uint32_t through_wave = wave_inclusive_scan(own);
  if (lane == 63) s_wave_total[wave] = through_wave;
  __syncthreads();
  uint32_t before = through_wave - own, total = 0;
#pragma unroll
  for (uint32_t w = 0; w < kSelectThreads / 64; ++w) {
    const uint32_t t = s_wave_total[w];
    if (w < wave) before += t;
    total += t;
  }
  if (threadIdx.x == 0) present[s] = total;
  if (total < wanted) {  // everything stays
    if (threadIdx.x == 0) {
      threshold[s] = kSelectBins - 1u;
      kept[s] = total;
    }
  } else if (before < wanted && before + own >= wanted) {  // exactly one lane
    uint32_t running = before;
    for (uint32_t b = 0; b < kOwn; ++b) {
      running += s_hist[threadIdx.x * kOwn + b];
      if (running >= wanted) {
        threshold[s] = threadIdx.x * kOwn + b;
        kept[s] = running;
        break;
      }
    }
  }
}

__device__ __forceinline__ bool select_keeps(uint32_t key, uint32_t threshold) {
  return key != kAbsentKey && (key >> (32u - kSelectBits)) <= threshold;
}

// Copies the kept entries of sample s into its part [ranked_start[s], ranked_start[s + 1]) of
// kept_key / kept_id, in whatever order the wavefronts get there (a wavefront claims room for
// the entries of a round with one atomic).  A few hundred of a sample's millions of keys stay:
// one workgroup per sample, whose wavefronts look at the best prefix of each stretch of 256 keys
// first and read only those that hold a kept key.  The sorts that follow fix the order.
__global__ __launch_bounds__(kSelectThreads) void select_collect(const uint32_t* __restrict__ keys,
                                                                 uint32_t keys_per_sample,
                                                                 const uint16_t* __restrict__ stretch_best,
                                                      const uint32_t* __restrict__ threshold_of,
                                                      const uint32_t* __restrict__ ranked_start,
                                                      uint32_t* __restrict__ claimed, uint32_t* __restrict__ kept_key,
                                                      uint32_t* __restrict__ kept_sample, int32_t* __restrict__ kept_id) {
  const uint32_t s = blockIdx.x;
  const uint32_t* mine = keys + (size_t)s * keys_per_sample;
  const uint32_t stretches = keys_per_sample / kCollectStretch;
  const uint16_t* best_of = stretch_best + (size_t)s * stretches;
  const uint32_t threshold = threshold_of[s];
  const uint32_t first = ranked_start[s];
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  // a wavefront looks at 64 stretches at a time: lane i knows whether stretch i holds a kept key
  for (uint32_t stretch_begin = wave * 64u; stretch_begin < stretches; stretch_begin += (kSelectThreads / 64u) * 64u) {
    const uint32_t my_stretch = stretch_begin + lane;
    const bool holds = my_stretch < stretches && best_of[my_stretch] <= threshold;
    uint64_t todo = __ballot(holds);
    while (todo) {  // the same for every lane
      const uint32_t stretch = stretch_begin + (uint32_t)__ffsll((long long)todo) - 1u;
      todo &= todo - 1ull;
      const uint32_t v0 = stretch * kCollectStretch + lane * 4u;
      const uint4 four = *(const uint4*)(mine + v0);
      const uint32_t key[4] = {four.x, four.y, four.z, four.w};
#pragma unroll
      for (uint32_t i = 0; i < 4; ++i) {
        const bool stays = select_keeps(key[i], threshold);
        const uint64_t mask = __ballot(stays);
        if (mask == 0) continue;
        uint32_t base = 0;
        if (lane == (uint32_t)__ffsll((long long)mask) - 1u) base = atomicAdd(&claimed[s], (uint32_t)__popcll(mask));
        base = __shfl(base, __ffsll((long long)mask) - 1, kWave);
        if (stays) {
          const uint32_t at = first + base + (uint32_t)__popcll(mask & ((1ull << lane) - 1ull));
          kept_key[at] = key[i];
          kept_sample[at] = s;
          kept_id[at] = (int32_t)(v0 + i);
        }
      }
    }
  }
}

struct LayerParams {
  CSRPartition csr;
  TransitView transits;   // base already points at the first sample of the chunk
  int step;
  uint32_t step_size;
  uint32_t chunk_samples; // samples in this launch
  uint32_t sample_begin;  // index of the chunk's first sample
  uint32_t final_size;
  uint32_t out_base;      // stepSizeAtStep(step - 1)
  int32_t invalid;
  uint64_t seed;
  uint64_t first_sample;  // index of the device's first sample (multi-device offset)
  int32_t* final_samples;
  void* samples;
  // kConcatenated: offsets are relative to the chunk
  const uint32_t* offsets;
  const int32_t* nbr_cols;
  const float* nbr_weights;
  // kRankedByLadiesImportance: the kept ids of sample ls in descending key order are
  // ranked_ids[ranked_start[ls] .. ranked_start[ls + 1])
  const uint32_t* ranked_start;
  const int32_t* ranked_ids;
  // kDistinctByDegreeSquared: bitmaps and their two levels of degree^2 sums
  const uint32_t* bitmap;
  uint32_t words_per_sample;
  const uint64_t* part_before;
  const uint64_t* group_through;
  const uint32_t* marked;        // marked vertices per sample
};

template <class SampleType, class App>
__global__ __launch_bounds__(256) void layer_execute_kernel(LayerParams P) {
  const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (uint64_t)P.chunk_samples * P.step_size) return;
  const uint32_t ls = (uint32_t)(i / P.step_size);  // sample inside the chunk
  const uint32_t nbr = (uint32_t)(i - (uint64_t)ls * P.step_size);
  const uint32_t s = P.sample_begin + ls;
  CSRPartition csr = P.csr;
  const int32_t* transits = P.transits.base + (size_t)ls * P.transits.stride;
  SampleType local_state;
  SampleType* state = std::is_empty<SampleType>::value ? &local_state : (SampleType*)P.samples + s;
  curandState rng;
  rng.reset(P.seed, (P.first_sample + s) * P.step_size + nbr, (uint32_t)P.step);
  const VertexID sample_id = (VertexID)(P.first_sample + s);
  VertexID neighbor = P.invalid;
  if constexpr (apps::neighborhood_form_of<App>::value == apps::kConcatenated) {
    // only the first transit decides whether next() runs (nextdoor.cu:1421)
    if (transits[0] != P.invalid && transits[0] != -1) {
      const uint32_t begin = P.offsets[ls];
      const CSR::Edge* edges = P.nbr_cols + begin;
      const float* weights = P.nbr_weights + begin;
      const VertexID r = App().template next<SampleType, const CSR::Edge*, const float*>(
          P.step, &csr, transits, sample_id, state, 0.0f, edges, weights, (EdgePos_t)(P.offsets[ls + 1] - begin),
          (VertexID_t)nbr, &rng);
      neighbor = r == -1 ? P.invalid : r;
    }
  } else if constexpr (apps::neighborhood_form_of<App>::value == apps::kDistinctByDegreeSquared) {
    const uint32_t parts = P.words_per_sample / kPartWords;
    DistinctByDegreeSquared distinct{P.bitmap + (size_t)ls * P.words_per_sample,
                                     P.part_before + (size_t)ls * (parts + 1),
                                     P.group_through + (size_t)ls * parts * kGroupsPerPart, csr.row_ptr, parts};
    const float* no_weights = nullptr;
    const VertexID r = App().template next<SampleType, DistinctByDegreeSquared, const float*>(
        P.step, &csr, transits, sample_id, state, 0.0f, distinct, no_weights, (EdgePos_t)P.marked[ls],
        (VertexID_t)nbr, &rng);
    neighbor = r == -1 ? P.invalid : r;
  } else {
    const uint32_t begin = P.ranked_start[ls];
    const CSR::Edge* ranked = P.ranked_ids + begin;
    const float* no_weights = nullptr;
    const VertexID r = App().template next<SampleType, const CSR::Edge*, const float*>(
        P.step, &csr, transits, sample_id, state, 0.0f, ranked, no_weights,
        (EdgePos_t)(P.ranked_start[ls + 1] - begin), (VertexID_t)nbr, &rng);
    neighbor = r == -1 ? P.invalid : r;
  }
  P.final_samples[(size_t)s * P.final_size + P.out_base + nbr] = neighbor;
}

// Entries of concatenated neighbourhood one chunk of samples may hold (about 70 bytes of
// device memory per entry across all work arrays).
constexpr uint64_t kLayerChunkEntries = 96ull << 20;
// Importance forms: nothing is stored per entry, so a chunk is bounded by the memory of its
// presence maps (and accumulators) and by the number of marking work items (entries / kBuildItemEntries) of one launch.
constexpr uint64_t kBitmapBudgetBytes = 48ull << 30;
constexpr uint64_t kBitmapChunkEntries = 1ull << 40;

template <class SampleType, class App>
class LayerEngine : public EngineBase {
 public:
  explicit LayerEngine(const char* name) : name_(name) {}
  ~LayerEngine() override { free_device(); }

  const char* app_name() const override { return name_; }
  int64_t num_samples() const override { return n_samples_; }
  int final_sample_size() const override { return nd::final_sample_size<App>(); }
  int steps() const override { return App().steps(); }
  int step_size(int k) const override { return App().stepSize(k); }
  int initial_sample_size() const override { return App().initialSampleSize(nullptr); }
  int sampling_type() const override { return App().samplingType(); }
  int32_t invalid_vertex() const override { return invalid_; }
  int max_bits() const override { return max_bits_; }
  size_t sample_state_bytes() const override {
    return std::is_empty<SampleType>::value ? 0 : sizeof(SampleType) * (size_t)n_samples_;
  }

  int set_graph(const CSR* graph) override {
    free_run_buffers();  // sized against the previous graph: alloc() is due again
    graph_ = nullptr;
    release(d_row_sums_);
    if (!dgraph_.upload(graph, false, app_uses_edge_lookup<App>::value, &last_error)) return -1;
    if (apps::neighborhood_form_of<App>::value == apps::kRankedByLadiesImportance) {
      // 1 / (weights of every vertex summed in edge order, sequential float adds)
      const size_t V = (size_t)graph->get_n_vertices();
      std::vector<float> sums(V);
      for (size_t v = 0; v < V; ++v) {
        float acc = 0.0f;
        for (EdgePos_t x = graph->row_ptr[v]; x < graph->row_ptr[v + 1]; ++x) acc = acc + graph->weight[x];
        sums[v] = 1.0f / acc;  // the kernels multiply by the inverse
      }
      ND_HIP_TRY(hipMalloc(&d_row_sums_, sizeof(float) * V));
      ND_HIP_TRY(hipMemcpy(d_row_sums_, sums.data(), sizeof(float) * V, hipMemcpyHostToDevice));
      const int rc = build_dense_pieces(graph, sums.data());
      if (rc != 0) return rc;
    }
    if (apps::neighborhood_form_of<App>::value == apps::kDistinctByDegreeSquared) {
      const int rc = build_dense_pieces(graph, nullptr);
      if (rc != 0) return rc;
    }
    graph_ = graph;
    return 0;
  }

  int alloc(uint64_t seed) override {
    if (!graph_) { last_error = "alloc before set_graph"; return -1; }
    free_run_buffers();
    seed_ = seed;
    CSR* csr = const_cast<CSR*>(graph_);
    App app;
    if (!is_collective<App>()) { last_error = "not a CollectiveNeighborhood app"; return -2; }
    if (app.hasExplicitTransits()) { last_error = "apps with explicit transits are not supported"; return -2; }
    const int n_steps = app.steps();
    if (n_steps < 1 || n_steps > kMaxSteps) { last_error = "steps() must be in [1, 128]"; return -2; }
    n_samples_ = app.numSamples(csr);
    init_size_ = app.initialSampleSize(csr);
    if (n_samples_ <= 0 || init_size_ <= 0) { last_error = "app yields no samples"; return -2; }
    if (n_samples_ >= (1ll << 31)) { last_error = "too many samples"; return -2; }
    uint32_t widest = (uint32_t)init_size_;
    for (int k = 0; k < n_steps; ++k) {
      if (app.stepSize(k) <= 0) { last_error = "stepSize must be positive"; return -2; }
      if ((uint32_t)app.stepSize(k) > widest) widest = (uint32_t)app.stepSize(k);
    }
    if (widest > kMaxLayerTransits) { last_error = "more than 1024 transits per sample"; return -2; }
    invalid_ = graph_->get_n_vertices();
    max_bits_ = 0;
    while ((invalid_ >> max_bits_) != 0) max_bits_++;

    samples_.clear();
    initialContents.clear();
    samples_.reserve((size_t)n_samples_);
    for (int64_t s = 0; s < n_samples_; ++s) {
      samples_.push_back(app.template initializeSample<SampleType>(csr, (VertexID_t)s));
      std::vector<VertexID_t> roots = app.initialSample((int)s, csr, samples_.back());
      if ((EdgePos_t)roots.size() != init_size_) {
        last_error = "initialSample size differs from initialSampleSize";
        return -2;
      }
      if (!roots_are_vertices(roots, graph_->get_n_vertices())) {
        last_error = "initialSample returned a root that is not a vertex of the graph";
        return -2;
      }
      initialContents.insert(initialContents.end(), roots.begin(), roots.end());
    }
    const size_t F = (size_t)final_sample_size();
    hFinalSamples.assign((size_t)n_samples_ * F, invalid_);
    h_sizes_.resize((size_t)n_samples_);
    chunk_entries_ = kLayerChunkEntries;
    bitmap_chunk_entries_ = kBitmapChunkEntries;
    progress_ = getenv("ND_PROGRESS") != nullptr;  // long layers report on stderr every 16 chunks
    if (const char* env = getenv("ND_LAYER_CHUNK_ENTRIES")) {  // smaller chunks, e.g. to exercise chunking
      const long long v = atoll(env);
      if (v > 0) chunk_entries_ = bitmap_chunk_entries_ = (uint64_t)v;
    }
    // one byte per vertex for the LADIES form, one bit for the FastGCN form
    bitmap_words_ = bitmap_words_for((uint32_t)invalid_);
    // bytes a sample of a chunk holds: its bitmap (FastGCN form) or one key per vertex, padded
    // to whole stretches (LADIES form)
    uint64_t bytes_per_sample = (uint64_t)bitmap_words_ * sizeof(uint32_t);
    if (apps::neighborhood_form_of<App>::value == apps::kRankedByLadiesImportance) {
      const uint32_t bin_words = kBinVerticesSums / 32u;
      bytes_per_sample = (uint64_t)((bitmap_words_ + bin_words - 1) / bin_words) * kBinVerticesSums * sizeof(uint32_t);
    }
    const uint64_t fit = kBitmapBudgetBytes / bytes_per_sample;
    bitmap_chunk_samples_ = fit < 1 ? 1u : fit > (uint64_t)n_samples_ ? (uint32_t)n_samples_ : (uint32_t)fit;
    // the selection kernels of the LADIES form index the samples of a chunk by blockIdx.y
    if (apps::neighborhood_form_of<App>::value == apps::kRankedByLadiesImportance && bitmap_chunk_samples_ > 65535u)
      bitmap_chunk_samples_ = 65535u;

    ND_HIP_TRY(hipStreamCreate(&stream_));
    ND_HIP_TRY(hipEventCreate(&ev_begin_));
    ND_HIP_TRY(hipEventCreate(&ev_end_));
    ND_HIP_TRY(hipEventCreate(&ev_a_));
    ND_HIP_TRY(hipEventCreate(&ev_b_));
    allocated_ = true;
    ND_HIP_TRY(hipMalloc(&d_initial_, sizeof(VertexID_t) * initialContents.size()));
    ND_HIP_TRY(hipMemcpy(d_initial_, initialContents.data(), sizeof(VertexID_t) * initialContents.size(),
                         hipMemcpyHostToDevice));
    if (!std::is_empty<SampleType>::value) {
      ND_HIP_TRY(hipMalloc(&d_samples_, sizeof(SampleType) * (size_t)n_samples_));
      ND_HIP_TRY(hipMalloc(&d_samples_init_, sizeof(SampleType) * (size_t)n_samples_));
      ND_HIP_TRY(hipMemcpy(d_samples_init_, samples_.data(), sizeof(SampleType) * (size_t)n_samples_,
                           hipMemcpyHostToDevice));
      // what fetch_sample_states gives before the first run
      ND_HIP_TRY(hipMemcpy(d_samples_, d_samples_init_, sizeof(SampleType) * (size_t)n_samples_,
                           hipMemcpyDeviceToDevice));
      std::vector<SampleType>().swap(samples_);  // the pristine copy now lives on the device
    }
    ND_HIP_TRY(hipMalloc(&d_final_, sizeof(VertexID_t) * (size_t)n_samples_ * F));
    ND_HIP_TRY(hipMalloc(&d_sizes_, sizeof(uint32_t) * ((size_t)n_samples_ + 1)));
    ND_HIP_TRY(hipMemset(d_sizes_, 0, sizeof(uint32_t) * ((size_t)n_samples_ + 1)));
    ND_HIP_TRY(hipMalloc(&d_offsets_, sizeof(uint32_t) * ((size_t)n_samples_ + 1)));
    ND_HIP_TRY(hipMalloc(&d_item_count_, sizeof(uint32_t) * ((size_t)n_samples_ + 1)));
    ND_HIP_TRY(hipMalloc(&d_item_start_, sizeof(uint32_t) * ((size_t)n_samples_ + 1)));
    ND_HIP_TRY(hipMalloc(&d_row_offsets_, sizeof(uint32_t) * (size_t)n_samples_ * widest));
    ND_HIP_TRY(hipMalloc(&d_small_scratch_, sizeof(uint32_t) * scan_scratch_elems((size_t)n_samples_ + 1)));
    if (apps::neighborhood_form_of<App>::value == apps::kRankedByLadiesImportance) {
      const size_t per_sample = sizeof(uint32_t) * ((size_t)n_samples_ + 1);
      ND_HIP_TRY(hipMalloc(&d_ranked_start_, per_sample));
      ND_HIP_TRY(hipMalloc(&d_select_kept_, per_sample));
      ND_HIP_TRY(hipMalloc(&d_select_threshold_, per_sample));
      ND_HIP_TRY(hipMalloc(&d_select_present_, per_sample));
    }
    return 0;
  }

  int sample(int) override {
    if (!allocated_) { last_error = "sample before alloc"; return -1; }
    App app;
    const int n_steps = app.steps();
    const size_t F = (size_t)final_sample_size();
    times = PhaseTimes();
    neighborhood_total_ = 0;
    distinct_total_ = 0;
    chunks_run_ = 0;
    if (!std::is_empty<SampleType>::value) {
      ND_HIP_TRY(hipMemcpyAsync(d_samples_, d_samples_init_, sizeof(SampleType) * (size_t)n_samples_,
                                hipMemcpyDeviceToDevice, stream_));
    }
    ND_HIP_TRY(hipStreamSynchronize(stream_));
    ND_HIP_TRY(hipEventRecord(ev_begin_, stream_));
    const uint32_t S = (uint32_t)n_samples_;
    for (int step = 0; step < n_steps; ++step) {
      TransitView all;
      if (step == 0) {
        all.base = d_initial_;
        all.stride = (uint32_t)init_size_;
        all.count = (uint32_t)init_size_;
      } else {
        all.base = d_final_ + step_size_at_step<App>(step - 2);
        all.stride = (uint32_t)F;
        all.count = (uint32_t)app.stepSize(step - 1);
      }
      // size of every sample's collective neighbourhood, then chunks of samples that fit the budget
      collective_sizes<<<dim3((S + 3) / 4), dim3(256), 0, stream_>>>(dgraph_.view, all, S, invalid_, d_sizes_);
      ND_HIP_TRY(hipMemcpyAsync(h_sizes_.data(), d_sizes_, sizeof(uint32_t) * S, hipMemcpyDeviceToHost, stream_));
      ND_HIP_TRY(hipStreamSynchronize(stream_));
      // chunk limits: entries of concatenation the work arrays hold, or (bitmap form) bitmaps
      // that fit the budget and a grid of marking work items that fits 31 bits
      constexpr bool by_bitmap = apps::neighborhood_form_of<App>::value != apps::kConcatenated;
      const uint64_t entry_budget = by_bitmap ? bitmap_chunk_entries_ : chunk_entries_;
      const uint32_t sample_budget = by_bitmap ? bitmap_chunk_samples_ : S;
      for (uint32_t s = 0; s < S; ++s)
        if (h_sizes_[s] >= (1u << 31)) { last_error = "collective neighbourhood of one sample has 2^31 or more entries"; return -2; }
      uint32_t s0 = 0;
      while (s0 < S) {
        uint64_t total = h_sizes_[s0];
        uint32_t s1 = s0 + 1;
        while (s1 < S && s1 - s0 < sample_budget && total + h_sizes_[s1] <= entry_budget) total += h_sizes_[s1++];
        if (run_chunk(step, all, s0, s1, total) != 0) return -1;
        neighborhood_total_ += total;
        chunks_run_++;
        if (progress_ && chunks_run_ % 16 == 0) {
          ND_HIP_TRY(hipStreamSynchronize(stream_));
          fprintf(stderr, "[nextdoor] layer %d: samples %u of %u done, %llu neighbourhood entries so far\n", step, s1,
                  S, (unsigned long long)neighborhood_total_);
          fflush(stderr);
        }
        s0 = s1;
      }
    }
    ND_HIP_TRY(hipEventRecord(ev_end_, stream_));
    ND_HIP_TRY(hipStreamSynchronize(stream_));
    ND_HIP_TRY(hipEventElapsedTime(&times.end_to_end, ev_begin_, ev_end_));
    return 0;
  }

  int fetch_final_samples() override {
    if (!allocated_) { last_error = "no device data"; return -1; }
    ND_HIP_TRY(hipMemcpy(hFinalSamples.data(), d_final_, sizeof(VertexID_t) * hFinalSamples.size(),
                         hipMemcpyDeviceToHost));
    return 0;
  }

  int fetch_sample_states(void* dst, size_t bytes) override {
    if (!allocated_ || std::is_empty<SampleType>::value) { last_error = "no sample state"; return -1; }
    if (bytes != sample_state_bytes()) { last_error = "sample state size mismatch"; return -1; }
    ND_HIP_TRY(hipMemcpy(dst, d_samples_, bytes, hipMemcpyDeviceToHost));
    return 0;
  }

  int distinct() override {
    last_error = "distinct applies to IndividualNeighborhood results";
    return -2;
  }

  // sizes of the last run, for the algorithmic-bytes figure
  int64_t counter(int which) const override {
    return which == 0 ? (int64_t)neighborhood_total_ : which == 1 ? (int64_t)distinct_total_
           : which == 2 ? (int64_t)chunks_run_ : which == 3 ? (int64_t)dense_pieces_ : 0;
  }

  void free_device() override {
    free_run_buffers();
    release(d_row_sums_);
    release_dense_pieces();
    dgraph_.release();
    graph_ = nullptr;
  }

 private:
  template <class T>
  static void release(T*& p) {
    if (p) (void)hipFree(p);
    p = nullptr;
  }

  // What the vertices with many edges into one stretch contribute to it, built once per graph
  // (see DensePieces).  inverse_row_sums: the LADIES form's 1 / rowsum per vertex, else nullptr.
  int build_dense_pieces(const CSR* graph, const float* inverse_row_sums) {
    release_dense_pieces();
    constexpr bool ladies = apps::neighborhood_form_of<App>::value == apps::kRankedByLadiesImportance;
    uint32_t threshold = ladies ? kDensePieceEntriesSums : kDensePieceEntries;
    if (const char* env = getenv("ND_DENSE_PIECE_ENTRIES")) {  // 0: no pieces; small: to exercise them on small graphs
      const long long v = atoll(env);
      if (v <= 0) return 0;
      threshold = (uint32_t)v;
    }
    constexpr uint32_t stretch_words = ladies ? kBinVerticesSums / 32u : kBinWordsBits;
    constexpr uint32_t stretch = stretch_words * 32u;
    // a piece: a bit per vertex of the stretch, or a 64-bit importance sum (kAbsentSum: no edge)
    constexpr size_t piece_words = ladies ? (size_t)stretch * 2u : (size_t)stretch_words;
    const uint32_t V = (uint32_t)graph->get_n_vertices();
    const uint32_t stretches = (bitmap_words_for(V) + stretch_words - 1) / stretch_words;
    const size_t most_pieces = kDensePieceBudgetBytes / (sizeof(uint32_t) * piece_words);
    std::vector<int32_t> hub_row(V, -1);
    std::vector<uint32_t> piece_of, words;
    size_t n_hubs = 0, n_pieces = 0;
    for (uint32_t v = 0; v < V; ++v) {
      const int32_t* const row = graph->col.data() + graph->row_ptr[v];
      const int32_t* first = row;
      const int32_t* last = graph->col.data() + graph->row_ptr[v + 1];
      if ((size_t)(last - first) < threshold) continue;
      while (first < last) {  // one sub-range of the sorted adjacency per stretch
        const uint32_t b = (uint32_t)*first / stretch;
        const uint32_t limit = (b + 1) * stretch;
        const int32_t* stop = std::partition_point(first, last, [limit](int32_t c) { return (uint32_t)c < limit; });
        if ((size_t)(stop - first) >= threshold && n_pieces < most_pieces) {
          if (hub_row[v] < 0) {
            hub_row[v] = (int32_t)n_hubs++;
            piece_of.resize(n_hubs * stretches, kNoPiece);
          }
          piece_of[(size_t)hub_row[v] * stretches + b] = (uint32_t)n_pieces;
          words.resize((n_pieces + 1) * piece_words, ladies ? 0xFFFFFFFFu : 0u);
          uint32_t* w = words.data() + n_pieces * piece_words;
          for (const int32_t* c = first; c < stop; ++c) {
            const uint32_t local = (uint32_t)*c - b * stretch;
            if (ladies) {
              // the term the marking kernel adds for this edge, in the same arithmetic
              const float p = graph->weight[(size_t)graph->row_ptr[v] + (size_t)(c - row)] * inverse_row_sums[v];
              unsigned long long sum;
              memcpy(&sum, w + 2u * local, sizeof(sum));
              if (sum == kAbsentSum) sum = 0;
              sum += importance_term_fixed(p * p);
              memcpy(w + 2u * local, &sum, sizeof(sum));
            } else {
              w[local >> 5] |= 1u << (local & 31u);
            }
          }
          ++n_pieces;
        }
        first = stop;
      }
    }
    if (n_pieces == 0) return 0;
    ND_HIP_TRY(hipMalloc(&d_hub_row_, sizeof(int32_t) * V));
    ND_HIP_TRY(hipMalloc(&d_piece_of_, sizeof(uint32_t) * piece_of.size()));
    ND_HIP_TRY(hipMalloc(&d_piece_words_, sizeof(uint32_t) * words.size()));
    ND_HIP_TRY(hipMemcpy(d_hub_row_, hub_row.data(), sizeof(int32_t) * V, hipMemcpyHostToDevice));
    ND_HIP_TRY(hipMemcpy(d_piece_of_, piece_of.data(), sizeof(uint32_t) * piece_of.size(), hipMemcpyHostToDevice));
    ND_HIP_TRY(hipMemcpy(d_piece_words_, words.data(), sizeof(uint32_t) * words.size(), hipMemcpyHostToDevice));
    dense_.hub_row = d_hub_row_;
    dense_.piece_of = d_piece_of_;
    dense_.words = d_piece_words_;
    dense_.sums = (const unsigned long long*)d_piece_words_;
    dense_pieces_ = n_pieces;
    return 0;
  }

  void release_dense_pieces() {
    release(d_hub_row_);
    release(d_piece_of_);
    release(d_piece_words_);
    dense_ = DensePieces();
    dense_pieces_ = 0;
  }


  // events around the neighbourhood kernel when profiling is on
  void tick() {
    if (profiling) (void)hipEventRecord(ev_a_, stream_);
  }
  void tock() {
    if (!profiling) return;
    (void)hipEventRecord(ev_b_, stream_);
    (void)hipEventSynchronize(ev_b_);
    float ms = 0;
    (void)hipEventElapsedTime(&ms, ev_a_, ev_b_);
    times.neighborhood += ms;
    times.neighborhood_launches++;
  }

  // One chunk of samples [s0, s1) of one layer: concatenate, post-process in the form the
  // app asks for, run next() for every (sample, nbr).
  int run_chunk(int step, const TransitView& all, uint32_t s0, uint32_t s1, uint64_t total) {
    App app;
    const uint32_t n = s1 - s0;
    const size_t F = (size_t)final_sample_size();
    constexpr int form = apps::neighborhood_form_of<App>::value;
    TransitView tv = all;
    tv.base = all.base + (size_t)s0 * all.stride;
    if (form != apps::kConcatenated) {
      if (build_distinct_by_bitmap(step, s0, tv, n) != 0) return -1;
    } else {
      // work items of the build: long neighbourhoods are spread over several workgroups
      uint64_t n_items = 0;
      for (uint32_t s = s0; s < s1; ++s) {
        const uint64_t items = ((uint64_t)h_sizes_[s] + kBuildItemEntries - 1) / kBuildItemEntries;
        n_items += items ? items : 1;
      }
      if (n_items >= (1ull << 31)) { last_error = "a chunk needs 2^31 or more work items"; return -2; }
      build_item_counts<<<dim3((n + 1 + 255) / 256), dim3(256), 0, stream_>>>(d_sizes_ + s0, n, d_item_count_);
      ND_HIP_TRY(exclusive_scan_u32(d_item_count_, d_item_start_, (size_t)n + 1, d_small_scratch_, stream_));
      if (ensure_neighborhood_capacity((uint32_t)total) != 0) return -1;
      // offsets of the chunk's samples, relative to the chunk (element n = total)
      ND_HIP_TRY(exclusive_scan_u32(d_sizes_ + s0, d_offsets_, (size_t)n + 1, d_small_scratch_, stream_));
      tick();
      collective_build<<<dim3((unsigned)n_items), dim3(256), 0, stream_>>>(
          dgraph_.view, tv, invalid_, d_offsets_, d_item_start_, n, d_nbr_cols_, d_nbr_weights_,
          d_row_offsets_ + (size_t)s0 * all.count);
      tock();
      ND_HIP_TRY(hipGetLastError());
    }

    LayerParams P{};
    P.csr = dgraph_.view;
    P.transits = tv;
    P.step = step;
    P.step_size = (uint32_t)app.stepSize(step);
    P.chunk_samples = n;
    P.sample_begin = s0;
    P.final_size = (uint32_t)F;
    P.out_base = (uint32_t)step_size_at_step<App>(step - 1);
    P.invalid = invalid_;
    P.seed = seed_;
    P.first_sample = 0;
    P.final_samples = d_final_;
    P.samples = d_samples_;
    P.offsets = d_offsets_;
    P.nbr_cols = d_nbr_cols_;
    P.nbr_weights = d_nbr_weights_;
    if (form != apps::kConcatenated) {
      P.ranked_start = d_ranked_start_;
      P.ranked_ids = d_ranked_ids_;
      P.bitmap = d_bitmap_;
      P.words_per_sample = bitmap_words_;
      P.part_before = d_part_before_;
      P.group_through = d_group_through_;
      P.marked = d_marked_;
    }
    const uint64_t outputs = (uint64_t)n * P.step_size;
    layer_execute_kernel<SampleType, App><<<dim3((unsigned)((outputs + 255) / 256)), dim3(256), 0, stream_>>>(P);
    ND_HIP_TRY(hipGetLastError());
    return 0;
  }

  // What next() of the importance forms is handed, for every sample of the chunk.
  int build_distinct_by_bitmap(int step, uint32_t s0, const TransitView& tv, uint32_t n) {
    constexpr bool ladies = apps::neighborhood_form_of<App>::value == apps::kRankedByLadiesImportance;
    constexpr uint32_t bin_words = ladies ? kBinVerticesSums / 32u : kBinWordsBits;
    const uint32_t bins = (bitmap_words_ + bin_words - 1) / bin_words;
    constexpr uint32_t per_group = ladies ? kBinsPerGroupSums : kBinsPerGroupBits;
    const uint32_t groups = (bins + per_group - 1) / per_group;
    if ((uint64_t)n * groups >= (1ull << 31)) { last_error = "a chunk needs 2^31 or more workgroups"; return -1; }
    if constexpr (ladies) {
      return rank_by_keys(step, s0, tv, n, bins, groups);
    } else {
      return list_distinct(tv, n, bins, groups);
    }
  }

  // FastGCN form: mark the vertices of every sample's neighbourhood in its bitmap and add up
  // degree^2 over the marked vertices at two levels (groups of 256 vertices, parts of 64 groups).
  int list_distinct(const TransitView& tv, uint32_t n, uint32_t bins, uint32_t groups) {
    const uint32_t parts_per_sample = bitmap_words_ / kPartWords;
    const size_t n_parts = (size_t)n * parts_per_sample;
    if (n_parts >= (1ull << 32)) { last_error = "a chunk needs 2^32 or more bitmap parts"; return -1; }
    if (n > bitmap_samples_) {
      release(d_bitmap_); release(d_group_through_); release(d_part_total_); release(d_part_before_); release(d_marked_);
      ND_HIP_TRY(hipMalloc(&d_bitmap_, sizeof(uint32_t) * (size_t)n * bitmap_words_));
      ND_HIP_TRY(hipMalloc(&d_group_through_, sizeof(uint64_t) * n_parts * kGroupsPerPart));
      ND_HIP_TRY(hipMalloc(&d_part_total_, sizeof(uint64_t) * n_parts));
      ND_HIP_TRY(hipMalloc(&d_part_before_, sizeof(uint64_t) * (size_t)n * (parts_per_sample + 1)));
      ND_HIP_TRY(hipMalloc(&d_marked_, sizeof(uint32_t) * (size_t)n));
      bitmap_samples_ = n;
    }
    tick();
    collective_mark_binned<false><<<dim3(n * groups), dim3(kBinThreads), 0, stream_>>>(
        dgraph_.view, tv, invalid_, n, bins, d_bitmap_, bitmap_words_, nullptr, 0u, dense_, KeysOnTheWayOut());
    tock();
    ND_HIP_TRY(hipMemsetAsync(d_marked_, 0, sizeof(uint32_t) * (size_t)n, stream_));
    const uint32_t sample_blocks = (n + kSumSamplesPerBlock - 1) / kSumSamplesPerBlock;
    bitmap_group_sums<<<dim3(parts_per_sample * sample_blocks), dim3(kSumThreads), 0, stream_>>>(
        d_bitmap_, bitmap_words_, n, (uint32_t)invalid_, dgraph_.row_ptr(), d_group_through_, d_part_total_, d_marked_);
    sample_part_sums<<<dim3(n), dim3(64), 0, stream_>>>(d_part_total_, parts_per_sample, d_part_before_);
    std::vector<uint32_t> marked(n);
    ND_HIP_TRY(hipMemcpyAsync(marked.data(), d_marked_, sizeof(uint32_t) * n, hipMemcpyDeviceToHost, stream_));
    ND_HIP_TRY(hipStreamSynchronize(stream_));
    for (uint32_t c : marked) distinct_total_ += c;
    return hipGetLastError() == hipSuccess ? 0 : -1;
  }

  // LADIES form: the marking leaves one sampling key per (sample, vertex); per sample, the
  // vertices that can be among its first `wanted` in key order are picked by a radix select on
  // the upper 14 bits of the key and ordered by descending key.  The distinct pairs of a
  // sample (2.4 M per batch at full size) are never listed.
  int rank_by_keys(int step, uint32_t s0, const TransitView& tv, uint32_t n, uint32_t bins, uint32_t groups) {
    const uint32_t keys_per_sample = bins * kBinVerticesSums;
    if (n > bitmap_samples_) {
      release(d_keys_dense_); release(d_stretch_best_);
      ND_HIP_TRY(hipMalloc(&d_keys_dense_, sizeof(uint32_t) * (size_t)n * keys_per_sample));
      ND_HIP_TRY(hipMalloc(&d_stretch_best_, sizeof(uint16_t) * (size_t)n * (keys_per_sample / kCollectStretch)));
      bitmap_samples_ = n;
    }
    KeysOnTheWayOut keys_out;
    keys_out.keys = d_keys_dense_;
    keys_out.seed = seed_;
    keys_out.first_sample = s0;
    keys_out.step = (uint32_t)step;
    keys_out.n_vertices = (uint32_t)invalid_;
    tick();
    collective_mark_binned<true><<<dim3(n * groups), dim3(kBinThreads), 0, stream_>>>(
        dgraph_.view, tv, invalid_, n, bins, nullptr, 0u, d_row_sums_, keys_per_sample, dense_, keys_out);
    tock();
    const uint32_t wanted = (uint32_t)App().stepSize(step);
    select_threshold<<<dim3(n), dim3(kSelectThreads), 0, stream_>>>(d_keys_dense_, keys_per_sample, wanted,
                                                                    d_select_threshold_, d_select_kept_,
                                                                    d_select_present_, d_stretch_best_);
    // where every sample's ranked list starts: exclusive scan of the kept counts
    fill_u32<<<dim3(1), dim3(1), 0, stream_>>>(d_select_kept_ + n, 1, 0u);
    ND_HIP_TRY(exclusive_scan_u32(d_select_kept_, d_ranked_start_, (size_t)n + 1, d_small_scratch_, stream_));
    uint32_t n_kept = 0;
    ND_HIP_TRY(hipMemcpyAsync(&n_kept, d_small_scratch_ + scan_num_tiles((size_t)n + 1), sizeof(uint32_t),
                              hipMemcpyDeviceToHost, stream_));
    std::vector<uint32_t> present(n);
    ND_HIP_TRY(hipMemcpyAsync(present.data(), d_select_present_, sizeof(uint32_t) * n, hipMemcpyDeviceToHost, stream_));
    ND_HIP_TRY(hipStreamSynchronize(stream_));
    for (uint32_t c : present) distinct_total_ += c;
    if (ensure_distinct_capacity(n_kept) != 0) return -1;
    ND_HIP_TRY(hipMemsetAsync(d_select_present_, 0, sizeof(uint32_t) * (size_t)n, stream_));  // now: room claimed
    select_collect<<<dim3(n), dim3(kSelectThreads), 0, stream_>>>(d_keys_dense_, keys_per_sample, d_stretch_best_, d_select_threshold_,
                                                     d_ranked_start_, d_select_present_, d_kept_key_, d_kept_sample_,
                                                     d_kept_id_);
    // order the kept vertices of every sample by descending key, equal keys by ascending
    // vertex id: stable sorts by vertex, then by key, then by sample
    if (n_kept > 0) {
      int chunk_bits = 1;
      while (((uint64_t)n >> chunk_bits) != 0) chunk_bits++;
      const unsigned blocks = (n_kept + 255) / 256;
      const SortPlan by_vertex = make_sort_plan(n_kept, max_bits_);
      uint32_t *k2 = nullptr, *j2 = nullptr;
      ND_HIP_TRY(radix_sort_pairs(by_vertex, (const uint32_t*)d_kept_id_, nullptr, d_keys_a_, d_vals_a_, d_keys_b_,
                                  d_vals_b_, d_hist_, d_scratch_, stream_, &k2, &j2));
      gather_u32<<<dim3(blocks), dim3(256), 0, stream_>>>(d_kept_key_, j2, n_kept, d_key2_, d_index2_);
      const SortPlan by_key = make_sort_plan(n_kept, 32);
      uint32_t *k3 = nullptr, *j3 = nullptr;
      ND_HIP_TRY(radix_sort_pairs(by_key, d_key2_, d_index2_, d_keys_a_, d_vals_a_, d_keys_b_, d_vals_b_, d_hist_,
                                  d_scratch_, stream_, &k3, &j3));
      gather_u32<<<dim3(blocks), dim3(256), 0, stream_>>>(d_kept_sample_, j3, n_kept, d_key2_, d_index2_);
      const SortPlan by_sample = make_sort_plan(n_kept, chunk_bits);
      uint32_t *k4 = nullptr, *j4 = nullptr;
      ND_HIP_TRY(radix_sort_pairs(by_sample, d_key2_, d_index2_, d_keys_a_, d_vals_a_, d_keys_b_, d_vals_b_, d_hist_,
                                  d_scratch_, stream_, &k4, &j4));
      gather_u32<<<dim3(blocks), dim3(256), 0, stream_>>>((const uint32_t*)d_kept_id_, j4, n_kept,
                                                          (uint32_t*)d_ranked_ids_, nullptr);
    }
    return hipGetLastError() == hipSuccess ? 0 : -1;
  }

  // Arrays with one entry per listed (sample, vertex) pair of a chunk: the distinct pairs
  // (FastGCN form) or the pairs the selection keeps (LADIES form).
  int ensure_distinct_capacity(uint32_t n_distinct) {
    if (n_distinct <= distinct_capacity_ && distinct_capacity_ > 0) return 0;
    constexpr int form = apps::neighborhood_form_of<App>::value;
    const size_t cap = (size_t)n_distinct + n_distinct / 8 + 1024;
    release_distinct_buffers();
    if (form == apps::kRankedByLadiesImportance) {
      ND_HIP_TRY(hipMalloc(&d_ranked_ids_, sizeof(int32_t) * cap));
      ND_HIP_TRY(hipMalloc(&d_kept_key_, sizeof(uint32_t) * cap));
      ND_HIP_TRY(hipMalloc(&d_kept_sample_, sizeof(uint32_t) * cap));
      ND_HIP_TRY(hipMalloc(&d_kept_id_, sizeof(int32_t) * cap));
      ND_HIP_TRY(hipMalloc(&d_keys_a_, sizeof(uint32_t) * cap));
      ND_HIP_TRY(hipMalloc(&d_vals_a_, sizeof(uint32_t) * cap));
      ND_HIP_TRY(hipMalloc(&d_keys_b_, sizeof(uint32_t) * cap));
      ND_HIP_TRY(hipMalloc(&d_vals_b_, sizeof(uint32_t) * cap));
      ND_HIP_TRY(hipMalloc(&d_key2_, sizeof(uint32_t) * cap));
      ND_HIP_TRY(hipMalloc(&d_index2_, sizeof(uint32_t) * cap));
      ND_HIP_TRY(hipMalloc(&d_hist_, sizeof(uint32_t) * sort_hist_capacity(cap)));
      size_t scratch = make_sort_plan(cap, 32).scratch_elems;
      ND_HIP_TRY(hipMalloc(&d_scratch_, sizeof(uint32_t) * scratch));
    }
    distinct_capacity_ = cap;
    return 0;
  }

  // The concatenated neighbourhood itself (kConcatenated form).
  int ensure_neighborhood_capacity(uint32_t total) {
    if (total <= capacity_ && capacity_ > 0) return 0;
    const size_t cap = (size_t)total + total / 8 + 1024;
    release(d_nbr_cols_); release(d_nbr_weights_);
    ND_HIP_TRY(hipMalloc(&d_nbr_cols_, sizeof(int32_t) * cap));
    ND_HIP_TRY(hipMalloc(&d_nbr_weights_, sizeof(float) * cap));
    capacity_ = cap;
    return 0;
  }

  void release_distinct_buffers() {
    release(d_ranked_ids_);
    release(d_keys_a_); release(d_vals_a_); release(d_keys_b_); release(d_vals_b_);
    release(d_key2_); release(d_index2_); release(d_hist_); release(d_scratch_);
    release(d_kept_key_); release(d_kept_sample_); release(d_kept_id_);
    distinct_capacity_ = 0;
  }

  void release_neighborhood_buffers() {
    release(d_nbr_cols_); release(d_nbr_weights_);
    release(d_bitmap_); release(d_keys_dense_); release(d_stretch_best_);
    release(d_group_through_); release(d_part_total_); release(d_part_before_); release(d_marked_);
    release_distinct_buffers();
    capacity_ = 0;
    bitmap_samples_ = 0;
  }

  void free_run_buffers() {
    release(d_initial_); release(d_samples_); release(d_samples_init_); release(d_final_);
    release(d_sizes_); release(d_offsets_); release(d_row_offsets_); release(d_small_scratch_);
    release(d_item_count_); release(d_item_start_);
    release(d_ranked_start_); release(d_select_kept_);
    release(d_select_threshold_); release(d_select_present_);
    release_neighborhood_buffers();
    // whatever exists, also after an alloc that failed half way
    for (hipEvent_t* ev : {&ev_a_, &ev_b_, &ev_begin_, &ev_end_}) {
      if (*ev) (void)hipEventDestroy(*ev);
      *ev = nullptr;
    }
    if (stream_) (void)hipStreamDestroy(stream_);
    stream_ = nullptr;
    allocated_ = false;
  }

  const char* name_;
  const CSR* graph_ = nullptr;
  DeviceGraph dgraph_;
  float* d_row_sums_ = nullptr;
  int32_t* d_hub_row_ = nullptr;       // dense pieces of the graph (FastGCN form)
  uint32_t* d_piece_of_ = nullptr;
  uint32_t* d_piece_words_ = nullptr;
  DensePieces dense_;
  size_t dense_pieces_ = 0;
  std::vector<SampleType> samples_;
  std::vector<uint32_t> h_sizes_;
  int64_t n_samples_ = 0;
  int init_size_ = 0;
  int32_t invalid_ = 0;
  int max_bits_ = 0;
  uint64_t seed_ = 0;
  bool allocated_ = false;
  size_t capacity_ = 0;
  uint32_t bitmap_words_ = 0;          // 32-bit words of one sample's presence map (a multiple of kBitmapTileWords)
  uint32_t bitmap_chunk_samples_ = 0;  // samples whose bitmaps fit the budget
  uint64_t bitmap_chunk_entries_ = 0;
  uint32_t bitmap_samples_ = 0;        // samples the allocated bitmaps hold
  size_t distinct_capacity_ = 0;
  uint32_t* d_bitmap_ = nullptr;
  // LADIES form: importance sums and sampling keys, [sample][vertex, padded to whole stretches]
  uint32_t* d_keys_dense_ = nullptr;
  uint16_t* d_stretch_best_ = nullptr;  // LADIES form: best key prefix of every 256 keys of every sample
  uint64_t neighborhood_total_ = 0, distinct_total_ = 0, chunks_run_ = 0;
  uint64_t chunk_entries_ = kLayerChunkEntries;
  bool progress_ = false;

  hipStream_t stream_ = nullptr;
  hipEvent_t ev_begin_ = nullptr, ev_end_ = nullptr, ev_a_ = nullptr, ev_b_ = nullptr;
  VertexID_t* d_initial_ = nullptr;
  SampleType* d_samples_ = nullptr;
  SampleType* d_samples_init_ = nullptr;
  VertexID_t* d_final_ = nullptr;
  uint32_t *d_sizes_ = nullptr, *d_offsets_ = nullptr, *d_row_offsets_ = nullptr, *d_small_scratch_ = nullptr;
  uint32_t *d_item_count_ = nullptr, *d_item_start_ = nullptr;
  // LADIES form: the selection of the best keys per sample
  uint32_t *d_ranked_start_ = nullptr, *d_select_kept_ = nullptr, *d_select_threshold_ = nullptr;
  uint32_t* d_select_present_ = nullptr;  // present[s]: distinct vertices of sample s's neighbourhood
  uint32_t *d_kept_key_ = nullptr, *d_kept_sample_ = nullptr;
  int32_t* d_kept_id_ = nullptr;
  int32_t* d_nbr_cols_ = nullptr;
  float* d_nbr_weights_ = nullptr;
  uint32_t *d_keys_a_ = nullptr, *d_vals_a_ = nullptr, *d_keys_b_ = nullptr, *d_vals_b_ = nullptr;
  uint32_t *d_key2_ = nullptr, *d_index2_ = nullptr, *d_hist_ = nullptr, *d_scratch_ = nullptr;
  // FastGCN form: degree^2 of the marked vertices, by group inside a part, by part, by sample
  uint64_t *d_group_through_ = nullptr, *d_part_total_ = nullptr, *d_part_before_ = nullptr;
  uint32_t* d_marked_ = nullptr;
  int32_t* d_ranked_ids_ = nullptr;
};

}  // namespace nd
