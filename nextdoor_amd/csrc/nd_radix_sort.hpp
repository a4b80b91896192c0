// Sample -> transit inversion: stable LSD radix sort of (transit vertex, slot) pairs.
//
// Takes the place of cub::DeviceRadixSort::SortPairs in the reference's step loop
// (src/nextdoor.cu:2924-2939; key width maxBits from 1993-1999): keys are transit vertex
// ids in [0, V] (V = INVALID_VERTEX sorts last), only the low `key_bits` bits are sorted.
// The value is the SLOT of the pair in the unsorted map (sample * transitsPerSample + j),
// not the sample id, so the step kernels can place outputs without atomics; on the first
// pass the values are generated from the index instead of being read.
//
// Per 8-bit digit pass: (1) per-tile digit histogram into a digit-major table, (2) one
// workgroup per digit turns its row into exclusive prefixes over tiles and leaves the row
// total, (3) scatter (every workgroup scans the 256 row totals itself).  The scatter ranks keys inside a tile with
// wave64 ballots (match-any on the digit), keeps one running counter per wave and digit in
// LDS, stages the tile digit-sorted in LDS and writes runs of equal digits to HBM.
// No spinning, no inter-workgroup waiting.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "nd_device_scan.hpp"

namespace nd {

constexpr int kSortThreads = 256;
constexpr int kSortWaves = kSortThreads / kWave;
// Keys per lane and tile: 10 (2560 pairs per workgroup) for sorts that are latency bound,
// 32 (8192 pairs) for large ones, where fewer, larger tiles keep the digit table small.
// Measured: inversion of a 100-step pass over 4.2 M walks 12.3 ms with 16, 11.5 ms with 8,
// 14.7 ms with 4; sorts of ~1e8 entries are 12 % slower with 8 than with 16.  Again, after the
// kernels had their loads batched: 13.96 / 11.50 / 10.80 / 10.24 / 10.62 ms with 4 / 6 / 8 / 10 / 12.
#ifndef ND_SORT_ITEMS_SMALL
#define ND_SORT_ITEMS_SMALL 10
#endif
constexpr int kSortItemsSmall = ND_SORT_ITEMS_SMALL;
// (5.2e7 pairs of the k-hop pass, three digit passes, with 12 / 16 / 20 / 24 / 28 / 32 keys per lane of the
// histogram kernel: 0.85 / 0.83 / 0.83 / 0.81 / 0.81 / 0.80 ms)
#ifndef ND_SORT_ITEMS_LARGE
#define ND_SORT_ITEMS_LARGE 32
#endif
constexpr int kSortItemsLarge = ND_SORT_ITEMS_LARGE;
constexpr size_t kSortLargeFrom = (size_t)16 << 20;  // pairs
constexpr int kSortMaxTile = kSortThreads * kSortItemsLarge;
constexpr int kRadixBits = 8;
constexpr int kRadix = 1 << kRadixBits;
constexpr uint32_t kPadKey = 0xFFFFFFFFu;  // never a real key: keys are <= V < 2^31

// Element `it` of lane `lane` in wave `wave` sits at this offset inside the tile: each
// wave owns a contiguous chunk and reads it 64 keys (256 B) at a time, so the order
// (wave, it, lane) is the input order and one running counter per wave keeps it stable.
template <int kSortItems>
__device__ __forceinline__ int tile_offset(int wave, int it, int lane) {
  return wave * (kWave * kSortItems) + it * kWave + lane;
}

// Where key i of the input sits: keys[i], or, when the keys are segments of rows of a wider
// table (seg_len keys at the start of every row of `pitch` words), keys[(i / seg_len) * pitch
// + i % seg_len].  Only the first pass of a sort reads such an input.
struct KeyLayout {
  uint32_t seg_len = 0;  // 0: contiguous
  uint32_t pitch = 0;
  uint64_t magic = 0;    // floor(2^64 / seg_len) + 1 (2^64 / seg_len for a power of two): i / seg_len is the
                         // upper half of i * magic for every i below 2^32, without a division per key
  void rows(uint32_t segment, uint32_t row_pitch) {
    seg_len = segment;
    pitch = row_pitch;
    magic = segment ? ~0ull / segment + 1ull : 0ull;
  }
  __host__ __device__ size_t at(size_t i) const {
    if (seg_len == 0) return i;
    if (seg_len == 1) return i * (size_t)pitch;  // (no 64-bit magic for 1)
#if defined(__HIP_DEVICE_COMPILE__)
    const uint64_t row = __umul64hi((uint64_t)i, magic);  // i < 2^32: the sorts take at most 2^32 - 1 keys
#else
    const uint64_t row = i / seg_len;
#endif
    return row * (size_t)pitch + (i - row * seg_len);
  }
};

// n_dev (nullable): element count kept in device memory; overrides n when given.
// drop_key: keys equal to it are left out of the sort (kPadKey: nothing is left out).
// (A workgroup counting four consecutive tiles, so that a digit's four counts leave as one 16-byte
// store instead of four pieces of four lines: 0.86 -> 0.85 ms of inversion on 5.2e7 pairs; not kept.)
template <int kSortItems>
__global__ __launch_bounds__(kSortThreads) void radix_histogram(const uint32_t* __restrict__ keys, size_t n,
                                                                const uint32_t* __restrict__ n_dev, int shift,
                                                                uint32_t mask, uint32_t drop_key,
                                                                uint32_t* __restrict__ hist, uint32_t num_tiles,
                                                                KeyLayout layout) {
  constexpr int kSortTile = kSortThreads * kSortItems;
  __shared__ uint32_t s_hist[kRadix];
  s_hist[threadIdx.x] = 0;
  __syncthreads();
  if (n_dev) n = *n_dev;
  const size_t tile_start = (size_t)blockIdx.x * kSortTile;
  // all of a lane's keys are fetched before the first is counted: with the count inside the
  // loop every key waited for the one before it (eight memory round trips one after the other)
  uint32_t mine[kSortItems];
#pragma unroll
  for (int it = 0; it < kSortItems; ++it) {
    const size_t idx = tile_start + (size_t)it * kSortThreads + threadIdx.x;
    mine[it] = idx < n ? keys[layout.at(idx)] : drop_key;
  }
#pragma unroll
  for (int it = 0; it < kSortItems; ++it) {
    const size_t idx = tile_start + (size_t)it * kSortThreads + threadIdx.x;
    if (idx < n && mine[it] != drop_key) atomicAdd(&s_hist[(mine[it] >> shift) & mask], 1u);
  }
  __syncthreads();
  if (threadIdx.x <= mask) hist[(size_t)threadIdx.x * num_tiles + blockIdx.x] = s_hist[threadIdx.x];
}

// One workgroup per digit: exclusive scan of the digit's row of the table (over tiles) in
// place, and the row total.  The row is taken in stretches of kSortThreads * kHeld counts: a
// thread holds kHeld consecutive counts of a stretch in registers (their loads are all under
// way at once, and the sweep that writes the prefixes reads nothing), the workgroup scans the
// threads' sums, and the stretch's total is carried to the next stretch.
__global__ __launch_bounds__(kSortThreads) void radix_row_scan(uint32_t* __restrict__ hist, uint32_t num_tiles,
                                                               uint32_t* __restrict__ row_totals) {
  __shared__ uint32_t s_scan_tmp[kSortWaves];
  uint32_t* row = hist + (size_t)blockIdx.x * num_tiles;
  constexpr uint32_t kHeld = 8;
  uint32_t carry = 0;
  for (uint32_t stretch = 0; stretch < num_tiles; stretch += kSortThreads * kHeld) {
    // a short row is spread over all threads rather than packed into the first few
    const uint32_t left = num_tiles - stretch;
    const uint32_t per_thread = left >= kSortThreads * kHeld ? kHeld : (left + kSortThreads - 1) / kSortThreads;
    const uint32_t begin = stretch + threadIdx.x * per_thread;
    uint32_t held[kHeld];
    uint32_t sum = 0;
#pragma unroll
    for (uint32_t k = 0; k < kHeld; ++k) held[k] = k < per_thread && begin + k < num_tiles ? row[begin + k] : 0u;
#pragma unroll
    for (uint32_t k = 0; k < kHeld; ++k) sum += held[k];
    uint32_t total;
    uint32_t running = carry + block_exclusive_scan_256(sum, s_scan_tmp, &total);
#pragma unroll
    for (uint32_t k = 0; k < kHeld; ++k) {
      if (k < per_thread && begin + k < num_tiles) row[begin + k] = running;
      running += held[k];
    }
    carry += total;
  }
  if (threadIdx.x == 0) row_totals[blockIdx.x] = carry;
}

// aux_in / aux_out (kAux): a second 32-bit payload that travels with the pair.  It goes
// through the LDS staging area of the values in a second round, after the keys and values
// of the tile have been written, so that the workgroup needs no more LDS than without it (with a
// staging area of its own and one round: inversion of the 4.2 M-walk pass 9.4 -> 10.5 ms).
// kSortItems is the keys per lane of the histogram's 256-lane workgroups; this kernel runs the
// same tile with kScatterThreads lanes, each taking kSortItems * 256 / kScatterThreads keys: the
// ranking of a lane's keys is a chain of ballots per key, one key after the other, and with
// twice the lanes the chain is half as long.  Inversion of the 100-step pass over 4.2 M walks: 256
// lanes 10.2 ms, 512 lanes 9.4 ms (with tiles of 2048 / 3072 keys: 11.0 / 9.7), 1024 lanes 10.8-11.8.
#ifndef ND_SCATTER_THREADS
#define ND_SCATTER_THREADS 512
#endif
constexpr int kScatterThreads = ND_SCATTER_THREADS;
constexpr int kScatterWaves = kScatterThreads / kWave;

template <int kSortItems, bool kIotaValues, bool kAux>
__global__ __launch_bounds__(kScatterThreads) void radix_scatter(const uint32_t* __restrict__ keys_in,
                                                                 const uint32_t* __restrict__ vals_in,
                                                                 const uint32_t* __restrict__ aux_in,
                                                                 uint32_t* __restrict__ keys_out,
                                                                 uint32_t* __restrict__ vals_out,
                                                                 uint32_t* __restrict__ aux_out, size_t n,
                                                                 const uint32_t* __restrict__ n_dev, int shift,
                                                                 uint32_t mask, int digit_bits, uint32_t drop_key,
                                                                 const uint32_t* __restrict__ scanned_hist,
                                                                 const uint32_t* __restrict__ row_totals,
                                                                 uint32_t num_tiles, uint32_t* __restrict__ kept_out,
                                                                 KeyLayout layout) {
  constexpr int kSortTile = kSortThreads * kSortItems;
  static_assert(kSortTile % kScatterThreads == 0, "the tile is a whole number of keys per lane");
  constexpr int kItems = kSortTile / kScatterThreads;  // keys per lane here
  __shared__ uint32_t s_keys[kSortTile];
  __shared__ uint32_t s_vals[kSortTile];
  __shared__ uint32_t s_wave_count[kScatterWaves][kRadix];
  __shared__ uint32_t s_digit_base[kRadix];
  __shared__ uint32_t s_global_base[kRadix];
  __shared__ uint32_t s_scan_tmp[kScatterWaves];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const bool digit_lane = tid < kRadix;  // lanes that own a digit in the per-digit steps
  if (n_dev) n = *n_dev;
  const size_t tile_start = (size_t)blockIdx.x * kSortTile;
  if (tile_start >= n && !(kept_out && blockIdx.x == 0)) return;
  // first position of every digit in the output: exclusive scan of the row totals
  uint32_t kept_total;
  const uint32_t digit_first = block_exclusive_scan<kScatterThreads>(
      digit_lane && (uint32_t)tid <= mask ? row_totals[tid] : 0u, s_scan_tmp, &kept_total);
  // number of keys the whole sort keeps; published once
  if (kept_out && blockIdx.x == 0 && tid == 0) kept_out[0] = kept_total;
  if (tile_start >= n) return;
  const uint32_t in_tile = (uint32_t)((n - tile_start) < (size_t)kSortTile ? (n - tile_start) : (size_t)kSortTile);
  // where the tile's keys of a digit go among all keys of that digit: fetched now, with the keys,
  // not after the ranking, where it would be one more round trip
  const uint32_t before_tile = digit_lane && (uint32_t)tid <= mask ? scanned_hist[(size_t)tid * num_tiles + blockIdx.x] : 0u;

  if (digit_lane) {
#pragma unroll
    for (int w = 0; w < kScatterWaves; ++w) s_wave_count[w][tid] = 0;
  }
  __syncthreads();

  uint32_t key[kItems], val[kItems], rank[kItems], aux[kAux ? kItems : 1];
  bool live[kItems];
#pragma unroll
  for (int it = 0; it < kItems; ++it) {
    const uint32_t off = (uint32_t)tile_offset<kItems>(wave, it, lane);
    const bool inside = off < in_tile;
    key[it] = inside ? keys_in[layout.at(tile_start + off)] : kPadKey;
    live[it] = inside && key[it] != drop_key;
    if (kIotaValues) val[it] = (uint32_t)(tile_start + off);
    else val[it] = inside ? vals_in[tile_start + off] : 0u;
    if (kAux) aux[it] = inside ? aux_in[tile_start + off] : 0u;  // fetched with the pair: no second round trip
  }

  const uint64_t lanes_below = (1ull << lane) - 1ull;
#pragma unroll
  for (int it = 0; it < kItems; ++it) {
    const uint32_t digit = (key[it] >> shift) & mask;
    // peers = live lanes of this wave holding the same digit
    uint64_t peers = __ballot(live[it]);
    for (int b = 0; b < digit_bits; ++b) {
      const bool bit = (digit >> b) & 1u;
      const uint64_t vote = __ballot(bit);
      peers &= bit ? vote : ~vote;
    }
    uint32_t before = 0;
    const int leader = peers ? __ffsll((unsigned long long)peers) - 1 : 0;
    if (live[it] && lane == leader) before = atomicAdd(&s_wave_count[wave][digit], (uint32_t)__popcll(peers));
    before = __shfl(before, leader, kWave);
    rank[it] = before + (uint32_t)__popcll(peers & lanes_below);
  }
  __syncthreads();

  // per digit: turn the per-wave counts into exclusive prefixes over waves, then scan
  // the tile totals over digits.
  uint32_t digit_total = 0;
  if (digit_lane) {
#pragma unroll
    for (int w = 0; w < kScatterWaves; ++w) {
      const uint32_t c = s_wave_count[w][tid];
      s_wave_count[w][tid] = digit_total;
      digit_total += c;
    }
  }
  uint32_t live_in_tile;
  const uint32_t digit_base = block_exclusive_scan<kScatterThreads>(digit_total, s_scan_tmp, &live_in_tile);
  if (digit_lane) {
    s_digit_base[tid] = digit_base;
    if ((uint32_t)tid <= mask)
      s_global_base[tid] = digit_first + before_tile - digit_base;
  }
  __syncthreads();

#pragma unroll
  for (int it = 0; it < kItems; ++it) {
    if (live[it]) {
      const uint32_t digit = (key[it] >> shift) & mask;
      const uint32_t pos = s_digit_base[digit] + s_wave_count[wave][digit] + rank[it];
      rank[it] = pos;  // position inside the digit-sorted tile
      s_keys[pos] = key[it];
      s_vals[pos] = val[it];
    }
  }
  __syncthreads();

  for (uint32_t p = tid; p < live_in_tile; p += kScatterThreads) {
    const uint32_t k = s_keys[p];
    const uint32_t out = s_global_base[(k >> shift) & mask] + p;
    keys_out[out] = k;
    vals_out[out] = s_vals[p];
  }
  if (kAux) {
    __syncthreads();
#pragma unroll
    for (int it = 0; it < kItems; ++it) {
      if (live[it]) s_vals[rank[it]] = aux[it];
    }
    __syncthreads();
    for (uint32_t p = tid; p < live_in_tile; p += kScatterThreads) {
      const uint32_t out = s_global_base[(s_keys[p] >> shift) & mask] + p;
      aux_out[out] = s_vals[p];
    }
  }
}

struct SortPlan {
  size_t n = 0;
  int key_bits = 0;
  int passes = 0;
  int items = kSortItemsSmall;  // keys per lane: tile = kSortThreads * items
  uint32_t num_tiles = 0;
  size_t hist_elems = 0;     // kRadix * num_tiles
  size_t scratch_elems = 0;  // digit row totals
};

inline SortPlan make_sort_plan(size_t n, int key_bits) {
  SortPlan p;
  p.n = n;
  // key_bits == 0: one pass in which every key has digit 0, i.e. a stable compaction of the
  // pairs the sort keeps (see SortJob::drop_key)
  p.key_bits = key_bits < 0 ? 0 : key_bits;
  p.passes = p.key_bits == 0 ? 1 : (p.key_bits + kRadixBits - 1) / kRadixBits;
  p.items = n >= kSortLargeFrom ? kSortItemsLarge : kSortItemsSmall;
  const size_t tile = (size_t)kSortThreads * p.items;
  p.num_tiles = (uint32_t)((n + tile - 1) / tile);
  p.hist_elems = (size_t)kRadix * p.num_tiles;
  p.scratch_elems = kRadix;  // row totals
  return p;
}

// Digit-table size (uint32) that serves every sort of at most n_max pairs: the tile size
// depends on the size of the sort, so a buffer kept across sorts of different sizes is
// sized for the smaller tile.
inline size_t sort_hist_capacity(size_t n_max) {
  const size_t tile = (size_t)kSortThreads * kSortItemsSmall;
  return (size_t)kRadix * ((n_max + tile - 1) / tile + 1);
}

// Everything one sort works with.  keys_in is not modified.  vals_in == nullptr means
// "value = index".  Two ping-pong buffer sets (a, b) of plan.n elements each; the result
// lands in keys_sorted / vals_sorted / aux_sorted (one of a / b).  hist needs plan.hist_elems
// and scratch plan.scratch_elems uint32.
//   aux_in (nullable): a second payload per pair, with aux_a / aux_b as its ping-pong buffers.
//   n_in_dev (nullable): the number of input pairs, in device memory (at most plan.n).
//   drop_key / kept_dev: pairs whose key equals drop_key are left out by the first pass and
//   the number of pairs kept is stored in kept_dev[0] (device memory, not the same word as
//   n_in_dev); later passes and the caller's kernels read the count from there, no host round
//   trip.  kPadKey and nullptr sort everything.
struct SortJob {
  const uint32_t* keys_in = nullptr;
  const uint32_t* vals_in = nullptr;
  const uint32_t* aux_in = nullptr;
  uint32_t *keys_a = nullptr, *vals_a = nullptr, *aux_a = nullptr;
  uint32_t *keys_b = nullptr, *vals_b = nullptr, *aux_b = nullptr;
  uint32_t* hist = nullptr;
  uint32_t* scratch = nullptr;
  const uint32_t* n_in_dev = nullptr;
  KeyLayout keys_in_layout;  // how keys_in is laid out (values are then the key's index i)
  uint32_t drop_key = kPadKey;
  uint32_t* kept_dev = nullptr;
  // results
  uint32_t *keys_sorted = nullptr, *vals_sorted = nullptr, *aux_sorted = nullptr;
};

// The three launches of one digit pass.
template <int kSortItems>
inline void sort_pass(const SortPlan& plan, const SortJob& job, const uint32_t* src_k, const uint32_t* src_v,
                      const uint32_t* src_x, uint32_t* dst_k, uint32_t* dst_v, uint32_t* dst_x, const uint32_t* n_dev,
                      int shift, uint32_t mask, int bits, uint32_t drop, uint32_t* kept_out, KeyLayout layout,
                      hipStream_t stream) {
  const dim3 grid(plan.num_tiles), block(kSortThreads);
  radix_histogram<kSortItems><<<grid, block, 0, stream>>>(src_k, plan.n, n_dev, shift, mask, drop, job.hist,
                                                          plan.num_tiles, layout);
  radix_row_scan<<<dim3(mask + 1), block, 0, stream>>>(job.hist, plan.num_tiles, job.scratch);
  const dim3 scatter_block(kScatterThreads);
  if (src_v == nullptr)
    radix_scatter<kSortItems, true, false><<<grid, scatter_block, 0, stream>>>(src_k, nullptr, nullptr, dst_k, dst_v, nullptr,
                                                                       plan.n, n_dev, shift, mask, bits, drop, job.hist,
                                                                       job.scratch, plan.num_tiles, kept_out, layout);
  else if (src_x == nullptr)
    radix_scatter<kSortItems, false, false><<<grid, scatter_block, 0, stream>>>(src_k, src_v, nullptr, dst_k, dst_v, nullptr,
                                                                        plan.n, n_dev, shift, mask, bits, drop,
                                                                        job.hist, job.scratch, plan.num_tiles, kept_out, layout);
  else
    radix_scatter<kSortItems, false, true><<<grid, scatter_block, 0, stream>>>(src_k, src_v, src_x, dst_k, dst_v, dst_x, plan.n,
                                                                       n_dev, shift, mask, bits, drop, job.hist,
                                                                       job.scratch, plan.num_tiles, kept_out, layout);
}

inline hipError_t radix_sort(const SortPlan& plan, SortJob& job, hipStream_t stream) {
  job.keys_sorted = job.keys_a;
  job.vals_sorted = job.vals_a;
  job.aux_sorted = job.aux_a;
  if (plan.n == 0) return hipSuccess;
  const bool aux = job.aux_in != nullptr;
  if (aux && job.vals_in == nullptr) return hipErrorInvalidValue;  // generated values carry no second payload
  // digits as even as possible: 23 bits -> 8, 8, 7
  const uint32_t* src_k = job.keys_in;
  const uint32_t* src_v = job.vals_in;
  const uint32_t* src_x = job.aux_in;
  uint32_t* dst_k = job.keys_a;
  uint32_t* dst_v = job.vals_a;
  uint32_t* dst_x = job.aux_a;
  int shift = 0;
  for (int pass = 0; pass < plan.passes; ++pass) {
    const int remaining = plan.key_bits - shift;
    const int passes_left = plan.passes - pass;
    const int bits = (remaining + passes_left - 1) / passes_left;
    const uint32_t mask = (1u << bits) - 1u;
    const uint32_t* n_dev = pass > 0 ? job.kept_dev : job.n_in_dev;
    const uint32_t drop = pass == 0 ? job.drop_key : kPadKey;
    uint32_t* kept_out = pass == 0 ? job.kept_dev : nullptr;
    const KeyLayout layout = pass == 0 ? job.keys_in_layout : KeyLayout();
    if (plan.items == kSortItemsLarge)
      sort_pass<kSortItemsLarge>(plan, job, src_k, src_v, src_x, dst_k, dst_v, dst_x, n_dev, shift, mask, bits, drop,
                                 kept_out, layout, stream);
    else
      sort_pass<kSortItemsSmall>(plan, job, src_k, src_v, src_x, dst_k, dst_v, dst_x, n_dev, shift, mask, bits, drop,
                                 kept_out, layout, stream);
    job.keys_sorted = dst_k;
    job.vals_sorted = dst_v;
    job.aux_sorted = dst_x;
    src_k = dst_k;
    src_v = dst_v;
    src_x = dst_x;
    if (dst_k == job.keys_a) { dst_k = job.keys_b; dst_v = job.vals_b; dst_x = job.aux_b; }
    else { dst_k = job.keys_a; dst_v = job.vals_a; dst_x = job.aux_a; }
    shift += bits;
  }
  return hipGetLastError();
}

// The common case: (key, value) pairs, no second payload, input count known on the host.
inline hipError_t radix_sort_pairs(const SortPlan& plan, const uint32_t* keys_in, const uint32_t* vals_in,
                                   uint32_t* keys_a, uint32_t* vals_a, uint32_t* keys_b, uint32_t* vals_b,
                                   uint32_t* hist, uint32_t* scratch, hipStream_t stream,
                                   uint32_t** keys_sorted, uint32_t** vals_sorted, uint32_t drop_key = kPadKey,
                                   uint32_t* kept_dev = nullptr) {
  SortJob job;
  job.keys_in = keys_in;
  job.vals_in = vals_in;
  job.keys_a = keys_a;
  job.vals_a = vals_a;
  job.keys_b = keys_b;
  job.vals_b = vals_b;
  job.hist = hist;
  job.scratch = scratch;
  job.drop_key = drop_key;
  job.kept_dev = kept_dev;
  const hipError_t e = radix_sort(plan, job, stream);
  *keys_sorted = job.keys_sorted;
  *vals_sorted = job.vals_sorted;
  return e;
}

}  // namespace nd
