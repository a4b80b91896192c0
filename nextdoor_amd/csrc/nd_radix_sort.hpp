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
constexpr int kSortItems = 16;
constexpr int kSortTile = kSortThreads * kSortItems;  // 4096 pairs per workgroup
constexpr int kRadixBits = 8;
constexpr int kRadix = 1 << kRadixBits;
constexpr uint32_t kPadKey = 0xFFFFFFFFu;  // never a real key: keys are <= V < 2^31

// Element `it` of lane `lane` in wave `wave` sits at this offset inside the tile: each
// wave owns a contiguous chunk and reads it 64 keys (256 B) at a time, so the order
// (wave, it, lane) is the input order and one running counter per wave keeps it stable.
__device__ __forceinline__ int tile_offset(int wave, int it, int lane) {
  return wave * (kWave * kSortItems) + it * kWave + lane;
}

// n_dev (nullable): element count kept in device memory; overrides n when given.
// drop_key: keys equal to it are left out of the sort (kPadKey: nothing is left out).
__global__ __launch_bounds__(kSortThreads) void radix_histogram(const uint32_t* __restrict__ keys, size_t n,
                                                                const uint32_t* __restrict__ n_dev, int shift,
                                                                uint32_t mask, uint32_t drop_key,
                                                                uint32_t* __restrict__ hist, uint32_t num_tiles) {
  __shared__ uint32_t s_hist[kRadix];
  s_hist[threadIdx.x] = 0;
  __syncthreads();
  if (n_dev) n = *n_dev;
  const size_t tile_start = (size_t)blockIdx.x * kSortTile;
#pragma unroll
  for (int it = 0; it < kSortItems; ++it) {
    const size_t idx = tile_start + (size_t)it * kSortThreads + threadIdx.x;
    if (idx < n) {
      const uint32_t k = keys[idx];
      if (k != drop_key) atomicAdd(&s_hist[(k >> shift) & mask], 1u);
    }
  }
  __syncthreads();
  if (threadIdx.x <= mask) hist[(size_t)threadIdx.x * num_tiles + blockIdx.x] = s_hist[threadIdx.x];
}

// One workgroup per digit: exclusive scan of the digit's row of the table (over tiles) in
// place, and the row total.
__global__ __launch_bounds__(kSortThreads) void radix_row_scan(uint32_t* __restrict__ hist, uint32_t num_tiles,
                                                               uint32_t* __restrict__ row_totals) {
  __shared__ uint32_t s_scan_tmp[kSortWaves];
  uint32_t* row = hist + (size_t)blockIdx.x * num_tiles;
  // thread t owns a contiguous stretch of the row
  const uint32_t per_thread = (num_tiles + kSortThreads - 1) / kSortThreads;
  const uint32_t begin = threadIdx.x * per_thread;
  const uint32_t end = begin + per_thread < num_tiles ? begin + per_thread : num_tiles;
  uint32_t sum = 0;
  for (uint32_t i = begin; i < end; ++i) sum += row[i];
  uint32_t total;
  uint32_t running = block_exclusive_scan_256(sum, s_scan_tmp, &total);
  for (uint32_t i = begin; i < end; ++i) {
    const uint32_t c = row[i];
    row[i] = running;
    running += c;
  }
  if (threadIdx.x == 0) row_totals[blockIdx.x] = total;
}

template <bool kIotaValues>
__global__ __launch_bounds__(kSortThreads) void radix_scatter(const uint32_t* __restrict__ keys_in,
                                                              const uint32_t* __restrict__ vals_in,
                                                              uint32_t* __restrict__ keys_out,
                                                              uint32_t* __restrict__ vals_out, size_t n,
                                                              const uint32_t* __restrict__ n_dev, int shift,
                                                              uint32_t mask, int digit_bits, uint32_t drop_key,
                                                              const uint32_t* __restrict__ scanned_hist,
                                                              const uint32_t* __restrict__ row_totals,
                                                              uint32_t num_tiles, uint32_t* __restrict__ kept_out) {
  __shared__ uint32_t s_keys[kSortTile];
  __shared__ uint32_t s_vals[kSortTile];
  __shared__ uint32_t s_wave_count[kSortWaves][kRadix];
  __shared__ uint32_t s_digit_base[kRadix];
  __shared__ uint32_t s_global_base[kRadix];
  __shared__ uint32_t s_scan_tmp[kSortWaves];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  if (n_dev) n = *n_dev;
  const size_t tile_start = (size_t)blockIdx.x * kSortTile;
  if (tile_start >= n && !(kept_out && blockIdx.x == 0)) return;
  // first position of every digit in the output: exclusive scan of the row totals
  uint32_t kept_total;
  const uint32_t digit_first = block_exclusive_scan_256((uint32_t)tid <= mask ? row_totals[tid] : 0u, s_scan_tmp,
                                                        &kept_total);
  // number of keys the whole sort keeps; published once
  if (kept_out && blockIdx.x == 0 && tid == 0) kept_out[0] = kept_total;
  if (tile_start >= n) return;
  const uint32_t in_tile = (uint32_t)((n - tile_start) < (size_t)kSortTile ? (n - tile_start) : (size_t)kSortTile);

#pragma unroll
  for (int w = 0; w < kSortWaves; ++w) s_wave_count[w][tid] = 0;
  __syncthreads();

  uint32_t key[kSortItems], val[kSortItems], rank[kSortItems];
  bool live[kSortItems];
#pragma unroll
  for (int it = 0; it < kSortItems; ++it) {
    const uint32_t off = (uint32_t)tile_offset(wave, it, lane);
    const bool inside = off < in_tile;
    key[it] = inside ? keys_in[tile_start + off] : kPadKey;
    live[it] = inside && key[it] != drop_key;
    if (kIotaValues) val[it] = (uint32_t)(tile_start + off);
    else val[it] = inside ? vals_in[tile_start + off] : 0u;
  }

  const uint64_t lanes_below = (1ull << lane) - 1ull;
#pragma unroll
  for (int it = 0; it < kSortItems; ++it) {
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
#pragma unroll
  for (int w = 0; w < kSortWaves; ++w) {
    const uint32_t c = s_wave_count[w][tid];
    s_wave_count[w][tid] = digit_total;
    digit_total += c;
  }
  uint32_t live_in_tile;
  const uint32_t digit_base = block_exclusive_scan_256(digit_total, s_scan_tmp, &live_in_tile);
  s_digit_base[tid] = digit_base;
  if ((uint32_t)tid <= mask)
    s_global_base[tid] = digit_first + scanned_hist[(size_t)tid * num_tiles + blockIdx.x] - digit_base;
  __syncthreads();

#pragma unroll
  for (int it = 0; it < kSortItems; ++it) {
    if (live[it]) {
      const uint32_t digit = (key[it] >> shift) & mask;
      const uint32_t pos = s_digit_base[digit] + s_wave_count[wave][digit] + rank[it];
      s_keys[pos] = key[it];
      s_vals[pos] = val[it];
    }
  }
  __syncthreads();

  for (uint32_t p = tid; p < live_in_tile; p += kSortThreads) {
    const uint32_t k = s_keys[p];
    const uint32_t out = s_global_base[(k >> shift) & mask] + p;
    keys_out[out] = k;
    vals_out[out] = s_vals[p];
  }
}

struct SortPlan {
  size_t n = 0;
  int key_bits = 0;
  int passes = 0;
  uint32_t num_tiles = 0;
  size_t hist_elems = 0;     // kRadix * num_tiles
  size_t scratch_elems = 0;  // digit row totals
};

inline SortPlan make_sort_plan(size_t n, int key_bits) {
  SortPlan p;
  p.n = n;
  p.key_bits = key_bits < 1 ? 1 : key_bits;
  p.passes = (p.key_bits + kRadixBits - 1) / kRadixBits;
  p.num_tiles = (uint32_t)((n + kSortTile - 1) / kSortTile);
  p.hist_elems = (size_t)kRadix * p.num_tiles;
  p.scratch_elems = kRadix;  // row totals
  return p;
}

// Sorts n pairs by the low key_bits bits of the key.  keys_in is not modified.
// vals_in == nullptr means "value = index".  Two ping-pong buffer pairs (a, b) of n
// elements each; the result lands in *keys_sorted / *vals_sorted (one of a / b).
// hist needs plan.hist_elems and scratch plan.scratch_elems uint32.
// drop_key / kept_dev: pairs whose key equals drop_key are left out by the first pass and
// the number of pairs kept is stored in kept_dev[0] (device memory); later passes and the
// caller's kernels read the count from there, no host round trip.  Pass kPadKey and
// nullptr to sort everything.
inline hipError_t radix_sort_pairs(const SortPlan& plan, const uint32_t* keys_in, const uint32_t* vals_in,
                                   uint32_t* keys_a, uint32_t* vals_a, uint32_t* keys_b, uint32_t* vals_b,
                                   uint32_t* hist, uint32_t* scratch, hipStream_t stream,
                                   uint32_t** keys_sorted, uint32_t** vals_sorted, uint32_t drop_key = kPadKey,
                                   uint32_t* kept_dev = nullptr) {
  *keys_sorted = keys_a;
  *vals_sorted = vals_a;
  if (plan.n == 0) return hipSuccess;
  // digits as even as possible: 23 bits -> 8, 8, 7
  const uint32_t* src_k = keys_in;
  const uint32_t* src_v = vals_in;
  uint32_t* dst_k = keys_a;
  uint32_t* dst_v = vals_a;
  int shift = 0;
  for (int pass = 0; pass < plan.passes; ++pass) {
    const int remaining = plan.key_bits - shift;
    const int passes_left = plan.passes - pass;
    const int bits = (remaining + passes_left - 1) / passes_left;
    const uint32_t mask = (1u << bits) - 1u;
    const uint32_t* n_dev = pass > 0 ? kept_dev : nullptr;
    const uint32_t drop = pass == 0 ? drop_key : kPadKey;
    radix_histogram<<<dim3(plan.num_tiles), dim3(kSortThreads), 0, stream>>>(src_k, plan.n, n_dev, shift, mask, drop,
                                                                            hist, plan.num_tiles);
    radix_row_scan<<<dim3(mask + 1), dim3(kSortThreads), 0, stream>>>(hist, plan.num_tiles, scratch);
    uint32_t* kept_out = pass == 0 ? kept_dev : nullptr;
    if (pass == 0 && src_v == nullptr)
      radix_scatter<true><<<dim3(plan.num_tiles), dim3(kSortThreads), 0, stream>>>(
          src_k, nullptr, dst_k, dst_v, plan.n, n_dev, shift, mask, bits, drop, hist, scratch, plan.num_tiles, kept_out);
    else
      radix_scatter<false><<<dim3(plan.num_tiles), dim3(kSortThreads), 0, stream>>>(
          src_k, src_v, dst_k, dst_v, plan.n, n_dev, shift, mask, bits, drop, hist, scratch, plan.num_tiles, kept_out);
    *keys_sorted = dst_k;
    *vals_sorted = dst_v;
    src_k = dst_k;
    src_v = dst_v;
    if (dst_k == keys_a) { dst_k = keys_b; dst_v = vals_b; }
    else { dst_k = keys_a; dst_v = vals_a; }
    shift += bits;
  }
  return hipGetLastError();
}

}  // namespace nd
