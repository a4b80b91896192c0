// Unique transits of the sorted (transit, slot) map and their extents.
//
// Where the reference trims the INVALID tail (invalidVertexStartPos,
// src/nextdoor.cu:1804-1836), run-length encodes the sorted transits
// (cub::DeviceRunLengthEncode::Encode, 2535-2545) and exclusive-sums the counts into
// start positions (cub::DeviceScan::ExclusiveSum, 2560-2567) with three blocking
// device->host copies in between, this does the same in three launches whose sizes are
// known on the host up front; every count the later kernels need stays in device memory.
//
// A building block with an entry point and tests of its own (nd_unique_transits): the engine's
// pass does not launch it.  The step loop needs no list of the unique transits - it finds each
// run's extent at the run's last pair and classifies it there (classify_run_tails in
// nd_engine.hpp); only RunsMeta below is shared with it.
//
// A run head is a position i with key[i] != INVALID and (i == 0 or key[i] != key[i-1]).
// run r = the r-th head: run_key[r], run_start[r]; run_start[n_runs] = n_valid, so the
// count of run r is run_start[r+1] - run_start[r] (the exclusive scan of the counts is
// run_start itself).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "nd_device_scan.hpp"

namespace nd {

// Device-resident per-step bookkeeping.  Written by compact_run_heads, consumed by the
// load-balancing kernels; never read by the host inside the step loop.
struct RunsMeta {
  uint32_t n_valid;    // pairs whose transit is a real vertex (sorted prefix length)
  uint32_t n_runs;     // unique transits in that prefix
  uint32_t n_chunks;   // work items emitted for the workgroup kernel
  uint32_t n_big_pairs;  // pairs covered by those work items
  uint32_t stamp;      // load-balanced steps: the value that marks the transits taken by work items at
                       // this step (see classify_run_tails in nd_engine.hpp); never 0
};

__device__ __forceinline__ bool is_run_head(const uint32_t* keys, size_t i, uint32_t invalid) {
  const uint32_t k = keys[i];
  return k != invalid && (i == 0 || keys[i - 1] != k);
}

__global__ __launch_bounds__(kScanThreads) void count_run_heads(const uint32_t* __restrict__ keys, size_t n,
                                                                uint32_t invalid, uint32_t* __restrict__ tile_counts) {
  __shared__ uint32_t s_wave[kScanThreads / kWave];
  const size_t base = (size_t)blockIdx.x * kScanTile;
  uint32_t heads = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    const size_t idx = base + (size_t)i * kScanThreads + threadIdx.x;
    if (idx < n && is_run_head(keys, idx, invalid)) heads++;
  }
  uint32_t total;
  block_exclusive_scan_256(heads, s_wave, &total);
  if (threadIdx.x == 0) tile_counts[blockIdx.x] = total;
}

// tile_offsets: exclusive scan of tile_counts, with the grand total at [num_tiles].
__global__ __launch_bounds__(kScanThreads) void compact_run_heads(const uint32_t* __restrict__ keys, size_t n,
                                                                  uint32_t invalid,
                                                                  const uint32_t* __restrict__ tile_offsets,
                                                                  uint32_t num_tiles, uint32_t* __restrict__ run_key,
                                                                  uint32_t* __restrict__ run_start,
                                                                  RunsMeta* __restrict__ meta) {
  __shared__ uint32_t s_wave[kScanThreads / kWave];
  const size_t base = (size_t)blockIdx.x * kScanTile + (size_t)threadIdx.x * kScanItems;
  const uint32_t total_runs = tile_offsets[num_tiles];
  bool head[kScanItems];
  uint32_t mine = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    const size_t idx = base + i;
    head[i] = idx < n && is_run_head(keys, idx, invalid);
    mine += head[i] ? 1u : 0u;
    if (idx < n) {
      // the single position that closes the valid prefix publishes the totals
      const uint32_t k = keys[idx];
      const bool last_valid = k != invalid && (idx + 1 == n || keys[idx + 1] == invalid);
      const bool nothing_valid = idx == 0 && k == invalid;
      if (last_valid || nothing_valid) {
        const uint32_t n_valid = nothing_valid ? 0u : (uint32_t)(idx + 1);
        meta->n_valid = n_valid;
        meta->n_runs = total_runs;
        meta->n_chunks = 0;
        meta->n_big_pairs = 0;
        run_start[total_runs] = n_valid;
      }
    }
  }
  uint32_t total;
  uint32_t r = block_exclusive_scan_256(mine, s_wave, &total) + tile_offsets[blockIdx.x];
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    if (head[i]) {
      run_key[r] = keys[base + i];
      run_start[r] = (uint32_t)(base + i);
      ++r;
    }
  }
}

// Scratch (uint32 elements) for find_transit_runs over n sorted pairs.
inline size_t runs_scratch_elems(size_t n) { return scan_num_tiles(n) + 1; }

// run_key needs n elements, run_start n + 1.
inline hipError_t find_transit_runs(const uint32_t* sorted_keys, size_t n, uint32_t invalid, uint32_t* run_key,
                                    uint32_t* run_start, RunsMeta* meta, uint32_t* scratch, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  const size_t tiles = scan_num_tiles(n);
  count_run_heads<<<dim3((unsigned)tiles), dim3(kScanThreads), 0, stream>>>(sorted_keys, n, invalid, scratch);
  scan_of_totals<<<dim3(1), dim3(kScanThreads), 0, stream>>>(scratch, tiles);
  compact_run_heads<<<dim3((unsigned)tiles), dim3(kScanThreads), 0, stream>>>(sorted_keys, n, invalid, scratch,
                                                                             (uint32_t)tiles, run_key, run_start, meta);
  return hipGetLastError();
}

}  // namespace nd
