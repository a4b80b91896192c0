// Device-wide exclusive prefix sum over uint32 (gfx950, wave64).
//
// Stands where the reference calls cub::DeviceScan::ExclusiveSum
// (src/nextdoor.cu:2560-2567) and is also the offset pass of the radix sort.
// Three launches, no spinning: tile totals -> scan of the totals by one workgroup ->
// rescan of each tile with its offset added.  All sizes are read on the host.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nd {

constexpr int kWave = 64;
constexpr int kScanThreads = 256;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanThreads * kScanItems;  // 2048 elements per workgroup

__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
  const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    uint32_t up = __shfl_up(v, d, kWave);
    if (lane >= d) v += up;
  }
  return v;
}

// Exclusive scan of one value per thread across a 256-thread workgroup.
// s_wave_totals must hold one uint32 per wavefront of the workgroup (kThreads / 64; 4 for the
// 256-thread form).  Returns the exclusive prefix; *block_total gets
// the sum over the workgroup.  Contains two barriers.
template <int kThreads>
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* s_wave_totals, uint32_t* block_total) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const uint32_t incl = wave_inclusive_scan(v);
  if (lane == kWave - 1) s_wave_totals[wave] = incl;
  __syncthreads();
  uint32_t before = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kThreads / kWave; ++w) {
    const uint32_t t = s_wave_totals[w];
    if (w < wave) before += t;
    total += t;
  }
  __syncthreads();
  *block_total = total;
  return before + incl - v;
}

__device__ __forceinline__ uint32_t block_exclusive_scan_256(uint32_t v, uint32_t* s_wave_totals,
                                                             uint32_t* block_total) {
  return block_exclusive_scan<kScanThreads>(v, s_wave_totals, block_total);
}

__global__ __launch_bounds__(kScanThreads) void scan_tile_totals(const uint32_t* __restrict__ in, size_t n,
                                                                 uint32_t* __restrict__ tile_totals) {
  __shared__ uint32_t s_wave[kScanThreads / kWave];
  const size_t base = (size_t)blockIdx.x * kScanTile;
  uint32_t sum = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    const size_t idx = base + (size_t)i * kScanThreads + threadIdx.x;
    if (idx < n) sum += in[idx];
  }
  uint32_t total;
  block_exclusive_scan_256(sum, s_wave, &total);
  if (threadIdx.x == 0) tile_totals[blockIdx.x] = total;
}

// One workgroup scans the tile totals in place (exclusive) and stores the grand
// total after the last entry: tile_totals[num_tiles] = sum of everything.
__global__ __launch_bounds__(kScanThreads) void scan_of_totals(uint32_t* __restrict__ tile_totals, size_t num_tiles) {
  __shared__ uint32_t s_wave[kScanThreads / kWave];
  uint32_t carry = 0;
  for (size_t start = 0; start < num_tiles; start += kScanThreads) {
    const size_t idx = start + threadIdx.x;
    const uint32_t v = idx < num_tiles ? tile_totals[idx] : 0u;
    uint32_t total;
    const uint32_t excl = block_exclusive_scan_256(v, s_wave, &total);
    if (idx < num_tiles) tile_totals[idx] = carry + excl;
    carry += total;
  }
  if (threadIdx.x == 0) tile_totals[num_tiles] = carry;
}

__global__ __launch_bounds__(kScanThreads) void scan_apply(const uint32_t* __restrict__ in, uint32_t* __restrict__ out,
                                                           size_t n, const uint32_t* __restrict__ tile_offsets) {
  __shared__ uint32_t s_wave[kScanThreads / kWave];
  // blocked arrangement: thread t owns kScanItems consecutive elements
  const size_t base = (size_t)blockIdx.x * kScanTile + (size_t)threadIdx.x * kScanItems;
  uint32_t v[kScanItems];
  uint32_t sum = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    v[i] = base + i < n ? in[base + i] : 0u;
    sum += v[i];
  }
  uint32_t total;
  uint32_t running = block_exclusive_scan_256(sum, s_wave, &total) + tile_offsets[blockIdx.x];
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    if (base + i < n) out[base + i] = running;
    running += v[i];
  }
}

// ---- 64-bit inclusive prefix sum (same three-launch scheme) ----

__device__ __forceinline__ uint64_t wave_inclusive_scan_u64(uint64_t v) {
  const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const uint32_t lo = __shfl_up((uint32_t)v, d, kWave);
    const uint32_t hi = __shfl_up((uint32_t)(v >> 32), d, kWave);
    if (lane >= d) v += ((uint64_t)hi << 32) | lo;
  }
  return v;
}

// Exclusive scan of one uint64 per thread across a 256-thread workgroup (two barriers).
__device__ __forceinline__ uint64_t block_exclusive_scan_256_u64(uint64_t v, uint64_t* s_wave_totals,
                                                                 uint64_t* block_total) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const uint64_t incl = wave_inclusive_scan_u64(v);
  if (lane == kWave - 1) s_wave_totals[wave] = incl;
  __syncthreads();
  uint64_t before = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kScanThreads / kWave; ++w) {
    const uint64_t t = s_wave_totals[w];
    if (w < wave) before += t;
    total += t;
  }
  __syncthreads();
  *block_total = total;
  return before + incl - v;
}

// The input of the 64-bit scan is a functor, so that values can be computed on the way in
// (e.g. degree^2 of a listed vertex) instead of being stored first.
struct LoadU64 {
  const uint64_t* p;
  __device__ __forceinline__ uint64_t operator()(size_t i) const { return p[i]; }
};

template <class Load>
__global__ __launch_bounds__(kScanThreads) void scan64_tile_totals(Load in, size_t n,
                                                                   uint64_t* __restrict__ tile_totals) {
  __shared__ uint64_t s_wave[kScanThreads / kWave];
  const size_t base = (size_t)blockIdx.x * kScanTile;
  uint64_t sum = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    const size_t idx = base + (size_t)i * kScanThreads + threadIdx.x;
    if (idx < n) sum += in(idx);
  }
  uint64_t total;
  block_exclusive_scan_256_u64(sum, s_wave, &total);
  if (threadIdx.x == 0) tile_totals[blockIdx.x] = total;
}

// One workgroup; a thread takes kTotalsPerThread consecutive totals per round.
constexpr int kTotalsPerThread = 16;
__global__ __launch_bounds__(kScanThreads) void scan64_of_totals(uint64_t* __restrict__ tile_totals, size_t num_tiles) {
  __shared__ uint64_t s_wave[kScanThreads / kWave];
  uint64_t carry = 0;
  for (size_t start = 0; start < num_tiles; start += (size_t)kScanThreads * kTotalsPerThread) {
    const size_t first = start + (size_t)threadIdx.x * kTotalsPerThread;
    uint64_t v[kTotalsPerThread];
    uint64_t sum = 0;
#pragma unroll
    for (int i = 0; i < kTotalsPerThread; ++i) {
      v[i] = first + i < num_tiles ? tile_totals[first + i] : 0ull;
      sum += v[i];
    }
    uint64_t total;
    uint64_t running = carry + block_exclusive_scan_256_u64(sum, s_wave, &total);
#pragma unroll
    for (int i = 0; i < kTotalsPerThread; ++i) {
      if (first + i < num_tiles) tile_totals[first + i] = running;
      running += v[i];
    }
    carry += total;
  }
  if (threadIdx.x == 0) tile_totals[num_tiles] = carry;
}

template <class Load>
__global__ __launch_bounds__(kScanThreads) void scan64_apply_inclusive(Load in, uint64_t* __restrict__ out, size_t n,
                                                                       const uint64_t* __restrict__ tile_offsets) {
  __shared__ uint64_t s_wave[kScanThreads / kWave];
  const size_t base = (size_t)blockIdx.x * kScanTile + (size_t)threadIdx.x * kScanItems;
  uint64_t v[kScanItems];
  uint64_t sum = 0;
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    v[i] = base + i < n ? in(base + i) : 0ull;
    sum += v[i];
  }
  uint64_t total;
  uint64_t running = block_exclusive_scan_256_u64(sum, s_wave, &total) + tile_offsets[blockIdx.x];
#pragma unroll
  for (int i = 0; i < kScanItems; ++i) {
    running += v[i];
    if (base + i < n) out[base + i] = running;
  }
}

inline size_t scan_num_tiles(size_t n) { return (n + kScanTile - 1) / kScanTile; }

// out[i] = in(0) + ... + in(i).  scratch needs scan_num_tiles(n) + 1 uint64.
template <class Load>
inline hipError_t inclusive_scan_u64_of(Load in, uint64_t* out, size_t n, uint64_t* scratch, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  const size_t tiles = (n + kScanTile - 1) / kScanTile;
  scan64_tile_totals<Load><<<dim3((unsigned)tiles), dim3(kScanThreads), 0, stream>>>(in, n, scratch);
  scan64_of_totals<<<dim3(1), dim3(kScanThreads), 0, stream>>>(scratch, tiles);
  scan64_apply_inclusive<Load><<<dim3((unsigned)tiles), dim3(kScanThreads), 0, stream>>>(in, out, n, scratch);
  return hipGetLastError();
}

// out[i] = sum of in[0..i]; in and out may alias.
inline hipError_t inclusive_scan_u64(const uint64_t* in, uint64_t* out, size_t n, uint64_t* scratch,
                                     hipStream_t stream) {
  return inclusive_scan_u64_of(LoadU64{in}, out, n, scratch, stream);
}

// Scratch needed by exclusive_scan_u32 for n elements, in uint32 units.
inline size_t scan_scratch_elems(size_t n) { return scan_num_tiles(n) + 1; }

// out[i] = sum of in[0..i); in and out may alias.  scratch[num_tiles] receives the
// grand total.  Returns the hipGetLastError() of the launches.
inline hipError_t exclusive_scan_u32(const uint32_t* in, uint32_t* out, size_t n, uint32_t* scratch,
                                     hipStream_t stream) {
  if (n == 0) return hipSuccess;
  const size_t tiles = scan_num_tiles(n);
  scan_tile_totals<<<dim3((unsigned)tiles), dim3(kScanThreads), 0, stream>>>(in, n, scratch);
  scan_of_totals<<<dim3(1), dim3(kScanThreads), 0, stream>>>(scratch, tiles);
  scan_apply<<<dim3((unsigned)tiles), dim3(kScanThreads), 0, stream>>>(in, out, n, scratch);
  return hipGetLastError();
}

}  // namespace nd
