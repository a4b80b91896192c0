// Per-sample distinct of k-hop results (GraphSAGE "sample with replacement, then distinct").
//
// For every sample and every hop segment of its result row: the ascending unique valid
// vertex ids packed to the left, the rest of the segment INVALID, and the number kept.
// The reference's k-hop app does not deduplicate; its only code for this is the unused
// per-root sort -> flag -> scan -> compact of src/distinct.cuh:1-111, whose behaviour
// (sort with a padding value above every vertex id, keep first of each run) this follows.
//
// One wavefront per segment of up to 256 ids: the segment sits in registers (1, 2 or 4 ids
// per lane), is sorted by a bitonic network whose cross-lane exchanges are wave shuffles,
// first-of-run flags become positions through wave ballots, and the packed ids are written
// back.  Longer segments (up to 4096 ids) use one workgroup and an LDS bitonic sort.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nd {

constexpr int32_t kDistinctPad = 0x7FFFFFFF;  // above INVALID (= |V|) and every vertex id

// kRegs ids per lane; element i of the segment is register i / 64 of lane i % 64.
template <int kRegs>
__global__ __launch_bounds__(256) void distinct_wave_kernel(int32_t* __restrict__ final_samples,
                                                            int32_t* __restrict__ counts, uint32_t n_samples,
                                                            uint32_t final_size, uint32_t seg_base, uint32_t seg_len,
                                                            int32_t invalid, uint32_t n_steps, uint32_t step) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t sample = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (sample >= n_samples) return;  // whole wave leaves together
  int32_t* seg = final_samples + (size_t)sample * final_size + seg_base;
  constexpr uint32_t kN = 64u * kRegs;

  int32_t v[kRegs];
#pragma unroll
  for (int r = 0; r < kRegs; ++r) {
    const uint32_t i = r * 64u + lane;
    v[r] = i < seg_len ? seg[i] : kDistinctPad;
  }

  // bitonic sort, ascending over i = r * 64 + lane
#pragma unroll
  for (uint32_t k = 2; k <= kN; k <<= 1) {
#pragma unroll
    for (uint32_t j = k >> 1; j > 0; j >>= 1) {
      if (j >= 64u) {
        const int dr = (int)(j >> 6);
#pragma unroll
        for (int r = 0; r < kRegs; ++r) {
          if ((r & dr) == 0) {
            const uint32_t i = r * 64u + lane;
            const bool ascending = (i & k) == 0;
            const int32_t a = v[r], b = v[r | dr];
            const bool swap = ascending ? a > b : a < b;
            v[r] = swap ? b : a;
            v[r | dr] = swap ? a : b;
          }
        }
      } else {
#pragma unroll
        for (int r = 0; r < kRegs; ++r) {
          const uint32_t i = r * 64u + lane;
          const int32_t other = __shfl_xor(v[r], (int)j, 64);
          const bool ascending = (i & k) == 0;
          const bool lower = (lane & j) == 0;  // this lane holds the lower index of the pair
          const bool take_min = ascending == lower;
          v[r] = take_min ? (v[r] < other ? v[r] : other) : (v[r] > other ? v[r] : other);
        }
      }
    }
  }

  // first of each run of equal valid ids
  const uint64_t lanes_below = (1ull << lane) - 1ull;
  uint32_t kept_before = 0;
#pragma unroll
  for (int r = 0; r < kRegs; ++r) {
    int32_t prev = __shfl_up(v[r], 1, 64);
    if (lane == 0) prev = -1;
    if (r > 0) {
      const int32_t carry = __shfl(v[r - 1], 63, 64);
      if (lane == 0) prev = carry;
    }
    const bool keep = v[r] < invalid && v[r] != prev;
    const uint64_t mask = __ballot(keep);
    if (keep) seg[kept_before + (uint32_t)__popcll(mask & lanes_below)] = v[r];
    kept_before += (uint32_t)__popcll(mask);
  }
  for (uint32_t i = kept_before + lane; i < seg_len; i += 64u) seg[i] = invalid;
  if (lane == 0) counts[(size_t)sample * n_steps + step] = (int32_t)kept_before;
}

// One workgroup per segment of up to 4096 ids, sorted in LDS.
__global__ __launch_bounds__(256) void distinct_workgroup_kernel(int32_t* __restrict__ final_samples,
                                                                 int32_t* __restrict__ counts, uint32_t final_size,
                                                                 uint32_t seg_base, uint32_t seg_len, uint32_t padded_len,
                                                                 int32_t invalid, uint32_t n_steps, uint32_t step) {
  __shared__ int32_t s_ids[4096];
  __shared__ uint32_t s_wave_kept[4];
  __shared__ uint32_t s_running;
  int32_t* seg = final_samples + (size_t)blockIdx.x * final_size + seg_base;
  for (uint32_t i = threadIdx.x; i < padded_len; i += 256) s_ids[i] = i < seg_len ? seg[i] : kDistinctPad;
  if (threadIdx.x == 0) s_running = 0;
  __syncthreads();
  for (uint32_t k = 2; k <= padded_len; k <<= 1) {
    for (uint32_t j = k >> 1; j > 0; j >>= 1) {
      for (uint32_t i = threadIdx.x; i < padded_len; i += 256) {
        const uint32_t partner = i ^ j;
        if (partner > i) {
          const int32_t a = s_ids[i], b = s_ids[partner];
          const bool ascending = (i & k) == 0;
          if (ascending ? a > b : a < b) {
            s_ids[i] = b;
            s_ids[partner] = a;
          }
        }
      }
      __syncthreads();
    }
  }
  // compact in chunks of 256 sorted ids
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  for (uint32_t chunk = 0; chunk < padded_len; chunk += 256) {
    const uint32_t i = chunk + threadIdx.x;
    const int32_t x = i < padded_len ? s_ids[i] : kDistinctPad;
    const int32_t prev = i == 0 ? -1 : s_ids[i - 1];
    const bool keep = i < padded_len && x < invalid && x != prev;
    const uint64_t mask = __ballot(keep);
    if (lane == 0) s_wave_kept[wave] = (uint32_t)__popcll(mask);
    __syncthreads();
    uint32_t before = s_running;
    for (uint32_t w = 0; w < wave; ++w) before += s_wave_kept[w];
    if (keep) seg[before + (uint32_t)__popcll(mask & ((1ull << lane) - 1ull))] = x;
    __syncthreads();
    if (threadIdx.x == 0) s_running += s_wave_kept[0] + s_wave_kept[1] + s_wave_kept[2] + s_wave_kept[3];
    __syncthreads();
  }
  const uint32_t kept = s_running;
  for (uint32_t i = kept + threadIdx.x; i < seg_len; i += 256) seg[i] = invalid;
  if (threadIdx.x == 0) counts[(size_t)blockIdx.x * n_steps + step] = (int32_t)kept;
}

constexpr uint32_t kDistinctMaxSegment = 4096;

// Launches the distinct pass of one step segment.  Returns false when the segment is too long.
inline bool launch_distinct_segment(int32_t* final_samples, int32_t* counts, uint32_t n_samples, uint32_t final_size,
                                    uint32_t seg_base, uint32_t seg_len, int32_t invalid, uint32_t n_steps,
                                    uint32_t step, hipStream_t stream) {
  const dim3 wave_grid((n_samples + 3) / 4), block(256);
  if (seg_len <= 64) {
    distinct_wave_kernel<1><<<wave_grid, block, 0, stream>>>(final_samples, counts, n_samples, final_size, seg_base,
                                                             seg_len, invalid, n_steps, step);
  } else if (seg_len <= 128) {
    distinct_wave_kernel<2><<<wave_grid, block, 0, stream>>>(final_samples, counts, n_samples, final_size, seg_base,
                                                             seg_len, invalid, n_steps, step);
  } else if (seg_len <= 256) {
    distinct_wave_kernel<4><<<wave_grid, block, 0, stream>>>(final_samples, counts, n_samples, final_size, seg_base,
                                                             seg_len, invalid, n_steps, step);
  } else if (seg_len <= kDistinctMaxSegment) {
    uint32_t padded = 512;
    while (padded < seg_len) padded <<= 1;
    distinct_workgroup_kernel<<<dim3(n_samples), block, 0, stream>>>(final_samples, counts, final_size, seg_base,
                                                                     seg_len, padded, invalid, n_steps, step);
  } else {
    return false;
  }
  return true;
}

}  // namespace nd
