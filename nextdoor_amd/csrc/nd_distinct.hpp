// Per-sample distinct of k-hop results (GraphSAGE "sample with replacement, then distinct").
//
// For every sample and every hop segment of its result row: the ascending unique valid
// vertex ids packed to the left, the rest of the segment INVALID, and the number kept.
// The reference's k-hop app does not deduplicate; its only code for this is the unused
// per-root sort -> flag -> scan -> compact of src/distinct.cuh:1-111, whose behaviour
// (sort with a padding value above every vertex id, keep first of each run) this follows.
//
// One wavefront per segment of up to 256 ids: the segment sits in registers (1, 2 or 4 ids
// per lane), is sorted by a bitonic network, first-of-run flags become positions through wave
// ballots, and the packed ids are written back.  Longer segments (up to 4096 ids) use one
// workgroup and an LDS bitonic sort.
//
// The network is the one whose comparators all point the same way: a merge of blocks of k
// starts by comparing element i with its mirror image i ^ (k - 1) and goes on with
// i ^ (k / 4), ..., i ^ 1, the lower index always keeping the smaller id.  Position i of the
// network is register i % kRegs of lane i / kRegs, so the strides below kRegs (15 of the 36
// stages at 256 ids) are a min and a max between two registers of a lane, and the others
// exchange whole registers between lanes lane ^ m: for m = 1, 2, 3, 7, 15 that is one DPP
// move (quad permutations, half-row and row mirrors), for m = 4 and 8 two of them (row shifts
// under bank masks), and only m = 16, 31, 63 (three stages) go through the LDS crossbar.  The
// exchange itself is one median-of-three per register.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nd {

constexpr int32_t kDistinctPad = 0x7FFFFFFF;  // above INVALID (= |V|) and every vertex id

// x of lane (lane ^ m); m is a constant wherever this is called (fully unrolled loops)
__device__ __forceinline__ int32_t value_of_lane_xor(int32_t x, uint32_t m) {
  switch (m) {
    // every lane has a source lane in these, so nothing of the destination's old content survives
    case 1: return __builtin_amdgcn_mov_dpp(x, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
    case 2: return __builtin_amdgcn_mov_dpp(x, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
    case 3: return __builtin_amdgcn_mov_dpp(x, 0x1B, 0xF, 0xF, true);   // quad_perm [3,2,1,0]
    case 7: return __builtin_amdgcn_mov_dpp(x, 0x141, 0xF, 0xF, true);  // row_half_mirror
    case 15: return __builtin_amdgcn_mov_dpp(x, 0x140, 0xF, 0xF, true); // row_mirror
    case 4: {  // banks (groups of four lanes) 0 and 2 of a row read four lanes up, banks 1 and 3 four lanes down
      const int32_t up = __builtin_amdgcn_mov_dpp(x, 0x104, 0xF, 0xF, true);          // row_shl:4, all banks
      return __builtin_amdgcn_update_dpp(up, x, 0x114, 0xF, 0xA, false);              // row_shr:4 into banks 1, 3
    }
    case 8: {
      const int32_t up = __builtin_amdgcn_mov_dpp(x, 0x108, 0xF, 0xF, true);          // row_shl:8, all banks
      return __builtin_amdgcn_update_dpp(up, x, 0x118, 0xF, 0xC, false);              // row_shr:8 into banks 2, 3
    }
    default: return __shfl_xor(x, (int)m, 64);
  }
}

// One stage of the network over positions i = lane * kRegs + r: partner of i is i ^ mask.
template <int kRegs>
__device__ __forceinline__ void network_stage(int32_t (&v)[kRegs], uint32_t lane, uint32_t mask) {
  const uint32_t reg_mask = mask & (uint32_t)(kRegs - 1);
  const uint32_t lane_mask = mask / (uint32_t)kRegs;
  if (lane_mask == 0) {
#pragma unroll
    for (int r = 0; r < kRegs; ++r) {
      const int q = r ^ (int)reg_mask;
      if (r < q) {
        const int32_t lo = v[r] < v[q] ? v[r] : v[q];
        const int32_t hi = v[r] < v[q] ? v[q] : v[r];
        v[r] = lo;
        v[q] = hi;
      }
    }
  } else {
    uint32_t top = lane_mask;  // highest bit of lane_mask: the lane without it holds the lower position
    top |= top >> 1; top |= top >> 2; top |= top >> 4;
    top = (top + 1) >> 1;
    // the lower position keeps min(mine, other) = median(mine, other, lowest int), the upper one
    // max(mine, other) = median(mine, other, highest int): one instruction for both kinds of lane
    const int32_t limit = (lane & top) != 0 ? 0x7FFFFFFF : (int32_t)0x80000000;
    int32_t other[kRegs];
#pragma unroll
    for (int r = 0; r < kRegs; ++r) other[r] = value_of_lane_xor(v[r ^ (int)reg_mask], lane_mask);
#pragma unroll
    for (int r = 0; r < kRegs; ++r) asm("v_med3_i32 %0, %1, %2, %3" : "=v"(v[r]) : "v"(v[r]), "v"(other[r]), "v"(limit));
  }
}

// One hop segment of one sample by one wavefront, kRegs ids per lane: sorts, keeps the first of
// each run of equal vertices, writes them back packed and returns how many.
template <int kRegs>
__device__ __forceinline__ uint32_t distinct_segment_in_wave(int32_t* __restrict__ seg, uint32_t seg_len,
                                                             int32_t invalid, uint32_t lane, int32_t* pack) {
  constexpr uint32_t kN = 64u * kRegs;
  // which id starts at which position of the network does not matter: load them coalesced
  int32_t v[kRegs];
  bool any_vertex = false;
#pragma unroll
  for (int r = 0; r < kRegs; ++r) {
    const uint32_t i = r * 64u + lane;
    v[r] = i < seg_len ? seg[i] : kDistinctPad;
    any_vertex = any_vertex || v[r] < invalid;
  }
  if (__ballot(any_vertex) == 0) return 0;  // nothing sampled here (a dead transit): all INVALID already

#pragma unroll
  for (uint32_t k = 2; k <= kN; k <<= 1) {
    network_stage<kRegs>(v, lane, k - 1);
#pragma unroll
    for (uint32_t j = k >> 2; j > 0; j >>= 1) network_stage<kRegs>(v, lane, j);
  }

  // first of each run of equal valid ids; position i = lane * kRegs + r is ascending
  int32_t before_mine = __builtin_amdgcn_update_dpp(-1, v[kRegs - 1], 0x138, 0xF, 0xF, false);  // wave_shr:1
  if (lane == 0) before_mine = -1;
  const uint64_t lanes_below = (1ull << lane) - 1ull;
  bool keep[kRegs];
  uint32_t kept_before = 0, kept_total = 0;
#pragma unroll
  for (int r = 0; r < kRegs; ++r) {
    keep[r] = v[r] < invalid && v[r] != (r == 0 ? before_mine : v[r - 1]);
    const uint64_t mask = __ballot(keep[r]);
    kept_before += (uint32_t)__popcll(mask & lanes_below);
    kept_total += (uint32_t)__popcll(mask);
  }
  // packed through the wavefront's piece of LDS, so that the stores to memory are whole lines:
  // a lane's kept ids are every kRegs-th position of the packed order
#pragma unroll
  for (int r = 0; r < kRegs; ++r) {
    if (keep[r]) pack[kept_before] = v[r];
    kept_before += keep[r] ? 1u : 0u;
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int r = 0; r < kRegs; ++r) {
    const uint32_t i = r * 64u + lane;
    if (i < seg_len) seg[i] = i < kept_total ? pack[i] : invalid;
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");  // the next segment packs into the same piece
  __builtin_amdgcn_wave_barrier();
  return kept_total;
}

// One wavefront per sample and segment.
template <int kRegs>
__global__ __launch_bounds__(256) void distinct_wave_kernel(int32_t* __restrict__ final_samples,
                                                            int32_t* __restrict__ counts, uint32_t n_samples,
                                                            uint32_t final_size, uint32_t seg_base, uint32_t seg_len,
                                                            int32_t invalid, uint32_t n_steps, uint32_t step) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t sample = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (sample >= n_samples) return;  // whole wave leaves together
  __shared__ int32_t s_pack[4][64 * kRegs];
  int32_t* seg = final_samples + (size_t)sample * final_size + seg_base;
  const uint32_t kept = distinct_segment_in_wave<kRegs>(seg, seg_len, invalid, lane, s_pack[threadIdx.x >> 6]);
  if (lane == 0) counts[(size_t)sample * n_steps + step] = (int32_t)kept;
}

// The hop segments of a result row, none longer than 256 ids.
constexpr int kDistinctRowSegments = 8;
struct RowSegments {
  uint32_t n;
  uint32_t base[kDistinctRowSegments];
  uint32_t len[kDistinctRowSegments];
};

// One wavefront per sample takes the segments of its row one after the other: the row is read
// as the one contiguous piece it is.  chained != 0: every hop's transits are the previous hop's
// vertices, so a row whose first hop found nothing holds nothing later either and is left after
// that look, its counts written as 0.
__global__ __launch_bounds__(256) void distinct_rows_kernel(int32_t* __restrict__ final_samples,
                                                            int32_t* __restrict__ counts, uint32_t n_samples,
                                                            uint32_t final_size, RowSegments segments, int32_t invalid,
                                                            uint32_t chained) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t sample = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (sample >= n_samples) return;  // whole wave leaves together
  __shared__ int32_t s_pack[4][256];
  int32_t* pack = s_pack[threadIdx.x >> 6];
  int32_t* row = final_samples + (size_t)sample * final_size;
  uint32_t kept_mine = 0;  // lane s keeps the count of segment s
  for (uint32_t s = 0; s < segments.n; ++s) {
    const uint32_t len = segments.len[s];
    int32_t* seg = row + segments.base[s];
    uint32_t kept;
    if (len <= 64u) kept = distinct_segment_in_wave<1>(seg, len, invalid, lane, pack);
    else if (len <= 128u) kept = distinct_segment_in_wave<2>(seg, len, invalid, lane, pack);
    else kept = distinct_segment_in_wave<4>(seg, len, invalid, lane, pack);
    if (lane == s) kept_mine = kept;
    if (chained && s == 0 && kept == 0) break;
  }
  if (lane < segments.n) counts[(size_t)sample * segments.n + lane] = (int32_t)kept_mine;
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

// All hop segments of every row in one launch; false when a segment is longer than 256 ids or
// there are more than kDistinctRowSegments of them (then: one launch per segment, below).
inline bool launch_distinct_rows(int32_t* final_samples, int32_t* counts, uint32_t n_samples, uint32_t final_size,
                                 const uint32_t* seg_base, const uint32_t* seg_len, uint32_t n_steps, int32_t invalid,
                                 bool chained, hipStream_t stream) {
  if (n_steps > (uint32_t)kDistinctRowSegments) return false;
  RowSegments segments{};
  segments.n = n_steps;
  for (uint32_t k = 0; k < n_steps; ++k) {
    if (seg_len[k] > 256u) return false;
    segments.base[k] = seg_base[k];
    segments.len[k] = seg_len[k];
  }
  distinct_rows_kernel<<<dim3((n_samples + 3) / 4), dim3(256), 0, stream>>>(final_samples, counts, n_samples, final_size,
                                                                          segments, invalid, chained ? 1u : 0u);
  return true;
}

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
