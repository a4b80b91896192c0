// Counter-based random numbers for the sampling engine (host + gfx950 device).
//
// Replaces the reference's per-thread-slot XORWOW states (src/nextdoor.cu:1838-1843,
// src/rand_num_gen.cuh:117-122): 48 bytes of state per launch thread are traded for a
// stateless Philox4x32-10 block keyed by WHAT is being sampled, so results do not depend
// on which kernel, workgroup or lane happens to execute an output slot.
//
//   block(slot, step, b) = Philox4x32-10(counter = {slot_lo, slot_hi, step, b},
//                                        key     = {seed_lo, seed_hi})
//   draw d of (slot, step) = word (d & 3) of block(slot, step, d >> 2)
//   uniform = (word >> 8) * 2^-24   in [0, 1)
//
// `slot` is the global index of the output being produced at `step`:
// ((sample * transitsPerSample + transitIdx) * stepSize + neighbourIdx).
//
// Steps that draw several outputs per transit (stepSize > 1: k-hop) use the GROUPED form of the
// stream: four consecutive output slots share one block for their first draw,
//   draw 0 of (slot, step)      = word (slot & 3) of block(slot >> 2, step | 2^31, 0)
//   draw d >= 1 of (slot, step) = draw d - 1 of the slot's own stream above,
// because such a step takes one draw per output (a uniform pick) and would otherwise spend a
// whole ten-round block on one word of it: the lane that produces the outputs of a transit
// computes one block per four of them.  (The multiplications of Philox are what a k-hop step
// waits for: 40 quarter-rate 32-bit multiplies per block.)  Walk steps (stepSize 1) draw several
// numbers per output and keep the plain form.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define ND_HD __host__ __device__ __forceinline__
#else
#define ND_HD inline
#endif

namespace nd {

struct PhiloxBlock {
  uint32_t w[4];
};

ND_HD uint32_t mul_hi_u32(uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __umulhi(a, b);
#else
  return (uint32_t)(((uint64_t)a * (uint64_t)b) >> 32);
#endif
}

ND_HD PhiloxBlock philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                uint32_t k0, uint32_t k1) {
  constexpr uint32_t kMulA = 0xD2511F53u, kMulB = 0xCD9E8D57u;
  constexpr uint32_t kWeylA = 0x9E3779B9u, kWeylB = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi_a = mul_hi_u32(kMulA, c0), lo_a = kMulA * c0;
    const uint32_t hi_b = mul_hi_u32(kMulB, c2), lo_b = kMulB * c2;
    c0 = hi_b ^ c1 ^ k0;
    c1 = lo_b;
    c2 = hi_a ^ c3 ^ k1;
    c3 = lo_a;
    k0 += kWeylA;
    k1 += kWeylB;
  }
  PhiloxBlock out;
  out.w[0] = c0; out.w[1] = c1; out.w[2] = c2; out.w[3] = c3;
  return out;
}

ND_HD float u32_to_unit_float(uint32_t word) {
  return (float)(word >> 8) * 5.9604644775390625e-08f;  // 2^-24, exact
}

constexpr uint32_t kGroupedStepFlag = 0x80000000u;

// The block the slots 4 * group .. 4 * group + 3 share for their first draw at a grouped step.
ND_HD PhiloxBlock grouped_first_block(uint64_t seed, uint64_t group, uint32_t step) {
  return philox4x32_10((uint32_t)group, (uint32_t)(group >> 32), step | kGroupedStepFlag, 0u, (uint32_t)seed,
                       (uint32_t)(seed >> 32));
}

// The same for a seed that is the same for every lane (a kernel argument).  The ten round keys
// are then scalars, and the compiler, seeing that they never change, computes all twenty words
// once per kernel and keeps them - more scalar registers than a step kernel has to spare, so
// they end up parked in lanes of a vector register and every use is a vector-pipe read (a fifth
// of the block's vector instructions).  The empty statement makes the key opaque at this point:
// the rounds add their constants on the scalar unit as they go.
ND_HD PhiloxBlock grouped_first_block_scalar_seed(uint64_t seed, uint64_t group, uint32_t step) {
#if defined(__HIP_DEVICE_COMPILE__)
  // (read from the first lane: a no-op for a value that is in scalar registers already, and
  // what makes it one where the compiler has moved the kernel's arguments to vector registers)
  uint32_t k0 = __builtin_amdgcn_readfirstlane((uint32_t)seed), k1 = __builtin_amdgcn_readfirstlane((uint32_t)(seed >> 32));
  asm volatile("" : "+s"(k0), "+s"(k1));
  return philox4x32_10((uint32_t)group, (uint32_t)(group >> 32), step | kGroupedStepFlag, 0u, k0, k1);
#else
  return grouped_first_block(seed, group, step);
#endif
}

// Word i (0..3) of a block, by comparisons: an index into the array would put it in memory.
ND_HD uint32_t block_word(const PhiloxBlock& b, uint32_t i) {
  return i == 0 ? b.w[0] : i == 1 ? b.w[1] : i == 2 ? b.w[2] : b.w[3];
}

// Cursor over the draws of one (slot, step).  This is the object an App's next()
// receives as its random-state handle.
struct RandState {
  uint32_t slot_lo, slot_hi, step, draw;  // draw: draws taken from the slot's own stream
  uint32_t key0, key1;
  uint32_t first_word;  // grouped form: the word of the shared block, until it is drawn
  uint32_t has_first;
  // The words of the current Philox block that have not been drawn yet, next one first.  A
  // draw takes word0 and moves the others up: no word is ever picked by an index, so the state
  // stays in registers (an array indexed by the draw number, or selects among its members,
  // end up as a memory object with a computed address).
  uint32_t word0, word1, word2, word3;

  ND_HD void reset(uint64_t seed, uint64_t slot, uint32_t step_) {
    slot_lo = (uint32_t)slot;
    slot_hi = (uint32_t)(slot >> 32);
    step = step_;
    draw = 0;
    key0 = (uint32_t)seed;
    key1 = (uint32_t)(seed >> 32);
    word0 = word1 = word2 = word3 = 0;
    first_word = 0;
    has_first = 0;
  }

  // Grouped form, the first draw given: the caller holds the shared block of the slot's group.
  ND_HD void reset_with_first(uint64_t seed, uint64_t slot, uint32_t step_, uint32_t first) {
    reset(seed, slot, step_);
    first_word = first;
    has_first = 1;
  }

  // Grouped form, computing the shared block here (host loops, one-off uses).
  ND_HD void reset_grouped(uint64_t seed, uint64_t slot, uint32_t step_) {
    reset_with_first(seed, slot, step_, block_word(grouped_first_block(seed, slot >> 2, step_), (uint32_t)slot & 3u));
  }

  ND_HD uint32_t next_word() {
    if (has_first) {
      has_first = 0;
      return first_word;
    }
    if ((draw & 3u) == 0) {
      const PhiloxBlock b = philox4x32_10(slot_lo, slot_hi, step, draw >> 2, key0, key1);
      word0 = b.w[0];
      word1 = b.w[1];
      word2 = b.w[2];
      word3 = b.w[3];
    }
    ++draw;
    const uint32_t word = word0;
    word0 = word1;
    word1 = word2;
    word2 = word3;
    return word;
  }

  ND_HD float next_uniform() { return u32_to_unit_float(next_word()); }
};

// One-shot form used by fills and host code.
ND_HD float uniform_at(uint64_t seed, uint64_t slot, uint32_t step, uint32_t draw) {
  PhiloxBlock b = philox4x32_10((uint32_t)slot, (uint32_t)(slot >> 32), step, draw >> 2,
                                (uint32_t)seed, (uint32_t)(seed >> 32));
  return u32_to_unit_float(b.w[draw & 3u]);
}

// Draw `draw` of the grouped form.
ND_HD float grouped_uniform_at(uint64_t seed, uint64_t slot, uint32_t step, uint32_t draw) {
  if (draw == 0) return u32_to_unit_float(block_word(grouped_first_block(seed, slot >> 2, step), (uint32_t)slot & 3u));
  return uniform_at(seed, slot, step, draw - 1);
}

// min((int)(u * n), n - 1): the reference's RandNumGen::rand_int
// (src/rand_num_gen.cuh:117-122) with u in [0,1).  The clamp still matters: u * n
// rounds up to n for u = 1 - 2^-24 and large n.
ND_HD int32_t rand_int_from_uniform(float u, int32_t n) {
  const float scaled = u * (float)n;
  const int32_t id = (int32_t)scaled;
  return id < n - 1 ? id : n - 1;
}

}  // namespace nd
