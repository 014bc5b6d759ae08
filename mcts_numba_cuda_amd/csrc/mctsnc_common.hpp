// Device-side building blocks shared by the MCTS-NC search kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "det_math.h"

namespace mctsnc {

constexpr int kWave = 64;

// ------------------------------------------------------------------------------------------------
// xoroshiro128+ (rotations 55/14/36) exactly as numba.cuda.random generates it: the reference draws
// every random number through xoroshiro128p_uniform_float32 (src/mctsnc.py:1435,1882,1971,2061).
// ------------------------------------------------------------------------------------------------
__host__ __device__ __forceinline__ uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

__host__ __device__ __forceinline__ uint64_t rng_next(uint64_t &s0, uint64_t &s1) {
    const uint64_t r = s0 + s1;
    const uint64_t t = s1 ^ s0;
    s0 = rotl64(s0, 55) ^ t ^ (t << 14);
    s1 = rotl64(t, 36);
    return r;
}

// float32((x >> 11) * 2^-53): the double product is exact, the narrowing rounds to nearest even and
// can therefore return exactly 1.0f.
__host__ __device__ __forceinline__ float rng_uniform(uint64_t &s0, uint64_t &s1) {
    return (float)((double)(rng_next(s0, s1) >> 11) * (1.0 / 9007199254740992.0));
}

// ------------------------------------------------------------------------------------------------
// Natural logarithm built only from IEEE-754 basic operations (no fused multiply-add, no library
// call), so that host and device evaluate bit-identical UCB values.  Classic table-free scheme:
// x = 2^k (1 + f), s = f / (2 + f), log(1 + f) = f - hfsq + s (hfsq + R(s^2)); error below 1 ulp.
// Valid for positive normal x (the callers pass visit counts >= 1).
// ------------------------------------------------------------------------------------------------
__host__ __device__ inline double det_log(double x) { return detm_log(x); }

#ifdef __HIPCC__
// float32((x >> 11) * 2^-53) for x = hi * 2^32 + lo (xoroshiro128p_uniform_float32 of numba.cuda.random as the
// reference calls it, src/mctsnc.py:1882): the 11 discarded bits are cleared, the remaining 53 significant bits are
// exact in float64 (two conversions and one fused multiply-add, all exact), the narrowing rounds once to nearest even
// as the reference's float32 cast does, and the scaling by 2^-64 is exact.  Five instructions per draw.
__device__ __forceinline__ float uniform_from_bits(uint32_t lo, uint32_t hi) {
    // (hi is usually the upper half of a 64-bit sum; without this the compiler converts that 64-bit value shifted down
    // instead, a longer sequence with an addition of zero that it does not fold)
    asm("" : "+v"(hi));
    const double d = __builtin_fma((double)hi, 4294967296.0, (double)(lo & 0xfffff800u));
    return (float)d * 0x1p-64f;
}

// xoroshiro128+ step on 32-bit halves (the 64-bit shifts of the generic form are slow vector instructions)
struct Rng32 { uint32_t s0l, s0h, s1l, s1h; };

__device__ __forceinline__ void rng_next32(Rng32 &r, uint32_t &out_lo, uint32_t &out_hi) {
    const uint64_t sum = (((uint64_t)r.s0h << 32) | r.s0l) + (((uint64_t)r.s1h << 32) | r.s1l);
    out_lo = (uint32_t)sum; out_hi = (uint32_t)(sum >> 32);
    const uint32_t tl = r.s1l ^ r.s0l, th = r.s1h ^ r.s0h;
    // rotl(s0, 55) = rotr(s0, 9); t << 14; rotl(t, 36) = halves swapped, then rotl 4
    const uint32_t r0l = __builtin_amdgcn_alignbit(r.s0h, r.s0l, 9), r0h = __builtin_amdgcn_alignbit(r.s0l, r.s0h, 9);
    const uint32_t shl = tl << 14, shh = __builtin_amdgcn_alignbit(th, tl, 18);
    r.s0l = r0l ^ tl ^ shl; r.s0h = r0h ^ th ^ shh;
    r.s1l = __builtin_amdgcn_alignbit(th, tl, 28); r.s1h = __builtin_amdgcn_alignbit(tl, th, 28);
}

// UCB of one child with the reference's numba typing (src/mctsnc.py:1337): float64 arithmetic on
// float32(child_n) and a float32 exploration constant, the sum narrowed to float32.
__device__ __forceinline__ float ucb_value(int32_t wins, int32_t n, double log_parent_n, float c) {
    const double q = (double)wins / (double)(float)n;
    const double e = (double)c * __dsqrt_rn(log_parent_n / (double)n);
    return (float)(q + e);
}

// Reverses the low three bits.  The reference's strided max-argmax keeps the left slot on ties
// (src/mctsnc.py:1343-1351), which makes the winner among tied slots the one whose bit-reversed index
// is smallest; for slots below 8 the order of the 3-bit reversal equals that of any wider reversal.
__device__ __forceinline__ uint32_t bitrev3(uint32_t a) { return ((a & 1u) << 2) | (a & 2u) | ((a >> 2) & 1u); }

// Maximum of a 32-bit key over each group of 8 adjacent lanes, in every lane of the group: one `v_max_u32` with a DPP
// operand per step (xor 1 and xor 2 inside a quad, then the mirror image within the half row) instead of LDS permutes.
// All 64 lanes must be active.
__device__ __forceinline__ uint32_t max_over_8_lanes(uint32_t key) {
    uint32_t o;
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)key, 0xB1, 0xf, 0xf, true); key = o > key ? o : key;
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)key, 0x4E, 0xf, 0xf, true); key = o > key ? o : key;
    o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)key, 0x141, 0xf, 0xf, true); key = o > key ? o : key;
    return key;
}

// ---- agent-scope synchronisation between workgroups --------------------------------------------
__device__ __forceinline__ uint32_t atomic_add_acq_rel(uint32_t *p, uint32_t v) {
    return __hip_atomic_fetch_add(p, v, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t atomic_load_acquire(const uint32_t *p) {
    return __hip_atomic_load(p, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t atomic_load_relaxed(const uint32_t *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void atomic_store_release(uint32_t *p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void atomic_store_relaxed(uint32_t *p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void fence_acquire_agent() { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent"); }
__device__ __forceinline__ void fence_release_agent() { __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent"); }

// Publishing to workgroups on the same XCC without an L2 write-back.  The vector L1 of a CU is write-through and the
// workgroups of one XCC share its L2, so a store is visible to them once it has been acknowledged: what a publish
// needs is that every earlier store of the publishing wavefront has completed before the flag store is issued.  A
// workgroup-scope release fence does NOT provide that (it lowers to no vector-memory wait when the workgroup runs on
// one CU, and stores to different L2 channels can land in either order), hence the explicit counter wait: vmcnt counts
// the wavefront's outstanding vector loads AND stores on gfx9.  Every wavefront that stored data a reader will look at
// must execute it before the flag store (or before the workgroup barrier that precedes the flag store).
__device__ __forceinline__ void wait_own_stores_at_l2() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
#endif

}  // namespace mctsnc
