/*
 * Synthetic evaluator of the Gomoku PUCT loop: stands in for a policy/value network with a pure function of the
 * position, so that a search is reproducible and the host can recompute every prior and value.  Plain C99 / C++ / HIP;
 * all arithmetic is 64-bit integer mixing plus IEEE basic operations and the deterministic log / exp of det_math.h, so
 * host and device agree bit for bit.
 *
 *   value(position)      uniform in [-1, 1) from a hash of the position (for the player to move)
 *   prior over the legal cells:  Dirichlet(alpha): one Gamma(alpha, 1) variate per legal cell from a hash of
 *                        (position, cell), in 2^-32 fixed point; the prior of a cell is its variate over the sum.
 *
 * The reference has no such loop (its PUCT kernels stop at select / backup, src/puct/puct_gpu_v3_cpp.cu,
 * src/puct/puct_gpu_v2.py:847-927); this evaluator is this library's own definition.
 */
#ifndef MCTSNC_PUCT_SYNTHETIC_H
#define MCTSNC_PUCT_SYNTHETIC_H
#include <stdint.h>

#include "det_math.h"

#if defined(__HIPCC__)
#define PSYN_FN __host__ __device__ inline
#else
#define PSYN_FN static inline
#endif

/* SplitMix64 finaliser applied to z + golden ratio. */
PSYN_FN uint64_t psyn_mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

/* Seed of tree `tree`: every tree sees its own synthetic network. */
PSYN_FN uint64_t psyn_tree_seed(uint64_t seed, int tree) { return psyn_mix64(seed ^ ((uint64_t)(uint32_t)tree << 32)); }

/* Hash of a position given as 16 words: words 0..7 the stones of the player with token +1 (bit = cell index), words
 * 8..15 those of the player with token -1.  The side to move follows from the stone counts. */
PSYN_FN uint64_t psyn_board_hash(uint64_t tree_seed, const uint32_t *w) {
    uint64_t h = psyn_mix64(tree_seed);
    for (int i = 0; i < 8; ++i) h = psyn_mix64(h ^ (((uint64_t)w[2 * i + 1] << 32) | w[2 * i]));
    return h;
}

/* Value of the position for the player to move, in [-1, 1): 24 hash bits, exactly representable. */
PSYN_FN float psyn_value(uint64_t board_hash) {
    const uint64_t h = psyn_mix64(board_hash ^ 0x76616C7565ull);
    return (float)((int32_t)(h >> 40) - 8388608) * (1.0f / 8388608.0f);
}

/* Uniform float in (0, 1), never 0 or 1, from 23 bits. */
PSYN_FN float psyn_unit(uint32_t h) { return ((float)(h >> 9) + 0.5f) * (1.0f / 8388608.0f); }

/* One round of the Ahrens-Dieter rejection sampler "GS" for Gamma(alpha, 1), 0 < alpha < 1, driven by the two halves
 * of word number `round` of the counter-based stream of `key`.  Writes the candidate to *x and returns whether it is
 * accepted.  The acceptance tests are taken in the log domain (log u2 <= -x, resp. log u2 <= (alpha - 1) log x).
 * Single precision throughout (a weight keeps 15 mantissa bits) and without a branch: a wavefront whose lanes take
 * different sides of the sampler runs the same instructions. */
PSYN_FN int psyn_gamma_round(float alpha, uint64_t key, int round, float *x) {
    const float b = 1.0f + alpha * 0.36787944117f; /* 1 + alpha / e */
    const float inv_alpha = 1.0f / alpha;
    const uint64_t h = psyn_mix64(key + (uint64_t)round);
    const float u1 = psyn_unit((uint32_t)(h >> 32));
    const float log_u2 = detm_logf(psyn_unit((uint32_t)h));
    const float p = b * u1;
    const int small = p <= 1.0f;
    float t = small ? p : (b - p) * inv_alpha;
    t = t < 1.17549435e-38f ? 1.17549435e-38f : t;
    const float log_t = detm_logf(t);
    const float x_small = detm_expf(log_t * inv_alpha);
    const float x_large = -log_t; /* > 1 on this side: b - p < alpha / e */
    const float bound = small ? -x_small : (alpha - 1.0f) * detm_logf(small ? 2.0f : x_large);
    *x = small ? x_small : x_large;
    return log_u2 <= bound;
}

#define PSYN_GAMMA_ROUNDS 16 /* the chance of needing more is below 1e-9; the last candidate is taken then */

PSYN_FN float psyn_gamma(float alpha, uint64_t key) {
    float x = 0.0f;
    for (int round = 0; round < PSYN_GAMMA_ROUNDS; ++round)
        if (psyn_gamma_round(alpha, key, round, &x)) break;
    return x;
}

/* Stream key of `cell` in the position with hash `board_hash`. */
PSYN_FN uint64_t psyn_cell_key(uint64_t board_hash, int cell) {
    return psyn_mix64(board_hash ^ (0x7072696F72ull + ((uint64_t)(uint32_t)cell << 40)));
}

/* The weight of a cell is its Gamma variate, capped at 255 and truncated to a float32 with 15 mantissa bits.  Two
 * views of the same number: a 32-bit sort key whose unsigned order is "larger weight first, then smaller cell" (0 is
 * reserved for cells that are not legal), and the weight in 2^-32 fixed point for the exact, order-independent sum
 * (a sum over 256 cells stays below 2^48). */
PSYN_FN uint32_t psyn_weight_key(float gamma, int cell) {
    union { float f; uint32_t u; } v;
    v.f = gamma > 255.0f ? 255.0f : gamma;
    return 0x80000000u | (v.u & 0xFFFFFF00u) | (uint32_t)(255 - cell);
}
PSYN_FN uint64_t psyn_key_weight(uint32_t key) {
    union { float f; uint32_t u; } v;
    v.u = key & 0x7FFFFF00u;
    return (uint64_t)((double)v.f * 4294967296.0);
}

/* Prior of a cell from its weight and the sum of the weights of all legal cells; uniform if every weight is 0. */
PSYN_FN float psyn_prior(uint64_t weight, uint64_t weight_sum, int n_legal) {
    if (weight_sum == 0) return (float)(1.0 / (double)n_legal);
    return (float)((double)weight / (double)weight_sum);
}

#endif
