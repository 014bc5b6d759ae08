/*
 * Synthetic evaluator of the Gomoku PUCT loop: stands in for a policy/value network with a pure function of the
 * position, so that a search is reproducible and the host can recompute every prior and value.  Plain C99 / C++ / HIP;
 * all arithmetic is 64-bit integer mixing plus IEEE double basic operations and the deterministic log / exp of
 * det_math.h, so host and device agree bit for bit.
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

/* Uniform double in (0, 1), never 0 or 1. */
PSYN_FN double psyn_unit(uint64_t h) { return ((double)(h >> 11) + 0.5) * (1.0 / 9007199254740992.0); }

/* One round of the Ahrens-Dieter rejection sampler "GS" for Gamma(alpha, 1), 0 < alpha < 1, driven by the uniforms
 * number 2 * round and 2 * round + 1 of the counter-based stream of `key`.  Writes the candidate to *x and returns
 * whether it is accepted.  The acceptance tests are taken in the log domain (log u2 <= -x, resp.
 * log u2 <= (alpha - 1) log x), which lets both branches share two of their three logarithms. */
PSYN_FN int psyn_gamma_round(double alpha, uint64_t key, int round, double *x) {
    const double b = 1.0 + alpha * 0.36787944117144233; /* 1 + alpha / e */
    const double inv_alpha = 1.0 / alpha;
    const double u1 = psyn_unit(psyn_mix64(key + 2u * (uint64_t)round));
    const double log_u2 = detm_log(psyn_unit(psyn_mix64(key + 2u * (uint64_t)round + 1u)));
    const double p = b * u1;
    const int small = p <= 1.0;
    const double log_t = detm_log(small ? p : (b - p) * inv_alpha);
    if (small) {
        *x = detm_exp(log_t * inv_alpha);
        return log_u2 <= -*x;
    }
    *x = -log_t;
    return log_u2 <= (alpha - 1.0) * detm_log(*x);
}

#define PSYN_GAMMA_ROUNDS 16 /* the chance of needing more is below 1e-9; the last candidate is taken then */

PSYN_FN double psyn_gamma(double alpha, uint64_t key) {
    double x = 0.0;
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
PSYN_FN uint32_t psyn_weight_key(double gamma, int cell) {
    union { float f; uint32_t u; } v;
    v.f = (float)(gamma > 255.0 ? 255.0 : gamma);
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
