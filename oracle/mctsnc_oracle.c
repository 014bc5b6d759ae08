/*
 * mctsnc_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain, sequential CPU restatement of the reference MCTS-NC search algorithm
 * (reference: src/mctsnc.py kernels :1259-2375, game mechanics
 * src/mctsnc_game_mechanics.py:89-280, RNG = numba.cuda.random xoroshiro128+).
 * It exists only so that tests, the smoke check and the CPU-baseline leg of the
 * benchmark can compare the HIP engine against something that follows the
 * reference line by line.  Nothing in the product path may call into it.
 *
 * Every function names the reference lines it restates.  Arrays keep the
 * reference's names, dtypes and index conventions (per tree instead of one
 * [T, S, ...] block, grown on demand instead of sized to max_tree_size).
 *
 * What pins this file (tests/test_oracle_golden.py, tests/test_oracle_units.py, tests/test_readme_examples.py):
 *   - the reference's recorded full-tree dumps extras/mctsnc_{ocp,acp}_thrifty_c4_1000steps.json
 *     (parents, children of expanded nodes, depths, turns, ns, ns_wins, last-step scratch);
 *   - the reference's recorded A100 experiment logs (root tables, tree statistics,
 *     RNG carry-over across consecutive searches);
 *   - the two complete runs printed in the reference's README.md: Connect 4 (8 trees x 128 playouts, all-children,
 *     6373 steps) and Gomoku 15x15 (same settings, 442 steps, 94 359 552 playouts), every printed root row, the best
 *     action and the tree statistics to the last digit: the Gomoku search end to end (legal list order, swap-remove,
 *     exactly-five, stream layout with 225 actions, reduction over 225 actions);
 *   - independent brute-force / textbook checks of the game rules, the tournament
 *     arg-max and the RNG jump.
 * Parity unpinned (no recorded artefact exercises them): the memory-exhausted (-3) paths.
 *
 * Deliberate deviations from the reference where the reference reads or writes
 * out of bounds (they are deterministic definitions, listed for the record):
 *   - tree-full (-3) step, OCP: the path is backed up, the out-of-bounds child
 *     update of _backup_ocp (src/mctsnc.py:2106-2114 with rand_child == -3) is
 *     skipped; _expand_2_thrifty (:1697-1754) is skipped instead of writing node -1.
 *   - node pool running out in the middle of an expansion: the reference gives every legal action that
 *     no longer fits the index of the last child that did (src/mctsnc.py:1427-1429 store the running
 *     shift for every action), after which several blocks write that one node concurrently; here such
 *     actions get no child (-1) and only the children that fit are created and played out.
 *   - OCP random child when the uniform draw rounds to 1.0f: the ordinal is
 *     clamped to count-1 (the reference indexes one past its list, :1435,:1511).
 *   - root action without a child node in the final reduction (:2236,:2278 read
 *     node -1): counted as n = 0, n_wins = 0.
 *   - never-written memory (child slots of leaves, local playout arrays) reads as
 *     -1 for child slots and 0 for local arrays.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define MAX_TREE_DEPTH 2048
#define GAME_C4 0
#define GAME_GOMOKU 1
#define V_OCP_THRIFTY 0
#define V_OCP_PRODIGAL 1
#define V_ACP_THRIFTY 2
#define V_ACP_PRODIGAL 3

typedef struct { uint64_t s0, s1; } rng_t;

typedef struct {
    int32_t size, cap;
    int32_t *trees;      /* [cap][1+A]: parent, children */
    int16_t *depths;
    int8_t *turns;
    uint8_t *leaves, *terminals;
    int8_t *outcomes;
    int32_t *ns, *ns_wins;
    int8_t *boards;      /* [cap][m*n] */
    int8_t *extras;      /* [cap][E] */
    int32_t selected;
    int32_t path[MAX_TREE_DEPTH + 2]; /* [-1] = length */
    int16_t *actions_expanded;        /* [A+2] */
    int32_t playout_outcomes[2];
    int32_t *playout_outcomes_children; /* [A][2] */
} tree_t;

typedef struct {
    int game, m, n, E, A, T, P, variant;
    float ucb_c;
    uint64_t seed;
    int64_t max_tree_size;
    int tpb_e1;
    int threads;
    tree_t *tr;
    rng_t *rng_expand;   /* OCP: [T*tpb_e1] */
    rng_t *rng_playout;  /* OCP: [T*P], ACP: [T*A*P] */
    int16_t *root_actions_expanded; /* [A+2] */
    int64_t *root_ns, *actions_ns, *actions_ns_wins; /* [A] */
    uint8_t *actions_win_flags;
    int32_t best_action; uint8_t best_win_flag; int64_t best_n, best_n_wins;
    int64_t steps;
    uint64_t u1_events;  /* playout draws that rounded to 1.0f */
    uint64_t plies;      /* playout moves made */
} oracle_t;

/* ----------------------------------------------------------------------------------------
 * RNG: numba.cuda.random (xoroshiro128+ with rotations 55/14/36, splitmix64 seeding, 2^64 jump)
 * -------------------------------------------------------------------------------------- */
static inline uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

uint64_t mo_rng_next(rng_t *s) {
    uint64_t s0 = s->s0, s1 = s->s1, r = s0 + s1;
    s1 ^= s0;
    s->s0 = rotl64(s0, 55) ^ s1 ^ (s1 << 14);
    s->s1 = rotl64(s1, 36);
    return r;
}

float mo_rng_uniform(rng_t *s) { /* uint64_to_unit_float32 */
    return (float)((double)(mo_rng_next(s) >> 11) * (1.0 / 9007199254740992.0));
}

void mo_rng_jump(rng_t *s) {
    static const uint64_t J[2] = {0xbeac0467eba5facbULL, 0xd86b048b86aa9922ULL};
    uint64_t s0 = 0, s1 = 0;
    for (int i = 0; i < 2; i++)
        for (int b = 0; b < 64; b++) {
            if (J[i] & (1ULL << b)) { s0 ^= s->s0; s1 ^= s->s1; }
            mo_rng_next(s);
        }
    s->s0 = s0; s->s1 = s1;
}

/* create_xoroshiro128p_states(n, seed): state 0 from splitmix64, state i = jump(state i-1) */
void mo_rng_init(rng_t *st, int64_t n, uint64_t seed) {
    if (n < 1) return;
    uint64_t z = seed + 0x9E3779B97F4A7C15ULL;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    z = z ^ (z >> 31);
    st[0].s0 = z; st[0].s1 = z;
    for (int64_t i = 1; i < n; i++) { st[i] = st[i - 1]; mo_rng_jump(&st[i]); }
}

/* ----------------------------------------------------------------------------------------
 * Game mechanics on byte boards with row stride `ld` (src/mctsnc_game_mechanics.py:89-280).
 * Row indices that went negative wrap by +32 as numba's indexing of the (32, 32) local
 * array does; only an over-full Connect 4 column can produce one.
 * -------------------------------------------------------------------------------------- */
#define BD(b, ld, i, j) ((b)[(((i) < 0) ? (i) + 32 : (i)) * (ld) + (j)])

static int is_action_legal(const oracle_t *o, const int8_t *board, int ld, const int8_t *extra, int action) {
    if (o->game == GAME_C4) return extra[action] < o->m;               /* :90-92 */
    return BD(board, ld, action / o->n, action % o->n) == 0;           /* :182-186 */
}

static void take_action(const oracle_t *o, int8_t *board, int ld, int8_t *extra, int turn, int action) {
    if (o->game == GAME_C4) {                                          /* :95-99 */
        extra[action] += 1;
        int row = o->m - extra[action];
        BD(board, ld, row, action) = (int8_t)turn;
    } else {                                                           /* :189-193 */
        BD(board, ld, action / o->n, action % o->n) = (int8_t)turn;
    }
}

/* legal[512] holds the count (the reference's legal_actions_with_count[-1]) */
static void legal_actions_playout(const oracle_t *o, const int8_t *board, int ld, const int8_t *extra, int16_t *legal) {
    if (o->game == GAME_C4) {                                          /* :102-109 */
        int count = 0;
        for (int j = 0; j < o->n; j++)
            if (extra[j] < o->m) legal[count++] = (int16_t)j;
        legal[512] = (int16_t)count;
    } else if (legal[512] == 0) {                                      /* :196-207 */
        int count = 0, k = 0;
        for (int i = 0; i < o->m; i++)
            for (int j = 0; j < o->n; j++) {
                if (BD(board, ld, i, j) == 0) legal[count++] = (int16_t)k;
                k++;
            }
        legal[512] = (int16_t)count;
    }
}

static void take_action_playout(const oracle_t *o, int8_t *board, int ld, int8_t *extra, int turn, int action, int action_ord, int16_t *legal) {
    if (o->game == GAME_C4) {                                          /* :112-116 */
        extra[action] += 1;
        int row = o->m - extra[action];
        BD(board, ld, row, action) = (int8_t)turn;
    } else {                                                           /* :210-217 */
        BD(board, ld, action / o->n, action % o->n) = (int8_t)turn;
        int16_t last = legal[legal[512] - 1];
        legal[action_ord] = last;
        legal[512] -= 1;
    }
}

static int compute_outcome(const oracle_t *o, const int8_t *board, int ld, const int8_t *extra, int turn, int last_action) {
    const int m = o->m, n = o->n;
    const int last_token = -turn;
    int i, j, reach, total;
    if (o->game == GAME_C4) { j = last_action; i = m - extra[j]; reach = 4; }   /* :119-123 */
    else { i = last_action / n; j = last_action % n; reach = 6; }              /* :220-224 */
    static const int DI[4][2] = {{-1, 1}, {0, 0}, {-1, 1}, {-1, 1}};
    static const int DJ[4][2] = {{0, 0}, {1, -1}, {1, -1}, {-1, 1}};
    for (int d = 0; d < 4; d++) {   /* N-S, E-W, NE-SW, NW-SE in the reference's order */
        total = 0;
        for (int h = 0; h < 2; h++) {
            int di = DI[d][h], dj = DJ[d][h];
            for (int k = 1; k < reach; k++) {
                int ii = i + di * k, jj = j + dj * k;
                if ((di < 0 && i - k < 0) || (di > 0 && i + k >= m) || (dj > 0 && j + k >= n) || (dj < 0 && j - k < 0))
                    break;
                if (BD(board, ld, ii, jj) != last_token) break;
                total++;
            }
        }
        if (o->game == GAME_C4 ? (total >= 3) : (total == 4)) return last_token; /* :134 / :235 */
    }
    if (o->game == GAME_C4) {                                          /* :172-178 */
        for (int jj = 0; jj < n; jj++) if (extra[jj] < m) return 2;
        return 0;
    }
    for (int ii = 0; ii < m; ii++)                                     /* :273-280 */
        for (int jj = 0; jj < n; jj++) if (BD(board, ld, ii, jj) == 0) return 2;
    return 0;
}

/* exported for the rule property tests (boards given with row stride n) */
int mo_game_outcome(int game, int m, int n, const int8_t *board, const int8_t *extra, int turn, int last_action) {
    oracle_t o; memset(&o, 0, sizeof o); o.game = game; o.m = m; o.n = n;
    return compute_outcome(&o, board, n, extra, turn, last_action);
}

/* ----------------------------------------------------------------------------------------
 * One playout (src/mctsnc.py:1870-1890, :1959-1979, :2049-2069) in the reference's local arrays.
 * Returns the outcome in {-1, 0, +1}.
 * -------------------------------------------------------------------------------------- */
static int playout(const oracle_t *o, const int8_t *node_board, const int8_t *node_extra, int turn, int last_action,
                   rng_t *rng, uint64_t *u1_events, uint64_t *plies) {
    int8_t lb[32 * 32];
    int8_t le[64];
    int16_t legal[513];
    memset(lb, 0, sizeof lb);
    memset(le, 0, sizeof le);
    memset(legal, 0, sizeof legal);
    for (int i = 0; i < o->m; i++) memcpy(lb + i * 32, node_board + i * o->n, (size_t)o->n);
    memcpy(le, node_extra, (size_t)(o->E < 64 ? o->E : 64));
    int outcome = (last_action != -1) ? compute_outcome(o, lb, 32, le, turn, last_action) : 2;
    for (;;) {
        if (outcome == -1 || outcome == 0 || outcome == 1) return outcome;
        legal_actions_playout(o, lb, 32, le, legal);
        int16_t count = legal[512];
        float u = mo_rng_uniform(rng);
        int16_t ord = (int16_t)(u * (float)count);   /* single-precision product, :1882 */
        if (ord == count) (*u1_events)++;
        last_action = legal[ord];
        take_action_playout(o, lb, 32, le, turn, last_action, ord, legal);
        (*plies)++;
        turn = -turn;
        outcome = compute_outcome(o, lb, 32, le, turn, last_action);
    }
}

/* ----------------------------------------------------------------------------------------
 * Tree storage
 * -------------------------------------------------------------------------------------- */
static void tree_reserve(const oracle_t *o, tree_t *t, int32_t need) {
    if (need <= t->cap) return;
    int32_t cap = t->cap ? t->cap : 1024;
    while (cap < need) cap *= 2;
    const int A = o->A, mn = o->m * o->n, E = o->E;
    t->trees = realloc(t->trees, sizeof(int32_t) * (size_t)cap * (1 + A));
    for (int64_t i = (int64_t)t->cap * (1 + A); i < (int64_t)cap * (1 + A); i++) t->trees[i] = -1;
    t->depths = realloc(t->depths, sizeof(int16_t) * cap);
    t->turns = realloc(t->turns, cap);
    t->leaves = realloc(t->leaves, cap);
    t->terminals = realloc(t->terminals, cap);
    t->outcomes = realloc(t->outcomes, cap);
    t->ns = realloc(t->ns, sizeof(int32_t) * cap);
    t->ns_wins = realloc(t->ns_wins, sizeof(int32_t) * cap);
    t->boards = realloc(t->boards, (size_t)cap * mn);
    t->extras = realloc(t->extras, (size_t)cap * E);
    t->cap = cap;
}

static int next_pow2(int x) { int p = 1; while (p < x) p *= 2; return p; }

oracle_t *mo_create(int game, int m, int n, int E, int A, int T, int P, int variant, double ucb_c,
                    uint64_t seed, int64_t max_tree_size) {
    oracle_t *o = calloc(1, sizeof *o);
    o->game = game; o->m = m; o->n = n; o->E = E < 1 ? 1 : E; o->A = A; o->T = T; o->P = P; o->variant = variant;
    o->ucb_c = (float)ucb_c; o->seed = seed; o->max_tree_size = max_tree_size;
    /* tpb table, src/mctsnc.py:360-365 with cuda_tpb_default = 512 */
    int tpb_board = next_pow2(m * n), tpb_extra = next_pow2(o->E), tpb_actions = next_pow2(A);
    int tpb_r = tpb_board > tpb_extra ? tpb_board : tpb_extra; if (tpb_r > 512) tpb_r = 512;
    o->tpb_e1 = tpb_r > tpb_actions ? tpb_r : tpb_actions; if (o->tpb_e1 > 512) o->tpb_e1 = 512;
    o->threads = 1;
    o->tr = calloc((size_t)T, sizeof(tree_t));
    for (int ti = 0; ti < T; ti++) {
        o->tr[ti].actions_expanded = calloc((size_t)A + 2, sizeof(int16_t));
        o->tr[ti].playout_outcomes_children = calloc((size_t)A * 2, sizeof(int32_t));
        tree_reserve(o, &o->tr[ti], 1024);
    }
    o->root_actions_expanded = calloc((size_t)A + 2, sizeof(int16_t));
    o->root_ns = calloc((size_t)A, sizeof(int64_t));
    o->actions_ns = calloc((size_t)A, sizeof(int64_t));
    o->actions_ns_wins = calloc((size_t)A, sizeof(int64_t));
    o->actions_win_flags = calloc((size_t)A, 1);
    /* RNG arrays, src/mctsnc.py:390-394 */
    if (variant <= V_OCP_PRODIGAL) {
        o->rng_expand = malloc(sizeof(rng_t) * (size_t)T * o->tpb_e1);
        mo_rng_init(o->rng_expand, (int64_t)T * o->tpb_e1, seed);
        o->rng_playout = malloc(sizeof(rng_t) * (size_t)T * P);
        mo_rng_init(o->rng_playout, (int64_t)T * P, seed);
    } else {
        o->rng_playout = malloc(sizeof(rng_t) * (size_t)T * A * P);
        mo_rng_init(o->rng_playout, (int64_t)T * A * P, seed);
    }
    return o;
}

void mo_destroy(oracle_t *o) {
    if (!o) return;
    for (int ti = 0; ti < o->T; ti++) {
        tree_t *t = &o->tr[ti];
        free(t->trees); free(t->depths); free(t->turns); free(t->leaves); free(t->terminals); free(t->outcomes);
        free(t->ns); free(t->ns_wins); free(t->boards); free(t->extras); free(t->actions_expanded);
        free(t->playout_outcomes_children);
    }
    free(o->tr); free(o->rng_expand); free(o->rng_playout); free(o->root_actions_expanded); free(o->root_ns);
    free(o->actions_ns); free(o->actions_ns_wins); free(o->actions_win_flags); free(o);
}

void mo_set_threads(oracle_t *o, int threads) { o->threads = threads < 1 ? 1 : threads; }

/* ----------------------------------------------------------------------------------------
 * The strided max-argmax "tournament" of the reference (src/mctsnc.py:1343-1351, :2318-2330):
 * slot t takes slot t+stride when strictly smaller.  less(a, b) decides "a < b".
 * -------------------------------------------------------------------------------------- */
int mo_argmax_tournament_f32(const float *vals, int count, int size) {
    float v[512]; int idx[512];
    for (int t = 0; t < size; t++) { v[t] = t < count ? vals[t] : -INFINITY; idx[t] = t; }
    for (int stride = size >> 1; stride > 0; stride >>= 1)
        for (int t = 0; t < stride; t++)
            if (v[t] < v[t + stride]) { v[t] = v[t + stride]; idx[t] = idx[t + stride]; }
    return idx[0];
}

/* Natural logarithm from IEEE-754 basic operations only (table-free reduction x = 2^k (1 + f),
 * s = f / (2 + f); error below 1 ulp).  The reference calls CUDA's log(), which is not correctly
 * rounded either; an implementation that is bit-reproducible on every processor is used instead, and
 * the recorded reference results pin that the choice does not change any search. */
double mo_det_log(double x) {
    const double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10;
    const double Lg1 = 6.666666666666735130e-01, Lg2 = 3.999999999940941908e-01, Lg3 = 2.857142874366239149e-01,
                 Lg4 = 2.222219843214978396e-01, Lg5 = 1.818357216161805012e-01, Lg6 = 1.531383769920937332e-01,
                 Lg7 = 1.479819860511658591e-01;
    union { double d; uint64_t u; } v;
    v.d = x;
    int32_t hx = (int32_t)(v.u >> 32);
    const uint32_t lx = (uint32_t)v.u;
    int32_t k = (hx >> 20) - 1023;
    hx &= 0x000fffff;
    int32_t i = (hx + 0x95f64) & 0x100000;
    v.u = ((uint64_t)(uint32_t)(hx | (i ^ 0x3ff00000)) << 32) | lx;  // normalise x or x/2
    k += (i >> 20);
    const double f = v.d - 1.0;
    const double dk = (double)k;
    if ((0x000fffff & (2 + hx)) < 3) {  // |f| < 2^-20
        if (f == 0.0) {
            if (k == 0) return 0.0;
            return dk * ln2_hi + dk * ln2_lo;
        }
        const double R = f * f * (0.5 - 0.33333333333333333 * f);
        if (k == 0) return f - R;
        return dk * ln2_hi - ((R - dk * ln2_lo) - f);
    }
    const double s = f / (2.0 + f);
    const double z = s * s;
    i = hx - 0x6147a;
    const double w = z * z;
    const int32_t j = 0x6b851 - hx;
    const double t1 = w * (Lg2 + w * (Lg4 + w * Lg6));
    const double t2 = z * (Lg1 + w * (Lg3 + w * (Lg5 + w * Lg7)));
    i |= j;
    const double R = t2 + t1;
    if (i > 0) {
        const double hfsq = 0.5 * f * f;
        if (k == 0) return f - (hfsq - s * (hfsq + R));
        return dk * ln2_hi - ((hfsq - (s * (hfsq + R) + dk * ln2_lo)) - f);
    }
    if (k == 0) return f - s * (f - R);
    return dk * ln2_hi - ((s * (f - R) - dk * ln2_lo) - f);
}

/* UCB value of one child as the reference's numba typing evaluates it (src/mctsnc.py:1337):
 * float64 arithmetic with float32(child_n) and float32 ucb_c, stored to a float32 array. */
float mo_ucb(int32_t child_ns_wins, int32_t child_n, int32_t parent_n, float ucb_c) {
    if (child_n == 0) return INFINITY;
    double q = (double)child_ns_wins / (double)(float)child_n;
    double e = (double)ucb_c * sqrt(mo_det_log((double)parent_n) / (double)child_n);
    return (float)(q + e);
}

/* _reset, src/mctsnc.py:1259-1290 */
static void k_reset(oracle_t *o, int ti, const int8_t *root_board, const int8_t *root_extra, int extra_len, int root_turn) {
    tree_t *t = &o->tr[ti];
    t->trees[0] = -1;
    t->size = 1;
    t->depths[0] = 0;
    t->turns[0] = (int8_t)root_turn;
    t->leaves[0] = 1;
    t->terminals[0] = 0;
    t->ns[0] = 0;
    t->ns_wins[0] = 0;
    memcpy(t->boards, root_board, (size_t)o->m * o->n);
    memset(t->extras, 0, (size_t)o->E);
    memcpy(t->extras, root_extra, (size_t)(extra_len < o->E ? extra_len : o->E));
}

/* _select, src/mctsnc.py:1292-1365 */
static void k_select(oracle_t *o, int ti) {
    tree_t *t = &o->tr[ti];
    const int A = o->A;
    float ucbs[512];
    int32_t node = 0; int depth = 0;
    t->path[0] = 0;
    while (!t->leaves[node]) {
        const int32_t *row = t->trees + (int64_t)node * (1 + A);
        for (int a = 0; a < A; a++) {
            int32_t child = row[1 + a];
            if (child == -1) ucbs[a] = -INFINITY;
            else ucbs[a] = mo_ucb(t->ns_wins[child], t->ns[child], t->ns[node], o->ucb_c);
        }
        int best = mo_argmax_tournament_f32(ucbs, A, 512);
        node = row[1 + best];
        depth++;
        t->path[depth] = node;
    }
    t->selected = node;
    t->path[MAX_TREE_DEPTH + 1] = depth + 1;
}

/* _expand_1_{ocp,acp}_{thrifty,prodigal}, src/mctsnc.py:1367-1681 */
static void k_expand_1(oracle_t *o, int ti) {
    tree_t *t = &o->tr[ti];
    const int A = o->A, mn = o->m * o->n;
    const int ocp = o->variant <= V_OCP_PRODIGAL;
    const int prodigal = (o->variant == V_OCP_PRODIGAL || o->variant == V_ACP_PRODIGAL);
    const int32_t selected = t->selected;
    uint8_t legal[512]; int16_t shifts[512]; int16_t map[512];
    memset(legal, 0, sizeof legal); memset(map, 0, sizeof map);
    const int8_t *board = t->boards + (int64_t)selected * mn;
    const int8_t *extra = t->extras + (int64_t)selected * o->E;
    const int terminal = t->terminals[selected];
    if (!terminal)
        for (int a = 0; a < A; a++) legal[a] = (uint8_t)is_action_legal(o, board, o->n, extra, a);
    const int32_t size_so_far = t->size;
    int16_t child_shift = -1, for_playout = -3;
    int16_t *ae = t->actions_expanded;
    for (int a = 0; a < A; a++) shifts[a] = -1;
    if (!terminal) {
        for (int i = 0; i < A; i++) {
            if (legal[i] && (int64_t)size_so_far + child_shift + 1 < o->max_tree_size) {
                child_shift++;
                map[child_shift] = (int16_t)i;
                shifts[i] = child_shift;
            }   /* a legal action that no longer fits gets no child: see file header */
        }
        if (child_shift >= 0) {
            ae[A + 1] = (int16_t)(child_shift + 1);
            t->leaves[selected] = 0;
            if (ocp) {
                float u = mo_rng_uniform(&o->rng_expand[(int64_t)ti * o->tpb_e1]);
                int16_t r = (int16_t)((double)u * (double)(child_shift + 1)); /* float32 * int64 -> float64 */
                if (r > child_shift) r = child_shift;                          /* u == 1.0f: see file header */
                for_playout = prodigal ? map[r] : r;
            } else for_playout = -2;
        } else ae[A + 1] = 1;
        ae[A] = for_playout;
    } else {
        ae[A + 1] = 1;
        ae[A] = -1;
    }
    tree_reserve(o, t, size_so_far + child_shift + 2);
    int32_t *row = t->trees + (int64_t)selected * (1 + A);
    for (int a = 0; a < A; a++) {
        int32_t child_index = -1;
        if (legal[a]) {
            int16_t cs = shifts[a];
            if (cs >= 0) {
                child_index = size_so_far + cs;
                if (prodigal) ae[a] = (int16_t)a; else ae[cs] = (int16_t)a;
            } else if (o->variant == V_ACP_PRODIGAL) ae[a] = -1;
        } else if (prodigal) ae[a] = -1;
        row[1 + a] = child_index;
    }
    t->size += child_shift + 1;
    if (!ocp && (terminal || for_playout == -3)) ae[0] = 0;
}

/* one block of _expand_2_{thrifty,prodigal}, src/mctsnc.py:1690-1821 */
static void k_expand_2_block(oracle_t *o, int ti, int action) {
    tree_t *t = &o->tr[ti];
    const int A = o->A, mn = o->m * o->n, E = o->E;
    const int32_t selected = t->selected;
    const int32_t child = t->trees[(int64_t)selected * (1 + A) + 1 + action];
    if (child < 0) return; /* stale row entry of an action that got no child in this step */
    int8_t *cb = t->boards + (int64_t)child * mn, *ce = t->extras + (int64_t)child * E;
    memcpy(cb, t->boards + (int64_t)selected * mn, (size_t)mn);
    memcpy(ce, t->extras + (int64_t)selected * E, (size_t)E);
    const int turn = t->turns[selected];
    take_action(o, cb, o->n, ce, turn, action);
    t->trees[(int64_t)child * (1 + A)] = selected;
    t->turns[child] = (int8_t)-turn;
    t->leaves[child] = 1;
    int outcome = compute_outcome(o, cb, o->n, ce, -turn, action);
    t->terminals[child] = (outcome == -1 || outcome == 0 || outcome == 1);
    t->outcomes[child] = (int8_t)outcome;
    t->ns[child] = 0;
    t->ns_wins[child] = 0;
    t->depths[child] = (int16_t)(t->depths[selected] + 1);
}

static void k_expand_2(oracle_t *o, int ti) {
    tree_t *t = &o->tr[ti];
    const int A = o->A;
    const int16_t *ae = t->actions_expanded;
    if (ae[A] == -1 || ae[A] == -3) return; /* :1766-1767; thrifty: see file header */
    if (t->terminals[t->selected]) return;
    if (o->variant == V_OCP_PRODIGAL || o->variant == V_ACP_PRODIGAL) {
        for (int a = 0; a < A; a++) if (ae[a] >= 0) k_expand_2_block(o, ti, a);
    } else {
        for (int i = 0; i < ae[A + 1]; i++) if (ae[i] >= 0) k_expand_2_block(o, ti, ae[i]);
    }
}

/* The playout blocks of one step for all trees: _playout_ocp (:1823-1902),
 * _playout_acp_thrifty (:1904-1991), _playout_acp_prodigal (:1993-2081). */
typedef struct { int ti, action; int32_t node; int last_action; int64_t rng_base; int32_t *dst; } pblock_t;

static void k_playouts(oracle_t *o) {
    const int A = o->A, P = o->P, mn = o->m * o->n, E = o->E, T = o->T;
    const int ocp = o->variant <= V_OCP_PRODIGAL;
    pblock_t *blocks = malloc(sizeof(pblock_t) * (size_t)T * (ocp ? 1 : A));
    int nb = 0;
    for (int ti = 0; ti < T; ti++) {
        tree_t *t = &o->tr[ti];
        const int16_t *ae = t->actions_expanded;
        const int32_t *row = t->trees + (int64_t)t->selected * (1 + A);
        if (ocp) {
            int32_t node = t->selected; int last_action = -1;
            if (ae[A] >= 0) { last_action = ae[ae[A]]; node = row[1 + last_action]; }
            if (t->terminals[node]) {
                int oc = t->outcomes[node];
                t->playout_outcomes[0] = oc == -1 ? P : 0;
                t->playout_outcomes[1] = oc == 1 ? P : 0;
            } else {
                pblock_t b = {ti, 0, node, last_action, (int64_t)ti * P, t->playout_outcomes};
                blocks[nb++] = b;
            }
        } else {
            const int prodigal = o->variant == V_ACP_PRODIGAL;
            const int nblk = prodigal ? A : ae[A + 1];
            for (int i = 0; i < nblk; i++) {
                int action = prodigal ? i : ae[i];
                if (prodigal && ae[i] < 0) continue;
                int32_t node = t->selected; int last_action = -1;
                const int fake = ae[A];
                if (fake == -2) { last_action = action; node = row[1 + action]; }
                if (t->terminals[node]) {
                    int oc = t->outcomes[node];
                    int32_t *dst = fake == -2 ? t->playout_outcomes_children + 2 * action : t->playout_outcomes;
                    dst[0] = oc == -1 ? P : 0;
                    dst[1] = oc == 1 ? P : 0;
                } else {
                    pblock_t b = {ti, action, node, last_action, ((int64_t)ti * A + action) * P,
                                  t->playout_outcomes_children + 2 * action};
                    blocks[nb++] = b;
                }
            }
        }
    }
    const int64_t total = (int64_t)nb * P;
    int32_t *res = calloc((size_t)nb * 2 + 2, sizeof(int32_t));
    uint64_t u1 = 0, plies = 0;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(o->threads) reduction(+ : u1, plies) if (o->threads > 1)
#endif
    for (int64_t w = 0; w < total; w++) {
        const pblock_t *b = &blocks[w / P];
        const tree_t *t = &o->tr[b->ti];
        int oc = playout(o, t->boards + (int64_t)b->node * mn, t->extras + (int64_t)b->node * E, t->turns[b->node],
                         b->last_action, &o->rng_playout[b->rng_base + (w % P)], &u1, &plies);
        if (oc != 0) {
#ifdef _OPENMP
#pragma omp atomic
#endif
            res[2 * (w / P) + (oc + 1) / 2] += 1;
        }
    }
    for (int i = 0; i < nb; i++) { blocks[i].dst[0] = res[2 * i]; blocks[i].dst[1] = res[2 * i + 1]; }
    o->u1_events += u1; o->plies += plies;
    free(res); free(blocks);
}

static void add_stats(tree_t *t, int32_t node, int32_t n, int32_t neg, int32_t pos) {
    t->ns[node] += n;
    t->ns_wins[node] += (t->turns[node] == 1) ? neg : pos;   /* :2099-2102 */
}

/* _backup_ocp (:2083-2114), _backup_1_acp_* (:2116-2194), _backup_2_acp (:2196-2220) */
static void k_backup(oracle_t *o, int ti) {
    tree_t *t = &o->tr[ti];
    const int A = o->A, P = o->P;
    const int16_t *ae = t->actions_expanded;
    const int32_t *row = t->trees + (int64_t)t->selected * (1 + A);
    const int path_length = t->path[MAX_TREE_DEPTH + 1];
    if (o->variant <= V_OCP_PRODIGAL) {
        const int32_t neg = t->playout_outcomes[0], pos = t->playout_outcomes[1];
        for (int e = 0; e < path_length; e++) add_stats(t, t->path[e], P, neg, pos);
        if (ae[A] >= 0) add_stats(t, row[1 + ae[ae[A]]], P, neg, pos);
    } else {
        if (ae[A] == -2) {
            int32_t sneg = 0, spos = 0;
            if (o->variant == V_ACP_THRIFTY) {
                for (int i = 0; i < ae[A + 1]; i++) {
                    int a = ae[i];
                    int32_t neg = t->playout_outcomes_children[2 * a], pos = t->playout_outcomes_children[2 * a + 1];
                    add_stats(t, row[1 + a], P, neg, pos);
                    sneg += neg; spos += pos;
                }
            } else {
                for (int a = 0; a < A; a++) {
                    if (ae[a] == -1) continue;
                    int32_t neg = t->playout_outcomes_children[2 * a], pos = t->playout_outcomes_children[2 * a + 1];
                    add_stats(t, row[1 + a], P, neg, pos);
                    sneg += neg; spos += pos;
                }
            }
            t->playout_outcomes[0] = sneg; t->playout_outcomes[1] = spos;
        }
        int n_expanded = ae[A + 1]; if (n_expanded == 0) n_expanded = 1;
        const int32_t neg = t->playout_outcomes[0], pos = t->playout_outcomes[1];
        for (int e = 0; e < path_length; e++) add_stats(t, t->path[e], P * n_expanded, neg, pos);
    }
}

/* lexicographic (win_flag, n, n_wins) tournament of _reduce_over_actions_* (:2318-2330, :2359-2370) */
int mo_argmax_tournament_lex(const uint8_t *flags, const int64_t *ns, const int64_t *ws, int count, int size) {
    uint8_t f[512]; int64_t n_[512], w[512]; int idx[512];
    for (int a = 0; a < size; a++) {
        idx[a] = a;
        f[a] = a < count ? flags[a] : 0; n_[a] = a < count ? ns[a] : 0; w[a] = a < count ? ws[a] : 0;
    }
    for (int stride = size >> 1; stride > 0; stride >>= 1)
        for (int a = 0; a < stride; a++) {
            int b = a + stride;
            if ((f[a] < f[b]) || (f[a] == f[b] && n_[a] < n_[b]) || (f[a] == f[b] && n_[a] == n_[b] && w[a] < w[b])) {
                idx[a] = idx[b]; f[a] = f[b]; n_[a] = n_[b]; w[a] = w[b];
            }
        }
    return idx[0];
}

/* _reduce_over_trees_* (:2222-2296) and _reduce_over_actions_* (:2298-2375) plus the host
 * remapping of the thrifty ordinal (:723). */
static void k_reduce(oracle_t *o, int root_turn) {
    const int A = o->A, T = o->T;
    const int thrifty = (o->variant == V_OCP_THRIFTY || o->variant == V_ACP_THRIFTY);
    const int16_t *rae = o->root_actions_expanded;
    memset(o->root_ns, 0, sizeof(int64_t) * A); memset(o->actions_ns, 0, sizeof(int64_t) * A);
    memset(o->actions_ns_wins, 0, sizeof(int64_t) * A); memset(o->actions_win_flags, 0, (size_t)A);
    const int nb = thrifty ? rae[A + 1] : A;
    for (int b = 0; b < nb; b++) {
        int action = thrifty ? rae[b] : b;
        if (!thrifty && rae[action] == -1) {
            /* sums stay zero; the win flag is still evaluated (:2295-2296) */
        } else {
            for (int ti = 0; ti < T; ti++) {
                tree_t *t = &o->tr[ti];
                o->root_ns[b] += t->ns[0];
                int32_t node = t->trees[1 + action];
                if (node >= 0) { o->actions_ns[b] += t->ns[node]; o->actions_ns_wins[b] += t->ns_wins[node]; }
            }
        }
        tree_t *t0 = &o->tr[0];
        int32_t node = t0->trees[1 + action];
        o->actions_win_flags[b] = (node != -1 && t0->terminals[node] && t0->outcomes[node] == root_turn);
    }
    const int size = next_pow2(A);
    int best = mo_argmax_tournament_lex(o->actions_win_flags, o->actions_ns, o->actions_ns_wins, nb, size);
    o->best_win_flag = best < nb ? o->actions_win_flags[best] : 0;
    o->best_n = best < nb ? o->actions_ns[best] : 0;
    o->best_n_wins = best < nb ? o->actions_ns_wins[best] : 0;
    o->best_action = thrifty ? rae[best] : best;
}

/* MCTSNC._run_<variant>, src/mctsnc.py:565-1257, with a fixed step budget */
int mo_run(oracle_t *o, const int8_t *root_board, const int8_t *root_extra, int extra_len, int root_turn, int64_t steps) {
    static const int8_t zero = 0;
    if (!root_extra) { root_extra = &zero; extra_len = 1; }
    for (int ti = 0; ti < o->T; ti++) k_reset(o, ti, root_board, root_extra, extra_len, root_turn);
    o->steps = 0;
    for (int64_t s = 0; s < steps; s++) {
        for (int ti = 0; ti < o->T; ti++) { k_select(o, ti); k_expand_1(o, ti); }
        if (s == 0) memcpy(o->root_actions_expanded, o->tr[0].actions_expanded, sizeof(int16_t) * (o->A + 2)); /* :1683-1688 */
        for (int ti = 0; ti < o->T; ti++) k_expand_2(o, ti);
        k_playouts(o);
        for (int ti = 0; ti < o->T; ti++) k_backup(o, ti);
        o->steps++;
    }
    k_reduce(o, root_turn);
    return o->best_action;
}

/* ---------------------------------------------------------------------------------------- accessors */
int32_t mo_tree_size(const oracle_t *o, int ti) { return o->tr[ti].size; }
int32_t mo_tree_selected(const oracle_t *o, int ti) { return o->tr[ti].selected; }
const void *mo_tree_array(const oracle_t *o, int ti, int which) {
    const tree_t *t = &o->tr[ti];
    switch (which) {
        case 0: return t->trees;
        case 1: return t->depths;
        case 2: return t->turns;
        case 3: return t->leaves;
        case 4: return t->terminals;
        case 5: return t->outcomes;
        case 6: return t->ns;
        case 7: return t->ns_wins;
        case 8: return t->boards;
        case 9: return t->extras;
        case 10: return t->path;
        case 11: return t->actions_expanded;
        case 12: return t->playout_outcomes;
        case 13: return t->playout_outcomes_children;
        default: return NULL;
    }
}
const void *mo_result_array(const oracle_t *o, int which) {
    switch (which) {
        case 0: return o->root_actions_expanded;
        case 1: return o->root_ns;
        case 2: return o->actions_ns;
        case 3: return o->actions_ns_wins;
        case 4: return o->actions_win_flags;
        default: return NULL;
    }
}
int32_t mo_best_action(const oracle_t *o) { return o->best_action; }
int32_t mo_best_win_flag(const oracle_t *o) { return o->best_win_flag; }
int64_t mo_best_n(const oracle_t *o) { return o->best_n; }
int64_t mo_best_n_wins(const oracle_t *o) { return o->best_n_wins; }
uint64_t mo_u1_events(const oracle_t *o) { return o->u1_events; }
uint64_t mo_plies(const oracle_t *o) { return o->plies; }
const rng_t *mo_rng_states(const oracle_t *o, int which) { return which == 0 ? o->rng_playout : o->rng_expand; }
