/*
 * mctsnc_hip.h -- C ABI of libmctsnc_hip.so, the MI355X (gfx950) MCTS-NC search engine.
 *
 * The reference implements this path as a Python class whose methods launch numba.cuda kernels
 * (src/mctsnc.py).  It has no C interface of its own for it, so each entry point below names the
 * reference method it stands in for; a Python (ctypes) class with the reference's constructor and
 * run() signature sits directly on top of these calls.
 *
 * Conventions: every function returns 0 on success and a negative MCTSNC_E_* code on failure;
 * mctsnc_last_error() returns a human-readable description of the last failure on the calling
 * thread.  All pointers are host pointers; the engine owns every device allocation.  One engine
 * may be used from one host thread at a time; several engines may coexist in a process.
 */
#ifndef MCTSNC_HIP_H
#define MCTSNC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MCTSNC_MAX_ACTIONS 512 /* MCTSNC.MAX_STATE_MAX_ACTIONS, src/mctsnc.py:193 */

enum { MCTSNC_GAME_C4 = 0, MCTSNC_GAME_GOMOKU = 1 };
/* order of MCTSNC.VARIANTS, src/mctsnc.py:180 */
enum { MCTSNC_OCP_THRIFTY = 0, MCTSNC_OCP_PRODIGAL = 1, MCTSNC_ACP_THRIFTY = 2, MCTSNC_ACP_PRODIGAL = 3 };

enum {
    MCTSNC_OK = 0,
    MCTSNC_E_INVALID = -1,     /* bad argument / unsupported configuration */
    MCTSNC_E_HIP = -2,         /* a HIP runtime call failed */
    MCTSNC_E_STATE = -3,       /* call order violated (e.g. run before init_device) */
    MCTSNC_E_ROOT = -4,        /* root position inconsistent with the game's rules */
    MCTSNC_E_DEVICE_SYNC = -5  /* the on-device step synchronisation timed out */
};

/* Constructor arguments of MCTSNC (src/mctsnc.py:199-204) after validation, plus the node-pool size that
 * init_device_side_arrays derives from device_memory (src/mctsnc.py:350-358). */
typedef struct mctsnc_config {
    int32_t game;               /* MCTSNC_GAME_* (the reference selects the game by editing source, src/mctsnc_game_mechanics.py:59-87) */
    int32_t board_m, board_n;   /* state_board_shape */
    int32_t extra_info_memory;  /* state_extra_info_memory, >= 1 */
    int32_t max_actions;        /* state_max_actions */
    int32_t n_trees;
    int32_t n_playouts;         /* power of two, <= 512 */
    int32_t variant;            /* MCTSNC_OCP_THRIFTY .. MCTSNC_ACP_PRODIGAL */
    float ucb_c;
    uint64_t seed;
    int64_t max_tree_size;      /* nodes per tree */
    int32_t device;             /* HIP device ordinal */
} mctsnc_config;

/* What run() leaves on the instance in the reference: best_* (src/mctsnc.py:1242-1247), the reduced root
 * table (dev_root_ns, dev_actions_*; :396-404), the memorised root expansion row (:1683-1688), step count,
 * timings (:448-470) and the tree statistics of _make_performance_info (:472-492). */
typedef struct mctsnc_result {
    int64_t steps;
    int32_t best_action;
    int32_t best_win_flag;
    int64_t best_n, best_n_wins;
    int32_t n_root_entries;                         /* thrifty: number of root actions; prodigal: max_actions */
    int16_t root_actions_expanded[MCTSNC_MAX_ACTIONS + 2];
    int64_t root_ns[MCTSNC_MAX_ACTIONS];
    int64_t actions_ns[MCTSNC_MAX_ACTIONS];
    int64_t actions_ns_wins[MCTSNC_MAX_ACTIONS];
    uint8_t actions_win_flags[MCTSNC_MAX_ACTIONS];
    double time_total, time_loop, time_reduce;      /* host wall clock, seconds */
    double time_device_loop;                        /* HIP-event time of the search kernels, seconds */
    int64_t depth_sum;                              /* sum of node depths over all trees */
    int64_t size_sum;                               /* sum of tree sizes */
    int32_t max_depth, max_size;
    uint64_t playout_plies;                         /* playout moves made during this run */
    uint64_t u1_events;                             /* playout draws that rounded up to 1.0f during this run */
    /* work counters summed over trees: tree levels walked by selection, children examined on those walks,
     * nodes created, nodes played out with real (non-terminal) playouts */
    uint64_t stat_levels, stat_children, stat_expanded, stat_played;
    /* per-stage device time of tree 0 in seconds (time_select/expand/playout/backup of the reference,
     * src/mctsnc.py:1121-1213); zero when stage timing is off */
    double time_select, time_expand, time_playout, time_backup;
    double time_exchange;   /* part of time_backup spent exchanging playout results between workgroups (incl. waiting) */
} mctsnc_result;

typedef struct mctsnc_engine mctsnc_engine;

/* MCTSNC.__init__ (src/mctsnc.py:199-276): validates the configuration; no device work. */
int mctsnc_create(const mctsnc_config *cfg, mctsnc_engine **out);

/* MCTSNC.init_device_side_arrays (src/mctsnc.py:318-407): allocates the node pools and seeds the
 * xoroshiro128+ streams exactly as create_xoroshiro128p_states does (stream i = stream i-1 jumped 2^64). */
int mctsnc_init_device(mctsnc_engine *e);

/* MCTSNC.run / _run_<variant> (src/mctsnc.py:409-434, :565-1257).  board: int8[m*n] row-major, values in
 * {-1, 0, +1}; extra: int8[extra_len] or NULL; turn: -1 or +1.  steps_limit / time_limit_s may be INFINITY;
 * forced_steps_limit < INFINITY overrides both (src/mctsnc.py:1112-1116).  Blocking. RNG streams carry over
 * from the previous run on the same engine, as in the reference.  Whatever the limits, a search ends after
 * floor((2^31 - 1) / (n_playouts * max_actions)) steps (one-child variants: / n_playouts), before an int32 visit
 * counter (the reference's dtype, src/mctsnc.py:334-335) could overflow. */
int mctsnc_run(mctsnc_engine *e, const int8_t *board, const int8_t *extra, int32_t extra_len, int32_t turn,
               double steps_limit, double time_limit_s, double forced_steps_limit, mctsnc_result *out);

/* Arrays of the last run in the reference's layout and dtypes, one tree at a time (what _json_dump copies
 * back, src/mctsnc.py:2393-2438).  mctsnc_read_size returns the byte size needed for (array_id, tree). */
enum {
    MCTSNC_ARR_TREES = 0,                     /* int32 [size][1 + A]: parent, children (-1 where absent) */
    MCTSNC_ARR_DEPTHS = 1,                    /* int16 [size] */
    MCTSNC_ARR_TURNS = 2,                     /* int8  [size] */
    MCTSNC_ARR_LEAVES = 3,                    /* uint8 [size] */
    MCTSNC_ARR_TERMINALS = 4,                 /* uint8 [size] */
    MCTSNC_ARR_OUTCOMES = 5,                  /* int8  [size] (root: 2) */
    MCTSNC_ARR_NS = 6,                        /* int32 [size] */
    MCTSNC_ARR_NS_WINS = 7,                   /* int32 [size] */
    MCTSNC_ARR_BOARDS = 8,                    /* int8  [size][m][n] */
    MCTSNC_ARR_EXTRA_INFOS = 9,               /* int8  [size][E] */
    MCTSNC_ARR_SELECTED_PATH = 10,            /* int32 [path_len] of the last step */
    MCTSNC_ARR_ACTIONS_EXPANDED = 11,         /* int16 [A + 2] of the last step */
    MCTSNC_ARR_PLAYOUT_OUTCOMES = 12,         /* int32 [2] */
    MCTSNC_ARR_PLAYOUT_OUTCOMES_CHILDREN = 13,/* int32 [A][2] (ACP variants) */
    MCTSNC_ARR_NODE_SELECTED = 14,            /* int32 [1] */
    MCTSNC_ARR_RNG_PLAYOUT = 15,              /* uint64 [n][2], whole array (tree argument ignored) */
    MCTSNC_ARR_RNG_EXPAND = 16                /* uint64 [n][2], OCP variants, whole array */
};
int64_t mctsnc_read_size(mctsnc_engine *e, int32_t array_id, int32_t tree);
int mctsnc_read(mctsnc_engine *e, int32_t array_id, int32_t tree, void *dst, size_t dst_bytes);

/* Re-creates the RNG streams from the engine's seed (what constructing a fresh MCTSNC + init_device_side_arrays
 * does to the generators, src/mctsnc.py:390-394). */
int mctsnc_reseed(mctsnc_engine *e);

/* Runs n engines of identical configuration concurrently, one search each, in a single device pass
 * (no counterpart in the reference, which runs one search at a time; results per engine equal those of
 * mctsnc_run; searches beyond what the device holds at once start as earlier ones finish).  boards: n * m*n bytes,
 * extras: n * extra_len bytes or NULL, turns: n entries. */
int mctsnc_run_batch(mctsnc_engine **engines, int32_t n, const int8_t *boards, const int8_t *extras, int32_t extra_len,
                     const int32_t *turns, double steps_limit, double time_limit_s, double forced_steps_limit,
                     mctsnc_result *out);

/* mctsnc_run_batch for callers that cannot allocate device memory while they run (tight serving loops, harnesses
 * that forbid hipMalloc; it has no counterpart in the reference).  Same arguments, same results, n >= 1.  The per-call
 * device buffers -- the gathered per-tree pointer records, the root positions and turns, the result blocks the
 * final reductions write -- come out of a static device array of MCTSNC_NOALLOC_SCRATCH_BYTES that the library holds
 * on every device it runs on until the process ends, instead of a hipMalloc / hipFree pair per call; the call makes
 * no hipMalloc, hipFree or other allocating device-runtime call (the engines' own pools were allocated by
 * mctsnc_init_device, which also looks up the array's address on the engine's device).  A batch whose buffers do not
 * fit is rejected with MCTSNC_E_INVALID and a message that states both sizes (Connect 4: 52 bytes per tree + 512 per
 * search, i.e. some 5000 searches of 4 trees; Gomoku 15x15: 140 bytes per tree + 6400 per search, i.e. some 500
 * searches of 8 trees).  All calls on one
 * device share the one array: a call that finds it in use by another host thread returns MCTSNC_E_STATE rather
 * than overwrite that call's buffers.  Every byte a call reads it has written first, so nothing needs clearing
 * between calls. */
#define MCTSNC_NOALLOC_SCRATCH_BYTES (4u << 20)
int mctsnc_run_batch_noalloc(mctsnc_engine **engines, int32_t n, const int8_t *boards, const int8_t *extras, int32_t extra_len,
                             const int32_t *turns, double steps_limit, double time_limit_s, double forced_steps_limit,
                             mctsnc_result *out);

/* How the search is laid out on the device and test hooks; none of them changes a search's results.  No counterpart in
 * the reference (it has one launch shape per kernel).  A batch call takes the options of its first engine.
 *   MCTSNC_OPT_AGENT_FENCES       1: the all-children kernels never take the shortcuts for trees whose workgroups share an
 *                                 XCC (full device-scope release and acquire every step: the path such trees take when
 *                                 they do not); 0 (default)
 *   MCTSNC_OPT_SOLO_TREES         Connect 4, all children: one workgroup per tree from this many trees of a pass on;
 *                                 0 = never, -1 (default) = by the number of trees per compute unit
 *   MCTSNC_OPT_SOLO_THREADS       threads of such a workgroup, a multiple of 64 up to 512; 0 (default) = by the playouts
 *   MCTSNC_OPT_TEAM_POOL          Connect 4, all children: a team's workgroups play their playouts as a pool of jobs on
 *                                 fewer lanes; 1 / 0 = always / never, -1 (default) = by the number of trees
 *   MCTSNC_OPT_TEAM_POOL_THREADS  lanes of such a workgroup, a multiple of 64 up to 512; 0 (default) = half the playouts
 *   MCTSNC_OPT_PREP_LEVELS        Gomoku, one child: the backup of paths up to this many levels is prepared during the
 *                                 playouts (at most 48); -1 (default) = 48
 *   MCTSNC_OPT_PLAIN_LAUNCH       1: the all-children kernels, whose workgroups wait for each other, are launched as
 *                                 ordinary kernels instead of cooperatively (same grid, sized to what the device keeps
 *                                 resident; what is given up is the runtime's guarantee of residency when other kernels
 *                                 share the device: a workgroup that never gets scheduled then ends the launch with
 *                                 MCTSNC_E_DEVICE_SYNC through the bounded waits).  For profilers that do not get along
 *                                 with the runtime's cooperative queue; 0 (default)
 *   MCTSNC_OPT_PROBE_STEPS        Connect 4 pass with more trees than stay resident: steps every tree runs before the
 *                                 searches are put in the order of what they cost; 0 = keep the order by stones,
 *                                 -1 (default) = a thirty-second of the step budget, 16 to 128
 *   MCTSNC_OPT_SPIN_LIMIT         polls after which a workgroup's wait for the others of its tree gives up and ends the
 *                                 launch (MCTSNC_E_DEVICE_SYNC); 0 (default) = 2^24.  1 makes the first wait that is not
 *                                 met at once give up: the hook with which the tests drive that path.
 * After MCTSNC_E_DEVICE_SYNC the search is void, the engines stay usable and their random streams are back at their
 * seeds (as after mctsnc_reseed). */
#define MCTSNC_OPT_AGENT_FENCES 0
#define MCTSNC_OPT_SOLO_TREES 1
#define MCTSNC_OPT_SOLO_THREADS 2
#define MCTSNC_OPT_TEAM_POOL 3
#define MCTSNC_OPT_TEAM_POOL_THREADS 4
#define MCTSNC_OPT_PREP_LEVELS 5
#define MCTSNC_OPT_PLAIN_LAUNCH 6
#define MCTSNC_OPT_PROBE_STEPS 7
#define MCTSNC_OPT_SPIN_LIMIT 8
#define MCTSNC_OPT_COUNT 9
int mctsnc_set_option(mctsnc_engine *e, int32_t option, int32_t value);

/* Switches the per-stage device timers on (default) or off. */
int mctsnc_set_stage_timing(mctsnc_engine *e, int32_t on);

void mctsnc_destroy(mctsnc_engine *e);
const char *mctsnc_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
