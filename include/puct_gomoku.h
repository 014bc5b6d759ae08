/*
 * C ABI of the Gomoku PUCT search loop with virtual loss (part of libpuct_hip.so, gfx950).
 *
 * The reference has no such loop: its PUCT kernels stop at selection (src/puct/puct_gpu_v3_cpp.cu:277-448) and backup
 * (src/puct/puct_gpu_v2.py:847-927) on synthetic trees.  This engine puts the step between them — committing the
 * claimed expansion slot, creating the child position, evaluating it — around the same selection and backup rules, for
 * Gomoku with the rules of the reference's game plugin (five in a row exactly,
 * src/mctsnc_game_mechanics.py:181-280) and a synthetic evaluator (Dirichlet priors over the legal cells and a value,
 * both pure functions of the position).
 *
 * One step = every tree runs `traversals` selections with virtual loss between them, then expands / evaluates the
 * selected leaves, then backs the values up.  All steps of a search run inside one kernel launch, one workgroup per
 * tree and one 64-lane wavefront per traversal.
 *
 * Selection.  Every decision of a traversal is the reference's (src/puct/puct_gpu_v3_cpp.cu:150-275): progressive
 * widening from the node's visits plus claims in flight, capped by the node's number of empty cells; an expansion
 * ticket if widening allows another child; otherwise the edge with the highest score q + cpuct * prior *
 * sqrt(parent) / (n + in flight + 1), ties broken by the edge index rotated by the traversal's number; one unit of
 * virtual loss on the chosen edge.  What this loop fixes, and the reference's kernel leaves to the timing of its
 * atomics, is the order in which the traversals of a tree take their claims: they descend in lockstep, one level per
 * round, and the traversals standing on the same node decide one after another, traversal number ascending, each
 * seeing the claims and tickets of those before it.  That is one of the interleavings the reference's kernel allows; a
 * claim taken in turn never loses, so the reference's winner-recalc retry and soft winner have nothing to do here, and a
 * search is reproducible: the same configuration gives the same trees, bit for bit, on every run.  A traversal ends BUSY
 * when it reaches a node that has no child yet and whose only allowed child is being created by a traversal before it;
 * it keeps its claims until the step's backup gives them back (no traversal of the same step reads those edges again).
 * With c_pw >= traversals a node without children admits one ticket per traversal and nothing ends BUSY.
 *
 * Storage is the loop's own, not the [trees, nodes, edges] arrays of the selection launcher (include/puct_select.h): one
 * 16-byte record per edge (visits, value sum, prior, child and claims in flight), one per node, up to 2^20 nodes per
 * tree; puct_gomoku_read() hands the fields out in the launcher's array shapes.
 *
 * All functions return 0 on success or a negative error code; puct_gomoku_last_error() describes the last failure
 * of the calling thread.  Host pointers only; the engine owns its device memory.
 */
#ifndef PUCT_GOMOKU_H
#define PUCT_GOMOKU_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PUCT_GOMOKU_OK 0
#define PUCT_GOMOKU_E_INVALID (-1)
#define PUCT_GOMOKU_E_HIP (-2)
#define PUCT_GOMOKU_E_ROOT (-3)
#define PUCT_GOMOKU_E_SYNC (-4)   /* workgroups of the search launch waited for each other in vain; the search was abandoned */

#define PUCT_GOMOKU_MAX_NODES (1 << 20)
#define PUCT_GOMOKU_MAX_PATH_DEPTH 256

/* Selection word of a traversal (array PUCT_GOMOKU_ARR_OUT_SELECTED): kind << 28 | expansion slot << 20 | node, kinds
 * as in include/puct_select.h (invalid 0, expand 1, terminal 2, depth limit 3, busy 4); node = all ones when the
 * traversal reached no node. */
#define PUCT_GOMOKU_SEL_NODE_MASK 0xFFFFF
#define PUCT_GOMOKU_SEL_SLOT_SHIFT 20
#define PUCT_GOMOKU_SEL_KIND_SHIFT 28

typedef struct {
    int32_t board_m, board_n;  /* rows, columns; m * n <= 256 */
    int32_t trees;             /* independent trees on the same root, each with its own synthetic evaluator */
    int32_t traversals;        /* selections per tree and step, 1..16 */
    int32_t max_nodes;         /* node capacity per tree, 2..2^20 */
    int32_t path_depth;        /* longest path a selection may take, 1..256 */
    float cpuct, c_pw, alpha_pw;
    float dirichlet_alpha;     /* in (0, 1) */
    uint64_t seed;
    int32_t device;
    int32_t evaluators;        /* 0..8: workgroups per tree that work out the priors of the step's new nodes on other
                                  compute units while the tree's own workgroup backs the step up (fused search only; fewer
                                  are used when the device cannot keep trees * (1 + evaluators) workgroups resident);
                                  0 = the tree's workgroup does it itself.  The trees are the same either way. */
    int32_t agent_fences;      /* 0: a tree and its evaluators hand over through the L2 they share when they find themselves
                                  on one XCD (they report where they run, and write the L2 back until all have), 1: they always
                                  write the L2 back, as they must on different XCDs.  Same trees either way; 1 is slower. */
} puct_gomoku_config;

typedef struct {
    int64_t steps;
    int32_t best_action;             /* cell with the most root visits over all trees (smallest index on ties), -1 if none */
    int64_t best_n;
    int64_t root_n[256];             /* visits per cell, summed over trees */
    double root_w[256];              /* value sums per cell (for the player to move at the root), summed over trees */
    int64_t selections[5];           /* per kind: invalid, expand, terminal, depth limit, busy */
    int64_t expansions_committed;    /* children created */
    int64_t nodes_total;             /* nodes over all trees after the search */
    int32_t max_nodes_in_tree;
    double time_total, time_device;  /* seconds */
    int64_t nodes_read;              /* node visits of the selections that loaded the node (its word and its expanded edges);
                                        traversals standing on the same node in the same round share one */
    int64_t edges_scored;            /* expanded edges loaded on those visits */
    double time_select, time_expand, time_backup; /* seconds of time_device per phase (fused search only; mean over the
                                        trees of what the first wavefront of each tree's workgroup measured) */
} puct_gomoku_result;

typedef struct puct_gomoku_engine puct_gomoku_engine;

int puct_gomoku_create(const puct_gomoku_config *config, puct_gomoku_engine **out);
void puct_gomoku_destroy(puct_gomoku_engine *engine);

/* Searches from `board` (int8 [m, n]: 0 empty, +1 / -1 stones) with `turn` (+1 / -1) to move for `steps` steps.
 * fused != 0: one kernel launch for the whole search; fused == 0: three launches per step (selection, expansion /
 * evaluation, backup) — same results.
 * Edge slots: an expansion puts the child into the node's next free edge slot, in traversal order (slots are in
 * descending prior order); the slot field of the selection word is the ticket that entitled the traversal to expand.
 * Node limit: a tree holds at most max_nodes nodes.  The expansions a step selects in one tree are committed together
 * or not at all: once they no longer all fit, none of that step is committed in that tree, each of those traversals
 * evaluates the node it reached as a leaf instead (the evaluator's value of its position), backs that value up its
 * path and gives its expansion ticket back (a traversal that was asked to widen the root itself has an empty path and
 * leaves no visit).  The search then goes on over a tree that no longer grows: node_count stays within
 * `traversals` of max_nodes and never exceeds it, nothing is left in flight, and result->expansions_committed stays
 * nodes_total - trees. */
int puct_gomoku_run(puct_gomoku_engine *engine, const int8_t *board, int32_t turn, int32_t steps, int32_t fused,
                    puct_gomoku_result *result);

/* Copies one array of the last search to the host (edge and node fields are gathered from their records on the device
 * first).  Shapes (T trees, N = max_nodes, E = 256, W traversals, D = path_depth): see the ids below.  `bytes` must equal
 * the array's size.  Rows of nodes that were never created hold no defined values. */
#define PUCT_GOMOKU_ARR_EDGE_CHILD 0       /* int32 [T, N, E]: -1 = no child */
#define PUCT_GOMOKU_ARR_EDGE_PRIOR 1       /* float32 [T, N, E] */
#define PUCT_GOMOKU_ARR_EDGE_W 2           /* float32 [T, N, E] */
#define PUCT_GOMOKU_ARR_EDGE_N 3           /* int32 [T, N, E] */
#define PUCT_GOMOKU_ARR_EDGE_INFLIGHT 4    /* int32 [T, N, E] */
#define PUCT_GOMOKU_ARR_EDGE_ACTION 5      /* uint8 [T, N, E] */
#define PUCT_GOMOKU_ARR_NODE_EXPANDED 6    /* int32 [T, N] */
#define PUCT_GOMOKU_ARR_NODE_EXPAND_INFLIGHT 7 /* int32 [T, N] */
#define PUCT_GOMOKU_ARR_NODE_COUNT 8       /* int32 [T] */
#define PUCT_GOMOKU_ARR_NODE_BOARD 9       /* uint32 [T, N, 16]: words 0..7 stones of +1, 8..15 stones of -1 */
#define PUCT_GOMOKU_ARR_NODE_TURN 10       /* int8 [T, N] */
#define PUCT_GOMOKU_ARR_NODE_VALUE 11      /* float32 [T, N]: value of a terminal node for its player to move */
#define PUCT_GOMOKU_ARR_OUT_SELECTED 12    /* int32 [T, W]: last step */
#define PUCT_GOMOKU_ARR_OUT_PATH 13        /* int32 [T, W, D]: last step, node << 8 | edge slot per level, -1 beyond the path */
#define PUCT_GOMOKU_ARR_OUT_LEN 14         /* int32 [T, W]: last step */
#define PUCT_GOMOKU_ARR_PATH_VALUES 15     /* float32 [T, W, D]: last step */
#define PUCT_GOMOKU_ARR_NODE_LEGAL 16      /* int32 [T, N]: empty cells of the node's position = most children it can have */
int64_t puct_gomoku_array_bytes(puct_gomoku_engine *engine, int32_t array_id);
int puct_gomoku_read(puct_gomoku_engine *engine, int32_t array_id, void *dst, size_t bytes);

const char *puct_gomoku_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
