/*
 * CPU oracle of the PUCT selection / backup path with virtual loss.  TEST INFRASTRUCTURE ONLY: nothing that ships may
 * link, load or call this file; the tests and the benchmark's CPU-baseline leg use it as the checker.
 *
 * Restates, as plain sequential C over host arrays, the algorithm of
 *   - puct_select_winner_recalc_kernel, src/puct/puct_gpu_v3_cpp.cu:277-448 (helpers :38-275);
 *   - _select_kernel_native and _select_kernel_winner_recalc, src/puct/puct_gpu_v2.py:573-840 (helpers :109-566);
 *   - _backup_kernel_native, src/puct/puct_gpu_v2.py:847-927;
 *   - _release_claims_kernel, src/puct/test_puct_gpu_v3.py:275-333 (edge-level claim release).
 *
 * The reference runs the traversals of one launch concurrently and its outcome depends on how their atomics
 * interleave.  This oracle runs them one after another, tree by tree and wid ascending, which is ONE of the legal
 * interleavings: a launch with a single traversal per tree must reproduce it exactly; a launch with several can only
 * be held to the invariants that every interleaving satisfies.
 *
 * Pins: the known answers of the reference's own kernel tests (src/puct/test_puct_gpu_v3.py:1154-1416,
 * src/puct/test_puct_gpu_v2.py:1006-1166) and hand-computed PUCT scores in tests/test_puct_oracle.py.
 * Parity unpinned: alpha_pw other than 0.5 (powf differs between math libraries in the last bit).
 */
#include <float.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>

#define TERMINAL (-1)
#define NODE_LIMIT 16384
#define NODE_MASK 0x3FFF
#define EDGE_MASK 0xFF
#define SLOT_SHIFT 14
#define KIND_SHIFT 22
#define KIND_MASK 0x7
#define REASON_SHIFT 25

enum { K_INVALID = 0, K_EXPAND = 1, K_TERMINAL = 2, K_DEPTH_LIMIT = 3, K_BUSY = 4 };
enum {
    R_UNSET = 0, R_OK_EXPAND = 1, R_OK_TERMINAL = 2, R_OK_DEPTH_LIMIT = 3, R_BUSY_EXPAND = 4, R_BUSY_RECALC = 5,
    R_SHAPE = 10, R_NODE_INFO = 11, R_NO_EDGE = 14, R_CHILD_OOB = 15, R_UNKNOWN = 16
};

static int pack(int kind, int node, int slot, int reason) {
    return (reason << REASON_SHIFT) | (kind << KIND_SHIFT) | (slot << SLOT_SHIFT) | node;
}

/* src/puct/puct_gpu_v3_cpp.cu:150-157 */
static int allowed_children(float c_pw, float alpha_pw, int n_node, int edges) {
    float val = (alpha_pw == 0.5f) ? c_pw * sqrtf((float)n_node) : c_pw * powf((float)n_node, alpha_pw);
    if (val >= (float)edges) return edges;
    int allowed = (int)ceilf(val);
    return allowed > 1 ? allowed : 1;
}

/* src/puct/puct_gpu_v3_cpp.cu:51-71: is (score, eid) ahead of (best_score, best_eid)? */
static int ahead(float score, int eid, float best_score, int best_eid, int tie_offset, int span) {
    if (score > best_score) return 1;
    if (score == best_score) {
        if (best_eid == INT32_MAX) return 1;
        int ka = eid - tie_offset, kb = best_eid - tie_offset;
        if (ka < 0) ka += span;
        if (kb < 0) kb += span;
        return ka < kb;
    }
    return 0;
}

static void rollback(int *edge_inflight, const int *path, int depth, size_t tree_row, int node_cnt, int edges) {
    for (int d = 0; d < depth; ++d) {
        int parent = path[d] >> 8, slot = path[d] & 0xFF;
        if (parent >= 0 && parent < node_cnt && slot < edges) edge_inflight[(tree_row + parent) * edges + slot] -= 1;
    }
}

/* One traversal (tree, wid) run to completion. */
static void select_one(float cpuct, float c_pw, float alpha_pw, int soft_winner, const int *edge_child_id,
                       const float *edge_prior, const float *edge_W, const int *edge_N, int *edge_inflight,
                       int *node_expand_inflight, const int *node_expanded, int node_cnt, int *out_selected,
                       int *path, int *out_len, int tree, int wid, int nodes, int edges, int path_depth,
                       const int *node_capacity) {
    (void)soft_winner; /* a sequential claim never loses its compare-and-swap, so the soft fallback cannot trigger */
    *out_selected = pack(K_INVALID, NODE_MASK, 0, R_UNSET);
    *out_len = 0;
    if (!(path_depth >= 1 && nodes > 0 && node_cnt > 0 && node_cnt <= nodes && node_cnt <= NODE_LIMIT && edges > 0 &&
          edges <= EDGE_MASK + 1)) {
        *out_selected = pack(K_INVALID, NODE_MASK, 0, R_SHAPE);
        return;
    }
    const size_t tree_row = (size_t)tree * nodes;
    int packed = pack(K_INVALID, NODE_MASK, 0, R_UNKNOWN), len = 0, node = 0, depth = 0;
    for (;;) {
        const size_t nrow = tree_row + node, erow = nrow * edges;
        const int info = node_expanded[nrow];
        if (info == TERMINAL) {
            packed = pack(K_TERMINAL, node, 0, R_OK_TERMINAL);
            len = depth + 1;
            break;
        }
        if (info < 0 || info > edges) {
            rollback(edge_inflight, path, depth, tree_row, node_cnt, edges);
            packed = pack(K_INVALID, NODE_MASK, 0, R_NODE_INFO);
            break;
        }
        if (depth >= path_depth) {
            packed = pack(K_DEPTH_LIMIT, node, 0, R_OK_DEPTH_LIMIT);
            len = depth + 1;
            break;
        }
        const int expanded = info;
        int parent_eff = 1, allowed = 1;
        if (expanded != 1 || c_pw != 0.0f) {
            int total = 0;
            for (int e = 0; e < expanded; ++e) total += edge_N[erow + e] + edge_inflight[erow + e];
            parent_eff = total > 1 ? total : 1;
            allowed = allowed_children(c_pw, alpha_pw, parent_eff, node_capacity ? node_capacity[nrow] : edges);
        }
        if (allowed > expanded) {
            int slot = -1;
            if (expanded + node_expand_inflight[nrow] < allowed) {
                const int ticket = node_expand_inflight[nrow]++;
                if (expanded + ticket < allowed) slot = expanded + ticket;
                else node_expand_inflight[nrow]--;
            }
            if (slot >= 0) {
                packed = pack(K_EXPAND, node, slot, R_OK_EXPAND);
                len = depth + 1;
                break;
            }
            if (expanded == 0) {
                rollback(edge_inflight, path, depth, tree_row, node_cnt, edges);
                packed = pack(K_BUSY, node, 0, R_BUSY_EXPAND);
                break;
            }
        }
        int tie_offset = wid;
        if (tie_offset >= expanded) tie_offset %= expanded;
        int best = 0, held = 0;
        if (expanded == 1) {
            edge_inflight[erow] += 1;
            held = 1;
        } else {
            const float sqrt_parent = sqrtf((float)parent_eff);
            float best_score = -FLT_MAX;
            best = INT32_MAX;
            for (int e = 0; e < expanded; ++e) {
                const int n = edge_N[erow + e];
                const float q = n > 0 ? edge_W[erow + e] / (float)n : 0.0f;
                const float u = cpuct * edge_prior[erow + e] * sqrt_parent / (float)(n + edge_inflight[erow + e] + 1);
                const float score = q + u;
                if (ahead(score, e, best_score, best, tie_offset, expanded)) {
                    best_score = score;
                    best = e;
                }
            }
            if (best != INT32_MAX) {
                edge_inflight[erow + best] += 1;
                held = 1;
            }
        }
        if (!held) {
            rollback(edge_inflight, path, depth, tree_row, node_cnt, edges);
            packed = pack(K_INVALID, NODE_MASK, 0, R_NO_EDGE);
            break;
        }
        const int child = edge_child_id[erow + best];
        if (child < 0 || child >= node_cnt) {
            edge_inflight[erow + best] -= 1;
            rollback(edge_inflight, path, depth, tree_row, node_cnt, edges);
            packed = pack(K_INVALID, NODE_MASK, 0, R_CHILD_OOB);
            break;
        }
        path[depth] = (node << 8) | best;
        node = child;
        depth += 1;
    }
    *out_selected = packed;
    *out_len = len;
}

/* node_capacity: optional int32 [trees, nodes] limit on the children of each node (NULL = `edges`, the reference). */
static void select_all(float cpuct, float c_pw, float alpha_pw, int soft_winner, const int *edge_child_id,
                       const float *edge_prior, const float *edge_W, const int *edge_N, int *edge_inflight,
                       int *node_expand_inflight, const int *node_expanded, const int *tree_nodes,
                       int *out_selected_node, int *out_path_eids, int *out_path_len, int trees, int nodes, int edges,
                       int warps, int path_depth, const int *node_capacity) {
    for (int tree = 0; tree < trees; ++tree)
        for (int wid = 0; wid < warps; ++wid) {
            const size_t out = (size_t)tree * warps + wid;
            select_one(cpuct, c_pw, alpha_pw, soft_winner, edge_child_id, edge_prior, edge_W, edge_N, edge_inflight,
                       node_expand_inflight, node_expanded, tree_nodes[tree], out_selected_node + out,
                       out_path_eids + out * path_depth, out_path_len + out, tree, wid, nodes, edges, path_depth,
                       node_capacity);
        }
}

void po_select(float cpuct, float c_pw, float alpha_pw, int soft_winner, const int *edge_child_id,
               const float *edge_prior, const float *edge_W, const int *edge_N, int *edge_inflight,
               int *node_expand_inflight, const int *node_expanded, const int *tree_nodes, int *out_selected_node,
               int *out_path_eids, int *out_path_len, int trees, int nodes, int edges, int warps, int path_depth) {
    select_all(cpuct, c_pw, alpha_pw, soft_winner, edge_child_id, edge_prior, edge_W, edge_N, edge_inflight,
               node_expand_inflight, node_expanded, tree_nodes, out_selected_node, out_path_eids, out_path_len, trees,
               nodes, edges, warps, path_depth, NULL);
}

/* ---------------------------------------------------------------------------------------------------------------------
 * Selection with node-level virtual loss: _select_kernel_native (preclaim != 0) and _select_kernel_winner_recalc
 * (preclaim == 0) of src/puct/puct_gpu_v2.py:573-840 with their helpers (:109-566), one traversal after another.
 * Sequentially, a preclaim that claims every candidate, scores it with the count found and releases the losers comes
 * to: score every candidate with its child's present count, then claim the winner; the counter compare-and-swap of
 * the winner-recalc variant never loses, and its conflict bit is "the child already carried claims".
 * Selection word: (kind << 22) | (slot << 14) | node, PACKED_INVALID = 0x3FFF with length 0 for every failure.
 * Pins: the known answers of src/puct/test_puct_gpu_v2.py:1006-1166 and hand-computed scores in
 * tests/test_puct_node_oracle.py.
 * ------------------------------------------------------------------------------------------------------------------ */
static void node_rollback(const int *edge_child_id, int *node_inflight, const int *path, int depth, size_t tree_row,
                          int limit, int edges) {
    for (int d = 0; d < depth; ++d) {      /* :291-310 */
        if (path[d] < 0) continue;
        const int parent = path[d] >> 8, slot = path[d] & 0xFF;
        if (parent < limit && slot < edges) {
            const int child = edge_child_id[(tree_row + parent) * edges + slot];
            if (child >= 0 && child < limit) node_inflight[tree_row + child] -= 1;
        }
    }
}

/* :420-445 / :448-472: the best candidate edge by (score, tie key), skipping `skip`; INT32_MAX when there is none */
static int node_best_edge(float cpuct, const int *edge_child_id, const float *edge_prior, const float *edge_W,
                          const int *edge_N, const int *node_inflight, size_t tree_row, size_t erow, int expanded,
                          int limit, float sqrt_parent, int skip, int tie_offset) {
    float best_score = -FLT_MAX;
    int best = INT32_MAX;
    for (int e = 0; e < expanded; ++e) {
        const int child = edge_child_id[erow + e];
        if (e == skip || child < 0 || child >= limit) continue;
        const int n = edge_N[erow + e];
        const float q = n > 0 ? edge_W[erow + e] / (float)n : 0.0f;
        const float u = cpuct * edge_prior[erow + e] * sqrt_parent / (float)(n + node_inflight[tree_row + child] + 1);
        const float score = q + u;
        if (ahead(score, e, best_score, best, tie_offset, expanded)) {
            best_score = score;
            best = e;
        }
    }
    return best;
}

static void node_select_one(int preclaim, float cpuct, float c_pw, float alpha_pw, const int *edge_child_id,
                            const float *edge_prior, const float *edge_W, const int *edge_N, int *node_inflight,
                            int *node_expand_inflight, const int *node_expanded, int limit, int *out_selected, int *path,
                            int *out_len, int tree, int wid, int nodes, int edges, int path_depth) {
    *out_selected = (K_INVALID << KIND_SHIFT) | NODE_MASK;
    *out_len = 0;
    if (!(path_depth >= 1 && nodes > 0 && limit > 0 && limit <= nodes && limit <= NODE_LIMIT && edges > 0 &&
          edges <= EDGE_MASK + 1))
        return;                                                                   /* :357-366 */
    const size_t tree_row = (size_t)tree * nodes;
    int node = 0, depth = 0;
    for (;;) {
        if (node < 0 || node >= limit) {
            node_rollback(edge_child_id, node_inflight, path, depth, tree_row, limit, edges);
            return;
        }
        if (depth >= path_depth) {
            *out_selected = (K_DEPTH_LIMIT << KIND_SHIFT) | node;
            *out_len = depth + 1;
            return;
        }
        const size_t nrow = tree_row + node, erow = nrow * edges;
        const int info = node_expanded[nrow];
        if (info == TERMINAL) {
            *out_selected = (K_TERMINAL << KIND_SHIFT) | node;
            *out_len = depth + 1;
            return;
        }
        if (info < 0 || info > edges) {
            node_rollback(edge_child_id, node_inflight, path, depth, tree_row, limit, edges);
            return;
        }
        const int expanded = info;
        int total = 0;                                                            /* :407-416 */
        for (int e = 0; e < expanded; ++e) {
            const int child = edge_child_id[erow + e];
            if (child >= 0 && child < limit) total += edge_N[erow + e] + node_inflight[tree_row + child];
        }
        const int parent_eff = total > 1 ? total : 1;
        const int allowed = (preclaim && expanded == 0) ? 1 : allowed_children(c_pw, alpha_pw, parent_eff, edges);
        if (allowed > expanded) {                                                 /* :389-403 */
            const int ticket = node_expand_inflight[nrow]++;
            if (expanded + ticket < allowed) {
                *out_selected = (K_EXPAND << KIND_SHIFT) | ((expanded + ticket) << SLOT_SHIFT) | node;
                *out_len = depth + 1;
            } else {
                node_expand_inflight[nrow]--;
                node_rollback(edge_child_id, node_inflight, path, depth, tree_row, limit, edges);
            }
            return;
        }
        const float sqrt_parent = sqrtf((float)parent_eff);
        int best, held = 0;
        if (preclaim) {
            int tie_offset = wid;
            if (tie_offset >= expanded) tie_offset %= expanded;
            best = node_best_edge(cpuct, edge_child_id, edge_prior, edge_W, edge_N, node_inflight, tree_row, erow, expanded,
                                  limit, sqrt_parent, -1, tie_offset);
            if (best != INT32_MAX) {
                node_inflight[tree_row + edge_child_id[erow + best]] += 1;
                held = 1;
            }
        } else {
            int skip = -1;
            best = INT32_MAX;
            for (int retry = 0; retry < 2; ++retry) {                             /* :520-560, MAX_RECALC_RETRY = 2 */
                best = node_best_edge(cpuct, edge_child_id, edge_prior, edge_W, edge_N, node_inflight, tree_row, erow,
                                      expanded, limit, sqrt_parent, skip, 0);
                if (best == INT32_MAX) {
                    if (skip < 0) break;
                    best = skip;
                }
                int *counter = &node_inflight[tree_row + edge_child_id[erow + best]];
                if (*counter < 0 || *counter >= INT32_MAX) break;                 /* :329-331: not claimable */
                const int conflict = *counter > 0;
                *counter += 1;
                held = 1;
                if (!conflict || expanded <= 1 || retry + 1 >= 2) break;
                *counter -= 1;
                skip = best;
                held = 0;
            }
        }
        if (!held) {
            node_rollback(edge_child_id, node_inflight, path, depth, tree_row, limit, edges);
            return;
        }
        path[depth] = (node << 8) | best;
        node = edge_child_id[erow + best];
        depth += 1;
    }
}

void po_node_select(int preclaim, float cpuct, float c_pw, float alpha_pw, const int *edge_child_id,
                    const float *edge_prior, const float *edge_W, const int *edge_N, int *node_inflight,
                    int *node_expand_inflight, const int *node_expanded, const int *node_count, int *out_selected_node,
                    int *out_path_eids, int *out_path_len, int trees, int nodes, int edges, int warps, int path_depth) {
    for (int tree = 0; tree < trees; ++tree)
        for (int wid = 0; wid < warps; ++wid) {
            const size_t out = (size_t)tree * warps + wid;
            node_select_one(preclaim, cpuct, c_pw, alpha_pw, edge_child_id, edge_prior, edge_W, edge_N, node_inflight,
                            node_expand_inflight, node_expanded, node_count[tree], out_selected_node + out,
                            out_path_eids + out * path_depth, out_path_len + out, tree, wid, nodes, edges, path_depth);
        }
}

/* node_level != 0: src/puct/puct_gpu_v2.py:847-927 as written.  node_level == 0: the same conversion applied to
 * edge-level claims (src/puct/test_puct_gpu_v3.py:275-333 for the release, statistics as in the v2 kernel). */
void po_backup(int node_level, int virtual_loss, const int *edge_child_id, float *edge_W, int *edge_N,
               int *edge_inflight, int *node_inflight, int *node_expand_inflight, const int *node_count,
               const int *out_selected_node, const int *out_path_eids, const int *out_path_len,
               const float *path_edge_values, int trees, int nodes, int edges, int warps, int path_depth) {
    for (int tree = 0; tree < trees; ++tree) {
        const int limit = node_count[tree];
        if (limit <= 0 || limit > nodes || limit > NODE_LIMIT) continue;
        const size_t tree_row = (size_t)tree * nodes;
        for (int wid = 0; wid < warps; ++wid) {
            const size_t out = (size_t)tree * warps + wid;
            const int raw = out_selected_node[out];
            if (raw < 0) continue;
            const int kind = node_level ? raw >> KIND_SHIFT : (raw >> KIND_SHIFT) & KIND_MASK;
            if (kind == K_INVALID || (!node_level && kind == K_BUSY)) continue;
            const int plen = out_path_len[out];
            if (plen <= 0) continue;
            int count = plen - 1;
            if (count > path_depth) count = path_depth;
            for (int d = 0; d < count; ++d) {
                const int enc = out_path_eids[out * path_depth + d];
                if (enc < 0) continue;
                const int parent = enc >> 8, slot = enc & 0xFF;
                if (parent >= limit || slot >= edges) continue;
                const size_t e = (tree_row + parent) * edges + slot;
                if (node_level) {
                    const int child = edge_child_id[e];
                    if (child >= 0 && child < limit) node_inflight[tree_row + child] -= virtual_loss;
                } else {
                    edge_inflight[e] -= virtual_loss;
                }
                if (path_edge_values) {
                    edge_N[e] += 1;
                    edge_W[e] += path_edge_values[out * path_depth + d];
                }
            }
            if (kind == K_EXPAND) {
                const int leaf = raw & NODE_MASK;
                if (leaf < limit) node_expand_inflight[tree_row + leaf] -= 1;
            }
        }
    }
}

/* ---------------------------------------------------------------------------------------------------------------------
 * Gomoku PUCT loop (selection -> expansion / evaluation -> backup per step).  The reference has no such loop; this
 * restates the library's own definition (include/puct_gomoku.h) as plain scalar code, so it is a second
 * implementation of the same specification rather than a restatement of reference code: PARITY UNPINNED against the
 * reference.  The synthetic evaluator (hash, value, Gamma weights) is shared with the library through its header,
 * because it is the definition of the workload's inputs; what is restated here is the tree logic.  Pins:
 * tests/test_puct_oracle.py checks the rules (five in a row exactly) against the brute-force outcome routine of the
 * MCTS-NC oracle, the priors against the Dirichlet moments, and structural invariants of the trees.
 *
 * The order in which the traversals of one step take their claims is part of that definition (it makes a search
 * reproducible): the traversals of a tree descend in lockstep, one level per round; within a round the traversals
 * standing on the same node decide one after another, wid ascending, each seeing the claims and expansion tickets of
 * those before it.  Every single decision is the reference's (src/puct/puct_gpu_v3_cpp.cu:150-275: progressive
 * widening, expansion ticket, score, order on edges with the rotated tie-break); a claim that is taken in turn never
 * loses, so the winner-recalc retry and the soft winner have nothing to do.  A traversal that ends BUSY keeps its
 * claims until the step's backup releases them (the reference's kernel rolls them back at once; no traversal of the
 * same step reads those edges again, so the difference cannot be observed).
 * ------------------------------------------------------------------------------------------------------------------ */
#include "../mcts_numba_cuda_amd/csrc/puct_synthetic.h"

#define G_EDGES 256
#define G_WORDS 16
#define G_MAX_WARPS 16
/* selection word of the loop: kind << 28 | slot << 20 | node (include/puct_gomoku.h) */
#define G_NODE_MASK 0xFFFFF
#define G_SLOT_SHIFT 20
#define G_KIND_SHIFT 28

typedef struct {
    int *edge_child; float *edge_prior; float *edge_w; int *edge_n; int *edge_inflight; uint8_t *edge_action;
    int *node_expanded; int *node_expand_inflight; int *node_count; uint32_t *node_board; int8_t *node_turn;
    float *node_value; int *out_selected; int *out_path; int *out_len; float *path_values; int *node_legal;
} po_gomoku_arrays;

static int g_pack(int kind, int node, int slot) { return (kind << G_KIND_SHIFT) | (slot << G_SLOT_SHIFT) | node; }

static int g_stone(const uint32_t *colour, int cell) { return (colour[cell >> 5] >> (cell & 31)) & 1u; }

static int g_popcount(const uint32_t *w) {
    int c = 0;
    for (int i = 0; i < G_WORDS; ++i) c += __builtin_popcount(w[i]);
    return c;
}

/* exactly five through `cell` for the colour `mine` */
static int g_makes_five(const uint32_t *mine, int cell, int m, int n) {
    static const int dirs[4][2] = {{0, 1}, {1, 0}, {1, 1}, {1, -1}};
    const int r0 = cell / n, c0 = cell % n;
    for (int d = 0; d < 4; ++d) {
        int run = 1;
        for (int s = -1; s <= 1; s += 2)
            for (int k = 1;; ++k) {
                const int r = r0 + s * k * dirs[d][0], c = c0 + s * k * dirs[d][1];
                if (r < 0 || r >= m || c < 0 || c >= n || !g_stone(mine, r * n + c)) break;
                ++run;
            }
        if (run == 5) return 1;
    }
    return 0;
}

static void g_write_priors(const po_gomoku_arrays *A, size_t node_row, const uint32_t *board, uint64_t bh, int cells,
                           float alpha) {
    uint32_t key[G_EDGES];
    uint64_t sum = 0;
    int n_legal = 0;
    for (int c = 0; c < cells; ++c) {
        key[c] = 0;
        if (!g_stone(board, c) && !g_stone(board + 8, c)) {
            key[c] = psyn_weight_key(psyn_gamma(alpha, psyn_cell_key(bh, c)), c);
            sum += psyn_key_weight(key[c]);
            ++n_legal;
        }
    }
    for (int c = 0; c < cells; ++c) {
        if (!key[c]) continue;
        int rank = 0;
        for (int o = 0; o < cells; ++o) rank += key[o] > key[c];
        const size_t e = node_row * G_EDGES + rank;
        A->edge_prior[e] = psyn_prior(psyn_key_weight(key[c]), sum, n_legal);
        A->edge_action[e] = (uint8_t)c;
        A->edge_child[e] = -1;
        A->edge_n[e] = 0;
        A->edge_w[e] = 0.0f;
        A->edge_inflight[e] = 0;
    }
}

/* Selection of one step in one tree: lockstep descent, claims in wid order within a node.  claims[w] = number of
 * path entries (claimed edges) traversal w holds when it ends, whatever its kind. */
static void g_select_step(const po_gomoku_arrays *A, int t, int nodes, int warps, int path_depth, float cpuct,
                          float c_pw, float alpha_pw, int *claims, int64_t *work) {
    const size_t trow = (size_t)t * nodes;
    int cur[G_MAX_WARPS], active[G_MAX_WARPS];
    for (int w = 0; w < warps; ++w) {
        cur[w] = 0;
        active[w] = 1;
        claims[w] = 0;
        A->out_selected[(size_t)t * warps + w] = g_pack(K_INVALID, G_NODE_MASK, 0);
        A->out_len[(size_t)t * warps + w] = 0;
    }
    for (int depth = 0;; ++depth) {
        int any = 0;
        for (int w = 0; w < warps; ++w) any |= active[w];
        if (!any) break;
        int next[G_MAX_WARPS], standing[G_MAX_WARPS];   /* standing: active when the round began */
        for (int w = 0; w < warps; ++w) next[w] = cur[w], standing[w] = active[w];
        for (int lead = 0; lead < warps; ++lead) {
            if (!standing[lead]) continue;
            int is_leader = 1;
            for (int w = 0; w < lead; ++w) is_leader &= !(standing[w] && cur[w] == cur[lead]);
            if (!is_leader) continue;
            const int node = cur[lead];
            const size_t nrow = trow + node, erow = nrow * G_EDGES;
            const int info = A->node_expanded[nrow];
            work[6] += 1;
            if (info >= 0 && depth < path_depth) work[7] += info;
            for (int w = lead; w < warps; ++w) {
                if (!standing[w] || cur[w] != node) continue;
                const size_t out = (size_t)t * warps + w;
                int *path = A->out_path + out * path_depth;
                claims[w] = depth;
                if (info == TERMINAL) {
                    A->out_selected[out] = g_pack(K_TERMINAL, node, 0);
                    A->out_len[out] = depth + 1;
                    active[w] = 0;
                    continue;
                }
                if (depth >= path_depth) {
                    A->out_selected[out] = g_pack(K_DEPTH_LIMIT, node, 0);
                    A->out_len[out] = depth + 1;
                    active[w] = 0;
                    continue;
                }
                const int expanded = info;
                int parent_eff = 1, allowed = 1;
                if (expanded != 1 || c_pw != 0.0f) {
                    int total = 0;
                    for (int e = 0; e < expanded; ++e) total += A->edge_n[erow + e] + A->edge_inflight[erow + e];
                    parent_eff = total > 1 ? total : 1;
                    allowed = allowed_children(c_pw, alpha_pw, parent_eff, A->node_legal[nrow]);
                }
                if (allowed > expanded) {
                    if (expanded + A->node_expand_inflight[nrow] < allowed) {
                        const int slot = expanded + A->node_expand_inflight[nrow]++;
                        A->out_selected[out] = g_pack(K_EXPAND, node, slot);
                        A->out_len[out] = depth + 1;
                        active[w] = 0;
                        continue;
                    }
                    if (expanded == 0) {
                        A->out_selected[out] = g_pack(K_BUSY, node, 0);
                        active[w] = 0;
                        continue;
                    }
                }
                int tie_offset = w;
                if (tie_offset >= expanded) tie_offset %= expanded;
                int best = 0;
                if (expanded > 1) {
                    const float sqrt_parent = sqrtf((float)parent_eff);
                    float best_score = -FLT_MAX;
                    best = INT32_MAX;
                    for (int e = 0; e < expanded; ++e) {
                        const int n = A->edge_n[erow + e];
                        const float q = n > 0 ? A->edge_w[erow + e] / (float)n : 0.0f;
                        const float u = cpuct * A->edge_prior[erow + e] * sqrt_parent / (float)(n + A->edge_inflight[erow + e] + 1);
                        const float score = q + u;
                        if (ahead(score, e, best_score, best, tie_offset, expanded)) {
                            best_score = score;
                            best = e;
                        }
                    }
                }
                if (best == INT32_MAX) {   /* no edge with a comparable score */
                    A->out_selected[out] = g_pack(K_INVALID, G_NODE_MASK, 0);
                    active[w] = 0;
                    continue;
                }
                A->edge_inflight[erow + best] += 1;
                path[depth] = (node << 8) | best;
                next[w] = A->edge_child[erow + best];
            }
        }
        for (int w = 0; w < warps; ++w) cur[w] = next[w];
    }
}

static void g_search_tree(const po_gomoku_arrays *A, int t, const uint32_t *root_words, int root_turn, int m, int n,
                          int nodes, int warps, int path_depth, int steps, float cpuct, float c_pw, float alpha_pw,
                          float alpha, uint64_t seed, int64_t *tally) {
    const int cells = m * n;
    const size_t trow = (size_t)t * nodes;
    const uint64_t tree_seed = psyn_tree_seed(seed, t);
    for (int i = 0; i < G_WORDS; ++i) A->node_board[trow * G_WORDS + i] = root_words[i];
    const int root_legal = cells - g_popcount(root_words);
    A->node_turn[trow] = (int8_t)root_turn;
    A->node_value[trow] = 0.0f;
    A->node_expanded[trow] = root_legal == 0 ? TERMINAL : 0;
    A->node_expand_inflight[trow] = 0;
    A->node_legal[trow] = root_legal;
    A->node_count[t] = 1;
    for (int k = 0; k < 8; ++k) tally[k] = 0;
    if (root_legal > 0) g_write_priors(A, trow, root_words, psyn_board_hash(tree_seed, root_words), cells, alpha);
    for (int step = 0; step < steps; ++step) {
        int claims[G_MAX_WARPS];
        g_select_step(A, t, nodes, warps, path_depth, cpuct, c_pw, alpha_pw, claims, tally);
        /* which traversals want a child, and does the tree have room for all of them? */
        int total = 0;
        for (int w = 0; w < warps; ++w) {
            const int raw = A->out_selected[(size_t)t * warps + w];
            const int kind = (raw >> G_KIND_SHIFT) & KIND_MASK, node = raw & G_NODE_MASK, slot = (raw >> G_SLOT_SHIFT) & EDGE_MASK;
            tally[kind] += 1;
            if (kind == K_EXPAND && slot < A->node_legal[trow + node]) ++total;
        }
        const int base = A->node_count[t];
        const int fits = base + total <= nodes;
        int next = base;
        if (fits) {
            A->node_count[t] = base + total;
            tally[5] += total;
        }
        for (int w = 0; w < warps; ++w) {
            const size_t out = (size_t)t * warps + w;
            const int raw = A->out_selected[out];
            const int kind = (raw >> G_KIND_SHIFT) & KIND_MASK, node = raw & G_NODE_MASK, slot = (raw >> G_SLOT_SHIFT) & EDGE_MASK;
            if (kind != K_EXPAND && kind != K_TERMINAL && kind != K_DEPTH_LIMIT) continue;
            uint32_t board[G_WORDS];
            for (int i = 0; i < G_WORDS; ++i) board[i] = A->node_board[(trow + node) * G_WORDS + i];
            const int n_legal = A->node_legal[trow + node];
            const int turn = A->node_turn[trow + node];
            float u;
            if (kind == K_EXPAND && slot < n_legal && fits) {
                /* the child goes into the node's next free edge slot (the expanded edges of a node stay contiguous
                 * whatever the tickets say), children numbered in traversal order */
                const int child = next++;
                const int taken = A->node_expanded[trow + node]++;
                const size_t e = (trow + node) * G_EDGES + taken;
                const int action = A->edge_action[e];
                uint32_t *mine = board + (turn > 0 ? 0 : 8);
                mine[action >> 5] |= 1u << (action & 31);
                const int win = g_makes_five(mine, action, m, n);
                const int terminal = win || n_legal - 1 == 0;
                const uint64_t bh = psyn_board_hash(tree_seed, board);
                const float v_child = win ? -1.0f : (terminal ? 0.0f : psyn_value(bh));
                for (int i = 0; i < G_WORDS; ++i) A->node_board[(trow + child) * G_WORDS + i] = board[i];
                A->node_turn[trow + child] = (int8_t)-turn;
                A->node_value[trow + child] = v_child;
                A->node_expanded[trow + child] = terminal ? TERMINAL : 0;
                A->node_expand_inflight[trow + child] = 0;
                A->node_legal[trow + child] = n_legal - 1;
                A->edge_child[e] = child;
                A->edge_n[e] = 1;
                A->edge_w[e] = -v_child;
                if (!terminal) g_write_priors(A, trow + child, board, bh, cells, alpha);
                u = -v_child;
            } else if (kind == K_TERMINAL) {
                u = A->node_value[trow + node];
            } else {
                u = psyn_value(psyn_board_hash(tree_seed, board));
            }
            const int L = A->out_len[out] - 1;
            for (int d = 0; d < L; ++d) A->path_values[out * path_depth + d] = ((L - d) & 1) ? -u : u;
        }
        /* backup: every traversal releases its claims; those that reached a node also leave a visit and a value */
        for (int w = 0; w < warps; ++w) {
            const size_t out = (size_t)t * warps + w;
            const int raw = A->out_selected[out];
            const int kind = (raw >> G_KIND_SHIFT) & KIND_MASK;
            const int counted = kind == K_EXPAND || kind == K_TERMINAL || kind == K_DEPTH_LIMIT;
            for (int d = 0; d < claims[w]; ++d) {
                const int enc = A->out_path[out * path_depth + d];
                const size_t e = (trow + (enc >> 8)) * G_EDGES + (enc & 0xFF);
                A->edge_inflight[e] -= 1;
                if (counted) {
                    A->edge_n[e] += 1;
                    A->edge_w[e] += A->path_values[out * path_depth + d];
                }
            }
            if (kind == K_EXPAND) A->node_expand_inflight[trow + (raw & G_NODE_MASK)] -= 1;
        }
    }
}

void po_gomoku_search(const po_gomoku_arrays *A, const int8_t *root, int root_turn, int m, int n, int trees, int nodes,
                      int warps, int path_depth, int steps, float cpuct, float c_pw, float alpha_pw,
                      float dirichlet_alpha, uint64_t seed, int threads, int64_t *tally /* [trees][8] */) {
    const int cells = m * n;
    uint32_t words[G_WORDS] = {0};
    for (int i = 0; i < cells; ++i) {
        if (root[i] == 1) words[i >> 5] |= 1u << (i & 31);
        if (root[i] == -1) words[8 + (i >> 5)] |= 1u << (i & 31);
    }
    if (warps > G_MAX_WARPS) warps = G_MAX_WARPS;
    /* trees are independent searches */
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads > 0 ? threads : 1)
    for (int t = 0; t < trees; ++t)
        g_search_tree(A, t, words, root_turn, m, n, nodes, warps, path_depth, steps, cpuct, c_pw, alpha_pw,
                      dirichlet_alpha, seed, tally + (size_t)t * 8);
}

/* helpers the tests use to pin the evaluator and the rule check */
float po_det_expf(float x) { return detm_expf(x); }
float po_det_logf(float x) { return detm_logf(x); }
float po_gamma(float alpha, uint64_t key) { return psyn_gamma(alpha, key); }
uint32_t po_cell_key(float alpha, uint64_t board_hash, int cell) { return psyn_weight_key(psyn_gamma(alpha, psyn_cell_key(board_hash, cell)), cell); }
float po_value(uint64_t board_hash) { return psyn_value(board_hash); }
uint64_t po_board_hash(uint64_t seed, int tree, const uint32_t *words) { return psyn_board_hash(psyn_tree_seed(seed, tree), words); }
int po_makes_five(const uint32_t *mine, int cell, int m, int n) { return g_makes_five(mine, cell, m, n); }
