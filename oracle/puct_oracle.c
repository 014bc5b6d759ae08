/*
 * CPU oracle of the PUCT selection / backup path with virtual loss.  TEST INFRASTRUCTURE ONLY: nothing that ships may
 * link, load or call this file; the tests and the benchmark's CPU-baseline leg use it as the checker.
 *
 * Restates, as plain sequential C over host arrays, the algorithm of
 *   - puct_select_winner_recalc_kernel, src/puct/puct_gpu_v3_cpp.cu:277-448 (helpers :38-275);
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
                       int *path, int *out_len, int tree, int wid, int nodes, int edges, int path_depth) {
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
            allowed = allowed_children(c_pw, alpha_pw, parent_eff, edges);
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

void po_select(float cpuct, float c_pw, float alpha_pw, int soft_winner, const int *edge_child_id,
               const float *edge_prior, const float *edge_W, const int *edge_N, int *edge_inflight,
               int *node_expand_inflight, const int *node_expanded, const int *tree_nodes, int *out_selected_node,
               int *out_path_eids, int *out_path_len, int trees, int nodes, int edges, int warps, int path_depth) {
    for (int tree = 0; tree < trees; ++tree)
        for (int wid = 0; wid < warps; ++wid) {
            const size_t out = (size_t)tree * warps + wid;
            select_one(cpuct, c_pw, alpha_pw, soft_winner, edge_child_id, edge_prior, edge_W, edge_N, edge_inflight,
                       node_expand_inflight, node_expanded, tree_nodes[tree], out_selected_node + out,
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
