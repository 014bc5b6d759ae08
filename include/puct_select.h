/*
 * C ABI of the PUCT selection / backup path with virtual loss (libpuct_hip.so, gfx950).
 *
 * All array arguments are raw DEVICE pointers to C-contiguous arrays owned by the caller.  Every launcher is
 * asynchronous on `stream` (a hipStream_t passed as void*, NULL = the default stream), returns the HIP runtime error
 * code of the launch (0 = success) and never synchronises; puct_cpp_cuda_error_string() turns a code into text.
 *
 * Array shapes (T = trees, N = nodes, E = edges, W = warps, D = path_depth):
 *   edge_child_id, edge_N, edge_inflight : int32 [T, N, E]       edge_prior, edge_W : float32 [T, N, E]
 *   node_expand_inflight, node_expanded, node_inflight : int32 [T, N]     tree_nodes / node_count : int32 [T]
 *   out_selected_node, out_path_len : int32 [T, W]     out_path_eids : int32 [T, W, D]
 *   path_edge_values : float32 [T, W, D]
 *
 * "warp" keeps the reference's meaning of one traversal: here one 64-lane wavefront runs traversal (tree, wid),
 * wid in [0, W), and wid feeds the tie rotation exactly as in the reference.
 */
#ifndef PUCT_SELECT_H
#define PUCT_SELECT_H

#ifdef __cplusplus
extern "C" {
#endif

/* node_expanded value of a terminal node (src/puct/puct_gpu_v3_cpp.cu:10). */
#define PUCT_NODE_EXPANDED_TERMINAL (-1)

/* Packed selection word: (reason << 25) | (kind << 22) | (expand_slot << 14) | node
 * (src/puct/puct_gpu_v3_cpp.cu:11-16,38-41). */
#define PUCT_PACKED_NODE_LIMIT 16384
#define PUCT_PACKED_NODE_MASK 0x3FFF
#define PUCT_PACKED_EDGE_MASK 0xFF
#define PUCT_PACKED_SLOT_SHIFT 14
#define PUCT_PACKED_KIND_SHIFT 22
#define PUCT_PACKED_KIND_MASK 0x7
#define PUCT_PACKED_REASON_SHIFT 25

/* Selection kinds (src/puct/puct_gpu_v3_cpp.cu:18-22). */
#define PUCT_SELECT_INVALID 0
#define PUCT_SELECT_EXPAND 1
#define PUCT_SELECT_TERMINAL 2
#define PUCT_SELECT_DEPTH_LIMIT 3
#define PUCT_SELECT_BUSY 4

/* Reason codes (src/puct/puct_gpu_v3_cpp.cu:24-34). */
#define PUCT_REASON_UNSET 0
#define PUCT_REASON_OK_EXPAND 1
#define PUCT_REASON_OK_TERMINAL 2
#define PUCT_REASON_OK_DEPTH_LIMIT 3
#define PUCT_REASON_BUSY_EXPAND_INFLIGHT 4
#define PUCT_REASON_BUSY_WINNER_RECALC 5
#define PUCT_REASON_INVALID_SHAPE 10
#define PUCT_REASON_INVALID_NODE_INFO 11
#define PUCT_REASON_INVALID_NO_VALID_EDGE 14
#define PUCT_REASON_INVALID_CHILD_OOB 15
#define PUCT_REASON_INVALID_UNKNOWN 16

/*
 * PUCT selection with edge-level virtual loss, winner-recalc claim and progressive widening.
 * Replaces puct_select_winner_recalc_launch of src/puct/puct_gpu_v3_cpp.cu:450-481 (kernel :277-448): same
 * signature, same semantics, same packing.  The reference launches `trees` blocks of `warps * 32` threads; this
 * library launches one 64-lane wavefront per (tree, wid) and splits trees with more than 16 traversals over several
 * workgroups, so `warps` is not limited to 32.  With up to 16 traversals per tree and nodes * edges <= 8192 a launch
 * keeps every tree's edge_inflight in the LDS of the one workgroup that runs the tree's traversals (read at the start,
 * written back at the end; the claims in between are LDS operations).  As with any output array, nothing else on the
 * device may read or write edge_inflight while the launch runs; launches on one stream, or ordered by events, are fine.
 */
int puct_select_winner_recalc_launch(float cpuct, float c_pw, float alpha_pw, int soft_winner,
                                     const int *edge_child_id, const float *edge_prior, const float *edge_W,
                                     const int *edge_N, int *edge_inflight, int *node_expand_inflight,
                                     const int *node_expanded, const int *tree_nodes, int *out_selected_node,
                                     int *out_path_eids, int *out_path_len, int trees, int nodes, int edges,
                                     int warps, int path_depth, void *stream);

/* Replaces puct_cpp_cuda_error_string of src/puct/puct_gpu_v3_cpp.cu:483-485. */
const char *puct_cpp_cuda_error_string(int code);

/*
 * Backup for the edge-level virtual loss that puct_select_winner_recalc_launch places.  For every traversal whose
 * kind is not INVALID or BUSY and whose path length is positive: along the path, edge_inflight -= virtual_loss,
 * and, when path_edge_values is not NULL, edge_N += 1 and edge_W += path_edge_values[tree, wid, d]; an EXPAND
 * selection also returns its expansion ticket (node_expand_inflight[leaf] -= 1).  With path_edge_values == NULL it is
 * the claim release of src/puct/test_puct_gpu_v3.py:275-333; the statistics update follows the reference's only
 * backup kernel, src/puct/puct_gpu_v2.py:847-927, moved from node-level to edge-level virtual loss.
 */
int puct_edge_backup_launch(int virtual_loss, float *edge_W, int *edge_N, int *edge_inflight,
                            int *node_expand_inflight, const int *node_count, const int *out_selected_node,
                            const int *out_path_eids, const int *out_path_len, const float *path_edge_values,
                            int trees, int nodes, int edges, int warps, int path_depth, void *stream);

/*
 * PUCT selection with node-level virtual loss (node_inflight[tree, child] += 1 along the selected path), the
 * counterpart of puct_node_backup_launch below.  The reference has these two kernels in numba only, so there is no C
 * symbol to replace: the entry points take the kernels' arguments in the kernels' order, the array shapes as trailing
 * integers and the stream, like the launchers above.
 *   puct_node_select_preclaim_launch       _select_kernel_native, src/puct/puct_gpu_v2.py:573-697: every candidate
 *                                          child is claimed before it is scored (the score sees the claims of the
 *                                          traversals ahead of it), the losers are released afterwards; ties go to
 *                                          the edge index rotated by wid.
 *   puct_node_select_winner_recalc_launch  _select_kernel_winner_recalc, :700-840: scores from the counters as read,
 *                                          a counter compare-and-swap on the winner only; when that child already
 *                                          carried claims the claim is released and the edges are scored once more
 *                                          without it; ties go to the smaller edge index.
 * Selection word (:352-354, no reason field, no BUSY kind): (kind << 22) | (expand_slot << 14) | node; a traversal
 * that ends without a selection (no expansion ticket left, no edge that leads to a node of the tree, inconsistent
 * node words) has given its claims back and reports PUCT_PACKED_INVALID_V2 with path length 0.
 * With up to 16 traversals per tree and up to 16384 nodes per tree a launch keeps every tree's node_inflight row in the
 * LDS of the one workgroup that runs the tree's traversals (read at the start, written back at the end; the claims in
 * between are LDS atomics).  As with any output array, nothing else on the device may read or write node_inflight
 * while the launch runs; launches on one stream, or ordered by events, are fine.
 */
#define PUCT_PACKED_INVALID_V2 ((PUCT_SELECT_INVALID << PUCT_PACKED_KIND_SHIFT) | PUCT_PACKED_NODE_MASK)
int puct_node_select_preclaim_launch(float cpuct, float c_pw, float alpha_pw, const int *edge_child_id,
                                     const float *edge_prior, const float *edge_W, const int *edge_N,
                                     int *node_inflight, int *node_expand_inflight, const int *node_expanded,
                                     const int *node_count, int *out_selected_node, int *out_path_eids,
                                     int *out_path_len, int trees, int nodes, int edges, int warps, int path_depth,
                                     void *stream);
int puct_node_select_winner_recalc_launch(float cpuct, float c_pw, float alpha_pw, const int *edge_child_id,
                                          const float *edge_prior, const float *edge_W, const int *edge_N,
                                          int *node_inflight, int *node_expand_inflight, const int *node_expanded,
                                          const int *node_count, int *out_selected_node, int *out_path_eids,
                                          int *out_path_len, int trees, int nodes, int edges, int warps,
                                          int path_depth, void *stream);

/*
 * Backup with node-level virtual loss: the kernel _backup_kernel_native of src/puct/puct_gpu_v2.py:847-927 with its
 * argument order (array shapes become the trailing integers).  The selection word is read with the v2 layout
 * (kind = word >> 22, no reason field, :879,903-905).
 */
int puct_node_backup_launch(int virtual_loss, const int *edge_child_id, float *edge_W, int *edge_N,
                            int *node_inflight, int *node_expand_inflight, const int *node_count,
                            const int *out_selected_node, const int *out_path_eids, const int *out_path_len,
                            const float *path_edge_values, int trees, int nodes, int edges, int warps,
                            int path_depth, void *stream);

#ifdef __cplusplus
}
#endif
#endif
