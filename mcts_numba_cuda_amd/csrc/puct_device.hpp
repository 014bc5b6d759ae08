// Device side of PUCT selection and backup with virtual loss for gfx950 (wave64): one 64-lane wavefront per traversal.
//
// Semantics follow src/puct/puct_gpu_v3_cpp.cu:38-448 (selection with edge-level virtual loss),
// src/puct/puct_gpu_v2.py:573-840 (the two selections with node-level virtual loss) and :847-927 (backup); the
// wavefront-level organisation is this library's own:
//   * the first 64 edges of a node (all of them for almost every node under progressive widening) are loaded once,
//     together with the node's own words, before anything about the node is known, so a level costs one round of
//     loads and one claim instead of a chain of dependent loads;
//   * the reference's total order on edges (score descending, rotated edge index ascending) is taken in two steps: the
//     largest score by a max-reduction of 32-bit keys over DPP row operations, the edge among the equal ones from the
//     lane masks of the comparison with it, on the scalar unit;
//   * a level is written once per number of 64-edge slices the node fills, and everything that is the same in all
//     lanes (node, depth, row addresses, branches) is kept on the scalar side: the kernels are bound by instruction
//     issue, not by the memory they read.
#pragma once
#include <hip/hip_runtime.h>
#include <float.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/puct_select.h"

namespace puct {


constexpr int kWave = 64;
constexpr int kMaxWavesPerBlock = 16;
constexpr int kRecalcAttempts = 2;  // MAX_RECALC_RETRY, src/puct/puct_gpu_v3_cpp.cu:36
constexpr int kPasses = (PUCT_PACKED_EDGE_MASK + 1) / kWave;  // 64-edge slices of the widest node
constexpr int kNoEdge = 0x7fffffff;

struct SelectArgs {
    float cpuct, c_pw, alpha_pw;
    int soft_winner;
    const int *edge_child_id;
    const float *edge_prior;
    const float *edge_W;
    const int *edge_N;
    int *edge_inflight;
    int *node_expand_inflight;
    const int *node_expanded;
    const int *tree_nodes;
    int *out_selected_node;
    int *out_path_eids;
    int *out_path_len;
    int trees, nodes, edges, warps, path_depth;
    // Optional per-node limit on the number of children, int32 [trees, nodes]; NULL = `edges` for every node, which is
    // the reference's behaviour.  A caller whose nodes have fewer possible children than `edges` (legal moves) passes
    // it so that progressive widening stops asking for slots a node cannot have.
    const int *node_capacity = nullptr;
    // Attempts of the winner-recalc claim per level; the reference has 2 compiled in.
    int recalc_attempts = kRecalcAttempts;
    // Optional work counters, uint64 [trees, 8]: entry 6 of a tree's row gains the tree levels its traversals read,
    // entry 7 the expanded edges examined on those levels (what the algorithmic byte count of a selection is made of).
    unsigned long long *work = nullptr;
};

// ---- cross-lane reductions -------------------------------------------------------------------------------------
// DPP controls: quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror.  After the four steps every
// lane holds the reduction of its 16-lane row; the four rows are combined through lane reads.
template <int CTRL>
__device__ __forceinline__ int dpp(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}

__device__ __forceinline__ int wave_sum(int v) {
    v += dpp<0xB1>(v);
    v += dpp<0x4E>(v);
    v += dpp<0x141>(v);
    v += dpp<0x140>(v);
    return __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) + __builtin_amdgcn_readlane(v, 32) +
           __builtin_amdgcn_readlane(v, 48);
}

template <int CTRL>
__device__ __forceinline__ uint64_t dpp_max64(uint64_t v) {
    const uint32_t lo = (uint32_t)dpp<CTRL>((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)dpp<CTRL>((int)(uint32_t)(v >> 32));
    const uint64_t o = ((uint64_t)hi << 32) | lo;
    return o > v ? o : v;
}

__device__ __forceinline__ uint64_t read_lane64(uint64_t v, int lane) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, lane);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), lane);
    return ((uint64_t)hi << 32) | lo;
}

__device__ __forceinline__ uint64_t wave_max(uint64_t v) {
    v = dpp_max64<0xB1>(v);
    v = dpp_max64<0x4E>(v);
    v = dpp_max64<0x141>(v);
    v = dpp_max64<0x140>(v);
    const uint64_t a = read_lane64(v, 0), b = read_lane64(v, 16), c = read_lane64(v, 32), d = read_lane64(v, 48);
    const uint64_t ab = a > b ? a : b, cd = c > d ? c : d;
    return ab > cd ? ab : cd;
}

__device__ __forceinline__ int load_relaxed(const int *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// A field of one edge of a tree: the tree's array (one address per wavefront, kept in scalar registers for the whole
// traversal) plus a 32-bit byte offset per lane.  A tree is at most 2^14 nodes of 256 edges, 16 MB per field, so the
// offset fits, and a load is one instruction with nothing to add to a 64-bit address first.
template <class T>
__device__ __forceinline__ T *at_bytes(T *tree_field, uint32_t byte_offset) {
    typedef std::conditional_t<std::is_const<T>::value, const char, char> Byte;
    return reinterpret_cast<T *>(reinterpret_cast<Byte *>(tree_field) + byte_offset);
}

// ---- selection ---------------------------------------------------------------------------------------------------
__device__ __forceinline__ int pack_selection(int kind, int node, int slot, int reason) {
    return (reason << PUCT_PACKED_REASON_SHIFT) | (kind << PUCT_PACKED_KIND_SHIFT) | (slot << PUCT_PACKED_SLOT_SHIFT) |
           node;
}

// src/puct/puct_gpu_v3_cpp.cu:43-49
__device__ __forceinline__ bool valid_select_shape(int path_depth, int nodes, int node_cnt, int edges) {
    return path_depth >= 1 && nodes > 0 && node_cnt > 0 && node_cnt <= nodes && node_cnt <= PUCT_PACKED_NODE_LIMIT &&
           edges > 0 && edges <= PUCT_PACKED_EDGE_MASK + 1;
}

// Progressive widening, src/puct/puct_gpu_v3_cpp.cu:150-157.
__device__ __forceinline__ int allowed_children(float c_pw, float alpha_pw, int n_node, int edges, float sqrt_n_node) {
    const float val = (alpha_pw == 0.5f) ? c_pw * sqrt_n_node : c_pw * powf((float)n_node, alpha_pw);
    if (val >= (float)edges) return edges;
    const int allowed = (int)ceilf(val);
    return allowed > 1 ? allowed : 1;
}
__device__ __forceinline__ int allowed_children(float c_pw, float alpha_pw, int n_node, int edges) {
    return allowed_children(c_pw, alpha_pw, n_node, edges, sqrtf((float)n_node));
}

// The score of an edge (src/puct/puct_gpu_v3_cpp.cu:171-180) is q + u with q = n > 0 ? w / n : 0 and
// u = cpuct * prior * sqrt_parent / (n + inflight + 1), in single precision, operation by operation.  The selections
// below keep q and the numerator of u per edge and divide again when the in-flight counts have been read again.

// One 64-bit key per candidate edge (used by the Gomoku search loop) whose unsigned order is the reference's order "higher score first, then smaller
// rotated edge index" (src/puct/puct_gpu_v3_cpp.cu:51-71).  0 means "not a candidate": the reference starts from
// (-FLT_MAX, no edge) and accepts a score that is greater than or equal to it, so NaN and -inf never win.  -0.0f is
// made +0.0f because the reference compares floats, for which the two are equal.
__device__ __forceinline__ uint64_t candidate_key(float score, int eid, int tie_offset, int span) {
    if (!(score >= -FLT_MAX)) return 0;
    const uint32_t b = __float_as_uint(score + 0.0f);
    const uint32_t ordered = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    int key = eid - tie_offset;
    if (key < 0) key += span;
    return ((uint64_t)ordered << 32) | ((uint32_t)(0xFFFF - key) << 16) | (uint32_t)eid;
}

// The same order with the score and the edge index kept apart, for the selection kernels of this file: a
// 32-bit key per edge whose unsigned order is the order of the scores (0 = not a candidate, as above), the largest of
// which is found with one `v_max_u32` per DPP step; the edge among the equal ones comes from the lane masks of the
// comparison with that maximum, on the scalar unit.
__device__ __forceinline__ uint32_t score_key(float score) {
    if (!(score >= -FLT_MAX)) return 0;
    const uint32_t b = __float_as_uint(score + 0.0f);
    return b ^ ((uint32_t)((int32_t)b >> 31) | 0x80000000u);
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    auto step = [](uint32_t x, auto ctrl) {
        const uint32_t o = (uint32_t)dpp<decltype(ctrl)::value>((int)x);
        return o > x ? o : x;
    };
    v = step(v, std::integral_constant<int, 0xB1>{});
    v = step(v, std::integral_constant<int, 0x4E>{});
    v = step(v, std::integral_constant<int, 0x141>{});
    v = step(v, std::integral_constant<int, 0x140>{});
    const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
    return ab > cd ? ab : cd;
}

// The edge with the largest key (keys[i] belongs to edge lane + 64 i; `skip` takes no part); among equal keys the one
// whose index rotated by tie_offset is smallest, i.e. the first at or after tie_offset, else the first.  kNoEdge if no
// key is above 0.  Every lane returns the same value.
template <int S>
__device__ __forceinline__ int best_edge(const uint32_t (&keys)[S], int lane, int skip, int tie_offset) {
    uint32_t k[S], m = 0;
#pragma unroll
    for (int i = 0; i < S; ++i) {
        k[i] = lane + i * kWave == skip ? 0u : keys[i];
        m = k[i] > m ? k[i] : m;
    }
    m = wave_max_u32(m);
    if (m == 0) return kNoEdge;
    int at_or_after = kNoEdge, first = kNoEdge;
#pragma unroll
    for (int i = 0; i < S; ++i) {
        const uint64_t equal = __builtin_amdgcn_ballot_w64(k[i] == m);
        const int from = tie_offset - i * kWave;   // lanes of this slice at or after the offset: from `from` on
        const uint64_t late = equal & (from <= 0 ? ~0ull : from >= kWave ? 0ull : ~0ull << from);
        if (first == kNoEdge && equal != 0) first = i * kWave + __builtin_ctzll(equal);
        if (at_or_after == kNoEdge && late != 0) at_or_after = i * kWave + __builtin_ctzll(late);
    }
    return at_or_after != kNoEdge ? at_or_after : first;
}

// The claims in flight on one tree's edges, edge_inflight[tree, :, :].  While a launch runs they are read and changed by
// the traversals of that tree only; when those are the wavefronts of one workgroup (up to 16 traversals per tree) and the
// tree is small enough (nodes * edges words), the workgroup keeps them in LDS for the launch (LOCAL): loaded at the
// start, stored at the end, every read of a node's row and every claim in between an LDS operation instead of an
// agent-scope load and an atomic performed at the memory side.
typedef __attribute__((address_space(3))) int *LdsInts;
template <bool LOCAL>
struct EdgeClaims {
    int *in_memory;     // edge_inflight + tree * nodes * edges
    LdsInts in_lds;     // the same counters, the workgroup's copy
    // (at: byte offset of the edge's slot in the tree, (node * edges + edge) * 4)
    __device__ __forceinline__ int peek(uint32_t at) const {
        if (LOCAL) return __hip_atomic_load(in_lds + (at >> 2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        return load_relaxed(at_bytes(in_memory, at));
    }
    __device__ __forceinline__ void add(uint32_t at, int v) const {
        if (LOCAL) __hip_atomic_fetch_add(in_lds + (at >> 2), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        else atomicAdd(at_bytes(in_memory, at), v);
    }
    __device__ __forceinline__ int cas(uint32_t at, int expected, int desired) const {   // returns the value found
        if (LOCAL) {
            __hip_atomic_compare_exchange_strong(in_lds + (at >> 2), &expected, desired, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            return expected;
        }
        return atomicCAS(at_bytes(in_memory, at), expected, desired);
    }
};

// Takes back the virtual loss of the first `depth` path entries (src/puct/puct_gpu_v3_cpp.cu:206-217).  The entries
// were stored by lane 0 of this wavefront; the fence completes those stores before other lanes read them back.
template <bool LOCAL>
__device__ __forceinline__ void rollback_path(const SelectArgs &a, const EdgeClaims<LOCAL> &claims, const int *path, int tree, int depth, int lane,
                                              int node_cnt) {
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "agent");
    for (int d = lane; d < depth; d += kWave) {
        const int encoded = load_relaxed(path + d);
        const int parent = encoded >> 8, slot = encoded & 0xFF;
        if (parent >= 0 && parent < node_cnt && slot < a.edges)
            claims.add(((uint32_t)parent * (uint32_t)a.edges + (uint32_t)slot) * 4u, -1);
    }
}

// One traversal (tree, wid) by one wavefront; every lane of the wavefront must call it.  A level is written once per
// number S of 64-edge slices that the node's expanded edges fill (1..4, the same for all lanes): these kernels are bound
// by the wavefronts' instruction issue, vector and scalar together, and a level written for "up to four slices" spends a
// third of it on finding out, slice by slice, that a slice is not there.
template <bool LOCAL>
__device__ __forceinline__ void select_traversal(const SelectArgs &a, const EdgeClaims<LOCAL> &claims, int tree, int wid, int lane) {
    static_assert(kPasses == 4, "the levels below are written for one to four slices");
    const size_t out = (size_t)tree * a.warps + wid;
    int *path = a.out_path_eids + out * a.path_depth;
    const int node_cnt = a.tree_nodes[tree];
    const int nodes = a.nodes, edges = a.edges;

    int final_packed = pack_selection(PUCT_SELECT_INVALID, PUCT_PACKED_NODE_MASK, 0, PUCT_REASON_INVALID_UNKNOWN);
    int final_len = 0;
    int levels = 0, edges_seen = 0;

    if (!valid_select_shape(a.path_depth, nodes, node_cnt, edges)) {
        final_packed = pack_selection(PUCT_SELECT_INVALID, PUCT_PACKED_NODE_MASK, 0, PUCT_REASON_INVALID_SHAPE);
    } else {
        const size_t tree_edges = (size_t)tree * nodes * edges;
        const int *const tree_n = a.edge_N + tree_edges, *const tree_c = a.edge_child_id + tree_edges;
        const float *const tree_p = a.edge_prior + tree_edges, *const tree_w = a.edge_W + tree_edges;
        int node = 0, depth = 0;
        while (true) {
            // (the same in all lanes; said so that the level's addresses and branches are worked out once per wavefront)
            node = __builtin_amdgcn_readfirstlane(node), depth = __builtin_amdgcn_readfirstlane(depth);
            levels += 1;
            const size_t nrow = (size_t)tree * nodes + node;
            const uint32_t row4 = (uint32_t)node * (uint32_t)edges * 4u;   // byte offset of the node's edges in the tree's fields

            // Everything a level can need from the first 64 edges, requested in one go, before the node's width is known
            // (lanes beyond the row read its last edge and take no part); the edges of wider nodes follow once it is
            // and stay in registers for the rest of the level.
            const uint32_t at0 = row4 + (uint32_t)(lane < edges ? lane : edges - 1) * 4u;
            const int n0 = *at_bytes(tree_n, at0), f0 = claims.peek(at0), c0 = *at_bytes(tree_c, at0);
            const float p0 = *at_bytes(tree_p, at0), w0 = *at_bytes(tree_w, at0);
            const int node_info = a.node_expanded[nrow];
            const int expand_inflight = load_relaxed(a.node_expand_inflight + nrow);
            const int capacity = a.node_capacity ? a.node_capacity[nrow] : edges;

            if (node_info == PUCT_NODE_EXPANDED_TERMINAL) {
                final_packed = pack_selection(PUCT_SELECT_TERMINAL, node, 0, PUCT_REASON_OK_TERMINAL);
                final_len = depth + 1;
                break;
            }
            if (node_info < 0 || node_info > edges) {
                rollback_path(a, claims, path, tree, depth, lane, node_cnt);
                final_packed =
                    pack_selection(PUCT_SELECT_INVALID, PUCT_PACKED_NODE_MASK, 0, PUCT_REASON_INVALID_NODE_INFO);
                break;
            }
            if (depth >= a.path_depth) {
                final_packed = pack_selection(PUCT_SELECT_DEPTH_LIMIT, node, 0, PUCT_REASON_OK_DEPTH_LIMIT);
                final_len = depth + 1;
                break;
            }

            const int cur_expanded = node_info;
            edges_seen += cur_expanded;

            // The level proper; returns the child the traversal moves on to, or -1 when it ends here.
            auto level = [&](auto slices) __attribute__((always_inline)) -> int {
                constexpr int S = decltype(slices)::value;   // (S - 1) * 64 < cur_expanded <= S * 64, or no edge at all (S = 1)
                constexpr int CS = S <= 2 ? S : 1;   // slices whose row of children is requested with the scores' fields (see best_child below)
                int n[S], f[S], c[CS];
                // byte offset of the edge that this lane looks at in slice i (lanes beyond the node's edges: its last edge)
                auto at = [&](int i) {
                    const int eid = lane + i * kWave;
                    return i == 0 ? at0 : row4 + (uint32_t)(i < S - 1 || eid < cur_expanded ? eid : cur_expanded - 1) * 4u;
                };
                float p[S], w[S];
                bool in_node[S];
                n[0] = n0, f[0] = f0, p[0] = p0, w[0] = w0, c[0] = c0;
#pragma unroll
                for (int i = 1; i < S; ++i) {
                    const uint32_t here = at(i);
                    n[i] = *at_bytes(tree_n, here), f[i] = claims.peek(here), p[i] = *at_bytes(tree_p, here), w[i] = *at_bytes(tree_w, here);
                    if (i < CS) c[i] = *at_bytes(tree_c, here);
                }
#pragma unroll
                for (int i = 0; i < S; ++i) in_node[i] = i < S - 1 || lane + i * kWave < cur_expanded;

                int parent_eff = 1, allowed = 1;
                float sqrt_parent = 1.0f;
                if (cur_expanded != 1 || a.c_pw != 0.0f) {
                    int total = 0;
#pragma unroll
                    for (int i = 0; i < S; ++i) total += in_node[i] ? n[i] + f[i] : 0;
                    total = wave_sum(total);
                    parent_eff = total > 1 ? total : 1;
                    sqrt_parent = sqrtf((float)parent_eff);
                    allowed = allowed_children(a.c_pw, a.alpha_pw, parent_eff, capacity, sqrt_parent);
                }

                if (allowed > cur_expanded) {
                    // Expansion ticket, src/puct/puct_gpu_v3_cpp.cu:219-233.
                    int expand_slot = -1;
                    if (cur_expanded + expand_inflight < allowed) {
                        if (lane == 0) {
                            const int slot = cur_expanded + atomicAdd(&a.node_expand_inflight[nrow], 1);
                            if (slot < allowed)
                                expand_slot = slot;
                            else
                                atomicSub(&a.node_expand_inflight[nrow], 1);
                        }
                        expand_slot = __builtin_amdgcn_readfirstlane(expand_slot);
                    }
                    if (expand_slot >= 0) {
                        final_packed = pack_selection(PUCT_SELECT_EXPAND, node, expand_slot, PUCT_REASON_OK_EXPAND);
                        final_len = depth + 1;
                        return -1;
                    }
                    if (cur_expanded == 0) {
                        rollback_path(a, claims, path, tree, depth, lane, node_cnt);
                        final_packed = pack_selection(PUCT_SELECT_BUSY, node, 0, PUCT_REASON_BUSY_EXPAND_INFLIGHT);
                        return -1;
                    }
                }

                int tie_offset = wid;
                if (tie_offset >= cur_expanded) tie_offset %= cur_expanded;

                auto of_edge = [&](const int (&v)[S], int eid) {
                    const int lane_of = eid & (kWave - 1), pass = eid / kWave;
                    int r = __builtin_amdgcn_readlane(v[0], lane_of);
#pragma unroll
                    for (int i = 1; i < S; ++i)
                        if (pass == i) r = __builtin_amdgcn_readlane(v[i], lane_of);
                    return r;
                };

                // Where the winner leads: for nodes of up to 128 edges the row of children came with the scores' fields; of a
                // wider node only its first 64, and beyond them just the winner's word is asked for, on its way while the
                // claim is made (the rest of that row is a sixth of what such a level reads -- and those launches are bound by
                // what they read -- and three registers per lane; at 128 edges waiting for the word cost more than the row).
                int best_eid = 0, held = 0, best_child = c0;   // (cur_expanded == 1: lane 0's is read below)
                if (cur_expanded == 1) {
                    if (lane == 0) claims.add(row4, 1);
                    held = 1;
                } else {
                    // Winner-recalc claim, src/puct/puct_gpu_v3_cpp.cu:235-275: score all edges, try to move the winner's
                    // in-flight count from the value the score was computed with to that value plus one, rescore once if
                    // another traversal got there first.  The mean value and the numerator of the exploration term do not
                    // depend on the in-flight counts, so a second evaluation divides once per edge, and only in the slices
                    // whose counts have changed (other traversals' claims sit on a few edges).
                    float q[S], num[S];
#pragma unroll
                    for (int i = 0; i < S; ++i) {
                        // (a slice none of whose edges has a visit or a value has q = +0 without dividing)
                        q[i] = 0.0f;
                        if (__builtin_amdgcn_ballot_w64(n[i] > 0 && __float_as_uint(w[i]) != 0u) != 0) q[i] = n[i] > 0 ? w[i] / (float)n[i] : 0.0f;
                        num[i] = a.cpuct * p[i] * sqrt_parent;
                    }
                    uint32_t keys[S];
                    auto score_slice = [&](int i, int inflight) {
                        return in_node[i] ? score_key(q[i] + num[i] / (float)(n[i] + inflight + 1)) : 0u;
                    };
                    best_eid = kNoEdge;
                    for (int attempt = 0; attempt < a.recalc_attempts; ++attempt) {
                        if (attempt == 0) {
#pragma unroll
                            for (int i = 0; i < S; ++i) keys[i] = score_slice(i, f[i]);
                        } else {
#pragma unroll
                            for (int i = 0; i < S; ++i) {
                                const int fi = claims.peek(at(i));
                                if (__builtin_amdgcn_ballot_w64(fi != f[i]) != 0) {
                                    f[i] = fi;
                                    keys[i] = score_slice(i, fi);
                                }
                            }
                        }
                        best_eid = best_edge<S>(keys, lane, -1, tie_offset);
                        if (best_eid == kNoEdge) break;
                        const int best_inflight = of_edge(f, best_eid);
                        if (best_eid < CS * kWave) {
                            best_child = __builtin_amdgcn_readlane(c[0], best_eid & (kWave - 1));
                            if (CS > 1 && best_eid >= kWave) best_child = __builtin_amdgcn_readlane(c[CS - 1], best_eid & (kWave - 1));
                        } else {
                            best_child = load_relaxed(at_bytes(tree_c, row4 + (uint32_t)best_eid * 4u));   // (every lane the same word)
                        }
                        int got = 0;
                        if (lane == 0) {
                            const int prev = claims.cas(row4 + (uint32_t)best_eid * 4u, best_inflight, best_inflight + 1);
                            got = prev == best_inflight ? 1 : 0;
                        }
                        held = __builtin_amdgcn_readfirstlane(got);
                        if (held) break;
                    }
                    if (a.soft_winner != 0 && held == 0 && best_eid != kNoEdge) {
                        if (lane == 0) claims.add(row4 + (uint32_t)best_eid * 4u, 1);
                        held = 1;
                    }
                }

                if (held == 0) {
                    rollback_path(a, claims, path, tree, depth, lane, node_cnt);
                    final_packed =
                        best_eid == kNoEdge
                            ? pack_selection(PUCT_SELECT_INVALID, PUCT_PACKED_NODE_MASK, 0, PUCT_REASON_INVALID_NO_VALID_EDGE)
                            : pack_selection(PUCT_SELECT_BUSY, node, 0, PUCT_REASON_BUSY_WINNER_RECALC);
                    return -1;
                }

                best_child = __builtin_amdgcn_readfirstlane(best_child);
                if (best_child < 0 || best_child >= node_cnt) {
                    if (lane == 0) claims.add(row4 + (uint32_t)best_eid * 4u, -1);
                    rollback_path(a, claims, path, tree, depth, lane, node_cnt);
                    final_packed =
                        pack_selection(PUCT_SELECT_INVALID, PUCT_PACKED_NODE_MASK, 0, PUCT_REASON_INVALID_CHILD_OOB);
                    return -1;
                }
                if (lane == 0) path[depth] = (node << 8) | best_eid;
                return best_child;
            };

            const int slices = (cur_expanded + kWave - 1) / kWave;
            int next;
            if (slices <= 1) next = level(std::integral_constant<int, 1>{});
            else if (slices == 2) next = level(std::integral_constant<int, 2>{});
            else if (slices == 3) next = level(std::integral_constant<int, 3>{});
            else next = level(std::integral_constant<int, 4>{});
            if (next < 0) break;
            node = next;
            depth += 1;
        }
    }

    if (lane == 0) {
        a.out_selected_node[out] = final_packed;
        a.out_path_len[out] = final_len;
        if (a.work != nullptr) {
            atomicAdd(&a.work[(size_t)tree * 8 + 6], (unsigned long long)levels);
            atomicAdd(&a.work[(size_t)tree * 8 + 7], (unsigned long long)edges_seen);
        }
    }
}

// ---- selection with node-level virtual loss ------------------------------------------------------------------------
// The two selection kernels of src/puct/puct_gpu_v2.py, whose virtual loss lives in node_inflight[tree, child] and is
// what backup_traversal<true> below takes back: _select_kernel_native (:573-697; every candidate child is claimed
// before it is scored and the losers are released afterwards) and _select_kernel_winner_recalc (:700-840; scores from
// the counters as read, a counter compare-and-swap on the winner only, one re-evaluation without the first winner
// when that child already carried claims).  Their selection word has no reason field and no BUSY kind: a traversal
// that cannot get an expansion ticket, or finds no edge, gives its claims back and reports PACKED_INVALID with length 0.
struct NodeSelectArgs {
    float cpuct, c_pw, alpha_pw;
    const int *edge_child_id;
    const float *edge_prior;
    const float *edge_W;
    const int *edge_N;
    int *node_inflight;
    int *node_expand_inflight;
    const int *node_expanded;
    const int *node_count;
    int *out_selected_node;
    int *out_path_eids;
    int *out_path_len;
    int trees, nodes, edges, warps, path_depth;
};

constexpr int kPackedInvalidV2 = (PUCT_SELECT_INVALID << PUCT_PACKED_KIND_SHIFT) | PUCT_PACKED_NODE_MASK;

__device__ __forceinline__ int pack_selection_v2(int kind, int node, int slot) {
    return (kind << PUCT_PACKED_KIND_SHIFT) | (slot << PUCT_PACKED_SLOT_SHIFT) | node;
}

// The virtual visits of one tree's nodes, node_inflight[tree, :].  While a launch runs they are read and changed by
// the traversals of that tree only; when those are the wavefronts of one workgroup (up to 16 traversals per tree) and the
// tree's counters fit, the workgroup keeps them in LDS for the launch (LOCAL): loaded at the start, stored at the end, and
// every claim in between is an LDS atomic instead of one performed at the memory side (the preclaim kernel makes two per
// edge and level; in device memory they were what bounded it).
template <bool LOCAL>
struct NodeVisits {
    int *in_memory;     // node_inflight + tree * nodes
    LdsInts in_lds;     // the same counters, workgroup's copy
    __device__ __forceinline__ int peek(int node) const {
        if (LOCAL) return __hip_atomic_load(in_lds + node, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        return load_relaxed(in_memory + node);
    }
    __device__ __forceinline__ int add(int node, int v) const {   // returns the count found
        if (LOCAL) return __hip_atomic_fetch_add(in_lds + node, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        return atomicAdd(in_memory + node, v);
    }
    __device__ __forceinline__ void sub(int node, int v) const {
        if (LOCAL) __hip_atomic_fetch_sub(in_lds + node, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        else atomicSub(in_memory + node, v);
    }
};

// src/puct/puct_gpu_v2.py:291-310: the claims of the first `depth` path entries live on the child each entry leads to.
template <bool LOCAL>
__device__ __forceinline__ void rollback_node_path(const NodeSelectArgs &a, const NodeVisits<LOCAL> &visits_of, const int *path, int tree, int depth, int lane,
                                                   int node_limit) {
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "agent");   // lane 0 stored the entries
    for (int d = lane; d < depth; d += kWave) {
        const int encoded = load_relaxed(path + d);
        if (encoded < 0) continue;
        const int parent = encoded >> 8, slot = encoded & 0xFF;
        if (parent < node_limit && slot < a.edges) {
            const int child = a.edge_child_id[((size_t)tree * a.nodes + parent) * a.edges + slot];
            if (child >= 0 && child < node_limit) visits_of.sub(child, 1);
        }
    }
}

// The claim of the winner-recalc kernel (src/puct/puct_gpu_v2.py:313-349) is one more virtual visit on the child's
// counter; "conflict" = the counter already held visits when the claim went in.  The reference moves the counter from the
// value it read to that value plus one with compare-and-swap, reads again when the exchange is lost, and after
// MAX_SELECT_RETRY lost exchanges adds one atomically instead: a counter, not a lock, so every claim goes in and all it
// learns is the value it found.  That is a fetch-and-add, which is what node_select_traversal does, without the lost
// exchanges (the traversals of a tree that reach a node together all claim the same child, and compare-and-swap then
// costs a round trip per traversal ahead).

// One traversal (tree, wid) by one wavefront; every lane of the wavefront must call it.  A level is written once per
// number S of 64-edge slices that the node's expanded edges fill (1..4, the same for all lanes): what bounds these
// kernels is the wavefronts' instruction issue, vector and scalar together, and a level written for "up to four slices"
// spends a third of it on finding out, slice by slice, that a slice is not there.
template <bool PRECLAIM, bool LOCAL>
__device__ __forceinline__ void node_select_traversal(const NodeSelectArgs &a, const NodeVisits<LOCAL> &visits_of, int tree, int wid, int lane) {
    static_assert(kPasses == 4, "the levels below are written for one to four slices");
    const size_t out = (size_t)tree * a.warps + wid;
    int *path = a.out_path_eids + out * a.path_depth;
    const int node_limit = a.node_count[tree];
    const int nodes = a.nodes, edges = a.edges;
    const size_t trow = (size_t)tree * nodes;

    int final_packed = kPackedInvalidV2, final_len = 0;
    // src/puct/puct_gpu_v2.py:357-366
    if (a.path_depth >= 1 && nodes > 0 && node_limit > 0 && node_limit <= nodes && node_limit <= PUCT_PACKED_NODE_LIMIT &&
        edges > 0 && edges <= PUCT_PACKED_EDGE_MASK + 1) {
        const size_t tree_edges = trow * edges;
        const int *const tree_c = a.edge_child_id + tree_edges, *const tree_n = a.edge_N + tree_edges;
        const float *const tree_p = a.edge_prior + tree_edges, *const tree_w = a.edge_W + tree_edges;
        int node = 0, depth = 0;
        while (true) {
            // (the same in all lanes; said so that the level's addresses and branches are worked out once per wavefront)
            node = __builtin_amdgcn_readfirstlane(node), depth = __builtin_amdgcn_readfirstlane(depth);
            if (node < 0 || node >= node_limit) {
                rollback_node_path(a, visits_of, path, tree, depth, lane, node_limit);
                break;
            }
            if (depth >= a.path_depth) {   // the path buffer is full: stop before reading or claiming anything here
                final_packed = pack_selection_v2(PUCT_SELECT_DEPTH_LIMIT, node, 0);
                final_len = depth + 1;
                break;
            }
            const size_t nrow = trow + node;
            const uint32_t row4 = (uint32_t)node * (uint32_t)edges * 4u;   // byte offset of the node's edges in the tree's fields
            // the first 64 edges are requested together with the node's own words, before the node's width is known
            // (lanes beyond the row read its last edge and take no part)
            const uint32_t at0 = row4 + (uint32_t)(lane < edges ? lane : edges - 1) * 4u;
            const int c0 = *at_bytes(tree_c, at0), n0 = *at_bytes(tree_n, at0);
            const float p0 = *at_bytes(tree_p, at0), w0 = *at_bytes(tree_w, at0);
            const int node_info = a.node_expanded[nrow];
            const int expand_inflight = load_relaxed(a.node_expand_inflight + nrow);
            if (node_info == PUCT_NODE_EXPANDED_TERMINAL) {
                final_packed = pack_selection_v2(PUCT_SELECT_TERMINAL, node, 0);
                final_len = depth + 1;
                break;
            }
            if (node_info < 0 || node_info > edges) {
                rollback_node_path(a, visits_of, path, tree, depth, lane, node_limit);
                break;
            }
            const int cur_expanded = node_info;

            // The level proper; returns the child the traversal moves on to, or -1 when it ends here.
            auto level = [&](auto slices) __attribute__((always_inline)) -> int {
                constexpr int S = decltype(slices)::value;   // (S - 1) * 64 < cur_expanded <= S * 64, or no edge at all (S = 1)
                int n[S], f[S], c[S];
                float p[S], w[S];
                bool cand[S];
                c[0] = c0, n[0] = n0, p[0] = p0, w[0] = w0;
#pragma unroll
                for (int i = 1; i < S; ++i) {
                    const int eid = lane + i * kWave;
                    const uint32_t at = row4 + (uint32_t)(i < S - 1 || eid < cur_expanded ? eid : cur_expanded - 1) * 4u;
                    c[i] = *at_bytes(tree_c, at), n[i] = *at_bytes(tree_n, at), p[i] = *at_bytes(tree_p, at), w[i] = *at_bytes(tree_w, at);
                }
                // an edge takes part when it is expanded and leads to a node of the tree; its virtual visits are its
                // child's (the other lanes read the root's counter and drop it)
                int total = 0;
#pragma unroll
                for (int i = 0; i < S; ++i) {
                    cand[i] = (i < S - 1 || lane + i * kWave < cur_expanded) && (uint32_t)c[i] < (uint32_t)node_limit;
                    const int visits = visits_of.peek(cand[i] ? c[i] : 0);
                    f[i] = cand[i] ? visits : 0;
                }
#pragma unroll
                for (int i = 0; i < S; ++i) total += cand[i] ? n[i] + f[i] : 0;
                total = wave_sum(total);
                const int parent_eff = total > 1 ? total : 1;   // :407-416
                const float sqrt_parent = sqrtf((float)parent_eff);
                const int allowed = (PRECLAIM && cur_expanded == 0) ? 1 : allowed_children(a.c_pw, a.alpha_pw, parent_eff, edges, sqrt_parent);

                if (allowed > cur_expanded) {
                    // Expansion ticket, :389-403.  Tickets are only given back by the backup, and a ticket beyond the quota is
                    // returned at once, so a counter that already shows the quota used up stays that way for this launch.
                    int expand_slot = -1;
                    if (cur_expanded + expand_inflight < allowed) {
                        if (lane == 0) {
                            const int slot = cur_expanded + atomicAdd(&a.node_expand_inflight[nrow], 1);
                            if (slot < allowed)
                                expand_slot = slot;
                            else
                                atomicSub(&a.node_expand_inflight[nrow], 1);
                        }
                        expand_slot = __builtin_amdgcn_readfirstlane(expand_slot);
                    }
                    if (expand_slot >= 0) {
                        final_packed = pack_selection_v2(PUCT_SELECT_EXPAND, node, expand_slot);
                        final_len = depth + 1;
                    } else {
                        rollback_node_path(a, visits_of, path, tree, depth, lane, node_limit);
                    }
                    return -1;
                }

                // puct_score in two parts: the mean value and the numerator of the exploration term do not depend on the
                // virtual visits, so an evaluation on counters read again divides once per edge, not twice
                float q[S], num[S];
#pragma unroll
                for (int i = 0; i < S; ++i) {
                    // (a slice none of whose edges has a visit or a value has q = +0 without dividing)
                    q[i] = 0.0f;
                    if (__builtin_amdgcn_ballot_w64(n[i] > 0 && __float_as_uint(w[i]) != 0u) != 0) q[i] = n[i] > 0 ? w[i] / (float)n[i] : 0.0f;
                    num[i] = a.cpuct * p[i] * sqrt_parent;
                }
                uint32_t keys[S];
                auto score_slice = [&](int i, int visits) {
                    return cand[i] ? score_key(q[i] + num[i] / (float)(n[i] + visits + 1)) : 0u;
                };
                auto of_edge = [&](const int (&v)[S], int eid) {
                    const int at = eid & (kWave - 1), pass = eid / kWave;
                    int r = __builtin_amdgcn_readlane(v[0], at);
#pragma unroll
                    for (int i = 1; i < S; ++i)
                        if (pass == i) r = __builtin_amdgcn_readlane(v[i], at);
                    return r;
                };
                int best_eid = kNoEdge, held = 0;
                if (PRECLAIM) {
                    // :448-483: claim every candidate, score it with the count found, keep the winner's claim
                    int tie_offset = wid;
                    if (tie_offset >= cur_expanded) tie_offset %= cur_expanded;
#pragma unroll
                    for (int i = 0; i < S; ++i) {
                        int before = 0;
                        if (cand[i]) before = visits_of.add(c[i], 1);
                        keys[i] = score_slice(i, before);
                    }
                    best_eid = best_edge<S>(keys, lane, -1, tie_offset);
#pragma unroll
                    for (int i = 0; i < S; ++i)
                        if (cand[i] && lane + i * kWave != best_eid) visits_of.sub(c[i], 1);
                    held = best_eid != kNoEdge ? 1 : 0;
                } else {
                    // :520-560 with MAX_RECALC_RETRY = 2 written out: the best edge by the counters as read; its child is
                    // claimed; if that child already carried claims and the node has other edges, the claim is given back and
                    // the best of the other edges is claimed and kept whatever it carries (none: the first winner again).
                    // The counters for the second evaluation are requested together with the first claim (just ahead of it, so
                    // that the wait for the claim's result covers them), before it is known whether they will be needed: the
                    // reference reads them after its release, but nothing orders those loads after its relaxed atomics on
                    // other counters, and the first winner's own counter is not among the ones the second evaluation looks at.
                    // one more visit on `child`'s counter, kept unless the counter was negative or full (:329-331): the value found
                    auto claim = [&](int child, int &found) {
                        int v = 0;
                        if (lane == 0) v = visits_of.add(child, 1);
                        found = __builtin_amdgcn_readfirstlane(v);
                        if (found < 0 || found >= INT32_MAX) {
                            if (lane == 0) visits_of.sub(child, 1);
                            return 0;
                        }
                        return 1;
                    };
#pragma unroll
                    for (int i = 0; i < S; ++i) keys[i] = score_slice(i, f[i]);
                    best_eid = best_edge<S>(keys, lane, -1, 0);
                    if (best_eid != kNoEdge) {
                        const int first_child = of_edge(c, best_eid), first_eid = best_eid;
                        const int seen = of_edge(f, first_eid);
                        bool second_round = false;
                        if (seen > 0 && seen < INT32_MAX && cur_expanded > 1) {
                            // The winner's counter already held visits when it was read.  In the execution in which no other
                            // traversal acts between that read and this traversal's claim, the claim finds the same value: a
                            // conflict, upon which the claim is given back and the other edges are evaluated on counters
                            // that are still the ones read (so the scores stand).  That execution is the one taken: nothing is
                            // added to the first winner's counter and nothing taken back.  (A claim that is added and taken back
                            // differs from it only in what other traversals may see in passing, and costs two of the three
                            // atomics and two of the five round trips of a level.)
                            second_round = true;
                        } else {
                            int again[S];
#pragma unroll
                            for (int i = 0; i < S; ++i) {
                                const int visits = visits_of.peek(cand[i] ? c[i] : 0);
                                again[i] = cand[i] ? visits : 0;
                            }
                            int found;
                            if (claim(first_child, found) == 0) {
                                // (the counter cannot be claimed: nothing is held)
                            } else if (found == 0 || cur_expanded <= 1) {
                                held = 1;
                            } else {
                                if (lane == 0) visits_of.sub(first_child, 1);
                                second_round = true;
                                // on the counters read again; other traversals' claims sit on a few edges, so most slices of a
                                // wide node read what they read before and keep their scores
#pragma unroll
                                for (int i = 0; i < S; ++i)
                                    if (S == 1 || __builtin_amdgcn_ballot_w64(again[i] != f[i]) != 0) keys[i] = score_slice(i, again[i]);
                            }
                        }
                        if (second_round) {
                            const int second = best_edge<S>(keys, lane, first_eid, 0);
                            if (second != kNoEdge) best_eid = second;
                            int found2;
                            held = claim(of_edge(c, best_eid), found2);
                        }
                    }
                }
                if (held == 0) {   // no edge leads anywhere (or the winner's counter cannot be claimed)
                    rollback_node_path(a, visits_of, path, tree, depth, lane, node_limit);
                    return -1;
                }
                // (only edges that lead to a node of the tree were candidates, so the child is one)
                if (lane == 0) path[depth] = (node << 8) | best_eid;
                return of_edge(c, best_eid);
            };

            const int slices = (cur_expanded + kWave - 1) / kWave;
            int next;
            if (slices <= 1) next = level(std::integral_constant<int, 1>{});
            else if (slices == 2) next = level(std::integral_constant<int, 2>{});
            else if (slices == 3) next = level(std::integral_constant<int, 3>{});
            else next = level(std::integral_constant<int, 4>{});
            if (next < 0) break;
            node = next;
            depth += 1;
        }
    }
    if (lane == 0) {
        a.out_selected_node[out] = final_packed;
        a.out_path_len[out] = final_len;
    }
}

// ---- backup --------------------------------------------------------------------------------------------------------
struct BackupArgs {
    int virtual_loss;
    const int *edge_child_id;
    float *edge_W;
    int *edge_N;
    int *edge_inflight;
    int *node_inflight;
    int *node_expand_inflight;
    const int *node_count;
    const int *out_selected_node;
    const int *out_path_eids;
    const int *out_path_len;
    const float *path_edge_values;
    int trees, nodes, edges, warps, path_depth;
};

// NODE_LEVEL = true: src/puct/puct_gpu_v2.py:847-927 as written (virtual loss lives in node_inflight[child], the
// selection word has no reason field).  NODE_LEVEL = false: the same conversion of virtual visits into real ones for
// the edge-level virtual loss of select_kernel; BUSY selections hold nothing and are skipped, as in
// src/puct/test_puct_gpu_v3.py:297-302.
template <bool NODE_LEVEL>
__device__ __forceinline__ void backup_traversal(const BackupArgs &a, int tree, int wid, int lane) {
    const int node_limit = a.node_count[tree];
    if (node_limit <= 0 || node_limit > a.nodes || node_limit > PUCT_PACKED_NODE_LIMIT) return;

    const size_t out = (size_t)tree * a.warps + wid;
    const int raw = a.out_selected_node[out];
    if (raw < 0) return;
    const int kind = NODE_LEVEL ? raw >> PUCT_PACKED_KIND_SHIFT : (raw >> PUCT_PACKED_KIND_SHIFT) & PUCT_PACKED_KIND_MASK;
    if (kind == PUCT_SELECT_INVALID) return;
    if (!NODE_LEVEL && kind == PUCT_SELECT_BUSY) return;
    const int plen = a.out_path_len[out];
    if (plen <= 0) return;

    int edge_count = plen - 1;
    if (edge_count > a.path_depth) edge_count = a.path_depth;
    const int *path = a.out_path_eids + out * a.path_depth;
    for (int d = lane; d < edge_count; d += kWave) {
        const int encoded = path[d];
        if (encoded < 0) continue;
        const int parent = encoded >> 8, slot = encoded & 0xFF;
        if (parent >= node_limit || slot >= a.edges) continue;
        const size_t e = ((size_t)tree * a.nodes + parent) * a.edges + slot;
        if (NODE_LEVEL) {
            const int child = a.edge_child_id[e];
            if (child >= 0 && child < node_limit)
                atomicSub(&a.node_inflight[(size_t)tree * a.nodes + child], a.virtual_loss);
        } else {
            atomicSub(&a.edge_inflight[e], a.virtual_loss);
        }
        if (a.path_edge_values != nullptr) {
            atomicAdd(&a.edge_N[e], 1);
            unsafeAtomicAdd(&a.edge_W[e], a.path_edge_values[out * a.path_depth + d]);
        }
    }

    if (lane == 0 && kind == PUCT_SELECT_EXPAND) {
        const int leaf = raw & PUCT_PACKED_NODE_MASK;
        if (leaf < node_limit) atomicSub(&a.node_expand_inflight[(size_t)tree * a.nodes + leaf], 1);
    }
}


}  // namespace puct
