// Gomoku PUCT search loop with virtual loss behind include/puct_gomoku.h: selection, expansion / evaluation and backup of
// all steps of a search in one launch, one workgroup per tree and one wavefront per traversal, on the loop's own tree
// storage (one 16-byte record per edge, one per node), and the host engine.  A tree belongs to one workgroup for the
// whole launch, so the traversals' claims are taken in a fixed order on registers instead of with atomics in memory,
// which also makes a search reproducible.
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "puct_device.hpp"
#include "puct_synthetic.h"
#include "../../include/puct_gomoku.h"

namespace {
using namespace puct;

constexpr int kEdges = 256;       // edge slots per node (MAX_ACTION of src/puct/puct_gpu_v2.py:72)
constexpr int kBoardWords = 16;   // 8 words per colour

struct Edge {
    int n;          // visits
    float w;        // value sum, for the player who moves along the edge
    float prior;
    uint32_t link;  // child << 8 | claims in flight (virtual loss); child 0 = none (node 0 is the root)
};
static_assert(sizeof(Edge) == 16, "one edge is one 16-byte load");

struct NodeInfo {
    int expanded;    // edge slots with a child, or PUCT_NODE_EXPANDED_TERMINAL
    int tickets;     // expansion tickets in flight
    int legal_turn;  // empty cells of the position (most children the node can have) | 0x10000 if -1 is to move
    float value;     // of the position for its player to move
};
static_assert(sizeof(NodeInfo) == 16, "one node word is one 16-byte load");
constexpr int kTurnBit = 0x10000;

constexpr int kTrav = kMaxWavesPerBlock;   // most traversals per tree: one wavefront each, one workgroup per tree
constexpr int kSlices = kEdges / kWave;    // 64-edge slices of the widest node
constexpr int kTally = 12;

struct LoopArgs {
    Edge *edges;       // [trees][max_nodes][256]
    NodeInfo *info;    // [trees][max_nodes]
    uint32_t *board;   // [trees][max_nodes][16]
    uint8_t *action;   // [trees][max_nodes][256]: cell of every edge slot
    int *node_count;   // [trees]
    // what the traversals of the last step ended with, [trees][traversals] (paths: [trees][traversals][path_depth])
    int *out_selected, *out_len, *out_claims, *out_path;
    float *out_value;
    unsigned long long *tally;   // [trees][12]: selections by kind (0..4), children created (5), nodes read (6), edges scored (7),
                                 // ticks of the 100 MHz clock that wavefront 0 spent selecting (8), expanding (9), backing up (10)
    float cpuct, c_pw, alpha_pw;
    int m, n, cells, max_nodes, traversals, path_depth, steps;
    uint64_t seed;
    float dirichlet_alpha;
    struct EvalRequests *requests;   // [trees]
    int evaluators;                  // workgroups per tree that work out the priors of new nodes (fused search), 0 = none
    int agent_fences;                // hand-overs between a tree and its evaluators always write the L2 back
};

// What a tree's workgroup hands to its evaluator workgroups, step by step: the non-terminal children the step created.
struct EvalRequests {
    int tag;     // step + 1 once the step's entries are complete; -1 when the search is over
    int done;    // entries the evaluators have worked off since the search began
    int abort;   // a bounded wait gave up: everybody leaves
    int n;       // entries of the step
    int child[kMaxWavesPerBlock];       // node to evaluate, -1 = nothing to do for this entry
    uint64_t hash[kMaxWavesPerBlock];   // its position's hash
    int xcc[1 + 8];                     // XCD that the tree's workgroup [0] and its evaluators [1..] run on, -1 = not known yet
};
constexpr int kMaxEvaluators = 8;
static_assert(sizeof(EvalRequests::xcc) == sizeof(int) * (1 + kMaxEvaluators), "one entry per workgroup of a tree");

__device__ __forceinline__ int my_xcc() { return (int)(__builtin_amdgcn_s_getreg(6164) & 0xfu); }   // HW_REG_XCC_ID, bits 3:0
constexpr unsigned long long kWaitTicks = 300000000ull;   // 3 s of the 100 MHz clock: a partner that is not there

// What a step keeps per traversal between its phases.  The paths ([traversals][path_depth] words) follow in dynamic LDS.
struct StepLds {
    int cur[2][kTrav];   // node every traversal stands on, -1 once it has ended; double buffered by level parity
    int sel[kTrav];      // selection word: kind << 28 | slot << 20 | node
    int len[kTrav];      // path length as reported (nodes on the path; 0 for a traversal that reached no node)
    int claims[kTrav];   // edges the traversal holds a claim on = path entries written
    float value[kTrav];  // of the reached node, for the player who moved into it
    int want[kTrav];     // node the traversal expands, -1 if none
    int node_count;
    int requests;        // evaluation requests of this step
    int requested;       // ... and of all steps so far
    int gave_up;
    uint32_t board[kTrav][kBoardWords];
    int stage[kTrav][kWave];   // per wavefront: edges on their way from four per lane to one per lane
};

__device__ __forceinline__ int pack_sel(int kind, int node, int slot) {
    return (kind << PUCT_GOMOKU_SEL_KIND_SHIFT) | (slot << PUCT_GOMOKU_SEL_SLOT_SHIFT) | node;
}

__device__ __forceinline__ uint64_t wave_sum64(uint64_t v) {
    auto step = [](uint64_t x, auto ctrl) {
        constexpr int C = decltype(ctrl)::value;
        const uint32_t lo = (uint32_t)dpp<C>((int)(uint32_t)x);
        const uint32_t hi = (uint32_t)dpp<C>((int)(uint32_t)(x >> 32));
        return x + (((uint64_t)hi << 32) | lo);
    };
    v = step(v, std::integral_constant<int, 0xB1>{});
    v = step(v, std::integral_constant<int, 0x4E>{});
    v = step(v, std::integral_constant<int, 0x141>{});
    v = step(v, std::integral_constant<int, 0x140>{});
    return read_lane64(v, 0) + read_lane64(v, 16) + read_lane64(v, 32) + read_lane64(v, 48);
}

// Orders this wavefront's LDS writes before its later LDS reads by other lanes.
__device__ __forceinline__ void wave_lds_fence() { __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup"); }

__device__ __forceinline__ bool stone_at(const uint32_t *colour, int cell) { return (colour[cell >> 5] >> (cell & 31)) & 1u; }

// Does the stone just placed at `cell` complete a row of exactly five (src/mctsnc_game_mechanics.py:181-280: a longer
// row does not win)?  Lanes 0..3 each scan one direction; the result is uniform.
__device__ __forceinline__ bool makes_five(const uint32_t *mine, int cell, int m, int n, int lane) {
    bool hit = false;
    if (lane < 4) {
        const int dr = lane == 0 ? 0 : 1, dc = lane == 0 ? 1 : (lane == 1 ? 0 : (lane == 2 ? 1 : -1));
        const int r0 = cell / n, c0 = cell % n;
        int run = 1;
        for (int s = -1; s <= 1; s += 2)
            for (int k = 1; k < 6; ++k) {
                const int r = r0 + s * k * dr, c = c0 + s * k * dc;
                if (r < 0 || r >= m || c < 0 || c >= n || !stone_at(mine, r * n + c)) break;
                ++run;
            }
        hit = run == 5;
    }
    return __ballot(hit) != 0;
}

// Bitonic sort of the wavefront's 256 keys, largest first: element e = 4 * lane + k lives in v[k] of `lane`.  Partners
// at element distance 1 and 2 are registers of the same lane; lane distances 1, 2 and 8 are DPP moves, 4 and 16 LDS
// swizzles (no memory), 32 an LDS permute.
template <int LANE_XOR>
__device__ __forceinline__ uint32_t from_lane_xor(uint32_t x, int lane) {
    if (LANE_XOR == 1) return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0xB1, 0xf, 0xf, true);    // quad_perm [1,0,3,2]
    if (LANE_XOR == 2) return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xf, 0xf, true);    // quad_perm [2,3,0,1]
    if (LANE_XOR == 8) return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x128, 0xf, 0xf, true);   // row_ror:8
    if (LANE_XOR == 4) return (uint32_t)__builtin_amdgcn_ds_swizzle((int)x, 0x101F);                      // bit mode: xor 4
    if (LANE_XOR == 16) return (uint32_t)__builtin_amdgcn_ds_swizzle((int)x, 0x401F);                     // bit mode: xor 16
    return (uint32_t)__builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, (int)x);
}
template <int SIZE, int DIST>
__device__ __forceinline__ void bitonic_step(uint32_t (&v)[4], int lane) {
    uint32_t p[4];
    if (DIST < 4) {
#pragma unroll
        for (int k = 0; k < 4; ++k) p[k] = v[k ^ DIST];
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) p[k] = from_lane_xor<DIST / 4>(v[k], lane);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int e = 4 * lane + k;
        const bool descending = (e & SIZE) == 0, first = (e & DIST) == 0;   // SIZE == 256: every block descends
        const uint32_t hi = v[k] > p[k] ? v[k] : p[k], lo = v[k] > p[k] ? p[k] : v[k];
        v[k] = (first == descending) ? hi : lo;
    }
}
template <int SIZE, int DIST>
__device__ __forceinline__ void bitonic_merge(uint32_t (&v)[4], int lane) {
    bitonic_step<SIZE, DIST>(v, lane);
    if constexpr (DIST > 1) bitonic_merge<SIZE, DIST / 2>(v, lane);
}
template <int SIZE>
__device__ __forceinline__ void bitonic_sort(uint32_t (&v)[4], int lane) {
    if constexpr (SIZE > 2) bitonic_sort<SIZE / 2>(v, lane);
    bitonic_merge<SIZE, SIZE / 2>(v, lane);
}
__device__ __forceinline__ void sort_keys_descending(uint32_t (&v)[4], int lane) { bitonic_sort<256>(v, lane); }

__device__ __forceinline__ Edge load_edge(const Edge *p) {
    const uint4 v = *reinterpret_cast<const uint4 *>(p);
    return Edge{(int)v.x, __uint_as_float(v.y), __uint_as_float(v.z), v.w};
}
__device__ __forceinline__ void store_edge(Edge *p, int n, float w, float prior, uint32_t link) {
    *reinterpret_cast<uint4 *>(p) = make_uint4((uint32_t)n, __float_as_uint(w), __float_as_uint(prior), link);
}
__device__ __forceinline__ NodeInfo load_info(const NodeInfo *p) {
    const uint4 v = *reinterpret_cast<const uint4 *>(p);
    return NodeInfo{(int)v.x, (int)v.y, (int)v.z, __uint_as_float(v.w)};
}
__device__ __forceinline__ uint64_t lanes_below(int lane) { return (1ull << lane) - 1ull; }

// Priors of a new node: one Gamma weight per legal cell, prior = weight / sum, edge slots in descending weight order
// (ties: smaller cell first), so that progressive widening opens the most promising moves first.  Writes the whole
// record of every legal slot (no visits, no child, nothing in flight) and the slot's cell.  All 64 lanes must call it
// together.
__device__ void write_priors(const LoopArgs &g, int tree, int node, const uint32_t *board, int lane, uint64_t board_hash,
                             int n_legal) {
    constexpr int kPer = kEdges / kWave;
    uint32_t mine[kPer];
    // Rejection sampling diverges between lanes; every lane walks through its own cells and rounds independently, so
    // the wavefront runs for the largest per-lane total instead of the sum of per-cell maxima.
    int i = 0, round = 0;
#pragma unroll
    for (int k = 0; k < kPer; ++k) mine[k] = 0u;
    auto legal_cell = [&](int k) {
        const int c = lane + k * kWave;
        return c < g.cells && !stone_at(board, c) && !stone_at(board + 8, c);
    };
    while (i < kPer && !legal_cell(i)) ++i;
    uint64_t key = i < kPer ? psyn_cell_key(board_hash, lane + i * kWave) : 0;
    while (__ballot(i < kPer) != 0) {
        float x;
        const int ok = psyn_gamma_round(g.dirichlet_alpha, key, round, &x);
        if (i < kPer) {
            if (ok || round == PSYN_GAMMA_ROUNDS - 1) {
                const uint32_t weight = psyn_weight_key(x, lane + i * kWave);
#pragma unroll
                for (int k = 0; k < kPer; ++k)
                    if (k == i) mine[k] = weight;
                ++i;
                round = 0;
                while (i < kPer && !legal_cell(i)) ++i;
                if (i < kPer) key = psyn_cell_key(board_hash, lane + i * kWave);
            } else {
                ++round;
            }
        }
    }
    uint64_t sum = 0;
#pragma unroll
    for (int k = 0; k < kPer; ++k) sum += mine[k] ? psyn_key_weight(mine[k]) : 0;
    sum = wave_sum64(sum);
    // slot of a cell = rank of its key among the node's keys, largest first (0 = not a legal cell: last)
    sort_keys_descending(mine, lane);
    const size_t erow = ((size_t)tree * g.max_nodes + node) * kEdges + (size_t)kPer * lane;
    uint32_t cells_packed = 0;
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        cells_packed |= (mine[k] ? 255u - (mine[k] & 0xFFu) : 0u) << (8 * k);
        if (mine[k] != 0u) store_edge(g.edges + erow + k, 0, 0.0f, psyn_prior(psyn_key_weight(mine[k]), sum, n_legal), 0u);
    }
    if (mine[0] != 0u) *reinterpret_cast<uint32_t *>(g.action + erow) = cells_packed;   // keys descend: slot 4 * lane is the lane's first
}

// Order-preserving integer image of a score that can win: the reference starts from (-FLT_MAX, no edge) and accepts
// a score that is greater than or equal to it, so NaN and -inf never win and get 0 (src/puct/puct_gpu_v3_cpp.cu:51-71);
// -0.0f counts as +0.0f because the reference compares floats.  The upper word of candidate_key().
__device__ __forceinline__ uint32_t score_image(float score) {
    if (!(score >= -FLT_MAX)) return 0u;
    const uint32_t b = __float_as_uint(score + 0.0f);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
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

// Progressive widening, src/puct/puct_gpu_v3_cpp.cu:150-157; sqrt_n = sqrtf((float)n_node), which the score needs too.
__device__ __forceinline__ int allowed_children(float c_pw, float alpha_pw, int n_node, float sqrt_n, int edges) {
    const float val = (alpha_pw == 0.5f) ? c_pw * sqrt_n : c_pw * powf((float)n_node, alpha_pw);
    if (val >= (float)edges) return edges;
    const int allowed = (int)ceilf(val);
    return allowed > 1 ? allowed : 1;
}

// ---- selection ---------------------------------------------------------------------------------------------------
// The edges of one node as the deciding traversals see them: up to NS per lane.
template <int NS>
struct EdgeSet {
    float q[NS], cp[NS];   // mean value, cpuct * prior
    int den[NS];           // visits + claims in flight + 1
    uint32_t link[NS], link_loaded[NS];
    int eid[NS];           // edge slot, -1 = none
};

template <int NS>
__device__ __forceinline__ float edge_score(const EdgeSet<NS> &e, int i, float sqrt_parent, int more_claims) {
    return e.q[i] + e.cp[i] * sqrt_parent / (float)(e.den[i] + more_claims);
}

// The traversals `members` decide one after another on the edges in `e` (which must include every edge that can come
// first for any of them); `total` = visits + claims over all expanded edges of the node, `tickets` = expansion tickets out.
template <int NS>
__device__ __forceinline__ void decide_in_turn(const LoopArgs &g, StepLds &s, int *paths, int *next, EdgeSet<NS> &e, int node,
                                               uint64_t members, int depth, int lane, int expanded, int legal, int &total,
                                               int &tickets, bool only_one = false) {
    // sqrt(parent) and the widening limit after 0, 1, 2 ... more claims, worked out side by side in lanes 0..15 (fewer
    // than 64 traversals decide here, and every claim adds one to the node's total)
    const bool widening = expanded != 1 || g.c_pw != 0.0f;
    const int claims_base = total;
    const int eff_lane = widening ? (total + lane > 1 ? total + lane : 1) : 1;
    const float sqrt_lane = widening ? sqrtf((float)eff_lane) : 1.0f;
    const int allowed_lane = widening ? allowed_children(g.c_pw, g.alpha_pw, eff_lane, sqrt_lane, legal) : 1;
    for (uint64_t rest = members; rest != 0; rest &= rest - 1) {
        const int j = __builtin_ctzll(rest);   // the traversal deciding now
        const int claimed = total - claims_base;
        const float sqrt_parent = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(sqrt_lane), claimed));
        const int allowed = __builtin_amdgcn_readlane(allowed_lane, claimed);
        if (allowed > expanded) {
            if (expanded + tickets < allowed) {   // expansion ticket
                if (lane == 0) {
                    s.sel[j] = pack_sel(PUCT_SELECT_EXPAND, node, expanded + tickets);
                    s.len[j] = depth + 1;
                    s.claims[j] = depth;
                    next[j] = -1;
                }
                tickets += 1;
                continue;
            }
            if (expanded == 0) {   // the node's only allowed child is being created by another traversal
                if (lane == 0) {
                    s.sel[j] = pack_sel(PUCT_SELECT_BUSY, node, 0);
                    s.len[j] = 0;
                    s.claims[j] = depth;
                    next[j] = -1;
                }
                continue;
            }
        }
        // The highest score first: its order-preserving integer image, reduced over the wavefront.  Only if more than
        // one edge attains it does the rotated edge index decide, through the full keys.  (A node's only edge is taken
        // whatever its score, as in the reference.)
        int best_lane = 0, best_slot = 0, hits = 1;
        if (expanded > 1 && !only_one) {
            float score[NS];
            uint32_t image[NS], lane_top = 0;
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                score[i] = edge_score(e, i, sqrt_parent, 0);
                image[i] = e.eid[i] >= 0 ? score_image(score[i]) : 0u;
                lane_top = image[i] > lane_top ? image[i] : lane_top;
            }
            const uint32_t top = wave_max_u32(lane_top);
            hits = 0;
#pragma unroll
            for (int i = 0; i < NS; ++i) {
                const uint64_t at = __ballot(image[i] == top);
                hits += __popcll(at);
                if (at != 0) best_lane = __builtin_ctzll(at), best_slot = i;
            }
            if (top == 0) {
                hits = 0;
            } else if (hits > 1) {
                int tie_offset = j;
                if (tie_offset >= expanded) tie_offset %= expanded;
                uint64_t key = 0;
                int key_slot = 0;
#pragma unroll
                for (int i = 0; i < NS; ++i) {
                    const uint64_t k = image[i] == top ? candidate_key(score[i], e.eid[i], tie_offset, expanded) : 0;
                    if (k > key) key = k, key_slot = i;
                }
                const uint64_t first = wave_max(key);
                best_lane = __builtin_ctzll(__ballot(key == first));
                best_slot = __builtin_amdgcn_readlane(key_slot, best_lane);
            }
        }
        int child = 0, best = 0;
        if (hits > 0) {
#pragma unroll
            for (int i = 0; i < NS; ++i)
                if (best_slot == i) {
                    child = (int)((uint32_t)__builtin_amdgcn_readlane((int)e.link[i], best_lane) >> 8);
                    best = __builtin_amdgcn_readlane(e.eid[i], best_lane);
                }
        }
        if (child <= 0 || child >= g.max_nodes) {   // no edge with a comparable score, or a link that leads nowhere
            if (lane == 0) {
                s.sel[j] = pack_sel(PUCT_SELECT_INVALID, PUCT_GOMOKU_SEL_NODE_MASK, 0);
                s.len[j] = 0;
                s.claims[j] = depth;
                next[j] = -1;
            }
            continue;
        }
#pragma unroll
        for (int i = 0; i < NS; ++i)
            if (best_slot == i && lane == best_lane) {
                e.den[i] += 1;
                e.link[i] += 1u;
            }
        total += 1;
        if (lane == 0) {
            paths[j * g.path_depth + depth] = (node << 8) | best;
            next[j] = child;
        }
    }
}

// The traversals of a tree descend in lockstep, one level per round.  The traversals that stand on the same node are
// served by one wavefront (that of the first of them), which loads the node's edges once and lets the traversals decide
// one after another, wid ascending, on registers: every decision is the reference's (progressive widening, expansion
// ticket, score, order on edges with the rotated tie-break: src/puct/puct_gpu_v3_cpp.cu:150-275) on the state that the
// claims of the traversals before it have left.  Taking the claims in turn is one of the interleavings the reference's
// atomics allow, needs no atomics itself, never loses a claim and makes a search reproducible.
__device__ void select_group(const LoopArgs &g, StepLds &s, int *paths, int *next, int tree, int node, uint64_t members,
                             int depth, int wave, int lane, uint32_t &nodes_read, uint32_t &edges_scored) {
    const size_t nrow = (size_t)tree * g.max_nodes + node;
    Edge *row = g.edges + nrow * kEdges;
    // all 256 edge slots are requested together with the node's own word, before anything about the node is known: one
    // round trip per level, whatever the node's width
    Edge loaded[kSlices];
#pragma unroll
    for (int i = 0; i < kSlices; ++i) loaded[i] = load_edge(row + lane + i * kWave);
    const NodeInfo ni = load_info(g.info + nrow);
    const int expanded = ni.expanded;
    nodes_read += 1;
    if (expanded == PUCT_NODE_EXPANDED_TERMINAL || depth >= g.path_depth) {
        const int kind = expanded == PUCT_NODE_EXPANDED_TERMINAL ? PUCT_SELECT_TERMINAL : PUCT_SELECT_DEPTH_LIMIT;
        if (lane < kTrav && ((members >> lane) & 1ull)) {
            s.sel[lane] = pack_sel(kind, node, 0);
            s.len[lane] = depth + 1;
            s.claims[lane] = depth;
            next[lane] = -1;
        }
        return;
    }
    edges_scored += (uint32_t)expanded;

    EdgeSet<kSlices> all;
    int total = 0;
#pragma unroll
    for (int i = 0; i < kSlices; ++i) {
        const Edge e = loaded[i];
        const bool valid = lane + i * kWave < expanded;
        all.q[i] = valid && e.n > 0 ? e.w / (float)e.n : 0.0f;
        all.cp[i] = g.cpuct * e.prior;
        all.link[i] = all.link_loaded[i] = e.link;
        all.den[i] = e.n + (int)(e.link & 0xFFu) + 1;
        all.eid[i] = valid ? lane + i * kWave : -1;
        total += valid ? all.den[i] - 1 : 0;
    }
    total = wave_sum(total);
    int tickets = ni.tickets;
    const int legal = ni.legal_turn & 0xFFFF, n_members = __popcll(members);

    // Every one of these traversals takes the same edge: all of them at once, a traversal per lane.
    auto take_all = [&](uint32_t link, int eid) {
        const int child = (int)(link >> 8);
        const bool leads_somewhere = child > 0 && child < g.max_nodes;
        if (lane < kTrav && ((members >> lane) & 1ull)) {
            if (leads_somewhere) {
                paths[lane * g.path_depth + depth] = (node << 8) | eid;
                next[lane] = child;
            } else {
                s.sel[lane] = pack_sel(PUCT_SELECT_INVALID, PUCT_GOMOKU_SEL_NODE_MASK, 0);
                s.len[lane] = 0;
                s.claims[lane] = depth;
                next[lane] = -1;
            }
        }
        if (leads_somewhere && lane == 0) row[eid].link = link + (uint32_t)n_members;
    };
    // No expansion ticket is to be had here however many of these traversals have claimed: the widening limit grows with
    // the claims, and its largest value, the one the last of them sees, does not exceed the children there are.
    const auto no_ticket_for_anyone = [&] {
        if (expanded < 1) return false;
        if (expanded == 1 && g.c_pw == 0.0f) return true;
        const int eff_last = total + n_members - 1 > 1 ? total + n_members - 1 : 1;
        return allowed_children(g.c_pw, g.alpha_pw, eff_last, sqrtf((float)eff_last), legal) <= expanded;
    };

    if (expanded <= kWave) {
        bool taken = false;
        if (n_members >= 3 && no_ticket_for_anyone()) {
            // one edge per lane: which of them can come first for any of these traversals (the bounds of the wide case below)
            uint64_t in = 1ull;   // (a node's only edge is taken whatever its score)
            if (expanded > 1) {
                const int now = total > 1 ? total : 1, then = total + n_members > 1 ? total + n_members : 1;
                const uint32_t l = all.eid[0] >= 0 ? score_image(edge_score(all, 0, sqrtf((float)now), n_members)) : 0u;
                const uint32_t h = all.eid[0] >= 0 ? score_image(edge_score(all, 0, sqrtf((float)then), 0)) : 0u;
                const uint32_t low = wave_max_u32(l);
                in = __ballot(low != 0 && h >= low && h != 0);
            }
            if (__popcll(in) == 1) {
                const int at = __builtin_ctzll(in);
                take_all((uint32_t)__builtin_amdgcn_readlane((int)all.link[0], at), at);
                taken = true;
            }
        }
        if (!taken) {
            EdgeSet<1> one{{all.q[0]}, {all.cp[0]}, {all.den[0]}, {all.link[0]}, {all.link_loaded[0]}, {all.eid[0]}};
            decide_in_turn<1>(g, s, paths, next, one, node, members, depth, lane, expanded, legal, total, tickets);
            if (one.link[0] != one.link_loaded[0]) row[lane].link = one.link[0];
        }
    } else {
        // A wide node with several traversals on it: most edges cannot come first for any of them.  While these
        // traversals decide, sqrt(parent) only grows (by their own claims) and an edge's claims only grow, and every
        // operation of the score is monotonic, so an edge's score stays below its score at the largest sqrt(parent) and
        // its present claims, and the best edge's score stays above the largest score at the present sqrt(parent) with
        // all of these traversals' claims on it.  Edges whose upper bound is below that lower bound are out; when at
        // most 64 remain they move to one edge per lane and a decision costs one division instead of four.
        bool pruned = false;
        if (n_members >= 3) {
            const int now = total > 1 ? total : 1, then = total + n_members > 1 ? total + n_members : 1;
            const float sqrt_now = sqrtf((float)now), sqrt_then = sqrtf((float)then);
            uint32_t low = 0, high[kSlices];
#pragma unroll
            for (int i = 0; i < kSlices; ++i) {
                const uint32_t l = all.eid[i] >= 0 ? score_image(edge_score(all, i, sqrt_now, n_members)) : 0u;
                high[i] = all.eid[i] >= 0 ? score_image(edge_score(all, i, sqrt_then, 0)) : 0u;
                low = l > low ? l : low;
            }
            low = wave_max_u32(low);
            int kept = 0, place[kSlices];
            uint64_t in_slice[kSlices];
#pragma unroll
            for (int i = 0; i < kSlices; ++i) {
                const bool in = low != 0 && high[i] >= low && high[i] != 0;
                const uint64_t mask = __ballot(in);
                in_slice[i] = mask;
                place[i] = in ? kept + __popcll(mask & lanes_below(lane)) : -1;
                kept += __popcll(mask);
            }
            // One edge left and no expansion ticket to be had: every one of these traversals takes that edge.
            if (kept == 1 && low != 0 && no_ticket_for_anyone()) {
                pruned = true;
#pragma unroll
                for (int i = 0; i < kSlices; ++i)
                    if (in_slice[i] != 0) {
                        const int at = __builtin_ctzll(in_slice[i]);
                        take_all((uint32_t)__builtin_amdgcn_readlane((int)all.link[i], at), at + i * kWave);
                    }
            }
            if (!pruned && kept >= 1 && kept <= kWave && low != 0) {
                pruned = true;
                // through LDS into one edge per lane
                EdgeSet<1> few{{0.0f}, {0.0f}, {1}, {0u}, {0u}, {-1}};
                int *stage = s.stage[wave];
#pragma unroll
                for (int f = 0; f < 5; ++f) {
#pragma unroll
                    for (int i = 0; i < kSlices; ++i)
                        if (place[i] >= 0)
                            stage[place[i]] = f == 0 ? __float_as_int(all.q[i]) : f == 1 ? __float_as_int(all.cp[i]) : f == 2 ? all.den[i]
                                            : f == 3 ? (int)all.link[i] : all.eid[i];
                    wave_lds_fence();
                    const int v = lane < kept ? stage[lane] : 0;
                    wave_lds_fence();
                    if (f == 0) few.q[0] = __int_as_float(v);
                    if (f == 1) few.cp[0] = __int_as_float(v);
                    if (f == 2) few.den[0] = lane < kept ? v : 1;
                    if (f == 3) few.link[0] = few.link_loaded[0] = (uint32_t)v;
                    if (f == 4) few.eid[0] = lane < kept ? v : -1;
                }
                decide_in_turn<1>(g, s, paths, next, few, node, members, depth, lane, expanded, legal, total, tickets, kept == 1);
                if (few.eid[0] >= 0 && few.link[0] != few.link_loaded[0]) row[few.eid[0]].link = few.link[0];
            }
        }
        if (!pruned) {
            decide_in_turn<kSlices>(g, s, paths, next, all, node, members, depth, lane, expanded, legal, total, tickets);
#pragma unroll
            for (int i = 0; i < kSlices; ++i)
                if (all.link[i] != all.link_loaded[i]) row[lane + i * kWave].link = all.link[i];
        }
    }
    if (lane == 0 && tickets != ni.tickets) g.info[nrow].tickets = tickets;
}

// Selection of one step for the traversals of one tree; all wavefronts of the workgroup call it.  Ends behind a
// workgroup barrier with every traversal's result in `s` and its path in `paths`.
__device__ void select_phase(const LoopArgs &g, StepLds &s, int *paths, int tree, int wave, int lane, int n_waves,
                             uint32_t &nodes_read, uint32_t &edges_scored) {
    if (threadIdx.x < kTrav) {
        const int t = threadIdx.x;
        s.cur[0][t] = t < n_waves ? 0 : -1;
        s.cur[1][t] = -1;
        s.sel[t] = pack_sel(PUCT_SELECT_INVALID, PUCT_GOMOKU_SEL_NODE_MASK, 0);
        s.len[t] = 0;
        s.claims[t] = 0;
        s.value[t] = 0.0f;
    }
    __syncthreads();
    for (int depth = 0;; ++depth) {
        const int *cur = s.cur[depth & 1];
        int *next = s.cur[(depth & 1) ^ 1];
        const int at = lane < kTrav ? cur[lane] : -1;
        if (__ballot(at >= 0) == 0) break;   // every wavefront reads the same words: all leave together
        const int mine = __builtin_amdgcn_readlane(at, wave);
        const uint64_t members = __ballot(at >= 0 && at == mine);
        if (mine < 0) {
            if (lane == 0) next[wave] = -1;
        } else if ((members & lanes_below(wave)) == 0) {
            select_group(g, s, paths, next, tree, mine, members, depth, wave, lane, nodes_read, edges_scored);
        }
        __syncthreads();
    }
}

// ---- expansion / evaluation -----------------------------------------------------------------------------------------
// Every wavefront handles the leaf of its own traversal.  Children get consecutive node ids in traversal order and go
// into the node's next free edge slots in traversal order (the expanded edges of a node stay contiguous whatever the
// tickets say); when the tree cannot take all expansions of a step none is committed (those traversals evaluate the
// node they reached instead).
template <bool FARM>
__device__ void expand_phase(const LoopArgs &g, StepLds &s, int tree, int wave, int lane, int n_waves, uint32_t &created) {
    const int raw = s.sel[wave];
    const int kind = (raw >> PUCT_GOMOKU_SEL_KIND_SHIFT) & 7;
    const int node = raw & PUCT_GOMOKU_SEL_NODE_MASK, ticket_slot = (raw >> PUCT_GOMOKU_SEL_SLOT_SHIFT) & 0xFF;
    const size_t trow = (size_t)tree * g.max_nodes;
    const uint64_t tree_seed = psyn_tree_seed(g.seed, tree);
    const bool has_node = kind == PUCT_SELECT_EXPAND || kind == PUCT_SELECT_TERMINAL || kind == PUCT_SELECT_DEPTH_LIMIT;
    uint32_t *board = s.board[wave];
    NodeInfo ni{0, 0, 0, 0.0f};
    if (has_node) {
        const uint32_t w = lane < kBoardWords ? g.board[(trow + node) * kBoardWords + lane] : 0u;
        ni = load_info(g.info + trow + node);
        if (lane < kBoardWords) board[lane] = w;
        wave_lds_fence();
    }
    const int n_legal = ni.legal_turn & 0xFFFF, turn = (ni.legal_turn & kTurnBit) ? -1 : 1;
    const bool wants = kind == PUCT_SELECT_EXPAND && ticket_slot < n_legal;
    if (lane == 0) s.want[wave] = wants ? node : -1;
    __syncthreads();
    if (FARM) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");   // the evaluators' priors of the step before (see search_kernel)
    const int other = lane < n_waves ? s.want[lane] : -1;
    const uint64_t all = __ballot(other >= 0), here = __ballot(other >= 0 && other == node);
    const int total = __popcll(all), before = __popcll(all & lanes_below(wave));
    const int rank = __popcll(here & lanes_below(wave)), siblings = __popcll(here);
    const int base = s.node_count;
    const bool fits = base + total <= g.max_nodes;
    __syncthreads();
    if (wave == 0 && lane == 0) {
        if (fits) s.node_count = base + total;
        s.requests = fits ? total : 0;
    }
    if (wave == 0 && fits) created += (uint32_t)total;

    float u = 0.0f;   // value of the reached node for the player who moved into it
    if (wants && fits) {
        const int child = base + before, slot = ni.expanded + rank;
        const size_t erow = (trow + node) * kEdges;
        const int action = g.action[erow + slot];
        uint32_t *mine = board + (turn > 0 ? 0 : 8);
        if (lane == 0) mine[action >> 5] |= 1u << (action & 31);
        wave_lds_fence();
        const bool win = makes_five(mine, action, g.m, g.n, lane);
        const int child_legal = n_legal - 1;
        const bool terminal = win || child_legal == 0;
        const uint64_t bh = psyn_board_hash(tree_seed, board);
        const float v_child = win ? -1.0f : (terminal ? 0.0f : psyn_value(bh));
        if (lane < kBoardWords) g.board[(trow + child) * kBoardWords + lane] = board[lane];
        if (lane == 0) {
            *reinterpret_cast<uint4 *>(g.info + trow + child) =
                make_uint4((uint32_t)(terminal ? PUCT_NODE_EXPANDED_TERMINAL : 0), 0u,
                           (uint32_t)(child_legal | (turn > 0 ? kTurnBit : 0)), __float_as_uint(v_child));
            Edge *e = g.edges + erow + slot;
            e->n = 1;
            e->w = -v_child;
            e->link = (uint32_t)child << 8;
            if (rank == 0) g.info[trow + node].expanded = ni.expanded + siblings;
        }
        if (FARM) {   // the child's priors are an evaluator workgroup's work
            if (lane == 0) {
                g.requests[tree].child[before] = terminal ? -1 : child;
                g.requests[tree].hash[before] = bh;
            }
        } else if (!terminal) {
            write_priors(g, tree, child, board, lane, bh, child_legal);
        }
        u = -v_child;
    } else if (kind == PUCT_SELECT_TERMINAL) {
        u = ni.value;
    } else if (has_node) {
        u = psyn_value(psyn_board_hash(tree_seed, board));
    }
    if (lane == 0) s.value[wave] = u;
}

// ---- backup ----------------------------------------------------------------------------------------------------------
// Every traversal gives back the claims along its path; one that reached a node (expansion, terminal, depth limit) also
// leaves a visit and the node's value, sign alternating, on every edge of the path (src/puct/puct_gpu_v2.py:847-927
// moved to edge-level virtual loss), and an expansion returns its ticket.  Lane = (traversal, one of four depths): the
// traversals whose paths share an edge at that depth meet inside a row of 16 lanes, and the last of them stores the
// edge after adding the values in traversal order, so the float sums do not depend on timing.
__device__ void backup_phase(const LoopArgs &g, StepLds &s, const int *paths, int tree, int wave, int lane, int n_waves) {
    const size_t trow = (size_t)tree * g.max_nodes;
    const int t = lane & (kTrav - 1), sub = lane >> 4;
    const int raw = s.sel[t], my_claims = s.claims[t];
    const int kind = (raw >> PUCT_GOMOKU_SEL_KIND_SHIFT) & 7;
    const int counted = (kind == PUCT_SELECT_EXPAND || kind == PUCT_SELECT_TERMINAL || kind == PUCT_SELECT_DEPTH_LIMIT) ? 1 : 0;
    const float u = s.value[t];
    int deepest = 0;
    for (int j = 0; j < n_waves; ++j) deepest = s.claims[j] > deepest ? s.claims[j] : deepest;
    for (int d0 = 4 * wave; d0 < deepest; d0 += 4 * n_waves) {
        const int d = d0 + sub;
        const int enc = d < my_claims ? paths[t * g.path_depth + d] : -1;
        const float val = ((my_claims - d) & 1) ? -u : u;   // a counted traversal's path has as many edges as claims
        Edge *e = nullptr;
        int n_old = 0;
        float acc = 0.0f;
        uint32_t link_old = 0;
        if (enc >= 0) {
            e = g.edges + (trow + (enc >> 8)) * kEdges + (enc & 0xFF);
            n_old = e->n;
            acc = e->w;
            link_old = e->link;
        }
        int visits = 0, released = 0;
        bool last = true;
#pragma unroll
        for (int j = 0; j < kTrav; ++j) {
            const int src = ((lane & ~(kTrav - 1)) | j) << 2;
            const int enc_j = __builtin_amdgcn_ds_bpermute(src, enc);
            const float val_j = __int_as_float(__builtin_amdgcn_ds_bpermute(src, __float_as_int(val)));
            const int counted_j = __builtin_amdgcn_ds_bpermute(src, counted);
            const bool same = enc >= 0 && enc_j == enc;
            if (same && j <= t) {
                released += 1;
                if (counted_j) {
                    acc += val_j;
                    visits += 1;
                }
            }
            if (same && j > t) last = false;
        }
        if (enc >= 0 && last) {
            e->n = n_old + visits;
            e->w = acc;
            e->link = link_old - (uint32_t)released;
        }
    }
    if (wave == 0) {   // expansion tickets back, once per node
        const int sel_l = lane < n_waves ? s.sel[lane] : 0;
        const bool is_exp = lane < n_waves && ((sel_l >> PUCT_GOMOKU_SEL_KIND_SHIFT) & 7) == PUCT_SELECT_EXPAND;
        const int node_l = sel_l & PUCT_GOMOKU_SEL_NODE_MASK;
        int returned = 0;
        bool first = true;
        for (int j = 0; j < n_waves; ++j) {
            const int node_j = __builtin_amdgcn_readlane(node_l, j);
            const bool exp_j = (__ballot(is_exp) >> j) & 1ull;
            if (exp_j && node_j == node_l) {
                returned += 1;
                if (j < lane) first = false;
            }
        }
        if (is_exp && first) g.info[trow + node_l].tickets -= returned;
    }
}

// Root of every tree: node 0 with the root position and its priors.
__global__ __launch_bounds__(kWave) void init_kernel(const LoopArgs g, const uint32_t *root_board, int root_turn) {
    __shared__ uint32_t board[kBoardWords];
    const int tree = blockIdx.x, lane = threadIdx.x;
    const size_t trow = (size_t)tree * g.max_nodes;
    const uint32_t w = lane < kBoardWords ? root_board[lane] : 0u;
    if (lane < kBoardWords) {
        board[lane] = w;
        g.board[trow * kBoardWords + lane] = w;
    }
    const int n_legal = g.cells - wave_sum(__popc(w));
    wave_lds_fence();
    if (lane < kTally) g.tally[(size_t)tree * kTally + lane] = 0ull;
    if (lane < g.traversals) {
        const size_t out = (size_t)tree * g.traversals + lane;
        g.out_selected[out] = pack_sel(PUCT_SELECT_INVALID, PUCT_GOMOKU_SEL_NODE_MASK, 0);
        g.out_len[out] = 0;
        g.out_claims[out] = 0;
        g.out_value[out] = 0.0f;
    }
    if (lane == 0) {
        *reinterpret_cast<uint4 *>(g.info + trow) =
            make_uint4((uint32_t)(n_legal == 0 ? PUCT_NODE_EXPANDED_TERMINAL : 0), 0u,
                       (uint32_t)(n_legal | (root_turn > 0 ? 0 : kTurnBit)), 0u);
        g.node_count[tree] = 1;
        EvalRequests &rq = g.requests[tree];
        rq.tag = 0;
        rq.done = 0;
        rq.abort = 0;
        rq.n = 0;
        for (int &x : rq.xcc) x = -1;
    }
    if (n_legal > 0) write_priors(g, tree, 0, board, lane, psyn_board_hash(psyn_tree_seed(g.seed, tree), board), n_legal);
}

// Makes the stores of a phase visible to the loads of the next one.  All wavefronts of a tree run on one CU and share
// its write-through L1 and the L2 behind it, so no L2 write-back is needed; what is needed is (1) that every
// wavefront's stores of the phase have been acknowledged by the L2 before any wavefront goes on -- a workgroup-scope
// release fence does not wait for that on one CU (it lowers to no vector-memory wait) -- hence the explicit wait on the
// wavefront's own outstanding vector memory operations; and (2) that the L1 drops the lines which other wavefronts have
// changed underneath it: the agent-scope acquire.
__device__ __forceinline__ void phase_barrier() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

// What the traversals of a step ended with, between the launches of the stepwise mode and for the host to read.
__device__ void state_to_memory(const LoopArgs &g, const StepLds &s, const int *paths, int tree, int n_waves) {
    const size_t out = (size_t)tree * g.traversals;
    for (int i = threadIdx.x; i < n_waves * g.path_depth; i += n_waves * kWave) {   // the workgroup's live threads
        const int t = i / g.path_depth, d = i - t * g.path_depth;
        g.out_path[out * g.path_depth + i] = d < s.claims[t] ? paths[i] : -1;
    }
    if (threadIdx.x < n_waves) {
        const int t = threadIdx.x;
        g.out_selected[out + t] = s.sel[t];
        g.out_len[out + t] = s.len[t];
        g.out_claims[out + t] = s.claims[t];
        g.out_value[out + t] = s.value[t];
    }
    if (threadIdx.x == 0) g.node_count[tree] = s.node_count;
}
__device__ void state_from_memory(const LoopArgs &g, StepLds &s, int *paths, int tree, int n_waves) {
    const size_t out = (size_t)tree * g.traversals;
    for (int i = threadIdx.x; i < n_waves * g.path_depth; i += n_waves * kWave) paths[i] = g.out_path[out * g.path_depth + i];
    if (threadIdx.x < kTrav) {
        const int t = threadIdx.x;
        const bool live = t < n_waves;
        s.sel[t] = live ? g.out_selected[out + t] : pack_sel(PUCT_SELECT_INVALID, PUCT_GOMOKU_SEL_NODE_MASK, 0);
        s.len[t] = live ? g.out_len[out + t] : 0;
        s.claims[t] = live ? g.out_claims[out + t] : 0;
        s.value[t] = live ? g.out_value[out + t] : 0.0f;
    }
    if (threadIdx.x == 0) s.node_count = g.node_count[tree];
    __syncthreads();
}

struct Work {
    uint32_t kinds[5] = {0, 0, 0, 0, 0}, created = 0, nodes_read = 0, edges_scored = 0;
    uint64_t ticks[3] = {0, 0, 0};   // selection, expansion, backup, on wavefront 0
    __device__ void count_kind(const StepLds &s, int wave) {
        const int kind = (s.sel[wave] >> PUCT_GOMOKU_SEL_KIND_SHIFT) & 7;
#pragma unroll
        for (int k = 0; k < 5; ++k) kinds[k] += kind == k ? 1u : 0u;
    }
    __device__ void to_memory(const LoopArgs &g, int tree, int lane) const {
        if (lane != 0) return;
        unsigned long long *row = g.tally + (size_t)tree * kTally;
#pragma unroll
        for (int k = 0; k < 5; ++k)
            if (kinds[k]) atomicAdd(row + k, (unsigned long long)kinds[k]);
        if (created) atomicAdd(row + 5, (unsigned long long)created);
        if (nodes_read) atomicAdd(row + 6, (unsigned long long)nodes_read);
        if (edges_scored) atomicAdd(row + 7, (unsigned long long)edges_scored);
#pragma unroll
        for (int k = 0; k < 3; ++k)
            if (ticks[k]) atomicAdd(row + 8 + k, (unsigned long long)ticks[k]);
    }
};

extern __shared__ int dynamic_lds[];

// ---- evaluator workgroups --------------------------------------------------------------------------------------------
// The priors of a new node are a pure function of its position, and nothing reads them before the next step's
// selection, so they need not be worked out on the compute unit that owns the tree: the tree's workgroup posts the
// step's new nodes, goes on with its backup, and picks the results up before the next step.  An evaluator workgroup
// takes two nodes at a time, four wavefronts and one cell per lane each; the slot of a cell is the number of larger keys
// among the node's 256, counted from LDS.  Same priors, bit for bit, as write_priors().
struct EvalLds {
    uint32_t keys[2][kEdges];
    unsigned long long weight[2][4];
    int legal[2][4];
    int tag;
};

__device__ __forceinline__ int poll_word(const int *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// Entries `first` and `first + 1` of the step, by wavefronts 0..3 and 4..7 of the workgroup; all eight must call it.
__device__ void evaluate_pair(const LoopArgs &g, EvalLds &L, int tree, int first, int n, int wave, int lane) {
    const EvalRequests &rq = g.requests[tree];
    const int group = wave >> 2, part = wave & 3, index = first + group;
    const int child = index < n ? rq.child[index] : -1;
    const bool active = child > 0;
    const size_t trow = (size_t)tree * g.max_nodes;
    const int cell = part * kWave + lane;
    uint32_t weight_key = 0;
    bool legal = false;
    if (active) {
        const uint32_t w = lane < kBoardWords ? g.board[(trow + child) * kBoardWords + lane] : 0u;
        // words of the lane's cell: the same for each half of the wavefront
        uint32_t plus = (uint32_t)__builtin_amdgcn_readlane((int)w, 2 * part), minus = (uint32_t)__builtin_amdgcn_readlane((int)w, 8 + 2 * part);
        const uint32_t plus_hi = (uint32_t)__builtin_amdgcn_readlane((int)w, 2 * part + 1);
        const uint32_t minus_hi = (uint32_t)__builtin_amdgcn_readlane((int)w, 8 + 2 * part + 1);
        if (lane >= 32) plus = plus_hi, minus = minus_hi;
        legal = cell < g.cells && !(((plus | minus) >> (lane & 31)) & 1u);
        const uint64_t key = psyn_cell_key(rq.hash[index], cell);
        bool pending = legal;
        for (int round = 0; __ballot(pending) != 0; ++round) {
            float x;
            const int ok = psyn_gamma_round(g.dirichlet_alpha, key, round, &x);
            if (pending && (ok || round == PSYN_GAMMA_ROUNDS - 1)) {
                weight_key = psyn_weight_key(x, cell);
                pending = false;
            }
        }
    }
    L.keys[group][cell] = weight_key;
    const uint64_t part_sum = wave_sum64(weight_key ? psyn_key_weight(weight_key) : 0);
    const int part_legal = __popcll(__ballot(legal));
    if (lane == 0) {
        L.weight[group][part] = part_sum;
        L.legal[group][part] = part_legal;
    }
    __syncthreads();
    if (legal) {
        const uint64_t sum = L.weight[group][0] + L.weight[group][1] + L.weight[group][2] + L.weight[group][3];
        const int n_legal = L.legal[group][0] + L.legal[group][1] + L.legal[group][2] + L.legal[group][3];
        int slot = 0;
        const uint4 *keys = reinterpret_cast<const uint4 *>(L.keys[group]);
#pragma unroll 8
        for (int c = 0; c < kEdges / 4; ++c) {
            const uint4 k = keys[c];
            slot += (k.x > weight_key) + (k.y > weight_key) + (k.z > weight_key) + (k.w > weight_key);
        }
        const size_t e = (trow + child) * kEdges + slot;
        store_edge(g.edges + e, 0, 0.0f, psyn_prior(psyn_key_weight(weight_key), sum, n_legal), 0u);
        g.action[e] = (uint8_t)cell;
    }
    __syncthreads();   // the keys are free again
}

__device__ void evaluator_loop(const LoopArgs &g, EvalLds &L, int tree, int helper, int wave, int lane) {
    EvalRequests &rq = g.requests[tree];
    if (threadIdx.x == 0) __hip_atomic_store(&rq.xcc[1 + helper], my_xcc(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int step = 0;; ++step) {
        if (threadIdx.x == 0) {
            const uint64_t start = wall_clock64();
            int tag;
            while ((tag = poll_word(&rq.tag)) >= 0 && tag <= step) {
                if (poll_word(&rq.abort) != 0 || wall_clock64() - start > kWaitTicks) {
                    __hip_atomic_store(&rq.abort, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    tag = -1;
                    break;
                }
                __builtin_amdgcn_s_sleep(2);
            }
            L.tag = tag;
        }
        __syncthreads();
        const int tag = L.tag;
        __syncthreads();
        if (tag < 0) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        const int n = rq.n;
        int worked_off = 0;
        for (int first = 2 * helper; first < n; first += 2 * g.evaluators) {
            evaluate_pair(g, L, tree, first, n, wave, lane);
            worked_off += n - first >= 2 ? 2 : 1;
        }
        // every wavefront's stores have reached the L2 before one of them reports; the release pushes them on
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (threadIdx.x == 0 && worked_off > 0) {
            // The tree's workgroup wrote its XCD down before it handed out its first step.  On the same XCD the priors
            // are where it reads them, in the L2 that both share; anywhere else the L2 must be written back first.
            if (g.agent_fences || poll_word(&rq.xcc[0]) != my_xcc()) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
            __hip_atomic_fetch_add(&rq.done, worked_off, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// Until the evaluators have worked off everything handed to them so far; gives up after a bounded wait.
__device__ void wait_for_evaluators(EvalRequests &rq, StepLds &s) {
    const uint64_t start = wall_clock64();
    while (poll_word(&rq.done) < s.requested) {
        if (poll_word(&rq.abort) != 0 || wall_clock64() - start > kWaitTicks) {
            __hip_atomic_store(&rq.abort, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s.gave_up = 1;
            break;
        }
        __builtin_amdgcn_s_sleep(1);
    }
}

// The whole search in one launch.  evaluators == 0: one workgroup per tree (grid = trees).  Otherwise every tree has
// 1 + evaluators workgroups; those of one tree have the same blockIdx.x % 8, which is how workgroups are dealt to the
// eight XCDs, so a tree's requests and results meet in one L2.
__global__ __launch_bounds__(kTrav *kWave) void search_kernel(const LoopArgs g, int trees) {
    __shared__ StepLds s;
    __shared__ EvalLds eval_lds;
    int *paths = dynamic_lds;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), n_waves = g.traversals;
    int tree = blockIdx.x, role = 0;
    if (g.evaluators > 0) {
        const int per_tree = 1 + g.evaluators, nth = blockIdx.x / 8;
        tree = (int)(blockIdx.x % 8) + 8 * (nth / per_tree);
        role = nth % per_tree;
    }
    if (tree >= trees) return;
    if (role > 0) {
        if (wave >= 8) return;   // an evaluator workgroup works with eight wavefronts
        evaluator_loop(g, eval_lds, tree, role - 1, wave, lane);
        return;
    }
    if (wave >= n_waves) return;   // the launch's workgroups are as large as the larger of the two kinds needs
    const bool farm = g.evaluators > 0;
    EvalRequests &rq = g.requests[tree];
    Work work;
    if (threadIdx.x == 0) {
        s.node_count = g.node_count[tree];
        s.requested = 0;
        s.gave_up = 0;
        if (farm) __hip_atomic_store(&rq.xcc[0], my_xcc(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    bool same_l2 = false;   // known: every evaluator of the tree runs on this workgroup's XCD
    uint64_t t0 = wave == 0 ? wall_clock64() : 0;
    for (int step = 0; step < g.steps; ++step) {
        select_phase(g, s, paths, tree, wave, lane, n_waves, work.nodes_read, work.edges_scored);
        work.count_kind(s, wave);
        uint64_t t1 = 0, t2 = 0;
        if (wave == 0) t1 = wall_clock64();
        if (farm) {
            // A node created in the step before can be expanded now at the earliest (selection hands out tickets without
            // looking at a node's priors), so this is where its priors must be there, not a step's length earlier.
            if (threadIdx.x == 0) wait_for_evaluators(rq, s);
            expand_phase<true>(g, s, tree, wave, lane, n_waves, work.created);
        } else {
            expand_phase<false>(g, s, tree, wave, lane, n_waves, work.created);
        }
        phase_barrier();   // the claims of the selection and the new nodes are in memory
        if (s.gave_up) break;
        if (farm && threadIdx.x == 0) {   // ... and the evaluators may start on this step's nodes
            rq.n = s.requests;
            s.requested += s.requests;
            if (!same_l2 && !g.agent_fences) {
                same_l2 = true;
                for (int h = 1; h <= g.evaluators; ++h) same_l2 = same_l2 && poll_word(&rq.xcc[h]) == my_xcc();
            }
            // The phase barrier above has the step's nodes and requests in the L2.  Evaluators on the same XCD read them
            // there (their acquire drops what their L1 holds); for any other, or one not heard of yet, the L2 is written
            // back first, which is the expensive part of an agent-scope release.
            if (same_l2) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // rq.n
            else __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
            __hip_atomic_store(&rq.tag, step + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (wave == 0) t2 = wall_clock64();
        backup_phase(g, s, paths, tree, wave, lane, n_waves);
        phase_barrier();
        if (wave == 0) {
            const uint64_t t3 = wall_clock64();
            work.ticks[0] += t1 - t0;
            work.ticks[1] += t2 - t1;
            work.ticks[2] += t3 - t2;
            t0 = t3;
        }
    }
    if (farm) {   // the last step's nodes
        if (threadIdx.x == 0) wait_for_evaluators(rq, s);
        __syncthreads();
    }
    if (farm && threadIdx.x == 0) __hip_atomic_store(&rq.tag, -1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    state_to_memory(g, s, paths, tree, n_waves);
    work.to_memory(g, tree, lane);
}

__global__ __launch_bounds__(kTrav *kWave) void select_step_kernel(const LoopArgs g) {
    __shared__ StepLds s;
    int *paths = dynamic_lds;
    const int tree = blockIdx.x, lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), n_waves = blockDim.x / kWave;
    Work work;
    if (threadIdx.x == 0) s.node_count = g.node_count[tree];
    select_phase(g, s, paths, tree, wave, lane, n_waves, work.nodes_read, work.edges_scored);
    work.count_kind(s, wave);
    state_to_memory(g, s, paths, tree, n_waves);
    work.to_memory(g, tree, lane);
}
__global__ __launch_bounds__(kTrav *kWave) void expand_step_kernel(const LoopArgs g) {
    __shared__ StepLds s;
    int *paths = dynamic_lds;
    const int tree = blockIdx.x, lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), n_waves = blockDim.x / kWave;
    Work work;
    state_from_memory(g, s, paths, tree, n_waves);
    expand_phase<false>(g, s, tree, wave, lane, n_waves, work.created);
    __syncthreads();
    state_to_memory(g, s, paths, tree, n_waves);
    work.to_memory(g, tree, lane);
}
__global__ __launch_bounds__(kTrav *kWave) void backup_step_kernel(const LoopArgs g) {
    __shared__ StepLds s;
    int *paths = dynamic_lds;
    const int tree = blockIdx.x, lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), n_waves = blockDim.x / kWave;
    state_from_memory(g, s, paths, tree, n_waves);
    backup_phase(g, s, paths, tree, wave, lane, n_waves);
}

// ---- the arrays as the host reads them -------------------------------------------------------------------------------
// One element of array `id` (include/puct_gomoku.h) per thread, written in the [trees, nodes, edges] / [trees, nodes]
// shapes of the selection and backup launchers' arrays.
__global__ void unpack_kernel(const LoopArgs g, int trees, int id, void *dst, size_t count) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    switch (id) {
    case PUCT_GOMOKU_ARR_EDGE_CHILD: {
        const int child = (int)(g.edges[i].link >> 8);
        static_cast<int *>(dst)[i] = child > 0 ? child : -1;
        break;
    }
    case PUCT_GOMOKU_ARR_EDGE_PRIOR: static_cast<float *>(dst)[i] = g.edges[i].prior; break;
    case PUCT_GOMOKU_ARR_EDGE_W: static_cast<float *>(dst)[i] = g.edges[i].w; break;
    case PUCT_GOMOKU_ARR_EDGE_N: static_cast<int *>(dst)[i] = g.edges[i].n; break;
    case PUCT_GOMOKU_ARR_EDGE_INFLIGHT: static_cast<int *>(dst)[i] = (int)(g.edges[i].link & 0xFFu); break;
    case PUCT_GOMOKU_ARR_NODE_EXPANDED: static_cast<int *>(dst)[i] = g.info[i].expanded; break;
    case PUCT_GOMOKU_ARR_NODE_EXPAND_INFLIGHT: static_cast<int *>(dst)[i] = g.info[i].tickets; break;
    case PUCT_GOMOKU_ARR_NODE_TURN: static_cast<int8_t *>(dst)[i] = (g.info[i].legal_turn & kTurnBit) ? -1 : 1; break;
    case PUCT_GOMOKU_ARR_NODE_VALUE: static_cast<float *>(dst)[i] = g.info[i].value; break;
    case PUCT_GOMOKU_ARR_NODE_LEGAL: static_cast<int *>(dst)[i] = g.info[i].legal_turn & 0xFFFF; break;
    case PUCT_GOMOKU_ARR_PATH_VALUES: {
        const size_t out = i / g.path_depth;
        const int d = (int)(i - out * g.path_depth), edges_on_path = g.out_len[out] - 1;
        const float u = g.out_value[out];
        static_cast<float *>(dst)[i] = d < edges_on_path ? (((edges_on_path - d) & 1) ? -u : u) : 0.0f;
        break;
    }
    default: break;
    }
}

// ---- host engine -----------------------------------------------------------------------------------------------------
thread_local std::string g_error;

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}

#define HIP_TRY(expr)                                                                                       \
    do {                                                                                                    \
        hipError_t err_ = (expr);                                                                           \
        if (err_ != hipSuccess) return fail(PUCT_GOMOKU_E_HIP, "%s failed: %s", #expr, hipGetErrorString(err_)); \
    } while (0)

double now_s() { return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count(); }

}  // namespace

struct puct_gomoku_engine {
    puct_gomoku_config cfg;
    LoopArgs args;
    uint32_t *d_root = nullptr;
    std::vector<void *> allocations;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
};

namespace {
template <typename T>
int alloc(puct_gomoku_engine *e, T **out, size_t count) {
    void *p = nullptr;
    HIP_TRY(hipMalloc(&p, sizeof(T) * count));
    e->allocations.push_back(p);
    *out = static_cast<T *>(p);
    return PUCT_GOMOKU_OK;
}

// Element size and count of array `id`, 0 if there is no such array.
size_t array_shape(const puct_gomoku_config &c, int id, size_t *count) {
    const size_t T = c.trees, N = c.max_nodes, W = c.traversals, D = c.path_depth;
    switch (id) {
    case PUCT_GOMOKU_ARR_EDGE_CHILD: case PUCT_GOMOKU_ARR_EDGE_PRIOR: case PUCT_GOMOKU_ARR_EDGE_W:
    case PUCT_GOMOKU_ARR_EDGE_N: case PUCT_GOMOKU_ARR_EDGE_INFLIGHT: *count = T * N * kEdges; return 4;
    case PUCT_GOMOKU_ARR_EDGE_ACTION: *count = T * N * kEdges; return 1;
    case PUCT_GOMOKU_ARR_NODE_EXPANDED: case PUCT_GOMOKU_ARR_NODE_EXPAND_INFLIGHT: case PUCT_GOMOKU_ARR_NODE_VALUE:
    case PUCT_GOMOKU_ARR_NODE_LEGAL: *count = T * N; return 4;
    case PUCT_GOMOKU_ARR_NODE_TURN: *count = T * N; return 1;
    case PUCT_GOMOKU_ARR_NODE_COUNT: *count = T; return 4;
    case PUCT_GOMOKU_ARR_NODE_BOARD: *count = T * N * kBoardWords; return 4;
    case PUCT_GOMOKU_ARR_OUT_SELECTED: case PUCT_GOMOKU_ARR_OUT_LEN: *count = T * W; return 4;
    case PUCT_GOMOKU_ARR_OUT_PATH: case PUCT_GOMOKU_ARR_PATH_VALUES: *count = T * W * D; return 4;
    default: *count = 0; return 0;
    }
}
}  // namespace

extern "C" const char *puct_gomoku_last_error(void) { return g_error.c_str(); }

extern "C" void puct_gomoku_destroy(puct_gomoku_engine *e) {
    if (!e) return;
    (void)hipSetDevice(e->cfg.device);
    for (void *p : e->allocations) (void)hipFree(p);
    if (e->ev0) (void)hipEventDestroy(e->ev0);
    if (e->ev1) (void)hipEventDestroy(e->ev1);
    if (e->stream) (void)hipStreamDestroy(e->stream);
    delete e;
}

extern "C" int puct_gomoku_create(const puct_gomoku_config *c, puct_gomoku_engine **out) {
    if (!c || !out) return fail(PUCT_GOMOKU_E_INVALID, "null argument");
    if (c->board_m < 5 && c->board_n < 5) return fail(PUCT_GOMOKU_E_INVALID, "board %dx%d cannot hold five in a row", c->board_m, c->board_n);
    if (c->board_m < 1 || c->board_n < 1 || c->board_m * c->board_n > kEdges)
        return fail(PUCT_GOMOKU_E_INVALID, "board %dx%d: need 1 <= m * n <= %d", c->board_m, c->board_n, kEdges);
    if (c->trees < 1) return fail(PUCT_GOMOKU_E_INVALID, "trees = %d, need >= 1", c->trees);
    if (c->traversals < 1 || c->traversals > kTrav)
        return fail(PUCT_GOMOKU_E_INVALID, "traversals = %d, need 1..%d", c->traversals, kTrav);
    if (c->max_nodes < 2 || c->max_nodes > PUCT_GOMOKU_MAX_NODES)
        return fail(PUCT_GOMOKU_E_INVALID, "max_nodes = %d, need 2..%d", c->max_nodes, PUCT_GOMOKU_MAX_NODES);
    if (c->path_depth < 1 || c->path_depth > PUCT_GOMOKU_MAX_PATH_DEPTH)
        return fail(PUCT_GOMOKU_E_INVALID, "path_depth = %d, need 1..%d", c->path_depth, PUCT_GOMOKU_MAX_PATH_DEPTH);
    if (!(c->dirichlet_alpha > 0.0f && c->dirichlet_alpha < 1.0f))
        return fail(PUCT_GOMOKU_E_INVALID, "dirichlet_alpha = %g, need 0 < alpha < 1", (double)c->dirichlet_alpha);
    if (!(c->cpuct >= 0.0f) || !(c->c_pw >= 0.0f)) return fail(PUCT_GOMOKU_E_INVALID, "cpuct and c_pw must not be negative");
    if (c->evaluators < 0 || c->evaluators > kMaxEvaluators)
        return fail(PUCT_GOMOKU_E_INVALID, "evaluators = %d, need 0..%d", c->evaluators, kMaxEvaluators);
    HIP_TRY(hipSetDevice(c->device));
    auto *e = new puct_gomoku_engine();
    e->cfg = *c;
    const size_t T = c->trees, N = c->max_nodes, W = c->traversals, D = c->path_depth;
    LoopArgs &g = e->args;
    int rc = 0;
    if ((rc = alloc(e, &g.edges, T * N * kEdges)) || (rc = alloc(e, &g.info, T * N)) || (rc = alloc(e, &g.board, T * N * kBoardWords)) ||
        (rc = alloc(e, &g.action, T * N * kEdges)) || (rc = alloc(e, &g.node_count, T)) || (rc = alloc(e, &g.out_selected, T * W)) ||
        (rc = alloc(e, &g.out_len, T * W)) || (rc = alloc(e, &g.out_claims, T * W)) || (rc = alloc(e, &g.out_path, T * W * D)) ||
        (rc = alloc(e, &g.out_value, T * W)) || (rc = alloc(e, &g.tally, T * kTally)) || (rc = alloc(e, &g.requests, T)) || (rc = alloc(e, &e->d_root, (size_t)kBoardWords))) {
        puct_gomoku_destroy(e);
        return rc;
    }
    g.cpuct = c->cpuct; g.c_pw = c->c_pw; g.alpha_pw = c->alpha_pw;
    g.m = c->board_m; g.n = c->board_n; g.cells = c->board_m * c->board_n; g.max_nodes = c->max_nodes;
    g.traversals = c->traversals; g.path_depth = c->path_depth; g.steps = 0;
    g.seed = c->seed; g.dirichlet_alpha = c->dirichlet_alpha; g.evaluators = c->evaluators;
    g.agent_fences = c->agent_fences != 0;
    hipError_t err = hipStreamCreate(&e->stream);
    if (err == hipSuccess) err = hipEventCreate(&e->ev0);
    if (err == hipSuccess) err = hipEventCreate(&e->ev1);
    if (err == hipSuccess) err = hipMemset(g.out_path, 0xFF, sizeof(int) * T * W * D);
    if (err != hipSuccess) {
        puct_gomoku_destroy(e);
        return fail(PUCT_GOMOKU_E_HIP, "engine set-up failed: %s", hipGetErrorString(err));
    }
    *out = e;
    return PUCT_GOMOKU_OK;
}

extern "C" int puct_gomoku_run(puct_gomoku_engine *e, const int8_t *board, int32_t turn, int32_t steps, int32_t fused,
                               puct_gomoku_result *res) {
    if (!e || !board || !res) return fail(PUCT_GOMOKU_E_INVALID, "null argument");
    if (turn != 1 && turn != -1) return fail(PUCT_GOMOKU_E_ROOT, "turn must be +1 or -1");
    if (steps < 0) return fail(PUCT_GOMOKU_E_INVALID, "steps must not be negative");
    const puct_gomoku_config &c = e->cfg;
    const int cells = c.board_m * c.board_n;
    uint32_t words[kBoardWords] = {0};
    int empty = 0;
    for (int i = 0; i < cells; ++i) {
        if (board[i] == 1) words[i >> 5] |= 1u << (i & 31);
        else if (board[i] == -1) words[8 + (i >> 5)] |= 1u << (i & 31);
        else if (board[i] == 0) ++empty;
        else return fail(PUCT_GOMOKU_E_ROOT, "cell %d holds %d, expected -1, 0 or +1", i, (int)board[i]);
    }
    if (empty == 0) return fail(PUCT_GOMOKU_E_ROOT, "the root position has no empty cell");
    const double t0 = now_s();
    HIP_TRY(hipSetDevice(c.device));
    LoopArgs g = e->args;
    g.steps = steps;
    hipStream_t s = e->stream;
    HIP_TRY(hipMemcpyAsync(e->d_root, words, sizeof words, hipMemcpyHostToDevice, s));
    hipLaunchKernelGGL(init_kernel, dim3(c.trees), dim3(kWave), 0, s, g, e->d_root, (int)turn);
    HIP_TRY(hipGetLastError());
    const dim3 grid(c.trees), block(c.traversals * kWave);
    const size_t lds = sizeof(int) * (size_t)c.traversals * c.path_depth;
    HIP_TRY(hipEventRecord(e->ev0, s));
    if (fused) {
        if (steps > 0) {
            // The tree workgroups and their evaluators wait for each other, so every workgroup of the launch must be
            // resident: as many evaluators per tree as the device takes at once, none if it comes to that.
            int waves = c.traversals, per_cu = 0;
            if (g.evaluators > 0 && waves < 8) waves = 8;
            hipDeviceProp_t prop;
            HIP_TRY(hipGetDeviceProperties(&prop, c.device));
            HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, search_kernel, waves * kWave, lds));
            const long resident = (long)per_cu * prop.multiProcessorCount, groups = 8L * ((c.trees + 7) / 8);
            while (g.evaluators > 0 && groups * (1 + g.evaluators) > resident) g.evaluators -= 1;
            if (g.evaluators == 0) waves = c.traversals;
            const dim3 all(g.evaluators > 0 ? (unsigned)(groups * (1 + g.evaluators)) : (unsigned)c.trees);
            hipLaunchKernelGGL(search_kernel, all, dim3(waves * kWave), lds, s, g, (int)c.trees);
            HIP_TRY(hipGetLastError());
        }
    } else {
        for (int i = 0; i < steps; ++i) {
            hipLaunchKernelGGL(select_step_kernel, grid, block, lds, s, g);
            hipLaunchKernelGGL(expand_step_kernel, grid, block, lds, s, g);
            hipLaunchKernelGGL(backup_step_kernel, grid, block, lds, s, g);
        }
        HIP_TRY(hipGetLastError());
    }
    HIP_TRY(hipEventRecord(e->ev1, s));
    HIP_TRY(hipStreamSynchronize(s));
    float ms = 0.0f;
    HIP_TRY(hipEventElapsedTime(&ms, e->ev0, e->ev1));
    if (fused && g.evaluators > 0 && steps > 0) {
        std::vector<EvalRequests> rq(c.trees);
        HIP_TRY(hipMemcpy(rq.data(), g.requests, sizeof(EvalRequests) * c.trees, hipMemcpyDeviceToHost));
        for (int t = 0; t < c.trees; ++t)
            if (rq[t].abort)
                return fail(PUCT_GOMOKU_E_SYNC, "tree %d: a workgroup waited for more than 3 s for its partners (are all %d workgroups of "
                            "the launch resident?); the search was abandoned", t, (int)(8 * ((c.trees + 7) / 8) * (1 + g.evaluators)));
    }

    // root tables of all trees
    const size_t T = c.trees, N = c.max_nodes;
    std::vector<Edge> root_edges(T * kEdges);
    std::vector<NodeInfo> root_info(T);
    std::vector<uint8_t> a_root(T * kEdges);
    std::vector<int> counts(T);
    std::vector<unsigned long long> tally(T * kTally);
    HIP_TRY(hipMemcpy2D(root_edges.data(), sizeof(Edge) * kEdges, g.edges, sizeof(Edge) * kEdges * N, sizeof(Edge) * kEdges, T, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy2D(root_info.data(), sizeof(NodeInfo), g.info, sizeof(NodeInfo) * N, sizeof(NodeInfo), T, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy2D(a_root.data(), kEdges, g.action, (size_t)kEdges * N, kEdges, T, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(counts.data(), g.node_count, sizeof(int) * T, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(tally.data(), g.tally, sizeof(unsigned long long) * T * kTally, hipMemcpyDeviceToHost));
    memset(res, 0, sizeof *res);
    res->steps = steps;
    for (size_t t = 0; t < T; ++t) {
        for (int sl = 0; sl < root_info[t].expanded && sl < kEdges; ++sl) {
            const int a = a_root[t * kEdges + sl];
            res->root_n[a] += root_edges[t * kEdges + sl].n;
            res->root_w[a] += (double)root_edges[t * kEdges + sl].w;
        }
        for (int k = 0; k < 5; ++k) res->selections[k] += (int64_t)tally[t * kTally + k];
        res->expansions_committed += (int64_t)tally[t * kTally + 5];
        res->nodes_read += (int64_t)tally[t * kTally + 6];
        res->edges_scored += (int64_t)tally[t * kTally + 7];
        res->time_select += 1e-8 * (double)tally[t * kTally + 8] / (double)T;
        res->time_expand += 1e-8 * (double)tally[t * kTally + 9] / (double)T;
        res->time_backup += 1e-8 * (double)tally[t * kTally + 10] / (double)T;
        res->nodes_total += counts[t];
        if (counts[t] > res->max_nodes_in_tree) res->max_nodes_in_tree = counts[t];
    }
    res->best_action = -1;
    for (int a = 0; a < cells; ++a)
        if (res->root_n[a] > res->best_n) { res->best_n = res->root_n[a]; res->best_action = a; }
    res->time_device = ms * 1e-3;
    res->time_total = now_s() - t0;
    return PUCT_GOMOKU_OK;
}

extern "C" int64_t puct_gomoku_array_bytes(puct_gomoku_engine *e, int32_t id) {
    size_t count = 0;
    const size_t elem = e ? array_shape(e->cfg, id, &count) : 0;
    if (elem == 0) return fail(PUCT_GOMOKU_E_INVALID, "unknown array id %d", id);
    return (int64_t)(elem * count);
}

extern "C" int puct_gomoku_read(puct_gomoku_engine *e, int32_t id, void *dst, size_t bytes) {
    size_t count = 0;
    const size_t elem = (e && dst) ? array_shape(e->cfg, id, &count) : 0;
    if (elem == 0) return fail(PUCT_GOMOKU_E_INVALID, "unknown array id %d", id);
    if (bytes != elem * count) return fail(PUCT_GOMOKU_E_INVALID, "array %d has %zu bytes, buffer has %zu", id, elem * count, bytes);
    HIP_TRY(hipSetDevice(e->cfg.device));
    const LoopArgs &g = e->args;
    const void *direct = nullptr;   // arrays the engine keeps in the shape the host reads
    switch (id) {
    case PUCT_GOMOKU_ARR_EDGE_ACTION: direct = g.action; break;
    case PUCT_GOMOKU_ARR_NODE_COUNT: direct = g.node_count; break;
    case PUCT_GOMOKU_ARR_NODE_BOARD: direct = g.board; break;
    case PUCT_GOMOKU_ARR_OUT_SELECTED: direct = g.out_selected; break;
    case PUCT_GOMOKU_ARR_OUT_LEN: direct = g.out_len; break;
    case PUCT_GOMOKU_ARR_OUT_PATH: direct = g.out_path; break;
    default: break;
    }
    if (direct) {
        HIP_TRY(hipMemcpy(dst, direct, bytes, hipMemcpyDeviceToHost));
        return PUCT_GOMOKU_OK;
    }
    // the others are fields of the edge and node records: gathered on the device, then copied
    void *staging = nullptr;
    HIP_TRY(hipMalloc(&staging, bytes));
    const unsigned threads = 256;
    hipLaunchKernelGGL(unpack_kernel, dim3((unsigned)((count + threads - 1) / threads)), dim3(threads), 0, e->stream, g, e->cfg.trees,
                       (int)id, staging, count);
    hipError_t err = hipGetLastError();
    if (err == hipSuccess) err = hipStreamSynchronize(e->stream);
    if (err == hipSuccess) err = hipMemcpy(dst, staging, bytes, hipMemcpyDeviceToHost);
    (void)hipFree(staging);
    if (err != hipSuccess) return fail(PUCT_GOMOKU_E_HIP, "reading array %d failed: %s", id, hipGetErrorString(err));
    return PUCT_GOMOKU_OK;
}
