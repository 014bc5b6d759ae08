// Gomoku PUCT search loop with virtual loss: the expansion / evaluation step between the selection and backup
// kernels, a kernel that runs all steps of a search in one launch (one workgroup per tree, one wavefront per
// traversal), and the host engine behind include/puct_gomoku.h.
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

struct GomokuArgs {
    SelectArgs sel;
    BackupArgs bk;
    int *node_expanded, *node_count, *node_expand_inflight, *node_legal;
    uint32_t *node_board;
    int8_t *node_turn;
    float *node_value;
    uint8_t *edge_action;
    int *edge_child;
    float *edge_prior;
    float *edge_W;
    int *edge_N;
    int *edge_inflight;
    float *path_values;
    unsigned long long *tally;   // [trees][8]: selections by kind (0..4), children created (5)
    int m, n, cells, max_nodes, steps;
    uint64_t seed;
    double dirichlet_alpha;
};

struct Lds {
    int want[kMaxWavesPerBlock];
    uint32_t board[kMaxWavesPerBlock][kBoardWords];
};

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

// Priors of a new node: one Gamma weight per legal cell, prior = weight / sum, edge slots in descending weight order
// (ties: smaller cell first), so that progressive widening opens the most promising moves first.  Initialises every
// edge field of the node's legal slots.  All 64 lanes must call it together.
__device__ void write_priors(const GomokuArgs &g, int tree, int node, const uint32_t *board, int lane, uint64_t board_hash,
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
    while (__ballot(i < kPer) != 0) {
        if (i < kPer) {
            const int c = lane + i * kWave;
            double x;
            const int ok = psyn_gamma_round(g.dirichlet_alpha, psyn_cell_key(board_hash, c), round, &x);
            if (ok || round == PSYN_GAMMA_ROUNDS - 1) {
                const uint32_t key = psyn_weight_key(x, c);
#pragma unroll
                for (int k = 0; k < kPer; ++k)
                    if (k == i) mine[k] = key;
                ++i;
                round = 0;
                while (i < kPer && !legal_cell(i)) ++i;
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
    const size_t erow = ((size_t)tree * g.sel.nodes + node) * kEdges + (size_t)kPer * lane;
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        if (mine[k] == 0u) continue;
        const size_t e = erow + k;
        g.edge_prior[e] = psyn_prior(psyn_key_weight(mine[k]), sum, n_legal);
        g.edge_action[e] = (uint8_t)(255u - (mine[k] & 0xFFu));
        g.edge_child[e] = -1;
        g.edge_N[e] = 0;
        g.edge_W[e] = 0.0f;
        g.edge_inflight[e] = 0;
    }
}

// Expansion / evaluation of one step for the traversals of one tree; all wavefronts of the workgroup call it.
// Children get consecutive node ids in traversal order; when the tree cannot take all expansions of a step none is
// committed (those traversals evaluate the node they reached instead).
__device__ void expand_phase(const GomokuArgs &g, Lds &lds, int tree, int wave, int lane, int n_waves) {
    const size_t out = (size_t)tree * g.sel.warps + wave;
    const int raw = g.sel.out_selected_node[out];
    const int kind = (raw >> PUCT_PACKED_KIND_SHIFT) & PUCT_PACKED_KIND_MASK;
    const int node = raw & PUCT_PACKED_NODE_MASK, ticket_slot = (raw >> PUCT_PACKED_SLOT_SHIFT) & PUCT_PACKED_EDGE_MASK;
    const int plen = g.sel.out_path_len[out];
    const size_t trow = (size_t)tree * g.sel.nodes;
    const uint64_t tree_seed = psyn_tree_seed(g.seed, tree);
    const bool has_node = kind == PUCT_SELECT_EXPAND || kind == PUCT_SELECT_TERMINAL || kind == PUCT_SELECT_DEPTH_LIMIT;
    uint32_t *board = lds.board[wave];
    int n_legal = 0, turn = 0;
    if (has_node) {
        const uint32_t w = lane < kBoardWords ? g.node_board[(trow + node) * kBoardWords + lane] : 0u;
        if (lane < kBoardWords) board[lane] = w;
        n_legal = g.cells - wave_sum(__popc(w));
        turn = g.node_turn[trow + node];
        wave_lds_fence();
    }
    const int wants = (kind == PUCT_SELECT_EXPAND && ticket_slot < n_legal) ? 1 : 0;
    if (lane == 0) {
        lds.want[wave] = wants;
        atomicAdd(&g.tally[(size_t)tree * 8 + kind], 1ull);
    }
    __syncthreads();
    int total = 0, before = 0;
    for (int w = 0; w < n_waves; ++w) {
        total += lds.want[w];
        before += w < wave ? lds.want[w] : 0;
    }
    const int base = load_relaxed(g.node_count + tree);
    const bool fits = base + total <= g.max_nodes;
    __syncthreads();
    if (wave == 0 && lane == 0 && fits && total > 0) {
        g.node_count[tree] = base + total;
        atomicAdd(&g.tally[(size_t)tree * 8 + 5], (unsigned long long)total);
    }

    float u = 0.0f;   // value of the reached node for its player to move
    if (wants && fits) {
        const int child = base + before;
        const size_t erow = (trow + node) * kEdges;
        // The edge slot the child goes into is the node's next free one, taken here, not the slot of the selection's
        // ticket: tickets of one step can leave a hole (a traversal whose widening limit, computed from visit counts
        // that include other traversals' virtual losses, is smaller gives its ticket back while one with a larger limit
        // has already drawn the next), and the expanded edges of a node must stay contiguous.  With one traversal per
        // tree the two are the same slot.
        int slot_taken = 0;
        if (lane == 0) slot_taken = atomicAdd(&g.node_expanded[trow + node], 1);
        const int slot = __builtin_amdgcn_readfirstlane(slot_taken);
        const int action = g.edge_action[erow + slot];
        uint32_t *mine = board + (turn > 0 ? 0 : 8);
        if (lane == 0) mine[action >> 5] |= 1u << (action & 31);
        wave_lds_fence();
        const bool win = makes_five(mine, action, g.m, g.n, lane);
        const int child_legal = n_legal - 1;
        const bool terminal = win || child_legal == 0;
        const uint64_t bh = psyn_board_hash(tree_seed, board);
        const float v_child = win ? -1.0f : (terminal ? 0.0f : psyn_value(bh));
        if (lane < kBoardWords) g.node_board[(trow + child) * kBoardWords + lane] = board[lane];
        if (lane == 0) {
            g.node_turn[trow + child] = (int8_t)-turn;
            g.node_value[trow + child] = v_child;
            g.node_expanded[trow + child] = terminal ? PUCT_NODE_EXPANDED_TERMINAL : 0;
            g.node_expand_inflight[trow + child] = 0;
            g.node_legal[trow + child] = child_legal;
            g.edge_child[erow + slot] = child;
            g.edge_N[erow + slot] = 1;
            g.edge_W[erow + slot] = -v_child;
        }
        if (!terminal) write_priors(g, tree, child, board, lane, bh, child_legal);
        u = -v_child;
    } else if (kind == PUCT_SELECT_TERMINAL) {
        u = g.node_value[trow + node];
    } else if (has_node) {
        u = psyn_value(psyn_board_hash(tree_seed, board));
    }
    if (has_node) {
        // edge d was played by the player to move at depth d; the reached node sits at depth L
        const int L = plen - 1;
        for (int d = lane; d < L; d += kWave) g.path_values[out * g.sel.path_depth + d] = ((L - d) & 1) ? -u : u;
    }
}

// Root of every tree: node 0 with the root position and its priors.
__global__ __launch_bounds__(kWave) void init_kernel(const GomokuArgs g, const uint32_t *root_board, int root_turn) {
    __shared__ uint32_t board[kBoardWords];
    const int tree = blockIdx.x, lane = threadIdx.x;
    const size_t trow = (size_t)tree * g.sel.nodes;
    const uint32_t w = lane < kBoardWords ? root_board[lane] : 0u;
    if (lane < kBoardWords) {
        board[lane] = w;
        g.node_board[trow * kBoardWords + lane] = w;
    }
    const int n_legal = g.cells - wave_sum(__popc(w));
    wave_lds_fence();
    if (lane < 8) g.tally[(size_t)tree * 8 + lane] = 0ull;
    if (lane == 0) {
        g.node_turn[trow] = (int8_t)root_turn;
        g.node_value[trow] = 0.0f;
        g.node_expanded[trow] = n_legal == 0 ? PUCT_NODE_EXPANDED_TERMINAL : 0;
        g.node_expand_inflight[trow] = 0;
        g.node_legal[trow] = n_legal;
        g.node_count[tree] = 1;
    }
    if (n_legal > 0) write_priors(g, tree, 0, board, lane, psyn_board_hash(psyn_tree_seed(g.seed, tree), board), n_legal);
}

// Makes the writes of a phase (plain stores and atomics) visible to the loads of the next one.  All wavefronts of a
// tree run on one CU and share its write-through L1 and the L2 behind it, so no L2 write-back is needed; what is needed
// is (1) that every wavefront's stores and atomics of the phase have been acknowledged by the L2 before any wavefront
// goes on -- a workgroup-scope release fence does not wait for that on one CU (it lowers to no vector-memory wait), and a
// counter that another wavefront changed with a fire-and-forget atomic could otherwise still be read with its old value
// after the barrier -- hence the explicit wait on the wavefront's own outstanding vector memory operations; and (2) that
// the L1 drops the lines which device-scope atomics of other wavefronts have changed underneath it: the agent-scope
// acquire.
__device__ __forceinline__ void phase_barrier() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

__global__ __launch_bounds__(kMaxWavesPerBlock *kWave) void search_kernel(const GomokuArgs g) {
    __shared__ Lds lds;
    const int tree = blockIdx.x, wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
    const int n_waves = blockDim.x / kWave;
    for (int step = 0; step < g.steps; ++step) {
        select_traversal(g.sel, tree, wave, lane);
        phase_barrier();
        expand_phase(g, lds, tree, wave, lane, n_waves);
        phase_barrier();
        backup_traversal<false>(g.bk, tree, wave, lane);
        phase_barrier();
    }
}

__global__ __launch_bounds__(kMaxWavesPerBlock *kWave) void select_step_kernel(const GomokuArgs g) {
    select_traversal(g.sel, blockIdx.x, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
}
__global__ __launch_bounds__(kMaxWavesPerBlock *kWave) void expand_step_kernel(const GomokuArgs g) {
    __shared__ Lds lds;
    expand_phase(g, lds, blockIdx.x, threadIdx.x / kWave, threadIdx.x & (kWave - 1), blockDim.x / kWave);
}
__global__ __launch_bounds__(kMaxWavesPerBlock *kWave) void backup_step_kernel(const GomokuArgs g) {
    backup_traversal<false>(g.bk, blockIdx.x, threadIdx.x / kWave, threadIdx.x & (kWave - 1));
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
    GomokuArgs args;
    uint32_t *d_root = nullptr;
    std::vector<void *> allocations;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    struct Array { void *ptr; size_t bytes; };
    Array arrays[17];
};

namespace {
template <typename T>
int alloc(puct_gomoku_engine *e, T **out, size_t count, int array_id) {
    void *p = nullptr;
    HIP_TRY(hipMalloc(&p, sizeof(T) * count));
    e->allocations.push_back(p);
    *out = static_cast<T *>(p);
    if (array_id >= 0) e->arrays[array_id] = {p, sizeof(T) * count};
    return PUCT_GOMOKU_OK;
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
    if (c->traversals < 1 || c->traversals > kMaxWavesPerBlock)
        return fail(PUCT_GOMOKU_E_INVALID, "traversals = %d, need 1..%d", c->traversals, kMaxWavesPerBlock);
    if (c->max_nodes < 2 || c->max_nodes > PUCT_PACKED_NODE_LIMIT)
        return fail(PUCT_GOMOKU_E_INVALID, "max_nodes = %d, need 2..%d", c->max_nodes, PUCT_PACKED_NODE_LIMIT);
    if (c->path_depth < 1 || c->path_depth > 1024) return fail(PUCT_GOMOKU_E_INVALID, "path_depth = %d, need 1..1024", c->path_depth);
    if (!(c->dirichlet_alpha > 0.0f && c->dirichlet_alpha < 1.0f))
        return fail(PUCT_GOMOKU_E_INVALID, "dirichlet_alpha = %g, need 0 < alpha < 1", (double)c->dirichlet_alpha);
    if (c->recalc_attempts < 0 || c->recalc_attempts > 64) return fail(PUCT_GOMOKU_E_INVALID, "recalc_attempts = %d, need 0..64", c->recalc_attempts);
    if (!(c->cpuct >= 0.0f) || !(c->c_pw >= 0.0f)) return fail(PUCT_GOMOKU_E_INVALID, "cpuct and c_pw must not be negative");
    HIP_TRY(hipSetDevice(c->device));
    auto *e = new puct_gomoku_engine();
    e->cfg = *c;
    memset(e->arrays, 0, sizeof e->arrays);
    const size_t T = c->trees, N = c->max_nodes, E = kEdges, W = c->traversals, D = c->path_depth;
    GomokuArgs &g = e->args;
    int *out_selected, *out_path, *out_len;
    int rc = 0;
    if ((rc = alloc(e, &g.edge_child, T * N * E, PUCT_GOMOKU_ARR_EDGE_CHILD)) || (rc = alloc(e, &g.edge_prior, T * N * E, PUCT_GOMOKU_ARR_EDGE_PRIOR)) ||
        (rc = alloc(e, &g.edge_W, T * N * E, PUCT_GOMOKU_ARR_EDGE_W)) || (rc = alloc(e, &g.edge_N, T * N * E, PUCT_GOMOKU_ARR_EDGE_N)) ||
        (rc = alloc(e, &g.edge_inflight, T * N * E, PUCT_GOMOKU_ARR_EDGE_INFLIGHT)) ||
        (rc = alloc(e, &g.edge_action, T * N * E, PUCT_GOMOKU_ARR_EDGE_ACTION)) ||
        (rc = alloc(e, &g.node_expanded, T * N, PUCT_GOMOKU_ARR_NODE_EXPANDED)) ||
        (rc = alloc(e, &g.node_expand_inflight, T * N, PUCT_GOMOKU_ARR_NODE_EXPAND_INFLIGHT)) ||
        (rc = alloc(e, &g.node_count, T, PUCT_GOMOKU_ARR_NODE_COUNT)) || (rc = alloc(e, &g.node_board, T * N * kBoardWords, PUCT_GOMOKU_ARR_NODE_BOARD)) ||
        (rc = alloc(e, &g.node_turn, T * N, PUCT_GOMOKU_ARR_NODE_TURN)) || (rc = alloc(e, &g.node_value, T * N, PUCT_GOMOKU_ARR_NODE_VALUE)) ||
        (rc = alloc(e, &out_selected, T * W, PUCT_GOMOKU_ARR_OUT_SELECTED)) || (rc = alloc(e, &out_path, T * W * D, PUCT_GOMOKU_ARR_OUT_PATH)) ||
        (rc = alloc(e, &out_len, T * W, PUCT_GOMOKU_ARR_OUT_LEN)) || (rc = alloc(e, &g.path_values, T * W * D, PUCT_GOMOKU_ARR_PATH_VALUES)) ||
        (rc = alloc(e, &g.node_legal, T * N, PUCT_GOMOKU_ARR_NODE_LEGAL)) || (rc = alloc(e, &g.tally, T * 8, -1)) || (rc = alloc(e, &e->d_root, (size_t)kBoardWords, -1))) {
        puct_gomoku_destroy(e);
        return rc;
    }
    g.sel = SelectArgs{c->cpuct, c->c_pw, c->alpha_pw, c->soft_winner, g.edge_child, g.edge_prior, g.edge_W, g.edge_N, g.edge_inflight,
                       g.node_expand_inflight, g.node_expanded, g.node_count, out_selected, out_path, out_len,
                       c->trees, c->max_nodes, kEdges, c->traversals, c->path_depth, g.node_legal,
                       c->recalc_attempts > 0 ? c->recalc_attempts : kRecalcAttempts, g.tally};
    g.bk = BackupArgs{1, nullptr, g.edge_W, g.edge_N, g.edge_inflight, nullptr, g.node_expand_inflight, g.node_count,
                      out_selected, out_path, out_len, g.path_values, c->trees, c->max_nodes, kEdges, c->traversals, c->path_depth};
    g.m = c->board_m; g.n = c->board_n; g.cells = c->board_m * c->board_n; g.max_nodes = c->max_nodes; g.steps = 0;
    g.seed = c->seed; g.dirichlet_alpha = (double)c->dirichlet_alpha;
    hipError_t err = hipStreamCreate(&e->stream);
    if (err == hipSuccess) err = hipEventCreate(&e->ev0);
    if (err == hipSuccess) err = hipEventCreate(&e->ev1);
    // the paths and values of slots a step does not write must still be readable
    if (err == hipSuccess) err = hipMemset(out_path, 0xFF, sizeof(int) * T * W * D);
    if (err == hipSuccess) err = hipMemset(g.path_values, 0, sizeof(float) * T * W * D);
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
    GomokuArgs g = e->args;
    g.steps = steps;
    hipStream_t s = e->stream;
    HIP_TRY(hipMemcpyAsync(e->d_root, words, sizeof words, hipMemcpyHostToDevice, s));
    hipLaunchKernelGGL(init_kernel, dim3(c.trees), dim3(kWave), 0, s, g, e->d_root, (int)turn);
    HIP_TRY(hipGetLastError());
    const dim3 grid(c.trees), block(c.traversals * kWave);
    HIP_TRY(hipEventRecord(e->ev0, s));
    if (fused) {
        if (steps > 0) {
            hipLaunchKernelGGL(search_kernel, grid, block, 0, s, g);
            HIP_TRY(hipGetLastError());
        }
    } else {
        for (int i = 0; i < steps; ++i) {
            hipLaunchKernelGGL(select_step_kernel, grid, block, 0, s, g);
            hipLaunchKernelGGL(expand_step_kernel, grid, block, 0, s, g);
            hipLaunchKernelGGL(backup_step_kernel, grid, block, 0, s, g);
        }
        HIP_TRY(hipGetLastError());
    }
    HIP_TRY(hipEventRecord(e->ev1, s));
    HIP_TRY(hipStreamSynchronize(s));
    float ms = 0.0f;
    HIP_TRY(hipEventElapsedTime(&ms, e->ev0, e->ev1));

    // root tables of all trees
    const size_t T = c.trees, N = c.max_nodes;
    std::vector<int> n_root(T * kEdges), expanded(T), counts(T);
    std::vector<float> w_root(T * kEdges);
    std::vector<uint8_t> a_root(T * kEdges);
    std::vector<unsigned long long> tally(T * 8);
    for (size_t t = 0; t < T; ++t) {
        HIP_TRY(hipMemcpy(n_root.data() + t * kEdges, g.edge_N + t * N * kEdges, sizeof(int) * kEdges, hipMemcpyDeviceToHost));
        HIP_TRY(hipMemcpy(w_root.data() + t * kEdges, g.edge_W + t * N * kEdges, sizeof(float) * kEdges, hipMemcpyDeviceToHost));
        HIP_TRY(hipMemcpy(a_root.data() + t * kEdges, g.edge_action + t * N * kEdges, kEdges, hipMemcpyDeviceToHost));
        HIP_TRY(hipMemcpy(&expanded[t], g.node_expanded + t * N, sizeof(int), hipMemcpyDeviceToHost));
    }
    HIP_TRY(hipMemcpy(counts.data(), g.node_count, sizeof(int) * T, hipMemcpyDeviceToHost));
    HIP_TRY(hipMemcpy(tally.data(), g.tally, sizeof(unsigned long long) * T * 8, hipMemcpyDeviceToHost));
    memset(res, 0, sizeof *res);
    res->steps = steps;
    for (size_t t = 0; t < T; ++t) {
        for (int sl = 0; sl < expanded[t] && sl < kEdges; ++sl) {
            const int a = a_root[t * kEdges + sl];
            res->root_n[a] += n_root[t * kEdges + sl];
            res->root_w[a] += (double)w_root[t * kEdges + sl];
        }
        for (int k = 0; k < 5; ++k) res->selections[k] += (int64_t)tally[t * 8 + k];
        res->expansions_committed += (int64_t)tally[t * 8 + 5];
        res->levels_read += (int64_t)tally[t * 8 + 6];
        res->edges_examined += (int64_t)tally[t * 8 + 7];
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
    if (!e || id < 0 || id > PUCT_GOMOKU_ARR_NODE_LEGAL || !e->arrays[id].ptr) return fail(PUCT_GOMOKU_E_INVALID, "unknown array id %d", id);
    return (int64_t)e->arrays[id].bytes;
}

extern "C" int puct_gomoku_read(puct_gomoku_engine *e, int32_t id, void *dst, size_t bytes) {
    if (!e || !dst || id < 0 || id > PUCT_GOMOKU_ARR_NODE_LEGAL || !e->arrays[id].ptr) return fail(PUCT_GOMOKU_E_INVALID, "unknown array id %d", id);
    if (bytes != e->arrays[id].bytes) return fail(PUCT_GOMOKU_E_INVALID, "array %d has %zu bytes, buffer has %zu", id, e->arrays[id].bytes, bytes);
    HIP_TRY(hipSetDevice(e->cfg.device));
    HIP_TRY(hipMemcpy(dst, e->arrays[id].ptr, bytes, hipMemcpyDeviceToHost));
    return PUCT_GOMOKU_OK;
}
