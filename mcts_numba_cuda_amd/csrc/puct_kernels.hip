// Kernels and C ABI of PUCT selection and backup with virtual loss (device code: puct_device.hpp).
#include "puct_device.hpp"

namespace {
using namespace puct;

// LOCAL: the tree's traversals are this workgroup's wavefronts (grid.y == 1) and the claims on its edges are kept in
// the workgroup's dynamic LDS for the launch (a.nodes * a.edges words).
template <bool LOCAL>
__global__ __launch_bounds__(kMaxWavesPerBlock *kWave) __attribute__((amdgpu_waves_per_eu(8, 8))) void select_kernel(const SelectArgs a) {
    extern __shared__ int tree_claims[];
    const int wid = __builtin_amdgcn_readfirstlane(blockIdx.y * (blockDim.x / kWave) + threadIdx.x / kWave);   // the same in all lanes
    const int words = a.nodes * a.edges;
    int *const in_memory = a.edge_inflight + (size_t)blockIdx.x * a.nodes * a.edges;
    const EdgeClaims<LOCAL> claims{in_memory, (LdsInts)tree_claims};
    if (LOCAL) {
        for (int i = threadIdx.x; i < words; i += blockDim.x) tree_claims[i] = in_memory[i];
        __syncthreads();
    }
    if (LOCAL || wid < a.warps) select_traversal<LOCAL>(a, claims, blockIdx.x, wid, threadIdx.x & (kWave - 1));
    if (LOCAL) {
        __syncthreads();
        for (int i = threadIdx.x; i < words; i += blockDim.x) in_memory[i] = tree_claims[i];
    }
}

// LOCAL: the tree's traversals are this workgroup's wavefronts (grid.y == 1) and its virtual-visit counters are kept
// in the workgroup's dynamic LDS for the launch (a.nodes words).
template <bool PRECLAIM, bool LOCAL>
__global__ __launch_bounds__(kMaxWavesPerBlock *kWave) __attribute__((amdgpu_waves_per_eu(8, 8))) void node_select_kernel(const NodeSelectArgs a) {
    extern __shared__ int tree_visits[];
    const int wid = __builtin_amdgcn_readfirstlane(blockIdx.y * (blockDim.x / kWave) + threadIdx.x / kWave);   // the same in all lanes
    int *const in_memory = a.node_inflight + (size_t)blockIdx.x * a.nodes;
    const NodeVisits<LOCAL> visits_of{in_memory, (LdsInts)tree_visits};
    if (LOCAL) {
        for (int i = threadIdx.x; i < a.nodes; i += blockDim.x) tree_visits[i] = in_memory[i];
        __syncthreads();
    }
    if (LOCAL || wid < a.warps) node_select_traversal<PRECLAIM, LOCAL>(a, visits_of, blockIdx.x, wid, threadIdx.x & (kWave - 1));
    if (LOCAL) {
        __syncthreads();
        for (int i = threadIdx.x; i < a.nodes; i += blockDim.x) in_memory[i] = tree_visits[i];
    }
}

template <bool NODE_LEVEL>
__global__ __launch_bounds__(kMaxWavesPerBlock *kWave) void backup_kernel(const BackupArgs a) {
    const int wid = blockIdx.y * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (wid >= a.warps) return;
    backup_traversal<NODE_LEVEL>(a, blockIdx.x, wid, threadIdx.x & (kWave - 1));
}

constexpr int kLocalVisitNodes = 16384;   // (what a selection word can name; 64 KB of LDS, two workgroups per CU: still ahead of counters in memory)
constexpr int kLocalClaimSlots = 8192;

// One wavefront per traversal; a tree with more than 16 traversals is spread over several workgroups.
inline void launch_shape(int trees, int warps, dim3 &grid, dim3 &block) {
    const int per_block = warps < kMaxWavesPerBlock ? warps : kMaxWavesPerBlock;
    block = dim3(per_block > 0 ? per_block * kWave : 0);
    grid = dim3(trees > 0 ? trees : 0, per_block > 0 ? (warps + per_block - 1) / per_block : 0);
}

}  // namespace

extern "C" int puct_select_winner_recalc_launch(float cpuct, float c_pw, float alpha_pw, int soft_winner,
                                                const int *edge_child_id, const float *edge_prior, const float *edge_W,
                                                const int *edge_N, int *edge_inflight, int *node_expand_inflight,
                                                const int *node_expanded, const int *tree_nodes,
                                                int *out_selected_node, int *out_path_eids, int *out_path_len, int trees,
                                                int nodes, int edges, int warps, int path_depth, void *stream) {
    SelectArgs a{cpuct,        c_pw,          alpha_pw,        soft_winner,          edge_child_id,
                 edge_prior,   edge_W,        edge_N,          edge_inflight,        node_expand_inflight,
                 node_expanded, tree_nodes,   out_selected_node, out_path_eids,      out_path_len,
                 trees,        nodes,         edges,           warps,                path_depth};
    dim3 grid, block;
    launch_shape(trees, warps, grid, block);
    // (the claims of a tree in LDS: up to 8192 edge slots, so that a CU still holds four workgroups)
    const long long slots = (long long)nodes * edges;
    if (grid.y == 1 && slots > 0 && slots <= kLocalClaimSlots)
        hipLaunchKernelGGL(select_kernel<true>, grid, block, sizeof(int) * (size_t)slots, reinterpret_cast<hipStream_t>(stream), a);
    else
        hipLaunchKernelGGL(select_kernel<false>, grid, block, 0, reinterpret_cast<hipStream_t>(stream), a);
    return static_cast<int>(hipGetLastError());
}

namespace {
template <bool PRECLAIM>
int launch_node_select(float cpuct, float c_pw, float alpha_pw, const int *edge_child_id, const float *edge_prior,
                       const float *edge_W, const int *edge_N, int *node_inflight, int *node_expand_inflight,
                       const int *node_expanded, const int *node_count, int *out_selected_node, int *out_path_eids,
                       int *out_path_len, int trees, int nodes, int edges, int warps, int path_depth, void *stream) {
    NodeSelectArgs a{cpuct,         c_pw,         alpha_pw,          edge_child_id, edge_prior,   edge_W, edge_N,
                     node_inflight, node_expand_inflight, node_expanded, node_count,    out_selected_node,
                     out_path_eids, out_path_len, trees,             nodes,         edges,        warps,  path_depth};
    dim3 grid, block;
    launch_shape(trees, warps, grid, block);
    // (the counters of a tree in LDS: up to 16384 nodes)
    if (grid.y == 1 && nodes > 0 && nodes <= kLocalVisitNodes)
        hipLaunchKernelGGL((node_select_kernel<PRECLAIM, true>), grid, block, sizeof(int) * (size_t)nodes, reinterpret_cast<hipStream_t>(stream), a);
    else
        hipLaunchKernelGGL((node_select_kernel<PRECLAIM, false>), grid, block, 0, reinterpret_cast<hipStream_t>(stream), a);
    return static_cast<int>(hipGetLastError());
}
}  // namespace

extern "C" int puct_node_select_preclaim_launch(float cpuct, float c_pw, float alpha_pw, const int *edge_child_id,
                                                const float *edge_prior, const float *edge_W, const int *edge_N,
                                                int *node_inflight, int *node_expand_inflight, const int *node_expanded,
                                                const int *node_count, int *out_selected_node, int *out_path_eids,
                                                int *out_path_len, int trees, int nodes, int edges, int warps,
                                                int path_depth, void *stream) {
    return launch_node_select<true>(cpuct, c_pw, alpha_pw, edge_child_id, edge_prior, edge_W, edge_N, node_inflight,
                                    node_expand_inflight, node_expanded, node_count, out_selected_node, out_path_eids,
                                    out_path_len, trees, nodes, edges, warps, path_depth, stream);
}

extern "C" int puct_node_select_winner_recalc_launch(float cpuct, float c_pw, float alpha_pw, const int *edge_child_id,
                                                     const float *edge_prior, const float *edge_W, const int *edge_N,
                                                     int *node_inflight, int *node_expand_inflight,
                                                     const int *node_expanded, const int *node_count,
                                                     int *out_selected_node, int *out_path_eids, int *out_path_len,
                                                     int trees, int nodes, int edges, int warps, int path_depth,
                                                     void *stream) {
    return launch_node_select<false>(cpuct, c_pw, alpha_pw, edge_child_id, edge_prior, edge_W, edge_N, node_inflight,
                                     node_expand_inflight, node_expanded, node_count, out_selected_node, out_path_eids,
                                     out_path_len, trees, nodes, edges, warps, path_depth, stream);
}

extern "C" const char *puct_cpp_cuda_error_string(int code) { return hipGetErrorString(static_cast<hipError_t>(code)); }

extern "C" int puct_edge_backup_launch(int virtual_loss, float *edge_W, int *edge_N, int *edge_inflight,
                                       int *node_expand_inflight, const int *node_count, const int *out_selected_node,
                                       const int *out_path_eids, const int *out_path_len, const float *path_edge_values,
                                       int trees, int nodes, int edges, int warps, int path_depth, void *stream) {
    BackupArgs a{virtual_loss, nullptr,    edge_W,           edge_N,        edge_inflight, nullptr,
                 node_expand_inflight, node_count, out_selected_node, out_path_eids, out_path_len, path_edge_values,
                 trees,        nodes,      edges,            warps,         path_depth};
    dim3 grid, block;
    launch_shape(trees, warps, grid, block);
    hipLaunchKernelGGL(backup_kernel<false>, grid, block, 0, reinterpret_cast<hipStream_t>(stream), a);
    return static_cast<int>(hipGetLastError());
}

extern "C" int puct_node_backup_launch(int virtual_loss, const int *edge_child_id, float *edge_W, int *edge_N,
                                       int *node_inflight, int *node_expand_inflight, const int *node_count,
                                       const int *out_selected_node, const int *out_path_eids, const int *out_path_len,
                                       const float *path_edge_values, int trees, int nodes, int edges, int warps,
                                       int path_depth, void *stream) {
    BackupArgs a{virtual_loss, edge_child_id, edge_W,        edge_N,        nullptr,       node_inflight,
                 node_expand_inflight, node_count, out_selected_node, out_path_eids, out_path_len, path_edge_values,
                 trees,        nodes,         edges,         warps,         path_depth};
    dim3 grid, block;
    launch_shape(trees, warps, grid, block);
    hipLaunchKernelGGL(backup_kernel<true>, grid, block, 0, reinterpret_cast<hipStream_t>(stream), a);
    return static_cast<int>(hipGetLastError());
}
