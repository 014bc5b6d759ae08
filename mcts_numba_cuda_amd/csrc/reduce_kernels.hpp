// Final reductions of a search on the device: MCTSNC._reduce_over_trees_{thrifty,prodigal} (src/mctsnc.py:2222-2296)
// and _reduce_over_actions_{thrifty,prodigal} (:2298-2375) in one kernel, one workgroup per search, whatever the game.
//
// Over trees: for every entry b of the root table (thrifty: the b-th expanded root action of tree 0's memorised
// row; prodigal: action b, counted if tree 0 expanded it) the int64 sums over all trees of the root's visits, the
// child's visits and the child's wins; the win flag is tree 0's (child terminal with the root mover's outcome,
// :2257-2258).  Over actions: the reference's strided max-argmax with the lexicographic key (win_flag, n, n_wins),
// the left slot kept on ties (:2318-2330), run as the same tournament: strides of a wavefront and more through LDS,
// smaller ones with cross-lane moves inside wavefront 0.  The per-tree bookkeeping the host reports (sizes, depth sums,
// work counters, stage clocks of tree 0) is summed here too, so one small block per search goes back to the host.
//
// A game provides `RootView` (see c4_kernels.hpp / gomoku_kernels.hpp): where the root's visit count, the memorised
// row and the counters of the root's children live in its tree layout.
#pragma once
#include "mctsnc_common.hpp"

namespace mctsnc {

constexpr int kReduceThreads = 512;   // MAX_STATE_MAX_ACTIONS of the reference (src/mctsnc.py:193): one tournament slot per thread

// What a search leaves for the host: this header, then root_ns[A], actions_ns[A], actions_ns_wins[A] (int64),
// root_actions_expanded[A + 2] (int16), actions_win_flags[A] (uint8); blocks of consecutive searches are
// reduced_stride(A) bytes apart.
struct __attribute__((aligned(256))) ReducedHeader {
    int32_t best_action, best_win_flag, n_root_entries, max_depth, max_size, pad0[3];
    int64_t best_n, best_n_wins, depth_sum, size_sum;
    unsigned long long plies, u1_events, stat_levels, stat_children, stat_expanded, stat_played;
    unsigned long long t_select, t_expand, t_playout, t_backup, t_exchange;   // of tree 0
};
static_assert(sizeof(ReducedHeader) == 256, "header of a reduced block");

__host__ __device__ inline size_t reduced_off_root_ns(int) { return sizeof(ReducedHeader); }
__host__ __device__ inline size_t reduced_off_ns(int A) { return sizeof(ReducedHeader) + (size_t)8 * A; }
__host__ __device__ inline size_t reduced_off_wins(int A) { return sizeof(ReducedHeader) + (size_t)16 * A; }
__host__ __device__ inline size_t reduced_off_rae(int A) { return sizeof(ReducedHeader) + (size_t)24 * A; }
__host__ __device__ inline size_t reduced_off_flags(int A) { return reduced_off_rae(A) + (size_t)2 * (A + 2); }
__host__ __device__ inline size_t reduced_stride(int A) { return (reduced_off_flags(A) + (size_t)A + 255) & ~(size_t)255; }

#ifdef __HIPCC__
// refs: the trees of the launch, those of search j at [j * T, (j + 1) * T) with its tree 0 first.
template <class Game>
__global__ void __launch_bounds__(kReduceThreads) reduce_kernel(const typename Game::Ref *refs, int T, int A, int thrifty, unsigned char *out) {
    using Ref = typename Game::Ref;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    refs += (size_t)blockIdx.x * T;
    unsigned char *const o = out + (size_t)blockIdx.x * reduced_stride(A);
    int A_pad = 1;
    while (A_pad < A) A_pad <<= 1;   // slots of the tournament: the next power of two (any larger padding gives the same winner)

    __shared__ int16_t s_rae[kReduceThreads + 2];
    __shared__ int32_t s_base[kReduceThreads], s_kids[kReduceThreads];   // per tree (T <= 512): first child and child set of the root
    __shared__ unsigned long long s_sum_ns[kReduceThreads], s_sum_ws[kReduceThreads];
    __shared__ unsigned long long s_tot[10];    // root visits, depth sum, size sum, plies, u1 events, four work counters
    __shared__ int32_t s_max[2];                // max depth, max size
    __shared__ uint8_t s_f[kReduceThreads];
    __shared__ int64_t s_n[kReduceThreads], s_w[kReduceThreads];
    __shared__ int16_t s_i[kReduceThreads];

    const Ref ref0 = refs[0];
    for (int i = tid; i < A + 2; i += kReduceThreads) s_rae[i] = Game::root_ae(ref0, i);
    s_sum_ns[tid] = 0; s_sum_ws[tid] = 0;
    if (tid < 10) s_tot[tid] = 0;
    if (tid == 0) { s_max[0] = -1; s_max[1] = 0; }
    __syncthreads();

    // ---- per tree: the root's child range, and the bookkeeping totals ----
    for (int t = tid; t < T; t += kReduceThreads) {
        const Ref r = refs[t];
        int32_t base, kids;
        Game::root_info(r, base, kids);
        s_base[t] = base; s_kids[t] = kids;
        const auto *h = r.hdr;
        atomicAdd(&s_tot[0], (unsigned long long)(long long)Game::root_ns(r));
        atomicAdd(&s_tot[1], (unsigned long long)h->depth_sum);
        atomicAdd(&s_tot[2], (unsigned long long)(long long)h->size);
        atomicAdd(&s_tot[3], h->plies); atomicAdd(&s_tot[4], h->u1_events);
        atomicAdd(&s_tot[5], h->stat_levels); atomicAdd(&s_tot[6], h->stat_children);
        atomicAdd(&s_tot[7], h->stat_expanded); atomicAdd(&s_tot[8], h->stat_played);
        atomicMax(&s_max[0], h->max_depth); atomicMax(&s_max[1], h->size);
    }
    __syncthreads();

    // ---- sums over trees (:2222-2296): thread = (group of trees, table entry) ----
    int nb = thrifty ? (int)s_rae[A + 1] : A;
    nb = nb < 0 ? 0 : (nb > A ? A : nb);
    const int groups = kReduceThreads / A_pad, b = tid & (A_pad - 1), grp = tid / A_pad;
    int action = -1;
    if (b < nb) {
        const int a = thrifty ? (int)s_rae[b] : b;
        if (a >= 0 && a < A && (thrifty || s_rae[a] != -1)) action = a;
    }
    const int slot = action >= 0 ? Game::action_slot(ref0, action) : -1;   // the same in every tree: they share the root position
    long long ns = 0, ws = 0;
    if (action >= 0) {
        for (int t = grp; t < T; t += groups) {
            const int32_t kids = s_kids[t];
            if (Game::has_child(kids, slot, action)) {
                int32_t cn, cw;
                Game::child_counts(refs[t], s_base[t], slot, action, cn, cw);
                ns += cn; ws += cw;
            }
        }
    }
    // the groups of a wavefront meet with cross-lane adds, the wavefronts in LDS
    for (int off = A_pad; off < 64; off <<= 1) { ns += __shfl_xor(ns, off); ws += __shfl_xor(ws, off); }
    if (A_pad >= 64 || lane < A_pad) {
        if (ns) atomicAdd(&s_sum_ns[b], (unsigned long long)ns);
        if (ws) atomicAdd(&s_sum_ws[b], (unsigned long long)ws);
    }
    __syncthreads();

    // ---- the table, and the tournament's slots ----
    uint8_t f = 0; int64_t n = 0, w = 0; int16_t idx = (int16_t)tid;
    if (tid < A) {
        const bool counted = grp == 0 && action >= 0;
        n = (int64_t)s_sum_ns[tid]; w = (int64_t)s_sum_ws[tid];
        if (counted && Game::has_child(s_kids[0], slot, action)) {   // win flag from tree 0 (:2257-2258)
            bool terminal; int outcome;
            Game::child_state(ref0, s_base[0], s_kids[0], slot, action, terminal, outcome);
            f = (terminal && outcome == ref0.hdr->root_turn) ? 1 : 0;
        }
        reinterpret_cast<int64_t *>(o + reduced_off_root_ns(A))[tid] = counted ? (int64_t)s_tot[0] : 0;
        reinterpret_cast<int64_t *>(o + reduced_off_ns(A))[tid] = n;
        reinterpret_cast<int64_t *>(o + reduced_off_wins(A))[tid] = w;
        (o + reduced_off_flags(A))[tid] = f;
    }
    for (int i = tid; i < A + 2; i += kReduceThreads) reinterpret_cast<int16_t *>(o + reduced_off_rae(A))[i] = s_rae[i];
    if (tid >= nb) { f = 0; n = 0; w = 0; }   // entries past the table take part as zeros (:2312-2316)

    // ---- max-argmax over (win_flag, n, n_wins), left slot kept on ties (:2318-2330) ----
    auto less = [](uint8_t fa, int64_t na, int64_t wa, uint8_t fb, int64_t nb_, int64_t wb) {
        return (fa < fb) || (fa == fb && na < nb_) || (fa == fb && na == nb_ && wa < wb);
    };
    if (A_pad > 64) {
        s_f[tid] = f; s_n[tid] = n; s_w[tid] = w; s_i[tid] = idx;
        __syncthreads();
        for (int stride = A_pad >> 1; stride >= 64; stride >>= 1) {
            if (tid < stride && less(s_f[tid], s_n[tid], s_w[tid], s_f[tid + stride], s_n[tid + stride], s_w[tid + stride])) {
                s_f[tid] = s_f[tid + stride]; s_n[tid] = s_n[tid + stride]; s_w[tid] = s_w[tid + stride]; s_i[tid] = s_i[tid + stride];
            }
            __syncthreads();
        }
        f = s_f[tid]; n = s_n[tid]; w = s_w[tid]; idx = s_i[tid];
    }
    if (wave == 0) {
        for (int stride = (A_pad > 64 ? 64 : A_pad) >> 1; stride > 0; stride >>= 1) {
            const int of = __shfl_down((int)f, stride), oi = __shfl_down((int)idx, stride);
            const long long on = __shfl_down((long long)n, stride), ow = __shfl_down((long long)w, stride);
            if (lane < stride && less(f, n, w, (uint8_t)of, on, ow)) { f = (uint8_t)of; n = on; w = ow; idx = (int16_t)oi; }
        }
        if (lane == 0) {
            ReducedHeader hd;
            hd.best_action = thrifty ? (idx < A + 2 ? (int32_t)s_rae[idx] : -1) : (int32_t)idx;
            hd.best_win_flag = f; hd.best_n = n; hd.best_n_wins = w;
            hd.n_root_entries = nb;
            hd.max_depth = s_max[0]; hd.max_size = s_max[1];
            hd.pad0[0] = hd.pad0[1] = hd.pad0[2] = 0;
            hd.depth_sum = (int64_t)s_tot[1]; hd.size_sum = (int64_t)s_tot[2];
            hd.plies = s_tot[3]; hd.u1_events = s_tot[4];
            hd.stat_levels = s_tot[5]; hd.stat_children = s_tot[6]; hd.stat_expanded = s_tot[7]; hd.stat_played = s_tot[8];
            const auto *h0 = ref0.hdr;
            hd.t_select = h0->t_select; hd.t_expand = h0->t_expand; hd.t_playout = h0->t_playout; hd.t_backup = h0->t_backup; hd.t_exchange = h0->t_exchange;
            *reinterpret_cast<ReducedHeader *>(o) = hd;
        }
    }
}
#endif

}  // namespace mctsnc
