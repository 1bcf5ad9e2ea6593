// How an expert kernel finds the slots (token, expert assignments) of its group.
#pragma once
#include "kernels.hpp"

namespace moe {

// View of one group's slots for one workgroup.
struct GroupSlots {
    int n;            // slots in the group
    int s_begin;      // dispatched mode: first slot
    const int* list;  // direct mode: LDS list of slot ids (ascending); nullptr when dispatched
    __device__ inline int slot(int i) const { return list ? list[i] : s_begin + i; }
};

// Builds the view.  All threads of the workgroup must call it (it contains barriers in direct
// mode).  `list_lds` holds DIRECT_MAX_SLOTS ints, `wtot_lds` one int per wave.
template <int NTHREADS>
__device__ inline GroupSlots group_slots(const ExpertParams& p, int grp, int* list_lds, int* wtot_lds) {
    GroupSlots gs;
    if (p.is_shared) {   // every token, in order, at slots T*k ..: needs nothing of the routing (nor of the dispatch pass)
        gs.s_begin = p.rb.T * p.rb.k;
        gs.n = p.rb.T;
        gs.list = nullptr;
        return gs;
    }
    if (!p.rb.direct) {
        gs.s_begin = p.rb.offsets[p.group0 + grp];
        gs.n = p.rb.offsets[p.group0 + grp + 1] - gs.s_begin;
        // the grid and the output hold max_rows rows per group: a table that says more is never followed past them
        if (gs.n > (int)p.max_rows) gs.n = (int)p.max_rows;
        gs.list = nullptr;
        return gs;
    }
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int A = p.rb.T * p.rb.k;
    gs.s_begin = 0;
    gs.list = list_lds;
    const int e = p.group0 + grp;
    int base = 0;
    const unsigned long long lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    for (int c0 = 0; c0 < A; c0 += NTHREADS) {
        const int a = c0 + tid;
        const bool m = a < A && p.rb.topk_idx[a] == e;
        const unsigned long long b = __ballot(m);
        if (lane == 0) wtot_lds[wave] = __popcll(b);
        __syncthreads();
        int off = base, tot = 0;
#pragma unroll
        for (int w = 0; w < NTHREADS / 64; w++) {
            const int c = wtot_lds[w];
            off += (w < wave) ? c : 0;
            tot += c;
        }
        if (m) list_lds[off + __popcll(b & lt)] = a;
        base += tot;
        __syncthreads();
    }
    gs.n = base;
    return gs;
}

// Group of a workgroup row.  Regular launches: the row index.  Launches by assignment: the expert of assignment
// `row`, or -1 when an earlier assignment has the same expert (its workgroups do the work).  Uniform per workgroup.
__device__ inline int group_of_row(const ExpertParams& p, int row) {
    if (!p.by_assignment) return row;
    const int lane = threadIdx.x & 63;
    const int e = p.rb.topk_idx[row];
    bool dup = false;
    for (int a = lane; a < row; a += 64) dup |= p.rb.topk_idx[a] == e;
    return __any(dup) ? -1 : e - p.group0;
}

// token row / routing weight of a slot
__device__ inline int slot_token(const ExpertParams& p, int slot) {
    if (p.is_shared) return slot - p.rb.T * p.rb.k;
    return p.rb.direct ? slot / p.rb.k : p.rb.perm_token[slot];
}
__device__ inline float slot_weight(const ExpertParams& p, int slot) {
    if (p.is_shared) return p.rb.shared_w[slot - p.rb.T * p.rb.k];
    return p.rb.direct ? p.rb.topk_w[slot] : p.rb.perm_w[slot];
}

// Hands one weighted expert output to the layer's result.  With top-2 routing and nothing else to add, a token's result is
// 0 + a + b (quantized_llama.rs:185-203 index_adds onto zeros in ascending expert order), and since a + b == b + a in
// floating point the two terms may arrive in either order: they are added to the zeroed output row with device-scope
// hardware float atomics and the combine pass is not needed.  Otherwise the output is stored per slot for that pass.
__device__ inline void emit_expert_output(const ExpertParams& p, int slot, int col, float v) {
    if (p.y_acc) unsafeAtomicAdd(p.y_acc + (int64_t)slot_token(p, slot) * p.H + col, v);
    else p.yw[(int64_t)slot * p.H + col] = v;
}

}  // namespace moe
