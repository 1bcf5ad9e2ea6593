// Router, dispatch and combine kernels.
//
//   front_kernel(s)         per token: optional rms-norm, gate product, softmax, top-k with
//                           renormalised weights, activation quantisation.
//   dispatch_kernel         per-expert token lists: histogram, prefix scan and a stable permutation
//                           from wavefront ballots, in one workgroup.  Small batches skip it: there
//                           the slot of (token t, rank r) is t*k + r and the expert kernels derive
//                           their lists from topk_idx themselves.
//   route_from_logits       the same routing starting from given logits (parity hook).
//   combine_kernel          routing-weighted sum of the expert outputs back in token order.
//
// Reference semantics restated here:
//   softmax_last_dim  candle-nn/src/ops.rs:313-351  (max cpu/kernels.rs:40-45, sum cpu/mod.rs:132-151
//                     in the 4 x 8-lane accumulator order of cpu/avx.rs:54-68)
//   top-k + lists     candle-transformers/src/models/quantized_llama.rs:158-179
//   combine           quantized_llama.rs:200-202 (index_add in ascending expert order)
//   rms_norm          candle-nn/src/ops.rs:504-515;  sigmoid candle-nn/src/ops.rs:59-61
#include <algorithm>
#include <cstdlib>

#include "act_quant.hpp"
#include "kernels.hpp"

namespace moe {

constexpr int FRONT_THREADS = 256;
constexpr int MAX_E = 256;
static_assert(MAX_E == DISPATCH_COUNT_STRIDE, "a workgroup's row of wg_counts holds every expert");
constexpr int MAX_K = 16;

// Sum over the wave by the butterfly lane ^ 32, ^ 16, ^ 8, ^ 4, ^ 2, ^ 1 (every lane ends with the same bits).  The last
// four steps run as rotations inside the rows of 16 lanes (DPP, no LDS traffic): after the steps before it the lanes of
// one residue class hold the same value, and lane i + o (mod 16) lies in the class of lane i ^ o, so a rotation by o adds
// the same number as the exchange would.
#define MOE_ROW_ROR(v, n) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x120 + (n), 0xf, 0xf, false))
__device__ inline float wave_sum(float v) {
    v += __shfl_xor(v, 32, 64);
    v += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401f));   // lane ^ 16
    v += MOE_ROW_ROR(v, 8);
    v += MOE_ROW_ROR(v, 4);
    v += MOE_ROW_ROR(v, 2);
    v += MOE_ROW_ROR(v, 1);
    return v;
}

__device__ inline float wave_max_f(float v) {
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401f)));
    v = fmaxf(v, MOE_ROW_ROR(v, 8));
    v = fmaxf(v, MOE_ROW_ROR(v, 4));
    v = fmaxf(v, MOE_ROW_ROR(v, 2));
    v = fmaxf(v, MOE_ROW_ROR(v, 1));
    return v;
}

// Sum of p[0..n) in the order candle's AVX2 build uses (vec_sum): for n >= 32 four 8-lane
// accumulators over blocks of 32, tree-reduced, then the tail left to right.
__device__ inline float vec_sum_ref_order(const float* p, int n) {
    int np = n & ~31;
    float b = 0.f;
    if (np) {
        float acc[32];
#pragma unroll
        for (int i = 0; i < 32; i++) acc[i] = 0.f;
        for (int i = 0; i < np; i += 32) {
#pragma unroll
            for (int j = 0; j < 32; j++) acc[j] = acc[j] + p[i + j];
        }
        float x0[8];
#pragma unroll
        for (int l = 0; l < 8; l++) x0[l] = (acc[l] + acc[8 + l]) + (acc[16 + l] + acc[24 + l]);
        float t0 = x0[0] + x0[4], t1 = x0[1] + x0[5], t2 = x0[2] + x0[6], t3 = x0[3] + x0[7];
        b = (t0 + t1) + (t2 + t3);
    }
    for (int i = np; i < n; i++) b += p[i];
    return b;
}

// One thread: softmax over E logits (in place -> probabilities) and top-k selection.
__device__ inline void route_one_token(float* p /*[E] logits in, probs out*/, int E, int k, int norm_topk,
                                       int32_t* idx_out, float* w_out) {
    float mx = p[0];
    for (int i = 1; i < E; i++) mx = fmaxf(mx, p[i]);
    for (int i = 0; i < E; i++) p[i] = expf_glibc(p[i] - mx);
    float s = vec_sum_ref_order(p, E);
    for (int i = 0; i < E; i++) p[i] = p[i] / s;
    // stable descending order by total_cmp == repeated arg-max with the lowest index winning ties
    int32_t sel[MAX_K];
    float sum = 0.f;
    for (int r = 0; r < k; r++) {
        int best = -1;
        int32_t bkey = 0;
        for (int i = 0; i < E; i++) {
            bool taken = false;
            for (int q = 0; q < r; q++) taken |= (sel[q] == i);
            if (taken) continue;
            int32_t key = total_key(p[i]);
            if (best < 0 || key > bkey) { best = i; bkey = key; }
        }
        sel[r] = best;
        sum += p[best];
    }
    for (int r = 0; r < k; r++) {
        idx_out[r] = sel[r];
        w_out[r] = norm_topk ? p[sel[r]] / sum : p[sel[r]];
    }
}

// ---------------------------------------------------------------------------------------------
// Per-expert lists.  Runs in ONE workgroup of DISPATCH_THREADS threads (16 waves).  Assignments are
// taken in (token, rank) order; within an expert the slots keep that order, i.e. ascending token
// index, exactly as the Vec pushes of the reference produce them.
constexpr int DISPATCH_THREADS = 1024;
struct DispatchShared {
    int cnt[DISPATCH_THREADS / 64][MAX_E];
    int off[MAX_E + 2];
    int tot[MAX_E];      // per expert: its assignments over all workgroups; after the scan: the tiles of the experts before it
    int before[MAX_E];
    int n_tiles;         // tiles of the E routed experts
};

// Mask of the valid lanes whose expert index equals this lane's: one ballot per bit of the index, whatever the number
// of distinct experts among the 64 lanes (a loop over the distinct values takes ~40 rounds with 60 experts and top-4).
__device__ inline unsigned long long same_expert_lanes(int e, bool valid, int ebits) {
    unsigned long long m = __ballot(valid);
    for (int b = 0; b < ebits; b++) {
        const unsigned long long set = __ballot((e >> b) & 1);
        m &= ((e >> b) & 1) ? set : ~set;
    }
    return m;
}

// One workgroup of G (`pass` 0 with G = 1: everything in one launch).  With G > 1 the assignments are cut into G stretches
// and the work into two launches: pass 1 counts a stretch's assignments per expert into rb.wg_counts[g][:], pass 2 repeats
// its own count, reads the others' and places its stretch behind the earlier ones'.
__device__ void dispatch_block(const RouteBufs& rb, int64_t T, int E, int k, bool shared, DispatchShared& sh, int g, int G, int pass) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    constexpr int NW = DISPATCH_THREADS / 64;
    const int64_t A = T * k;
    // a workgroup's stretch is a multiple of 64 * NW assignments, a wave's chunk of 64 (and so of every k <= 16 that is a
    // power of two: such a token's assignments stay in one wave's 64 lanes)
    const int64_t stretch = ((A + G - 1) / G + 64 * NW - 1) / (64 * NW) * (64 * NW);
    const int64_t a_lo = g * stretch, a_hi = a_lo + stretch < A ? a_lo + stretch : A;
    const int64_t chunk = stretch / NW;
    const int64_t lo = a_lo + wave * chunk, hi = lo + chunk < a_hi ? lo + chunk : a_hi;
    const unsigned long long lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));   // the lanes below this one
    const int ebits = 32 - __clz(E > 1 ? E - 1 : 1);                              // bits of an expert index
    for (int i = tid; i < NW * MAX_E; i += DISPATCH_THREADS) (&sh.cnt[0][0])[i] = 0;
    __syncthreads();
    // phase 1: per-wave histogram from ballots (topk_idx comes from the previous kernel: plain loads,
    // the next 64 assignments requested while these are counted)
    {
        int e_next = (lo + lane < hi) ? rb.topk_idx[lo + lane] : -1;
        for (int64_t base = lo; base < hi; base += 64) {
            const int e = e_next;
            const bool valid = base + lane < hi;
            e_next = (base + 64 + lane < hi) ? rb.topk_idx[base + 64 + lane] : -1;
            // lanes of this wave with the same expert; the lowest of them adds the group's size
            const unsigned long long m = same_expert_lanes(e, valid, ebits);
            if (valid && (m & lt) == 0) sh.cnt[wave][e] += __popcll(m);
        }
    }
    __syncthreads();
    // phase 2: totals per expert (over all workgroups), exclusive scan over experts (one wave, four experts per lane),
    // per-wave bases behind the earlier workgroups' assignments
    for (int e = tid; e < MAX_E; e += DISPATCH_THREADS) {
        int mine = 0, all = 0, before = 0;
        if (e < E) {
            for (int w = 0; w < NW; w++) mine += sh.cnt[w][e];
            all = mine;
            if (pass == 2)
                for (int gg = 0; gg < G; gg++) {
                    if (gg == g) continue;
                    const int c = rb.wg_counts[gg * MAX_E + e];
                    all += c;
                    if (gg < g) before += c;
                }
        }
        if (pass == 1) rb.wg_counts[g * MAX_E + e] = mine;
        sh.tot[e] = all;
        sh.before[e] = before;
    }
    if (pass == 1) return;
    __syncthreads();
    if (wave == 0) {
        static_assert(MAX_E == 256, "four experts per lane");
        const int t0 = sh.tot[4 * lane], t1 = sh.tot[4 * lane + 1], t2 = sh.tot[4 * lane + 2], t3 = sh.tot[4 * lane + 3];
        int incl = t0 + t1 + t2 + t3;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_up(incl, o, 64);
            if (lane >= o) incl += v;
        }
        const int base = incl - (t0 + t1 + t2 + t3);
        sh.off[4 * lane] = base;
        sh.off[4 * lane + 1] = base + t0;
        sh.off[4 * lane + 2] = base + t0 + t1;
        sh.off[4 * lane + 3] = base + t0 + t1 + t2;
        if (lane == 63) sh.off[MAX_E] = incl;   // = A
        // the same scan over the experts' tile counts (work list of the tiled kernels; the tile size is a power of two)
        const int tsh = 31 - __clz(rb.tile_slots > 0 ? rb.tile_slots : 1), tm = (1 << tsh) - 1;
        const int l0 = (t0 + tm) >> tsh, l1 = (t1 + tm) >> tsh, l2 = (t2 + tm) >> tsh, l3 = (t3 + tm) >> tsh;
        int tincl = l0 + l1 + l2 + l3;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_up(tincl, o, 64);
            if (lane >= o) tincl += v;
        }
        const int tbase = tincl - (l0 + l1 + l2 + l3);
        sh.tot[4 * lane] = tbase;
        sh.tot[4 * lane + 1] = tbase + l0;
        sh.tot[4 * lane + 2] = tbase + l0 + l1;
        sh.tot[4 * lane + 3] = tbase + l0 + l1 + l2;
        if (lane == 63) sh.n_tiles = tincl;
    }
    __syncthreads();
    if (tid == 0) {   // experts past E have no assignments: off[E] == A already; the shared expert follows
        sh.off[E] = (int)A;
        sh.off[E + 1] = (int)A + (shared ? (int)T : 0);
    }
    for (int e = tid; e < E; e += DISPATCH_THREADS) {
        int run = sh.off[e] + sh.before[e];
        for (int w = 0; w < NW; w++) {
            int c = sh.cnt[w][e];
            sh.cnt[w][e] = run;  // becomes the wave's running cursor
            run += c;
        }
    }
    __syncthreads();
    if (g == 0) {
        for (int e = tid; e <= E + (shared ? 1 : 0); e += DISPATCH_THREADS) rb.offsets[e] = sh.off[e];
        if (rb.tile_tab) {  // work list of the tiled expert kernels: a group's tiles follow those of the groups before it
            const int NG = E + (shared ? 1 : 0), ts = rb.tile_slots;
            for (int gi = tid; gi < NG; gi += DISPATCH_THREADS) {
                int n = gi < E ? sh.tot[gi] : sh.n_tiles;
                const int len = sh.off[gi + 1] - sh.off[gi];
                for (int pos = 0; pos < len; pos += ts, n++) {
                    rb.tile_tab[1 + 2 * n] = gi;
                    rb.tile_tab[2 + 2 * n] = pos;
                }
                if (gi == NG - 1) rb.tile_tab[0] = n;
            }
        }
    }
    // phase 3: stable placement; the token's row of tok_slots lists its slots by ascending expert index (the order
    // of the combine pass): an assignment's place there is the number of the token's experts below its own.  With k a
    // power of two a token's assignments lie in one wave's 64 lanes, otherwise its experts are read back.
    const int kk = k + (shared ? 1 : 0);
    const bool in_wave = (k & (k - 1)) == 0;   // k <= 16
    {
        int e_next = (lo + lane < hi) ? rb.topk_idx[lo + lane] : -1;
        float w_next = (lo + lane < hi) ? rb.topk_w[lo + lane] : 0.f;
        for (int64_t base = lo; base < hi; base += 64) {
            const int64_t a = base + lane;
            const bool valid = a < hi;
            const int e = e_next;
            const float w = w_next;
            e_next = (a + 64 < hi) ? rb.topk_idx[a + 64] : -1;
            w_next = (a + 64 < hi) ? rb.topk_w[a + 64] : 0.f;
            const unsigned long long m = same_expert_lanes(e, valid, ebits);
            const int t = (int)((uint32_t)a / (uint32_t)k), r0 = (int)a - t * k;
            int place = 0;
            if (in_wave) {
                const int first = lane - r0;
                for (int j = 0; j < k; j++) {
                    const int ej = __shfl(e, first + j, 64);
                    place += (ej < e || (ej == e && j < r0)) ? 1 : 0;
                }
            } else if (valid) {
#pragma unroll 4
                for (int j = 0; j < k; j++) {
                    const int ej = rb.topk_idx[(int64_t)t * k + j];
                    place += (ej < e || (ej == e && j < r0)) ? 1 : 0;
                }
            }
            int slot = -1;
            if (valid) {
                const int cur = sh.cnt[wave][e];
                slot = cur + __popcll(m & lt);
                // every lane of the group has read `cur` before its lowest lane updates it (one wave, program order)
                if ((m & lt) == 0) sh.cnt[wave][e] = cur + __popcll(m);
            }
            if (valid) {
                rb.perm_token[slot] = t;
                rb.perm_w[slot] = w;
                rb.tok_slots[(int64_t)t * kk + place] = slot;
            }
        }
    }
    // phase 4: the always-on expert's slots follow the routed ones
    if (shared)
        for (int64_t t = (int64_t)g * DISPATCH_THREADS + tid; t < T; t += (int64_t)G * DISPATCH_THREADS) {
            const int slot = (int)(A + t);
            rb.tok_slots[t * kk + k] = slot;
            rb.perm_token[slot] = (int)t;
            rb.perm_w[slot] = rb.shared_w[t];
        }
}

// ---------------------------------------------------------------------------------------------
__device__ inline void route_one_token_wave(float logit, int lane, int E, int k, int norm_topk, int32_t* idx_out, float* w_out);
__device__ inline void route_one_token_wave_lds(float* p, int lane, int E, int k, int norm_topk, int32_t* idx_out, float* w_out, int* sel, long long* order);

template <int VDT>
__global__ __launch_bounds__(FRONT_THREADS) void front_kernel(FrontParams p) {
    extern __shared__ float xrow[];  // [H]
    __shared__ float probs[MAX_E];
    __shared__ int sel_lds[MAX_K];
    __shared__ __align__(16) long long order_lds[MAX_E];
    __shared__ float red[FRONT_THREADS / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t t = blockIdx.x;
    const int H = p.H, E = p.E;
    const float* x = p.x + t * H;

    // ---- load the row (and normalise it if the layer carries the pre-norm)
    for (int h = tid * 4; h < H; h += FRONT_THREADS * 4) *reinterpret_cast<float4*>(xrow + h) = *reinterpret_cast<const float4*>(x + h);
    if (p.rms_alpha) {
        // sum of squares left to right, as the reference does (see front_fast_kernel)
        __syncthreads();
        if (tid == 0) {
            float tot = 0.f;
            for (int h = 0; h < H; h++) tot += xrow[h] * xrow[h];
            red[0] = sqrtf(tot / (float)H + p.rms_eps);
        }
        __syncthreads();
        const float m = red[0];
        __syncthreads();
        for (int h = tid; h < H; h += FRONT_THREADS) xrow[h] = xrow[h] / m * p.rms_alpha[h];
    }
    __syncthreads();

    // ---- gate product: wave w owns experts w, w+4, ...; the shared-expert gate is "expert" E
    const int n_dot = E + (p.shared_gate ? 1 : 0);
    for (int e = wave; e < n_dot; e += FRONT_THREADS / 64) {
        const float* wrow = (e < E) ? p.gate + (int64_t)e * H : p.shared_gate;
        float acc = 0.f;
        for (int h = lane * 4; h < H; h += 256) {
            float4 wv = *reinterpret_cast<const float4*>(wrow + h);
            float4 xv = *reinterpret_cast<const float4*>(xrow + h);
            acc = __builtin_fmaf(wv.x, xv.x, acc);
            acc = __builtin_fmaf(wv.y, xv.y, acc);
            acc = __builtin_fmaf(wv.z, xv.z, acc);
            acc = __builtin_fmaf(wv.w, xv.w, acc);
        }
        acc = wave_sum(acc);
        if (lane == 0) {
            if (e < E) {
                if (p.gate_bias) acc += p.gate_bias[e];
                probs[e] = acc;
                p.rb.logits[t * E + e] = acc;
            } else {
                p.rb.shared_w[t] = 1.0f / (expf_glibc(-acc) + 1.0f);
            }
        }
    }
    __syncthreads();

    // the row of x is in LDS by now (the output may be the input buffer): clear the token's output row if the down
    // kernels are to accumulate into it
    if (p.y_zero)
        for (int h = tid * 4; h < H; h += FRONT_THREADS * 4) *reinterpret_cast<float4*>(p.y_zero + t * H + h) = make_float4(0.f, 0.f, 0.f, 0.f);

    // ---- wave 0 routes, then joins the others in quantising the row
    if (wave == 0) {
        if (E <= 64) route_one_token_wave(lane < E ? probs[lane] : 0.f, lane, E, p.k, p.norm_topk, p.rb.topk_idx + t * p.k, p.rb.topk_w + t * p.k);
        else route_one_token_wave_lds(probs, lane, E, p.k, p.norm_topk, p.rb.topk_idx + t * p.k, p.rb.topk_w + t * p.k, sel_lds, order_lds);
    }

    if (VDT == MOE_GGML_Q8K) {
        const int nb = H / 256;
        for (int b = wave; b < nb; b += FRONT_THREADS / 64) {
            float4 v = *reinterpret_cast<const float4*>(xrow + b * 256 + lane * 4);
            quantize_q8k_block(v, lane, p.xq.qs + t * H + b * 256, p.xq.d + t * nb + b,
                               reinterpret_cast<__half*>(p.xq.bsum) + (t * nb + b) * 16);
        }
    } else {
        const int nb = H / 32;
        for (int h = tid; h < H; h += FRONT_THREADS) {
            int b = h / 32;
            quantize_q8_0_block(p.vdt, xrow[h], lane, p.xq.qs + t * H + h, p.xq.d + t * nb + b,
                                reinterpret_cast<int32_t*>(p.xq.bsum) + t * nb + b);
        }
    }

}

// ---------------------------------------------------------------------------------------------
// Wave-parallel routing for E <= 64: lane e holds expert e.  Same arithmetic, in the same order,
// as route_one_token: the exp values are summed left to right (E < 32) or in the 4 x 8
// accumulator order followed by the serial tail (E >= 32); the rank of an expert is the number of
// experts that precede it in the (total_cmp key descending, index ascending) order.  Cross-lane
// traffic goes through v_readlane (scalar broadcast), not LDS.  Call with all 64 lanes active.
__device__ inline float lane_bcast(float v, int i) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), i));
}
__device__ inline void route_one_token_wave(float logit, int lane, int E, int k, int norm_topk,
                                            int32_t* idx_out, float* w_out) {
    const bool valid = lane < E;
    float mx = -__builtin_inff();
    for (int i = 0; i < E; i++) mx = fmaxf(mx, lane_bcast(logit, i));
    const float ex = valid ? expf_glibc(logit - mx) : 0.f;
    float s;
    if (E < 32) {
        s = 0.f;
        for (int i = 0; i < E; i++) s += lane_bcast(ex, i);
    } else {
        // acc[j] (lane j < 32) = sum over complete blocks of 32 of ex[32*b + j]
        const int np = E & ~31;
        float a = ex;                                  // block 0 (0 + ex, exact)
        float hi = __shfl(ex, (lane & 31) + 32, 64);   // block 1
        if (np >= 64) a = a + hi;
        const int l = lane & 7;
        float x0 = (__shfl(a, l, 64) + __shfl(a, 8 + l, 64)) + (__shfl(a, 16 + l, 64) + __shfl(a, 24 + l, 64));
        float t0 = lane_bcast(x0, 0) + lane_bcast(x0, 4);
        float t1 = lane_bcast(x0, 1) + lane_bcast(x0, 5);
        float t2 = lane_bcast(x0, 2) + lane_bcast(x0, 6);
        float t3 = lane_bcast(x0, 3) + lane_bcast(x0, 7);
        s = (t0 + t1) + (t2 + t3);
        for (int i = np; i < E; i++) s += lane_bcast(ex, i);
    }
    const float pr = ex / s;
    const int key = total_key(pr);
    int rank = 0;
    for (int i = 0; i < E; i++) {
        const int ki = __builtin_amdgcn_readlane(key, i);
        rank += (ki > key || (ki == key && i < lane)) ? 1 : 0;
    }
    if (!valid) rank = 0x7fffffff;
    // probabilities in rank order: sum, then the (renormalised) weights
    float sum = 0.f;
    float my_p = 0.f;
    int my_e = 0;
    for (int r = 0; r < k; r++) {
        const unsigned long long m = __ballot(rank == r);
        const int e = __ffsll((long long)m) - 1;
        const float pe = lane_bcast(pr, e);
        sum += pe;
        if (lane == r) { my_p = pe; my_e = e; }
    }
    if (lane < k) {
        idx_out[lane] = my_e;
        w_out[lane] = norm_topk ? my_p / sum : my_p;
    }
}

// Wave-parallel routing for 64 < E <= 256, the logits in LDS (`p`, overwritten with the probabilities): lane l holds
// experts l, l + 64, l + 128, l + 192.  Same arithmetic and order as route_one_token: the maximum (any order gives the
// same float), the exp values summed as vec_sum_ref_order sums them (lane j < 32 carries accumulator j over the blocks
// of 32, then the tree, then the tail left to right), the rank of an expert = the number of experts that precede it in
// the (total_cmp key descending, index ascending) order.  `sel` (LDS, k ints) receives the experts in rank order.
// Call with all 64 lanes of one wave active; p, sel and order (LDS, MAX_E entries, 16-byte aligned) belong to that wave.
// Ranks of a lane's NQ experts among all E: order[i] = (total_cmp key of p[i], ~i) as one signed 64-bit integer, so that
// "i precedes e" is one comparison; four entries per LDS read pair.
template <int NQ>
__device__ __forceinline__ void count_ranks(const long long* order, int E, const long long (&mine)[4], int (&rank)[4]) {
    for (int i = 0; i < E; i += 4) {
        const longlong2 a = *reinterpret_cast<const longlong2*>(order + i), b = *reinterpret_cast<const longlong2*>(order + i + 2);
        const long long c[4] = {a.x, a.y, b.x, b.y};
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int q = 0; q < NQ; q++) rank[q] += c[j] > mine[q] ? 1 : 0;
    }
}
__device__ inline void route_one_token_wave_lds(float* p, int lane, int E, int k, int norm_topk, int32_t* idx_out, float* w_out, int* sel, long long* order_lds) {
    float mx = -__builtin_inff();
    bool any = false;   // fmaxf skips NaNs; with nothing but NaNs the serial loop is left with one
    for (int e = lane; e < E; e += 64) {
        const float v = p[e];
        if (v == v) { mx = fmaxf(mx, v); any = true; }
    }
    mx = wave_max_f(mx);
    if (__ballot(any) == 0ull) mx = p[0];
    for (int e = lane; e < E; e += 64) p[e] = expf_glibc(p[e] - mx);
    __builtin_amdgcn_wave_barrier();
    const int np = E & ~31;
    float acc = 0.f;
    for (int b = 0; b < np; b += 32) acc = acc + p[b + (lane & 31)];
    const int l8 = lane & 7;
    const float x0 = (__shfl(acc, l8, 64) + __shfl(acc, 8 + l8, 64)) + (__shfl(acc, 16 + l8, 64) + __shfl(acc, 24 + l8, 64));
    const float t0 = lane_bcast(x0, 0) + lane_bcast(x0, 4);
    const float t1 = lane_bcast(x0, 1) + lane_bcast(x0, 5);
    const float t2 = lane_bcast(x0, 2) + lane_bcast(x0, 6);
    const float t3 = lane_bcast(x0, 3) + lane_bcast(x0, 7);
    float s = (t0 + t1) + (t2 + t3);
    for (int i = np; i < E; i++) s += p[i];
    static_assert(MAX_E == 256, "four experts per lane");
    float pr[4];
    long long mine[4];
    int rank[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const int e = lane + 64 * q;
        pr[q] = e < E ? p[e] / s : 0.f;
        // experts past E sort behind everything (the loop reads the table in fours)
        mine[q] = e < E ? (long long)(((unsigned long long)(uint32_t)total_key(pr[q]) << 32) | (uint32_t)~(uint32_t)e)
                        : (long long)0x8000000000000000ull;
        rank[q] = 0;
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int q = 0; q < 4; q++) {
        if (lane + 64 * q < E) p[lane + 64 * q] = pr[q];
        order_lds[lane + 64 * q] = mine[q];
    }
    __builtin_amdgcn_wave_barrier();
    if (E <= 128) count_ranks<2>(order_lds, E, mine, rank);
    else if (E <= 192) count_ranks<3>(order_lds, E, mine, rank);
    else count_ranks<4>(order_lds, E, mine, rank);
#pragma unroll
    for (int q = 0; q < 4; q++)
        if (lane + 64 * q < E && rank[q] < k) sel[rank[q]] = lane + 64 * q;
    __builtin_amdgcn_wave_barrier();
    float sum = 0.f;
    for (int r = 0; r < k; r++) sum += p[sel[r]];
    if (lane < k) {
        const int e = sel[lane];
        idx_out[lane] = e;
        w_out[lane] = norm_topk ? p[e] / sum : p[e];
    }
}

// Low-latency front end for H = NCH * 256 (NCH <= 32) and E <= 64.  512 threads per token: waves
// 0-3 compute the gate products (two experts at a time, all loads issued up front), waves 4-7
// quantise the row, then one barrier and wave 0 routes.  Every wave keeps the activation row in
// registers (lane l holds elements 256*i + 4l .. +3); with the pre-norm every wave evaluates the
// same sum of squares in the same order, so all of them normalise with the same divisor.
// Plain float arrays with compile-time indices only: nothing here may end up in scratch memory.
constexpr int FAST_THREADS = 512;

// Quantises chunk `chunk` (256 elements, this lane holds 4) of token row t; phases are written so
// that a caller looping over several chunks gets independent dependency chains.
template <int VDT>
__device__ inline void quantize_chunk(const FrontParams& p, int64_t t, int H, int chunk, const float e[4], int lane) {
    if (VDT == MOE_GGML_Q8K) {
        const int nb = H / 256;
        float4 v = make_float4(e[0], e[1], e[2], e[3]);
        quantize_q8k_block(v, lane, p.xq.qs + t * H + chunk * 256, p.xq.d + t * nb + chunk,
                           reinterpret_cast<__half*>(p.xq.bsum) + (t * nb + chunk) * 16);
    } else {
        const int nb = H / 32;
        float amax = fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3])));
#pragma unroll
        for (int o = 4; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));  // eight lanes share a block
        const float d = amax / 127.0f;
        const float id = (d != 0.f) ? 1.0f / d : 0.f;
        uint32_t packed = 0;
        int sum = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int qv = round_as_i8(e[j] * id);
            sum += qv;
            packed |= (uint32_t)(uint8_t)qv << (8 * j);
        }
#pragma unroll
        for (int o = 4; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
        *reinterpret_cast<uint32_t*>(p.xq.qs + t * H + chunk * 256 + lane * 4) = packed;
        if ((lane & 7) == 0) {
            const int b = chunk * 8 + (lane >> 3);
            const float dh = __half2float(__float2half_rn(d));
            p.xq.d[t * nb + b] = dh;
            reinterpret_cast<int32_t*>(p.xq.bsum)[t * nb + b] = q8_block_word(p.vdt, sum, dh);
        }
    }
}

// Sum of the squares of a row in the reference's order: ((x0^2 + x1^2) + x2^2) + ..., every product and every
// partial sum rounded to f32 (candle-nn/src/ops.rs:504-515 folds the row with `sum::<f32>()`).  Taken literally that is
// a chain of H dependent adds, ten cycles each for a lone wave (20 us at H = 4096).  The chain is cut into 64 chunks:
// while a running sum S = k * u (k its 24-bit significand, u its ulp) stays inside one binade, adding a term v moves
// k by round-to-nearest-even(v / u), i.e. by floor(v / u), plus one if the fraction exceeds 1/2, plus the parity of the
// result if the fraction is exactly 1/2.  Such steps compose: a run of them maps k to k + (k even ? a0 : a1), and two
// runs compose into a pair of the same kind.  Every chunk is summarised this way in parallel for the binade that an
// approximate prefix sum predicts for it; one wave then walks the chunks with the exact running sum and takes the
// summary when the sum enters the chunk in the predicted binade and leaves it in the same one (the partial sums only
// grow, so the end decides), and adds the chunk term by term otherwise (chunk 0, binade crossings, NaN / overflow: a
// handful of chunks per row).  Either way the bits equal those of the term-by-term sum.  Call with all FAST_THREADS
// threads; every wave holds the row (xr[4 i + j] = x[256 i + 4 lane + j]); `serial_only` adds every chunk term by term.
template <int NCH>
__device__ inline float ordered_sum_of_squares(const float* xr, int tid, bool serial_only, float* sqp) {
    constexpr int L = NCH * 4, LP = L + 1;     // chunk length; chunks are padded by one word so that lanes reading
                                               // the same position of 64 chunks hit 64 different banks (sqp: 64 * LP floats)
    __shared__ int part[8][64][2];
    __shared__ float result;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr bool kSummaries = NCH >= 4 && NCH % 2 == 0;
    const bool summaries = kSummaries && !serial_only;
#pragma unroll
    for (int i = 0; i < NCH; i++)
        if ((i & 7) == wave) {
            const int idx = i * 256 + lane * 4;
            float* d = sqp + idx + idx / L;
            d[0] = xr[4 * i] * xr[4 * i]; d[1] = xr[4 * i + 1] * xr[4 * i + 1];
            d[2] = xr[4 * i + 2] * xr[4 * i + 2]; d[3] = xr[4 * i + 3] * xr[4 * i + 3];
        }
    __syncthreads();
    const float* mine = sqp + lane * LP;
    int e = 0;   // biased exponent predicted for the running sum at the start of chunk `lane`; 0 = no summary
    if (summaries) {
        float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll
        for (int j = 0; j < L; j += 4) { s0 += mine[j]; s1 += mine[j + 1]; s2 += mine[j + 2]; s3 += mine[j + 3]; }
        float incl = (s0 + s1) + (s2 + s3);
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const float o = __shfl_up(incl, d, 64);
            if (lane >= d) incl += o;
        }
        const float excl = __shfl_up(incl, 1, 64);
        const int eb = (int)(__float_as_uint(excl) >> 23);
        // 1 / u = 2^(150 - eb) has to be a normal float
        if (lane > 0 && eb >= 23 && eb <= 254) e = eb;
        int a0 = 0, a1 = 0;
        if (e) {
            const float inv_u = __uint_as_float((uint32_t)(277 - e) << 23);
#pragma unroll
            for (int jj = 0; jj < L / 8; jj++) {
                float sc = mine[wave * (L / 8) + jj] * inv_u;   // a power of two: exact
                if (!(sc < 16777216.f)) sc = 16777216.f;         // too large for this binade (or NaN): the end test fails
                const float q = floorf(sc), f = sc - q;
                const int n = (int)q + (f > 0.5f ? 1 : 0);
                const bool tie = f == 0.5f;
                a0 += n + (tie ? ((a0 + n) & 1) : 0);
                a1 += n + (tie ? ((1 + a1 + n) & 1) : 0);
            }
        }
        part[wave][lane][0] = a0;
        part[wave][lane][1] = a1;
    }
    __syncthreads();
    if (wave == 0) {
        int a0 = 0, a1 = 0;
        if (summaries) {
            a0 = part[0][lane][0]; a1 = part[0][lane][1];
#pragma unroll
            for (int w = 1; w < 8; w++) {
                const int b0 = part[w][lane][0], b1 = part[w][lane][1];
                a0 += (a0 & 1) ? b1 : b0;
                a1 += ((1 + a1) & 1) ? b1 : b0;
                a0 = a0 < (1 << 25) ? a0 : (1 << 25);   // anything from 2^24 on fails the end test; keeps the sums in range
                a1 = a1 < (1 << 25) ? a1 : (1 << 25);
            }
        }
        // bits of the first float of the predicted binade; all ones where the chunk has no summary
        const uint32_t lo_v = e ? (uint32_t)e << 23 : 0xffffffffu;
        uint32_t b = 0;   // bits of the running sum, the same in every lane
        for (int c = 0; c < 64; c++) {
            const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)lo_v, c);
            const uint32_t s0 = (uint32_t)__builtin_amdgcn_readlane(a0, c), s1 = (uint32_t)__builtin_amdgcn_readlane(a1, c);
            const uint32_t nb = b + ((b & 1u) ? s1 : s0);   // inside a binade the significand's increment adds to the bits
            // taken when the sum enters the chunk in the predicted binade and leaves it there: both share lo's top nine bits
            if ((((b ^ lo) | (nb ^ lo)) >> 23) == 0u) {
                b = nb;
            } else {
                float S = __uint_as_float(b);
                const float* ch = sqp + c * LP;
#pragma unroll
                for (int j0 = 0; j0 < L; j0 += 16) {
                    float v[16];
#pragma unroll
                    for (int j = 0; j < 16 && j0 + j < L; j++) v[j] = ch[j0 + j];
#pragma unroll
                    for (int j = 0; j < 16 && j0 + j < L; j++) S += v[j];
                }
                b = __builtin_amdgcn_readfirstlane(__float_as_uint(S));
            }
        }
        if (lane == 0) result = __uint_as_float(b);
    }
    __syncthreads();
    return result;
}

// WIDE (layers with dozens of experts, small batches): all eight waves take gate products, after sharing out the
// quantisation -- a token's gate rows are a megabyte at 128 experts, and a workgroup that requests two rows per wave at a
// time from four waves spends its time waiting for them (one token, 128 experts of 2048: 28 us).
template <int VDT, int NCH, bool LEAN, bool WIDE = false>
__device__ __forceinline__ void front_fast_body(const FrontParams& p) {
    __shared__ float logit_lds[MAX_E];
    __shared__ int sel_lds[MAX_K];
    __shared__ __align__(16) long long order_lds[MAX_E];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t t = blockIdx.x;
    constexpr int H = NCH * 256;
    const int E = p.E;
    float xr[NCH * 4];
    // the rms-norm's workspace; also the row exchange of a folded-in combine pass
    __shared__ float row_lds[LEAN ? 1 : 64 * (NCH * 4 + 1)];
    if (!LEAN && p.prev.yw) {
        // the previous layer's combine pass: its terms in ascending expert order onto zero, then its residual
        // (combine_kernel's additions in combine_kernel's order).  Wave i % 8 sums chunk i -- all of a wave's loads are in
        // flight together -- stores it as the previous layer's output and shares it through the LDS.
        constexpr int PK = 8;   // terms requested together
        const int pk = p.prev.k;
        const int e = lane < pk ? p.prev.topk_idx[t * pk + lane] : 0x7fffffff;
        int rank = 0;
        for (int j = 0; j < pk; j++) {
            const int ej = __shfl(e, j, 64);
            rank += (ej < e || (ej == e && j < lane)) ? 1 : 0;
        }
        // lane j learns which of the token's slots comes j-th
        int nth = 0;
        for (int j = 0; j < pk; j++) {
            const int rj = __shfl(rank, j, 64);
            if (rj == lane) nth = j;
        }
        const int64_t slot0 = t * pk;
#pragma unroll
        for (int i = 0; i < NCH; i++)
            if ((i & 7) == wave) {
                float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
                float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
                if (p.prev.residual) r = *reinterpret_cast<const float4*>(p.prev.residual + t * H + i * 256 + lane * 4);
                for (int j0 = 0; j0 < pk; j0 += PK) {
                    float4 a[PK];
#pragma unroll
                    for (int j = 0; j < PK; j++)
                        if (j0 + j < pk) {
                            const int64_t slot = slot0 + __builtin_amdgcn_readlane(nth, (j0 + j) & 63);
                            a[j] = *reinterpret_cast<const float4*>(p.prev.yw + slot * H + i * 256 + lane * 4);
                        }
#pragma unroll
                    for (int j = 0; j < PK; j++)
                        if (j0 + j < pk) { acc.x += a[j].x; acc.y += a[j].y; acc.z += a[j].z; acc.w += a[j].w; }
                }
                if (p.prev.residual) { acc.x += r.x; acc.y += r.y; acc.z += r.z; acc.w += r.w; }
                *reinterpret_cast<float4*>(p.prev.x_out + t * H + i * 256 + lane * 4) = acc;
                *reinterpret_cast<float4*>(row_lds + i * 256 + lane * 4) = acc;
            }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const float4 v = *reinterpret_cast<const float4*>(row_lds + i * 256 + lane * 4);
            xr[4 * i] = v.x; xr[4 * i + 1] = v.y; xr[4 * i + 2] = v.z; xr[4 * i + 3] = v.w;
        }
        __syncthreads();   // the norm below writes row_lds again
    } else {
        const float* x = p.x + t * H;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const float4 v = *reinterpret_cast<const float4*>(x + i * 256 + lane * 4);
            xr[4 * i] = v.x; xr[4 * i + 1] = v.y; xr[4 * i + 2] = v.z; xr[4 * i + 3] = v.w;
        }
    }
    // Gate rows of experts e0 and e0 + 4 (the shared-expert gate counts as expert E).  Waves 0..3 request their first
    // pair here, ahead of the rms-norm: nothing has touched the gate since the layer last ran, and the fetch from HBM
    // then overlaps the norm instead of following its barriers.
    const int n_dot = E + (p.shared_gate ? 1 : 0);
    float4 wa[NCH], wb[NCH];
    auto load_gate_pair = [&](int e0) {
        const int e1 = e0 + (WIDE ? 8 : 4) < n_dot ? e0 + (WIDE ? 8 : 4) : e0;
        const float* w0 = (e0 < E) ? p.gate + (int64_t)e0 * H : p.shared_gate;
        const float* w1 = (e1 < E) ? p.gate + (int64_t)e1 * H : p.shared_gate;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            wa[i] = *reinterpret_cast<const float4*>(w0 + i * 256 + lane * 4);
            wb[i] = *reinterpret_cast<const float4*>(w1 + i * 256 + lane * 4);
        }
    };
    // (only with an rms-norm ahead: without one the early request measured 0.9 us slower on a gate that is still in the
    // L2; and not for rows beyond 4096, where two gate rows and the token's row exceed the registers)
    const bool early_gate = !LEAN && NCH <= 16 && p.rms_alpha != nullptr;
    if (early_gate && wave < (WIDE ? 8 : 4) && wave < n_dot) load_gate_pair(wave);
    if (!LEAN && p.rms_alpha) {
        // rms_norm (candle-nn/src/ops.rs:504-515) sums the squares left to right in f32.  A different
        // order changes the divisor in the last ulp, which flips quantised activations now and then
        // and moves a whole output row by 1e-3 of its rms, so the sum keeps the reference's order.
        const float sum2 = ordered_sum_of_squares<NCH>(xr, tid, p.rms_serial != 0, row_lds);
        const float m = sqrtf(sum2 / (float)H + p.rms_eps);
        // every wave holds the whole row: each normalises an eighth of it (a correctly rounded division per element)
        // and the waves exchange the results (the sum's last barrier has released row_lds)
#pragma unroll
        for (int i = 0; i < NCH; i++)
            if ((i & 7) == wave) {
                const float4 a = *reinterpret_cast<const float4*>(p.rms_alpha + i * 256 + lane * 4);
                *reinterpret_cast<float4*>(row_lds + i * 256 + lane * 4) =
                    make_float4(xr[4 * i] / m * a.x, xr[4 * i + 1] / m * a.y, xr[4 * i + 2] / m * a.z, xr[4 * i + 3] / m * a.w);
            }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const float4 v = *reinterpret_cast<const float4*>(row_lds + i * 256 + lane * 4);
            xr[4 * i] = v.x; xr[4 * i + 1] = v.y; xr[4 * i + 2] = v.z; xr[4 * i + 3] = v.w;
        }
    }
    // rows of 4096 and more leave no registers for a second buffer (and few experts per wave to run ahead over)
    // gate products: waves 0..3 while waves 4..7 quantise (all eight waves on the products with the quantisation shared
    // out afterwards measured no better at 61 products per token and worse at 8)
    static_assert(!(LEAN && WIDE), "one or the other");
    constexpr int GW = WIDE ? 8 : 4;
    constexpr bool LEAN_PIPE = NCH < 16;
    constexpr int LEAN_PIECE = LEAN_PIPE ? 2 : 4, LEAN_NP = LEAN ? NCH / LEAN_PIECE : 2;
    static_assert(!LEAN || (NCH % LEAN_PIECE == 0 && LEAN_NP % 2 == 0), "the pieces alternate between two buffers");
    float4 qa[2][LEAN_PIECE], qb[2][LEAN_PIECE];
    auto load_piece = [&](int e0, int pc, int buf) {
        const int e1 = e0 + GW < n_dot ? e0 + GW : e0;
        const float* w0 = (e0 < E) ? p.gate + (int64_t)e0 * H : p.shared_gate;
        const float* w1 = (e1 < E) ? p.gate + (int64_t)e1 * H : p.shared_gate;
#pragma unroll
        for (int j = 0; j < LEAN_PIECE; j++) {
            qa[buf][j] = *reinterpret_cast<const float4*>(w0 + (pc * LEAN_PIECE + j) * 256 + lane * 4);
            qb[buf][j] = *reinterpret_cast<const float4*>(w1 + (pc * LEAN_PIECE + j) * 256 + lane * 4);
        }
    };
    if constexpr (WIDE) {   // every wave quantises its share of the row (chunks wave, wave + 8, ...), then joins the products
#pragma unroll
        for (int i = 0; i < NCH; i++)
            if ((i & 7) == wave) {
                const float e4[4] = {xr[4 * i], xr[4 * i + 1], xr[4 * i + 2], xr[4 * i + 3]};
                quantize_chunk<VDT>(p, t, H, i, e4, lane);
            }
    }
    if (wave < GW) {
        // gate products
        if (LEAN && LEAN_PIPE && wave < n_dot) load_piece(wave, 0, 0);
        for (int e0 = wave; e0 < n_dot; e0 += 2 * GW) {
            const int e1 = e0 + GW < n_dot ? e0 + GW : e0;
            float acc0 = 0.f, acc1 = 0.f;
            if constexpr (LEAN) {
                // the gate rows pass through in pieces of two or four chunks (same products, same order; a quarter of
                // the registers, so that two workgroups fit a CU); short rows: each piece is requested while the one before
                // it is multiplied, across the wave's experts too
#pragma unroll
                for (int pc = 0; pc < LEAN_NP; pc++) {
                    if (!LEAN_PIPE) load_piece(e0, pc, 0);
                    else if (pc + 1 < LEAN_NP) load_piece(e0, pc + 1, (pc + 1) & 1);
                    else if (e0 + 2 * GW < n_dot) load_piece(e0 + 2 * GW, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    const int buf = LEAN_PIPE ? (pc & 1) : 0;
#pragma unroll
                    for (int j = 0; j < LEAN_PIECE; j++) {
                        const int i = pc * LEAN_PIECE + j;
                        const float4 a = qa[buf][j], b = qb[buf][j];
                        acc0 = __builtin_fmaf(a.x, xr[4 * i], acc0);     acc1 = __builtin_fmaf(b.x, xr[4 * i], acc1);
                        acc0 = __builtin_fmaf(a.y, xr[4 * i + 1], acc0); acc1 = __builtin_fmaf(b.y, xr[4 * i + 1], acc1);
                        acc0 = __builtin_fmaf(a.z, xr[4 * i + 2], acc0); acc1 = __builtin_fmaf(b.z, xr[4 * i + 2], acc1);
                        acc0 = __builtin_fmaf(a.w, xr[4 * i + 3], acc0); acc1 = __builtin_fmaf(b.w, xr[4 * i + 3], acc1);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                if (!early_gate || e0 != wave) load_gate_pair(e0);
#pragma unroll
                for (int i = 0; i < NCH; i++) {
                    acc0 = __builtin_fmaf(wa[i].x, xr[4 * i], acc0);     acc1 = __builtin_fmaf(wb[i].x, xr[4 * i], acc1);
                    acc0 = __builtin_fmaf(wa[i].y, xr[4 * i + 1], acc0); acc1 = __builtin_fmaf(wb[i].y, xr[4 * i + 1], acc1);
                    acc0 = __builtin_fmaf(wa[i].z, xr[4 * i + 2], acc0); acc1 = __builtin_fmaf(wb[i].z, xr[4 * i + 2], acc1);
                    acc0 = __builtin_fmaf(wa[i].w, xr[4 * i + 3], acc0); acc1 = __builtin_fmaf(wb[i].w, xr[4 * i + 3], acc1);
                }
            }
            acc0 = wave_sum(acc0);
            acc1 = wave_sum(acc1);
            if (lane == 0) {
                if (e0 < E) {
                    if (p.gate_bias) acc0 += p.gate_bias[e0];
                    logit_lds[e0] = acc0;
                    p.rb.logits[t * E + e0] = acc0;
                } else {
                    p.rb.shared_w[t] = 1.0f / (expf_glibc(-acc0) + 1.0f);
                }
                if (e1 != e0) {
                    if (e1 < E) {
                        if (p.gate_bias) acc1 += p.gate_bias[e1];
                        logit_lds[e1] = acc1;
                        p.rb.logits[t * E + e1] = acc1;
                    } else {
                        p.rb.shared_w[t] = 1.0f / (expf_glibc(-acc1) + 1.0f);
                    }
                }
            }
        }
    }
    if constexpr (!WIDE) {
        if (wave >= GW) {
            // quantise: wave 4+q owns chunks q, q+4, ...; the branches are wave-uniform
            const int q = wave - GW;
#pragma unroll
            for (int i = 0; i < NCH; i++)
                if ((i & 3) == q) {
                    const float e4[4] = {xr[4 * i], xr[4 * i + 1], xr[4 * i + 2], xr[4 * i + 3]};
                    quantize_chunk<VDT>(p, t, H, i, e4, lane);
                }
        }
    }
    __syncthreads();
    // every wave read the row of x at the start (the output may be the input buffer): clear the token's output row if
    // the down kernels are to accumulate into it
    if (p.y_zero)
        for (int i = tid; i < H / 4; i += FAST_THREADS) reinterpret_cast<float4*>(p.y_zero + t * H)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (wave == 0) {
        if (E <= 64) route_one_token_wave(lane < E ? logit_lds[lane] : 0.f, lane, E, p.k, p.norm_topk, p.rb.topk_idx + t * p.k, p.rb.topk_w + t * p.k);
        else route_one_token_wave_lds(logit_lds, lane, E, p.k, p.norm_topk, p.rb.topk_idx + t * p.k, p.rb.topk_w + t * p.k, sel_lds, order_lds);
    }
}
template <int VDT, int NCH>
__global__ __launch_bounds__(FAST_THREADS) void front_fast_kernel(FrontParams p) {
    front_fast_body<VDT, NCH, false>(p);
}
template <int VDT, int NCH>
__global__ __launch_bounds__(FAST_THREADS) void front_fast_kernel_wide(FrontParams p) {
    front_fast_body<VDT, NCH, false, true>(p);
}
// The same for large batches: at most 128 registers, so that two workgroups share a CU (a batch of thousands of tokens
// is bound by how many of these latency chains run at once, a decode batch by the length of one).
template <int VDT, int NCH>
__global__ __launch_bounds__(FAST_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void front_fast_kernel_dense(FrontParams p) {
    front_fast_body<VDT, NCH, true>(p);   // layers without the pre-norm only
}

// RmsNorm::forward as a kernel of its own (candle-nn/src/ops.rs:504-515; the `(attn + residual)` that precedes the
// ffn_norm at quantized_llama.rs:884-888 folded in when `residual` is given): one workgroup per row.
template <int NCH>
__global__ __launch_bounds__(FAST_THREADS) void rms_norm_fast_kernel(const float* x, const float* residual, const float* alpha, float eps,
                                                                     float* sum, float* y, int serial) {
    constexpr int H = NCH * 256;
    __shared__ float row_lds[64 * (NCH * 4 + 1)];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t t = blockIdx.x;
    float xr[NCH * 4];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        float4 v = *reinterpret_cast<const float4*>(x + t * H + i * 256 + lane * 4);
        if (residual) {
            const float4 r = *reinterpret_cast<const float4*>(residual + t * H + i * 256 + lane * 4);
            v.x = v.x + r.x; v.y = v.y + r.y; v.z = v.z + r.z; v.w = v.w + r.w;
            if ((i & 7) == wave) *reinterpret_cast<float4*>(sum + t * H + i * 256 + lane * 4) = v;
        }
        xr[4 * i] = v.x; xr[4 * i + 1] = v.y; xr[4 * i + 2] = v.z; xr[4 * i + 3] = v.w;
    }
    const float sum2 = ordered_sum_of_squares<NCH>(xr, tid, serial != 0, row_lds);
    const float m = sqrtf(sum2 / (float)H + eps);
#pragma unroll
    for (int i = 0; i < NCH; i++)
        if ((i & 7) == wave) {
            const float4 a = *reinterpret_cast<const float4*>(alpha + i * 256 + lane * 4);
            *reinterpret_cast<float4*>(y + t * H + i * 256 + lane * 4) =
                make_float4(xr[4 * i] / m * a.x, xr[4 * i + 1] / m * a.y, xr[4 * i + 2] / m * a.z, xr[4 * i + 3] / m * a.w);
        }
}

// any other row length: the row in LDS, one thread adds the squares
__global__ __launch_bounds__(FRONT_THREADS) void rms_norm_generic_kernel(const float* x, const float* residual, const float* alpha, float eps,
                                                                         float* sum, float* y, int H) {
    extern __shared__ float xrow[];
    __shared__ float mval;
    const int tid = threadIdx.x;
    const int64_t t = blockIdx.x;
    for (int h = tid; h < H; h += FRONT_THREADS) {
        float v = x[t * H + h];
        if (residual) {
            v = v + residual[t * H + h];
            sum[t * H + h] = v;
        }
        xrow[h] = v;
    }
    __syncthreads();
    if (tid == 0) {
        float tot = 0.f;
        for (int h = 0; h < H; h++) tot += xrow[h] * xrow[h];
        mval = sqrtf(tot / (float)H + eps);
    }
    __syncthreads();
    const float m = mval;
    for (int h = tid; h < H; h += FRONT_THREADS) y[t * H + h] = xrow[h] / m * alpha[h];
}

__global__ __launch_bounds__(256) void fill_or_copy_kernel(const float* src, float* y, int64_t n4) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    reinterpret_cast<float4*>(y)[i] = src ? reinterpret_cast<const float4*>(src)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
}

__global__ __launch_bounds__(FRONT_THREADS) void route_from_logits_kernel(const float* logits, int64_t T, int E, int k,
                                                                         int norm_topk, RouteBufs rb) {
    __shared__ float probs[FRONT_THREADS / 64][MAX_E];
    __shared__ int sel_lds[FRONT_THREADS / 64][MAX_K];
    __shared__ __align__(16) long long order_lds[FRONT_THREADS / 64][MAX_E];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // one wave per token (4 tokens per workgroup)
    int64_t t = (int64_t)blockIdx.x * (FRONT_THREADS / 64) + wave;
    if (t < T) {
        for (int e = lane; e < E; e += 64) {
            float v = logits[t * E + e];
            probs[wave][e] = v;
            rb.logits[t * E + e] = v;
        }
    }
    __syncthreads();
    if (E <= 64) {
        if (t < T) route_one_token_wave(lane < E ? probs[wave][lane] : 0.f, lane, E, k, norm_topk, rb.topk_idx + t * k, rb.topk_w + t * k);
    } else if (t < T) {
        route_one_token_wave_lds(probs[wave], lane, E, k, norm_topk, rb.topk_idx + t * k, rb.topk_w + t * k, sel_lds[wave], order_lds[wave]);
    }
}

__global__ __launch_bounds__(DISPATCH_THREADS) void dispatch_kernel(RouteBufs rb, int64_t T, int E, int k, int shared, int pass) {
    __shared__ DispatchShared dsh;
    dispatch_block(rb, T, E, k, shared != 0, dsh, (int)blockIdx.x, (int)gridDim.x, pass);
}

__global__ void identity_routing_kernel(RouteBufs rb, int64_t rows) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i == 0) { rb.offsets[0] = 0; rb.offsets[1] = (int)rows; }
    if (i < rows) { rb.perm_token[i] = (int)i; rb.perm_w[i] = 1.0f; rb.tok_slots[i] = (int)i; }
    if (rb.tile_tab) {  // work list of the tiled kernels: one group cut into tiles of tile_slots rows
        const int64_t n_tiles = (rows + rb.tile_slots - 1) / rb.tile_slots;
        if (i == 0) rb.tile_tab[0] = (int)n_tiles;
        if (i < n_tiles) { rb.tile_tab[1 + 2 * i] = 0; rb.tile_tab[2 + 2 * i] = (int)(i * rb.tile_slots); }
    }
}

// y[t, :] = sum_j yw[slot_j, :] in ascending expert order (shared expert last), starting from
// zero as `zeros_like` does, each term already rounded (broadcast_mul happens before index_add in
// the reference).
__global__ __launch_bounds__(256) void combine_kernel(const float* yw, RouteBufs rb, int shared, const float* residual,
                                                      float* y, int64_t T, int H) {
    const int64_t t = blockIdx.x;
    const int k = rb.k;
    const int n = k + (shared ? 1 : 0);
    // the token's slots in the order of the sum: one wave ranks the selected experts (they are distinct) ...
    __shared__ int slots[MAX_K + 1];
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        if (rb.direct) {
            const int e = lane < k ? rb.topk_idx[t * k + lane] : 0x7fffffff;
            int rank = 0;
            for (int j = 0; j < k; j++) {
                const int ej = __shfl(e, j, 64);
                rank += (ej < e || (ej == e && j < lane)) ? 1 : 0;
            }
            if (lane < k) slots[rank] = (int)(t * k + lane);
            if (shared && lane == 0) slots[k] = (int)(T * k + t);
        } else if (lane < n) {   // ... or the dispatch pass has
            slots[lane] = rb.tok_slots[t * n + lane];
        }
    }
    __syncthreads();
    // a workgroup walks the token's row in steps of 1024 floats, two steps' loads in flight
    const int h0 = (blockIdx.y * 256 + threadIdx.x) * 4, hstep = gridDim.y * 1024;
    for (int h = h0; h < H; h += 2 * hstep) {
        const int h2 = h + hstep;
        const bool two = h2 < H;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f), acc2 = acc;
        if (n == 2) {   // the common case: both terms of both steps requested before the first add
            const int s0 = slots[0], s1 = slots[1];
            const float4 a0 = *reinterpret_cast<const float4*>(yw + (int64_t)s0 * H + h);
            const float4 a1 = *reinterpret_cast<const float4*>(yw + (int64_t)s1 * H + h);
            float4 b0 = acc, b1 = acc;
            if (two) {
                b0 = *reinterpret_cast<const float4*>(yw + (int64_t)s0 * H + h2);
                b1 = *reinterpret_cast<const float4*>(yw + (int64_t)s1 * H + h2);
            }
            acc.x += a0.x; acc.y += a0.y; acc.z += a0.z; acc.w += a0.w;
            acc.x += a1.x; acc.y += a1.y; acc.z += a1.z; acc.w += a1.w;
            acc2.x += b0.x; acc2.y += b0.y; acc2.z += b0.z; acc2.w += b0.w;
            acc2.x += b1.x; acc2.y += b1.y; acc2.z += b1.z; acc2.w += b1.w;
        } else {
            // four terms requested at a time, added in order
            for (int j0 = 0; j0 < n; j0 += 4) {
                float4 v[4], u[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int sl = slots[j0 + i < n ? j0 + i : n - 1];
                    v[i] = *reinterpret_cast<const float4*>(yw + (int64_t)sl * H + h);
                    if (two) u[i] = *reinterpret_cast<const float4*>(yw + (int64_t)sl * H + h2);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    if (j0 + i < n) {   // uniform
                        acc.x += v[i].x; acc.y += v[i].y; acc.z += v[i].z; acc.w += v[i].w;
                        if (two) { acc2.x += u[i].x; acc2.y += u[i].y; acc2.z += u[i].z; acc2.w += u[i].w; }
                    }
                }
            }
        }
        if (residual) {
            const float4 r = *reinterpret_cast<const float4*>(residual + t * H + h);
            acc.x += r.x; acc.y += r.y; acc.z += r.z; acc.w += r.w;
            if (two) {
                const float4 r2 = *reinterpret_cast<const float4*>(residual + t * H + h2);
                acc2.x += r2.x; acc2.y += r2.y; acc2.z += r2.z; acc2.w += r2.w;
            }
        }
        *reinterpret_cast<float4*>(y + t * H + h) = acc;
        if (two) *reinterpret_cast<float4*>(y + t * H + h2) = acc2;
    }
}

// ---------------------------------------------------------------------------------------------
// The front end in two launches, for layers with dozens of experts and for large batches (no pre-norm): the gate product
// of all tokens as an f32 matrix product on the matrix cores, then routing and quantisation per token.  One workgroup per
// token computing its own E products reads the whole gate (a megabyte at 128 experts of 2048) through one CU.
//
// logits[t, e] = x[t, :] . gate[e, :] (+ bias[e]); row E of the product is the always-on expert's gate, whose sigmoid goes
// to shared_w[t].  A workgroup owns 16 tokens x NB * 16 gate rows; its four waves split K and add their parts in wave
// order (v_mfma_f32_16x16x4_f32: lane l holds A[l % 16][l / 16], B[l / 16][l % 16] and D[4 (l / 16) + r][l % 16]).
typedef float v4f_front __attribute__((ext_vector_type(4)));
template <int NB>
__global__ __launch_bounds__(256) void gate_logits_kernel(FrontParams p) {
    __shared__ float part[4][NB][4][64];
    const int tid = threadIdx.x, lane = tid & 63, m = lane & 15, kq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int H = p.H, E = p.E;
    const int NE = E + (p.shared_gate ? 1 : 0);
    const int64_t t0 = (int64_t)blockIdx.x * 16;
    const int e0 = blockIdx.y * (NB * 16);
    const int64_t trow = t0 + m < p.T ? t0 + m : p.T - 1;
    const int kw = (H / 64) * 16;   // K of a wave: a multiple of 64
    // a batch is 16 * DEPTH consecutive k: lane group kq takes 4 * DEPTH consecutive ones of them (whole cache lines per
    // row and batch; which k a lane group multiplies only permutes the sum), DEPTH loads of four
    constexpr int DEPTH = NB == 1 ? 4 : 2;
    const float* xp = p.x + trow * H + wave * kw + 4 * DEPTH * kq;
    const float* gp[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        int e = e0 + nb * 16 + m;
        e = e < NE ? e : NE - 1;   // rows past the last are computed and dropped
        gp[nb] = (e < E ? p.gate + (int64_t)e * H : p.shared_gate) + wave * kw + 4 * DEPTH * kq;
    }
    v4f_front acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) acc[nb] = v4f_front{0.f, 0.f, 0.f, 0.f};
    // a batch is requested ahead of the one being multiplied
    float4 xa[DEPTH], ga[DEPTH][NB];
    auto request = [&](int kc, float4 (&xo)[DEPTH], float4 (&go)[DEPTH][NB]) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            xo[d] = *reinterpret_cast<const float4*>(xp + kc + 4 * d);
#pragma unroll
            for (int nb = 0; nb < NB; nb++) go[d][nb] = *reinterpret_cast<const float4*>(gp[nb] + kc + 4 * d);
        }
    };
    request(0, xa, ga);
    for (int kc = 0; kc < kw; kc += 16 * DEPTH) {
        float4 xn[DEPTH], gn[DEPTH][NB];
        request(kc + 16 * DEPTH < kw ? kc + 16 * DEPTH : kc, xn, gn);
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            const float xs[4] = {xa[d].x, xa[d].y, xa[d].z, xa[d].w};
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                const float gs[4] = {ga[d][nb].x, ga[d][nb].y, ga[d][nb].z, ga[d][nb].w};
#pragma unroll
                for (int j = 0; j < 4; j++) acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xs[j], gs[j], acc[nb], 0, 0, 0);
            }
        }
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            xa[d] = xn[d];
#pragma unroll
            for (int nb = 0; nb < NB; nb++) ga[d][nb] = gn[d][nb];
        }
    }
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int r = 0; r < 4; r++) part[wave][nb][r][lane] = acc[nb][r];
    __syncthreads();
    for (int v = wave; v < NB * 4; v += 4) {
        const int nb = v >> 2, r = v & 3;
        float sum = part[0][nb][r][lane];
        sum += part[1][nb][r][lane];
        sum += part[2][nb][r][lane];
        sum += part[3][nb][r][lane];
        const int64_t t = t0 + 4 * kq + r;
        const int e = e0 + nb * 16 + m;
        if (t < p.T && e < NE) {
            if (e < E) p.rb.logits[t * E + e] = p.gate_bias ? sum + p.gate_bias[e] : sum;
            else p.rb.shared_w[t] = 1.0f / (expf_glibc(-sum) + 1.0f);
        }
    }
}

// Routing and quantisation of one token whose logits are in memory: wave 0 routes, waves 1 to 3 quantise the row.
template <int VDT>
__global__ __launch_bounds__(256) void front_route_kernel(FrontParams p) {
    __shared__ float logit_lds[MAX_E];
    __shared__ int sel_lds[MAX_K];
    __shared__ __align__(16) long long order_lds[MAX_E];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t t = blockIdx.x;
    const int H = p.H, E = p.E, nch = H / 256;
    if (wave == 0) {
        if (E <= 64) {
            const float v = lane < E ? p.rb.logits[t * E + lane] : 0.f;
            route_one_token_wave(v, lane, E, p.k, p.norm_topk, p.rb.topk_idx + t * p.k, p.rb.topk_w + t * p.k);
        } else {
            for (int e = lane; e < E; e += 64) logit_lds[e] = p.rb.logits[t * E + e];
            __builtin_amdgcn_wave_barrier();
            route_one_token_wave_lds(logit_lds, lane, E, p.k, p.norm_topk, p.rb.topk_idx + t * p.k, p.rb.topk_w + t * p.k, sel_lds, order_lds);
        }
    } else {
        // chunks wave - 1, wave + 2, ...: two of them side by side
        for (int i = wave - 1; i < nch; i += 6) {
            const int i2 = i + 3;
            const float4 a = *reinterpret_cast<const float4*>(p.x + t * H + i * 256 + lane * 4);
            float4 b = a;
            if (i2 < nch) b = *reinterpret_cast<const float4*>(p.x + t * H + i2 * 256 + lane * 4);
            const float ea[4] = {a.x, a.y, a.z, a.w}, eb[4] = {b.x, b.y, b.z, b.w};
            quantize_chunk<VDT>(p, t, H, i, ea, lane);
            if (i2 < nch) quantize_chunk<VDT>(p, t, H, i2, eb, lane);
        }
    }
    if (p.y_zero)
        for (int i = tid; i < H / 4; i += 256) reinterpret_cast<float4*>(p.y_zero + t * H)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
}

// Logits of a quantised router: the dense product's [T, n_pad] rows cut to E columns, the optional bias added.
__global__ void logits_unpad_kernel(const float* padded, int n_pad, const float* bias, float* logits, int64_t T, int E) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= T * E) return;
    const int64_t t = i / E;
    const int e = (int)(i - t * E);
    const float v = padded[t * n_pad + e];
    logits[i] = bias ? v + bias[e] : v;
}
hipError_t launch_logits_unpad(const float* padded, int n_pad, const float* bias, float* logits, int64_t T, int E, hipStream_t s) {
    if (T == 0) return hipSuccess;
    hipLaunchKernelGGL(logits_unpad_kernel, dim3((unsigned)((T * E + 255) / 256)), dim3(256), 0, s, padded, n_pad, bias, logits, T, E);
    return hipGetLastError();
}
// Routing and activation quantisation from logits that are already in p.rb.logits (no gate product, no pre-norm: p.x is
// the row the experts see).
hipError_t launch_front_route(const FrontParams& p, hipStream_t s) {
    if (p.T == 0) return hipSuccess;
    if (p.H % 256 || p.E > MAX_E) return hipErrorInvalidValue;
    if (p.vdt == MOE_GGML_Q8K) hipLaunchKernelGGL(front_route_kernel<MOE_GGML_Q8K>, dim3((unsigned)p.T), dim3(256), 0, s, p);
    else hipLaunchKernelGGL(front_route_kernel<MOE_GGML_Q8_0>, dim3((unsigned)p.T), dim3(256), 0, s, p);
    return hipGetLastError();
}

static bool launch_front_split(const FrontParams& p, hipStream_t s) {
    const int sw = switches().front_split;
    const int NE = p.E + (p.shared_gate ? 1 : 0);
    if (sw == 0 || p.rms_alpha || p.H % 256 || p.E > MAX_E) return false;
    // (measured, front stage fused / split: 128 experts of 2048: 25 / 17 us at 512 tokens, 179 / 57 at 4096; 64 experts and
    // the always-on gate: 18 / 18 at 512, 118 / 51 at 4096; 60 experts and that gate: 19 / 21 at 512, 112 / 42 at 4096; 8 experts
    // of 4096: 54 / 46 at 4096, 5 / 18 at 32: the product kernel takes 2 us + 3.3 us per 1024 of H whatever its grid)
    if (sw < 0 && !(NE >= 32 && p.T * (int64_t)NE >= 49152)) return false;
    const unsigned tiles = (unsigned)((p.T + 15) / 16);
    // four blocks of gate rows per workgroup when that still leaves a workgroup per CU
    if (NE > 16 && (int64_t)tiles * ((NE + 63) / 64) >= 256) hipLaunchKernelGGL(gate_logits_kernel<4>, dim3(tiles, (unsigned)((NE + 63) / 64)), dim3(256), 0, s, p);
    else hipLaunchKernelGGL(gate_logits_kernel<1>, dim3(tiles, (unsigned)((NE + 15) / 16)), dim3(256), 0, s, p);
    if (p.vdt == MOE_GGML_Q8K) hipLaunchKernelGGL(front_route_kernel<MOE_GGML_Q8K>, dim3((unsigned)p.T), dim3(256), 0, s, p);
    else hipLaunchKernelGGL(front_route_kernel<MOE_GGML_Q8_0>, dim3((unsigned)p.T), dim3(256), 0, s, p);
    return true;
}

// ---------------------------------------------------------------------------------------------
template <int VDT>
static bool launch_front_fast(const FrontParams& p, hipStream_t s) {
    if (p.E > MAX_E || p.H % 256) return false;
    dim3 grid((unsigned)p.T), block(FAST_THREADS);
    switch (p.H / 256) {
        case 1: hipLaunchKernelGGL((front_fast_kernel<VDT, 1>), grid, block, 0, s, p); return true;
        case 2: hipLaunchKernelGGL((front_fast_kernel<VDT, 2>), grid, block, 0, s, p); return true;
        case 4: hipLaunchKernelGGL((front_fast_kernel<VDT, 4>), grid, block, 0, s, p); return true;
        case 8:
            if (p.T >= 256 && !p.rms_alpha) hipLaunchKernelGGL((front_fast_kernel_dense<VDT, 8>), grid, block, 0, s, p);
            else if (p.E > 32) hipLaunchKernelGGL((front_fast_kernel_wide<VDT, 8>), grid, block, 0, s, p);
            else hipLaunchKernelGGL((front_fast_kernel<VDT, 8>), grid, block, 0, s, p);
            return true;
        case 12: hipLaunchKernelGGL((front_fast_kernel<VDT, 12>), grid, block, 0, s, p); return true;
        case 16:
            if (p.T >= 1024 && !p.rms_alpha) hipLaunchKernelGGL((front_fast_kernel_dense<VDT, 16>), grid, block, 0, s, p);
            else if (p.E > 32) hipLaunchKernelGGL((front_fast_kernel_wide<VDT, 16>), grid, block, 0, s, p);
            else hipLaunchKernelGGL((front_fast_kernel<VDT, 16>), grid, block, 0, s, p);
            return true;
        case 20: hipLaunchKernelGGL((front_fast_kernel<VDT, 20>), grid, block, 0, s, p); return true;
        case 24: hipLaunchKernelGGL((front_fast_kernel<VDT, 24>), grid, block, 0, s, p); return true;
        case 28: hipLaunchKernelGGL((front_fast_kernel<VDT, 28>), grid, block, 0, s, p); return true;
        case 32: hipLaunchKernelGGL((front_fast_kernel<VDT, 32>), grid, block, 0, s, p); return true;
    }
    return false;
}

// The fast kernel in its plain or wide form (not the two-launch front end, not the lean form of large batches without a
// pre-norm, not the generic kernel): the one that can fold the previous layer's combine pass in.
bool front_takes_prev_combine(const FrontParams& p) {
    if (switches().front_generic || p.E > MAX_E || p.H % 256 || p.T == 0) return false;
    const int nch = p.H / 256;
    if (!(nch == 1 || nch == 2 || (nch % 4 == 0 && nch <= 32))) return false;
    const int sw = switches().front_split;
    const int NE = p.E + (p.shared_gate ? 1 : 0);
    if (!p.rms_alpha && sw != 0 && (sw > 0 || (NE >= 32 && p.T * (int64_t)NE >= 49152))) return false;   // two launches
    if (!p.rms_alpha && ((nch == 8 && p.T >= 256) || (nch == 16 && p.T >= 1024))) return false;              // lean form
    return true;
}

hipError_t launch_fill_or_copy(const float* src, float* y, int64_t n, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    const int64_t n4 = n / 4;
    hipLaunchKernelGGL(fill_or_copy_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, s, src, y, n4);
    return hipGetLastError();
}

hipError_t launch_add_rms_norm(const float* x, const float* residual, const float* alpha, float eps, int64_t rows, int hidden,
                               float* sum, float* y, hipStream_t s) {
    if (rows == 0) return hipSuccess;
    const int serial = switches().rms_serial;
    dim3 grid((unsigned)rows), block(FAST_THREADS);
#define MOE_RMS_CASE(N) case N: hipLaunchKernelGGL((rms_norm_fast_kernel<N>), grid, block, 0, s, x, residual, alpha, eps, sum, y, serial); return hipGetLastError();
    if (hidden % 256 == 0 && !switches().front_generic) switch (hidden / 256) {
        MOE_RMS_CASE(1) MOE_RMS_CASE(2) MOE_RMS_CASE(4) MOE_RMS_CASE(8) MOE_RMS_CASE(12) MOE_RMS_CASE(16)
        MOE_RMS_CASE(20) MOE_RMS_CASE(24) MOE_RMS_CASE(28) MOE_RMS_CASE(32)
    }
#undef MOE_RMS_CASE
    if ((size_t)hidden * 4 > 64 * 1024 - 512) return hipErrorInvalidValue;
    hipLaunchKernelGGL(rms_norm_generic_kernel, grid, dim3(FRONT_THREADS), (size_t)hidden * sizeof(float), s, x, residual, alpha, eps, sum, y, hidden);
    return hipGetLastError();
}

hipError_t launch_front(const FrontParams& p_in, hipStream_t s) {
    if (p_in.T == 0) return hipSuccess;
    const FrontParams& p = p_in;
    const bool no_fast = switches().front_generic != 0;
    const bool q8k = p.vdt == MOE_GGML_Q8K;
    if (!no_fast && launch_front_split(p, s)) return hipGetLastError();
    if (!no_fast && (q8k ? launch_front_fast<MOE_GGML_Q8K>(p, s) : launch_front_fast<MOE_GGML_Q8_0>(p, s))) return hipGetLastError();
    size_t lds = (size_t)p.H * sizeof(float);
    if (q8k)
        hipLaunchKernelGGL(front_kernel<MOE_GGML_Q8K>, dim3((unsigned)p.T), dim3(FRONT_THREADS), lds, s, p);
    else
        hipLaunchKernelGGL(front_kernel<MOE_GGML_Q8_0>, dim3((unsigned)p.T), dim3(FRONT_THREADS), lds, s, p);
    return hipGetLastError();
}

hipError_t launch_route_from_logits(const float* logits, int64_t T, int E, int k, int norm_topk,
                                    const RouteBufs& rb, hipStream_t s) {
    if (T == 0) return hipSuccess;
    unsigned blocks = (unsigned)((T + FRONT_THREADS / 64 - 1) / (FRONT_THREADS / 64));
    hipLaunchKernelGGL(route_from_logits_kernel, dim3(blocks), dim3(FRONT_THREADS), 0, s, logits, T, E, k, norm_topk, rb);
    return hipGetLastError();
}

hipError_t launch_identity_routing(const RouteBufs& rb, int64_t rows, hipStream_t s) {
    unsigned blocks = (unsigned)((rows + 255) / 256);
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(identity_routing_kernel, dim3(blocks), dim3(256), 0, s, rb, rows);
    return hipGetLastError();
}

hipError_t launch_dispatch(const RouteBufs& rb, int64_t T, int E, int k, bool shared, hipStream_t s) {
    if (T == 0) return hipSuccess;
    // one workgroup up to 16k assignments (8192: 13 us); beyond, a counting and a placing launch of a workgroup per 4096
    const int64_t A = T * k;
    const unsigned G = (unsigned)std::min<int64_t>(DISPATCH_MAX_WGS, (A + 4095) / 4096);
    if (A <= 16384 || !rb.wg_counts || switches().dispatch_one) {
        hipLaunchKernelGGL(dispatch_kernel, dim3(1), dim3(DISPATCH_THREADS), 0, s, rb, T, E, k, shared ? 1 : 0, 0);
    } else {
        hipLaunchKernelGGL(dispatch_kernel, dim3(G), dim3(DISPATCH_THREADS), 0, s, rb, T, E, k, shared ? 1 : 0, 1);
        hipLaunchKernelGGL(dispatch_kernel, dim3(G), dim3(DISPATCH_THREADS), 0, s, rb, T, E, k, shared ? 1 : 0, 2);
    }
    return hipGetLastError();
}

hipError_t launch_combine(const float* yw, const RouteBufs& rb, bool shared, const float* residual, float* y,
                          int64_t T, int H, hipStream_t s) {
    if (T == 0) return hipSuccess;
    // few tokens: one workgroup per 1024 floats of a row; many: one or two per row, each walking it
    const unsigned per_row = (unsigned)((H / 4 + 255) / 256);
    const unsigned split = T >= 2048 ? 1u : T >= 512 ? std::min(per_row, 2u) : per_row;
    dim3 grid((unsigned)T, split);
    hipLaunchKernelGGL(combine_kernel, grid, dim3(256), 0, s, yw, rb, shared ? 1 : 0, residual, y, T, H);
    return hipGetLastError();
}

}  // namespace moe
