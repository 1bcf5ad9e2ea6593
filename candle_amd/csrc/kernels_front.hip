// Router, dispatch and combine kernels.
//
//   front_kernel            per token: optional rms-norm, gate product, softmax, top-k with
//                           renormalised weights, activation quantisation; the last workgroup to
//                           retire builds the per-expert token lists (histogram, prefix scan and a
//                           stable permutation from wavefront ballots).
//   route_from_logits       the same routing starting from given logits (parity hook).
//   combine_kernel          routing-weighted sum of the expert outputs back in token order.
//
// Reference semantics restated here:
//   softmax_last_dim  candle-nn/src/ops.rs:313-351  (max cpu/kernels.rs:40-45, sum cpu/mod.rs:132-151
//                     in the 4 x 8-lane accumulator order of cpu/avx.rs:54-68)
//   top-k + lists     candle-transformers/src/models/quantized_llama.rs:158-179
//   combine           quantized_llama.rs:200-202 (index_add in ascending expert order)
//   rms_norm          candle-nn/src/ops.rs:504-515;  sigmoid candle-nn/src/ops.rs:59-61
#include "act_quant.hpp"
#include "kernels.hpp"

namespace moe {

constexpr int FRONT_THREADS = 256;
constexpr int MAX_E = 256;
constexpr int MAX_K = 16;

__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
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
// Per-expert lists.  Runs in ONE workgroup of FRONT_THREADS threads.  Assignments are taken in
// (token, rank) order; within an expert the slots keep that order, i.e. ascending token index,
// exactly as the Vec pushes of the reference produce them.
struct DispatchShared {
    int cnt[FRONT_THREADS / 64][MAX_E];
    int off[MAX_E + 2];
};

__device__ inline int ld_i32(const int32_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ inline float ld_f32(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

__device__ void dispatch_block(const RouteBufs& rb, int64_t T, int E, int k, bool shared, DispatchShared& sh) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    constexpr int NW = FRONT_THREADS / 64;
    const int64_t A = T * k;
    const int64_t chunk = ((A + NW - 1) / NW + 63) / 64 * 64;
    const int64_t lo = wave * chunk, hi = (lo + chunk < A) ? lo + chunk : A;
    for (int i = tid; i < NW * MAX_E; i += FRONT_THREADS) (&sh.cnt[0][0])[i] = 0;
    __syncthreads();
    // phase 1: per-wave histogram from ballots
    for (int64_t base = lo; base < hi; base += 64) {
        int64_t a = base + lane;
        bool valid = a < hi;
        int e = valid ? ld_i32(rb.topk_idx + a) : -1;
        unsigned long long rem = __ballot(valid);
        while (rem) {
            int leader = __ffsll((long long)rem) - 1;
            int e0 = __shfl(e, leader, 64);
            unsigned long long m = __ballot(valid && e == e0);
            if (lane == leader) sh.cnt[wave][e0] += __popcll(m);
            rem &= ~m;
        }
    }
    __syncthreads();
    // phase 2: exclusive scan over experts, then per-wave bases
    if (tid == 0) {
        int run = 0;
        for (int e = 0; e < E; e++) {
            sh.off[e] = run;
            for (int w = 0; w < NW; w++) run += sh.cnt[w][e];
        }
        sh.off[E] = run;
        sh.off[E + 1] = run + (shared ? (int)T : 0);
    }
    __syncthreads();
    for (int e = tid; e < E; e += FRONT_THREADS) {
        int run = sh.off[e];
        for (int w = 0; w < NW; w++) {
            int c = sh.cnt[w][e];
            sh.cnt[w][e] = run;  // becomes the wave's running cursor
            run += c;
        }
    }
    for (int e = tid; e <= E + (shared ? 1 : 0); e += FRONT_THREADS) rb.offsets[e] = sh.off[e];
    __syncthreads();
    // phase 3: stable placement
    const int kk = k + (shared ? 1 : 0);
    for (int64_t base = lo; base < hi; base += 64) {
        int64_t a = base + lane;
        bool valid = a < hi;
        int e = valid ? ld_i32(rb.topk_idx + a) : -1;
        float w = valid ? ld_f32(rb.topk_w + a) : 0.f;
        unsigned long long rem = __ballot(valid);
        unsigned long long lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
        int slot = -1;
        while (rem) {
            int leader = __ffsll((long long)rem) - 1;
            int e0 = __shfl(e, leader, 64);
            unsigned long long m = __ballot(valid && e == e0);
            int cur = sh.cnt[wave][e0];
            if (valid && e == e0) slot = cur + __popcll(m & lt);
            // all lanes have read `cur` before the leader updates it (same wave, program order)
            if (lane == leader) sh.cnt[wave][e0] = cur + __popcll(m);
            rem &= ~m;
        }
        if (valid) {
            int t = (int)(a / k);
            rb.perm_token[slot] = t;
            rb.perm_w[slot] = w;
            // stash (slot) per assignment in tok_slots, unsorted for now
            rb.tok_slots[(int64_t)t * kk + (int)(a % k)] = slot;
        }
    }
    __syncthreads();
    // phase 4: per token, order its slots by ascending expert index (combine order); append shared
    for (int64_t t = tid; t < T; t += FRONT_THREADS) {
        int es[MAX_K], ss[MAX_K];
        for (int r = 0; r < k; r++) {
            es[r] = ld_i32(rb.topk_idx + t * k + r);
            ss[r] = ld_i32(rb.tok_slots + t * kk + r);
        }
        for (int i = 1; i < k; i++) {
            int ev = es[i], sv = ss[i], j = i - 1;
            while (j >= 0 && es[j] > ev) { es[j + 1] = es[j]; ss[j + 1] = ss[j]; j--; }
            es[j + 1] = ev; ss[j + 1] = sv;
        }
        for (int r = 0; r < k; r++) rb.tok_slots[t * kk + r] = ss[r];
        if (shared) {
            int slot = (int)(A + t);
            rb.tok_slots[t * kk + k] = slot;
            rb.perm_token[slot] = (int)t;
            rb.perm_w[slot] = ld_f32(rb.shared_w + t);
        }
    }
}

// Returns true in every thread of the last workgroup of the grid to get here.
__device__ inline bool last_block_done(uint32_t* counter, int* flag_lds) {
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned ticket = atomicAdd(counter, 1u);
        *flag_lds = (ticket == gridDim.x - 1);
    }
    __syncthreads();
    bool last = *flag_lds != 0;
    if (last) __threadfence();
    return last;
}

// ---------------------------------------------------------------------------------------------
template <int VDT>
__global__ __launch_bounds__(FRONT_THREADS) void front_kernel(FrontParams p) {
    extern __shared__ float xrow[];  // [H]
    __shared__ float probs[MAX_E];
    __shared__ float red[FRONT_THREADS / 64];
    __shared__ int last_flag;
    __shared__ DispatchShared dsh;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t t = blockIdx.x;
    const int H = p.H, E = p.E;
    const float* x = p.x + t * H;

    // ---- load the row (and normalise it if the layer carries the pre-norm)
    float sum2 = 0.f;
    for (int h = tid * 4; h < H; h += FRONT_THREADS * 4) {
        float4 v = *reinterpret_cast<const float4*>(x + h);
        *reinterpret_cast<float4*>(xrow + h) = v;
        sum2 += v.x * v.x;
        sum2 += v.y * v.y;
        sum2 += v.z * v.z;
        sum2 += v.w * v.w;
    }
    if (p.rms_alpha) {
        sum2 = wave_sum(sum2);
        if (lane == 0) red[wave] = sum2;
        __syncthreads();
        float tot = 0.f;
        for (int w = 0; w < FRONT_THREADS / 64; w++) tot += red[w];
        float m = sqrtf(tot / (float)H + p.rms_eps);
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

    // ---- one thread routes while the waves quantise the row
    if (tid == 0) route_one_token(probs, E, p.k, p.norm_topk, p.rb.topk_idx + t * p.k, p.rb.topk_w + t * p.k);

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
            quantize_q8_0_block(xrow[h], lane, p.xq.qs + t * H + h, p.xq.d + t * nb + b,
                                reinterpret_cast<int32_t*>(p.xq.bsum) + t * nb + b);
        }
    }

    // ---- the last workgroup builds the expert lists
    if (last_block_done(p.rb.counter, &last_flag)) {
        dispatch_block(p.rb, p.T, E, p.k, p.shared_gate != nullptr, dsh);
        if (tid == 0) *p.rb.counter = 0u;
    }
}

__global__ __launch_bounds__(FRONT_THREADS) void route_from_logits_kernel(const float* logits, int64_t T, int E, int k,
                                                                         int norm_topk, RouteBufs rb) {
    __shared__ float probs[FRONT_THREADS / 64][MAX_E];
    __shared__ int last_flag;
    __shared__ DispatchShared dsh;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // one wave per token (4 tokens per workgroup); lane 0 routes
    int64_t t = (int64_t)blockIdx.x * (FRONT_THREADS / 64) + wave;
    if (t < T) {
        for (int e = lane; e < E; e += 64) {
            float v = logits[t * E + e];
            probs[wave][e] = v;
            rb.logits[t * E + e] = v;
        }
    }
    __syncthreads();
    if (t < T && lane == 0) route_one_token(probs[wave], E, k, norm_topk, rb.topk_idx + t * k, rb.topk_w + t * k);
    if (last_block_done(rb.counter, &last_flag)) {
        dispatch_block(rb, T, E, k, false, dsh);
        if (tid == 0) *rb.counter = 0u;
    }
}

__global__ void identity_routing_kernel(RouteBufs rb, int64_t rows) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i == 0) { rb.offsets[0] = 0; rb.offsets[1] = (int)rows; }
    if (i < rows) { rb.perm_token[i] = (int)i; rb.perm_w[i] = 1.0f; rb.tok_slots[i] = (int)i; }
}

// y[t, :] = sum_j yw[slot_j, :] in ascending expert order, starting from zero as `zeros_like`
// does, each term already rounded (broadcast_mul happens before index_add in the reference).
__global__ __launch_bounds__(256) void combine_kernel(const float* yw, const int32_t* tok_slots, int spt,
                                                      const float* residual, float* y, int64_t T, int H) {
    int64_t t = blockIdx.x;
    int h = (blockIdx.y * 256 + threadIdx.x) * 4;
    if (h >= H) return;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int j = 0; j < spt; j++) {
        int slot = tok_slots[t * spt + j];
        float4 v = *reinterpret_cast<const float4*>(yw + (int64_t)slot * H + h);
        acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
    }
    if (residual) {
        float4 r = *reinterpret_cast<const float4*>(residual + t * H + h);
        acc.x += r.x; acc.y += r.y; acc.z += r.z; acc.w += r.w;
    }
    *reinterpret_cast<float4*>(y + t * H + h) = acc;
}

// ---------------------------------------------------------------------------------------------
hipError_t launch_front(const FrontParams& p, hipStream_t s) {
    if (p.T == 0) return hipSuccess;
    size_t lds = (size_t)p.H * sizeof(float);
    if (p.vdt == MOE_GGML_Q8K)
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

hipError_t launch_combine(const float* yw, const int32_t* tok_slots, int spt, const float* residual, float* y,
                          int64_t T, int H, hipStream_t s) {
    if (T == 0) return hipSuccess;
    dim3 grid((unsigned)T, (unsigned)((H / 4 + 255) / 256));
    hipLaunchKernelGGL(combine_kernel, grid, dim3(256), 0, s, yw, tok_slots, spt, residual, y, T, H);
    return hipGetLastError();
}

}  // namespace moe
