// Grouped expert products over Q4K weights with Q8K activations (gfx950, wave64, int8 MFMA).
//
// Arithmetic restated from BlockQ4K::vec_dot, candle-core/src/quantized/k_quants.rs:1205-1285:
// per 256-element super-block
//     d * y.d * sum_j sc_j * (q4_j . q8_j)  -  dmin * y.d * sum_j m_j * (bsum_2j + bsum_2j+1)
// The integer parts are exact: the 32-element dots come from v_mfma_i32_16x16x32_i8 (one
// sub-block per instruction), the 6-bit scales are applied in 32-bit integers, and the `mins`
// term is an exact f16 MFMA over the 16 block sums (|bsum| <= 2048, m <= 63, products summed in
// f32 stay below 2^24).  Only the f32 accumulation across super-blocks is ordered differently from
// the scalar reference.
//
// MFMA orientation: A = activations (M = 16 slots), B = weights (N = 16 rows), so lane l ends up
// with D[slot 4*(l/16)+i][row l%16]: one weight row per lane, hence one set of scales per lane.
//
//   q4k_up_kernel    h[slot, f] = silu(W1 x) * (W3 x) for a 256-row block of F, then the block is
//                    quantised to Q8K in the epilogue (Mlp::forward, quantized_llama.rs:124-131;
//                    the re-quantisation is what k_quants::matmul does to the lhs of w2).
//   q4k_down_kernel  yw[slot, :] = (W2 h[slot]) * routing weight (quantized_llama.rs:199-201).
#include "act_quant.hpp"
#include "kernels.hpp"

namespace moe {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

struct Q4KTile {
    uint4 q0, q1, sc;
};

__device__ inline Q4KTile load_q4k_tile(const uint8_t* tile, int lane) {
    Q4KTile t;
    t.q0 = *reinterpret_cast<const uint4*>(tile + lane * 16);
    t.q1 = *reinterpret_cast<const uint4*>(tile + 1024 + lane * 16);
    t.sc = *reinterpret_cast<const uint4*>(tile + 2048 + (lane & 15) * 16);
    return t;
}

// Activation operand of one 16-slot tile for one super-block.
struct Q8KOperand {
    uint4 a[4];   // pair P: sub-block 2P (x,y) and 2P+1 (z,w), this lane's 8-element chunk
    v4h bs;       // bsums 4g..4g+3 of the lane's slot (l%16)
    float yd[4];  // Q8K scale of the lane's four output slots (4g+i)
};

__device__ inline Q8KOperand load_q8k_operand(const ActBuf& ab, int K, int nsb, int sb, int rowA, const int rowD[4], int g) {
    Q8KOperand o;
    const int8_t* base = ab.qs + (int64_t)rowA * K + sb * 256 + g * 16;
#pragma unroll
    for (int P = 0; P < 4; P++) o.a[P] = *reinterpret_cast<const uint4*>(base + P * 64);
    o.bs = *reinterpret_cast<const v4h*>(reinterpret_cast<const __half*>(ab.bsum) + ((int64_t)rowA * nsb + sb) * 16 + 4 * g);
#pragma unroll
    for (int i = 0; i < 4; i++) o.yd[i] = ab.d[(int64_t)rowD[i] * nsb + sb];
    return o;
}

__device__ inline long pack64(uint32_t lo, uint32_t hi) { return (long)(((uint64_t)hi << 32) | lo); }

// acc[i] += contribution of one (16 rows x 256 k) weight tile against one 16-slot operand.
__device__ inline void q4k_mac(const Q4KTile& w, const Q8KOperand& A, int g, float acc[4]) {
    const uint32_t M4 = 0x0f0f0f0fu;
    const uint32_t hdr = w.sc.x, u0 = w.sc.y, u1 = w.sc.z, u2 = w.sc.w;
    const float d = __half2float(__ushort_as_half((unsigned short)(hdr & 0xffffu)));
    const float dmin = __half2float(__ushort_as_half((unsigned short)(hdr >> 16)));
    // get_scale_min_k4 (utils.rs:50-60) for all eight sub-blocks at once
    const uint32_t sc03 = u0 & 0x3f3f3f3fu;
    const uint32_t sc47 = (u2 & M4) | (((u0 >> 6) & 0x03030303u) << 4);
    const uint32_t m03 = u1 & 0x3f3f3f3fu;
    const uint32_t m47 = ((u2 >> 4) & M4) | (((u1 >> 6) & 0x03030303u) << 4);
    const v4i zero = {0, 0, 0, 0};
    v4i isum = {0, 0, 0, 0};
    const uint32_t qw[8] = {w.q0.x, w.q0.y, w.q0.z, w.q0.w, w.q1.x, w.q1.y, w.q1.z, w.q1.w};
#pragma unroll
    for (int P = 0; P < 4; P++) {
        const uint32_t wx = qw[2 * P], wy = qw[2 * P + 1];
        const long b_lo = pack64(wx & M4, wy & M4);
        const long b_hi = pack64((wx >> 4) & M4, (wy >> 4) & M4);
        const long a_lo = pack64(A.a[P].x, A.a[P].y);
        const long a_hi = pack64(A.a[P].z, A.a[P].w);
        v4i D0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_lo, b_lo, zero, 0, 0, 0);
        v4i D1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_hi, b_hi, zero, 0, 0, 0);
        const uint32_t scw = (P < 2) ? sc03 : sc47;
        const int s0 = (int)((scw >> (16 * (P & 1))) & 0xffu);
        const int s1 = (int)((scw >> (16 * (P & 1) + 8)) & 0xffu);
#pragma unroll
        for (int i = 0; i < 4; i++) isum[i] += __mul24(s0, D0[i]) + __mul24(s1, D1[i]);
    }
    // mins term: sum_k bsum16[slot][k] * m[row][k/2], k = 0..15, as an exact f16 MFMA; this lane
    // supplies k = 4g..4g+3, i.e. sub-blocks 2g and 2g+1
    const uint32_t mw = (g < 2) ? m03 : m47;
    const _Float16 ma = (_Float16)(int)((mw >> (16 * (g & 1))) & 0xffu);
    const _Float16 mb = (_Float16)(int)((mw >> (16 * (g & 1) + 8)) & 0xffu);
    const v4h mB = {ma, ma, mb, mb};
    const v4f zf = {0.f, 0.f, 0.f, 0.f};
    v4f Dm = __builtin_amdgcn_mfma_f32_16x16x16f16(A.bs, mB, zf, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float dd = d * A.yd[i];
        const float dm = dmin * A.yd[i];
        acc[i] += dd * (float)isum[i];
        acc[i] -= dm * Dm[i];
    }
}

__device__ inline float silu_ref(float v) { return v / (1.0f + expf_glibc(-v)); }  // op.rs:646-648

// ---------------------------------------------------------------------------------------------
constexpr int UP_THREADS = 512;
constexpr int UP_ROWS = 256;     // rows of F per workgroup = one Q8K block of h per slot
constexpr int HBUF_STRIDE = 260;

template <int TT>
__global__ __launch_bounds__(UP_THREADS) void q4k_up_kernel(ExpertParams p) {
    __shared__ float hbuf[TT * 16][HBUF_STRIDE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, g = lane >> 4;
    const int grp = blockIdx.y;
    const int s_begin = p.rb.offsets[p.group0 + grp], s_end = p.rb.offsets[p.group0 + grp + 1];
    const int tg0 = blockIdx.z * (TT * 16);
    if (s_begin + tg0 >= s_end) return;
    const int H = p.H, F = p.F, nsb = H / 256;
    const int rb = blockIdx.x;

    int rowA[TT], rowD[TT][4];
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        int s = s_begin + tg0 + tt * 16 + r;
        rowA[tt] = p.rb.perm_token[s < s_end ? s : s_end - 1];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int sd = s_begin + tg0 + tt * 16 + 4 * g + i;
            rowD[tt][i] = p.rb.perm_token[sd < s_end ? sd : s_end - 1];
        }
    }
    const GroupWeights gw = p.groups[grp];
    const int rt0 = rb * (UP_ROWS / 16) + wave * 2;
    const uint8_t* tp[4] = {gw.w1 + (size_t)rt0 * nsb * Q4K_TILE_BYTES, gw.w1 + (size_t)(rt0 + 1) * nsb * Q4K_TILE_BYTES,
                            gw.w3 + (size_t)rt0 * nsb * Q4K_TILE_BYTES, gw.w3 + (size_t)(rt0 + 1) * nsb * Q4K_TILE_BYTES};
    float acc[4][TT][4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int tt = 0; tt < TT; tt++)
#pragma unroll
            for (int i = 0; i < 4; i++) acc[j][tt][i] = 0.f;

    Q4KTile cur[4], nxt[4];
    Q8KOperand Acur[TT], Anxt[TT];
#pragma unroll
    for (int j = 0; j < 4; j++) cur[j] = load_q4k_tile(tp[j], lane);
#pragma unroll
    for (int tt = 0; tt < TT; tt++) Acur[tt] = load_q8k_operand(p.xq, H, nsb, 0, rowA[tt], rowD[tt], g);

    for (int sb = 0; sb < nsb; sb++) {
        if (sb + 1 < nsb) {
#pragma unroll
            for (int j = 0; j < 4; j++) nxt[j] = load_q4k_tile(tp[j] + (size_t)(sb + 1) * Q4K_TILE_BYTES, lane);
#pragma unroll
            for (int tt = 0; tt < TT; tt++) Anxt[tt] = load_q8k_operand(p.xq, H, nsb, sb + 1, rowA[tt], rowD[tt], g);
        }
#pragma unroll
        for (int tt = 0; tt < TT; tt++)
#pragma unroll
            for (int j = 0; j < 4; j++) q4k_mac(cur[j], Acur[tt], g, acc[j][tt]);
#pragma unroll
        for (int j = 0; j < 4; j++) cur[j] = nxt[j];
#pragma unroll
        for (int tt = 0; tt < TT; tt++) Acur[tt] = Anxt[tt];
    }

    // epilogue: h = silu(w1 x) * (w3 x), then Q8K-quantise the 256-row block of every slot
#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                hbuf[tt * 16 + 4 * g + i][wave * 32 + j * 16 + r] = silu_ref(acc[j][tt][i]) * acc[2 + j][tt][i];
    __syncthreads();
    const int nfb = F / 256;
    for (int tok = wave; tok < TT * 16; tok += UP_THREADS / 64) {
        int slot = s_begin + tg0 + tok;
        if (slot >= s_end) break;
        float4 v = *reinterpret_cast<const float4*>(&hbuf[tok][lane * 4]);
        int64_t hrow = slot - p.slot_origin;
        quantize_q8k_block(v, lane, p.hq.qs + hrow * F + rb * 256, p.hq.d + hrow * nfb + rb,
                           reinterpret_cast<__half*>(p.hq.bsum) + (hrow * nfb + rb) * 16);
    }
}

// ---------------------------------------------------------------------------------------------
constexpr int DOWN_THREADS = 256;
constexpr int DOWN_STEP = 4;  // super-blocks in flight per wave

template <int TT>
__global__ __launch_bounds__(DOWN_THREADS) void q4k_down_kernel(ExpertParams p) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, g = lane >> 4;
    const int grp = blockIdx.y;
    const int s_begin = p.rb.offsets[p.group0 + grp], s_end = p.rb.offsets[p.group0 + grp + 1];
    const int tg0 = blockIdx.z * (TT * 16);
    if (s_begin + tg0 >= s_end) return;
    const int H = p.H, F = p.F, nsb = F / 256;
    const int rt = blockIdx.x * (DOWN_THREADS / 64) + wave;
    if (rt >= H / 16) return;

    int rowA[TT], rowD[TT][4];
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        int s = s_begin + tg0 + tt * 16 + r;
        rowA[tt] = (s < s_end ? s : s_end - 1) - p.slot_origin;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int sd = s_begin + tg0 + tt * 16 + 4 * g + i;
            rowD[tt][i] = (sd < s_end ? sd : s_end - 1) - p.slot_origin;
        }
    }
    const uint8_t* tp = p.groups[grp].w2 + (size_t)rt * nsb * Q4K_TILE_BYTES;
    float acc[TT][4];
#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[tt][i] = 0.f;

    Q4KTile cur[DOWN_STEP], nxt[DOWN_STEP];
#pragma unroll
    for (int j = 0; j < DOWN_STEP; j++)
        if (j < nsb) cur[j] = load_q4k_tile(tp + (size_t)j * Q4K_TILE_BYTES, lane);

    for (int sb0 = 0; sb0 < nsb; sb0 += DOWN_STEP) {
#pragma unroll
        for (int j = 0; j < DOWN_STEP; j++)
            if (sb0 + DOWN_STEP + j < nsb) nxt[j] = load_q4k_tile(tp + (size_t)(sb0 + DOWN_STEP + j) * Q4K_TILE_BYTES, lane);
#pragma unroll
        for (int j = 0; j < DOWN_STEP; j++) {
            if (sb0 + j < nsb) {
#pragma unroll
                for (int tt = 0; tt < TT; tt++) {
                    Q8KOperand A = load_q8k_operand(p.hq, F, nsb, sb0 + j, rowA[tt], rowD[tt], g);
                    q4k_mac(cur[j], A, g, acc[tt]);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < DOWN_STEP; j++) cur[j] = nxt[j];
    }

#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int slot = s_begin + tg0 + tt * 16 + 4 * g + i;
            if (slot < s_end) p.yw[(int64_t)slot * H + rt * 16 + r] = acc[tt][i] * p.rb.perm_w[slot];
        }
}

// ---------------------------------------------------------------------------------------------
static inline int pick_tt(const ExpertParams& p) { return p.slot_tiles >= 2 ? 2 : 1; }

hipError_t launch_q4k_up(const ExpertParams& p, hipStream_t s) {
    if (p.max_rows == 0 || p.n_groups == 0) return hipSuccess;
    const int tt = pick_tt(p);
    dim3 grid((unsigned)(p.F / UP_ROWS), (unsigned)p.n_groups, (unsigned)((p.max_rows + tt * 16 - 1) / (tt * 16)));
    if (tt == 1)
        hipLaunchKernelGGL(q4k_up_kernel<1>, grid, dim3(UP_THREADS), 0, s, p);
    else
        hipLaunchKernelGGL(q4k_up_kernel<2>, grid, dim3(UP_THREADS), 0, s, p);
    return hipGetLastError();
}

hipError_t launch_q4k_down(const ExpertParams& p, hipStream_t s) {
    if (p.max_rows == 0 || p.n_groups == 0) return hipSuccess;
    const int tt = pick_tt(p);
    const int wpb = DOWN_THREADS / 64;
    dim3 grid((unsigned)((p.H / 16 + wpb - 1) / wpb), (unsigned)p.n_groups, (unsigned)((p.max_rows + tt * 16 - 1) / (tt * 16)));
    if (tt == 1)
        hipLaunchKernelGGL(q4k_down_kernel<1>, grid, dim3(DOWN_THREADS), 0, s, p);
    else
        hipLaunchKernelGGL(q4k_down_kernel<2>, grid, dim3(DOWN_THREADS), 0, s, p);
    return hipGetLastError();
}

}  // namespace moe
