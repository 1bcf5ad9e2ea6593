// Grouped expert products over the 32-element block formats (gfx950, int8 MFMA): Q4_0, Q5_0, Q8_0 weights
// with Q8_0 activations, Q4_1 and Q5_1 weights with Q8_1 activations.
//
// Arithmetic restated from candle-core/src/quantized/k_quants.rs:241-258 (Q4_0 . Q8_0), :381-402
// (Q5_0 . Q8_0) and :650-668 (Q8_0 . Q8_0): per 32-element block  sumf += (sum_i as f32) * d_w * d_x;
// :270-297 (Q4_1 . Q8_1) and :477-509 (Q5_1 . Q8_1): sumf += (sum_i as f32) * d_w * d_x + m_w * s_x.  One
// v_mfma_i32_16x16x32_i8 yields the exact integer dot of a block for 16 rows x 16 slots, and every
// lane adds its (row, slot) blocks in ascending block order with separately rounded products, so
// the f32 result is bit-identical to the scalar reference loop.
//
// Q4_0 stores nibble - 8 and Q5_0 code - 16; the kernel multiplies the raw codes (0..15, 0..31) and
// subtracts 8 or 16 times sum(q8) of the block, which is the same integer.  Q4_1 and Q5_1 codes are
// unsigned as stored.
#include <cstdlib>
#include "act_quant.hpp"
#include "kernels.hpp"
#include "slots.hpp"

namespace moe {

typedef int v4i __attribute__((ext_vector_type(4)));

// Placement of one format's 16-row tile (see moe_common.hpp) and what its block carries.
template <int DT>
struct Q32Fmt {
    static constexpr bool NIB = DT != MOE_GGML_Q8_0;                             // two codes per byte
    static constexpr bool FIFTH = DT == MOE_GGML_Q5_0 || DT == MOE_GGML_Q5_1;    // a fifth bit per code
    static constexpr bool HAS_M = DT == MOE_GGML_Q4_1 || DT == MOE_GGML_Q5_1;    // a block minimum (and Q8_1 activations)
    static constexpr int OFFSET = DT == MOE_GGML_Q4_0 ? 8 : DT == MOE_GGML_Q5_0 ? 16 : 0;  // stored code - value
    static constexpr int TB = DT == MOE_GGML_Q8_0 ? Q8_0_TILE_BYTES : DT == MOE_GGML_Q4_0 ? Q4_0_TILE_BYTES
                            : DT == MOE_GGML_Q4_1 ? Q4_1_TILE_BYTES : DT == MOE_GGML_Q5_0 ? Q5_0_TILE_BYTES : Q5_1_TILE_BYTES;
    static constexpr uint32_t H_OFF = 256;
    static constexpr uint32_t D_OFF = !NIB ? 512 : FIFTH ? 320 : 256;
    static constexpr uint32_t D_STRIDE = HAS_M ? 4 : 2;
    __device__ static uint32_t q_off(int lane) { return NIB ? (uint32_t)((lane & 15) * 16 + 8 * (lane >> 5)) : (uint32_t)lane * 8u; }
    __device__ static uint32_t d_off(int lane) { return D_OFF + D_STRIDE * (uint32_t)(lane & 15); }
    __device__ static uint32_t h_off(int lane) { return H_OFF + 4u * (uint32_t)(lane & 15); }
};

template <int DT>
struct Q32Tile {
    uint2 q;
    float d;
    float m;   // formats with a block minimum only
};

// element offset inside a block of this lane's 8-element MFMA chunk
template <int DT>
__device__ inline int chunk_start(int g) {
    return DT == MOE_GGML_Q8_0 ? 8 * g : (g & 1) * 16 + (g >> 1) * 8;
}

typedef const __attribute__((address_space(1))) uint8_t* gbytes32;
typedef uint32_t u32x2g __attribute__((ext_vector_type(2)));
typedef float f32x4g __attribute__((ext_vector_type(4)));
typedef int i32x4g __attribute__((ext_vector_type(4)));
template <typename T>
__device__ __forceinline__ T ldg(const void* uniform_base, uint32_t off) {
    return *reinterpret_cast<const __attribute__((address_space(1))) T*>((gbytes32)uniform_base + off);
}
template <typename T>
__device__ __forceinline__ T ldg_stream(const void* uniform_base, uint32_t off) {
    return __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) T*>((gbytes32)uniform_base + off));
}

// One lane's share of a tile as it is fetched: 8 code bytes, the row's d (and m), the row's fifth bits.
struct Q32Raw {
    u32x2g q;
    uint32_t dm;
    uint32_t h;
};
// ONCE: the weights are read by one pass only (non-temporal: they should not displace the activations
// in the caches); otherwise further workgroups stream the same tiles again and should find them in L2
template <int DT, bool ONCE>
__device__ __forceinline__ Q32Raw load_q32_raw(const uint8_t* tile, uint32_t q_off, uint32_t d_off, uint32_t h_off) {
    typedef Q32Fmt<DT> F;
    Q32Raw t;
    t.h = 0;
    if (ONCE) {
        t.q = ldg_stream<u32x2g>(tile, q_off);
        t.dm = F::HAS_M ? ldg_stream<uint32_t>(tile, d_off) : (uint32_t)ldg_stream<unsigned short>(tile, d_off);
        if (F::FIFTH) t.h = ldg_stream<uint32_t>(tile, h_off);
    } else {
        t.q = ldg<u32x2g>(tile, q_off);
        t.dm = F::HAS_M ? ldg<uint32_t>(tile, d_off) : (uint32_t)ldg<unsigned short>(tile, d_off);
        if (F::FIFTH) t.h = ldg<uint32_t>(tile, h_off);
    }
    return t;
}
// bits 0..3 of x to bit 4 of bytes 0..3 (the four shifted copies of x do not overlap, so no carries)
__device__ __forceinline__ uint32_t fifth_bits(uint32_t x) { return ((x * 0x00204081u) & 0x01010101u) << 4; }
template <int DT>
__device__ __forceinline__ Q32Tile<DT> q32_unpack(const Q32Raw& raw, int g) {
    typedef Q32Fmt<DT> F;
    Q32Tile<DT> t;
    if (!F::NIB) {
        t.q = make_uint2(raw.q.x, raw.q.y);
    } else {
        uint32_t x = raw.q.x, y = raw.q.y;
        if (g & 1) { x >>= 4; y >>= 4; }
        x &= 0x0f0f0f0fu; y &= 0x0f0f0f0fu;
        if (F::FIFTH) {   // bit e of the word belongs to element e; this lane's elements start at chunk_start
            const uint32_t hb = raw.h >> chunk_start<DT>(g);
            x |= fifth_bits(hb & 15u);
            y |= fifth_bits((hb >> 4) & 15u);
        }
        t.q = make_uint2(x, y);
    }
    t.d = __half2float(__ushort_as_half((unsigned short)(raw.dm & 0xffffu)));
    t.m = F::HAS_M ? __half2float(__ushort_as_half((unsigned short)(raw.dm >> 16))) : 0.f;
    return t;
}

template <int DT>
__device__ inline Q32Tile<DT> load_q32_tile(const uint8_t* tile, int lane) {
    typedef Q32Fmt<DT> F;
    return q32_unpack<DT>(load_q32_raw<DT, true>(tile, F::q_off(lane), F::d_off(lane), F::h_off(lane)), lane >> 4);
}

struct Q8_0Operand {
    uint2 a;
    float yd[4];
    int bs[4];
};

template <int DT>
__device__ inline Q8_0Operand load_q8_0_operand(const ActBuf& ab, int K, int nkb, int kb, int rowA, const int rowD[4], int g) {
    Q8_0Operand o;
    o.a = *reinterpret_cast<const uint2*>(ab.qs + (int64_t)rowA * K + kb * 32 + chunk_start<DT>(g));
#pragma unroll
    for (int i = 0; i < 4; i++) {
        o.yd[i] = ab.d[(int64_t)rowD[i] * nkb + kb];
        o.bs[i] = (Q32Fmt<DT>::OFFSET || Q32Fmt<DT>::HAS_M) ? reinterpret_cast<const int32_t*>(ab.bsum)[(int64_t)rowD[i] * nkb + kb] : 0;
    }
    return o;
}

template <int DT>
__device__ inline void q32_mac(const Q32Tile<DT>& w, const Q8_0Operand& A, float acc[4]) {
    const v4i zero = {0, 0, 0, 0};
    const long a = (long)(((uint64_t)A.a.y << 32) | A.a.x);
    const long b = (long)(((uint64_t)w.q.y << 32) | w.q.x);
    v4i D = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b, zero, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int isum = D[i];
        if (Q32Fmt<DT>::OFFSET) isum -= Q32Fmt<DT>::OFFSET * A.bs[i];
        float t = (float)isum * w.d;
        t = t * A.yd[i];
        if (Q32Fmt<DT>::HAS_M) t = t + w.m * __int_as_float(A.bs[i]);   // the word holds the activation block's s
        acc[i] += t;
    }
}

__device__ inline float silu_ref32(float v) { return v / (1.0f + expf_glibc(-v)); }

constexpr int Q32_THREADS = 256;

template <int DT, int TT>
__global__ __launch_bounds__(Q32_THREADS) void q32_up_kernel(ExpertParams p) {
    __shared__ int list_lds[DIRECT_MAX_SLOTS];
    __shared__ int wtot_lds[Q32_THREADS / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, g = lane >> 4;
    const int grp = blockIdx.y;
    const GroupSlots gs = group_slots<Q32_THREADS>(p, grp, list_lds, wtot_lds);
    const int tg0 = blockIdx.z * (TT * 16);
    if (tg0 >= gs.n) return;
    const int H = p.H, F = p.F, nkb = H / 32;
    const int rt0 = (blockIdx.x * (Q32_THREADS / 64) + wave) * 2;
    if (rt0 >= F / 16) return;
    constexpr int TB = Q32Fmt<DT>::TB;

    int rowA[TT], rowD[TT][4];
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        int ia = tg0 + tt * 16 + r;
        rowA[tt] = slot_token(p, gs.slot(ia < gs.n ? ia : gs.n - 1));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int id = tg0 + tt * 16 + 4 * g + i;
            rowD[tt][i] = slot_token(p, gs.slot(id < gs.n ? id : gs.n - 1));
        }
    }
    const GroupWeights gw = p.groups[grp];
    const uint8_t* tp[4] = {gw.w1 + (size_t)rt0 * nkb * TB, gw.w1 + (size_t)(rt0 + 1) * nkb * TB,
                            gw.w3 + (size_t)rt0 * nkb * TB, gw.w3 + (size_t)(rt0 + 1) * nkb * TB};
    float acc[4][TT][4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int tt = 0; tt < TT; tt++)
#pragma unroll
            for (int i = 0; i < 4; i++) acc[j][tt][i] = 0.f;

    Q32Tile<DT> cur[4], nxt[4];
#pragma unroll
    for (int j = 0; j < 4; j++) cur[j] = load_q32_tile<DT>(tp[j], lane);
    for (int kb = 0; kb < nkb; kb++) {
        if (kb + 1 < nkb) {
#pragma unroll
            for (int j = 0; j < 4; j++) nxt[j] = load_q32_tile<DT>(tp[j] + (size_t)(kb + 1) * TB, lane);
        }
#pragma unroll
        for (int tt = 0; tt < TT; tt++) {
            Q8_0Operand A = load_q8_0_operand<DT>(p.xq, H, nkb, kb, rowA[tt], rowD[tt], g);
#pragma unroll
            for (int j = 0; j < 4; j++) q32_mac<DT>(cur[j], A, acc[j][tt]);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) cur[j] = nxt[j];
    }

    // epilogue: h = silu(w1 x) * (w3 x); the wave's 32 rows are exactly one Q8_0 block per slot
    const int nfb = F / 32;
    const int fb = rt0 / 2;
#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float h0 = silu_ref32(acc[0][tt][i]) * acc[2][tt][i];
            float h1 = silu_ref32(acc[1][tt][i]) * acc[3][tt][i];
            float amax = fmaxf(fabsf(h0), fabsf(h1));
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
            float d = amax / 127.0f;
            float id = (d != 0.f) ? 1.0f / d : 0.f;
            int q0 = sat_i8(roundf(h0 * id)), q1 = sat_i8(roundf(h1 * id));
            int sum = q0 + q1;
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
            const int pos = tg0 + tt * 16 + 4 * g + i;
            if (pos < gs.n) {
                int64_t hrow = gs.slot(pos) - p.slot_origin;
                p.hq.qs[hrow * F + rt0 * 16 + r] = (int8_t)q0;
                p.hq.qs[hrow * F + rt0 * 16 + 16 + r] = (int8_t)q1;
                if (r == 0) {
                    const float dh = __half2float(__float2half_rn(d));
                    p.hq.d[hrow * nfb + fb] = dh;
                    reinterpret_cast<int32_t*>(p.hq.bsum)[hrow * nfb + fb] = q8_block_word(vecdot_dtype(DT), sum, dh);
                }
            }
        }
}

constexpr int Q32_DOWN_STEP = 4;

template <int DT, int TT>
__global__ __launch_bounds__(Q32_THREADS) void q32_down_kernel(ExpertParams p) {
    __shared__ int list_lds[DIRECT_MAX_SLOTS];
    __shared__ int wtot_lds[Q32_THREADS / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, g = lane >> 4;
    const int grp = blockIdx.y;
    const GroupSlots gs = group_slots<Q32_THREADS>(p, grp, list_lds, wtot_lds);
    const int tg0 = blockIdx.z * (TT * 16);
    if (tg0 >= gs.n) return;
    const int H = p.H, F = p.F, nkb = F / 32;
    const int rt = blockIdx.x * (Q32_THREADS / 64) + wave;
    if (rt >= H / 16) return;
    constexpr int TB = Q32Fmt<DT>::TB;

    int rowA[TT], rowD[TT][4];
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        int ia = tg0 + tt * 16 + r;
        rowA[tt] = gs.slot(ia < gs.n ? ia : gs.n - 1) - p.slot_origin;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int id = tg0 + tt * 16 + 4 * g + i;
            rowD[tt][i] = gs.slot(id < gs.n ? id : gs.n - 1) - p.slot_origin;
        }
    }
    const uint8_t* tp = p.groups[grp].w2 + (size_t)rt * nkb * TB;
    float acc[TT][4];
#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[tt][i] = 0.f;

    Q32Tile<DT> cur[Q32_DOWN_STEP], nxt[Q32_DOWN_STEP];
#pragma unroll
    for (int j = 0; j < Q32_DOWN_STEP; j++)
        if (j < nkb) cur[j] = load_q32_tile<DT>(tp + (size_t)j * TB, lane);
    for (int kb0 = 0; kb0 < nkb; kb0 += Q32_DOWN_STEP) {
#pragma unroll
        for (int j = 0; j < Q32_DOWN_STEP; j++)
            if (kb0 + Q32_DOWN_STEP + j < nkb) nxt[j] = load_q32_tile<DT>(tp + (size_t)(kb0 + Q32_DOWN_STEP + j) * TB, lane);
#pragma unroll
        for (int j = 0; j < Q32_DOWN_STEP; j++) {
            if (kb0 + j < nkb) {
#pragma unroll
                for (int tt = 0; tt < TT; tt++) {
                    Q8_0Operand A = load_q8_0_operand<DT>(p.hq, F, nkb, kb0 + j, rowA[tt], rowD[tt], g);
                    q32_mac<DT>(cur[j], A, acc[tt]);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < Q32_DOWN_STEP; j++) cur[j] = nxt[j];
    }
#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int pos = tg0 + tt * 16 + 4 * g + i;
            if (pos < gs.n) {
                const int slot = gs.slot(pos);
                p.yw[(int64_t)slot * H + rt * 16 + r] = acc[tt][i] * slot_weight(p, slot);
            }
        }
}

// ---------------------------------------------------------------------------------------------
// Streaming versions of the two kernels above (same arithmetic, same order of additions): STEP blocks
// per trip, the next trip's weight tiles requested before this trip's arithmetic (double buffer),
// non-temporal global loads with a scalar base and 32-bit lane offsets, the activation scales and
// block sums of a trip fetched as one 16-byte load per output slot.  They need K / 32 to be a
// multiple of STEP; other shapes take the kernels above.
// activation operand of one 16-slot tile for STEP consecutive blocks
template <int STEP>
struct Q8_0Trip {
    u32x2g a[STEP];
    f32x4g yd[4][STEP / 4];
    i32x4g bs[4][STEP / 4];
};
template <int DT, int STEP>
__device__ __forceinline__ Q8_0Trip<STEP> load_q8_0_trip(const ActBuf& ab, int K, int nkb, int kb0, int rowA, const int rowD[4], int g) {
    Q8_0Trip<STEP> o;
    const uint32_t abase = (uint32_t)rowA * (uint32_t)K + (uint32_t)(kb0 * 32 + chunk_start<DT>(g));
#pragma unroll
    for (int j = 0; j < STEP; j++) o.a[j] = ldg<u32x2g>(ab.qs, abase + j * 32);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t doff = ((uint32_t)rowD[i] * (uint32_t)nkb + (uint32_t)kb0) * 4;
#pragma unroll
        for (int q = 0; q < STEP / 4; q++) {
            o.yd[i][q] = ldg<f32x4g>(ab.d, doff + q * 16);
            if (Q32Fmt<DT>::OFFSET || Q32Fmt<DT>::HAS_M) o.bs[i][q] = ldg<i32x4g>(ab.bsum, doff + q * 16);
        }
    }
    return o;
}

template <int DT, int STEP>
__device__ __forceinline__ void q32_mac_trip(const Q32Tile<DT>& w, const Q8_0Trip<STEP>& A, int j, float acc[4]) {
    const v4i zero = {0, 0, 0, 0};
    const long a = (long)(((uint64_t)A.a[j].y << 32) | A.a[j].x);
    const long b = (long)(((uint64_t)w.q.y << 32) | w.q.x);
    v4i D = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b, zero, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int isum = D[i];
        if (Q32Fmt<DT>::OFFSET) isum -= Q32Fmt<DT>::OFFSET * A.bs[i][j / 4][j % 4];
        float t = (float)isum * w.d;
        t = t * A.yd[i][j / 4][j % 4];
        if (Q32Fmt<DT>::HAS_M) t = t + w.m * __int_as_float(A.bs[i][j / 4][j % 4]);
        acc[i] += t;
    }
}

// One wave: NT weight tile streams (tp[j], advancing TB bytes per block) against TT slot tiles, all of K.
template <int DT, int TT, int NT, int STEP, bool ONCE>
__device__ __forceinline__ void q32_engine(const uint8_t* const tp[NT], const ActBuf& ab, int K, const int rowA[TT], const int rowD[TT][4],
                                           int lane, float acc[NT][TT][4]) {
    constexpr int TB = Q32Fmt<DT>::TB;
    const int g = lane >> 4;
    const int nkb = K / 32;
    const uint32_t q_off = Q32Fmt<DT>::q_off(lane), d_off = Q32Fmt<DT>::d_off(lane), h_off = Q32Fmt<DT>::h_off(lane);
    // ONCE (the weights come from HBM): the next trip's tiles are requested a whole trip ahead.  Otherwise they
    // are in L2 after the first pass and are fetched where they are used: half the registers, twice the waves.
    Q32Raw nxt[ONCE ? NT : 1][ONCE ? STEP : 1];
    if (ONCE) {
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int j = 0; j < STEP; j++) nxt[t][j] = load_q32_raw<DT, ONCE>(tp[t] + (size_t)j * TB, q_off, d_off, h_off);
    }
    // With several slot tiles the activation operand is requested one step ahead too: the one of slot
    // tile tt+1, or of the next trip's first slot tile, is on its way while this one is multiplied.
    // (With one slot tile the extra registers cost a wave per SIMD, which costs more than the wait.)
    constexpr bool AHEAD = TT > 1;
    Q8_0Trip<STEP> An;
    if (AHEAD) An = load_q8_0_trip<DT, STEP>(ab, K, nkb, 0, rowA[0], rowD[0], g);
    for (int kb0 = 0; kb0 < nkb; kb0 += STEP) {
        Q32Raw cur[NT][STEP];
        // the trip after this one; past the end the last trip is requested again (no branch around a load)
        const int kbn = kb0 + STEP < nkb ? kb0 + STEP : kb0;
        if (ONCE) {
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int j = 0; j < STEP; j++) cur[t][j] = nxt[t][j];
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int j = 0; j < STEP; j++) nxt[t][j] = load_q32_raw<DT, ONCE>(tp[t] + (size_t)(kbn + j) * TB, q_off, d_off, h_off);
        } else {
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int j = 0; j < STEP; j++) cur[t][j] = load_q32_raw<DT, ONCE>(tp[t] + (size_t)(kb0 + j) * TB, q_off, d_off, h_off);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int tt = 0; tt < TT; tt++) {
            Q8_0Trip<STEP> A;
            if (AHEAD) {
                A = An;
                An = tt + 1 < TT ? load_q8_0_trip<DT, STEP>(ab, K, nkb, kb0, rowA[tt + 1 < TT ? tt + 1 : 0], rowD[tt + 1 < TT ? tt + 1 : 0], g)
                                 : load_q8_0_trip<DT, STEP>(ab, K, nkb, kbn, rowA[0], rowD[0], g);
                __builtin_amdgcn_sched_barrier(0);
            } else {
                A = load_q8_0_trip<DT, STEP>(ab, K, nkb, kb0, rowA[tt], rowD[tt], g);
            }
#pragma unroll
            for (int j = 0; j < STEP; j++)
#pragma unroll
                for (int t = 0; t < NT; t++) q32_mac_trip<DT, STEP>(q32_unpack<DT>(cur[t][j], g), A, j, acc[t][tt]);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

constexpr int Q32_STEP = 4;

template <int DT, int TT, bool ONCE>
__global__ __launch_bounds__(Q32_THREADS) void q32_up_stream_kernel(ExpertParams p) {
    __shared__ int list_lds[DIRECT_MAX_SLOTS];
    __shared__ int wtot_lds[Q32_THREADS / 64];
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = blockIdx.y;
    const GroupSlots gs = group_slots<Q32_THREADS>(p, grp, list_lds, wtot_lds);
    const int tg0 = blockIdx.z * (TT * 16);
    if (tg0 >= gs.n) return;
    const int H = p.H, F = p.F, nkb = H / 32;
    const int rt0 = (blockIdx.x * (Q32_THREADS / 64) + wave) * 2;
    if (rt0 >= F / 16) return;
    constexpr int TB = Q32Fmt<DT>::TB;

    int rowA[TT], rowD[TT][4];
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        int ia = tg0 + tt * 16 + r;
        rowA[tt] = slot_token(p, gs.slot(ia < gs.n ? ia : gs.n - 1));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int id = tg0 + tt * 16 + 4 * g + i;
            rowD[tt][i] = slot_token(p, gs.slot(id < gs.n ? id : gs.n - 1));
        }
    }
    const GroupWeights gw = p.groups[grp];
    const uint8_t* tp[4] = {gw.w1 + (size_t)rt0 * nkb * TB, gw.w1 + (size_t)(rt0 + 1) * nkb * TB,
                            gw.w3 + (size_t)rt0 * nkb * TB, gw.w3 + (size_t)(rt0 + 1) * nkb * TB};
    float acc[4][TT][4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int tt = 0; tt < TT; tt++)
#pragma unroll
            for (int i = 0; i < 4; i++) acc[j][tt][i] = 0.f;

    q32_engine<DT, TT, 4, Q32_STEP, ONCE>(tp, p.xq, H, rowA, rowD, lane, acc);

    // epilogue: h = silu(w1 x) * (w3 x); the wave's 32 rows are exactly one Q8_0 block per slot
    const int nfb = F / 32;
    const int fb = rt0 / 2;
#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float h0 = silu_ref32(acc[0][tt][i]) * acc[2][tt][i];
            float h1 = silu_ref32(acc[1][tt][i]) * acc[3][tt][i];
            float amax = fmaxf(fabsf(h0), fabsf(h1));
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
            float d = amax / 127.0f;
            float id = (d != 0.f) ? 1.0f / d : 0.f;
            int q0 = sat_i8(roundf(h0 * id)), q1 = sat_i8(roundf(h1 * id));
            int sum = q0 + q1;
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
            const int pos = tg0 + tt * 16 + 4 * g + i;
            if (pos < gs.n) {
                int64_t hrow = gs.slot(pos) - p.slot_origin;
                p.hq.qs[hrow * F + rt0 * 16 + r] = (int8_t)q0;
                p.hq.qs[hrow * F + rt0 * 16 + 16 + r] = (int8_t)q1;
                if (r == 0) {
                    const float dh = __half2float(__float2half_rn(d));
                    p.hq.d[hrow * nfb + fb] = dh;
                    reinterpret_cast<int32_t*>(p.hq.bsum)[hrow * nfb + fb] = q8_block_word(vecdot_dtype(DT), sum, dh);
                }
            }
        }
}

template <int DT, int TT, bool ONCE>
__global__ __launch_bounds__(Q32_THREADS) void q32_down_stream_kernel(ExpertParams p) {
    __shared__ int list_lds[DIRECT_MAX_SLOTS];
    __shared__ int wtot_lds[Q32_THREADS / 64];
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = blockIdx.y;
    const GroupSlots gs = group_slots<Q32_THREADS>(p, grp, list_lds, wtot_lds);
    const int tg0 = blockIdx.z * (TT * 16);
    if (tg0 >= gs.n) return;
    const int H = p.H, F = p.F, nkb = F / 32;
    const int rt = blockIdx.x * (Q32_THREADS / 64) + wave;
    if (rt >= H / 16) return;
    constexpr int TB = Q32Fmt<DT>::TB;

    int rowA[TT], rowD[TT][4];
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        int ia = tg0 + tt * 16 + r;
        rowA[tt] = gs.slot(ia < gs.n ? ia : gs.n - 1) - p.slot_origin;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int id = tg0 + tt * 16 + 4 * g + i;
            rowD[tt][i] = gs.slot(id < gs.n ? id : gs.n - 1) - p.slot_origin;
        }
    }
    const uint8_t* tp[1] = {p.groups[grp].w2 + (size_t)rt * nkb * TB};
    float acc[1][TT][4];
#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[0][tt][i] = 0.f;

    q32_engine<DT, TT, 1, ONCE ? 2 * Q32_STEP : Q32_STEP, ONCE>(tp, p.hq, F, rowA, rowD, lane, acc);

#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int pos = tg0 + tt * 16 + 4 * g + i;
            if (pos < gs.n) {
                const int slot = gs.slot(pos);
                p.yw[(int64_t)slot * H + rt * 16 + r] = acc[0][tt][i] * slot_weight(p, slot);
            }
        }
}

template <int DT>
static hipError_t launch_q32_up_t(const ExpertParams& p, hipStream_t s) {
    const int tt = p.slot_tiles >= 2 ? 2 : 1;
    const int wpb = Q32_THREADS / 64;
    const int n_pairs = p.F / 32;
    dim3 grid((unsigned)((n_pairs + wpb - 1) / wpb), (unsigned)p.n_groups, (unsigned)((p.max_rows + tt * 16 - 1) / (tt * 16)));
    static const bool plain = getenv("MOE_Q32_PLAIN") != nullptr;
    const bool stream = !plain && (p.H / 32) % Q32_STEP == 0;
    if (tt == 1) {
        if (stream) hipLaunchKernelGGL((q32_up_stream_kernel<DT, 1, true>), grid, dim3(Q32_THREADS), 0, s, p);
        else hipLaunchKernelGGL((q32_up_kernel<DT, 1>), grid, dim3(Q32_THREADS), 0, s, p);
    } else {
        if (stream && grid.z == 1) hipLaunchKernelGGL((q32_up_stream_kernel<DT, 2, true>), grid, dim3(Q32_THREADS), 0, s, p);
        else if (stream) hipLaunchKernelGGL((q32_up_stream_kernel<DT, 2, false>), grid, dim3(Q32_THREADS), 0, s, p);
        else hipLaunchKernelGGL((q32_up_kernel<DT, 2>), grid, dim3(Q32_THREADS), 0, s, p);
    }
    return hipGetLastError();
}
template <int DT>
static hipError_t launch_q32_down_t(const ExpertParams& p, hipStream_t s) {
    const int tt = p.slot_tiles >= 2 ? 2 : 1;
    const int wpb = Q32_THREADS / 64;
    dim3 grid((unsigned)((p.H / 16 + wpb - 1) / wpb), (unsigned)p.n_groups, (unsigned)((p.max_rows + tt * 16 - 1) / (tt * 16)));
    static const bool plain = getenv("MOE_Q32_PLAIN") != nullptr;
    const bool stream = !plain && (p.F / 32) % (2 * Q32_STEP) == 0;
    const bool stream_again = !plain && (p.F / 32) % Q32_STEP == 0;   // the several-pass variant walks K in shorter trips
    if (tt == 1) {
        if (stream) hipLaunchKernelGGL((q32_down_stream_kernel<DT, 1, true>), grid, dim3(Q32_THREADS), 0, s, p);
        else hipLaunchKernelGGL((q32_down_kernel<DT, 1>), grid, dim3(Q32_THREADS), 0, s, p);
    } else {
        if (stream && grid.z == 1) hipLaunchKernelGGL((q32_down_stream_kernel<DT, 2, true>), grid, dim3(Q32_THREADS), 0, s, p);
        else if (stream_again && grid.z > 1) hipLaunchKernelGGL((q32_down_stream_kernel<DT, 2, false>), grid, dim3(Q32_THREADS), 0, s, p);
        else hipLaunchKernelGGL((q32_down_kernel<DT, 2>), grid, dim3(Q32_THREADS), 0, s, p);
    }
    return hipGetLastError();
}

hipError_t launch_q4k_up(const ExpertParams& p, hipStream_t s);
hipError_t launch_q4k_down(const ExpertParams& p, hipStream_t s);

hipError_t launch_expert_up(const ExpertParams& p, hipStream_t s) {
    if (p.max_rows == 0 || p.n_groups == 0) return hipSuccess;
    switch (p.dt) {
        case MOE_GGML_Q2K: case MOE_GGML_Q3K: case MOE_GGML_Q4K: case MOE_GGML_Q5K: case MOE_GGML_Q6K: return launch_q4k_up(p, s);
        case MOE_GGML_Q8_0: return launch_q32_up_t<MOE_GGML_Q8_0>(p, s);
        case MOE_GGML_Q4_0: return launch_q32_up_t<MOE_GGML_Q4_0>(p, s);
        case MOE_GGML_Q4_1: return launch_q32_up_t<MOE_GGML_Q4_1>(p, s);
        case MOE_GGML_Q5_0: return launch_q32_up_t<MOE_GGML_Q5_0>(p, s);
        case MOE_GGML_Q5_1: return launch_q32_up_t<MOE_GGML_Q5_1>(p, s);
    }
    return hipErrorInvalidValue;
}
hipError_t launch_expert_down(const ExpertParams& p, hipStream_t s) {
    if (p.max_rows == 0 || p.n_groups == 0) return hipSuccess;
    switch (p.dt_down ? p.dt_down : p.dt) {
        case MOE_GGML_Q2K: case MOE_GGML_Q3K: case MOE_GGML_Q4K: case MOE_GGML_Q5K: case MOE_GGML_Q6K: return launch_q4k_down(p, s);
        case MOE_GGML_Q8_0: return launch_q32_down_t<MOE_GGML_Q8_0>(p, s);
        case MOE_GGML_Q4_0: return launch_q32_down_t<MOE_GGML_Q4_0>(p, s);
        case MOE_GGML_Q4_1: return launch_q32_down_t<MOE_GGML_Q4_1>(p, s);
        case MOE_GGML_Q5_0: return launch_q32_down_t<MOE_GGML_Q5_0>(p, s);
        case MOE_GGML_Q5_1: return launch_q32_down_t<MOE_GGML_Q5_1>(p, s);
    }
    return hipErrorInvalidValue;
}

}  // namespace moe
