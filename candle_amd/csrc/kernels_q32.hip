// Grouped expert products over Q4_0 / Q8_0 weights with Q8_0 activations (gfx950, int8 MFMA).
//
// Arithmetic restated from candle-core/src/quantized/k_quants.rs:241-258 (Q4_0 . Q8_0) and
// :650-668 (Q8_0 . Q8_0): per 32-element block  sumf += (sum_i as f32) * d_w * d_x.  One
// v_mfma_i32_16x16x32_i8 yields the exact integer dot of a block for 16 rows x 16 slots, and every
// lane adds its (row, slot) blocks in ascending block order with separately rounded products, so
// the f32 result is bit-identical to the scalar reference loop.
//
// Q4_0 stores nibble - 8; the kernel multiplies the raw nibbles (0..15) and subtracts
// 8 * sum(q8) of the block, which is the same integer.
#include <cstdlib>
#include "act_quant.hpp"
#include "kernels.hpp"
#include "slots.hpp"

namespace moe {

typedef int v4i __attribute__((ext_vector_type(4)));

template <int DT>
struct Q32Tile {
    uint2 q;
    float d;
};

// weight tiles are read once per launch: non-temporal loads keep them from displacing the activations
// and routing lists in the caches
typedef uint32_t u32x2_q32 __attribute__((ext_vector_type(2)));
__device__ inline uint2 load_stream8(const uint8_t* p) {
    const u32x2_q32 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2_q32*>(p));
    return make_uint2(v.x, v.y);
}
__device__ inline float load_stream_half(const uint8_t* p) {
    const unsigned short h = __builtin_nontemporal_load(reinterpret_cast<const unsigned short*>(p));
    return __half2float(__ushort_as_half(h));
}

template <int DT>
__device__ inline Q32Tile<DT> load_q32_tile(const uint8_t* tile, int lane) {
    Q32Tile<DT> t;
    const int r = lane & 15, g = lane >> 4;
    if (DT == MOE_GGML_Q8_0) {
        t.q = load_stream8(tile + lane * 8);
        t.d = load_stream_half(tile + 512 + 2 * r);
    } else {
        uint2 w = load_stream8(tile + r * 16 + 8 * (g >> 1));
        if (g & 1) { w.x >>= 4; w.y >>= 4; }
        t.q.x = w.x & 0x0f0f0f0fu;
        t.q.y = w.y & 0x0f0f0f0fu;
        t.d = load_stream_half(tile + 256 + 2 * r);
    }
    return t;
}

struct Q8_0Operand {
    uint2 a;
    float yd[4];
    int bs[4];
};

// element offset inside a block of this lane's 8-element MFMA chunk
template <int DT>
__device__ inline int chunk_start(int g) {
    return DT == MOE_GGML_Q8_0 ? 8 * g : (g & 1) * 16 + (g >> 1) * 8;
}

template <int DT>
__device__ inline Q8_0Operand load_q8_0_operand(const ActBuf& ab, int K, int nkb, int kb, int rowA, const int rowD[4], int g) {
    Q8_0Operand o;
    o.a = *reinterpret_cast<const uint2*>(ab.qs + (int64_t)rowA * K + kb * 32 + chunk_start<DT>(g));
#pragma unroll
    for (int i = 0; i < 4; i++) {
        o.yd[i] = ab.d[(int64_t)rowD[i] * nkb + kb];
        o.bs[i] = (DT == MOE_GGML_Q4_0) ? reinterpret_cast<const int32_t*>(ab.bsum)[(int64_t)rowD[i] * nkb + kb] : 0;
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
        if (DT == MOE_GGML_Q4_0) isum -= 8 * A.bs[i];
        float t = (float)isum * w.d;
        t = t * A.yd[i];
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
    constexpr int TB = (DT == MOE_GGML_Q8_0) ? Q8_0_TILE_BYTES : Q4_0_TILE_BYTES;

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
                    p.hq.d[hrow * nfb + fb] = __half2float(__float2half_rn(d));
                    reinterpret_cast<int32_t*>(p.hq.bsum)[hrow * nfb + fb] = sum;
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
    constexpr int TB = (DT == MOE_GGML_Q8_0) ? Q8_0_TILE_BYTES : Q4_0_TILE_BYTES;

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

struct Q32Raw {
    u32x2g q;
    unsigned short d;
};
// ONCE: the weights are read by one pass only (non-temporal: they should not displace the activations
// in the caches); otherwise further workgroups stream the same tiles again and should find them in L2
template <int DT, bool ONCE>
__device__ __forceinline__ Q32Raw load_q32_raw(const uint8_t* tile, uint32_t q_off, uint32_t d_off) {
    Q32Raw t;
    if (ONCE) {
        t.q = ldg_stream<u32x2g>(tile, q_off);
        t.d = ldg_stream<unsigned short>(tile, d_off);
    } else {
        t.q = ldg<u32x2g>(tile, q_off);
        t.d = ldg<unsigned short>(tile, d_off);
    }
    return t;
}
template <int DT>
__device__ __forceinline__ Q32Tile<DT> q32_unpack(const Q32Raw& raw, int g) {
    Q32Tile<DT> t;
    if (DT == MOE_GGML_Q8_0) {
        t.q = make_uint2(raw.q.x, raw.q.y);
    } else {
        uint32_t x = raw.q.x, y = raw.q.y;
        if (g & 1) { x >>= 4; y >>= 4; }
        t.q = make_uint2(x & 0x0f0f0f0fu, y & 0x0f0f0f0fu);
    }
    t.d = __half2float(__ushort_as_half(raw.d));
    return t;
}

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
            if (DT == MOE_GGML_Q4_0) o.bs[i][q] = ldg<i32x4g>(ab.bsum, doff + q * 16);
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
        if (DT == MOE_GGML_Q4_0) isum -= 8 * A.bs[i][j / 4][j % 4];
        float t = (float)isum * w.d;
        t = t * A.yd[i][j / 4][j % 4];
        acc[i] += t;
    }
}

// One wave: NT weight tile streams (tp[j], advancing TB bytes per block) against TT slot tiles, all of K.
template <int DT, int TT, int NT, int STEP, bool ONCE>
__device__ __forceinline__ void q32_engine(const uint8_t* const tp[NT], const ActBuf& ab, int K, const int rowA[TT], const int rowD[TT][4],
                                           int lane, float acc[NT][TT][4]) {
    constexpr int TB = (DT == MOE_GGML_Q8_0) ? Q8_0_TILE_BYTES : Q4_0_TILE_BYTES;
    const int r = lane & 15, g = lane >> 4;
    const int nkb = K / 32;
    const uint32_t q_off = DT == MOE_GGML_Q8_0 ? (uint32_t)lane * 8u : (uint32_t)(r * 16 + 8 * (g >> 1));
    const uint32_t d_off = (DT == MOE_GGML_Q8_0 ? 512u : 256u) + 2u * (uint32_t)r;
    // ONCE (the weights come from HBM): the next trip's tiles are requested a whole trip ahead.  Otherwise they
    // are in L2 after the first pass and are fetched where they are used: half the registers, twice the waves.
    Q32Raw nxt[ONCE ? NT : 1][ONCE ? STEP : 1];
    if (ONCE) {
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int j = 0; j < STEP; j++) nxt[t][j] = load_q32_raw<DT, ONCE>(tp[t] + (size_t)j * TB, q_off, d_off);
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
                for (int j = 0; j < STEP; j++) nxt[t][j] = load_q32_raw<DT, ONCE>(tp[t] + (size_t)(kbn + j) * TB, q_off, d_off);
        } else {
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int j = 0; j < STEP; j++) cur[t][j] = load_q32_raw<DT, ONCE>(tp[t] + (size_t)(kb0 + j) * TB, q_off, d_off);
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
    constexpr int TB = (DT == MOE_GGML_Q8_0) ? Q8_0_TILE_BYTES : Q4_0_TILE_BYTES;

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
                    p.hq.d[hrow * nfb + fb] = __half2float(__float2half_rn(d));
                    reinterpret_cast<int32_t*>(p.hq.bsum)[hrow * nfb + fb] = sum;
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
    constexpr int TB = (DT == MOE_GGML_Q8_0) ? Q8_0_TILE_BYTES : Q4_0_TILE_BYTES;

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
    }
    return hipErrorInvalidValue;
}
hipError_t launch_expert_down(const ExpertParams& p, hipStream_t s) {
    if (p.max_rows == 0 || p.n_groups == 0) return hipSuccess;
    switch (p.dt_down ? p.dt_down : p.dt) {
        case MOE_GGML_Q2K: case MOE_GGML_Q3K: case MOE_GGML_Q4K: case MOE_GGML_Q5K: case MOE_GGML_Q6K: return launch_q4k_down(p, s);
        case MOE_GGML_Q8_0: return launch_q32_down_t<MOE_GGML_Q8_0>(p, s);
        case MOE_GGML_Q4_0: return launch_q32_down_t<MOE_GGML_Q4_0>(p, s);
    }
    return hipErrorInvalidValue;
}

}  // namespace moe
