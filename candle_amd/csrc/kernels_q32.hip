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
// the same with the exp table in LDS (32 entries, filled by the caller): a table fetched from memory per element makes
// a run of these a chain of memory latencies
__device__ inline float silu_ref32(float v, const uint64_t* lds_tab) {
    return v / (1.0f + expf_glibc_with(-v, [lds_tab](int i) { return lds_tab[i]; }));
}

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
            int q0 = round_as_i8(h0 * id), q1 = round_as_i8(h1 * id);
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
                emit_expert_output(p, slot, rt * 16 + r, acc[tt][i] * slot_weight(p, slot));
            }
        }
}

// ---------------------------------------------------------------------------------------------
// Streaming versions of the two kernels above (same arithmetic, same order of additions) for matrices
// whose K is a multiple of 128: those are kept in "super-tiles" of 16 rows x four blocks (moe_common.hpp),
// so a lane fetches the codes of four blocks with one or two 16-byte loads and their scales with one.
//
// The four waves of a workgroup work on different rows against the SAME slots, so the activation operand
// is staged once per workgroup: every K step (four blocks) the 256 threads copy the 16 x 128 quants of each
// slot tile and their 64 (scale, word) pairs from global memory into LDS in MFMA operand order (double
// buffered, one barrier per step); the waves read them back with conflict-free 8-byte reads and broadcast
// 16-byte reads.  The weights go global -> registers, one step ahead.
typedef uint32_t u32x4g __attribute__((ext_vector_type(4)));

template <int DT>
struct Q32SFmt {
    typedef Q32Fmt<DT> F;
    static constexpr uint32_t QB = F::NIB ? 1024 : 2048;     // codes: lane l at 16 l (Q8_0: blocks 0,1 then, 1 KiB on, 2,3)
    static constexpr uint32_t HB = F::FIFTH ? 256 : 0;       // fifth-bit words: row r at 16 r, one word per block
    static constexpr uint32_t DB = F::HAS_M ? 256 : 128;     // d (and m) per block: row r at 8 r (16 r)
    static constexpr uint32_t STB = QB + HB + DB;            // = 4 tiles of the one-block layout
};

template <int DT>
struct Q32SRaw {
    u32x4g q0, q1;   // q1: Q8_0 only
    u32x4g h;        // five-bit formats only
    u32x4g dm;       // formats with a minimum: (d, m) of the four blocks; else .x / .y = the four d
};
template <int DT, bool ONCE>
__device__ __forceinline__ Q32SRaw<DT> load_q32s(const uint8_t* tile, int lane) {
    typedef Q32Fmt<DT> F;
    typedef Q32SFmt<DT> S;
    Q32SRaw<DT> t;
    const uint32_t r = (uint32_t)(lane & 15);
    t.q0 = ONCE ? ldg_stream<u32x4g>(tile, (uint32_t)lane * 16u) : ldg<u32x4g>(tile, (uint32_t)lane * 16u);
    if (!F::NIB) t.q1 = ONCE ? ldg_stream<u32x4g>(tile, 1024u + (uint32_t)lane * 16u) : ldg<u32x4g>(tile, 1024u + (uint32_t)lane * 16u);
    if (F::FIFTH) t.h = ONCE ? ldg_stream<u32x4g>(tile, S::QB + 16u * r) : ldg<u32x4g>(tile, S::QB + 16u * r);
    if (F::HAS_M) {
        t.dm = ONCE ? ldg_stream<u32x4g>(tile, S::QB + S::HB + 16u * r) : ldg<u32x4g>(tile, S::QB + S::HB + 16u * r);
    } else {
        const u32x2g d = ONCE ? ldg_stream<u32x2g>(tile, S::QB + S::HB + 8u * r) : ldg<u32x2g>(tile, S::QB + S::HB + 8u * r);
        t.dm.x = d.x; t.dm.y = d.y;
    }
    return t;
}
// Block b (compile-time) of a super-tile as an MFMA operand.  Lane (row, g) holds the codes of elements
// 4g .. 4g+3 (low word) and 16+4g .. 16+4g+3 (high word) of the block.
template <int DT, int B>
__device__ __forceinline__ Q32Tile<DT> q32s_block(const Q32SRaw<DT>& raw, int g) {
    typedef Q32Fmt<DT> F;
    Q32Tile<DT> t;
    if (!F::NIB) {
        const u32x4g& q = B < 2 ? raw.q0 : raw.q1;
        t.q = (B & 1) ? make_uint2(q.z, q.w) : make_uint2(q.x, q.y);
    } else {
        const uint32_t w = raw.q0[B];
        uint32_t lo = w & 0x0f0f0f0fu, hi = (w >> 4) & 0x0f0f0f0fu;
        if (F::FIFTH) {   // bit e of the word belongs to element e
            const uint32_t hb = raw.h[B] >> (4 * g);
            lo |= fifth_bits(hb & 15u);
            hi |= fifth_bits((hb >> 16) & 15u);
        }
        t.q = make_uint2(lo, hi);
    }
    if (F::HAS_M) {
        t.d = __half2float(__ushort_as_half((unsigned short)(raw.dm[B] & 0xffffu)));
        t.m = __half2float(__ushort_as_half((unsigned short)(raw.dm[B] >> 16)));
    } else {
        const uint32_t w = B < 2 ? raw.dm.x : raw.dm.y;
        t.d = __half2float(__ushort_as_half((unsigned short)((B & 1) ? (w >> 16) : (w & 0xffffu))));
        t.m = 0.f;
    }
    return t;
}

constexpr int Q32S_ACT_Q = 2048;                  // LDS bytes of one slot tile's quants for one K step
constexpr int Q32S_ACT_BYTES = Q32S_ACT_Q + 512;  // ... and of its 4 x 16 (scale, word) pairs

// Which rows of the activation buffer this thread copies: quants of slot tid / 16 (8 bytes at element 8 (tid % 16) of
// the step), and the (scale, word) pair of slot (tid / 4) % 16, block tid % 4 (the four waves copy the same 64 pairs:
// no divergent branch in the K loop, whose body has to stay one basic block for the scheduler fences to hold).
template <int TT>
struct Q32SRows {
    uint32_t q_row[TT], s_row[TT];
};
template <int TT>
struct Q32SStage {
    u32x2g q[TT];
    float d[TT];
    int w[TT];
};
// Requests step ks of the activations.  A step past the end of K (the K loop runs in whole rounds of its prefetch
// ring) re-reads the last one; q32s_commit zeroes its scale and word, so that its products add +-0.  (Nothing here
// may touch the loaded values: that would wait for the loads where they are issued.)
template <int TT>
__device__ __forceinline__ void q32s_issue(Q32SStage<TT>& st, const Q32SRows<TT>& rows, const ActBuf& ab, int K, int nkb, int ks, int tid) {
    const int nks = K / 128;
    const int kc = ks >= nks ? nks - 1 : ks;
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        st.q[tt] = ldg<u32x2g>(ab.qs, rows.q_row[tt] * (uint32_t)K + (uint32_t)(kc * 128 + 8 * (tid & 15)));
        const uint32_t off = (rows.s_row[tt] * (uint32_t)nkb + (uint32_t)(kc * 4 + (tid & 3))) * 4u;
        st.d[tt] = ldg<float>(ab.d, off);
        st.w[tt] = ldg<int>(ab.bsum, off);
    }
}
// The integer products reach the vector ALU as floats without a conversion: the MFMA's addend is the bit pattern of
// 1.5 * 2^23, so its result, read as a float, is exactly 1.5 * 2^23 + isum (|isum| < 2^22), and
// fma(that, d, -(1.5 * 2^23) * d) = isum * d with one rounding, as (isum as f32) * d has (the subtrahend is exact:
// d has an 11-bit significand).  OFFSET: the format's code offset leaves through the same addend, staged per
// block and slot as magic - OFFSET * (sum of the block's quants).
constexpr int Q32S_MAGIC_BITS = 0x4B400000;
constexpr float Q32S_MAGIC = 12582912.0f;
template <int TT, int OFFSET>
__device__ __forceinline__ void q32s_commit(const Q32SStage<TT>& st, uint8_t* buf, int tid, bool past) {
    const int slot = tid >> 4, c = tid & 15, b = c >> 2, cc = c & 3;
    // elements 8cc .. 8cc+3 of the block belong to chunk g0 = 2 (cc % 2), the next four to chunk g0 + 1; both are the
    // low (cc < 2) or the high half of their lane's operand
    const int at = ((b * 64 + 2 * (cc & 1) * 16 + slot) * 8) + (cc >> 1) * 4;
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        uint8_t* base = buf + tt * Q32S_ACT_BYTES;
        *reinterpret_cast<uint32_t*>(base + at) = st.q[tt].x;
        *reinterpret_cast<uint32_t*>(base + at + 128) = st.q[tt].y;
        const int at_s = Q32S_ACT_Q + ((tid & 3) * 16 + ((tid >> 2) & 15)) * 4;   // [block][slot] scales, then words
        *reinterpret_cast<float*>(base + at_s) = past ? 0.f : st.d[tt];
        *reinterpret_cast<int*>(base + at_s + 256) = OFFSET ? Q32S_MAGIC_BITS - st.w[tt] * OFFSET : (past ? 0 : st.w[tt]);
    }
}

template <int DT>
__device__ __forceinline__ void q32s_mac(const Q32Tile<DT>& w, uint2 a, const f32x4g& yd, const v4i& wd, float acc[4]) {
    const v4i magic = {Q32S_MAGIC_BITS, Q32S_MAGIC_BITS, Q32S_MAGIC_BITS, Q32S_MAGIC_BITS};
    const long av = (long)(((uint64_t)a.y << 32) | a.x);
    const long bv = (long)(((uint64_t)w.q.y << 32) | w.q.x);
    v4i D = __builtin_amdgcn_mfma_i32_16x16x32_i8(av, bv, Q32Fmt<DT>::OFFSET ? wd : magic, 0, 0, 0);
    const float c = -(Q32S_MAGIC * w.d);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float t = __builtin_fmaf(__int_as_float(D[i]), w.d, c);
        t = t * yd[i];
        if (Q32Fmt<DT>::HAS_M) t = t + w.m * __int_as_float(wd[i]);   // the word holds the activation block's s
        acc[i] += t;
    }
}

// Block B of the step: every slot tile's operand and scales from LDS against the NT weight tiles.
template <int DT, int TT, int NT, int B>
__device__ __forceinline__ void q32s_step(const Q32SRaw<DT> (&cur)[NT], const uint8_t* buf, int lane, float acc[NT][TT][4]) {
    const int g = lane >> 4;
    Q32Tile<DT> w[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) w[t] = q32s_block<DT, B>(cur[t], g);
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        const uint8_t* base = buf + tt * Q32S_ACT_BYTES;
        const uint2 a = *reinterpret_cast<const uint2*>(base + (B * 64 + lane) * 8);
        const f32x4g yd = *reinterpret_cast<const f32x4g*>(base + Q32S_ACT_Q + (B * 16 + 4 * g) * 4);
        v4i wd = {0, 0, 0, 0};
        if (Q32Fmt<DT>::OFFSET || Q32Fmt<DT>::HAS_M) wd = *reinterpret_cast<const v4i*>(base + Q32S_ACT_Q + 256 + (B * 16 + 4 * g) * 4);
#pragma unroll
        for (int t = 0; t < NT; t++) q32s_mac<DT>(w[t], a, yd, wd, acc[t][tt]);
    }
    __builtin_amdgcn_sched_barrier(0);
}

// One wave: NT super-tile streams (tp[t], advancing `stride` bytes per K step) against the workgroup's TT slot tiles,
// all of K.  Every thread of the workgroup must call it (barriers).  D = steps the weights and the activations are
// requested ahead (register rings; the K loop is unrolled D times so that ring positions are compile-time).  A wave
// with one weight stream does little arithmetic per step, so only a deep ring keeps enough bytes in flight.
template <int DT, int TT, int NT, bool ONCE, int D>
__device__ __forceinline__ void q32s_engine(const uint8_t* const tp[NT], size_t stride, const ActBuf& ab, int K, const Q32SRows<TT>& rows,
                                            uint8_t* act_lds, int tid, float acc[NT][TT][4]) {
    const int lane = tid & 63;
    const int nkb = K / 32, nks = K / 128;
    Q32SStage<TT> st[D];
    Q32SRaw<DT> ring[D][NT];
#pragma unroll
    for (int j = 0; j < D; j++) {
        q32s_issue<TT>(st[j], rows, ab, K, nkb, j, tid);
        // past the end the last step is requested again (no branch around a load)
#pragma unroll
        for (int t = 0; t < NT; t++) ring[j][t] = load_q32s<DT, ONCE>(tp[t] + (size_t)(j < nks ? j : nks - 1) * stride, lane);
    }
    q32s_commit<TT, Q32Fmt<DT>::OFFSET>(st[0], act_lds, tid, false);
    q32s_issue<TT>(st[0], rows, ab, K, nkb, D, tid);
    __syncthreads();
    for (int ks0 = 0; ks0 < nks; ks0 += D) {
#pragma unroll
        for (int j = 0; j < D; j++) {
            const int ks = ks0 + j;
            Q32SRaw<DT> cur[NT];
            const int ksn = ks + D < nks ? ks + D : nks - 1;
#pragma unroll
            for (int t = 0; t < NT; t++) { cur[t] = ring[j][t]; ring[j][t] = load_q32s<DT, ONCE>(tp[t] + (size_t)ksn * stride, lane); }
            __builtin_amdgcn_sched_barrier(0);
            const uint8_t* buf = act_lds + (ks & 1) * (TT * Q32S_ACT_BYTES);
            q32s_step<DT, TT, NT, 0>(cur, buf, lane, acc);
            q32s_step<DT, TT, NT, 1>(cur, buf, lane, acc);
            q32s_step<DT, TT, NT, 2>(cur, buf, lane, acc);
            q32s_step<DT, TT, NT, 3>(cur, buf, lane, acc);
            __builtin_amdgcn_sched_barrier(0);
            // step ks + 1 goes into the other buffer (nobody reads it before the barrier below), its ring position
            // takes the request for step ks + 1 + D
            q32s_commit<TT, Q32Fmt<DT>::OFFSET>(st[(j + 1) % D], act_lds + ((ks + 1) & 1) * (TT * Q32S_ACT_BYTES), tid, ks + 1 >= nks);
            q32s_issue<TT>(st[(j + 1) % D], rows, ab, K, nkb, ks + 1 + D, tid);
            __syncthreads();
        }
    }
}

// (a fixed number of waves per SIMD also makes the compiler keep the MFMA results in ordinary registers)
template <int DT, int TT, bool ONCE, int WPE, int DEPTH>
__global__ __launch_bounds__(Q32_THREADS) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void q32s_up_kernel(ExpertParams p) {
    __shared__ int list_lds[DIRECT_MAX_SLOTS];
    __shared__ int wtot_lds[Q32_THREADS / 64];
    __shared__ __align__(16) uint8_t act_lds[2 * TT * Q32S_ACT_BYTES];
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = blockIdx.y;
    const GroupSlots gs = group_slots<Q32_THREADS>(p, grp, list_lds, wtot_lds);
    const int tg0 = blockIdx.z * (TT * 16);
    if (tg0 >= gs.n) return;
    const int H = p.H, F = p.F, n_rt = F / 16;
    int rt0 = (blockIdx.x * (Q32_THREADS / 64) + wave) * 2;
    const bool live = rt0 < n_rt;      // a wave past the last rows still stages activations and meets the barriers
    if (!live) rt0 = 0;
    constexpr size_t STB = Q32SFmt<DT>::STB;

    Q32SRows<TT> st;
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        const int iq = tg0 + tt * 16 + (tid >> 4), is = tg0 + tt * 16 + ((tid >> 2) & 15);
        st.q_row[tt] = (uint32_t)slot_token(p, gs.slot(iq < gs.n ? iq : gs.n - 1));
        st.s_row[tt] = (uint32_t)slot_token(p, gs.slot(is < gs.n ? is : gs.n - 1));
    }
    const GroupWeights gw = p.groups[grp];
    const uint8_t* tp[4] = {gw.w1 + (size_t)rt0 * STB, gw.w1 + (size_t)(rt0 + 1) * STB,
                            gw.w3 + (size_t)rt0 * STB, gw.w3 + (size_t)(rt0 + 1) * STB};
    float acc[4][TT][4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int tt = 0; tt < TT; tt++)
#pragma unroll
            for (int i = 0; i < 4; i++) acc[j][tt][i] = 0.f;

    q32s_engine<DT, TT, 4, ONCE, DEPTH>(tp, (size_t)n_rt * STB, p.xq, H, st, act_lds, tid, acc);
    if (!live) return;

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
            int q0 = round_as_i8(h0 * id), q1 = round_as_i8(h1 * id);
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

template <int DT, int TT, bool ONCE, int WPE, int DEPTH>
__global__ __launch_bounds__(Q32_THREADS) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void q32s_down_kernel(ExpertParams p) {
    __shared__ int list_lds[DIRECT_MAX_SLOTS];
    __shared__ int wtot_lds[Q32_THREADS / 64];
    __shared__ __align__(16) uint8_t act_lds[2 * TT * Q32S_ACT_BYTES];
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = blockIdx.y;
    const GroupSlots gs = group_slots<Q32_THREADS>(p, grp, list_lds, wtot_lds);
    const int tg0 = blockIdx.z * (TT * 16);
    if (tg0 >= gs.n) return;
    const int H = p.H, F = p.F, n_rt = H / 16;
    int rt = blockIdx.x * (Q32_THREADS / 64) + wave;
    const bool live = rt < n_rt;
    if (!live) rt = 0;
    constexpr size_t STB = Q32SFmt<DT>::STB;

    Q32SRows<TT> st;
#pragma unroll
    for (int tt = 0; tt < TT; tt++) {
        const int iq = tg0 + tt * 16 + (tid >> 4), is = tg0 + tt * 16 + ((tid >> 2) & 15);
        st.q_row[tt] = (uint32_t)(gs.slot(iq < gs.n ? iq : gs.n - 1) - p.slot_origin);
        st.s_row[tt] = (uint32_t)(gs.slot(is < gs.n ? is : gs.n - 1) - p.slot_origin);
    }
    const uint8_t* tp[1] = {p.groups[grp].w2 + (size_t)rt * STB};
    float acc[1][TT][4];
#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[0][tt][i] = 0.f;

    q32s_engine<DT, TT, 1, ONCE, DEPTH>(tp, (size_t)n_rt * STB, p.hq, F, st, act_lds, tid, acc);
    if (!live) return;

#pragma unroll
    for (int tt = 0; tt < TT; tt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int pos = tg0 + tt * 16 + 4 * g + i;
            if (pos < gs.n) {
                const int slot = gs.slot(pos);
                emit_expert_output(p, slot, rt * 16 + r, acc[0][tt][i] * slot_weight(p, slot));
            }
        }
}

template <int DT, int TT>
static void launch_q32s_up(const ExpertParams& p, dim3 grid, hipStream_t s) {
    // waves per SIMD the register count of each variant allows (the five-bit formats carry their fifth-bit words)
    constexpr bool fat = Q32Fmt<DT>::FIFTH || Q32Fmt<DT>::HAS_M || !Q32Fmt<DT>::NIB;
    constexpr int WPE = TT == 1 ? (fat ? 3 : 4) : (Q32Fmt<DT>::FIFTH ? 2 : 3);
    // one-tile launches are chosen for short lists: a second pass is the exception there, and the stream stays non-temporal
    if (TT == 1 || grid.z == 1) hipLaunchKernelGGL((q32s_up_kernel<DT, TT, true, WPE, 1>), grid, dim3(Q32_THREADS), 0, s, p);
    else hipLaunchKernelGGL((q32s_up_kernel<DT, TT, false, WPE, 1>), grid, dim3(Q32_THREADS), 0, s, p);
}
template <int DT>
static hipError_t launch_q32_up_t(const ExpertParams& p, hipStream_t s) {
    const bool stream = q32_super_layout(p.H);   // the layout of w1 / w3 decides
    const int tt = p.slot_tiles >= 2 ? 2 : 1;
    const int wpb = Q32_THREADS / 64;
    const int n_pairs = p.F / 32;
    dim3 grid((unsigned)((n_pairs + wpb - 1) / wpb), (unsigned)p.n_groups, (unsigned)((p.max_rows + tt * 16 - 1) / (tt * 16)));
    if (stream) {
        if (tt == 1) launch_q32s_up<DT, 1>(p, grid, s);
        else launch_q32s_up<DT, 2>(p, grid, s);
    } else if (tt == 1) {
        hipLaunchKernelGGL((q32_up_kernel<DT, 1>), grid, dim3(Q32_THREADS), 0, s, p);
    } else {
        hipLaunchKernelGGL((q32_up_kernel<DT, 2>), grid, dim3(Q32_THREADS), 0, s, p);
    }
    return hipGetLastError();
}
template <int DT, int TT>
static void launch_q32s_down(const ExpertParams& p, dim3 grid, hipStream_t s) {
    constexpr int WPE = TT == 1 ? (Q32Fmt<DT>::FIFTH ? 3 : 4) : 4;
    if constexpr (TT == 1) {
        // one weight stream per wave: a deep request ring when K is long enough to pay for its prologue
        if (p.F >= 24 * 128) hipLaunchKernelGGL((q32s_down_kernel<DT, 1, true, WPE, 6>), grid, dim3(Q32_THREADS), 0, s, p);
        else hipLaunchKernelGGL((q32s_down_kernel<DT, 1, true, WPE + 1, 2>), grid, dim3(Q32_THREADS), 0, s, p);
    } else if (grid.z == 1) {
        hipLaunchKernelGGL((q32s_down_kernel<DT, TT, true, WPE, 2>), grid, dim3(Q32_THREADS), 0, s, p);
    } else {
        hipLaunchKernelGGL((q32s_down_kernel<DT, TT, false, WPE, 2>), grid, dim3(Q32_THREADS), 0, s, p);
    }
}
template <int DT>
static hipError_t launch_q32_down_t(const ExpertParams& p, hipStream_t s) {
    const bool stream = q32_super_layout(p.F);   // the layout of w2 decides
    const int tt = p.slot_tiles >= 2 ? 2 : 1;
    const int wpb = Q32_THREADS / 64;
    dim3 grid((unsigned)((p.H / 16 + wpb - 1) / wpb), (unsigned)p.n_groups, (unsigned)((p.max_rows + tt * 16 - 1) / (tt * 16)));
    if (stream) {
        if (tt == 1) launch_q32s_down<DT, 1>(p, grid, s);
        else launch_q32s_down<DT, 2>(p, grid, s);
    } else if (tt == 1) {
        hipLaunchKernelGGL((q32_down_kernel<DT, 1>), grid, dim3(Q32_THREADS), 0, s, p);
    } else {
        hipLaunchKernelGGL((q32_down_kernel<DT, 2>), grid, dim3(Q32_THREADS), 0, s, p);
    }
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// Tiled grouped products for Q8_0 weights, and for Q4_0 / Q5_0 / Q4_1 / Q5_1 (batches whose slots are grouped by expert): one pass over an expert's
// weights for up to 64 of its slots, where the streaming kernels above take a pass per 32.
//
// Same arithmetic and the same order of additions as q32s_mac (bit-identical results): one
// v_mfma_i32_16x16x32_i8 per 32-element block, its four integers per lane turned into
// ((isum as f32) * d_w) * d_x and added in ascending block order.  Three vector instructions per result and
// block is what exactness costs, so these kernels are bound by the vector ALU, not by HBM; what the tiled
// form buys is one read of the weights per 64 slots and enough independent work per wave to keep that ALU busy.
//
// Work split: a workgroup (8 waves) owns one tile of up to 64 slots of one group (from the dispatch kernel's tile
// list; the always-on expert's tiles follow from the token count) and eight 16-row weight operands, one per wave
// (MODE 0: four of w1 and the same rows of w3; MODE 1: eight of w2).  Per K step of 128 (four blocks, one super-tile
// per wave) the tile's quants go from global memory straight into LDS as 16-byte pieces ([operand][piece][slot], piece
// p = bytes 16p .. 16p+15 of the step: the two dwords of a lane's MFMA operand are 256 bytes apart), with the scales
// of the step's four blocks per slot beside them; both double-buffered, one barrier per step.  16-slot operands past
// the end of the list are skipped, so the work follows the list length in steps of 16.
constexpr int QG_NOP = 4;
constexpr int QG_THREADS = 512;
struct alignas(16) QGemmLds {
    alignas(16) uint8_t q[2][QG_NOP][8][256];       // [buffer][operand][piece][slot m] 16 bytes
    alignas(16) float yd[2][QG_NOP * 16][4];          // [buffer][slot][block of the step]
    alignas(16) int bs[2][QG_NOP * 16][4];            // the blocks' sums of quants (formats with a code offset)
};
__device__ __forceinline__ uint32_t qg_lds_address(const void* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}
// direct global -> LDS load: lane i of the wave writes 16 bytes at lds + 16 i (the issuing wave waits for it with vmcnt)
__device__ __forceinline__ void qg_dma16(const void* gbase, uint32_t voff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(gbase), "s"(lds));
}

// WOPS (MODE 1): 16-slot operands per wave.  With 4 the eight waves hold eight weight operands (128 rows) and every one of
// them takes the tile's four slot operands; with 2 (1) they hold four (two) weight operands, 64 (32) rows, and split
// the slot operands between them: a grid of few tiles -- the always-on expert's down projection, 16 row blocks of 128 x 8
// tiles at 512 tokens of 2048 -- becomes twice (four times) as many workgroups, each of half (a quarter of) the length.
template <int DT, int MODE, int WOPS = QG_NOP>
__global__ __launch_bounds__(QG_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void q8_0_gemm_kernel(ExpertParams p) {
    static_assert(DT == MOE_GGML_Q8_0 || DT == MOE_GGML_Q4_0 || DT == MOE_GGML_Q5_0 || DT == MOE_GGML_Q4_1 || DT == MOE_GGML_Q5_1, "the 32-element formats");
    static_assert(MODE == 1 || WOPS == QG_NOP, "the up projection pairs w1 and w3 waves");
    constexpr int RTW = 8 * WOPS / QG_NOP;   // MODE 1: weight operands (16 rows) per workgroup
    constexpr int OFFSET = Q32Fmt<DT>::OFFSET;
    constexpr bool HAS_M = Q32Fmt<DT>::HAS_M;    // Q4_1 / Q5_1: the block minimum times the activation block's s (Q8_1 rows)
    constexpr bool WORDS = OFFSET != 0 || HAS_M;   // the activation blocks' words (sum of quants, or s) are staged too
    constexpr size_t STB = Q32SFmt<DT>::STB;
    __shared__ QGemmLds L;
    __shared__ float hx[MODE == 0 ? QG_NOP * 16 : 1][MODE == 0 ? 65 : 1];   // MODE 0: h of the tile's slots x the workgroup's 64 rows
    __shared__ uint64_t exp_tab[MODE == 0 ? 32 : 1];
    const int tid = threadIdx.x, lane = tid & 63;
    if (MODE == 0 && tid < 32) exp_tab[tid] = exp2f_tab(tid);   // published by the barrier ahead of the K loop
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // workgroup -> (row block, slot tile), in patches per XCD (patch_position)
    const int n_rb = MODE == 0 ? p.F / 64 : p.H / (16 * RTW);
    const PatchPos pp = patch_position((int)blockIdx.x, n_rb, p.patch);
    const int rblk = pp.rblk, tile = pp.tile;
    if (rblk >= n_rb) return;
    int gi, pos0;
    if (p.is_shared) {   // one group holding every token: its tiles need no list
        gi = p.group0; pos0 = tile * (QG_NOP * 16);
        if (pos0 >= p.rb.T) return;
    } else {
        if (tile >= p.rb.tile_tab[0]) return;
        gi = p.rb.tile_tab[1 + 2 * tile]; pos0 = p.rb.tile_tab[2 + 2 * tile];
        if (gi < p.group0 || gi >= p.group0 + p.n_groups) return;
    }
    const int grp = gi - p.group0;
    const int s_begin = p.rb.offsets[gi], n_g = p.rb.offsets[gi + 1] - s_begin;
    const int n_here = n_g - pos0 < QG_NOP * 16 ? n_g - pos0 : QG_NOP * 16;   // slots of this tile
    const int n_op = __builtin_amdgcn_readfirstlane((n_here + 15) >> 4);       // live 16-slot operands
    const int K = MODE == 0 ? p.H : p.F;
    const int N = MODE == 0 ? p.F : p.H;
    const int nks = K / 128, nkb = K / 32;
    const size_t step_stride = (size_t)(N / 16) * STB;
    const ActBuf& ab = MODE == 0 ? p.xq : p.hq;

    auto act_row = [&](int r) {   // positions past the list repeat its last row (read, never stored)
        const int pos = pos0 + r;
        const int slot = s_begin + (pos < n_g ? pos : n_g - 1);
        return MODE == 0 ? p.rb.perm_token[slot] : slot - p.slot_origin;
    };
    // Row r of a 16-slot operand holds the tile's position 4 (r % 4) + r / 4, so that a lane's result register i (rows
    // 4 g + i of the matrix instruction's output) covers positions 4 i .. 4 i + 3: the result arithmetic of a short last
    // operand then follows the list length in steps of four slots, not sixteen.
    auto pos_of_row = [](int r) { return (r & ~15) + ((r & 3) << 2) + ((r >> 2) & 3); };
    // transfers of a step: wave w stages half w % 2 (pieces 4 (w % 2) .. +3) of operand w / 2; wave 0 also the scales
    const uint32_t q_src = (uint32_t)act_row(pos_of_row(16 * (wave >> 1) + (lane & 15))) * (uint32_t)K + (uint32_t)((4 * (wave & 1) + (lane >> 4)) * 16);
    const uint32_t d_src = (uint32_t)act_row(pos_of_row(lane)) * (uint32_t)nkb * 4u;
    auto stage = [&](int ks, int buf) {
        qg_dma16(ab.qs, q_src + (uint32_t)(ks * 128), qg_lds_address(&L.q[buf][wave >> 1][4 * (wave & 1)][0]));
        if (wave == 0) qg_dma16(ab.d, d_src + (uint32_t)(ks * 16), qg_lds_address(&L.yd[buf][0][0]));
        if (WORDS && wave == 1) qg_dma16(ab.bsum, d_src + (uint32_t)(ks * 16), qg_lds_address(&L.bs[buf][0][0]));
    };

    const GroupWeights gw = p.groups[grp];
    const uint8_t* wp;
    int row0;
    if (MODE == 0) {
        row0 = rblk * 64 + (wave & 3) * 16;
        wp = (wave < 4 ? gw.w1 : gw.w3) + (size_t)(row0 / 16) * STB;
    } else {
        row0 = rblk * (16 * RTW) + (wave % RTW) * 16;
        wp = gw.w2 + (size_t)(row0 / 16) * STB;
    }
    const int ob = MODE == 0 ? 0 : (wave / RTW) * WOPS;   // the wave's first slot operand
    const int m = lane & 15, g = lane >> 4;
    float acc[WOPS][4];
#pragma unroll
    for (int o = 0; o < WOPS; o++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[o][i] = 0.f;

    stage(0, 0);
    Q32SRaw<DT> cur = load_q32s<DT, false>(wp, lane);
    Q32SRaw<DT> nxt = load_q32s<DT, false>(wp + (size_t)(1 < nks ? 1 : 0) * step_stride, lane);
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    __syncthreads();
    const v4i magic = {Q32S_MAGIC_BITS, Q32S_MAGIC_BITS, Q32S_MAGIC_BITS, Q32S_MAGIC_BITS};
    const int last_regs = __builtin_amdgcn_readfirstlane((n_here - 16 * (n_op - 1) + 3) >> 2);   // live result registers of the last operand
    for (int ks = 0; ks < nks; ks++) {
        const int buf = ks & 1;
        const int ks1 = ks + 1 < nks ? ks + 1 : ks, ks2 = ks + 2 < nks ? ks + 2 : nks - 1;
        stage(ks1, buf ^ 1);
        const Q32SRaw<DT> w = cur;
        cur = nxt;
        nxt = load_q32s<DT, false>(wp + (size_t)ks2 * step_stride, lane);
        const Q32Tile<DT> w0 = q32s_block<DT, 0>(w, g), w1 = q32s_block<DT, 1>(w, g), w2 = q32s_block<DT, 2>(w, g), w3 = q32s_block<DT, 3>(w, g);
        const float dwv[4] = {w0.d, w1.d, w2.d, w3.d};
        const float wm[4] = {w0.m, w1.m, w2.m, w3.m};
        const uint2 wq[4] = {w0.q, w1.q, w2.q, w3.q};
        float cneg[4];
#pragma unroll
        for (int b = 0; b < 4; b++) cneg[b] = -(Q32S_MAGIC * dwv[b]);
#pragma unroll
        for (int ow = 0; ow < WOPS; ow++) {
            const int o = ob + ow;
            if (o < n_op) {   // wave-uniform
                f32x4g ydv[4];
#pragma unroll
                for (int i = 0; i < 4; i++) ydv[i] = *reinterpret_cast<const f32x4g*>(&L.yd[buf][o * 16 + 4 * g + i][0]);
                f32x4g ysv[4];   // the activation blocks' s
                if (HAS_M) {
#pragma unroll
                    for (int i = 0; i < 4; i++) ysv[i] = *reinterpret_cast<const f32x4g*>(&L.bs[buf][o * 16 + 4 * g + i][0]);
                }
                v4i D[4];
                __builtin_amdgcn_s_setprio(2);   // issue priority while the matrix instructions go out (as in q4k_gemm_kernel)
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const uint8_t* ap = &L.q[buf][o][2 * b][0] + m * 16 + 4 * g;
                    const uint32_t alo = *reinterpret_cast<const uint32_t*>(ap), ahi = *reinterpret_cast<const uint32_t*>(ap + 256);
                    const long av = (long)(((uint64_t)ahi << 32) | alo);
                    const long bv = (long)(((uint64_t)wq[b].y << 32) | wq[b].x);
                    v4i addend = magic;
                    if (OFFSET) {   // stored code = value + OFFSET: the block's sum of quants leaves through the addend
#pragma unroll
                        for (int i = 0; i < 4; i++) addend[i] = Q32S_MAGIC_BITS - OFFSET * L.bs[buf][o * 16 + 4 * g + i][b];
                    }
                    D[b] = __builtin_amdgcn_mfma_i32_16x16x32_i8(av, bv, addend, 0, 0, 0);
                }
                __builtin_amdgcn_s_setprio(0);
                // ascending block order per (row, slot), every product rounded where the reference rounds it; result
                // registers beyond the end of the list are left alone
                const int regs = o + 1 < n_op ? 4 : last_regs;
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (i < regs) {   // wave-uniform
#pragma unroll
                        for (int b = 0; b < 4; b++) {
                            float t = __builtin_fmaf(__int_as_float(D[b][i]), dwv[b], cneg[b]);
                            t = t * ydv[i][b];
                            if (HAS_M) t = t + wm[b] * ysv[i][b];   // (isum d_w) d_x + m_w s_x, then the sum (k_quants.rs:294-295)
                            acc[ow][i] += t;
                        }
                    }
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);   // the next step's transfers (and tiles) have landed
        __syncthreads();
    }

    // epilogue: lane holds weight row n = lane % 16 and the tile's positions 16 o + 4 i + lane / 16
    const int n = lane & 15;
    if (MODE == 0) {
        // Wave w < 4 holds w1 x of 16 rows, wave w + 4 holds w3 x of the same rows.  Each of the two parks half of its sums
        // in LDS (the staging buffers are free now) and combines the other half: the w1 wave slot operands 0 and 1, the
        // w3 wave operands 2 and 3 -- a wave's silu evaluations are a chain of dependent double-precision operations, and
        // eight waves carry eight of them each instead of four waves sixteen.
        float* xch = reinterpret_cast<float*>(&L.q[0][0][0][0]);   // [8 waves][2 operands][4 i][64 lanes] floats
        static_assert(8 * 2 * 4 * 64 * 4 <= sizeof(L.q) && QG_NOP == 4, "exchange area");
#pragma unroll
        for (int oo = 0; oo < 2; oo++)
#pragma unroll
            for (int i = 0; i < 4; i++) xch[((wave * 2 + oo) * 4 + i) * 64 + lane] = wave < 4 ? acc[2 + oo][i] : acc[oo][i];
        __syncthreads();
        const int partner = wave ^ 4;
#pragma unroll
        for (int oo = 0; oo < 2; oo++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float other = xch[((partner * 2 + oo) * 4 + i) * 64 + lane];
                const int o = (wave < 4 ? 0 : 2) + oo;
                // silu(w1 x) * (w3 x): the operand this wave kept, times / under the partner's
                const float gate_v = wave < 4 ? acc[oo][i] : other, up_v = wave < 4 ? other : acc[2 + oo][i];
                hx[o * 16 + 4 * i + g][(wave & 3) * 16 + n] = silu_ref32(gate_v, exp_tab) * up_v;
            }
        __syncthreads();
        // Q8_0 blocks of h (BlockQ8_0::from_float, k_quants.rs:605-634): the workgroup's 64 rows are two blocks per slot;
        // half a wave quantises one (slot, block)
        const int nfb = p.F / 32;
#pragma unroll
        for (int it = 0; it < QG_NOP * 16 * 2 / 16; it++) {
            const int pair = (wave * (QG_NOP * 2) + it) * 2 + (lane >> 5);
            const int slot_in_tile = pair >> 1, blk = pair & 1, e = lane & 31;
            const float x = hx[slot_in_tile][blk * 32 + e];
            float amax = fabsf(x);
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
            const float d = amax / 127.0f;
            const float id = (d != 0.f) ? 1.0f / d : 0.f;
            const int q = round_as_i8(x * id);
            int sum = q;
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
            if (slot_in_tile < n_here) {
                const int64_t hrow = s_begin + pos0 + slot_in_tile - p.slot_origin;
                p.hq.qs[hrow * p.F + rblk * 64 + blk * 32 + e] = (int8_t)q;
                if (e == 0) {
                    const float dh = __half2float(__float2half_rn(d));
                    p.hq.d[hrow * nfb + rblk * 2 + blk] = dh;
                    reinterpret_cast<int32_t*>(p.hq.bsum)[hrow * nfb + rblk * 2 + blk] = q8_block_word(vecdot_dtype(DT), sum, dh);
                }
            }
        }
    } else {
#pragma unroll
        for (int ow = 0; ow < WOPS; ow++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int pos = (ob + ow) * 16 + i * 4 + g;
                if (pos >= n_here) continue;
                const int slot = s_begin + pos0 + pos;
                p.yw[(int64_t)slot * p.H + row0 + n] = acc[ow][i] * p.rb.perm_w[slot];
            }
    }
}

static bool qg_format(int dt) { return dt == MOE_GGML_Q8_0 || dt == MOE_GGML_Q4_0 || dt == MOE_GGML_Q5_0 || dt == MOE_GGML_Q4_1 || dt == MOE_GGML_Q5_1; }
bool q8_0_gemm_usable(int dt, int dt_down, int64_t H, int64_t F) {
    return qg_format(dt) && (dt_down == 0 || qg_format(dt_down)) && H % 128 == 0 && F % 128 == 0;
}
static int64_t qg_tiles(const ExpertParams& p) {
    return p.is_shared ? (p.max_rows + QG_NOP * 16 - 1) / (QG_NOP * 16) : max_gemm_tiles(p.n_slots, p.n_groups + 1, QG_NOP * 16);
}
template <int MODE, int WOPS = QG_NOP>
static hipError_t qg_launch(int dt, const ExpertParams& p, dim3 grid, hipStream_t s) {
    switch (dt) {
        case MOE_GGML_Q8_0: hipLaunchKernelGGL((q8_0_gemm_kernel<MOE_GGML_Q8_0, MODE, WOPS>), grid, dim3(QG_THREADS), 0, s, p); break;
        case MOE_GGML_Q4_0: hipLaunchKernelGGL((q8_0_gemm_kernel<MOE_GGML_Q4_0, MODE, WOPS>), grid, dim3(QG_THREADS), 0, s, p); break;
        case MOE_GGML_Q5_0: hipLaunchKernelGGL((q8_0_gemm_kernel<MOE_GGML_Q5_0, MODE, WOPS>), grid, dim3(QG_THREADS), 0, s, p); break;
        case MOE_GGML_Q4_1: hipLaunchKernelGGL((q8_0_gemm_kernel<MOE_GGML_Q4_1, MODE, WOPS>), grid, dim3(QG_THREADS), 0, s, p); break;
        case MOE_GGML_Q5_1: hipLaunchKernelGGL((q8_0_gemm_kernel<MOE_GGML_Q5_1, MODE, WOPS>), grid, dim3(QG_THREADS), 0, s, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}
hipError_t launch_q8_0_gemm_up(const ExpertParams& p_in, hipStream_t s) {
    if (p_in.max_rows == 0 || p_in.n_groups == 0) return hipSuccess;
    ExpertParams p = p_in;
    p.patch = p.is_shared ? patch_all_tiles(p.F / 64, qg_tiles(p)) : patch_edge(p.F / 64, qg_tiles(p));
    return qg_launch<0>(p.dt, p, dim3(patch_grid(p.F / 64, qg_tiles(p), p.patch)), s);
}
hipError_t launch_q8_0_gemm_down(const ExpertParams& p_in, hipStream_t s) {
    if (p_in.max_rows == 0 || p_in.n_groups == 0) return hipSuccess;
    ExpertParams p = p_in;
    const int dt = p.dt_down ? p.dt_down : p.dt;
    const int64_t tiles = qg_tiles(p);
    // fewer than a workgroup per CU: narrower workgroups (64 or 32 rows), whose waves split the slot operands
    const int rows = (p.H / 128) * tiles >= 256 ? 128 : (p.H / 64) * tiles >= 256 ? 64 : 32;
    p.patch = p.is_shared ? patch_all_tiles(p.H / rows, tiles) : patch_edge(p.H / rows, tiles);
    const dim3 grid(patch_grid(p.H / rows, tiles, p.patch));
    return rows == 128 ? qg_launch<1, 4>(dt, p, grid, s) : rows == 64 ? qg_launch<1, 2>(dt, p, grid, s) : qg_launch<1, 1>(dt, p, grid, s);
}

// ---------------------------------------------------------------------------------------------
// Dense matrix (super-tile layout) times one to four rows in one launch, for single-stream decoding.  The streaming down
// kernel gives a row tile to one wave, which walks all of K -- 256 waves for a matrix of 4096 rows -- because the
// reference adds a row's block values in ascending block order and the results have to carry the same bits.  Here the four
// waves of a workgroup share a row tile's K all the same: they compute the block values ((isum as f32) * d_w) * d_x
// (+ m_w * s_x) in parallel, 64 blocks at a time, and park them in LDS; one wave then adds them to the running sums in
// block order.  The rows are quantised inside the kernel (BlockQ8_0 / BlockQ8_1::from_float, k_quants.rs:605-634, 700-729:
// the arithmetic of quantize_q8_0_block, eight pairs of blocks side by side), each wave the blocks it multiplies.
// Maximum / sum over the 32 lanes that hold one block, left in all of them: four rotations inside the rows of 16 lanes
// (DPP: no LDS traffic, no address arithmetic) and one exchange between the two rows.
__device__ __forceinline__ float block32_max(float v) {
#define GV_ROR_MAX(n) v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x120 + (n), 0xf, 0xf, false)))
    GV_ROR_MAX(8); GV_ROR_MAX(4); GV_ROR_MAX(2); GV_ROR_MAX(1);
#undef GV_ROR_MAX
    return fmaxf(v, __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401f)));   // lane ^ 16
}
__device__ __forceinline__ int block32_sum(int v) {
#define GV_ROR_ADD(n) v += __builtin_amdgcn_update_dpp(0, v, 0x120 + (n), 0xf, 0xf, false)
    GV_ROR_ADD(8); GV_ROR_ADD(4); GV_ROR_ADD(2); GV_ROR_ADD(1);
#undef GV_ROR_ADD
    return v + __builtin_amdgcn_ds_swizzle(v, 0x401f);
}

constexpr int GV_MAX_ROWS = 4;
constexpr int GV_STEPS = 4;                     // K steps (of four blocks) a wave takes per chunk
constexpr int GV_BLOCKS = 4 * GV_STEPS;         // blocks per wave and chunk
constexpr int GV_CHUNK = 4 * GV_BLOCKS;         // blocks per workgroup and chunk

template <int DT, bool QUANTISED>
__global__ __launch_bounds__(256) void q32_rows_fused_kernel(FusedRows f) {
    typedef Q32Fmt<DT> F;
    const float* x = f.x;
    const int m = (int)f.m, n = (int)f.n, K = (int)f.k;
    const uint8_t* w = blockIdx.y ? f.w_b : f.w;
    float* y = blockIdx.y ? f.y_b : f.y;
    constexpr size_t STB = Q32SFmt<DT>::STB;
    constexpr int VDT = F::HAS_M ? MOE_GGML_Q8_1 : MOE_GGML_Q8_0;
    __shared__ float terms[2][GV_CHUNK][4][16];                       // [buffer][block of the chunk][row of x][weight row]
    __shared__ __align__(16) int8_t xq[4][GV_BLOCKS][GV_MAX_ROWS][32];  // [wave][block][row]: quants
    __shared__ float xd[4][GV_BLOCKS][GV_MAX_ROWS];
    __shared__ int32_t xw[4][GV_BLOCKS][GV_MAX_ROWS];
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n_rt = n / 16, nks = K / 128, nkb = K / 32;
    const int rt = blockIdx.x;
    const uint8_t* tp = w + (size_t)rt * STB;
    const size_t step_stride = (size_t)n_rt * STB;
    const int n_chunks = (nks + 4 * GV_STEPS - 1) / (4 * GV_STEPS);
    const int my_row = r < m ? r : m - 1;
    float acc = 0.f;   // wave 0: lane (weight row r, row g of x)
    // weights of the wave's steps of a chunk: requested a chunk ahead, the rows are quantised while they travel
    Q32SRaw<DT> raw[GV_STEPS];
    auto request = [&](int c) {
#pragma unroll
        for (int st = 0; st < GV_STEPS; st++) {
            int ks = c * 4 * GV_STEPS + wave * GV_STEPS + st;
            ks = ks < nks ? ks : nks - 1;
            raw[st] = load_q32s<DT, true>(tp + (size_t)ks * step_stride, lane);
        }
    };
    request(0);
    auto fetch = [&](uint32_t off) {
        float a = ldg<float>(x, off);
        if (f.x2) a *= ldg<float>(f.x2, off);
        return a;
    };
    float xnext[8];
    // rows that arrive quantised: per row and chunk a lane copies 8 quants of the wave's 512, lanes 0..15 a block's scale
    // and word; requested a chunk ahead like the weights
    uint2 qnext[GV_MAX_ROWS];
    float dnext[GV_MAX_ROWS];
    int wnext[GV_MAX_ROWS];
    auto request_rows = [&](int ks0) {
        const int e = ks0 * 128 + lane * 8;
        const int b = ks0 * 4 + (lane & 15);
#pragma unroll
        for (int row = 0; row < GV_MAX_ROWS; row++) {
            const size_t rr = (size_t)(row < m ? row : m - 1);
            qnext[row] = *reinterpret_cast<const uint2*>(f.xq.qs + rr * K + (e < K ? e : K - 8));
            dnext[row] = f.xq.d[rr * nkb + (b < nkb ? b : nkb - 1)];
            wnext[row] = static_cast<const int32_t*>(f.xq.bsum)[rr * nkb + (b < nkb ? b : nkb - 1)];
        }
    };
    if constexpr (QUANTISED) {
        request_rows(wave * GV_STEPS);
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int e = wave * GV_STEPS * 128 + j * 64 + lane;
            xnext[j] = fetch((uint32_t)(e < K ? e : K - 1) * 4u);
        }
    }
    for (int c = 0; c < n_chunks; c++) {
        const int ks0 = c * 4 * GV_STEPS + wave * GV_STEPS;       // this wave's first K step of the chunk
        const int n_steps = nks - ks0 < GV_STEPS ? (nks - ks0 < 0 ? 0 : nks - ks0) : GV_STEPS;
        if constexpr (QUANTISED) {
            uint2 qc[GV_MAX_ROWS];
            float dc[GV_MAX_ROWS];
            int wc[GV_MAX_ROWS];
#pragma unroll
            for (int row = 0; row < GV_MAX_ROWS; row++) { qc[row] = qnext[row]; dc[row] = dnext[row]; wc[row] = wnext[row]; }
            request_rows(ks0 + 4 * GV_STEPS);
#pragma unroll
            for (int row = 0; row < GV_MAX_ROWS; row++) {
                if (row < m) {   // uniform
                    *reinterpret_cast<uint2*>(&xq[wave][lane >> 2][row][(lane & 3) * 8]) = qc[row];
                    if (lane < GV_BLOCKS) {
                        xd[wave][lane][row] = dc[row];
                        xw[wave][lane][row] = wc[row];
                    }
                }
            }
        } else
        // the rows' blocks of these steps: 512 elements per row, lane l holds elements l, l + 64, ... (pair of blocks j)
        for (int row = 0; row < m; row++) {
            float xv[8];
#pragma unroll
            for (int j = 0; j < 8; j++) xv[j] = xnext[j];
            {   // the values of the next row (after the last one: of row 0 of the next chunk) are requested a turn ahead
                const int nrow = row + 1 < m ? row + 1 : 0;
                const int nks0 = row + 1 < m ? ks0 : ks0 + 4 * GV_STEPS;
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int e = nks0 * 128 + j * 64 + lane;
                    xnext[j] = fetch(((uint32_t)nrow * (uint32_t)K + (uint32_t)(e < K ? e : K - 1)) * 4u);
                }
            }
            float amax[8];
#pragma unroll
            for (int j = 0; j < 8; j++) amax[j] = fabsf(xv[j]);
#pragma unroll
            for (int j = 0; j < 8; j++) amax[j] = block32_max(amax[j]);
            int q[8], sum[8];
            float d[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                d[j] = amax[j] / 127.0f;
                const float id = (d[j] != 0.f) ? 1.0f / d[j] : 0.f;
                q[j] = round_as_i8(xv[j] * id);
                sum[j] = q[j];
            }
#pragma unroll
            for (int j = 0; j < 8; j++) sum[j] = block32_sum(sum[j]);
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int blk = 2 * j + (lane >> 5);
                xq[wave][blk][row][lane & 31] = (int8_t)q[j];
                if ((lane & 31) == 0) {
                    const float dh = __half2float(__float2half_rn(d[j]));
                    xd[wave][blk][row] = dh;
                    xw[wave][blk][row] = q8_block_word(VDT, sum[j], dh);
                }
            }
        }
        // the wave reads what its other lanes have written: LDS serves a wave's requests in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int buf = c & 1;
#pragma unroll
        for (int st = 0; st < GV_STEPS; st++) {
            if (st < n_steps) {   // uniform
                const Q32Tile<DT> wb[4] = {q32s_block<DT, 0>(raw[st], g), q32s_block<DT, 1>(raw[st], g), q32s_block<DT, 2>(raw[st], g),
                                           q32s_block<DT, 3>(raw[st], g)};
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    const int blk = st * 4 + b;
                    const int8_t* ap = &xq[wave][blk][my_row][0];
                    const uint32_t alo = *reinterpret_cast<const uint32_t*>(ap + 4 * g), ahi = *reinterpret_cast<const uint32_t*>(ap + 16 + 4 * g);
                    const long av = (long)(((uint64_t)ahi << 32) | alo);
                    const long bv = (long)(((uint64_t)wb[b].q.y << 32) | wb[b].q.x);
                    const v4i zero = {0, 0, 0, 0};
                    const v4i D = __builtin_amdgcn_mfma_i32_16x16x32_i8(av, bv, zero, 0, 0, 0);
                    if (g == 0) {   // D[i]: row i of x, weight row r
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            if (i >= m) break;   // uniform
                            const int xr = i;
                            const int word = xw[wave][blk][xr];
                            int isum = D[i];
                            if (F::OFFSET) isum -= F::OFFSET * word;
                            float t = (float)isum * wb[b].d;
                            t = t * xd[wave][blk][xr];
                            if (F::HAS_M) t = t + wb[b].m * __int_as_float(word);   // the word holds the activation block's s
                            terms[buf][wave * GV_BLOCKS + blk][i][r] = t;
                        }
                    }
                }
            }
        }
        if (c + 1 < n_chunks) request(c + 1);
        __syncthreads();
        if (wave == 0) {   // the chunk's block values join the running sums in ascending block order
            const int nb = nkb - c * GV_CHUNK < GV_CHUNK ? nkb - c * GV_CHUNK : GV_CHUNK;
            for (int b = 0; b < nb; b++) acc += terms[buf][b][g][r];
        }
    }
    if (wave == 0 && g < m) {
        if (f.row_scale) acc *= f.row_scale[g];
        if (f.silu_y && blockIdx.y == 0) acc = silu_ref32(acc);
        y[(size_t)g * n + (size_t)rt * 16 + r] = acc;
    }
}

bool q32_rows_fused_usable(int dt, int64_t m, int64_t n, int64_t k) {
    const bool fmt = dt == MOE_GGML_Q8_0 || dt == MOE_GGML_Q4_0 || dt == MOE_GGML_Q5_0 || dt == MOE_GGML_Q4_1 || dt == MOE_GGML_Q5_1;
    return fmt && m >= 1 && m <= GV_MAX_ROWS && n % 16 == 0 && q32_super_layout(k) && k >= 128 && m * k < ((int64_t)1 << 29);
}
template <int DT>
static void launch_q32_rows_fused_t(const FusedRows& f, hipStream_t s) {
    const dim3 grid((unsigned)(f.n / 16), f.w_b ? 2u : 1u), block(256);
    if (f.x) hipLaunchKernelGGL((q32_rows_fused_kernel<DT, false>), grid, block, 0, s, f);
    else hipLaunchKernelGGL((q32_rows_fused_kernel<DT, true>), grid, block, 0, s, f);
}
hipError_t launch_q32_rows_fused(int dt, const FusedRows& f, hipStream_t s) {
    if (!q32_rows_fused_usable(dt, f.m, f.n, f.k) || !(f.x || f.xq.qs) || !f.w || !f.y || (f.w_b && !f.y_b)) return hipErrorInvalidValue;
    switch (dt) {
        case MOE_GGML_Q8_0: launch_q32_rows_fused_t<MOE_GGML_Q8_0>(f, s); break;
        case MOE_GGML_Q4_0: launch_q32_rows_fused_t<MOE_GGML_Q4_0>(f, s); break;
        case MOE_GGML_Q5_0: launch_q32_rows_fused_t<MOE_GGML_Q5_0>(f, s); break;
        case MOE_GGML_Q4_1: launch_q32_rows_fused_t<MOE_GGML_Q4_1>(f, s); break;
        case MOE_GGML_Q5_1: launch_q32_rows_fused_t<MOE_GGML_Q5_1>(f, s); break;
        default: return hipErrorInvalidValue;
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
