// Grouped expert products over Q2K, Q3K, Q4K, Q5K and Q6K weights with Q8K activations (gfx950, wave64, int8 MFMA).
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
// Q6K (BlockQ6K::vec_dot, k_quants.rs:1613-1671): d * y.d * sum_j sc_j * ((code_j - 32) . q8_j) over
// the sixteen 16-element sub-blocks, sc_j an i8.  One v_mfma_i32_16x16x32_i8 spans two sub-blocks with
// different scales, so each is issued twice, with the weight operand of the lane groups that hold the
// other sub-block zeroed; the codes stay unsigned (0..63) and the -32 is taken out through the
// activations' 16-element sums: sum_j sc_j * bsum_j is one exact f16 MFMA (|bsum| <= 2032,
// |sc| <= 128, the sum of sixteen products stays below 2^24).
//
//   q4k_up_kernel    h[slot, f] = silu(W1 x) * (W3 x) for a 256-row block of F, then the block is
//                    quantised to Q8K in the epilogue (Mlp::forward, quantized_llama.rs:124-131;
//                    the re-quantisation is what k_quants::matmul does to the lhs of w2).
//   q4k_down_kernel  yw[slot, :] = (W2 h[slot]) * routing weight (quantized_llama.rs:199-201).
#include <type_traits>
#include <cstdlib>

#include "act_quant.hpp"
#include "kernels.hpp"
#include "slots.hpp"

namespace moe {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

struct Q4KTile {
    uint4 q0, q1, sc;
};

// Loads go through explicit global-address-space pointers made of a wave-uniform base and a 32-bit
// per-lane offset: the base then lives in scalar registers and the instruction is a global (not
// flat) load, which keeps 64-bit addresses out of the vector register file.
typedef const __attribute__((address_space(1))) uint8_t* gbytes;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <typename T>
__device__ inline T gload(const void* uniform_base, uint32_t off) {
    return *reinterpret_cast<const __attribute__((address_space(1))) T*>((gbytes)uniform_base + off);
}
template <>
__device__ inline uint4 gload<uint4>(const void* uniform_base, uint32_t off) {
    u32x4 v = *reinterpret_cast<const __attribute__((address_space(1))) u32x4*>((gbytes)uniform_base + off);
    return make_uint4(v.x, v.y, v.z, v.w);
}

typedef float f32x4 __attribute__((ext_vector_type(4)));
template <>
__device__ inline float4 gload<float4>(const void* uniform_base, uint32_t off) {
    f32x4 v = *reinterpret_cast<const __attribute__((address_space(1))) f32x4*>((gbytes)uniform_base + off);
    return make_float4(v.x, v.y, v.z, v.w);
}

// weight tiles are read once per launch: non-temporal loads keep them from displacing the activations
// and routing lists in the caches
__device__ inline uint4 gload_stream(const void* uniform_base, uint32_t off) {
    u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) u32x4*>((gbytes)uniform_base + off));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ inline Q4KTile load_q4k_tile(const uint8_t* tile, int lane) {
    Q4KTile t;
    t.q0 = gload_stream(tile, (uint32_t)lane * 16u);
    t.q1 = gload_stream(tile, 1024u + (uint32_t)lane * 16u);
    t.sc = gload_stream(tile, 2048u + (uint32_t)(lane & 15) * 16u);
    return t;
}

// Activation operand of one 16-slot tile for one super-block.
struct Q8KOperand {
    uint4 a[4];   // pair P: sub-block 2P (x,y) and 2P+1 (z,w), this lane's 8-element chunk
    v4h bs;       // bsums 4g..4g+3 of the lane's slot (l%16)
    float yd;     // Q8K scale of the lane's own slot (l%16)
};

__device__ inline Q8KOperand load_q8k_operand(const ActBuf& ab, int K, int nsb, int sb, int rowA, int g) {
    Q8KOperand o;
    // uniform base pointers + 32-bit per-lane offsets (rows * K < 2^31 is checked on the host)
    const uint32_t qoff = (uint32_t)rowA * (uint32_t)K + (uint32_t)(sb * 256 + g * 16);
    const uint32_t boff = ((uint32_t)rowA * (uint32_t)nsb + (uint32_t)sb);
#pragma unroll
    for (int P = 0; P < 4; P++) o.a[P] = gload<uint4>(ab.qs, qoff + P * 64);
    o.bs = gload<v4h>(ab.bsum, (boff * 16 + 4 * g) * 2);
    o.yd = gload<float>(ab.d, boff * 4);
    return o;
}

__device__ inline long pack64(uint32_t lo, uint32_t hi) { return (long)(((uint64_t)hi << 32) | lo); }

// acc[i] += contribution of one (16 rows x 256 k) weight tile against one 16-slot operand.
// yd[i] is the activation scale of output slot 4g+i.  FIFTH: the tile is Q5K, h0 / h1 hold the lane's
// fifth bits (pairs 0,1 / 2,3; four bits per byte and pair), else Q4K.
template <bool FIFTH>
__device__ inline void q45k_mac(const uint4& q0, const uint4& q1, const uint4& sc, uint32_t h0, uint32_t h1, const Q8KOperand& A,
                                const float yd[4], int g, float acc[4]) {
    const uint32_t M4 = 0x0f0f0f0fu, M1 = 0x01010101u;
    const uint32_t hdr = sc.x, u0 = sc.y, u1 = sc.z, u2 = sc.w;
    const float d = __half2float(__ushort_as_half((unsigned short)(hdr & 0xffffu)));
    const float dmin = __half2float(__ushort_as_half((unsigned short)(hdr >> 16)));
    // get_scale_min_k4 (utils.rs:50-60) for all eight sub-blocks at once
    const uint32_t sc03 = u0 & 0x3f3f3f3fu;
    const uint32_t sc47 = (u2 & M4) | (((u0 >> 6) & 0x03030303u) << 4);
    const uint32_t m03 = u1 & 0x3f3f3f3fu;
    const uint32_t m47 = ((u2 >> 4) & M4) | (((u1 >> 6) & 0x03030303u) << 4);
    const v4i zero = {0, 0, 0, 0};
    v4i isum = {0, 0, 0, 0};
    const uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
    for (int P = 0; P < 4; P++) {
        const uint32_t wx = qw[2 * P], wy = qw[2 * P + 1];
        uint32_t lx = wx & M4, ly = wy & M4, hx = (wx >> 4) & M4, hy = (wy >> 4) & M4;
        if (FIFTH) {   // codes 0..31: nibble | fifth bit << 4
            const uint32_t h = (P < 2 ? h0 : h1) >> (4 * (P & 1));
            lx |= (h & M1) << 4;
            ly |= ((h >> 1) & M1) << 4;
            hx |= ((h >> 2) & M1) << 4;
            hy |= ((h >> 3) & M1) << 4;
        }
        const long b_lo = pack64(lx, ly);
        const long b_hi = pack64(hx, hy);
        const long a_lo = pack64(A.a[P].x, A.a[P].y);
        const long a_hi = pack64(A.a[P].z, A.a[P].w);
        v4i D0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_lo, b_lo, zero, 0, 0, 0);
        v4i D1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_hi, b_hi, zero, 0, 0, 0);
        const uint32_t scw = (P < 2) ? sc03 : sc47;
        const int s0 = (int)((scw >> (16 * (P & 1))) & 0xffu);
        const int s1 = (int)((scw >> (16 * (P & 1) + 8)) & 0xffu);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // one v_mad_i32_i24 per product: the empty asm keeps the compiler from regrouping the two into two
            // multiplies and a three-way add (1.5 instructions per product)
            isum[i] += __mul24(s0, D0[i]);
            asm("" : "+v"(isum[i]));
            isum[i] += __mul24(s1, D1[i]);
            asm("" : "+v"(isum[i]));
        }
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
        // The reference rounds d_w * d_x first and then each product; (d_w isum - dmin_w mins) d_x with fused
        // multiply-adds would save two instructions per result, but every rounding that differs from the reference's
        // moves more intermediate values across a re-quantisation boundary (measured: the 64-token case of the
        // Mixtral-shape test went from inside to outside the 2e-3 bar).
        const float dd = d * yd[i];
        const float dm = dmin * yd[i];
        acc[i] += dd * (float)isum[i];
        acc[i] -= dm * Dm[i];
    }
}

__device__ inline void q4k_mac(const Q4KTile& w, const Q8KOperand& A, const float yd[4], int g, float acc[4]) {
    q45k_mac<false>(w.q0, w.q1, w.sc, 0u, 0u, A, yd, g, acc);
}

// The same Q4K contribution with the 6-bit scale inside the weight operand, for workgroups that carry two or four
// slot tiles: sc = 8 hi + lo (3-bit digits), the byte planes hi * q4 and lo * q4 (<= 105, packed 16-bit multiplies,
// no carry between bytes) are each multiplied by the activations with v_mfma_i32_16x16x64_i8 (a pair of sub-blocks
// per instruction, its two scales already applied) and accumulated over the super-block; 8 acc_hi + acc_lo is the
// integer of vec_dot.  The planes are built once per weight tile and serve every slot tile, whereas q45k_mac spends
// an integer multiply-add per result and sub-block: 80 + 32 TT vector instructions per tile against 39 + 72 TT.
typedef unsigned short u16x2p __attribute__((ext_vector_type(2)));
__device__ inline uint32_t digit_times_codes(uint32_t q, uint32_t digit) {
    const u16x2p a = __builtin_bit_cast(u16x2p, q);
    const u16x2p b = {(unsigned short)digit, (unsigned short)digit};
    return __builtin_bit_cast(uint32_t, (u16x2p)(a * b));
}
struct Q4KPlanes {
    v4i hi[4], lo[4];   // pair P: operand of one 16x16x64 MFMA (sub-block 2P chunk, sub-block 2P+1 chunk)
    float d, dmin;
    v4h mB;
};
__device__ inline Q4KPlanes q4k_planes(const Q4KTile& w, int g) {
    const uint32_t M4 = 0x0f0f0f0fu;
    Q4KPlanes pl;
    const uint32_t hdr = w.sc.x, u0 = w.sc.y, u1 = w.sc.z, u2 = w.sc.w;
    pl.d = __half2float(__ushort_as_half((unsigned short)(hdr & 0xffffu)));
    pl.dmin = __half2float(__ushort_as_half((unsigned short)(hdr >> 16)));
    const uint32_t sc03 = u0 & 0x3f3f3f3fu;
    const uint32_t sc47 = (u2 & M4) | (((u0 >> 6) & 0x03030303u) << 4);
    const uint32_t m03 = u1 & 0x3f3f3f3fu;
    const uint32_t m47 = ((u2 >> 4) & M4) | (((u1 >> 6) & 0x03030303u) << 4);
    const uint32_t qw[8] = {w.q0.x, w.q0.y, w.q0.z, w.q0.w, w.q1.x, w.q1.y, w.q1.z, w.q1.w};
#pragma unroll
    for (int P = 0; P < 4; P++) {
        const uint32_t wx = qw[2 * P], wy = qw[2 * P + 1];
        const uint32_t lx = wx & M4, ly = wy & M4, hx = (wx >> 4) & M4, hy = (wy >> 4) & M4;
        // the digits of four scales at a time, then one bit-field extract per digit
        const uint32_t scw = (P < 2) ? sc03 : sc47;
        const uint32_t hiw = (scw >> 3) & 0x07070707u, low = scw & 0x07070707u;
        const uint32_t s0h = (hiw >> (16 * (P & 1))) & 0xffu, s1h = (hiw >> (16 * (P & 1) + 8)) & 0xffu;
        const uint32_t s0l = (low >> (16 * (P & 1))) & 0xffu, s1l = (low >> (16 * (P & 1) + 8)) & 0xffu;
        pl.hi[P] = v4i{(int)digit_times_codes(lx, s0h), (int)digit_times_codes(ly, s0h), (int)digit_times_codes(hx, s1h), (int)digit_times_codes(hy, s1h)};
        pl.lo[P] = v4i{(int)digit_times_codes(lx, s0l), (int)digit_times_codes(ly, s0l), (int)digit_times_codes(hx, s1l), (int)digit_times_codes(hy, s1l)};
    }
    const uint32_t mw = (g < 2) ? m03 : m47;
    const _Float16 ma = (_Float16)(int)((mw >> (16 * (g & 1))) & 0xffu);
    const _Float16 mb = (_Float16)(int)((mw >> (16 * (g & 1) + 8)) & 0xffu);
    pl.mB = v4h{ma, ma, mb, mb};
    return pl;
}
__device__ inline void q4k_mac_planes(const Q4KPlanes& pl, const Q8KOperand& A, const float yd[4], float acc[4]) {
    const v4i zero = {0, 0, 0, 0};
    v4i acc_hi = zero, acc_lo = zero;
#pragma unroll
    for (int P = 0; P < 4; P++) {
        const v4i a = {(int)A.a[P].x, (int)A.a[P].y, (int)A.a[P].z, (int)A.a[P].w};
        acc_hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, pl.hi[P], acc_hi, 0, 0, 0);
        acc_lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, pl.lo[P], acc_lo, 0, 0, 0);
    }

    const v4f zf = {0.f, 0.f, 0.f, 0.f};
    v4f Dm = __builtin_amdgcn_mfma_f32_16x16x16f16(A.bs, pl.mB, zf, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float dd = pl.d * yd[i];
        const float dm = pl.dmin * yd[i];
        acc[i] += dd * (float)(8 * acc_hi[i] + acc_lo[i]);
        acc[i] -= dm * Dm[i];
    }
}

// Q5K (BlockQ5K::vec_dot, k_quants.rs:1394-1485): the Q4K arithmetic on 5-bit codes
struct Q5KTile {
    uint4 q0, q1, sc;
    uint2 qh;
};
__device__ inline Q5KTile load_q5k_tile(const uint8_t* tile, int lane) {
    Q5KTile t;
    t.q0 = gload_stream(tile, (uint32_t)lane * 16u);
    t.q1 = gload_stream(tile, 1024u + (uint32_t)lane * 16u);
    t.sc = gload_stream(tile, 2048u + (uint32_t)(lane & 15) * 16u);
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 h = __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) u32x2*>((gbytes)tile + 2304u + (uint32_t)lane * 8u));
    t.qh = make_uint2(h.x, h.y);
    return t;
}
__device__ inline void q5k_mac(const Q5KTile& w, const Q8KOperand& A, const float yd[4], int g, float acc[4]) {
    q45k_mac<true>(w.q0, w.q1, w.sc, w.qh.x, w.qh.y, A, yd, g, acc);
}

// Q2K (BlockQ2K::vec_dot, k_quants.rs:755-805): d * y.d * sum_j sc_j * (code_j . q8_j) - dmin * y.d *
// sum_j min_j * bsum_j over the sixteen 16-element sub-blocks, sc and min four bits each.  sc * code <= 45
// fits a byte, so the scale goes into the weight operand (a lane's eight elements of a 32-element stretch
// lie in one sub-block) and the eight MFMAs of a super-block accumulate into one exact integer.
struct Q2KTile {
    uint4 q, sc;
    uint32_t dd;   // d | dmin << 16 of the lane's row
};
__device__ inline Q2KTile load_q2k_tile(const uint8_t* tile, int lane) {
    Q2KTile t;
    t.q = gload_stream(tile, (uint32_t)lane * 16u);
    t.sc = gload_stream(tile, 1024u + (uint32_t)(lane & 15) * 16u);
    t.dd = __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) uint32_t*>((gbytes)tile + 1280u + (uint32_t)(lane & 15) * 4u));
    return t;
}
// four bytes (each <= 3) times a scale (<= 15) with the packed 16-bit multiply: no byte overflows
typedef unsigned short u16x2s __attribute__((ext_vector_type(2)));
__device__ inline uint32_t scale_codes(uint32_t q, uint32_t s) {
    const u16x2s a = __builtin_bit_cast(u16x2s, q);
    const u16x2s b = {(unsigned short)s, (unsigned short)s};
    return __builtin_bit_cast(uint32_t, (u16x2s)(a * b));
}
__device__ inline void q2k_mac(const Q2KTile& w, const Q8KOperand& A, const float yd[4], int g, float acc[4]) {
    const uint32_t M3 = 0x03030303u;
    const float d = __half2float(__ushort_as_half((unsigned short)(w.dd & 0xffffu)));
    const float dmin = __half2float(__ushort_as_half((unsigned short)(w.dd >> 16)));
    const uint32_t qw[4] = {w.q.x, w.q.y, w.q.z, w.q.w};
    const uint32_t sw[4] = {w.sc.x, w.sc.y, w.sc.z, w.sc.w};
    const int sel = 8 * (g >> 1);   // groups 0,1 hold the first 16 elements of a 32-element stretch, 2,3 the second
    v4i isum = {0, 0, 0, 0};
#pragma unroll
    for (int P = 0; P < 4; P++) {
        const uint32_t q = qw[P];
        const uint32_t s_lo = (sw[P] >> sel) & 0xFu, s_hi = (sw[P] >> (16 + sel)) & 0xFu;
        const long b_lo = pack64(scale_codes(q & M3, s_lo), scale_codes((q >> 2) & M3, s_lo));
        const long b_hi = pack64(scale_codes((q >> 4) & M3, s_hi), scale_codes((q >> 6) & M3, s_hi));
        isum = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(A.a[P].x, A.a[P].y), b_lo, isum, 0, 0, 0);
        isum = __builtin_amdgcn_mfma_i32_16x16x32_i8(pack64(A.a[P].z, A.a[P].w), b_hi, isum, 0, 0, 0);
    }
    // mins term: sum_j min_j * bsum_j as an exact f16 MFMA; this lane supplies sub-blocks 4g..4g+3
    const uint32_t mg = (sw[g] >> 4) & 0x0f0f0f0fu;
    const v4h mB = {(_Float16)(int)(mg & 0xffu), (_Float16)(int)((mg >> 8) & 0xffu), (_Float16)(int)((mg >> 16) & 0xffu), (_Float16)(int)(mg >> 24)};
    const v4f zf = {0.f, 0.f, 0.f, 0.f};
    v4f Dm = __builtin_amdgcn_mfma_f32_16x16x16f16(A.bs, mB, zf, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; i++)   // sumf += dall * isum - dmin * summs, rounded where the reference rounds (k_quants.rs:772-773, 801)
        acc[i] += (yd[i] * d) * (float)isum[i] - (yd[i] * dmin) * Dm[i];
}

struct Q6KTile {
    uint4 q0, q1, qh, sc;
    uint32_t d;   // f16 bits of the lane's row
};
__device__ inline Q6KTile load_q6k_tile(const uint8_t* tile, int lane) {
    Q6KTile t;
    t.q0 = gload_stream(tile, (uint32_t)lane * 16u);
    t.q1 = gload_stream(tile, 1024u + (uint32_t)lane * 16u);
    t.qh = gload_stream(tile, 2048u + (uint32_t)lane * 16u);
    t.sc = gload_stream(tile, 3072u + (uint32_t)(lane & 15) * 16u);
    t.d = __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) uint16_t*>((gbytes)tile + 3328u + (uint32_t)(lane & 15) * 2u));
    return t;
}

// acc[i] += contribution of one (16 rows x 256 k) Q6K tile against one 16-slot operand.
__device__ inline void q6k_mac(const Q6KTile& w, const Q8KOperand& A, const float yd[4], int g, float acc[4]) {
    const uint32_t M4 = 0x0f0f0f0fu, M2 = 0x03030303u;
    const float d = __half2float(__ushort_as_half((unsigned short)w.d));
    // lane groups 0,1 carry elements 0..15 of a 32-element stretch, groups 2,3 elements 16..31
    const uint32_t first = g < 2 ? 0xffffffffu : 0u, second = ~first;
    const v4i zero = {0, 0, 0, 0};
    v4i isum = {0, 0, 0, 0};
    const uint32_t qw[8] = {w.q0.x, w.q0.y, w.q0.z, w.q0.w, w.q1.x, w.q1.y, w.q1.z, w.q1.w};
    const uint32_t hw[4] = {w.qh.x, w.qh.y, w.qh.z, w.qh.w};
    const uint32_t sw[4] = {w.sc.x, w.sc.y, w.sc.z, w.sc.w};
#pragma unroll
    for (int P = 0; P < 4; P++) {
        const uint32_t wx = qw[2 * P], wy = qw[2 * P + 1], h = hw[P];
        const uint32_t lx = (wx & M4) | ((h & M2) << 4), ly = (wy & M4) | (((h >> 2) & M2) << 4);
        const uint32_t hx = ((wx >> 4) & M4) | (((h >> 4) & M2) << 4), hy = ((wy >> 4) & M4) | (((h >> 6) & M2) << 4);
        const long a_lo = pack64(A.a[P].x, A.a[P].y);
        const long a_hi = pack64(A.a[P].z, A.a[P].w);
        // sub-blocks 4P .. 4P+3 (16 elements each)
        v4i D0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_lo, pack64(lx & first, ly & first), zero, 0, 0, 0);
        v4i D1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_lo, pack64(lx & second, ly & second), zero, 0, 0, 0);
        v4i D2 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_hi, pack64(hx & first, hy & first), zero, 0, 0, 0);
        v4i D3 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a_hi, pack64(hx & second, hy & second), zero, 0, 0, 0);
        const int s0 = (int)(int8_t)(sw[P] & 0xffu), s1 = (int)(int8_t)((sw[P] >> 8) & 0xffu);
        const int s2 = (int)(int8_t)((sw[P] >> 16) & 0xffu), s3 = (int)(int8_t)(sw[P] >> 24);
#pragma unroll
        for (int i = 0; i < 4; i++) isum[i] += __mul24(s0, D0[i]) + __mul24(s1, D1[i]) + __mul24(s2, D2[i]) + __mul24(s3, D3[i]);
    }
    // offset term: sum_j sc_j * bsum_j as an exact f16 MFMA; this lane supplies sub-blocks 4g..4g+3
    const uint32_t sg = sw[g];
    const v4h sB = {(_Float16)(int)(int8_t)(sg & 0xffu), (_Float16)(int)(int8_t)((sg >> 8) & 0xffu),
                    (_Float16)(int)(int8_t)((sg >> 16) & 0xffu), (_Float16)(int)(int8_t)(sg >> 24)};
    const v4f zf = {0.f, 0.f, 0.f, 0.f};
    v4f Ds = __builtin_amdgcn_mfma_f32_16x16x16f16(A.bs, sB, zf, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int tot = isum[i] - 32 * (int)Ds[i];   // exact: |tot| < 2^28
        acc[i] += (d * yd[i]) * (float)tot;
    }
}

// Q3K (BlockQ3K::vec_dot, k_quants.rs:927-1045): d * y.d * sum_j (sc_j - 32) * (code_j . q8_j), codes -4..3, one
// signed 6-bit scale per 16 elements: the Q6K scheme with 3-bit unsigned codes (code + 4 = low two bits |
// high bit << 2) and the offset -4 taken out through the activations' 16-element sums.
struct Q3KTile {
    uint4 q, sc;
    uint2 qh;
    uint32_t d;
};
__device__ inline Q3KTile load_q3k_tile(const uint8_t* tile, int lane) {
    Q3KTile t;
    t.q = gload_stream(tile, (uint32_t)lane * 16u);
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 h = __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) u32x2*>((gbytes)tile + 1024u + (uint32_t)lane * 8u));
    t.qh = make_uint2(h.x, h.y);
    t.sc = gload_stream(tile, 1536u + (uint32_t)(lane & 15) * 16u);
    t.d = __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) uint16_t*>((gbytes)tile + 1792u + (uint32_t)(lane & 15) * 2u));
    return t;
}
// The scale of a 16-element group goes into the weight operand, as for Q4K with several slot tiles: a lane's eight
// codes of a 32-element stretch lie in one group, so the lane knows its scale.  sc * (code - 4) can reach +128, one too
// many for a byte; instead sc + 32 = 8 hi + lo (3-bit digits) multiplies the unsigned code (<= 49 per plane) and the
// plain codes form a third plane:
//     sum sc (code - 4) a = 8 P_hi + P_lo - 32 P_code - 4 sum_j sc_j bsum_j
// (the last term the exact f16 MFMA over the 16-element sums as before).  Twelve v_mfma_i32_16x16x64_i8 per tile and
// slot tile instead of sixteen half-masked 16x16x32 ones, and no integer multiply-add per result and group.
struct Q3KPlanes {
    v4i hi[4], lo[4], code[4];
    float d;
    v4h sB;
};
__device__ inline Q3KPlanes q3k_planes(const Q3KTile& w, int g) {
    const uint32_t M3 = 0x03030303u, M1 = 0x01010101u;
    Q3KPlanes pl;
    pl.d = __half2float(__ushort_as_half((unsigned short)w.d));
    const uint32_t qw[4] = {w.q.x, w.q.y, w.q.z, w.q.w};
    const uint32_t sw[4] = {w.sc.x, w.sc.y, w.sc.z, w.sc.w};
    const int half = g < 2 ? 0 : 8;   // which group of its stretch this lane's codes belong to
#pragma unroll
    for (int P = 0; P < 4; P++) {
        const uint32_t q = qw[P], h = (P < 2 ? w.qh.x : w.qh.y) >> (4 * (P & 1));
        const uint32_t lx = (q & M3) | ((h & M1) << 2), ly = ((q >> 2) & M3) | (((h >> 1) & M1) << 2);
        const uint32_t hx = ((q >> 4) & M3) | (((h >> 2) & M1) << 2), hy = ((q >> 6) & M3) | (((h >> 3) & M1) << 2);
        // stored scale - 32 was decoded at re-lay time; + 32 gives back the unsigned 6-bit value
        const uint32_t s_lo = (uint32_t)((int)(int8_t)((sw[P] >> half) & 0xffu) + 32);
        const uint32_t s_hi = (uint32_t)((int)(int8_t)((sw[P] >> (16 + half)) & 0xffu) + 32);
        pl.hi[P] = v4i{(int)digit_times_codes(lx, s_lo >> 3), (int)digit_times_codes(ly, s_lo >> 3),
                       (int)digit_times_codes(hx, s_hi >> 3), (int)digit_times_codes(hy, s_hi >> 3)};
        pl.lo[P] = v4i{(int)digit_times_codes(lx, s_lo & 7u), (int)digit_times_codes(ly, s_lo & 7u),
                       (int)digit_times_codes(hx, s_hi & 7u), (int)digit_times_codes(hy, s_hi & 7u)};
        pl.code[P] = v4i{(int)lx, (int)ly, (int)hx, (int)hy};
    }
    const uint32_t sg = sw[g];
    pl.sB = v4h{(_Float16)(int)(int8_t)(sg & 0xffu), (_Float16)(int)(int8_t)((sg >> 8) & 0xffu),
                (_Float16)(int)(int8_t)((sg >> 16) & 0xffu), (_Float16)(int)(int8_t)(sg >> 24)};
    return pl;
}
__device__ inline void q3k_mac(const Q3KPlanes& pl, const Q8KOperand& A, const float yd[4], float acc[4]) {
    const v4i zero = {0, 0, 0, 0};
    v4i p_hi = zero, p_lo = zero, p_c = zero;
#pragma unroll
    for (int P = 0; P < 4; P++) {
        const v4i a = {(int)A.a[P].x, (int)A.a[P].y, (int)A.a[P].z, (int)A.a[P].w};
        p_hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, pl.hi[P], p_hi, 0, 0, 0);
        p_lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, pl.lo[P], p_lo, 0, 0, 0);
        p_c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, pl.code[P], p_c, 0, 0, 0);
    }
    const v4f zf = {0.f, 0.f, 0.f, 0.f};
    v4f Ds = __builtin_amdgcn_mfma_f32_16x16x16f16(A.bs, pl.sB, zf, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int tot = 8 * p_hi[i] + p_lo[i] - 32 * p_c[i] - 4 * (int)Ds[i];   // exact: |tot| < 2^28
        acc[i] += (pl.d * yd[i]) * (float)tot;
    }
}

// Weight formats of the engine below: tile type, bytes per (16 rows x 256 k) tile, load and multiply.
struct FmtQ4K {
    typedef Q4KTile Tile;
    static constexpr int TILE_BYTES = Q4K_TILE_BYTES;
    static __device__ inline Tile load(const uint8_t* tile, int lane) { return load_q4k_tile(tile, lane); }
    static __device__ inline const Tile& prepare(const Tile& w, int) { return w; }
    static __device__ inline void mac(const Tile& w, const Q8KOperand& A, const float yd[4], int g, float acc[4]) { q4k_mac(w, A, yd, g, acc); }
};
// Q4K with the scales inside the weight operand (see q4k_planes): for two and four slot tiles per pass
struct FmtQ4KP {
    typedef Q4KTile Tile;
    static constexpr int TILE_BYTES = Q4K_TILE_BYTES;
    static __device__ inline Tile load(const uint8_t* tile, int lane) { return load_q4k_tile(tile, lane); }
    static __device__ inline Q4KPlanes prepare(const Tile& w, int g) { return q4k_planes(w, g); }
    static __device__ inline void mac(const Q4KPlanes& pl, const Q8KOperand& A, const float yd[4], int, float acc[4]) { q4k_mac_planes(pl, A, yd, acc); }
};
struct FmtQ2K {
    typedef Q2KTile Tile;
    static constexpr int TILE_BYTES = Q2K_TILE_BYTES;
    static __device__ inline Tile load(const uint8_t* tile, int lane) { return load_q2k_tile(tile, lane); }
    static __device__ inline const Tile& prepare(const Tile& w, int) { return w; }
    static __device__ inline void mac(const Tile& w, const Q8KOperand& A, const float yd[4], int g, float acc[4]) { q2k_mac(w, A, yd, g, acc); }
};
struct FmtQ3K {
    typedef Q3KTile Tile;
    static constexpr int TILE_BYTES = Q3K_TILE_BYTES;
    static __device__ inline Tile load(const uint8_t* tile, int lane) { return load_q3k_tile(tile, lane); }
    static __device__ inline Q3KPlanes prepare(const Tile& w, int g) { return q3k_planes(w, g); }
    static __device__ inline void mac(const Q3KPlanes& pl, const Q8KOperand& A, const float yd[4], int, float acc[4]) { q3k_mac(pl, A, yd, acc); }
};
struct FmtQ5K {
    typedef Q5KTile Tile;
    static constexpr int TILE_BYTES = Q5K_TILE_BYTES;
    static __device__ inline Tile load(const uint8_t* tile, int lane) { return load_q5k_tile(tile, lane); }
    static __device__ inline const Tile& prepare(const Tile& w, int) { return w; }
    static __device__ inline void mac(const Tile& w, const Q8KOperand& A, const float yd[4], int g, float acc[4]) { q5k_mac(w, A, yd, g, acc); }
};
struct FmtQ6K {
    typedef Q6KTile Tile;
    static constexpr int TILE_BYTES = Q6K_TILE_BYTES;
    static __device__ inline Tile load(const uint8_t* tile, int lane) { return load_q6k_tile(tile, lane); }
    static __device__ inline const Tile& prepare(const Tile& w, int) { return w; }
    static __device__ inline void mac(const Tile& w, const Q8KOperand& A, const float yd[4], int g, float acc[4]) { q6k_mac(w, A, yd, g, acc); }
};

// One wave, NT weight tiles per super-block (tp[0..NT), each walking along K), TT 16-slot operand
// tiles shared by all of them.  RING tile buffers rotate over the item sequence (sb, j): a buffer
// is refilled with the item RING places ahead as soon as it has been consumed, so RING tiles
// (2304 B each per wave) are in flight while one is being multiplied.
// Tiles of one matrix are ordered [super-block][row tile] (sb-major): all the waves of the grid that
// are at the same step of their K walk then read one contiguous region, which spreads the requests
// evenly over the HBM channels.  `sb_stride` = row tiles of the matrix * Q4K_TILE_BYTES.
template <class FMT, int NT, int RING>
__device__ inline void q4k_engine_prefetch(const uint8_t* const tp[NT], size_t sb_stride, int sb_lo, int sb_last, int lane, typename FMT::Tile t[RING]) {
#pragma unroll
    for (int j = 0; j < RING; j++) {
        const int sb = sb_lo + j / NT < sb_last ? sb_lo + j / NT : sb_last;
        t[j] = FMT::load(tp[j % NT] + (size_t)sb * sb_stride, lane);
    }
}

// `t` must have been filled by q4k_engine_prefetch for sb_lo (callers issue it before they know
// their slot list, so the first weight tiles are already on their way while the list is built).
// RING <= NT: the ring rotates inside a super-block.  RING a multiple of NT (few tiles per wave):
// the ring spans RING/NT super-blocks, so that a wave with little work per super-block still keeps
// RING tiles in flight; the loop then advances RING/NT super-blocks per trip, and a trip that runs
// past the end multiplies its surplus super-blocks by a zero activation scale.
template <class FMT, int TT, int NT, int RING>
__device__ inline void q4k_engine(const uint8_t* const tp[NT], size_t sb_stride, typename FMT::Tile t[RING], const ActBuf& ab, int K, int nsb,
                                  int sb_lo, int sb_hi, const int rowA[TT], int lane, int g, float acc[NT][TT][4], int a_step = 1, int a_off = 0) {
    static_assert(NT % RING == 0 || RING % NT == 0, "ring must divide, or be a multiple of, the tiles per super-block");
    constexpr int U = RING > NT ? RING / NT : 1;   // super-blocks per trip
    if (sb_lo >= sb_hi) return;
    Q8KOperand A[TT];
#pragma unroll
    for (int tt = 0; tt < TT; tt++) A[tt] = load_q8k_operand(ab, K, nsb, sb_lo * a_step + a_off, rowA[tt], g);
    // The loop body is one basic block: prefetches past the end are redirected to the last
    // super-block (a harmless repeated load) instead of being branched around, so that the
    // scheduling fences below really bound the live ranges.
    for (int sb0 = sb_lo; sb0 < sb_hi; sb0 += U) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int sb = sb0 + u;
            const bool live = U == 1 || sb < sb_hi;
            float yd[TT][4];
#pragma unroll
            for (int tt = 0; tt < TT; tt++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float v = __shfl(A[tt].yd, 4 * g + i, 64);
                    yd[tt][i] = live ? v : 0.f;
                }
            const int sb_next = (sb + 1 < sb_hi) ? sb + 1 : sb_hi - 1;
#pragma unroll
            for (int j = 0; j < NT; j++) {
                const int idx = u * NT + j;            // position in the trip
                const typename FMT::Tile w = t[idx % RING];
                const int ahead = idx + RING;          // the item that takes this ring place
                const int jn = ahead % NT;
                int sbn = sb0 + ahead / NT;
                sbn = sbn < sb_hi ? sbn : sb_hi - 1;
                // (issue priority for the refill: the sooner the request leaves, the longer the memory system has for it;
                // 1 % at batch 64, 0.3 % at batch 32)
                __builtin_amdgcn_s_setprio(3);
                t[idx % RING] = FMT::load(tp[jn] + (size_t)sbn * sb_stride, lane);
                __builtin_amdgcn_s_setprio(0);
                __builtin_amdgcn_sched_barrier(0);
                const auto prep = FMT::prepare(w, g);   // what of the tile's unpacking serves every slot tile
#pragma unroll
                for (int tt = 0; tt < TT; tt++) FMT::mac(prep, A[tt], yd[tt], g, acc[j][tt]);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int tt = 0; tt < TT; tt++) A[tt] = load_q8k_operand(ab, K, nsb, sb_next * a_step + a_off, rowA[tt], g);
        }
    }
}

// silu for the Q4K path: v / (1 + exp(-v)) with the hardware exp2.  The first product is not
// bit-identical to the CPU's anyway (f32 order), so the last-ulp accuracy of exp buys nothing here,
// while the double-precision exp costs microseconds in every workgroup's epilogue.
__device__ inline float silu_fast(float v) { return v / (1.0f + __expf(-v)); }
__device__ inline float silu_ref(float v) { return v / (1.0f + expf_glibc(-v)); }  // op.rs:646-648

// ---------------------------------------------------------------------------------------------
// Up projection.  A workgroup owns UP_ROWS rows of F of one expert; wave w carries rows
// [w*UP_ROWS/NW, (w+1)*UP_ROWS/NW) of both w1 and w3 over the whole of K.  UP_ROWS = 256 is one Q8K
// block of h per slot, quantised in the epilogue.  UP_ROWS = 64 (very small batches, where only a
// few experts are active and 256-row workgroups would leave most CUs without work) writes f32 h to
// p.hbuf instead and leaves the quantisation to a pass of its own.
constexpr int HBUF_STRIDE = 260;

template <class FMT, int TT, int NW, int RING, int UP_ROWS = 256>
__device__ inline void q4k_up_body(const ExpertParams& p, float (*hbuf)[HBUF_STRIDE], int* list_lds, int* wtot_lds) {
    constexpr int RTW = (UP_ROWS / 16) / NW;  // row tiles per wave and matrix
    constexpr int NT = 2 * RTW;
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: tile addresses stay in scalar registers
    const int grp = __builtin_amdgcn_readfirstlane(group_of_row(p, blockIdx.y));
    if (grp < 0) return;
    const int H = p.H, F = p.F, nsb = H / 256;
    const int rb = blockIdx.x;
    const GroupWeights gw = p.groups[grp];
    const int rt0 = rb * (UP_ROWS / 16) + wave * RTW;
    const uint8_t* tp[NT];
#pragma unroll
    for (int j = 0; j < RTW; j++) {
        tp[j] = gw.w1 + (size_t)(rt0 + j) * FMT::TILE_BYTES;
        tp[RTW + j] = gw.w3 + (size_t)(rt0 + j) * FMT::TILE_BYTES;
    }
    const size_t sb_stride = (size_t)(F / 16) * FMT::TILE_BYTES;
    // The grid's passes cover the longest list there could be; with many experts most of them find nothing.  A later pass
    // over a list that the dispatch kernel has measured looks at its length before it requests anything.
    if (blockIdx.z > 0 && !p.rb.direct && !p.is_shared) {
        const int gi = p.group0 + grp;
        if ((int)blockIdx.z * (TT * 16) >= p.rb.offsets[gi + 1] - p.rb.offsets[gi]) return;
    }
    // first weight tiles go out before anything else; an expert without tokens wastes them
    typename FMT::Tile ring[RING];
    q4k_engine_prefetch<FMT, NT, RING>(tp, sb_stride, 0, nsb - 1, lane, ring);

    const GroupSlots gs = group_slots<NW * 64>(p, grp, list_lds, wtot_lds);
    const int tg0 = blockIdx.z * (TT * 16);
    if (tg0 >= gs.n) return;

    // A two-tile pass over a list that ends inside its first tile runs the one-tile arithmetic (wave-uniform): the second
    // tile's matrix instructions and result steps are a fifth of the vector work of such a workgroup.
    auto run = [&](auto ttl_tag) {
        constexpr int TTL = decltype(ttl_tag)::value;   // live slot tiles of this pass
        int rowA[TTL];
#pragma unroll
        for (int tt = 0; tt < TTL; tt++) {
            int i = tg0 + tt * 16 + r;
            rowA[tt] = slot_token(p, gs.slot(i < gs.n ? i : gs.n - 1));
        }
        float acc[NT][TTL][4];
#pragma unroll
        for (int j = 0; j < NT; j++)
#pragma unroll
            for (int tt = 0; tt < TTL; tt++)
#pragma unroll
                for (int i = 0; i < 4; i++) acc[j][tt][i] = 0.f;

        q4k_engine<FMT, TTL, NT, RING>(tp, sb_stride, ring, p.xq, H, nsb, 0, nsb, rowA, lane, g, acc);

        if (UP_ROWS != 256) {   // h = silu(w1 x) * (w3 x) straight to memory
#pragma unroll
            for (int tt = 0; tt < TTL; tt++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int pos = tg0 + tt * 16 + 4 * g + i;
                    if (pos >= gs.n) continue;
                    const int64_t hrow = gs.slot(pos) - p.slot_origin;
#pragma unroll
                    for (int j = 0; j < RTW; j++)
                        p.hbuf[hrow * F + rb * UP_ROWS + (wave * RTW + j) * 16 + r] = silu_fast(acc[j][tt][i]) * acc[RTW + j][tt][i];
                }
            return;
        }
        // epilogue: h = silu(w1 x) * (w3 x), then Q8K-quantise the 256-row block of every slot
#pragma unroll
        for (int tt = 0; tt < TTL; tt++)
#pragma unroll
            for (int j = 0; j < RTW; j++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    hbuf[tt * 16 + 4 * g + i][(wave * RTW + j) * 16 + r] = silu_fast(acc[j][tt][i]) * acc[RTW + j][tt][i];
        __syncthreads();
        const int nfb = F / 256;
        // every wave quantises its TTL*16/NW tokens side by side
        constexpr int NQ = TTL * 16 / NW;
        float4 v[NQ];
        bool valid[NQ];
        int8_t* qs_out[NQ];
        float* d_out[NQ];
        __half* bs_out[NQ];
#pragma unroll
        for (int n = 0; n < NQ; n++) {
            const int tok = wave + n * NW;
            valid[n] = tg0 + tok < gs.n;
            v[n] = *reinterpret_cast<const float4*>(&hbuf[tok][lane * 4]);
            const int64_t hrow = gs.slot(valid[n] ? tg0 + tok : gs.n - 1) - p.slot_origin;
            qs_out[n] = p.hq.qs + hrow * F + rb * 256;
            d_out[n] = p.hq.d + hrow * nfb + rb;
            bs_out[n] = reinterpret_cast<__half*>(p.hq.bsum) + (hrow * nfb + rb) * 16;
        }
        quantize_q8k_blocks<NQ>(v, valid, lane, qs_out, d_out, bs_out);
    };
    if (TT == 2 && gs.n - tg0 <= 16) run(std::integral_constant<int, 1>{});
    else run(std::integral_constant<int, TT>{});
}

// ---------------------------------------------------------------------------------------------
// Down projection: a workgroup owns NTD row tiles (64 weight rows; 32 for very small batches) of one
// expert; its NW waves split K, every wave carrying the tiles over its K range, and the partial sums
// meet in LDS.
template <class FMT, int TT, int NW, int RING, int NTD = 4>
__device__ inline void q4k_down_body(const ExpertParams& p, float (*part)[NTD * TT * 4][64], int* list_lds, int* wtot_lds) {
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: tile addresses stay in scalar registers
    const int grp = __builtin_amdgcn_readfirstlane(group_of_row(p, blockIdx.y));
    if (grp < 0) return;
    const int H = p.H, F = p.F, nsb = F / 256;
    const int n_rt = H / 16;
    const int rt0 = blockIdx.x * NTD;
    const uint8_t* w2 = p.groups[grp].w2;
    const uint8_t* tp[NTD];
#pragma unroll
    for (int j = 0; j < NTD; j++) {
        int rt = rt0 + j < n_rt ? rt0 + j : n_rt - 1;  // tiles past the last row are computed and dropped
        tp[j] = w2 + (size_t)rt * FMT::TILE_BYTES;
    }
    size_t sb_stride = (size_t)n_rt * FMT::TILE_BYTES;
    int sb_lo = (int)((int64_t)nsb * wave / NW), sb_hi = (int)((int64_t)nsb * (wave + 1) / NW);
    int a_step = 1, a_off = 0;
    const bool ILV = p.down_interleaved != 0;
    if (ILV) {   // wave w takes super-blocks w, w + NW, ...: the waves of a workgroup read neighbouring slabs of the matrix
        const int mine = wave < nsb ? (nsb - wave + NW - 1) / NW : 0;
        a_step = NW; a_off = mine ? wave : 0;
#pragma unroll
        for (int j = 0; j < NTD; j++) tp[j] += (size_t)a_off * sb_stride;
        sb_stride *= NW;
        sb_lo = 0; sb_hi = mine;
    }
    if (blockIdx.z > 0 && !p.rb.direct && !p.is_shared) {   // (a later pass: see the up kernel)
        const int gi = p.group0 + grp;
        if ((int)blockIdx.z * (TT * 16) >= p.rb.offsets[gi + 1] - p.rb.offsets[gi]) return;
    }
    typename FMT::Tile ring[RING];
    if (ILV) q4k_engine_prefetch<FMT, NTD, RING>(tp, sb_stride, 0, sb_hi > 0 ? sb_hi - 1 : 0, lane, ring);
    else q4k_engine_prefetch<FMT, NTD, RING>(tp, sb_stride, sb_lo < nsb ? sb_lo : nsb - 1, sb_hi > sb_lo ? sb_hi - 1 : (sb_lo < nsb ? sb_lo : nsb - 1), lane, ring);

    const GroupSlots gs = group_slots<NW * 64>(p, grp, list_lds, wtot_lds);
    const int tg0 = blockIdx.z * (TT * 16);
    if (tg0 >= gs.n) return;

    // (a two-tile pass over a list that ends inside its first tile: the one-tile arithmetic, as in the up kernel)
    auto run = [&](auto ttl_tag) {
        constexpr int TTL = decltype(ttl_tag)::value;
        int rowA[TTL];
#pragma unroll
        for (int tt = 0; tt < TTL; tt++) {
            int i = tg0 + tt * 16 + r;
            rowA[tt] = gs.slot(i < gs.n ? i : gs.n - 1) - p.slot_origin;
        }
        float acc[NTD][TTL][4];
#pragma unroll
        for (int j = 0; j < NTD; j++)
#pragma unroll
            for (int tt = 0; tt < TTL; tt++)
#pragma unroll
                for (int i = 0; i < 4; i++) acc[j][tt][i] = 0.f;

        q4k_engine<FMT, TTL, NTD, RING>(tp, sb_stride, ring, p.hq, F, nsb, sb_lo, sb_hi, rowA, lane, g, acc, a_step, a_off);

#pragma unroll
        for (int j = 0; j < NTD; j++)
#pragma unroll
            for (int tt = 0; tt < TTL; tt++)
#pragma unroll
                for (int i = 0; i < 4; i++) part[wave][(j * TTL + tt) * 4 + i][lane] = acc[j][tt][i];
        __syncthreads();
        // NTD*TTL*4 value planes of 64 lanes; wave w reduces planes w, w+NW, ... (a fixed trip count, so that the routing
        // weights of all its planes are fetched together rather than one per trip)
        constexpr int NPL = NTD * TTL * 4;
#pragma unroll
        for (int n = 0; n < (NPL + NW - 1) / NW; n++) {
            const int v = wave + n * NW;
            if (NPL % NW != 0 && v >= NPL) break;
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < NW; w++) sum += part[w][v][lane];
            const int j = v / (TTL * 4), tt = (v / 4) % TTL, i = v % 4;
            const int pos = tg0 + tt * 16 + 4 * g + i;
            if (pos < gs.n && rt0 + j < n_rt) {
                const int slot = gs.slot(pos);
                emit_expert_output(p, slot, (rt0 + j) * 16 + r, sum * slot_weight(p, slot));
            }
        }
    };
    if (TT == 2 && gs.n - tg0 <= 16) run(std::integral_constant<int, 1>{});
    else run(std::integral_constant<int, TT>{});
}

#define DEF_UP_NARROW(NAME, FMT, NW, RING, WPE)                                                               \
    __global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void NAME(ExpertParams p) { \
        __shared__ int list_lds[DIRECT_MAX_SLOTS];                                                          \
        __shared__ int wtot_lds[NW];                                                                        \
        q4k_up_body<FMT, 1, NW, RING, 64>(p, nullptr, list_lds, wtot_lds);                                  \
    }
#define DEF_DOWN_NARROW(NAME, FMT, NW, RING, WPE)                                                             \
    __global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void NAME(ExpertParams p) { \
        __shared__ float part[NW][2 * 4][64];                                                               \
        __shared__ int list_lds[DIRECT_MAX_SLOTS];                                                          \
        __shared__ int wtot_lds[NW];                                                                        \
        q4k_down_body<FMT, 1, NW, RING, 2>(p, part, list_lds, wtot_lds);                                    \
    }
#define DEF_UP(NAME, FMT, TT, NW, RING, WPE)                                                                  \
    __global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void NAME(ExpertParams p) { \
        __shared__ float hbuf[TT * 16][HBUF_STRIDE];                                                        \
        __shared__ int list_lds[DIRECT_MAX_SLOTS];                                                          \
        __shared__ int wtot_lds[NW];                                                                        \
        q4k_up_body<FMT, TT, NW, RING>(p, hbuf, list_lds, wtot_lds);                                        \
    }
#define DEF_DOWN(NAME, FMT, TT, NW, RING, WPE)                                                              \
    __global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void NAME(ExpertParams p) { \
        __shared__ float part[NW][4 * TT * 4][64];                                                          \
        __shared__ int list_lds[DIRECT_MAX_SLOTS];                                                          \
        __shared__ int wtot_lds[NW];                                                                        \
        q4k_down_body<FMT, TT, NW, RING>(p, part, list_lds, wtot_lds);                                      \
    }

// Down-projection workgroups of one row tile (16 rows) instead of four: dense matrices of a few thousand rows, whose
// 64-row workgroups would leave most CUs without work.
#define DEF_DOWN_FINE(NAME, FMT, TT, NW, RING, WPE)                                                         \
    __global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void NAME(ExpertParams p) { \
        __shared__ float part[NW][1 * TT * 4][64];                                                          \
        __shared__ int list_lds[DIRECT_MAX_SLOTS];                                                          \
        __shared__ int wtot_lds[NW];                                                                        \
        q4k_down_body<FMT, TT, NW, RING, 1>(p, part, list_lds, wtot_lds);                                   \
    }

// One 16-slot tile per pass (small batches): variant 1 (default) 4 waves, 168 VGPRs, three workgroups
// per CU; variant 0 8 waves, 128 VGPRs.  Two and four tiles per pass (up to 32 / 64 rows per expert
// without streaming its weights twice) need the registers of a two-waves-per-SIMD launch.
DEF_UP(q4k_up_t1_v0, FmtQ4K, 1, 8, 2, 4)
DEF_UP(q4k_up_t1_v1, FmtQ4K, 1, 4, 2, 3)
DEF_UP_NARROW(q4k_up_t1_narrow, FmtQ4K, 4, 2, 4)   // 127 registers: a fourth wave per SIMD is free (batch 2: 85 -> 80 us per step)
DEF_UP(q4k_up_t2, FmtQ4KP, 2, 4, 2, 2)
DEF_UP(q4k_up_t4, FmtQ4KP, 4, 8, 2, 2)
DEF_DOWN(q4k_down_t1_v0, FmtQ4K, 1, 8, 2, 4)
DEF_DOWN(q4k_down_t1_v1, FmtQ4K, 1, 4, 2, 3)
DEF_DOWN_NARROW(q4k_down_t1_narrow, FmtQ4K, 8, 2, 4)
DEF_DOWN(q4k_down_t2, FmtQ4KP, 2, 4, 2, 2)
DEF_DOWN(q4k_down_t4, FmtQ4KP, 4, 8, 2, 2)
// Q2K: nine registers per tile; one and two slot tiles per pass
DEF_UP(q2k_up_t1, FmtQ2K, 1, 4, 2, 3)
DEF_UP_NARROW(q2k_up_t1_narrow, FmtQ2K, 4, 2, 3)
DEF_UP(q2k_up_t2, FmtQ2K, 2, 4, 2, 2)
DEF_DOWN(q2k_down_t1, FmtQ2K, 1, 4, 2, 3)
DEF_DOWN_NARROW(q2k_down_t1_narrow, FmtQ2K, 8, 2, 4)
DEF_DOWN(q2k_down_t2, FmtQ2K, 2, 4, 2, 2)
// Q3K: eleven registers per tile, sixteen MFMAs per tile and operand like Q6K
DEF_UP(q3k_up_t1, FmtQ3K, 1, 4, 2, 3)
DEF_UP_NARROW(q3k_up_t1_narrow, FmtQ3K, 4, 2, 3)
DEF_UP(q3k_up_t2, FmtQ3K, 2, 4, 2, 2)
DEF_DOWN(q3k_down_t1, FmtQ3K, 1, 4, 2, 3)
DEF_DOWN_NARROW(q3k_down_t1_narrow, FmtQ3K, 8, 2, 3)
DEF_DOWN(q3k_down_t2, FmtQ3K, 2, 4, 2, 2)
// Q5K: the Q4K variants with two more registers per tile; one and two slot tiles per pass
DEF_UP(q5k_up_t1, FmtQ5K, 1, 4, 2, 3)
DEF_UP_NARROW(q5k_up_t1_narrow, FmtQ5K, 4, 2, 3)
DEF_UP(q5k_up_t2, FmtQ5K, 2, 4, 2, 2)
DEF_DOWN(q5k_down_t1, FmtQ5K, 1, 4, 2, 3)
DEF_DOWN_NARROW(q5k_down_t1_narrow, FmtQ5K, 8, 2, 3)
DEF_DOWN(q5k_down_t2, FmtQ5K, 2, 4, 2, 2)
// Q6K: the same bodies; its tiles take five loads and seventeen registers, so every variant gets the
// registers of a two-waves-per-SIMD launch, and four slot tiles per pass would spill: two at most
DEF_UP(q6k_up_t1, FmtQ6K, 1, 4, 2, 2)
DEF_UP_NARROW(q6k_up_t1_narrow, FmtQ6K, 4, 2, 2)
DEF_UP(q6k_up_t2, FmtQ6K, 2, 4, 2, 2)
DEF_DOWN(q6k_down_t1, FmtQ6K, 1, 4, 2, 2)
DEF_DOWN_NARROW(q6k_down_t1_narrow, FmtQ6K, 8, 2, 2)
DEF_DOWN(q6k_down_t2, FmtQ6K, 2, 4, 2, 2)

DEF_DOWN_FINE(q4k_down_t1_fine, FmtQ4K, 1, 4, 4, 3)
DEF_DOWN_FINE(q4k_down_t2_fine, FmtQ4KP, 2, 4, 4, 2)
DEF_DOWN_FINE(q4k_down_t4_fine, FmtQ4KP, 4, 8, 2, 2)
DEF_DOWN_FINE(q2k_down_t1_fine, FmtQ2K, 1, 4, 4, 3)
DEF_DOWN_FINE(q2k_down_t2_fine, FmtQ2K, 2, 4, 4, 2)
DEF_DOWN_FINE(q3k_down_t1_fine, FmtQ3K, 1, 4, 4, 3)
DEF_DOWN_FINE(q3k_down_t2_fine, FmtQ3K, 2, 4, 4, 2)
DEF_DOWN_FINE(q5k_down_t1_fine, FmtQ5K, 1, 4, 4, 3)
DEF_DOWN_FINE(q5k_down_t2_fine, FmtQ5K, 2, 4, 4, 2)
DEF_DOWN_FINE(q6k_down_t1_fine, FmtQ6K, 1, 4, 4, 2)
DEF_DOWN_FINE(q6k_down_t2_fine, FmtQ6K, 2, 4, 4, 2)

// ---------------------------------------------------------------------------------------------
// Dense matrix times a few rows (single-stream decoding: attention projections, output head) in one launch: the rows
// are quantised to Q8K inside the kernel.  A wave multiplies super-blocks w, w + 4, ... of its workgroup's row tiles, as
// the streaming down kernel's waves do; just before each of them it quantises that block of every row (the wave-level
// BlockQ8K::from_float of act_quant.hpp, 64 lanes x 4 elements) into a few hundred bytes of LDS of its own and reads
// its MFMA operand back from there.  Every workgroup repeats the quantisation of the rows -- ~80 instructions per block
// and row -- which is why this pays for a handful of rows only: against it stand a kernel launch and a round trip of the
// quantised rows through memory.  Same blocks, same products, partial sums added in the same order as quantize_rows_kernel
// followed by the streaming down kernel: the results carry the same bits.
constexpr int FUSED_MAX_ROWS = 4;
constexpr int XQ_BSUM = 256, XQ_D = 288, XQ_BYTES = 320;   // one quantised block in LDS: 256 quants, 16 f16 sums, f32 scale
constexpr int FUSED_NW = 4;
constexpr size_t FUSED_MAX_LDS = 44 * 1024;   // beside the 16 KiB at most of partial sums: below the 64 KiB a workgroup gets without asking
// LDS for the quantised rows: every wave keeps its own super-blocks of every row
__host__ __device__ inline int fused_blocks_per_wave(int K) { return (K / 256 + FUSED_NW - 1) / FUSED_NW; }
static size_t fused_lds_bytes(int64_t m, int64_t K) { return (size_t)FUSED_NW * (size_t)fused_blocks_per_wave((int)K) * (size_t)m * XQ_BYTES; }

template <class FMT, int NTD, bool QUANTISED>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void qlinear_fused_kernel(FusedRows f) {
    constexpr int NW = FUSED_NW;
    const float* x = f.x;
    const int m = (int)f.m, n = (int)f.n, K = (int)f.k;
    const uint8_t* w = blockIdx.y ? f.w_b : f.w;
    float* y = blockIdx.y ? f.y_b : f.y;
    constexpr int RING = 4, U = RING / NTD;   // tiles in flight per wave; super-blocks per trip of the loop
    static_assert(RING % NTD == 0, "the ring holds whole super-blocks");
    __shared__ float part[NW][NTD * 4][64];
    extern __shared__ __align__(16) uint8_t xq_all[];   // [wave][block of the wave][row][XQ_BYTES]
    const int tid = threadIdx.x, lane = tid & 63, r = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nsb = K / 256, n_rt = n / 16;
    const int rt0 = blockIdx.x * NTD;
    const int mine = wave < nsb ? (nsb - wave + NW - 1) / NW : 0;   // super-blocks wave, wave + NW, ...
    const size_t sb_stride = (size_t)n_rt * FMT::TILE_BYTES * NW;
    const uint8_t* tp[NTD];
#pragma unroll
    for (int j = 0; j < NTD; j++) {
        const int rt = rt0 + j < n_rt ? rt0 + j : n_rt - 1;   // tiles past the last row are computed and dropped
        tp[j] = w + (size_t)rt * FMT::TILE_BYTES + (size_t)(mine ? wave : 0) * (size_t)n_rt * FMT::TILE_BYTES;
    }
    float acc[NTD][4];
#pragma unroll
    for (int j = 0; j < NTD; j++)
#pragma unroll
        for (int i = 0; i < 4; i++) acc[j][i] = 0.f;
    if (mine > 0) {
        // the first weight tiles are requested before anything else: the rows are quantised while they travel
        typename FMT::Tile ring[RING];
#pragma unroll
        for (int q = 0; q < RING; q++) {
            const int it = q / NTD < mine ? q / NTD : mine - 1;
            ring[q] = FMT::load(tp[q % NTD] + (size_t)it * sb_stride, lane);
        }
        uint8_t* xq = xq_all + (size_t)wave * fused_blocks_per_wave(K) * m * XQ_BYTES;
        if constexpr (QUANTISED) {
            // the wave's blocks of all rows, numbered b = it * m + row, copied from the Q8K rows in memory, four per turn
            constexpr int NQ = 4;
            const int n_blk = mine * m;
            const uint32_t* bsum = static_cast<const uint32_t*>(f.xq.bsum);
            for (int b0 = 0; b0 < n_blk; b0 += NQ) {
                uint32_t q[NQ], bs[NQ];
                float d[NQ];
#pragma unroll
                for (int i = 0; i < NQ; i++) {
                    const int bb = b0 + i < n_blk ? b0 + i : n_blk - 1;
                    const int it = bb / m, row = bb - it * m;
                    const size_t blk = (size_t)row * nsb + (size_t)(wave + it * NW);
                    q[i] = *reinterpret_cast<const uint32_t*>(f.xq.qs + blk * 256 + lane * 4);
                    bs[i] = bsum[blk * 8 + (lane & 7)];
                    d[i] = f.xq.d[blk];
                }
#pragma unroll
                for (int i = 0; i < NQ; i++) {
                    if (b0 + i < n_blk) {   // uniform
                        uint8_t* blk = xq + (size_t)(b0 + i) * XQ_BYTES;
                        *reinterpret_cast<uint32_t*>(blk + lane * 4) = q[i];
                        if (lane < 8) *reinterpret_cast<uint32_t*>(blk + XQ_BSUM + lane * 4) = bs[i];
                        if (lane == 0) *reinterpret_cast<float*>(blk + XQ_D) = d[i];
                    }
                }
            }
        } else {
            // the wave's blocks of all rows, numbered b = it * m + row, four at a time side by side (their loads, wave
            // reductions and divisions overlap); 32-bit byte offsets: m * K * 4 < 2^31
            constexpr int NQ = 4;
            const int n_blk = mine * m;
            auto x_offset = [&](int b) {
                const int bb = b < n_blk ? b : n_blk - 1;
                const int it = bb / m, row = bb - it * m;
                return ((uint32_t)row * (uint32_t)K + (uint32_t)((wave + it * NW) * 256 + lane * 4)) * 4u;
            };
            auto fetch = [&](int b) {
                const uint32_t off = x_offset(b);
                float4 a = gload<float4>(x, off);
                if (f.x2) {
                    const float4 c = gload<float4>(f.x2, off);
                    a = make_float4(a.x * c.x, a.y * c.y, a.z * c.z, a.w * c.w);
                }
                return a;
            };
            float4 v[NQ];
#pragma unroll
            for (int i = 0; i < NQ; i++) v[i] = fetch(i);
            for (int b0 = 0; b0 < n_blk; b0 += NQ) {
                bool valid[NQ];
                int8_t* qs_out[NQ];
                float* d_out[NQ];
                __half* bs_out[NQ];
                float4 cur[NQ];
#pragma unroll
                for (int i = 0; i < NQ; i++) {
                    valid[i] = b0 + i < n_blk;
                    uint8_t* blk = xq + (size_t)(valid[i] ? b0 + i : 0) * XQ_BYTES;
                    qs_out[i] = reinterpret_cast<int8_t*>(blk);
                    bs_out[i] = reinterpret_cast<__half*>(blk + XQ_BSUM);
                    d_out[i] = reinterpret_cast<float*>(blk + XQ_D);
                    cur[i] = v[i];
                }
#pragma unroll
                for (int i = 0; i < NQ; i++) v[i] = fetch(b0 + NQ + i);
                quantize_q8k_blocks<NQ>(cur, valid, lane, qs_out, d_out, bs_out);
            }
        }
        // the wave reads what its other lanes have written: LDS serves a wave's requests in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int my_row = r < m ? r : m - 1;
        for (int it0 = 0; it0 < mine; it0 += U) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int it = it0 + u;
                if (it < mine) {   // uniform
                    const uint8_t* blk = xq + (size_t)it * m * XQ_BYTES;
                    Q8KOperand A;
#pragma unroll
                    for (int P = 0; P < 4; P++) A.a[P] = *reinterpret_cast<const uint4*>(blk + my_row * XQ_BYTES + P * 64 + g * 16);
                    A.bs = *reinterpret_cast<const v4h*>(blk + my_row * XQ_BYTES + XQ_BSUM + g * 8);
                    float yd[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int row = 4 * g + i;
                        yd[i] = *reinterpret_cast<const float*>(blk + (row < m ? row : m - 1) * XQ_BYTES + XQ_D);
                    }
                    A.yd = yd[0];
                    __builtin_amdgcn_sched_barrier(0);   // (the fences bound the live ranges: one tile's arithmetic at a time)
#pragma unroll
                    for (int j = 0; j < NTD; j++) {
                        const int q = u * NTD + j;
                        const typename FMT::Tile wt = ring[q];
                        int ita = it0 + U + u;               // the super-block that takes this ring place
                        ita = ita < mine ? ita : mine - 1;
                        ring[q] = FMT::load(tp[j] + (size_t)ita * sb_stride, lane);
                        __builtin_amdgcn_sched_barrier(0);
                        const auto prep = FMT::prepare(wt, g);
                        FMT::mac(prep, A, yd, g, acc[j]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < NTD; j++)
#pragma unroll
        for (int i = 0; i < 4; i++) part[wave][j * 4 + i][lane] = acc[j][i];
    __syncthreads();
    for (int v2 = wave; v2 < NTD * 4; v2 += NW) {
        float sum = 0.f;
#pragma unroll
        for (int ww = 0; ww < NW; ww++) sum += part[ww][v2][lane];
        const int j = v2 / 4, i = v2 % 4;
        const int row = 4 * g + i;
        if (f.row_scale && row < m) sum *= f.row_scale[row];
        if (f.silu_y && blockIdx.y == 0) sum = silu_fast(sum);
        if (row < m && rt0 + j < n_rt) y[(size_t)row * n + (size_t)(rt0 + j) * 16 + r] = sum;
    }
}

bool qlinear_fused_usable(int dt, int64_t m, int64_t n, int64_t k) {
    return vecdot_dtype(dt) == MOE_GGML_Q8K && m >= 1 && m <= FUSED_MAX_ROWS && n % 16 == 0 && k % 256 == 0 && k >= 256 &&
           m * k < ((int64_t)1 << 29) && fused_lds_bytes(m, k) <= FUSED_MAX_LDS;
}

template <class FMT, bool QUANTISED>
static void launch_fused_src(const FusedRows& f, hipStream_t s) {
    // enough workgroups for two per CU where the matrices have the rows for it
    const int n_rt = (int)(f.n / 16);
    const unsigned ny = f.w_b ? 2u : 1u;
    const size_t lds = fused_lds_bytes(f.m, f.k);
    if (n_rt * (int)ny >= 2048) hipLaunchKernelGGL((qlinear_fused_kernel<FMT, 4, QUANTISED>), dim3((unsigned)((n_rt + 3) / 4), ny), dim3(256), lds, s, f);
    else if (n_rt * (int)ny >= 1024) hipLaunchKernelGGL((qlinear_fused_kernel<FMT, 2, QUANTISED>), dim3((unsigned)((n_rt + 1) / 2), ny), dim3(256), lds, s, f);
    else hipLaunchKernelGGL((qlinear_fused_kernel<FMT, 1, QUANTISED>), dim3((unsigned)n_rt, ny), dim3(256), lds, s, f);
}
template <class FMT>
static void launch_fused_fmt(const FusedRows& f, hipStream_t s) {
    if (f.x) launch_fused_src<FMT, false>(f, s);
    else launch_fused_src<FMT, true>(f, s);
}

hipError_t launch_qlinear_fused(int dt, const FusedRows& f, hipStream_t s) {
    if (!qlinear_fused_usable(dt, f.m, f.n, f.k) || !(f.x || f.xq.qs) || !f.w || !f.y || (f.w_b && !f.y_b)) return hipErrorInvalidValue;
    switch (dt) {
        case MOE_GGML_Q2K: launch_fused_fmt<FmtQ2K>(f, s); break;
        case MOE_GGML_Q3K: launch_fused_fmt<FmtQ3K>(f, s); break;
        case MOE_GGML_Q4K: launch_fused_fmt<FmtQ4K>(f, s); break;
        case MOE_GGML_Q5K: launch_fused_fmt<FmtQ5K>(f, s); break;
        case MOE_GGML_Q6K: launch_fused_fmt<FmtQ6K>(f, s); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
static int variant(const char* name, int dflt) {
    const char* e = getenv(name);
    return e ? atoi(e) : dflt;
}

// The kernels of one weight format.  t4 (four slot tiles per pass) exists for Q4K only.
typedef void (*ExpertKernel)(ExpertParams);
struct KernelFamily {
    ExpertKernel up_t1, up_narrow, up_t2, up_t4;
    ExpertKernel down_t1, down_narrow, down_t2, down_t4;
    ExpertKernel down_t1_fine, down_t2_fine, down_t4_fine;
};
static const KernelFamily* kernel_family(int dt) {
    static const int uv = variant("MOE_UP_VARIANT", 1), dv = variant("MOE_DOWN_VARIANT", 1);
    static const KernelFamily q4k = {uv == 0 ? q4k_up_t1_v0 : q4k_up_t1_v1, q4k_up_t1_narrow, q4k_up_t2, q4k_up_t4,
                                     dv == 0 ? q4k_down_t1_v0 : q4k_down_t1_v1, q4k_down_t1_narrow, q4k_down_t2, q4k_down_t4,
                                     q4k_down_t1_fine, q4k_down_t2_fine, q4k_down_t4_fine};
    static const KernelFamily q2k = {q2k_up_t1, q2k_up_t1_narrow, q2k_up_t2, nullptr, q2k_down_t1, q2k_down_t1_narrow, q2k_down_t2, nullptr,
                                     q2k_down_t1_fine, q2k_down_t2_fine, nullptr};
    static const KernelFamily q3k = {q3k_up_t1, q3k_up_t1_narrow, q3k_up_t2, nullptr, q3k_down_t1, q3k_down_t1_narrow, q3k_down_t2, nullptr,
                                     q3k_down_t1_fine, q3k_down_t2_fine, nullptr};
    static const KernelFamily q5k = {q5k_up_t1, q5k_up_t1_narrow, q5k_up_t2, nullptr, q5k_down_t1, q5k_down_t1_narrow, q5k_down_t2, nullptr,
                                     q5k_down_t1_fine, q5k_down_t2_fine, nullptr};
    static const KernelFamily q6k = {q6k_up_t1, q6k_up_t1_narrow, q6k_up_t2, nullptr, q6k_down_t1, q6k_down_t1_narrow, q6k_down_t2, nullptr,
                                     q6k_down_t1_fine, q6k_down_t2_fine, nullptr};
    switch (dt) {
        case MOE_GGML_Q2K: return &q2k;
        case MOE_GGML_Q3K: return &q3k;
        case MOE_GGML_Q4K: return &q4k;
        case MOE_GGML_Q5K: return &q5k;
        case MOE_GGML_Q6K: return &q6k;
    }
    return nullptr;
}

hipError_t launch_q4k_up(const ExpertParams& p, hipStream_t s) {
    if (p.max_rows == 0 || p.n_groups == 0) return hipSuccess;
    const KernelFamily* f = kernel_family(p.dt);
    if (!f) return hipErrorInvalidValue;
    static const int uv = variant("MOE_UP_VARIANT", 1);
    const int tt = p.slot_tiles >= 4 && f->up_t4 ? 4 : p.slot_tiles >= 2 ? 2 : 1;
    if (p.hbuf && tt == 1) {   // narrow workgroups (64 rows), f32 h to p.hbuf
        dim3 ngrid((unsigned)(p.F / 64), (unsigned)(p.by_assignment ? p.rb.T * p.rb.k : p.n_groups), (unsigned)((p.max_rows + 15) / 16));
        hipLaunchKernelGGL(f->up_narrow, ngrid, dim3(256), 0, s, p);
        return hipGetLastError();
    }
    dim3 grid((unsigned)(p.F / 256), (unsigned)p.n_groups, (unsigned)((p.max_rows + tt * 16 - 1) / (tt * 16)));
    if (tt == 4) hipLaunchKernelGGL(f->up_t4, grid, dim3(512), 0, s, p);
    else if (tt == 2) hipLaunchKernelGGL(f->up_t2, grid, dim3(256), 0, s, p);
    else hipLaunchKernelGGL(f->up_t1, grid, dim3(p.dt == MOE_GGML_Q4K && uv == 0 ? 512 : 256), 0, s, p);
    return hipGetLastError();
}

hipError_t launch_q4k_down(const ExpertParams& p_in, hipStream_t s) {
    if (p_in.max_rows == 0 || p_in.n_groups == 0) return hipSuccess;
    static const int ilv = variant("MOE_DOWN_ILV", 1);
    ExpertParams p = p_in;
    p.down_interleaved = ilv;
    const int dtd = p.dt_down ? p.dt_down : p.dt;
    const KernelFamily* f = kernel_family(dtd);
    if (!f) return hipErrorInvalidValue;
    static const int dv = variant("MOE_DOWN_VARIANT", 1);
    const int tt = p.slot_tiles >= 4 && f->down_t4 ? 4 : p.slot_tiles >= 2 ? 2 : 1;
    if (p.hbuf && tt == 1) {   // narrow workgroups (32 rows), eight waves split K
        dim3 ngrid((unsigned)((p.H / 16 + 1) / 2), (unsigned)(p.by_assignment ? p.rb.T * p.rb.k : p.n_groups), (unsigned)((p.max_rows + 15) / 16));
        hipLaunchKernelGGL(f->down_narrow, ngrid, dim3(512), 0, s, p);
        return hipGetLastError();
    }
    // one group whose 64-row workgroups would not fill the chip (a dense matrix of a few thousand rows): 16-row workgroups
    const int64_t passes = (p.max_rows + tt * 16 - 1) / (tt * 16);
    static const int fine_sw = variant("MOE_DOWN_FINE", -1);
    // (measured in a HIP graph, us per call, 64-row / 16-row workgroups: Q4_K 4096 x 4096: 13.1 / 9.7 at 3 rows, 18.2 / 13.6 at
    // 32, 24.6 / 19.2 at 64, 25.8 / 27.7 at 90; 8192 x 4096: 13.9 / 11.7 at 3 rows, 18.7 / 20.4 at 32; 4096 x 14336: 41.0 / 31.9
    // at 32 rows; 32000 x 4096: 20.4 / 29.2 at 3 rows; Q6_K 4096 x 4096: 25.3 / 14.6 at 32 rows, 25.4 / 19.8 at 48 (two passes
    // of two slot tiles), 8192 x 4096: 25.6 / 22.4 at 32 rows)
    const int64_t n_rt = p.H / 16;
    const bool fine = fine_sw >= 0 ? fine_sw > 0 : (p.n_groups == 1 && (n_rt * passes <= (dtd == MOE_GGML_Q6K ? 512 : 256) || (n_rt <= 512 && tt == 1)));
    if (fine) {
        dim3 fgrid((unsigned)(p.H / 16), (unsigned)p.n_groups, (unsigned)passes);
        if (tt == 4) hipLaunchKernelGGL(f->down_t4_fine, fgrid, dim3(512), 0, s, p);
        else if (tt == 2) hipLaunchKernelGGL(f->down_t2_fine, fgrid, dim3(256), 0, s, p);
        else hipLaunchKernelGGL(f->down_t1_fine, fgrid, dim3(256), 0, s, p);
        return hipGetLastError();
    }
    dim3 grid((unsigned)((p.H / 16 + 3) / 4), (unsigned)p.n_groups, (unsigned)passes);
    if (tt == 4) hipLaunchKernelGGL(f->down_t4, grid, dim3(512), 0, s, p);
    else if (tt == 2) hipLaunchKernelGGL(f->down_t2, grid, dim3(256), 0, s, p);
    else hipLaunchKernelGGL(f->down_t1, grid, dim3(dtd == MOE_GGML_Q4K && dv == 0 ? 512 : 256), 0, s, p);
    return hipGetLastError();
}

}  // namespace moe
