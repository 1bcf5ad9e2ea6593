// Tiled grouped expert products for large batches (prefill): Q4K (also Q2K, Q3K, Q5K and Q6K) weights x
// Q8K activations on v_mfma_i32_16x16x64_i8, a full-rate int8 MFMA shape of gfx950.
//
// Same integers as BlockQ4K::vec_dot (candle-core/src/quantized/k_quants.rs:1205-1285):
//     sum_j sc_j * (q4_j . q8_j)      and      sum_j m_j * (bsum_2j + bsum_2j+1).
// Applying the 6-bit scale to every block of MFMA results would cost one integer multiply-add per
// result and 32 elements of K -- twice the time of the MFMA itself -- so the scale is moved into the
// weight operand instead: sc = 8*hi + lo with hi, lo <= 7, and the two byte planes hi*q4 and lo*q4
// (<= 105, no carry between bytes) are multiplied by the activations in two MFMAs that accumulate over
// the whole 256-element super-block.  8*acc_hi + acc_lo is then the exact integer the reference
// computes; the mins term is an exact f16 MFMA over the 16 block sums.
//
// Work split: a workgroup (8 waves) owns one tile of 128 slots of one expert (from the dispatch
// kernel's tile list, so a skewed routing is balanced by tiles, not by experts) and eight 16-row
// weight operands, one per wave.  The 128 activation rows of a super-block go straight from global
// memory into LDS (double-buffered, no staging registers) and every wave reads them as MFMA A
// operands.  A wave unpacks and pre-scales its 16 weight rows of the super-block once, keeps the two
// planes in registers (32 VGPRs) and runs them against the eight 16-slot operands one after the other.
// The 16-row operand keeps a wave below 128 VGPRs, so four waves share a SIMD: a single wave issues
// at most one vector instruction every ~5 cycles and stalls on every MFMA result, and it takes that
// many waves to keep the MFMA pipe and the vector ALU busy at the same time.
//
// Q6K weights (the w2 of mixed files) take the same kernel for the down projection.  BlockQ6K::vec_dot
// (k_quants.rs:1613-1671) is d * y.d * sum_j sc_j * ((code_j - 32) . q8_j) with an i8 scale per 16 elements; the
// products W = sc * (code - 32) (|W| <= 4096) are formed in packed 16-bit arithmetic and cut into two signed bytes,
// W = 256 * H + L with L in [-128, 127], which are the two planes: 256 * acc_H + acc_L is the reference's integer, and
// no term over the block sums is left.
//
// Q2K weights (BlockQ2K::vec_dot, k_quants.rs:755-805) need one plane only: a 4-bit scale times a 2-bit code is at most 45,
// so the scaled codes are the weight operand as they are and a super-block takes four int8 MFMAs per operand instead of
// eight; the minimums leave through the sixteen block sums as for Q4K.
#include <type_traits>
#include "act_quant.hpp"
#include "kernels.hpp"

namespace moe {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef const __attribute__((address_space(1))) uint8_t* gbytes;

template <typename T>
__device__ __forceinline__ T gld(const void* uniform_base, uint32_t off) {
    return *reinterpret_cast<const __attribute__((address_space(1))) T*>((gbytes)uniform_base + off);
}

// four bytes (each <= 15) times a digit (<= 7): no byte overflows, and the packed 16-bit multiply does
// both halves of the register in one full-rate instruction (a 24-bit multiply would drop the top byte)
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t scale_bytes(uint32_t q, uint32_t s) {
    const u16x2 a = __builtin_bit_cast(u16x2, q);
    const u16x2 b = {(unsigned short)s, (unsigned short)s};
    return __builtin_bit_cast(uint32_t, (u16x2)(a * b));
}

// A tile is NOP 16-slot MFMA operands: 8 (128 slots) for big batches, 4 (64 slots) when the experts'
// lists are short, so that less of a tile is padding.
constexpr int G_WAVES = 8;
constexpr int G_THREADS = 64 * G_WAVES;
// Activations in LDS, laid out so that what one MFMA reads is one contiguous stretch in lane order
// (any other placement of a 16-lane x 4-chunk operand runs into LDS bank conflicts at half the read
// rate), and so that one direct global->LDS load of a wave (lane i lands at byte 16 i) writes exactly
// such a stretch:
//   quants [operand o][pair P][chunk g][row m] 16-byte pieces: 1 KiB per (o, P);
//   block sums [operand o][half h][row m] 16-byte pieces (8 sums): lane (m, g) reads 8 bytes at
//          piece (g/2, m), offset 8 (g%2);
//   scales [slot].
template <int NOP>
struct alignas(16) GemmLds {
    alignas(16) uint8_t q[2][NOP * 16 * 256];
    alignas(16) _Float16 bs[2][NOP][2][16][8];
    alignas(16) float yd[2][NOP * 16];
};

__device__ __forceinline__ uint32_t lds_address(const void* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}
// Direct global->LDS loads: lane i of the wave writes SIZE bytes at lds + SIZE*i; nothing passes through
// registers, so a whole super-block of activations can be in flight while the wave computes.  The
// compiler does not see these loads: the issuing wave waits for them (vmcnt) before the barrier that
// publishes the buffer.
__device__ __forceinline__ void dma16(const void* gbase, uint32_t voff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(gbase), "s"(lds));
}
__device__ __forceinline__ void dma4(const void* gbase, uint32_t voff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(voff), "s"(gbase), "s"(lds));
}
__device__ __forceinline__ void wait_all_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }   // vmcnt(0)

// Measurement aid, Q4K only, never set in the product (`python -m candle_amd.build --out-dir DIR --flag=-DMOE_WHATIF=N`
// builds a second library; its results are WRONG by construction, only its kernel times mean something).  Each bit
// takes one cost out of the tiled kernel's K loop, to show what the loop's other parts alone would take:
//   1  the result step: one vector instruction per result keeps the matrix instructions alive, no mins product
//   2  the unpacking of the weights into two scaled digit planes (the raw bytes go to the matrix cores)
//   4  the transfers of the next super-block's activations into LDS
//   8  the LDS reads of the activation operands (one register set for every operand)
#ifndef MOE_WHATIF
#define MOE_WHATIF 0
#endif

// What a lane fetches for the tile.  Quants: the NOP*4 (operand, pair) stretches of 1 KiB are dealt to
// the eight waves, NOP/2 each: lane (m = l%16, g = l/16) fetches piece (P, g) of row 16 o + m.  Block
// sums: one transfer covers two operands: lane fetches half (l/16)%2 of row 32 x + 16 (l/32) + l%16.
// Scales: row 64 x + l.  Waves without a share of the sums and scales repeat another wave's transfer:
// same bytes to the same place, and no branch around a load.
struct StageRows {
    uint32_t q;        // byte offset of the row's quants
    uint32_t bs, yd;   // row index
};
// transfer number I (0 .. NOP/2+1) of a wave's share of the tile: NOP/2 quant stretches, block sums, scales
template <int I, int NOP>
__device__ __forceinline__ void stage_piece(const ActBuf& ab, const StageRows& r, int nsb, int sb, GemmLds<NOP>& L, int buf, int wave, int lane) {
    constexpr int NB = NOP / 2;
    if (I < NB) {
        const int blk = wave * NB + I;            // = 4 o + P with o the wave's operand (r.q is its row)
        dma16(ab.qs, r.q + (uint32_t)(sb * 256 + ((blk & 3) * 4 + (lane >> 4)) * 16), lds_address(L.q[buf]) + (uint32_t)(blk * 1024));
    } else if (I == NB) {
        dma16(ab.bsum, ((r.bs * (uint32_t)nsb + (uint32_t)sb) * 16 + ((lane >> 4) & 1) * 8) * 2,
              lds_address(&L.bs[buf][0][0][0][0]) + (uint32_t)((wave % (NOP / 2)) * 1024));
    } else {
        dma4(ab.d, (r.yd * (uint32_t)nsb + (uint32_t)sb) * 4, lds_address(&L.yd[buf][0]) + (uint32_t)((wave % (NOP / 4)) * 256));
    }
}

// One wave's weights for one super-block: the 16 rows of one tile of the device layout.  Lane
// (n = l%16, g = l/16) owns row n and k-chunk g of every sub-block: exactly the tile's own lane order.
struct BRegs {
    u32x4 c[2];   // plane pl: (x,y) = 8 bytes of pair 2pl, chunk g; (z,w) = pair 2pl+1 (Q6K: the codes' low nibbles)
    u32x4 hdr;    // Q4K: d, dmin, 12 scale bytes of row n; Q6K: the row's sixteen i8 scales
    u32x4 qh;     // Q6K: the codes' top two bits, word P for pair P
    u32x2 q5;     // Q5K: the lane's fifth bits (pairs 0,1 / 2,3; four bits per byte and pair); Q3K: the codes' third bits, placed alike
    uint32_t d16; // Q6K, Q3K: d (f16 bits); Q2K: d | dmin << 16
};
template <int FMT>
__device__ __forceinline__ BRegs b_load(const uint8_t* tile, int lane) {
    BRegs b;
    b.c[0] = gld<u32x4>(tile, (uint32_t)(lane * 16));
    if (FMT == MOE_GGML_Q3K) {   // the codes' low two bits (placed as Q2K's codes), their high bits, the row's sixteen i8 scales, d
        b.q5 = gld<u32x2>(tile, (uint32_t)(1024 + lane * 8));
        b.hdr = gld<u32x4>(tile, (uint32_t)(1536 + (lane & 15) * 16));
        b.d16 = gld<uint16_t>(tile, (uint32_t)(1792 + (lane & 15) * 2));
        return b;
    }
    if (FMT == MOE_GGML_Q2K) {   // word P of the lane: the 2-bit codes of pair P; then the row's 16 (scale | min << 4) bytes and d | dmin << 16
        b.hdr = gld<u32x4>(tile, (uint32_t)(1024 + (lane & 15) * 16));
        b.d16 = gld<uint32_t>(tile, (uint32_t)(1280 + (lane & 15) * 4));
        return b;
    }
    b.c[1] = gld<u32x4>(tile, (uint32_t)(1024 + lane * 16));
    if (FMT == MOE_GGML_Q6K) {
        b.qh = gld<u32x4>(tile, (uint32_t)(2048 + lane * 16));
        b.hdr = gld<u32x4>(tile, (uint32_t)(3072 + (lane & 15) * 16));
        b.d16 = gld<uint16_t>(tile, (uint32_t)(3328 + (lane & 15) * 2));
    } else {
        b.hdr = gld<u32x4>(tile, (uint32_t)(2048 + (lane & 15) * 16));
        if (FMT == MOE_GGML_Q5K) b.q5 = gld<u32x2>(tile, (uint32_t)(Q4K_TILE_BYTES + lane * 8));
    }
    return b;
}

// The unpacked, pre-scaled operand of one super-block.  MFMA number P multiplies activation piece
// (pair P, chunk g) = [8 values of sub-block 2P | 8 values of sub-block 2P+1] by the low and the high
// nibbles of the same 8 weight bytes, each half scaled by its own sub-block's digit (the planes are
// accumulated over the whole super-block, so an MFMA may mix sub-blocks).
struct BPlanes {
    v4i lo[4], hi[4];
    v4h mB;
    float d, dmin;
};

__device__ __forceinline__ BPlanes b_prepare(const BRegs& b, int lane) {
    const int g = lane >> 4;
    const uint32_t M4 = 0x0f0f0f0fu;
    if (MOE_WHATIF & 2) {   // measurement aid: no unpacking
        BPlanes o;
        o.d = __uint_as_float(b.hdr.x); o.dmin = __uint_as_float(b.hdr.y);
#pragma unroll
        for (int P = 0; P < 4; P++) {
            const u32x4 c = b.c[P >> 1];
            o.lo[P] = v4i{(int)c.x, (int)c.y, (int)c.z, (int)c.w};
            o.hi[P] = v4i{(int)c.y, (int)c.z, (int)c.w, (int)c.x};
        }
        o.mB = v4h{0, 0, 0, 0};
        return o;
    }
    const uint32_t u0 = b.hdr.y, u1 = b.hdr.z, u2 = b.hdr.w;
    BPlanes o;
    o.d = __half2float(__ushort_as_half((unsigned short)(b.hdr.x & 0xffffu)));
    o.dmin = __half2float(__ushort_as_half((unsigned short)(b.hdr.x >> 16)));
    const uint32_t sc03 = u0 & 0x3f3f3f3fu;
    const uint32_t sc47 = (u2 & M4) | (((u0 >> 6) & 0x03030303u) << 4);
    const uint32_t m03 = u1 & 0x3f3f3f3fu;
    const uint32_t m47 = ((u2 >> 4) & M4) | (((u1 >> 6) & 0x03030303u) << 4);
    // scales split into two 3-bit digits, still one byte per sub-block
    const uint32_t lo03 = sc03 & 0x07070707u, hi03 = (sc03 >> 3) & 0x07070707u;
    const uint32_t lo47 = sc47 & 0x07070707u, hi47 = (sc47 >> 3) & 0x07070707u;
#pragma unroll
    for (int P = 0; P < 4; P++) {
        const u32x4 c = b.c[P >> 1];
        const uint32_t w0 = (P & 1) ? c.z : c.x, w1 = (P & 1) ? c.w : c.y;
        const uint32_t lw = (P < 2) ? lo03 : lo47, hw = (P < 2) ? hi03 : hi47;
        const uint32_t slo_a = (lw >> (16 * (P & 1))) & 0xffu, slo_b = (lw >> (16 * (P & 1) + 8)) & 0xffu;
        const uint32_t shi_a = (hw >> (16 * (P & 1))) & 0xffu, shi_b = (hw >> (16 * (P & 1) + 8)) & 0xffu;
        const uint32_t a0 = w0 & M4, a1 = w1 & M4, b0 = (w0 >> 4) & M4, b1 = (w1 >> 4) & M4;
        o.lo[P] = v4i{(int)scale_bytes(a0, slo_a), (int)scale_bytes(a1, slo_a), (int)scale_bytes(b0, slo_b), (int)scale_bytes(b1, slo_b)};
        o.hi[P] = v4i{(int)scale_bytes(a0, shi_a), (int)scale_bytes(a1, shi_a), (int)scale_bytes(b0, shi_b), (int)scale_bytes(b1, shi_b)};
    }
    // mins: the f16 MFMA's k = 4g + j is block sum 4g + j, which belongs to sub-block 2g + j/2
    const uint32_t mw = (g < 2) ? m03 : m47;
    const uint32_t ma = (mw >> (16 * (g & 1))) & 0xffu, mb = (mw >> (16 * (g & 1) + 8)) & 0xffu;
    o.mB = v4h{(_Float16)(int)ma, (_Float16)(int)ma, (_Float16)(int)mb, (_Float16)(int)mb};
    return o;
}

// Q6K: both planes of W = sc * (code - 32).  A word of four codes is spread over two registers of two 16-bit lanes
// (even and odd bytes), each multiplied and offset in one packed multiply-add: W + 128 = code * sc + (128 - 32 sc).
// The high bytes of W + 128 are H = floor((W + 128) / 256); its low bytes, with the top bit flipped, are W - 256 H as a
// signed byte.
__device__ __forceinline__ uint32_t pk_mad_u16(uint32_t a, uint32_t b, uint32_t c) {
    return __builtin_bit_cast(uint32_t, (u16x2)(__builtin_bit_cast(u16x2, a) * __builtin_bit_cast(u16x2, b) + __builtin_bit_cast(u16x2, c)));
}
__device__ __forceinline__ void q6k_planes(uint32_t codes, uint32_t s2, uint32_t add2, int& lo, int& hi) {
    const uint32_t ev = codes & 0x00ff00ffu;
    const uint32_t od = __builtin_amdgcn_perm(0u, codes, 0x0c030c01u);
    const uint32_t we = pk_mad_u16(ev, s2, add2), wo = pk_mad_u16(od, s2, add2);
    lo = (int)(__builtin_amdgcn_perm(wo, we, 0x06020400u) ^ 0x80808080u);
    hi = (int)__builtin_amdgcn_perm(wo, we, 0x07030501u);
}
__device__ __forceinline__ BPlanes b_prepare_q6k(const BRegs& b, int lane) {
    const int g = lane >> 4;
    const uint32_t M4 = 0x0f0f0f0fu, M2H = 0x30303030u;
    BPlanes o;
    o.d = __half2float(__ushort_as_half((unsigned short)b.d16));
    o.dmin = 0.f;
    o.mB = v4h{0, 0, 0, 0};
    const uint32_t sel = (uint32_t)(g >> 1) * 8u;   // elements 8g .. 8g+7 of a 32-element stretch: its first or second 16
#pragma unroll
    for (int P = 0; P < 4; P++) {
        const u32x4 c = b.c[P >> 1];
        const uint32_t w0 = (P & 1) ? c.z : c.x, w1 = (P & 1) ? c.w : c.y;
        const uint32_t h = b.qh[P], sw = b.hdr[P];
        // i8 scales of sub-blocks 4P + g/2 (first stretch of the pair) and 4P + 2 + g/2 (second), in both 16-bit lanes
        const int sa = __builtin_amdgcn_sbfe(sw, sel, 8), sb = __builtin_amdgcn_sbfe(sw, sel + 16u, 8);
        const uint32_t sa2 = __builtin_amdgcn_perm((uint32_t)sa, (uint32_t)sa, 0x05040100u);
        const uint32_t sb2 = __builtin_amdgcn_perm((uint32_t)sb, (uint32_t)sb, 0x05040100u);
        const uint32_t aa2 = pk_mad_u16(sa2, 0xffe0ffe0u, 0x00800080u), ab2 = pk_mad_u16(sb2, 0xffe0ffe0u, 0x00800080u);
        const uint32_t c0 = (w0 & M4) | ((h << 4) & M2H), c1 = (w1 & M4) | ((h << 2) & M2H);
        const uint32_t c2 = ((w0 >> 4) & M4) | (h & M2H), c3 = ((w1 >> 4) & M4) | ((h >> 2) & M2H);
        int l0, l1, l2, l3, h0, h1, h2, h3;
        q6k_planes(c0, sa2, aa2, l0, h0);
        q6k_planes(c1, sa2, aa2, l1, h1);
        q6k_planes(c2, sb2, ab2, l2, h2);
        q6k_planes(c3, sb2, ab2, l3, h3);
        o.lo[P] = v4i{l0, l1, l2, l3};
        o.hi[P] = v4i{h0, h1, h2, h3};
    }
    return o;
}

// Q5K (BlockQ5K::vec_dot, k_quants.rs:1394-1485): the Q4K sums on 5-bit codes.  A 3-bit digit times a code of up to 31
// no longer fits a signed byte, so the planes are the two bytes of W = sc * code (<= 1953), formed and cut as for Q6K
// (no offset: the minimum leaves through the block sums, as for Q4K).
__device__ __forceinline__ BPlanes b_prepare_q5k(const BRegs& b, int lane) {
    const int g = lane >> 4;
    const uint32_t M4 = 0x0f0f0f0fu, M1H = 0x10101010u;
    const uint32_t u0 = b.hdr.y, u1 = b.hdr.z, u2 = b.hdr.w;
    BPlanes o;
    o.d = __half2float(__ushort_as_half((unsigned short)(b.hdr.x & 0xffffu)));
    o.dmin = __half2float(__ushort_as_half((unsigned short)(b.hdr.x >> 16)));
    const uint32_t sc03 = u0 & 0x3f3f3f3fu;
    const uint32_t sc47 = (u2 & M4) | (((u0 >> 6) & 0x03030303u) << 4);
    const uint32_t m03 = u1 & 0x3f3f3f3fu;
    const uint32_t m47 = ((u2 >> 4) & M4) | (((u1 >> 6) & 0x03030303u) << 4);
#pragma unroll
    for (int P = 0; P < 4; P++) {
        const u32x4 c = b.c[P >> 1];
        const uint32_t w0 = (P & 1) ? c.z : c.x, w1 = (P & 1) ? c.w : c.y;
        const uint32_t h = ((P < 2) ? b.q5.x : b.q5.y) >> (4 * (P & 1));
        const uint32_t scw = (P < 2) ? sc03 : sc47;
        const uint32_t sa = (scw >> (16 * (P & 1))) & 0xffu, sb = (scw >> (16 * (P & 1) + 8)) & 0xffu;
        const uint32_t sa2 = sa | (sa << 16), sb2 = sb | (sb << 16);
        const uint32_t c0 = (w0 & M4) | ((h << 4) & M1H), c1 = (w1 & M4) | ((h << 3) & M1H);
        const uint32_t c2 = ((w0 >> 4) & M4) | ((h << 2) & M1H), c3 = ((w1 >> 4) & M4) | ((h << 1) & M1H);
        int l0, l1, l2, l3, h0, h1, h2, h3;
        q6k_planes(c0, sa2, 0x00800080u, l0, h0);
        q6k_planes(c1, sa2, 0x00800080u, l1, h1);
        q6k_planes(c2, sb2, 0x00800080u, l2, h2);
        q6k_planes(c3, sb2, 0x00800080u, l3, h3);
        o.lo[P] = v4i{l0, l1, l2, l3};
        o.hi[P] = v4i{h0, h1, h2, h3};
    }
    const uint32_t mw = (g < 2) ? m03 : m47;
    const uint32_t ma = (mw >> (16 * (g & 1))) & 0xffu, mb = (mw >> (16 * (g & 1) + 8)) & 0xffu;
    o.mB = v4h{(_Float16)(int)ma, (_Float16)(int)ma, (_Float16)(int)mb, (_Float16)(int)mb};
    return o;
}

// Q3K (BlockQ3K::vec_dot, k_quants.rs:923-1047): d * y.d * sum_j sc_j * ((code_j - 4) . q8_j) with a signed 6-bit scale per
// 16 elements.  W = sc * (code - 4) lies in [-124, 128] -- one too many for a signed byte -- so it is formed and cut into two
// signed bytes exactly as the Q6K products are, W + 128 = code * sc + (128 - 4 sc); the high plane is zero but where W = 128.
__device__ __forceinline__ BPlanes b_prepare_q3k(const BRegs& b, int lane) {
    const int g = lane >> 4;
    const uint32_t M3 = 0x03030303u, M1H = 0x04040404u;
    BPlanes o;
    o.d = __half2float(__ushort_as_half((unsigned short)b.d16));
    o.dmin = 0.f;
    o.mB = v4h{0, 0, 0, 0};
    const uint32_t sel = (uint32_t)(g >> 1) * 8u;   // elements 8g .. 8g+7 of a 32-element stretch: its first or second 16
#pragma unroll
    for (int P = 0; P < 4; P++) {
        const uint32_t q = b.c[0][P], sw = b.hdr[P];
        const uint32_t h = ((P < 2) ? b.q5.x : b.q5.y) >> (4 * (P & 1));
        const int sa = __builtin_amdgcn_sbfe(sw, sel, 8), sb = __builtin_amdgcn_sbfe(sw, sel + 16u, 8);
        const uint32_t sa2 = __builtin_amdgcn_perm((uint32_t)sa, (uint32_t)sa, 0x05040100u);
        const uint32_t sb2 = __builtin_amdgcn_perm((uint32_t)sb, (uint32_t)sb, 0x05040100u);
        const uint32_t aa2 = pk_mad_u16(sa2, 0xfffcfffcu, 0x00800080u), ab2 = pk_mad_u16(sb2, 0xfffcfffcu, 0x00800080u);
        const uint32_t c0 = (q & M3) | ((h << 2) & M1H), c1 = ((q >> 2) & M3) | ((h << 1) & M1H);
        const uint32_t c2 = ((q >> 4) & M3) | (h & M1H), c3 = ((q >> 6) & M3) | ((h >> 1) & M1H);
        int l0, l1, l2, l3, h0, h1, h2, h3;
        q6k_planes(c0, sa2, aa2, l0, h0);
        q6k_planes(c1, sa2, aa2, l1, h1);
        q6k_planes(c2, sb2, ab2, l2, h2);
        q6k_planes(c3, sb2, ab2, l3, h3);
        o.lo[P] = v4i{l0, l1, l2, l3};
        o.hi[P] = v4i{h0, h1, h2, h3};
    }
    return o;
}

// Q2K: the one plane sc * code (<= 45).  A lane's eight elements of a 32-element stretch lie in one 16-element sub-block
// (the first for chunks 0 and 1, the second for chunks 2 and 3), so each half of an MFMA operand takes one scale.
__device__ __forceinline__ BPlanes b_prepare_q2k(const BRegs& b, int lane) {
    const int g = lane >> 4;
    const uint32_t M3 = 0x03030303u;
    BPlanes o;
    o.d = __half2float(__ushort_as_half((unsigned short)(b.d16 & 0xffffu)));
    o.dmin = __half2float(__ushort_as_half((unsigned short)(b.d16 >> 16)));
    const int sel = 8 * (g >> 1);
#pragma unroll
    for (int P = 0; P < 4; P++) {
        const uint32_t q = b.c[0][P], sw = b.hdr[P];
        const uint32_t s_a = (sw >> sel) & 0xFu, s_b = (sw >> (16 + sel)) & 0xFu;
        o.lo[P] = v4i{(int)scale_bytes(q & M3, s_a), (int)scale_bytes((q >> 2) & M3, s_a),
                      (int)scale_bytes((q >> 4) & M3, s_b), (int)scale_bytes((q >> 6) & M3, s_b)};
    }
    // mins: the f16 MFMA's k = 4g + j is block sum 4g + j = sub-block 4g + j
    const uint32_t mg = (b.hdr[g] >> 4) & 0x0f0f0f0fu;
    o.mB = v4h{(_Float16)(int)(mg & 0xffu), (_Float16)(int)((mg >> 8) & 0xffu), (_Float16)(int)((mg >> 16) & 0xffu), (_Float16)(int)(mg >> 24)};
    return o;
}

// one super-block of the wave's 16 weight rows against 16-slot operand o of the staged tile
// `while_busy` runs right after the MFMAs are issued: this is where the next super-block's loads go.
template <int FMT, int NOP, typename Fill>
__device__ __forceinline__ void gemm_operand(const BPlanes& B, const GemmLds<NOP>& L, int buf, int o, int lane, v4f& facc, Fill while_busy) {
    const int m = lane & 15, g = lane >> 4;
    const v4i zero4 = {0, 0, 0, 0};
    v4i acc_lo, acc_hi;
    const uint8_t* arow = L.q[buf] + o * 4096 + lane * 16;
    // the wave takes issue priority while its matrix instructions go out: they keep the matrix pipe fed while the other
    // waves of the SIMD work through their result steps (2 % on the kernel)
    __builtin_amdgcn_s_setprio(2);
#pragma unroll
    for (int P = 0; P < 4; P++) {
        v4i a;
        if (MOE_WHATIF & 8) a = v4i{lane, lane + 1, lane + 2, lane + 3};   // measurement aid: no LDS read (one register set for all)
        else a = *reinterpret_cast<const v4i*>(arow + P * 1024);
        acc_lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, B.lo[P], P == 0 ? zero4 : acc_lo, 0, 0, 0);
        if constexpr (FMT != MOE_GGML_Q2K) acc_hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, B.hi[P], P == 0 ? zero4 : acc_hi, 0, 0, 0);
    }
    __builtin_amdgcn_s_setprio(0);
    // D[i] belongs to slot 16 o + 4 g + i, weight row n = lane%16
    if constexpr (FMT == MOE_GGML_Q6K || FMT == MOE_GGML_Q3K) {
        const v4f yd = *reinterpret_cast<const v4f*>(&L.yd[buf][o * 16 + g * 4]);
        while_busy();
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int isum = (acc_hi[i] << 8) + acc_lo[i];
            facc[i] = __builtin_fmaf(B.d * yd[i], (float)isum, facc[i]);
        }
    } else if ((MOE_WHATIF & 1) && FMT == MOE_GGML_Q4K) {   // measurement aid: no result step
        while_busy();
#pragma unroll
        for (int i = 0; i < 4; i++) facc[i] = __int_as_float(acc_lo[i] + acc_hi[i] + __float_as_int(facc[i]));
    } else {
        const v4h mA = *reinterpret_cast<const v4h*>(&L.bs[buf][o][g >> 1][m][(g & 1) * 4]);
        const v4f zf = {0.f, 0.f, 0.f, 0.f};
        const v4f Dm = __builtin_amdgcn_mfma_f32_16x16x16f16(mA, B.mB, zf, 0, 0, 0);
        const v4f yd = *reinterpret_cast<const v4f*>(&L.yd[buf][o * 16 + g * 4]);
        while_busy();
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if constexpr (FMT == MOE_GGML_Q2K) {
                // the reference's own order, every product and the difference rounded (k_quants.rs:772-773, 801): with unsigned
                // 2-bit codes the two terms are large and nearly cancel, and the scalar path's sum has one order only -- a
                // wave walks K in that order, so the up projection repeats vec_dot_unopt bit for bit
                const float dall = yd[i] * B.d, dminy = yd[i] * B.dmin;
                facc[i] += dall * (float)acc_lo[i] - dminy * Dm[i];
            } else {
                const int isum = (acc_hi[i] << (FMT == MOE_GGML_Q5K ? 8 : 3)) + acc_lo[i];
                const float v = __builtin_fmaf(B.d, (float)isum, -(B.dmin * Dm[i]));
                facc[i] = __builtin_fmaf(yd[i], v, facc[i]);
            }
        }
    }
}

__device__ __forceinline__ float silu_gemm(float v) { return v / (1.0f + __expf(-v)); }

// ---------------------------------------------------------------------------------------------
// One 16-row weight operand per wave, eight waves per workgroup, two workgroups per CU; a tile of
// NOP*16 slots.
// MODE 0: up   -- a workgroup owns 64 rows of F: waves 0-3 carry those rows of w1, waves 4-7 the same
//                 rows of w3; the w3 waves hand their sums over through LDS and the w1 waves write
//                 h = silu(a) * b (f32).
// MODE 1: down -- a workgroup owns 128 rows of H of w2, one 16-row operand per wave; writes yw.
// FMT: the weights' format (Q2K ... Q6K).
template <int FMT, int MODE, int NOP>
__global__ __launch_bounds__(G_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void q4k_gemm_kernel(ExpertParams p) {
    static_assert(FMT == MOE_GGML_Q2K || FMT == MOE_GGML_Q3K || FMT == MOE_GGML_Q4K || FMT == MOE_GGML_Q5K || FMT == MOE_GGML_Q6K, "formats of the tiled kernel");
    constexpr int NB = NOP / 2;
    constexpr int TILE_BYTES = FMT == MOE_GGML_Q6K ? Q6K_TILE_BYTES : FMT == MOE_GGML_Q5K ? Q5K_TILE_BYTES : FMT == MOE_GGML_Q2K ? Q2K_TILE_BYTES : FMT == MOE_GGML_Q3K ? Q3K_TILE_BYTES : Q4K_TILE_BYTES;
    constexpr bool kSums = FMT != MOE_GGML_Q6K && FMT != MOE_GGML_Q3K;   // block sums staged (the mins term)
    __shared__ GemmLds<NOP> L;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n_tiles = p.rb.tile_tab[0];
    // workgroup -> (row block, slot tile), in patches per XCD (patch_position)
    const int n_rb = MODE == 0 ? p.F / 64 : p.H / 128;
    const PatchPos pos = patch_position((int)blockIdx.x, n_rb, p.patch);
    const int rblk = pos.rblk, tile = pos.tile;
    if (tile >= n_tiles || rblk >= n_rb) return;
    const int gi = p.rb.tile_tab[1 + 2 * tile], pos0 = p.rb.tile_tab[2 + 2 * tile];
    if (gi < p.group0 || gi >= p.group0 + p.n_groups) return;
    const int grp = gi - p.group0;
    const int s_begin = p.rb.offsets[gi], n_g = p.rb.offsets[gi + 1] - s_begin;
    const int K = MODE == 0 ? p.H : p.F;        // reduction length
    const int N = MODE == 0 ? p.F : p.H;        // weight rows of the matrix
    const int nsb = K / 256;
    const size_t sb_stride = (size_t)(N / 16) * TILE_BYTES;
    const ActBuf& ab = MODE == 0 ? p.xq : p.hq;

    // activation row behind position r of the tile (positions past the expert's list repeat its last row)
    auto act_row = [&](int r) {
        const int pos = pos0 + r;
        const int slot = s_begin + (pos < n_g ? pos : n_g - 1);
        return MODE == 0 ? p.rb.perm_token[slot] : slot - p.slot_origin;
    };
    StageRows rows;
    rows.q = (uint32_t)act_row(16 * ((wave * NB) >> 2) + (lane & 15)) * (uint32_t)K;
    rows.bs = (uint32_t)act_row(32 * (wave % (NOP / 2)) + 16 * (lane >> 5) + (lane & 15));
    rows.yd = (uint32_t)act_row(64 * (wave % (NOP / 4)) + lane);

    // weight operand of this wave
    const GroupWeights gw = p.groups[grp];
    const uint8_t* wp;
    int row0;
    if (MODE == 0) {
        row0 = rblk * 64 + (wave & 3) * 16;
        wp = (wave < 4 ? gw.w1 : gw.w3) + (size_t)(row0 / 16) * TILE_BYTES;
    } else {
        row0 = rblk * 128 + wave * 16;
        wp = gw.w2 + (size_t)(row0 / 16) * TILE_BYTES;
    }
    v4f facc[NOP];
#pragma unroll
    for (int o = 0; o < NOP; o++) facc[o] = v4f{0.f, 0.f, 0.f, 0.f};

    // transfer t of the wave's share (quant stretches, sums, scales), then the weight tile
    auto stage = [&](auto I, int sb, int buf) {
        if ((MOE_WHATIF & 4) && sb > 0) return;   // measurement aid: the first super-block's transfers only
        if constexpr (!kSums && decltype(I)::value == NB) return;
        stage_piece<decltype(I)::value, NOP>(ab, rows, nsb, sb, L, buf, wave, lane);
    };
    auto prepare = [&](const BRegs& r) {
        if constexpr (FMT == MOE_GGML_Q6K) return b_prepare_q6k(r, lane);
        else if constexpr (FMT == MOE_GGML_Q2K) return b_prepare_q2k(r, lane);
        else if constexpr (FMT == MOE_GGML_Q3K) return b_prepare_q3k(r, lane);
        else if constexpr (FMT == MOE_GGML_Q5K) return b_prepare_q5k(r, lane);
        else return b_prepare(r, lane);
    };
    using std::integral_constant;
    stage(integral_constant<int, 0>{}, 0, 0);
    stage(integral_constant<int, 1>{}, 0, 0);
    stage(integral_constant<int, NB>{}, 0, 0);
    stage(integral_constant<int, NB + 1>{}, 0, 0);
    if constexpr (NB == 4) { stage(integral_constant<int, 2>{}, 0, 0); stage(integral_constant<int, 3>{}, 0, 0); }
    BRegs raw = b_load<FMT>(wp, lane);
    wait_all_loads();
    __syncthreads();
    for (int sb = 0; sb < nsb; sb++) {
        const int buf = sb & 1, nb = buf ^ 1;
        const int sbn = sb + 1 < nsb ? sb + 1 : sb;
        const BPlanes B = prepare(raw);
        // the next super-block's activations and weights are requested while the operands' MFMAs drain
        if constexpr (NOP == 8) {
            gemm_operand<FMT>(B, L, buf, 0, lane, facc[0], [&] { stage(integral_constant<int, 0>{}, sbn, nb); });
            gemm_operand<FMT>(B, L, buf, 1, lane, facc[1], [&] { stage(integral_constant<int, 1>{}, sbn, nb); });
            gemm_operand<FMT>(B, L, buf, 2, lane, facc[2], [&] { stage(integral_constant<int, 2>{}, sbn, nb); });
            gemm_operand<FMT>(B, L, buf, 3, lane, facc[3], [&] { stage(integral_constant<int, 3>{}, sbn, nb); });
            gemm_operand<FMT>(B, L, buf, 4, lane, facc[4], [&] { stage(integral_constant<int, 4>{}, sbn, nb); });
            gemm_operand<FMT>(B, L, buf, 5, lane, facc[5], [&] { stage(integral_constant<int, 5>{}, sbn, nb); });
            gemm_operand<FMT>(B, L, buf, 6, lane, facc[6], [&] { raw = b_load<FMT>(wp + (size_t)sbn * sb_stride, lane); });
            gemm_operand<FMT>(B, L, buf, 7, lane, facc[7], [&] {});
        } else {
            gemm_operand<FMT>(B, L, buf, 0, lane, facc[0], [&] { stage(integral_constant<int, 0>{}, sbn, nb); stage(integral_constant<int, 1>{}, sbn, nb); });
            gemm_operand<FMT>(B, L, buf, 1, lane, facc[1], [&] { stage(integral_constant<int, NB>{}, sbn, nb); stage(integral_constant<int, NB + 1>{}, sbn, nb); });
            gemm_operand<FMT>(B, L, buf, 2, lane, facc[2], [&] { raw = b_load<FMT>(wp + (size_t)sbn * sb_stride, lane); });
            gemm_operand<FMT>(B, L, buf, 3, lane, facc[3], [&] {});
        }
        wait_all_loads();
        __syncthreads();
    }

    // epilogue: lane holds weight row n = lane%16 and slots 16 o + 4 (lane/16) + i
    const int n = lane & 15, g = lane >> 4;
    if (MODE == 0) {
        // w3 waves (4-7) park their sums in LDS (the activation buffers are free now), w1 waves combine
        float* xch = reinterpret_cast<float*>(L.q[0]);   // [4 waves][NOP][4 i][64 lanes] floats
        static_assert(4 * NOP * 4 * 64 * 4 <= sizeof(L.q), "exchange area");
        if (wave >= 4) {
#pragma unroll
            for (int o = 0; o < NOP; o++)
#pragma unroll
                for (int i = 0; i < 4; i++) xch[(((wave - 4) * NOP + o) * 4 + i) * 64 + lane] = facc[o][i];
        }
        __syncthreads();
        if (wave < 4) {
#pragma unroll
            for (int o = 0; o < NOP; o++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int pos = pos0 + o * 16 + g * 4 + i;
                    if (pos >= n_g) continue;
                    const float bsum = xch[((wave * NOP + o) * 4 + i) * 64 + lane];
                    p.hbuf[(int64_t)(s_begin + pos - p.slot_origin) * p.F + row0 + n] = silu_gemm(facc[o][i]) * bsum;
                }
        }
    } else {
#pragma unroll
        for (int o = 0; o < NOP; o++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int pos = pos0 + o * 16 + g * 4 + i;
                if (pos >= n_g) continue;
                const int slot = s_begin + pos;
                p.yw[(int64_t)slot * p.H + row0 + n] = facc[o][i] * p.rb.perm_w[slot];
            }
    }
}

template <int FMT, int MODE>
static void launch_gemm(const ExpertParams& p, dim3 grid, hipStream_t s) {
    if (p.rb.tile_slots == 64) hipLaunchKernelGGL((q4k_gemm_kernel<FMT, MODE, 4>), grid, dim3(G_THREADS), 0, s, p);
    else hipLaunchKernelGGL((q4k_gemm_kernel<FMT, MODE, 8>), grid, dim3(G_THREADS), 0, s, p);
}
bool q4k_gemm_up_format(int dt) { return dt == MOE_GGML_Q2K || dt == MOE_GGML_Q3K || dt == MOE_GGML_Q4K || dt == MOE_GGML_Q5K || dt == MOE_GGML_Q6K; }
bool q4k_gemm_down_format(int dt) { return q4k_gemm_up_format(dt); }
hipError_t launch_q4k_gemm_up(const ExpertParams& p_in, hipStream_t s) {
    ExpertParams p = p_in;
    const int64_t tiles = max_gemm_tiles(p.n_slots, p.n_groups + 1, p.rb.tile_slots);
    p.patch = patch_edge(p.F / 64, tiles);
    dim3 grid(patch_grid(p.F / 64, tiles, p.patch));
    if (p.dt == MOE_GGML_Q6K) launch_gemm<MOE_GGML_Q6K, 0>(p, grid, s);
    else if (p.dt == MOE_GGML_Q5K) launch_gemm<MOE_GGML_Q5K, 0>(p, grid, s);
    else if (p.dt == MOE_GGML_Q4K) launch_gemm<MOE_GGML_Q4K, 0>(p, grid, s);
    else if (p.dt == MOE_GGML_Q2K) launch_gemm<MOE_GGML_Q2K, 0>(p, grid, s);
    else if (p.dt == MOE_GGML_Q3K) launch_gemm<MOE_GGML_Q3K, 0>(p, grid, s);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}
hipError_t launch_q4k_gemm_down(const ExpertParams& p_in, hipStream_t s) {
    ExpertParams p = p_in;
    const int64_t tiles = max_gemm_tiles(p.n_slots, p.n_groups + 1, p.rb.tile_slots);
    p.patch = patch_edge(p.H / 128, tiles);
    dim3 grid(patch_grid(p.H / 128, tiles, p.patch));
    const int dtd = p.dt_down ? p.dt_down : p.dt;
    if (dtd == MOE_GGML_Q6K) launch_gemm<MOE_GGML_Q6K, 1>(p, grid, s);
    else if (dtd == MOE_GGML_Q5K) launch_gemm<MOE_GGML_Q5K, 1>(p, grid, s);
    else if (dtd == MOE_GGML_Q4K) launch_gemm<MOE_GGML_Q4K, 1>(p, grid, s);
    else if (dtd == MOE_GGML_Q2K) launch_gemm<MOE_GGML_Q2K, 1>(p, grid, s);
    else if (dtd == MOE_GGML_Q3K) launch_gemm<MOE_GGML_Q3K, 1>(p, grid, s);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace moe
