// Layout and format kernels: re-laying GGML blocks into the tiled device layout, `to_float`
// from either layout, and the stand-alone activation quantiser used by the parity hooks.
//
// to_float restated from candle-core/src/quantized/k_quants.rs:166-186 (Q4_0), 340-359 (Q4_1), 443-465 (Q5_0), 556-581 (Q5_1), 587-603 (Q8_0), 872-908 (Q2K), 1131-1186 (Q3K),
// 1347-1374 (Q4K, with get_scale_min_k4 of utils.rs:50-60), 1563-1595 (Q5K), 1753-1790 (Q6K) and 1858-1870 (Q8K).  The library is
// built with -ffp-contract=off: `d1 * q - m1` must round the product before the subtraction.
#include <algorithm>
#include "act_quant.hpp"
#include "kernels.hpp"

namespace moe {

__device__ inline float f16_bits_to_f32(uint16_t h) { return __half2float(__ushort_as_half(h)); }

__device__ inline void scale_min_k4(int j, const uint8_t* q, int* sc, int* m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4);
        *m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
    }
}

// value of element `i` (0..255) of a Q4K block given its header (16 B) and the byte holding it
__device__ inline float q4k_value(const uint8_t* hdr, int i, uint8_t qbyte) {
    float d = f16_bits_to_f32((uint16_t)(hdr[0] | (hdr[1] << 8)));
    float mn = f16_bits_to_f32((uint16_t)(hdr[2] | (hdr[3] << 8)));
    int sc, m;
    scale_min_k4(i / 32, hdr + 4, &sc, &m);
    float d1 = d * (float)sc;
    float m1 = mn * (float)m;
    int q = ((i / 32) & 1) ? (qbyte >> 4) : (qbyte & 0xF);
    return d1 * (float)q - m1;
}

// to_float of one Q2K element, k_quants.rs:885-903: `dl * code - ml` with dl = d * (sc & 0xF), ml = min * (sc >> 4)
__device__ inline float q2k_value(float d, float mn, uint8_t sc, int code) {
    const float dl = d * (float)(sc & 0xF), ml = mn * (float)(sc >> 4);
    return dl * (float)code - ml;
}

// Q3K: the sixteen 6-bit scales of a raw block (low nibbles in scales[0..8), two per byte; high bit pairs in
// scales[8..12): the KMASK shuffle of k_quants.rs:1137-1145), and a code (-4..3) from its bit fields
__device__ inline int q3k_scale_raw(const uint8_t* scales, int j) {
    const int lo = j < 8 ? (scales[j] & 0xF) : (scales[j - 8] >> 4);
    return lo | (((scales[8 + j % 4] >> (2 * (j / 4))) & 3) << 4);
}
__device__ inline int q3k_code_raw(const uint8_t* blk, int e) {
    const int G = e / 32, l = e % 32;
    return ((blk[32 + 32 * (G / 4) + l] >> (2 * (G % 4))) & 3) - (((blk[l] >> G) & 1) ? 0 : 4);
}
// to_float of one Q3K element, k_quants.rs:1160-1172: `d_all * (scale as f32 - 32.0)`, then times the code
__device__ inline float q3k_value(float d, int8_t scale_minus_32, int code) {
    const float dl = d * (float)scale_minus_32;
    return dl * (float)code;
}

// value of element `i` of a Q5K block: header as Q4K, nibble byte, fifth bit (k_quants.rs:1582-1591:
// `d1 * (nibble as f32 + to_add) - m1`)
__device__ inline float q5k_value(const uint8_t* hdr, int i, uint8_t qbyte, int hbit) {
    float d = f16_bits_to_f32((uint16_t)(hdr[0] | (hdr[1] << 8)));
    float mn = f16_bits_to_f32((uint16_t)(hdr[2] | (hdr[3] << 8)));
    int sc, m;
    scale_min_k4(i / 32, hdr + 4, &sc, &m);
    float d1 = d * (float)sc;
    float m1 = mn * (float)m;
    int q = ((i / 32) & 1) ? (qbyte >> 4) : (qbyte & 0xF);
    return d1 * ((float)q + (hbit ? 16.f : 0.f)) - m1;
}

// code (0..63) of element e (0..255) of a raw BlockQ6K: the bit fields of k_quants.rs:1772-1778
__device__ inline int q6k_code(const uint8_t* blk, int e) {
    const int half = e / 128, q = (e % 128) / 32, l = e % 32;
    const uint8_t b = blk[64 * half + 32 * (q & 1) + l];
    const int nib = q >= 2 ? (b >> 4) : (b & 0xF);
    const int hi = (blk[128 + 32 * half + l] >> (2 * q)) & 3;
    return nib | (hi << 4);
}
// to_float of one Q6K element, k_quants.rs:1779-1782: `d * sc as f32 * q as f32`, left to right
__device__ inline float q6k_value(float d, int8_t sc, int code) { return d * (float)sc * (float)(int8_t)(code - 32); }

// ------------------------------------------------------------------ standard layout to_float
// 32-element block formats with two codes per byte (Q4_0, Q4_1, Q5_0, Q5_1): where the pieces of a raw block sit
// (d first; m, the fifth-bit word and the 16 nibble bytes after it) and where the tile keeps them.
// to_float: k_quants.rs:166-186, 340-359, 443-465, 556-581.
struct NibFmt {
    int bytes, m_pos, h_pos, q_pos;   // raw block; a position of 0 = the format has no such field
    int offset;                       // stored code - value (formats without a minimum)
    int tile_bytes, tile_d, tile_d_stride;
};
__host__ __device__ inline bool is_nib(int dt) { return dt == MOE_GGML_Q4_0 || dt == MOE_GGML_Q4_1 || dt == MOE_GGML_Q5_0 || dt == MOE_GGML_Q5_1; }
__host__ __device__ inline NibFmt nib_fmt(int dt) {
    switch (dt) {
        case MOE_GGML_Q4_1: return {20, 2, 0, 4, 0, Q4_1_TILE_BYTES, 256, 4};
        case MOE_GGML_Q5_0: return {22, 0, 2, 6, 16, Q5_0_TILE_BYTES, 320, 2};
        case MOE_GGML_Q5_1: return {24, 2, 4, 8, 0, Q5_1_TILE_BYTES, 320, 4};
        default: return {18, 0, 0, 2, 8, Q4_0_TILE_BYTES, 256, 2};
    }
}
// element e of a block: low nibbles are elements 0..15, high nibbles 16..31, bit e of h is the fifth bit
__device__ inline float nib_value(const NibFmt& f, uint16_t d_bits, uint16_t m_bits, uint8_t q, uint32_t h, int e) {
    const int code = (e < 16 ? (q & 0xF) : (q >> 4)) | (int)(((h >> e) & 1u) << 4);
    const float d = f16_bits_to_f32(d_bits);
    if (!f.m_pos) return (float)(code - f.offset) * d;
    return (float)code * d + f16_bits_to_f32(m_bits);
}

__global__ void dequant_std_kernel(int dt, const uint8_t* blocks, float* out, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    if (dt == MOE_GGML_Q4K) {
        const uint8_t* b = blocks + (i / 256) * 144;
        int e = (int)(i % 256);
        out[i] = q4k_value(b, e, b[16 + (e / 64) * 32 + (e % 32)]);
    } else if (dt == MOE_GGML_Q2K) {
        const uint8_t* b = blocks + (i / 256) * 84;
        int e = (int)(i % 256);
        int code = (b[16 + 32 * (e / 128) + e % 32] >> (2 * ((e % 128) / 32))) & 3;
        out[i] = q2k_value(f16_bits_to_f32((uint16_t)(b[80] | (b[81] << 8))), f16_bits_to_f32((uint16_t)(b[82] | (b[83] << 8))), b[e / 16], code);
    } else if (dt == MOE_GGML_Q3K) {
        const uint8_t* b = blocks + (i / 256) * 110;
        int e = (int)(i % 256);
        out[i] = q3k_value(f16_bits_to_f32((uint16_t)(b[108] | (b[109] << 8))), (int8_t)(q3k_scale_raw(b + 96, e / 16) - 32), q3k_code_raw(b, e));
    } else if (dt == MOE_GGML_Q5K) {
        const uint8_t* b = blocks + (i / 256) * 176;
        int e = (int)(i % 256);
        out[i] = q5k_value(b, e, b[48 + (e / 64) * 32 + (e % 32)], (b[16 + e % 32] >> (e / 32)) & 1);
    } else if (dt == MOE_GGML_Q6K) {
        const uint8_t* b = blocks + (i / 256) * 210;
        int e = (int)(i % 256);
        out[i] = q6k_value(f16_bits_to_f32((uint16_t)(b[208] | (b[209] << 8))), (int8_t)b[192 + e / 16], q6k_code(b, e));
    } else if (is_nib(dt)) {
        const NibFmt f = nib_fmt(dt);
        const uint8_t* b = blocks + (i / 32) * f.bytes;
        int e = (int)(i % 32);
        uint32_t h = f.h_pos ? (uint32_t)b[f.h_pos] | ((uint32_t)b[f.h_pos + 1] << 8) | ((uint32_t)b[f.h_pos + 2] << 16) | ((uint32_t)b[f.h_pos + 3] << 24) : 0u;
        out[i] = nib_value(f, (uint16_t)(b[0] | (b[1] << 8)), (uint16_t)(b[2] | (b[3] << 8)), b[f.q_pos + (e % 16)], h, e);
    } else if (dt == MOE_GGML_Q8_0) {
        const uint8_t* b = blocks + (i / 32) * 34;
        float d = f16_bits_to_f32((uint16_t)(b[0] | (b[1] << 8)));
        out[i] = (float)(int8_t)b[2 + (i % 32)] * d;
    } else {  // Q8K
        const uint8_t* b = blocks + (i / 256) * 292;
        float d;
        __builtin_memcpy(&d, b, 4);
        out[i] = d * (float)(int8_t)b[4 + (i % 256)];
    }
}

// ------------------------------------------------------------------ re-lay (one thread per 16/8/2-byte piece)
__global__ void relayout_q4k_kernel(const uint8_t* raw, uint8_t* tiled, int64_t n_rt, int nsb) {
    // one thread per 16-byte destination chunk: 144 chunks per tile
    int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t total = n_rt * nsb * 144;
    if (c >= total) return;
    int64_t tile = c / 144;
    int ch = (int)(c % 144);
    int64_t rt = tile / nsb;
    int sb = (int)(tile % nsb);
    uint8_t* dst = tiled + (sb * n_rt + rt) * Q4K_TILE_BYTES + ch * 16;  // tiles ordered [sb][rt]
    if (ch < 128) {
        int half = ch / 64, l = ch % 64, r = l % 16, g = l / 16;
        const uint8_t* blk = raw + ((rt * 16 + r) * nsb + sb) * 144 + 16;
        const uint8_t* s0 = blk + (2 * half) * 32 + 8 * g;
        const uint8_t* s1 = blk + (2 * half + 1) * 32 + 8 * g;
        for (int i = 0; i < 8; i++) { dst[i] = s0[i]; dst[8 + i] = s1[i]; }
    } else {
        int r = ch - 128;
        const uint8_t* blk = raw + ((rt * 16 + r) * nsb + sb) * 144;
        for (int i = 0; i < 16; i++) dst[i] = blk[i];
    }
}

__global__ void relayout_q2k_kernel(const uint8_t* raw, uint8_t* tiled, int64_t n_rt, int nsb) {
    // one thread per (tile, lane): its 64 two-bit codes; lanes < 16 also move the row's scales, d and dmin
    int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= n_rt * nsb * 64) return;
    int64_t tile = c / 64;
    int l = (int)(c % 64), r = l % 16, g = l / 16;
    int64_t rt = tile / nsb;
    int sb = (int)(tile % nsb);
    const uint8_t* blk = raw + ((rt * 16 + r) * nsb + sb) * 84;
    uint8_t* dst = tiled + (sb * n_rt + rt) * Q2K_TILE_BYTES;  // tiles ordered [sb][rt]
    auto code = [&](int e) { return (blk[16 + 32 * (e / 128) + e % 32] >> (2 * ((e % 128) / 32))) & 3; };
    for (int P = 0; P < 4; P++)
        for (int i = 0; i < 4; i++) {
            const int e = 64 * P + 8 * g + i;
            dst[l * 16 + P * 4 + i] = (uint8_t)(code(e) | (code(e + 4) << 2) | (code(e + 32) << 4) | (code(e + 36) << 6));
        }
    if (g == 0) {
        for (int j = 0; j < 16; j++) dst[1024 + r * 16 + j] = blk[j];
        for (int j = 0; j < 4; j++) dst[1280 + r * 4 + j] = blk[80 + j];
    }
}

__global__ void relayout_q3k_kernel(const uint8_t* raw, uint8_t* tiled, int64_t n_rt, int nsb) {
    // one thread per (tile, lane): 16 bytes of low bits, 8 bytes of high bits; lanes < 16 also decode the row's scales
    int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= n_rt * nsb * 64) return;
    int64_t tile = c / 64;
    int l = (int)(c % 64), r = l % 16, g = l / 16;
    int64_t rt = tile / nsb;
    int sb = (int)(tile % nsb);
    const uint8_t* blk = raw + ((rt * 16 + r) * nsb + sb) * 110;
    uint8_t* dst = tiled + (sb * n_rt + rt) * Q3K_TILE_BYTES;  // tiles ordered [sb][rt]
    auto cu = [&](int e) { return q3k_code_raw(blk, e) + 4; };   // 0..7: low two bits | high bit << 2
    for (int P = 0; P < 4; P++)
        for (int i = 0; i < 4; i++) {
            const int e = 64 * P + 8 * g + i;
            dst[l * 16 + P * 4 + i] = (uint8_t)((cu(e) & 3) | ((cu(e + 4) & 3) << 2) | ((cu(e + 32) & 3) << 4) | ((cu(e + 36) & 3) << 6));
        }
    for (int w = 0; w < 2; w++)
        for (int i = 0; i < 4; i++) {
            int byte = 0;
            for (int q = 0; q < 2; q++) {
                const int e = 64 * (2 * w + q) + 8 * g + i;
                byte |= ((cu(e) >> 2) | ((cu(e + 4) >> 2) << 1) | ((cu(e + 32) >> 2) << 2) | ((cu(e + 36) >> 2) << 3)) << (4 * q);
            }
            dst[1024 + l * 8 + w * 4 + i] = (uint8_t)byte;
        }
    if (g == 0) {
        for (int j = 0; j < 16; j++) dst[1536 + r * 16 + j] = (uint8_t)(int8_t)(q3k_scale_raw(blk + 96, j) - 32);
        dst[1792 + 2 * r] = blk[108];
        dst[1792 + 2 * r + 1] = blk[109];
    }
}

__global__ void relayout_q5k_kernel(const uint8_t* raw, uint8_t* tiled, int64_t n_rt, int nsb) {
    // one thread per (tile, lane): 32 nibble bytes and 8 bytes of fifth bits; lanes < 16 also move the header
    int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= n_rt * nsb * 64) return;
    int64_t tile = c / 64;
    int l = (int)(c % 64), r = l % 16, g = l / 16;
    int64_t rt = tile / nsb;
    int sb = (int)(tile % nsb);
    const uint8_t* blk = raw + ((rt * 16 + r) * nsb + sb) * 176;
    const uint8_t* qh = blk + 16;
    const uint8_t* qs = blk + 48;
    uint8_t* dst = tiled + (sb * n_rt + rt) * Q5K_TILE_BYTES;  // tiles ordered [sb][rt]
    for (int P = 0; P < 4; P++)
        for (int i = 0; i < 8; i++) dst[(P / 2) * 1024 + l * 16 + (P % 2) * 8 + i] = qs[32 * P + 8 * g + i];
    auto hb = [&](int j, int t) { return (qh[t] >> j) & 1; };   // fifth bit of element t of sub-block j
    for (int w = 0; w < 2; w++)
        for (int i = 0; i < 4; i++) {
            int byte = 0;
            for (int q = 0; q < 2; q++) {
                const int P = 2 * w + q;
                const int bits = hb(2 * P, 8 * g + i) | (hb(2 * P, 8 * g + 4 + i) << 1) | (hb(2 * P + 1, 8 * g + i) << 2) | (hb(2 * P + 1, 8 * g + 4 + i) << 3);
                byte |= bits << (4 * q);
            }
            dst[2304 + l * 8 + w * 4 + i] = (uint8_t)byte;
        }
    if (g == 0)
        for (int j = 0; j < 16; j++) dst[2048 + r * 16 + j] = blk[j];
}

__global__ void relayout_q6k_kernel(const uint8_t* raw, uint8_t* tiled, int64_t n_rt, int nsb) {
    // one thread per (tile, lane): its 32 nibble bytes and 16 high-bit bytes; lanes < 16 also move the
    // row's scales and d
    int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= n_rt * nsb * 64) return;
    int64_t tile = c / 64;
    int l = (int)(c % 64), r = l % 16, g = l / 16;
    int64_t rt = tile / nsb;
    int sb = (int)(tile % nsb);
    const uint8_t* blk = raw + ((rt * 16 + r) * nsb + sb) * 210;
    uint8_t* dst = tiled + (sb * n_rt + rt) * Q6K_TILE_BYTES;  // tiles ordered [sb][rt]
    for (int P = 0; P < 4; P++) {
        int ca[8], cb[8];
        for (int i = 0; i < 8; i++) {
            ca[i] = q6k_code(blk, 64 * P + 8 * g + i);
            cb[i] = q6k_code(blk, 64 * P + 32 + 8 * g + i);
            dst[(P / 2) * 1024 + l * 16 + (P % 2) * 8 + i] = (uint8_t)((ca[i] & 15) | ((cb[i] & 15) << 4));
        }
        for (int i = 0; i < 4; i++)
            dst[2048 + l * 16 + P * 4 + i] = (uint8_t)((ca[i] >> 4) | ((ca[i + 4] >> 4) << 2) | ((cb[i] >> 4) << 4) | ((cb[i + 4] >> 4) << 6));
    }
    if (g == 0) {
        for (int j = 0; j < 16; j++) dst[3072 + r * 16 + j] = blk[192 + j];
        dst[3328 + 2 * r] = blk[208];
        dst[3328 + 2 * r + 1] = blk[209];
    }
}

__global__ void relayout_q8_0_kernel(const uint8_t* raw, uint8_t* tiled, int64_t n_rt, int nkb) {
    // one thread per (tile, lane): 8 quant bytes; lanes < 16 also move the scale
    int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= n_rt * nkb * 64) return;
    int64_t tile = c / 64;
    int l = (int)(c % 64), r = l % 16, g = l / 16;
    int64_t rt = tile / nkb;
    int kb = (int)(tile % nkb);
    const uint8_t* blk = raw + ((rt * 16 + r) * nkb + kb) * 34;
    uint8_t* dst = tiled + tile * Q8_0_TILE_BYTES;
    for (int i = 0; i < 8; i++) dst[l * 8 + i] = blk[2 + 8 * g + i];
    if (g == 0) { dst[512 + 2 * r] = blk[0]; dst[512 + 2 * r + 1] = blk[1]; }
}

__global__ void relayout_nib_kernel(int dt, const uint8_t* raw, uint8_t* tiled, int64_t n_rt, int nkb) {
    // one thread per (tile, row)
    int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= n_rt * nkb * 16) return;
    const NibFmt f = nib_fmt(dt);
    int64_t tile = c / 16;
    int r = (int)(c % 16);
    int64_t rt = tile / nkb;
    int kb = (int)(tile % nkb);
    const uint8_t* blk = raw + ((rt * 16 + r) * nkb + kb) * f.bytes;
    uint8_t* dst = tiled + tile * f.tile_bytes;
    for (int i = 0; i < 16; i++) dst[r * 16 + i] = blk[f.q_pos + i];
    if (f.h_pos)
        for (int i = 0; i < 4; i++) dst[256 + 4 * r + i] = blk[f.h_pos + i];
    for (int i = 0; i < f.tile_d_stride; i++) dst[f.tile_d + f.tile_d_stride * r + i] = blk[i];   // d, then m, lead the block
}

// Super-tiles of the 32-element formats (K % 128 == 0): 16 rows x four blocks, ordered [step][row-tile].
// One thread per (super-tile, lane l = (row r, chunk g)): the lane's 4 (nibble formats) or 8 (Q8_0) code bytes of each
// of the four blocks; the lanes of chunk 0 also move the row's fifth-bit words and scales.
struct SuperFmt {
    uint32_t qb, hb, db;   // section sizes: codes, fifth-bit words, scales
};
__host__ __device__ inline SuperFmt super_fmt(int dt) {
    const uint32_t qb = dt == MOE_GGML_Q8_0 ? 2048u : 1024u;
    const uint32_t hb = (dt == MOE_GGML_Q5_0 || dt == MOE_GGML_Q5_1) ? 256u : 0u;
    const uint32_t db = (dt == MOE_GGML_Q4_1 || dt == MOE_GGML_Q5_1) ? 256u : 128u;
    return {qb, hb, db};
}
__global__ void relayout_q32_super_kernel(int dt, const uint8_t* raw, uint8_t* tiled, int64_t n_rt, int nks) {
    int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= n_rt * nks * 64) return;
    const SuperFmt sf = super_fmt(dt);
    const bool nib = is_nib(dt);
    const NibFmt f = nib_fmt(dt);
    const int bytes = nib ? f.bytes : 34, q_pos = nib ? f.q_pos : 2, m_pos = nib ? f.m_pos : 0, h_pos = nib ? f.h_pos : 0;
    int64_t tile = c / 64;
    int l = (int)(c % 64), r = l % 16, g = l / 16;
    int ks = (int)(tile / n_rt);
    int64_t rt = tile % n_rt;
    uint8_t* dst = tiled + tile * (sf.qb + sf.hb + sf.db);
    for (int b = 0; b < 4; b++) {
        const uint8_t* blk = raw + ((rt * 16 + r) * (int64_t)(nks * 4) + ks * 4 + b) * bytes;
        if (nib) {
            for (int i = 0; i < 4; i++) dst[l * 16 + 4 * b + i] = blk[q_pos + 4 * g + i];
        } else {
            uint8_t* q = dst + (b / 2) * 1024 + l * 16 + (b & 1) * 8;
            for (int i = 0; i < 4; i++) { q[i] = blk[q_pos + 4 * g + i]; q[4 + i] = blk[q_pos + 16 + 4 * g + i]; }
        }
        if (g == 0) {
            if (h_pos)
                for (int i = 0; i < 4; i++) dst[sf.qb + 16 * r + 4 * b + i] = blk[h_pos + i];
            const int nd = m_pos ? 4 : 2;   // d, then m, lead the block
            for (int i = 0; i < nd; i++) dst[sf.qb + sf.hb + nd * 4 * r + nd * b + i] = blk[i];
        }
    }
}

// ------------------------------------------------------------------ to_float from the tiled layout
__global__ void dequant_tiled_kernel(int dt, const uint8_t* tiled, float* out, int64_t rows, int64_t k) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * k) return;
    int64_t row = i / k;
    int col = (int)(i % k);
    int64_t rt = row / 16;
    int r = (int)(row % 16);
    if (dt == MOE_GGML_Q4K) {
        int sb = col / 256, e = col % 256;
        const uint8_t* tile = tiled + ((int64_t)sb * (rows / 16) + rt) * Q4K_TILE_BYTES;
        // original qs byte index of element e: (e/64)*32 + e%32 ; that byte sits in pair P = byte/32,
        // chunk g = (byte%32)/8, position byte%8
        int byte = (e / 64) * 32 + (e % 32);
        int P = byte / 32, g = (byte % 32) / 8, pos = byte % 8;
        int l = g * 16 + r;
        uint8_t q = tile[(P / 2) * 1024 + l * 16 + (P % 2) * 8 + pos];
        out[i] = q4k_value(tile + 2048 + r * 16, e, q);
    } else if (dt == MOE_GGML_Q2K) {
        int sb = col / 256, e = col % 256;
        const uint8_t* tile = tiled + ((int64_t)sb * (rows / 16) + rt) * Q2K_TILE_BYTES;
        int P = e / 64, sub = (e % 64) / 32, g = (e % 32) / 8, pos = e % 8;
        int l = g * 16 + r;
        int code = (tile[l * 16 + P * 4 + pos % 4] >> (2 * (2 * sub + pos / 4))) & 3;
        const uint8_t* dd = tile + 1280 + r * 4;
        out[i] = q2k_value(f16_bits_to_f32((uint16_t)(dd[0] | (dd[1] << 8))), f16_bits_to_f32((uint16_t)(dd[2] | (dd[3] << 8))),
                           tile[1024 + r * 16 + e / 16], code);
    } else if (dt == MOE_GGML_Q3K) {
        int sb = col / 256, e = col % 256;
        const uint8_t* tile = tiled + ((int64_t)sb * (rows / 16) + rt) * Q3K_TILE_BYTES;
        int P = e / 64, sub = (e % 64) / 32, g = (e % 32) / 8, pos = e % 8;
        int l = g * 16 + r;
        int low = (tile[l * 16 + P * 4 + pos % 4] >> (2 * (2 * sub + pos / 4))) & 3;
        int hb = (tile[1024 + l * 8 + (P / 2) * 4 + pos % 4] >> ((P % 2) * 4 + sub * 2 + pos / 4)) & 1;
        float d = f16_bits_to_f32((uint16_t)(tile[1792 + 2 * r] | (tile[1792 + 2 * r + 1] << 8)));
        out[i] = q3k_value(d, (int8_t)tile[1536 + r * 16 + e / 16], low - (hb ? 0 : 4));
    } else if (dt == MOE_GGML_Q5K) {
        int sb = col / 256, e = col % 256;
        const uint8_t* tile = tiled + ((int64_t)sb * (rows / 16) + rt) * Q5K_TILE_BYTES;
        int P = e / 64, sub = (e % 64) / 32, g = (e % 32) / 8, pos = e % 8;
        int l = g * 16 + r;
        uint8_t q = tile[(P / 2) * 1024 + l * 16 + (P % 2) * 8 + pos];
        uint8_t hbyte = tile[2304 + l * 8 + (P / 2) * 4 + pos % 4];
        out[i] = q5k_value(tile + 2048 + r * 16, e, q, (hbyte >> ((P % 2) * 4 + sub * 2 + pos / 4)) & 1);
    } else if (dt == MOE_GGML_Q6K) {
        int sb = col / 256, e = col % 256;
        const uint8_t* tile = tiled + ((int64_t)sb * (rows / 16) + rt) * Q6K_TILE_BYTES;
        int P = e / 64, sub = (e % 64) / 32, g = (e % 32) / 8, pos = e % 8;
        int l = g * 16 + r;
        uint8_t nb = tile[(P / 2) * 1024 + l * 16 + (P % 2) * 8 + pos];
        uint8_t hb = tile[2048 + l * 16 + P * 4 + pos % 4];
        int code = (sub ? (nb >> 4) : (nb & 0xF)) | (((hb >> (2 * (2 * sub + pos / 4))) & 3) << 4);
        float d = f16_bits_to_f32((uint16_t)(tile[3328 + 2 * r] | (tile[3328 + 2 * r + 1] << 8)));
        out[i] = q6k_value(d, (int8_t)tile[3072 + r * 16 + e / 16], code);
    } else if (q32_super_layout(k)) {  // the 32-element formats in super-tiles
        const SuperFmt sf = super_fmt(dt);
        const int ks = col / 128, b = (col % 128) / 32, e = col % 32;
        const uint8_t* tile = tiled + ((int64_t)ks * (rows / 16) + rt) * (sf.qb + sf.hb + sf.db);
        const int g = (e % 16) / 4, bi = e % 4, l = g * 16 + r;
        if (dt == MOE_GGML_Q8_0) {
            const uint8_t* dp = tile + sf.qb + 8 * r + 2 * b;
            float d = f16_bits_to_f32((uint16_t)(dp[0] | (dp[1] << 8)));
            out[i] = (float)(int8_t)tile[(b / 2) * 1024 + l * 16 + (b & 1) * 8 + (e / 16) * 4 + bi] * d;
        } else {
            const NibFmt f = nib_fmt(dt);
            const int nd = f.m_pos ? 4 : 2;
            const uint8_t* dm = tile + sf.qb + sf.hb + nd * 4 * r + nd * b;
            const uint8_t* hp = tile + sf.qb + 16 * r + 4 * b;
            uint32_t h = f.h_pos ? (uint32_t)hp[0] | ((uint32_t)hp[1] << 8) | ((uint32_t)hp[2] << 16) | ((uint32_t)hp[3] << 24) : 0u;
            uint16_t m_bits = f.m_pos ? (uint16_t)(dm[2] | (dm[3] << 8)) : (uint16_t)0;
            out[i] = nib_value(f, (uint16_t)(dm[0] | (dm[1] << 8)), m_bits, tile[l * 16 + 4 * b + bi], h, e);
        }
    } else if (dt == MOE_GGML_Q8_0) {
        int nkb = (int)(k / 32), kb = col / 32, e = col % 32;
        const uint8_t* tile = tiled + (rt * nkb + kb) * Q8_0_TILE_BYTES;
        float d = f16_bits_to_f32((uint16_t)(tile[512 + 2 * r] | (tile[512 + 2 * r + 1] << 8)));
        int l = (e / 8) * 16 + r;
        out[i] = (float)(int8_t)tile[l * 8 + e % 8] * d;
    } else {  // Q4_0, Q4_1, Q5_0, Q5_1
        const NibFmt f = nib_fmt(dt);
        int nkb = (int)(k / 32), kb = col / 32, e = col % 32;
        const uint8_t* tile = tiled + (rt * nkb + kb) * f.tile_bytes;
        const uint8_t* dm = tile + f.tile_d + f.tile_d_stride * r;
        const uint8_t* hp = tile + 256 + 4 * r;
        uint32_t h = f.h_pos ? (uint32_t)hp[0] | ((uint32_t)hp[1] << 8) | ((uint32_t)hp[2] << 16) | ((uint32_t)hp[3] << 24) : 0u;
        uint16_t m_bits = f.m_pos ? (uint16_t)(dm[2] | (dm[3] << 8)) : (uint16_t)0;
        out[i] = nib_value(f, (uint16_t)(dm[0] | (dm[1] << 8)), m_bits, tile[r * 16 + e % 16], h, e);
    }
}

// ------------------------------------------------------------------ activation quantiser on plain rows
template <int VDT>
__global__ __launch_bounds__(256) void quantize_rows_kernel(const float* x, int64_t rows, int k, ActBuf out) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t row = blockIdx.x;
    const float* xr = x + row * k;
    if (VDT == MOE_GGML_Q8K) {
        // blocks of a row are dealt to the waves of gridDim.y workgroups (few rows: many workgroups per row)
        // (four blocks of a wave side by side: their loads, wave reductions and divisions overlap)
        const int nb = k / 256;
        constexpr int NQ = 4;
        const int stride = 4 * gridDim.y;
        for (int b0 = blockIdx.y * 4 + wave; b0 < nb; b0 += NQ * stride) {
            float4 v[NQ];
            bool valid[NQ];
            int8_t* qs_out[NQ];
            float* d_out[NQ];
            __half* bs_out[NQ];
#pragma unroll
            for (int n = 0; n < NQ; n++) {
                valid[n] = b0 + n * stride < nb;
                const int b = valid[n] ? b0 + n * stride : b0;
                v[n] = *reinterpret_cast<const float4*>(xr + b * 256 + lane * 4);
                qs_out[n] = out.qs + row * k + b * 256;
                d_out[n] = out.d + row * nb + b;
                bs_out[n] = reinterpret_cast<__half*>(out.bsum) + (row * nb + b) * 16;
            }
            quantize_q8k_blocks<NQ>(v, valid, lane, qs_out, d_out, bs_out);
        }
    } else {
        const int nb = k / 32;
        for (int h = blockIdx.y * 256 + tid; h < k; h += 256 * gridDim.y)
            quantize_q8_0_block(VDT, xr[h], lane, out.qs + row * k + h, out.d + row * nb + h / 32,
                                reinterpret_cast<int32_t*>(out.bsum) + row * nb + h / 32);
    }
}

// ActBuf -> the reference's block structs (BlockQ8K 292 B: d f32, qs[256], bsums i16[16];
// BlockQ8_0 34 B: d f16, qs[32]; BlockQ8_1 36 B: d f16, s f16, qs[32])
__global__ void actbuf_to_std_kernel(int vdt, ActBuf in, int64_t rows, int k, uint8_t* out) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * k) return;
    int64_t row = i / k;
    int col = (int)(i % k);
    if (vdt == MOE_GGML_Q8K) {
        int nb = k / 256, b = col / 256, e = col % 256;
        uint8_t* blk = out + (row * nb + b) * 292;
        blk[4 + e] = (uint8_t)in.qs[row * k + b * 256 + q8k_act_offset(e)];
        if (e == 0) __builtin_memcpy(blk, &in.d[row * nb + b], 4);
        if (e < 16) {
            int16_t s = (int16_t)__half2int_rn(reinterpret_cast<const __half*>(in.bsum)[(row * nb + b) * 16 + e]);
            __builtin_memcpy(blk + 260 + 2 * e, &s, 2);
        }
    } else {
        const bool q81 = vdt == MOE_GGML_Q8_1;
        int nb = k / 32, b = col / 32, e = col % 32;
        uint8_t* blk = out + (row * nb + b) * (q81 ? 36 : 34);
        blk[(q81 ? 4 : 2) + e] = (uint8_t)in.qs[row * k + col];
        if (e == 0) {
            // the stored f32 values are exactly widened f16
            uint16_t h = __half_as_ushort(__float2half_rn(in.d[row * nb + b]));
            __builtin_memcpy(blk, &h, 2);
            if (q81) {
                uint16_t sh = __half_as_ushort(__float2half_rn(reinterpret_cast<const float*>(in.bsum)[row * nb + b]));
                __builtin_memcpy(blk + 2, &sh, 2);
            }
        }
    }
}

// ------------------------------------------------------------------ launchers
static inline unsigned nblk(int64_t n, int bs) { return (unsigned)((n + bs - 1) / bs); }

hipError_t launch_relayout(int dt, const uint8_t* raw, uint8_t* tiled, int64_t rows, int64_t k, hipStream_t s) {
    int64_t n_rt = rows / 16;
    int nkb = (int)(k / block_elems(dt));
    if (n_rt == 0 || nkb == 0) return hipSuccess;
    if (dt == MOE_GGML_Q4K)
        hipLaunchKernelGGL(relayout_q4k_kernel, dim3(nblk(n_rt * nkb * 144, 256)), dim3(256), 0, s, raw, tiled, n_rt, nkb);
    else if (dt == MOE_GGML_Q2K)
        hipLaunchKernelGGL(relayout_q2k_kernel, dim3(nblk(n_rt * nkb * 64, 256)), dim3(256), 0, s, raw, tiled, n_rt, nkb);
    else if (dt == MOE_GGML_Q3K)
        hipLaunchKernelGGL(relayout_q3k_kernel, dim3(nblk(n_rt * nkb * 64, 256)), dim3(256), 0, s, raw, tiled, n_rt, nkb);
    else if (dt == MOE_GGML_Q5K)
        hipLaunchKernelGGL(relayout_q5k_kernel, dim3(nblk(n_rt * nkb * 64, 256)), dim3(256), 0, s, raw, tiled, n_rt, nkb);
    else if (dt == MOE_GGML_Q6K)
        hipLaunchKernelGGL(relayout_q6k_kernel, dim3(nblk(n_rt * nkb * 64, 256)), dim3(256), 0, s, raw, tiled, n_rt, nkb);
    else if (q32_super_layout(k))
        hipLaunchKernelGGL(relayout_q32_super_kernel, dim3(nblk(n_rt * (nkb / 4) * 64, 256)), dim3(256), 0, s, dt, raw, tiled, n_rt, nkb / 4);
    else if (dt == MOE_GGML_Q8_0)
        hipLaunchKernelGGL(relayout_q8_0_kernel, dim3(nblk(n_rt * nkb * 64, 256)), dim3(256), 0, s, raw, tiled, n_rt, nkb);
    else
        hipLaunchKernelGGL(relayout_nib_kernel, dim3(nblk(n_rt * nkb * 16, 256)), dim3(256), 0, s, dt, raw, tiled, n_rt, nkb);
    return hipGetLastError();
}

hipError_t launch_dequant_tiled(int dt, const uint8_t* tiled, float* out, int64_t rows, int64_t k, hipStream_t s) {
    if (rows * k == 0) return hipSuccess;
    hipLaunchKernelGGL(dequant_tiled_kernel, dim3(nblk(rows * k, 256)), dim3(256), 0, s, dt, tiled, out, rows, k);
    return hipGetLastError();
}

hipError_t launch_dequant_std(int dt, const uint8_t* blocks, float* out, int64_t n, hipStream_t s) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(dequant_std_kernel, dim3(nblk(n, 256)), dim3(256), 0, s, dt, blocks, out, n);
    return hipGetLastError();
}

hipError_t launch_quantize_rows(int vdt, const float* x, int64_t rows, int k, const ActBuf& out, hipStream_t s) {
    if (rows == 0) return hipSuccess;
    const int64_t per_row = vdt == MOE_GGML_Q8K ? (k / 256 + 3) / 4 : (k + 255) / 256;   // workgroups that have a share of a row
    const unsigned split = (unsigned)std::max<int64_t>(1, std::min<int64_t>(per_row, 2048 / rows));
    if (vdt == MOE_GGML_Q8K)
        hipLaunchKernelGGL(quantize_rows_kernel<MOE_GGML_Q8K>, dim3((unsigned)rows, split), dim3(256), 0, s, x, rows, k, out);
    else if (vdt == MOE_GGML_Q8_1)
        hipLaunchKernelGGL(quantize_rows_kernel<MOE_GGML_Q8_1>, dim3((unsigned)rows, split), dim3(256), 0, s, x, rows, k, out);
    else
        hipLaunchKernelGGL(quantize_rows_kernel<MOE_GGML_Q8_0>, dim3((unsigned)rows, split), dim3(256), 0, s, x, rows, k, out);
    return hipGetLastError();
}

hipError_t launch_actbuf_to_std(int vdt, const ActBuf& in, int64_t rows, int k, uint8_t* out, hipStream_t s) {
    if (rows == 0) return hipSuccess;
    hipLaunchKernelGGL(actbuf_to_std_kernel, dim3(nblk(rows * k, 256)), dim3(256), 0, s, vdt, in, rows, k, out);
    return hipGetLastError();
}

}  // namespace moe
