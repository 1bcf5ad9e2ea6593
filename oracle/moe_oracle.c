/*
 * CPU oracle for candle's quantized sparse-MoE path.  TEST INFRASTRUCTURE ONLY
 * (see moe_oracle.h for the pinning status of every function).
 *
 * Build: no fused multiply-add contraction and no fast-math, because the Rust
 * reference never contracts `a*b+c` (see oracle/Makefile).
 */
#include "moe_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ f16 */
/* half 2.5.0 `f16::to_f32` / `f16::from_f32` semantics (IEEE binary16, RNE). */
float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t orc_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xff;
    uint32_t man = x & 0x7fffffu;
    if (exp == 255) { /* inf / nan */
        if (man == 0) return (uint16_t)(sign | 0x7c00u);
        return (uint16_t)(sign | 0x7c00u | 0x200u | (man >> 13)); /* quiet NaN, payload kept */
    }
    int32_t e = (int32_t)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u); /* overflow -> inf */
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign; /* too small: rounds to zero */
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1))) half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half_man = man >> 13;
    uint32_t rem = man & 0x1fffu;
    uint16_t h = (uint16_t)(sign | ((uint32_t)e << 10) | half_man);
    if (rem > 0x1000u || (rem == 0x1000u && (half_man & 1))) h++; /* may carry into exponent / inf */
    return h;
}

/* ------------------------------------------------------------------ helpers */
/* Rust `f as i32`: truncate toward zero, saturate, NaN -> 0. */
static inline int32_t sat_i32(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}
static inline uint8_t sat_u8(float v) {
    if (v != v) return 0;
    if (v >= 255.0f) return 255;
    if (v <= 0.0f) return 0;
    return (uint8_t)v;
}
static inline int8_t sat_i8(float v) {
    if (v != v) return 0;
    if (v >= 127.0f) return 127;
    if (v <= -128.0f) return -128;
    return (int8_t)v;
}
/* utils.rs:1-3 : f32::round (half away from zero) then `as i32` */
static inline int32_t nearest_int(float v) { return sat_i32(roundf(v)); }
/* Rust f32::max / f32::min ignore a NaN operand */
static inline float rmax(float a, float b) { return fmaxf(a, b); }
static inline float rmin(float a, float b) { return fminf(a, b); }

int64_t orc_block_elems(int dtype) {
    switch (dtype) {
        case ORC_Q4_0: case ORC_Q4_1: case ORC_Q5_0: case ORC_Q5_1: case ORC_Q8_0: case ORC_Q8_1: return 32;
        case ORC_Q2K: case ORC_Q3K: case ORC_Q4K: case ORC_Q5K: case ORC_Q6K: case ORC_Q8K: return 256;
        default: return -1;
    }
}
int64_t orc_block_bytes(int dtype) {
    switch (dtype) {
        case ORC_Q4_0: return 18;
        case ORC_Q4_1: return 20;
        case ORC_Q5_0: return 22;
        case ORC_Q5_1: return 24;
        case ORC_Q8_0: return 34;
        case ORC_Q8_1: return 36;
        case ORC_Q2K: return 84;
        case ORC_Q3K: return 110;
        case ORC_Q4K: return 144;
        case ORC_Q5K: return 176;
        case ORC_Q6K: return 210;
        case ORC_Q8K: return 292;
        default: return -1;
    }
}
int orc_vecdot_dtype(int dtype) {
    switch (dtype) {
        case ORC_Q4_0: case ORC_Q5_0: case ORC_Q8_0: return ORC_Q8_0;
        case ORC_Q4_1: case ORC_Q5_1: case ORC_Q8_1: return ORC_Q8_1;
        case ORC_Q2K: case ORC_Q3K: case ORC_Q4K: case ORC_Q5K: case ORC_Q6K: case ORC_Q8K: return ORC_Q8K;
        default: return -1;
    }
}

/* ------------------------------------------------------------------ Q4_0 */
/* k_quants.rs:188-224 */
static void quantize_q4_0(const float* xs, int64_t k, orc_block_q4_0* ys) {
    const int qk = 32;
    for (int64_t i = 0; i < k / qk; i++) {
        float amax = 0.f, max = 0.f;
        const float* x = xs + i * qk;
        for (int j = 0; j < qk; j++) {
            if (amax < fabsf(x[j])) { amax = fabsf(x[j]); max = x[j]; }
        }
        float d = max / -8.0f;
        float id = (d != 0.f) ? 1.f / d : 0.f;
        ys[i].d = orc_f32_to_f16(d);
        for (int j = 0; j < qk / 2; j++) {
            float x0 = x[j] * id;
            float x1 = x[qk / 2 + j] * id;
            uint8_t xi0 = sat_u8(x0 + 8.5f); if (xi0 > 15) xi0 = 15;
            uint8_t xi1 = sat_u8(x1 + 8.5f); if (xi1 > 15) xi1 = 15;
            ys[i].qs[j] = (uint8_t)(xi0 | (xi1 << 4));
        }
    }
}
/* k_quants.rs:166-186 */
static void dequantize_q4_0(const orc_block_q4_0* xs, int64_t k, float* ys) {
    const int qk = 32;
    for (int64_t i = 0; i < k / qk; i++) {
        float d = orc_f16_to_f32(xs[i].d);
        for (int j = 0; j < qk / 2; j++) {
            int x0 = (int)(xs[i].qs[j] & 0x0F) - 8;
            int x1 = (int)(xs[i].qs[j] >> 4) - 8;
            ys[i * qk + j] = (float)x0 * d;
            ys[i * qk + j + qk / 2] = (float)x1 * d;
        }
    }
}
/* k_quants.rs:241-258 */
static float vec_dot_q4_0_q8_0(int64_t n, const orc_block_q4_0* xs, const orc_block_q8_0* ys) {
    float sumf = 0.f;
    for (int64_t b = 0; b < n / 32; b++) {
        int32_t sum_i = 0;
        for (int j = 0; j < 16; j++) {
            int v0 = (int)(xs[b].qs[j] & 0x0F) - 8;
            int v1 = (int)(xs[b].qs[j] >> 4) - 8;
            sum_i += v0 * (int)ys[b].qs[j] + v1 * (int)ys[b].qs[j + 16];
        }
        sumf += (float)sum_i * orc_f16_to_f32(xs[b].d) * orc_f16_to_f32(ys[b].d);
    }
    return sumf;
}

/* ------------------------------------------------------------------ Q4_1 */
/* k_quants.rs:299-337 */
static void quantize_q4_1(const float* xs, int64_t k, orc_block_q4_1* ys) {
    const int qk = 32;
    for (int64_t i = 0; i < k / qk; i++) {
        const float* x = xs + i * qk;
        float min = INFINITY, max = -INFINITY;
        for (int j = 0; j < qk; j++) { min = rmin(x[j], min); max = rmax(x[j], max); }
        float d = (max - min) / 15.0f;
        float id = (d != 0.f) ? 1.f / d : 0.f;
        ys[i].d = orc_f32_to_f16(d);
        ys[i].m = orc_f32_to_f16(min);
        for (int j = 0; j < qk / 2; j++) {
            float x0 = (x[j] - min) * id;
            float x1 = (x[qk / 2 + j] - min) * id;
            uint8_t xi0 = sat_u8(x0 + 0.5f); if (xi0 > 15) xi0 = 15;
            uint8_t xi1 = sat_u8(x1 + 0.5f); if (xi1 > 15) xi1 = 15;
            ys[i].qs[j] = (uint8_t)(xi0 | (xi1 << 4));
        }
    }
}
/* k_quants.rs:340-359 */
static void dequantize_q4_1(const orc_block_q4_1* xs, int64_t k, float* ys) {
    const int qk = 32;
    for (int64_t i = 0; i < k / qk; i++) {
        float d = orc_f16_to_f32(xs[i].d), m = orc_f16_to_f32(xs[i].m);
        for (int j = 0; j < qk / 2; j++) {
            int x0 = xs[i].qs[j] & 0x0F, x1 = xs[i].qs[j] >> 4;
            ys[i * qk + j] = (float)x0 * d + m;
            ys[i * qk + j + qk / 2] = (float)x1 * d + m;
        }
    }
}
/* k_quants.rs:270-297 */
static float vec_dot_q4_1_q8_1(int64_t n, const orc_block_q4_1* xs, const orc_block_q8_1* ys) {
    float sumf = 0.f;
    for (int64_t b = 0; b < n / 32; b++) {
        int32_t sumi = 0;
        for (int j = 0; j < 16; j++) {
            int v0 = xs[b].qs[j] & 0x0F, v1 = xs[b].qs[j] >> 4;
            sumi += v0 * (int)ys[b].qs[j] + v1 * (int)ys[b].qs[j + 16];
        }
        sumf += (float)sumi * orc_f16_to_f32(xs[b].d) * orc_f16_to_f32(ys[b].d)
              + orc_f16_to_f32(xs[b].m) * orc_f16_to_f32(ys[b].s);
    }
    return sumf;
}

/* ------------------------------------------------------------------ Q5_0 */
static inline uint32_t rd_u32le(const uint8_t* p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24); }
static inline void wr_u32le(uint8_t* p, uint32_t v) { p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); p[2] = (uint8_t)(v >> 16); p[3] = (uint8_t)(v >> 24); }
/* k_quants.rs:404-440 */
static void quantize_q5_0(const float* xs, int64_t k, orc_block_q5_0* ys) {
    const int qk = 32;
    for (int64_t i = 0; i < k / qk; i++) {
        const float* x = xs + i * qk;
        float amax = 0.f, max = 0.f;
        for (int j = 0; j < qk; j++) {
            if (amax < fabsf(x[j])) { amax = fabsf(x[j]); max = x[j]; }
        }
        float d = max / -16.0f;
        float id = (d != 0.f) ? 1.f / d : 0.f;
        ys[i].d = orc_f32_to_f16(d);
        uint32_t qh = 0;
        for (int j = 0; j < qk / 2; j++) {
            float x0 = x[j] * id, x1 = x[j + qk / 2] * id;
            int8_t s0 = sat_i8(x0 + 16.5f); if (s0 > 31) s0 = 31;     /* `as i8` then .min(31) then `as u8` */
            int8_t s1 = sat_i8(x1 + 16.5f); if (s1 > 31) s1 = 31;
            uint8_t xi0 = (uint8_t)s0, xi1 = (uint8_t)s1;
            ys[i].qs[j] = (uint8_t)((xi0 & 0x0F) | ((xi1 & 0x0F) << 4));
            qh |= (((uint32_t)xi0 & 0x10u) >> 4) << j;
            qh |= (((uint32_t)xi1 & 0x10u) >> 4) << (j + qk / 2);
        }
        wr_u32le(ys[i].qh, qh);
    }
}
/* k_quants.rs:443-465 */
static void dequantize_q5_0(const orc_block_q5_0* xs, int64_t k, float* ys) {
    const int qk = 32;
    for (int64_t i = 0; i < k / qk; i++) {
        float d = orc_f16_to_f32(xs[i].d);
        uint32_t qh = rd_u32le(xs[i].qh);
        for (int j = 0; j < qk / 2; j++) {
            uint8_t xh_0 = (uint8_t)(((qh >> j) << 4) & 0x10);
            uint8_t xh_1 = (uint8_t)((qh >> (j + 12)) & 0x10);
            int x0 = (int)((xs[i].qs[j] & 0x0F) | xh_0) - 16;
            int x1 = (int)((xs[i].qs[j] >> 4) | xh_1) - 16;
            ys[i * qk + j] = (float)x0 * d;
            ys[i * qk + j + qk / 2] = (float)x1 * d;
        }
    }
}
/* k_quants.rs:381-402 (vec_dot is vec_dot_unopt on every target, :367-379) */
static float vec_dot_q5_0_q8_0(int64_t n, const orc_block_q5_0* xs, const orc_block_q8_0* ys) {
    float sumf = 0.f;
    for (int64_t b = 0; b < n / 32; b++) {
        uint32_t qh = rd_u32le(xs[b].qh);
        int32_t sumi = 0;
        for (int j = 0; j < 16; j++) {
            uint8_t xh_0 = (uint8_t)(((qh & (1u << j)) >> j) << 4);
            uint8_t xh_1 = (uint8_t)((qh & (1u << (j + 16))) >> (j + 12));
            int x0 = ((int)(xs[b].qs[j] & 0x0F) | (int)xh_0) - 16;
            int x1 = ((int)(xs[b].qs[j] >> 4) | (int)xh_1) - 16;
            sumi += x0 * (int)ys[b].qs[j] + x1 * (int)ys[b].qs[j + 16];
        }
        sumf += (float)sumi * orc_f16_to_f32(xs[b].d) * orc_f16_to_f32(ys[b].d);
    }
    return sumf;
}

/* ------------------------------------------------------------------ Q5_1 */
/* k_quants.rs:511-553 */
static void quantize_q5_1(const float* xs, int64_t k, orc_block_q5_1* ys) {
    const int qk = 32;
    for (int64_t i = 0; i < k / qk; i++) {
        const float* x = xs + i * qk;
        float min = INFINITY, max = -INFINITY;
        for (int j = 0; j < qk; j++) { min = rmin(x[j], min); max = rmax(x[j], max); }
        float d = (max - min) / 31.0f;
        float id = (d != 0.f) ? 1.f / d : 0.f;
        ys[i].d = orc_f32_to_f16(d);
        ys[i].m = orc_f32_to_f16(min);
        uint32_t qh = 0;
        for (int j = 0; j < qk / 2; j++) {
            float x0 = (x[j] - min) * id, x1 = (x[qk / 2 + j] - min) * id;
            uint8_t xi0 = sat_u8(x0 + 0.5f), xi1 = sat_u8(x1 + 0.5f);
            ys[i].qs[j] = (uint8_t)((xi0 & 0x0F) | ((xi1 & 0x0F) << 4));
            qh |= (((uint32_t)xi0 & 0x10u) >> 4) << j;
            qh |= (((uint32_t)xi1 & 0x10u) >> 4) << (j + qk / 2);
        }
        wr_u32le(ys[i].qh, qh);
    }
}
/* k_quants.rs:556-581 */
static void dequantize_q5_1(const orc_block_q5_1* xs, int64_t k, float* ys) {
    const int qk = 32;
    for (int64_t i = 0; i < k / qk; i++) {
        float d = orc_f16_to_f32(xs[i].d), m = orc_f16_to_f32(xs[i].m);
        uint32_t qh = rd_u32le(xs[i].qh);
        for (int j = 0; j < qk / 2; j++) {
            uint8_t xh_0 = (uint8_t)(((qh >> j) << 4) & 0x10);
            uint8_t xh_1 = (uint8_t)((qh >> (j + 12)) & 0x10);
            int x0 = (xs[i].qs[j] & 0x0F) | xh_0;
            int x1 = (xs[i].qs[j] >> 4) | xh_1;
            ys[i * qk + j] = (float)x0 * d + m;
            ys[i * qk + j + qk / 2] = (float)x1 * d + m;
        }
    }
}
/* k_quants.rs:477-509 */
static float vec_dot_q5_1_q8_1(int64_t n, const orc_block_q5_1* xs, const orc_block_q8_1* ys) {
    float sumf = 0.f;
    for (int64_t b = 0; b < n / 32; b++) {
        uint32_t qh = rd_u32le(xs[b].qh);
        int32_t sumi = 0;
        for (int j = 0; j < 16; j++) {
            int xh_0 = (int)(((qh >> j) << 4) & 0x10);
            int xh_1 = (int)((qh >> (j + 12)) & 0x10);
            int x0 = (xs[b].qs[j] & 0xF) | xh_0;
            int x1 = (xs[b].qs[j] >> 4) | xh_1;
            sumi += x0 * (int)ys[b].qs[j] + x1 * (int)ys[b].qs[j + 16];
        }
        sumf += (float)sumi * orc_f16_to_f32(xs[b].d) * orc_f16_to_f32(ys[b].d)
              + orc_f16_to_f32(xs[b].m) * orc_f16_to_f32(ys[b].s);
    }
    return sumf;
}

/* ------------------------------------------------------------------ Q8_1 */
/* k_quants.rs:700-729.  `s` is computed in f16 arithmetic: f16(sum) * d, i.e. the two f16 values widened,
 * multiplied in f32 and rounded once (half 2.5.0, binary16 arithmetic through f32). */
static void quantize_q8_1(const float* xs, int64_t k, orc_block_q8_1* ys) {
    for (int64_t i = 0; i < k / 32; i++) {
        const float* x = xs + i * 32;
        float amax = 0.f;
        for (int j = 0; j < 32; j++) amax = rmax(amax, fabsf(x[j]));
        float d = amax / 127.0f;
        float id = (d != 0.f) ? 1.f / d : 0.f;
        ys[i].d = orc_f32_to_f16(d);
        int32_t sum = 0;
        for (int j = 0; j < 16; j++) {
            ys[i].qs[j] = sat_i8(roundf(x[j] * id));
            ys[i].qs[j + 16] = sat_i8(roundf(x[j + 16] * id));
            sum += (int32_t)ys[i].qs[j] + (int32_t)ys[i].qs[j + 16];
        }
        ys[i].s = orc_f32_to_f16(orc_f16_to_f32(orc_f32_to_f16((float)sum)) * orc_f16_to_f32(ys[i].d));
    }
}
/* k_quants.rs:680-698 */
static float vec_dot_q8_1_q8_1(int64_t n, const orc_block_q8_1* xs, const orc_block_q8_1* ys) {
    float sumf = 0.f;
    for (int64_t b = 0; b < n / 32; b++) {
        int32_t sum_i = 0;
        for (int j = 0; j < 32; j++) sum_i += (int)xs[b].qs[j] * (int)ys[b].qs[j];
        sumf += (float)sum_i * orc_f16_to_f32(xs[b].d) * orc_f16_to_f32(ys[b].d);
    }
    return sumf;
}

/* ------------------------------------------------------------------ Q8_0 */
/* k_quants.rs:605-634 */
static void quantize_q8_0(const float* xs, int64_t k, orc_block_q8_0* ys) {
    for (int64_t i = 0; i < k / 32; i++) {
        const float* x = xs + i * 32;
        float amax = 0.f;
        for (int j = 0; j < 32; j++) amax = rmax(amax, fabsf(x[j]));
        float d = amax / 127.0f;
        float id = (d != 0.f) ? 1.f / d : 0.f;
        ys[i].d = orc_f32_to_f16(d);
        for (int j = 0; j < 32; j++) ys[i].qs[j] = sat_i8(roundf(x[j] * id));
    }
}
/* k_quants.rs:587-603 */
static void dequantize_q8_0(const orc_block_q8_0* xs, int64_t k, float* ys) {
    for (int64_t i = 0; i < k / 32; i++) {
        float d = orc_f16_to_f32(xs[i].d);
        for (int j = 0; j < 32; j++) ys[i * 32 + j] = (float)xs[i].qs[j] * d;
    }
}
/* k_quants.rs:650-668 */
static float vec_dot_q8_0_q8_0(int64_t n, const orc_block_q8_0* xs, const orc_block_q8_0* ys) {
    float sumf = 0.f;
    for (int64_t b = 0; b < n / 32; b++) {
        int32_t sum_i = 0;
        for (int j = 0; j < 32; j++) sum_i += (int)xs[b].qs[j] * (int)ys[b].qs[j];
        sumf += (float)sum_i * orc_f16_to_f32(xs[b].d) * orc_f16_to_f32(ys[b].d);
    }
    return sumf;
}

/* ------------------------------------------------------------------ Q4K */
/* utils.rs:50-60 */
static inline void get_scale_min_k4(int j, const uint8_t* q, uint8_t* d, uint8_t* m) {
    if (j < 4) {
        *d = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}
/* Total order of Rust's f32::total_cmp as a sortable integer key. */
static inline int32_t total_key(float f) {
    int32_t b;
    memcpy(&b, &f, 4);
    b ^= (int32_t)(((uint32_t)(b >> 31)) >> 1);
    return b;
}
/* utils.rs:202-259 */
static void make_qkx1_quants(int nmax, int ntry, const float* x, int n, float* out_scale, float* out_min) {
    uint8_t l[32];
    memset(l, 0, sizeof l);
    float min = x[0], max = x[0];
    for (int i = 1; i < n; i++) {
        if (total_key(x[i]) < total_key(min)) min = x[i];   /* min_by keeps the first minimum */
        if (total_key(x[i]) >= total_key(max)) max = x[i];  /* max_by keeps the last maximum  */
    }
    if (max == min) { *out_scale = 0.f; *out_min = 0.f; return; }
    min = rmin(min, 0.f);
    float iscale = (float)nmax / (max - min);
    float scale = 1.0f / iscale;
    for (int t = 0; t < ntry; t++) {
        float sumlx = 0.f;
        int32_t suml2 = 0;
        int did_change = 0;
        for (int i = 0; i < n; i++) {
            int32_t li = nearest_int(iscale * (x[i] - min));
            if (li < 0) li = 0;
            if (li > nmax) li = nmax;
            uint8_t c = (uint8_t)li;
            if (c != l[i]) { l[i] = c; did_change = 1; }
            sumlx += (x[i] - min) * (float)li;
            suml2 += li * li;
        }
        scale = sumlx / (float)suml2;
        float sum = 0.f;
        for (int i = 0; i < n; i++) sum += x[i] - scale * (float)l[i];
        min = sum / (float)n;
        if (min > 0.f) min = 0.f;
        iscale = 1.0f / scale;
        if (!did_change) break;
    }
    *out_scale = scale;
    *out_min = -min;
}
/* k_quants.rs:1287-1345 */
static void quantize_q4k(const float* xs, int64_t k, orc_block_q4k* ys) {
    for (int64_t b = 0; b < k / 256; b++) {
        const float* x = xs + b * 256;
        orc_block_q4k* block = &ys[b];
        float mins[8], scales[8];
        for (int j = 0; j < 8; j++) make_qkx1_quants(15, 5, x + 32 * j, 32, &scales[j], &mins[j]);
        float max_scale = 0.f, max_min = 0.f;
        for (int j = 0; j < 8; j++) { max_scale = rmax(scales[j], max_scale); max_min = rmax(mins[j], max_min); }
        float inv_scale = max_scale > 0.f ? 63.0f / max_scale : 0.f;
        float inv_min = max_min > 0.f ? 63.0f / max_min : 0.f;
        for (int j = 0; j < 8; j++) {
            int32_t lsi = nearest_int(inv_scale * scales[j]); if (lsi > 63) lsi = 63;
            int32_t lmi = nearest_int(inv_min * mins[j]);     if (lmi > 63) lmi = 63;
            uint8_t ls = (uint8_t)lsi, lm = (uint8_t)lmi;
            if (j < 4) {
                block->scales[j] = ls;
                block->scales[j + 4] = lm;
            } else {
                block->scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                block->scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
                block->scales[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        block->d = orc_f32_to_f16(max_scale / 63.0f);
        block->dmin = orc_f32_to_f16(max_min / 63.0f);
        uint8_t l[256];
        memset(l, 0, sizeof l);
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m;
            get_scale_min_k4(j, block->scales, &sc, &m);
            float d = orc_f16_to_f32(block->d) * (float)sc;
            if (d != 0.f) {
                float dm = orc_f16_to_f32(block->dmin) * (float)m;
                for (int ii = 0; ii < 32; ii++) {
                    int32_t lv = nearest_int((x[32 * j + ii] + dm) / d);
                    if (lv < 0) lv = 0;
                    if (lv > 15) lv = 15;
                    l[32 * j + ii] = (uint8_t)lv;
                }
            }
        }
        for (int j = 0; j < 256; j += 64)
            for (int lv = 0; lv < 32; lv++)
                block->qs[(j / 64) * 32 + lv] = (uint8_t)(l[j + lv] | (l[j + lv + 32] << 4));
    }
}
/* k_quants.rs:1347-1374 */
static void dequantize_q4k(const orc_block_q4k* xs, int64_t k, float* ys) {
    for (int64_t b = 0; b < k / 256; b++) {
        const orc_block_q4k* block = &xs[b];
        float* y = ys + b * 256;
        float d = orc_f16_to_f32(block->d);
        float min = orc_f16_to_f32(block->dmin);
        int is = 0, yi = 0;
        for (int j = 0; j < 256; j += 64) {
            const uint8_t* q = block->qs + j / 2;
            uint8_t sc, m;
            get_scale_min_k4(is, block->scales, &sc, &m);
            float d1 = d * (float)sc, m1 = min * (float)m;
            get_scale_min_k4(is + 1, block->scales, &sc, &m);
            float d2 = d * (float)sc, m2 = min * (float)m;
            for (int t = 0; t < 32; t++) y[yi++] = d1 * (float)(q[t] & 0xF) - m1;
            for (int t = 0; t < 32; t++) y[yi++] = d2 * (float)(q[t] >> 4) - m2;
            is += 2;
        }
    }
}
/* k_quants.rs:1205-1285 */
static float vec_dot_q4k_q8k(int64_t n, const orc_block_q4k* xs, const orc_block_q8k* ys) {
    int8_t aux8[256];
    int16_t aux16[8];
    float sums[8] = {0};
    int32_t aux32[8];
    float sumf = 0.f;
    for (int64_t b = 0; b < n / 256; b++) {
        const orc_block_q4k* x = &xs[b];
        const orc_block_q8k* y = &ys[b];
        memset(aux32, 0, sizeof aux32);
        int8_t* a = aux8;
        const uint8_t* q4 = x->qs;
        for (int j = 0; j < 4; j++) {
            for (int l = 0; l < 32; l++) a[l] = (int8_t)(q4[l] & 0xF);
            a += 32;
            for (int l = 0; l < 32; l++) a[l] = (int8_t)(q4[l] >> 4);
            a += 32;
            q4 += 32;
        }
        uint8_t scales[8], mins[8];
        for (int j = 0; j < 8; j++) get_scale_min_k4(j, x->scales, &scales[j], &mins[j]);
        int32_t sumi = 0;
        for (int j = 0; j < 16; j++) sumi += (int32_t)y->bsums[j] * (int32_t)mins[j / 2];
        a = aux8;
        const int8_t* q8 = y->qs;
        for (int s = 0; s < 8; s++) {
            int32_t scale = scales[s];
            for (int r = 0; r < 4; r++) {
                for (int l = 0; l < 8; l++) aux16[l] = (int16_t)((int16_t)q8[l] * (int16_t)a[l]);
                for (int l = 0; l < 8; l++) aux32[l] += scale * (int32_t)aux16[l];
                q8 += 8;
                a += 8;
            }
        }
        float d = orc_f16_to_f32(x->d) * y->d;
        for (int l = 0; l < 8; l++) sums[l] += d * (float)aux32[l];
        float dmin = orc_f16_to_f32(x->dmin) * y->d;
        sumf -= dmin * (float)sumi;
    }
    float tail = 0.f;
    for (int l = 0; l < 8; l++) tail += sums[l];
    return sumf + tail;
}

/* ------------------------------------------------------------------ Q2K */
/* k_quants.rs:808-870 */
static void quantize_q2k(const float* xs, int64_t k, orc_block_q2k* ys) {
    const float Q4SCALE = 15.0f;
    for (int64_t b = 0; b < k / 256; b++) {
        const float* x = xs + b * 256;
        orc_block_q2k* block = &ys[b];
        float mins[16], scales[16];
        for (int j = 0; j < 16; j++) make_qkx1_quants(3, 5, x + 16 * j, 16, &scales[j], &mins[j]);
        float max_scale = 0.f, max_min = 0.f;
        for (int j = 0; j < 16; j++) { max_scale = rmax(scales[j], max_scale); max_min = rmax(mins[j], max_min); }
        if (max_scale > 0.f) {
            float iscale = Q4SCALE / max_scale;
            for (int j = 0; j < 16; j++) block->scales[j] = (uint8_t)nearest_int(iscale * scales[j]);
            block->d = orc_f32_to_f16(max_scale / Q4SCALE);
        } else {
            for (int j = 0; j < 16; j++) block->scales[j] = 0;
            block->d = orc_f32_to_f16(0.f);
        }
        if (max_min > 0.f) {
            float iscale = Q4SCALE / max_min;
            for (int j = 0; j < 16; j++) {
                uint8_t l = (uint8_t)nearest_int(iscale * mins[j]);
                block->scales[j] |= (uint8_t)(l << 4);
            }
            block->dmin = orc_f32_to_f16(max_min / Q4SCALE);
        } else {
            block->dmin = orc_f32_to_f16(0.f);
        }
        uint8_t big_l[256];
        memset(big_l, 0, sizeof big_l);
        for (int j = 0; j < 16; j++) {
            float d = orc_f16_to_f32(block->d) * (float)(block->scales[j] & 0xF);
            if (d == 0.f) continue;
            float dm = orc_f16_to_f32(block->dmin) * (float)(block->scales[j] >> 4);
            for (int ii = 0; ii < 16; ii++) {
                int32_t ll = nearest_int((x[16 * j + ii] + dm) / d);
                big_l[16 * j + ii] = (uint8_t)(ll < 0 ? 0 : ll > 3 ? 3 : ll);
            }
        }
        for (int j = 0; j < 256; j += 128)
            for (int ll = 0; ll < 32; ll++)
                block->qs[j / 4 + ll] = (uint8_t)(big_l[j + ll] | (big_l[j + ll + 32] << 2) | (big_l[j + ll + 64] << 4) | (big_l[j + ll + 96] << 6));
    }
}
/* k_quants.rs:872-908 */
static void dequantize_q2k(const orc_block_q2k* xs, int64_t k, float* ys) {
    for (int64_t b = 0; b < k / 256; b++) {
        const orc_block_q2k* block = &xs[b];
        float d = orc_f16_to_f32(block->d);
        float min = orc_f16_to_f32(block->dmin);
        int is = 0;
        for (int n = 0; n < 256; n += 128) {
            const uint8_t* qs = block->qs + n / 4;
            float* y = ys + b * 256 + n;
            int yi = 0, shift = 0;
            for (int j = 0; j < 4; j++) {
                uint8_t sc = block->scales[is++];
                float dl = d * (float)(sc & 0xF), ml = min * (float)(sc >> 4);
                for (int l = 0; l < 16; l++) y[yi++] = dl * (float)((qs[l] >> shift) & 3) - ml;
                sc = block->scales[is++];
                dl = d * (float)(sc & 0xF);
                ml = min * (float)(sc >> 4);
                for (int l = 16; l < 32; l++) y[yi++] = dl * (float)((qs[l] >> shift) & 3) - ml;
                shift += 2;
            }
        }
    }
}
/* k_quants.rs:755-805 (vec_dot_unopt) */
static float vec_dot_q2k_q8k(int64_t n, const orc_block_q2k* xs, const orc_block_q8k* ys) {
    float sumf = 0.f;
    for (int64_t b = 0; b < n / 256; b++) {
        const orc_block_q2k* x = &xs[b];
        const orc_block_q8k* y = &ys[b];
        const uint8_t* q2 = x->qs;
        const int8_t* q8 = y->qs;
        int32_t summs = 0;
        for (int j = 0; j < 16; j++) summs += (int32_t)y->bsums[j] * (int32_t)(x->scales[j] >> 4);
        float dall = y->d * orc_f16_to_f32(x->d);
        float dmin = y->d * orc_f16_to_f32(x->dmin);
        int32_t isum = 0;
        int is = 0;
        for (int h = 0; h < 2; h++) {
            int shift = 0;
            for (int j = 0; j < 4; j++) {
                int32_t d = x->scales[is++] & 0xF;
                int32_t isuml = 0;
                for (int l = 0; l < 16; l++) isuml += (int32_t)q8[l] * (int32_t)((q2[l] >> shift) & 3);
                isum += d * isuml;
                d = x->scales[is++] & 0xF;
                isuml = 0;
                for (int l = 16; l < 32; l++) isuml += (int32_t)q8[l] * (int32_t)((q2[l] >> shift) & 3);
                isum += d * isuml;
                shift += 2;
                q8 += 32;
            }
            q2 += 32;
        }
        sumf += dall * (float)isum - dmin * (float)summs;
    }
    return sumf;
}

/* ------------------------------------------------------------------ Q3K */
/* make_q3_quants, utils.rs:262-328 */
static float make_q3_quants(const float* x, int n, int nmax, int do_rmse) {
    int8_t l[16];
    float max = 0.f, amax = 0.f;
    for (int i = 0; i < n; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; max = x[i]; }
    }
    if (amax == 0.f) return 0.f;
    float iscale = -(float)nmax / max;
    if (do_rmse) {
        float sumlx = 0.f, suml2 = 0.f;
        for (int i = 0; i < n; i++) {
            int32_t li = nearest_int(iscale * x[i]);
            li = li < -nmax ? -nmax : li > nmax - 1 ? nmax - 1 : li;
            l[i] = (int8_t)li;
            float w = x[i] * x[i];
            sumlx += w * x[i] * (float)li;
            suml2 += w * (float)(li * li);
        }
        for (int t = 0; t < 5; t++) {
            int n_changed = 0;
            for (int i = 0; i < n; i++) {
                float w = x[i] * x[i];
                float slx = sumlx - w * x[i] * (float)l[i];
                if (slx > 0.f) {
                    float sl2 = suml2 - w * (float)((int32_t)l[i] * (int32_t)l[i]);
                    int32_t new_l = nearest_int(x[i] * sl2 / slx);
                    new_l = new_l < -nmax ? -nmax : new_l > nmax - 1 ? nmax - 1 : new_l;
                    if (new_l != (int32_t)l[i]) {
                        slx += w * x[i] * (float)new_l;
                        sl2 += w * (float)(new_l * new_l);
                        if (sl2 > 0.f && slx * slx * suml2 > sumlx * sumlx * sl2) {
                            l[i] = (int8_t)new_l;
                            sumlx = slx;
                            suml2 = sl2;
                            n_changed++;
                        }
                    }
                }
            }
            if (n_changed == 0) break;
        }
        return sumlx / suml2;
    }
    return 1.0f / iscale;
}
/* the sixteen 6-bit scales (stored + 32) of a block: low four bits in scales[0..8) (two per byte), high
 * two bits in scales[8..12) -- the KMASK shuffle of k_quants.rs:1013-1019 / 1137-1145 */
static inline int q3k_scale(const uint8_t* scales, int j) {
    int lo = j < 8 ? (scales[j] & 0xF) : (scales[j - 8] >> 4);
    int hi = (scales[8 + j % 4] >> (2 * (j / 4))) & 3;
    return lo | (hi << 4);
}
/* k_quants.rs:1047-1129 */
static void quantize_q3k(const float* xs, int64_t k, orc_block_q3k* ys) {
    for (int64_t b = 0; b < k / 256; b++) {
        const float* x = xs + b * 256;
        orc_block_q3k* block = &ys[b];
        float scales[16];
        for (int j = 0; j < 16; j++) scales[j] = make_q3_quants(x + 16 * j, 16, 4, 1);
        float max_scale = 0.f;
        for (int j = 0; j < 16; j++)
            if (fabsf(scales[j]) > fabsf(max_scale)) max_scale = scales[j];
        memset(block->scales, 0, sizeof block->scales);
        if (max_scale != 0.f) {
            float iscale = -32.0f / max_scale;
            for (int j = 0; j < 16; j++) {
                int32_t lv = nearest_int(iscale * scales[j]);
                lv = (lv < -32 ? -32 : lv > 31 ? 31 : lv) + 32;
                if (j < 8) block->scales[j] = (uint8_t)(lv & 0xF);
                else block->scales[j - 8] |= (uint8_t)((lv & 0xF) << 4);
                lv >>= 4;
                block->scales[j % 4 + 8] |= (uint8_t)(lv << (2 * (j / 4)));
            }
            block->d = orc_f32_to_f16(1.0f / iscale);
        } else {
            block->d = orc_f32_to_f16(0.f);
        }
        int8_t l[256];
        memset(l, 0, sizeof l);
        for (int j = 0; j < 16; j++) {
            int sc = q3k_scale(block->scales, j) - 32;
            float d = orc_f16_to_f32(block->d) * (float)sc;
            if (d != 0.f)
                for (int ii = 0; ii < 16; ii++) {
                    int32_t lv = nearest_int(x[16 * j + ii] / d);
                    l[16 * j + ii] = (int8_t)((lv < -4 ? -4 : lv > 3 ? 3 : lv) + 4);
                }
        }
        memset(block->hmask, 0, sizeof block->hmask);
        int m = 0;
        uint8_t hm = 1;
        for (int i = 0; i < 256; i++) {
            if (l[i] > 3) { block->hmask[m] |= hm; l[i] -= 4; }
            if (++m == 32) { m = 0; hm <<= 1; }
        }
        for (int j = 0; j < 256; j += 128)
            for (int lv = 0; lv < 32; lv++)
                block->qs[j / 4 + lv] = (uint8_t)(l[j + lv] | (l[j + lv + 32] << 2) | (l[j + lv + 64] << 4) | (l[j + lv + 96] << 6));
    }
}
/* k_quants.rs:1131-1186 */
static void dequantize_q3k(const orc_block_q3k* xs, int64_t k, float* ys) {
    for (int64_t b = 0; b < k / 256; b++) {
        const orc_block_q3k* block = &xs[b];
        float d_all = orc_f16_to_f32(block->d);
        uint8_t m = 1;
        int is = 0;
        for (int n = 0; n < 256; n += 128) {
            const uint8_t* qs = block->qs + n / 4;
            float* y = ys + b * 256 + n;
            int shift = 0;
            for (int j = 0; j < 4; j++) {
                for (int half = 0; half < 2; half++) {
                    float dl = d_all * ((float)(int8_t)q3k_scale(block->scales, is) - 32.0f);
                    for (int i = 0; i < 16; i++) {
                        int8_t q = (int8_t)((int8_t)((qs[i + 16 * half] >> shift) & 3) - ((block->hmask[i + 16 * half] & m) == 0 ? 4 : 0));
                        y[32 * j + 16 * half + i] = dl * (float)q;
                    }
                    is++;
                }
                shift += 2;
                m <<= 1;
            }
        }
    }
}
/* k_quants.rs:927-1045 (vec_dot_unopt) */
static float vec_dot_q3k_q8k(int64_t n, const orc_block_q3k* xs, const orc_block_q8k* ys) {
    int8_t aux8[256];
    int16_t aux16[8];
    float sums[8] = {0};
    int32_t aux32[8];
    for (int64_t b = 0; b < n / 256; b++) {
        const orc_block_q3k* x = &xs[b];
        const orc_block_q8k* y = &ys[b];
        memset(aux32, 0, sizeof aux32);
        int8_t* a = aux8;
        const uint8_t* q3 = x->qs;
        uint8_t m = 1;
        for (int h = 0; h < 2; h++) {
            for (int sh = 0; sh < 8; sh += 2) {
                for (int l = 0; l < 32; l++) a[l] = (int8_t)(((q3[l] >> sh) & 3) - ((x->hmask[l] & m) ? 0 : 4));
                a += 32;
                m <<= 1;
            }
            q3 += 32;
        }
        a = aux8;
        const int8_t* q8 = y->qs;
        for (int j = 0; j < 16; j++) {
            int32_t scale = (int32_t)(int8_t)q3k_scale(x->scales, j) - 32;
            for (int r = 0; r < 2; r++) {
                for (int l = 0; l < 8; l++) aux16[l] = (int16_t)((int16_t)q8[l] * (int16_t)a[l]);
                for (int l = 0; l < 8; l++) aux32[l] += scale * (int32_t)aux16[l];
                q8 += 8;
                a += 8;
            }
        }
        float d = orc_f16_to_f32(x->d) * y->d;
        for (int l = 0; l < 8; l++) sums[l] += d * (float)aux32[l];
    }
    float total = 0.f;
    for (int l = 0; l < 8; l++) total += sums[l];
    return total;
}

/* ------------------------------------------------------------------ Q5K */
/* k_quants.rs:1487-1561 */
static void quantize_q5k(const float* xs, int64_t k, orc_block_q5k* ys) {
    for (int64_t b = 0; b < k / 256; b++) {
        const float* x = xs + b * 256;
        orc_block_q5k* block = &ys[b];
        float mins[8], scales[8];
        for (int j = 0; j < 8; j++) make_qkx1_quants(31, 5, x + 32 * j, 32, &scales[j], &mins[j]);
        float max_scale = 0.f, max_min = 0.f;
        for (int j = 0; j < 8; j++) { max_scale = rmax(scales[j], max_scale); max_min = rmax(mins[j], max_min); }
        float inv_scale = max_scale > 0.f ? 63.0f / max_scale : 0.f;
        float inv_min = max_min > 0.f ? 63.0f / max_min : 0.f;
        for (int j = 0; j < 8; j++) {
            int32_t lsi = nearest_int(inv_scale * scales[j]); if (lsi > 63) lsi = 63;
            int32_t lmi = nearest_int(inv_min * mins[j]);     if (lmi > 63) lmi = 63;
            uint8_t ls = (uint8_t)lsi, lm = (uint8_t)lmi;
            if (j < 4) {
                block->scales[j] = ls;
                block->scales[j + 4] = lm;
            } else {
                block->scales[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                block->scales[j - 4] |= (uint8_t)((ls >> 4) << 6);
                block->scales[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        block->d = orc_f32_to_f16(max_scale / 63.0f);
        block->dmin = orc_f32_to_f16(max_min / 63.0f);
        uint8_t l[256];
        memset(l, 0, sizeof l);
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m;
            get_scale_min_k4(j, block->scales, &sc, &m);
            float d = orc_f16_to_f32(block->d) * (float)sc;
            if (d == 0.f) continue;
            float dm = orc_f16_to_f32(block->dmin) * (float)m;
            for (int ii = 0; ii < 32; ii++) {
                int32_t lv = nearest_int((x[32 * j + ii] + dm) / d);
                l[32 * j + ii] = (uint8_t)(lv < 0 ? 0 : lv > 31 ? 31 : lv);
            }
        }
        memset(block->qh, 0, sizeof block->qh);
        uint8_t m1 = 1, m2 = 2;
        for (int n = 0; n < 256; n += 64) {
            int offset = (n / 64) * 32;
            for (int j = 0; j < 32; j++) {
                uint8_t l1 = l[n + j], l2 = l[n + j + 32];
                if (l1 > 15) { l1 -= 16; block->qh[j] |= m1; }
                if (l2 > 15) { l2 -= 16; block->qh[j] |= m2; }
                block->qs[offset + j] = (uint8_t)(l1 | (l2 << 4));
            }
            m1 <<= 2;
            m2 <<= 2;
        }
    }
}
/* k_quants.rs:1563-1595 */
static void dequantize_q5k(const orc_block_q5k* xs, int64_t k, float* ys) {
    for (int64_t b = 0; b < k / 256; b++) {
        const orc_block_q5k* block = &xs[b];
        float* y = ys + b * 256;
        float d = orc_f16_to_f32(block->d);
        float min = orc_f16_to_f32(block->dmin);
        int is = 0, yi = 0;
        uint8_t u1 = 1, u2 = 2;
        for (int j = 0; j < 256; j += 64) {
            const uint8_t* ql = block->qs + j / 2;
            uint8_t sc, m;
            get_scale_min_k4(is, block->scales, &sc, &m);
            float d1 = d * (float)sc, m1 = min * (float)m;
            get_scale_min_k4(is + 1, block->scales, &sc, &m);
            float d2 = d * (float)sc, m2 = min * (float)m;
            for (int t = 0; t < 32; t++) {
                float to_add = (block->qh[t] & u1) ? 16.f : 0.f;
                y[yi++] = d1 * ((float)(ql[t] & 0xF) + to_add) - m1;
            }
            for (int t = 0; t < 32; t++) {
                float to_add = (block->qh[t] & u2) ? 16.f : 0.f;
                y[yi++] = d2 * ((float)(ql[t] >> 4) + to_add) - m2;
            }
            is += 2;
            u1 <<= 2;
            u2 <<= 2;
        }
    }
}
/* k_quants.rs:1394-1485 (vec_dot_unopt) */
static float vec_dot_q5k_q8k(int64_t n, const orc_block_q5k* xs, const orc_block_q8k* ys) {
    int8_t aux8[256];
    int16_t aux16[8];
    float sums[8] = {0};
    int32_t aux32[8];
    float sumf = 0.f;
    for (int64_t b = 0; b < n / 256; b++) {
        const orc_block_q5k* x = &xs[b];
        const orc_block_q8k* y = &ys[b];
        memset(aux32, 0, sizeof aux32);
        int8_t* a = aux8;
        const uint8_t* q5 = x->qs;
        uint8_t m = 1;
        for (int j = 0; j < 4; j++) {
            for (int l = 0; l < 32; l++) a[l] = (int8_t)((q5[l] & 0xF) + ((x->qh[l] & m) ? 16 : 0));
            a += 32;
            m <<= 1;
            for (int l = 0; l < 32; l++) a[l] = (int8_t)((q5[l] >> 4) + ((x->qh[l] & m) ? 16 : 0));
            a += 32;
            m <<= 1;
            q5 += 32;
        }
        uint8_t scales[8], mins[8];
        for (int j = 0; j < 8; j++) get_scale_min_k4(j, x->scales, &scales[j], &mins[j]);
        int32_t sumi = 0;
        for (int j = 0; j < 16; j++) sumi += (int32_t)y->bsums[j] * (int32_t)mins[j / 2];
        a = aux8;
        const int8_t* q8 = y->qs;
        for (int s = 0; s < 8; s++) {
            int32_t scale = scales[s];
            for (int r = 0; r < 4; r++) {
                for (int l = 0; l < 8; l++) aux16[l] = (int16_t)((int16_t)q8[l] * (int16_t)a[l]);
                for (int l = 0; l < 8; l++) aux32[l] += scale * (int32_t)aux16[l];
                q8 += 8;
                a += 8;
            }
        }
        float d = orc_f16_to_f32(x->d) * y->d;
        for (int l = 0; l < 8; l++) sums[l] += d * (float)aux32[l];
        float dmin = orc_f16_to_f32(x->dmin) * y->d;
        sumf -= dmin * (float)sumi;
    }
    float tail = 0.f;
    for (int l = 0; l < 8; l++) tail += sums[l];
    return sumf + tail;
}

/* ------------------------------------------------------------------ Q6K */
/* make_qx_quants, utils.rs:62-203 (the caller below uses rmse_type 1: unit weights, early return) */
static float make_qx_quants(int n, int nmax, const float* x, int8_t* ls, int rmse_type) {
    float max = 0.f, amax = 0.f;
    for (int i = 0; i < n; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; max = x[i]; }
    }
    if (amax == 0.f) {
        for (int i = 0; i < n; i++) ls[i] = 0;
        return 0.f;
    }
    float iscale = -(float)nmax / max;
    if (rmse_type == 0) {
        for (int i = 0; i < n; i++) {
            int32_t l = nearest_int(iscale * x[i]);
            l = l < -nmax ? -nmax : l > nmax - 1 ? nmax - 1 : l;
            ls[i] = (int8_t)(nmax + l);
        }
        return 1.0f / iscale;
    }
    const int weight_type = rmse_type % 2;
    float sumlx = 0.f, suml2 = 0.f;
    for (int i = 0; i < n; i++) {
        int32_t l = nearest_int(iscale * x[i]);
        l = l < -nmax ? -nmax : l > nmax - 1 ? nmax - 1 : l;
        ls[i] = (int8_t)(l + nmax);
        float w = weight_type == 1 ? x[i] * x[i] : 1.0f;
        float lf = (float)l;
        sumlx += w * x[i] * lf;
        suml2 += w * lf * lf;
    }
    float scale = sumlx / suml2;
    float best = scale * sumlx;
    for (int itry = 0; itry < 3; itry++) {
        float is2 = 1.0f / scale;
        float slx = 0.f, sl2 = 0.f;
        int changed = 0;
        for (int i = 0; i < n; i++) {
            int32_t l = nearest_int(is2 * x[i]);
            l = l < -nmax ? -nmax : l > nmax - 1 ? nmax - 1 : l;
            if (l + nmax != (int32_t)ls[i]) changed = 1;
            float w = weight_type == 1 ? x[i] * x[i] : 1.0f;
            float lf = (float)l;
            slx += w * x[i] * lf;
            sl2 += w * lf * lf;
        }
        if (!changed || sl2 == 0.0f || slx * slx <= best * sl2) break;
        for (int i = 0; i < n; i++) {
            int32_t l = nearest_int(is2 * x[i]);
            l = l < -nmax ? -nmax : l > nmax - 1 ? nmax - 1 : l;
            ls[i] = (int8_t)(nmax + l);
        }
        sumlx = slx;
        suml2 = sl2;
        scale = sumlx / suml2;
        best = scale * sumlx;
    }
    for (int itry = 0; itry < 5; itry++) {
        int n_changed = 0;
        for (int i = 0; i < n; i++) {
            float w = weight_type == 1 ? x[i] * x[i] : 1.0f;
            int32_t l = (int32_t)ls[i] - nmax;
            float slx = sumlx - w * x[i] * (float)l;
            if (slx > 0.f) {
                float sl2 = suml2 - w * (float)l * (float)l;
                int32_t new_l = nearest_int(x[i] * sl2 / slx);
                new_l = new_l < -nmax ? -nmax : new_l > nmax - 1 ? nmax - 1 : new_l;
                if (new_l != l) {
                    slx += w * x[i] * (float)new_l;
                    sl2 += w * (float)new_l * (float)new_l;
                    if (sl2 > 0.f && slx * slx * suml2 > sumlx * sumlx * sl2) {
                        ls[i] = (int8_t)(nmax + new_l);
                        sumlx = slx;
                        suml2 = sl2;
                        scale = sumlx / suml2;
                        best = scale * sumlx;
                        n_changed++;
                    }
                }
            }
        }
        if (n_changed == 0) break;
    }
    if (rmse_type < 3) return scale;
    for (int is = -4; is < 4; is++) {
        if (is == 0) continue;
        iscale = -((float)nmax + 0.1f * (float)is) / max;
        float slx = 0.f, sl2 = 0.f;
        for (int i = 0; i < n; i++) {
            int32_t l = nearest_int(iscale * x[i]);
            l = l < -nmax ? -nmax : l > nmax - 1 ? nmax - 1 : l;
            float w = weight_type == 1 ? x[i] * x[i] : 1.0f;
            float lf = (float)l;
            slx += w * x[i] * lf;
            sl2 += w * lf * lf;
        }
        if (sl2 > 0.f && slx * slx > best * sl2) {
            for (int i = 0; i < n; i++) {
                int32_t l = nearest_int(iscale * x[i]);
                l = l < -nmax ? -nmax : l > nmax - 1 ? nmax - 1 : l;
                ls[i] = (int8_t)(nmax + l);
            }
            scale = slx / sl2;
            best = scale * slx;
        }
    }
    return scale;
}
/* k_quants.rs:1673-1751 */
static void quantize_q6k(const float* xs, int64_t k, orc_block_q6k* ys) {
    int8_t l[256];
    float scales[16];
    for (int64_t b = 0; b < k / 256; b++) {
        const float* x = xs + b * 256;
        orc_block_q6k* y = &ys[b];
        float max_scale = 0.f, max_abs_scale = 0.f;
        for (int ib = 0; ib < 16; ib++) {
            float scale = make_qx_quants(16, 32, x + 16 * ib, l + 16 * ib, 1);
            scales[ib] = scale;
            float a = fabsf(scale);
            if (a > max_abs_scale) { max_abs_scale = a; max_scale = scale; }
        }
        float iscale = -128.0f / max_scale;
        y->d = orc_f32_to_f16(1.0f / iscale);
        for (int j = 0; j < 16; j++) {
            int32_t v = nearest_int(iscale * scales[j]);
            y->scales[j] = (int8_t)(v < 127 ? v : 127);   /* `as i8` wraps below -128; cannot occur: |v| <= 128 */
        }
        for (int j = 0; j < 16; j++) {
            float d = orc_f16_to_f32(y->d) * (float)y->scales[j];
            if (d == 0.f) continue;
            for (int ii = 0; ii < 16; ii++) {
                int32_t ll = nearest_int(x[16 * j + ii] / d);
                ll = ll < -32 ? -32 : ll > 31 ? 31 : ll;
                l[16 * j + ii] = (int8_t)(ll + 32);
            }
        }
        uint8_t* ql = y->ql;
        uint8_t* qh = y->qh;
        for (int j = 0; j < 256; j += 128) {
            for (int i = 0; i < 32; i++) {
                uint8_t q1 = (uint8_t)l[j + i] & 0xF, q2 = (uint8_t)l[j + i + 32] & 0xF;
                uint8_t q3 = (uint8_t)l[j + i + 64] & 0xF, q4 = (uint8_t)l[j + i + 96] & 0xF;
                ql[i] = (uint8_t)(q1 | (q3 << 4));
                ql[i + 32] = (uint8_t)(q2 | (q4 << 4));
                /* arithmetic shifts of i8 values 0..63: same as unsigned here */
                qh[i] = (uint8_t)((l[j + i] >> 4) | ((l[j + i + 32] >> 4) << 2) | ((l[j + i + 64] >> 4) << 4) |
                                  ((l[j + i + 96] >> 4) << 6));
            }
            ql += 64;
            qh += 32;
        }
    }
}
/* k_quants.rs:1753-1790 */
static void dequantize_q6k(const orc_block_q6k* xs, int64_t k, float* ys) {
    for (int64_t b = 0; b < k / 256; b++) {
        const orc_block_q6k* x = &xs[b];
        float d = orc_f16_to_f32(x->d);
        for (int n = 0; n < 256; n += 128) {
            int idx = n / 128;
            float* y = ys + b * 256 + n;
            const int8_t* sc = x->scales + 8 * idx;
            const uint8_t* ql = x->ql + 64 * idx;
            const uint8_t* qh = x->qh + 32 * idx;
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int8_t q1 = (int8_t)((int8_t)((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32);
                int8_t q2 = (int8_t)((int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
                int8_t q3 = (int8_t)((int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
                int8_t q4 = (int8_t)((int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
                y[l] = d * (float)sc[is] * (float)q1;           /* (d * sc) * q, left to right */
                y[l + 32] = d * (float)sc[is + 2] * (float)q2;
                y[l + 64] = d * (float)sc[is + 4] * (float)q3;
                y[l + 96] = d * (float)sc[is + 6] * (float)q4;
            }
        }
    }
}
/* k_quants.rs:1613-1671 (vec_dot_unopt) */
static float vec_dot_q6k_q8k(int64_t n, const orc_block_q6k* xs, const orc_block_q8k* ys) {
    int8_t aux8[256];
    int16_t aux16[8];
    float sums[8] = {0};
    float aux32[8];
    for (int64_t b = 0; b < n / 256; b++) {
        const orc_block_q6k* x = &xs[b];
        const orc_block_q8k* y = &ys[b];
        for (int l = 0; l < 8; l++) aux32[l] = 0.f;
        for (int j = 0; j < 256; j += 128) {
            int8_t* a = aux8 + j;
            const uint8_t* q4 = x->ql + j / 2;
            const uint8_t* qh = x->qh + j / 4;
            for (int l = 0; l < 32; l++) {
                a[l] = (int8_t)((int32_t)((q4[l] & 0xF) | ((qh[l] & 3) << 4)) - 32);
                a[l + 32] = (int8_t)((int32_t)((q4[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
                a[l + 64] = (int8_t)((int32_t)((q4[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
                a[l + 96] = (int8_t)((int32_t)((q4[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
            }
        }
        for (int j = 0; j < 16; j++) {
            float scale = (float)x->scales[j];
            const int8_t* q8 = y->qs + 16 * j;
            const int8_t* a = aux8 + 16 * j;
            for (int l = 0; l < 8; l++) aux16[l] = (int16_t)((int16_t)q8[l] * (int16_t)a[l]);
            for (int l = 0; l < 8; l++) aux32[l] += scale * (float)aux16[l];
            q8 += 8;
            a += 8;
            for (int l = 0; l < 8; l++) aux16[l] = (int16_t)((int16_t)q8[l] * (int16_t)a[l]);
            for (int l = 0; l < 8; l++) aux32[l] += scale * (float)aux16[l];
        }
        float d = orc_f16_to_f32(x->d) * y->d;
        for (int l = 0; l < 8; l++) sums[l] += aux32[l] * d;
    }
    float total = 0.f;
    for (int l = 0; l < 8; l++) total += sums[l];
    return total;
}

/* ------------------------------------------------------------------ Q8K */
/* k_quants.rs:1819-1856 */
static void quantize_q8k(const float* xs, int64_t k, orc_block_q8k* ys) {
    for (int64_t i = 0; i < k / 256; i++) {
        const float* x = xs + i * 256;
        orc_block_q8k* y = &ys[i];
        float max = 0.f, amax = 0.f;
        for (int j = 0; j < 256; j++) {
            if (amax < fabsf(x[j])) { amax = fabsf(x[j]); max = x[j]; }
        }
        if (amax == 0.f) {
            /* the reference leaves bsums untouched here; blocks are zero-initialised by
             * matmul (k_quants.rs:1893) so they read as zero */
            y->d = 0.f;
            memset(y->qs, 0, 256);
            memset(y->bsums, 0, sizeof y->bsums);
        } else {
            float iscale = -128.0f / max;
            for (int j = 0; j < 256; j++) {
                float v = roundf(iscale * x[j]);
                y->qs[j] = sat_i8(rmin(v, 127.f));
            }
            for (int j = 0; j < 16; j++) {
                int32_t sum = 0;
                for (int ii = 0; ii < 16; ii++) sum += y->qs[j * 16 + ii];
                y->bsums[j] = (int16_t)sum;
            }
            y->d = 1.0f / iscale;
        }
    }
}
/* k_quants.rs:1858-1870 */
static void dequantize_q8k(const orc_block_q8k* xs, int64_t k, float* ys) {
    for (int64_t i = 0; i < k / 256; i++)
        for (int j = 0; j < 256; j++) ys[i * 256 + j] = xs[i].d * (float)xs[i].qs[j];
}
/* k_quants.rs:1798-1817 */
static float vec_dot_q8k_q8k(int64_t n, const orc_block_q8k* xs, const orc_block_q8k* ys) {
    float sumf = 0.f;
    for (int64_t b = 0; b < n / 256; b++) {
        int32_t sum_i = 0;
        for (int j = 0; j < 256; j++) sum_i += (int)xs[b].qs[j] * (int)ys[b].qs[j];
        sumf += (float)sum_i * xs[b].d * ys[b].d;
    }
    return sumf;
}

/* ------------------------------------------------------------------ dispatch by dtype */
int orc_quantize(int dtype, const float* x, int64_t n, void* blocks) {
    int64_t be = orc_block_elems(dtype);
    if (be < 0 || n % be) return -1;
    switch (dtype) {
        case ORC_Q4_0: quantize_q4_0(x, n, (orc_block_q4_0*)blocks); return 0;
        case ORC_Q8_0: quantize_q8_0(x, n, (orc_block_q8_0*)blocks); return 0;
        case ORC_Q4_1: quantize_q4_1(x, n, (orc_block_q4_1*)blocks); return 0;
        case ORC_Q5_0: quantize_q5_0(x, n, (orc_block_q5_0*)blocks); return 0;
        case ORC_Q5_1: quantize_q5_1(x, n, (orc_block_q5_1*)blocks); return 0;
        case ORC_Q8_1: quantize_q8_1(x, n, (orc_block_q8_1*)blocks); return 0;
        case ORC_Q4K: memset(blocks, 0, (size_t)(n / 256) * 144); quantize_q4k(x, n, (orc_block_q4k*)blocks); return 0;
        case ORC_Q2K: memset(blocks, 0, (size_t)(n / 256) * 84); quantize_q2k(x, n, (orc_block_q2k*)blocks); return 0;
        case ORC_Q3K: memset(blocks, 0, (size_t)(n / 256) * 110); quantize_q3k(x, n, (orc_block_q3k*)blocks); return 0;
        case ORC_Q5K: memset(blocks, 0, (size_t)(n / 256) * 176); quantize_q5k(x, n, (orc_block_q5k*)blocks); return 0;
        case ORC_Q6K: memset(blocks, 0, (size_t)(n / 256) * 210); quantize_q6k(x, n, (orc_block_q6k*)blocks); return 0;
        case ORC_Q8K: quantize_q8k(x, n, (orc_block_q8k*)blocks); return 0;
    }
    return -1;
}
int orc_dequantize(int dtype, const void* blocks, int64_t n, float* y) {
    int64_t be = orc_block_elems(dtype);
    if (be < 0 || n % be) return -1;
    switch (dtype) {
        case ORC_Q4_0: dequantize_q4_0((const orc_block_q4_0*)blocks, n, y); return 0;
        case ORC_Q8_0: dequantize_q8_0((const orc_block_q8_0*)blocks, n, y); return 0;
        case ORC_Q4_1: dequantize_q4_1((const orc_block_q4_1*)blocks, n, y); return 0;
        case ORC_Q5_0: dequantize_q5_0((const orc_block_q5_0*)blocks, n, y); return 0;
        case ORC_Q5_1: dequantize_q5_1((const orc_block_q5_1*)blocks, n, y); return 0;
        case ORC_Q4K: dequantize_q4k((const orc_block_q4k*)blocks, n, y); return 0;
        case ORC_Q2K: dequantize_q2k((const orc_block_q2k*)blocks, n, y); return 0;
        case ORC_Q3K: dequantize_q3k((const orc_block_q3k*)blocks, n, y); return 0;
        case ORC_Q5K: dequantize_q5k((const orc_block_q5k*)blocks, n, y); return 0;
        case ORC_Q6K: dequantize_q6k((const orc_block_q6k*)blocks, n, y); return 0;
        case ORC_Q8K: dequantize_q8k((const orc_block_q8k*)blocks, n, y); return 0;
    }
    return -1;
}
float orc_vec_dot(int dtype, int64_t n, const void* w, const void* a) {
    switch (dtype) {
        case ORC_Q4_0: return vec_dot_q4_0_q8_0(n, (const orc_block_q4_0*)w, (const orc_block_q8_0*)a);
        case ORC_Q8_0: return vec_dot_q8_0_q8_0(n, (const orc_block_q8_0*)w, (const orc_block_q8_0*)a);
        case ORC_Q4_1: return vec_dot_q4_1_q8_1(n, (const orc_block_q4_1*)w, (const orc_block_q8_1*)a);
        case ORC_Q5_0: return vec_dot_q5_0_q8_0(n, (const orc_block_q5_0*)w, (const orc_block_q8_0*)a);
        case ORC_Q5_1: return vec_dot_q5_1_q8_1(n, (const orc_block_q5_1*)w, (const orc_block_q8_1*)a);
        case ORC_Q8_1: return vec_dot_q8_1_q8_1(n, (const orc_block_q8_1*)w, (const orc_block_q8_1*)a);
        case ORC_Q4K: return vec_dot_q4k_q8k(n, (const orc_block_q4k*)w, (const orc_block_q8k*)a);
        case ORC_Q2K: return vec_dot_q2k_q8k(n, (const orc_block_q2k*)w, (const orc_block_q8k*)a);
        case ORC_Q3K: return vec_dot_q3k_q8k(n, (const orc_block_q3k*)w, (const orc_block_q8k*)a);
        case ORC_Q5K: return vec_dot_q5k_q8k(n, (const orc_block_q5k*)w, (const orc_block_q8k*)a);
        case ORC_Q6K: return vec_dot_q6k_q8k(n, (const orc_block_q6k*)w, (const orc_block_q8k*)a);
        case ORC_Q8K: return vec_dot_q8k_q8k(n, (const orc_block_q8k*)w, (const orc_block_q8k*)a);
    }
    return NAN;
}

/* AVX2 inner loops live in moe_oracle_avx2.c (built with -mavx2 -mfma). */
float orc_vec_dot_avx2(int dtype, int64_t n, const void* w, const void* a);

int orc_has_avx2(void) {
#if defined(__x86_64__)
    return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma");
#else
    return 0;
#endif
}

/* k_quants.rs:1873-1920 */
int orc_matmul(int dtype, int64_t m, int64_t k, int64_t n, const float* lhs, const void* rhs_t,
               float* dst, int simd, int threads) {
    int64_t be = orc_block_elems(dtype);
    if (be < 0 || k % be) return -1;
    int vdt = orc_vecdot_dtype(dtype);
    int64_t kb = k / be;
    int64_t abytes = orc_block_bytes(vdt), wbytes = orc_block_bytes(dtype);
    char* lhs_b = (char*)calloc((size_t)(m * kb), (size_t)abytes);
    if (!lhs_b) return -1;
    for (int64_t r = 0; r < m; r++) orc_quantize(vdt, lhs + r * k, k, lhs_b + r * kb * abytes);
    if (simd && !orc_has_avx2()) simd = 0;
    const char* w = (const char*)rhs_t;
    for (int64_t r = 0; r < m; r++) {
        const char* lrow = lhs_b + r * kb * abytes;
        float* drow = dst + r * n;
        /* rayon splits the columns into pieces of 128..512 and runs them on the pool;
         * a static schedule over the same column range is arithmetically identical. */
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(threads > 1 ? threads : 1) if (threads > 1 && n >= 256)
#endif
        for (int64_t c = 0; c < n; c++) {
            const char* wcol = w + c * kb * wbytes;
            drow[c] = simd ? orc_vec_dot_avx2(dtype, k, wcol, lrow) : orc_vec_dot(dtype, k, wcol, lrow);
        }
    }
    free(lhs_b);
    return 0;
}

/* ------------------------------------------------------------------ softmax & friends */
/* cpu/mod.rs:132-151 with cpu/avx.rs:10-12,54-68 (STEP 32, 4 accumulators of 8 lanes) */
static float vec_sum_avx2_order(const float* row, int64_t k) {
    int64_t np = k & ~(int64_t)31;
    float acc[4][8];
    memset(acc, 0, sizeof acc);
    for (int64_t i = 0; i < np; i += 32)
        for (int j = 0; j < 4; j++)
            for (int l = 0; l < 8; l++) acc[j][l] = acc[j][l] + row[i + j * 8 + l];
    float x0[8];
    for (int l = 0; l < 8; l++) {
        float a = acc[0][l] + acc[1][l];
        float b = acc[2][l] + acc[3][l];
        x0[l] = a + b;
    }
    float t0[4];
    for (int l = 0; l < 4; l++) t0[l] = x0[l] + x0[l + 4];
    float t1a = t0[0] + t0[1], t1b = t0[2] + t0[3];
    float b = t1a + t1b;
    for (int64_t i = np; i < k; i++) b += row[i];
    return b;
}
void orc_softmax_last_dim(const float* x, int64_t rows, int64_t cols, float* y) {
    for (int64_t r = 0; r < rows; r++) {
        const float* s = x + r * cols;
        float* d = y + r * cols;
        float max = s[0];
        for (int64_t i = 1; i < cols; i++) max = rmax(max, s[i]);
        for (int64_t i = 0; i < cols; i++) d[i] = expf(s[i] - max);
        float sum = vec_sum_avx2_order(d, cols);
        for (int64_t i = 0; i < cols; i++) d[i] /= sum;
    }
}
float orc_silu(float v) { return v / (1.0f + expf(-v)); }
float orc_sigmoid(float v) { return 1.0f / (expf(-v) + 1.0f); }

void orc_rms_norm(const float* x, int64_t rows, int64_t cols, const float* alpha, float eps, float* y) {
    for (int64_t r = 0; r < rows; r++) {
        const float* s = x + r * cols;
        float sum2 = 0.f;
        for (int64_t i = 0; i < cols; i++) sum2 += s[i] * s[i];
        float m = sqrtf(sum2 / (float)cols + eps);
        for (int64_t i = 0; i < cols; i++) y[r * cols + i] = s[i] / m * alpha[i];
    }
}

void orc_gate_logits(const float* xs, int64_t T, int64_t H, const float* wg, int64_t E, float* logits) {
    for (int64_t t = 0; t < T; t++)
        for (int64_t e = 0; e < E; e++) {
            float acc = 0.f;
            for (int64_t h = 0; h < H; h++) acc += xs[t * H + h] * wg[e * H + h];
            logits[t * E + e] = acc;
        }
}

/* ------------------------------------------------------------------ routing */
int orc_route(const float* probs, int64_t T, int64_t E, int64_t k, int norm_topk,
              int32_t* topk_idx, float* topk_w, int32_t* offsets, int32_t* perm_token, float* perm_w) {
    if (k < 0 || k > E || E <= 0) return -1;
    int32_t* order = (int32_t*)malloc(sizeof(int32_t) * (size_t)E);
    int32_t* counts = (int32_t*)calloc((size_t)E + 1, sizeof(int32_t));
    if (!order || !counts) { free(order); free(counts); return -1; }
    /* pass 1: per-token selection (quantized_llama.rs:162-179) */
    for (int64_t t = 0; t < T; t++) {
        const float* rw = probs + t * E;
        /* stable sort, descending by total_cmp: insertion sort keeps equal keys in index order */
        for (int32_t i = 0; i < E; i++) {
            int32_t j = i;
            while (j > 0 && total_key(rw[order[j - 1]]) < total_key(rw[i])) { order[j] = order[j - 1]; j--; }
            order[j] = i;
        }
        float sum = 0.f;
        for (int64_t r = 0; r < k; r++) sum += rw[order[r]];
        for (int64_t r = 0; r < k; r++) {
            int32_t e = order[r];
            topk_idx[t * k + r] = e;
            topk_w[t * k + r] = norm_topk ? rw[e] / sum : rw[e];
            counts[e + 1]++;
        }
    }
    /* pass 2: per-expert lists in token order = the Vec pushes of the reference */
    offsets[0] = 0;
    for (int64_t e = 0; e < E; e++) offsets[e + 1] = offsets[e] + counts[e + 1];
    int32_t* cursor = (int32_t*)malloc(sizeof(int32_t) * (size_t)E);
    if (!cursor) { free(order); free(counts); return -1; }
    for (int64_t e = 0; e < E; e++) cursor[e] = offsets[e];
    for (int64_t t = 0; t < T; t++)
        for (int64_t r = 0; r < k; r++) {
            int32_t e = topk_idx[t * k + r];
            int32_t slot = cursor[e]++;
            perm_token[slot] = (int32_t)t;
            perm_w[slot] = topk_w[t * k + r];
        }
    free(order); free(counts); free(cursor);
    return 0;
}

/* ------------------------------------------------------------------ block */
/* Mlp::forward quantized_llama.rs:124-131 on n rows */
static int expert_mlp(int dtype, int dtype_down, int64_t n, int64_t H, int64_t F, const float* x, const void* w1,
                      const void* w3, const void* w2, float* out, int simd, int threads) {
    float* a = (float*)malloc(sizeof(float) * (size_t)(n * F));
    float* b = (float*)malloc(sizeof(float) * (size_t)(n * F));
    if (!a || !b) { free(a); free(b); return -1; }
    int rc = orc_matmul(dtype, n, H, F, x, w1, a, simd, threads);
    if (!rc) rc = orc_matmul(dtype, n, H, F, x, w3, b, simd, threads);
    if (!rc) {
        for (int64_t i = 0; i < n * F; i++) a[i] = orc_silu(a[i]) * b[i];
        rc = orc_matmul(dtype_down, n, F, H, a, w2, out, simd, threads);
    }
    free(a); free(b);
    return rc;
}

int orc_moe_forward(const orc_layer* L, const float* xs_in, int64_t T, const float* logits_in,
                    float* logits_out, float* ys, int simd, int threads) {
    const int64_t H = L->H, E = L->E, k = L->k;
    const int dtype_down = L->dtype_down ? L->dtype_down : L->dtype;
    int rc = 0;
    float* xn = NULL;
    const float* xs = xs_in;
    if (L->rms_alpha) {
        xn = (float*)malloc(sizeof(float) * (size_t)(T * H));
        if (!xn) return -1;
        orc_rms_norm(xs_in, T, H, L->rms_alpha, L->rms_eps, xn);
        xs = xn;
    }
    float* logits = (float*)malloc(sizeof(float) * (size_t)(T * E));
    float* probs = (float*)malloc(sizeof(float) * (size_t)(T * E));
    int32_t* topk_idx = (int32_t*)malloc(sizeof(int32_t) * (size_t)(T * k + 1));
    float* topk_w = (float*)malloc(sizeof(float) * (size_t)(T * k + 1));
    int32_t* offsets = (int32_t*)malloc(sizeof(int32_t) * (size_t)(E + 1));
    int32_t* perm = (int32_t*)malloc(sizeof(int32_t) * (size_t)(T * k + 1));
    float* perm_w = (float*)malloc(sizeof(float) * (size_t)(T * k + 1));
    if (logits_in) {
        memcpy(logits, logits_in, sizeof(float) * (size_t)(T * E));
    } else {
        orc_gate_logits(xs, T, H, L->gate, E, logits);
        if (L->gate_bias)
            for (int64_t t = 0; t < T; t++)
                for (int64_t e = 0; e < E; e++) logits[t * E + e] += L->gate_bias[e];
    }
    if (logits_out) memcpy(logits_out, logits, sizeof(float) * (size_t)(T * E));
    orc_softmax_last_dim(logits, T, E, probs);
    rc = orc_route(probs, T, E, k, L->norm_topk, topk_idx, topk_w, offsets, perm, perm_w);
    memset(ys, 0, sizeof(float) * (size_t)(T * H));
    for (int64_t e = 0; e < E && !rc; e++) {
        int64_t n = offsets[e + 1] - offsets[e];
        if (n == 0) continue;
        const int32_t* rows = perm + offsets[e];
        float* cur = (float*)malloc(sizeof(float) * (size_t)(n * H));
        float* out = (float*)malloc(sizeof(float) * (size_t)(n * H));
        if (!cur || !out) { free(cur); free(out); rc = -1; break; }
        for (int64_t i = 0; i < n; i++) memcpy(cur + i * H, xs + (int64_t)rows[i] * H, sizeof(float) * (size_t)H);
        rc = expert_mlp(L->dtype, dtype_down, n, H, L->F, cur, L->w1[e], L->w3[e], L->w2[e], out, simd, threads);
        if (!rc)
            for (int64_t i = 0; i < n; i++) {
                float w = perm_w[offsets[e] + i];
                float* dst = ys + (int64_t)rows[i] * H;
                for (int64_t h = 0; h < H; h++) {
                    float scaled = out[i * H + h] * w; /* broadcast_mul, then index_add */
                    dst[h] += scaled;
                }
            }
        free(cur); free(out);
    }
    if (!rc && L->Fs > 0) { /* qwen2_moe.rs:315-319 */
        float* so = (float*)malloc(sizeof(float) * (size_t)(T * H));
        if (!so) rc = -1;
        if (!rc) rc = expert_mlp(L->dtype, dtype_down, T, H, L->Fs, xs, L->sw1, L->sw3, L->sw2, so, simd, threads);
        if (!rc)
            for (int64_t t = 0; t < T; t++) {
                float g = 0.f;
                for (int64_t h = 0; h < H; h++) g += xs[t * H + h] * L->shared_gate[h];
                float s = orc_sigmoid(g);
                for (int64_t h = 0; h < H; h++) {
                    float v = so[t * H + h] * s;
                    ys[t * H + h] = ys[t * H + h] + v;
                }
            }
        free(so);
    }
    if (!rc && L->rms_alpha)
        for (int64_t i = 0; i < T * H; i++) ys[i] = ys[i] + xs_in[i]; /* quantized_llama.rs:891 */
    free(xn); free(logits); free(probs); free(topk_idx); free(topk_w); free(offsets); free(perm); free(perm_w);
    return rc;
}

/* ------------------------------------------------------------------ synthetic data */
static inline uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}
static inline void normal_pair(uint64_t seed, uint64_t idx, float* a, float* b) {
    uint64_t r = splitmix64(seed * 0xD1342543DE82EF95ull + idx);
    uint32_t u1 = (uint32_t)(r >> 32), u2 = (uint32_t)r;
    float f1 = ((float)(u1 >> 8) + 0.5f) * (1.0f / 16777216.0f);
    float f2 = (float)(u2 >> 8) * (1.0f / 16777216.0f);
    float rad = sqrtf(-2.0f * logf(f1));
    float ang = 6.28318530717958647692f * f2;
    *a = rad * cosf(ang);
    *b = rad * sinf(ang);
}
static void fill_range(uint64_t seed, int64_t base, int64_t n, float mean, float std, float* out) {
    /* element i is the (i&1) member of pair i>>1, so any split gives identical values */
    for (int64_t i = 0; i < n; i++) {
        int64_t g = base + i;
        float a, b;
        normal_pair(seed, (uint64_t)(g >> 1), &a, &b);
        out[i] = mean + std * ((g & 1) ? b : a);
    }
}
void orc_fill_normal(uint64_t seed, int64_t n, float mean, float std, float* out, int threads) {
    const int64_t chunk = 1 << 16;
    int64_t nchunks = (n + chunk - 1) / chunk;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic) num_threads(threads > 1 ? threads : 1)
#endif
    for (int64_t c = 0; c < nchunks; c++) {
        int64_t lo = c * chunk, hi = lo + chunk > n ? n : lo + chunk;
        fill_range(seed, lo, hi - lo, mean, std, out + lo);
    }
}
int orc_fill_normal_quantized(uint64_t seed, int dtype, int64_t rows, int64_t k, float std,
                              void* blocks, int threads) {
    int64_t be = orc_block_elems(dtype);
    if (be < 0 || k % be) return -1;
    int64_t row_bytes = k / be * orc_block_bytes(dtype);
    int err = 0;
#ifdef _OPENMP
#pragma omp parallel num_threads(threads > 1 ? threads : 1)
#endif
    {
        float* buf = (float*)malloc(sizeof(float) * (size_t)k);
        if (!buf) {
            err = 1;
        } else {
#ifdef _OPENMP
#pragma omp for schedule(dynamic, 16)
#endif
            for (int64_t r = 0; r < rows; r++) {
                fill_range(seed, r * k, k, 0.f, std, buf);
                orc_quantize(dtype, buf, k, (char*)blocks + r * row_bytes);
            }
        }
        free(buf);
    }
    return err ? -1 : 0;
}
