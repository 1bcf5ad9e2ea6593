/*
 * AVX2 inner loops of the CPU oracle.  TEST INFRASTRUCTURE ONLY.
 *
 * These restate the x86 vec_dot kernels the reference runs when it is built with
 * `target-cpu=native` (its .cargo/config.toml:1-2):
 *   vec_dot_q4_0_q8_0  candle-core/src/quantized/avx.rs:50-68
 *   vec_dot_q8_0_q8_0  candle-core/src/quantized/avx.rs:71-87
 *   vec_dot_q4k_q8k    candle-core/src/quantized/avx.rs:443-525
 *   vec_dot_q2k_q8k    candle-core/src/quantized/avx.rs:224-304
 *   vec_dot_q3k_q8k    candle-core/src/quantized/avx.rs:306-441
 *   vec_dot_q5k_q8k    candle-core/src/quantized/avx.rs:527-638
 *   vec_dot_q6k_q8k    candle-core/src/quantized/avx.rs:131-216
 * The integer parts are exact; the f32 accumulation order differs from the scalar
 * vec_dot_unopt, which the reference's own tests allow up to 1e-6 * k
 * (candle-core/tests/quantized_tests.rs:869-876).  Used for the CPU-baseline timing.
 */
#include "moe_oracle.h"
#include <immintrin.h>
#include <math.h>
#include <string.h>

static inline float hsum_float_8(__m256 x) { /* avx.rs:26-32 */
    __m128 res = _mm256_extractf128_ps(x, 1);
    res = _mm_add_ps(res, _mm256_castps256_ps128(x));
    res = _mm_add_ps(res, _mm_movehl_ps(res, res));
    res = _mm_add_ss(res, _mm_movehdup_ps(res));
    return _mm_cvtss_f32(res);
}
static inline __m256 mul_sum_i8_pairs_float(__m256i x, __m256i y) { /* avx.rs:12-24,43-48 */
    __m256i ax = _mm256_sign_epi8(x, x);
    __m256i sy = _mm256_sign_epi8(y, x);
    __m256i dot = _mm256_maddubs_epi16(ax, sy);
    __m256i summed = _mm256_madd_epi16(_mm256_set1_epi16(1), dot);
    return _mm256_cvtepi32_ps(summed);
}
static inline __m256i bytes_from_nibbles_32(const uint8_t* p) { /* avx.rs:34-41 */
    __m128i tmp = _mm_loadu_si128((const __m128i*)p);
    __m256i bytes = _mm256_insertf128_si256(_mm256_castsi128_si256(tmp), _mm_srli_epi16(tmp, 4), 1);
    return _mm256_and_si256(_mm256_set1_epi8(0xF), bytes);
}

static float dot_q4_0(int64_t n, const orc_block_q4_0* xs, const orc_block_q8_0* ys) {
    __m256 acc = _mm256_setzero_ps();
    for (int64_t b = 0; b < n / 32; b++) {
        __m256 d = _mm256_set1_ps(orc_f16_to_f32(xs[b].d) * orc_f16_to_f32(ys[b].d));
        __m256i bx = _mm256_sub_epi8(bytes_from_nibbles_32(xs[b].qs), _mm256_set1_epi8(8));
        __m256i by = _mm256_loadu_si256((const __m256i*)ys[b].qs);
        acc = _mm256_fmadd_ps(d, mul_sum_i8_pairs_float(bx, by), acc);
    }
    return hsum_float_8(acc);
}
static float dot_q8_0(int64_t n, const orc_block_q8_0* xs, const orc_block_q8_0* ys) {
    __m256 acc = _mm256_setzero_ps();
    for (int64_t b = 0; b < n / 32; b++) {
        __m256 d = _mm256_set1_ps(orc_f16_to_f32(xs[b].d) * orc_f16_to_f32(ys[b].d));
        __m256i bx = _mm256_loadu_si256((const __m256i*)xs[b].qs);
        __m256i by = _mm256_loadu_si256((const __m256i*)ys[b].qs);
        acc = _mm256_fmadd_ps(d, mul_sum_i8_pairs_float(bx, by), acc);
    }
    return hsum_float_8(acc);
}
static float dot_q4k(int64_t n, const orc_block_q4k* xs, const orc_block_q8k* ys) {
    const uint32_t KMASK1 = 0x3f3f3f3f, KMASK2 = 0x0f0f0f0f, KMASK3 = 0x03030303;
    const __m256i m4 = _mm256_set1_epi8(0xF);
    __m256 acc = _mm256_setzero_ps();
    __m128 acc_m = _mm_setzero_ps();
    for (int64_t b = 0; b < n / 256; b++) {
        const orc_block_q4k* x = &xs[b];
        const orc_block_q8k* y = &ys[b];
        float d = y->d * orc_f16_to_f32(x->d);
        float dmin = -y->d * orc_f16_to_f32(x->dmin);
        uint32_t utmp[4];
        memcpy(utmp, x->scales, 12);
        utmp[3] = ((utmp[2] >> 4) & KMASK2) | (((utmp[1] >> 6) & KMASK3) << 4);
        uint32_t uaux = utmp[1] & KMASK1;
        utmp[1] = (utmp[2] & KMASK2) | (((utmp[0] >> 6) & KMASK3) << 4);
        utmp[2] = uaux;
        utmp[0] &= KMASK1;
        const uint8_t* q4 = x->qs;
        const int8_t* q8 = y->qs;
        __m256i mins_and_scales = _mm256_cvtepu8_epi16(
            _mm_set_epi32((int)utmp[3], (int)utmp[2], (int)utmp[1], (int)utmp[0]));
        __m256i q8sums = _mm256_loadu_si256((const __m256i*)y->bsums);
        __m128i q8s = _mm_hadd_epi16(_mm256_extracti128_si256(q8sums, 0), _mm256_extracti128_si256(q8sums, 1));
        __m128i prod = _mm_madd_epi16(_mm256_extracti128_si256(mins_and_scales, 1), q8s);
        acc_m = _mm_fmadd_ps(_mm_set1_ps(dmin), _mm_cvtepi32_ps(prod), acc_m);
        __m128i sc128 = _mm256_extracti128_si256(mins_and_scales, 0);
        __m256i scales = _mm256_set_m128i(sc128, sc128);
        __m256i sumi = _mm256_setzero_si256();
        for (int j = 0; j < 4; j++) {
            /* 16-bit scale 2j (resp. 2j+1) broadcast to every lane: bytes {2s, 2s+1} repeated */
            __m256i shuf_l = _mm256_set1_epi16((short)(((4 * j + 1) << 8) | (4 * j)));
            __m256i shuf_h = _mm256_set1_epi16((short)(((4 * j + 3) << 8) | (4 * j + 2)));
            __m256i scale_l = _mm256_shuffle_epi8(scales, shuf_l);
            __m256i scale_h = _mm256_shuffle_epi8(scales, shuf_h);
            __m256i q4bits = _mm256_loadu_si256((const __m256i*)q4);
            q4 += 32;
            __m256i q4l = _mm256_and_si256(q4bits, m4);
            __m256i q4h = _mm256_and_si256(_mm256_srli_epi16(q4bits, 4), m4);
            __m256i q8l = _mm256_loadu_si256((const __m256i*)q8);
            q8 += 32;
            __m256i p16l = _mm256_madd_epi16(scale_l, _mm256_maddubs_epi16(q4l, q8l));
            sumi = _mm256_add_epi32(sumi, p16l);
            __m256i q8h = _mm256_loadu_si256((const __m256i*)q8);
            q8 += 32;
            __m256i p16h = _mm256_madd_epi16(scale_h, _mm256_maddubs_epi16(q4h, q8h));
            sumi = _mm256_add_epi32(sumi, p16h);
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    acc_m = _mm_add_ps(acc_m, _mm_movehl_ps(acc_m, acc_m));
    acc_m = _mm_add_ss(acc_m, _mm_movehdup_ps(acc_m));
    return hsum_float_8(acc) + _mm_cvtss_f32(acc_m);
}

static float dot_q2k(int64_t n, const orc_block_q2k* xs, const orc_block_q8k* ys) {
    const __m256i m3 = _mm256_set1_epi8(3);
    const __m128i m4 = _mm_set1_epi8(0xF);
    __m256 acc = _mm256_setzero_ps();
    for (int64_t b = 0; b < n / 256; b++) {
        const orc_block_q2k* x = &xs[b];
        const orc_block_q8k* y = &ys[b];
        float d = y->d * orc_f16_to_f32(x->d);
        float dmin = -y->d * orc_f16_to_f32(x->dmin);
        const uint8_t* q2 = x->qs;
        const int8_t* q8 = y->qs;
        __m128i mins_and_scales = _mm_loadu_si128((const __m128i*)x->scales);
        __m128i scales8 = _mm_and_si128(mins_and_scales, m4);
        __m128i mins8 = _mm_and_si128(_mm_srli_epi16(mins_and_scales, 4), m4);
        __m256i mins = _mm256_cvtepi8_epi16(mins8);
        __m256i prod = _mm256_madd_epi16(mins, _mm256_loadu_si256((const __m256i*)y->bsums));
        acc = _mm256_fmadd_ps(_mm256_set1_ps(dmin), _mm256_cvtepi32_ps(prod), acc);
        __m256i all_scales = _mm256_cvtepi8_epi16(scales8);
        __m128i l_scales = _mm256_extracti128_si256(all_scales, 0);
        __m128i h_scales = _mm256_extracti128_si256(all_scales, 1);
        __m256i scales[2] = {_mm256_set_m128i(l_scales, l_scales), _mm256_set_m128i(h_scales, h_scales)};
        __m256i sumi = _mm256_setzero_si256();
        for (int h = 0; h < 2; h++) {
            __m256i q2bits = _mm256_loadu_si256((const __m256i*)q2);
            q2 += 32;
            __m256i p[4];
            for (int t = 0; t < 4; t++) {
                __m256i q8v = _mm256_loadu_si256((const __m256i*)q8);
                q8 += 32;
                __m256i q2v = _mm256_and_si256(_mm256_srl_epi16(q2bits, _mm_cvtsi32_si128(2 * t)), m3);
                /* 16-bit scale 2t in the low 128 bits, 2t+1 in the high (get_scale_shuffle_q3k, avx.rs:118-129) */
                __m256i shuf = _mm256_set_m128i(_mm_set1_epi16((short)(((4 * t + 3) << 8) | (4 * t + 2))),
                                                _mm_set1_epi16((short)(((4 * t + 1) << 8) | (4 * t))));
                p[t] = _mm256_madd_epi16(_mm256_shuffle_epi8(scales[h], shuf), _mm256_maddubs_epi16(q2v, q8v));
            }
            sumi = _mm256_add_epi32(sumi, _mm256_add_epi32(_mm256_add_epi32(p[0], p[1]), _mm256_add_epi32(p[2], p[3])));
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    return hsum_float_8(acc);
}
static float dot_q3k(int64_t n, const orc_block_q3k* xs, const orc_block_q8k* ys) {
    const uint32_t KMASK1 = 0x03030303, KMASK2 = 0x0f0f0f0f;
    const __m256i m3 = _mm256_set1_epi8(3), mone = _mm256_set1_epi8(1);
    __m256 acc = _mm256_setzero_ps();
    for (int64_t b = 0; b < n / 256; b++) {
        const orc_block_q3k* x = &xs[b];
        const orc_block_q8k* y = &ys[b];
        float d = y->d * orc_f16_to_f32(x->d);
        const uint8_t* q3 = x->qs;
        const int8_t* q8 = y->qs;
        uint32_t aux[3];
        memcpy(aux, x->scales, 12);
        __m128i scales128 = _mm_set_epi32((int)(((aux[1] >> 4) & KMASK2) | (((aux[2] >> 6) & KMASK1) << 4)),
                                          (int)(((aux[0] >> 4) & KMASK2) | (((aux[2] >> 4) & KMASK1) << 4)),
                                          (int)((aux[1] & KMASK2) | (((aux[2] >> 2) & KMASK1) << 4)),
                                          (int)((aux[0] & KMASK2) | ((aux[2] & KMASK1) << 4)));
        scales128 = _mm_sub_epi8(scales128, _mm_set1_epi8(32));
        __m256i all_scales = _mm256_cvtepi8_epi16(scales128);
        __m128i l_scales = _mm256_extracti128_si256(all_scales, 0);
        __m128i h_scales = _mm256_extracti128_si256(all_scales, 1);
        __m256i scales[2] = {_mm256_set_m128i(l_scales, l_scales), _mm256_set_m128i(h_scales, h_scales)};
        __m256i hbits = _mm256_loadu_si256((const __m256i*)x->hmask);
        __m256i sumi = _mm256_setzero_si256();
        for (int j = 0; j < 2; j++) {
            __m256i q3bits = _mm256_loadu_si256((const __m256i*)q3);
            q3 += 32;
            __m256i p[4];
            for (int t = 0; t < 4; t++) {
                const int bit = 4 * j + t;
                __m256i q3l = _mm256_and_si256(_mm256_srl_epi16(q3bits, _mm_cvtsi32_si128(2 * t)), m3);
                /* 4 where the high bit is NOT set, else 0 */
                __m256i q3h = _mm256_slli_epi16(
                    _mm256_srl_epi16(_mm256_andnot_si256(hbits, _mm256_sll_epi16(mone, _mm_cvtsi32_si128(bit))), _mm_cvtsi32_si128(bit)), 2);
                __m256i q8v = _mm256_loadu_si256((const __m256i*)q8);
                q8 += 32;
                __m256i p16 = _mm256_sub_epi16(_mm256_maddubs_epi16(q3l, q8v), _mm256_maddubs_epi16(q3h, q8v));
                __m256i shuf = _mm256_set_m128i(_mm_set1_epi16((short)(((4 * t + 3) << 8) | (4 * t + 2))),
                                                _mm_set1_epi16((short)(((4 * t + 1) << 8) | (4 * t))));
                p[t] = _mm256_madd_epi16(_mm256_shuffle_epi8(scales[j], shuf), p16);
            }
            sumi = _mm256_add_epi32(sumi, _mm256_add_epi32(_mm256_add_epi32(p[0], p[1]), _mm256_add_epi32(p[2], p[3])));
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    return hsum_float_8(acc);
}
static float dot_q5k(int64_t n, const orc_block_q5k* xs, const orc_block_q8k* ys) {
    const uint32_t KMASK1 = 0x3f3f3f3f, KMASK2 = 0x0f0f0f0f, KMASK3 = 0x03030303;
    const __m256i m4 = _mm256_set1_epi8(0xF);
    __m256 acc = _mm256_setzero_ps();
    float summs = 0.f;
    for (int64_t b = 0; b < n / 256; b++) {
        const orc_block_q5k* x = &xs[b];
        const orc_block_q8k* y = &ys[b];
        float d = y->d * orc_f16_to_f32(x->d);
        float dmin = -y->d * orc_f16_to_f32(x->dmin);
        uint32_t utmp[4];
        memcpy(utmp, x->scales, 12);
        utmp[3] = ((utmp[2] >> 4) & KMASK2) | (((utmp[1] >> 6) & KMASK3) << 4);
        uint32_t uaux = utmp[1] & KMASK1;
        utmp[1] = (utmp[2] & KMASK2) | (((utmp[0] >> 6) & KMASK3) << 4);
        utmp[2] = uaux;
        utmp[0] &= KMASK1;
        const uint8_t* q5 = x->qs;
        const int8_t* q8 = y->qs;
        __m256i mins_and_scales = _mm256_cvtepu8_epi16(
            _mm_set_epi32((int)utmp[3], (int)utmp[2], (int)utmp[1], (int)utmp[0]));
        __m256i q8sums = _mm256_loadu_si256((const __m256i*)y->bsums);
        __m128i q8s = _mm_hadd_epi16(_mm256_extracti128_si256(q8sums, 0), _mm256_extracti128_si256(q8sums, 1));
        __m128i prod = _mm_madd_epi16(_mm256_extracti128_si256(mins_and_scales, 1), q8s);
        __m128i hsum = _mm_hadd_epi32(_mm_hadd_epi32(prod, _mm_setzero_si128()), _mm_setzero_si128());
        summs += dmin * (float)_mm_extract_epi32(hsum, 0);
        __m128i sc128 = _mm256_extracti128_si256(mins_and_scales, 0);
        __m256i scales = _mm256_set_m128i(sc128, sc128);
        __m256i hbits = _mm256_loadu_si256((const __m256i*)x->qh);
        __m256i sumi = _mm256_setzero_si256();
        for (int j = 0; j < 4; j++) {
            __m256i scale_0 = _mm256_shuffle_epi8(scales, _mm256_set1_epi16((short)(((4 * j + 1) << 8) | (4 * j))));
            __m256i scale_1 = _mm256_shuffle_epi8(scales, _mm256_set1_epi16((short)(((4 * j + 3) << 8) | (4 * j + 2))));
            __m256i q5bits = _mm256_loadu_si256((const __m256i*)q5);
            q5 += 32;
            /* high bit 2j of every byte -> bit 4 (the reference hard-codes the same shifts per j) */
            __m256i h0 = _mm256_and_si256(_mm256_srl_epi16(hbits, _mm_cvtsi32_si128(2 * j)), _mm256_set1_epi8(1));
            __m256i h1 = _mm256_and_si256(_mm256_srl_epi16(hbits, _mm_cvtsi32_si128(2 * j + 1)), _mm256_set1_epi8(1));
            __m256i q5_0 = _mm256_add_epi8(_mm256_and_si256(q5bits, m4), _mm256_slli_epi16(h0, 4));
            __m256i q5_1 = _mm256_add_epi8(_mm256_and_si256(_mm256_srli_epi16(q5bits, 4), m4), _mm256_slli_epi16(h1, 4));
            __m256i q8_0 = _mm256_loadu_si256((const __m256i*)q8);
            q8 += 32;
            __m256i q8_1 = _mm256_loadu_si256((const __m256i*)q8);
            q8 += 32;
            __m256i p16_0 = _mm256_madd_epi16(scale_0, _mm256_maddubs_epi16(q5_0, q8_0));
            __m256i p16_1 = _mm256_madd_epi16(scale_1, _mm256_maddubs_epi16(q5_1, q8_1));
            sumi = _mm256_add_epi32(sumi, _mm256_add_epi32(p16_0, p16_1));
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    return hsum_float_8(acc) + summs;
}
static float dot_q6k(int64_t n, const orc_block_q6k* xs, const orc_block_q8k* ys) {
    const __m256i m4 = _mm256_set1_epi8(0xF), m2 = _mm256_set1_epi8(3), m32s = _mm256_set1_epi8(32);
    __m256 acc = _mm256_setzero_ps();
    for (int64_t b = 0; b < n / 256; b++) {
        const orc_block_q6k* x = &xs[b];
        const orc_block_q8k* y = &ys[b];
        float d = y->d * orc_f16_to_f32(x->d);
        const uint8_t* q4 = x->ql;
        const uint8_t* qh = x->qh;
        const int8_t* q8 = y->qs;
        __m128i scales = _mm_loadu_si128((const __m128i*)x->scales);
        __m256i sumi = _mm256_setzero_si256();
        for (int j = 0; j < 2; j++) {
            __m256i sc[4];
            for (int t = 0; t < 4; t++) {
                /* scale 2i in the low eight bytes, scale 2i+1 in the high eight (get_scale_shuffle, avx.rs:89-99) */
                const int i = 4 * j + t;
                __m128i shuf = _mm_set_epi64x(0x0101010101010101LL * (2 * i + 1), 0x0101010101010101LL * (2 * i));
                sc[t] = _mm256_cvtepi8_epi16(_mm_shuffle_epi8(scales, shuf));
            }
            __m256i q4bits1 = _mm256_loadu_si256((const __m256i*)q4);
            __m256i q4bits2 = _mm256_loadu_si256((const __m256i*)(q4 + 32));
            q4 += 64;
            __m256i q4bits_h = _mm256_loadu_si256((const __m256i*)qh);
            qh += 32;
            __m256i qv[4];
            qv[0] = _mm256_or_si256(_mm256_and_si256(q4bits1, m4), _mm256_slli_epi16(_mm256_and_si256(q4bits_h, m2), 4));
            qv[1] = _mm256_or_si256(_mm256_and_si256(q4bits2, m4),
                                    _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(q4bits_h, 2), m2), 4));
            qv[2] = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(q4bits1, 4), m4),
                                    _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(q4bits_h, 4), m2), 4));
            qv[3] = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(q4bits2, 4), m4),
                                    _mm256_slli_epi16(_mm256_and_si256(_mm256_srli_epi16(q4bits_h, 6), m2), 4));
            __m256i p[4];
            for (int t = 0; t < 4; t++) {
                __m256i q8v = _mm256_loadu_si256((const __m256i*)q8);
                q8 += 32;
                __m256i q8s = _mm256_maddubs_epi16(m32s, q8v);
                __m256i p16 = _mm256_sub_epi16(_mm256_maddubs_epi16(qv[t], q8v), q8s);
                p[t] = _mm256_madd_epi16(sc[t], p16);
            }
            sumi = _mm256_add_epi32(sumi, _mm256_add_epi32(p[0], p[1]));
            sumi = _mm256_add_epi32(sumi, _mm256_add_epi32(p[2], p[3]));
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    return hsum_float_8(acc);
}

float orc_vec_dot_avx2(int dtype, int64_t n, const void* w, const void* a) {
    switch (dtype) {
        case ORC_Q4_0: return dot_q4_0(n, (const orc_block_q4_0*)w, (const orc_block_q8_0*)a);
        case ORC_Q8_0: return dot_q8_0(n, (const orc_block_q8_0*)w, (const orc_block_q8_0*)a);
        case ORC_Q4K: return dot_q4k(n, (const orc_block_q4k*)w, (const orc_block_q8k*)a);
        case ORC_Q2K: return dot_q2k(n, (const orc_block_q2k*)w, (const orc_block_q8k*)a);
        case ORC_Q3K: return dot_q3k(n, (const orc_block_q3k*)w, (const orc_block_q8k*)a);
        case ORC_Q5K: return dot_q5k(n, (const orc_block_q5k*)w, (const orc_block_q8k*)a);
        case ORC_Q6K: return dot_q6k(n, (const orc_block_q6k*)w, (const orc_block_q8k*)a);
        default: return orc_vec_dot(dtype, n, w, a);
    }
}
