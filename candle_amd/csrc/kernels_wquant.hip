// Weight quantisers: f32 -> GGML blocks on the GPU, bit-identical to candle's CPU quantiser
// (QTensor::quantize, candle-core/src/quantized/mod.rs:331-349):
//   BlockQ4_0::from_float  candle-core/src/quantized/k_quants.rs:188-224
//   BlockQ8_0::from_float  k_quants.rs:605-634
//   BlockQ4K::from_float   k_quants.rs:1287-1345 with make_qkx1_quants(15, 5, .) of
//                          candle-core/src/quantized/utils.rs:202-259 and nearest_int = round()
//   BlockQ2K / Q3K / Q5K / Q6K::from_float  k_quants.rs:808-870, 1049-1129, 1484-1561, 1675-1751
// Every f32 sum runs in the reference's element order inside one thread; the build does not
// contract multiply-adds, so each intermediate rounds as on the CPU.
#include "kernels.hpp"

namespace moe {

__device__ inline int nearest_int_ref(float v) {  // utils.rs:1-3: f32::round, then a saturating cast
    v = roundf(v);
    if (v != v) return 0;
    if (v >= 2147483648.0f) return 2147483647;
    if (v <= -2147483648.0f) return -2147483647 - 1;
    return (int)v;
}

__device__ inline uint16_t f32_to_f16_bits(float f) { return __half_as_ushort(__float2half_rn(f)); }

// one thread per 32-element block
__global__ void wquant_q4_0_kernel(const float* x, int64_t nblocks, uint8_t* out) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float* xs = x + b * 32;
    float amax = 0.f, max = 0.f;
    for (int j = 0; j < 32; j++) {
        float a = fabsf(xs[j]);
        if (amax < a) { amax = a; max = xs[j]; }
    }
    float d = max / -8.0f;
    float id = (d != 0.f) ? 1.0f / d : 0.f;
    uint8_t* o = out + b * 18;
    uint16_t h = f32_to_f16_bits(d);
    // the compiler folds `max * -0.125` and the f16 conversion into one fma-mix with a +0 addend,
    // which turns d = -0.0 (an all-zero block: 0 / -8) into +0.0; keep the sign of a zero scale
    if (d == 0.f) h = (uint16_t)((__float_as_uint(d) >> 16) & 0x8000u);
    o[0] = (uint8_t)(h & 0xff);
    o[1] = (uint8_t)(h >> 8);
    for (int j = 0; j < 16; j++) {
        float x0 = xs[j] * id + 8.5f, x1 = xs[16 + j] * id + 8.5f;
        // `as u8` saturates and truncates, NaN -> 0; then min(15)
        int q0 = (x0 != x0) ? 0 : (int)fminf(fmaxf(x0, 0.f), 255.f);
        int q1 = (x1 != x1) ? 0 : (int)fminf(fmaxf(x1, 0.f), 255.f);
        q0 = q0 > 15 ? 15 : q0;
        q1 = q1 > 15 ? 15 : q1;
        o[2 + j] = (uint8_t)(q0 | (q1 << 4));
    }
}

__global__ void wquant_q8_0_kernel(const float* x, int64_t nblocks, uint8_t* out) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const float* xs = x + b * 32;
    float amax = 0.f;
    for (int j = 0; j < 32; j++) amax = fmaxf(amax, fabsf(xs[j]));
    float d = amax / 127.0f;
    float id = (d != 0.f) ? 1.0f / d : 0.f;
    uint8_t* o = out + b * 34;
    uint16_t h = f32_to_f16_bits(d);
    o[0] = (uint8_t)(h & 0xff);
    o[1] = (uint8_t)(h >> 8);
    for (int j = 0; j < 32; j++) o[2 + j] = (uint8_t)sat_i8(roundf(xs[j] * id));
}

// make_qkx1_quants(15, 5, x[0..32)) -> (scale, min)
__device__ inline void make_qkx1(const float* x, float* out_scale, float* out_min) {
    const int n = 32, nmax = 15, ntry = 5;
    float min = x[0], max = x[0];
    for (int i = 1; i < n; i++) {
        min = x[i] < min ? x[i] : min;
        max = x[i] > max ? x[i] : max;
    }
    if (max == min) { *out_scale = 0.f; *out_min = 0.f; return; }
    min = fminf(min, 0.f);
    float iscale = (float)nmax / (max - min);
    float scale = 1.0f / iscale;
    uint32_t lbits[4] = {0, 0, 0, 0};  // the 32 4-bit levels of the previous pass
    for (int t = 0; t < ntry; t++) {
        float sumlx = 0.f;
        int suml2 = 0;
        bool did_change = false;
        for (int i = 0; i < n; i++) {
            int li = nearest_int_ref(iscale * (x[i] - min));
            li = li < 0 ? 0 : (li > nmax ? nmax : li);
            uint32_t prev = (lbits[i >> 3] >> ((i & 7) * 4)) & 0xfu;
            if ((uint32_t)li != prev) {
                lbits[i >> 3] = (lbits[i >> 3] & ~(0xfu << ((i & 7) * 4))) | ((uint32_t)li << ((i & 7) * 4));
                did_change = true;
            }
            sumlx += (x[i] - min) * (float)li;
            suml2 += li * li;
        }
        scale = sumlx / (float)suml2;
        float sum = 0.f;
        for (int i = 0; i < n; i++) {
            uint32_t li = (lbits[i >> 3] >> ((i & 7) * 4)) & 0xfu;
            sum += x[i] - scale * (float)li;
        }
        min = sum / (float)n;
        if (min > 0.f) min = 0.f;
        iscale = 1.0f / scale;
        if (!did_change) break;
    }
    *out_scale = scale;
    *out_min = -min;
}

// eight consecutive lanes own one 256-element super-block, one 32-element sub-block each
__global__ __launch_bounds__(256) void wquant_q4k_kernel(const float* x, int64_t nsub, uint8_t* out) {
    int64_t sub = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int lane = threadIdx.x & 63;
    const int j = lane & 7;                 // sub-block inside the super-block
    const bool live = sub < nsub;           // nsub is a multiple of 8, so groups are all-or-nothing
    float xs[32];
    const float* src = x + (live ? sub : 0) * 32;
#pragma unroll
    for (int i = 0; i < 32; i += 4) {
        float4 v = *reinterpret_cast<const float4*>(src + i);
        xs[i] = v.x; xs[i + 1] = v.y; xs[i + 2] = v.z; xs[i + 3] = v.w;
    }
    float scale, mn;
    make_qkx1(xs, &scale, &mn);
    // fold(0.0, max) over the eight sub-blocks
    float max_scale = fmaxf(scale, 0.f), max_min = fmaxf(mn, 0.f);
#pragma unroll
    for (int o = 1; o < 8; o <<= 1) {
        max_scale = fmaxf(max_scale, __shfl_xor(max_scale, o, 64));
        max_min = fmaxf(max_min, __shfl_xor(max_min, o, 64));
    }
    float inv_scale = max_scale > 0.f ? 63.0f / max_scale : 0.f;
    float inv_min = max_min > 0.f ? 63.0f / max_min : 0.f;
    int ls = nearest_int_ref(inv_scale * scale); ls = ls > 63 ? 63 : ls;
    int lm = nearest_int_ref(inv_min * mn);      lm = lm > 63 ? 63 : lm;
    ls &= 0xff; lm &= 0xff;
    const uint16_t dh = f32_to_f16_bits(max_scale / 63.0f), dmh = f32_to_f16_bits(max_min / 63.0f);
    // the reference re-reads the packed 6-bit values; ls, lm <= 63 so that is the identity here
    const float d = __half2float(__ushort_as_half(dh)) * (float)ls;
    uint32_t lv[4] = {0, 0, 0, 0};  // 32 levels, 4 bits each
    if (d != 0.f) {
        const float dm = __half2float(__ushort_as_half(dmh)) * (float)lm;
#pragma unroll
        for (int i = 0; i < 32; i++) {
            int l = nearest_int_ref((xs[i] + dm) / d);
            l = l < 0 ? 0 : (l > 15 ? 15 : l);
            lv[i >> 3] |= (uint32_t)l << ((i & 7) * 4);
        }
    }
    // gather the eight (ls, lm) pairs of the super-block
    int all_ls[8], all_lm[8];
#pragma unroll
    for (int s = 0; s < 8; s++) {
        all_ls[s] = __shfl(ls, (lane & ~7) | s, 64);
        all_lm[s] = __shfl(lm, (lane & ~7) | s, 64);
    }
    // sub-blocks 2p (low nibbles) and 2p+1 (high nibbles) share 32 bytes; the even lane writes them
    uint32_t hi[4];
#pragma unroll
    for (int w = 0; w < 4; w++) hi[w] = __shfl(lv[w], lane | 1, 64);
    if (!live) return;
    uint8_t* blk = out + (sub >> 3) * 144;
    if (j == 0) {
        uint8_t sc[12];
        for (int s = 0; s < 12; s++) sc[s] = 0;
        for (int s = 0; s < 8; s++) {
            if (s < 4) {
                sc[s] = (uint8_t)all_ls[s];
                sc[s + 4] = (uint8_t)all_lm[s];
            } else {
                sc[s + 4] = (uint8_t)((all_ls[s] & 0xF) | ((all_lm[s] & 0xF) << 4));
                sc[s - 4] |= (uint8_t)((all_ls[s] >> 4) << 6);
                sc[s] |= (uint8_t)((all_lm[s] >> 4) << 6);
            }
        }
        blk[0] = (uint8_t)(dh & 0xff); blk[1] = (uint8_t)(dh >> 8);
        blk[2] = (uint8_t)(dmh & 0xff); blk[3] = (uint8_t)(dmh >> 8);
        for (int s = 0; s < 12; s++) blk[4 + s] = sc[s];
    }
    if ((j & 1) == 0) {
        uint8_t* q = blk + 16 + (j >> 1) * 32;
#pragma unroll
        for (int i = 0; i < 32; i++) {
            uint32_t lo4 = (lv[i >> 3] >> ((i & 7) * 4)) & 0xfu;
            uint32_t hi4 = (hi[i >> 3] >> ((i & 7) * 4)) & 0xfu;
            q[i] = (uint8_t)(lo4 | (hi4 << 4));
        }
    }
}


// ---------------------------------------------------------------------------------------------
// Q2K, Q3K, Q5K and Q6K (BlockQ2K / Q3K / Q5K / Q6K::from_float, k_quants.rs:808-870, 1049-1129, 1484-1561,
// 1675-1751).  One lane per sub-block (16 elements; 32 for Q5K) runs the reference's per-sub-block search in its
// element order; the lanes of a super-block meet in LDS, where its first lane derives the block's header serially, as
// the reference does, and the lanes then share out the packing of the bytes.

__device__ inline int32_t total_key_dev(float f) {   // the order of f32::total_cmp as an integer
    int32_t b = __float_as_int(f);
    b ^= (int32_t)(((uint32_t)(b >> 31)) >> 1);
    return b;
}

// make_qkx1_quants(nmax, 5, x[0..N)) of utils.rs:202-259 -> (scale, -min)
template <int N>
__device__ inline void make_qkx1_n(const float (&x)[N], int nmax, float* out_scale, float* out_min) {
    uint8_t l[N];
#pragma unroll
    for (int i = 0; i < N; i++) l[i] = 0;
    float min = x[0], max = x[0];
#pragma unroll
    for (int i = 1; i < N; i++) {
        if (total_key_dev(x[i]) < total_key_dev(min)) min = x[i];    // min_by keeps the first minimum
        if (total_key_dev(x[i]) >= total_key_dev(max)) max = x[i];   // max_by keeps the last maximum
    }
    if (max == min) { *out_scale = 0.f; *out_min = 0.f; return; }
    min = fminf(min, 0.f);
    float iscale = (float)nmax / (max - min);
    float scale = 1.0f / iscale;
    for (int t = 0; t < 5; t++) {
        float sumlx = 0.f;
        int suml2 = 0;
        bool did_change = false;
#pragma unroll
        for (int i = 0; i < N; i++) {
            int li = nearest_int_ref(iscale * (x[i] - min));
            li = li < 0 ? 0 : (li > nmax ? nmax : li);
            if ((uint8_t)li != l[i]) { l[i] = (uint8_t)li; did_change = true; }
            sumlx += (x[i] - min) * (float)li;
            suml2 += li * li;
        }
        scale = sumlx / (float)suml2;
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < N; i++) sum += x[i] - scale * (float)l[i];
        min = sum / (float)N;
        if (min > 0.f) min = 0.f;
        iscale = 1.0f / scale;
        if (!did_change) break;
    }
    *out_scale = scale;
    *out_min = -min;
}

// make_q3_quants(x[0..16), nmax = 4, do_rmse) of k_quants.rs:872-908
__device__ inline float make_q3_quants_16(const float (&x)[16]) {
    const int nmax = 4;
    int8_t l[16];
    float max = 0.f, amax = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; max = x[i]; }
    }
    if (amax == 0.f) return 0.f;
    const float iscale = -(float)nmax / max;
    float sumlx = 0.f, suml2 = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        int li = nearest_int_ref(iscale * x[i]);
        li = li < -nmax ? -nmax : li > nmax - 1 ? nmax - 1 : li;
        l[i] = (int8_t)li;
        const float w = x[i] * x[i];
        sumlx += w * x[i] * (float)li;
        suml2 += w * (float)(li * li);
    }
    for (int t = 0; t < 5; t++) {
        int n_changed = 0;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float w = x[i] * x[i];
            float slx = sumlx - w * x[i] * (float)l[i];
            if (slx > 0.f) {
                float sl2 = suml2 - w * (float)((int)l[i] * (int)l[i]);
                int new_l = nearest_int_ref(x[i] * sl2 / slx);
                new_l = new_l < -nmax ? -nmax : new_l > nmax - 1 ? nmax - 1 : new_l;
                if (new_l != (int)l[i]) {
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

// make_qx_quants(16, 32, x, ls, rmse_type = 1) of utils.rs:77-200: weights x^2, no scan over neighbouring scales
__device__ inline float make_qx_quants_16(const float (&x)[16], int8_t (&ls)[16]) {
    const int nmax = 32;
    float max = 0.f, amax = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float ax = fabsf(x[i]);
        if (ax > amax) { amax = ax; max = x[i]; }
    }
    if (amax == 0.f) {
#pragma unroll
        for (int i = 0; i < 16; i++) ls[i] = 0;
        return 0.f;
    }
    const float iscale = -(float)nmax / max;
    float sumlx = 0.f, suml2 = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        int l = nearest_int_ref(iscale * x[i]);
        l = l < -nmax ? -nmax : l > nmax - 1 ? nmax - 1 : l;
        ls[i] = (int8_t)(l + nmax);
        const float w = x[i] * x[i];
        const float lf = (float)l;
        sumlx += w * x[i] * lf;
        suml2 += w * lf * lf;
    }
    float scale = sumlx / suml2;
    float best = scale * sumlx;
    for (int itry = 0; itry < 3; itry++) {
        const float is2 = 1.0f / scale;
        float slx = 0.f, sl2 = 0.f;
        bool changed = false;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            int l = nearest_int_ref(is2 * x[i]);
            l = l < -nmax ? -nmax : l > nmax - 1 ? nmax - 1 : l;
            if (l + nmax != (int)ls[i]) changed = true;
            const float w = x[i] * x[i];
            const float lf = (float)l;
            slx += w * x[i] * lf;
            sl2 += w * lf * lf;
        }
        if (!changed || sl2 == 0.0f || slx * slx <= best * sl2) break;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            int l = nearest_int_ref(is2 * x[i]);
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
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float w = x[i] * x[i];
            const int l = (int)ls[i] - nmax;
            float slx = sumlx - w * x[i] * (float)l;
            if (slx > 0.f) {
                float sl2 = suml2 - w * (float)l * (float)l;
                int new_l = nearest_int_ref(x[i] * sl2 / slx);
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
    return scale;
}

__device__ inline void put_f16(uint8_t* p, uint16_t h) { p[0] = (uint8_t)(h & 0xff); p[1] = (uint8_t)(h >> 8); }

template <int DT>
__global__ __launch_bounds__(256) void wquant_kquant_kernel(const float* x, int64_t nsuper, uint8_t* out) {
    constexpr int SUBS = DT == MOE_GGML_Q5K ? 8 : 16;   // sub-blocks per super-block = lanes per super-block
    constexpr int N = 256 / SUBS;                        // elements per sub-block
    constexpr int PER_WG = 256 / SUBS;                   // super-blocks per workgroup
    constexpr int BYTES = DT == MOE_GGML_Q2K ? 84 : DT == MOE_GGML_Q3K ? 110 : DT == MOE_GGML_Q5K ? 176 : 210;
    __shared__ float s_scale[PER_WG][16], s_min[PER_WG][16];
    __shared__ uint8_t s_l[PER_WG][256];
    __shared__ int s_q[PER_WG][16];            // the block's quantised (scale, min) bytes as the level pass reads them
    __shared__ float s_d[PER_WG], s_dmin[PER_WG];
    const int tid = threadIdx.x, g = tid / SUBS, j = tid % SUBS;
    const int64_t sb = (int64_t)blockIdx.x * PER_WG + g;
    const bool live = sb < nsuper;
    float xs[N];
    const float* src = x + (live ? sb : 0) * 256 + j * N;
#pragma unroll
    for (int i = 0; i < N; i += 4) {
        const float4 v = *reinterpret_cast<const float4*>(src + i);
        xs[i] = v.x; xs[i + 1] = v.y; xs[i + 2] = v.z; xs[i + 3] = v.w;
    }
    uint8_t* blk = out + (live ? sb : 0) * BYTES;

    // ---- the sub-block's scale (and minimum)
    if constexpr (DT == MOE_GGML_Q2K || DT == MOE_GGML_Q5K) {
        float sc, mn;
        make_qkx1_n<N>(xs, DT == MOE_GGML_Q2K ? 3 : 31, &sc, &mn);
        s_scale[g][j] = sc;
        s_min[g][j] = mn;
    } else if constexpr (DT == MOE_GGML_Q3K) {
        s_scale[g][j] = make_q3_quants_16(xs);
    } else {
        int8_t ls[16];
        s_scale[g][j] = make_qx_quants_16(xs, ls);
#pragma unroll
        for (int i = 0; i < 16; i++) s_l[g][j * 16 + i] = (uint8_t)ls[i];   // kept where the final scale turns out zero
    }
    __syncthreads();

    // ---- the block's header, by the super-block's first lane, in the reference's order
    if (j == 0 && live) {
        if constexpr (DT == MOE_GGML_Q2K) {
            float max_scale = 0.f, max_min = 0.f;
            for (int s = 0; s < 16; s++) { max_scale = fmaxf(s_scale[g][s], max_scale); max_min = fmaxf(s_min[g][s], max_min); }
            uint8_t q[16];
            uint16_t dh, dmh;
            if (max_scale > 0.f) {
                const float iscale = 15.0f / max_scale;
                for (int s = 0; s < 16; s++) q[s] = (uint8_t)nearest_int_ref(iscale * s_scale[g][s]);
                dh = f32_to_f16_bits(max_scale / 15.0f);
            } else {
                for (int s = 0; s < 16; s++) q[s] = 0;
                dh = f32_to_f16_bits(0.f);
            }
            if (max_min > 0.f) {
                const float iscale = 15.0f / max_min;
                for (int s = 0; s < 16; s++) q[s] |= (uint8_t)((uint8_t)nearest_int_ref(iscale * s_min[g][s]) << 4);
                dmh = f32_to_f16_bits(max_min / 15.0f);
            } else {
                dmh = f32_to_f16_bits(0.f);
            }
            for (int s = 0; s < 16; s++) { blk[s] = q[s]; s_q[g][s] = q[s]; }
            put_f16(blk + 80, dh);
            put_f16(blk + 82, dmh);
            s_d[g] = __half2float(__ushort_as_half(dh));
            s_dmin[g] = __half2float(__ushort_as_half(dmh));
        } else if constexpr (DT == MOE_GGML_Q3K) {
            float max_scale = 0.f;
            for (int s = 0; s < 16; s++)
                if (fabsf(s_scale[g][s]) > fabsf(max_scale)) max_scale = s_scale[g][s];
            uint8_t sc[12];
            for (int s = 0; s < 12; s++) sc[s] = 0;
            uint16_t dh;
            if (max_scale != 0.f) {
                const float iscale = -32.0f / max_scale;
                for (int s = 0; s < 16; s++) {
                    int lv = nearest_int_ref(iscale * s_scale[g][s]);
                    lv = (lv < -32 ? -32 : lv > 31 ? 31 : lv) + 32;
                    s_q[g][s] = lv;
                    if (s < 8) sc[s] = (uint8_t)(lv & 0xF);
                    else sc[s - 8] |= (uint8_t)((lv & 0xF) << 4);
                    lv >>= 4;
                    sc[s % 4 + 8] |= (uint8_t)(lv << (2 * (s / 4)));
                }
                dh = f32_to_f16_bits(1.0f / iscale);
            } else {
                for (int s = 0; s < 16; s++) s_q[g][s] = 0;   // stored scale bits 0 -> scale -32
                dh = f32_to_f16_bits(0.f);
            }
            for (int s = 0; s < 12; s++) blk[96 + s] = sc[s];
            put_f16(blk + 108, dh);
            s_d[g] = __half2float(__ushort_as_half(dh));
        } else if constexpr (DT == MOE_GGML_Q5K) {
            float max_scale = 0.f, max_min = 0.f;
            for (int s = 0; s < 8; s++) { max_scale = fmaxf(s_scale[g][s], max_scale); max_min = fmaxf(s_min[g][s], max_min); }
            const float inv_scale = max_scale > 0.f ? 63.0f / max_scale : 0.f;
            const float inv_min = max_min > 0.f ? 63.0f / max_min : 0.f;
            uint8_t sc[12];
            for (int s = 0; s < 12; s++) sc[s] = 0;
            for (int s = 0; s < 8; s++) {
                int lsi = nearest_int_ref(inv_scale * s_scale[g][s]); lsi = lsi > 63 ? 63 : lsi;
                int lmi = nearest_int_ref(inv_min * s_min[g][s]);     lmi = lmi > 63 ? 63 : lmi;
                const uint8_t ls = (uint8_t)lsi, lm = (uint8_t)lmi;
                if (s < 4) {
                    sc[s] = ls;
                    sc[s + 4] = lm;
                } else {
                    sc[s + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                    sc[s - 4] |= (uint8_t)((ls >> 4) << 6);
                    sc[s] |= (uint8_t)((lm >> 4) << 6);
                }
            }
            // the level pass reads the packed bytes back (get_scale_min_k4, utils.rs:50-60)
            for (int s = 0; s < 8; s++) {
                int d6, m6;
                if (s < 4) { d6 = sc[s] & 63; m6 = sc[s + 4] & 63; }
                else { d6 = (sc[s + 4] & 0xF) | ((sc[s - 4] >> 6) << 4); m6 = (sc[s + 4] >> 4) | ((sc[s] >> 6) << 4); }
                s_q[g][s] = d6 | (m6 << 8);
            }
            const uint16_t dh = f32_to_f16_bits(max_scale / 63.0f), dmh = f32_to_f16_bits(max_min / 63.0f);
            put_f16(blk, dh);
            put_f16(blk + 2, dmh);
            for (int s = 0; s < 12; s++) blk[4 + s] = sc[s];
            s_d[g] = __half2float(__ushort_as_half(dh));
            s_dmin[g] = __half2float(__ushort_as_half(dmh));
        } else {
            float max_scale = 0.f, max_abs_scale = 0.f;
            for (int s = 0; s < 16; s++) {
                const float a = fabsf(s_scale[g][s]);
                if (a > max_abs_scale) { max_abs_scale = a; max_scale = s_scale[g][s]; }
            }
            const float iscale = -128.0f / max_scale;
            const uint16_t dh = f32_to_f16_bits(1.0f / iscale);
            for (int s = 0; s < 16; s++) {
                const int v = nearest_int_ref(iscale * s_scale[g][s]);
                const int8_t q = (int8_t)(v < 127 ? v : 127);
                s_q[g][s] = (int)q;
                blk[192 + s] = (uint8_t)q;
            }
            put_f16(blk + 208, dh);
            s_d[g] = __half2float(__ushort_as_half(dh));
        }
    }
    __syncthreads();

    // ---- the sub-block's levels against the stored header
    if constexpr (DT == MOE_GGML_Q2K) {
        const float d = s_d[g] * (float)(s_q[g][j] & 0xF);
        const float dm = s_dmin[g] * (float)(s_q[g][j] >> 4);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            int ll = 0;
            if (d != 0.f) { ll = nearest_int_ref((xs[i] + dm) / d); ll = ll < 0 ? 0 : ll > 3 ? 3 : ll; }
            s_l[g][j * 16 + i] = (uint8_t)ll;
        }
    } else if constexpr (DT == MOE_GGML_Q3K) {
        const float d = s_d[g] * (float)(s_q[g][j] - 32);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            int lv = 0;
            if (d != 0.f) { lv = nearest_int_ref(xs[i] / d); lv = (lv < -4 ? -4 : lv > 3 ? 3 : lv) + 4; }
            s_l[g][j * 16 + i] = (uint8_t)lv;
        }
    } else if constexpr (DT == MOE_GGML_Q5K) {
        const float d = s_d[g] * (float)(s_q[g][j] & 0xff);
        const float dm = s_dmin[g] * (float)(s_q[g][j] >> 8);
#pragma unroll
        for (int i = 0; i < 32; i++) {
            int lv = 0;
            if (d != 0.f) { lv = nearest_int_ref((xs[i] + dm) / d); lv = lv < 0 ? 0 : lv > 31 ? 31 : lv; }
            s_l[g][j * 32 + i] = (uint8_t)lv;
        }
    } else {
        const float d = s_d[g] * (float)s_q[g][j];
        if (d != 0.f) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                int ll = nearest_int_ref(xs[i] / d);
                ll = ll < -32 ? -32 : ll > 31 ? 31 : ll;
                s_l[g][j * 16 + i] = (uint8_t)(ll + 32);
            }
        }
    }
    __syncthreads();
    if (!live) return;

    // ---- packing, shared out over the super-block's lanes
    const uint8_t* l = s_l[g];
    if constexpr (DT == MOE_GGML_Q2K || DT == MOE_GGML_Q3K) {
        uint8_t* qs = blk + (DT == MOE_GGML_Q2K ? 16 : 32);
        for (int b = j * 4; b < j * 4 + 4; b++) {   // 64 bytes, four per lane
            const int h = b >> 5, ll = b & 31, base = 128 * h + ll;
            qs[b] = (uint8_t)((l[base] & 3) | ((l[base + 32] & 3) << 2) | ((l[base + 64] & 3) << 4) | ((l[base + 96] & 3) << 6));
        }
        if constexpr (DT == MOE_GGML_Q3K) {
            for (int m = j * 2; m < j * 2 + 2; m++) {   // hmask[m]: bit i/32 of element i = 32 * bit + m
                uint8_t hm = 0;
                for (int bit = 0; bit < 8; bit++) hm |= (uint8_t)((l[32 * bit + m] > 3 ? 1 : 0) << bit);
                blk[m] = hm;
            }
        }
    } else if constexpr (DT == MOE_GGML_Q5K) {
        for (int b = j * 16; b < j * 16 + 16; b++) {   // qs: 128 bytes, sixteen per lane
            const int q = b >> 5, jj = b & 31, n = 64 * q;
            blk[48 + b] = (uint8_t)((l[n + jj] & 15) | ((l[n + jj + 32] & 15) << 4));
        }
        for (int jj = j * 4; jj < j * 4 + 4; jj++) {   // qh: 32 bytes, four per lane
            uint8_t h = 0;
            for (int q = 0; q < 4; q++) h |= (uint8_t)(((l[64 * q + jj] > 15 ? 1 : 0) << (2 * q)) | ((l[64 * q + jj + 32] > 15 ? 1 : 0) << (2 * q + 1)));
            blk[16 + jj] = h;
        }
    } else {
        for (int b = j * 4; b < j * 4 + 4; b++) {   // per half of 128 elements: 64 bytes of ql, 32 of qh
            const int h = b >> 5, i = b & 31, base = 128 * h + i;
            blk[64 * h + i] = (uint8_t)((l[base] & 0xF) | ((l[base + 64] & 0xF) << 4));
            blk[64 * h + i + 32] = (uint8_t)((l[base + 32] & 0xF) | ((l[base + 96] & 0xF) << 4));
            blk[128 + 32 * h + i] = (uint8_t)((l[base] >> 4) | ((l[base + 32] >> 4) << 2) | ((l[base + 64] >> 4) << 4) | ((l[base + 96] >> 4) << 6));
        }
    }
}

hipError_t launch_quantize_weights(int dt, const float* x, int64_t n, uint8_t* out, hipStream_t s) {
    if (n == 0) return hipSuccess;
    if (dt == MOE_GGML_Q4K) {
        int64_t nsub = n / 32;
        hipLaunchKernelGGL(wquant_q4k_kernel, dim3((unsigned)((nsub + 255) / 256)), dim3(256), 0, s, x, nsub, out);
    } else if (dt == MOE_GGML_Q8_0) {
        int64_t nb = n / 32;
        hipLaunchKernelGGL(wquant_q8_0_kernel, dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, s, x, nb, out);
    } else if (dt == MOE_GGML_Q4_0) {
        int64_t nb = n / 32;
        hipLaunchKernelGGL(wquant_q4_0_kernel, dim3((unsigned)((nb + 255) / 256)), dim3(256), 0, s, x, nb, out);
    } else if (dt == MOE_GGML_Q2K || dt == MOE_GGML_Q3K || dt == MOE_GGML_Q5K || dt == MOE_GGML_Q6K) {
        const int64_t nsuper = n / 256;
        const int per_wg = dt == MOE_GGML_Q5K ? 32 : 16;
        const dim3 grid((unsigned)((nsuper + per_wg - 1) / per_wg));
        if (dt == MOE_GGML_Q2K) hipLaunchKernelGGL(wquant_kquant_kernel<MOE_GGML_Q2K>, grid, dim3(256), 0, s, x, nsuper, out);
        else if (dt == MOE_GGML_Q3K) hipLaunchKernelGGL(wquant_kquant_kernel<MOE_GGML_Q3K>, grid, dim3(256), 0, s, x, nsuper, out);
        else if (dt == MOE_GGML_Q5K) hipLaunchKernelGGL(wquant_kquant_kernel<MOE_GGML_Q5K>, grid, dim3(256), 0, s, x, nsuper, out);
        else hipLaunchKernelGGL(wquant_kquant_kernel<MOE_GGML_Q6K>, grid, dim3(256), 0, s, x, nsuper, out);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace moe
