// Weight quantisers: f32 -> GGML blocks on the GPU, bit-identical to candle's CPU quantiser
// (QTensor::quantize, candle-core/src/quantized/mod.rs:331-349):
//   BlockQ4_0::from_float  candle-core/src/quantized/k_quants.rs:188-224
//   BlockQ8_0::from_float  k_quants.rs:605-634
//   BlockQ4K::from_float   k_quants.rs:1287-1345 with make_qkx1_quants(15, 5, .) of
//                          candle-core/src/quantized/utils.rs:202-259 and nearest_int = round()
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
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace moe
