// Wave-level activation quantisers.  They restate, per block, exactly what candle's
// k_quants::matmul applies to every lhs row before the integer dot products:
//   BlockQ8K::from_float   candle-core/src/quantized/k_quants.rs:1819-1856
//   BlockQ8_0::from_float  candle-core/src/quantized/k_quants.rs:605-634
//   BlockQ8_1::from_float  candle-core/src/quantized/k_quants.rs:700-729
// so the int8 operands are bit-identical to the CPU path's.
#pragma once
#include "moe_common.hpp"

namespace moe {

__device__ inline float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Byte offset of element k (0..K) inside a Q8K-quantised activation row (see moe_common.hpp).
__host__ __device__ inline int q8k_act_offset(int k) {
    return (k / 64) * 64 + ((k % 32) / 8) * 16 + ((k / 32) % 2) * 8 + (k % 8);
}

// One wave quantises one 256-element block; lane l holds elements 4l..4l+3 in v.
//   qs_block : the block's 256 quant bytes (device layout), d_out / bs_out: scale and 16 bsums.
__device__ inline void quantize_q8k_block(float4 v, int lane, int8_t* qs_block, float* d_out, __half* bs_out) {
    // first element of largest magnitude, scanning in index order with a strict '<'
    float amax = 0.f, mx = 0.f;
    float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float a = fabsf(e[i]);
        if (amax < a) { amax = a; mx = e[i]; }
    }
    float wmax = wave_max(amax);
    if (wmax == 0.f) {
        *reinterpret_cast<uint32_t*>(qs_block + q8k_act_offset(4 * lane)) = 0u;
        if (lane == 0) *d_out = 0.f;
        if (lane < 16) bs_out[lane] = __float2half(0.f);
        return;
    }
    unsigned long long winners = __ballot(amax == wmax);
    int first = __ffsll((long long)winners) - 1;
    float max = __shfl(mx, first, 64);
    float iscale = -128.0f / max;
    int sum = 0;
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float r = roundf(iscale * e[i]);
        int q = sat_i8(fminf(r, 127.f));
        sum += q;
        packed |= (uint32_t)(uint8_t)q << (8 * i);
    }
    *reinterpret_cast<uint32_t*>(qs_block + q8k_act_offset(4 * lane)) = packed;
    sum += __shfl_xor(sum, 1, 64);
    sum += __shfl_xor(sum, 2, 64);
    if ((lane & 3) == 0) bs_out[lane >> 2] = __int2half_rn(sum);
    if (lane == 0) *d_out = 1.0f / iscale;
}

// N blocks at once, lane l holding elements 4l..4l+3 of each: the arithmetic of quantize_q8k_block without its
// branch, so that the N chains of wave reductions and the divisions overlap instead of running one after the other
// (the epilogue of the up projection, where nothing else hides their latency).  Blocks with valid[n] == false are
// computed and not stored.
template <int N>
__device__ inline void quantize_q8k_blocks(const float4 (&v)[N], const bool (&valid)[N], int lane, int8_t* const (&qs_block)[N],
                                           float* const (&d_out)[N], __half* const (&bs_out)[N]) {
    float amax[N], mx[N], wmax[N], iscale[N];
#pragma unroll
    for (int n = 0; n < N; n++) {
        const float e[4] = {v[n].x, v[n].y, v[n].z, v[n].w};
        amax[n] = 0.f; mx[n] = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float a = fabsf(e[i]);
            if (amax[n] < a) { amax[n] = a; mx[n] = e[i]; }
        }
    }
#pragma unroll
    for (int n = 0; n < N; n++) wmax[n] = wave_max(amax[n]);
#pragma unroll
    for (int n = 0; n < N; n++) {
        const unsigned long long winners = __ballot(amax[n] == wmax[n]);
        const int first = __ffsll((long long)winners) - 1;
        const float max = __shfl(mx[n], first, 64);
        iscale[n] = wmax[n] == 0.f ? 0.f : -128.0f / max;   // an all-zero block quantises to zeros with d = 0
    }
#pragma unroll
    for (int n = 0; n < N; n++) {
        const float e[4] = {v[n].x, v[n].y, v[n].z, v[n].w};
        int sum = 0;
        uint32_t packed = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float r = roundf(iscale[n] * e[i]);
            const int q = sat_i8(fminf(r, 127.f));
            sum += q;
            packed |= (uint32_t)(uint8_t)q << (8 * i);
        }
        sum += __shfl_xor(sum, 1, 64);
        sum += __shfl_xor(sum, 2, 64);
        if (valid[n]) {
            *reinterpret_cast<uint32_t*>(qs_block[n] + q8k_act_offset(4 * lane)) = packed;
            if ((lane & 3) == 0) bs_out[n][lane >> 2] = __int2half_rn(sum);
            if (lane == 0) *d_out[n] = wmax[n] == 0.f ? 0.f : 1.0f / iscale[n];
        }
    }
}

// The word kept beside a 32-element activation block.  Q8_0: the sum of the block's quants (the -8 / -16 code
// offsets of Q4_0 / Q5_0 weights leave through it).  Q8_1: the block's `s` widened to f32, s = f16(sum) * d in
// binary16 arithmetic (two 11-bit significands: the f32 product is exact, so one rounding to f16 remains).
__device__ inline int32_t q8_block_word(int vdt, int sum, float d_f16) {
    if (vdt != MOE_GGML_Q8_1) return sum;
    const float fs = __half2float(__float2half_rn((float)sum));
    return __float_as_int(__half2float(__float2half_rn(fs * d_f16)));
}

// Half a wave (32 lanes) quantises one 32-element block; lane holds element (lane & 31).  Q8_0 and Q8_1 blocks
// hold the same scale and quants.
//   q_out: the element's quant byte; d_out: f16-rounded scale widened to f32; word_out: see q8_block_word.
__device__ inline void quantize_q8_0_block(int vdt, float x, int lane, int8_t* q_out, float* d_out, int32_t* word_out) {
    float amax = fabsf(x);
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
    float d = amax / 127.0f;
    float id = (d != 0.f) ? 1.0f / d : 0.f;
    int q = sat_i8(roundf(x * id));
    *q_out = (int8_t)q;
    int sum = q;
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
    if ((lane & 31) == 0) {
        const float dh = __half2float(__float2half_rn(d));
        *d_out = dh;
        *word_out = q8_block_word(vdt, sum, dh);
    }
}

}  // namespace moe
