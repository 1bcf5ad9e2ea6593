// Wave-level activation quantisers.  They restate, per block, exactly what candle's
// k_quants::matmul applies to every lhs row before the integer dot products:
//   BlockQ8K::from_float   candle-core/src/quantized/k_quants.rs:1819-1856
//   BlockQ8_0::from_float  candle-core/src/quantized/k_quants.rs:605-634
//   BlockQ8_1::from_float  candle-core/src/quantized/k_quants.rs:700-729
// so the int8 operands are bit-identical to the CPU path's.
#pragma once
#include "moe_common.hpp"

namespace moe {

// `v.round() as i8` of the activation quantisers (f32::round: half away from zero; `as i8`: saturating, NaN -> 0) in five
// instructions.  For every float with |v| <= 130, trunc(v + copysign(0.49999997, v)) == v.round() (0.49999997 is the
// float below one half; checked over all 2.2e9 such floats), beyond that both sides of the clamp agree anyway, and the
// conversion instruction truncates toward zero, saturates and turns NaN into 0.
__device__ inline int round_as_i8(float v) {
    const int q = __float2int_rz(v + copysignf(0.49999997f, v));
    return min(max(q, -128), 127);
}
// `v.round().min(127.) as i8` (BlockQ8K::from_float, k_quants.rs:1843-1844): f32::min returns the other operand for a
// NaN, so a NaN becomes 127.
__device__ inline int round_min127_as_i8(float v) {
    const int q = __float2int_rz(fminf(v + copysignf(0.49999997f, v), 127.0f));
    return max(q, -128);
}


// Maximum over the wave, in every lane: four rotations inside the rows of 16 lanes (DPP: no LDS traffic, no address
// arithmetic), one exchange between neighbouring rows, and the two halves' values read back as scalars.
__device__ inline float wave_max(float v) {
#define MOE_ROR_MAX(n) v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x120 + (n), 0xf, 0xf, false)))
    MOE_ROR_MAX(8); MOE_ROR_MAX(4); MOE_ROR_MAX(2); MOE_ROR_MAX(1);
#undef MOE_ROR_MAX
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401f)));   // lane ^ 16
    const float lo = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float hi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    return fmaxf(lo, hi);
}
// v + (lane ^ 1's v) + (lane ^ 2's) + (lane ^ 3's): the sum over a quad, in each of its lanes
__device__ inline int quad_sum(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false);   // quad_perm [1, 0, 3, 2]
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, false);   // quad_perm [2, 3, 0, 1]
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
        int q = round_min127_as_i8(iscale * e[i]);
        sum += q;
        packed |= (uint32_t)(uint8_t)q << (8 * i);
    }
    *reinterpret_cast<uint32_t*>(qs_block + q8k_act_offset(4 * lane)) = packed;
    sum = quad_sum(sum);
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
            const int q = round_min127_as_i8(iscale[n] * e[i]);
            sum += q;
            packed |= (uint32_t)(uint8_t)q << (8 * i);
        }
        sum = quad_sum(sum);
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
    int q = round_as_i8(x * id);
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
