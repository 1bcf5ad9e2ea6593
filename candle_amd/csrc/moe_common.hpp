// Shared declarations of the gfx950 quantized-MoE library: error handling, block formats,
// device-side layouts and the small numeric helpers whose exact rounding decides parity with
// candle's CPU path.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <string>

#include "../../include/candle_amd_moe.h"

namespace moe {

// ---------------------------------------------------------------- errors
void set_error(int code, const std::string& msg);
int fail(int code, const std::string& msg);
#define MOE_HIP_CHECK(expr)                                                                       \
    do {                                                                                          \
        hipError_t _e = (expr);                                                                   \
        if (_e != hipSuccess)                                                                     \
            return ::moe::fail(MOE_E_HIP, std::string(#expr) + ": " + hipGetErrorString(_e));     \
    } while (0)

int ensure_device();  // 0 if a gfx950 device is usable

// ---------------------------------------------------------------- GGML block formats
// Sizes per candle-core/src/quantized/k_quants.rs:45-51 (Q4_0), 53-60 (Q4_1), 62-69 (Q5_0), 71-79 (Q5_1), 81-87 (Q8_0), 89-96 (Q8_1), 98-106 (Q2K), 108-116 (Q3K), 118-127 (Q4K),
// 129-137 (Q5K), 142-149 (Q6K), 151-158 (Q8K).
constexpr int QK_K = 256;
inline int64_t block_elems(int dt) {
    switch (dt) {
        case MOE_GGML_Q4_0: case MOE_GGML_Q4_1: case MOE_GGML_Q5_0: case MOE_GGML_Q5_1: case MOE_GGML_Q8_0: case MOE_GGML_Q8_1: return 32;
        case MOE_GGML_Q2K: case MOE_GGML_Q3K: case MOE_GGML_Q4K: case MOE_GGML_Q5K: case MOE_GGML_Q6K: case MOE_GGML_Q8K: return 256;
        default: return -1;
    }
}
inline int64_t block_bytes(int dt) {
    switch (dt) {
        case MOE_GGML_Q4_0: return 18;
        case MOE_GGML_Q4_1: return 20;
        case MOE_GGML_Q5_0: return 22;
        case MOE_GGML_Q5_1: return 24;
        case MOE_GGML_Q8_0: return 34;
        case MOE_GGML_Q8_1: return 36;
        case MOE_GGML_Q2K: return 84;
        case MOE_GGML_Q3K: return 110;
        case MOE_GGML_Q4K: return 144;
        case MOE_GGML_Q5K: return 176;
        case MOE_GGML_Q6K: return 210;
        case MOE_GGML_Q8K: return 292;
        default: return -1;
    }
}
__host__ __device__ constexpr int vecdot_dtype(int dt) {  // GgmlType::VecDotType, k_quants.rs:163,264,365,471,584,1189,1600
    return (dt == MOE_GGML_Q2K || dt == MOE_GGML_Q3K || dt == MOE_GGML_Q4K || dt == MOE_GGML_Q5K || dt == MOE_GGML_Q6K || dt == MOE_GGML_Q8K) ? MOE_GGML_Q8K
         : (dt == MOE_GGML_Q4_1 || dt == MOE_GGML_Q5_1 || dt == MOE_GGML_Q8_1) ? MOE_GGML_Q8_1 : MOE_GGML_Q8_0;
}
inline bool weight_dtype_supported(int dt) {
    return dt == MOE_GGML_Q4_0 || dt == MOE_GGML_Q4_1 || dt == MOE_GGML_Q5_0 || dt == MOE_GGML_Q5_1 || dt == MOE_GGML_Q8_0 || dt == MOE_GGML_Q2K || dt == MOE_GGML_Q3K || dt == MOE_GGML_Q4K || dt == MOE_GGML_Q5K || dt == MOE_GGML_Q6K;
}

// ---------------------------------------------------------------- device layouts
//
// WEIGHTS.  A matrix [N rows, K] is cut into row-tiles of 16 rows.  The values of every GGML
// block are kept bit-identical; only their placement changes so that a 64-lane wave fetches
// the operand of an int8 MFMA (16 rows x 32 k, lane l <-> row l%16, k-chunk l/16) with
// contiguous 16-byte-per-lane loads.
//
//  Q4K  tile(rt, sb) = 2304 B for 16 rows x one 256-element super-block:
//         [0,1024)    lane l: qs[row l%16][ 0+8g .. 0+8g+8) | qs[row][32+8g .. +8)   (g = l/16)
//         [1024,2048) lane l: qs[row l%16][64+8g ..       ) | qs[row][96+8g .. +8)
//         [2048,2304) row r : the block's first 16 bytes (d, dmin, 12 packed scale bytes)
//       tiles ordered [sb][rt]: the waves of a launch that are at the same step of their walk along
//       K read one contiguous region, which keeps the HBM channels evenly loaded.
//  Q2K  tile(rt, sb) = 1344 B, ordered [sb][rt]:
//         [0,1024)    lane l: word P (pair of 32-element stretches 2P, 2P+1), byte i: bits 1:0 / 3:2 = codes of
//                     elements 64P + 8g + i / + 4, bits 5:4 / 7:6 = codes of elements 64P + 32 + 8g + i / + 4
//         [1024,1280) row r : the 16 (scale | min << 4) bytes, one per 16 elements
//         [1280,1344) row r : d, dmin (f16 each)
//  Q3K  tile(rt, sb) = 1824 B, ordered [sb][rt]:
//         [0,1024)    lane l: the low two bits of the codes, placed as in the Q2K tile
//         [1024,1536) lane l: 8 bytes of high bits, placed as the fifth bits of the Q5K tile (set = no -4)
//         [1536,1792) row r : the sixteen scales, decoded to i8 (stored value - 32)
//         [1792,1824) row r : d (f16)
//  Q5K  tile(rt, sb) = 2816 B: the Q4K tile (nibbles, then d / dmin / scales of the 16 rows) followed by
//         [2304,2816) lane l: 8 bytes of fifth bits; byte i of word w (0..3, 0..1) holds, for pair 2w in
//                     bits 0..3 and pair 2w+1 in bits 4..7: the bits of elements 8g+i and 8g+4+i of the
//                     pair's first sub-block, then of its second
//  Q6K  tile(rt, sb) = 3360 B for 16 rows x one super-block, ordered [sb][rt] like Q4K.  The 6-bit
//       codes are split so that the low nibbles sit exactly where Q4K keeps its quants:
//         [0,1024)    lane l: byte i of pair P in {0,1}: low nibble = code[64P + 8g + i] & 15,
//         [1024,2048)         high nibble = code[64P + 32 + 8g + i] & 15   (pairs 2,3 in the second KiB)
//         [2048,3072) lane l: word P, byte i (0..3): bits 1:0 / 3:2 = code >> 4 of elements
//                     64P + 8g + i / + 4, bits 5:4 / 7:6 = the same of elements 64P + 32 + 8g + i / + 4
//         [3072,3328) row r : the 16 i8 scales (one per 16 elements)
//         [3328,3360) row r : d (f16)
//  Q8_0 tile(rt, kb) = 544 B for 16 rows x one 32-element block:
//         [0,512)   lane l: qs[row l%16][8g .. 8g+8)
//         [512,544) row r : d (f16)
//  Q4_0 tile(rt, kb) = 288 B:
//         [0,256)   (row r, half h): qs[row r][8h .. 8h+8)   (16 rows x 2 x 8 B)
//         [256,288) row r : d (f16)
//       MFMA k-chunk g of a Q4_0 block covers elements {0-7, 16-23, 8-15, 24-31}[g]: low / high
//       nibbles of byte half g>>1.
//  Q4_1 / Q5_0 / Q5_1 tiles (320 / 352 / 384 B): the 256 nibble bytes as in the Q4_0 tile, then, for the
//       five-bit formats, row r's 32 fifth bits as one little-endian word (bit e = element e), then row
//       r's d (f16) and, for the formats with a block minimum, m (f16) as one 4-byte pair.
//  Super-tiles of these five formats (matrices with K % 128 == 0; 16 rows x blocks 4s .. 4s+3, ordered
//       [step s][row-tile], four times the bytes of the one-block tile).  MFMA k-chunk g of a block covers
//       elements 4g .. 4g+3 and 16+4g .. 16+4g+3:
//         codes   lane l = (row l%16, g = l/16) at 16 l.  Nibble formats: word b = bytes 4g .. 4g+3 of block b's qs
//                 (low nibbles = elements 4g .., high nibbles = elements 16+4g ..).  Q8_0: 2 KiB, blocks 0,1 then 2,3;
//                 per block 8 bytes: elements 4g .. 4g+3, then 16+4g .. 16+4g+3.
//         fifth bits (Q5_0, Q5_1)  row r at 16 r: the four blocks' words
//         scales  row r at 8 r: the four d (f16); with a minimum, at 16 r: (d, m) per block
//
// ACTIVATIONS are quantised exactly as the reference does (Q8K for Q2K ... Q6K weights, Q8_1 for Q4_1 and
// Q5_1, Q8_0 otherwise) and stored per row as
//  Q8K  qs[K] with element k at ((k/64)*64 + ((k%32)/8)*16 + ((k/32)%2)*8 + k%8), so that lane
//       (row, g) fetches sub-blocks 2P and 2P+1, chunk g, with one 16-byte load;
//       d[K/256] f32;  bsums[K/256][16] as f16 (|sum of 16 quants| <= 2048 is exact in f16).
//  Q8_0 qs[K] in natural order; d[K/32] f32 (the f16-rounded scale widened);
//       bsum[K/32] i32 = sum of the block's 32 quants (used for the -8 / -16 offsets of Q4_0 / Q5_0).
//  Q8_1 as Q8_0, except that the word beside every block holds the block's `s` widened to f32:
//       s = f16(sum of quants) * d in binary16 arithmetic (k_quants.rs:727).
constexpr int Q4K_TILE_BYTES = 2304;
constexpr int Q2K_TILE_BYTES = 1344;
constexpr int Q3K_TILE_BYTES = 1824;
constexpr int Q5K_TILE_BYTES = 2816;
constexpr int Q6K_TILE_BYTES = 3360;
constexpr int Q8_0_TILE_BYTES = 544;
constexpr int Q4_0_TILE_BYTES = 288;
constexpr int Q4_1_TILE_BYTES = 320;
constexpr int Q5_0_TILE_BYTES = 352;
constexpr int Q5_1_TILE_BYTES = 384;

inline int64_t tile_bytes(int dt) {
    switch (dt) {
        case MOE_GGML_Q4K: return Q4K_TILE_BYTES;
        case MOE_GGML_Q2K: return Q2K_TILE_BYTES;
        case MOE_GGML_Q3K: return Q3K_TILE_BYTES;
        case MOE_GGML_Q5K: return Q5K_TILE_BYTES;
        case MOE_GGML_Q6K: return Q6K_TILE_BYTES;
        case MOE_GGML_Q8_0: return Q8_0_TILE_BYTES;
        case MOE_GGML_Q4_0: return Q4_0_TILE_BYTES;
        case MOE_GGML_Q4_1: return Q4_1_TILE_BYTES;
        case MOE_GGML_Q5_0: return Q5_0_TILE_BYTES;
        case MOE_GGML_Q5_1: return Q5_1_TILE_BYTES;
        default: return -1;
    }
}
// The 32-element formats keep a matrix whose K is a multiple of 128 in super-tiles of 16 rows x four blocks
// (same bytes in total), other matrices in the one-block tiles.
__host__ __device__ inline bool q32_super_layout(int64_t k) { return k % 128 == 0; }
// bytes of a re-laid [rows, k] matrix (rows % 16 == 0)
inline int64_t relaid_bytes(int dt, int64_t rows, int64_t k) {
    return (rows / 16) * (k / block_elems(dt)) * tile_bytes(dt);
}

// Quantised activation rows (device).
struct ActBuf {
    int8_t* qs = nullptr;    // [rows][K]
    float* d = nullptr;      // [rows][K/block]
    void* bsum = nullptr;    // Q8K: __half [rows][K/256][16]; Q8_0: int32 [rows][K/32]; Q8_1: float s [rows][K/32]
};

// ---------------------------------------------------------------- exp with the CPU's rounding
//
// candle's softmax and silu call Rust's f32::exp, i.e. the platform expf.  glibc's expf is not
// correctly rounded (about 0.502 ulp), so rounding a double-precision exp would differ from it
// in a fraction of a percent of the inputs and break bit-exact routing.  This is the algorithm
// glibc >= 2.27 uses (sysdeps/ieee754/flt-32/e_expf.c with the exp2f_data table, N = 32):
// exp(x) = 2^(k/N) * 2^(r/N), cubic polynomial in r, everything in double, one final rounding.
// All operations are IEEE double operations, identical on the CPU and on gfx950.
__host__ __device__ inline uint64_t exp2f_tab(int i) {
    constexpr uint64_t T[32] = {
        0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
        0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
        0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
        0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
        0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
        0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
        0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
        0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull};
    return T[i];
}

// `tab(i)`: entry i of the table above, from wherever the caller keeps it
template <class Tab>
__host__ __device__ inline float expf_glibc_with(float x, Tab tab) {
    if (x != x) return x;
    if (x > 0x1.62e42ep6f) return __builtin_inff();      // overflow
    if (x < -0x1.9fe368p6f) return 0.0f;                 // underflow (also -inf)
    const double InvLn2N = 0x1.71547652b82fep+0 * 32.0;
    const double Shift = 0x1.8p+52;
    const double C0 = 0x1.c6af84b912394p-5 / 32.0 / 32.0 / 32.0;
    const double C1 = 0x1.ebfce50fac4f3p-3 / 32.0 / 32.0;
    const double C2 = 0x1.62e42ff0c52d6p-1 / 32.0;
    double xd = (double)x;
    double z = InvLn2N * xd;
    double kd = z + Shift;
    uint64_t ki;
    __builtin_memcpy(&ki, &kd, 8);
    kd -= Shift;
    double r = z - kd;
    uint64_t t = tab((int)(ki % 32));
    t += ki << (52 - 5);
    double s;
    __builtin_memcpy(&s, &t, 8);
    // the x86-64 glibc build selected on FMA-capable CPUs contracts these three expressions
    z = __builtin_fma(C0, r, C1);
    double r2 = r * r;
    double y = __builtin_fma(C2, r, 1.0);
    y = __builtin_fma(z, r2, y);
    y = y * s;
    return (float)y;
}
__host__ __device__ inline float expf_glibc(float x) {
    return expf_glibc_with(x, [](int i) { return exp2f_tab(i); });
}

// Total order of Rust's f32::total_cmp as a sortable signed integer.
__host__ __device__ inline int32_t total_key(float f) {
    int32_t b;
    __builtin_memcpy(&b, &f, 4);
    b ^= (int32_t)(((uint32_t)(b >> 31)) >> 1);
    return b;
}

// Rust `as i8` after f32::round: saturating, NaN -> 0.
__device__ inline int8_t sat_i8(float v) {
    if (v != v) return 0;
    v = fminf(fmaxf(v, -128.f), 127.f);
    return (int8_t)(int)v;
}

}  // namespace moe
