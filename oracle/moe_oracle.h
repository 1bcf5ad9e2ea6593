/*
 * CPU oracle for candle's quantized sparse-MoE path.  TEST INFRASTRUCTURE ONLY:
 * nothing in the shipped library links or calls this code.  It is used by the
 * tests, the smoke check and the CPU-baseline leg of the benchmark.
 *
 * Every function is a restatement, in plain C, of one function of the
 * reference (john-sharratt/candle v0.9.1).  The reference location is given
 * beside each declaration as file:line relative to the reference root.
 *
 * Pinning status (what independent evidence each function is checked against):
 *   f16 conversions        exhaustive against numpy float16
 *   q4_0 quantize/dequant  exact 128-value vector of candle-core/tests/quantized_tests.rs:262-291
 *   q4_0 x q8_0 matmul     exact integers of quantized_tests.rs:89-104 and :149-169
 *   q4_1, q5_0, q5_1       exact 128-value round trips of quantized_tests.rs:296-392 (to three decimals, as the reference
 *                          states them), ggml RMSE / dot-error bounds :821-911, independent numpy block decoders,
 *                          float64 dot of the dequantised operands
 *   q8_1 quantize, dots    closed form (the Q8_0 block plus s = f16(sum) * d), ggml dot-error bound :836
 *   q8_0 quantize/dequant  closed form + ggml RMSE / dot-error bounds (quantized_tests.rs:428-469,821-911)
 *   q4k  quantize/dequant  spot values and error bounds of quantized_tests.rs:566-611, and the seeded
 *                          (11,512,21) mat-mul spot values of :1102-1121 through a restated rand-0.9 StdRng
 *   q2k  quantize/dequant  spot values and error bounds of quantized_tests.rs:471-517, ggml dot error :821-911,
 *                          the seeded (11,512,21) mat-mul spot values of :1048-1074, independent decoder
 *   q3k  quantize/dequant  spot values and error bounds of quantized_tests.rs:519-563, ggml dot error :821-911,
 *                          the seeded (11,512,21) mat-mul spot values of :1076-1100, independent decoder
 *   q5k  quantize/dequant  spot values and error bounds of quantized_tests.rs:613-658, ggml dot error :821-911,
 *                          the seeded (11,512,21) mat-mul spot values of :1129-1152, independent decoder
 *   q6k  quantize/dequant  spot values and error bound of quantized_tests.rs:660-700, ggml dot error :821-911,
 *                          the seeded (11,512,21) mat-mul spot values of :1156-1178, and an independent
 *                          bit-field decoder of the block layout (tests/test_oracle_quant.py)
 *   q8k  quantize/dequant  spot values quantized_tests.rs:707-752
 *   softmax                candle-nn/tests/ops.rs:9-53 + float64 closed form
 *   rms_norm, sigmoid      candle-nn/tests/ops.rs:55-78, :317-325
 *   top-k routing / lists  NO reference test exists; pinned by invariants, constructed ties and
 *                          brute force (see tests/test_oracle_routing.py)
 *   whole block            NO reference test exists; pinned by composition + a float64
 *                          dequantised-weights model (tests/test_oracle_block.py)
 *   router logits bits     parity unpinned: the reference computes them with the un-vendored
 *                          `gemm` crate 0.18.2 whose f32 summation order is not in the tree.
 */
#ifndef MOE_ORACLE_H
#define MOE_ORACLE_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml dtype numbering: candle-core/src/quantized/mod.rs:153-174 */
enum { ORC_Q4_0 = 2, ORC_Q4_1 = 3, ORC_Q5_0 = 6, ORC_Q5_1 = 7, ORC_Q8_0 = 8, ORC_Q8_1 = 9, ORC_Q2K = 10, ORC_Q3K = 11, ORC_Q4K = 12, ORC_Q5K = 13, ORC_Q6K = 14, ORC_Q8K = 15 };

#pragma pack(push, 1)
typedef struct { uint16_t d; uint8_t qs[16]; } orc_block_q4_0;            /* k_quants.rs:45-51  */
typedef struct { uint16_t d; int8_t qs[32]; } orc_block_q8_0;             /* k_quants.rs:81-87  */
typedef struct { uint16_t d, m; uint8_t qs[16]; } orc_block_q4_1;         /* k_quants.rs:53-60  */
typedef struct { uint16_t d; uint8_t qh[4]; uint8_t qs[16]; } orc_block_q5_0;     /* k_quants.rs:62-69  */
typedef struct { uint16_t d, m; uint8_t qh[4]; uint8_t qs[16]; } orc_block_q5_1;  /* k_quants.rs:71-79  */
typedef struct { uint16_t d, s; int8_t qs[32]; } orc_block_q8_1;          /* k_quants.rs:89-96  */
typedef struct { uint16_t d, dmin; uint8_t scales[12]; uint8_t qs[128]; } orc_block_q4k; /* :118-127 */
typedef struct { uint8_t scales[16]; uint8_t qs[64]; uint16_t d, dmin; } orc_block_q2k;   /* k_quants.rs:98-106 */
typedef struct { uint8_t hmask[32]; uint8_t qs[64]; uint8_t scales[12]; uint16_t d; } orc_block_q3k; /* k_quants.rs:108-116 */
typedef struct { uint16_t d, dmin; uint8_t scales[12]; uint8_t qh[32]; uint8_t qs[128]; } orc_block_q5k; /* :129-137 */
typedef struct { uint8_t ql[128]; uint8_t qh[64]; int8_t scales[16]; uint16_t d; } orc_block_q6k; /* :142-149 */
typedef struct { float d; int8_t qs[256]; int16_t bsums[16]; } orc_block_q8k;            /* :151-158 */
#pragma pack(pop)

/* half crate 2.5 f16 <-> f32 (IEEE, round-to-nearest-even, subnormals kept) */
float    orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_f16(float f);

/* type_size / block_size table: candle-core/src/quantized/mod.rs:218-252 */
int64_t orc_block_elems(int dtype);
int64_t orc_block_bytes(int dtype);
/* VecDotType of a weight dtype: k_quants.rs:163,584,1189 */
int     orc_vecdot_dtype(int dtype);

/* from_float / to_float: k_quants.rs:166-224 (Q4_0), 299-359 (Q4_1), 404-465 (Q5_0), 511-581 (Q5_1), 587-634 (Q8_0), 700-729 (Q8_1, from_float only), 808-908 (Q2K), 1047-1186 (Q3K), 1287-1374 (Q4K), 1487-1595 (Q5K), 1673-1790 (Q6K),
 * 1819-1871 (Q8K).
 * n must be a multiple of the block size.  Return 0 or -1 (bad dtype / size). */
int orc_quantize(int dtype, const float* x, int64_t n, void* blocks);
int orc_dequantize(int dtype, const void* blocks, int64_t n, float* y);

/* vec_dot_unopt: k_quants.rs:241-258, 270-297 (Q4_1), 381-402 (Q5_0), 477-509 (Q5_1), 650-668, 680-698 (Q8_1), 755-805 (Q2K), 927-1045 (Q3K), 1205-1285, 1394-1485 (Q5K), 1613-1671 (Q6K) */
float orc_vec_dot(int dtype, int64_t n, const void* w_blocks, const void* act_blocks);

/* k_quants::matmul, k_quants.rs:1873-1920: dst[m,n] = lhs[m,k] . rhs_t[n,k]^T, lhs quantised
 * row by row to the VecDotType.  simd=0 uses vec_dot_unopt, simd=1 the AVX2 loops that restate
 * candle-core/src/quantized/avx.rs:50-87,131-216,224-441,443-638 (falls back to 0 if the CPU lacks AVX2+FMA).
 * threads<=1 runs serially; otherwise output columns are split over threads as rayon does. */
int orc_matmul(int dtype, int64_t m, int64_t k, int64_t n, const float* lhs, const void* rhs_t,
               float* dst, int simd, int threads);
int orc_has_avx2(void);

/* softmax_last_dim: candle-nn/src/ops.rs:313-351, max cpu/kernels.rs:40-45, sum cpu/mod.rs:132-151
 * with the AVX2 accumulator order of cpu/avx.rs:54-68 (plain left-to-right when cols < 32). */
void orc_softmax_last_dim(const float* x, int64_t rows, int64_t cols, float* y);

/* silu op.rs:646-648, sigmoid candle-nn/src/ops.rs:59-61 */
float orc_silu(float v);
float orc_sigmoid(float v);

/* rms_norm: candle-nn/src/ops.rs:504-515 */
void orc_rms_norm(const float* x, int64_t rows, int64_t cols, const float* alpha, float eps, float* y);

/* Router gate xs[T,H] . wg[E,H]^T in f32, plain left-to-right accumulation without fused
 * multiply-add.  The reference does this with the gemm crate (cpu_backend/mod.rs:1308-1392);
 * its summation order is not pinned, so this is one admissible answer, not THE answer. */
void orc_gate_logits(const float* xs, int64_t T, int64_t H, const float* wg, int64_t E, float* logits);

/* Routing given probabilities: quantized_llama.rs:158-179 (Mixtral flavour, always renormalised)
 * and qwen2_moe.rs:270-293 (norm_topk selectable).  Outputs:
 *   topk_idx[T*k], topk_w[T*k]  in rank order per token
 *   offsets[E+1]                exclusive prefix of per-expert list lengths
 *   perm_token[T*k]             token row of every list slot (lists concatenated in expert order,
 *                               each ascending in token index)
 *   perm_w[T*k]                 routing weight of every list slot */
int orc_route(const float* probs, int64_t T, int64_t E, int64_t k, int norm_topk,
              int32_t* topk_idx, float* topk_w, int32_t* offsets, int32_t* perm_token, float* perm_w);

/* Description of one MoE layer for the block-level oracle. */
typedef struct {
    int64_t H, F, E, k;
    int dtype;                 /* expert weight dtype */
    int norm_topk;             /* 1 for Mixtral */
    const float* gate;         /* [E,H] f32 */
    const float* gate_bias;    /* optional [E], added to the logits (harness construct) */
    const void* const* w1;     /* E pointers, each [F,H] blocks */
    const void* const* w3;     /* E pointers, each [F,H] blocks */
    const void* const* w2;     /* E pointers, each [H,F] blocks */
    int64_t Fs;                /* shared expert width, 0 if none (qwen2_moe.rs:315-319) */
    const void *sw1, *sw3, *sw2;
    const float* shared_gate;  /* [H] */
    const float* rms_alpha;    /* optional [H]: y = x + moe(rms_norm(x)) (quantized_llama.rs:888-892) */
    float rms_eps;
    int dtype_down;            /* dtype of w2 (and sw2) when it differs from `dtype`, as in files that store
                                  ffn_down as Q6K beside Q4K gate/up matrices; 0 = same as `dtype` */
} orc_layer;

/* MlpOrMoe::forward (MoE arm) quantized_llama.rs:143-211.  If logits_in != NULL they are used
 * instead of computing the gate product (routing "given the same router logits").
 * logits_out (optional) receives the logits actually used. */
int orc_moe_forward(const orc_layer* L, const float* xs, int64_t T, const float* logits_in,
                    float* logits_out, float* ys, int simd, int threads);

/* Deterministic N(0,std) filler (splitmix64 counter + Box-Muller), identical for any thread count. */
void orc_fill_normal(uint64_t seed, int64_t n, float mean, float std, float* out, int threads);
/* Fill + quantise row by row without materialising the f32 tensor. */
int orc_fill_normal_quantized(uint64_t seed, int dtype, int64_t rows, int64_t k, float std,
                              void* blocks, int threads);

#ifdef __cplusplus
}
#endif
#endif
