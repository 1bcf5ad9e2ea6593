/*
 * candle_amd_moe.h -- C ABI of the MI355X (gfx950) quantized sparse-MoE block.
 *
 * The library replaces ONE path of candle: the `MlpOrMoe::MoE` arm of
 * candle-transformers/src/models/quantized_llama.rs:143-211 together with the per-expert
 * `QMatMul::forward` calls it makes (candle-core/src/quantized/mod.rs:533-556 ->
 * k_quants::matmul, candle-core/src/quantized/k_quants.rs:1873-1920).  candle has no C FFI
 * for this path; its interface is the Rust trait
 *     candle::Module { fn forward(&self, xs: &Tensor) -> Result<Tensor> }   (candle-core/src/lib.rs:148-150)
 * and, for user ops, `CustomOp1::cpu_fwd` (candle-core/src/custom_op.rs:7-41).  candle's `Device`
 * has no HIP variant (candle-core/src/device.rs:16-20), so a drop-in op receives and returns HOST
 * f32 storage; the quantized weights live on the GPU inside the layer object.
 *
 * Conventions
 *   - every function returns 0 on success, a non-zero MOE_E_* code on failure;
 *     moe_last_error() returns the message of the calling thread's last failure
 *     (the Rust side maps it to candle::Error::Msg, candle-core/src/error.rs:233).
 *   - host pointers passed to moe_layer_create are BORROWED for the duration of the call only;
 *     the library copies and re-lays the blocks on the device and owns that memory.
 *   - activations are contiguous row-major f32 [n_tokens, hidden]; the reference bails on
 *     anything else (candle-core/src/quantized/mod.rs:480-482,501).
 *   - a layer may be used from several threads (QuantizedType: Send + Sync,
 *     candle-core/src/quantized/mod.rs:256); calls on one layer are serialised internally.
 *   - there is no CPU fallback: without a usable HIP device every entry point fails.
 */
#ifndef CANDLE_AMD_MOE_H
#define CANDLE_AMD_MOE_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GgmlDType numbering, candle-core/src/quantized/mod.rs:153-174 (also the GGUF on-disk ids). */
#define MOE_GGML_Q4_0 2
#define MOE_GGML_Q4_1 3
#define MOE_GGML_Q5_0 6
#define MOE_GGML_Q5_1 7
#define MOE_GGML_Q8_0 8
#define MOE_GGML_Q8_1 9   /* activations only (VecDotType of Q4_1 and Q5_1) */
#define MOE_GGML_Q2K 10
#define MOE_GGML_Q3K 11
#define MOE_GGML_Q4K 12
#define MOE_GGML_Q5K 13
#define MOE_GGML_Q6K 14
#define MOE_GGML_Q8K 15

#define MOE_OK 0
#define MOE_E_INVALID 1   /* bad argument / unsupported shape or dtype */
#define MOE_E_HIP 2       /* HIP runtime error (message carries hipGetErrorString) */
#define MOE_E_NODEVICE 3  /* no gfx950 device visible */
#define MOE_E_NOMEM 4

typedef struct moe_layer moe_layer;

/* One MoE layer.  Replaces the fields of `MlpOrMoe::MoE` (quantized_llama.rs:133-141):
 * `feed_forward_gate_inp` -> gate, `experts[e].feed_forward_w{1,2,3}` -> w1/w2/w3,
 * `n_expert_used` -> top_k.  Weight matrices are the raw bytes of a CPU QTensor
 * (`QTensor::data()`, candle-core/src/quantized/mod.rs:394-396): rows of GGML blocks,
 * w1 and w3 are [ffn, hidden], w2 is [hidden, ffn]. */
typedef struct {
    int64_t hidden;              /* H */
    int64_t ffn;                 /* F: per-expert intermediate size */
    int64_t n_experts;           /* E (1..256) */
    int64_t top_k;               /* n_expert_used (0..min(E,16)); 0 is what the reference runs with when the file lacks
                                    llama.expert_used_count (quantized_llama.rs:507-512): `take(0)` at :167 selects no
                                    expert and the block returns zeros (plus the residual when rms_alpha is set).  Not
                                    accepted together with a shared expert. */
    int32_t ggml_dtype;          /* MOE_GGML_Q4_0 | Q4_1 | Q5_0 | Q5_1 | Q8_0 | Q2K | Q3K | Q4K | Q5K | Q6K: dtype of every w1 and w3 (and of w2
                                    unless ggml_dtype_down says otherwise) */
    int32_t norm_topk;           /* 1: weights renormalised over the selected experts (Mixtral,
                                    quantized_llama.rs:175-178); 0: raw softmax probability
                                    (qwen2_moe.rs:287 with norm_topk_prob=false) */
    const float* gate;           /* [E, H] f32: an F32 / F16 / BF16 router is dequantised at load (mod.rs:429-436) */
    const float* gate_bias;      /* optional [E], added to the logits; NULL for the reference's models */
    const void* const* w1;       /* E pointers */
    const void* const* w3;       /* E pointers */
    const void* const* w2;       /* E pointers */
    /* always-on shared expert, qwen2_moe.rs:315-319; shared_ffn == 0 disables it */
    int64_t shared_ffn;
    const void* shared_w1;       /* [shared_ffn, H] */
    const void* shared_w3;       /* [shared_ffn, H] */
    const void* shared_w2;       /* [H, shared_ffn] */
    const float* shared_gate;    /* [H] f32, sigmoid gate */
    /* optional fused pre-norm + residual, quantized_llama.rs:888-892: y = x + moe(rms_norm(x)) */
    const float* rms_alpha;      /* [H] or NULL */
    float rms_eps;
    /* dtype of every w2 (and shared_w2) when it differs from ggml_dtype, 0 = the same.  GGUF files of
     * the Q4_K_M flavour store ffn_down of some layers as Q6K beside Q4K gate / up matrices; the two
     * dtypes must quantise activations the same way (Q2K ... Q6K use Q8K; Q4_0, Q5_0 and Q8_0 use Q8_0;
     * Q4_1 and Q5_1 use Q8_1). */
    int32_t ggml_dtype_down;
    /* A router tensor that is not F32 / F16 / BF16 stays quantised in the reference: `QMatMul::from_arc`
     * (candle-core/src/quantized/mod.rs:428-447) dequantises those three only, any other `ffn_gate_inp` runs as
     * `QMatMul::QTensor`, i.e. the logits are a quantised product over the rows quantised to the gate dtype's
     * activation format (mod.rs:533-537 -> k_quants::matmul, k_quants.rs:1873-1920).  gate_dtype != 0 selects that arm:
     * gate_blocks holds the raw GGML blocks of the [E, H] tensor in that dtype (any dtype ggml_dtype accepts) and `gate`
     * is not read.  hidden has to be a multiple of 256; not accepted together with a shared expert. */
    int32_t gate_dtype;
    const void* gate_blocks;
} moe_desc;

/* Uploads and re-lays the weights.  Replaces the construction at quantized_llama.rs:553-578. */
int moe_layer_create(const moe_desc* desc, moe_layer** out);
void moe_layer_destroy(moe_layer* layer);

/* hidden, ffn, n_experts and top_k of a layer (what a caller that built it from a GGUF file needs for its shape
 * checks; the reference reads the same from `feed_forward_gate_inp` / `n_expert_used`).  Any pointer may be NULL. */
int moe_layer_shape(const moe_layer* layer, int64_t* hidden, int64_t* ffn, int64_t* n_experts, int64_t* top_k);

/* `MlpOrMoe::forward`, quantized_llama.rs:143-211 (== CustomOp1::cpu_fwd for the drop-in op):
 * x and y are HOST f32 [n_tokens, hidden]; synchronous. */
int moe_layer_forward(moe_layer* layer, const float* x, int64_t n_tokens, float* y);

/* moe_layer_forward_device may be recorded into a HIP graph (stream capture): it then allocates nothing
 * and fails with a message if its workspace was not reserved by an earlier forward of the same size.  The graph's
 * nodes hold addresses inside the layer's workspace: from the first capture on, the layer never frees workspace
 * memory before moe_layer_destroy (a later, larger eager forward moves to new memory and keeps the old alive), so a
 * replay stays valid; a replay and another call on the same layer must not overlap in time (they share the layer). */
/* (Both entries cut inputs of more than (2^31 - 1) / (top_k * max(hidden, ffn)) tokens into several passes;
 * after such a call the moe_layer_last_* hooks fail, since they describe one pass.) */

/* Same computation on DEVICE pointers, enqueued on `hip_stream` (a hipStream_t, NULL = default
 * stream) without synchronising.  d_x and d_y must not alias or overlap, and d_y is the call's to
 * write from its first kernel on (top-2 layers clear it early and accumulate the two expert terms of
 * a token in place), so nothing else may read or write it while the call runs.  This is the entry a
 * caller that already keeps activations on the GPU uses (no PCIe in the path). */
int moe_layer_forward_device(moe_layer* layer, const void* d_x, int64_t n_tokens, void* d_y, void* hip_stream);

/* The MoE blocks of consecutive transformer layers as one call: y = layer[n-1](... layer[1](layer[0](x))), each layer's own
 * forward (with rms_alpha: x + moe(rms_norm(x)), `ModelWeights::forward`, quantized_llama.rs:886-892, without the attention
 * half of the layer).  Same results, bit for bit, as n calls of moe_layer_forward_device; what the call adds is that
 * between two layers of a small (decode) batch the first layer's combine pass and residual add and the second layer's
 * rms-norm, router and activation quantiser are ONE launch.  The layers must be distinct objects of one hidden size;
 * n_tokens at most what one pass carries.  Like moe_layer_forward_device it can be recorded into a HIP graph after one
 * eager call of the same size.  d_x and d_y must not overlap. */
int moe_stack_forward_device(moe_layer* const* layers, int64_t n_layers, const void* d_x, int64_t n_tokens, void* d_y, void* hip_stream);

/* No counterpart in the reference.  For callers that cannot allocate device memory while they run: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  The same forward as
 * moe_layer_forward_device (same kernels, same results), but its workspace (routing lists, quantised activations,
 * the experts' weighted outputs) is a file-scope device array of MOE_STATIC_SCRATCH_BYTES bytes that every GPU the
 * library runs on holds until the process ends; the call makes no hipMalloc / hipFree.  A batch whose workspace
 * exceeds the array is rejected with MOE_E_INVALID and a message (Mixtral-8x7B shape: batches of up to 119 tokens fit; the
 * need grows with n_tokens * top_k * (ffn + 4 hidden)).  All layers and all calls on one GPU share the array: calls
 * that overlap in time on one GPU race (same-stream calls are ordered by the stream). */
#define MOE_STATIC_SCRATCH_BYTES (8 * 1024 * 1024)
int moe_layer_forward_device_noalloc(moe_layer* layer, const void* d_x, int64_t n_tokens, void* d_y, void* hip_stream);
int64_t moe_static_scratch_bytes(void);

/* Measurement aid (no counterpart in the reference): one forward as moe_layer_forward_device with
 * HIP events recorded on `hip_stream` between the launches; waits for completion and returns the
 * elapsed milliseconds of the seven stages in stage_ms[0..6]: front (router + activation quantiser),
 * dispatch (0 for small batches), up (w1/w3 + SiLU), requant (Q8K/Q8_0 quantisation of the
 * intermediate as a pass of its own: large Q4_K batches only, otherwise part of up), down (w2),
 * shared expert, combine. */
int moe_layer_forward_timed(moe_layer* layer, const void* d_x, int64_t n_tokens, void* d_y, void* hip_stream, float* stage_ms);

/* Router logits [n_tokens, E] (after the optional bias) that the last forward on this layer
 * computed, copied to the host.  Debug / parity hook: candle computes these with the `gemm`
 * crate whose f32 summation order is not part of the reference tree. */
int moe_layer_last_logits(moe_layer* layer, float* logits, int64_t n_tokens);

/* Routing that the last forward produced (host copies): topk_idx/topk_w [n_tokens, k] in rank
 * order, expert_offsets [E+1], perm_token / perm_w [n_tokens*k] (per-expert token lists).
 * Any pointer may be NULL. */
int moe_layer_last_routing(moe_layer* layer, int64_t n_tokens, int32_t* topk_idx, float* topk_w,
                           int32_t* expert_offsets, int32_t* perm_token, float* perm_w);

/* Device-layout check: dequantises expert `expert` (0..E-1, or E for the shared expert), matrix
 * `which` (1, 2 or 3) from the re-laid device copy into host f32 [rows*cols] in the ORIGINAL
 * row-major order.  Must equal `to_float` of the bytes passed at create. */
int moe_layer_dequantize_weight(moe_layer* layer, int64_t expert, int which, float* out, int64_t n_elems);

/* Parity hook: router + dispatch given logits (host pointers).  Restates softmax_last_dim
 * (candle-nn/src/ops.rs:313-351) + the host top-k loop (quantized_llama.rs:158-179) on the GPU.
 * Outputs as for moe_layer_last_routing.  The reference has no FFI for this step, so the signature is this
 * library's own: it takes no layer handle (routing needs E, k and the renormalisation flag only) and also returns
 * the per-slot weights perm_w that `selected_rws` holds (quantized_llama.rs:174-178).  A NaN probability is ranked as
 * f32::total_cmp ranks it (:166): above every number when its sign bit is clear, below when set. */
int moe_route(const float* logits, int64_t n_tokens, int64_t n_experts, int64_t top_k, int32_t norm_topk,
              int32_t* topk_idx, float* topk_w, int32_t* expert_offsets, int32_t* perm_token, float* perm_w);

/* Parity hook: GgmlType::to_float on raw blocks (host pointers), k_quants.rs:166-186 (Q4_0), 340-359 (Q4_1),
 * 443-465 (Q5_0), 556-581 (Q5_1), 587-603 (Q8_0), 872-908 (Q2K), 1131-1186 (Q3K), 1347-1374 (Q4K), 1563-1595 (Q5K), 1753-1790 (Q6K), 1858-1870 (Q8K). */
int moe_dequantize(int32_t ggml_dtype, const void* blocks, int64_t n_elems, float* out);

/* Parity hook: the activation quantiser k_quants::matmul applies to every lhs row
 * (k_quants.rs:1893-1903): vecdot_dtype MOE_GGML_Q8_0 (k_quants.rs:605-634), MOE_GGML_Q8_1
 * (k_quants.rs:700-729) or MOE_GGML_Q8K (k_quants.rs:1819-1856).  x is host f32 [rows, k]; out receives rows*k/block standard blocks. */
int moe_quantize_act(int32_t vecdot_dtype, const float* x, int64_t rows, int64_t k, void* out);

/* Parity hook: QMatMul::forward on one quantized matrix (quantized/mod.rs:533-537 ->
 * k_quants.rs:1873-1920): y[m, n] = x[m, k] . W[n, k]^T, host pointers, W as raw blocks.
 * (moe_qlinear_create + moe_qlinear_forward + moe_qlinear_destroy in one call.) */
int moe_qmatmul(int32_t ggml_dtype, const void* w_blocks, int64_t n, int64_t k, const float* x, int64_t m, float* y);

/* ---- dense quantized projection --------------------------------------------------------------
 * The QMatMul::QTensor arm of candle-core/src/quantized/mod.rs:428-447 (from_arc / from_qtensor) and
 * 533-537 (forward): the attention projections and the output head around the MoE block
 * (quantized_llama.rs:590-593 attention_wq/wk/wv/wo, :608 output; applied at :275-277, :345, :897).
 * create uploads the [n, k] matrix of raw GGML blocks once (n % 16 == 0, k a multiple of the block
 * size; Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2K, Q3K, Q4K, Q5K, Q6K) and keeps it resident in the kernels' layout; forward quantises the m rows
 * of x as k_quants::matmul does (k_quants.rs:1893-1903) and writes y[m, n] = x . W^T.
 * forward takes host pointers and returns when y is filled; forward_device takes device pointers and
 * enqueues on hip_stream.  Calls on one object serialise (a call on another stream waits for the previous call's
 * kernels); captures into HIP graphs follow the rules given for moe_layer_forward_device.  dequantize is QMatMul::dequantize
 * (QTensor::dequantize, mod.rs:367-371) of the resident copy: [n, k] f32. */
typedef struct moe_qlinear moe_qlinear;
int moe_qlinear_create(int32_t ggml_dtype, const void* w_blocks, int64_t n, int64_t k, moe_qlinear** out);
void moe_qlinear_destroy(moe_qlinear* q);
int moe_qlinear_forward(moe_qlinear* q, const float* x, int64_t m, float* y);
int moe_qlinear_forward_device(moe_qlinear* q, const void* d_x, int64_t m, void* d_y, void* hip_stream);
int moe_qlinear_dequantize(moe_qlinear* q, float* out, int64_t n_elems);
int moe_qlinear_shape(const moe_qlinear* q, int64_t* n, int64_t* k, int32_t* ggml_dtype);

/* ---- rms-norm as an operation of its own --------------------------------------------------------
 * RmsNorm::forward (candle-transformers/src/quantized_nn.rs:100-126 -> candle_nn::ops::rms_norm,
 * candle-nn/src/ops.rs:504-515): y = x / sqrt(sum(x^2) / hidden + eps) * alpha per row, the squares summed left
 * to right in f32 as the reference does (bit-identical divisor).  moe_add_rms_norm_device also folds in the
 * `(attn + residual)` that precedes `ffn_norm` in the decoder layer (quantized_llama.rs:884-888): with d_residual
 * set it stores v = x + residual to d_sum (the layer's new residual stream) and normalises v.  hidden % 4 == 0,
 * hidden <= 16256.  (The norm + residual around the MoE block itself is fused into the layer: moe_desc.rms_alpha.) */
int moe_rms_norm(const float* x, const float* alpha, float eps, int64_t rows, int64_t hidden, float* y);
int moe_add_rms_norm_device(const void* d_x, const void* d_residual, const void* d_alpha, float eps, int64_t rows, int64_t hidden,
                            void* d_sum, void* d_y, void* hip_stream);

/* QTensor::quantize (candle-core/src/quantized/mod.rs:331-349) on the GPU: f32 [n_elems] -> raw
 * GGML blocks, bit-identical to GgmlType::from_float of k_quants.rs:188-224 (Q4_0), 605-634 (Q8_0), 808-870 (Q2K),
 * 1049-1129 (Q3K), 1287-1345 (Q4K), 1484-1561 (Q5K) and 1675-1751 (Q6K); other formats are refused.  Host pointers /
 * device pointers (the latter enqueued on hip_stream). */
int moe_quantize_weights(int32_t ggml_dtype, const float* x, int64_t n_elems, void* out_blocks);
int moe_quantize_weights_device(int32_t ggml_dtype, const void* d_x, int64_t n_elems, void* d_out_blocks, void* hip_stream);

/* ---- GGUF expert loader -------------------------------------------------------------------
 * `Content::read` (candle-core/src/quantized/gguf_file.rs:439-511) on a memory-mapped file: magic and
 * version 1-3, metadata table, tensor table (dimensions reversed to outermost-first), tensor data
 * start rounded up to `general.alignment` (default 32).  Host code only: usable without a GPU. */
typedef struct moe_gguf moe_gguf;
int moe_gguf_open(const char* path, moe_gguf** out);
void moe_gguf_close(moe_gguf* file);
int moe_gguf_version(const moe_gguf* file);
int64_t moe_gguf_tensor_count(const moe_gguf* file);
uint64_t moe_gguf_tensor_data_offset(const moe_gguf* file);          /* Content::tensor_data_offset */
const char* moe_gguf_tensor_name(const moe_gguf* file, int64_t index); /* file order; NULL past the end */
/* Metadata accessors, `Value::to_*` (gguf_file.rs:226-294): value_type is the on-disk ValueType id
 * (gguf_file.rs:402-420); u64 upcasts u8/u16/u32/bool as Value::to_u64 does. */
int moe_gguf_metadata_type(const moe_gguf* file, const char* key, int* value_type);
int moe_gguf_metadata_u64(const moe_gguf* file, const char* key, uint64_t* out);
int moe_gguf_metadata_i64(const moe_gguf* file, const char* key, int64_t* out);
int moe_gguf_metadata_f64(const moe_gguf* file, const char* key, double* out);
int moe_gguf_metadata_str(const moe_gguf* file, const char* key, char* buf, uint64_t cap);
int moe_gguf_metadata_array_len(const moe_gguf* file, const char* key, uint64_t* len, int* elem_type);
/* `TensorInfo::read_from_mmap` (gguf_file.rs:91-126): dtype id, shape (outermost first, up to 8 dims)
 * and a pointer into the mapping, valid until moe_gguf_close; same divisibility and bounds checks. */
int moe_gguf_tensor(const moe_gguf* file, const char* name, int* ggml_dtype, int* n_dims, int64_t dims[8], const void** data,
                    uint64_t* nbytes);
/* The MoE arm of `ModelWeights::from_gguf` for ONE layer (quantized_llama.rs:506-512, 553-578):
 * `llama.expert_count`, `llama.expert_used_count` (0 when absent, as there: a layer that selects no expert),
 * `blk.{l}.ffn_gate_inp.weight` (F32, F16 or BF16, the dtypes QMatMul::from_arc dequantises, quantized/mod.rs:429-443;
 * a quantised router tensor is refused) and `blk.{l}.ffn_{gate,down,up}.{i}.weight` as w1 / w2 / w3.  All gate / up
 * matrices of the layer must share one supported dtype and all down matrices one (Q4K gate / up with
 * Q6K down, as Q4_K_M files have it, or Q5K with Q6K, is accepted).  Needs the GPU. */
int moe_layer_create_from_gguf(const moe_gguf* file, int layer_index, int norm_topk, moe_layer** out);
/* One named two-dimensional quantized tensor of the file as a resident projection: what
 * `QMatMul::from_qtensor(ct.tensor(reader, name, device)?)` builds for `blk.{l}.attn_q.weight`,
 * `blk.{l}.attn_output.weight`, `output.weight` ... (quantized_llama.rs:533-547, 590-593, 608).  Needs the GPU. */
int moe_qlinear_create_from_gguf(const moe_gguf* file, const char* tensor_name, moe_qlinear** out);

/* Message of the calling thread's last error ("" if none). */
const char* moe_last_error(void);

/* Name of the device the library runs on, e.g. "gfx950"; NULL (and an error message) if none. */
const char* moe_device_arch(void);

/* Identifies the sources this library was compiled from (no counterpart in the reference): sixteen hex digits of the
 * SHA-256 over the library's source files, as the build step computed it; "unknown" for a build that did not pass it.
 * Counter summaries of a kernel are tied to a build with it: a figure measured on other sources is not this library's. */
const char* moe_build_id(void);

/* Test aid (no counterpart in the reference): sets one of the process-wide tuning switches that are otherwise
 * read once from the MOE_* environment variables: "combine_pass", "rms_serial", "max_tokens_per_pass", "no_gemm",
 * "front_generic", "tile_slots", "slot_tiles", "narrow", "fused_rows", "front_split", "dispatch_one".  Not for use while forwards are in flight. */
int moe_debug_set_switch(const char* name, int64_t value);

/* Host restatement of the exp used by the device router (same source, compiled for the CPU), so
 * that its agreement with the platform's expf can be checked without a GPU. */
float moe_debug_expf(float x);

#ifdef __cplusplus
}
#endif
#endif
