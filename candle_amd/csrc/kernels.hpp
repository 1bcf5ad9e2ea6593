// Launchers of the gfx950 kernels (definitions in the kernels_*.hip files).
#pragma once
#include "moe_common.hpp"

namespace moe {

// Tuning and test switches of the whole process: read once from the MOE_* environment variables, changed afterwards
// only through moe_debug_set_switch.  Nothing on a forward's path reads the environment.
struct Switches {
    int combine_pass = 0;             // MOE_COMBINE_PASS: keep the combine pass for top-2 layers
    int rms_serial = 0;               // MOE_RMS_SERIAL: rms-norm sum of squares term by term
    int64_t max_tokens_per_pass = 0;  // MOE_MAX_TOKENS_PER_PASS: lower the per-pass token bound (0 = the real bound)
    int no_gemm = 0;                  // MOE_NO_GEMM: never take the tiled kernels
    int front_generic = 0;            // MOE_FRONT_GENERIC: generic front kernel
    int dispatch_one = 0;             // MOE_DISPATCH_ONE: the dispatch pass always as one workgroup
    int front_split = -1;             // MOE_FRONT_SPLIT: gate product as a kernel of its own ahead of routing: 0 | 1 (-1 = by shape)
    int tile_slots = 0;               // MOE_TILE_SLOTS: 64 | 128 (0 = by batch size)
    int slot_tiles = 0;               // MOE_SLOT_TILES: 16-slot tiles per streaming pass (0 = by batch size)
    int narrow = -1;                  // MOE_NARROW: 0 | 1 (-1 = by batch size)
    int fused_rows = 0;               // MOE_FUSED_ROWS: dense products of a few rows in one launch: 1 = never, 2 = whenever possible (0 = by size)
};
Switches& switches();

// Routing state of one forward call (all device pointers).  "Groups" are the E routed experts
// plus, when the layer has one, the always-on shared expert as group E.
struct RouteBufs {
    float* logits = nullptr;        // [T, E]
    int32_t* topk_idx = nullptr;    // [T, k] rank order
    float* topk_w = nullptr;        // [T, k]
    float* shared_w = nullptr;      // [T] sigmoid gate of the shared expert (or null)
    int32_t* offsets = nullptr;     // [G+1] slot ranges per group
    int32_t* perm_token = nullptr;  // [S] token row of every slot
    float* perm_w = nullptr;        // [S] routing weight of every slot
    int32_t* tok_slots = nullptr;   // [T, k(+1)] slots of a token, ascending expert index
    // Work list of the tiled (prefill) expert kernels, written by the dispatch kernel: [0] = number
    // of tiles of `tile_slots` slots, then (group, first position inside the group) per tile.  Built
    // from the real list lengths, so a skewed routing yields tiles in proportion to each expert's load.
    int32_t* tile_tab = nullptr;
    int32_t* wg_counts = nullptr;   // [DISPATCH_MAX_WGS][DISPATCH_COUNT_STRIDE] assignments per expert of each workgroup of a dispatch pass in two launches
    int tile_slots = 128;           // 128, or 64 when the lists are short
    // Slot numbering.  direct == 0: slots are grouped by expert (offsets / perm_* built by the
    // dispatch kernel).  direct == 1 (small batches): slot of assignment (token t, rank r) is
    // simply t*k + r, the shared expert's slots are T*k + t, and every consumer derives its
    // expert's ascending list from topk_idx itself -- no dispatch pass on the critical path.
    int direct = 0;
    int T = 0, k = 0;
};
constexpr int DISPATCH_MAX_WGS = 32;      // workgroups of a dispatch pass in two launches
constexpr int DISPATCH_COUNT_STRIDE = 256;  // ints per workgroup in wg_counts: the largest expert count
constexpr int DIRECT_MAX_SLOTS = 1024;  // largest T*k (and T) served without a dispatch pass
constexpr int GEMM_MIN_TILE_SLOTS = 64;  // smallest tile of the tiled expert kernels
inline int64_t max_gemm_tiles(int64_t slots, int64_t groups, int tile_slots = GEMM_MIN_TILE_SLOTS) { return slots / tile_slots + groups + 1; }

// Tiled kernels: workgroup id -> (row block, slot tile).  Hardware hands consecutive workgroup ids to the eight XCDs in
// turn, each with its own L2; the ids that land on one XCD are walked in patches of edge x edge (row blocks x tiles), so
// that the workgroups an XCD runs at a time share their weight rows and their activation tiles through that L2.  The
// edge is 8 when that still gives every XCD at least two patches, else 4 or 2: a grid of a few hundred workgroups cut
// into 8 x 8 patches would leave XCDs without work.
struct PatchPos { int rblk, tile; };
// `patch` = rows edge + 256 * tiles edge (a tiles edge of 0: a square patch)
__host__ __device__ inline PatchPos patch_position(int block, int n_rb, int patch) {
    const int er = patch & 255, et = (patch >> 8) ? (patch >> 8) : er;
    const int per = er * et, RG = (n_rb + er - 1) / er;
    const int xcd = block & 7, q = block >> 3;
    const int st = (q / per) * 8 + xcd, within = q % per;
    return PatchPos{(st % RG) * er + within % er, (st / RG) * et + within / er};
}
inline int patch_edge(int64_t n_rb, int64_t tiles) {
    for (int e = 8; e > 2; e >>= 1)
        if (((n_rb + e - 1) / e) * ((tiles + e - 1) / e) >= 16) return e;
    return 2;
}
// One group of a few tiles (the always-on expert, a dense product): a patch holds every tile of its row blocks, so that
// each weight row is fetched into one XCD's L2 only (square patches of 4 x 4 fetched the rows of eight tiles twice).
inline int patch_all_tiles(int64_t n_rb, int64_t tiles) {
    if (tiles < 1 || tiles > 16) return patch_edge(n_rb, tiles);
    int er = 4;
    while (er > 1 && (n_rb + er - 1) / er < 16) er >>= 1;
    return er + 256 * (int)tiles;
}
inline unsigned patch_grid(int64_t n_rb, int64_t tiles, int patch) {
    const int er = patch & 255, et = (patch >> 8) ? (patch >> 8) : er;
    const int64_t RG = (n_rb + er - 1) / er, TG = (tiles + et - 1) / et;
    return (unsigned)((RG * TG + 7) / 8 * 8 * er * et);
}

// The combine pass of the layer BEFORE this one, folded into this layer's front kernel (stacks of layers, small batches):
// the token's input row is  sum of that layer's weighted expert outputs in ascending expert order (+ that layer's
// input, its residual) -- the additions of combine_kernel in combine_kernel's order -- and is stored to x_out, where this
// layer's own residual is read from later.  Slots are numbered t * k + r (no dispatch pass ran in that layer).
struct PrevCombine {
    const float* yw = nullptr;          // [T * k, H] weighted expert outputs of the previous layer
    const int32_t* topk_idx = nullptr;  // [T, k] its routing
    int k = 0;
    const float* residual = nullptr;    // [T, H] its input, or null for a layer without the pre-norm
    float* x_out = nullptr;             // [T, H]
};

struct FrontParams {
    const float* x = nullptr;       // [T, H]
    int64_t T = 0;
    int H = 0, E = 0, k = 0, norm_topk = 1;
    const float* gate = nullptr;        // [E, H]
    const float* gate_bias = nullptr;   // [E] or null
    const float* shared_gate = nullptr; // [H] or null
    const float* rms_alpha = nullptr;   // [H] or null
    float rms_eps = 0.f;
    int rms_serial = 0;                 // 1: the fast kernel adds the squares of a row term by term (checks the chunked evaluation)
    int vdt = MOE_GGML_Q8K;             // activation format
    ActBuf xq;                          // token-indexed quantised activations (output)
    float* y_zero = nullptr;            // [T, H] or null: rows the kernel clears for the down kernels to accumulate into
    RouteBufs rb;
    PrevCombine prev;                   // fast kernel only (front_takes_prev_combine): x is not read then
};
// whether launch_front will take the kernel that can fold the previous layer's combine pass in
bool front_takes_prev_combine(const FrontParams& p);
// rms-norm (optional) + gate product + softmax + top-k + activation quantisation per token.
hipError_t launch_front(const FrontParams& p, hipStream_t s);
// The front end of a layer whose router stays quantised: logits from the dense product's padded rows, then routing and
// activation quantisation from rb.logits.
hipError_t launch_logits_unpad(const float* padded, int n_pad, const float* bias, float* logits, int64_t T, int E, hipStream_t s);
hipError_t launch_front_route(const FrontParams& p, hipStream_t s);
// softmax + top-k from given logits (parity hook).
hipError_t launch_route_from_logits(const float* logits, int64_t T, int E, int k, int norm_topk,
                                    const RouteBufs& rb, hipStream_t s);
// Per-expert lists from topk_idx / topk_w: histogram, prefix scan, stable permutation (one workgroup).
hipError_t launch_dispatch(const RouteBufs& rb, int64_t T, int E, int k, bool shared, hipStream_t s);

struct GroupWeights {
    const uint8_t* w1;
    const uint8_t* w3;
    const uint8_t* w2;
};

struct ExpertParams {
    int dt = 0;                     // dtype of w1 / w3
    int dt_down = 0;                // dtype of w2 when it differs from dt (same activation format), else 0
    int H = 0, F = 0;
    int n_groups = 0;               // groups handled by this launch
    int group0 = 0;                 // index of the first of them in rb.offsets
    const GroupWeights* groups = nullptr;  // device array [n_groups]
    RouteBufs rb;
    ActBuf xq;                      // token-indexed, K = H
    ActBuf hq;                      // slot-indexed (row = slot - slot_origin), K = F
    int slot_origin = 0;
    float* yw = nullptr;            // [S, H] weighted expert outputs, slot-indexed (absolute)
    float* y_acc = nullptr;         // when set: the down kernels add their weighted outputs to y_acc[token, :] (zeroed by the
                                    // front kernel) instead of storing yw, and no combine pass runs
    int64_t max_rows = 0;           // upper bound of rows in any group of this launch
    int slot_tiles = 1;             // 16-slot tiles a workgroup carries per pass over the weights (1, 2 or, Q4K only, 4)
    int is_shared = 0;              // this launch is the always-on shared expert (one group, all tokens)
    int patch = 8;                  // tiled kernels: edge of the (row block x tile) patches dealt to the XCDs (set by the launchers)
    // Narrow launches of tiny batches (direct slot numbering, T*k <= E): the grid's y dimension counts assignments
    // instead of experts, workgroup row y serves the expert of assignment y unless an earlier assignment names the
    // same expert.  No workgroups (and no weight prefetches) for experts without tokens.
    int by_assignment = 0;
    int down_interleaved = 0;   // down projection: wave w of a workgroup takes super-blocks w, w + NW, ... instead of a contiguous range
    float* hbuf = nullptr;          // tiled path only: f32 intermediate [slots, F] before re-quantisation
    int64_t n_slots = 0;            // tiled path only: total slots (bounds the tile grid)
};
// h = silu(W1 x) * (W3 x), quantised to the activation format, for every slot of every group.
hipError_t launch_expert_up(const ExpertParams& p, hipStream_t s);
// yw[slot] = (W2 h[slot]) * perm_w[slot]
hipError_t launch_expert_down(const ExpertParams& p, hipStream_t s);

// Tiled (prefill) variants for Q4K in dispatched mode: activations staged through LDS, weights
// unpacked and pre-scaled per wave, v_mfma_i32_32x32x32_i8.  up writes f32 h into p.hbuf (the
// caller re-quantises it), down writes yw.
bool q4k_gemm_up_format(int dt);
bool q4k_gemm_down_format(int dt);
// Dense matrix [n, k] (device layout) times m <= 4 rows of f32 in one launch (the rows are quantised in the kernel).
struct FusedRows {
    const float* x = nullptr;          // [m, k] rows ...
    const float* x2 = nullptr;         // ... optionally times the rows x2 (the two halves of a SwiGLU intermediate in f32)
    ActBuf xq;                         // x == nullptr: the rows, already quantised to the matrix format's activation type
    int64_t m = 0, n = 0, k = 0;
    const uint8_t* w = nullptr;        // the matrix
    float* y = nullptr;                // [m, n]
    const uint8_t* w_b = nullptr;      // optional second matrix of the same shape against the same rows ...
    float* y_b = nullptr;              // ... and its output
    const float* row_scale = nullptr;  // optional: row r of y is multiplied by row_scale[r]
    int silu_y = 0;                    // y = silu(w x) (y_b stays w_b x)
};
// K-quant matrices:
bool qlinear_fused_usable(int dt, int64_t m, int64_t n, int64_t k);
hipError_t launch_qlinear_fused(int dt, const FusedRows& f, hipStream_t s);
// The 32-element formats (super-tile layout): bit-identical to the streaming kernel's results.
bool q32_rows_fused_usable(int dt, int64_t m, int64_t n, int64_t k);
hipError_t launch_q32_rows_fused(int dt, const FusedRows& f, hipStream_t s);
hipError_t launch_q4k_gemm_up(const ExpertParams& p, hipStream_t s);
hipError_t launch_q4k_gemm_down(const ExpertParams& p, hipStream_t s);

// Tiled products for Q8_0 layers whose slots are grouped by expert (tiles of 64 slots, rb.tile_slots == 64; F a multiple
// of 128 for the reduction of w2 and of 64 for the row blocks of w1 / w3, H a multiple of 128): up quantises the
// intermediate into p.hq in its epilogue, down writes yw.  With p.is_shared the launch covers the always-on expert
// (one group of p.max_rows tokens) and needs no tile list.
bool q8_0_gemm_usable(int dt, int dt_down, int64_t H, int64_t F);
hipError_t launch_q8_0_gemm_up(const ExpertParams& p, hipStream_t s);
hipError_t launch_q8_0_gemm_down(const ExpertParams& p, hipStream_t s);

// y[t] = sum over the token's slots (ascending expert index, shared expert last) of yw[slot] (+ residual[t]).
hipError_t launch_combine(const float* yw, const RouteBufs& rb, bool shared, const float* residual, float* y,
                          int64_t T, int H, hipStream_t s);

// y[i] = src ? src[i] : 0 for n floats (n % 4 == 0): the output of a layer that selects no expert.
hipError_t launch_fill_or_copy(const float* src, float* y, int64_t n, hipStream_t s);
// RmsNorm::forward (candle-nn/src/ops.rs:504-515) on rows of `hidden` floats: v = x (+ residual, stored to sum when
// given), y = v / sqrt(sum(v^2) / hidden + eps) * alpha, the squares summed left to right as the reference does.
hipError_t launch_add_rms_norm(const float* x, const float* residual, const float* alpha, float eps, int64_t rows, int hidden,
                               float* sum, float* y, hipStream_t s);

// Re-lay raw GGML blocks [rows, k] (device, standard layout) into the tiled device layout.
hipError_t launch_relayout(int dt, const uint8_t* raw, uint8_t* tiled, int64_t rows, int64_t k, hipStream_t s);
// to_float from the tiled layout back to row-major f32 (layout check).
hipError_t launch_dequant_tiled(int dt, const uint8_t* tiled, float* out, int64_t rows, int64_t k, hipStream_t s);
// to_float on standard blocks.
hipError_t launch_dequant_std(int dt, const uint8_t* blocks, float* out, int64_t n, hipStream_t s);
// Activation quantiser on plain rows [rows, k] into an ActBuf (same device code the front kernel uses).
hipError_t launch_quantize_rows(int vdt, const float* x, int64_t rows, int k, const ActBuf& out, hipStream_t s);
// ActBuf -> standard BlockQ8K / BlockQ8_0 bytes.
hipError_t launch_actbuf_to_std(int vdt, const ActBuf& in, int64_t rows, int k, uint8_t* out, hipStream_t s);
// Identity routing for a dense product over `rows` rows: one group, slot i = row i, weight 1.
hipError_t launch_identity_routing(const RouteBufs& rb, int64_t rows, hipStream_t s);

// QTensor::quantize on the GPU: f32 [n] (device) -> standard GGML blocks (device).
hipError_t launch_quantize_weights(int dt, const float* x, int64_t n, uint8_t* out, hipStream_t s);

// bytes of the ActBuf members for `rows` rows of length k
inline size_t act_qs_bytes(int64_t rows, int64_t k) { return (size_t)rows * k; }
inline size_t act_d_bytes(int vdt, int64_t rows, int64_t k) { return (size_t)rows * (k / block_elems(vdt)) * 4; }
inline size_t act_bsum_bytes(int vdt, int64_t rows, int64_t k) {
    return vdt == MOE_GGML_Q8K ? (size_t)rows * (k / 256) * 16 * 2 : (size_t)rows * (k / 32) * 4;
}

}  // namespace moe
