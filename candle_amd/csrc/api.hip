// C ABI of the library (see include/candle_amd_moe.h): layer objects, device memory and the
// sequence of kernel launches of one forward pass.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <vector>

#include "kernels.hpp"

namespace moe {

static thread_local std::string g_err;
void set_error(int, const std::string& msg) { g_err = msg; }
int fail(int code, const std::string& msg) {
    g_err = msg;
    return code;
}

static std::once_flag g_dev_once;
static int g_dev_rc = MOE_E_NODEVICE;
static std::string g_dev_msg, g_arch;

int ensure_device() {
    std::call_once(g_dev_once, [] {
        int n = 0;
        hipError_t e = hipGetDeviceCount(&n);
        if (e != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            g_dev_msg = std::string("no HIP device visible (") + (e != hipSuccess ? hipGetErrorString(e) : "device count 0") +
                        "); this library has no CPU fallback";
            g_dev_rc = MOE_E_NODEVICE;
            return;
        }
        int dev = 0;
        (void)hipGetDevice(&dev);
        hipDeviceProp_t prop;
        e = hipGetDeviceProperties(&prop, dev);
        if (e != hipSuccess) {
            g_dev_msg = std::string("hipGetDeviceProperties: ") + hipGetErrorString(e);
            g_dev_rc = MOE_E_HIP;
            return;
        }
        g_arch = prop.gcnArchName;
        if (g_arch.rfind("gfx950", 0) != 0) {
            g_dev_msg = "device architecture is " + g_arch + "; the kernels are built for gfx950 only";
            g_dev_rc = MOE_E_NODEVICE;
            return;
        }
        g_dev_rc = MOE_OK;
    });
    if (g_dev_rc != MOE_OK) g_err = g_dev_msg;
    return g_dev_rc;
}

// ------------------------------------------------------------------ device buffers
struct DevBuf {
    void* p = nullptr;
    size_t cap = 0;
    ~DevBuf() {
        if (p) (void)hipFree(p);
    }
    DevBuf() = default;
    DevBuf(const DevBuf&) = delete;
    DevBuf& operator=(const DevBuf&) = delete;
    int reserve(size_t bytes) {
        if (bytes <= cap) return MOE_OK;
        if (p) MOE_HIP_CHECK(hipFree(p));
        p = nullptr;
        cap = 0;
        size_t want = std::max<size_t>(bytes, 256);
        hipError_t e = hipMalloc(&p, want);
        if (e != hipSuccess) {
            p = nullptr;
            return fail(MOE_E_NOMEM, std::string("hipMalloc(") + std::to_string(want) + "): " + hipGetErrorString(e));
        }
        cap = want;
        return MOE_OK;
    }
    template <typename T>
    T* as() const { return reinterpret_cast<T*>(p); }
};

struct ActStore {
    DevBuf qs, d, bsum;
    int reserve(int vdt, int64_t rows, int64_t k) {
        int rc;
        if ((rc = qs.reserve(act_qs_bytes(rows, k)))) return rc;
        if ((rc = d.reserve(act_d_bytes(vdt, rows, k)))) return rc;
        return bsum.reserve(act_bsum_bytes(vdt, rows, k));
    }
    ActBuf view() const {
        ActBuf a;
        a.qs = qs.as<int8_t>();
        a.d = d.as<float>();
        a.bsum = bsum.p;
        return a;
    }
};

struct RouteStore {
    DevBuf logits, topk_idx, topk_w, shared_w, offsets, perm_token, perm_w, tok_slots, tile_tab, wg_counts;
    int reserve(int64_t T, int E, int k, bool shared) {
        int rc;
        const int64_t S = T * k + (shared ? T : 0);
        if ((rc = logits.reserve((size_t)T * E * 4))) return rc;
        if ((rc = topk_idx.reserve((size_t)T * k * 4))) return rc;
        if ((rc = topk_w.reserve((size_t)T * k * 4))) return rc;
        if ((rc = shared_w.reserve((size_t)T * 4))) return rc;
        if ((rc = offsets.reserve((size_t)(E + 2) * 4))) return rc;
        if ((rc = perm_token.reserve((size_t)S * 4))) return rc;
        if ((rc = perm_w.reserve((size_t)S * 4))) return rc;
        if ((rc = tok_slots.reserve((size_t)T * (k + 1) * 4))) return rc;
        if ((rc = tile_tab.reserve((size_t)(1 + 2 * max_gemm_tiles(S, E + 1)) * 4))) return rc;
        if ((rc = wg_counts.reserve((size_t)DISPATCH_MAX_WGS * DISPATCH_COUNT_STRIDE * 4))) return rc;
        return MOE_OK;
    }
    RouteBufs view() const {
        RouteBufs r;
        r.logits = logits.as<float>();
        r.topk_idx = topk_idx.as<int32_t>();
        r.topk_w = topk_w.as<float>();
        r.shared_w = shared_w.as<float>();
        r.offsets = offsets.as<int32_t>();
        r.perm_token = perm_token.as<int32_t>();
        r.perm_w = perm_w.as<float>();
        r.tok_slots = tok_slots.as<int32_t>();
        r.tile_tab = tile_tab.as<int32_t>();
        r.wg_counts = wg_counts.as<int32_t>();
        return r;
    }
};

// A call's device workspace as one stretch of memory cut into 256-byte aligned pieces.  With base == nullptr the
// cuts only measure: `off` ends up as the number of bytes the same cuts need.
struct Carver {
    uint8_t* base = nullptr;
    size_t off = 0;
    template <typename T>
    T* take(size_t bytes) {
        const size_t at = (off + 255) & ~(size_t)255;
        off = at + bytes;
        return base ? reinterpret_cast<T*>(base + at) : nullptr;
    }
    ActBuf take_act(int vdt, int64_t rows, int64_t k) {
        ActBuf a;
        a.qs = take<int8_t>(act_qs_bytes(rows, k));
        a.d = take<float>(act_d_bytes(vdt, rows, k));
        a.bsum = take<uint8_t>(act_bsum_bytes(vdt, rows, k));
        return a;
    }
    RouteBufs take_route(int64_t T, int E, int k, bool shared, bool tile_tab) {
        RouteBufs r;
        const int64_t S = T * k + (shared ? T : 0);
        r.logits = take<float>((size_t)T * E * 4);
        r.topk_idx = take<int32_t>((size_t)T * k * 4);
        r.topk_w = take<float>((size_t)T * k * 4);
        r.shared_w = take<float>((size_t)T * 4);
        r.offsets = take<int32_t>((size_t)(E + 2) * 4);
        r.perm_token = take<int32_t>((size_t)S * 4);
        r.perm_w = take<float>((size_t)S * 4);
        r.tok_slots = take<int32_t>((size_t)T * (k + 1) * 4);
        r.tile_tab = tile_tab ? take<int32_t>((size_t)(1 + 2 * max_gemm_tiles(S, E + 1)) * 4) : nullptr;
        if (T * k > 16384) r.wg_counts = take<int32_t>((size_t)DISPATCH_MAX_WGS * DISPATCH_COUNT_STRIDE * 4);
        return r;
    }
};

// A workspace that graph captures may have baked into their nodes: once `captured` is set, growing it keeps the old
// memory alive until the owner goes (a replay of the capture still reads and writes it).
struct GrowBuf {
    void* p = nullptr;
    size_t cap = 0;
    bool captured = false;
    std::vector<void*> retired;
    GrowBuf() = default;
    GrowBuf(const GrowBuf&) = delete;
    GrowBuf& operator=(const GrowBuf&) = delete;
    ~GrowBuf() {
        if (p) (void)hipFree(p);
        for (void* q : retired) (void)hipFree(q);
    }
    int reserve(size_t bytes) {
        if (bytes <= cap) return MOE_OK;
        void* fresh = nullptr;
        const size_t want = std::max<size_t>(bytes, 256);
        hipError_t e = hipMalloc(&fresh, want);
        if (e != hipSuccess) return fail(MOE_E_NOMEM, std::string("hipMalloc(") + std::to_string(want) + "): " + hipGetErrorString(e));
        if (p) {
            if (captured) retired.push_back(p);
            else MOE_HIP_CHECK(hipFree(p));   // waits for the work that still uses it
        }
        p = fresh;
        cap = want;
        return MOE_OK;
    }
};

// Calls on one object share its workspace, so a call must not start before the previous one has finished.  On one
// stream the stream's own order sees to that; the event is recorded (on the previous call's stream) only when a call
// arrives on another stream or the host wants the results: an event record between every two calls costs a 5.6 us
// bubble per step.
struct CallOrder {
    hipEvent_t done = nullptr;
    hipStream_t last_stream = nullptr;
    bool pending = false;           // work enqueued on last_stream that `done` does not cover yet
    int init() {
        MOE_HIP_CHECK(hipEventCreateWithFlags(&done, hipEventDisableTiming));
        return MOE_OK;
    }
    void destroy() {
        if (done) (void)hipEventDestroy(done);
        done = nullptr;
    }
    // Marks the end of everything enqueued so far in `done`.  If the stream of the last call has gone (the caller
    // destroyed it; its work completes all the same) the device is synchronised instead.
    int close() {
        if (!pending) return MOE_OK;
        if (hipEventRecord(done, last_stream) != hipSuccess) {
            (void)hipGetLastError();
            MOE_HIP_CHECK(hipDeviceSynchronize());
            MOE_HIP_CHECK(hipEventRecord(done, nullptr));
        }
        pending = false;
        return MOE_OK;
    }
    // before the first launch of an eager call on stream s
    int enter(hipStream_t s) {
        if (pending && last_stream == s) return MOE_OK;
        if (int rc = close()) return rc;
        MOE_HIP_CHECK(hipStreamWaitEvent(s, done, 0));
        return MOE_OK;
    }
    void leave(hipStream_t s) { last_stream = s; pending = true; }
    // host side: wait for everything enqueued so far
    int wait() {
        if (int rc = close()) return rc;
        MOE_HIP_CHECK(hipEventSynchronize(done));
        return MOE_OK;
    }
};

// ------------------------------------------------------------------ tuning / test switches
static std::once_flag g_sw_once;
static Switches g_sw;
Switches& switches() {
    std::call_once(g_sw_once, [] {
        auto num = [](const char* name, long long dflt) {
            const char* e = getenv(name);
            return e ? atoll(e) : dflt;
        };
        g_sw.combine_pass = getenv("MOE_COMBINE_PASS") != nullptr;
        g_sw.rms_serial = getenv("MOE_RMS_SERIAL") != nullptr;
        g_sw.max_tokens_per_pass = num("MOE_MAX_TOKENS_PER_PASS", 0);
        g_sw.no_gemm = getenv("MOE_NO_GEMM") != nullptr;
        g_sw.front_generic = getenv("MOE_FRONT_GENERIC") != nullptr;
        g_sw.front_split = (int)num("MOE_FRONT_SPLIT", -1);
        g_sw.dispatch_one = (int)num("MOE_DISPATCH_ONE", 0);
        g_sw.tile_slots = (int)num("MOE_TILE_SLOTS", 0);
        g_sw.slot_tiles = (int)num("MOE_SLOT_TILES", 0);
        g_sw.narrow = (int)num("MOE_NARROW", -1);
        g_sw.fused_rows = (int)num("MOE_FUSED_ROWS", 0);
    });
    return g_sw;
}

}  // namespace moe

using namespace moe;

struct moe_qlinear;
static int enqueue_qlinear(moe_qlinear* Q, const float* d_x, int64_t m, float* d_y, hipStream_t s);

// The pieces of one forward's workspace (device pointers).
struct Workspace {
    RouteBufs rb;
    ActBuf xq, hq, hq_shared;
    float* yw = nullptr;
    float* hbuf = nullptr;
    float* ab_shared = nullptr;   // [2][T][Fs]: silu(w1 x) and w3 x of the always-on expert at a few tokens
    float* xin = nullptr;         // stacks: the layer's input row [T][H] when the layer before leaves its combine pass to this one
    float* xn = nullptr;          // quantised router, layers with the pre-norm: the normed rows [T][H]
    float* logits_pad = nullptr;  // quantised router: the dense product's rows [T][E rounded up to 16]
};

// Which kernels a forward of T tokens takes.
struct ForwardPlan {
    bool tiled = false, tiled_down = false, tiled32 = false, direct = false, accumulate = false, narrow = false, hbuf = false;
    bool shared_rows = false;   // the always-on expert as two dense few-row products
    int tile_slots = 128, slot_tiles = 1;
};

struct moe_layer {
    int64_t H = 0, F = 0, E = 0, k = 0, Fs = 0;
    int dt = 0, dt_down = 0, vdt = 0, norm_topk = 1;   // dt: w1 / w3, dt_down: w2 (same activation format)
    bool has_bias = false, has_rms = false;
    float rms_eps = 0.f;
    DevBuf weights;                 // all re-laid expert matrices
    DevBuf gate, gate_bias, shared_gate, rms_alpha, groups;
    // a router tensor kept quantised (moe_desc.gate_dtype): the [E, H] blocks as a dense projection of E16 = E rounded up
    // to the layout's 16-row tiles (the extra rows are zero blocks), applied to the rows the experts see
    moe_qlinear* gate_q = nullptr;
    int64_t E16 = 0;
    std::vector<GroupWeights> host_groups;  // E routed (+1 shared)
    std::mutex mu;
    GrowBuf ws;                     // per-call workspace, grown on demand, cut anew for every call
    DevBuf x_dev, y_dev;            // staging of the host-pointer entry
    hipStream_t stream = nullptr;   // used by the host-pointer entry
    // layers with a shared expert: its two kernels run on this stream beside the routed experts' (fork after the front
    // kernels, join before the combine pass); nothing but the workspace pieces of its own is shared with them
    hipStream_t side = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    CallOrder order;
    int64_t last_T = 0;             // -1: several passes, -2: a layer with top_k = 0 routes nothing
    bool last_direct = false;       // the last forward skipped the dispatch pass
    Workspace last_ws;              // where the last forward left its logits and routing
};

static int check_desc(const moe_desc* d) {
    if (!d) return fail(MOE_E_INVALID, "desc is NULL");
    const int dt = d->ggml_dtype, dtd = d->ggml_dtype_down ? d->ggml_dtype_down : dt;
    if (!weight_dtype_supported(dt) || !weight_dtype_supported(dtd))
        return fail(MOE_E_INVALID, "unsupported ggml_dtype " + std::to_string(weight_dtype_supported(dt) ? dtd : dt) +
                                       " (supported: Q4_0=2, Q4_1=3, Q5_0=6, Q5_1=7, Q8_0=8, Q2K=10, Q3K=11, Q4K=12, Q5K=13, Q6K=14)");
    // w2 consumes the intermediate in the activation format of its own dtype; the up kernels emit the one of dt
    if (vecdot_dtype(dt) != vecdot_dtype(dtd))
        return fail(MOE_E_INVALID, "ggml_dtype " + std::to_string(dt) + " and ggml_dtype_down " + std::to_string(dtd) +
                                       " quantise activations differently (Q8_0, Q8_1 or Q8K); such a layer is not supported");
    const int64_t be = block_elems(dt);
    if (d->hidden <= 0 || d->ffn <= 0) return fail(MOE_E_INVALID, "hidden and ffn must be positive");
    // the reference rejects a last dimension that is not a multiple of the block size
    // (candle-core/src/quantized/mod.rs:310-322)
    if (d->hidden % be || d->ffn % be)
        return fail(MOE_E_INVALID, "hidden and ffn must be multiples of the block size " + std::to_string(be));
    if (d->hidden % 16 || d->ffn % 32) return fail(MOE_E_INVALID, "hidden must be a multiple of 16 and ffn of 32");
    if (d->hidden > 16384) return fail(MOE_E_INVALID, "hidden > 16384 is not supported");
    if (d->n_experts < 1 || d->n_experts > 256) return fail(MOE_E_INVALID, "n_experts must be in 1..256");
    // top_k = 0 is what the reference runs with when the file lacks llama.expert_used_count (quantized_llama.rs:507-512
    // defaults the key to 0): `take(0)` at :167 selects nothing and the block returns zeros
    if (d->top_k < 0 || d->top_k > d->n_experts || d->top_k > 16)
        return fail(MOE_E_INVALID, "top_k must be in 0..min(n_experts,16)");
    if (d->top_k == 0 && d->shared_ffn > 0) return fail(MOE_E_INVALID, "top_k = 0 with a shared expert is not supported");
    if ((!d->gate && !d->gate_dtype) || !d->w1 || !d->w2 || !d->w3) return fail(MOE_E_INVALID, "gate, w1, w2, w3 must be set");
    if (d->gate_dtype) {
        if (!weight_dtype_supported(d->gate_dtype)) return fail(MOE_E_INVALID, "unsupported gate_dtype " + std::to_string(d->gate_dtype));
        if (!d->gate_blocks) return fail(MOE_E_INVALID, "gate_dtype is set but gate_blocks is NULL");
        if (d->hidden % 256) return fail(MOE_E_INVALID, "a quantised router needs hidden to be a multiple of 256");
        if (d->shared_ffn > 0) return fail(MOE_E_INVALID, "a quantised router together with a shared expert is not supported");
    }
    for (int64_t e = 0; e < d->n_experts; e++)
        if (!d->w1[e] || !d->w2[e] || !d->w3[e]) return fail(MOE_E_INVALID, "expert " + std::to_string(e) + " has a NULL matrix");
    if (d->shared_ffn < 0) return fail(MOE_E_INVALID, "shared_ffn < 0");
    if (d->shared_ffn > 0) {
        if (d->shared_ffn % be || d->shared_ffn % 32) return fail(MOE_E_INVALID, "shared_ffn must be a multiple of the block size and of 32");
        if (!d->shared_w1 || !d->shared_w2 || !d->shared_w3 || !d->shared_gate)
            return fail(MOE_E_INVALID, "shared expert needs shared_w1, shared_w2, shared_w3 and shared_gate");
    }
    return MOE_OK;
}

static int upload_f32(DevBuf& b, const float* src, size_t n) {
    int rc = b.reserve(n * 4);
    if (rc) return rc;
    MOE_HIP_CHECK(hipMemcpy(b.p, src, n * 4, hipMemcpyHostToDevice));
    return MOE_OK;
}

extern "C" int moe_layer_create(const moe_desc* d, moe_layer** out) {
    if (!out) return fail(MOE_E_INVALID, "out is NULL");
    *out = nullptr;
    int rc = ensure_device();
    if (rc) return rc;
    if ((rc = check_desc(d))) return rc;
    moe_layer* L = new moe_layer();
    auto bail = [&](int code) {
        moe_layer_destroy(L);
        return code;
    };
    L->H = d->hidden; L->F = d->ffn; L->E = d->n_experts; L->k = d->top_k; L->Fs = d->shared_ffn;
    L->dt = d->ggml_dtype; L->dt_down = d->ggml_dtype_down ? d->ggml_dtype_down : L->dt;
    L->vdt = vecdot_dtype(L->dt); L->norm_topk = d->norm_topk ? 1 : 0;
    L->rms_eps = d->rms_eps;
    if (d->gate_dtype) {
        // QMatMul::QTensor arm (quantized/mod.rs:428-447, 533-537): the blocks stay as they are, padded with zero blocks
        // (every format reads all-zero bytes as zeros) to the 16-row tiles of the dense projections
        L->E16 = (L->E + 15) / 16 * 16;
        const size_t row_bytes = (size_t)(L->H / block_elems(d->gate_dtype) * block_bytes(d->gate_dtype));
        std::vector<uint8_t> padded((size_t)L->E16 * row_bytes, 0);
        memcpy(padded.data(), d->gate_blocks, (size_t)L->E * row_bytes);
        if ((rc = moe_qlinear_create(d->gate_dtype, padded.data(), L->E16, L->H, &L->gate_q))) return bail(rc);
    } else if ((rc = upload_f32(L->gate, d->gate, (size_t)L->E * L->H))) return bail(rc);
    if (d->gate_bias) {
        L->has_bias = true;
        if ((rc = upload_f32(L->gate_bias, d->gate_bias, (size_t)L->E))) return bail(rc);
    }
    if (L->Fs > 0 && (rc = upload_f32(L->shared_gate, d->shared_gate, (size_t)L->H))) return bail(rc);
    if (d->rms_alpha) {
        L->has_rms = true;
        if ((rc = upload_f32(L->rms_alpha, d->rms_alpha, (size_t)L->H))) return bail(rc);
    }
    // one allocation for all matrices
    auto raw_bytes_of = [](int dt, int64_t elems) { return (size_t)(elems / block_elems(dt) * block_bytes(dt)); };
    const size_t total = (size_t)(2 * relaid_bytes(L->dt, L->F, L->H) + relaid_bytes(L->dt_down, L->H, L->F)) * L->E +
                         (L->Fs ? (size_t)(2 * relaid_bytes(L->dt, L->Fs, L->H) + relaid_bytes(L->dt_down, L->H, L->Fs)) : 0);
    if ((rc = L->weights.reserve(total))) return bail(rc);
    const size_t raw_mat = raw_bytes_of(L->dt, L->F * L->H), raw_mat_down = raw_bytes_of(L->dt_down, L->F * L->H);
    const size_t raw_smat = raw_bytes_of(L->dt, L->Fs * L->H), raw_smat_down = raw_bytes_of(L->dt_down, L->Fs * L->H);
    DevBuf staging;
    if ((rc = staging.reserve(std::max(std::max(raw_mat, raw_smat), std::max(raw_mat_down, raw_smat_down))))) return bail(rc);
    uint8_t* wbase = L->weights.as<uint8_t>();
    size_t off = 0;
    auto put = [&](int dt, const void* src, size_t raw_bytes, int64_t rows, int64_t cols, const uint8_t** dst) -> int {
        hipError_t e = hipMemcpy(staging.p, src, raw_bytes, hipMemcpyHostToDevice);
        if (e != hipSuccess) return fail(MOE_E_HIP, std::string("hipMemcpy(weights): ") + hipGetErrorString(e));
        e = launch_relayout(dt, staging.as<uint8_t>(), wbase + off, rows, cols, nullptr);
        if (e == hipSuccess) e = hipDeviceSynchronize();
        if (e != hipSuccess) return fail(MOE_E_HIP, std::string("relayout: ") + hipGetErrorString(e));
        *dst = wbase + off;
        off += (size_t)relaid_bytes(dt, rows, cols);
        return MOE_OK;
    };
    L->host_groups.resize(L->E + (L->Fs ? 1 : 0));
    for (int64_t e = 0; e < L->E; e++) {
        GroupWeights& g = L->host_groups[e];
        if ((rc = put(L->dt, d->w1[e], raw_mat, L->F, L->H, &g.w1))) return bail(rc);
        if ((rc = put(L->dt, d->w3[e], raw_mat, L->F, L->H, &g.w3))) return bail(rc);
        if ((rc = put(L->dt_down, d->w2[e], raw_mat_down, L->H, L->F, &g.w2))) return bail(rc);
    }
    if (L->Fs) {
        GroupWeights& g = L->host_groups[L->E];
        if ((rc = put(L->dt, d->shared_w1, raw_smat, L->Fs, L->H, &g.w1))) return bail(rc);
        if ((rc = put(L->dt, d->shared_w3, raw_smat, L->Fs, L->H, &g.w3))) return bail(rc);
        if ((rc = put(L->dt_down, d->shared_w2, raw_smat_down, L->H, L->Fs, &g.w2))) return bail(rc);
    }
    if ((rc = L->groups.reserve(L->host_groups.size() * sizeof(GroupWeights)))) return bail(rc);
    hipError_t e = hipMemcpy(L->groups.p, L->host_groups.data(), L->host_groups.size() * sizeof(GroupWeights), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&L->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        fail(MOE_E_HIP, std::string("layer setup: ") + hipGetErrorString(e));
        return bail(MOE_E_HIP);
    }
    if ((rc = L->order.init())) return bail(rc);
    if (L->Fs > 0) {
        e = hipStreamCreateWithFlags(&L->side, hipStreamNonBlocking);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&L->fork, hipEventDisableTiming);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&L->join, hipEventDisableTiming);
        if (e != hipSuccess) {
            fail(MOE_E_HIP, std::string("layer setup: ") + hipGetErrorString(e));
            return bail(MOE_E_HIP);
        }
    }
    *out = L;
    return MOE_OK;
}

extern "C" void moe_layer_destroy(moe_layer* L) {
    if (!L) return;
    (void)hipDeviceSynchronize();
    if (L->gate_q) moe_qlinear_destroy(L->gate_q);
    if (L->stream) (void)hipStreamDestroy(L->stream);
    if (L->side) (void)hipStreamDestroy(L->side);
    if (L->fork) (void)hipEventDestroy(L->fork);
    if (L->join) (void)hipEventDestroy(L->join);
    L->order.destroy();
    delete L;
}

// Stage marks for moe_layer_forward_timed: events recorded between the launches.
enum { ST_BEGIN = 0, ST_FRONT, ST_DISPATCH, ST_UP, ST_REQUANT, ST_DOWN, ST_SHARED, ST_COMBINE, ST_COUNT };

// The expert kernels address quantised activation rows with 32-bit byte offsets (rows * K): a call carries
// at most this many tokens; longer inputs are cut into chunks (tokens are independent of each other).
static int64_t max_tokens_per_pass(const moe_layer* L) {
    const int64_t widest = std::max(std::max(L->H, L->F), L->Fs);
    int64_t limit = std::max<int64_t>(1, (((int64_t)1 << 31) - 1) / (std::max<int64_t>(L->k, 1) * widest));
    const int64_t forced = switches().max_tokens_per_pass;   // testing aid: force several passes on small inputs
    if (forced > 0) limit = std::min(limit, forced);
    return limit;
}

static ForwardPlan plan_forward(const moe_layer* L, int64_t T) {
    const Switches& sw = switches();
    ForwardPlan pl;
    const bool shared = L->Fs > 0;
    // K-quant batches with more than 34 rows per expert take the tiled MFMA kernel for the up projection (F a
    // multiple of 64, H of 128; those kernels address activation rows with 32-bit byte offsets), from ~64 rows per
    // expert on for the down projection too (measured at the Mixtral shape: 36 rows per expert, 316 against 326 us per
    // step, 32 rows 310 against 296; 48 rows per expert, up 198 us tiled
    // against 230 us streamed with four slot tiles, down 170 against 120 us; 64 rows: down 177 against 170).
    // Their tiles hold 64 slots while the lists are short (less padding), 128 beyond ~72 rows per expert (Mixtral shape:
    // 64 rows per expert 449 against 485 us per step, 80 rows 531 against 498).
    // (w2 may be Q4K, Q5K or Q6K whatever w1 / w3 are: mixed files store part of it as Q6K)
    pl.tiled = !sw.no_gemm && q4k_gemm_up_format(L->dt) && L->F % 64 == 0 && L->H % 128 == 0 && T * L->k > 34 * L->E;
    pl.tiled_down = pl.tiled && q4k_gemm_down_format(L->dt_down) && T * L->k > 64 * L->E;
    // 16-slot tiles a workgroup carries per pass over the weights, from the expected rows per expert
    // (a list longer than a pass covers is finished by further workgroups that stream the weights again)
    // (measured at the Mixtral shape: two tiles per pass, with a second pass for the longer lists, beat four
    // tiles per pass up to ~34 rows per expert)
    // (the 32-element kernels carry at most two tiles: three or four per pass measured slower at the Mixtral shape and
    // 8 % faster at best where sixty small experts' weights exceed the caches)
    // (K-quants, Mixtral shape: one tile with a second pass for the lists beyond 16 rows beats two tiles up to ~13 rows per
    // expert on average: 48 tokens 168 against 181 us per step, 64 tokens 214 against 185)
    const int64_t two_from = (L->vdt == MOE_GGML_Q8K ? 13 : 9) * L->E;
    pl.slot_tiles = (T * L->k > 34 * L->E) ? 4 : (T * L->k > two_from) ? 2 : 1;
    if (sw.slot_tiles) pl.slot_tiles = sw.slot_tiles;
    // small batches: slots are numbered t*k + r and no dispatch pass runs; every workgroup then finds its expert's slots
    // by scanning the assignments, and the grid holds a pass for every 16 * slot_tiles tokens there could be in a list.
    // With many experts most of those passes are empty: beyond four of them the dispatch pass is worth its 5 us (its
    // lists let an empty pass leave at once; 128 experts, 512 tokens: 386 -> 303 us).
    const int64_t passes = (T + 16 * pl.slot_tiles - 1) / (16 * pl.slot_tiles);
    pl.direct = !pl.tiled && T * L->k <= DIRECT_MAX_SLOTS && T <= DIRECT_MAX_SLOTS && (passes <= 4 || L->E <= 16);
    pl.tile_slots = sw.tile_slots == 64 || sw.tile_slots == 128 ? sw.tile_slots : T * L->k >= 72 * L->E ? 128 : 64;
    // Top-2 routing with nothing else to add to a token's result (no shared expert, no residual): the streaming down
    // kernels add their two terms per token straight into the output, which the front kernel clears, and no combine
    // pass runs (a + b is the same float in either order; with three or more terms the order would matter).  Batches
    // served without a dispatch pass only: a prefill's tens of millions of atomic adds cost more than its combine pass.
    pl.accumulate = pl.direct && L->k == 2 && !shared && !L->has_rms && !sw.combine_pass;
    // very small K-quant batches: at most half of the experts can be active, so the weights are cut
    // into four times as many workgroups; those write f32 h and a small pass quantises it
    pl.narrow = pl.direct && L->vdt == MOE_GGML_Q8K && L->F % 64 == 0 && L->H % 32 == 0 && pl.slot_tiles == 1 &&
                (sw.narrow >= 0 ? sw.narrow > 0 : T * L->k <= L->E);
    pl.hbuf = pl.tiled || pl.narrow;
    // The always-on expert of a few tokens: its regular up launch has Fs / 256 (K-quants) or Fs / 128 workgroups, a
    // handful for a matrix of megabytes, and it is the step's critical path then.  The dense few-row kernels split K over
    // the waves of a workgroup per 16 rows instead (hundreds of workgroups): one launch for w1 and w3, one for w2.
    if (shared && sw.fused_rows != 1) {
        const bool kq = L->vdt == MOE_GGML_Q8K;
        const bool can = kq ? qlinear_fused_usable(L->dt, T, L->Fs, L->H) && qlinear_fused_usable(L->dt_down, T, L->H, L->Fs)
                            : q32_rows_fused_usable(L->dt, T, L->Fs, L->H) && q32_rows_fused_usable(L->dt_down, T, L->H, L->Fs);
        // (measured, step with / without: Qwen-MoE shape Q8_0, Fs = 5632: 73 / 94 us at one token, 88 / 100 at two, 103 / 107
        // at three, 115 / 112 at four; 64 Q4_K experts top-6 with Fs = 3072: 63 / 70, 65 / 75, 67 / 76, 70 / 81)
        pl.shared_rows = can && (sw.fused_rows == 2 || T <= (kq ? 4 : 3));
    }
    // Q8_0 / Q4_0 / Q5_0 layers whose slots are grouped by expert (more than DIRECT_MAX_SLOTS assignments): the tiled
    // kernels of kernels_q32.hip read an expert's weights once for up to 64 of its slots
    pl.tiled32 = !sw.no_gemm && !pl.direct && q8_0_gemm_usable(L->dt, L->dt_down, L->H, L->F) && T * L->k > 20 * L->E;
    if (pl.tiled32) pl.tile_slots = 64;
    return pl;
}

// Cuts the workspace of a forward of T tokens out of `base`; returns the bytes it takes (base == nullptr: only that).
static size_t carve_workspace(const moe_layer* L, int64_t T, const ForwardPlan& pl, uint8_t* base, Workspace* ws, bool stack_input = false) {
    Carver c;
    c.base = base;
    const bool shared = L->Fs > 0;
    const int64_t S = T * L->k + (shared ? T : 0);
    Workspace w;
    w.rb = c.take_route(T, (int)L->E, (int)L->k, shared, true);
    w.xq = c.take_act(L->vdt, T, L->H);
    w.hq = c.take_act(L->vdt, T * L->k, L->F);
    if (shared) w.hq_shared = c.take_act(L->vdt, T, L->Fs);
    w.yw = c.take<float>((size_t)S * L->H * 4);
    if (pl.hbuf) w.hbuf = c.take<float>((size_t)T * L->k * L->F * 4);
    if (pl.shared_rows) w.ab_shared = c.take<float>((size_t)2 * T * L->Fs * 4);
    if (stack_input) w.xin = c.take<float>((size_t)T * L->H * 4);
    if (L->gate_q) {
        if (L->has_rms) w.xn = c.take<float>((size_t)T * L->H * 4);
        w.logits_pad = c.take<float>((size_t)T * L->E16 * 4);
    }
    if (ws) *ws = w;
    return c.off;
}

// Enqueues one forward of T tokens on `s` with the workspace `ws`.  Caller holds L->mu.
// In a stack (moe_stack_forward_device): `prev` = the layer before left its combine pass to this layer's front kernel,
// which writes this layer's input to ws.xin (d_x is not read); `leave_combine` = this layer leaves its own to the next.
static int enqueue_forward(moe_layer* L, const ForwardPlan& pl, const Workspace& ws, const float* d_x, int64_t T, float* d_y,
                           hipStream_t s, hipEvent_t* marks = nullptr, const PrevCombine* prev = nullptr, bool leave_combine = false) {
#define MOE_MARK(i) do { if (marks) MOE_HIP_CHECK(hipEventRecord(marks[i], s)); } while (0)
    if (L->k == 0) {
        // nothing is selected: the block's output is zero (quantized_llama.rs:167 `take(0)`), plus the residual of a
        // layer that carries the pre-norm
        MOE_HIP_CHECK(launch_fill_or_copy(L->has_rms ? d_x : nullptr, d_y, T * L->H, s));
        L->last_T = -2;
        return MOE_OK;
    }
    const bool shared = L->Fs > 0;
    FrontParams fp;
    fp.x = d_x; fp.T = T; fp.H = (int)L->H; fp.E = (int)L->E; fp.k = (int)L->k; fp.norm_topk = L->norm_topk;
    fp.gate = L->gate.as<float>();
    fp.gate_bias = L->has_bias ? L->gate_bias.as<float>() : nullptr;
    fp.shared_gate = shared ? L->shared_gate.as<float>() : nullptr;
    fp.rms_alpha = L->has_rms ? L->rms_alpha.as<float>() : nullptr;
    fp.rms_eps = L->rms_eps;
    fp.rms_serial = switches().rms_serial;
    fp.vdt = L->vdt;
    fp.xq = ws.xq;
    fp.rb = ws.rb;
    fp.rb.T = (int)T; fp.rb.k = (int)L->k;
    fp.rb.direct = pl.direct ? 1 : 0;
    fp.rb.tile_slots = pl.tile_slots;
    if (pl.accumulate) fp.y_zero = d_y;
    if (prev) {
        fp.prev = *prev;
        fp.prev.x_out = ws.xin;
        d_x = ws.xin;   // this layer's residual
    }
    MOE_MARK(ST_BEGIN);
    if (L->gate_q) {
        // The quantised router: logits = the gate matrix's quantised product over the rows the experts see, quantised to
        // the gate dtype's own activation format; then routing and the experts' activation quantisation from those logits.
        if (L->has_rms) {
            MOE_HIP_CHECK(launch_add_rms_norm(d_x, nullptr, fp.rms_alpha, fp.rms_eps, T, (int)L->H, nullptr, ws.xn, s));
            fp.x = ws.xn;
            fp.rms_alpha = nullptr;
        }
        if (int rc = enqueue_qlinear(L->gate_q, fp.x, T, ws.logits_pad, s)) return rc;
        MOE_HIP_CHECK(launch_logits_unpad(ws.logits_pad, (int)L->E16, fp.gate_bias, fp.rb.logits, T, (int)L->E, s));
        MOE_HIP_CHECK(launch_front_route(fp, s));
    } else
    MOE_HIP_CHECK(launch_front(fp, s));
    MOE_MARK(ST_FRONT);
    if (!pl.direct) MOE_HIP_CHECK(launch_dispatch(fp.rb, T, (int)L->E, (int)L->k, shared, s));
    MOE_MARK(ST_DISPATCH);
    // The always-on expert's stream forks here.  (Its kernels need nothing of the dispatch pass and could start before it;
    // measured at the Qwen-MoE shape, 512 tokens, they then crowd the one-workgroup dispatch kernel and the start of the
    // routed launch: 308 against 298 us per step.)
    const bool overlap_shared = shared && !marks;
    if (overlap_shared) {
        MOE_HIP_CHECK(hipEventRecord(L->fork, s));
        MOE_HIP_CHECK(hipStreamWaitEvent(L->side, L->fork, 0));
    }

    ExpertParams ep;
    ep.dt = L->dt; ep.dt_down = L->dt_down; ep.H = (int)L->H; ep.F = (int)L->F;
    ep.n_groups = (int)L->E; ep.group0 = 0;
    ep.groups = L->groups.as<GroupWeights>();
    ep.rb = fp.rb; ep.xq = fp.xq; ep.hq = ws.hq; ep.slot_origin = 0;
    ep.yw = ws.yw;
    ep.y_acc = pl.accumulate ? d_y : nullptr;
    ep.max_rows = T;
    ep.slot_tiles = pl.slot_tiles;
    // The always-on expert reads the quantised activations and writes its own slots of yw: independent of the routed
    // experts until the combine pass, so its kernels go to the side stream and fill the CUs the routed launches leave idle
    // (the timed entry keeps one stream: its stage marks would mean nothing otherwise).
    hipStream_t ss = overlap_shared ? L->side : s;
    auto run_shared = [&]() -> int {
        if (pl.shared_rows) {
            const GroupWeights& g = L->host_groups[L->E];
            const bool kq = L->vdt == MOE_GGML_Q8K;
            FusedRows up;
            up.xq = fp.xq; up.m = T; up.n = L->Fs; up.k = L->H;
            up.w = g.w1; up.y = ws.ab_shared; up.silu_y = 1;
            up.w_b = g.w3; up.y_b = ws.ab_shared + T * L->Fs;
            MOE_HIP_CHECK(kq ? launch_qlinear_fused(L->dt, up, ss) : launch_q32_rows_fused(L->dt, up, ss));
            FusedRows down;   // quantises silu(w1 x) * (w3 x) as the up kernels' epilogues do, scales by the expert's gate
            down.x = up.y; down.x2 = up.y_b; down.m = T; down.n = L->H; down.k = L->Fs;
            down.w = g.w2; down.y = ws.yw + T * L->k * L->H; down.row_scale = fp.rb.shared_w;
            MOE_HIP_CHECK(kq ? launch_qlinear_fused(L->dt_down, down, ss) : launch_q32_rows_fused(L->dt_down, down, ss));
            return MOE_OK;
        }
        ExpertParams sp = ep;
        // the always-on expert takes the regular kernels (which quantise its intermediate in their epilogue) also when
        // the routed experts of a tiny batch took the narrow ones with their separate quantisation pass
        sp.hbuf = nullptr; sp.by_assignment = 0;
        sp.F = (int)L->Fs; sp.n_groups = 1; sp.group0 = (int)L->E; sp.is_shared = 1;
        sp.groups = L->groups.as<GroupWeights>() + L->E;
        sp.hq = ws.hq_shared; sp.slot_origin = (int)(T * L->k);
        sp.max_rows = T; sp.slot_tiles = T > 32 ? 4 : T > 16 ? 2 : 1;
        // Tiled kernels for the always-on expert too once its up projection fills the chip twice over.  (Qwen-MoE shape,
        // 512 tokens: alone on the GPU the tiled pair takes 132 us against 116 us streamed -- its down projection has
        // 8 tiles x 16 row blocks = 128 workgroups -- but beside the routed launches the step takes 291 against 300 us:
        // the tiled kernels read the expert's weights once, the streaming ones 16 times out of the caches.)
        const bool shared_tiled = pl.tiled32 && L->Fs % 128 == 0 && (L->Fs / 64) * ((T + 63) / 64) >= 512;
        if (shared_tiled) {
            MOE_HIP_CHECK(launch_q8_0_gemm_up(sp, ss));
            MOE_HIP_CHECK(launch_q8_0_gemm_down(sp, ss));
        } else {
            MOE_HIP_CHECK(launch_expert_up(sp, ss));
            MOE_HIP_CHECK(launch_expert_down(sp, ss));
        }
        return MOE_OK;
    };
    if (overlap_shared) {
        if (int rc = run_shared()) return rc;
        MOE_HIP_CHECK(hipEventRecord(L->join, ss));
    }
    if (pl.tiled) {
        ep.hbuf = ws.hbuf;
        ep.n_slots = T * L->k;
        MOE_HIP_CHECK(launch_q4k_gemm_up(ep, s));
        MOE_MARK(ST_UP);
        MOE_HIP_CHECK(launch_quantize_rows(L->vdt, ep.hbuf, T * L->k, (int)L->F, ep.hq, s));
        MOE_MARK(ST_REQUANT);
        if (pl.tiled_down) {
            MOE_HIP_CHECK(launch_q4k_gemm_down(ep, s));
        } else {
            ExpertParams dp = ep;
            dp.hbuf = nullptr;
            MOE_HIP_CHECK(launch_expert_down(dp, s));
        }
        MOE_MARK(ST_DOWN);
    } else if (pl.tiled32) {
        ep.n_slots = T * L->k;
        // (Q4_0 w1 / w3 stay with the streaming kernel: its nibble unpacking and offset addends per block put the tiled
        // up kernel 3 % behind it at the Mixtral shape, 4832 against 4683 us for 4096 tokens; both quantise the
        // intermediate in their epilogue)
        if (L->dt == MOE_GGML_Q4_0) MOE_HIP_CHECK(launch_expert_up(ep, s));
        else MOE_HIP_CHECK(launch_q8_0_gemm_up(ep, s));
        MOE_MARK(ST_UP);
        MOE_MARK(ST_REQUANT);
        MOE_HIP_CHECK(launch_q8_0_gemm_down(ep, s));
        MOE_MARK(ST_DOWN);
    } else if (pl.narrow) {
        ep.hbuf = ws.hbuf;
        ep.by_assignment = T * L->k <= L->E ? 1 : 0;   // one row of workgroups per assignment: none for idle experts
        MOE_HIP_CHECK(launch_expert_up(ep, s));
        MOE_MARK(ST_UP);
        MOE_HIP_CHECK(launch_quantize_rows(L->vdt, ep.hbuf, T * L->k, (int)L->F, ep.hq, s));
        MOE_MARK(ST_REQUANT);
        MOE_HIP_CHECK(launch_expert_down(ep, s));
        MOE_MARK(ST_DOWN);
        ep.by_assignment = 0;
    } else {
        MOE_HIP_CHECK(launch_expert_up(ep, s));   // re-quantises the intermediate in its epilogue
        MOE_MARK(ST_UP);
        MOE_MARK(ST_REQUANT);
        MOE_HIP_CHECK(launch_expert_down(ep, s));
        MOE_MARK(ST_DOWN);
    }
    if (overlap_shared) MOE_HIP_CHECK(hipStreamWaitEvent(s, L->join, 0));
    else if (shared)
        if (int rc = run_shared()) return rc;
    MOE_MARK(ST_SHARED);
    if (!pl.accumulate && !leave_combine) MOE_HIP_CHECK(launch_combine(ws.yw, fp.rb, shared, L->has_rms ? d_x : nullptr, d_y, T, (int)L->H, s));
    MOE_MARK(ST_COMBINE);
#undef MOE_MARK
    L->last_direct = pl.direct;
    L->last_T = T;
    L->last_ws = ws;
    L->last_ws.rb = fp.rb;
    return MOE_OK;
}

// One pass (T within max_tokens_per_pass) on the layer's own workspace.  Under stream capture (the caller records the
// forward into a HIP graph) nothing may be allocated, the event that orders eager calls on different streams stays out
// of the graph, and the workspace is from then on never freed before the layer goes: a replay uses its addresses.
static int forward_pass(moe_layer* L, const float* d_x, int64_t T, float* d_y, hipStream_t s, hipEvent_t* marks = nullptr) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (s) MOE_HIP_CHECK(hipStreamIsCapturing(s, &cap));
    const bool capturing = cap != hipStreamCaptureStatusNone;
    const ForwardPlan pl = plan_forward(L, T);
    Workspace ws;
    if (L->k > 0) {
        const size_t need = carve_workspace(L, T, pl, nullptr, nullptr);
        if (capturing && need > L->ws.cap)
            return fail(MOE_E_INVALID, "forward under stream capture needs its workspace: run one forward of the same number of tokens before capturing");
        if (need > L->ws.cap) {
            // a call on another stream may still be using the old workspace
            if (int rc = L->order.wait()) return rc;
            if (int rc = L->ws.reserve(need)) return rc;
        }
        carve_workspace(L, T, pl, static_cast<uint8_t*>(L->ws.p), &ws);
        if (capturing) L->ws.captured = true;
    }
    // a previous call may still be running on another stream and shares the workspace
    if (!capturing)
        if (int rc = L->order.enter(s)) return rc;
    const int rc = enqueue_forward(L, pl, ws, d_x, T, d_y, s, marks);
    if (!capturing) L->order.leave(s);   // also after a failure: what was enqueued before it is pending work on s
    return rc;
}

extern "C" int moe_layer_forward_device(moe_layer* L, const void* d_x, int64_t T, void* d_y, void* hip_stream) {
    if (!L || T < 0 || (T > 0 && (!d_x || !d_y))) return fail(MOE_E_INVALID, "bad argument to moe_layer_forward_device");
    if (d_x == d_y && T > 0) return fail(MOE_E_INVALID, "d_x and d_y must not alias");
    if (T > (1 << 20)) return fail(MOE_E_INVALID, "n_tokens > 2^20 is not supported");
    std::lock_guard<std::mutex> lk(L->mu);
    if (T == 0) { L->last_T = 0; return MOE_OK; }
    const int64_t step = max_tokens_per_pass(L);
    for (int64_t t0 = 0; t0 < T; t0 += step) {
        const int rc = forward_pass(L, static_cast<const float*>(d_x) + t0 * L->H, std::min(step, T - t0),
                                    static_cast<float*>(d_y) + t0 * L->H, static_cast<hipStream_t>(hip_stream));
        if (rc) return rc;
    }
    if (T > step && L->k > 0) L->last_T = -1;   // the routing hooks describe one pass only
    return MOE_OK;
}

// ------------------------------------------------------------------ a stack of layers
// y = layer[n-1](... layer[1](layer[0](x))), quantized_llama.rs:886-892 for the MoE blocks of consecutive transformer layers.
// Between two layers of a decode batch the first one's combine pass (+ residual) and the second one's front kernel
// (rms-norm, gate, routing, quantisation) are one launch: the front kernel forms its input row from the first layer's
// weighted expert outputs with the combine pass's own additions, in its order.  Where a boundary does not qualify (a
// dispatch pass, a shared expert, top-2 layers that accumulate in place, a front end in two launches, a quantised router)
// the two launches stay apart; the results are the same bits either way.
static bool stack_boundary_fuses(const moe_layer* A, const ForwardPlan& pa, const moe_layer* B, int64_t T) {
    if (A->k == 0 || B->k == 0 || A->Fs > 0 || !pa.direct || pa.accumulate || B->gate_q) return false;
    FrontParams fp;
    fp.T = T; fp.H = (int)B->H; fp.E = (int)B->E;
    fp.shared_gate = B->Fs > 0 ? B->shared_gate.as<float>() : nullptr;
    fp.rms_alpha = B->has_rms ? B->rms_alpha.as<float>() : nullptr;
    return front_takes_prev_combine(fp);
}

extern "C" int moe_stack_forward_device(moe_layer* const* layers, int64_t n_layers, const void* d_x, int64_t T, void* d_y, void* hip_stream) {
    if (!layers || n_layers <= 0 || T < 0 || (T > 0 && (!d_x || !d_y))) return fail(MOE_E_INVALID, "bad argument to moe_stack_forward_device");
    if (d_x == d_y && T > 0) return fail(MOE_E_INVALID, "d_x and d_y must not alias");
    for (int64_t l = 0; l < n_layers; l++) {
        if (!layers[l]) return fail(MOE_E_INVALID, "moe_stack_forward_device: layer " + std::to_string(l) + " is NULL");
        if (layers[l]->H != layers[0]->H) return fail(MOE_E_INVALID, "moe_stack_forward_device: the layers differ in hidden size");
        for (int64_t m = 0; m < l; m++)
            if (layers[m] == layers[l]) return fail(MOE_E_INVALID, "moe_stack_forward_device: a layer appears twice (every layer owns one workspace)");
    }
    if (T == 0) return MOE_OK;
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    // every layer of the stack is locked for the call (in address order: two stacks that share layers cannot deadlock)
    std::vector<moe_layer*> order(layers, layers + n_layers);
    std::sort(order.begin(), order.end());
    std::vector<std::unique_lock<std::mutex>> locks;
    for (moe_layer* L : order) locks.emplace_back(L->mu);
    for (int64_t l = 0; l < n_layers; l++)
        if (T > max_tokens_per_pass(layers[l])) return fail(MOE_E_INVALID, "moe_stack_forward_device: more tokens than one pass carries; call the layers one by one");
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (s) MOE_HIP_CHECK(hipStreamIsCapturing(s, &cap));
    const bool capturing = cap != hipStreamCaptureStatusNone;
    // plans, workspaces and which boundaries fuse
    std::vector<ForwardPlan> plans((size_t)n_layers);
    std::vector<char> fused_in((size_t)n_layers, 0);   // layer l takes layer l-1's combine pass
    for (int64_t l = 0; l < n_layers; l++) plans[(size_t)l] = plan_forward(layers[l], T);
    for (int64_t l = 1; l < n_layers; l++) fused_in[(size_t)l] = stack_boundary_fuses(layers[l - 1], plans[(size_t)l - 1], layers[l], T) ? 1 : 0;
    std::vector<Workspace> wss((size_t)n_layers);
    // Whatever was enqueued for a layer counts as its pending work on this stream, also when a later step of the call
    // fails: a following call from another stream then still waits for it.
    struct Entered {
        moe_layer* const* layers;
        hipStream_t s;
        int64_t n = 0;
        ~Entered() {
            for (int64_t l = 0; l < n; l++) layers[l]->order.leave(s);
        }
    } entered{layers, s};
    for (int64_t l = 0; l < n_layers; l++) {
        moe_layer* L = layers[l];
        // the layer's input row lives in its own workspace when the layer before writes it (fused) and, otherwise, in
        // the workspace too: every layer but the last writes its output into the next layer's xin
        const size_t need = L->k > 0 ? carve_workspace(L, T, plans[(size_t)l], nullptr, nullptr, l > 0) : (l > 0 ? (size_t)T * L->H * 4 + 256 : 0);
        if (capturing && need > L->ws.cap)
            return fail(MOE_E_INVALID, "moe_stack_forward_device under stream capture needs its workspaces: run the stack once with the same number of tokens before capturing");
        if (need > L->ws.cap) {
            if (int rc = L->order.wait()) return rc;
            if (int rc = L->ws.reserve(need)) return rc;
        }
        if (L->k > 0) carve_workspace(L, T, plans[(size_t)l], static_cast<uint8_t*>(L->ws.p), &wss[(size_t)l], l > 0);
        else if (l > 0) wss[(size_t)l].xin = reinterpret_cast<float*>(L->ws.p);
        if (capturing) L->ws.captured = true;
        if (!capturing) {
            if (int rc = L->order.enter(s)) return rc;
            entered.n = l + 1;
        }
    }
    // Layer l reads its input from d_x (l = 0) or from its own xin, which either the layer before wrote (its combine pass)
    // or this layer's front kernel writes (the combine pass folded in); its output goes to the next layer's xin, or to d_y.
    const float* in_prev = nullptr;
    for (int64_t l = 0; l < n_layers; l++) {
        moe_layer* L = layers[l];
        const bool last = l + 1 == n_layers;
        const bool leave = !last && fused_in[(size_t)l + 1];
        const float* in = l == 0 ? static_cast<const float*>(d_x) : wss[(size_t)l].xin;
        float* out = last ? static_cast<float*>(d_y) : wss[(size_t)l + 1].xin;
        PrevCombine prev;
        if (fused_in[(size_t)l]) {
            const moe_layer* P = layers[l - 1];
            prev.yw = wss[(size_t)l - 1].yw;
            prev.topk_idx = wss[(size_t)l - 1].rb.topk_idx;
            prev.k = (int)P->k;
            prev.residual = P->has_rms ? in_prev : nullptr;
        }
        if (int rc = enqueue_forward(L, plans[(size_t)l], wss[(size_t)l], in, T, out, s, nullptr, fused_in[(size_t)l] ? &prev : nullptr, leave)) return rc;
        in_prev = in;
    }
    return MOE_OK;   // `entered` marks the layers' work as pending on s
}

// ------------------------------------------------------------------ the entry point that allocates nothing
// Its workspace is this array instead of memory from hipMalloc.  The name below is a host-side stand-in: the device
// address comes from hipGetSymbolAddress, once per device, and only that address is handed to kernels.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)MOE_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];
constexpr int MAX_DEVICES = 64;
static std::mutex g_scratch_mu;
static void* g_scratch_ptr[MAX_DEVICES] = {};

static int static_scratch(uint8_t** out) {
    int dev = 0;
    MOE_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return fail(MOE_E_INVALID, "device index out of range");
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        MOE_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return fail(MOE_E_HIP, "hipGetSymbolAddress returned no address for the static scratch array");
        g_scratch_ptr[dev] = ptr;
    }
    *out = static_cast<uint8_t*>(g_scratch_ptr[dev]);
    return MOE_OK;
}

extern "C" int64_t moe_static_scratch_bytes(void) { return (int64_t)STATIC_SCRATCH_BYTES; }

extern "C" int moe_layer_forward_device_noalloc(moe_layer* L, const void* d_x, int64_t T, void* d_y, void* hip_stream) {
    if (!L || T < 0 || (T > 0 && (!d_x || !d_y))) return fail(MOE_E_INVALID, "bad argument to moe_layer_forward_device_noalloc");
    if (d_x == d_y && T > 0) return fail(MOE_E_INVALID, "d_x and d_y must not alias");
    std::lock_guard<std::mutex> lk(L->mu);
    if (T == 0) { L->last_T = 0; return MOE_OK; }
    if (T > max_tokens_per_pass(L))
        return fail(MOE_E_INVALID, "moe_layer_forward_device_noalloc: " + std::to_string(T) + " tokens are more than one pass carries");
    if (L->gate_q) return fail(MOE_E_INVALID, "moe_layer_forward_device_noalloc: a layer with a quantised router allocates the workspace of its gate product; use moe_layer_forward_device");
    const ForwardPlan pl = plan_forward(L, T);
    const size_t need = L->k > 0 ? carve_workspace(L, T, pl, nullptr, nullptr) : 0;
    if (need > STATIC_SCRATCH_BYTES)
        return fail(MOE_E_INVALID, "moe_layer_forward_device_noalloc: " + std::to_string(T) + " tokens need a workspace of " + std::to_string(need) +
                                       " bytes, the static scratch array holds " + std::to_string(STATIC_SCRATCH_BYTES) +
                                       "; use moe_layer_forward_device for batches of this size");
    uint8_t* base = nullptr;
    if (int rc = static_scratch(&base)) return rc;
    Workspace ws;
    if (L->k > 0) carve_workspace(L, T, pl, base, &ws);
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (s) MOE_HIP_CHECK(hipStreamIsCapturing(s, &cap));
    // An earlier call on this layer may still run on another stream: it shares the layer's side stream and events (and
    // a later allocating call must find this one in the order).  An event record and a stream wait: no allocation.
    const bool capturing = cap != hipStreamCaptureStatusNone;
    if (!capturing)
        if (int rc = L->order.enter(s)) return rc;
    const int rc = enqueue_forward(L, pl, ws, static_cast<const float*>(d_x), T, static_cast<float*>(d_y), s);
    // the hooks that read the last call's logits and routing wait for this stream (after a failure too: what was
    // enqueued before it is pending work on s)
    if (!capturing) L->order.leave(s);
    return rc;
}

extern "C" int moe_layer_forward_timed(moe_layer* L, const void* d_x, int64_t T, void* d_y, void* hip_stream, float* stage_ms) {
    if (!L || T <= 0 || !d_x || !d_y || !stage_ms || d_x == d_y) return fail(MOE_E_INVALID, "bad argument to moe_layer_forward_timed");
    if (T > (1 << 20)) return fail(MOE_E_INVALID, "n_tokens > 2^20 is not supported");
    std::lock_guard<std::mutex> lk(L->mu);
    if (L->k == 0) return fail(MOE_E_INVALID, "moe_layer_forward_timed: the layer has top_k = 0 and launches no stages");
    if (T > max_tokens_per_pass(L)) return fail(MOE_E_INVALID, "moe_layer_forward_timed: more tokens than one pass carries (" + std::to_string(max_tokens_per_pass(L)) + ")");
    hipStream_t s = static_cast<hipStream_t>(hip_stream);
    hipEvent_t marks[ST_COUNT] = {};
    int rc = MOE_OK;
    for (int i = 0; i < ST_COUNT && !rc; i++)
        if (hipEventCreate(&marks[i]) != hipSuccess) rc = fail(MOE_E_HIP, "hipEventCreate failed");
    if (!rc) rc = forward_pass(L, static_cast<const float*>(d_x), T, static_cast<float*>(d_y), s, marks);
    if (!rc && hipEventSynchronize(marks[ST_COMBINE]) != hipSuccess) rc = fail(MOE_E_HIP, "hipEventSynchronize failed");
    for (int i = 0; i + 1 < ST_COUNT && !rc; i++)
        if (hipEventElapsedTime(&stage_ms[i], marks[i], marks[i + 1]) != hipSuccess) rc = fail(MOE_E_HIP, "hipEventElapsedTime failed");
    for (int i = 0; i < ST_COUNT; i++)
        if (marks[i]) (void)hipEventDestroy(marks[i]);
    return rc;
}

extern "C" int moe_layer_forward(moe_layer* L, const float* x, int64_t T, float* y) {
    if (!L || T < 0 || (T > 0 && (!x || !y))) return fail(MOE_E_INVALID, "bad argument to moe_layer_forward");
    if (T > (1 << 20)) return fail(MOE_E_INVALID, "n_tokens > 2^20 is not supported");
    std::lock_guard<std::mutex> lk(L->mu);
    if (T == 0) { L->last_T = 0; return MOE_OK; }
    int rc;
    const size_t bytes = (size_t)T * L->H * 4;
    if ((rc = L->x_dev.reserve(bytes))) return rc;
    if ((rc = L->y_dev.reserve(bytes))) return rc;
    MOE_HIP_CHECK(hipMemcpyAsync(L->x_dev.p, x, bytes, hipMemcpyHostToDevice, L->stream));
    const int64_t step = max_tokens_per_pass(L);
    for (int64_t t0 = 0; t0 < T; t0 += step)
        if ((rc = forward_pass(L, L->x_dev.as<float>() + t0 * L->H, std::min(step, T - t0), L->y_dev.as<float>() + t0 * L->H, L->stream))) return rc;
    if (T > step && L->k > 0) L->last_T = -1;   // the routing hooks describe one pass only
    MOE_HIP_CHECK(hipMemcpyAsync(y, L->y_dev.p, bytes, hipMemcpyDeviceToHost, L->stream));
    MOE_HIP_CHECK(hipStreamSynchronize(L->stream));
    return MOE_OK;
}

static int d2h(void* dst, const void* src, size_t bytes) {
    if (!dst || bytes == 0) return MOE_OK;
    MOE_HIP_CHECK(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return MOE_OK;
}

static int check_last(const moe_layer* L, int64_t T) {
    if (L->last_T == -2) return fail(MOE_E_INVALID, "the layer has top_k = 0: its forward computes no logits and no routing");
    if (T != L->last_T) return fail(MOE_E_INVALID, "n_tokens differs from the last forward on this layer");
    return MOE_OK;
}

extern "C" int moe_layer_last_logits(moe_layer* L, float* logits, int64_t T) {
    if (!L || !logits) return fail(MOE_E_INVALID, "bad argument to moe_layer_last_logits");
    std::lock_guard<std::mutex> lk(L->mu);
    if (int rc = check_last(L, T)) return rc;
    if (int rc = L->order.wait()) return rc;
    return d2h(logits, L->last_ws.rb.logits, (size_t)T * L->E * 4);
}

extern "C" int moe_layer_last_routing(moe_layer* L, int64_t T, int32_t* topk_idx, float* topk_w, int32_t* offsets,
                                      int32_t* perm_token, float* perm_w) {
    if (!L) return fail(MOE_E_INVALID, "layer is NULL");
    std::lock_guard<std::mutex> lk(L->mu);
    int rc;
    if ((rc = check_last(L, T))) return rc;
    if ((rc = L->order.wait())) return rc;
    const size_t A = (size_t)T * L->k;
    const RouteBufs& rb = L->last_ws.rb;
    if (L->last_direct && T > 0) {  // the forward needed no lists; build them now for the caller
        MOE_HIP_CHECK(launch_dispatch(rb, T, (int)L->E, (int)L->k, L->Fs > 0, nullptr));
        MOE_HIP_CHECK(hipDeviceSynchronize());
        L->last_direct = false;
    }
    if (T == 0) {
        if (offsets) std::memset(offsets, 0, (size_t)(L->E + 1) * 4);
        return MOE_OK;
    }
    if ((rc = d2h(topk_idx, rb.topk_idx, A * 4))) return rc;
    if ((rc = d2h(topk_w, rb.topk_w, A * 4))) return rc;
    if ((rc = d2h(offsets, rb.offsets, (size_t)(L->E + 1) * 4))) return rc;
    if ((rc = d2h(perm_token, rb.perm_token, A * 4))) return rc;
    return d2h(perm_w, rb.perm_w, A * 4);
}

extern "C" int moe_layer_shape(const moe_layer* L, int64_t* hidden, int64_t* ffn, int64_t* n_experts, int64_t* top_k) {
    if (!L) return fail(MOE_E_INVALID, "layer is NULL");
    if (hidden) *hidden = L->H;
    if (ffn) *ffn = L->F;
    if (n_experts) *n_experts = L->E;
    if (top_k) *top_k = L->k;
    return MOE_OK;
}

extern "C" int moe_layer_dequantize_weight(moe_layer* L, int64_t expert, int which, float* out, int64_t n_elems) {
    if (!L || !out) return fail(MOE_E_INVALID, "bad argument to moe_layer_dequantize_weight");
    if (expert < 0 || expert >= (int64_t)L->host_groups.size() || which < 1 || which > 3)
        return fail(MOE_E_INVALID, "expert / which out of range");
    const int64_t F = expert == L->E ? L->Fs : L->F;
    const int64_t rows = which == 2 ? L->H : F, cols = which == 2 ? F : L->H;
    if (n_elems != rows * cols) return fail(MOE_E_INVALID, "n_elems must be rows*cols = " + std::to_string(rows * cols));
    const GroupWeights& g = L->host_groups[expert];
    const uint8_t* src = which == 1 ? g.w1 : which == 2 ? g.w2 : g.w3;
    DevBuf tmp;
    int rc = tmp.reserve((size_t)n_elems * 4);
    if (rc) return rc;
    MOE_HIP_CHECK(launch_dequant_tiled(which == 2 ? L->dt_down : L->dt, src, tmp.as<float>(), rows, cols, nullptr));
    MOE_HIP_CHECK(hipDeviceSynchronize());
    return d2h(out, tmp.p, (size_t)n_elems * 4);
}

extern "C" int moe_route(const float* logits, int64_t T, int64_t E, int64_t k, int32_t norm_topk, int32_t* topk_idx,
                         float* topk_w, int32_t* offsets, int32_t* perm_token, float* perm_w) {
    int rc = ensure_device();
    if (rc) return rc;
    if (T < 0 || E < 1 || E > 256 || k < 0 || k > E || k > 16) return fail(MOE_E_INVALID, "moe_route: need 1<=E<=256, 0<=k<=min(E,16)");
    if (T > 0 && !logits) return fail(MOE_E_INVALID, "logits is NULL");
    if (T == 0 || k == 0) {   // k = 0: `take(0)` selects nothing, every list is empty
        if (offsets) std::memset(offsets, 0, (size_t)(E + 1) * 4);
        return MOE_OK;
    }
    RouteStore rs;
    DevBuf dl;
    if ((rc = rs.reserve(T, (int)E, (int)k, false))) return rc;
    if ((rc = dl.reserve((size_t)T * E * 4))) return rc;
    MOE_HIP_CHECK(hipMemcpy(dl.p, logits, (size_t)T * E * 4, hipMemcpyHostToDevice));
    MOE_HIP_CHECK(launch_route_from_logits(dl.as<float>(), T, (int)E, (int)k, norm_topk ? 1 : 0, rs.view(), nullptr));
    MOE_HIP_CHECK(launch_dispatch(rs.view(), T, (int)E, (int)k, false, nullptr));
    MOE_HIP_CHECK(hipDeviceSynchronize());
    const size_t A = (size_t)T * k;
    if ((rc = d2h(topk_idx, rs.topk_idx.p, A * 4))) return rc;
    if ((rc = d2h(topk_w, rs.topk_w.p, A * 4))) return rc;
    if ((rc = d2h(offsets, rs.offsets.p, (size_t)(E + 1) * 4))) return rc;
    if ((rc = d2h(perm_token, rs.perm_token.p, A * 4))) return rc;
    return d2h(perm_w, rs.perm_w.p, A * 4);
}

extern "C" int moe_dequantize(int32_t dt, const void* blocks, int64_t n, float* out) {
    int rc = ensure_device();
    if (rc) return rc;
    const int64_t be = block_elems(dt);
    if (be < 0 || dt == MOE_GGML_Q8_1)   // BlockQ8_1 has no to_float (k_quants.rs:731-733)
        return fail(MOE_E_INVALID, "moe_dequantize: unsupported dtype " + std::to_string(dt));
    if (n < 0 || n % be) return fail(MOE_E_INVALID, "n_elems must be a non-negative multiple of the block size");
    if (n == 0) return MOE_OK;
    if (!blocks || !out) return fail(MOE_E_INVALID, "NULL pointer");
    DevBuf src, dst;
    const size_t bytes = (size_t)(n / be * block_bytes(dt));
    if ((rc = src.reserve(bytes))) return rc;
    if ((rc = dst.reserve((size_t)n * 4))) return rc;
    MOE_HIP_CHECK(hipMemcpy(src.p, blocks, bytes, hipMemcpyHostToDevice));
    MOE_HIP_CHECK(launch_dequant_std(dt, src.as<uint8_t>(), dst.as<float>(), n, nullptr));
    MOE_HIP_CHECK(hipDeviceSynchronize());
    return d2h(out, dst.p, (size_t)n * 4);
}

extern "C" int moe_quantize_act(int32_t vdt, const float* x, int64_t rows, int64_t k, void* out) {
    int rc = ensure_device();
    if (rc) return rc;
    if (vdt != MOE_GGML_Q8_0 && vdt != MOE_GGML_Q8_1 && vdt != MOE_GGML_Q8K) return fail(MOE_E_INVALID, "vecdot_dtype must be Q8_0 (8), Q8_1 (9) or Q8K (15)");
    const int64_t be = block_elems(vdt);
    if (rows < 0 || k <= 0 || k % be || k > (1 << 24)) return fail(MOE_E_INVALID, "k must be a positive multiple of the block size");
    if (rows == 0) return MOE_OK;
    if (!x || !out) return fail(MOE_E_INVALID, "NULL pointer");
    DevBuf dx, dout;
    ActStore as;
    const size_t out_bytes = (size_t)(rows * k / be * block_bytes(vdt));
    if ((rc = dx.reserve((size_t)rows * k * 4))) return rc;
    if ((rc = dout.reserve(out_bytes))) return rc;
    if ((rc = as.reserve(vdt, rows, k))) return rc;
    MOE_HIP_CHECK(hipMemcpy(dx.p, x, (size_t)rows * k * 4, hipMemcpyHostToDevice));
    MOE_HIP_CHECK(launch_quantize_rows(vdt, dx.as<float>(), rows, (int)k, as.view(), nullptr));
    MOE_HIP_CHECK(launch_actbuf_to_std(vdt, as.view(), rows, (int)k, dout.as<uint8_t>(), nullptr));
    MOE_HIP_CHECK(hipDeviceSynchronize());
    return d2h(out, dout.p, out_bytes);
}

// ------------------------------------------------------------------ dense quantized linear
// One quantized matrix kept resident in the tiled layout, applied to f32 rows: the attention and
// output projections around the MoE block use the same matmul as the experts.
struct moe_qlinear {
    int64_t n = 0, k = 0;
    int dt = 0, vdt = 0;
    DevBuf weights, group;
    std::mutex mu;
    GrowBuf ws;                     // quantised rows and the identity routing table, cut anew for every call
    CallOrder order;
    int64_t routed_m = -1;          // row count the identity routing table currently describes (with routed_tile)
    int routed_tile = 0;
    bool routed_tab = false;
    hipStream_t routed_stream = nullptr;
    DevBuf x_dev, y_dev;
    hipStream_t stream = nullptr;
};

extern "C" void moe_qlinear_destroy(moe_qlinear* Q) {
    if (!Q) return;
    (void)hipDeviceSynchronize();
    if (Q->stream) (void)hipStreamDestroy(Q->stream);
    Q->order.destroy();
    delete Q;
}

extern "C" int moe_qlinear_create(int32_t dt, const void* w_blocks, int64_t n, int64_t k, moe_qlinear** out) {
    if (out) *out = nullptr;
    int rc = ensure_device();
    if (rc) return rc;
    if (!out || !w_blocks) return fail(MOE_E_INVALID, "moe_qlinear_create: NULL pointer");
    if (!weight_dtype_supported(dt))
        return fail(MOE_E_INVALID, "moe_qlinear_create: unsupported ggml_dtype " + std::to_string(dt) + " (supported: Q4_0=2, Q4_1=3, Q5_0=6, Q5_1=7, Q8_0=8, Q2K=10, Q3K=11, Q4K=12, Q5K=13, Q6K=14)");
    const int64_t be = block_elems(dt);
    if (n <= 0 || n % 16 || k <= 0 || k % be || k > (1 << 24))
        return fail(MOE_E_INVALID, "moe_qlinear_create: need n % 16 == 0 and k a multiple of the block size (" + std::to_string(be) + ")");
    std::unique_ptr<moe_qlinear, void (*)(moe_qlinear*)> Q(new moe_qlinear, moe_qlinear_destroy);
    Q->n = n; Q->k = k; Q->dt = dt; Q->vdt = vecdot_dtype(dt);
    DevBuf raw;
    const size_t raw_bytes = (size_t)(n * k / be * block_bytes(dt));
    if ((rc = raw.reserve(raw_bytes))) return rc;
    if ((rc = Q->weights.reserve((size_t)relaid_bytes(dt, n, k)))) return rc;
    if ((rc = Q->group.reserve(sizeof(GroupWeights)))) return rc;
    MOE_HIP_CHECK(hipMemcpy(raw.p, w_blocks, raw_bytes, hipMemcpyHostToDevice));
    MOE_HIP_CHECK(launch_relayout(dt, raw.as<uint8_t>(), Q->weights.as<uint8_t>(), n, k, nullptr));
    GroupWeights g{nullptr, nullptr, Q->weights.as<uint8_t>()};
    MOE_HIP_CHECK(hipMemcpy(Q->group.p, &g, sizeof g, hipMemcpyHostToDevice));
    MOE_HIP_CHECK(hipDeviceSynchronize());
    MOE_HIP_CHECK(hipStreamCreateWithFlags(&Q->stream, hipStreamNonBlocking));
    if ((rc = Q->order.init())) return rc;
    *out = Q.release();
    return MOE_OK;
}

static size_t carve_qlinear(const moe_qlinear* Q, int64_t m, uint8_t* base, RouteBufs* rb, ActBuf* xq) {
    Carver c;
    c.base = base;
    const RouteBufs r = c.take_route(m, 1, 1, false, true);
    const ActBuf a = c.take_act(Q->vdt, m, Q->k);
    if (rb) *rb = r;
    if (xq) *xq = a;
    return c.off;
}

// quantise the rows, then one pass over the matrix: streamed for short batches, tiled MFMA beyond
static int enqueue_qlinear(moe_qlinear* Q, const float* d_x, int64_t m, float* d_y, hipStream_t s) {
    // One or two rows of a K-quant matrix (single-stream decoding): one launch that quantises the rows itself; no workspace,
    // nothing shared between calls.  Every workgroup repeats the quantisation, which costs a wave ~0.5 us per block and
    // row, so the two passes win from three rows on and for the widest matrices (measured inside a HIP graph, Q4_K,
    // fused / two passes: 4096 x 4096: 5.8 / 12.6 us at one row, 7.8 / 13.0 at two, 11.6 / 13.4 at four -- the graph's two
    // passes carry a table kernel that eager calls skip, ~2.5 us; 4096 x 14336: 16.9 / 28.0 at one row; 16384 x 4096:
    // 10.7 / 14.5; 32000 x 4096: 21.2 / 19.5).  fused_rows: 1 = never, 2 = whenever the kernel can (test aid).
    const int fr = switches().fused_rows;
    if (fr != 1 && qlinear_fused_usable(Q->dt, m, Q->n, Q->k) && (fr == 2 || (m <= 2 && Q->n <= 16384))) {
        FusedRows f;
        f.x = d_x; f.m = m; f.n = Q->n; f.k = Q->k; f.w = Q->weights.as<uint8_t>(); f.y = d_y;
        MOE_HIP_CHECK(launch_qlinear_fused(Q->dt, f, s));
        return MOE_OK;
    }
    // the 32-element formats: the same, with the block values added in the reference's order by one wave (in a graph,
    // Q8_0, fused / two passes: 4096 x 4096: 9.3 / 22.1 us at one row, 13.6 / 22.4 at two, 21.4 / 22.8 at four; 4096 x 14336:
    // 27.6 / 57.0 at one row; 8192 x 4096: 11.4 / 22.7; 32000 x 4096: 33.1 / 30.3)
    if (fr != 1 && q32_rows_fused_usable(Q->dt, m, Q->n, Q->k) && (fr == 2 || (m <= 3 && Q->n <= 16384))) {
        FusedRows f;
        f.x = d_x; f.m = m; f.n = Q->n; f.k = Q->k; f.w = Q->weights.as<uint8_t>(); f.y = d_y;
        MOE_HIP_CHECK(launch_q32_rows_fused(Q->dt, f, s));
        return MOE_OK;
    }
    // under stream capture nothing may be allocated, the graph carries its own copy of the routing table pass, and the
    // workspace is never freed afterwards (a replay uses its addresses)
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (s) MOE_HIP_CHECK(hipStreamIsCapturing(s, &cap));
    const bool capturing = cap != hipStreamCaptureStatusNone;
    const size_t need = carve_qlinear(Q, m, nullptr, nullptr, nullptr);
    if (capturing && need > Q->ws.cap)
        return fail(MOE_E_INVALID, "forward under stream capture needs its workspace: run one forward of the same number of rows before capturing");
    if (need > Q->ws.cap) {
        if (int rc = Q->order.wait()) return rc;   // a call on another stream may still be using the old workspace
        if (int rc = Q->ws.reserve(need)) return rc;
        Q->routed_m = -1;   // the table has moved
    }
    if (capturing) Q->ws.captured = true;
    RouteBufs rb;
    ActBuf xq;
    carve_qlinear(Q, m, static_cast<uint8_t*>(Q->ws.p), &rb, &xq);
    // Calls share the quantised rows and the table: a call on another stream waits for the previous one.
    if (!capturing)
        if (int rc = Q->order.enter(s)) return rc;
    // The tiled MFMA kernel runs one workgroup per (128 weight rows, tile of 64 or 128 x rows): it pays
    // once that grid fills most of the 256 CUs; below, the streamed kernels split the matrix finer.
    const int64_t row_blocks = Q->n / 128;
    const int tile_slots = row_blocks * ((m + 127) / 128) >= 512 ? 128 : 64;
    const bool tiled = !switches().no_gemm && q4k_gemm_down_format(Q->dt) && Q->n % 128 == 0 && m >= 96 &&
                       row_blocks * ((m + tile_slots - 1) / tile_slots) >= 192;
    // Q8_0 / Q4_0 / Q5_0 matrices: the tiled kernel of the 32-element formats (64-row tiles of the one group, no tile list)
    // once its grid holds a workgroup per CU (Q8_0, 4096 x 4096: 58 against 65 us at 512 rows, 53 against 42 us at 256)
    const bool tiled32 = !switches().no_gemm && q8_0_gemm_usable(Q->dt, 0, Q->n, Q->k) && row_blocks * ((m + 63) / 64) >= 256;
    rb.T = (int)m; rb.k = 1;
    rb.tile_slots = tiled32 ? 64 : tile_slots;
    if (!tiled) rb.tile_tab = nullptr;
    MOE_HIP_CHECK(launch_quantize_rows(Q->vdt, d_x, m, (int)Q->k, xq, s));
    // The identity table depends on the row count only: a decode loop that calls with the same m finds it in place.
    // Once a graph has been captured on this object the host no longer knows what the table holds -- a replay rewrites
    // it for the captured row count, in the workspace eager calls share -- so from then on every call writes it again.
    if (Q->ws.captured || Q->routed_m != m || Q->routed_tile != tile_slots || Q->routed_tab != tiled || Q->routed_stream != s) {
        MOE_HIP_CHECK(launch_identity_routing(rb, m, s));
        Q->routed_m = m; Q->routed_tile = tile_slots; Q->routed_tab = tiled; Q->routed_stream = s;
    }
    ExpertParams ep;
    ep.dt = Q->dt; ep.H = (int)Q->n; ep.F = (int)Q->k; ep.n_groups = 1; ep.group0 = 0;
    ep.groups = Q->group.as<GroupWeights>();
    ep.rb = rb; ep.hq = xq; ep.slot_origin = 0; ep.yw = d_y;
    ep.max_rows = m; ep.n_slots = m; ep.slot_tiles = m > 32 ? 4 : m > 16 ? 2 : 1;
    if (tiled) {
        MOE_HIP_CHECK(launch_q4k_gemm_down(ep, s));
    } else if (tiled32) {
        ep.is_shared = 1;
        MOE_HIP_CHECK(launch_q8_0_gemm_down(ep, s));
    } else {
        MOE_HIP_CHECK(launch_expert_down(ep, s));
    }
    if (!capturing) Q->order.leave(s);
    return MOE_OK;
}

// 32-bit byte offsets into the quantised rows (rows * k): longer inputs go through in several passes
static int64_t qlinear_rows_per_pass(const moe_qlinear* Q) { return std::max<int64_t>(1, (((int64_t)1 << 31) - 1) / Q->k); }

static int check_qlinear_call(moe_qlinear* Q, const void* x, int64_t m, const void* y, const char* who) {
    if (!Q || m < 0 || (m > 0 && (!x || !y))) return fail(MOE_E_INVALID, std::string("bad argument to ") + who);
    if (m > (1 << 20)) return fail(MOE_E_INVALID, std::string(who) + ": more than 2^20 rows is not supported");
    return MOE_OK;
}

extern "C" int moe_qlinear_forward_device(moe_qlinear* Q, const void* d_x, int64_t m, void* d_y, void* hip_stream) {
    int rc = check_qlinear_call(Q, d_x, m, d_y, "moe_qlinear_forward_device");
    if (rc || m == 0) return rc;
    if (d_x == d_y) return fail(MOE_E_INVALID, "d_x and d_y must not alias");
    std::lock_guard<std::mutex> lk(Q->mu);
    const int64_t step = qlinear_rows_per_pass(Q);
    for (int64_t r0 = 0; r0 < m; r0 += step)
        if ((rc = enqueue_qlinear(Q, static_cast<const float*>(d_x) + r0 * Q->k, std::min(step, m - r0), static_cast<float*>(d_y) + r0 * Q->n,
                                  static_cast<hipStream_t>(hip_stream))))
            return rc;
    return MOE_OK;
}

extern "C" int moe_qlinear_forward(moe_qlinear* Q, const float* x, int64_t m, float* y) {
    int rc = check_qlinear_call(Q, x, m, y, "moe_qlinear_forward");
    if (rc || m == 0) return rc;
    std::lock_guard<std::mutex> lk(Q->mu);
    const size_t xb = (size_t)m * Q->k * 4, yb = (size_t)m * Q->n * 4;
    if ((rc = Q->x_dev.reserve(xb))) return rc;
    if ((rc = Q->y_dev.reserve(yb))) return rc;
    MOE_HIP_CHECK(hipMemcpyAsync(Q->x_dev.p, x, xb, hipMemcpyHostToDevice, Q->stream));
    const int64_t step = qlinear_rows_per_pass(Q);
    for (int64_t r0 = 0; r0 < m; r0 += step)
        if ((rc = enqueue_qlinear(Q, Q->x_dev.as<float>() + r0 * Q->k, std::min(step, m - r0), Q->y_dev.as<float>() + r0 * Q->n, Q->stream))) return rc;
    MOE_HIP_CHECK(hipMemcpyAsync(y, Q->y_dev.p, yb, hipMemcpyDeviceToHost, Q->stream));
    MOE_HIP_CHECK(hipStreamSynchronize(Q->stream));
    return MOE_OK;
}

extern "C" int moe_qlinear_dequantize(moe_qlinear* Q, float* out, int64_t n_elems) {
    if (!Q || !out) return fail(MOE_E_INVALID, "bad argument to moe_qlinear_dequantize");
    if (n_elems != Q->n * Q->k) return fail(MOE_E_INVALID, "n_elems must be n*k = " + std::to_string(Q->n * Q->k));
    DevBuf tmp;
    int rc = tmp.reserve((size_t)n_elems * 4);
    if (rc) return rc;
    MOE_HIP_CHECK(launch_dequant_tiled(Q->dt, Q->weights.as<uint8_t>(), tmp.as<float>(), Q->n, Q->k, nullptr));
    MOE_HIP_CHECK(hipDeviceSynchronize());
    return d2h(out, tmp.p, (size_t)n_elems * 4);
}

extern "C" int moe_qlinear_shape(const moe_qlinear* Q, int64_t* n, int64_t* k, int32_t* dt) {
    if (!Q) return fail(MOE_E_INVALID, "qlinear is NULL");
    if (n) *n = Q->n;
    if (k) *k = Q->k;
    if (dt) *dt = Q->dt;
    return MOE_OK;
}

extern "C" int moe_qmatmul(int32_t dt, const void* w_blocks, int64_t n, int64_t k, const float* x, int64_t m, float* y) {
    if (m < 0) return fail(MOE_E_INVALID, "moe_qmatmul: negative row count");
    moe_qlinear* Q = nullptr;
    int rc = moe_qlinear_create(dt, w_blocks, n, k, &Q);
    if (rc) return rc;
    rc = moe_qlinear_forward(Q, x, m, y);
    moe_qlinear_destroy(Q);
    return rc;
}

static bool weight_quantiser_exists(int dt) {
    return dt == MOE_GGML_Q4_0 || dt == MOE_GGML_Q8_0 || dt == MOE_GGML_Q2K || dt == MOE_GGML_Q3K || dt == MOE_GGML_Q4K ||
           dt == MOE_GGML_Q5K || dt == MOE_GGML_Q6K;
}

extern "C" int moe_quantize_weights_device(int32_t dt, const void* d_x, int64_t n, void* d_out, void* hip_stream) {
    int rc = ensure_device();
    if (rc) return rc;
    if (!weight_quantiser_exists(dt)) return fail(MOE_E_INVALID, "moe_quantize_weights: unsupported dtype");
    if (n < 0 || n % block_elems(dt)) return fail(MOE_E_INVALID, "n_elems must be a non-negative multiple of the block size");
    if (n == 0) return MOE_OK;
    if (!d_x || !d_out) return fail(MOE_E_INVALID, "NULL pointer");
    MOE_HIP_CHECK(launch_quantize_weights(dt, static_cast<const float*>(d_x), n, static_cast<uint8_t*>(d_out), static_cast<hipStream_t>(hip_stream)));
    return MOE_OK;
}

extern "C" int moe_quantize_weights(int32_t dt, const float* x, int64_t n, void* out) {
    int rc = ensure_device();
    if (rc) return rc;
    if (!weight_quantiser_exists(dt)) return fail(MOE_E_INVALID, "moe_quantize_weights: unsupported dtype");
    if (n < 0 || n % block_elems(dt)) return fail(MOE_E_INVALID, "n_elems must be a non-negative multiple of the block size");
    if (n == 0) return MOE_OK;
    if (!x || !out) return fail(MOE_E_INVALID, "NULL pointer");
    DevBuf dx, dout;
    const size_t out_bytes = (size_t)(n / block_elems(dt) * block_bytes(dt));
    if ((rc = dx.reserve((size_t)n * 4))) return rc;
    if ((rc = dout.reserve(out_bytes))) return rc;
    MOE_HIP_CHECK(hipMemcpy(dx.p, x, (size_t)n * 4, hipMemcpyHostToDevice));
    MOE_HIP_CHECK(launch_quantize_weights(dt, dx.as<float>(), n, dout.as<uint8_t>(), nullptr));
    MOE_HIP_CHECK(hipDeviceSynchronize());
    return d2h(out, dout.p, out_bytes);
}

// ------------------------------------------------------------------ rms-norm as an operation of its own
static int check_rms_args(const void* x, const void* alpha, int64_t rows, int64_t hidden, const void* y, const char* who) {
    if (rows < 0 || hidden <= 0 || hidden > 16256) return fail(MOE_E_INVALID, std::string(who) + ": need rows >= 0 and 0 < hidden <= 16256");
    if (rows > 0 && (!x || !alpha || !y)) return fail(MOE_E_INVALID, std::string(who) + ": NULL pointer");
    if (hidden % 4) return fail(MOE_E_INVALID, std::string(who) + ": hidden must be a multiple of 4");
    return MOE_OK;
}

extern "C" int moe_add_rms_norm_device(const void* d_x, const void* d_residual, const void* d_alpha, float eps, int64_t rows, int64_t hidden,
                                       void* d_sum, void* d_y, void* hip_stream) {
    int rc = ensure_device();
    if (rc) return rc;
    if ((rc = check_rms_args(d_x, d_alpha, rows, hidden, d_y, "moe_add_rms_norm_device"))) return rc;
    if (rows == 0) return MOE_OK;
    if (d_residual && !d_sum) return fail(MOE_E_INVALID, "moe_add_rms_norm_device: d_sum must be given with d_residual");
    MOE_HIP_CHECK(launch_add_rms_norm(static_cast<const float*>(d_x), static_cast<const float*>(d_residual), static_cast<const float*>(d_alpha), eps,
                                      rows, (int)hidden, static_cast<float*>(d_sum), static_cast<float*>(d_y), static_cast<hipStream_t>(hip_stream)));
    return MOE_OK;
}

extern "C" int moe_rms_norm(const float* x, const float* alpha, float eps, int64_t rows, int64_t hidden, float* y) {
    int rc = ensure_device();
    if (rc) return rc;
    if ((rc = check_rms_args(x, alpha, rows, hidden, y, "moe_rms_norm"))) return rc;
    if (rows == 0) return MOE_OK;
    DevBuf dx, da, dy;
    const size_t bytes = (size_t)rows * hidden * 4;
    if ((rc = dx.reserve(bytes))) return rc;
    if ((rc = dy.reserve(bytes))) return rc;
    if ((rc = da.reserve((size_t)hidden * 4))) return rc;
    MOE_HIP_CHECK(hipMemcpy(dx.p, x, bytes, hipMemcpyHostToDevice));
    MOE_HIP_CHECK(hipMemcpy(da.p, alpha, (size_t)hidden * 4, hipMemcpyHostToDevice));
    MOE_HIP_CHECK(launch_add_rms_norm(dx.as<float>(), nullptr, da.as<float>(), eps, rows, (int)hidden, nullptr, dy.as<float>(), nullptr));
    MOE_HIP_CHECK(hipDeviceSynchronize());
    return d2h(y, dy.p, bytes);
}

extern "C" int moe_debug_set_switch(const char* name, int64_t value) {
    if (!name) return fail(MOE_E_INVALID, "moe_debug_set_switch: name is NULL");
    Switches& sw = switches();
    const std::string n(name);
    if (n == "combine_pass") sw.combine_pass = value != 0;
    else if (n == "rms_serial") sw.rms_serial = value != 0;
    else if (n == "max_tokens_per_pass") sw.max_tokens_per_pass = value;
    else if (n == "no_gemm") sw.no_gemm = value != 0;
    else if (n == "front_generic") sw.front_generic = value != 0;
    else if (n == "tile_slots") sw.tile_slots = (int)value;
    else if (n == "slot_tiles") sw.slot_tiles = (int)value;
    else if (n == "narrow") sw.narrow = (int)value;
    else if (n == "fused_rows") sw.fused_rows = (int)value;
    else if (n == "front_split") sw.front_split = (int)value;
    else if (n == "dispatch_one") sw.dispatch_one = (int)value;
    else return fail(MOE_E_INVALID, "moe_debug_set_switch: unknown switch '" + n + "'");
    return MOE_OK;
}

extern "C" const char* moe_last_error(void) { return g_err.c_str(); }

#ifndef MOE_BUILD_ID
#define MOE_BUILD_ID "unknown"
#endif
extern "C" const char* moe_build_id(void) { return MOE_BUILD_ID; }

extern "C" const char* moe_device_arch(void) {
    if (ensure_device()) return nullptr;
    return g_arch.c_str();
}

extern "C" float moe_debug_expf(float x) { return expf_glibc(x); }
