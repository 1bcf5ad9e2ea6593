// GGUF container reader for the expert loader (host code only).
//
// Restates `Content::read` of candle-core/src/quantized/gguf_file.rs:439-511 on a memory-mapped file:
// magic and version (:16-45), counts (u32 in version 1, u64 from version 2 on), the metadata key/value
// table (`Value::read`, :296-357; strings :135-150 with trailing NULs dropped), the tensor table
// (name, dimensions stored innermost first and reversed on read, GgmlDType id, offset; :467-494) and
// the start of the tensor data, the position after the tables rounded up to `general.alignment`
// (default 32; :496-505).  Tensor bytes are handed out as pointers into the mapping
// (`TensorInfo::read_from_mmap`, :91-126), with the same size and bounds checks.
//
// `moe_layer_create_from_gguf` then does for ONE layer what `ModelWeights::from_gguf` does for the MoE
// arm (candle-transformers/src/models/quantized_llama.rs:506-512, 553-578): `llama.expert_count`,
// `llama.expert_used_count`, `blk.{l}.ffn_gate_inp.weight` and `blk.{l}.ffn_{gate,down,up}.{i}.weight`
// as w1 / w2 / w3.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstring>
#include <new>
#include <stdexcept>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "moe_common.hpp"

namespace {

using moe::fail;

struct Value {
    uint32_t type = 0;          // ValueType id, gguf_file.rs:402-420
    uint64_t u = 0;             // integers and bool
    int64_t i = 0;
    double f = 0.0;
    std::string s;
    std::vector<Value> arr;
};

struct TensorInfo {
    int ggml_dtype = 0;
    std::vector<int64_t> dims;  // outermost first, as candle's Shape
    uint64_t offset = 0;
};

// (block elements, block bytes) per GgmlDType id; candle-core/src/quantized/mod.rs:153-174, 218-252
bool dtype_geometry(int dt, uint64_t* elems, uint64_t* bytes) {
    switch (dt) {
        case 0: *elems = 1; *bytes = 4; return true;       // F32
        case 1: *elems = 1; *bytes = 2; return true;       // F16
        case 2: *elems = 32; *bytes = 18; return true;     // Q4_0
        case 3: *elems = 32; *bytes = 20; return true;     // Q4_1
        case 6: *elems = 32; *bytes = 22; return true;     // Q5_0
        case 7: *elems = 32; *bytes = 24; return true;     // Q5_1
        case 8: *elems = 32; *bytes = 34; return true;     // Q8_0
        case 9: *elems = 32; *bytes = 36; return true;     // Q8_1
        case 10: *elems = 256; *bytes = 84; return true;   // Q2K
        case 11: *elems = 256; *bytes = 110; return true;  // Q3K
        case 12: *elems = 256; *bytes = 144; return true;  // Q4K
        case 13: *elems = 256; *bytes = 176; return true;  // Q5K
        case 14: *elems = 256; *bytes = 210; return true;  // Q6K
        case 15: *elems = 256; *bytes = 292; return true;  // Q8K
        case 30: *elems = 1; *bytes = 2; return true;      // BF16
        default: return false;
    }
}

struct Reader {
    const uint8_t* p;
    size_t len, pos = 0;
    int version = 0;
    bool ok = true;
    template <typename T>
    T get() {
        T v{};
        if (pos + sizeof(T) > len) { ok = false; pos = len; return v; }
        memcpy(&v, p + pos, sizeof(T));
        pos += sizeof(T);
        return v;
    }
    uint64_t count() { return version == 1 ? get<uint32_t>() : get<uint64_t>(); }
    std::string str() {
        const uint64_t n = count();
        if (!ok || n > len - pos) { ok = false; pos = len; return {}; }
        std::string s(reinterpret_cast<const char*>(p + pos), (size_t)n);
        pos += (size_t)n;
        while (!s.empty() && s.back() == '\0') s.pop_back();
        return s;
    }
};

bool read_value(Reader& r, uint32_t type, Value& v, int depth, std::string& err) {
    v.type = type;
    switch (type) {
        case 0: v.u = r.get<uint8_t>(); break;
        case 1: v.i = r.get<int8_t>(); break;
        case 2: v.u = r.get<uint16_t>(); break;
        case 3: v.i = r.get<int16_t>(); break;
        case 4: v.u = r.get<uint32_t>(); break;
        case 5: v.i = r.get<int32_t>(); break;
        case 6: v.f = r.get<float>(); break;
        case 7: {
            const uint8_t b = r.get<uint8_t>();
            if (b > 1) { err = "unexpected bool value " + std::to_string(b); return false; }
            v.u = b;
            break;
        }
        case 8: v.s = r.str(); break;
        case 9: {
            if (depth > 8) { err = "arrays nested too deeply"; return false; }
            const uint32_t et = r.get<uint32_t>();
            if (et > 12) { err = "unrecognized value-type " + std::to_string(et); return false; }
            const uint64_t n = r.count();
            if (!r.ok || n > r.len - r.pos) { err = "array length past the end of the file"; return false; }   // every element takes a byte or more
            v.arr.resize((size_t)n);
            for (auto& e : v.arr)
                if (!read_value(r, et, e, depth + 1, err)) return false;
            break;
        }
        case 10: v.u = r.get<uint64_t>(); break;
        case 11: v.i = r.get<int64_t>(); break;
        case 12: v.f = r.get<double>(); break;
        default: err = "unrecognized value-type " + std::to_string(type); return false;
    }
    if (!r.ok) { err = "unexpected end of file in the metadata"; return false; }
    return true;
}

}  // namespace

struct moe_gguf {
    int fd = -1;
    const uint8_t* map = nullptr;
    size_t len = 0;
    int version = 0;
    uint64_t tensor_data_offset = 0;
    std::map<std::string, Value> metadata;
    std::map<std::string, TensorInfo> tensors;
    std::vector<std::string> tensor_names;  // file order
    ~moe_gguf() {
        if (map) munmap(const_cast<uint8_t*>(map), len);
        if (fd >= 0) close(fd);
    }
};

static int gguf_open_impl(const char* path, moe_gguf** out);

extern "C" int moe_gguf_open(const char* path, moe_gguf** out) {
    if (!path || !out) return fail(MOE_E_INVALID, "moe_gguf_open: NULL argument");
    *out = nullptr;
    try {
        return gguf_open_impl(path, out);
    } catch (const std::bad_alloc&) {   // a table that claims more entries than memory holds
        return fail(MOE_E_NOMEM, std::string(path) + ": out of memory while reading the GGUF tables");
    } catch (const std::exception& e) {
        return fail(MOE_E_INVALID, std::string(path) + ": " + e.what());
    }
}

static int gguf_open_impl(const char* path, moe_gguf** out) {
    auto g = std::make_unique<moe_gguf>();
    g->fd = open(path, O_RDONLY);
    if (g->fd < 0) return fail(MOE_E_INVALID, std::string("cannot open ") + path + ": " + strerror(errno));
    struct stat st;
    if (fstat(g->fd, &st) != 0 || st.st_size < 8) return fail(MOE_E_INVALID, std::string(path) + ": not a GGUF file (too short)");
    g->len = (size_t)st.st_size;
    void* m = mmap(nullptr, g->len, PROT_READ, MAP_PRIVATE, g->fd, 0);
    if (m == MAP_FAILED) return fail(MOE_E_NOMEM, std::string("mmap failed for ") + path + ": " + strerror(errno));
    g->map = static_cast<const uint8_t*>(m);

    Reader r{g->map, g->len};
    const uint32_t magic = r.get<uint32_t>();
    if (magic != 0x46554747u && magic != 0x47475546u) {
        char b[32];
        snprintf(b, sizeof b, "0x%08x", magic);
        return fail(MOE_E_INVALID, std::string("unknown magic ") + b);
    }
    const uint32_t version = r.get<uint32_t>();
    if (version < 1 || version > 3) return fail(MOE_E_INVALID, "gguf: unsupported version " + std::to_string(version));
    r.version = g->version = (int)version;
    const uint64_t tensor_count = r.count();
    const uint64_t kv_count = r.count();
    if (!r.ok || tensor_count > g->len || kv_count > g->len) return fail(MOE_E_INVALID, "gguf: truncated header");
    std::string err;
    for (uint64_t i = 0; i < kv_count; i++) {
        std::string key = r.str();
        const uint32_t vt = r.get<uint32_t>();
        Value v;
        if (!r.ok) return fail(MOE_E_INVALID, "gguf: unexpected end of file in the metadata");
        if (!read_value(r, vt, v, 0, err)) return fail(MOE_E_INVALID, "gguf: " + err + " (key " + key + ")");
        g->metadata[key] = std::move(v);
    }
    for (uint64_t i = 0; i < tensor_count; i++) {
        std::string name = r.str();
        const uint32_t nd = r.get<uint32_t>();
        if (!r.ok || nd > 8) return fail(MOE_E_INVALID, "gguf: bad tensor table entry " + std::to_string(i));
        TensorInfo ti;
        ti.dims.resize(nd);
        for (uint32_t d = 0; d < nd; d++) ti.dims[nd - 1 - d] = (int64_t)r.count();   // stored innermost first
        const uint32_t dt = r.get<uint32_t>();
        uint64_t be, bb;
        if (!dtype_geometry((int)dt, &be, &bb)) return fail(MOE_E_INVALID, "unknown dtype for tensor " + std::to_string(dt));
        ti.ggml_dtype = (int)dt;
        ti.offset = r.get<uint64_t>();
        if (!r.ok) return fail(MOE_E_INVALID, "gguf: unexpected end of file in the tensor table");
        g->tensor_names.push_back(name);
        g->tensors[name] = std::move(ti);
    }
    uint64_t alignment = 32;
    auto it = g->metadata.find("general.alignment");
    if (it != g->metadata.end()) {
        const Value& v = it->second;
        if (v.type == 0 || v.type == 2 || v.type == 4) alignment = v.u;
        else if ((v.type == 1 || v.type == 3 || v.type == 5) && v.i >= 0) alignment = (uint64_t)v.i;
    }
    if (alignment == 0 || alignment > (1u << 30)) return fail(MOE_E_INVALID, "gguf: general.alignment is " + std::to_string(alignment));
    g->tensor_data_offset = (r.pos + alignment - 1) / alignment * alignment;
    *out = g.release();
    return MOE_OK;
}

extern "C" void moe_gguf_close(moe_gguf* g) { delete g; }

extern "C" int moe_gguf_version(const moe_gguf* g) { return g ? g->version : 0; }
extern "C" int64_t moe_gguf_tensor_count(const moe_gguf* g) { return g ? (int64_t)g->tensor_names.size() : 0; }
extern "C" uint64_t moe_gguf_tensor_data_offset(const moe_gguf* g) { return g ? g->tensor_data_offset : 0; }

extern "C" const char* moe_gguf_tensor_name(const moe_gguf* g, int64_t index) {
    if (!g || index < 0 || index >= (int64_t)g->tensor_names.size()) return nullptr;
    return g->tensor_names[(size_t)index].c_str();
}

static const Value* find_value(const moe_gguf* g, const char* key) {
    if (!g || !key) { fail(MOE_E_INVALID, "moe_gguf: NULL argument"); return nullptr; }
    auto it = g->metadata.find(key);
    if (it == g->metadata.end()) { fail(MOE_E_INVALID, std::string("cannot find ") + key + " in metadata"); return nullptr; }
    return &it->second;
}

extern "C" int moe_gguf_metadata_type(const moe_gguf* g, const char* key, int* value_type) {
    const Value* v = find_value(g, key);
    if (!v) return MOE_E_INVALID;
    if (value_type) *value_type = (int)v->type;
    return MOE_OK;
}

extern "C" int moe_gguf_metadata_u64(const moe_gguf* g, const char* key, uint64_t* out) {
    const Value* v = find_value(g, key);
    if (!v || !out) return MOE_E_INVALID;
    // Value::to_u64 upcasts the unsigned types and bool (gguf_file.rs:268-279)
    if (v->type == 0 || v->type == 2 || v->type == 4 || v->type == 7 || v->type == 10) { *out = v->u; return MOE_OK; }
    return fail(MOE_E_INVALID, std::string(key) + ": not a u64 or upcastable to u64");
}

extern "C" int moe_gguf_metadata_i64(const moe_gguf* g, const char* key, int64_t* out) {
    const Value* v = find_value(g, key);
    if (!v || !out) return MOE_E_INVALID;
    if (v->type == 1 || v->type == 3 || v->type == 5 || v->type == 11) { *out = v->i; return MOE_OK; }
    return fail(MOE_E_INVALID, std::string(key) + ": not a signed integer");
}

extern "C" int moe_gguf_metadata_f64(const moe_gguf* g, const char* key, double* out) {
    const Value* v = find_value(g, key);
    if (!v || !out) return MOE_E_INVALID;
    if (v->type == 6 || v->type == 12) { *out = v->f; return MOE_OK; }
    return fail(MOE_E_INVALID, std::string(key) + ": not a float");
}

extern "C" int moe_gguf_metadata_str(const moe_gguf* g, const char* key, char* buf, uint64_t cap) {
    const Value* v = find_value(g, key);
    if (!v || !buf || cap == 0) return MOE_E_INVALID;
    if (v->type != 8) return fail(MOE_E_INVALID, std::string(key) + ": not a string");
    if (v->s.size() + 1 > cap) return fail(MOE_E_INVALID, std::string(key) + ": buffer too small");
    memcpy(buf, v->s.c_str(), v->s.size() + 1);
    return MOE_OK;
}

extern "C" int moe_gguf_metadata_array_len(const moe_gguf* g, const char* key, uint64_t* len, int* elem_type) {
    const Value* v = find_value(g, key);
    if (!v) return MOE_E_INVALID;
    if (v->type != 9) return fail(MOE_E_INVALID, std::string(key) + ": not an array");
    if (len) *len = v->arr.size();
    if (elem_type) *elem_type = v->arr.empty() ? 4 : (int)v->arr[0].type;
    return MOE_OK;
}

extern "C" int moe_gguf_tensor(const moe_gguf* g, const char* name, int* ggml_dtype, int* n_dims, int64_t dims[8], const void** data,
                               uint64_t* nbytes) {
    if (!g || !name) return fail(MOE_E_INVALID, "moe_gguf_tensor: NULL argument");
    auto it = g->tensors.find(name);
    if (it == g->tensors.end()) return fail(MOE_E_INVALID, std::string("cannot find tensor info for ") + name);
    const TensorInfo& ti = it->second;
    uint64_t elems = 1;
    for (int64_t d : ti.dims) {   // a hostile table must not wrap the element count around
        if (d < 0 || (d > 0 && elems > UINT64_MAX / (uint64_t)d))
            return fail(MOE_E_INVALID, std::string(name) + ": tensor dimensions overflow");
        elems *= (uint64_t)d;
    }
    uint64_t be = 1, bb = 1;
    dtype_geometry(ti.ggml_dtype, &be, &bb);
    if (elems % be)
        return fail(MOE_E_INVALID, "the number of elements " + std::to_string(elems) + " is not divisible by the block size " + std::to_string(be));
    if (elems / be > UINT64_MAX / bb) return fail(MOE_E_INVALID, std::string(name) + ": tensor dimensions overflow");
    const uint64_t size = elems / be * bb;
    const uint64_t start = g->tensor_data_offset + ti.offset;
    if (ti.offset > g->len || start > g->len || size > g->len - start)
        return fail(MOE_E_INVALID, "tensor data extends beyond file boundary: offset=" + std::to_string(start) + ", size=" + std::to_string(size) +
                                       ", file_len=" + std::to_string(g->len));
    if (ggml_dtype) *ggml_dtype = ti.ggml_dtype;
    if (n_dims) *n_dims = (int)ti.dims.size();
    if (dims)
        for (size_t d = 0; d < ti.dims.size(); d++) dims[d] = ti.dims[d];
    if (data) *data = g->map + start;
    if (nbytes) *nbytes = size;
    return MOE_OK;
}

static float half_bits_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu, bits;
    if (exp == 0) {
        if (man == 0) bits = sign;
        else {
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
    else bits = sign | ((exp + 112) << 23) | (man << 13);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

extern "C" int moe_layer_create_from_gguf(const moe_gguf* g, int layer_index, int norm_topk, moe_layer** out) {
    if (!g || !out || layer_index < 0) return fail(MOE_E_INVALID, "moe_layer_create_from_gguf: bad argument");
    *out = nullptr;
    // quantized_llama.rs:507-512: both keys default to 0 when absent
    // (`md_get(..).and_then(|v| v.to_u32()).unwrap_or(0)`: `Value::to_u32`, gguf_file.rs:249-254, takes the U32 variant
    // only, so a key of any other type counts as 0 too instead of failing the load)
    auto u32_or_zero = [&](const char* key) -> uint64_t {
        const Value* v = find_value(g, key);
        return v && v->type == 4 ? v->u : 0;
    };
    const uint64_t n_expert = u32_or_zero("llama.expert_count"), n_used = u32_or_zero("llama.expert_used_count");
    if (n_expert <= 1) return fail(MOE_E_INVALID, "llama.expert_count is " + std::to_string(n_expert) + ": the file has dense feed-forward layers, no MoE block");
    // n_used == 0 (key absent or zero): the reference builds the block all the same and its forward selects no expert
    // (`take(0)`, quantized_llama.rs:167): a layer with top_k = 0 whose output is zero
    const std::string prefix = "blk." + std::to_string(layer_index);

    int dt = 0, nd = 0;
    int64_t dims[8];
    const void* data = nullptr;
    uint64_t nbytes = 0;
    int rc = moe_gguf_tensor(g, (prefix + ".ffn_gate_inp.weight").c_str(), &dt, &nd, dims, &data, &nbytes);
    if (rc) return rc;
    if (nd != 2 || (uint64_t)dims[0] != n_expert) return fail(MOE_E_INVALID, prefix + ".ffn_gate_inp.weight: expected shape [expert_count, hidden]");
    const int64_t E = dims[0], H = dims[1];
    int gate_dtype = 0;
    const void* gate_blocks = nullptr;
    std::vector<float> gate((size_t)(E * H));
    if (dt == 0) memcpy(gate.data(), data, gate.size() * 4);
    else if (dt == 1) {
        const uint16_t* h = static_cast<const uint16_t*>(data);
        for (size_t i = 0; i < gate.size(); i++) gate[i] = half_bits_to_float(h[i]);
    } else if (dt == 30) {   // BF16: the upper half of an f32
        const uint16_t* h = static_cast<const uint16_t*>(data);
        for (size_t i = 0; i < gate.size(); i++) {
            const uint32_t bits = (uint32_t)h[i] << 16;
            memcpy(&gate[i], &bits, 4);
        }
    } else {
        // QMatMul::from_arc (candle-core/src/quantized/mod.rs:429-443) dequantises F32, F16 and BF16 only; any other
        // router tensor stays a QTensor and its logits are a quantised product over Q8-quantised rows (moe_desc.gate_dtype)
        gate_dtype = dt;
        gate_blocks = data;
    }

    std::vector<const void*> w1((size_t)E), w2((size_t)E), w3((size_t)E);
    int up_dt = -1, down_dt = -1;   // gate / up matrices share one dtype, down matrices one
    int64_t F = -1;
    for (int64_t e = 0; e < E; e++) {
        struct { const char* stem; std::vector<const void*>* dst; bool up; } parts[3] = {{"ffn_gate", &w1, true}, {"ffn_down", &w2, false}, {"ffn_up", &w3, true}};
        for (auto& part : parts) {
            const std::string name = prefix + "." + part.stem + "." + std::to_string(e) + ".weight";
            if ((rc = moe_gguf_tensor(g, name.c_str(), &dt, &nd, dims, &data, &nbytes))) return rc;
            if (nd != 2) return fail(MOE_E_INVALID, name + ": expected a matrix");
            if (F < 0) F = part.up ? dims[0] : dims[1];
            int& want = part.up ? up_dt : down_dt;
            if (want < 0) want = dt;
            if (dt != want)
                return fail(MOE_E_INVALID, name + ": dtype " + std::to_string(dt) + " differs from the layer's other " + (part.up ? "gate / up" : "down") +
                                               " matrices (" + std::to_string(want) + ")");
            const int64_t rows = part.up ? F : H, cols = part.up ? H : F;
            if (dims[0] != rows || dims[1] != cols)
                return fail(MOE_E_INVALID, name + ": shape [" + std::to_string(dims[0]) + ", " + std::to_string(dims[1]) + "] does not match hidden " + std::to_string(H) +
                                               " / ffn " + std::to_string(F));
            (*part.dst)[(size_t)e] = data;
        }
    }
    moe_desc d;
    memset(&d, 0, sizeof d);
    d.hidden = H; d.ffn = F; d.n_experts = E; d.top_k = (int64_t)n_used;
    d.ggml_dtype = up_dt; d.ggml_dtype_down = down_dt == up_dt ? 0 : down_dt; d.norm_topk = norm_topk;
    d.gate = gate.data();
    d.gate_dtype = gate_dtype; d.gate_blocks = gate_blocks;
    d.w1 = w1.data(); d.w3 = w3.data(); d.w2 = w2.data();
    return moe_layer_create(&d, out);
}

// One named matrix of the file as a resident dense projection: what `QMatMul::from_qtensor(ct.tensor(
// reader, name, device)?)` builds for `blk.{l}.attn_q.weight` ... `output.weight`
// (quantized_llama.rs:533-547, 590-593, 608).
extern "C" int moe_qlinear_create_from_gguf(const moe_gguf* g, const char* tensor_name, moe_qlinear** out) {
    if (out) *out = nullptr;
    if (!g || !tensor_name || !out) return fail(MOE_E_INVALID, "moe_qlinear_create_from_gguf: bad argument");
    int dt = 0, nd = 0;
    int64_t dims[8];
    const void* data = nullptr;
    uint64_t nbytes = 0;
    int rc = moe_gguf_tensor(g, tensor_name, &dt, &nd, dims, &data, &nbytes);
    if (rc) return rc;
    if (nd != 2) return fail(MOE_E_INVALID, std::string(tensor_name) + ": a projection matrix has two dimensions, this tensor has " + std::to_string(nd));
    if (!moe::weight_dtype_supported(dt))
        return fail(MOE_E_INVALID, std::string(tensor_name) + ": unsupported dtype " + std::to_string(dt) + " (supported: Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2K, Q3K, Q4K, Q5K, Q6K)");
    return moe_qlinear_create(dt, data, dims[0], dims[1], out);
}
