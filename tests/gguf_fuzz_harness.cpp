// Host-only robustness check of the GGUF reader: the library's gguf.cpp is compiled with AddressSanitizer and
// UndefinedBehaviorSanitizer (no GPU code), the entry points that would touch the GPU are replaced by stubs that
// read every byte the reader hands them, and mutated copies of a valid file are pushed through every public call.
// A reader that follows a hostile length, offset or dimension out of the mapping dies here.
//
// usage: gguf_fuzz <valid.gguf> <scratch path> <iterations> <seed>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../include/candle_amd_moe.h"

namespace moe {
static thread_local std::string g_err;
void set_error(int, const std::string& msg) { g_err = msg; }
int fail(int code, const std::string& msg) { g_err = msg; return code; }
int ensure_device() { return MOE_OK; }
}  // namespace moe

static volatile uint64_t g_sink;
static void touch(const void* p, uint64_t n) {
    const uint8_t* b = static_cast<const uint8_t*>(p);
    uint64_t s = 0;
    for (uint64_t i = 0; i < n; i++) s += b[i];
    g_sink += s;
}
static uint64_t blocks_bytes(int dt, int64_t elems) {
    switch (dt) {
        case MOE_GGML_Q4_0: return (uint64_t)elems / 32 * 18;
        case MOE_GGML_Q8_0: return (uint64_t)elems / 32 * 34;
        case MOE_GGML_Q2K: return (uint64_t)elems / 256 * 84;
        case MOE_GGML_Q3K: return (uint64_t)elems / 256 * 110;
        case MOE_GGML_Q4K: return (uint64_t)elems / 256 * 144;
        case MOE_GGML_Q5K: return (uint64_t)elems / 256 * 176;
        case MOE_GGML_Q6K: return (uint64_t)elems / 256 * 210;
    }
    return 0;
}

extern "C" const char* moe_last_error(void) { return moe::g_err.c_str(); }
extern "C" int moe_dequantize(int32_t dt, const void* blocks, int64_t n, float* out) {
    touch(blocks, blocks_bytes(dt, n));
    for (int64_t i = 0; i < n; i++) out[i] = 0.f;
    return MOE_OK;
}
extern "C" int moe_layer_create(const moe_desc* d, moe_layer** out) {
    // what the real constructor reads: E matrices of hidden*ffn elements per family, the gate
    const int dtd = d->ggml_dtype_down ? d->ggml_dtype_down : d->ggml_dtype;
    touch(d->gate, (uint64_t)d->n_experts * d->hidden * 4);
    for (int64_t e = 0; e < d->n_experts; e++) {
        touch(d->w1[e], blocks_bytes(d->ggml_dtype, d->hidden * d->ffn));
        touch(d->w3[e], blocks_bytes(d->ggml_dtype, d->hidden * d->ffn));
        touch(d->w2[e], blocks_bytes(dtd, d->hidden * d->ffn));
    }
    *out = nullptr;
    return MOE_E_NODEVICE;
}
extern "C" int moe_qlinear_create(int32_t dt, const void* w, int64_t n, int64_t k, moe_qlinear** out) {
    touch(w, blocks_bytes(dt, n * k));
    *out = nullptr;
    return MOE_E_NODEVICE;
}

static uint64_t rng_state;
static uint64_t rnd() {
    rng_state += 0x9E3779B97F4A7C15ull;
    uint64_t z = rng_state;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static void exercise(const char* path) {
    moe_gguf* g = nullptr;
    if (moe_gguf_open(path, &g) != MOE_OK) return;
    (void)moe_gguf_version(g);
    (void)moe_gguf_tensor_data_offset(g);
    const int64_t nt = moe_gguf_tensor_count(g);
    for (int64_t i = 0; i < nt && i < 4096; i++) {
        const char* name = moe_gguf_tensor_name(g, i);
        if (!name) continue;
        int dt = 0, nd = 0;
        int64_t dims[8];
        const void* data = nullptr;
        uint64_t nbytes = 0;
        if (moe_gguf_tensor(g, name, &dt, &nd, dims, &data, &nbytes) == MOE_OK) touch(data, nbytes);
        moe_qlinear* q = nullptr;
        (void)moe_qlinear_create_from_gguf(g, name, &q);
    }
    static const char* keys[] = {"general.architecture", "general.alignment", "llama.expert_count", "llama.expert_used_count",
                                 "llama.embedding_length", "tokenizer.ggml.tokens", "missing.key"};
    for (const char* key : keys) {
        int vt = 0;
        uint64_t u = 0, len = 0;
        int64_t iv = 0;
        double f = 0;
        char buf[64];
        (void)moe_gguf_metadata_type(g, key, &vt);
        (void)moe_gguf_metadata_u64(g, key, &u);
        (void)moe_gguf_metadata_i64(g, key, &iv);
        (void)moe_gguf_metadata_f64(g, key, &f);
        (void)moe_gguf_metadata_str(g, key, buf, sizeof buf);
        (void)moe_gguf_metadata_array_len(g, key, &len, &vt);
    }
    for (int layer = 0; layer < 2; layer++) {
        moe_layer* l = nullptr;
        (void)moe_layer_create_from_gguf(g, layer, 1, &l);
    }
    moe_gguf_close(g);
}

int main(int argc, char** argv) {
    if (argc != 5) return 2;
    FILE* f = fopen(argv[1], "rb");
    if (!f) return 2;
    std::vector<uint8_t> good;
    uint8_t tmp[65536];
    size_t n;
    while ((n = fread(tmp, 1, sizeof tmp, f)) > 0) good.insert(good.end(), tmp, tmp + n);
    fclose(f);
    const int iters = atoi(argv[3]);
    rng_state = strtoull(argv[4], nullptr, 10);
    exercise(argv[1]);   // the unmodified file first
    // the tables end where the tensor data starts; mutations concentrate there
    size_t tables = good.size() < 4096 ? good.size() : 4096;
    for (int it = 0; it < iters; it++) {
        std::vector<uint8_t> m = good;
        const int kind = (int)(rnd() % 4);
        if (kind == 0) {                       // flip a few bytes of the tables
            const int flips = 1 + (int)(rnd() % 4);
            for (int j = 0; j < flips; j++) m[rnd() % tables] = (uint8_t)rnd();
        } else if (kind == 1) {                // overwrite an aligned 8-byte field with an extreme value
            static const uint64_t extremes[] = {0, 1, 0x7fffffffffffffffull, 0xffffffffffffffffull, 0x8000000000000000ull, 1ull << 32, (1ull << 40) + 7};
            const size_t at = (rnd() % (tables > 8 ? tables - 8 : 1));
            const uint64_t v = extremes[rnd() % 7];
            memcpy(&m[at], &v, at + 8 <= m.size() ? 8 : 0);
        } else if (kind == 2) {                // truncate
            m.resize(rnd() % (m.size() + 1));
        } else {                               // flip one bit anywhere in the tables
            m[rnd() % tables] ^= (uint8_t)(1u << (rnd() % 8));
        }
        FILE* o = fopen(argv[2], "wb");
        if (!o) return 2;
        if (!m.empty()) fwrite(m.data(), 1, m.size(), o);
        fclose(o);
        exercise(argv[2]);
    }
    printf("gguf fuzz: %d mutants survived\n", iters);
    return 0;
}
