// Tiled grouped expert products for large batches (prefill): Q4K weights x Q8K activations on
// v_mfma_i32_32x32x32_i8, the full-rate int8 MFMA shape of gfx950 whose K = 32 is one Q4K sub-block.
//
// Same integers as BlockQ4K::vec_dot (candle-core/src/quantized/k_quants.rs:1205-1285):
//     sum_j sc_j * (q4_j . q8_j)      and      sum_j m_j * (bsum_2j + bsum_2j+1).
// Applying the 6-bit scale to every 32x32 block of MFMA results would cost 16 integer multiply-adds
// per lane and instruction -- twice the time of the instruction itself -- so the scale is moved into
// the weight operand instead: sc = 8*hi + lo with hi, lo <= 7, and the two byte planes hi*q4 and
// lo*q4 (<= 105, no carry between bytes) are multiplied by the activations in two MFMAs that
// accumulate over the whole 256-element super-block.  8*acc_hi + acc_lo is then the exact integer
// the reference computes; the mins term is an exact f16 MFMA over the 16 block sums.
//
// Work split: a workgroup owns one tile of 64 slots of one expert (from the dispatch kernel's tile
// list, so a skewed routing is balanced by tiles, not by experts) and four 32-row operands; the 64
// activation rows of a super-block are staged once in LDS (double-buffered) and every wave reads them
// as MFMA A operands, while each wave unpacks and pre-scales its own 32 weight rows in registers.
#include "act_quant.hpp"
#include "kernels.hpp"

namespace moe {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef const __attribute__((address_space(1))) uint8_t* gbytes;

template <typename T>
__device__ __forceinline__ T gld(const void* uniform_base, uint32_t off) {
    return *reinterpret_cast<const __attribute__((address_space(1))) T*>((gbytes)uniform_base + off);
}

// four bytes (each <= 15) times a digit (<= 7): no byte overflows, and the packed 16-bit multiply does
// both halves of the register in one full-rate instruction (a 24-bit multiply would drop the top byte)
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t scale_bytes(uint32_t q, uint32_t s) {
    const u16x2 a = __builtin_bit_cast(u16x2, q);
    const u16x2 b = {(unsigned short)s, (unsigned short)s};
    return __builtin_bit_cast(uint32_t, (u16x2)(a * b));
}

constexpr int GT = GEMM_TILE_SLOTS;   // 64 slots per tile = two 32-row MFMA operands
constexpr int QSTRIDE = 272;          // LDS row stride of the quants (256 + 16: conflict-free b128 reads)
constexpr int G_THREADS = 256;

struct alignas(16) GemmLds {
    alignas(16) uint8_t q[2][GT * QSTRIDE];   // activation quants, natural k order inside a row
    alignas(16) _Float16 bs[2][GT][16];       // block sums
    alignas(16) float yd[2][GT];              // activation scales
};

// registers holding one thread's share of an activation tile on its way from global memory to LDS
struct AStage {
    u32x4 q[4];
    u32x4 bs;
    float yd;
};

// Thread t moves quant chunks c = t + 256*j (row c/16, piece c%16 = pair*4 + chunk), the block sums
// (row (t%128)/2, half t%2) and the scales (row t%64).  Every thread issues every load -- the upper
// threads repeat the lower ones' addresses and drop the result -- so that the loop body has no
// divergent branch around a load: with branches the compiler can no longer count the loads in flight
// and falls back to waiting for all of them at the top of the next iteration.
__device__ __forceinline__ AStage a_stage_load(const ActBuf& ab, int K, int nsb, int sb, const int rows4[4], int row_bs, int row_yd, int tid) {
    AStage st;
    const int piece = tid & 15;
#pragma unroll
    for (int j = 0; j < 4; j++)
        st.q[j] = gld<u32x4>(ab.qs, (uint32_t)rows4[j] * (uint32_t)K + (uint32_t)(sb * 256 + piece * 16));
    st.bs = gld<u32x4>(ab.bsum, (((uint32_t)row_bs * (uint32_t)nsb + (uint32_t)sb) * 16 + (tid & 1) * 8) * 2);
    st.yd = gld<float>(ab.d, ((uint32_t)row_yd * (uint32_t)nsb + (uint32_t)sb) * 4);
    return st;
}

__device__ __forceinline__ void a_stage_store(const AStage& st, GemmLds& L, int buf, int tid) {
    const int piece = tid & 15, P = piece >> 2, g = piece & 3;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int row = (tid >> 4) + 16 * j;
        uint8_t* base = L.q[buf] + row * QSTRIDE;
        // the 16 bytes are [sub-block 2P, chunk g | sub-block 2P+1, chunk g]
        *reinterpret_cast<u32x2*>(base + (2 * P) * 32 + g * 8) = u32x2{st.q[j].x, st.q[j].y};
        *reinterpret_cast<u32x2*>(base + (2 * P + 1) * 32 + g * 8) = u32x2{st.q[j].z, st.q[j].w};
    }
    // duplicates write the same value to the same place
    *reinterpret_cast<u32x4*>(&L.bs[buf][(tid & 127) >> 1][(tid & 1) * 8]) = st.bs;
    L.yd[buf][tid & 63] = st.yd;
}

// One wave's weights for one super-block: 32 rows = row tiles rt, rt+1 of the 16-row tile layout.
// Lane (n = l%32, half = l/32) owns row n and k-chunks 2*half, 2*half+1 of every sub-block.
struct BRegs {
    u32x4 c0[2], c1[2];   // [plane of the tile: pairs (0,1) / (2,3)]: chunk 2*half and chunk 2*half+1
    u32x4 hdr;            // d, dmin, 12 scale bytes of row n
};

__device__ __forceinline__ BRegs b_load(const uint8_t* tile_pair /* tile of row-tile rt at this super-block */, int lane) {
    const int n = lane & 31, half = lane >> 5;
    const uint32_t tile_off = (uint32_t)(n >> 4) * Q4K_TILE_BYTES;   // row tiles are adjacent in the [sb][rt] order
    const int r = n & 15;
    BRegs b;
#pragma unroll
    for (int pl = 0; pl < 2; pl++) {
        b.c0[pl] = gld<u32x4>(tile_pair, tile_off + pl * 1024 + ((2 * half) * 16 + r) * 16);
        b.c1[pl] = gld<u32x4>(tile_pair, tile_off + pl * 1024 + ((2 * half + 1) * 16 + r) * 16);
    }
    b.hdr = gld<u32x4>(tile_pair, tile_off + 2048 + r * 16);
    return b;
}

// accumulate one super-block of one 32-row weight operand against MT 32-slot activation operands
template <int MT>
__device__ __forceinline__ void gemm_superblock(const BRegs& b, const GemmLds& L, int buf, int lane, v16f facc[MT]) {
    const int m = lane & 31, half = lane >> 5;
    const uint32_t M4 = 0x0f0f0f0fu;
    const uint32_t u0 = b.hdr.y, u1 = b.hdr.z, u2 = b.hdr.w;
    const float d = __half2float(__ushort_as_half((unsigned short)(b.hdr.x & 0xffffu)));
    const float dmin = __half2float(__ushort_as_half((unsigned short)(b.hdr.x >> 16)));
    const uint32_t sc03 = u0 & 0x3f3f3f3fu;
    const uint32_t sc47 = (u2 & M4) | (((u0 >> 6) & 0x03030303u) << 4);
    const uint32_t m03 = u1 & 0x3f3f3f3fu;
    const uint32_t m47 = ((u2 >> 4) & M4) | (((u1 >> 6) & 0x03030303u) << 4);
    // scales split into two 3-bit digits, still one byte per sub-block
    const uint32_t lo03 = sc03 & 0x07070707u, hi03 = (sc03 >> 3) & 0x07070707u;
    const uint32_t lo47 = sc47 & 0x07070707u, hi47 = (sc47 >> 3) & 0x07070707u;

    v16i acc_hi[MT], acc_lo[MT];
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};  // first MFMA of a chain takes the constant 0 as C

#pragma unroll
    for (int s = 0; s < 8; s++) {
        // sub-block s = pair P (s/2), low (s even) or high (s odd) nibbles; pair P lives in plane P/2,
        // bytes (x,y) for P even and (z,w) for P odd of both chunk registers
        const int P = s >> 1, pl = P >> 1;
        const uint32_t w0 = (P & 1) ? b.c0[pl].z : b.c0[pl].x, w1 = (P & 1) ? b.c0[pl].w : b.c0[pl].y;
        const uint32_t w2 = (P & 1) ? b.c1[pl].z : b.c1[pl].x, w3 = (P & 1) ? b.c1[pl].w : b.c1[pl].y;
        const int sh = (s & 1) ? 4 : 0;
        const uint32_t q0 = (w0 >> sh) & M4, q1 = (w1 >> sh) & M4, q2 = (w2 >> sh) & M4, q3 = (w3 >> sh) & M4;
        const uint32_t lw = (s < 4) ? lo03 : lo47, hw = (s < 4) ? hi03 : hi47;
        const uint32_t slo = (lw >> (8 * (s & 3))) & 0xffu, shi = (hw >> (8 * (s & 3))) & 0xffu;
        const v4i blo = {(int)scale_bytes(q0, slo), (int)scale_bytes(q1, slo), (int)scale_bytes(q2, slo), (int)scale_bytes(q3, slo)};
        const v4i bhi = {(int)scale_bytes(q0, shi), (int)scale_bytes(q1, shi), (int)scale_bytes(q2, shi), (int)scale_bytes(q3, shi)};
#pragma unroll
        for (int t = 0; t < MT; t++) {
            const v4i a = *reinterpret_cast<const v4i*>(L.q[buf] + (t * 32 + m) * QSTRIDE + s * 32 + half * 16);
            acc_lo[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, blo, s == 0 ? zero16 : acc_lo[t], 0, 0, 0);
            acc_hi[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bhi, s == 0 ? zero16 : acc_hi[t], 0, 0, 0);
        }
    }
    // mins: k = 8*half + j is block sum j of this half; it belongs to sub-block 4*half + j/2
    const uint32_t mw = half ? m47 : m03;
    v8h mB;
#pragma unroll
    for (int j = 0; j < 8; j++) mB[j] = (_Float16)(int)((mw >> (8 * (j >> 1))) & 0xffu);
#pragma unroll
    for (int t = 0; t < MT; t++) {
        const v8h mA = *reinterpret_cast<const v8h*>(&L.bs[buf][t * 32 + m][half * 8]);
        const v16f zf = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const v16f Dm = __builtin_amdgcn_mfma_f32_32x32x16_f16(mA, mB, zf, 0, 0, 0);
        // D[i] belongs to slot (i/4)*8 + half*4 + i%4 of operand t, weight row n = lane%32
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
            typedef float v4fl __attribute__((ext_vector_type(4)));
            const v4fl yd = *reinterpret_cast<const v4fl*>(&L.yd[buf][t * 32 + i4 * 8 + half * 4]);
            const float ydv[4] = {yd.x, yd.y, yd.z, yd.w};
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const int i = i4 * 4 + c;
                const int isum = (acc_hi[t][i] << 3) + acc_lo[t][i];
                const float v = __builtin_fmaf(d, (float)isum, -(dmin * Dm[i]));
                facc[t][i] = __builtin_fmaf(ydv[c], v, facc[t][i]);
            }
        }
    }
}

__device__ __forceinline__ float silu_gemm(float v) { return v / (1.0f + __expf(-v)); }

// ---------------------------------------------------------------------------------------------
// One 32-row weight operand per wave (keeps the accumulators in architectural registers and two
// waves per SIMD, so one wave's integer/float work overlaps the other's MFMAs).
// MODE 0: up   -- a workgroup owns 64 rows of F: waves 0,1 carry those rows of w1, waves 2,3 the same
//                 rows of w3; the w3 waves hand their sums over through LDS and the w1 waves write
//                 h = silu(a) * b (f32).
// MODE 1: down -- a workgroup owns 128 rows of H of w2, one 32-row operand per wave; writes yw.
template <int MODE>
__global__ __launch_bounds__(G_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void q4k_gemm_kernel(ExpertParams p) {
    __shared__ GemmLds L;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n_tiles = p.rb.tile_tab[0];
    // Workgroup -> (row block, slot tile).  Hardware hands consecutive workgroup ids to the eight XCDs
    // in turn, each with its own L2; the ids that land on one XCD are therefore walked in 8 x 8
    // super-tiles (8 row blocks x 8 slot tiles), so that the ~64 workgroups an XCD runs at a time share
    // their weight rows and their activation tiles through that L2.
    const int n_rb = MODE == 0 ? p.F / 64 : p.H / 128;
    const int RG = (n_rb + 7) / 8;
    const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
    const int st = (q >> 6) * 8 + xcd, within = q & 63;
    const int rblk = (st % RG) * 8 + (within & 7);
    const int tile = (st / RG) * 8 + (within >> 3);
    if (tile >= n_tiles || rblk >= n_rb) return;
    const int gi = p.rb.tile_tab[1 + 2 * tile], pos0 = p.rb.tile_tab[2 + 2 * tile];
    if (gi < p.group0 || gi >= p.group0 + p.n_groups) return;
    const int grp = gi - p.group0;
    const int s_begin = p.rb.offsets[gi], n_g = p.rb.offsets[gi + 1] - s_begin;
    const int K = MODE == 0 ? p.H : p.F;        // reduction length
    const int N = MODE == 0 ? p.F : p.H;        // weight rows of the matrix
    const int nsb = K / 256;
    const size_t sb_stride = (size_t)(N / 16) * Q4K_TILE_BYTES;
    const ActBuf& ab = MODE == 0 ? p.xq : p.hq;

    // which activation rows this thread stages: rows tid/16 + 16 j (quants), tid/2 (sums), tid-128 (scales)
    auto act_row = [&](int r) {
        const int pos = pos0 + r;
        const int slot = s_begin + (pos < n_g ? pos : n_g - 1);
        return MODE == 0 ? p.rb.perm_token[slot] : slot - p.slot_origin;
    };
    int rows4[4];
#pragma unroll
    for (int j = 0; j < 4; j++) rows4[j] = act_row((tid >> 4) + 16 * j);
    const int row_bs = act_row((tid & 127) >> 1), row_yd = act_row(tid & 63);

    // weight operand of this wave
    const GroupWeights gw = p.groups[grp];
    const uint8_t* wp;
    int row0;
    if (MODE == 0) {
        row0 = rblk * 64 + (wave & 1) * 32;
        wp = (wave < 2 ? gw.w1 : gw.w3) + (size_t)(row0 / 16) * Q4K_TILE_BYTES;
    } else {
        row0 = rblk * 128 + wave * 32;
        wp = gw.w2 + (size_t)(row0 / 16) * Q4K_TILE_BYTES;
    }
    v16f facc[2];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) facc[t][i] = 0.f;

    {
        AStage st = a_stage_load(ab, K, nsb, 0, rows4, row_bs, row_yd, tid);
        a_stage_store(st, L, 0, tid);
    }
    BRegs b0 = b_load(wp, lane);
    __syncthreads();
    for (int sb = 0; sb < nsb; sb++) {
        const int buf = sb & 1;
        const int sbn = sb + 1 < nsb ? sb + 1 : sb;
        const BRegs n0 = b_load(wp + (size_t)sbn * sb_stride, lane);
        AStage st = a_stage_load(ab, K, nsb, sbn, rows4, row_bs, row_yd, tid);
        __builtin_amdgcn_sched_barrier(0);   // the prefetches must be in flight before the MFMA work, not after it
        gemm_superblock<2>(b0, L, buf, lane, facc);
        __builtin_amdgcn_sched_barrier(0);
        a_stage_store(st, L, buf ^ 1, tid);
        b0 = n0;
        __syncthreads();
    }

    // epilogue: lane holds weight row n = lane%32 and slots t*32 + (i/4)*8 + half*4 + i%4
    const int n = lane & 31, half = lane >> 5;
    if (MODE == 0) {
        // w3 waves (2,3) park their sums in LDS (the activation buffers are free now), w1 waves combine
        float* xch = reinterpret_cast<float*>(L.q[0]);   // [2 waves][2 t][16 i][64 lanes] = 16 KB <= sizeof(L.q[0])
        if (wave >= 2) {
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int i = 0; i < 16; i++) xch[(((wave - 2) * 2 + t) * 16 + i) * 64 + lane] = facc[t][i];
        }
        __syncthreads();
        if (wave < 2) {
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int pos = pos0 + t * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
                    if (pos >= n_g) continue;
                    const float bsum = xch[((wave * 2 + t) * 16 + i) * 64 + lane];
                    p.hbuf[(int64_t)(s_begin + pos - p.slot_origin) * p.F + row0 + n] = silu_gemm(facc[t][i]) * bsum;
                }
        }
    } else {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int pos = pos0 + t * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
                if (pos >= n_g) continue;
                const int slot = s_begin + pos;
                p.yw[(int64_t)slot * p.H + row0 + n] = facc[t][i] * p.rb.perm_w[slot];
            }
    }
}

static unsigned gemm_grid(int n_rb, int64_t max_tiles) {
    const int64_t RG = (n_rb + 7) / 8, TG = (max_tiles + 7) / 8;
    return (unsigned)(RG * TG * 64);
}
hipError_t launch_q4k_gemm_up(const ExpertParams& p, hipStream_t s) {
    dim3 grid(gemm_grid(p.F / 64, max_gemm_tiles(p.n_slots, p.n_groups + 1)));
    hipLaunchKernelGGL(q4k_gemm_kernel<0>, grid, dim3(G_THREADS), 0, s, p);
    return hipGetLastError();
}
hipError_t launch_q4k_gemm_down(const ExpertParams& p, hipStream_t s) {
    dim3 grid(gemm_grid(p.H / 128, max_gemm_tiles(p.n_slots, p.n_groups + 1)));
    hipLaunchKernelGGL(q4k_gemm_kernel<1>, grid, dim3(G_THREADS), 0, s, p);
    return hipGetLastError();
}

}  // namespace moe
