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
// Work split: a workgroup owns one tile of 128 slots of one expert (from the dispatch kernel's tile
// list, so a skewed routing is balanced by tiles, not by experts) and four 32-row weight operands,
// one per wave.  The 128 activation rows of a super-block go straight from global memory into LDS
// (double-buffered, no staging registers) and every wave reads them as MFMA A operands.  A wave unpacks and pre-scales its 32 weight rows of
// the super-block once, keeps the two planes in registers (64 VGPRs) and runs them against the four
// 32-slot operands one after the other, so the unpacking cost is spread over 128 slots while only
// one operand's integer accumulators are live at a time.
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

constexpr int GT = GEMM_TILE_SLOTS;   // 128 slots per tile = four 32-row MFMA operands
constexpr int MT = GT / 32;
constexpr int G_THREADS = 256;
// Activation quants in LDS: the tile's rows go in chunks of four; a chunk is 1 KiB, written by ONE
// direct global->LDS load of a wave (lane i lands at byte 16 i), and holds [16-byte piece c][row r%4].
// Chunks are 1088 bytes apart, so the 16 rows that one phase of a 16-byte LDS read touches (four
// chunks x four rows, same piece) fall into 16 different 16-byte bank groups.
constexpr int CHUNK = 1088;
constexpr int QBUF = (GT / 4) * CHUNK;

struct alignas(16) GemmLds {
    alignas(16) uint8_t q[2][QBUF];           // activation quants (device order of the row: pieces (pair P, chunk g))
    alignas(16) _Float16 bs[2][GT][16];       // block sums
    alignas(16) float yd[2][GT];              // activation scales
};

__device__ __forceinline__ uint32_t lds_address(const void* p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}
// Direct global->LDS loads: lane i of the wave writes SIZE bytes at lds + SIZE*i; nothing passes through
// registers, so a whole super-block of activations can be in flight while the wave computes.  The
// compiler does not see these loads: the issuing wave waits for them (vmcnt) before the barrier that
// publishes the buffer.
__device__ __forceinline__ void dma16(const void* gbase, uint32_t voff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(gbase), "s"(lds));
}
__device__ __forceinline__ void dma4(const void* gbase, uint32_t voff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(voff), "s"(gbase), "s"(lds));
}
__device__ __forceinline__ void wait_all_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }   // vmcnt(0)

// What a lane fetches for the tile: quants of rows 4*(8 wave + j) + lane%4 (piece lane/4), block sums of
// row 32 wave + lane/2, scale of row 64 (wave%2) + lane (waves 2,3 repeat waves 0,1: same bytes to the
// same place, and no branch around a load).
struct StageRows {
    uint32_t q[8];     // byte offset of the row's quants
    uint32_t bs, yd;   // row index
};
// transfer number i (0..9) of a wave's share of the tile: eight quant chunks, the block sums, the scales
template <int I>
__device__ __forceinline__ void stage_piece(const ActBuf& ab, const StageRows& r, int nsb, int sb, GemmLds& L, int buf, int wave, int lane) {
    if (I < 8)
        dma16(ab.qs, r.q[I] + (uint32_t)(sb * 256 + (lane >> 2) * 16), lds_address(L.q[buf]) + (uint32_t)((wave * 8 + I) * CHUNK));
    else if (I == 8)
        dma16(ab.bsum, ((r.bs * (uint32_t)nsb + (uint32_t)sb) * 16 + (lane & 1) * 8) * 2, lds_address(&L.bs[buf][0][0]) + (uint32_t)(wave * 1024));
    else
        dma4(ab.d, (r.yd * (uint32_t)nsb + (uint32_t)sb) * 4, lds_address(&L.yd[buf][0]) + (uint32_t)((wave & 1) * 256));
}
__device__ __forceinline__ void stage_tile(const ActBuf& ab, const StageRows& r, int nsb, int sb, GemmLds& L, int buf, int wave, int lane) {
    stage_piece<0>(ab, r, nsb, sb, L, buf, wave, lane); stage_piece<1>(ab, r, nsb, sb, L, buf, wave, lane);
    stage_piece<2>(ab, r, nsb, sb, L, buf, wave, lane); stage_piece<3>(ab, r, nsb, sb, L, buf, wave, lane);
    stage_piece<4>(ab, r, nsb, sb, L, buf, wave, lane); stage_piece<5>(ab, r, nsb, sb, L, buf, wave, lane);
    stage_piece<6>(ab, r, nsb, sb, L, buf, wave, lane); stage_piece<7>(ab, r, nsb, sb, L, buf, wave, lane);
    stage_piece<8>(ab, r, nsb, sb, L, buf, wave, lane); stage_piece<9>(ab, r, nsb, sb, L, buf, wave, lane);
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

// The unpacked, pre-scaled operand of one super-block.  MFMA number 2P+e of the super-block multiplies
// activation piece (pair P, chunk 2*half+e) = [8 values of sub-block 2P | 8 values of sub-block 2P+1]
// by the low and the high nibbles of the same 8 weight bytes, each half scaled by its own sub-block's
// digit (the planes are accumulated over the whole super-block, so an MFMA may mix sub-blocks).
struct BPlanes {
    v4i lo[8], hi[8];
    v8h mB;
    float d, dmin;
};

__device__ __forceinline__ BPlanes b_prepare(const BRegs& b, int lane) {
    const int half = lane >> 5;
    const uint32_t M4 = 0x0f0f0f0fu;
    const uint32_t u0 = b.hdr.y, u1 = b.hdr.z, u2 = b.hdr.w;
    BPlanes o;
    o.d = __half2float(__ushort_as_half((unsigned short)(b.hdr.x & 0xffffu)));
    o.dmin = __half2float(__ushort_as_half((unsigned short)(b.hdr.x >> 16)));
    const uint32_t sc03 = u0 & 0x3f3f3f3fu;
    const uint32_t sc47 = (u2 & M4) | (((u0 >> 6) & 0x03030303u) << 4);
    const uint32_t m03 = u1 & 0x3f3f3f3fu;
    const uint32_t m47 = ((u2 >> 4) & M4) | (((u1 >> 6) & 0x03030303u) << 4);
    // scales split into two 3-bit digits, still one byte per sub-block
    const uint32_t lo03 = sc03 & 0x07070707u, hi03 = (sc03 >> 3) & 0x07070707u;
    const uint32_t lo47 = sc47 & 0x07070707u, hi47 = (sc47 >> 3) & 0x07070707u;
#pragma unroll
    for (int P = 0; P < 4; P++) {
        // pair P lives in plane P/2 of the tile, dwords (x,y) for P even and (z,w) for P odd
        const int pl = P >> 1;
        const uint32_t lw = (P < 2) ? lo03 : lo47, hw = (P < 2) ? hi03 : hi47;
        const uint32_t slo_a = (lw >> (16 * (P & 1))) & 0xffu, slo_b = (lw >> (16 * (P & 1) + 8)) & 0xffu;
        const uint32_t shi_a = (hw >> (16 * (P & 1))) & 0xffu, shi_b = (hw >> (16 * (P & 1) + 8)) & 0xffu;
#pragma unroll
        for (int e = 0; e < 2; e++) {
            const u32x4 c = e ? b.c1[pl] : b.c0[pl];
            const uint32_t w0 = (P & 1) ? c.z : c.x, w1 = (P & 1) ? c.w : c.y;
            const uint32_t a0 = w0 & M4, a1 = w1 & M4, b0 = (w0 >> 4) & M4, b1 = (w1 >> 4) & M4;
            o.lo[P * 2 + e] = v4i{(int)scale_bytes(a0, slo_a), (int)scale_bytes(a1, slo_a), (int)scale_bytes(b0, slo_b), (int)scale_bytes(b1, slo_b)};
            o.hi[P * 2 + e] = v4i{(int)scale_bytes(a0, shi_a), (int)scale_bytes(a1, shi_a), (int)scale_bytes(b0, shi_b), (int)scale_bytes(b1, shi_b)};
        }
    }
    // mins: k = 8*half + j is block sum j of this half; it belongs to sub-block 4*half + j/2
    const uint32_t mw = half ? m47 : m03;
#pragma unroll
    for (int j = 0; j < 8; j++) o.mB[j] = (_Float16)(int)((mw >> (8 * (j >> 1))) & 0xffu);
    return o;
}

// one super-block of the wave's 32 weight rows against 32-slot operand t of the staged tile
// `while_busy` runs right after the MFMAs are issued: the wave would otherwise idle until they drain,
// so this is where the next super-block's loads are issued.
template <typename Fill>
__device__ __forceinline__ void gemm_operand(const BPlanes& B, const GemmLds& L, int buf, int t, int lane, v16f& facc, Fill while_busy) {
    const int m = lane & 31, half = lane >> 5;
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};  // first MFMA of a chain takes the constant 0 as C
    v16i acc_lo, acc_hi;
    // row t*32+m: chunk t*8 + m/4, slot m%4 of every piece; pieces 4P + 2*half + e
    const uint8_t* arow = L.q[buf] + (t * 8 + (m >> 2)) * CHUNK + (m & 3) * 16 + half * 128;
#pragma unroll
    for (int u = 0; u < 8; u++) {
        const v4i a = *reinterpret_cast<const v4i*>(arow + (u >> 1) * 256 + (u & 1) * 64);
        acc_lo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, B.lo[u], u == 0 ? zero16 : acc_lo, 0, 0, 0);
        acc_hi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, B.hi[u], u == 0 ? zero16 : acc_hi, 0, 0, 0);
    }
    const v8h mA = *reinterpret_cast<const v8h*>(&L.bs[buf][t * 32 + m][half * 8]);
    const v16f zf = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const v16f Dm = __builtin_amdgcn_mfma_f32_32x32x16_f16(mA, B.mB, zf, 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    while_busy();
    __builtin_amdgcn_sched_barrier(0);
    // D[i] belongs to slot (i/4)*8 + half*4 + i%4 of operand t, weight row n = lane%32.
    // The 16 values go through each step together (the fences keep the compiler from re-serialising
    // them into 16 dependent chains: a lone dependent VALU chain issues at half rate).
    typedef float v4fl __attribute__((ext_vector_type(4)));
    float ydv[16];
#pragma unroll
    for (int i4 = 0; i4 < 4; i4++) {
        const v4fl yd = *reinterpret_cast<const v4fl*>(&L.yd[buf][t * 32 + i4 * 8 + half * 4]);
        ydv[i4 * 4 + 0] = yd.x; ydv[i4 * 4 + 1] = yd.y; ydv[i4 * 4 + 2] = yd.z; ydv[i4 * 4 + 3] = yd.w;
    }
    int isum[16];
    float fs[16], mm[16], v[16];
#pragma unroll
    for (int i = 0; i < 16; i++) isum[i] = (acc_hi[i] << 3) + acc_lo[i];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 16; i++) fs[i] = (float)isum[i];
#pragma unroll
    for (int i = 0; i < 16; i++) mm[i] = B.dmin * Dm[i];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 16; i++) v[i] = __builtin_fmaf(B.d, fs[i], -mm[i]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 16; i++) facc[i] = __builtin_fmaf(ydv[i], v[i], facc[i]);
}


__device__ __forceinline__ float silu_gemm(float v) { return v / (1.0f + __expf(-v)); }

// ---------------------------------------------------------------------------------------------
// One 32-row weight operand per wave, two workgroups per CU (two waves per SIMD from different
// workgroups, so one wave's integer/float work overlaps the other's MFMAs).
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

    // activation row behind position r of the tile (positions past the expert's list repeat its last row)
    auto act_row = [&](int r) {
        const int pos = pos0 + r;
        const int slot = s_begin + (pos < n_g ? pos : n_g - 1);
        return MODE == 0 ? p.rb.perm_token[slot] : slot - p.slot_origin;
    };
    StageRows rows;
#pragma unroll
    for (int j = 0; j < 8; j++) rows.q[j] = (uint32_t)act_row(4 * (wave * 8 + j) + (lane & 3)) * (uint32_t)K;
    rows.bs = (uint32_t)act_row(32 * wave + (lane >> 1));
    rows.yd = (uint32_t)act_row(64 * (wave & 1) + lane);

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
    v16f facc[MT];
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) facc[t][i] = 0.f;

    stage_tile(ab, rows, nsb, 0, L, 0, wave, lane);
    BRegs raw = b_load(wp, lane);
    wait_all_loads();
    __syncthreads();
    for (int sb = 0; sb < nsb; sb++) {
        const int buf = sb & 1;
        const int sbn = sb + 1 < nsb ? sb + 1 : sb;
        const BPlanes B = b_prepare(raw, lane);
        const int nb = buf ^ 1;
        gemm_operand(B, L, buf, 0, lane, facc[0], [&] {
            stage_piece<0>(ab, rows, nsb, sbn, L, nb, wave, lane); stage_piece<1>(ab, rows, nsb, sbn, L, nb, wave, lane);
            stage_piece<2>(ab, rows, nsb, sbn, L, nb, wave, lane); });
        __builtin_amdgcn_sched_barrier(0);
        gemm_operand(B, L, buf, 1, lane, facc[1], [&] {
            stage_piece<3>(ab, rows, nsb, sbn, L, nb, wave, lane); stage_piece<4>(ab, rows, nsb, sbn, L, nb, wave, lane);
            stage_piece<5>(ab, rows, nsb, sbn, L, nb, wave, lane); });
        __builtin_amdgcn_sched_barrier(0);
        gemm_operand(B, L, buf, 2, lane, facc[2], [&] {
            stage_piece<6>(ab, rows, nsb, sbn, L, nb, wave, lane); stage_piece<7>(ab, rows, nsb, sbn, L, nb, wave, lane);
            stage_piece<8>(ab, rows, nsb, sbn, L, nb, wave, lane); stage_piece<9>(ab, rows, nsb, sbn, L, nb, wave, lane); });
        __builtin_amdgcn_sched_barrier(0);
        gemm_operand(B, L, buf, 3, lane, facc[3], [&] { raw = b_load(wp + (size_t)sbn * sb_stride, lane); });
        __builtin_amdgcn_sched_barrier(0);
        wait_all_loads();
        __syncthreads();
    }

    // epilogue: lane holds weight row n = lane%32 and slots t*32 + (i/4)*8 + half*4 + i%4
    const int n = lane & 31, half = lane >> 5;
    if (MODE == 0) {
        // w3 waves (2,3) park their sums in LDS (the activation buffers are free now), w1 waves combine
        float* xch = reinterpret_cast<float*>(L.q[0]);   // [2 waves][MT][16 i][64 lanes] floats
        static_assert(2 * MT * 16 * 64 * 4 <= sizeof(L.q[0]), "exchange area");
        if (wave >= 2) {
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int i = 0; i < 16; i++) xch[(((wave - 2) * MT + t) * 16 + i) * 64 + lane] = facc[t][i];
        }
        __syncthreads();
        if (wave < 2) {
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int pos = pos0 + t * 32 + (i >> 2) * 8 + half * 4 + (i & 3);
                    if (pos >= n_g) continue;
                    const float bsum = xch[((wave * MT + t) * 16 + i) * 64 + lane];
                    p.hbuf[(int64_t)(s_begin + pos - p.slot_origin) * p.F + row0 + n] = silu_gemm(facc[t][i]) * bsum;
                }
        }
    } else {
#pragma unroll
        for (int t = 0; t < MT; t++)
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
