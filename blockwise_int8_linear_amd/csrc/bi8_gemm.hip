// int8 GEMM with the per-K-block dequantize fused into the K loop (bi8_gemm_nt_dequant) and its int32
// block partials (bi8_gemm_nt_partials).  Replaces _int8_matmul_block64_rowwise_dequantize,
// triton_functions.py:70-139 (SPLIT_K = 1 path).
//
//   C[m,n] = cast( (1/127^2) * sum_j sA[j,m] * sW[j,n] * P_j[m,n] ),   P_j = int32 dot over K-block j
//
// NT GEMM, both operands K-contiguous.  The kernels, chosen by shape in plan_gemm():
//   gemm_wide    blocks 128 / 64, problems of >= 129 tiles of 256x256: v_mfma_i32_16x16x64_i8, 64x128 per wave, persistent
//                grid; when its last round of tiles would be mostly empty it runs on the leading rows or columns only and
//                a gemm_tile launch takes the rest;
//   gemm_wide32  block 32, same problems and tile: v_mfma_i32_32x32x32_i8, 32x256 per wave;
//   gemm_wide<.., 4>  the same kernel on 256x128 tiles (64x64 per wave) for problems of more than 256 tiles of 128x128 that
//                do not fill the chip with 256x256 tiles (Llama prefill at 2048 tokens, the GPT-2 layer GEMMs);
//   gemm_tile    blocks 32/64/128: v_mfma_i32_32x32x32_i8, 256x128 / 128x128 / 64x128 tiles; also the int32
//                block partials, and (SPLIT) fp32 partial sums over part of K for problems of fewer tiles than CUs, which
//                splitk_reduce adds up;
//   gemv_rows    M <= 2, blocks 64/128 (single-token decode; also bi8_linear_few_rows, which quantizes the activations in
//                the same launch): one pass over W in 1 KiB runs of whole rows, v_dot4_i32_i8 on the vector unit;
//   gemv_staged  M <= 32, blocks 64/128 (small decode batches): one pass over W, 16 columns per workgroup, K split over
//                4 or 8 waves that each stream whole cache lines of W through a private LDS ring into 16x16x64 MFMAs;
//   gemm_skinny  M <= 32 at block 32 (when nothing splits): operands gathered in operand layout, 32x32x32 MFMAs, one stage
//                of lookahead;
//   gemm_generic anything else (K not a multiple of 128, rows not 16-byte aligned, other block sizes): same
//                MFMA, operands gathered straight from global memory with byte loads.
// Common to the tiled kernels:
//   - the int32 partial of a K-block stays in registers and is folded into an fp32 accumulator with two vector
//     ops per output as soon as the block's MFMAs are issued;
//   - A and W tiles (128 bytes of K per row per stage) and the stage's scale rows go L2 -> LDS directly
//     (buffer_load ... lds, 16 bytes per lane), two LDS stage buffers, one barrier per stage;
//   - LDS rows are 128 bytes with the 16-byte chunk index XOR-ed with ((row >> 1) & 7): 16 consecutive rows of
//     one chunk column cover all 64 banks, so the MFMA operand reads (ds_read_b128) run at full LDS rate;
//   - the workgroup index is remapped so that the 32 workgroups resident on one XCD (one L2) cover a
//     compact patch of output tiles.
#include <atomic>
#include <type_traits>

#include "bi8_common.h"

namespace {

constexpr int kStageK = 128;       // bytes of K per LDS stage

// Raw buffer resource (V#) over [base, base + bytes): loads beyond the end return zeros.
typedef bi8_v4i bi8_rsrc;
__device__ __forceinline__ bi8_rsrc bi8_make_rsrc(const void *base, int64_t bytes) {
    const uint64_t a = (uint64_t)base;
    const int n = bytes > 0x7fffffffLL ? 0x7fffffff : (bytes < 0 ? 0 : (int)bytes);    // never a wrapped (huge) range
    // dword0-1: 48-bit base, stride 0; dword2: size in bytes; dword3: raw 32-bit-format buffer (gfx9 family)
    return bi8_rsrc{(int)(uint32_t)a, (int)(uint32_t)((a >> 32) & 0xffffu), n, 0x00020000};
}
// The same resource as the compiler's buffer type, for loads into registers (the compiler tracks their completion):
// the address is one VGPR offset plus one SGPR offset plus an immediate, instead of a 64-bit VGPR pointer per load.
typedef __amdgpu_buffer_rsrc_t bi8_brsrc;
__device__ __forceinline__ bi8_brsrc bi8_make_brsrc(const void *base, int64_t bytes) {
    const int n = bytes > 0x7fffffffLL ? 0x7fffffff : (bytes < 0 ? 0 : (int)bytes);
    return __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, n, 0x00020000);
}
constexpr int kBufNT = 2;          // cache policy bit "nt": streamed once
constexpr int kBufOut = 0x40000000;  // added to a VGPR offset: beyond any range this file gives a buffer (< 2^31 bytes)
__device__ __forceinline__ bi8_v4i bi8_buffer_load16(bi8_brsrc r, int voff, int soff, bool nt) {
    return nt ? (bi8_v4i)__builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, kBufNT)
              : (bi8_v4i)__builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0);
}
__device__ __forceinline__ float bi8_buffer_load_f32(bi8_brsrc r, int voff, int soff) {
    return bi8_u2f(__builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
__device__ __forceinline__ uint32_t bi8_lds_address(const void *p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
}
// 64 lanes x 16 (or 4) bytes from buffer offset voff + soff straight into LDS at lds_addr + lane * 16 (or 4);
// rsrc, lds_addr and soff are wave-uniform.  Written as inline asm on purpose: the loads complete
// asynchronously and are fenced by this file's own `s_waitcnt vmcnt(n)`, which lets later stages stay in
// flight across a barrier; through the compiler's builtin every barrier would wait for all of them.
__device__ __forceinline__ void bi8_buffer_to_lds16(bi8_rsrc r, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(r), "s"(soff)
                 : "memory", "m0", "vcc");      // vcc listed so that no operand is allocated to it (not encodable as soffset)
}
// Same with the scalar offset given as a sum: the addition sits between the write of M0 and the load, where the
// hardware needs one independent instruction anyway.
__device__ __forceinline__ void bi8_buffer_to_lds16_sum(bi8_rsrc r, uint32_t lds_addr, uint32_t voff, uint32_t soff_a, uint32_t soff_b) {
    uint32_t soff;
    asm volatile("s_mov_b32 m0, %1\n\ts_add_u32 %0, %4, %5\n\tbuffer_load_dwordx4 %2, %3, %0 offen lds"
                 : "=&s"(soff)
                 : "s"(lds_addr), "v"(voff), "s"(r), "s"(soff_a), "s"(soff_b)
                 : "memory", "m0", "scc", "vcc");
}
// 64 lanes x one 16-bit element, each zero-extended into its own dword of LDS
__device__ __forceinline__ void bi8_buffer_to_lds2(bi8_rsrc r, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_ushort %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(r), "s"(soff)
                 : "memory", "m0", "vcc");
}
__device__ __forceinline__ void bi8_buffer_to_lds4(bi8_rsrc r, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(r), "s"(soff)
                 : "memory", "m0", "vcc");      // vcc listed so that no operand is allocated to it (not encodable as soffset)
}

// Workgroups are dealt round-robin to the 8 XCDs.  Give XCD x the x-th contiguous eighth of a
// tile order in which consecutive indices form kGroupM-row bands walked column by column.
constexpr int kXcds = 8;
constexpr int kGroupM = 4;
__device__ __forceinline__ void tile_of_workgroup(int pid, int tiles_m, int tiles_n, int &tm, int &tn) {
    const int total = tiles_m * tiles_n;
    const int per = total / kXcds;                 // full rounds
    int idx;
    if (pid < per * kXcds) idx = (pid % kXcds) * per + pid / kXcds;
    else idx = pid;                                // remainder keeps its place at the end
    const int band = kGroupM * tiles_n;
    const int b = idx / band;
    const int rows = (tiles_m - b * kGroupM < kGroupM) ? (tiles_m - b * kGroupM) : kGroupM;
    const int in = idx % band;
    tm = b * kGroupM + in % rows;
    tn = in / rows;
}

// The same order for a kernel that walks several tiles: pid is wave-uniform and every step stays on the scalar unit
// (no division: band_magic = floor(2^32 / (kGroupM * tiles_n)) comes from the host).
__device__ __forceinline__ void tile_of_workgroup_scalar(int pid, int tiles_m, int tiles_n, uint32_t band_magic, int &tm, int &tn) {
    const int total = tiles_m * tiles_n;
    const int per = total >> 3;
    const int idx = pid < per * kXcds ? (pid & (kXcds - 1)) * per + (pid >> 3) : pid;
    const int band = kGroupM * tiles_n;
    int b = (int)__umulhi((uint32_t)idx, band_magic);          // floor(idx / band) or one less
    int in = idx - b * band;
    if (in >= band) {
        in -= band;
        ++b;
    }
    const int left = tiles_m - b * kGroupM;
    const int rows = left < kGroupM ? left : kGroupM;          // 1 .. 4
    static_assert(kGroupM == 4 && kXcds == 8, "the shifts below");
    const int q = rows == 4 ? in >> 2 : rows == 3 ? (int)__umulhi((uint32_t)in, 0x55555556u) : rows == 2 ? in >> 1 : in;
    tm = b * kGroupM + (in - q * rows);
    tn = q;
}

template <int CDT> __device__ __forceinline__ void store_c(void *C, int64_t idx, float acc, bool has_bias, float bias) {
    float c = bi8_round_to<CDT>(acc);                      // acc.to(C.dtype)             triton_functions.py:127
    if (has_bias) c = c + bi8_round_to<CDT>(bias);         // + bias.to(C.dtype), in C's dtype   :129-131
    bi8_store_elem<CDT>(C, idx, c);
}

struct GemmArgs {
    const int8_t *A, *W;
    const float *sA, *sW;
    const void *bias;
    void *C;
    int32_t *P;
    int64_t M, N, K, lda, ldw, ldc;
    int tiles_m, tiles_n;
    int bias_dtype;
    // split of the contraction over `splits` workgroups (<= 1: none), each of which writes fp32 partial sums (scaled,
    // no bias) of `split_stages` 128-byte stages of K to slabs ws[...][BM][BN], in one of two forms:
    //   split_per_tile > 0: that many workgroups per tile; workgroup w takes stages (w % split_per_tile) * split_stages
    //     ... of tile w / split_per_tile of the XCD-aware order, slab t * split_per_tile + w % split_per_tile (t = the
    //     tile's row-major index);
    //   split_per_tile == 0: the (tile, stage) pairs, tiles in row-major order and a tile's stages ascending, are one
    //     sequence, and workgroup w takes the run of split_stages pairs from w * split_stages on.  A run touches one
    //     tile or the end of one and the start of the next; slab w + t for each.
    float *ws;
    int64_t ws_bytes;
    int splits, split_stages;
    uint32_t band_magic;            // gemm_wide: floor(2^32 / (kGroupM * tiles_n))
    int split_per_tile;
    // a launch that computes part of the output only: tiles_m x tiles_n tiles from tile (tile_m0, tile_n0) on (M, N and
    // the pointers stay those of the whole problem)
    int tile_m0, tile_n0;
    // gemm_panel: columns from one tile to the next where that is less than the tile's width (0: its width): the tile's
    // remaining columns are loaded as zeros, from beyond the buffer's range, and not stored
    int panel_pitch;
};
// The rectangle of the output that one launch computes (the whole of it unless the plan cuts the problem in two).
struct Part {
    int64_t row0, col0, rows, cols;
};

__device__ __forceinline__ float load_bias(const GemmArgs &g, int64_t n) {
    if (g.bias_dtype == BI8_F32) return ((const float *)g.bias)[n];
    if (g.bias_dtype == BI8_BF16) return bi8_from_bf16_bits(((const uint16_t *)g.bias)[n]);
    return bi8_from_f16_bits(((const uint16_t *)g.bias)[n]);
}

// A slab element of a split contraction (gemm_tile): stored with device scope (cache policy sc1: written through to
// memory instead of staying in the writing XCD's L2 until the kernel ends, when all of it would be written back at
// once).  Measured against plain stores, both kernels of the call: 128 x 4096 x 4096 14.7 -> 14.1 us, 128 x 11008 x 4096
// 22.2 -> 21.6, 256 x 4096 x 4096 20.7 -> 20.1; on the 256x128 slabs of gemm_wide's split +-1 %, not used there.
__device__ __forceinline__ void slab_store(float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
constexpr int kSplitMax = 8;                   // most slabs per tile

// LDS map of gemm_tile: one region per operand, each a ring of kBufs stage buffers.
template <int BM, int BN, int BLK, int NBUF> struct TileLds {
    static constexpr int kBufs = NBUF;
    static constexpr int NBS = kStageK / BLK;        // K-blocks per stage
    static constexpr int kABuf = BM * kStageK, kWBuf = BN * kStageK;
    static constexpr int kSABuf = NBS * BM * 4, kSWBuf = NBS * BN * 4;
    static constexpr int kAReg = 0;
    static constexpr int kWReg = kAReg + kBufs * kABuf;
    static constexpr int kSAReg = kWReg + kBufs * kWBuf;
    static constexpr int kSWReg = kSAReg + kBufs * kSABuf;
    static constexpr int kBytes = kSWReg + kBufs * kSWBuf;
    static constexpr bool kFits = kBytes <= 160 * 1024;   // LDS per CU
};

// BM x BN output tile per workgroup, WM x WN waves (each TM x TN subtiles of 32x32), BLK = quantization block.
// One tile (tile_m, tile_n) of the problem `g`, by one workgroup.
// SLAB: the output is a slab of a split contraction (fp32, no bias), stored with slab_store.
template <int BM, int BN, int WM, int WN, int NBUF, int BLK, int CDT, bool PARTIALS, bool SLAB = false>
__device__ __forceinline__ void gemm_tile_body(const GemmArgs g, const int tile_m, const int tile_n) {
    using L = TileLds<BM, BN, BLK, NBUF>;
    constexpr int kBufs = NBUF;
    constexpr int NW = WM * WN;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int NBS = L::NBS;
    constexpr int KSB = BLK / 32;                  // MFMA k-steps per K-block
    constexpr int NSUB = TM * TN;
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tiling");
    static_assert(BM % 64 == 0 && BN % 64 == 0, "scale rows are loaded 64 floats per wave instruction");
    static_assert((BM / 8) % NW == 0 && (BN / 8) % NW == 0, "operand rows split evenly over the waves");

    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, h = lane >> 5;

    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    const int nstages = (int)(g.K / kStageK);

    // ---- loader: buffer loads straight into LDS.  One buffer resource per operand, based at this tile's
    // first row and sized to the end of the matrix, so rows past the edge read as zeros; a 32-bit per-lane
    // offset per wave instruction (constant over the K loop) and the K position in a scalar register.
    // wave-instruction i covers tile rows 8i .. 8i+7; lane -> (row 8i + lane/8, LDS chunk lane%8), which
    // holds source chunk (lane%8) ^ ((row >> 1) & 7).  Every wave's instruction indices i = wave + it*NW have
    // the parity of `wave` (NW is even), so (row >> 1) & 7 = (4 * (wave & 1) + lane/16) & 7.
    static_assert(NW % 2 == 0, "swizzle term must not depend on the iteration");
    const int ld_row = lane >> 3;
    const int ld_chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);
    constexpr int kAIter = BM / 8 / NW, kWIter = BN / 8 / NW;
    const int64_t a_rows = (g.M - m0 < BM) ? (g.M - m0) : BM, w_rows = (g.N - n0 < BN) ? (g.N - n0) : BN;
    const bi8_rsrc a_rsrc = bi8_make_rsrc(g.A + m0 * g.lda, (a_rows - 1) * g.lda + g.K);
    const bi8_rsrc w_rsrc = bi8_make_rsrc(g.W + n0 * g.ldw, (w_rows - 1) * g.ldw + g.K);
    // per-lane part of the offset (one register per operand); the rows of wave instruction `it` start
    // (wave + it*NW) * 8 rows further down, which goes into the scalar offset together with the K position
    const uint32_t a_off = (uint32_t)(ld_row * g.lda + ld_chunk * 16), w_off = (uint32_t)(ld_row * g.ldw + ld_chunk * 16);
    const uint32_t a_wave = (uint32_t)(wave * 8 * g.lda), w_wave = (uint32_t)(wave * 8 * g.ldw);
    const uint32_t a_step = (uint32_t)(NW * 8 * g.lda), w_step = (uint32_t)(NW * 8 * g.ldw);
    // scale rows: 64 floats per wave instruction; instruction i -> K-block i / kSPer of the stage, and inside
    // it the first BM/64 instructions fetch sA, the rest sW.  Waves beyond the last instruction repeat an
    // earlier one (same bytes to the same place) rather than branch around it.
    constexpr int kSPer = BM / 64 + BN / 64;
    constexpr int kSInstr = PARTIALS ? 0 : NBS * kSPer;
    constexpr int kSIter = (kSInstr + NW - 1) / NW;
    constexpr int kSI = kSIter > 0 ? kSIter : 1;
    const int64_t nblk = g.K / BLK;
    const bi8_rsrc sa_rsrc = bi8_make_rsrc(g.sA + m0, PARTIALS ? 0 : ((nblk - 1) * g.M + (g.M - m0)) * 4);
    const bi8_rsrc sw_rsrc = bi8_make_rsrc(g.sW + n0, PARTIALS ? 0 : ((nblk - 1) * g.N + (g.N - n0)) * 4);
    uint32_t s_off[kSI], s_pos[kSI], s_inc[kSI];   // per-lane offset; scale-row position of the next stage and its step
    int s_dst[kSI], s_bufstep[kSI];
    bi8_rsrc s_rsrc[kSI];
#pragma unroll
    for (int it = 0; it < kSIter; ++it) {
        const int i = (wave + it * NW) % (kSInstr > 0 ? kSInstr : 1);
        const int b = i / kSPer, r = i % kSPer;
        const bool is_a = r < BM / 64;             // wave-uniform: everything below is selected, not branched
        s_rsrc[it] = is_a ? sa_rsrc : sw_rsrc;
        s_off[it] = is_a ? (uint32_t)((b * g.M + r * 64 + lane) * 4) : (uint32_t)((b * g.N + (r - BM / 64) * 64 + lane) * 4);
        s_dst[it] = is_a ? L::kSAReg + (b * BM + r * 64) * 4 : L::kSWReg + (b * BN + (r - BM / 64) * 64) * 4;
        s_bufstep[it] = is_a ? L::kSABuf : L::kSWBuf;
        s_inc[it] = (uint32_t)(NBS * (is_a ? g.M : g.N) * 4);
        s_pos[it] = 0;
    }
    uint32_t k_pos = 0;                            // K offset of the next stage to load (bytes)

    constexpr int kLoadsPerStage = kAIter + kWIter + kSIter;     // VMEM instructions one wave issues per stage
    const uint32_t lds_base = bi8_lds_address(lds);
    // the same in two halves (A rows; W rows + scales + advance), so that a stage's loads need not all be issued at once
    auto issue_half = [&](int buf, int half) {
        if (half == 0) {
#pragma unroll
            for (int it = 0; it < kAIter; ++it) bi8_buffer_to_lds16_sum(a_rsrc, lds_base + L::kAReg + buf * L::kABuf + (wave + it * NW) * 1024, a_off, k_pos, a_wave + it * a_step);
        } else {
#pragma unroll
            for (int it = 0; it < kWIter; ++it) bi8_buffer_to_lds16_sum(w_rsrc, lds_base + L::kWReg + buf * L::kWBuf + (wave + it * NW) * 1024, w_off, k_pos, w_wave + it * w_step);
            k_pos += kStageK;
#pragma unroll
            for (int it = 0; it < kSIter; ++it) {
                bi8_buffer_to_lds4(s_rsrc[it], lds_base + s_dst[it] + buf * s_bufstep[it], s_off[it], s_pos[it]);
                s_pos[it] += s_inc[it];
            }
        }
    };
    auto issue_stage = [&](int buf) {             // buf is wave-uniform: LDS destinations and K position are scalars
#pragma unroll
        for (int it = 0; it < kAIter; ++it) bi8_buffer_to_lds16(a_rsrc, lds_base + L::kAReg + buf * L::kABuf + (wave + it * NW) * 1024, a_off, k_pos + a_wave + it * a_step);
#pragma unroll
        for (int it = 0; it < kWIter; ++it) bi8_buffer_to_lds16(w_rsrc, lds_base + L::kWReg + buf * L::kWBuf + (wave + it * NW) * 1024, w_off, k_pos + w_wave + it * w_step);
        k_pos += kStageK;
#pragma unroll
        for (int it = 0; it < kSIter; ++it) {
            bi8_buffer_to_lds4(s_rsrc[it], lds_base + s_dst[it] + buf * s_bufstep[it], s_off[it], s_pos[it]);
            s_pos[it] += s_inc[it];
        }
    };

    // ---- operand fragment addresses (buffer 0).  Row r = ... + l32, 16-byte chunk (2*ks + h) ^ ((r >> 1) & 7):
    // address(ks) = base ^ (ks << 5).  One register per ks; buffer and subtile offsets are immediates.
    const int frag_sw = ((h ^ ((l32 >> 1) & 7)) << 4);
    int a_addr[4], w_addr[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        a_addr[ks] = (L::kAReg + (wm * (BM / WM) + l32) * kStageK + frag_sw) ^ (ks << 5);
        w_addr[ks] = (L::kWReg + (wn * (BN / WN) + l32) * kStageK + frag_sw) ^ (ks << 5);
    }
    int sa_addr = L::kSAReg + (wm * (BM / WM) + 4 * h) * 4;
    int sw_addr = L::kSWReg + (wn * (BN / WN) + l32) * 4;
    // keep the region offsets inside these ten registers (every access = one of them + an immediate under 64 KiB);
    // otherwise the compiler folds them into immediates too large for the instruction and keeps an address register
    // per access
    asm volatile("" : "+v"(a_addr[0]), "+v"(a_addr[1]), "+v"(a_addr[2]), "+v"(a_addr[3]), "+v"(w_addr[0]), "+v"(w_addr[1]), "+v"(w_addr[2]),
                 "+v"(w_addr[3]), "+v"(sa_addr), "+v"(sw_addr));

    float acc[TM][TN][16];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    // Loop-carried pipeline state.  The last subtile ("item") of a stage is folded into the accumulator
    // during the first MFMAs of the NEXT stage (after the barrier, while the new operands are still on their
    // way from LDS), so its int32 partial and its scales stay live across the stage boundary.
    constexpr int NITEM = NBS * NSUB;
    static_assert(NITEM % 2 == 0, "the two partial buffers alternate consistently across stages");
    bi8_v16i p[2];
    constexpr int kMagicBits = 0x4B400000;        // bit pattern of 1.5 * 2^23
    const int mg = PARTIALS ? 0 : kMagicBits;
    const bi8_v16i magic = {mg, mg, mg, mg, mg, mg, mg, mg, mg, mg, mg, mg, mg, mg, mg, mg};
    p[0] = p[1] = magic;                           // "partial 0" for the fold that precedes the first stage
    float swv[2][TN], swc[2][TN];                  // [K-block parity][column subtile]: scale b and -(1.5*2^23)*b
    bi8_v4f sxv[2][TM][4];                         // [K-block parity][row subtile][row group of 8]
#pragma unroll
    for (int q = 0; q < 2; ++q) {
#pragma unroll
        for (int b = 0; b < TN; ++b) swv[q][b] = swc[q][b] = 0.0f;
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int i = 0; i < 4; ++i) sxv[q][a][i] = bi8_v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }

    // Fold elements [16*ks/KSB, 16*(ks+1)/KSB) of an item's partial into the accumulator, two vector ops each.
    // The MFMA chain starts from kMagicBits in every accumulator lane, so the int32 result P + kMagicBits,
    // read as a float, IS the number 1.5*2^23 + P (exact for |P| < 2^22): no int->float conversion.  With the
    // column scale b rounded to 22 significant bits, c = -(1.5*2^23)*b is exact, and fma(f, b, c) = fl(b*P)
    // with a single rounding; the second fma applies the row scale and accumulates.
    auto fold_slice = [&](const bi8_v16i &pt, const bi8_v4f *sx, float sw, float swc, float *dst, int ks) {
#pragma unroll
        for (int r = ks * (16 / KSB); r < (ks + 1) * (16 / KSB); ++r) {
            const float u = __builtin_fmaf(bi8_u2f((uint32_t)pt[r]), sw, swc);
            dst[r] = __builtin_fmaf(u, sx[r >> 2][r & 3], dst[r]);
        }
    };

    // One stage = NBS K-blocks x NSUB subtiles ("items"), KSB MFMAs each.  The instruction order below is the
    // schedule: sched_barrier(0) fences keep the compiler from reordering across steps.  Step (t, ks) issues
    // one MFMA of item t and folds one slice of item t-1, so the matrix pipe and the vector ALU overlap;
    // operand reads are issued at the top of the stage in order of first use, scale reads as soon as the
    // registers they overwrite have been consumed.
    auto compute_stage = [&](int buf, int s) {     // buf is wave-uniform
        const int oa = buf * L::kABuf, ow = buf * L::kWBuf, osa = buf * L::kSABuf, osw = buf * L::kSWBuf;
        bi8_v4i af[TM][4], wf[TN][4];
        auto load_scales = [&](int blk, int a0, int a1, int b0, int b1) {
#pragma unroll
            for (int b = b0; b < b1; ++b) swv[blk & 1][b] = *(const float *)(lds + (sw_addr + osw) + (blk * BN + b * 32) * 4);
#pragma unroll
            for (int a = a0; a < a1; ++a)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    sxv[blk & 1][a][i] = *(const bi8_v4f *)(lds + (sa_addr + osa) + (blk * BM + a * 32 + 8 * i) * 4);
        };
        // column scale -> 22 significant bits (relative change <= 2^-22) and its product with -1.5*2^23 (exact)
        auto prep_scales = [&](int blk, int b0, int b1) {
#pragma unroll
            for (int b = b0; b < b1; ++b) {
                const float bq = bi8_u2f((bi8_f2u(swv[blk & 1][b]) + 2u) & ~3u);
                swv[blk & 1][b] = bq;
                swc[blk & 1][b] = -BI8_MAGIC * bq;
            }
        };
        // Operands are read just in time: item (0,0)'s at the top of the stage, row subtile a / column subtile b
        // during the item that precedes their first use, so the LDS traffic is spread over the stage.
        auto load_a = [&](int a) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) af[a][ks] = *(const bi8_v4i *)(lds + (a_addr[ks] + oa) + a * 32 * kStageK);
        };
        auto load_w = [&](int b) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) wf[b][ks] = *(const bi8_v4i *)(lds + (w_addr[ks] + ow) + b * 32 * kStageK);
        };
        // K-block blk of every row / column subtile (blocks shorter than the stage: their operands are read one
        // block at a time, during the last subtile of the block before, so a stage's operands are never all live)
        auto load_block = [&](int blk) {
#pragma unroll
            for (int ks = blk * KSB; ks < (blk + 1) * KSB; ++ks) {
#pragma unroll
                for (int b = 0; b < TN; ++b) wf[b][ks] = *(const bi8_v4i *)(lds + (w_addr[ks] + ow) + b * 32 * kStageK);
#pragma unroll
                for (int a = 0; a < TM; ++a) af[a][ks] = *(const bi8_v4i *)(lds + (a_addr[ks] + oa) + a * 32 * kStageK);
            }
        };
        if constexpr (PARTIALS) {                  // the simple order: everything up front
#pragma unroll
            for (int b = 0; b < TN; ++b) load_w(b);
#pragma unroll
            for (int a = 0; a < TM; ++a) load_a(a);
        } else if constexpr (NBS > 1) {
            load_block(0);
        } else {
            load_a(0);
            load_w(0);
        }

        if constexpr (PARTIALS) {
#pragma unroll
            for (int t = 0; t < NITEM; ++t) {
                const int blk = t / NSUB, a = (t % NSUB) / TN, b = t % TN;
                bi8_v16i pt = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int ks = 0; ks < KSB; ++ks)
                    pt = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[a][blk * KSB + ks], wf[b][blk * KSB + ks], pt, 0, 0, 0);
                const int64_t jb = (int64_t)s * NBS + blk;
                const int64_t n = n0 + wn * (BN / WN) + b * 32 + l32;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t m = m0 + wm * (BM / WM) + a * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                    if (m < g.M && n < g.N) g.P[(jb * g.M + m) * g.N + n] = pt[r];
                }
            }
        } else {
            // The pending item of the previous stage reads parity (NBS-1)&1, row subtile TM-1, column TN-1.
            constexpr bool kClash = ((NBS - 1) & 1) == 0;          // K-block 0 of this stage reuses those registers
            load_scales(0, 0, kClash ? TM - 1 : TM, 0, kClash ? TN - 1 : TN);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < NITEM; ++t) {
                const int blk = t / NSUB, a = (t % NSUB) / TN, b = t % TN;
                // item t-1 (for t = 0: the last item of the previous stage)
                const int u = (t + NITEM - 1) % NITEM, ub = u / NSUB, ua = (u % NSUB) / TN, un = u % TN;
                if constexpr (NBS == 1) {           // operands of the next item: column subtile b+1, then row subtile a+1
                    if (a == 0 && b + 1 < TN) load_w(b + 1);
                    if (b == TN - 1 && a + 1 < TM) load_a(a + 1);
                    __builtin_amdgcn_sched_barrier(0);
                } else {
                    if (t % NSUB == NSUB - 1 && blk + 1 < NBS) {
                        load_block(blk + 1);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
#pragma unroll
                for (int ks = 0; ks < KSB; ++ks) {
                    // at the top of a stage the fold goes first: its inputs are ready, the operands are not yet
                    if (t == 0) fold_slice(p[u & 1], sxv[ub & 1][ua], swv[ub & 1][un], swc[ub & 1][un], acc[ua][un], ks);
                    if (ks == 0)
                        p[t & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[a][blk * KSB], wf[b][blk * KSB], magic, 0, 0, 0);
                    else
                        p[t & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[a][blk * KSB + ks], wf[b][blk * KSB + ks], p[t & 1], 0, 0, 0);
                    if (t != 0) fold_slice(p[u & 1], sxv[ub & 1][ua], swv[ub & 1][un], swc[ub & 1][un], acc[ua][un], ks);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (t == 0) {
                    if (kClash) {
                        load_scales(0, TM - 1, TM, 0, 0);
                        load_scales(0, 0, 0, TN - 1, TN);
                    }
                    prep_scales(0, 0, TN);
                    __builtin_amdgcn_sched_barrier(0);
                }

                // the registers of parity (blk+1)&1 were last read by the fold that just finished when t opens a block
                if (t % NSUB == 0 && blk + 1 < NBS) {
                    load_scales(blk + 1, 0, TM, 0, TN);
                    prep_scales(blk + 1, 0, TN);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };

    // vmcnt(n) alone: wait until at most n of this wave's VMEM instructions are outstanding
    auto wait_vm = [&](auto pending_c) {
        constexpr int kPending = decltype(pending_c)::value;
        static_assert(kPending < 64, "vmcnt is a 6-bit field");
        __builtin_amdgcn_s_waitcnt(0x0F70 | (kPending & 15) | ((kPending >> 4) << 14));
    };
    using Drained = std::integral_constant<int, 0>;

    constexpr bool kPipelined = !PARTIALS && NBS == 1 && TM == 2 && TN == 2 && kBufs == 2;
    if constexpr (kPipelined) {
        // ---- block-128 pipeline: two stage buffers, barrier in the MIDDLE of a stage ------------------------
        // Stage s lives in buffer q = s & 1 and runs the four subtiles in the order (0,f) (0,g) (1,g) (1,f) with
        // f = q, g = 1 - q.  All of its operands are in registers after the second subtile; then ONE barrier
        // certifies for every wave that stage s+1 has landed and that buffer q is no longer read, the loads of
        // stage s+2 start into buffer q, and the operands of stage s+1's first subtile (row subtile 0, column
        // subtile g) are read during subtiles three and four into the registers that subtiles one and two have
        // released.  No wave waits for LDS data right behind a barrier, the stage body is one basic block, and
        // every LDS address is "base register + immediate".
        // Stages past the end of K (the trip count is rounded up to even, and loads run two stages ahead) read
        // their scales through the buffers' range check as zeros, so they add exactly 0 to the accumulators.
        bi8_v4i A0[4], A1[4], Bq[2][4];
        bi8_v4f sx0[4], sx1[4];
        float sw2[2] = {0.0f, 0.0f}, swc2[2] = {0.0f, 0.0f}, pend_sw = 0.0f, pend_swc = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) sx0[i] = sx1[i] = bi8_v4f{0.0f, 0.0f, 0.0f, 0.0f};
        using InFlight1 = std::integral_constant<int, kLoadsPerStage>;

        auto read_a = [&](bi8_v4i *dst, int a, int buf) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) dst[ks] = *(const bi8_v4i *)(lds + a_addr[ks] + buf * L::kABuf + a * 32 * kStageK);
        };
        auto read_w = [&](bi8_v4i *dst, int b, int buf) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) dst[ks] = *(const bi8_v4i *)(lds + w_addr[ks] + buf * L::kWBuf + b * 32 * kStageK);
        };
        auto read_sx = [&](bi8_v4f *dst, int a, int buf) {
#pragma unroll
            for (int i = 0; i < 4; ++i) dst[i] = *(const bi8_v4f *)(lds + sa_addr + buf * L::kSABuf + (a * 32 + 8 * i) * 4);
        };
        // one subtile: four MFMAs, each followed by a slice of the previous subtile's fold
        auto item = [&](bi8_v16i &pdst, const bi8_v4i *af, const bi8_v4i *wf, const bi8_v16i &psrc, const bi8_v4f *sx, float sw,
                        float swcv, float *dst, bool fold_first) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                if (fold_first) fold_slice(psrc, sx, sw, swcv, dst, ks);
                pdst = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[ks], wf[ks], ks == 0 ? magic : pdst, 0, 0, 0);
                if (!fold_first) fold_slice(psrc, sx, sw, swcv, dst, ks);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        auto stage = [&](auto par_c) {
            constexpr int F = decltype(par_c)::value, G = 1 - F;       // F is also this stage's buffer, G the next one's
            // subtile (0,F): its operands were read during the previous stage
            read_w(Bq[G], G, F);
            read_sx(sx0, 0, F);
            float swn[2];
            swn[0] = *(const float *)(lds + sw_addr + F * L::kSWBuf);
            swn[1] = *(const float *)(lds + sw_addr + F * L::kSWBuf + 32 * 4);
            __builtin_amdgcn_sched_barrier(0);
            item(p[0], A0, Bq[F], p[1], sx1, pend_sw, pend_swc, acc[1][G], true);      // folds the previous stage's (1,G)
#pragma unroll
            for (int b = 0; b < 2; ++b) {          // column scales -> 22 significant bits, and -(1.5*2^23) times them
                sw2[b] = bi8_u2f((bi8_f2u(swn[b]) + 2u) & ~3u);
                swc2[b] = -BI8_MAGIC * sw2[b];
            }
            // subtile (0,G)
            read_a(A1, 1, F);
            read_sx(sx1, 1, F);
            __builtin_amdgcn_sched_barrier(0);
            item(p[1], A0, Bq[G], p[0], sx0, sw2[F], swc2[F], acc[0][F], false);
            // every operand of this stage is in registers (or on its way: lgkmcnt below); synchronize
            __builtin_amdgcn_s_waitcnt(0xC07F);    // lgkmcnt(0) only
            wait_vm(Drained{});                    // this wave's loads of stage s+1 have landed
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
            issue_half(F, 0);                      // stage s+2 into the buffer just released: A rows now, the rest one subtile later
            // subtile (1,G), meanwhile the next stage's row subtile 0
            read_a(A0, 0, G);
            __builtin_amdgcn_sched_barrier(0);
            item(p[0], A1, Bq[G], p[1], sx0, sw2[G], swc2[G], acc[0][G], false);
            issue_half(F, 1);
            // subtile (1,F), meanwhile the next stage's column subtile G (its first)
            read_w(Bq[G], G, G);
            __builtin_amdgcn_sched_barrier(0);
            item(p[1], A1, Bq[F], p[0], sx1, sw2[G], swc2[G], acc[1][G], false);
            pend_sw = sw2[F];
            pend_swc = swc2[F];
        };
        using P0 = std::integral_constant<int, 0>;
        using P1 = std::integral_constant<int, 1>;
        // prologue: two stages of loads, wait for the first, read the first subtile's operands
        issue_stage(0);
        issue_stage(1);
        wait_vm(InFlight1{});
        __syncthreads();
        read_a(A0, 0, 0);
        read_w(Bq[0], 0, 0);
        for (int s = 0; s < nstages; s += 2) {
            stage(P0{});
            stage(P1{});
        }
        wait_vm(Drained{});                        // nothing may still be writing LDS when the wave ends
        // the last subtile of the last (possibly padding) stage: always (1,1)
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) fold_slice(p[1], sx1, pend_sw, pend_swc, acc[1][1], ks);
    } else {
    // ---- generic pipeline: barrier at the top of every stage ---------------------------------------------------
    // Ring of kBufs stage buffers.  Before computing stage s every wave waits until only the loads of later
    // stages are still outstanding (its own direct-to-LDS loads of stage s have landed), then the barrier makes
    // that true for all waves and frees the buffer computed one stage earlier.
    auto sync_stage = [&](auto pending_c) {
        __builtin_amdgcn_sched_barrier(0);
        wait_vm(pending_c);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
    };
    // kBufs - 1 stages of loads are in flight while one stage is computed
    using InFlight = std::integral_constant<int, (kBufs - 2) * kLoadsPerStage>;
#pragma unroll
    for (int q = 0; q < kBufs - 1; ++q)
        if (q < nstages) issue_stage(q);
    int s = 0, buf = 0, fill = kBufs - 1;
    for (; s + kBufs - 1 < nstages; ++s) {         // steady state: start the loads of stage s+kBufs-1, compute stage s
        sync_stage(InFlight{});
        issue_stage(fill);
        compute_stage(buf, s);
        buf = (buf == kBufs - 1) ? 0 : buf + 1;
        fill = (fill == kBufs - 1) ? 0 : fill + 1;
    }
    for (; s < nstages; ++s) {                     // drain: nothing left to start; wait for everything each time
        sync_stage(Drained{});
        compute_stage(buf, s);
        buf = (buf == kBufs - 1) ? 0 : buf + 1;
    }
    if constexpr (!PARTIALS)
#pragma unroll
        for (int ks = 0; ks < KSB; ++ks)
            fold_slice(p[(NITEM - 1) & 1], sxv[(NBS - 1) & 1][TM - 1], swv[(NBS - 1) & 1][TN - 1], swc[(NBS - 1) & 1][TN - 1], acc[TM - 1][TN - 1], ks);
    }

    if constexpr (!PARTIALS) {
        const float div = (float)(1.0 / (127.0 * 127.0));
        const bool has_bias = g.bias != nullptr;
#pragma unroll
        for (int b = 0; b < TN; ++b) {
            const int64_t n = n0 + wn * (BN / WN) + b * 32 + l32;
            const bool n_ok = n < g.N;
            const float bias = (has_bias && n_ok) ? load_bias(g, n) : 0.0f;
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t m = m0 + wm * (BM / WM) + a * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                    if constexpr (SLAB) {
                        if (n_ok && m < g.M) slab_store((float *)g.C + (m * g.ldc + n), acc[a][b][r] * div);
                    } else {
                        if (n_ok && m < g.M) store_c<CDT>(g.C, m * g.ldc + n, acc[a][b][r] * div, has_bias, bias);
                    }
                }
        }
    }
}

// SPLIT: the kernel of a split contraction (GemmArgs::splits workgroups, fp32 slabs), a kernel of its own so that the
// one-tile-per-workgroup form stays the code it is.
template <int BM, int BN, int WM, int WN, int NBUF, int BLK, int CDT, bool PARTIALS, bool SPLIT = false>
__global__ __launch_bounds__(WM *WN * 64) void gemm_tile(const GemmArgs g_in) {
    if constexpr (SPLIT) {
        static_assert(!PARTIALS && CDT == BI8_F32, "the slabs are fp32 sums");
        // A piece of a tile's K is the same problem on shifted operands: codes from byte k0 of every row, scale rows from
        // K-block k0 / BLK, and as output the slab, addressed so that element (m0 + i, n0 + j) is slab[i][j].
        // (The divisions below run on the vector unit; their results are wave-uniform and go back to scalar registers,
        // where buffer descriptors and LDS addresses have to be.)
        const int nst = (int)(g_in.K / kStageK), per = g_in.split_per_tile, S = g_in.split_stages;
        const bool runs = per == 0;
        // runs: this workgroup's run of (tile, stage) pairs [u, u_end), piece by piece (at most two: a run is shorter than a
        // tile's K); per-tile splits: one piece
        const int total = g_in.tiles_m * g_in.tiles_n * nst;                 // below 2^30: the plan splits nothing larger
        int u = runs ? (int)blockIdx.x * S : 0;
        const int u_end = runs ? (u + S < total ? u + S : total) : 1;
        while (u < u_end) {
            int tile_m, tile_n, s_lo, s_hi, slab;
            if (runs) {
                const int tile = __builtin_amdgcn_readfirstlane(u / nst);
                s_lo = u - tile * nst;
                s_hi = u_end - u < nst - s_lo ? s_lo + (u_end - u) : nst;
                tile_m = __builtin_amdgcn_readfirstlane(tile / g_in.tiles_n);
                tile_n = tile - tile_m * g_in.tiles_n;
                slab = (int)blockIdx.x + tile;
                u += s_hi - s_lo;
            } else {
                const int tw = __builtin_amdgcn_readfirstlane((int)blockIdx.x / per), part = (int)blockIdx.x - tw * per;
                tile_of_workgroup(tw, g_in.tiles_m, g_in.tiles_n, tile_m, tile_n);
                tile_m = __builtin_amdgcn_readfirstlane(tile_m);
                tile_n = __builtin_amdgcn_readfirstlane(tile_n);
                s_lo = part * S;
                s_hi = s_lo + S < nst ? s_lo + S : nst;
                slab = (tile_m * g_in.tiles_n + tile_n) * per + part;
                u = u_end;
            }
            tile_m += g_in.tile_m0;                // from the launch's tiles to the problem's
            tile_n += g_in.tile_n0;
            GemmArgs g = g_in;
            const int64_t k0 = (int64_t)s_lo * kStageK;
            g.A += k0;
            g.W += k0;
            g.sA += (k0 / BLK) * g.M;
            g.sW += (k0 / BLK) * g.N;
            g.K = (int64_t)(s_hi - s_lo) * kStageK;
            g.C = g.ws + (int64_t)slab * (BM * BN) - ((int64_t)tile_m * BM * BN + (int64_t)tile_n * BN);
            g.ldc = BN;
            g.bias = nullptr;
            gemm_tile_body<BM, BN, WM, WN, NBUF, BLK, CDT, PARTIALS, true>(g, tile_m, tile_n);
            __syncthreads();                       // the next piece's loads reuse the stage buffers
        }
    } else {
        int tile_m, tile_n;
        tile_of_workgroup(blockIdx.x, g_in.tiles_m, g_in.tiles_n, tile_m, tile_n);
        // (the divisions of the tile order run on the vector unit; the tile's coordinates go back to scalar registers,
        // where buffer descriptors have to be)
        gemm_tile_body<BM, BN, WM, WN, NBUF, BLK, CDT, PARTIALS>(g_in, __builtin_amdgcn_readfirstlane(tile_m) + g_in.tile_m0,
                                                                 __builtin_amdgcn_readfirstlane(tile_n) + g_in.tile_n0);
    }
}

// ---- 128 x (16 ... 64) tiles for problems of few tiles, the whole contraction in one workgroup -------------------------
// A problem of a few hundred rows against a wide W fills the chip only if either the contraction is split (slabs, a
// second kernel: the split tile kernels) or the tiles are so narrow that there is one for every CU.  This kernel is
// the second way.  A workgroup streams ALL 128 rows of A (from L2) next to its few rows of W (from memory), 16 KiB of A
// per stage of K whatever the tile's width; in exchange nothing is written twice and nothing waits for a second
// launch, so it wins where K is short (the plan's rule and the measurements behind it: kPanelMaxStages).
// Twelve waves.  Eight compute, each 16 rows x 16 * NJ columns (NJ subtiles of 16 x 16 on v_mfma_i32_16x16x64_i8): stacked,
// a tile of 128 rows (described here), or as 4 x 2 a tile of 64 rows x 32 * NJ columns for up to 64 rows (half the bytes
// of A), or as 2 x 4 a tile of 32 rows x 64 * NJ columns for up to 32.  Four only load: a ring of six to eight stage buffers is filled by their `buffer_load ... lds`, each loader its
// share of a stage's wave-instructions (rows of A, rows of W, scale rows); stages past the end of K are loaded from
// beyond the buffers' ranges (zeros, no memory access), so a loader's count of loads in flight is the same everywhere.
// ONE barrier per stage, which all twelve waves meet: a loader arrives when its loads of stage s + 1 have landed, and
// behind the barrier asks for the stage that goes into the buffer stage s - 1 has left; a computing wave arrives when
// the MFMAs of stage s are issued, and behind the barrier reads the operand fragments of stage s + 1 from LDS, folds
// the partials of stage s - 1 while those reads and the MFMAs are under way, and reads the scales of stage s + 1 into
// the registers that held those of stage s - 1.  Partials and scales are double-buffered in registers by stage parity.
// Why waves that only load.  In the first form of this kernel the eight computing waves loaded as well (three or four
// wave-instructions each per stage).  Timestamps inside that kernel and parts switched off (128 x 4096 x 4096, 32
// stages of 0.31 us each): without the loop's loads 0.18 us per stage, without the fragment reads 0.24, without the MFMAs
// 0.23, without the fold 0.26, without the barrier 0.28 -- the parts of a stage ran one after the other, in all waves at
// once, and a wave that offers a load to a busy path into LDS (one wave-instruction per 16-19 clocks, whoever issues it:
// a stage of A alone streams in 0.13-0.15 us from one, two, four, eight or sixteen waves alike) stands still.  With the
// loads in waves of their own the two run side by side: 128 x 4096 x 2048 8.1 -> 6.6 us, 512 x 1024 x 4096 12.5 -> 9.6,
// 128 x 11008 x 4096 20.1 -> 18.5, 128 x 4096 x 4096 13.4 -> 12.6 (256 workgroups reading the same lines of A: the L2 is the
// limit there).  The loaders' code is specialised per loader at compile time (which item of the stage is of which kind);
// as one copy with a four-way branch per load it ran at 0.6 us per stage.  Measured and not kept in the first form: the
// fragments read a stage earlier into a second set of registers, the ring filled while the first stages are computed
// instead of in front of them (both the same), every wave repeating somebody else's W or scale row to keep the waves'
// counts equal (0.26 against 0.25 us).
// CG = column groups of the eight waves: 1 -> 8 x 1 waves, tiles of 128 rows x 16 * NJ columns; 2 -> 4 x 2 waves, tiles of
// 64 rows x 32 * NJ columns (for up to 64 rows: half the bytes of A per stage); 4 -> 2 x 4 waves, tiles of 32 rows x 64 * NJ
// columns (for up to 32 rows: a quarter)
// NI = 16-row subtiles per wave (1 or 2): with two, 4 x 2 waves make a tile of 128 rows x 32 * NJ columns (the square form below)
template <int NBS, int NJ, int CG, int NI = 1> struct PanelLds {
    static constexpr int BM = 128 * NI / CG, BN = 16 * NJ * CG;
    static constexpr int kSWRow = (BN + 63) / 64 * 64;                       // (a scale row is loaded 64 floats at a time)
    static constexpr int kABuf = BM * kStageK, kWBuf = BN * kStageK;         // 16, 8 or 4 KiB; 2 ... 32 KiB
    static constexpr int kSARow = BM > 64 ? BM : 64;                         // (... and so is a row of row scales)
    static constexpr int kSABuf = NBS * kSARow * 4, kSWBuf = NBS * kSWRow * 4;
    static constexpr int kStage = kABuf + kWBuf + kSABuf + kSWBuf;
    static constexpr int kBufs = (158 * 1024 / kStage) >= 8 ? 8 : (158 * 1024 / kStage) >= 6 ? (158 * 1024 / kStage) : 4;
    static constexpr int kAReg = 0;
    static constexpr int kWReg = kAReg + kBufs * kABuf;
    static constexpr int kSAReg = kWReg + kBufs * kWBuf;
    static constexpr int kSWReg = kSAReg + kBufs * kSABuf;
    static constexpr int kBytes = kSWReg + kBufs * kSWBuf;
    static_assert(kBytes <= 160 * 1024, "LDS per CU");
};

constexpr int kPanelLoaders = 4;               // waves of a gemm_panel workgroup that only load
constexpr int kPanelThreads = (8 + kPanelLoaders) * 64;
// The computing waves of the forms with one 16-row subtile per wave: `wave` = row group rg (16 rows), column group cg
// (16 * NJ columns).
template <int BLK, int CDT, int NJ, int CG, bool SPLIT>
__device__ __forceinline__ void panel_compute_rows(const GemmArgs &g, uint8_t *lds, int wave, int lane, int64_t m0, int64_t n0, int64_t n_end, int nst) {
    constexpr int NBS = kStageK / BLK;
    using L = PanelLds<NBS, NJ, CG>;
    constexpr int BM = L::BM, BN = L::BN, RG = 8 / CG, kBufs = L::kBufs;     // RG = row groups of 16 rows
    auto next_buf = [](int buf) { return buf + 1 == kBufs ? 0 : buf + 1; };      // the ring's buffer after `buf`
    const int rg = wave % RG, cg = wave / RG;
    const int r16 = lane & 15, q = lane >> 4;
    // operand fragments: lane -> row r16 of a 16-row subtile, 16-byte chunk 4*kb + q of the stage's eight, stored at chunk
    // position (4*kb + q) ^ (r16 >> 1): the address of kb = 1 is that of kb = 0 with bit 6 flipped
    int a_base = L::kAReg + (rg * 16 + r16) * kStageK + ((q ^ (r16 >> 1)) << 4);
    int w_base = L::kWReg + (cg * 16 * NJ + r16) * kStageK + ((q ^ (r16 >> 1)) << 4);
    // a subtile's outputs: lane -> column r16, rows 4q .. 4q+3
    int sa_base = L::kSAReg + (rg * 16 + 4 * q) * 4;
    int sw_base = L::kSWReg + (cg * 16 * NJ + r16) * 4;
    asm volatile("" : "+v"(a_base), "+v"(w_base), "+v"(sa_base), "+v"(sw_base));
    constexpr int kMagicBits = 0x4B400000;        // bit pattern of 1.5 * 2^23
    const bi8_v4i magic = {kMagicBits, kMagicBits, kMagicBits, kMagicBits};

    float acc[NJ][4];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[j][r] = 0.0f;
    bi8_v4i A[2], B[NJ][2];                        // [kb], [column subtile][kb]: the current stage's operands
    bi8_v4i c[2][NBS][NJ];                         // [stage parity][K-block][column subtile]
    bi8_v4f sx[2][NBS];                            // [stage parity][K-block]: row scales
    float bw[2][NBS][NJ];                          // ... [column subtile]: column scales

    auto read_frags = [&](int buf) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            A[kb] = *(const bi8_v4i *)(lds + (a_base ^ (kb * 64)) + buf * L::kABuf);
#pragma unroll
            for (int j = 0; j < NJ; ++j) B[j][kb] = *(const bi8_v4i *)(lds + (w_base ^ (kb * 64)) + buf * L::kWBuf + j * 16 * kStageK);
        }
    };
    auto read_scales = [&](int buf, auto par_c) {
        constexpr int P = decltype(par_c)::value;
#pragma unroll
        for (int kb = 0; kb < NBS; ++kb) {
            sx[P][kb] = *(const bi8_v4f *)(lds + sa_base + buf * L::kSABuf + kb * L::kSARow * 4);
#pragma unroll
            for (int j = 0; j < NJ; ++j) bw[P][kb][j] = *(const float *)(lds + sw_base + buf * L::kSWBuf + (kb * L::kSWRow + j * 16) * 4);
        }
    };
    auto mfmas = [&](auto par_c) {
        constexpr int P = decltype(par_c)::value;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int blk = NBS == 2 ? kb : 0;
                const bool first = NBS == 2 || kb == 0;
                c[P][blk][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[kb], B[j][kb], first ? magic : c[P][blk][j], 0, 0, 0);
            }
    };
    // a stage's partials into the accumulators: per K-block and subtile four products, then four accumulations
    auto fold = [&](auto par_c) {
        constexpr int P = decltype(par_c)::value;
#pragma unroll
        for (int kb = 0; kb < NBS; ++kb)
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const float b = bi8_u2f((bi8_f2u(bw[P][kb][j]) + 2u) & ~3u);     // 22 significant bits: -(1.5*2^23)*b is exact
                const float cm = -BI8_MAGIC * b;
                float t[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) t[r] = __builtin_fmaf(bi8_u2f((uint32_t)c[P][kb][j][r]), b, cm);
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[j][r] = __builtin_fmaf(t[r], sx[P][kb][r], acc[j][r]);
            }
    };
    // stage s (parity P, its operands in A and B): MFMAs; the barrier that publishes stage s + 1; its operands from LDS; the
    // fold of stage s - 1; the scales of stage s + 1 into the registers that held those of stage s - 1
    int buf = 0;
    auto step = [&](auto par_c, bool fold_prev) {
        constexpr int P = decltype(par_c)::value;
        using Q = std::integral_constant<int, 1 - P>;
        mfmas(par_c);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        buf = next_buf(buf);
        read_frags(buf);
        __builtin_amdgcn_sched_barrier(0);
        if (fold_prev) fold(Q{});
        __builtin_amdgcn_sched_barrier(0);
        read_scales(buf, Q{});
    };

    __syncthreads();                               // stage 0 is published
    read_frags(0);
    read_scales(0, std::integral_constant<int, 0>{});
    step(std::integral_constant<int, 0>{}, false);
    int s = 1;
    for (; s + 1 < nst; s += 2) {
        step(std::integral_constant<int, 1>{}, true);
        step(std::integral_constant<int, 0>{}, true);
    }
    if (s < nst) {                                 // an even number of stages: one more, of odd parity
        step(std::integral_constant<int, 1>{}, true);
        fold(std::integral_constant<int, 1>{});
    } else {
        fold(std::integral_constant<int, 0>{});
    }

    const float div = (float)(1.0 / (127.0 * 127.0));
    const bool has_bias = !SPLIT && g.bias != nullptr;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int64_t n = n0 + cg * 16 * NJ + j * 16 + r16;
        const bool n_ok = n < n_end;
        const float bias = (has_bias && n_ok) ? load_bias(g, n) : 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int64_t m = m0 + rg * 16 + 4 * q + r;
            if constexpr (SPLIT) {
                float *slab = g.ws + ((int64_t)blockIdx.x * gridDim.y + blockIdx.y) * (BM * BN);
                if (n_ok && m < g.M) slab_store(slab + (rg * 16 + 4 * q + r) * BN + cg * 16 * NJ + j * 16 + r16, acc[j][r] * div);
            } else {
                if (n_ok && m < g.M) store_c<CDT>(g.C, m * g.ldc + n, acc[j][r] * div, has_bias, bias);
            }
        }
    }
}

// The computing waves of the square form (NI = 2): 4 x 2 waves, each 32 rows x 16 * NJ columns as 2 x NJ subtiles, a tile of
// 128 rows x 32 * NJ columns.  Per byte read from LDS a wave does twice the MFMAs of the one-subtile-high forms (a stage's
// fragment reads are what bounds those at 64 columns per wave).  To stay within the 168 registers that twelve waves leave
// each lane, the int32 partials are double-buffered by HALF stages, and the next stage's fragments are read in two parts, each
// right behind the MFMAs that were the last to read the registers it goes into, so that the LDS reads run under MFMAs and
// folds (the order of a stage: at `step` below).
template <int BLK, int CDT, int NJ, bool SPLIT>
__device__ __forceinline__ void panel_compute_square(const GemmArgs &g, uint8_t *lds, int wave, int lane, int64_t m0, int64_t n0, int64_t n_end, int nst) {
    constexpr int NBS = kStageK / BLK, NI = 2, CG = 2, RG = 4, NH = NJ / 2;
    using L = PanelLds<NBS, NJ, CG, NI>;
    constexpr int BM = L::BM, BN = L::BN, kBufs = L::kBufs;
    auto next_buf = [](int buf) { return buf + 1 == kBufs ? 0 : buf + 1; };
    const int rg = wave % RG, cg = wave / RG;
    const int r16 = lane & 15, q = lane >> 4;
    int a_base = L::kAReg + (rg * 16 * NI + r16) * kStageK + ((q ^ (r16 >> 1)) << 4);
    int w_base = L::kWReg + (cg * 16 * NJ + r16) * kStageK + ((q ^ (r16 >> 1)) << 4);
    int sa_base = L::kSAReg + (rg * 16 * NI + 4 * q) * 4;
    int sw_base = L::kSWReg + (cg * 16 * NJ + r16) * 4;
    asm volatile("" : "+v"(a_base), "+v"(w_base), "+v"(sa_base), "+v"(sw_base));
    constexpr int kMagicBits = 0x4B400000;        // bit pattern of 1.5 * 2^23
    const bi8_v4i magic = {kMagicBits, kMagicBits, kMagicBits, kMagicBits};

    float acc[NI][NJ][4];
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;
    bi8_v4i A[NI][2], B[NJ][2];                    // [subtile][kb]: the current stage's operands
    bi8_v4i c[2][NBS][NI][NH];                     // [half of the columns][K-block][row subtile][column subtile of the half]
    bi8_v4f sx[2][NBS][NI];                        // [stage parity][K-block][row subtile]: row scales
    float bw[2][NBS][NJ];                          // ... [column subtile]: column scales

    auto read_a = [&](int buf) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < NI; ++i) A[i][kb] = *(const bi8_v4i *)(lds + (a_base ^ (kb * 64)) + buf * L::kABuf + i * 16 * kStageK);
    };
    auto read_b = [&](int buf, auto half_c) {      // the W fragments of one half of the columns
        constexpr int H = decltype(half_c)::value;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int jj = 0; jj < NH; ++jj)
                B[H * NH + jj][kb] = *(const bi8_v4i *)(lds + (w_base ^ (kb * 64)) + buf * L::kWBuf + (H * NH + jj) * 16 * kStageK);
    };
    auto read_scales = [&](int buf, auto par_c) {
        constexpr int P = decltype(par_c)::value;
#pragma unroll
        for (int kb = 0; kb < NBS; ++kb) {
#pragma unroll
            for (int i = 0; i < NI; ++i) sx[P][kb][i] = *(const bi8_v4f *)(lds + sa_base + buf * L::kSABuf + (kb * L::kSARow + i * 16) * 4);
#pragma unroll
            for (int j = 0; j < NJ; ++j) bw[P][kb][j] = *(const float *)(lds + sw_base + buf * L::kSWBuf + (kb * L::kSWRow + j * 16) * 4);
        }
    };
    auto mfmas = [&](auto half_c) {
        constexpr int H = decltype(half_c)::value;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
                for (int jj = 0; jj < NH; ++jj) {
                    const int blk = NBS == 2 ? kb : 0;
                    const bool first = NBS == 2 || kb == 0;
                    c[H][blk][i][jj] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[i][kb], B[H * NH + jj][kb], first ? magic : c[H][blk][i][jj], 0, 0, 0);
                }
    };
    // half H of a stage (its scales in parity P) into the accumulators: per K-block and subtile four products, then four accumulations
    auto fold = [&](auto half_c, auto par_c) {
        constexpr int H = decltype(half_c)::value, P = decltype(par_c)::value;
#pragma unroll
        for (int kb = 0; kb < NBS; ++kb)
#pragma unroll
            for (int jj = 0; jj < NH; ++jj) {
                const float b = bi8_u2f((bi8_f2u(bw[P][kb][H * NH + jj]) + 2u) & ~3u);      // 22 significant bits: -(1.5*2^23)*b is exact
                const float cm = -BI8_MAGIC * b;
#pragma unroll
                for (int i = 0; i < NI; ++i) {
                    float t[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) t[r] = __builtin_fmaf(bi8_u2f((uint32_t)c[H][kb][i][jj][r]), b, cm);
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[i][H * NH + jj][r] = __builtin_fmaf(t[r], sx[P][kb][i][r], acc[i][H * NH + jj][r]);
                }
            }
    };
    using H0 = std::integral_constant<int, 0>;
    using H1 = std::integral_constant<int, 1>;
    // stage s (its operands in A and B, its scales in parity P): the barrier that publishes stage s + 1; the MFMAs of the left
    // columns, behind them the left W fragments of stage s + 1 into the registers they have just read; the fold of the right
    // columns of stage s - 1; the MFMAs of the right columns, behind them the A and the right W fragments of stage s + 1; the
    // fold of the left columns; the scales of stage s + 1 into the registers that held those of stage s - 1
    int buf = 0;
    auto step = [&](auto par_c, bool fold_prev) {
        constexpr int P = decltype(par_c)::value;
        using Q = std::integral_constant<int, 1 - P>;
        __syncthreads();
        buf = next_buf(buf);
        __builtin_amdgcn_sched_barrier(0);
        mfmas(H0{});
        __builtin_amdgcn_sched_barrier(0);
        read_b(buf, H0{});
        __builtin_amdgcn_sched_barrier(0);
        if (fold_prev) fold(H1{}, Q{});
        __builtin_amdgcn_sched_barrier(0);
        mfmas(H1{});
        __builtin_amdgcn_sched_barrier(0);
        read_a(buf);
        read_b(buf, H1{});
        __builtin_amdgcn_sched_barrier(0);
        fold(H0{}, par_c);
        __builtin_amdgcn_sched_barrier(0);
        read_scales(buf, Q{});
    };

    __syncthreads();                               // stage 0 is published
    read_a(0);
    read_b(0, H0{});
    read_b(0, H1{});
    read_scales(0, std::integral_constant<int, 0>{});
    step(std::integral_constant<int, 0>{}, false);
    int s = 1;
    for (; s + 1 < nst; s += 2) {
        step(std::integral_constant<int, 1>{}, true);
        step(std::integral_constant<int, 0>{}, true);
    }
    if (s < nst) {                                 // an even number of stages: one more, of odd parity
        step(std::integral_constant<int, 1>{}, true);
        fold(H1{}, std::integral_constant<int, 1>{});
    } else {
        fold(H1{}, std::integral_constant<int, 0>{});
    }

    const float div = (float)(1.0 / (127.0 * 127.0));
    const bool has_bias = !SPLIT && g.bias != nullptr;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int64_t n = n0 + cg * 16 * NJ + j * 16 + r16;
        const bool n_ok = n < n_end;
        const float bias = (has_bias && n_ok) ? load_bias(g, n) : 0.0f;
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = rg * 16 * NI + i * 16 + 4 * q + r;
                const int64_t m = m0 + row;
                if constexpr (SPLIT) {
                    float *slab = g.ws + ((int64_t)blockIdx.x * gridDim.y + blockIdx.y) * (BM * BN);
                    if (n_ok && m < g.M) slab_store(slab + row * BN + cg * 16 * NJ + j * 16 + r16, acc[i][j][r] * div);
                } else {
                    if (n_ok && m < g.M) store_c<CDT>(g.C, m * g.ldc + n, acc[i][j][r] * div, has_bias, bias);
                }
            }
    }
}

// SPLIT: K in gridDim.y pieces of GemmArgs::split_stages stages; workgroup (t, y) writes the fp32 sums of its piece, scaled,
// without bias, to slab t * gridDim.y + y of the workspace ([BM][BN] each), and splitk_reduce adds a tile's slabs.
template <int BLK, int CDT, int NJ, int CG = 1, bool SPLIT = false, int NI = 1>
__global__ __launch_bounds__(kPanelThreads) void gemm_panel(const GemmArgs g) {
    static_assert(!SPLIT || CDT == BI8_F32, "the slabs are fp32 sums");
    static_assert(BLK == 128 || BLK == 64, "a K-block is one or two MFMAs of 64 bytes of K");
    static_assert(NJ >= 1 && NJ <= 4 && (CG == 1 || CG == 2 || CG == 4), "16 ... 64 columns per wave, one, two or four waves side by side");
    static_assert(NI == 1 || (NI == 2 && CG == 2 && NJ % 2 == 0), "two row subtiles per wave: the square form, its columns in two halves");
    constexpr int NBS = kStageK / BLK;
    using L = PanelLds<NBS, NJ, CG, NI>;
    constexpr int BM = L::BM, BN = L::BN;
    constexpr int kBufs = L::kBufs;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t lds_base = bi8_lds_address(lds);
    const int tile_m = (int)blockIdx.x / g.tiles_n, tile_n = (int)blockIdx.x - tile_m * g.tiles_n;
    const int pitch = !SPLIT && g.panel_pitch > 0 ? g.panel_pitch : BN;
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * pitch;
    const int64_t n_end = g.N - n0 < pitch ? g.N : n0 + pitch;                  // the tile's columns: n0 ... n_end - 1
    const int stage_lo = SPLIT ? (int)blockIdx.y * g.split_stages : 0;          // this workgroup's first stage of K, and how many
    const int nst = SPLIT ? ((int)(g.K / kStageK) - stage_lo < g.split_stages ? (int)(g.K / kStageK) - stage_lo : g.split_stages)
                          : (int)(g.K / kStageK);
    auto wait_vm = [&](auto pending_c) {
        constexpr int kPending = decltype(pending_c)::value;
        static_assert(kPending < 64, "vmcnt is a 6-bit field");
        __builtin_amdgcn_s_waitcnt(0x0F70 | (kPending & 15) | ((kPending >> 4) << 14));
    };
    auto next_buf = [](int buf) { return buf + 1 == kBufs ? 0 : buf + 1; };      // the ring's buffer after `buf`

    if (wave >= 8) {
        // ---- the loading waves.  A stage is a list of wave-instructions: BM / 8 of rows of A and BN / 8 of rows of W (an
        // instruction covers tile rows 8i .. 8i+7, lane -> row 8i + lane/8, LDS chunk lane%8, which holds source chunk
        // (lane%8) ^ ((row >> 1) & 7)), then per K-block the row scales and the column scales, 64 floats per instruction.
        // Loader P takes items P, P + 4, ... (all its row items have the parity of P); which item is of which kind is known
        // at compile time, one copy of the code per loader.  Stages past the end of K are loaded from beyond the buffers'
        // ranges (zeros, no memory access), so a loader's count of loads in flight never changes.
        constexpr int kAItems = BM / 8, kWItems = BN / 8;
        constexpr int kSAParts = L::kSARow / 64, kSWParts = L::kSWRow / 64, kSParts = kSAParts + kSWParts;
        constexpr int kItems = kAItems + kWItems + kSParts * NBS, kSlots = (kItems + kPanelLoaders - 1) / kPanelLoaders;
        static_assert(kAItems % 2 == 0 && kPanelLoaders % 2 == 0, "the swizzle term of a loader's row items does not depend on the slot");
        static_assert((kBufs - 1) * kSlots < 64, "a loader's loads in flight fit the counter");
        const int64_t nblk = g.K / BLK;
        const int64_t a_rows = g.M - m0 < BM ? g.M - m0 : BM, w_rows = n_end - n0;
        const bi8_rsrc a_rsrc = bi8_make_rsrc(g.A + m0 * g.lda, (a_rows - 1) * g.lda + g.K);
        const bi8_rsrc w_rsrc = bi8_make_rsrc(g.W + n0 * g.ldw, (w_rows - 1) * g.ldw + g.K);
        const bi8_rsrc sa_rsrc = bi8_make_rsrc(g.sA + m0, ((nblk - 1) * g.M + (g.M - m0)) * 4);
        const bi8_rsrc sw_rsrc = bi8_make_rsrc(g.sW + n0, ((nblk - 1) * g.N + (g.N - n0)) * 4);
        const uint32_t sa_row = (uint32_t)(g.M * 4), sw_row = (uint32_t)(g.N * 4);          // bytes from one K-block's scales to the next
        auto loader = [&](auto p_c) {
            constexpr int P = decltype(p_c)::value;
            constexpr int kMine = (kItems - P + kPanelLoaders - 1) / kPanelLoaders;          // this loader's items per stage
            const int ld_row = lane >> 3;
            const int ld_chunk = (lane & 7) ^ ((4 * (P & 1) + (lane >> 4)) & 7);
            const uint32_t a_lane = (uint32_t)(ld_row * g.lda + ld_chunk * 16), w_lane = (uint32_t)(ld_row * g.ldw + ld_chunk * 16);
            const uint32_t a_item = (uint32_t)(8 * g.lda), w_item = (uint32_t)(8 * g.ldw);  // from one row item to the next
            const uint32_t s_lane = (uint32_t)(lane * 4);
            auto issue_stage = [&](int buf, int s) {   // both wave-uniform
                const bool real = s < nst;
                const uint32_t k_pos = real ? (uint32_t)((stage_lo + s) * kStageK) : (uint32_t)kBufOut;
                const uint32_t kb0 = (uint32_t)((stage_lo + s) * NBS);
#pragma unroll
                for (int e = 0; e < kMine; ++e) {
                    constexpr int kA = kAItems, kW = kWItems;
                    const int item = e * kPanelLoaders + P;            // a constant after unrolling
                    if (item < kA) {
                        bi8_buffer_to_lds16_sum(a_rsrc, lds_base + L::kAReg + buf * L::kABuf + item * 1024, a_lane, k_pos, (uint32_t)item * a_item);
                    } else if (item < kA + kW) {
                        bi8_buffer_to_lds16_sum(w_rsrc, lds_base + L::kWReg + buf * L::kWBuf + (item - kA) * 1024, w_lane, k_pos, (uint32_t)(item - kA) * w_item);
                    } else {
                        const int sc = item - kA - kW, kb = sc / kSParts, r = sc % kSParts;
                        if (r < kSAParts) {
                            const uint32_t pos = real ? (kb0 + kb) * sa_row + r * 256 : (uint32_t)kBufOut;
                            bi8_buffer_to_lds4(sa_rsrc, lds_base + L::kSAReg + buf * L::kSABuf + (kb * L::kSARow + r * 64) * 4, s_lane, pos);
                        } else {
                            const uint32_t pos = real ? (kb0 + kb) * sw_row + (r - kSAParts) * 256 : (uint32_t)kBufOut;
                            bi8_buffer_to_lds4(sw_rsrc, lds_base + L::kSWReg + buf * L::kSWBuf + (kb * L::kSWRow + (r - kSAParts) * 64) * 4, s_lane, pos);
                        }
                    }
                }
            };
#pragma unroll
            for (int s = 0; s < kBufs - 1; ++s) issue_stage(s, s);
            wait_vm(std::integral_constant<int, (kBufs - 2) * kMine>{});                 // stage 0 has landed
            __syncthreads();
            int fill = kBufs - 1;
            for (int s = 0; s < nst; ++s) {
                wait_vm(std::integral_constant<int, (kBufs - 3) * kMine>{});             // stage s + 1 has landed
                __syncthreads();                   // ... for every loader: published; and the computing waves have left stage s - 1
                issue_stage(fill, s + kBufs - 1);
                fill = next_buf(fill);
            }
            wait_vm(std::integral_constant<int, 0>{});     // (the loads past the end of K) nothing may still be writing LDS when the wave ends
        };
        static_assert(kPanelLoaders == 4, "one copy of the loader per loading wave");
        if (wave == 8) loader(std::integral_constant<int, 0>{});
        else if (wave == 9) loader(std::integral_constant<int, 1>{});
        else if (wave == 10) loader(std::integral_constant<int, 2>{});
        else loader(std::integral_constant<int, 3>{});
        return;
    }

    if constexpr (NI == 2) panel_compute_square<BLK, CDT, NJ, SPLIT>(g, lds, wave, lane, m0, n0, n_end, nst);
    else panel_compute_rows<BLK, CDT, NJ, CG, SPLIT>(g, lds, wave, lane, m0, n0, n_end, nst);
}

// ---- 256x256 tile, block 128 ------------------------------------------------------------------------------------
// The large-problem kernel.  Twice the output per byte of operand moved from L2 to LDS compared to the 256x128
// tile, which is what bounds gemm_tile at large sizes.  8 waves as 4 (rows) x 2 (columns); one wave owns 64 x 128
// outputs as 4 x 8 subtiles of 16x16 (v_mfma_i32_16x16x64_i8: four accumulator registers per subtile, so the
// int32 partials of two columns in flight cost 32 registers and the row scales of a stage 16), 128 fp32
// accumulators per lane.  Per stage (128 bytes of K = one K-block) a wave keeps its 64 rows of A in registers and
// streams the eight column subtiles of W through two register buffers, one column ahead.  A column's eight MFMAs
// are issued back to back, then the whole fold of the column before: a wave's vector instructions run under its own
// MFMAs only (the two waves of a SIMD do not overlap one's MFMAs with the other's vector work), and long runs of
// each measured faster than alternating instruction by instruction.  Two LDS stage buffers, ONE barrier per stage, placed where the last
// operand of the stage has been read (top of the eighth column): it certifies that the next stage has landed
// and releases this stage's buffer to the loads of the stage after next.
// Measured on MI355X: a SIMD issues about one instruction of any kind per 4 cycles, so the kernel is bound by its
// instruction count; two fold instructions per output per K-block are 2/3 of it.
// The grid is persistent, one workgroup per CU (the LDS admits no second one): a workgroup walks tiles b, b + grid, ...
// of the XCD-aware order and never drains its pipeline between them, so a tile's outputs leave (through a small
// wave-private LDS strip) while the next tile's first stages land.  Measured against one workgroup per tile:
// 8192^3 -1.5 %, 8192 x 50257 x 768 -13 %.
template <int NBS, int BN = 256> struct WideLds {   // NBS = K-blocks per stage, BN = columns of the tile (256 or 128)
    static constexpr int kABuf = 256 * kStageK, kWBuf = BN * kStageK;        // 32 KiB (16 KiB) per operand per stage
    static constexpr int kSRow = 256 * 4;                                    // one row-scale row of the tile
    static constexpr int kSBuf = NBS * kSRow;                                // the stage's row scales, one row per K-block
    // column scales are stored prepared: per column the pair (b, -1.5*2^23*b), b = the scale rounded to 22 significant
    // bits; a wave's BN/2 columns as [column pair 2p, 2p+1][r16][b0, c0, b1, c1], so a lane reads two columns' pairs at once
    static constexpr int kCRow = BN * 8;
    static constexpr int kCBuf = NBS * kCRow;
    static constexpr int kAReg = 0;
    static constexpr int kWReg = kAReg + 2 * kABuf;
    static constexpr int kSAReg = kWReg + 2 * kWBuf;
    static constexpr int kSWReg = kSAReg + 2 * kSBuf;
    // after the K loop the same memory holds each wave's 64x128 tile of 16-bit outputs, row-major; the pitch
    // (256 + 16 bytes) puts the four row groups of one accumulator register into different banks
    static constexpr int kOutPitch = 272;
    static constexpr int kDummy = kSWReg + 2 * kCBuf;                        // gemm_wide32: 1 KiB written and never read
    static constexpr int kBiasReg = kDummy;                                  // gemm_wide: the tile's bias, BN x 4 bytes
    static constexpr int kStages = kDummy + 1024;                            // 135 / 141 KiB
    // gemm_wide: next to the stage buffers every wave owns a strip of 16 rows x 64 columns of 16-bit outputs, through
    // which its accumulators leave as row-major runs while the next tile's first stages are already landing in the
    // stage buffers; the pitch (128 + 16 bytes) puts the four row groups of one accumulator register into different banks
    static constexpr int kStripPitch = 144;
    static constexpr int kStripBytes = 16 * kStripPitch;
    static constexpr int kStrips = kStages;
    static constexpr int kBytesPersistent = kStages + 8 * kStripBytes;       // 153 / 159 KiB of the CU's 160
    static constexpr int kOut = 8 * 64 * kOutPitch;                          // 136 KiB
    static constexpr int kBytes = kOut > kStages ? kOut : kStages;           // of the CU's 160 KiB
};

// NJ = column subtiles of a wave: 8 is the 256x256 tile described above; 4 a 256x128 tile (64x64 per wave) for problems
// that do not fill the chip with 256x256 tiles -- the same loop on half the columns, so half the MFMAs per LDS read of A.
// SPLIT: the contraction is split over gridDim.y workgroups per tile (GemmArgs::split_stages stages of K each, an even
// number, so that the padding stage of an odd trip count exists only at the end of K, where the scales read as zeros);
// workgroup (t, y) writes the fp32 sums of its piece, scaled, without bias, to slab (row-major tile index) * gridDim.y + y
// of the workspace, and splitk_reduce adds a tile's slabs.  One piece per workgroup: the grid is not persistent.
template <int BLK, int CDT, int NJ = 8, bool SPLIT = false>
__global__ __launch_bounds__(512) void gemm_wide(const GemmArgs g) {
    static_assert(BLK == 128 || BLK == 64, "a K-block is one or two 64-byte MFMAs");
    static_assert(NJ == 8 || NJ == 4, "64x128 or 64x64 per wave");
    static_assert(!SPLIT || CDT == BI8_F32, "the slabs are fp32 sums");
    constexpr int NBS = kStageK / BLK;
    constexpr int BM = 256, BN = 32 * NJ, WC = 16 * NJ, NW = 8;       // WC = columns of a wave
    using L = WideLds<NBS, BN>;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int r16 = lane & 15, q = lane >> 4;

    // The grid is persistent: workgroup b computes tiles b, b + gridDim.x, ... of the XCD-aware tile order, and the
    // stage pipeline runs on across tile boundaries: while a tile's last two stages are computed the loader already
    // fetches the first two stages of the workgroup's next tile, and they land while the accumulators leave.
    const int ntiles = g.tiles_m * g.tiles_n;
    const int stage_lo = SPLIT ? (int)blockIdx.y * g.split_stages : 0;          // this workgroup's first stage of K
    const int nstages = SPLIT ? ((int)(g.K / kStageK) - stage_lo < g.split_stages ? (int)(g.K / kStageK) - stage_lo : g.split_stages)
                              : (int)(g.K / kStageK);
    const int npairs = (nstages + 1) >> 1;         // the trip count is rounded up to even (see below)
    int pid = blockIdx.x;                          // the tile being computed
    int m0, n0, slab = 0;
    {
        int tile_m, tile_n;
        tile_of_workgroup_scalar(pid, g.tiles_m, g.tiles_n, g.band_magic, tile_m, tile_n);
        m0 = (tile_m + g.tile_m0) * BM;
        n0 = (tile_n + g.tile_n0) * BN;
        if constexpr (SPLIT) slab = (tile_m * g.tiles_n + tile_n) * (int)gridDim.y + (int)blockIdx.y;
    }

    // ---- loader (same scheme as gemm_tile): wave instruction i covers tile rows 8i .. 8i+7, lane -> row
    // 8i + lane/8, LDS chunk lane%8, which holds source chunk (lane%8) ^ ((row >> 1) & 7); i = wave + 8*it.
    // One buffer per operand over the whole matrix (the host checks that each is below 2 GiB); the tile and the K
    // position are scalar offsets.  Rows past the end of a matrix are past the end of its buffer and read as zeros.
    const int ld_row = lane >> 3;
    const int ld_chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);
    const bi8_rsrc a_rsrc = bi8_make_rsrc(g.A, (g.M - 1) * g.lda + g.K);
    const bi8_rsrc w_rsrc = bi8_make_rsrc(g.W, (g.N - 1) * g.ldw + g.K);
    const uint32_t a_off = (uint32_t)(ld_row * g.lda + ld_chunk * 16), w_off = (uint32_t)(ld_row * g.ldw + ld_chunk * 16);
    const uint32_t a_wave = (uint32_t)(wave * 8 * g.lda), w_wave = (uint32_t)(wave * 8 * g.ldw);
    const uint32_t a_step = (uint32_t)(NW * 8 * g.lda), w_step = (uint32_t)(NW * 8 * g.ldw);
    // scale rows of the stage's K-blocks: waves 0-3 fetch 64 row scales each, waves 4-7 64 column scales each (of a
    // 128-column tile: waves 6 and 7 repeat what waves 4 and 5 do)
    const int64_t nblk = g.K / BLK;
    const bool s_is_a = wave < 4;
    const int s_part = s_is_a ? wave : (wave & 3) % (BN / 64);
    const bi8_brsrc s_brsrc = s_is_a ? bi8_make_brsrc(g.sA, nblk * g.M * 4) : bi8_make_brsrc(g.sW, nblk * g.N * 4);
    const uint32_t s_off = (uint32_t)((s_part * 64 + lane) * 4);
    const uint32_t s_inc = (uint32_t)((s_is_a ? g.M : g.N) * 4);
    // The scales come into a register of the fetching lane, which stores them to LDS just before the barrier that
    // publishes the stage.  Row scales are stored as they are.  Column scales are stored prepared, so that the
    // preparation is done once per column instead of once per wave row and lane group: lane -> tile column
    // s_part * 64 + lane = wave column wn, subtile j, r16 = lane % 16; pair j / 2, half j % 2 of its 16 bytes.
    // Both kinds run the same instructions (no branch: a branch in the K loop costs the register allocator its
    // footing): two 4-byte stores, the second of a row-scale lane to a slot nobody reads.
    float s_raw[NBS];
#pragma unroll
    for (int kb = 0; kb < NBS; ++kb) s_raw[kb] = 0.0f;
    const int c_col = s_part * 64 + lane, c_j = (c_col % WC) >> 4;
    const int c_dst = L::kSWReg + (c_col / WC) * (WC * 8) + (((c_j >> 1) * 16 + (lane & 15)) * 2 + (c_j & 1)) * 8;
    int p_dst0 = s_is_a ? L::kSAReg + (s_part * 64 + lane) * 4 : c_dst;
    int p_dst1 = s_is_a ? L::kStrips + wave * L::kStripBytes + lane * 4 : c_dst + 4;     // the wave's strip is idle during the K loop
    const int p_buf0 = s_is_a ? L::kSBuf : L::kCBuf, p_row0 = s_is_a ? L::kSRow : L::kCRow;
    const int p_buf1 = s_is_a ? 0 : L::kCBuf, p_row1 = s_is_a ? 0 : L::kCRow;
    // The loader walks the stream of stages (this tile's, then the next tile's) at two positions one stage apart:
    // E, where a stage gets its first kEarly loads (rows of A), and L, where it gets the others.  A position is the
    // byte offset of (tile, K position) in each operand; all of them are wave-uniform.
    uint32_t ao_E = (uint32_t)(m0 * g.lda + stage_lo * kStageK), ao_L = ao_E, wo_L = (uint32_t)(n0 * g.ldw + stage_lo * kStageK);
    uint32_t so_L = (uint32_t)((s_is_a ? m0 : n0) * 4) + (uint32_t)(stage_lo * NBS) * s_inc;
    uint32_t ao_nxt = 0, wo_nxt = 0, so_nxt = 0;   // the workgroup's next tile
    int m0_nxt = 0, n0_nxt = 0;
    auto aim_next = [&](int p) {
        int tile_m, tile_n;
        // past the last tile: tile 0 once more, a stage or two loaded and never used
        tile_of_workgroup_scalar(p < ntiles ? p : 0, g.tiles_m, g.tiles_n, g.band_magic, tile_m, tile_n);
        m0_nxt = (tile_m + g.tile_m0) * BM;
        n0_nxt = (tile_n + g.tile_n0) * BN;
        ao_nxt = (uint32_t)(m0_nxt * g.lda);
        wo_nxt = (uint32_t)(n0_nxt * g.ldw);
        so_nxt = (uint32_t)((s_is_a ? m0_nxt : n0_nxt) * 4);
    };
    constexpr int kWLoads = BN / 64;                // a wave's load instructions for the rows of W
    constexpr int kLoadsPerStage = 4 + kWLoads + NBS;
    // A wave's nine or ten (seven or eight) load instructions of a stage are spread out so that the texture path never sees all of
    // the workgroup's at once: the first kEarly right after the barrier that releases their buffer (last column
    // step of the stage two before), the others two per step during the first steps of the stage before.
    constexpr int kEarly = 3, kLateCols = (kLoadsPerStage - kEarly + 1) / 2;
    static_assert(kEarly <= 4, "the early loads are rows of A");
    static_assert(kLateCols <= NJ - 1, "the late loads are issued before the last column step of the stage before");
    // The stage in buffer F gives the stage after it (buffer G) its late loads, at L, and the stage after that
    // (buffer F again) its early loads, at E.

    const uint32_t lds_base = bi8_lds_address(lds);
    // load instruction idx of a stage: 0-3 = A rows, then kWLoads of W rows, then the scale rows; the K position advances after the last
    auto issue_one = [&](int buf, int idx) {
        if (idx < 4) {
            bi8_buffer_to_lds16_sum(a_rsrc, lds_base + L::kAReg + buf * L::kABuf + (wave + idx * NW) * 1024, a_off, idx < kEarly ? ao_E : ao_L, a_wave + idx * a_step);
        } else if (idx < 4 + kWLoads) {
            bi8_buffer_to_lds16_sum(w_rsrc, lds_base + L::kWReg + buf * L::kWBuf + (wave + (idx - 4) * NW) * 1024, w_off, wo_L, w_wave + (idx - 4) * w_step);
        } else if (idx < kLoadsPerStage) {
            s_raw[idx - 4 - kWLoads] = bi8_buffer_load_f32(s_brsrc, (int)s_off, (int)so_L);
            so_L += s_inc;
        }
    };

    // the fetching lanes' scales of the stage that goes to buffer `buf` (all loads have been waited for)
    auto publish_scales = [&](int buf) {
#pragma unroll
        for (int kb = 0; kb < NBS; ++kb) {
            const float b = bi8_u2f((bi8_f2u(s_raw[kb]) + 2u) & ~3u);     // 22 significant bits
            *(float *)(lds + p_dst0 + buf * p_buf0 + kb * p_row0) = s_is_a ? s_raw[kb] : b;
            *(float *)(lds + p_dst1 + buf * p_buf1 + kb * p_row1) = -BI8_MAGIC * b;          // exact
        }
    };

    // ---- operand fragments: lane -> row r16 of a 16-row subtile, 16-byte chunk 4*kb + q of the stage's eight;
    // stored at chunk position (4*kb + q) ^ ((row >> 1) & 7) and (row >> 1) & 7 = r16 >> 1 for every subtile,
    // so the address of kb = 1 is the address of kb = 0 with bit 6 flipped.
    int a_base[2], w_base[2];
    a_base[0] = L::kAReg + (wm * 64 + r16) * kStageK + ((q ^ (r16 >> 1)) << 4);
    w_base[0] = L::kWReg + (wn * WC + r16) * kStageK + ((q ^ (r16 >> 1)) << 4);
    a_base[1] = a_base[0] ^ 64;
    w_base[1] = w_base[0] ^ 64;
    // a subtile's outputs: lane -> column r16, rows 4q .. 4q+3
    int sa_base = L::kSAReg + (wm * 64 + 4 * q) * 4;
    int sw_base = L::kSWReg + wn * (WC * 8) + r16 * 16;
    // The region offsets (64 KiB and up) stay inside these six registers: every access below is one of them plus an
    // immediate under 64 KiB.  Left to itself the compiler folds each region offset into the immediates, finds them
    // too large for the instruction's 16-bit field, and keeps a separate address register per access (24 spilled).
    asm volatile("" : "+v"(a_base[0]), "+v"(a_base[1]), "+v"(w_base[0]), "+v"(w_base[1]), "+v"(sa_base), "+v"(sw_base), "+v"(p_dst0), "+v"(p_dst1));

    float acc[4][NJ][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;

    constexpr int kMagicBits = 0x4B400000;        // bit pattern of 1.5 * 2^23
    const bi8_v4i magic = {kMagicBits, kMagicBits, kMagicBits, kMagicBits};
    bi8_v4i A[4][2], Bf[2][2];                     // [row subtile][kb], [column parity][kb]
    bi8_v4f sx[4];                                 // row scales per row subtile
    bi8_v4f bc[2];                                 // per column pair (parity of the pair): b, -(1.5*2^23)*b of its two columns
    bc[0] = bc[1] = bi8_v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < 4; ++i) sx[i] = bi8_v4f{0.0f, 0.0f, 0.0f, 0.0f};

    auto read_a = [&](bi8_v4i *dst, int i, int buf) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) dst[kb] = *(const bi8_v4i *)(lds + a_base[kb] + buf * L::kABuf + i * 16 * kStageK);
    };
    auto read_b = [&](bi8_v4i *dst, int j, int buf) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) dst[kb] = *(const bi8_v4i *)(lds + w_base[kb] + buf * L::kWBuf + j * 16 * kStageK);
        if ((j & 1) == 0) bc[(j >> 1) & 1] = *(const bi8_v4f *)(lds + sw_base + buf * L::kCBuf + (j >> 1) * 256);
    };
    auto read_sx = [&](bi8_v4f &dst, int i, int buf) { dst = *(const bi8_v4f *)(lds + sa_base + buf * L::kSBuf + i * 16 * 4); };
    // two elements of a finished partial: fma(f, b, c) = fl(b * P) (the partial carries the 1.5*2^23 offset), then
    // the row scale and the accumulation
    auto fold2 = [&](const bi8_v4i &pt, int r0, const bi8_v4f &s, int col, float *dst) {
        const float b = bc[(col >> 1) & 1][2 * (col & 1)], cm = bc[(col >> 1) & 1][2 * (col & 1) + 1];
#pragma unroll
        for (int r = r0; r < r0 + 2; ++r) {
            const float u = __builtin_fmaf(bi8_u2f((uint32_t)pt[r]), b, cm);
            dst[r] = __builtin_fmaf(u, s[r], dst[r]);
        }
    };
    // the same for the four elements of a partial, the four products first, so that no instruction reads the result of
    // the one before it (measured: a dependent pair of FMAs whose sources share a register bank costs 12 % more than an
    // independent one; 8192^3 0.535 -> 0.530 ms, at block 64 0.692 -> 0.680)
    auto fold4 = [&](const bi8_v4i &pt, const bi8_v4f &s, int col, float *dst) {
        const float b = bc[(col >> 1) & 1][2 * (col & 1)], cm = bc[(col >> 1) & 1][2 * (col & 1) + 1];
        float u[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) u[r] = __builtin_fmaf(bi8_u2f((uint32_t)pt[r]), b, cm);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < 4; ++r) dst[r] = __builtin_fmaf(u[r], s[r], dst[r]);
        __builtin_amdgcn_sched_barrier(0);
    };
    auto wait_vm = [&](auto pending_c) {
        constexpr int kPending = decltype(pending_c)::value;
        __builtin_amdgcn_s_waitcnt(0x0F70 | (kPending & 15) | ((kPending >> 4) << 14));
    };

    // Column-burst schedule (BLK = 128): the eight MFMAs of column j back to back, then the whole fold of column
    // j - 1 (32 FMAs).  cB[parity][row subtile] are the partials; on entry A[0..3], Bf[0], swr[0] hold this stage's
    // operands of column 0 and cB[1] the previous stage's column 7, still to be folded with the OLD sx, swb[1], swc[1].
    bi8_v4i cB[2][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) cB[0][i] = cB[1][i] = magic;
    auto stage = [&](auto buf_c) {                  // BLK = 128
        constexpr int F = decltype(buf_c)::value, G = 1 - F;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            constexpr int kPrevCol[8] = {NJ - 1, 0, 1, 2, 3, 4, 5, 6};
            const int jb = j & 1;
            if (j < kLateCols) issue_one(G, kEarly + 2 * j);
            if (j < NJ - 1) {
                read_b(Bf[jb ^ 1], j + 1, F);
            } else {
                __builtin_amdgcn_s_waitcnt(0xC07F);
                wait_vm(std::integral_constant<int, 0>{});
                publish_scales(G);
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int idx = 0; idx < kEarly - 1; ++idx) issue_one(F, idx);
                read_b(Bf[0], 0, G);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 4; ++i) cB[jb][i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[i][0], Bf[jb][0], magic, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) cB[jb][i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[i][1], Bf[jb][1], cB[jb][i], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (j == NJ - 1) {                     // every MFMA of this stage is issued: the next stage's row subtiles
                issue_one(F, kEarly - 1);
#pragma unroll
                for (int i = 0; i < 4; ++i) read_a(A[i], i, G);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) fold4(cB[jb ^ 1][i], sx[i], kPrevCol[j], acc[i][kPrevCol[j]]);
            __builtin_amdgcn_sched_barrier(0);
            if (j == 0) {                          // this stage's row scales: first needed by the fold in column 1
#pragma unroll
                for (int i = 0; i < 4; ++i) read_sx(sx[i], i, F);
            }
            if (j < kLateCols) issue_one(G, kEarly + 2 * j + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- BLK = 64: a stage is two K-blocks, each ONE MFMA per subtile.  The stage runs as 16 column steps (K-block
    // kb = step / 8, column = step % 8): the four MFMAs of a step, then the whole fold of the step before (twice the
    // vector work per MFMA of the block-128 schedule).  W fragments (one 16-byte chunk column) and column scales are
    // read one step ahead, the row scales of K-block 1 after the fold of step 8.
    bi8_v4i Bh[2];                                 // [step parity]
    auto read_bh = [&](bi8_v4i &dst, int step, int buf) {
        const int kb = step / NJ, j = step % NJ;
        dst = *(const bi8_v4i *)(lds + w_base[kb] + buf * L::kWBuf + j * 16 * kStageK);
        if ((j & 1) == 0) bc[(j >> 1) & 1] = *(const bi8_v4f *)(lds + sw_base + buf * L::kCBuf + kb * L::kCRow + (j >> 1) * 256);
    };
    auto read_sx64 = [&](bi8_v4f &dst, int i, int kb, int buf) {
        dst = *(const bi8_v4f *)(lds + sa_base + buf * L::kSBuf + kb * L::kSRow + i * 16 * 4);
    };
    auto stage64 = [&](auto buf_c) {               // same burst schedule: four MFMAs, then the fold of the step before
        constexpr int F = decltype(buf_c)::value, G = 1 - F;
#pragma unroll
        for (int h = 0; h < 2 * NJ; ++h) {
            const int kb = h / NJ, hb = h & 1, jprev = (h + 2 * NJ - 1) % NJ;
            if (h < kLateCols) issue_one(G, kEarly + 2 * h);
            if (h < 2 * NJ - 1) {
                read_bh(Bh[hb ^ 1], h + 1, F);
            } else {
                __builtin_amdgcn_s_waitcnt(0xC07F);                // lgkmcnt(0) only
                wait_vm(std::integral_constant<int, 0>{});
                publish_scales(G);
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int idx = 0; idx < kEarly - 1; ++idx) issue_one(F, idx);
                read_bh(Bh[0], 0, G);                              // the next stage's first step
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 4; ++i) cB[hb][i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[i][kb], Bh[hb], magic, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (h == 2 * NJ - 1) {                                 // every MFMA of this stage is issued
                issue_one(F, kEarly - 1);
#pragma unroll
                for (int i = 0; i < 4; ++i) read_a(A[i], i, G);
                __builtin_amdgcn_sched_barrier(0);
            }
            // the step before: at h = 0 the previous stage's last step, at h = NJ the last step of K-block 0, both with
            // the row scales still in sx
#pragma unroll
            for (int i = 0; i < 4; ++i) fold4(cB[hb ^ 1][i], sx[i], jprev, acc[i][jprev]);
            __builtin_amdgcn_sched_barrier(0);
            if (h == 0 || h == NJ) {                               // this K-block's row scales: first needed one step on
#pragma unroll
                for (int i = 0; i < 4; ++i) read_sx64(sx[i], i, kb, F);
            }
            if (h < kLateCols) issue_one(G, kEarly + 2 * h + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // 16-bit outputs: the bias of the tile's columns waits in LDS for the tile's end, one dword per column (a
    // 16-bit element zero-extended), fetched by waves 4-7 (4-5 for 128 columns), 64 columns each.  The waits and barriers of the stages
    // that follow complete and publish it; columns past N read as zeros.
    const bi8_rsrc bias_rsrc = bi8_make_rsrc(g.bias, g.bias ? g.N * (g.bias_dtype == BI8_F32 ? 4 : 2) : 0);
    auto fetch_bias = [&]() {
        if (wave >= 4 && wave < 4 + BN / 64) {
            const uint32_t dst = lds_base + L::kBiasReg + (wave - 4) * 256, col = (uint32_t)(n0 + (wave - 4) * 64);
            if (g.bias_dtype == BI8_F32) bi8_buffer_to_lds4(bias_rsrc, dst, (uint32_t)(lane * 4), col * 4);
            else bi8_buffer_to_lds2(bias_rsrc, dst, (uint32_t)(lane * 2), col * 2);
        }
    };
    if (CDT != BI8_F32 && g.bias != nullptr) fetch_bias();

    // prologue: the first stage's loads and the early part of the second's; wait for the first stage
#pragma unroll
    for (int idx = 0; idx < kLoadsPerStage; ++idx) issue_one(0, idx);
    ao_E += kStageK;
#pragma unroll
    for (int idx = 0; idx < kEarly; ++idx) issue_one(1, idx);
    ao_L = ao_E;
    wo_L += kStageK;
    wait_vm(std::integral_constant<int, kEarly>{});
    publish_scales(0);
    __syncthreads();
    read_a(A[0], 0, 0);
    read_a(A[1], 1, 0);
    read_a(A[2], 2, 0);
    read_a(A[3], 3, 0);
    if constexpr (BLK == 128) read_b(Bf[0], 0, 0);
    else read_bh(Bh[0], 0, 0);
    // The trip count is rounded up to even and loads run two stages ahead: stages past the end of K read their
    // scales through the buffers' range check as zeros, so they add exactly 0 to the accumulators.
    const float div = (float)(1.0 / (127.0 * 127.0));
    const bool has_bias = g.bias != nullptr;
    for (;;) {
        aim_next(pid + (int)gridDim.x);
        for (int pi = 0; pi < npairs; ++pi) {
            // Stages 2pi (buffer 0) and 2pi + 1 (buffer 1).  In the tile's last pair E is in the next tile from the
            // start, and L follows it there after the first of the two stages.
            const bool last = pi == npairs - 1;
            ao_E = last ? ao_nxt : ao_L + kStageK;
            if constexpr (BLK == 128) stage(std::integral_constant<int, 0>{});
            else stage64(std::integral_constant<int, 0>{});
            ao_L = ao_E;
            wo_L = last ? wo_nxt : wo_L + kStageK;
            so_L = last ? so_nxt : so_L;
            ao_E += kStageK;
            if constexpr (BLK == 128) stage(std::integral_constant<int, 1>{});
            else stage64(std::integral_constant<int, 1>{});
            ao_L = ao_E;
            wo_L += kStageK;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {              // the last column of the last (possibly padding) stage
            fold2(cB[1][i], 0, sx[i], NJ - 1, acc[i][NJ - 1]);
            fold2(cB[1][i], 2, sx[i], NJ - 1, acc[i][NJ - 1]);
        }

        if constexpr (CDT != BI8_F32) {
            // 16-bit outputs leave through the wave's LDS strip, 16 rows x 64 columns at a time: in the accumulator
            // layout a store instruction would write 32-byte runs of four rows; from the row-major strip it writes
            // 128-byte runs.  The strip is the wave's own, so no barrier: LDS serves a wave's instructions in order.
            // Nothing here waits for memory (the bias comes from LDS, addresses are rebuilt from the lane number
            // rather than kept in registers across the K loop): the next tile's loads and this tile's stores stay in flight.
            int lane_e = lane;
            asm volatile("" : "+v"(lane_e));
            const int er16 = lane_e & 15, eq = lane_e >> 4;
            uint8_t *strip = lds + L::kStrips + wave * L::kStripBytes;
            uint8_t *strip_w = strip + 4 * eq * L::kStripPitch + er16 * 2;
            const uint8_t *strip_r = strip + (lane_e >> 3) * L::kStripPitch + (lane_e & 7) * 16;
            const int row_e = lane_e >> 3, col_e = (lane_e & 7) * 8;        // of the strip, as read back
            const int m_left = (int)(g.M - m0) - wm * 64 - row_e;             // rows 16i + 8p below this are inside C
            const int n_e = n0 + wn * WC + col_e;
            uint8_t *c_tile = (uint8_t *)g.C + ((int64_t)(m0 + wm * 64) * g.ldc + n0 + wn * WC) * 2;
            const uint32_t c_lane = (uint32_t)((row_e * g.ldc + col_e) * 2);
            const uint8_t *bias_lds = lds + L::kBiasReg + (wn * WC + er16) * 4;
            auto leave = [&](auto with_bias_c, auto streaming_c) {
                constexpr bool kBias = decltype(with_bias_c)::value, kStreaming = decltype(streaming_c)::value;
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int jh = 0; jh < NJ / 4; ++jh) {
#pragma unroll
                        for (int jj = 0; jj < 4; ++jj) {
                            float bias = 0.0f;
                            if constexpr (kBias) {
                                const int j = 4 * jh + jj;
                                const uint32_t raw = *(const uint32_t *)(bias_lds + j * 64);
                                bias = g.bias_dtype == BI8_F32 ? bi8_u2f(raw) : g.bias_dtype == BI8_BF16 ? bi8_from_bf16_bits(raw) : bi8_from_f16_bits(raw);
                                bias = bi8_round_to<CDT>(bias);
                            }
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                float v = bi8_round_to<CDT>(acc[i][4 * jh + jj][r] * div);    // acc.to(C.dtype), then + bias in C's dtype
                                if constexpr (kBias) v = v + bias;
                                const uint32_t bits = (CDT == BI8_BF16) ? bi8_bf16_bits(v) : bi8_f16_bits(v);
                                *(uint16_t *)(strip_w + r * L::kStripPitch + jj * 32) = (uint16_t)bits;
                            }
                        }
                        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                        __builtin_amdgcn_wave_barrier();
                        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                        // lane -> row 8p + lane/8 of the strip, 8 outputs (16 bytes) at column 8 * (lane % 8)
#pragma unroll
                        for (int p = 0; p < 2; ++p) {
                            const bi8_v4u v = *(const bi8_v4u *)(strip_r + 8 * p * L::kStripPitch);
                            if (16 * i + 8 * p < m_left) {
                                uint8_t *dst = c_tile + ((int64_t)(16 * i + 8 * p) * g.ldc + jh * 64) * 2 + c_lane;
                                if (n_e + jh * 64 + 8 <= g.N) {
                                    // (rows of odd length start on 2-byte boundaries)
                                    if constexpr (kStreaming) __builtin_nontemporal_store(v, (bi8_v4u_unaligned *)dst);
                                    else *(bi8_v4u_unaligned *)dst = v;
                                } else {
#pragma nounroll
                                    for (int e = 0; e < 8 && n_e + jh * 64 + e < g.N; ++e) ((uint16_t *)dst)[e] = (uint16_t)(v[e >> 1] >> (16 * (e & 1)));
                                }
                            }
                        }
                        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                        __builtin_amdgcn_wave_barrier();
                    }
            };
            // The workgroup's last tile leaves with non-temporal stores: nothing is left to run while the L2 writes its
            // lines back at the kernel's end (2048 x 4096 x 4096, one tile per workgroup: 44.3 -> 43.2 us; the tiles before
            // the last, whose stores run under the next tile's K loop, measured 0.5 % slower with them).
            const bool last_tile = pid + (int)gridDim.x >= ntiles;
            if (has_bias) {
                if (last_tile) leave(std::true_type{}, std::true_type{});
                else leave(std::true_type{}, std::false_type{});
            } else {
                if (last_tile) leave(std::false_type{}, std::true_type{});
                else leave(std::false_type{}, std::false_type{});
            }
        } else if constexpr (SPLIT) {
            // the piece's sums, scaled, to its slab [256][BN]: the whole tile (rows and columns past the matrix hold zeros)
            float *out = g.ws + (int64_t)slab * (BM * BN) + (wm * 64 + 4 * q) * BN + wn * WC + r16;
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
#pragma unroll
                    for (int r = 0; r < 4; ++r) out[(i * 16 + r) * BN + j * 16] = acc[i][j][r] * div;
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int64_t n = (int64_t)n0 + wn * WC + j * 16 + r16;
                const bool n_ok = n < g.N;
                const float bias = (has_bias && n_ok) ? load_bias(g, n) : 0.0f;
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int64_t m = (int64_t)m0 + wm * 64 + i * 16 + 4 * q + r;
                        if (n_ok && m < g.M) store_c<CDT>(g.C, m * g.ldc + n, acc[i][j][r] * div, has_bias, bias);
                    }
            }
        }

        pid += (int)gridDim.x;
        if (SPLIT || pid >= ntiles) break;
        // The next tile: its first stage is published, its operands of column 0 are in A and Bf[0].  The first step
        // folds "the column before" from an empty partial with zero scales, as at the start of the kernel.
        m0 = m0_nxt;
        n0 = n0_nxt;
        if (CDT != BI8_F32 && has_bias) {
            __syncthreads();                       // every wave has read the tile's bias
            fetch_bias();
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            cB[1][i] = magic;
            sx[i] = bi8_v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;
        }
        bc[1] = bi8_v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }
    wait_vm(std::integral_constant<int, 0>{});     // nothing may still be writing LDS when the wave ends
}

// ---- 256x256 tile on v_mfma_i32_32x32x32_i8 ---------------------------------------------------------------------------
// Same workgroup tile, loader, stage buffers and single barrier per stage as gemm_wide; what differs is the shape of
// the matrix instruction and with it the wave tile.  A 32x32x32 MFMA does twice the work of a 16x16x64 one for the
// same hold on the issue port, so half as many of them are issued per K-block; the price is its accumulator layout
// (16 rows per lane instead of 4), which makes a wave's row scales cost 16 registers per 32 rows.  The eight waves
// therefore stack along M: one wave owns 32 rows x 256 columns = 8 subtiles of 32x32.  Per stage it keeps its 32 rows
// of A (16 registers) and the K-block's row scales (16) in registers and streams the eight column subtiles of W
// through ONE register buffer: the 16-byte chunk of W that MFMA k-step ks has just consumed is refilled with the same
// chunk of the next subtile, which is needed four MFMAs later.  An item = one (K-block, column subtile): BLK/32
// chained MFMAs, each followed by a slice of the fold of the item before (the chain is dependent, so the fold's
// vector instructions fill the wait for the previous MFMA's result).
// Used for block 32, where a K-block is exactly one such MFMA (8192^3: 1.23 ms against 1.47 ms on 128x128 tiles).
// For blocks 128 and 64 it measured SLOWER than gemm_wide (0.65 against 0.53 ms, 0.81 against 0.71 ms at 8192^3): its
// three 16-register tuples (two partials and the 1.5*2^23 start value, which the compiler then rebuilds with eight
// moves per item rather than keep) and the 32x256 wave tile's extra LDS reads (48 against 36 per wave and stage) cost
// more than the halved MFMA count gives back; a 64x128 wave tile with this instruction does not fit 256 registers.
template <int NBS> struct Wide32Lds {
    using W = WideLds<NBS>;
    static constexpr int kOutPitch = 512 + 16;                                // a wave's 32 x 256 tile of 16-bit outputs
    static constexpr int kOut = 8 * 32 * kOutPitch;                          // 132 KiB
    static constexpr int kBytes = kOut > W::kStages ? kOut : W::kStages;
};

template <int BLK, int CDT>
__global__ __launch_bounds__(512) void gemm_wide32(const GemmArgs g) {
    static_assert(BLK == 128 || BLK == 64 || BLK == 32, "a K-block is 1, 2 or 4 MFMAs of 32 bytes of K");
    constexpr int NBS = kStageK / BLK;             // K-blocks per stage
    constexpr int KSB = BLK / 32;                  // MFMAs per K-block and subtile
    constexpr int NJ = 8;                          // column subtiles of a wave
    constexpr int NI = NBS * NJ;                   // items per stage
    using L = WideLds<NBS>;
    constexpr int BM = 256, BN = 256, NW = 8;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, h = lane >> 5;

    int tile_m, tile_n;
    tile_of_workgroup(blockIdx.x, g.tiles_m, g.tiles_n, tile_m, tile_n);
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    const int nstages = (int)(g.K / kStageK);

    // ---- loader: exactly gemm_wide's (wave instruction i covers tile rows 8i .. 8i+7, chunk swizzle (row >> 1) & 7)
    const int ld_row = lane >> 3;
    const int ld_chunk = (lane & 7) ^ ((4 * (wave & 1) + (lane >> 4)) & 7);
    const int64_t a_rows = (g.M - m0 < BM) ? (g.M - m0) : BM, w_rows = (g.N - n0 < BN) ? (g.N - n0) : BN;
    const bi8_rsrc a_rsrc = bi8_make_rsrc(g.A + m0 * g.lda, (a_rows - 1) * g.lda + g.K);
    const bi8_rsrc w_rsrc = bi8_make_rsrc(g.W + n0 * g.ldw, (w_rows - 1) * g.ldw + g.K);
    const uint32_t a_off = (uint32_t)(ld_row * g.lda + ld_chunk * 16), w_off = (uint32_t)(ld_row * g.ldw + ld_chunk * 16);
    const uint32_t a_wave = (uint32_t)(wave * 8 * g.lda), w_wave = (uint32_t)(wave * 8 * g.ldw);
    const uint32_t a_step = (uint32_t)(NW * 8 * g.lda), w_step = (uint32_t)(NW * 8 * g.ldw);
    const int64_t nblk = g.K / BLK;
    const bool s_is_a = wave < 4;
    const int s_part = wave & 3;
    const bi8_brsrc sa_brsrc = bi8_make_brsrc(g.sA + m0, ((nblk - 1) * g.M + (g.M - m0)) * 4);
    const bi8_brsrc sw_brsrc = bi8_make_brsrc(g.sW + n0, ((nblk - 1) * g.N + (g.N - n0)) * 4);
    const bi8_brsrc s_brsrc = s_is_a ? sa_brsrc : sw_brsrc;
    const uint32_t s_off = (uint32_t)((s_part * 64 + lane) * 4);
    const uint32_t s_inc = (uint32_t)((s_is_a ? g.M : g.N) * 4);
    float s_raw[NBS];
#pragma unroll
    for (int kb = 0; kb < NBS; ++kb) s_raw[kb] = 0.0f;
    // Column scales are stored prepared, as the pair (b, -1.5*2^23*b) with b rounded to 22 significant bits, in the
    // order [column within its subtile][subtile][b, c]: a lane reads the pairs of two subtiles with one 16-byte read.
    // The fetching lane holds tile column s_part * 64 + lane = subtile 2 * s_part + lane / 32, column lane % 32.
    const int c_dst = L::kSWReg + ((lane & 31) * NJ + 2 * s_part + (lane >> 5)) * 8;
    // (a row-scale lane's second store repeats its first: both kinds of lane run the same instructions)
    int p_dst0 = s_is_a ? L::kSAReg + (s_part * 64 + lane) * 4 : c_dst;
    const int p_second = s_is_a ? 0 : 4;           // wave-uniform
    const int p_buf0 = s_is_a ? L::kSBuf : L::kCBuf, p_row0 = s_is_a ? L::kSRow : L::kCRow;
    uint32_t s_pos = 0, k_pos = 0;
    constexpr int kLoadsPerStage = 4 + 4 + NBS;
    constexpr int kEarly = 3, kLateItems = (kLoadsPerStage - kEarly + 1) / 2;
    static_assert(kLateItems <= NI - 1, "the late loads are issued before the last item of the stage before");

    const uint32_t lds_base = bi8_lds_address(lds);
    auto issue_one = [&](int buf, int idx) {
        if (idx < 4) {
            bi8_buffer_to_lds16_sum(a_rsrc, lds_base + L::kAReg + buf * L::kABuf + (wave + idx * NW) * 1024, a_off, k_pos, a_wave + idx * a_step);
        } else if (idx < 8) {
            bi8_buffer_to_lds16_sum(w_rsrc, lds_base + L::kWReg + buf * L::kWBuf + (wave + (idx - 4) * NW) * 1024, w_off, k_pos, w_wave + (idx - 4) * w_step);
        } else if (idx < kLoadsPerStage) {
            s_raw[idx - 8] = bi8_buffer_load_f32(s_brsrc, (int)s_off, (int)s_pos);
            s_pos += s_inc;
            if (idx == kLoadsPerStage - 1) k_pos += kStageK;
        }
    };
    auto publish_scales = [&](int buf) {           // buf is wave-uniform
        const int dst = p_dst0 + buf * p_buf0;
#pragma unroll
        for (int kb = 0; kb < NBS; ++kb) {
            const float b = bi8_u2f((bi8_f2u(s_raw[kb]) + 2u) & ~3u);     // 22 significant bits
            *(float *)(lds + dst + kb * p_row0) = s_is_a ? s_raw[kb] : b;
            *(float *)(lds + (dst + p_second) + kb * p_row0) = s_is_a ? s_raw[kb] : -BI8_MAGIC * b;   // exact
        }
    };

    // ---- operand fragments of a 32x32x32 MFMA: lane -> row l32 of the subtile, 16-byte chunk 2*ks + h of the stage's
    // eight, stored at chunk position (2*ks + h) ^ ((row >> 1) & 7): address(ks) = address(0) ^ (ks << 5)
    const int frag_sw = ((h ^ ((l32 >> 1) & 7)) << 4);
    // (W: one address register per ks, read 32 times a stage; A is read four times a stage and derives its addresses)
    int a_addr0 = L::kAReg + (wave * 32 + l32) * kStageK + frag_sw, w_addr[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) w_addr[ks] = (L::kWReg + l32 * kStageK + frag_sw) ^ (ks << 5);
    // outputs of a subtile: lane -> column l32, rows 8 * (r >> 2) + 4 * h + (r & 3) for accumulator register r
    int sa_base = L::kSAReg + (wave * 32 + 4 * h) * 4;
    int sw_base = L::kSWReg + l32 * NJ * 8;
    asm volatile("" : "+v"(a_addr0), "+v"(w_addr[0]), "+v"(w_addr[1]), "+v"(w_addr[2]), "+v"(w_addr[3]), "+v"(sa_base), "+v"(sw_base), "+v"(p_dst0));

    float acc[NJ][16];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;

    constexpr int kMagicBits = 0x4B400000;        // bit pattern of 1.5 * 2^23
    const bi8_v16i magic = {kMagicBits, kMagicBits, kMagicBits, kMagicBits, kMagicBits, kMagicBits, kMagicBits, kMagicBits,
                            kMagicBits, kMagicBits, kMagicBits, kMagicBits, kMagicBits, kMagicBits, kMagicBits, kMagicBits};
    bi8_v4i A[4], Wf[4];                           // this stage's A chunks; the current subtile's W chunks
    bi8_v4f sx[4];                                 // row scales of the K-block being folded: rows 8*g + 4*h + 0..3
    bi8_v2f bc[2];                                 // (b, c) of a subtile, by parity of the item
    bi8_v16i P[2];
    P[0] = P[1] = magic;
    bc[0] = bc[1] = bi8_v2f{0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < 4; ++i) sx[i] = bi8_v4f{0.0f, 0.0f, 0.0f, 0.0f};

    auto read_a = [&](int ks) {
        int addr = a_addr0;
        if (ks) asm volatile("v_xor_b32 %0, %1, %2" : "=v"(addr) : "v"(a_addr0), "v"(ks << 5));    // not hoisted out of the loop
        A[ks] = *(const bi8_v4i *)(lds + addr);
    };
    auto read_w = [&](int ks, int j) { Wf[ks] = *(const bi8_v4i *)(lds + w_addr[ks] + j * 32 * kStageK); };
    auto read_bc = [&](int kb, int j) { bc[j & 1] = *(const bi8_v2f *)(lds + sw_base + kb * L::kCRow + j * 8); };
    auto read_sx = [&](int kb) {
#pragma unroll
        for (int i = 0; i < 4; ++i) sx[i] = *(const bi8_v4f *)(lds + sa_base + kb * L::kSRow + i * 8 * 4);
    };
    // The read addresses above point into the stage buffer that the reads of the moment are for; they move to the other
    // buffer right behind the barrier of a stage, after which every read is for the next stage.
    auto switch_buffers = [&](int to) {            // to: wave-uniform, 0 or 1
        const int d = to ? 1 : -1;
        a_addr0 += d * L::kABuf;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) w_addr[ks] += d * L::kWBuf;
        sa_base += d * L::kSBuf;
        sw_base += d * L::kCBuf;
    };
    // elements [16 * q / KSB, 16 * (q + 1) / KSB) of a finished partial: fma(f, b, c) = fl(b * P) (the partial carries
    // the 1.5*2^23 offset), then the row scale and the accumulation
    auto fold_slice = [&](const bi8_v16i &pt, int j, int q) {
        const float b = bc[j & 1][0], cm = bc[j & 1][1];
        // in groups of four: the four products first, so that no instruction reads the result of the one before it
        // (block 32 at 8192^3: 1.241 -> 1.220 ms)
#pragma unroll
        for (int r0 = q * (16 / KSB); r0 < (q + 1) * (16 / KSB); r0 += 4) {
            float u[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) u[r] = __builtin_fmaf(bi8_u2f((uint32_t)pt[r0 + r]), b, cm);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[j][r0 + r] = __builtin_fmaf(u[r], sx[(r0 + r) >> 2][r], acc[j][r0 + r]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto wait_vm = [&](auto pending_c) {
        constexpr int kPending = decltype(pending_c)::value;
        __builtin_amdgcn_s_waitcnt(0x0F70 | (kPending & 15) | ((kPending >> 4) << 14));
    };

    // One stage, in stage buffer `cur` (wave-uniform; the loop below is not unrolled over the two buffers, so that the
    // registers keep their roles from one stage to the next).  Item t = (K-block t / 8, subtile t % 8).  On entry A[]
    // and Wf[] hold this stage's operands of item 0, and P[1], sx[], bc[1] the last item of the stage before, still to
    // be folded.
    auto stage = [&](int cur) {
        const int nxt = 1 - cur;
#pragma unroll
        for (int t = 0; t < NI; ++t) {
            const int kb = t / NJ, j = t % NJ;
            const int tp = (t + NI - 1) % NI, jp = tp % NJ;             // the item before
            if (t < kLateItems) issue_one(nxt, kEarly + 2 * t);
            // this item's pair: first used by the fold one item on (the other register serves the fold below)
            read_bc(kb, j);
            if (t == NI - 1) {
                // every operand of this stage is in registers or on its way: publish the next stage, release this one
                __builtin_amdgcn_s_waitcnt(0xC07F);                    // lgkmcnt(0) only
                wait_vm(std::integral_constant<int, 0>{});
                publish_scales(nxt);
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
                switch_buffers(nxt);
#pragma unroll
                for (int idx = 0; idx < kEarly - 1; ++idx) issue_one(cur, idx);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q = 0; q < KSB; ++q) {
                const int ks = kb * KSB + q;
                P[t & 1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(A[ks], Wf[ks], q == 0 ? magic : P[t & 1], 0, 0, 0);
                // the chunk just consumed is refilled: W with the next item's, A (after its last use) with the next stage's
                if (t == NI - 1) {
                    read_w(q, 0);
                    // no A chunk is needed any more once this stage's last MFMA on it is issued: the next stage's
#pragma unroll
                    for (int kk = q; kk < 4; kk += KSB) read_a(kk);
                } else {
                    const int tn = t + 1;
                    read_w((tn / NJ) * KSB + q, tn % NJ);
                }
                __builtin_amdgcn_sched_barrier(0);
                fold_slice(P[tp & 1], jp, q);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (t == NI - 1) issue_one(cur, kEarly - 1);
            // the fold above was the last of its K-block when the item before was a subtile 7: its row scales make way
            // for those of the block whose first item has just been issued
            if (j == 0) read_sx(kb);
            if (t < kLateItems) issue_one(nxt, kEarly + 2 * t + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // prologue: the first stage's loads and the early part of the second's; wait for the first stage
#pragma unroll
    for (int idx = 0; idx < kLoadsPerStage; ++idx) issue_one(0, idx);
#pragma unroll
    for (int idx = 0; idx < kEarly; ++idx) issue_one(1, idx);
    wait_vm(std::integral_constant<int, kEarly>{});
    publish_scales(0);
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        read_a(ks);
        if (ks < KSB) read_w(ks, 0);
    }
    // The trip count is rounded up to even and loads run two stages ahead: stages past the end of K read their
    // scales through the buffers' range check as zeros, so they add exactly 0 to the accumulators.
    {
        const int trips = (nstages + 1) & ~1;
        int cur = 0;
#pragma nounroll
        for (int s = 0; s < trips; ++s) {
            stage(cur);
            cur = 1 - cur;
        }
    }
    wait_vm(std::integral_constant<int, 0>{});     // nothing may still be writing LDS when the wave ends
#pragma unroll
    for (int q = 0; q < KSB; ++q) fold_slice(P[(NI - 1) & 1], NJ - 1, q);   // the last item of the last (possibly padding) stage

    const float div = (float)(1.0 / (127.0 * 127.0));
    const bool has_bias = g.bias != nullptr;
    if constexpr (CDT != BI8_F32) {
        // 16-bit outputs leave through LDS: a row-major copy of the wave's 32 x 256 tile, stored as 512-byte row runs
        __syncthreads();                           // every wave is done with the stage buffers
        uint8_t *tile = lds + wave * (32 * Wide32Lds<NBS>::kOutPitch);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int64_t n = n0 + j * 32 + l32;
            const float bias = (has_bias && n < g.N) ? bi8_round_to<CDT>(load_bias(g, n)) : 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float v = bi8_round_to<CDT>(acc[j][r] * div);          // acc.to(C.dtype), then + bias in C's dtype
                if (has_bias) v = v + bias;
                const uint32_t bits = (CDT == BI8_BF16) ? bi8_bf16_bits(v) : bi8_f16_bits(v);
                *(uint16_t *)(tile + (8 * (r >> 2) + 4 * h + (r & 3)) * Wide32Lds<NBS>::kOutPitch + (j * 32 + l32) * 2) = (uint16_t)bits;
            }
        }
        // lane -> row 2p + lane / 32 of the tile, 8 outputs (16 bytes) at column 8 * (lane % 32)
        const int64_t n = n0 + l32 * 8;
#pragma unroll
        for (int p = 0; p < 16; ++p) {
            const int row = 2 * p + h;
            const int64_t m = m0 + wave * 32 + row;
            const bi8_v4u v = *(const bi8_v4u *)(tile + row * Wide32Lds<NBS>::kOutPitch + l32 * 16);
            if (m < g.M) {
                uint16_t *dst = (uint16_t *)g.C + m * g.ldc + n;
                if (n + 8 <= g.N) {
                    *(bi8_v4u_unaligned *)dst = v;
                } else {
                    for (int e = 0; e < 8 && n + e < g.N; ++e) dst[e] = (uint16_t)(v[e >> 1] >> (16 * (e & 1)));
                }
            }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int64_t n = n0 + j * 32 + l32;
        const bool n_ok = n < g.N;
        const float bias = (has_bias && n_ok) ? load_bias(g, n) : 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int64_t m = m0 + wave * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
            if (n_ok && m < g.M) store_c<CDT>(g.C, m * g.ldc + n, acc[j][r] * div, has_bias, bias);
        }
    }
}

// Skinny GEMM (M <= 32), HBM-bound on W: the whole problem is one pass over the N*K bytes of weight codes.
// One workgroup = 32 output columns, 8 waves that split K in interleaved 128-byte stages; every wave gathers its
// MFMA operands straight from global memory in operand layout (16 bytes per lane; the four k-steps of a stage
// touch each 128-byte line of a weight row once), folds each K-block into 16 fp32 accumulators per lane, and the
// eight partial accumulators are summed through LDS in wave order (deterministic).  Rows m >= M are zero operands.
template <int BLK, int CDT>
__global__ __launch_bounds__(512) void gemm_skinny(const GemmArgs g) {
    constexpr int NW = 8;
    constexpr int NBS = kStageK / BLK, KSB = BLK / 32;
    __shared__ float red[NW][16][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int l32 = lane & 31, h = lane >> 5;
    const int64_t n0 = (int64_t)blockIdx.x * 32;
    const int64_t m0 = (int64_t)blockIdx.y * 32;      // row group of this workgroup
    const int64_t n = n0 + l32;
    const int64_t nc = n < g.N ? n : g.N - 1;                      // clamped: never stored
    const int64_t mc = m0 + l32 < g.M ? m0 + l32 : g.M - 1;
    const bool m_ok = m0 + l32 < g.M;
    const int8_t *wrow = g.W + nc * g.ldw + h * 16;
    const int8_t *arow = g.A + mc * g.lda + h * 16;
    const int nstages = (int)(g.K / kStageK);
    float acc[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

    auto load_stage = [&](int s, bi8_v4i *wf, bi8_v4i *af) {
        const int64_t k0 = (int64_t)s * kStageK;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            wf[ks] = __builtin_nontemporal_load((const bi8_v4i *)(wrow + k0 + ks * 32));
            af[ks] = m_ok ? *(const bi8_v4i *)(arow + k0 + ks * 32) : bi8_v4i{0, 0, 0, 0};
        }
    };
    bi8_v4i wf[2][4], af[2][4];
    int s = wave;
    if (s < nstages) load_stage(s, wf[0], af[0]);
    int cur = 0;
    for (; s < nstages; s += NW, cur ^= 1) {
        if (s + NW < nstages) load_stage(s + NW, wf[cur ^ 1], af[cur ^ 1]);      // next stage of this wave in flight
#pragma unroll
        for (int blk = 0; blk < NBS; ++blk) {
            const int64_t jb = (int64_t)s * NBS + blk;
            const float sw = g.sW[jb * g.N + nc];
            bi8_v16i p = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int ks = 0; ks < KSB; ++ks)
                p = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[cur][blk * KSB + ks], wf[cur][blk * KSB + ks], p, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int64_t row = m0 + 8 * i + 4 * h + j;
                    const float sx = (row < g.M) ? g.sA[jb * g.M + row] : 0.0f;
                    acc[4 * i + j] = __builtin_fmaf((float)p[4 * i + j] * sx, sw, acc[4 * i + j]);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) red[wave][r][lane] = acc[r];
    __syncthreads();
    if (wave == 0) {
        const float div = (float)(1.0 / (127.0 * 127.0));
        const bool has_bias = g.bias != nullptr;
        const float bias = (has_bias && n < g.N) ? load_bias(g, n) : 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float v = red[0][r][lane];
#pragma unroll
            for (int w = 1; w < NW; ++w) v += red[w][r][lane];
            const int64_t m = m0 + 8 * (r >> 2) + 4 * h + (r & 3);
            if (m < g.M && n < g.N) store_c<CDT>(g.C, m * g.ldc + n, v * div, has_bias, bias);
        }
    }
}

// ---- up to 32 rows, weight rows read as whole cache lines through LDS ----------------------------------------------------
// Few-row GEMM (M <= 32 as one or two groups of 16 rows, blocks 64 and 128): decode.  HBM-bound on W: one pass over the weight codes.  A load in MFMA
// operand layout would fetch 64 bytes of 16 rows (half a cache line per row and instruction); here a wave's load
// instruction fetches whole 128-byte lines (8 rows x 128 bytes, straight into LDS), and the operands are read back from
// LDS in operand layout.  One workgroup = 16 output columns; its NW waves split K in interleaved 128-byte chunks and
// never wait for one another: every wave owns a ring of kLdsGemvSlotsW stages of W (16 rows x 128 bytes each) with the
// scales of their K-blocks, and a ring of two stages of A (all 16 rows, zeros past M).  The partial accumulators of
// the waves are summed through LDS in wave order (deterministic).  Stages past the end of K load zeros (codes and
// scales).  Measured at M = 16, block 128, against the same kernel with operands gathered from global memory in operand
// layout through an 8-stage register ring: 4096 -> 11008 16.0 -> 12.8 us, 11008 -> 4096 17.1 -> 14.4 us.
constexpr int kLdsGemvSlotsW = 4, kLdsGemvSlotsA = 2;
constexpr int kLdsGemvSlot = 16 * 128;             // bytes of one stage of W, or of 16 rows of A
// MT = groups of 16 rows of A (1, 2 or 4: M <= 16, 32, 64).  One stage's scales: [K-block][16] column scales (128 bytes),
// then [K-block][16 * MT] row scales.
template <int MT> struct GemvLds {
    static constexpr int kAStage = MT * kLdsGemvSlot;
    static constexpr int kScales = 128 + 128 * MT;
    static constexpr int kAReg = kLdsGemvSlotsW * kLdsGemvSlot;
    static constexpr int kScReg = kAReg + kLdsGemvSlotsA * kAStage;
    static constexpr int kWaveBytes = kScReg + kLdsGemvSlotsW * kScales;
};
template <int BLK, int CDT, int NW, int MT>
__global__ __launch_bounds__(NW * 64) void gemv_staged(const GemmArgs g) {
    using L = GemvLds<MT>;
    constexpr int KW = 128;                        // bytes of K per wave and stage
    constexpr int NSW = kLdsGemvSlotsW, NSA = kLdsGemvSlotsA;
    constexpr int BPS = KW / BLK;                  // K-blocks per stage of a wave
    constexpr int kSlot = kLdsGemvSlot;
    static_assert(BLK == 64 || BLK == 128, "one or two 64-byte MFMAs per K-block");
    static_assert(NSW == 4 && NSA == 2, "the K loop is unrolled over the period of both rings");
    static_assert(MT == 1 || MT == 2 || MT == 4, "16 to 64 rows of A");
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r16 = lane & 15, q = lane >> 4;
    const int64_t n0 = (int64_t)blockIdx.x * 16;
    const int64_t n = n0 + r16;
    const int nchunks = (int)(g.K / KW);
    const int nst = (((nchunks + NW - 1) / NW) + 3) & ~3;           // stages of every wave; those past the end of K load zeros
    const int nblk = (int)(g.K / BLK);
    constexpr int wave_bytes = L::kWaveBytes;
    uint8_t *mine = lds + wave * wave_bytes;
    const uint32_t mine_addr = bi8_lds_address(lds) + (uint32_t)(wave * wave_bytes);
    constexpr int kAReg = L::kAReg, kScReg = L::kScReg;

    const int64_t wrows = g.N - n0 < 16 ? g.N - n0 : 16;
    const bi8_rsrc rw = bi8_make_rsrc(g.W + n0 * g.ldw, (wrows - 1) * g.ldw + g.K);
    const bi8_rsrc ra = bi8_make_rsrc(g.A, (g.M - 1) * g.lda + g.K);
    const bi8_rsrc rsw = bi8_make_rsrc(g.sW, (int64_t)nblk * g.N * 4);
    const bi8_rsrc rsa = bi8_make_rsrc(g.sA, (int64_t)nblk * g.M * 4);
    // scales of a stage: column scales lane -> K-block lane / 16 of the stage's BPS, column lane % 16; row scales: element
    // e = 64 u + lane of load instruction u -> K-block e / (16 MT), row e % (16 MT); rows past M read as zeros
    constexpr int kRowsA = 16 * MT;
    constexpr int kSaLoads = (kRowsA * BPS + 63) / 64;        // load instructions for a stage's row scales
    const uint32_t vsw = (uint32_t)((q * (int)g.N + (int)(n < g.N ? n : g.N - 1)) * 4);
    uint32_t vsa[kSaLoads];
#pragma unroll
    for (int u = 0; u < kSaLoads; ++u) {
        const int e = 64 * u + lane;
        vsa[u] = e % kRowsA < g.M ? (uint32_t)(((e / kRowsA) * (int)g.M + e % kRowsA) * 4) : (uint32_t)kBufOut;
    }

    // ---- loader: instruction i of a stage covers rows 8i .. 8i+7, lane -> row 8i + lane/8, LDS chunk lane%8, which
    // holds source chunk (lane%8) ^ ((row >> 1) & 7) = (lane%8) ^ (lane/16) ^ 4(i & 1)
    const int ld_row = lane >> 3;
    const int ld_chunk = (lane & 7) ^ ((lane >> 4) & 3);
    // (of A, instruction i = 2 t + p: the 16 rows of group t go into the scalar offset, so two registers serve all groups)
    uint32_t vw[2], va[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) vw[i] = (uint32_t)((8 * i + ld_row) * (int)g.ldw + 16 * (ld_chunk ^ (4 * i)));
#pragma unroll
    for (int i = 0; i < 2; ++i) va[i] = (uint32_t)((8 * i + ld_row) * (int)g.lda + 16 * (ld_chunk ^ (4 * i)));
    const uint32_t a_group = (uint32_t)(16 * (int)g.lda);
    auto issue_w = [&](int s, int slot) {          // s, slot: wave-uniform; four load instructions
        const int c = s * NW + wave;
        const bool live = c < nchunks;
        const uint32_t k0 = live ? (uint32_t)(c * KW) : (uint32_t)kBufOut;
#pragma unroll
        for (int i = 0; i < 2; ++i) bi8_buffer_to_lds16(rw, mine_addr + slot * kSlot + i * 1024, vw[i], k0);
        if (lane < 16 * BPS)                       // (the loads write LDS for the active lanes only)
            bi8_buffer_to_lds4(rsw, mine_addr + kScReg + slot * L::kScales, vsw, live ? (uint32_t)(c * BPS * (int)g.N * 4) : (uint32_t)kBufOut);
#pragma unroll
        for (int u = 0; u < kSaLoads; ++u)
            if (64 * u + lane < kRowsA * BPS)
                bi8_buffer_to_lds4(rsa, mine_addr + kScReg + slot * L::kScales + 128 + u * 256, vsa[u], live ? (uint32_t)(c * BPS * (int)g.M * 4) : (uint32_t)kBufOut);
    };
    auto issue_a = [&](int s, int slot) {          // 2 MT load instructions
        const int c = s * NW + wave;
        const uint32_t k0 = c < nchunks ? (uint32_t)(c * KW) : (uint32_t)kBufOut;
        // (a dead stage's offset stays past the end of the buffer with the rows of a group added: below 2^31, see the plan)
#pragma unroll
        for (int i = 0; i < 2 * MT; ++i) bi8_buffer_to_lds16(ra, mine_addr + kAReg + slot * L::kAStage + i * 1024, va[i & 1], k0 + (i >> 1) * a_group);
    };
    // operand fragments: lane -> row r16 (of W, or of a group of 16 rows of A), chunk 4j + q of the stage's eight, stored
    // at (4j + q) ^ ((r16 >> 1) & 7)
    const int frag = r16 * KW + ((q ^ ((r16 >> 1) & 7)) << 4);

    float acc[MT][4];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[t][r] = 0.0f;
    // in flight at the top of stage s, oldest first: ..., A(s), W(s + NSW - 2)
#pragma unroll
    for (int d = 0; d < NSW - 2; ++d) issue_w(d, d);
    issue_a(0, 0);
    issue_w(NSW - 2, NSW - 2);
    auto stage = [&](int s, auto slot_c) {
        constexpr int SW = decltype(slot_c)::value, SA = SW & 1;
        // The loads below overwrite the slots that the stage before has read.  Its ds_reads may still be in flight (the
        // compiler waits for them where their results are first used, which it places after these loads), and a load of A,
        // which every workgroup reads and the CU's L1 therefore often holds, can land within their latency: the reads
        // have to be complete first.  (Without this wait, a workgroup that shares its CU with an older one now and then
        // multiplied a stage's W by the A of two stages on.)
        __builtin_amdgcn_s_waitcnt(0xC07F);        // lgkmcnt(0)
        issue_a(s + 1, SA ^ 1);
        issue_w(s + NSW - 1, (SW + NSW - 1) % NSW);
        // everything up to A(s) has landed when only W(s + 3), A(s + 1) and W(s + 2) are outstanding
        constexpr int kPending = 2 * (3 + kSaLoads) + 2 * MT;
        static_assert(kPending < 64, "vmcnt is a 6-bit field");
        __builtin_amdgcn_s_waitcnt(0x0F70 | (kPending & 15) | ((kPending >> 4) << 14));
        const bi8_v4i zero = {0, 0, 0, 0};
        bi8_v4i wf[2], af[MT][2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            wf[j] = *(const bi8_v4i *)(mine + SW * kSlot + (frag ^ (j << 6)));
#pragma unroll
            for (int t = 0; t < MT; ++t) af[t][j] = *(const bi8_v4i *)(mine + kAReg + SA * L::kAStage + t * kSlot + (frag ^ (j << 6)));
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            bi8_v4i p[BPS];
            if constexpr (BPS == 1) {
                p[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[t][0], wf[0], zero, 0, 0, 0);
                p[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[t][1], wf[1], p[0], 0, 0, 0);
            } else {
                p[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[t][0], wf[0], zero, 0, 0, 0);
                p[1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[t][1], wf[1], zero, 0, 0, 0);
            }
#pragma unroll
            for (int b = 0; b < BPS; ++b) {
                const float sw = *(const float *)(mine + kScReg + SW * L::kScales + b * 64 + r16 * 4);
                const bi8_v4f sx = *(const bi8_v4f *)(mine + kScReg + SW * L::kScales + 128 + b * (64 * MT) + t * 64 + q * 16);
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[t][r] = __builtin_fmaf((float)p[b][r] * sx[r], sw, acc[t][r]);
            }
        }
    };
    for (int s = 0; s < nst; s += NSW) {
        stage(s, std::integral_constant<int, 0>{});
        stage(s + 1, std::integral_constant<int, 1>{});
        stage(s + 2, std::integral_constant<int, 2>{});
        stage(s + 3, std::integral_constant<int, 3>{});
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);            // vmcnt(0): nothing may still be writing LDS when the rings are reused
    __syncthreads();
    float(*red)[MT * 4][64] = (float(*)[MT * 4][64])lds;            // [wave][register][lane], over the rings
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave][t * 4 + r][lane] = acc[t][r];
    __syncthreads();
    if (wave == 0) {
        const float div = (float)(1.0 / (127.0 * 127.0));
        const bool has_bias = g.bias != nullptr;
        const float bias = (has_bias && n < g.N) ? load_bias(g, n) : 0.0f;
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float v = red[0][t * 4 + r][lane];
#pragma unroll
                for (int w = 1; w < NW; ++w) v += red[w][t * 4 + r][lane];
                const int64_t m = 16 * t + 4 * q + r;
                if (m < g.M && n < g.N) store_c<CDT>(g.C, m * g.ldc + n, v * div, has_bias, bias);
            }
    }
}

// ---- one or two rows, weight rows read as whole runs -------------------------------------------------------------------
// One or two rows of activations against all of W: single-token decode.  The problem is one pass over the N*K bytes of
// weight codes and nothing else matters.  Gathering W in the operand layout of an MFMA (16 rows x 64
// bytes per load instruction) reads 64-byte pieces of sixteen rows at a time, which this chip's memory pipeline serves
// at 3.8 - 4.5 TB/s; whole 1 KiB runs of one row per load instruction (lane -> 16 consecutive bytes) come in at 5.3 -
// 6.2 TB/s (a read-only micro-benchmark of the two patterns on the same grid).  With so few rows the matrix pipe has
// nothing to offer anyway (a 16-row MFMA would be 1/16 to 1/4 used), so the dot products are v_dot4_i32_i8 on the
// vector unit: per 16 bytes of W and row of activations four of them, then an integer sum over the lanes of a K-block
// (DPP), the conversion and the two scale products.  One workgroup = 16 output columns, a wave = four of them, each
// walked along K in runs of 1 KiB with sixteen loads in flight per lane (four rows x four runs).  The activations'
// codes [M][K] and row scales, and the 16 columns' scales, sit in LDS; with FUSED the codes are made here from the
// un-quantized activations by the row quantizer's own arithmetic (BlockInt8Linear.infer, block_linear.py:141-144, as one
// launch).  The fp32 sums run over the K-blocks in a fixed order (per lane group ascending, then a butterfly over the
// groups): the same code and therefore the same bits with and without FUSED.
constexpr int kRowsMax = 2;                        // rows of activations (with four the kernel needs more registers than three
                                                   // workgroups per CU leave it, and the MFMA kernel is as fast)
constexpr size_t kRowsLdsMax = 64 * 1024;
// scale rows in LDS: the K-blocks of whole runs, plus one run of zeros for loop slots past the end of K, rounded up to
// 16 rows (the rows are filled 64 floats at a time)
template <int BLK> constexpr int rows_blocks_padded(int64_t K) { return ((int)((K + 1023) / 1024 + 1) * (1024 / BLK) + 15) & ~15; }
// the kernel is compiled for 1 and for 2 rows
static inline int rows_compiled_for(int64_t M) { return M <= 1 ? 1 : 2; }
constexpr int64_t kRowsDeepK = 8192;               // from here on a single row of activations runs with six runs of W in flight per row
// x_bytes: size of an element of the un-quantized activations that the fused form stages in LDS (0: codes are given)
template <int BLK> static size_t rows_lds_bytes(int64_t M, int64_t K, int64_t x_bytes) {
    return (size_t)rows_blocks_padded<BLK>(K) * (4 + 16) * sizeof(float) + (size_t)rows_compiled_for(M) * (size_t)K + 1024 +
           (size_t)M * (size_t)K * (size_t)x_bytes;
}
template <int CTRL> __device__ __forceinline__ int bi8_dpp_i(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false); }

template <int BLK, int DT, bool FUSED, int MM, int CG>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3))) void gemv_rows(const GemmArgs g, const void *__restrict__ x, int64_t ldx) {
    static_assert(BLK == 64 || BLK == 128, "a K-block is 4 or 8 lanes of 16 bytes");
    constexpr int LB = BLK / 16;                   // lanes per K-block
    constexpr int BPC = 1024 / BLK;                // K-blocks per run of 1 KiB
    constexpr int R = 4;                           // rows of W per wave; CG = runs in flight per row
    extern __shared__ __attribute__((aligned(16))) float rows_lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int K = (int)g.K, M = (int)g.M;
    const int nblk = K / BLK;
    const int nrun = (K + 1023) / 1024;            // runs per row; the last one may be partial (K is a multiple of 128)
    const int nblk_pad = rows_blocks_padded<BLK>(K);
    float *s_sx = rows_lds;                        // [K-block][4 rows of activations], zeros past M and past K
    float *s_sw = s_sx + (size_t)nblk_pad * 4;     // [K-block][16 columns], zeros past N and past K
    int8_t *s_a = (int8_t *)(s_sw + (size_t)nblk_pad * 16);          // [M][K] codes (+ 1 KiB that partial runs may read)
    const int64_t n0 = (int64_t)blockIdx.x * 16;
    const int64_t wrows = g.N - n0 < 16 ? g.N - n0 : 16;
    const bi8_brsrc rw = bi8_make_brsrc(g.W + n0 * g.ldw, (wrows - 1) * g.ldw + g.K);   // rows past N read as zeros

    // ---- Order of the memory traffic.  Loads complete in the order they are issued, so what the prologue needs goes
    // out FIRST (a few KiB: the activations, their scales, the 16 columns' scales), then this wave's first R*CG runs
    // of W; the prologue then waits for its own data only ("at most R*CG loads still outstanding"), and the loop works
    // on the runs of W as they arrive.  Scales (and, without FUSED, the codes) go global -> LDS directly, no registers.
    // The workgroup barrier is a bare s_barrier behind an LDS wait: a fence would wait for the W loads as well.
    const uint32_t lds0 = bi8_lds_address(rows_lds);
    {
        const bi8_rsrc sw_rsrc = bi8_make_rsrc(g.sW, (int64_t)nblk * g.N * 4);
        for (int i0 = wave * 64; i0 < nblk_pad * 16; i0 += 256) {
            const int i = i0 + lane, jb = i >> 4, n = i & 15;
            const uint32_t off = (jb < nblk && n < wrows) ? (uint32_t)(((int64_t)jb * g.N + n0 + n) * 4) : (uint32_t)kBufOut;
            bi8_buffer_to_lds4(sw_rsrc, lds0 + (uint32_t)(nblk_pad * 4 + i0) * 4, off, 0);
        }
    }
    constexpr int VEC = FUSED ? Bi8Vec<DT>::kElems : 16;
    const int cpr = K / VEC;                       // 16-byte chunks per row of activations
    const int total = M * cpr;
    // FUSED: the un-quantized activations are staged in LDS behind the codes, chunk c at byte 16 * c
    const uint32_t stage0 = lds0 + (uint32_t)(nblk_pad * 20) * 4 + (uint32_t)(MM * K + 1024);
    if constexpr (FUSED) {
        constexpr int ES = 16 / VEC;
        const bi8_rsrc x_rsrc = bi8_make_rsrc(x, ((int64_t)(M - 1) * ldx + K) * ES);
        for (int c0 = wave * 64; c0 < total; c0 += 256) {
            const int c = c0 + lane;
            const uint32_t off = c < total ? (uint32_t)(((c / cpr) * (int)ldx + (c % cpr) * VEC) * ES) : (uint32_t)kBufOut;
            bi8_buffer_to_lds16(x_rsrc, stage0 + (uint32_t)c0 * 16, off, 0);
        }
    } else {
        // codes [M][K] (rows are 16-byte aligned; LDS keeps them densely, so chunk c lands at byte 16 * c) and the row
        // scales [K-block][M] into [K-block][4]
        const bi8_rsrc a_rsrc = bi8_make_rsrc(g.A, (int64_t)(M - 1) * g.lda + K);
        for (int c0 = wave * 64; c0 < total; c0 += 256) {
            const int c = c0 + lane;
            const uint32_t off = c < total ? (uint32_t)((c / cpr) * (int)g.lda + (c % cpr) * 16) : (uint32_t)kBufOut;
            bi8_buffer_to_lds16(a_rsrc, lds0 + (uint32_t)(nblk_pad * 20) * 4 + (uint32_t)c0 * 16, off, 0);
        }
        const bi8_rsrc sa_rsrc = bi8_make_rsrc(g.sA, (int64_t)nblk * M * 4);
        for (int i0 = wave * 64; i0 < nblk_pad * 4; i0 += 256) {
            const int i = i0 + lane, jb = i >> 2, m = i & 3;
            const uint32_t off = (jb < nblk && m < M) ? (uint32_t)((jb * M + m) * 4) : (uint32_t)kBufOut;
            bi8_buffer_to_lds4(sa_rsrc, lds0 + (uint32_t)i0 * 4, off, 0);
        }
    }
    // (the compiler must not move the loads of W, which it knows to be plain loads, above the ones before)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    bi8_v4i w[CG][R];
    auto load_w = [&](int c, int cc, int r) {      // run c of row 4 * wave + r into slot (cc, r)
        const int k = c * 1024 + lane * 16;
        const int voff = (k < K ? (4 * wave + r) * (int)g.ldw + k : kBufOut);          // past K: no access, zeros
        w[cc][r] = bi8_buffer_load16(rw, voff, 0, true);
    };
#pragma unroll
    for (int cc = 0; cc < CG; ++cc)
#pragma unroll
        for (int r = 0; r < R; ++r) load_w(cc, cc, r);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    if constexpr (FUSED) {
        // x [M,K] of type DT -> codes and scales, with the row quantizer's helpers (same results).  Every wave works on
        // the chunks that it fetched itself (they have landed once at most the R*CG runs of W are outstanding);
        // K % 128 == 0 makes every aligned group of L chunks one K-block of one row.
        constexpr int L = BLK / VEC;
        constexpr int NCORR = (DT == BI8_F32) ? 2 : 1;
        __builtin_amdgcn_s_waitcnt(0x0F70 | ((R * CG) & 15) | (((R * CG) >> 4) << 14));   // vmcnt(R * CG)
        const uint8_t *stage = (const uint8_t *)s_a + (size_t)MM * K + 1024;
        for (int c0 = wave * 64; c0 < total; c0 += 256) {
            const int c = c0 + lane;                                   // (total is a multiple of L: whole groups are in or out)
            const bi8_v4u raw = c < total ? *(const bi8_v4u *)(stage + (size_t)c * 16) : bi8_v4u{0u, 0u, 0u, 0u};
            const int row = c / cpr, col = (c % cpr) * VEC;
            float f[VEC];
            bi8_unpack<DT>(raw, f);
            float m = 0.0f;
            bool special = false;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                m = __builtin_fmaxf(m, __builtin_fabsf(f[e]));
                special |= (f[e] != f[e]);
            }
            m = bi8_group_max<L>(m);
            special |= !bi8_scale_is_ordinary(m);
            uint32_t code[VEC];
            if (__builtin_expect(special, 0)) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) code[e] = bi8_code_slow(f[e], m);
            } else {
                const float y = 1.0f / m;
#pragma unroll
                for (int e = 0; e < VEC; ++e) code[e] = bi8_code_fast<NCORR>(f[e], m, y);
            }
            if (c < total) {
                if ((lane & (L - 1)) == 0) s_sx[(col / BLK) * 4 + row] = m;
                int8_t *dst = s_a + row * K + col;
                if constexpr (VEC == 4) {
                    *(uint32_t *)dst = bi8_pack4(code[0], code[1], code[2], code[3]);
                } else {
                    *(bi8_v2u *)dst = bi8_v2u{bi8_pack4(code[0], code[1], code[2], code[3]), bi8_pack4(code[4], code[5], code[6], code[7])};
                }
            }
        }
        for (int i = tid; i < nblk_pad * 4; i += 256)
            if (i >= nblk * 4 || (i & 3) >= M) s_sx[i] = 0.0f;
    }
    // the direct-to-LDS loads were all issued before the R*CG runs of W
    __builtin_amdgcn_s_waitcnt(0x0F70 | ((R * CG) & 15) | (((R * CG) >> 4) << 14));       // vmcnt(R * CG)
    __builtin_amdgcn_s_waitcnt(0xC07F);                                                     // lgkmcnt(0): this wave's LDS writes
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    float acc[R][MM];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MM; ++m) acc[r][m] = 0.0f;
    const int8_t *a_lane = s_a + lane * 16;
    const int grp = lane / LB;                     // this lane's K-block inside a run
    // one group of CG runs: every slot is consumed (run, then row) and, with REFILL, loaded again with the run CG on
    auto group = [&](int c0, auto refill) {
        constexpr bool REFILL = decltype(refill)::value;
#pragma unroll
        for (int cc = 0; cc < CG; ++cc) {
            const int c = c0 + cc;
            const int kc = (c < nrun ? c : nrun - 1) * 1024;           // runs past the end: zero W against any codes ...
            const int jb = (c < nrun ? c : nrun) * BPC + grp;          // ... and zero scales
            bi8_v4i xa[MM];                                            // (rows past M: whatever the LDS holds, against zero scales)
#pragma unroll
            for (int m = 0; m < MM; ++m) xa[m] = *(const bi8_v4i *)(a_lane + m * K + kc);
            const bi8_v4f sxv = *(const bi8_v4f *)(s_sx + jb * 4);
            const bi8_v4f swv = *(const bi8_v4f *)(s_sw + jb * 16 + 4 * wave);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const bi8_v4i wv = w[cc][r];
                if constexpr (REFILL) load_w(c + CG, cc, r);
                const float swr = swv[r];
#pragma unroll
                for (int m = 0; m < MM; ++m) {
                    int p = __builtin_amdgcn_sdot4(wv[0], xa[m][0], 0, false);
                    p = __builtin_amdgcn_sdot4(wv[1], xa[m][1], p, false);
                    p = __builtin_amdgcn_sdot4(wv[2], xa[m][2], p, false);
                    p = __builtin_amdgcn_sdot4(wv[3], xa[m][3], p, false);
                    p += bi8_dpp_i<0xB1>(p);                           // lanes ^1
                    p += bi8_dpp_i<0x4E>(p);                           // lanes ^2
                    if constexpr (LB == 8) p += bi8_dpp_i<0x141>(p);       // the other quad of the K-block (half-row mirror)
                    acc[r][m] = __builtin_fmaf((float)p * sxv[m], swr, acc[r][m]);
                }
            }
        }
    };
    int c0 = 0;
    for (; c0 + CG < nrun; c0 += CG) group(c0, std::true_type{});
    group(c0, std::false_type{});

    // every lane of a K-block's group holds the same sums: add up the groups (butterfly over the lane bits above a group)
    const float div = (float)(1.0 / (127.0 * 127.0));
    const bool has_bias = g.bias != nullptr;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t n = n0 + 4 * wave + r;
        const float bias = (has_bias && n < g.N) ? load_bias(g, n) : 0.0f;
#pragma unroll
        for (int m = 0; m < MM; ++m) {
            if (m < M) {
                float v = acc[r][m];
                if constexpr (LB == 4) v += bi8_dpp<0x141>(v);         // groups ^1 (lanes ^4: half-row mirror across the quads)
                v += bi8_dpp<0x140>(v);                                // lanes ^8 (row mirror across the halves of a row)
                v += __shfl_xor(v, 16, 64);
                v += __shfl_xor(v, 32, 64);
                if (lane == 0 && n < g.N) store_c<DT>(g.C, (int64_t)m * g.ldc + n, v * div, has_bias, bias);
            }
        }
    }
}

// Fallback for any K, block, alignment: 4 waves, each a 32x32 output subtile; every lane gathers its own
// 16-byte MFMA operands with byte loads (zero outside the matrix and outside the current K-block).
template <int CDT, bool PARTIALS>
__global__ __launch_bounds__(256) void gemm_generic(const GemmArgs g, int block) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int tile_m = blockIdx.x / g.tiles_n, tile_n = blockIdx.x % g.tiles_n;
    const int64_t m_base = (int64_t)tile_m * 64 + (wave >> 1) * 32;
    const int64_t n_base = (int64_t)tile_n * 64 + (wave & 1) * 32;
    const int64_t am = m_base + l32, wnr = n_base + l32;
    const int64_t nblk = (g.K + block - 1) / block;
    const float div = (float)(1.0 / (127.0 * 127.0));
    float acc[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

    for (int64_t jb = 0; jb < nblk; ++jb) {
        const int64_t kb = jb * block;
        const int64_t ke = (kb + block < g.K) ? (kb + block) : g.K;
        bi8_v16i p = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        for (int64_t k = kb; k < ke; k += 32) {
            bi8_v4i af = {0, 0, 0, 0}, wf = {0, 0, 0, 0};
            const int64_t kk = k + h * 16;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int64_t ki = kk + e;
                uint32_t av = 0, wv = 0;
                if (ki < ke) {
                    if (am < g.M) av = (uint8_t)g.A[am * g.lda + ki];
                    if (wnr < g.N) wv = (uint8_t)g.W[wnr * g.ldw + ki];
                }
                af[e >> 2] |= (int)(av << (8 * (e & 3)));
                wf[e >> 2] |= (int)(wv << (8 * (e & 3)));
            }
            p = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, wf, p, 0, 0, 0);
        }
        const int64_t n = n_base + l32;
        if constexpr (PARTIALS) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t m = m_base + 8 * (r >> 2) + 4 * h + (r & 3);
                if (m < g.M && n < g.N) g.P[(jb * g.M + m) * g.N + n] = p[r];
            }
        } else {
            const float sw = (n < g.N) ? g.sW[jb * g.N + n] : 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t m = m_base + 8 * (r >> 2) + 4 * h + (r & 3);
                const float sx = (m < g.M) ? g.sA[jb * g.M + m] : 0.0f;
                acc[r] = __builtin_fmaf((float)p[r] * sx, sw, acc[r]);
            }
        }
    }
    if constexpr (!PARTIALS) {
        const int64_t n = n_base + l32;
        const bool has_bias = g.bias != nullptr;
        const float bias = (has_bias && n < g.N) ? load_bias(g, n) : 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int64_t m = m_base + 8 * (r >> 2) + 4 * h + (r & 3);
            if (m < g.M && n < g.N) store_c<CDT>(g.C, m * g.ldc + n, acc[r] * div, has_bias, bias);
        }
    }
}

// Sum of a tile's slabs in ascending workgroup order (deterministic), then the cast and the bias of the one-pass
// epilogue.  One workgroup = 8 rows of one tile (16 or 32 of a tile of 64 or 32 columns), a thread = four consecutive columns; a tile has at most kSplitMax slabs,
// all loaded before the first addition.  With split_per_tile workgroups per tile, tile t's slabs are
// t * split_per_tile ... ; with runs, the workgroups whose runs touch tile t are floor(t * nst / S) ...
// floor(((t + 1) * nst - 1) / S), and workgroup w's slab for it is ws[w + t].
template <int CDT, int BM, int BN>
__global__ __launch_bounds__(256) void splitk_reduce(const GemmArgs g) {
    constexpr int kCols4 = BN / 4, kRowsPerGroup = 256 / kCols4;     // BN = 128: 32 threads per row, 8 rows per workgroup; 64: 16 and 16; 32: 8 and 32
    static_assert((BN == 128 || BN == 64 || BN == 32) && BM % kRowsPerGroup == 0, "whole rows per workgroup (grid y = BM / rows per workgroup)");
    const int t = blockIdx.x, tile_m = t / g.tiles_n, tile_n = t - tile_m * g.tiles_n;
    const int nst = (int)(g.K / kStageK), S = g.split_stages;
    int first, count;
    if (g.split_per_tile > 0) {
        first = t * g.split_per_tile;
        count = (nst + S - 1) / S;
    } else {
        const int w0 = (t * nst) / S, w1 = ((t + 1) * nst - 1) / S;
        first = w0 + t;
        count = w1 - w0 + 1;
    }
    const int i = blockIdx.y * kRowsPerGroup + (int)threadIdx.x / kCols4, j = ((int)threadIdx.x % kCols4) * 4;
    const int64_t m = (int64_t)(tile_m + g.tile_m0) * BM + i;
    if (m >= g.M) return;
    const float *src = g.ws + (int64_t)first * (BM * BN) + i * BN + j;
    bi8_v4f x[kSplitMax];
#pragma unroll
    for (int q = 0; q < kSplitMax; ++q) x[q] = q < count ? *(const bi8_v4f *)(src + (int64_t)q * (BM * BN)) : bi8_v4f{0.0f, 0.0f, 0.0f, 0.0f};
    bi8_v4f v = x[0];
#pragma unroll
    for (int q = 1; q < kSplitMax; ++q)
        if (q < count) v += x[q];
    const bool has_bias = g.bias != nullptr;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int64_t n = (int64_t)(tile_n + g.tile_n0) * BN + j + q;
        if (n < g.N) store_c<CDT>(g.C, m * g.ldc + n, v[q], has_bias, has_bias ? load_bias(g, n) : 0.0f);
    }
}

// How to split a problem that the tile kernels would run on fewer workgroups than the chip has CUs, and with which tile
// (kind 0: 64x128, 1: 128x128).
// Up to 128 tiles: the same number of workgroups per tile, as many as fill the 256 CUs once, at least kSplitMinStages
// stages of K each, at most kSplitMax (measured: 4 x 8 stages beat 8 x 4 at K = 4096, 8 x 11 beat 4 x 22 at K = 11008).
// 129 to 255 tiles: the (tile, stage) pairs are dealt to 256 workgroups in equal runs that need not end where tiles end
// (144 tiles of 64 stages are 256 runs of 36), when that saves kRunMinSaved stages and a quarter of a tile's K: a
// workgroup whose run crosses into a second tile fills its pipeline twice and writes two slabs, and all tiles go through
// the second kernel (measured: 3072 x 768 x 8192 at block 64 62.1 -> 54.3 us, 1500 x 1500 x 16384 at block 128
// 84.8 -> 70.6; runs in place of the equal split of few tiles cost 10-25 %).
constexpr int64_t kCus = 256;                  // compute units the plan counts rounds of workgroups against (MI355X)
constexpr int kSplitMinStages = 8, kRunMinSaved = 28;
// The split of 256x128 tiles on gemm_wide's loop pays where pieces are long and the tiles few: every piece writes and the
// second kernel reads a slab of 128 KiB.  Measured against the split (or unsplit) 128x128 tiles, bf16 out: block 64, K = 8192
// (the GPT-2 grad-weight GEMMs), 3072 x 768 (3 pieces of 22 stages per tile) 50.2 -> 43.5 us, 768 x 3072 49.2 -> 42.8, 2304 x
// 768 (4 x 16) 40.3 -> 35.1; block 128: 1024 x 2048 x 8192 (4 x 16) 34.9 -> 34.2, but 512 x 4096 x 4096 (4 x 8) 23.5 -> 24.9,
// 256 x 4096 x 11008 (8 x 12) 27.3 -> 29.2, 1024 x 4096 x 4096 (2 x 16, 256 slabs) 28.0 -> 34.7, 256 x 11008 x 4096 25.9 -> 30.5.
constexpr int64_t kWideSplitMinGroups = 160;   // workgroups that the split 256x128 tiles have to put to work,
constexpr int64_t kWideSplitMinStages = 16;    // ... the least stages of K per piece
constexpr int64_t kWideSplitMinPer = 3;        // ... and pieces per tile
struct SplitGrid {
    int groups, stages, per_tile;                  // workgroups, stages of K per workgroup, workgroups per tile (0: runs); groups <= 1: no split
};
static SplitGrid split_grid(int64_t tiles, int64_t nstages) {
    const SplitGrid none{1, 0, 0};
    if (tiles <= 0 || tiles >= kCus || tiles * nstages >= (1ll << 30)) return none;
    if (tiles <= 128) {
        int64_t sp = kCus / tiles;
        if (sp > kSplitMax) sp = kSplitMax;
        if (sp > nstages / kSplitMinStages) sp = nstages / kSplitMinStages;
        if (sp < 2) return none;
        const int64_t stages = (nstages + sp - 1) / sp;
        const int64_t per = (nstages + stages - 1) / stages;               // every workgroup has work
        return per < 2 ? none : SplitGrid{(int)(tiles * per), (int)stages, (int)per};
    }
    const int64_t run = (tiles * nstages + kCus - 1) / kCus;
    if (nstages - run < kRunMinSaved || 4 * run > 3 * nstages) return none;
    return SplitGrid{(int)((tiles * nstages + run - 1) / run), (int)run, 0};
}
static SplitGrid plan_split(int64_t M, int64_t N, int64_t K, int &kind) {
    const int64_t nstages = K / kStageK;
    kind = M > 64 ? 1 : 0;
    const int64_t t128 = ((M + 127) / 128) * ((N + 127) / 128), t64 = ((M + 63) / 64) * ((N + 127) / 128);
    // (splitting the 256x128 tile where the 128x128 tiles are too many to split measured slower than not splitting)
    const SplitGrid sg = split_grid(kind ? t128 : t64, nstages);
    // a short K caps the number of splits: when the 128x128 tiles then fill at most half of the CUs, the 64x128 tile
    // puts twice as many workgroups to work
    const int64_t wgs = sg.groups > 1 ? sg.groups : t128;
    if (kind == 1 && wgs <= 128) {
        const SplitGrid s64 = split_grid(t64, nstages);
        if (s64.groups > 1 && s64.per_tile > 0 && s64.groups > wgs) {
            kind = 0;
            return s64;
        }
    }
    return sg;
}

// A kernel that uses more than 64 KiB of dynamic LDS has to be allowed to, once per device: remembered here so that
// the launch path makes that runtime call only the first time.
struct LdsOptIn {
    std::atomic<uint64_t> done{0};                 // bit d: device d has the attribute
    int ensure(const void *kern, int bytes) {
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return bi8_hip_rc(e);
        if (dev >= 0 && dev < 64 && ((done.load(std::memory_order_acquire) >> dev) & 1)) return BI8_OK;
        e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e != hipSuccess) return bi8_hip_rc(e);
        if (dev >= 0 && dev < 64) done.fetch_or(1ull << dev, std::memory_order_release);
        return BI8_OK;
    }
};

// Compute units of the current device, rounded down to whole rounds over the XCDs so that a workgroup of a persistent
// grid keeps to its own XCD's share of the tile order (looked up once per device).
static int compute_units(int *out) {
    static std::atomic<int> cached[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return bi8_hip_rc(e);
    int n = (dev >= 0 && dev < 64) ? cached[dev].load(std::memory_order_acquire) : 0;
    if (n <= 0) {
        e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return bi8_hip_rc(e);
        n = n >= kXcds ? n - n % kXcds : kXcds;
        if (dev >= 0 && dev < 64) cached[dev].store(n, std::memory_order_release);
    }
    *out = n;
    return BI8_OK;
}

// gemm_wide addresses each operand through one buffer with 32-bit offsets
static bool wide_addressable(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int block) {
    const int64_t lim = 0x7fffffffLL, nblk = K / block;
    return (M - 1) * lda + K <= lim && (N - 1) * ldw + K <= lim && nblk * M * 4 <= lim && nblk * N * 4 <= lim && M + 256 <= lim && N + 256 <= lim;
}

template <int BM, int BN, int WM, int WN, int NBUF, int BLK, int CDT, bool PARTIALS, bool SPLIT = false>
int launch_tile(GemmArgs g, const Part &part, hipStream_t st) {
    constexpr int kLds = TileLds<BM, BN, BLK, NBUF>::kBytes;
    static_assert(TileLds<BM, BN, BLK, NBUF>::kFits, "tile does not fit the LDS");
    if (part.row0 % BM != 0 || part.col0 % BN != 0) return BI8_ERR_UNSUPPORTED;     // (the plan cuts at multiples of 256 only)
    const int64_t tm = (part.rows + BM - 1) / BM, tn = (part.cols + BN - 1) / BN;
    if (tm * tn > 0x7fffffffLL) return BI8_ERR_TOO_LARGE;
    g.tiles_m = (int)tm;
    g.tiles_n = (int)tn;
    g.tile_m0 = (int)(part.row0 / BM);
    g.tile_n0 = (int)(part.col0 / BN);
    auto kern = gemm_tile<BM, BN, WM, WN, NBUF, BLK, CDT, PARTIALS, SPLIT>;
    if (SPLIT != (g.splits > 1)) return BI8_ERR_UNSUPPORTED;         // (the plan pairs them)
    if (kLds > 64 * 1024) {
        static LdsOptIn opted;                     // one per kernel instantiation
        const int rc = opted.ensure((const void *)kern, kLds);
        if (rc != BI8_OK) return rc;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)(SPLIT ? g.splits : tm * tn)), dim3(WM * WN * 64), kLds, st, g);
    return bi8_launch_rc();
}

template <int BLK, int CDT, int NJ = 8, bool SPLIT = false> int launch_wide(GemmArgs g, const Part &part, hipStream_t st) {
    constexpr int BN = 32 * NJ;
    using L = WideLds<kStageK / BLK, BN>;
    if (part.row0 % 256 != 0 || part.col0 % BN != 0) return BI8_ERR_UNSUPPORTED;   // (the plan cuts at multiples of 256 only)
    const int64_t tm = (part.rows + 255) / 256, tn = (part.cols + BN - 1) / BN;
    if (tm * tn > 0x7fffffffLL) return BI8_ERR_TOO_LARGE;
    g.tiles_m = (int)tm;
    g.tiles_n = (int)tn;
    g.tile_m0 = (int)(part.row0 / 256);
    g.tile_n0 = (int)(part.col0 / BN);
    if (!wide_addressable(g.M, g.N, g.K, g.lda, g.ldw, BLK)) return BI8_ERR_TOO_LARGE;       // the plan does not send such a problem here
    g.band_magic = (uint32_t)((1ull << 32) / (uint64_t)(kGroupM * tn));
    auto kern = gemm_wide<BLK, CDT, NJ, SPLIT>;
    static LdsOptIn opted;                         // one per kernel instantiation
    const int rc = opted.ensure((const void *)kern, L::kBytesPersistent);
    if (rc != BI8_OK) return rc;
    if constexpr (SPLIT) {                         // one piece per workgroup: split_per_tile pieces of every tile
        if (g.split_per_tile < 2 || g.split_stages < 2 || g.split_stages % 2 != 0 || tm * tn * g.split_per_tile > kCus) return BI8_ERR_UNSUPPORTED;
        hipLaunchKernelGGL(kern, dim3((unsigned)(tm * tn), (unsigned)g.split_per_tile), dim3(512), L::kBytesPersistent, st, g);
        return bi8_launch_rc();
    }
    int cus = 0;
    const int rc_cus = compute_units(&cus);
    if (rc_cus != BI8_OK) return rc_cus;
    const int64_t grid = tm * tn < cus ? tm * tn : cus;        // the kernel's LDS leaves room for one workgroup per CU
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), L::kBytesPersistent, st, g);
    return bi8_launch_rc();
}

template <int BLK, int CDT> int launch_wide32(GemmArgs g, hipStream_t st) {
    using L = Wide32Lds<kStageK / BLK>;
    const int64_t tm = (g.M + 255) / 256, tn = (g.N + 255) / 256;
    if (tm * tn > 0x7fffffffLL) return BI8_ERR_TOO_LARGE;
    g.tiles_m = (int)tm;
    g.tiles_n = (int)tn;
    auto kern = gemm_wide32<BLK, CDT>;
    static LdsOptIn opted;                         // one per kernel instantiation
    const int rc = opted.ensure((const void *)kern, L::kBytes);
    if (rc != BI8_OK) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)(tm * tn)), dim3(512), L::kBytes, st, g);
    return bi8_launch_rc();
}

template <int CDT, bool PARTIALS> int launch_generic(GemmArgs g, int block, hipStream_t st) {
    const int64_t tm = (g.M + 63) / 64, tn = (g.N + 63) / 64;
    if (tm * tn > 0x7fffffffLL) return BI8_ERR_TOO_LARGE;
    g.tiles_m = (int)tm;
    g.tiles_n = (int)tn;
    hipLaunchKernelGGL((gemm_generic<CDT, PARTIALS>), dim3((unsigned)(tm * tn)), dim3(256), 0, st, g, block);
    return bi8_launch_rc();
}


// ---- which kernel runs a problem ------------------------------------------------------------------------------------
// One rule, used by the launcher, by bi8_gemm_workspace_bytes and by bi8_gemm_kernel_name.
enum GemmKernel { kKGeneric = 0, kKGemv, kKSkinny, kKWide, kKTile256x128, kKTile128x128, kKTile64x128, kKSplit128x128, kKSplit64x128, kKRows, kKWideHalf, kKSplitWideHalf, kKPanel, kKSplitPanel };
static const char *const kGemmKernelNames[] = {"gemm_generic", "gemv_staged", "gemm_skinny", "gemm_wide", "gemm_tile_256x128",
                                                "gemm_tile_128x128", "gemm_tile_64x128", "gemm_tile_128x128_splitk",
                                                "gemm_tile_64x128_splitk", "gemv_rows", "gemm_wide_256x128", "gemm_wide_256x128_splitk", "gemm_panel", "gemm_panel_splitk"};
struct GemmPlan {
    int kernel;
    int splits, split_stages;      // of the split kernels: workgroups of the split grid and 128-byte stages of K per workgroup,
    int split_per_tile;            // ... workgroups per tile (0: runs across tiles)
    int64_t ws_need;               // ... and the bytes of scratch memory for their slabs
    // a problem cut in two launches (cut_axis 0: one launch): `kernel` (the 256x256 kernel) on the leading `lead` rows
    // (cut_axis 1) or columns (2) of the output, the rest_* kernel of the tile family on the others
    int cut_axis;
    int64_t lead;
    int rest_kernel, rest_splits, rest_split_stages, rest_split_per_tile;
};
// Up to 128 tiles of 256x256 the same problem is at most 256 tiles of 256x128: one round of workgroups on the 256 CUs,
// where the smaller tile wins (1424 against 1072 TOP/s at 2048x4096x4096).  From 129 on the 256x128 grid needs a second,
// mostly empty round and the 256x256 kernel wins (1284 against 978 TOP/s at 2304x4096x4096, 144 tiles).
// (choosing between the two by the fill of the last round of workgroups changed nothing measurable)
constexpr int64_t kWideMinTiles = 129;
// gemm_panel: at most one tile of 128 x (16 ... 64) -- up to 64 rows: 64 x (32 ... 128), up to 32: 32 x (64 ... 256) -- per CU, and a
// short K: every workgroup streams all rows of A, so its time grows with K faster than that of the kernels that split the
// contraction.  Measured against what ran these shapes before (one-pass or split 64x128 / 128x128 tiles), W from HBM,
// block 128, us at K = 768 / 2048 / 4096 / 8192: 128 x 768 8.4 -> 4.3, 10.8 -> 6.0, 11.0 -> 8.7, 12.7 -> 13.8; 128 x 4096
// 8.6 -> 4.9, 12.8 -> 6.6, 14.9 -> 12.3, 21.7 -> 21.8; 128 x 11008 9.2 -> 6.5, 19.3 -> 10.9, 22.5 -> 18.2, 35.0 -> 35.2;
// 512 x 2048 8.6 -> 5.3, 15.1 -> 8.0, 22.3 -> 12.0, 24.7 -> 23.6; 1024 x 1024 (512 x 1024: the same tiles) 8.6 -> 4.7,
// 15.2 -> 6.5, 22.4 -> 9.6; block 64, 128 x 4096 (first form of the kernel) 9.6 -> 5.8, 14.8 -> 9.1, 16.6 -> 15.3.
constexpr int64_t kPanelMinRows = 64;          // more rows: tiles of 128 rows; 33 ... 64: tiles of 64 rows
constexpr int64_t kPanelMaxStages = 32;        // K <= 4096
constexpr int64_t kPanelSplitMinStages = 8;    // the split form: the least stages of K per piece ...
constexpr int64_t kPanelSplitMaxStages = 96;   // ... and the longest K (12288)
constexpr int64_t kPanelSplitFewRowsMin = 16;  // the split form on tiles of 32 rows: more rows than this, ...
constexpr int64_t kPanelSplitFewRowsMinStages = 64, kPanelSplitFewRowsTwoStages = 80;      // ... K from 8192 on; two pieces per tile from 10240 on, ...
constexpr int64_t kPanelSplitFewRowsMinGroups = 192;                                       // ... and this many workgroups
constexpr int64_t kPanelSplit64RowsMinStages = 40, kPanelSplit64RowsMaxTiles = 32;         // on tiles of 64 rows: K from 5120 on, up to 2048 columns
constexpr int64_t kPanelOverStagedStages = 8;  // 33 ... 64 rows inside gemv_staged's band: only up to K = 1024 ...
constexpr int64_t kPanelOverStagedMinCols = 3072;      // ... or from this many columns on
constexpr int64_t kPanelSquareSplitMinTiles = 100, kPanelSquareSplitMinStages = 64;     // the square form on two pieces of K: 100 ... 128 tiles, K from 8192 on
constexpr int64_t kPanelSquareMinTiles = 176;  // the square form outright from this many tiles on; with fewer only where nothing splits K
constexpr int64_t kPanelHalfHeightMaxSubtiles = 4;     // more than 64 rows on tiles of 64 rows: where those are at most 64 columns wide
constexpr int64_t kPanelFewRows = 32;          // up to 32 rows: tiles of 32 rows x (64 ... 256) columns ...
constexpr int64_t kPanelFewRowsMinCols = 5120; // ... from this many columns on (fewer leave most CUs without a tile)
// the widest tile, in 16-column subtiles (block 64 at 64 columns needs more registers than a wave has)
constexpr int panel_max_subtiles(int block) { return block == 64 ? 3 : 4; }
constexpr int64_t kStagedMaxRows = 32;         // gemv_staged: one or two groups of 16 rows whatever the shape ...
// ... and up to four where one round of workgroups covers the columns and a workgroup's pass over all of A stays short: every
// workgroup streams the whole of A through its LDS, which a split of K divides.  Measured against the split 64x128 tiles,
// W from HBM, block 128, 48 / 64 rows: 4096 -> 4096 12.8 -> 9.6 / 13.3 -> 10.3 us, but 4096 -> 11008 (2.7 rounds) 17.4 -> 23.8 /
// 17.9 -> 26.0 and 11008 -> 4096 16.7 -> 19.8 / 17.2 -> 21.8; eight groups (128 rows, three waves) lose everywhere (4096 -> 4096
// 14.7 -> 17.0, 4096 -> 11008 21.9 -> 45.3).
constexpr int64_t kStagedWideRows = 64, kStagedWideMaxGroups = 288, kStagedWideMaxCodes = 320 * 1024;
// `aligned`: A and W 16-byte aligned, the scales 4-byte aligned (the partials entry point has no scales);
// ws_bytes: scratch memory the split kernels may use (0: none).
// A last round of 256x256 tiles that is mostly empty costs as much as a full one (1280 x 11008 x 4096: 215 tiles, 69 us;
// 1536 x 11008 x 4096: 258 tiles, 125 us).  When whole rows or columns of tiles can be cut off so that the leading part
// is full rounds and the rest at most kCutMaxRest tiles' worth, the rest runs as a second launch on the smaller tiles
// that suit it (measured, both launches: 1536 x 11008 x 4096 123 -> 93 us, 2304 x 8192 x 8192 229 -> 170, 4352 x 4096 x
// 4096 120 -> 91, 2048 x 11008 x 4096 123 -> 114, 8192 x 2304 x 768 at block 64 43 -> 37; a rest of 96 tiles, 8192 x
// 11008 x 4096, 378 -> 383: not cut).
constexpr int64_t kCutMaxRest = 90;
static GemmPlan plan_gemm(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int block, bool aligned, bool partials,
                          int64_t ws_bytes, bool rest_of_cut = false) {
    GemmPlan p{kKGeneric, 1, 0, 0, 0, 0, 0, kKGeneric, 1, 0, 0};
    // the tiled kernels address a tile's operand rows and the scale rows with 32-bit byte offsets
    const int64_t max_ld = lda > ldw ? lda : ldw, max_mn = M > N ? M : N;
    const bool offsets_ok = max_ld < (1 << 22) && (block <= 0 || (K / block + 1) * max_mn * 4 < 0x7fffffffLL);
    const bool tile_ok = K > 0 && K % kStageK == 0 && lda % 16 == 0 && ldw % 16 == 0 && aligned && offsets_ok &&
                         (block == 32 || block == 64 || block == 128);
    if (!tile_ok) return p;
    // few tiles and scratch memory: split K over the workgroups, then sum the slabs
    bool panel_if_no_split = false;                // gemm_panel's tiles would give one round, but K is beyond what it is given outright
    bool square_if_no_split = false;               // its square tiles would, but they are few enough that a split of K may be ahead
    auto try_split = [&](bool few_rows_split = false) {
        if (partials || ws_bytes <= 0) return false;
        // 65 ... 128 rows and K up to 12288: gemm_panel on pieces of K, tiles of 128 rows x 64 columns (block 64: 32).  Measured
        // against the split 64x128 / 128x128 tiles, block 128, W from HBM, us at K = 8192 / 11008 / 16384: 128 x 768 12.9 -> 11.1,
        // 13.7 -> 11.8, 17.4 -> 14.1; 128 x 4096 21.7 -> 18.8, 24.8 -> 20.1, 25.8 -> 31.2; 128 x 8192 28.4 -> 26.3, 35.4 -> 32.9,
        // 43.7 -> 46.7; 512 x 768 18.7 -> 15.1, 19.9 -> 20.3; 512 x 2048 25.8 -> 23.6, 28.5 -> 28.8; 1024 x 768 21.8 -> 23.0
        // (256 workgroups that each stream all of A: the longer the pieces and the more rows of tiles, the less it pays).
        // 17 ... 32 rows and K from 8192 on: the same on tiles of 32 x 64 where the columns leave three pieces of K or more per tile,
        // or two of 40 stages, and 192 workgroups or more; 33 ... 64 rows and K from 5120 on: tiles of 64 x 64 where there are at most
        // 32 of them.  Measured against gemv_staged and the split 64x128 tiles, block 128, W from HBM, us at K = 8192 / 11008 / 12288:
        // 32 x 1024 7.3 -> 7.7; 32 x 2048 10.0 -> 8.8, 13.6 -> 10.0, 15.0 -> 10.4; 32 x 4096 11.8 -> 11.5, 16.5 -> 14.2, 16.3 -> 15.0;
        // 32 x 5120 17.5 -> 13.1, 25.4 -> 18.0; 32 x 8192 19.3 -> 20.3, 28.1 -> 23.0, 30.2 -> 23.2; at K = 5120 / 7168 32 x 2048 7.4 -> 8.0,
        // 9.2 -> 8.3, 32 x 4096 9.9 -> 9.6, 10.9 -> 11.1; 16 rows stay with gemv_staged: 16 x 4096 9.7 -> 11.3, 13.8 -> 13.9, 13.0 -> 14.6.
        // 64 x 1024 at K = 5120 / 7168 / 8192 9.2 -> 8.6, 11.1 -> 8.4, 11.2 -> 8.4; 64 x 2048 9.9 -> 8.6, 12.1 -> 9.4, 12.6 -> 10.0, at
        // K = 11008 14.0 -> 11.2; 40 x 2048 8.6 -> 8.4, 11.6 -> 9.0; 64 x 4096 (two runs) 12.2 -> 11.2, 15.5 -> 14.2, 14.0 -> 12.7 and 14.5 -> 15.4,
        // block 64 16.2 -> 16.4, at K = 11008 18.8 -> 19.8: not taken.
        const bool few = M <= kPanelMinRows;
        const int64_t ps_bm = M <= kPanelFewRows ? 32 : few ? 64 : 128, ps_nst = K / kStageK;
        if (block != 32 && M > (few_rows_split ? kPanelSplitFewRowsMin : kPanelMinRows) && M <= 128 && ps_nst <= kPanelSplitMaxStages &&
            (!few || ps_nst >= (ps_bm == 32 ? kPanelSplitFewRowsMinStages : kPanelSplit64RowsMinStages)) && !rest_of_cut &&
            (K / block + 1) * max_mn * 4 < kBufOut) {
            const int64_t bm = ps_bm, nst = ps_nst, bn = block == 64 && bm == 128 ? 32 : 64, t = (N + bn - 1) / bn;
            int64_t per = t > 0 && t <= kCus / 2 ? kCus / t : 0;
            if (per > kSplitMax) per = kSplitMax;
            if (per > nst / kPanelSplitMinStages) per = nst / kPanelSplitMinStages;
            const int64_t least = bm == 128 ? 2 : bm == 64 ? 4 : nst >= kPanelSplitFewRowsTwoStages ? 2 : 3;
            const bool enough = bm == 128 || (bm == 64 ? t <= kPanelSplit64RowsMaxTiles : t * per >= kPanelSplitFewRowsMinGroups);
            if (per >= least && enough) {
                const int64_t stages = (nst + per - 1) / per;
                per = (nst + stages - 1) / stages;
                const int64_t need = t * per * bm * bn * 4;
                if (per >= least && need <= ws_bytes) {
                    p.kernel = kKSplitPanel;
                    p.splits = (int)(t * per);
                    p.split_stages = (int)stages;
                    p.split_per_tile = (int)per;
                    p.ws_need = need;
                    return true;
                }
            }
        }
        if (few_rows_split) return false;          // (asked ahead of gemv_staged: only for that rule)
        // more than 128 rows, 100 to 128 square tiles (128 x 128, block 64: 128 x 64) and K from 8192 on: two pieces per tile on
        // gemm_panel's square form.  Measured against the split 256x128 tiles, block 128, W from HBM, us at K = 8192 / 11008 /
        // 16384: 512 x 4096 38.2 -> 34.0, 45.2 -> 42.7, 59.2 -> 56.4; 1024 x 2048 37.7 -> 33.1, 45.5 -> 43.7, 59.6 -> 55.7; 256 x 8192
        // 39.1 -> 35.7, 47.1 -> 47.0, 62.8 -> 60.9.  With fewer tiles and more pieces it is level with or behind the split tile
        // kernels (256 x 4096: 25.9 -> 26.5, 30.5 -> 31.7; 512 x 1024: 21.2 -> 18.4, 22.3 -> 21.3, 25.0 -> 28.7): not taken there.
        if (block != 32 && M > 128 && !rest_of_cut && K / kStageK >= kPanelSquareSplitMinStages && (K / block + 1) * max_mn * 4 < kBufOut) {
            const int64_t bn = block == 64 ? 64 : 128, t = ((M + 127) / 128) * ((N + bn - 1) / bn), nst = K / kStageK;
            if (t >= kPanelSquareSplitMinTiles && t <= kCus / 2) {
                const int64_t stages = (nst + 1) / 2, need = t * 2 * 128 * bn * 4;
                if (need <= ws_bytes) {
                    p.kernel = kKSplitPanel;
                    p.splits = (int)(t * 2);
                    p.split_stages = (int)stages;
                    p.split_per_tile = 2;
                    p.ws_need = need;
                    return true;
                }
            }
        }
        // 256x128 tiles on gemm_wide's loop, split evenly, where that puts most of the CUs to work
        if (block != 32 && M > 128 && wide_addressable(M, N, K, lda, ldw, block)) {
            const int64_t t = ((M + 255) / 256) * ((N + 127) / 128), nst = K / kStageK;
            int64_t per = t > 0 && t <= kCus / 2 ? kCus / t : 0;
            if (per > kSplitMax) per = kSplitMax;
            if (per > nst / kSplitMinStages) per = nst / kSplitMinStages;
            if (per >= 2) {
                int64_t stages = (nst + per - 1) / per;
                stages += stages & 1;              // even: a piece's padding stage (odd trip count) only at the end of K
                per = (nst + stages - 1) / stages;
                const int64_t need = t * per * 256 * 128 * 4;
                if (per >= kWideSplitMinPer && stages >= kWideSplitMinStages && t * per >= kWideSplitMinGroups && need <= ws_bytes) {
                    p.kernel = kKSplitWideHalf;
                    p.splits = (int)(t * per);
                    p.split_stages = (int)stages;
                    p.split_per_tile = (int)per;
                    p.ws_need = need;
                    return true;
                }
            }
        }
        int kind;
        const SplitGrid sg = plan_split(M, N, K, kind);
        if (sg.groups <= 1) return false;
        // one slab of a tile's size per (workgroup, tile it touches); with runs the slab indices are workgroup + tile
        const int64_t tiles = ((M + (kind ? 127 : 63)) / (kind ? 128 : 64)) * ((N + 127) / 128);
        const int64_t need = (sg.per_tile > 0 ? sg.groups : sg.groups + tiles - 1) * (kind ? 128 : 64) * 128 * 4;
        if (need > ws_bytes) return false;
        p.kernel = kind == 1 ? kKSplit128x128 : kKSplit64x128;
        p.splits = sg.groups;
        p.split_stages = sg.stages;
        p.split_per_tile = sg.per_tile;
        p.ws_need = need;
        return true;
    };
    // (the rest of a cut problem shares the whole problem's pointers and strides, which only the tile kernels take)
    if (!partials && !rest_of_cut) {
        if (M <= kRowsMax && (block == 64 || block == 128) &&
            (block == 64 ? rows_lds_bytes<64>(M, K, 0) : rows_lds_bytes<128>(M, K, 0)) <= kRowsLdsMax && (K / block + 16) * N * 4 < kBufOut) {
            // (offsets of kBufOut and beyond mark lanes that load nothing: every buffer of the kernel has to end below it)
            p.kernel = kKRows;
            return p;
        }
        // 17 ... 64 rows against a long K, given scratch memory: gemm_panel on pieces of K where the rule in try_split has it
        if (M > kPanelSplitFewRowsMin && M <= kPanelMinRows && try_split(true)) return p;
        // 33 ... 64 rows: gemm_panel on tiles of 64 rows where the columns fit one round of them and K is at most 4096 --
        // unless gemv_staged's four groups of rows apply, which are ahead from K = 1152 on (measured, 64 rows, block 128, W from
        // HBM, us, gemv_staged or the split 64x128 tiles -> gemm_panel, K = 768 / 2048 / 4096 / 8192: N = 4096 5.7 -> 4.7,
        // 6.0 -> 7.2, 10.1 -> 11.6, 16.9 -> 19.6; N = 8192 7.1 -> 5.0, 12.4 -> 7.9, 15.5 -> 13.1, 21.1 -> 23.1; N = 11008 7.5 -> 5.9,
        // 13.6 -> 10.2, 17.4 -> 16.2, 29.4 -> 28.0; N = 16384 8.0 -> 6.6, 15.5 -> 12.5, 22.4 -> 19.4, 39.4 -> 33.5).  With tiles of as few
        // 16-column subtiles as give one tile per CU, and of 32 rows where those are at most 32 columns wide (launch_panel), the
        // kernel is ahead of gemv_staged from 3072 columns on whatever K up to 4096: N = 4096 at K = 2048 / 4096, 48 rows 5.6 -> 5.4,
        // 9.4 -> 8.3, 64 rows 5.9 -> 5.4, 10.0 -> 8.5; level at N = 2048 (5.5 -> 5.4, 7.6 -> 7.7), behind at N = 1024 (7.2 -> 7.6)
        const bool staged_band = M <= kStagedWideRows && (N + 15) / 16 <= kStagedWideMaxGroups && M * K <= kStagedWideMaxCodes;
        if (M > kStagedMaxRows && M <= kPanelMinRows && (block == 64 || block == 128) && (K / block + 1) * max_mn * 4 < kBufOut) {
            const int64_t widest = 32 * panel_max_subtiles(block), nst = K / kStageK;
            if ((N + widest - 1) / widest <= kCus && nst <= kPanelMaxStages && (!staged_band || nst <= kPanelOverStagedStages || N >= kPanelOverStagedMinCols)) {
                p.kernel = kKPanel;
                return p;
            }
            panel_if_no_split = (N + widest - 1) / widest <= kCus && !staged_band;
        }
        // 3 ... 32 rows against many columns: gemm_panel on tiles of 32 rows x 64 ... 256 columns, one per CU, where gemv_staged's
        // workgroups of 16 columns run in several rounds (measured, block 128, W from HBM, us, gemv_staged -> gemm_panel at
        // K = 1024 / 4096: 16 rows N = 6144 7.2 -> 4.2, 10.4 -> 9.4; N = 11008 6.1 -> 4.7, 13.6 -> 11.9; N = 32000 13.8 -> 9.1, 31.8 -> 29.8;
        // 32 rows N = 8192 5.7 -> 4.1, 12.3 -> 11.4; N = 11008 7.8 -> 4.3, 16.4 -> 12.5; N = 16384 10.1 -> 5.0, 21.6 -> 16.3; N = 32000
        // 17.9 -> 8.1, 37.3 -> 30.0.  A tile's columns are a multiple of 16 (the tile's remaining subtiles stay empty: panel_pitch), as
        // few as give one tile per CU: N = 6144 / 8192 at K = 4096 on 192 / 256 tiles of 32 columns instead of 96 / 128 of 64: 16 rows
        // 9.9 -> 8.6, 10.5 -> 9.8; 32 rows 10.8 -> 9.0, 11.3 -> 10.2; N = 5120 (gemv_staged before) 9.2 -> 8.2, 10.9 -> 8.6; at N = 4096
        // gemv_staged stays ahead: 16 rows 6.4 -> 8.5, 32 rows 7.8 -> 8.6 at K = 4096)
        if (M > kRowsMax && M <= kPanelFewRows && N >= kPanelFewRowsMinCols && (block == 64 || block == 128) &&
            (K / block + 1) * max_mn * 4 < kBufOut && K / kStageK <= kPanelMaxStages) {
            const int64_t widest = 64 * panel_max_subtiles(block);
            if ((N + widest - 1) / widest <= kCus) {
                p.kernel = kKPanel;
                return p;
            }
        }
        const bool staged_rows = M <= kStagedMaxRows || staged_band;
        if (staged_rows && (block == 64 || block == 128) && (K / block + 16) * N * 4 < 0x3fffffffLL && 16 * ldw + K < 0x3fffffffLL &&
            128 * lda + K < 0x3fffffffLL && (K / block + 16) * M * 4 < 0x3fffffffLL) {         // (gemv_staged addresses its buffers with 32-bit offsets)
            p.kernel = kKGemv;
            return p;
        }
        // few tiles and a short K: one narrow tile per CU, no split (gemm_panel)
        if (M > kPanelMinRows && (block == 64 || block == 128) && (K / block + 1) * max_mn * 4 < kBufOut) {
            const int64_t rows = (M + 127) / 128, widest = 16 * panel_max_subtiles(block), nst = K / kStageK;
            const bool one_round = rows * ((N + widest - 1) / widest) <= kCus;
            if (one_round && nst <= kPanelMaxStages) {
                p.kernel = kKPanel;
                return p;
            }
            // more rows of tiles than that: the square form, tiles of 128 x 128 (block 64: 128 x 64), where that is one round.
            // Measured against the 128x128 tile kernel, W from HBM, us: block 128 1024 x 4096 x 1024 / 4096 / 11008 12.7 -> 11.2,
            // 33.1 -> 28.2, 74.2 -> 61.7; 256 x 11008 x 4096 27.5 -> 26.0; 1024 x 3072 x 16384 (split) 89.0 -> 74.9; block 64
            // 512 x 4096 x 768 / 4096 9.9 -> 7.1, 25.7 -> 19.4; 1024 x 2048 x 3072 22.9 -> 15.5.  With fewer than 176 tiles a split
            // of K, where the rules below find one, is level or ahead (1024 x 2176 x 8192 / 11008 / 16384, 136 tiles, against
            // the split 256x128 tiles: 41.5 -> 40.1, 50.1 -> 60.9, 68.1 -> 68.4; 160 tiles: 42.1 -> 38.3, 52.6 -> 56.7, 70.4 -> 68.9).
            if (!one_round && M > 128) {
                const int64_t bn = block == 64 ? 64 : 128, sq = rows * ((N + bn - 1) / bn);
                if (sq <= kCus && sq >= kPanelSquareMinTiles) {
                    p.kernel = kKPanel;
                    return p;
                }
                square_if_no_split = sq <= kCus;
            }
            panel_if_no_split = one_round;
        }
        if (M <= 32) {
            // (block 32) with scratch memory the split 64x128 tiles are ahead of the kernel that gathers its operands (measured
            // at block 128, 4096 -> 11008, 17 to 32 rows: 30-34 us against 17)
            if (!try_split()) p.kernel = kKSkinny;
            return p;
        }
        // 256x256 tiles when there is enough work to fill the 256 CUs with them
        const int64_t tm = (M + 255) / 256, tn = (N + 255) / 256;
        if (tm * tn >= kWideMinTiles && (block == 32 || wide_addressable(M, N, K, lda, ldw, block))) {
            p.kernel = kKWide;
            const int64_t full = (tm * tn / kCus) * kCus;             // tiles of the full rounds
            if (block != 32 && full > 0 && tm * tn > full) {
                // the largest leading part of whole tile rows (columns) within the full rounds, and what the rest costs
                int64_t best_rest = kCutMaxRest + 1;
                for (int axis = 1; axis <= 2; ++axis) {
                    const int64_t across = axis == 1 ? tn : tm, along = axis == 1 ? tm : tn;
                    const int64_t lead = full / across;                // whole rows (columns) of tiles
                    if (lead < 1 || lead >= along) continue;
                    const int64_t rest_tiles = (along - lead) * across;
                    if (rest_tiles >= best_rest) continue;
                    const int64_t rm = axis == 1 ? M - lead * 256 : M, rn = axis == 1 ? N : N - lead * 256;
                    const GemmPlan r = plan_gemm(rm, rn, K, lda, ldw, block, aligned, false, ws_bytes, true);
                    const bool tile_family = r.kernel == kKTile256x128 || r.kernel == kKWideHalf || r.kernel == kKSplitWideHalf || r.kernel == kKTile128x128 || r.kernel == kKTile64x128 ||
                                             r.kernel == kKSplit128x128 || r.kernel == kKSplit64x128;
                    if (!tile_family) continue;
                    best_rest = rest_tiles;
                    p.cut_axis = axis;
                    p.lead = lead * 256;
                    p.rest_kernel = r.kernel;
                    p.rest_splits = r.splits;
                    p.rest_split_stages = r.split_stages;
                    p.rest_split_per_tile = r.split_per_tile;
                    p.ws_need = r.ws_need;
                }
            }
            return p;
        }
    }
    // 128x128 tiles while they fit one round of workgroups on the 256 CUs; beyond that the 256x128 tile (measured
    // 25-40 % faster than two rounds of 128x128 tiles at 288-320 of them)
    const int64_t t128 = ((M + 127) / 128) * ((N + 127) / 128);
    static_assert(!TileLds<256, 128, 32, 3>::kFits && TileLds<256, 128, 64, 3>::kFits, "block 32 has no 256x128 tile: its stage ring exceeds the LDS");
    if (M > 128 && t128 > 256 && block != 32) {
        // 256x128 tiles: on gemm_wide's loop (64x64 per wave) where its 32-bit operand offsets reach, else (and for the
        // int32 partials) on the tile kernel.  Measured, bf16 out, gemm_tile 256x128 (block 64: 128x192 tiles, since
        // removed) -> gemm_wide<.., 4>: 2048 x 4096 x 4096 47.1 -> 44.8 us, 2048 x 4096 x 11008 111.8 -> 107.5, 1024 x 8192 x
        // 8192 85.4 -> 81.8; block 64: 8192 x 768 x 768 15.4 -> 14.3, 8192 x 768 x 3072 39.1 -> 37.0, 2048 x 4096 x 4096
        // 61.8 -> 54.0, 4096 x 2048 x 2048 34.8 -> 30.9; same output bits.
        p.kernel = (!partials && wide_addressable(M, N, K, lda, ldw, block)) ? kKWideHalf : kKTile256x128;
        return p;
    }
    // small grids: one workgroup per CU at best, so the tile is spread over as many waves as its shape allows
    // (measured 25-37 % faster than 2x2 waves of 64x64 at M = 96 ... 1024)
    if (try_split()) return p;
    // a long K and nothing to split it with (no scratch memory, or too little): one round of narrow tiles is still ahead of a
    // few 128x128 tiles (measured without scratch memory, block 128, us, K = 8192 / 16384: 128 x 768 45.0 -> 13.9, 88.6 -> 35.9;
    // 128 x 11008 48.7 -> 32.2, 90.3 -> 57.6; 512 x 4096 49.7 -> 34.9, 88.5 -> 63.2; 1024 x 256 at K = 32768 167 -> 53)
    if (panel_if_no_split || square_if_no_split) {     // (the square tiles: 12-18 % ahead of the 128x128 tile kernel on the same grid)
        p.kernel = kKPanel;
        return p;
    }
    // (64x128 tiles for problems of 129-255 tiles of 128x128 measured 5-10 % slower than the half-empty 128x128 grid)
    p.kernel = M > 64 ? kKTile128x128 : kKTile64x128;
    return p;
}

template <int BLK, int CDT> int launch_skinny(GemmArgs g, hipStream_t st) {
    const int64_t tn = (g.N + 31) / 32, tm = (g.M + 31) / 32;
    if (tn > 0x7fffffffLL || tm > 65535) return BI8_ERR_TOO_LARGE;
    hipLaunchKernelGGL((gemm_skinny<BLK, CDT>), dim3((unsigned)tn, (unsigned)tm), dim3(512), 0, st, g);
    return bi8_launch_rc();
}

template <int BLK, int CDT, int NW, int MT> int launch_staged_as(const GemmArgs &g, unsigned tn, hipStream_t st) {
    constexpr int lds = NW * GemvLds<MT>::kWaveBytes;
    auto kern = gemv_staged<BLK, CDT, NW, MT>;
    if (lds > 64 * 1024) {
        static LdsOptIn opted;                     // one per kernel instantiation
        const int rc = opted.ensure((const void *)kern, lds);
        if (rc != BI8_OK) return rc;
    }
    hipLaunchKernelGGL(kern, dim3(tn), dim3(NW * 64), lds, st, g);
    return bi8_launch_rc();
}
template <int BLK, int CDT> int launch_staged(const GemmArgs &g, hipStream_t st) {
    const int64_t tn = (g.N + 15) / 16;
    if (tn > 0x7fffffffLL) return BI8_ERR_TOO_LARGE;
    // eight waves per workgroup (one workgroup per CU) where that is one round of workgroups; else four: up to 16 rows three
    // workgroups of four waves share a CU, up to 32 rows (twice the A ring) two (measured, 16 rows, block 128, W from HBM, eight
    // waves -> four: N = 4112, K = 1024 / 4096 / 11008 6.7 -> 4.3, 9.6 -> 8.7, 19.5 -> 18.9 us; N = 5120 6.9 -> 4.5, 10.1 -> 9.2,
    // 21.4 -> 20.5; 32 rows N = 5120 8.9 -> 5.6, 12.7 -> 11.0, 27.0 -> 25.4)
    if (g.M <= 16) return tn <= kCus ? launch_staged_as<BLK, CDT, 8, 1>(g, (unsigned)tn, st) : launch_staged_as<BLK, CDT, 4, 1>(g, (unsigned)tn, st);
    if (g.M <= 32) return tn <= kCus ? launch_staged_as<BLK, CDT, 8, 2>(g, (unsigned)tn, st) : launch_staged_as<BLK, CDT, 4, 2>(g, (unsigned)tn, st);
    // up to 64 rows the rings of A leave room for four waves, one workgroup per CU (the plan asks for no more rows)
    if (g.M <= 64) return launch_staged_as<BLK, CDT, 4, 4>(g, (unsigned)tn, st);
    return BI8_ERR_UNSUPPORTED;
}

// gemm_panel on the narrowest tiles that give at most one per CU
template <int BLK, int CDT, int NJ, int CG, int NI = 1> int launch_panel_as(GemmArgs g, hipStream_t st) {
    using L = PanelLds<kStageK / BLK, NJ, CG, NI>;
    const int pitch = g.panel_pitch > 0 ? g.panel_pitch : L::BN;
    if (pitch > L::BN) return BI8_ERR_UNSUPPORTED;
    g.tiles_m = (int)((g.M + L::BM - 1) / L::BM);
    g.tiles_n = (int)((g.N + pitch - 1) / pitch);
    auto kern = gemm_panel<BLK, CDT, NJ, CG, false, NI>;
    static LdsOptIn opted;                         // one per kernel instantiation
    const int rc = opted.ensure((const void *)kern, L::kBytes);
    if (rc != BI8_OK) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)(g.tiles_m * g.tiles_n)), dim3(kPanelThreads), L::kBytes, st, g);
    return bi8_launch_rc();
}
template <int BLK, int CDT, int CG> int launch_panel_cg(GemmArgs g, hipStream_t st) {
    const int64_t rows = (g.M + 128 / CG - 1) / (128 / CG);                    // rows of tiles
    // the fewest 16-column subtiles per tile that give at most one tile per CU; the narrowest kernel form that holds them
    // (two or four waves side by side: the tile's last subtiles may then be empty)
    const int64_t sub = (g.N + 15) / 16, across = kCus / rows;
    const int64_t per_tile = across > 0 ? (sub + across - 1) / across : 0;
    if (per_tile < 1 || per_tile > CG * panel_max_subtiles(BLK)) return BI8_ERR_UNSUPPORTED;        // (the plan sends no other problem here)
    g.panel_pitch = (int)(16 * per_tile);
    switch ((per_tile + CG - 1) / CG) {
    case 1: return launch_panel_as<BLK, CDT, 1, CG>(g, st);
    case 2: return launch_panel_as<BLK, CDT, 2, CG>(g, st);
    case 3: return launch_panel_as<BLK, CDT, 3, CG>(g, st);
    default:
        if constexpr (panel_max_subtiles(BLK) >= 4) return launch_panel_as<BLK, CDT, 4, CG>(g, st);
        return BI8_ERR_UNSUPPORTED;
    }
}
// the split form: tiles of 128 rows x 64 columns (block 64: 32), split_per_tile pieces of split_stages stages each, then the sum
template <int BLK, int CDT, int NJ, int CG, int NI = 1> int launch_panel_split_as(GemmArgs g, hipStream_t st) {
    using L = PanelLds<kStageK / BLK, NJ, CG, NI>;
    g.tiles_m = (int)((g.M + L::BM - 1) / L::BM);
    g.tiles_n = (int)((g.N + L::BN - 1) / L::BN);
    g.tile_m0 = g.tile_n0 = 0;
    if (g.split_per_tile < 2 || g.split_per_tile > kSplitMax || (int64_t)g.tiles_m * g.tiles_n * g.split_per_tile > 2 * kCus) return BI8_ERR_UNSUPPORTED;
    auto kern = gemm_panel<BLK, BI8_F32, NJ, CG, true, NI>;
    static LdsOptIn opted;                         // one per kernel instantiation
    const int rc = opted.ensure((const void *)kern, L::kBytes);
    if (rc != BI8_OK) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)(g.tiles_m * g.tiles_n), (unsigned)g.split_per_tile), dim3(kPanelThreads), L::kBytes, st, g);
    const int rc_launch = bi8_launch_rc();
    if (rc_launch != BI8_OK) return rc_launch;
    hipLaunchKernelGGL((splitk_reduce<CDT, L::BM, L::BN>), dim3((unsigned)(g.tiles_m * g.tiles_n), L::BM / (256 / (L::BN / 4))), dim3(256), 0, st, g);
    return bi8_launch_rc();
}
// (the tiles the plan has counted: 32 rows x 64 columns up to 32 rows, 64 x 64 up to 64, 128 x 64 -- at block 64 128 x 32 -- up to
// 128, and beyond that the square form's 128 x 128, at block 64 128 x 64)
template <int BLK, int CDT> int launch_panel_split(const GemmArgs &g, hipStream_t st) {
    if (g.M <= kPanelFewRows) return launch_panel_split_as<BLK, CDT, 1, 4>(g, st);
    if (g.M <= kPanelMinRows) return launch_panel_split_as<BLK, CDT, 2, 2>(g, st);
    if (g.M > 128) return launch_panel_split_as<BLK, CDT, BLK == 64 ? 2 : 4, 2, 2>(g, st);
    return launch_panel_split_as<BLK, CDT, BLK == 64 ? 2 : 4, 1>(g, st);
}
template <int BLK, int CDT> int launch_panel(const GemmArgs &g, hipStream_t st) {
    if (g.M <= kPanelFewRows) return launch_panel_cg<BLK, CDT, 4>(g, st);
    // (more rows of narrow tiles than one round: the plan has counted the square form's)
    if (g.M > 128 && ((g.M + 127) / 128) * ((g.N + 16 * panel_max_subtiles(BLK) - 1) / (16 * panel_max_subtiles(BLK))) > kCus)
        return launch_panel_as<BLK, CDT, BLK == 64 ? 2 : 4, 2, 2>(g, st);
    if (g.M <= 64) {
        // 33 ... 64 rows: two rows of 32-row tiles where one round of them is at most 32 columns wide (a fifth less traffic into
        // LDS than one row of 64 x 16 tiles: 64 x 4096 x 4096 9.1 -> 8.5 us, 48 rows 8.7 -> 8.3; level at 8192 columns, behind beyond)
        if ((g.N + 15) / 16 <= 2 * (kCus / 2)) return launch_panel_cg<BLK, CDT, 4>(g, st);
        return launch_panel_cg<BLK, CDT, 2>(g, st);
    }
    // more than 64 rows: tiles of 64 rows where one round of them is at most 64 columns wide, else of 128 rows.  A workgroup
    // streams its tile's rows of A and of W, and what bounds these problems is that traffic: 256 tiles of 64 x 32 move a third
    // less than 256 of 128 x 16.  Measured, block 128, W from HBM, us at K = 1024 / 4096, tiles of 128 -> 64 rows: 128 x 768
    // 4.7 -> 4.2, 8.6 -> 7.8; 128 x 4096 5.1 -> 4.5, 12.4 -> 9.8; 128 x 8192 6.1 -> 5.6, 15.7 -> 15.1; 256 x 2048 5.1 -> 4.5, 9.5 -> 8.3;
    // 256 x 4096 5.8 -> 5.6, 14.2 -> 12.9; 512 x 768 5.0 -> 4.4, 9.0 -> 8.3; but 128 x 11008 (tiles of 64 x 96) 7.3 -> 8.0, 18.1 -> 19.4;
    // tiles of 32 rows: the same as 64 at up to 4096 columns, behind from there (128 x 8192 x 4096 16.5, 128 x 11008 x 4096 29.3).
    const int64_t across = kCus / ((g.M + 63) / 64);
    if (across >= 1 && ((g.N + 15) / 16 + across - 1) / across <= kPanelHalfHeightMaxSubtiles) return launch_panel_cg<BLK, CDT, 2>(g, st);
    return launch_panel_cg<BLK, CDT, 1>(g, st);
}

template <int BLK, int CDT> int launch_rows(const GemmArgs &g, hipStream_t st) {
    const int64_t tn = (g.N + 15) / 16;
    if (tn > 0x7fffffffLL) return BI8_ERR_TOO_LARGE;
    const size_t lds = rows_lds_bytes<BLK>(g.M, g.K, 0);
    // one row against a long K: six runs of every weight row in flight instead of four (11008 -> 4096: 12.6 -> 12.0 us; at
    // K = 4096, where four runs are the whole row, six measured 3 % slower, and eight spill)
    if (rows_compiled_for(g.M) == 1 && g.K >= kRowsDeepK) hipLaunchKernelGGL((gemv_rows<BLK, CDT, false, 1, 6>), dim3((unsigned)tn), dim3(256), lds, st, g, nullptr, 0);
    else if (rows_compiled_for(g.M) == 1) hipLaunchKernelGGL((gemv_rows<BLK, CDT, false, 1, 4>), dim3((unsigned)tn), dim3(256), lds, st, g, nullptr, 0);
    else hipLaunchKernelGGL((gemv_rows<BLK, CDT, false, 2, 4>), dim3((unsigned)tn), dim3(256), lds, st, g, nullptr, 0);
    return bi8_launch_rc();
}

// kernel `kernel` (with the split parameters, if it is one of the split kernels) on the rectangle `part` of the output
template <int BLK, int CDT, bool PARTIALS>
int launch_kernel(const GemmArgs &g, int kernel, int splits, int split_stages, int split_per_tile, const Part &part, hipStream_t st) {
    constexpr int kRing = 3;                       // stage buffers of the tile kernels that are not software-pipelined
    const bool whole = part.row0 == 0 && part.col0 == 0 && part.rows == g.M && part.cols == g.N;
    switch (kernel) {
    case kKTile256x128:
        if constexpr (TileLds<256, 128, BLK, kRing>::kFits)
            return launch_tile<256, 128, 4, 2, (BLK == 128 && !PARTIALS) ? 2 : kRing, BLK, CDT, PARTIALS>(g, part, st);
        break;
    case kKTile128x128: return launch_tile<128, 128, 4, 2, kRing, BLK, CDT, PARTIALS>(g, part, st);
    case kKTile64x128: return launch_tile<64, 128, 2, 2, kRing, BLK, CDT, PARTIALS>(g, part, st);
    default: break;
    }
    if constexpr (!PARTIALS) {
        if (!whole && kernel != kKWide && kernel != kKWideHalf && kernel != kKSplitWideHalf && kernel != kKSplit128x128 && kernel != kKSplit64x128)
            return BI8_ERR_UNSUPPORTED;
        switch (kernel) {
        case kKRows:
            if constexpr (BLK != 32) return launch_rows<BLK, CDT>(g, st);
            break;
        case kKGemv:
            if constexpr (BLK != 32) return launch_staged<BLK, CDT>(g, st);
            break;
        case kKSkinny: return launch_skinny<BLK, CDT>(g, st);
        case kKWide:
            // blocks 128 and 64: 16x16x64 MFMAs, 64x128 per wave; block 32 (one MFMA per K-block): 32x32x32, 32x256 per wave
            if constexpr (BLK == 32) return whole ? launch_wide32<BLK, CDT>(g, st) : BI8_ERR_UNSUPPORTED;
            else return launch_wide<BLK, CDT>(g, part, st);
        case kKWideHalf:
            if constexpr (BLK != 32) return launch_wide<BLK, CDT, 4>(g, part, st);
            break;
        case kKSplitWideHalf:
            if constexpr (BLK != 32) {
                GemmArgs gs = g;
                gs.splits = splits;
                gs.split_stages = split_stages;
                gs.split_per_tile = split_per_tile;
                const int rc = launch_wide<BLK, BI8_F32, 4, true>(gs, part, st);
                if (rc != BI8_OK) return rc;
                gs.tiles_m = (int)((part.rows + 255) / 256);
                gs.tiles_n = (int)((part.cols + 127) / 128);
                gs.tile_m0 = (int)(part.row0 / 256);
                gs.tile_n0 = (int)(part.col0 / 128);
                hipLaunchKernelGGL((splitk_reduce<CDT, 256, 128>), dim3((unsigned)(gs.tiles_m * gs.tiles_n), 32), dim3(256), 0, st, gs);
                return bi8_launch_rc();
            }
            break;
        case kKPanel:
            if constexpr (BLK != 32) {
                if (!whole) return BI8_ERR_UNSUPPORTED;
                return launch_panel<BLK, CDT>(g, st);
            }
            break;
        case kKSplitPanel:
            if constexpr (BLK != 32) {
                if (!whole) return BI8_ERR_UNSUPPORTED;
                GemmArgs gs = g;
                gs.splits = splits;
                gs.split_stages = split_stages;
                gs.split_per_tile = split_per_tile;
                return launch_panel_split<BLK, CDT>(gs, st);
            }
            break;
        case kKSplit128x128:
        case kKSplit64x128: {
            GemmArgs gs = g;
            gs.splits = splits;
            gs.split_stages = split_stages;
            gs.split_per_tile = split_per_tile;
            const bool big = kernel == kKSplit128x128;
            const int bm = big ? 128 : 64;
            const int rc = big ? launch_tile<128, 128, 4, 2, kRing, BLK, BI8_F32, false, true>(gs, part, st)
                               : launch_tile<64, 128, 2, 2, kRing, BLK, BI8_F32, false, true>(gs, part, st);
            if (rc != BI8_OK) return rc;
            gs.tiles_m = (int)((part.rows + bm - 1) / bm);
            gs.tiles_n = (int)((part.cols + 127) / 128);
            gs.tile_m0 = (int)(part.row0 / bm);
            gs.tile_n0 = (int)(part.col0 / 128);
            const dim3 grid((unsigned)(gs.tiles_m * gs.tiles_n), big ? 16 : 8);     // fewer than 256 tiles, 8 rows each
            if (big) hipLaunchKernelGGL((splitk_reduce<CDT, 128, 128>), grid, dim3(256), 0, st, gs);
            else hipLaunchKernelGGL((splitk_reduce<CDT, 64, 128>), grid, dim3(256), 0, st, gs);
            return bi8_launch_rc();
        }
        default: break;
        }
    }
    return BI8_ERR_UNSUPPORTED;                    // plan_gemm never pairs these (kernel, block)
}

template <int BLK, int CDT, bool PARTIALS> int launch_plan(const GemmArgs &g, const GemmPlan &p, hipStream_t st) {
    if (p.cut_axis == 0)
        return launch_kernel<BLK, CDT, PARTIALS>(g, p.kernel, p.splits, p.split_stages, p.split_per_tile, Part{0, 0, g.M, g.N}, st);
    const Part lead = p.cut_axis == 1 ? Part{0, 0, p.lead, g.N} : Part{0, 0, g.M, p.lead};
    const Part rest = p.cut_axis == 1 ? Part{p.lead, 0, g.M - p.lead, g.N} : Part{0, p.lead, g.M, g.N - p.lead};
    const int rc = launch_kernel<BLK, CDT, PARTIALS>(g, p.kernel, 1, 0, 0, lead, st);
    if (rc != BI8_OK) return rc;
    return launch_kernel<BLK, CDT, PARTIALS>(g, p.rest_kernel, p.rest_splits, p.rest_split_stages, p.rest_split_per_tile, rest, st);
}

template <int CDT, bool PARTIALS> int dispatch(const GemmArgs &g, int block, hipStream_t st) {
    const bool aligned = bi8_aligned(g.A, 16) && bi8_aligned(g.W, 16) && (PARTIALS || (bi8_aligned(g.sA, 4) && bi8_aligned(g.sW, 4)));
    const int64_t ws_bytes = (g.ws && bi8_aligned(g.ws, 16)) ? g.ws_bytes : 0;
    const GemmPlan p = plan_gemm(g.M, g.N, g.K, g.lda, g.ldw, block, aligned, PARTIALS, ws_bytes);
    if (p.kernel == kKGeneric) return launch_generic<CDT, PARTIALS>(g, block, st);
    switch (block) {
    case 32: return launch_plan<32, CDT, PARTIALS>(g, p, st);
    case 64: return launch_plan<64, CDT, PARTIALS>(g, p, st);
    default: return launch_plan<128, CDT, PARTIALS>(g, p, st);
    }
}

}  // namespace

extern "C" int bi8_gemm_nt_dequant_ws(const int8_t *A, const int8_t *W, const float *sA, const float *sW, const void *bias,
                                      int bias_dtype, void *C, int c_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw,
                                      int64_t ldc, int block, void *workspace, int64_t workspace_bytes, void *stream) {
    if (c_dtype < 0 || c_dtype > 2 || (bias && (bias_dtype < 0 || bias_dtype > 2))) return BI8_ERR_BAD_DTYPE;
    if (block < 1 || block > (1 << 20)) return BI8_ERR_BAD_BLOCK;
    if (M < 0 || N < 0 || K < 0 || lda < K || ldw < K || ldc < N || workspace_bytes < 0) return BI8_ERR_BAD_SHAPE;
    if (M == 0 || N == 0) return BI8_OK;
    if (!C || (K > 0 && (!A || !W || !sA || !sW))) return BI8_ERR_NULL_POINTER;
    GemmArgs g{A, W, sA, sW, bias, C, nullptr, M, N, K, lda, ldw, ldc, 0, 0, bias_dtype, (float *)workspace,
               workspace ? workspace_bytes : 0, 0, 0};
    hipStream_t st = (hipStream_t)stream;
    switch (c_dtype) {
    case BI8_F32: return dispatch<BI8_F32, false>(g, block, st);
    case BI8_BF16: return dispatch<BI8_BF16, false>(g, block, st);
    default: return dispatch<BI8_F16, false>(g, block, st);
    }
}

extern "C" int bi8_gemm_nt_dequant(const int8_t *A, const int8_t *W, const float *sA, const float *sW, const void *bias,
                                   int bias_dtype, void *C, int c_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw,
                                   int64_t ldc, int block, void *stream) {
    return bi8_gemm_nt_dequant_ws(A, W, sA, sW, bias, bias_dtype, C, c_dtype, M, N, K, lda, ldw, ldc, block, nullptr, 0, stream);
}

// ---- the entry point that allocates nothing ---------------------------------------------------------------------------
// The split of K needs scratch memory for its fp32 slabs.  bi8_gemm_nt_dequant_ws takes it from the caller;
// bi8_gemm_nt_dequant_static takes it from this array, one copy per GPU that loads the library, for callers that cannot
// allocate (HIP graph capture, serving loops, harnesses that forbid hipMalloc).  A split never wants more than
// workgroups + tiles - 1 <= 256 + 254 slabs of 128 x 128 fp32 < 32 MiB (plan_split), which is the size of the array.
constexpr int64_t kScratchBytes = 32ll << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// In host code `scratch` is only a handle for the runtime: the array's address on the current device comes from
// hipGetSymbolAddress, once per device, and is what the kernels are given.
constexpr int kMaxDevices = 64;
static std::atomic<void *> scratch_ptr[kMaxDevices];
static int scratch_of_current_device(void **out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return bi8_hip_rc(e);
    if (dev < 0 || dev >= kMaxDevices) return BI8_ERR_UNSUPPORTED;
    void *p = scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return bi8_hip_rc(e);
        if (!p) return BI8_ERR_NULL_POINTER;
        scratch_ptr[dev].store(p, std::memory_order_release);       // two threads racing here store the same address
    }
    *out = p;
    return BI8_OK;
}

extern "C" int64_t bi8_static_scratch_bytes(void) { return kScratchBytes; }


extern "C" int bi8_gemm_nt_dequant_static(const int8_t *A, const int8_t *W, const float *sA, const float *sW, const void *bias,
                                          int bias_dtype, void *C, int c_dtype, int64_t M, int64_t N, int64_t K, int64_t lda,
                                          int64_t ldw, int64_t ldc, int block, void *stream) {
    if (block < 1 || block > (1 << 20)) return BI8_ERR_BAD_BLOCK;
    if (M < 0 || N < 0 || K < 0 || lda < K || ldw < K || ldc < N) return BI8_ERR_BAD_SHAPE;
    // what the split of this problem wants, were scratch memory unlimited; more than the array holds is refused
    // rather than run differently from bi8_gemm_nt_dequant_ws
    const GemmPlan p = plan_gemm(M, N, K, lda, ldw, block, true, false, INT64_MAX);
    if (p.ws_need > kScratchBytes) return BI8_ERR_SCRATCH_TOO_SMALL;
    void *ws = nullptr;
    if (p.ws_need > 0) {
        const int rc = scratch_of_current_device(&ws);
        if (rc != BI8_OK) return rc;
    }
    return bi8_gemm_nt_dequant_ws(A, W, sA, sW, bias, bias_dtype, C, c_dtype, M, N, K, lda, ldw, ldc, block, ws, ws ? kScratchBytes : 0,
                                  stream);
}

extern "C" int64_t bi8_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int block) {
    if (M <= 0 || N <= 0 || K <= 0 || block < 1) return 0;
    const GemmPlan p = plan_gemm(M, N, K, K, K, block, true, false, INT64_MAX);
    return p.ws_need;
}

extern "C" const char *bi8_gemm_kernel_name(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw, int block,
                                            int64_t workspace_bytes) {
    if (M <= 0 || N <= 0 || K < 0 || block < 1) return "none";
    const GemmPlan p = plan_gemm(M, N, K, lda, ldw, block, true, false, workspace_bytes);
    if (p.cut_axis != 0) {                         // two launches: the 256x256 kernel, then the rest on smaller tiles
        switch (p.rest_kernel) {
        case kKTile256x128: return "gemm_wide+gemm_tile_256x128";
        case kKWideHalf: return "gemm_wide+gemm_wide_256x128";
        case kKSplitWideHalf: return "gemm_wide+gemm_wide_256x128_splitk";
        case kKTile128x128: return "gemm_wide+gemm_tile_128x128";
        case kKTile64x128: return "gemm_wide+gemm_tile_64x128";
        case kKSplit128x128: return "gemm_wide+gemm_tile_128x128_splitk";
        default: return "gemm_wide+gemm_tile_64x128_splitk";
        }
    }
    return kGemmKernelNames[p.kernel];
}

template <int DT> int launch_few_rows(const GemmArgs &g, const void *x, int64_t ldx, int block, size_t lds, hipStream_t st) {
    const unsigned tn = (unsigned)((g.N + 15) / 16);
    const int mm = rows_compiled_for(g.M);
    if (block == 64) {
        if (mm == 1 && g.K >= kRowsDeepK) hipLaunchKernelGGL((gemv_rows<64, DT, true, 1, 6>), dim3(tn), dim3(256), lds, st, g, x, ldx);
        else if (mm == 1) hipLaunchKernelGGL((gemv_rows<64, DT, true, 1, 4>), dim3(tn), dim3(256), lds, st, g, x, ldx);
        else hipLaunchKernelGGL((gemv_rows<64, DT, true, 2, 4>), dim3(tn), dim3(256), lds, st, g, x, ldx);
    } else {
        if (mm == 1 && g.K >= kRowsDeepK) hipLaunchKernelGGL((gemv_rows<128, DT, true, 1, 6>), dim3(tn), dim3(256), lds, st, g, x, ldx);
        else if (mm == 1) hipLaunchKernelGGL((gemv_rows<128, DT, true, 1, 4>), dim3(tn), dim3(256), lds, st, g, x, ldx);
        else hipLaunchKernelGGL((gemv_rows<128, DT, true, 2, 4>), dim3(tn), dim3(256), lds, st, g, x, ldx);
    }
    return bi8_launch_rc();
}

extern "C" int bi8_linear_few_rows(const void *x, int dtype, const int8_t *W, const float *sW, const void *bias, int bias_dtype,
                                   void *C, int64_t M, int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldc, int block,
                                   void *stream) {
    if (dtype < 0 || dtype > 2 || (bias && (bias_dtype < 0 || bias_dtype > 2))) return BI8_ERR_BAD_DTYPE;
    if (block < 1 || block > (1 << 20)) return BI8_ERR_BAD_BLOCK;
    if (M < 0 || N < 0 || K < 0 || ldx < K || ldw < K || ldc < N) return BI8_ERR_BAD_SHAPE;
    if (!x || !W || !sW || !C) return BI8_ERR_NULL_POINTER;
    const int64_t vec = dtype == BI8_F32 ? 4 : 8;
    if (M < 1 || M > kRowsMax || N < 1 || (block != 64 && block != 128) || K < kStageK || K % kStageK != 0 || ldx % vec != 0 ||
        ldw % 16 != 0 || ldw >= (1 << 22) || (K / block + 16) * N * 4 >= kBufOut || !bi8_aligned(x, 16) || !bi8_aligned(W, 16) ||
        !bi8_aligned(sW, 4) || (N + 15) / 16 > 0x7fffffffLL)
        return BI8_ERR_UNSUPPORTED;
    const size_t lds = block == 64 ? rows_lds_bytes<64>(M, K, bi8_dtype_size(dtype)) : rows_lds_bytes<128>(M, K, bi8_dtype_size(dtype));
    if (lds > kRowsLdsMax) return BI8_ERR_UNSUPPORTED;
    GemmArgs g{nullptr, W, nullptr, sW, bias, C, nullptr, M, N, K, 0, ldw, ldc, 0, 0, bias_dtype};
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
    case BI8_F32: return launch_few_rows<BI8_F32>(g, x, ldx, block, lds, st);
    case BI8_BF16: return launch_few_rows<BI8_BF16>(g, x, ldx, block, lds, st);
    default: return launch_few_rows<BI8_F16>(g, x, ldx, block, lds, st);
    }
}

extern "C" int bi8_gemm_nt_partials(const int8_t *A, const int8_t *W, int32_t *P, int64_t M, int64_t N, int64_t K, int64_t lda,
                                    int64_t ldw, int block, void *stream) {
    if (block < 1 || block > (1 << 20)) return BI8_ERR_BAD_BLOCK;
    if (M < 0 || N < 0 || K < 0 || lda < K || ldw < K) return BI8_ERR_BAD_SHAPE;
    if (M == 0 || N == 0 || K == 0) return BI8_OK;
    if (!A || !W || !P) return BI8_ERR_NULL_POINTER;
    GemmArgs g{A, W, nullptr, nullptr, nullptr, nullptr, P, M, N, K, lda, ldw, 0, 0, 0, 0};
    return dispatch<BI8_F32, true>(g, block, (hipStream_t)stream);
}
