// int8 GEMM with the per-K-block dequantize fused into the K loop (bi8_gemm_nt_dequant) and its int32
// block partials (bi8_gemm_nt_partials).  Replaces _int8_matmul_block64_rowwise_dequantize,
// triton_functions.py:70-139 (SPLIT_K = 1 path).
//
//   C[m,n] = cast( (1/127^2) * sum_j sA[j,m] * sW[j,n] * P_j[m,n] ),   P_j = int32 dot over K-block j
//
// Main kernel (gemm_tile): NT GEMM, both operands K-contiguous.
//   - v_mfma_i32_32x32x32_i8; one wave owns TM x TN subtiles of 32x32, int32 partial per K-block in
//     registers, converted and folded into an fp32 accumulator as soon as the block's MFMAs are issued;
//   - A and W tiles (128 bytes of K per row per stage) and the stage's scale rows go HBM -> LDS directly
//     (global_load_lds, 16 bytes per lane), two stages in flight, one barrier per stage;
//   - LDS rows are 128 bytes with the 16-byte chunk index XOR-ed with (row & 7), which makes both the
//     direct-to-LDS writes and the MFMA operand reads (ds_read_b128) conflict-free;
//   - the workgroup index is remapped so that the 32 workgroups resident on one XCD (one L2) cover a
//     compact patch of output tiles.
// Shapes the main kernel cannot take (K not a multiple of 128, rows not 16-byte aligned, other block
// sizes) go to gemm_generic: same MFMA, operands gathered straight from global memory with byte loads.
#include <type_traits>

#include "bi8_common.h"

namespace {

constexpr int kStageK = 128;       // bytes of K per LDS stage

__device__ __forceinline__ void lds_dma16(const void *gsrc, void *lds_dst) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gsrc,
                                     (__attribute__((address_space(3))) void *)lds_dst, 16, 0, 0);
}
__device__ __forceinline__ void lds_dma4(const void *gsrc, void *lds_dst) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gsrc,
                                     (__attribute__((address_space(3))) void *)lds_dst, 4, 0, 0);
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
};

__device__ __forceinline__ float load_bias(const GemmArgs &g, int64_t n) {
    if (g.bias_dtype == BI8_F32) return ((const float *)g.bias)[n];
    if (g.bias_dtype == BI8_BF16) return bi8_from_bf16_bits(((const uint16_t *)g.bias)[n]);
    return bi8_from_f16_bits(((const uint16_t *)g.bias)[n]);
}

// LDS map of gemm_tile: operand regions first, each with two stage buffers, so that every ds_read of the
// main loop is "per-lane base register + immediate".
template <int BM, int BN, int BLK> struct TileLds {
    static constexpr int NBS = kStageK / BLK;        // K-blocks per stage
    static constexpr int kABuf = BM * kStageK, kWBuf = BN * kStageK;
    static constexpr int kSABuf = NBS * BM * 4, kSWBuf = NBS * BN * 4;
    static constexpr int kAReg = 0;
    static constexpr int kWReg = kAReg + 2 * kABuf;
    static constexpr int kSAReg = kWReg + 2 * kWBuf;
    static constexpr int kSWReg = kSAReg + 2 * kSABuf;
    static constexpr int kBytes = kSWReg + 2 * kSWBuf;
};

// BM x BN output tile per workgroup, WM x WN waves (each TM x TN subtiles of 32x32), BLK = quantization block.
template <int BM, int BN, int WM, int WN, int BLK, int CDT, bool PARTIALS>
__global__ __launch_bounds__(WM *WN * 64) void gemm_tile(const GemmArgs g) {
    using L = TileLds<BM, BN, BLK>;
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

    int tile_m, tile_n;
    tile_of_workgroup(blockIdx.x, g.tiles_m, g.tiles_n, tile_m, tile_n);
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    const int nstages = (int)(g.K / kStageK);

    // ---- loader state: per-lane source pointers, advanced by one stage after every issue ----
    // wave-instruction i covers tile rows 8i .. 8i+7; lane -> (row 8i + lane/8, LDS chunk lane%8), which
    // holds source chunk (lane%8) ^ (lane/8).  Rows outside the matrix are clamped to its last row.
    const int ld_row = lane >> 3;
    const int ld_chunk = (lane & 7) ^ ld_row;
    constexpr int kAIter = BM / 8 / NW, kWIter = BN / 8 / NW;
    const int8_t *a_src[kAIter];
    const int8_t *w_src[kWIter];
#pragma unroll
    for (int it = 0; it < kAIter; ++it) {
        int64_t r = m0 + (wave + it * NW) * 8 + ld_row;
        if (r > g.M - 1) r = g.M - 1;
        a_src[it] = g.A + r * g.lda + ld_chunk * 16;
    }
#pragma unroll
    for (int it = 0; it < kWIter; ++it) {
        int64_t r = n0 + (wave + it * NW) * 8 + ld_row;
        if (r > g.N - 1) r = g.N - 1;
        w_src[it] = g.W + r * g.ldw + ld_chunk * 16;
    }
    // scale rows: 64 floats per wave instruction; instruction i -> K-block i / kSPer of the stage, and inside
    // it the first BM/64 instructions fetch sA, the rest sW
    constexpr int kSPer = BM / 64 + BN / 64;
    constexpr int kSInstr = PARTIALS ? 0 : NBS * kSPer;
    constexpr int kSIter = (kSInstr + NW - 1) / NW;
    const float *s_src[kSIter > 0 ? kSIter : 1];
    int s_dst[kSIter > 0 ? kSIter : 1];
    int64_t s_step[kSIter > 0 ? kSIter : 1];
#pragma unroll
    for (int it = 0; it < kSIter; ++it) {
        const int i = wave + it * NW;
        const int b = i / kSPer, r = i % kSPer;
        if (r < BM / 64) {
            int64_t m = m0 + r * 64 + lane;
            if (m > g.M - 1) m = g.M - 1;
            s_src[it] = g.sA + (int64_t)b * g.M + m;
            s_dst[it] = L::kSAReg + (b * BM + r * 64) * 4;
            s_step[it] = (int64_t)NBS * g.M;
        } else {
            int64_t n = n0 + (r - BM / 64) * 64 + lane;
            if (n > g.N - 1) n = g.N - 1;
            s_src[it] = g.sW + (int64_t)b * g.N + n;
            s_dst[it] = L::kSWReg + (b * BN + (r - BM / 64) * 64) * 4;
            s_step[it] = (int64_t)NBS * g.N;
        }
    }

    auto issue_stage = [&](int buf) {             // buf is wave-uniform: the LDS destinations are scalars
#pragma unroll
        for (int it = 0; it < kAIter; ++it) {
            lds_dma16(a_src[it], lds + L::kAReg + buf * L::kABuf + (wave + it * NW) * 1024);
            a_src[it] += kStageK;
        }
#pragma unroll
        for (int it = 0; it < kWIter; ++it) {
            lds_dma16(w_src[it], lds + L::kWReg + buf * L::kWBuf + (wave + it * NW) * 1024);
            w_src[it] += kStageK;
        }
#pragma unroll
        for (int it = 0; it < kSIter; ++it) {
            const int i = wave + it * NW;
            if (i < kSInstr) {
                const bool is_a = (i % kSPer) < BM / 64;
                lds_dma4(s_src[it], lds + s_dst[it] + buf * (is_a ? L::kSABuf : L::kSWBuf));
                s_src[it] += s_step[it];
            }
        }
    };

    // ---- operand fragment addresses of the buffer being computed.  Row r = ... + l32, 16-byte chunk
    // (2*ks + h) ^ (r & 7): address(ks) = base ^ (ks << 5).  One register per ks; subtile offsets are immediates.
    const int frag_sw = ((h ^ (lane & 7)) << 4);
    int a_addr[4], w_addr[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        a_addr[ks] = (L::kAReg + (wm * (BM / WM) + l32) * kStageK + frag_sw) ^ (ks << 5);
        w_addr[ks] = (L::kWReg + (wn * (BN / WN) + l32) * kStageK + frag_sw) ^ (ks << 5);
    }
    int sa_addr = L::kSAReg + (wm * (BM / WM) + 4 * h) * 4;
    int sw_addr = L::kSWReg + (wn * (BN / WN) + l32) * 4;
    int flip = 1;                                  // +1: the next stage is in buffer 1, -1: in buffer 0

    float acc[TM][TN][16];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    // The last subtile of a stage is folded into the accumulator during the first MFMAs of the NEXT stage
    // (after the barrier, while the new operands are still on their way from LDS).
    bi8_v16i pend_p = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    bi8_v4f pend_sx[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) pend_sx[i] = bi8_v4f{0.0f, 0.0f, 0.0f, 0.0f};
    float pend_sw = 0.0f;

    auto fold = [&](const bi8_v16i &pt, const bi8_v4f *sx, float sw, float *dst) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float f = (float)pt[r] * sx[r >> 2][r & 3];
            dst[r] = __builtin_fmaf(f, sw, dst[r]);
        }
    };

    // One stage = NBS K-blocks x NSUB subtiles ("items").  The MFMAs of item t are issued before the fp32
    // fold of item t-1, so the matrix pipe works while the vector ALU converts and accumulates.
    auto compute_stage = [&](int s) {
        bi8_v4i af[TM][4], wf[TN][4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
            for (int a = 0; a < TM; ++a) af[a][ks] = *(const bi8_v4i *)(lds + a_addr[ks] + a * 32 * kStageK);
#pragma unroll
            for (int b = 0; b < TN; ++b) wf[b][ks] = *(const bi8_v4i *)(lds + w_addr[ks] + b * 32 * kStageK);
        }
        float swv[2][TN];
        bi8_v4f sxv[2][TM][4];
        auto load_scales = [&](int blk) {
#pragma unroll
            for (int b = 0; b < TN; ++b) swv[blk & 1][b] = *(const float *)(lds + sw_addr + (blk * BN + b * 32) * 4);
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int i = 0; i < 4; ++i) sxv[blk & 1][a][i] = *(const bi8_v4f *)(lds + sa_addr + (blk * BM + a * 32 + 8 * i) * 4);
        };
        auto chain = [&](int t) {
            const int blk = t / NSUB, a = (t % NSUB) / TN, b = t % TN;
            bi8_v16i acc_i = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int ks = 0; ks < KSB; ++ks)
                acc_i = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[a][blk * KSB + ks], wf[b][blk * KSB + ks], acc_i, 0, 0, 0);
            return acc_i;
        };
        constexpr int NITEM = NBS * NSUB;
        if constexpr (PARTIALS) {
#pragma unroll
            for (int t = 0; t < NITEM; ++t) {
                const int blk = t / NSUB, a = (t % NSUB) / TN, b = t % TN;
                const bi8_v16i pt = chain(t);
                const int64_t jb = (int64_t)s * NBS + blk;
                const int64_t n = n0 + wn * (BN / WN) + b * 32 + l32;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t m = m0 + wm * (BM / WM) + a * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                    if (m < g.M && n < g.N) g.P[(jb * g.M + m) * g.N + n] = pt[r];
                }
            }
        } else {
            bi8_v16i p[2];
#pragma unroll
            for (int t = 0; t < NITEM; ++t) {
                const int blk = t / NSUB;
                if (t % NSUB == 0) load_scales(blk);
                p[t & 1] = chain(t);
                if (t == 0) {
                    fold(pend_p, pend_sx, pend_sw, acc[TM - 1][TN - 1]);
                } else {
                    const int u = t - 1, ub = u / NSUB, ua = (u % NSUB) / TN, un = u % TN;
                    fold(p[u & 1], sxv[ub & 1][ua], swv[ub & 1][un], acc[ua][un]);
                }
#pragma unroll
                for (int ks = 0; ks < KSB; ++ks) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);              // one MFMA of item t
                    __builtin_amdgcn_sched_group_barrier(0x002, 48 / KSB, 0);       // a slice of item t-1's fold
                }
            }
            pend_p = p[(NITEM - 1) & 1];
#pragma unroll
            for (int i = 0; i < 4; ++i) pend_sx[i] = sxv[(NBS - 1) & 1][TM - 1][i];
            pend_sw = swv[(NBS - 1) & 1][TN - 1];
        }
        // point the fragment addresses at the other buffer
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            a_addr[ks] += flip * L::kABuf;
            w_addr[ks] += flip * L::kWBuf;
        }
        sa_addr += flip * L::kSABuf;
        sw_addr += flip * L::kSWBuf;
        flip = -flip;
    };

    issue_stage(0);
    int fill = 1;
    for (int s = 0; s + 1 < nstages; ++s) {
        __builtin_amdgcn_s_waitcnt(0x0F70);        // vmcnt(0): this wave's direct-to-LDS loads have landed
        __syncthreads();                           // ... and everyone's; the other buffer is free again
        issue_stage(fill);
        fill ^= 1;
        compute_stage(s);
    }
    if (nstages > 0) {
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        compute_stage(nstages - 1);
    }
    if constexpr (!PARTIALS) fold(pend_p, pend_sx, pend_sw, acc[TM - 1][TN - 1]);

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
                    if (n_ok && m < g.M) store_c<CDT>(g.C, m * g.ldc + n, acc[a][b][r] * div, has_bias, bias);
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

template <int BM, int BN, int WM, int WN, int BLK, int CDT, bool PARTIALS>
int launch_tile(GemmArgs g, hipStream_t st) {
    constexpr int kLds = TileLds<BM, BN, BLK>::kBytes;
    const int64_t tm = (g.M + BM - 1) / BM, tn = (g.N + BN - 1) / BN;
    if (tm * tn > 0x7fffffffLL) return BI8_ERR_TOO_LARGE;
    g.tiles_m = (int)tm;
    g.tiles_n = (int)tn;
    auto kern = gemm_tile<BM, BN, WM, WN, BLK, CDT, PARTIALS>;
    if (kLds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
        if (e != hipSuccess) return bi8_hip_rc(e);
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)(tm * tn)), dim3(WM * WN * 64), kLds, st, g);
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

// tile shape by problem shape: the big tile when there is enough work to fill 256 CUs with it
template <int BLK, int CDT, bool PARTIALS> int pick_tile(const GemmArgs &g, hipStream_t st) {
#ifdef BI8_FORCE_TILE
    if (BI8_FORCE_TILE == 0) return launch_tile<256, 128, 4, 2, BLK, CDT, PARTIALS>(g, st);
    if (BI8_FORCE_TILE == 1) return launch_tile<128, 128, 2, 2, BLK, CDT, PARTIALS>(g, st);
    if (BI8_FORCE_TILE == 2) return launch_tile<64, 128, 1, 2, BLK, CDT, PARTIALS>(g, st);
#endif
    const int64_t big = ((g.M + 255) / 256) * ((g.N + 127) / 128);
    if (g.M > 128 && big >= 192) return launch_tile<256, 128, 4, 2, BLK, CDT, PARTIALS>(g, st);
    if (g.M > 64) return launch_tile<128, 128, 2, 2, BLK, CDT, PARTIALS>(g, st);
    return launch_tile<64, 128, 1, 2, BLK, CDT, PARTIALS>(g, st);
}

template <int CDT, bool PARTIALS> int dispatch(const GemmArgs &g, int block, hipStream_t st) {
    const bool tile_ok = g.K % kStageK == 0 && g.lda % 16 == 0 && g.ldw % 16 == 0 && bi8_aligned(g.A, 16) && bi8_aligned(g.W, 16) &&
                         (PARTIALS || (bi8_aligned(g.sA, 4) && bi8_aligned(g.sW, 4)));
    if (tile_ok) {
        switch (block) {
        case 32: return pick_tile<32, CDT, PARTIALS>(g, st);
        case 64: return pick_tile<64, CDT, PARTIALS>(g, st);
        case 128: return pick_tile<128, CDT, PARTIALS>(g, st);
        }
    }
    return launch_generic<CDT, PARTIALS>(g, block, st);
}

}  // namespace

extern "C" int bi8_gemm_nt_dequant(const int8_t *A, const int8_t *W, const float *sA, const float *sW, const void *bias,
                                   int bias_dtype, void *C, int c_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldw,
                                   int64_t ldc, int block, void *stream) {
    if (c_dtype < 0 || c_dtype > 2 || (bias && (bias_dtype < 0 || bias_dtype > 2))) return BI8_ERR_BAD_DTYPE;
    if (block < 1 || block > (1 << 20)) return BI8_ERR_BAD_BLOCK;
    if (M < 0 || N < 0 || K < 0 || lda < K || ldw < K || ldc < N) return BI8_ERR_BAD_SHAPE;
    if (M == 0 || N == 0) return BI8_OK;
    if (!C || (K > 0 && (!A || !W || !sA || !sW))) return BI8_ERR_NULL_POINTER;
    GemmArgs g{A, W, sA, sW, bias, C, nullptr, M, N, K, lda, ldw, ldc, 0, 0, bias_dtype};
    hipStream_t st = (hipStream_t)stream;
    switch (c_dtype) {
    case BI8_F32: return dispatch<BI8_F32, false>(g, block, st);
    case BI8_BF16: return dispatch<BI8_BF16, false>(g, block, st);
    default: return dispatch<BI8_F16, false>(g, block, st);
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
