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

// BM x BN output tile per workgroup, WM x WN waves, BLK = quantization block (32, 64 or 128).
template <int BM, int BN, int WM, int WN, int BLK, int CDT, bool PARTIALS>
__global__ __launch_bounds__(WM *WN * 64) void gemm_tile(const GemmArgs g) {
    constexpr int NW = WM * WN;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int NBS = kStageK / BLK;             // K-blocks per stage
    constexpr int KSB = BLK / 32;                  // MFMA k-steps per K-block
    constexpr int kAOff = 0;
    constexpr int kWOff = BM * kStageK;
    constexpr int kSAOff = (BM + BN) * kStageK;
    constexpr int kSWOff = kSAOff + NBS * BM * 4;
    constexpr int kStageBytes = kSWOff + NBS * BN * 4;
    static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "wave tiling");
    static_assert(BM % 64 == 0 && BN % 64 == 0, "scale rows are loaded 64 floats per wave instruction");

    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int l32 = lane & 31, h = lane >> 5;

    int tile_m, tile_n;
    tile_of_workgroup(blockIdx.x, g.tiles_m, g.tiles_n, tile_m, tile_n);
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    const int nstages = (int)(g.K / kStageK);
    const int64_t nblk = g.K / BLK;

    // ---- loader: this lane's source rows (clamped into the matrix) and swizzled source chunk ----
    // wave-instruction i covers tile rows 8i .. 8i+7; lane -> (row 8i + lane/8, LDS chunk lane%8),
    // which holds source chunk (lane%8) ^ (lane/8).
    const int ld_row = lane >> 3;
    const int ld_chunk = (lane & 7) ^ ld_row;
    constexpr int kAInstr = BM / 8, kWInstr = BN / 8;
    constexpr int kAIter = (kAInstr + NW - 1) / NW, kWIter = (kWInstr + NW - 1) / NW;
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
    // scale rows: 64 floats per wave instruction; instruction i < BM/64 -> sA, else sW (per K-block of the stage)
    constexpr int kSAInstr = BM / 64, kSWInstr = BN / 64;
    int64_t sa_col = m0 + lane, sw_col = n0 + lane;

    auto issue_stage = [&](int s, int buf) {
        uint8_t *base = lds + buf * kStageBytes;
        const int64_t k0 = (int64_t)s * kStageK;
#pragma unroll
        for (int it = 0; it < kAIter; ++it) {
            const int i = wave + it * NW;
            if (kAInstr % NW == 0 || i < kAInstr) lds_dma16(a_src[it] + k0, base + kAOff + i * 1024);
        }
#pragma unroll
        for (int it = 0; it < kWIter; ++it) {
            const int i = wave + it * NW;
            if (kWInstr % NW == 0 || i < kWInstr) lds_dma16(w_src[it] + k0, base + kWOff + i * 1024);
        }
        if constexpr (!PARTIALS) {
            constexpr int kSInstr = NBS * (kSAInstr + kSWInstr);
#pragma unroll
            for (int it = 0; it < (kSInstr + NW - 1) / NW; ++it) {
                const int i = wave + it * NW;
                if (i < kSInstr) {
                    const int b = i / (kSAInstr + kSWInstr);
                    const int r = i % (kSAInstr + kSWInstr);
                    const int64_t jb = (int64_t)s * NBS + b;
                    if (r < kSAInstr) {
                        int64_t m = sa_col + r * 64;
                        if (m > g.M - 1) m = g.M - 1;
                        lds_dma4(g.sA + jb * g.M + m, base + kSAOff + (b * BM + r * 64) * 4);
                    } else {
                        int64_t n = sw_col + (r - kSAInstr) * 64;
                        if (n > g.N - 1) n = g.N - 1;
                        lds_dma4(g.sW + jb * g.N + n, base + kSWOff + (b * BN + (r - kSAInstr) * 64) * 4);
                    }
                }
            }
        }
    };

    // ---- operand fragment addresses: row r = ... + l32, chunk (2*ks + h) ^ (r & 7) ----
    const int frag_sw = ((h ^ (lane & 7)) << 4);
    const int a_frag = kAOff + (wm * (BM / WM) + l32) * kStageK + frag_sw;
    const int w_frag = kWOff + (wn * (BN / WN) + l32) * kStageK + frag_sw;
    const int sa_frag = kSAOff + (wm * (BM / WM) + 4 * h) * 4;
    const int sw_frag = kSWOff + (wn * (BN / WN) + l32) * 4;

    float acc[TM][TN][16];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    auto compute_stage = [&](int s, int buf) {
        const uint8_t *base = lds + buf * kStageBytes;
        bi8_v4i af[TM][4], wf[TN][4];
#pragma unroll
        for (int a = 0; a < TM; ++a)
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) af[a][ks] = *(const bi8_v4i *)(base + ((a_frag + a * 32 * kStageK) ^ (ks << 5)));
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) wf[b][ks] = *(const bi8_v4i *)(base + ((w_frag + b * 32 * kStageK) ^ (ks << 5)));

#pragma unroll
        for (int blk = 0; blk < NBS; ++blk) {
            float swv[TN];
            if constexpr (!PARTIALS) {
#pragma unroll
                for (int b = 0; b < TN; ++b) swv[b] = *(const float *)(base + sw_frag + (blk * BN + b * 32) * 4);
            }
#pragma unroll
            for (int a = 0; a < TM; ++a) {
                bi8_v4f sxv[4];
                if constexpr (!PARTIALS) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) sxv[i] = *(const bi8_v4f *)(base + sa_frag + (blk * BM + a * 32 + 8 * i) * 4);
                }
#pragma unroll
                for (int b = 0; b < TN; ++b) {
                    bi8_v16i p = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                    for (int ks = 0; ks < KSB; ++ks)
                        p = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[a][blk * KSB + ks], wf[b][blk * KSB + ks], p, 0, 0, 0);
                    if constexpr (PARTIALS) {
                        const int64_t jb = (int64_t)s * NBS + blk;
                        const int64_t n = n0 + wn * (BN / WN) + b * 32 + l32;
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const int64_t m = m0 + wm * (BM / WM) + a * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                            if (m < g.M && n < g.N) g.P[(jb * g.M + m) * g.N + n] = p[r];
                        }
                    } else {
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const float t = (float)p[r] * sxv[r >> 2][r & 3];
                            acc[a][b][r] = __builtin_fmaf(t, swv[b], acc[a][b][r]);
                        }
                    }
                }
            }
        }
    };

    issue_stage(0, 0);
    for (int s = 0; s < nstages; ++s) {
        __builtin_amdgcn_s_waitcnt(0x0F70);        // vmcnt(0): this wave's direct-to-LDS loads have landed
        __syncthreads();                           // ... and everyone's; the other buffer is free again
        if (s + 1 < nstages) issue_stage(s + 1, (s + 1) & 1);
        compute_stage(s, s & 1);
    }
    (void)nblk;

    if constexpr (!PARTIALS) {
        const float div = (float)(1.0 / (127.0 * 127.0));
#pragma unroll
        for (int b = 0; b < TN; ++b) {
            const int64_t n = n0 + wn * (BN / WN) + b * 32 + l32;
            const bool n_ok = n < g.N;
            const bool has_bias = g.bias != nullptr;
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
    constexpr int NBS = kStageK / BLK;
    constexpr int kStageBytes = (BM + BN) * kStageK + NBS * (BM + BN) * 4;
    constexpr int kLds = 2 * kStageBytes;
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
    const int64_t big = ((g.M + 255) / 256) * ((g.N + 255) / 256);
    if (g.M > 128 && big >= 192) return launch_tile<256, 256, 4, 2, BLK, CDT, PARTIALS>(g, st);
    if (g.M > 64) return launch_tile<128, 128, 2, 2, BLK, CDT, PARTIALS>(g, st);
    return launch_tile<64, 128, 1, 4, BLK, CDT, PARTIALS>(g, st);
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
