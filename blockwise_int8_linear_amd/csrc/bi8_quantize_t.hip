// Block quantize of the transpose (bi8_quantize_transposed): x [R,C] -> codes [C,R], scales [ceil(R/B), C],
// blocks running down the columns of x.  The backward pass of the reference materializes x.t().contiguous()
// and then calls the row quantizer (block_linear.py:93-94, :100-103): two extra full passes over HBM.
// Here a workgroup reads a 128-row x 64-column tile once with 128-bit row loads (the next tile's loads already in
// flight while this one is processed), keeps it in LDS in its own type (16 bytes per store), reduces and quantizes
// down the columns one 32-bit word at a time (two columns of a 16-bit type), transposes the codes through LDS
// (16 bytes per access on both sides) and writes them as 128-byte runs of the output rows.  The kernel is bound by
// the number of LDS instructions, not by arithmetic.  Results are identical to the two-step form.
#include "bi8_common.h"

namespace {

constexpr int kTR = 128;           // tile rows (source rows = output columns)
constexpr int kTC = 64;            // tile columns (source columns = output rows)
constexpr int kThreads = 256;
// Tile order: the tiles in flight at one time (a few hundred) should form a compact patch of the matrix, so that both
// the reads (runs along the source rows) and the writes (runs along the output rows = down the source columns) of
// the patch are long contiguous runs in memory.  Bands of kSBR tile rows, inside a band chunks of kSBC tile columns,
// inside a chunk row by row.
// Measured on bf16 [8192,8192]: 16 x 32 tiles (2048 rows x 2048 columns) 42 us against 45 us row by row; 8 x 64, 32 x 16,
// 16 x 16 and 16 x 64 are in between.
constexpr int kSBR = 16, kSBC = 32;
__device__ __forceinline__ void tile_coords(int64_t t, int64_t tiles_r, int64_t tiles_c, int64_t &tr, int64_t &tc) {
    const int64_t band = t / (kSBR * tiles_c);
    const int64_t rows_b = (tiles_r - band * kSBR < kSBR) ? (tiles_r - band * kSBR) : kSBR;
    const int64_t in = t - band * kSBR * tiles_c;
    const int64_t chunk = in / (rows_b * kSBC);
    const int64_t wc = (tiles_c - chunk * kSBC < kSBC) ? (tiles_c - chunk * kSBC) : kSBC;
    const int64_t in2 = in - chunk * rows_b * kSBC;
    tr = band * kSBR + in2 / wc;
    tc = chunk * kSBC + in2 % wc;
}
constexpr int kQPitch = kTR + 16;  // code tile pitch in bytes: rows stay 16-byte aligned

// B in {32, 64, 128}: a thread owns one 32-bit word column of the tile (one fp32 column, two 16-bit columns) over
// 32 or 16 consecutive source rows: 32 elements either way.
// VLOAD: the source rows are 16-byte aligned and C is a multiple of the elements per 16 bytes; without it whole
// chunks are read with unaligned 16-byte loads and the last, partial chunk of a row element by element.  VSTORE: the
// output rows are 16-byte aligned, so a lane stores 16 codes at a time; without it the code tile is written byte by
// byte (64 consecutive bytes per wave instruction).  Odd leading dimensions such as the GPT-2 vocabulary, 50257.
template <int DT, int B, bool VLOAD, bool VSTORE>
__global__ __launch_bounds__(kThreads) void quantize_cols_tile(const void *__restrict__ x, int8_t *__restrict__ qT,
                                                               float *__restrict__ scalesT, int64_t R, int64_t C,
                                                               int64_t ldx, int64_t ldq, int64_t tiles_c, int64_t ntiles) {
    constexpr int VEC = Bi8Vec<DT>::kElems;
    constexpr int64_t ES = 16 / VEC;
    constexpr int LPR = kTC / VEC;                 // lanes per tile row
    constexpr int RPP = kThreads / LPR;            // rows per load pass
    constexpr int NCORR = (DT == BI8_F32) ? 2 : 1;
    constexpr int ESZ = (int)ES;                   // bytes per element
    constexpr int CPT = 4 / ESZ;                   // columns per thread in the column walk: one 32-bit word
    constexpr int G = kThreads / (kTC / CPT);      // row groups: 4 (fp32) or 8
    constexpr int RPT = kTR / G;                   // rows per thread: 32 (fp32) or 16
    constexpr int GPW = B / RPT;                   // row groups per block
    // row pitch in bytes, 16-byte aligned: fp32 rows are 64 words, so a wave's 64 word columns cover the 64 banks;
    // 16-bit rows are 32 words + 4, a wave reads two rows 16 apart (half the banks shared: two passes)
    constexpr int kXPitch = kTC * ESZ + (ESZ == 4 ? 0 : 16);
    __shared__ __attribute__((aligned(16))) uint8_t s_x[kTR * kXPitch];
    __shared__ float s_max[G][kTC];
    __shared__ __attribute__((aligned(16))) uint8_t s_q[kTC * kQPitch];

    const int tid = threadIdx.x;
    const char *xb = (const char *)x;
    constexpr int NP = kTR / RPP;                  // 16-byte loads per thread per tile

    // A workgroup walks tiles blockIdx.x, blockIdx.x + gridDim.x, ...; the loads of the next tile are issued before
    // the current one is processed, so every workgroup has global loads in flight all the time.
    const int64_t tiles_r = (R + kTR - 1) / kTR;
    auto load_tile = [&](int64_t tile, bi8_v4u *raw) {
        int64_t tr = 0, tc = 0;
        if (tile < ntiles) tile_coords(tile, tiles_r, tiles_c, tr, tc);
        const int64_t r0 = tr * kTR;
        const int64_t c0 = tc * kTC;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int r = p * RPP + tid / LPR;
            const int cc = (tid % LPR) * VEC;
            raw[p] = bi8_v4u{0u, 0u, 0u, 0u};
            if (tile < ntiles && r0 + r < R && c0 + cc < C) {
                const char *src = xb + ((r0 + r) * ldx + c0 + cc) * ES;
                if constexpr (VLOAD) {
                    raw[p] = __builtin_nontemporal_load((const bi8_v4u *)src);
                } else if (c0 + cc + VEC <= C) {
                    raw[p] = *(const bi8_v4u_unaligned *)src;
                } else {                           // the row ends inside this chunk
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        if (c0 + cc + e < C) {
                            if constexpr (DT == BI8_F32) raw[p][e] = ((const uint32_t *)src)[e];
                            else raw[p][e >> 1] |= (uint32_t)((const uint16_t *)src)[e] << (16 * (e & 1));
                        }
                    }
                }
            }
        }
    };
    bi8_v4u raw[NP];
    load_tile(blockIdx.x, raw);
    for (int64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        int64_t tr, tc;
        tile_coords(tile, tiles_r, tiles_c, tr, tc);
        const int64_t r0 = tr * kTR;
        const int64_t c0 = tc * kTC;

        // phase 1: rows of the tile -> LDS as they are; then start the next tile's loads
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int r = p * RPP + tid / LPR;
            *(bi8_v4u *)&s_x[r * kXPitch + (tid % LPR) * 16] = raw[p];
        }
        load_tile(tile + gridDim.x, raw);
        __syncthreads();

        // phase 2: column maxima over this thread's rows, then over the block's row groups
        const int cw = tid % (kTC / CPT);          // word column
        const int g = tid / (kTC / CPT);           // row group
        float v[CPT][RPT];
        float m[CPT];
        bool special = false;
#pragma unroll
        for (int k = 0; k < CPT; ++k) m[k] = 0.0f;
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            const uint32_t d = *(const uint32_t *)&s_x[(g * RPT + i) * kXPitch + cw * 4];
            if constexpr (DT == BI8_F32) {
                v[0][i] = bi8_u2f(d);
            } else if constexpr (DT == BI8_BF16) {
                v[0][i] = bi8_u2f(d << 16);
                v[1][i] = bi8_u2f(d & 0xffff0000u);
            } else {
                v[0][i] = bi8_from_f16_bits(d & 0xffffu);
                v[1][i] = bi8_from_f16_bits(d >> 16);
            }
#pragma unroll
            for (int k = 0; k < CPT; ++k) {
                m[k] = __builtin_fmaxf(m[k], __builtin_fabsf(v[k][i]));
                special |= (v[k][i] != v[k][i]);
            }
        }
        if constexpr (GPW > 1) {
#pragma unroll
            for (int k = 0; k < CPT; ++k) s_max[g][cw * CPT + k] = m[k];
            __syncthreads();
            const int gb = g & ~(GPW - 1);
#pragma unroll
            for (int q = 0; q < GPW; ++q)
#pragma unroll
                for (int k = 0; k < CPT; ++k) m[k] = __builtin_fmaxf(m[k], s_max[gb + q][cw * CPT + k]);
        }
        if ((g & (GPW - 1)) == 0) {
            const int64_t jb = (r0 + g * RPT) / B;
#pragma unroll
            for (int k = 0; k < CPT; ++k)
                if (r0 + g * RPT < R && c0 + cw * CPT + k < C) scalesT[jb * C + c0 + cw * CPT + k] = m[k];
        }

        // phase 3: codes of this thread's rows -> byte tile [column][row], 16 bytes per store
#pragma unroll
        for (int k = 0; k < CPT; ++k) {
            uint32_t code[RPT];
            if (__builtin_expect(special || !bi8_scale_is_ordinary(m[k]), 0)) {
#pragma unroll
                for (int i = 0; i < RPT; ++i) code[i] = bi8_code_slow(v[k][i], m[k]);
            } else {
                const float y = 1.0f / m[k];
#pragma unroll
                for (int i = 0; i < RPT; ++i) code[i] = bi8_code_fast<NCORR>(v[k][i], m[k], y);
            }
#pragma unroll
            for (int i = 0; i < RPT / 16; ++i) {
                bi8_v4u w;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    w[e] = bi8_pack4(code[16 * i + 4 * e], code[16 * i + 4 * e + 1], code[16 * i + 4 * e + 2], code[16 * i + 4 * e + 3]);
                *(bi8_v4u *)&s_q[(cw * CPT + k) * kQPitch + g * RPT + 16 * i] = w;
            }
        }
        __syncthreads();

        // phase 4: 16 codes per lane, 8 lanes per output row.  The next iteration's writes to s_x come after this
        // barrier (all column reads are done), its writes to s_q after its own first barrier (all reads below are done).
        if constexpr (!VSTORE) {
            // byte e = tid + 256 * k of the code tile [64 output rows][128]: 64 consecutive bytes per wave instruction
#pragma unroll 4
            for (int k = 0; k < (kTC * kTR) / kThreads; ++k) {
                const int e = tid + kThreads * k;
                const int oc = e / kTR, ob = e % kTR;
                const int64_t orow = c0 + oc, ocol = r0 + ob;
                if (orow < C && ocol < R) qT[orow * ldq + ocol] = (int8_t)s_q[oc * kQPitch + ob];
            }
        } else
#pragma unroll
        for (int p = 0; p < (kTC * kTR / 16) / kThreads; ++p) {
            const int idx = p * kThreads + tid;
            const int oc = idx / (kTR / 16);       // output row inside the tile = source column
            const int seg = idx % (kTR / 16);
            const int64_t orow = c0 + oc;
            const int64_t ocol = r0 + seg * 16;
            if (orow < C && ocol < R) {
                const bi8_v4u w = *(const bi8_v4u *)&s_q[oc * kQPitch + seg * 16];
                int8_t *dst = qT + orow * ldq + ocol;
                if (ocol + 16 <= R) {
                    *(bi8_v4u *)dst = w;
                } else {
                    for (int e = 0; e < (int)(R - ocol); ++e) dst[e] = (int8_t)((w[e >> 2] >> (8 * (e & 3))) & 0xffu);
                }
            }
        }
    }
}

// Any block size / alignment: one thread per (output row, block); consecutive threads read consecutive columns.
template <int DT>
__global__ __launch_bounds__(kThreads) void quantize_cols_generic(const void *__restrict__ x, int8_t *__restrict__ qT,
                                                                  float *__restrict__ scalesT, int64_t R, int64_t C,
                                                                  int64_t ldx, int64_t ldq, int64_t nblk, int block) {
    const int64_t units = C * nblk;
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    for (int64_t u = (int64_t)blockIdx.x * kThreads + threadIdx.x; u < units; u += stride) {
        const int64_t j = u / C, c = u % C;
        const int64_t ra = j * block;
        const int64_t n = (R - ra < block) ? (R - ra) : block;
        float m = 0.0f;
        for (int64_t i = 0; i < n; ++i) m = __builtin_fmaxf(m, __builtin_fabsf(bi8_load_elem<DT>(x, (ra + i) * ldx + c)));
        scalesT[j * C + c] = m;
        for (int64_t i = 0; i < n; ++i)
            qT[c * ldq + ra + i] = (int8_t)(bi8_code_slow(bi8_load_elem<DT>(x, (ra + i) * ldx + c), m) & 0xffu);
    }
}

template <int DT, int B, bool VLOAD, bool VSTORE>
int launch_tile(const void *x, int8_t *qT, float *scalesT, int64_t R, int64_t C, int64_t ldx, int64_t ldq, hipStream_t st) {
    const int64_t tiles_c = (C + kTC - 1) / kTC;
    const int64_t tiles_r = (R + kTR - 1) / kTR;
    const int64_t ntiles = tiles_c * tiles_r;
    // three workgroups per CU (fp32 tiles take 42 KiB of LDS each; 16-bit tiles would fit four or five, measured
    // slower); more tiles than that are walked by resident workgroups
    const int64_t resident = 3 * 256;
    const int64_t grid = ntiles < resident ? ntiles : resident;
    hipLaunchKernelGGL((quantize_cols_tile<DT, B, VLOAD, VSTORE>), dim3((unsigned)grid), dim3(kThreads), 0, st, x, qT, scalesT, R, C,
                       ldx, ldq, tiles_c, ntiles);
    return bi8_launch_rc();
}

template <int DT, int B>
int launch_tile_any(const void *x, int8_t *qT, float *scalesT, int64_t R, int64_t C, int64_t ldx, int64_t ldq, hipStream_t st) {
    constexpr int VEC = Bi8Vec<DT>::kElems;
    const bool vload = C % VEC == 0 && ldx % VEC == 0 && bi8_aligned(x, 16);
    const bool vstore = ldq % 16 == 0 && bi8_aligned(qT, 16);
    if (vload && vstore) return launch_tile<DT, B, true, true>(x, qT, scalesT, R, C, ldx, ldq, st);
    if (vload) return launch_tile<DT, B, true, false>(x, qT, scalesT, R, C, ldx, ldq, st);
    if (vstore) return launch_tile<DT, B, false, true>(x, qT, scalesT, R, C, ldx, ldq, st);
    return launch_tile<DT, B, false, false>(x, qT, scalesT, R, C, ldx, ldq, st);
}

template <int DT>
int dispatch(const void *x, int8_t *qT, float *scalesT, int64_t R, int64_t C, int64_t ldx, int64_t ldq, int block, hipStream_t st) {
    switch (block) {
    case 32: return launch_tile_any<DT, 32>(x, qT, scalesT, R, C, ldx, ldq, st);
    case 64: return launch_tile_any<DT, 64>(x, qT, scalesT, R, C, ldx, ldq, st);
    case 128: return launch_tile_any<DT, 128>(x, qT, scalesT, R, C, ldx, ldq, st);
    }
    const int64_t nblk = (R + block - 1) / block;
    int64_t grid = (C * nblk + kThreads - 1) / kThreads;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL((quantize_cols_generic<DT>), dim3((unsigned)grid), dim3(kThreads), 0, st, x, qT, scalesT, R, C, ldx, ldq, nblk,
                       block);
    return bi8_launch_rc();
}

}  // namespace

extern "C" int bi8_quantize_transposed(const void *x, int x_dtype, int8_t *qT, float *scalesT, int64_t R, int64_t C, int64_t ldx,
                                       int64_t ldq, int block, void *stream) {
    if (x_dtype < 0 || x_dtype > 2) return BI8_ERR_BAD_DTYPE;
    if (block < 1 || block > (1 << 20)) return BI8_ERR_BAD_BLOCK;
    if (R < 0 || C < 0 || ldx < C || ldq < R) return BI8_ERR_BAD_SHAPE;
    if (R == 0 || C == 0) return BI8_OK;
    if (!x || !qT || !scalesT) return BI8_ERR_NULL_POINTER;
    hipStream_t st = (hipStream_t)stream;
    switch (x_dtype) {
    case BI8_F32: return dispatch<BI8_F32>(x, qT, scalesT, R, C, ldx, ldq, block, st);
    case BI8_BF16: return dispatch<BI8_BF16>(x, qT, scalesT, R, C, ldx, ldq, block, st);
    default: return dispatch<BI8_F16>(x, qT, scalesT, R, C, ldx, ldq, block, st);
    }
}
