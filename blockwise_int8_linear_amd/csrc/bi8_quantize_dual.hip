// Block quantize in both directions at once (bi8_quantize_dual): x [R,C] -> codes [R,C] with scales [ceil(C/B), R]
// (blocks along the rows, what bi8_quantize_rowwise writes) AND codes [C,R] with scales [ceil(R/B), C] (blocks down
// the columns, what bi8_quantize_transposed writes), from one pass over x.  A training step of the reference
// quantizes each of X, W and G twice, once per direction (block_linear.py:77-78, :92-94, :100-103): with this kernel
// every one of them is read from HBM once.
//
// A workgroup owns a 128 x 128 tile, held in registers as two 64-column halves (16 bytes per lane per row pass; the
// next tile's loads are issued while this one is processed).  The row direction is finished straight from the
// registers: the lanes of one row reduce their absmax with DPP, quantize and store their codes.  The column direction
// runs half by half through LDS exactly as in bi8_quantize_transposed (tile kept in its own type, 16-byte LDS accesses).  Both outputs are bit for bit those of the
// two separate entry points.
//
// bi8_quantize_dual_colsum also returns the column sums of x (the bias gradient G.sum(dim=0) of block_linear.py:110,
// when x is the output gradient G): the column walk has every element in a register anyway, so each thread adds up its
// rows, the tile's row groups are added in ascending order, the tiles' sums go to a workspace [tile row][column] and a
// second, tiny kernel adds them in ascending order (fp32 sums in a fixed order: deterministic) and casts.
#include "bi8_common.h"

namespace {

constexpr int kTR = 128;           // tile rows
constexpr int kTC = 64;            // columns of one half
constexpr int kThreads = 256;
// Tile order, as in bi8_quantize_transposed: the tiles in flight at one time form a compact patch of the matrix
// (bands of kSBR tile rows, chunks of kSBC tile columns inside a band, row by row inside a chunk), so that the reads
// and row-direction writes (runs along the rows) and the column-direction writes (runs down the columns) of the patch
// are all long runs in memory.
// Measured on bf16 [8192,8192]: 16 x 16 tiles 64.0 us, row by row 65.4, 8 x 32 64.6, 32 x 8 69.
constexpr int kSBR = 16, kSBC = 16;
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

// ALIGNED: rows of x start on 16-byte boundaries and C is a multiple of the elements per 16 bytes, rows of q on 8-byte
// boundaries.  Otherwise whole 16-byte chunks move with unaligned accesses and the last, partial chunk of a row
// element by element.
// NH: halves per tile.  2 is the tile described above; 1 (a 128 x 64 tile, blocks of at most 64) doubles the number of
// workgroups for inputs too small to occupy the chip with full tiles.
template <int DT, int B, bool ALIGNED, bool SUM, int NH>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(DT == BI8_F32 ? 2 : 3))) void quantize_dual_tile(const void *__restrict__ x, int8_t *__restrict__ q,
                                                               float *__restrict__ scales, int8_t *__restrict__ qT,
                                                               float *__restrict__ scalesT, float *__restrict__ colsum_part, int64_t R,
                                                               int64_t C, int64_t ldx, int64_t ldq, int64_t ldqt, int64_t tiles_c,
                                                               int64_t ntiles) {
    constexpr int VEC = Bi8Vec<DT>::kElems;
    constexpr int64_t ES = 16 / VEC;
    constexpr int LPR = kTC / VEC;                 // lanes per half row: 8 (16-bit) or 16 (fp32)
    constexpr int RPP = kThreads / LPR;            // rows per load pass
    constexpr int NP = kTR / RPP;                  // load passes per half
    constexpr int NCORR = (DT == BI8_F32) ? 2 : 1;
    constexpr int ESZ = (int)ES;                   // bytes per element
    constexpr int CPT = 4 / ESZ;                   // columns per thread in the column walk: one 32-bit word
    constexpr int G = kThreads / (kTC / CPT);      // row groups: 4 (fp32) or 8
    constexpr int RPT = kTR / G;                   // rows per thread: 32 (fp32) or 16
    constexpr int GPW = B / RPT;                   // row groups per column block
    constexpr int kXPitch = kTC * ESZ + (ESZ == 4 ? 0 : 16);   // bytes, 16-byte aligned (as in bi8_quantize_transposed)
    constexpr int LB = (B < kTC ? B : kTC) / VEC;  // lanes of one half row that share a row block
    static_assert(B == 32 || B == 64 || B == 128, "tile = one or more whole blocks in both directions");
    static_assert(NH == 2 || (NH == 1 && B <= kTC), "a row block lies inside the tile");
    __shared__ __attribute__((aligned(16))) uint8_t s_x[kTR * kXPitch];
    __shared__ float s_max[G][kTC];
    __shared__ float s_sum[SUM ? G : 1][kTC];
    __shared__ __attribute__((aligned(16))) uint8_t s_q[kTC * kQPitch];
    // the tile's row-direction scales, [block along the row][tile row]: stored from here as runs of kTR consecutive rows
    // (single 4-byte stores from the lanes that hold them cost the fabric a 32-byte write each)
    constexpr int NRB = (NH * kTC + B - 1) / B;
    __shared__ float s_rs[NRB][kTR];

    const int tid = threadIdx.x;
    const char *xb = (const char *)x;
    const bool wide_q = (((uintptr_t)q | (uintptr_t)ldq) & 15) == 0;     // rows of q on 16-byte boundaries: 16-byte code stores
    const int lr = tid / LPR;                      // row inside a pass
    const int cc = (tid % LPR) * VEC;              // first column of this lane inside a half

    const int64_t tiles_r = (R + kTR - 1) / kTR;
    auto load_half = [&](int64_t tile, int h, bi8_v4u *raw) {
        int64_t tr = 0, tc = 0;
        if (tile < ntiles) tile_coords(tile, tiles_r, tiles_c, tr, tc);
        const int64_t r0 = tr * kTR;
        const int64_t c0 = tc * (NH * kTC) + h * kTC;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int r = p * RPP + lr;
            raw[p] = bi8_v4u{0u, 0u, 0u, 0u};
            if (tile < ntiles && r0 + r < R && c0 + cc < C) {
                const char *src = xb + ((r0 + r) * ldx + c0 + cc) * ES;
                if constexpr (ALIGNED) {
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

    bi8_v4u raw[NH][NP];
#pragma unroll
    for (int h = 0; h < NH; ++h) load_half(blockIdx.x, h, raw[h]);
    for (int64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        int64_t tr, tc;
        tile_coords(tile, tiles_r, tiles_c, tr, tc);
        const int64_t r0 = tr * kTR;
        const int64_t cbase = tc * (NH * kTC);

        // ---- along the rows, from the registers ----------------------------------------------------------------
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int64_t row = r0 + p * RPP + lr;
            float f[NH][VEC];
            float m[NH];
            bool special[NH];
#pragma unroll
            for (int h = 0; h < NH; ++h) {
                bi8_unpack<DT>(raw[h][p], f[h]);
                m[h] = 0.0f;
                special[h] = false;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    m[h] = __builtin_fmaxf(m[h], __builtin_fabsf(f[h][e]));
                    special[h] |= (f[h][e] != f[h][e]);
                }
            }
            if constexpr (B == 2 * kTC) {
                m[0] = m[NH - 1] = bi8_group_max<LPR>(__builtin_fmaxf(m[0], m[NH - 1]));
            } else {
#pragma unroll
                for (int h = 0; h < NH; ++h) m[h] = bi8_group_max<LB>(m[h]);
            }
            // (16-bit inputs, two halves, aligned: a lane's 8 codes of each half are exchanged with its neighbour's so that the
            // even lane stores 16 consecutive codes of the left half and the odd lane 16 of the right half -- the eight lanes of
            // a row then write the row's whole 128-byte line in one instruction instead of two halves in two)
            constexpr bool kPairStores = ALIGNED && VEC == 8 && NH == 2;
            bi8_v2u wq[NH];
#pragma unroll
            for (int h = 0; h < NH; ++h) {
                const int64_t col = cbase + h * kTC + cc;
                const bool live = row < R && col < C;
                if ((tid % LB) == 0 && (B != 2 * kTC || h == 0)) s_rs[(h * kTC + cc) / B][p * RPP + lr] = m[h];
                const bool slow = special[h] | !bi8_scale_is_ordinary(m[h]);
                uint32_t code[VEC];
                if (__builtin_expect(slow, 0)) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) code[e] = bi8_code_slow(f[h][e], m[h]);
                } else {
                    const float y = 1.0f / m[h];
#pragma unroll
                    for (int e = 0; e < VEC; ++e) code[e] = bi8_code_fast<NCORR>(f[h][e], m[h], y);
                }
                if constexpr (kPairStores) {
                    wq[h] = bi8_v2u{bi8_pack4(code[0], code[1], code[2], code[3]), bi8_pack4(code[4], code[5], code[6], code[7])};
                    if (!wide_q && live) __builtin_nontemporal_store(wq[h], (bi8_v2u *)(q + row * ldq + col));
                } else if (live) {
                    int8_t *dst = q + row * ldq + col;
                    if (ALIGNED || col + VEC <= C) {
                        if constexpr (VEC == 4) {
                            const uint32_t w = bi8_pack4(code[0], code[1], code[2], code[3]);
                            if constexpr (ALIGNED) __builtin_nontemporal_store(w, (uint32_t *)dst);
                            else *(bi8_u32_unaligned *)dst = w;
                        } else {
                            const bi8_v2u w = {bi8_pack4(code[0], code[1], code[2], code[3]), bi8_pack4(code[4], code[5], code[6], code[7])};
                            if constexpr (ALIGNED) __builtin_nontemporal_store(w, (bi8_v2u *)dst);
                            else *(bi8_v2u_unaligned *)dst = w;
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < VEC; ++e)
                            if (col + e < C) dst[e] = (int8_t)(code[e] & 0xffu);
                    }
                }
            }
            if constexpr (kPairStores) {
                if (wide_q) {
                    const bool odd = (tid & 1) != 0;
                    const bi8_v2u send = odd ? wq[0] : wq[1];              // what the neighbour stores of this lane's codes
                    bi8_v2u recv;
                    recv[0] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send[0], 0xB1, 0xf, 0xf, false);   // quad_perm [1,0,3,2]
                    recv[1] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send[1], 0xB1, 0xf, 0xf, false);
                    const bi8_v4u w = odd ? bi8_v4u{recv[0], recv[1], wq[1][0], wq[1][1]} : bi8_v4u{wq[0][0], wq[0][1], recv[0], recv[1]};
                    const int64_t col = cbase + (odd ? kTC + cc - VEC : cc);       // 16 consecutive codes from here
                    if (row < R && col < C) {
                        int8_t *dst = q + row * ldq + col;
                        if (col + 2 * VEC <= C) __builtin_nontemporal_store(w, (bi8_v4u *)dst);
                        else __builtin_nontemporal_store(bi8_v2u{w[0], w[1]}, (bi8_v2u *)dst);      // (C is a multiple of 8: the row ends after the first 8)
                    }
                }
            }
        }

        // ---- down the columns, one half at a time through LDS --------------------------------------------------
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            const int64_t c0 = cbase + h * kTC;
            // phase 1: this half -> LDS as it is (the previous half's column reads ended before the barrier that
            // precedes its phase 4); then start the next tile's loads of this half
#pragma unroll
            for (int p = 0; p < NP; ++p) *(bi8_v4u *)&s_x[(p * RPP + lr) * kXPitch + (tid % LPR) * 16] = raw[h][p];
            load_half(tile + gridDim.x, h, raw[h]);
            __syncthreads();
            if (h == 0) {
                for (int i = tid; i < NRB * kTR; i += kThreads) {
                    const int b = i / kTR, r = i % kTR;
                    if (r0 + r < R && cbase + b * B < C) scales[(cbase / B + b) * R + r0 + r] = s_rs[b][r];
                }
            }

            // phase 2: column maxima over this thread's rows (one 32-bit word column: one fp32 column or two 16-bit
            // columns), then over the block's row groups
            const int cw = tid % (kTC / CPT);
            const int g = tid / (kTC / CPT);
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
            if constexpr (SUM) {
                // this thread's rows of its columns, top to bottom (rows past R were loaded as zeros)
#pragma unroll
                for (int k = 0; k < CPT; ++k) {
                    float t = v[k][0];
#pragma unroll
                    for (int i = 1; i < RPT; ++i) t += v[k][i];
                    s_sum[g][cw * CPT + k] = t;
                }
            }
            if constexpr (GPW > 1 || SUM) {
#pragma unroll
                for (int k = 0; k < CPT; ++k) s_max[g][cw * CPT + k] = m[k];
                __syncthreads();
                if constexpr (SUM) {
                    // the tile's row groups in ascending order; read before the barrier that follows phase 3, written
                    // again after the one that follows the next phase 1
                    if (g == 0) {
#pragma unroll
                        for (int k = 0; k < CPT; ++k) {
                            float t = s_sum[0][cw * CPT + k];
#pragma unroll
                            for (int qg = 1; qg < G; ++qg) t += s_sum[qg][cw * CPT + k];
                            if (c0 + cw * CPT + k < C) colsum_part[tr * C + c0 + cw * CPT + k] = t;
                        }
                    }
                }
                const int gb = g & ~(GPW - 1);
#pragma unroll
                for (int qg = 0; qg < GPW; ++qg)
#pragma unroll
                    for (int k = 0; k < CPT; ++k) m[k] = __builtin_fmaxf(m[k], s_max[gb + qg][cw * CPT + k]);
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

            // phase 4: 16 codes per lane, 8 lanes per output row.  The next writes to s_x come after this barrier, the
            // next writes to s_q after the next phase-1 barrier.
#pragma unroll
            for (int p = 0; p < (kTC * kTR / 16) / kThreads; ++p) {
                const int idx = p * kThreads + tid;
                const int oc = idx / (kTR / 16);       // output row inside the half = source column
                const int seg = idx % (kTR / 16);
                const int64_t orow = c0 + oc;
                const int64_t ocol = r0 + seg * 16;
                if (orow < C && ocol < R) {
                    const bi8_v4u w = *(const bi8_v4u *)&s_q[oc * kQPitch + seg * 16];
                    int8_t *dst = qT + orow * ldqt + ocol;
                    if (ocol + 16 <= R) {
                        __builtin_nontemporal_store(w, (bi8_v4u *)dst);
                    } else {
                        for (int e = 0; e < (int)(R - ocol); ++e) dst[e] = (int8_t)((w[e >> 2] >> (8 * (e & 3))) & 0xffu);
                    }
                }
            }
        }
    }
}

template <int DT, int B, bool ALIGNED>
int launch_dual(const void *x, int8_t *q, float *scales, int8_t *qT, float *scalesT, float *colsum_part, int64_t R, int64_t C, int64_t ldx,
                int64_t ldq, int64_t ldqt, hipStream_t st) {
    const int64_t tiles_r = (R + kTR - 1) / kTR;
    // workgroups per CU: four with 16-bit inputs (29 KiB of LDS, under 128 registers: 62.7 us against 65.9 with three at
    // bf16 [8192,8192]), three with fp32 (42 KiB)
    const int64_t resident = (DT == BI8_F32 ? 3 : 4) * 256;
    if constexpr (B <= kTC) {
        // an input of fewer full tiles than the chip holds workgroups: half tiles, twice as many workgroups
        const int64_t tiles_c1 = (C + kTC - 1) / kTC;
        if (((C + 2 * kTC - 1) / (2 * kTC)) * tiles_r < resident) {
            const int64_t ntiles = tiles_c1 * tiles_r, grid = ntiles < resident ? ntiles : resident;
            if (colsum_part)
                hipLaunchKernelGGL((quantize_dual_tile<DT, B, ALIGNED, true, 1>), dim3((unsigned)grid), dim3(kThreads), 0, st, x, q, scales, qT,
                                   scalesT, colsum_part, R, C, ldx, ldq, ldqt, tiles_c1, ntiles);
            else
                hipLaunchKernelGGL((quantize_dual_tile<DT, B, ALIGNED, false, 1>), dim3((unsigned)grid), dim3(kThreads), 0, st, x, q, scales, qT,
                                   scalesT, colsum_part, R, C, ldx, ldq, ldqt, tiles_c1, ntiles);
            return bi8_launch_rc();
        }
    }
    const int64_t tiles_c = (C + 2 * kTC - 1) / (2 * kTC);
    const int64_t ntiles = tiles_c * tiles_r;
    const int64_t grid = ntiles < resident ? ntiles : resident;
    if (colsum_part)
        hipLaunchKernelGGL((quantize_dual_tile<DT, B, ALIGNED, true, 2>), dim3((unsigned)grid), dim3(kThreads), 0, st, x, q, scales, qT, scalesT,
                           colsum_part, R, C, ldx, ldq, ldqt, tiles_c, ntiles);
    else
        hipLaunchKernelGGL((quantize_dual_tile<DT, B, ALIGNED, false, 2>), dim3((unsigned)grid), dim3(kThreads), 0, st, x, q, scales, qT, scalesT,
                           colsum_part, R, C, ldx, ldq, ldqt, tiles_c, ntiles);
    return bi8_launch_rc();
}

template <int DT, bool ALIGNED>
int dispatch(const void *x, int8_t *q, float *scales, int8_t *qT, float *scalesT, float *colsum_part, int64_t R, int64_t C, int64_t ldx,
             int64_t ldq, int64_t ldqt, int block, hipStream_t st) {
    switch (block) {
    case 32: return launch_dual<DT, 32, ALIGNED>(x, q, scales, qT, scalesT, colsum_part, R, C, ldx, ldq, ldqt, st);
    case 64: return launch_dual<DT, 64, ALIGNED>(x, q, scales, qT, scalesT, colsum_part, R, C, ldx, ldq, ldqt, st);
    default: return launch_dual<DT, 128, ALIGNED>(x, q, scales, qT, scalesT, colsum_part, R, C, ldx, ldq, ldqt, st);
    }
}

// Column sums without the quantizer (the shapes that the one-pass kernel does not take): the same grouping of the
// rows -- groups of kTR / G rows top to bottom, the groups of a 128-row tile in ascending order -- so that the sums
// do not depend on which kernel made them.  One thread per column.
template <int DT>
__global__ __launch_bounds__(256) void colsum_tiles(const void *__restrict__ x, float *__restrict__ part, int64_t R, int64_t C, int64_t ldx) {
    constexpr int RPT = (DT == BI8_F32) ? 32 : 16;
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t tr = blockIdx.y;
    if (c >= C) return;
    float total = 0.0f;
    for (int g = 0; g < kTR / RPT; ++g) {
        float t = 0.0f;
        for (int i = 0; i < RPT; ++i) {
            const int64_t r = tr * kTR + g * RPT + i;
            const float v = r < R ? bi8_load_elem<DT>(x, r * ldx + c) : 0.0f;
            t = i == 0 ? v : t + v;
        }
        total = g == 0 ? t : total + t;
    }
    part[tr * C + c] = total;
}

// out[c] = cast(sum over the row tiles, ascending)
template <int DT>
__global__ __launch_bounds__(256) void colsum_finish(const float *__restrict__ part, void *__restrict__ out, int64_t tiles_r, int64_t C) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    // sixteen independent loads at a time (a chain of dependent ones costs a memory latency each), added in order
    float t = 0.0f;
    for (int64_t t0 = 0; t0 < tiles_r; t0 += 16) {
        float v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = t0 + i < tiles_r ? part[(t0 + i) * C + c] : 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i)
            if (t0 + i < tiles_r) t = (t0 + i == 0) ? v[i] : t + v[i];
    }
    bi8_store_elem<DT>(out, c, t);
}

template <int DT> int launch_colsum_finish(const float *part, void *out, int64_t tiles_r, int64_t C, hipStream_t st) {
    hipLaunchKernelGGL((colsum_finish<DT>), dim3((unsigned)((C + 255) / 256)), dim3(256), 0, st, part, out, tiles_r, C);
    return bi8_launch_rc();
}
template <int DT> int launch_colsum_tiles(const void *x, float *part, int64_t R, int64_t C, int64_t ldx, hipStream_t st) {
    const int64_t tiles_r = (R + kTR - 1) / kTR;
    if (tiles_r > 65535) return BI8_ERR_TOO_LARGE;
    hipLaunchKernelGGL((colsum_tiles<DT>), dim3((unsigned)((C + 255) / 256), (unsigned)tiles_r), dim3(256), 0, st, x, part, R, C, ldx);
    return bi8_launch_rc();
}

}  // namespace

static int quantize_dual(const void *x, int x_dtype, int8_t *q, float *scales, int8_t *qT, float *scalesT, float *colsum_part, int64_t R,
                         int64_t C, int64_t ldx, int64_t ldq, int64_t ldqt, int block, void *stream) {
    if (x_dtype < 0 || x_dtype > 2) return BI8_ERR_BAD_DTYPE;
    if (block < 1 || block > (1 << 20)) return BI8_ERR_BAD_BLOCK;
    if (R < 0 || C < 0 || ldx < C || ldq < C || ldqt < R) return BI8_ERR_BAD_SHAPE;
    if (R == 0 || C == 0) return BI8_OK;
    if (!x || !q || !scales || !qT || !scalesT) return BI8_ERR_NULL_POINTER;
    const int64_t vec = x_dtype == BI8_F32 ? 4 : 8;
    const int64_t esize = x_dtype == BI8_F32 ? 4 : 2;
    // one kernel: block 32 / 64 / 128, x aligned to its element type, the transposed codes in 16-byte aligned rows
    const bool one_pass = (block == 32 || block == 64 || block == 128) && bi8_aligned(x, esize) && ldqt % 16 == 0 && bi8_aligned(qT, 16);
    if (!one_pass) {
        // other block sizes, transposed rows of odd length: the two single-direction entry points, same results
        int rc = bi8_quantize_rowwise(x, x_dtype, q, scales, R, C, ldx, ldq, block, stream);
        if (rc != BI8_OK) return rc;
        rc = bi8_quantize_transposed(x, x_dtype, qT, scalesT, R, C, ldx, ldqt, block, stream);
        if (rc != BI8_OK || !colsum_part) return rc;
        switch (x_dtype) {
        case BI8_F32: return launch_colsum_tiles<BI8_F32>(x, colsum_part, R, C, ldx, (hipStream_t)stream);
        case BI8_BF16: return launch_colsum_tiles<BI8_BF16>(x, colsum_part, R, C, ldx, (hipStream_t)stream);
        default: return launch_colsum_tiles<BI8_F16>(x, colsum_part, R, C, ldx, (hipStream_t)stream);
        }
    }
    const bool aligned = C % vec == 0 && ldx % vec == 0 && bi8_aligned(x, 16) && ldq % 8 == 0 && bi8_aligned(q, 8);
    hipStream_t st = (hipStream_t)stream;
    if (aligned) {
        switch (x_dtype) {
        case BI8_F32: return dispatch<BI8_F32, true>(x, q, scales, qT, scalesT, colsum_part, R, C, ldx, ldq, ldqt, block, st);
        case BI8_BF16: return dispatch<BI8_BF16, true>(x, q, scales, qT, scalesT, colsum_part, R, C, ldx, ldq, ldqt, block, st);
        default: return dispatch<BI8_F16, true>(x, q, scales, qT, scalesT, colsum_part, R, C, ldx, ldq, ldqt, block, st);
        }
    }
    switch (x_dtype) {
    case BI8_F32: return dispatch<BI8_F32, false>(x, q, scales, qT, scalesT, colsum_part, R, C, ldx, ldq, ldqt, block, st);
    case BI8_BF16: return dispatch<BI8_BF16, false>(x, q, scales, qT, scalesT, colsum_part, R, C, ldx, ldq, ldqt, block, st);
    default: return dispatch<BI8_F16, false>(x, q, scales, qT, scalesT, colsum_part, R, C, ldx, ldq, ldqt, block, st);
    }
}

extern "C" int bi8_quantize_dual(const void *x, int x_dtype, int8_t *q, float *scales, int8_t *qT, float *scalesT, int64_t R, int64_t C,
                                 int64_t ldx, int64_t ldq, int64_t ldqt, int block, void *stream) {
    return quantize_dual(x, x_dtype, q, scales, qT, scalesT, nullptr, R, C, ldx, ldq, ldqt, block, stream);
}

extern "C" int64_t bi8_colsum_workspace_bytes(int64_t R, int64_t C) {
    if (R <= 0 || C <= 0) return 0;
    return ((R + kTR - 1) / kTR) * C * (int64_t)sizeof(float);
}

extern "C" int bi8_quantize_dual_colsum(const void *x, int x_dtype, int8_t *q, float *scales, int8_t *qT, float *scalesT, void *colsum,
                                        void *workspace, int64_t workspace_bytes, int64_t R, int64_t C, int64_t ldx, int64_t ldq,
                                        int64_t ldqt, int block, void *stream) {
    if (x_dtype < 0 || x_dtype > 2) return BI8_ERR_BAD_DTYPE;
    if (R < 0 || C < 0) return BI8_ERR_BAD_SHAPE;
    if (C == 0) return BI8_OK;
    if (!colsum) return BI8_ERR_NULL_POINTER;
    if (R == 0) {                                  // an empty sum: zeros, written by the finishing kernel (no tiles to add)
        switch (x_dtype) {
        case BI8_F32: return launch_colsum_finish<BI8_F32>(nullptr, colsum, 0, C, (hipStream_t)stream);
        case BI8_BF16: return launch_colsum_finish<BI8_BF16>(nullptr, colsum, 0, C, (hipStream_t)stream);
        default: return launch_colsum_finish<BI8_F16>(nullptr, colsum, 0, C, (hipStream_t)stream);
        }
    }
    if (!workspace || !bi8_aligned(workspace, 4)) return BI8_ERR_NULL_POINTER;
    if (workspace_bytes < bi8_colsum_workspace_bytes(R, C)) return BI8_ERR_BAD_SHAPE;
    const int rc = quantize_dual(x, x_dtype, q, scales, qT, scalesT, (float *)workspace, R, C, ldx, ldq, ldqt, block, stream);
    if (rc != BI8_OK) return rc;
    const int64_t tiles_r = (R + kTR - 1) / kTR;
    switch (x_dtype) {
    case BI8_F32: return launch_colsum_finish<BI8_F32>((const float *)workspace, colsum, tiles_r, C, (hipStream_t)stream);
    case BI8_BF16: return launch_colsum_finish<BI8_BF16>((const float *)workspace, colsum, tiles_r, C, (hipStream_t)stream);
    default: return launch_colsum_finish<BI8_F16>((const float *)workspace, colsum, tiles_r, C, (hipStream_t)stream);
    }
}
