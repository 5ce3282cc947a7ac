// Block quantize along rows (bi8_quantize_rowwise): per (row, K-block) absmax -> fp32 scale, int8 codes
// rint_even(127 * (x / absmax)).  HBM-bound: every input byte is read once with 128-bit loads, every
// code written once; the scales go through LDS so that each K-block's scales leave the workgroup as
// runs of 16 consecutive rows (the scale array is block-major / row-minor).
//
// Replaces _quantize_block_rowwise, triton_functions.py:193-216 (one program per row, serial over the
// row's blocks) with a 2-D tiling: one workgroup = 16 rows x 1 KiB of row, one lane = 16 input bytes,
// one K-block = L adjacent lanes (L = block * sizeof(elem) / 16), absmax by DPP inside the lane group.
#include "bi8_common.h"

namespace {

constexpr int kRowsPerWave = 4;            // = 16-byte loads in flight per lane; 2 and 8 both measured slower
constexpr int kRows = 4 * kRowsPerWave;    // rows per workgroup tile
constexpr int kChunks = 1;                 // 1 KiB wave-loads per row per tile (2 and 4 measured slower)
constexpr int kThreads = 256;

// ALIGNED: rows of x on 16-byte boundaries, K a multiple of the elements per 16 bytes, rows of q aligned to their
// 4- or 8-byte stores.  Otherwise (odd row length or leading dimension, e.g. the GPT-2 vocabulary 50257) whole chunks
// move with unaligned 16-byte loads and 4- or 8-byte stores, the last, partial chunk of a row element by element.
template <int DT, int L, bool ALIGNED>
__global__ __launch_bounds__(kThreads) void quantize_rows_vec(const void *__restrict__ x, int8_t *__restrict__ q,
                                                              float *__restrict__ scales, int64_t M, int64_t K,
                                                              int64_t ldx, int64_t ldq, int64_t nblk, int tiles_k) {
    constexpr int VEC = Bi8Vec<DT>::kElems;
    constexpr int B = L * VEC;                       // block size in elements
    constexpr int TE = kChunks * BI8_WAVE * VEC;     // elements of one row covered by a tile
    constexpr int NB = TE / B;                       // K-blocks per tile row
    constexpr int NCORR = (DT == BI8_F32) ? 2 : 1;
    constexpr int64_t ES = 16 / VEC;                 // bytes per element
    __shared__ float s_tile[NB][kRows + 1];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int64_t tile_m = blockIdx.x / tiles_k;
    const int tile_k = blockIdx.x % tiles_k;
    const int64_t row0 = tile_m * kRows;
    const int64_t col0 = (int64_t)tile_k * TE;
    const char *xb = (const char *)x;

    bi8_v4u raw[kRowsPerWave][kChunks];
#pragma unroll
    for (int i = 0; i < kRowsPerWave; ++i) {
        const int64_t row = row0 + wave * kRowsPerWave + i;
#pragma unroll
        for (int c = 0; c < kChunks; ++c) {
            const int64_t col = col0 + (c * BI8_WAVE + lane) * VEC;
            bi8_v4u v = {0u, 0u, 0u, 0u};
            if (row < M && col < K) {
                const char *src = xb + (row * ldx + col) * ES;
                if constexpr (ALIGNED) {
                    v = __builtin_nontemporal_load((const bi8_v4u *)src);
                } else if (col + VEC <= K) {
                    v = *(const bi8_v4u_unaligned *)src;
                } else {                           // the row ends inside this chunk
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        if (col + e < K) {
                            if constexpr (DT == BI8_F32) v[e] = ((const uint32_t *)src)[e];
                            else v[e >> 1] |= (uint32_t)((const uint16_t *)src)[e] << (16 * (e & 1));
                        }
                    }
                }
            }
            raw[i][c] = v;
        }
    }

#pragma unroll
    for (int i = 0; i < kRowsPerWave; ++i) {
        const int64_t row = row0 + wave * kRowsPerWave + i;
#pragma unroll
        for (int c = 0; c < kChunks; ++c) {
            const int64_t col = col0 + (c * BI8_WAVE + lane) * VEC;
            float f[VEC];
            bi8_unpack<DT>(raw[i][c], f);
            float m = 0.0f;
            bool special = false;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                m = __builtin_fmaxf(m, __builtin_fabsf(f[e]));      // ignores NaN
                special |= (f[e] != f[e]);
            }
            m = bi8_group_max<L>(m);
            if ((lane & (L - 1)) == 0) s_tile[(c * BI8_WAVE + lane) / L][wave * kRowsPerWave + i] = m;
            special |= !bi8_scale_is_ordinary(m);

            uint32_t code[VEC];
            if (__builtin_expect(special, 0)) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) code[e] = bi8_code_slow(f[e], m);
            } else {
                const float y = 1.0f / m;                               // correctly rounded reciprocal
#pragma unroll
                for (int e = 0; e < VEC; ++e) code[e] = bi8_code_fast<NCORR>(f[e], m, y);
            }
            if (row < M && col < K) {
                int8_t *dst = q + row * ldq + col;
                if (ALIGNED || col + VEC <= K) {
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
                        if (col + e < K) dst[e] = (int8_t)(code[e] & 0xffu);
                }
            }
        }
    }
    __syncthreads();
    const int64_t jb0 = col0 / B;
    for (int t = tid; t < NB * kRows; t += kThreads) {
        const int j = t / kRows, r = t % kRows;
        if (row0 + r < M && jb0 + j < nblk) scales[(jb0 + j) * M + row0 + r] = s_tile[j][r];
    }
}

// Any block size, any alignment: one wave per (row, block); lanes stride over the block.
template <int DT>
__global__ __launch_bounds__(kThreads) void quantize_rows_generic(const void *__restrict__ x, int8_t *__restrict__ q,
                                                                  float *__restrict__ scales, int64_t M, int64_t K,
                                                                  int64_t ldx, int64_t ldq, int64_t nblk, int block) {
    const int lane = threadIdx.x & 63;
    const int64_t wave0 = (int64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    const int64_t nwaves = (int64_t)gridDim.x * (kThreads / 64);
    const int64_t units = M * nblk;
    for (int64_t u = wave0; u < units; u += nwaves) {       // wave-uniform trip count
        // consecutive waves take consecutive blocks of one row
        const int64_t row = u / nblk, j = u % nblk;
        const int64_t k0 = j * block;
        const int64_t n = (K - k0 < block) ? (K - k0) : block;
        float m = 0.0f;
        for (int64_t k = lane; k < n; k += 64) m = __builtin_fmaxf(m, __builtin_fabsf(bi8_load_elem<DT>(x, row * ldx + k0 + k)));
        m = bi8_group_max<64>(m);
        if (lane == 0) scales[j * M + row] = m;
        for (int64_t k = lane; k < n; k += 64) {
            const float v = bi8_load_elem<DT>(x, row * ldx + k0 + k);
            q[row * ldq + k0 + k] = (int8_t)(bi8_code_slow(v, m) & 0xffu);
        }
    }
}

template <int DT, int L, bool ALIGNED>
int launch_vec(const void *x, int8_t *q, float *scales, int64_t M, int64_t K, int64_t ldx, int64_t ldq, hipStream_t st) {
    constexpr int VEC = Bi8Vec<DT>::kElems;
    constexpr int B = L * VEC;
    constexpr int TE = kChunks * BI8_WAVE * VEC;
    const int64_t tiles_k = (K + TE - 1) / TE;
    const int64_t tiles_m = (M + kRows - 1) / kRows;
    if (tiles_k * tiles_m > 0x7fffffffLL) return BI8_ERR_TOO_LARGE;
    const int64_t nblk = (K + B - 1) / B;
    hipLaunchKernelGGL((quantize_rows_vec<DT, L, ALIGNED>), dim3((unsigned)(tiles_k * tiles_m)), dim3(kThreads), 0, st, x, q, scales, M, K,
                       ldx, ldq, nblk, (int)tiles_k);
    return bi8_launch_rc();
}

template <int DT, bool ALIGNED>
int dispatch_vec(const void *x, int8_t *q, float *scales, int64_t M, int64_t K, int64_t ldx, int64_t ldq, int lanes, hipStream_t st) {
    switch (lanes) {
    case 1: return launch_vec<DT, 1, ALIGNED>(x, q, scales, M, K, ldx, ldq, st);
    case 2: return launch_vec<DT, 2, ALIGNED>(x, q, scales, M, K, ldx, ldq, st);
    case 4: return launch_vec<DT, 4, ALIGNED>(x, q, scales, M, K, ldx, ldq, st);
    case 8: return launch_vec<DT, 8, ALIGNED>(x, q, scales, M, K, ldx, ldq, st);
    case 16: return launch_vec<DT, 16, ALIGNED>(x, q, scales, M, K, ldx, ldq, st);
    case 32: return launch_vec<DT, 32, ALIGNED>(x, q, scales, M, K, ldx, ldq, st);
    default: return launch_vec<DT, 64, ALIGNED>(x, q, scales, M, K, ldx, ldq, st);
    }
}

template <int DT>
int dispatch(const void *x, int8_t *q, float *scales, int64_t M, int64_t K, int64_t ldx, int64_t ldq, int block, hipStream_t st) {
    constexpr int VEC = Bi8Vec<DT>::kElems;
    // one K-block = 1 .. 64 lanes of 16 input bytes each
    const bool vec_ok = bi8_pow2(block) && block >= VEC && block <= 64 * VEC && bi8_aligned(x, 16 / VEC);
    if (vec_ok) {
        const bool aligned = K % VEC == 0 && ldx % VEC == 0 && ldq % VEC == 0 && bi8_aligned(x, 16) && bi8_aligned(q, VEC);
        return aligned ? dispatch_vec<DT, true>(x, q, scales, M, K, ldx, ldq, block / VEC, st)
                       : dispatch_vec<DT, false>(x, q, scales, M, K, ldx, ldq, block / VEC, st);
    }
    const int64_t nblk = (K + block - 1) / block;
    const int64_t units = M * nblk;
    int64_t grid = (units + 3) / 4;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL((quantize_rows_generic<DT>), dim3((unsigned)grid), dim3(kThreads), 0, st, x, q, scales, M, K, ldx, ldq, nblk,
                       block);
    return bi8_launch_rc();
}

}  // namespace

extern "C" int bi8_quantize_rowwise(const void *x, int x_dtype, int8_t *q, float *scales, int64_t M, int64_t K, int64_t ldx,
                                    int64_t ldq, int block, void *stream) {
    if (x_dtype < 0 || x_dtype > 2) return BI8_ERR_BAD_DTYPE;
    if (block < 1 || block > (1 << 20)) return BI8_ERR_BAD_BLOCK;
    if (M < 0 || K < 0 || ldx < K || ldq < K) return BI8_ERR_BAD_SHAPE;
    if (M == 0 || K == 0) return BI8_OK;
    if (!x || !q || !scales) return BI8_ERR_NULL_POINTER;
    hipStream_t st = (hipStream_t)stream;
    switch (x_dtype) {
    case BI8_F32: return dispatch<BI8_F32>(x, q, scales, M, K, ldx, ldq, block, st);
    case BI8_BF16: return dispatch<BI8_BF16>(x, q, scales, M, K, ldx, ldq, block, st);
    default: return dispatch<BI8_F16>(x, q, scales, M, K, ldx, ldq, block, st);
    }
}
