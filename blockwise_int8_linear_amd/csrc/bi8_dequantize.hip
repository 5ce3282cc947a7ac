// Block dequantize (bi8_dequantize_rowwise): out = (scale * float(code)) * fp32(1/127), cast on store.
// Replaces _dequantize_block_rowwise, triton_functions.py:468-490.  HBM-bound: one lane = 16 codes
// (one 128-bit load) -> 16 outputs (two or four 128-bit stores).  Same tiling as the quantizer: a
// workgroup owns 16 rows x 1024 codes and first pulls its scales in through LDS, so the block-major /
// row-minor scale array is read as runs of 16 consecutive rows.
#include "bi8_common.h"

namespace {

constexpr int kRows = 16;
constexpr int kTileK = 1024;       // codes per tile row = 64 lanes x 16
constexpr int kThreads = 256;

template <int DT> __device__ __forceinline__ void store16(void *out, int64_t idx, const float *v) {
    if constexpr (DT == BI8_F32) {
        bi8_v4f *dst = (bi8_v4f *)((float *)out + idx);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            bi8_v4f w = {v[4 * g], v[4 * g + 1], v[4 * g + 2], v[4 * g + 3]};
            __builtin_nontemporal_store(w, dst + g);
        }
    } else {
        bi8_v4u *dst = (bi8_v4u *)((uint16_t *)out + idx);
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            bi8_v4u w;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                uint32_t lo, hi;
                if constexpr (DT == BI8_BF16) {
                    lo = bi8_bf16_bits(v[8 * g + 2 * e]);
                    hi = bi8_bf16_bits(v[8 * g + 2 * e + 1]);
                } else {
                    lo = bi8_f16_bits(v[8 * g + 2 * e]);
                    hi = bi8_f16_bits(v[8 * g + 2 * e + 1]);
                }
                w[e] = lo | (hi << 16);
            }
            __builtin_nontemporal_store(w, dst + g);
        }
    }
}

// LOG2B: log2 of the block size (>= 4, so that one lane's 16 codes share a scale)
template <int DT>
__global__ __launch_bounds__(kThreads) void dequantize_rows_vec(const int8_t *__restrict__ q, const float *__restrict__ scales,
                                                                void *__restrict__ out, int64_t M, int64_t K, int64_t ldq,
                                                                int64_t ldo, int64_t nblk, int log2b, int tiles_k) {
    __shared__ float s_tile[kTileK / 16][kRows + 1];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int64_t tile_m = blockIdx.x / tiles_k;
    const int tile_k = blockIdx.x % tiles_k;
    const int64_t row0 = tile_m * kRows;
    const int64_t col0 = (int64_t)tile_k * kTileK;
    const int nb = kTileK >> log2b;                 // blocks per tile row
    const int64_t jb0 = col0 >> log2b;

    bi8_v4u raw[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t row = row0 + wave * 4 + i;
        const int64_t col = col0 + lane * 16;
        bi8_v4u v = {0u, 0u, 0u, 0u};
        if (row < M && col < K) v = __builtin_nontemporal_load((const bi8_v4u *)(q + row * ldq + col));
        raw[i] = v;
    }
    for (int t = tid; t < nb * kRows; t += kThreads) {
        const int j = t / kRows, r = t % kRows;
        float s = 0.0f;
        if (row0 + r < M && jb0 + j < nblk) s = scales[(jb0 + j) * M + row0 + r];
        s_tile[j][r] = s;
    }
    __syncthreads();

    const float inv127 = (float)(1.0 / 127.0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t row = row0 + wave * 4 + i;
        const int64_t col = col0 + lane * 16;
        if (row < M && col < K) {
            const float s = s_tile[(lane * 16) >> log2b][wave * 4 + i];
            float v[16];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const int code = (int)(raw[i][e] << (24 - 8 * b)) >> 24;     // sign-extended byte b
                    v[4 * e + b] = (s * (float)code) * inv127;                   // two roundings, left to right
                }
            }
            store16<DT>(out, row * ldo + col, v);
        }
    }
}

template <int DT>
__global__ __launch_bounds__(kThreads) void dequantize_rows_generic(const int8_t *__restrict__ q, const float *__restrict__ scales,
                                                                    void *__restrict__ out, int64_t M, int64_t K, int64_t ldq,
                                                                    int64_t ldo, int block) {
    const float inv127 = (float)(1.0 / 127.0);
    const int64_t total = M * K;
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
        const int64_t row = i / K, k = i % K;
        const float s = scales[(k / block) * M + row];
        bi8_store_elem<DT>(out, row * ldo + k, (s * (float)q[row * ldq + k]) * inv127);
    }
}

template <int DT>
int dispatch(const int8_t *q, const float *scales, void *out, int64_t M, int64_t K, int64_t ldq, int64_t ldo, int block,
             hipStream_t st) {
    const bool vec_ok = bi8_pow2(block) && block >= 16 && block <= kTileK && K % 16 == 0 && ldq % 16 == 0 && ldo % 16 == 0 &&
                        bi8_aligned(q, 16) && bi8_aligned(out, 16);
    if (vec_ok) {
        const int64_t tiles_k = (K + kTileK - 1) / kTileK;
        const int64_t tiles_m = (M + kRows - 1) / kRows;
        if (tiles_k * tiles_m > 0x7fffffffLL) return BI8_ERR_TOO_LARGE;
        const int64_t nblk = (K + block - 1) / block;
        hipLaunchKernelGGL((dequantize_rows_vec<DT>), dim3((unsigned)(tiles_k * tiles_m)), dim3(kThreads), 0, st, q, scales, out, M,
                           K, ldq, ldo, nblk, __builtin_ctz((unsigned)block), (int)tiles_k);
        return bi8_launch_rc();
    }
    int64_t grid = (M * K + kThreads - 1) / kThreads;
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL((dequantize_rows_generic<DT>), dim3((unsigned)grid), dim3(kThreads), 0, st, q, scales, out, M, K, ldq, ldo,
                       block);
    return bi8_launch_rc();
}

}  // namespace

extern "C" int bi8_dequantize_rowwise(const int8_t *q, const float *scales, void *out, int out_dtype, int64_t M, int64_t K,
                                      int64_t ldq, int64_t ldo, int block, void *stream) {
    if (out_dtype < 0 || out_dtype > 2) return BI8_ERR_BAD_DTYPE;
    if (block < 1 || block > (1 << 20)) return BI8_ERR_BAD_BLOCK;
    if (M < 0 || K < 0 || ldq < K || ldo < K) return BI8_ERR_BAD_SHAPE;
    if (M == 0 || K == 0) return BI8_OK;
    if (!q || !scales || !out) return BI8_ERR_NULL_POINTER;
    hipStream_t st = (hipStream_t)stream;
    switch (out_dtype) {
    case BI8_F32: return dispatch<BI8_F32>(q, scales, out, M, K, ldq, ldo, block, st);
    case BI8_BF16: return dispatch<BI8_BF16>(q, scales, out, M, K, ldq, ldo, block, st);
    default: return dispatch<BI8_F16>(q, scales, out, M, K, ldq, ldo, block, st);
    }
}
