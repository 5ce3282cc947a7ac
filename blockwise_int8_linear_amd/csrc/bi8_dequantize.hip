// Block dequantize (bi8_dequantize_rowwise): out = (scale * float(code)) * fp32(1/127), cast on store.
// Replaces _dequantize_block_rowwise, triton_functions.py:468-490.  HBM-bound: one lane = one 128-bit store
// of outputs (8 bf16/f16 or 4 fp32) per step, so every wave store covers 1 KiB of contiguous output.  Same
// tiling as the quantizer: a workgroup owns 8 rows x 2 KiB of output row and first pulls its scales in
// through LDS, so the block-major / row-minor scale array is read as runs of 8 consecutive rows.
#include "bi8_common.h"

namespace {

constexpr int kLoads = 4;          // wave-loads per lane per tile (8 and 16 measured slower)
constexpr int kRpw = kLoads / 2;   // rows per wave
constexpr int kRows = 4 * kRpw;    // rows per workgroup tile
constexpr int kThreads = 256;

// One lane = kOut outputs = one 16-byte store (8 bf16/f16 or 4 fp32), so every store instruction of a wave
// writes 1 KiB of contiguous output; the codes come in as one 8- or 4-byte load per lane.
template <int DT> struct Out {
    static constexpr int kElems = (DT == BI8_F32) ? 4 : 8;
};

template <int DT> __device__ __forceinline__ void store_vec(void *out, int64_t idx, const float *v) {
    if constexpr (DT == BI8_F32) {
        bi8_v4f w = {v[0], v[1], v[2], v[3]};
        __builtin_nontemporal_store(w, (bi8_v4f *)((float *)out + idx));
    } else {
        bi8_v4u w;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            uint32_t lo, hi;
            if constexpr (DT == BI8_BF16) {
                lo = bi8_bf16_bits(v[2 * e]);
                hi = bi8_bf16_bits(v[2 * e + 1]);
            } else {
                lo = bi8_f16_bits(v[2 * e]);
                hi = bi8_f16_bits(v[2 * e + 1]);
            }
            w[e] = lo | (hi << 16);
        }
        __builtin_nontemporal_store(w, (bi8_v4u *)((uint16_t *)out + idx));
    }
}


// workgroup tile: 8 rows x (2 * 64 * kOut) codes; wave w owns rows 2w, 2w+1, two chunks of 64 * kOut codes each
template <int DT>
__global__ __launch_bounds__(kThreads) void dequantize_rows_vec(const int8_t *__restrict__ q, const float *__restrict__ scales,
                                                                void *__restrict__ out, int64_t M, int64_t K, int64_t ldq,
                                                                int64_t ldo, int64_t nblk, int log2b, int tiles_k) {
    constexpr int VEC = Out<DT>::kElems;
    constexpr int TE = 2 * BI8_WAVE * VEC;         // codes per tile row
    __shared__ float s_tile[TE / 8][kRows + 1];    // block size >= 8 on this path
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int64_t tile_m = blockIdx.x / tiles_k;
    const int tile_k = blockIdx.x % tiles_k;
    const int64_t row0 = tile_m * kRows;
    const int64_t col0 = (int64_t)tile_k * TE;
    const int nb = (TE >> log2b) > 0 ? (TE >> log2b) : 1;      // blocks per tile row
    const int64_t jb0 = col0 >> log2b;

    uint32_t raw[kLoads][VEC / 4];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        const int64_t row = row0 + wave * kRpw + (i >> 1);
        const int64_t col = col0 + ((i & 1) * BI8_WAVE + lane) * VEC;
#pragma unroll
        for (int e = 0; e < VEC / 4; ++e) raw[i][e] = 0u;
        if (row < M && col < K) {
            if constexpr (VEC == 8) {
                const bi8_v2u v = __builtin_nontemporal_load((const bi8_v2u *)(q + row * ldq + col));
                raw[i][0] = v[0];
                raw[i][1] = v[1];
            } else {
                raw[i][0] = __builtin_nontemporal_load((const uint32_t *)(q + row * ldq + col));
            }
        }
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
    for (int i = 0; i < kLoads; ++i) {
        const int64_t row = row0 + wave * kRpw + (i >> 1);
        const int incol = ((i & 1) * BI8_WAVE + lane) * VEC;
        const int64_t col = col0 + incol;
        if (row < M && col < K) {
            const float s = s_tile[incol >> log2b][wave * kRpw + (i >> 1)];
            float v[VEC];
#pragma unroll
            for (int e = 0; e < VEC / 4; ++e) {
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const int code = (int)(raw[i][e] << (24 - 8 * b)) >> 24;     // sign-extended byte b
                    v[4 * e + b] = (s * (float)code) * inv127;                   // two roundings, left to right
                }
            }
            store_vec<DT>(out, row * ldo + col, v);
        }
    }
}

template <int DT>
__global__ __launch_bounds__(kThreads) void dequantize_rows_generic(const int8_t *__restrict__ q, const float *__restrict__ scales,
                                                                    void *__restrict__ out, int64_t M, int64_t K, int64_t ldq,
                                                                    int64_t ldo, int block) {
    // one workgroup per (row, run of 2048 columns): consecutive lanes take consecutive elements, no 64-bit division
    const float inv127 = (float)(1.0 / 127.0);
    const int64_t runs = (K + 2047) / 2048;
    const int64_t units = M * runs;
    for (int64_t u = blockIdx.x; u < units; u += gridDim.x) {
        const int64_t row = u / runs, k0 = (u % runs) * 2048;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const int64_t k = k0 + t * kThreads + threadIdx.x;
            if (k < K) {
                const float s = scales[(k / block) * M + row];
                bi8_store_elem<DT>(out, row * ldo + k, (s * (float)q[row * ldq + k]) * inv127);
            }
        }
    }
}

template <int DT>
int dispatch(const int8_t *q, const float *scales, void *out, int64_t M, int64_t K, int64_t ldq, int64_t ldo, int block,
             hipStream_t st) {
    constexpr int VEC = Out<DT>::kElems;
    constexpr int TE = 2 * BI8_WAVE * VEC;
    const bool vec_ok = bi8_pow2(block) && block >= 8 && K % VEC == 0 && ldq % VEC == 0 && ldo % VEC == 0 &&
                        bi8_aligned(q, VEC) && bi8_aligned(out, 16);
    if (vec_ok) {
        const int64_t tiles_k = (K + TE - 1) / TE;
        const int64_t tiles_m = (M + kRows - 1) / kRows;
        if (tiles_k * tiles_m > 0x7fffffffLL) return BI8_ERR_TOO_LARGE;
        const int64_t nblk = (K + block - 1) / block;
        hipLaunchKernelGGL((dequantize_rows_vec<DT>), dim3((unsigned)(tiles_k * tiles_m)), dim3(kThreads), 0, st, q, scales, out, M,
                           K, ldq, ldo, nblk, __builtin_ctz((unsigned)block), (int)tiles_k);
        return bi8_launch_rc();
    }
    int64_t grid = M * ((K + 2047) / 2048);
    if (grid > (1 << 20)) grid = 1 << 20;
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
