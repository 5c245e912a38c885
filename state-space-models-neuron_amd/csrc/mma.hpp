// MFMA tile helpers for gfx950 (CDNA4, 64-lane wavefronts).
//
// All SSD contractions are expressed as  OUT[m][n] += sum_k A[m][k] * Bt[n][k]  with BOTH
// operands staged in LDS with k contiguous, so every lane fetches its MFMA fragment with one
// 16-byte ds_read (bf16) and the two operands use the same code path.
//
//   bf16: v_mfma_f32_32x32x16_bf16   lane -> row (lane & 31), k = 8 * (lane >> 5) + 0..7
//   fp32: v_mfma_f32_32x32x2_f32     lane -> row (lane & 31), k = (lane >> 5)
//   accumulator (both): 16 floats per lane; register v of lane holds
//        column  (lane & 31),   row  8 * (v >> 2) + 4 * (lane >> 5) + (v & 3)
#pragma once
#include "common.hpp"

namespace m2 {

constexpr int kQ = M2_CHUNK;   // 128 tokens per chunk

template <typename T> struct MmaTraits;
template <> struct MmaTraits<bf16_t> { static constexpr int kPad = 8; };
template <> struct MmaTraits<float> { static constexpr int kPad = 4; };

// leading dimension (elements) of an LDS tile with `k` contiguous columns; the pad keeps
// 16-byte alignment of every row and spreads rows over banks.
template <typename T> __host__ __device__ constexpr int lds_ld(int k) { return k + MmaTraits<T>::kPad; }

__device__ __forceinline__ int acc_row(int lane, int v) { return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3); }
__device__ __forceinline__ int acc_col(int lane) { return lane & 31; }

template <int BM, int BN>
__device__ __forceinline__ void acc_zero(floatx16 (&acc)[BM][BN]) {
#pragma unroll
    for (int i = 0; i < BM; ++i)
#pragma unroll
        for (int j = 0; j < BN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
}

// One wave: acc[i][j] (32x32 blocks) += A[rows i*32.., k0:k1] * Bt[rows j*32.., k0:k1]^T.
// A points at the first of this wave's BM*32 rows, Bt at the first of its BN*32 rows.
// k0, k1 multiples of 16.
template <int BM, int BN>
__device__ __forceinline__ void wave_mma(floatx16 (&acc)[BM][BN], const bf16_t* __restrict__ A, int lda,
                                         const bf16_t* __restrict__ Bt, int ldb, int k0, int k1) {
    const int lane = threadIdx.x & 63;
    const int r = lane & 31, kh = (lane >> 5) * 8;
    for (int k = k0; k < k1; k += 16) {
        bf16x8 a[BM], b[BN];
#pragma unroll
        for (int i = 0; i < BM; ++i) a[i] = *reinterpret_cast<const bf16x8*>(A + (i * 32 + r) * lda + k + kh);
#pragma unroll
        for (int j = 0; j < BN; ++j) b[j] = *reinterpret_cast<const bf16x8*>(Bt + (j * 32 + r) * ldb + k + kh);
#pragma unroll
        for (int i = 0; i < BM; ++i)
#pragma unroll
            for (int j = 0; j < BN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
}

template <int BM, int BN>
__device__ __forceinline__ void wave_mma(floatx16 (&acc)[BM][BN], const float* __restrict__ A, int lda,
                                         const float* __restrict__ Bt, int ldb, int k0, int k1) {
    const int lane = threadIdx.x & 63;
    const int r = lane & 31, kh = lane >> 5;
    for (int k = k0; k < k1; k += 2) {
        float a[BM], b[BN];
#pragma unroll
        for (int i = 0; i < BM; ++i) a[i] = A[(i * 32 + r) * lda + k + kh];
#pragma unroll
        for (int j = 0; j < BN; ++j) b[j] = Bt[(j * 32 + r) * ldb + k + kh];
#pragma unroll
        for (int i = 0; i < BM; ++i)
#pragma unroll
            for (int j = 0; j < BN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
}

// ------------------------------------------------------------------------------------------
// Cooperative staging, global -> LDS.  NT threads; `tid` in [0, NT).
//
// stage_rows: global tile [ROWS][COLS] (COLS contiguous, row stride gstride) -> LDS [ROWS][ld].
// Rows >= valid are zero-filled.  If SCALE, row r is multiplied by rowscale[r] (fp32) first.
template <typename T, int ROWS, int COLS, int NT, bool SCALE>
__device__ __forceinline__ void stage_rows(T* __restrict__ s, int ld, const T* __restrict__ g, int64_t gstride,
                                           int valid, const float* __restrict__ rowscale, int tid) {
    constexpr int V = VecTraits<T>::kVec;
    constexpr int VPR = COLS / V;
    constexpr int TOTAL = ROWS * VPR;
    static_assert(COLS % V == 0, "tile width must be a multiple of the vector width");
#pragma unroll 4
    for (int e = tid; e < TOTAL; e += NT) {
        const int r = e / VPR, cv = e % VPR;
        float v[V];
        if (r < valid) load16(g + (int64_t)r * gstride + cv * V, v);
        else {
#pragma unroll
            for (int i = 0; i < V; ++i) v[i] = 0.f;
        }
        if (SCALE) {
            const float sc = rowscale[r];
#pragma unroll
            for (int i = 0; i < V; ++i) v[i] *= sc;
        }
        store16(s + r * ld + cv * V, v);
    }
}

// stage_transposed: global tile [ROWS][COLS] (COLS contiguous) -> LDS [COLS][ld], element (c, r).
// Global reads stay 16-byte and coalesced; the transpose happens in the (2- or 4-byte) LDS writes.
template <typename T, int ROWS, int COLS, int NT, bool SCALE>
__device__ __forceinline__ void stage_transposed(T* __restrict__ s, int ld, const T* __restrict__ g, int64_t gstride,
                                                 int valid, const float* __restrict__ rowscale, int tid) {
    constexpr int V = VecTraits<T>::kVec;
    constexpr int VPR = COLS / V;
    constexpr int TOTAL = ROWS * VPR;
    static_assert(COLS % V == 0, "tile width must be a multiple of the vector width");
#pragma unroll 4
    for (int e = tid; e < TOTAL; e += NT) {
        // consecutive threads take consecutive tokens of the same channel vector: the LDS writes of a
        // wave then fall into consecutive addresses of V rows (few bank conflicts), while the global
        // reads of a wave are 64 rows x 16 bytes.
        const int cv = e / ROWS, r = e % ROWS;
        float v[V];
        if (r < valid) load16(g + (int64_t)r * gstride + cv * V, v);
        else {
#pragma unroll
            for (int i = 0; i < V; ++i) v[i] = 0.f;
        }
        const float sc = SCALE ? rowscale[r] : 1.f;
#pragma unroll
        for (int i = 0; i < V; ++i) s[(cv * V + i) * ld + r] = from_f32<T>(SCALE ? v[i] * sc : v[i]);
    }
}

// Inclusive cumulative sum l[t] = sum_{s<=t} A * dt[s] over one chunk (kQ = 128 tokens), in fp32.
// Tokens >= valid behave as dt = 0 (no decay, no input).  Results in LDS: s_l[kQ], s_dt[kQ].
// Must be called by all threads of the block (contains barriers); blockDim.x >= 128.
template <typename DT>
__device__ __forceinline__ void chunk_cumsum(const DT* __restrict__ dt, int64_t stride_l, int valid, float A,
                                             float* __restrict__ s_l, float* __restrict__ s_dt,
                                             float* __restrict__ s_tmp, int tid) {
    float a = 0.f, d = 0.f;
    if (tid < kQ) {
        if (tid < valid) d = to_f32(dt[(int64_t)tid * stride_l]);
        a = A * d;
        const int lane = tid & 63;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const float nb = __shfl_up(a, off, 64);
            if (lane >= off) a += nb;
        }
        if (tid == 63) s_tmp[0] = a;
    }
    __syncthreads();
    if (tid < kQ) {
        if (tid >= 64) a += s_tmp[0];
        s_l[tid] = a;
        s_dt[tid] = d;
    }
    __syncthreads();
}

// dt is stored either as fp32 or in the activation type T; `off` is the element offset of token 0.
template <typename T>
__device__ __forceinline__ void chunk_cumsum_any(const void* __restrict__ dt, int dt_f32, int64_t off, int64_t stride_l,
                                                 int valid, float A, float* __restrict__ s_l, float* __restrict__ s_dt,
                                                 float* __restrict__ s_tmp, int tid) {
    if (dt_f32) chunk_cumsum<float>(static_cast<const float*>(dt) + off, stride_l, valid, A, s_l, s_dt, s_tmp, tid);
    else chunk_cumsum<T>(static_cast<const T*>(dt) + off, stride_l, valid, A, s_l, s_dt, s_tmp, tid);
}

}  // namespace m2
