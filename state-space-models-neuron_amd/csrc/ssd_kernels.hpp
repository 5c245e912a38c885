// SSD chunked-scan building blocks shared by the forward and the backward (gfx950).
//
// Notation (one head, one chunk of kQ = 128 tokens, local indices i, j):
//   a_j = A * dt_j,  l_i = sum_{j<=i} a_j (inclusive, fp32),  Lam = l_{Q-1}
//   G[i][j]  = C_i . B_j                         (per group)
//   y_i      = sum_{j<=i} e^{l_i-l_j} dt_j G[i][j] x_j  +  e^{l_i} C_i . S_prev  +  D x_i
//   S_new    = e^{Lam} S_prev + sum_j e^{Lam-l_j} dt_j x_j (x) B_j          (S is [p][n])
// The decay is always evaluated on the DIFFERENCE l_i - l_j <= 0 (the factorised form
// overflows fp32: with A = -16, dt = 0.1 the cumulative sum reaches -204.8 in one chunk),
// as the reference does (mamba2/mamba2_kernel.py:32-33).
//
// Kernels here (all launched with the chunk index in blockIdx.x so consecutive workgroups,
// which the hardware deals round-robin to the 8 XCDs, still share B/C/G tiles of one batch
// row through the MALL, and each XCD's L2 sees whole (head, chunk) tiles):
//   cb_kernel          G = C B^T per (batch, chunk, group)          -> workspace, fp32
//   chunk_state_kernel local chunk state  sum_j scale_j x_j (x) B_j -> workspace, fp32
//                      (DSTATE variant: sum_i e^{l_i} dy_i (x) C_i for the backward)
//   state_scan_kernel  sequential-in-chunks, parallel-in-(b,h,p,n) fp32 recurrence; writes the
//                      state ENTERING each chunk in the MFMA operand type, and the final state
//                      (REVERSE variant: gradient recurrence + <dS, S> per chunk)
#pragma once
#include "mma.hpp"

namespace m2 {

struct SsdDims {
    int64_t batch, seqlen, nheads, ngroups, nchunks;
};

// ------------------------------------------------------------------------------------------
// G[b][c][g][i][j] = sum_n C[i][n] * B[j][n].   grid (nchunks, ngroups, batch), 256 threads.
// Only 32x32 blocks with block-row >= block-col are consumed (causal); the upper-right
// 64x64 quadrant is neither computed nor written.
template <typename T, int N>
__global__ void __launch_bounds__(256)
cb_kernel(const T* __restrict__ Bm, const T* __restrict__ Cm, float* __restrict__ G,
          int64_t seqlen, int64_t ngroups, int64_t nchunks,
          int64_t Bsb, int64_t Bsl, int64_t Bsg, int64_t Csb, int64_t Csl, int64_t Csg) {
    constexpr int KB = 64;
    constexpr int LD = lds_ld<T>(KB);
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* sC = reinterpret_cast<T*>(smem_raw);
    T* sB = sC + kQ * LD;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int64_t c = blockIdx.x, g = blockIdx.y, b = blockIdx.z;
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    const T* Bp = Bm + b * Bsb + t0 * Bsl + g * Bsg;
    const T* Cp = Cm + b * Csb + t0 * Csl + g * Csg;
    const int wm = wave >> 1, wn = wave & 1;
    floatx16 acc[2][2];
    acc_zero(acc);
    for (int k0 = 0; k0 < N; k0 += KB) {
        stage_rows<T, kQ, KB, 256, false>(sC, LD, Cp + k0, Csl, valid, nullptr, tid);
        stage_rows<T, kQ, KB, 256, false>(sB, LD, Bp + k0, Bsl, valid, nullptr, tid);
        __syncthreads();
        if (!(wm == 0 && wn == 1)) wave_mma<2, 2>(acc, sC + wm * 64 * LD, LD, sB + wn * 64 * LD, LD, 0, KB);
        __syncthreads();
    }
    if (wm == 0 && wn == 1) return;
    float* Gp = G + ((b * nchunks + c) * ngroups + g) * (int64_t)(kQ * kQ);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = wm * 64 + i * 32 + acc_row(lane, v);
                const int col = wn * 64 + j * 32 + acc_col(lane);
                Gp[row * kQ + col] = acc[i][j][v];
            }
}

// ------------------------------------------------------------------------------------------
// Local chunk state.  grid (nchunks, nheads, batch), 256 threads.
//   DSTATE == false:  out[p][n] = sum_j (dt_j e^{Lam-l_j}) x[j][p] * B[j][n]      (forward)
//   DSTATE == true :  out[p][n] = sum_i e^{l_i} dy[i][p] * C[i][n]                (backward)
// Also writes lam[b][h][c] = Lam.  `X` is x or dy, `M` is B or C.
template <typename T, int P, int N, bool DSTATE>
__global__ void __launch_bounds__(256)
chunk_state_kernel(const T* __restrict__ X, const void* __restrict__ dt, int dt_f32, const float* __restrict__ A,
                   const T* __restrict__ M, float* __restrict__ out, float* __restrict__ lam,
                   int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t nchunks,
                   int64_t Xsb, int64_t Xsl, int64_t Xsh, int64_t dtsb, int64_t dtsl,
                   int64_t Msb, int64_t Msl, int64_t Msg) {
    constexpr int LD = lds_ld<T>(kQ);
    extern __shared__ __align__(16) unsigned char smem_raw[];
    float* s_l = reinterpret_cast<float*>(smem_raw);
    float* s_dt = s_l + kQ;
    float* s_sc = s_dt + kQ;
    float* s_tmp = s_sc + kQ;          // 4 floats
    T* sX = reinterpret_cast<T*>(s_tmp + 4);   // [P][LD]
    T* sM = sX + P * LD;                       // [N][LD]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int64_t c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int64_t g = h / (nheads / ngroups);
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);

    chunk_cumsum_any<T>(dt, dt_f32, b * dtsb + t0 * dtsl + h, dtsl, valid, A[h], s_l, s_dt, s_tmp, tid);
    const float Lam = s_l[kQ - 1];
    if (tid < kQ) s_sc[tid] = DSTATE ? __expf(s_l[tid]) : s_dt[tid] * __expf(Lam - s_l[tid]);
    __syncthreads();

    stage_transposed<T, kQ, P, 256, true>(sX, LD, X + b * Xsb + t0 * Xsl + h * Xsh, Xsl, valid, s_sc, tid);
    stage_transposed<T, kQ, N, 256, false>(sM, LD, M + b * Msb + t0 * Msl + g * Msg, Msl, valid, nullptr, tid);
    __syncthreads();

    constexpr int BM = P / 64, BN = N / 64;
    const int wm = wave >> 1, wn = wave & 1;
    floatx16 acc[BM][BN];
    acc_zero(acc);
    wave_mma<BM, BN>(acc, sX + wm * (P / 2) * LD, LD, sM + wn * (N / 2) * LD, LD, 0, kQ);

    float* op = out + ((b * nchunks + c) * nheads + h) * (int64_t)(P * N);
#pragma unroll
    for (int i = 0; i < BM; ++i)
#pragma unroll
        for (int j = 0; j < BN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = wm * (P / 2) + i * 32 + acc_row(lane, v);
                const int col = wn * (N / 2) + j * 32 + acc_col(lane);
                op[row * N + col] = acc[i][j][v];
            }
    if (tid == 0 && lam) lam[(b * nheads + h) * nchunks + c] = Lam;
}

// ------------------------------------------------------------------------------------------
// Inter-chunk recurrence.  grid (nheads, batch), 256 threads; each thread owns EPT float4
// slices of the [p][n] state and walks the chunks with the running state in registers (fp32).
//
// forward (REVERSE == false):
//     run = init;  for c = 0..nc-1:  prev[c] = T(run);  run = e^{lam_c} run + local[c];  final = run
// reverse (REVERSE == true), the gradient recurrence:
//     run = dfinal;  for c = nc-1..0:  prev[c] = T(run)   (= dL/dS_new(c));
//                                      dlam[c] = <run, S_new(c)>;   run = e^{lam_c} run + local[c]
//     dinit = run.     S_new(c) = sprev[c+1] for c < nc-1, the fp32 final state for c = nc-1.
template <typename T, int PN, bool REVERSE>
__global__ void __launch_bounds__(256)
state_scan_kernel(const float* __restrict__ local, const float* __restrict__ lam, const float* __restrict__ init,
                  T* __restrict__ prev, float* __restrict__ final_out,
                  const T* __restrict__ sprev, const float* __restrict__ sfinal, float* __restrict__ dlam,
                  int64_t nheads, int64_t nchunks) {
    constexpr int EPT = PN / 4 / 256;
    static_assert(PN % 1024 == 0, "state size must be a multiple of 1024 elements");
    __shared__ float red[4];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int64_t h = blockIdx.x, b = blockIdx.y;
    const int64_t bh = b * nheads + h;
    floatx4 run[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        if (init) run[e] = *reinterpret_cast<const floatx4*>(init + bh * PN + (e * 256 + tid) * 4);
        else run[e] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll 1
    for (int64_t cc = 0; cc < nchunks; ++cc) {
        const int64_t c = REVERSE ? nchunks - 1 - cc : cc;
        const int64_t tile = ((b * nchunks + c) * nheads + h) * (int64_t)PN;
        const float dec = __expf(lam[bh * nchunks + c]);
        float dot = 0.f;
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            const int off = (e * 256 + tid) * 4;
            const floatx4 loc = *reinterpret_cast<const floatx4*>(local + tile + off);
            // store the state entering (forward) / the gradient leaving (reverse) this chunk
            T o[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) o[q] = from_f32<T>(run[e][q]);
            if (sizeof(T) == 2) *reinterpret_cast<uint2*>(prev + tile + off) = *reinterpret_cast<const uint2*>(o);
            else *reinterpret_cast<uint4*>(prev + tile + off) = *reinterpret_cast<const uint4*>(o);
            if (REVERSE) {
                float sn[4];
                if (c == nchunks - 1) {
                    const floatx4 f = *reinterpret_cast<const floatx4*>(sfinal + bh * PN + off);
#pragma unroll
                    for (int q = 0; q < 4; ++q) sn[q] = f[q];
                } else {
                    const int64_t nxt = ((b * nchunks + c + 1) * nheads + h) * (int64_t)PN;
                    T tv[4];
                    if (sizeof(T) == 2) *reinterpret_cast<uint2*>(tv) = *reinterpret_cast<const uint2*>(sprev + nxt + off);
                    else *reinterpret_cast<uint4*>(tv) = *reinterpret_cast<const uint4*>(sprev + nxt + off);
#pragma unroll
                    for (int q = 0; q < 4; ++q) sn[q] = to_f32(tv[q]);
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) dot += run[e][q] * sn[q];
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) run[e][q] = dec * run[e][q] + loc[q];
        }
        if (REVERSE) {
            dot = warp_sum(dot);
            __syncthreads();               // red[] free again
            if (lane == 0) red[wave] = dot;
            __syncthreads();
            if (tid == 0) dlam[bh * nchunks + c] = red[0] + red[1] + red[2] + red[3];
        }
    }
    if (final_out) {
#pragma unroll
        for (int e = 0; e < EPT; ++e)
            *reinterpret_cast<floatx4*>(final_out + bh * PN + (e * 256 + tid) * 4) = run[e];
    }
}

}  // namespace m2
