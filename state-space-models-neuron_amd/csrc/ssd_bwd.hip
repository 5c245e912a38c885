// SSD chunked-scan backward for gfx950.
//
// Replaces the reference's NKI kernel mamba_kernel_bwd_ (mamba2/mamba2_kernel.py:277-485): same
// gradients (ddt, dA, dX, dB, dC, dD), forward recomputed per chunk instead of storing the decay
// matrix L, any batch size (the reference is batch-1 only, :315-317), optional gradient of the
// final state and of the initial state.
//
// Per head and chunk, with l the in-chunk cumulative sum of A*dt, Lam = l_{Q-1}, xd = dt*x,
// dS the gradient w.r.t. the state LEAVING the chunk and S_prev the state ENTERING it:
//   dxd_j = sum_{i>=j} e^{l_i-l_j} G[i][j] dy_i + e^{Lam-l_j} dS B_j          dx = dt dxd + D dy
//   dG[i][j] = sum_h e^{l_i-l_j} dt_j (dy_i . x_j)           (i >= j, summed over the heads of a group)
//   dC_i = sum_j dG[i][j] B_j + sum_h e^{l_i} dy_i^T S_prev
//   dB_j = sum_i dG[i][j] C_i + sum_h dt_j e^{Lam-l_j} x_j^T dS
//   dl_i = sum_n (C_i o dC_i^h - B_i o dB_i^h)               (row role minus column role of l_i, per head;
//                                                             the reference's C o dC - B o dB, :401,456)
//        = rowsum_i(dG^h o G) - colsum_i(dG^h o G) + C_i . dCoff_i^h - B_i . dBoff_i^h
//   da_j = sum_{i>=j, same chunk} dl_i + <dS, S_new>         ddt_j = A da_j + dxd_j . x_j
//   dA   = sum_j da_j dt_j                                   dD = sum dy . x
// Row sums and column sums are taken from the SAME fp32 tile dG^h o G, so pairs (i, j) that both lie
// in a suffix cancel exactly and only pairs straddling the position contribute, as in exact
// arithmetic.  (Forming dl from dy . (y - D x) with the stored bf16 y loses everything to
// cancellation once D x dominates y.)  <dS, S_new> is exact per chunk, so rounding does not
// accumulate along the sequence as it would with a global reverse cumulative sum (:459-461).
//
// Launch sequence:
//   cb_kernel, chunk_state_kernel, state_scan_kernel          recompute G, S_prev, final state
//   chunk_state_kernel<DSTATE>                                local dS contributions  e^{l} dy^T C
//   state_scan_kernel<REVERSE>                                dS per chunk, <dS, S_new>, d initial state
//   group_grad_kernel      per (b, chunk, group, head slice)  partial dB, dC (heads reduced in registers), dl per head
//   dx_kernel              per (b, chunk, head)               dx, ddt, partial dA, dD
//   bc_reduce_kernel, ad_reduce_kernel                        sum the partials (fixed order, no atomics)
#include "ssd_host.hpp"

namespace m2 {
namespace {

__device__ __forceinline__ float half_wave_sum(float v) {   // sum over the 32 lanes sharing (lane >> 5)
#pragma unroll
    for (int off = 16; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// ------------------------------------------------------------------------------------------
// grid (nchunks, nheads, batch), 256 threads; wave w owns token rows 32w..32w+31.
template <typename T, int P, int N>
__global__ void __launch_bounds__(256)
dx_kernel(const T* __restrict__ X, const void* __restrict__ dt, int dt_f32, const float* __restrict__ A,
          const T* __restrict__ Bm, const float* __restrict__ D, const float* __restrict__ G,
          const float* __restrict__ dl, const T* __restrict__ dY, const T* __restrict__ dprev, const float* __restrict__ dlam,
          T* __restrict__ dX, void* __restrict__ ddt, float* __restrict__ dAp, float* __restrict__ dDp,
          int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t nchunks,
          int64_t Xsb, int64_t Xsl, int64_t Xsh, int64_t dtsb, int64_t dtsl,
          int64_t Bsb, int64_t Bsl, int64_t Bsg,
          int64_t dYsb, int64_t dYsl, int64_t dYsh, int64_t dXsb, int64_t dXsl, int64_t dXsh,
          int64_t ddtsb, int64_t ddtsl) {
    constexpr int LDN = lds_ld<T>(N);
    constexpr int LDQ = lds_ld<T>(kQ);
    constexpr int BN = P / 32;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    float* s_l = reinterpret_cast<float*>(smem_raw);
    float* s_dt = s_l + kQ;
    float* s_w = s_dt + kQ;
    float* s_dir = s_w + kQ;
    float* s_tmp = s_dir + kQ;                     // 4 floats
    float* s_red = s_tmp + 4;                      // 8 floats
    T* buf = reinterpret_cast<T*>(s_red + 8);
    T* sB = buf;                                   // phase 1: [kQ][LDN]
    T* sdS = buf + kQ * LDN;                       //          [P][LDN]
    T* sMt = buf;                                  // phase 2: [kQ][LDQ]   Mt[j][i]
    T* sdYt = buf + kQ * LDQ;                      //          [P][LDQ]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int64_t c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int64_t g = h / (nheads / ngroups);
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    const float Ah = A[h];

    chunk_cumsum_any<T>(dt, dt_f32, b * dtsb + t0 * dtsl + h, dtsl, valid, Ah, s_l, s_dt, s_tmp, tid);
    const float Lam = s_l[kQ - 1];

    // ---- phase 1: acc[j][p] = e^{Lam-l_j} * sum_n B[j][n] dS[p][n]
    const int64_t tile = ((b * nchunks + c) * nheads + h) * (int64_t)(P * N);
    stage_rows<T, kQ, N, 256, false>(sB, LDN, Bm + b * Bsb + t0 * Bsl + g * Bsg, Bsl, valid, nullptr, tid);
    stage_rows<T, P, N, 256, false>(sdS, LDN, dprev + tile, N, P, nullptr, tid);
    __syncthreads();
    floatx16 acc[1][BN];
    acc_zero(acc);
    wave_mma<1, BN>(acc, sB + wave * 32 * LDN, LDN, sdS, LDN, 0, N);
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const float e = __expf(Lam - s_l[wave * 32 + acc_row(lane, v)]);
#pragma unroll
        for (int j = 0; j < BN; ++j) acc[0][j][v] *= e;
    }
    __syncthreads();

    // ---- phase 2: acc[j][p] += sum_{i>=j} (e^{l_i-l_j} G[i][j]) dy[i][p]
    const float* Gp = G + ((b * nchunks + c) * ngroups + g) * (int64_t)(kQ * kQ);
    for (int e = tid; e < kQ * (kQ / 4); e += 256) {
        const int i = e / (kQ / 4), j4 = (e % (kQ / 4)) * 4;
        if ((j4 >> 5) > (i >> 5)) continue;
        const floatx4 g4 = *reinterpret_cast<const floatx4*>(Gp + i * kQ + j4);
        const float li = s_l[i];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int j = j4 + q;
            const float m = (j <= i) ? __expf(li - s_l[j]) * g4[q] : 0.f;
            sMt[j * LDQ + i] = from_f32<T>(m);
        }
    }
    stage_transposed<T, kQ, P, 256, false>(sdYt, LDQ, dY + b * dYsb + t0 * dYsl + h * dYsh, dYsl, valid, nullptr, tid);
    __syncthreads();
    wave_mma<1, BN>(acc, sMt + wave * 32 * LDQ, LDQ, sdYt, LDQ, wave * 32, kQ);

    // ---- epilogue
    const float Dh = D ? D[h] : 0.f;
    const T* Xp = X + b * Xsb + t0 * Xsl + h * Xsh;
    T* dXp = dX + b * dXsb + t0 * dXsl + h * dXsh;
    float dD_loc = 0.f;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int row = wave * 32 + acc_row(lane, v);
        float edir = 0.f;
        if (row < valid) {
            const float dtj = s_dt[row];
#pragma unroll
            for (int j = 0; j < BN; ++j) {
                const int col = j * 32 + acc_col(lane);
                const float xv = to_f32(Xp[(int64_t)row * Xsl + col]);
                const float gy = to_f32(sdYt[col * LDQ + row]);
                const float dxd = acc[0][j][v];
                dXp[(int64_t)row * dXsl + col] = from_f32<T>(dtj * dxd + Dh * gy);
                edir += dxd * xv;
                dD_loc += gy * xv;
            }
        }
        edir = half_wave_sum(edir);
        if ((lane & 31) == 0) s_dir[row] = edir;
    }
    dD_loc = warp_sum(dD_loc);
    if (lane == 0) s_red[wave] = dD_loc;
    __syncthreads();

    // ---- da_j = (suffix sum of dl inside the chunk) + <dS, S_new>;  ddt, partial dA, partial dD
    float da_dt = 0.f;
    if (tid < kQ) {
        const int j = kQ - 1 - tid;                // thread t scans token Q-1-t: prefix over t == suffix over j
        float s = dl[((b * nheads + h) * nchunks + c) * kQ + j];
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const float nb = __shfl_up(s, off, 64);
            if (lane >= off) s += nb;
        }
        if (tid == 63) s_tmp[1] = s;
        s_w[j] = s;                                // own slot only; completed after the barrier
    }
    __syncthreads();
    if (tid < kQ) {
        const int j = kQ - 1 - tid;
        float s = s_w[j];
        if (tid >= 64) s += s_tmp[1];
        const float da = s + dlam[(b * nheads + h) * nchunks + c];
        if (j < valid) {
            const float val = Ah * da + s_dir[j];
            const int64_t o = b * ddtsb + (t0 + j) * ddtsl + h;
            if (dt_f32) static_cast<float*>(ddt)[o] = val;
            else static_cast<T*>(ddt)[o] = from_f32<T>(val);
            da_dt = da * s_dt[j];
        }
    }
    da_dt = warp_sum(da_dt);
    if (lane == 0) s_red[4 + wave] = da_dt;
    __syncthreads();
    if (tid == 0) {
        const int64_t o = (b * nheads + h) * nchunks + c;
        dAp[o] = s_red[4] + s_red[5] + s_red[6] + s_red[7];
        dDp[o] = s_red[0] + s_red[1] + s_red[2] + s_red[3];
    }
}

// ------------------------------------------------------------------------------------------
// grid (nchunks, ngroups * nslices, batch), 512 threads (8 waves).
// Wave w owns 32x32 blocks: row block (w >> 1), column blocks (w & 1) * NB + {0..NB-1}.
template <typename T, int P, int N>
__global__ void __launch_bounds__(512)
group_grad_kernel(const T* __restrict__ X, const void* __restrict__ dt, int dt_f32, const float* __restrict__ A,
                  const T* __restrict__ Bm, const T* __restrict__ Cm, const T* __restrict__ dY,
                  const T* __restrict__ Sprev, const T* __restrict__ dprev, const float* __restrict__ G,
                  float* __restrict__ dBp, float* __restrict__ dCp, float* __restrict__ dl,
                  int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t nchunks, int64_t nslices, int64_t hps,
                  int64_t Xsb, int64_t Xsl, int64_t Xsh, int64_t dtsb, int64_t dtsl,
                  int64_t Bsb, int64_t Bsl, int64_t Bsg, int64_t Csb, int64_t Csl, int64_t Csg,
                  int64_t dYsb, int64_t dYsl, int64_t dYsh) {
    constexpr int LDP = lds_ld<T>(P);
    constexpr int LDQ = lds_ld<T>(kQ);
    constexpr int NB = N / 64;                    // column blocks per wave for [Q][N] outputs
    constexpr int SZ1 = 2 * kQ * LDP, SZ2 = (kQ + N) * LDQ, SZ3 = (kQ + N) * LDP;
    constexpr int SZ = SZ1 > SZ2 ? (SZ1 > SZ3 ? SZ1 : SZ3) : (SZ2 > SZ3 ? SZ2 : SZ3);
    (void)SZ;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    float* s_l = reinterpret_cast<float*>(smem_raw);
    float* s_dt = s_l + kQ;
    float* s_e = s_dt + kQ;                        // e^{l_i}
    float* s_d = s_e + kQ;                         // dt_j e^{Lam - l_j}
    float* s_tmp = s_d + kQ;                       // 4 floats
    float* s_rs = s_tmp + 4;                       // [2][kQ] row sums of dG^h o G   (one slot per column half)
    float* s_cs = s_rs + 2 * kQ;                   // [4][kQ] column sums of dG^h o G (one slot per row block)
    float* s_rc = s_cs + 4 * kQ;                   // [2][kQ] C_i . dCoff_i^h
    float* s_rb = s_rc + 2 * kQ;                   // [2][kQ] B_j . dBoff_j^h
    T* buf = reinterpret_cast<T*>(s_rb + 2 * kQ);
    T* sA = buf;                                   // first tile  [kQ][LDP]  (or [kQ][LDQ] in the final steps)
    T* sT = buf + kQ * LDP;                        // second tile [kQ or N][LDP]
    T* sA2 = buf;                                  // final: [kQ][LDQ]
    T* sT2 = buf + kQ * LDQ;                       // final: [N][LDQ]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int64_t c = blockIdx.x, b = blockIdx.z;
    const int64_t g = blockIdx.y / nslices, slice = blockIdx.y % nslices;
    const int64_t hpg = nheads / ngroups;
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    const int rb = wave >> 1, cb0 = (wave & 1) * 2;       // [Q][Q] blocks: 2 per wave
    const int nb0 = (wave & 1) * NB;                        // [Q][N] blocks: NB per wave

    floatx16 dG[1][2], dC[1][NB], dB[1][NB];
    acc_zero(dG); acc_zero(dC); acc_zero(dB);

    for (int64_t hh = 0; hh < hps; ++hh) {
        const int64_t h = g * hpg + slice * hps + hh;
        chunk_cumsum_any<T>(dt, dt_f32, b * dtsb + t0 * dtsl + h, dtsl, valid, A[h], s_l, s_dt, s_tmp, tid);
        const float Lam = s_l[kQ - 1];
        if (tid < kQ) { s_e[tid] = __expf(s_l[tid]); s_d[tid] = s_dt[tid] * __expf(Lam - s_l[tid]); }
        const T* Xp = X + b * Xsb + t0 * Xsl + h * Xsh;
        const T* dYp = dY + b * dYsb + t0 * dYsl + h * dYsh;
        const int64_t tile = ((b * nchunks + c) * nheads + h) * (int64_t)(P * N);

        // ---- A: dG[i][j] += e^{l_i-l_j} dt_j (dy_i . x_j),  i >= j
        stage_rows<T, kQ, P, 512, false>(sA, LDP, dYp, dYsl, valid, nullptr, tid);
        stage_rows<T, kQ, P, 512, false>(sT, LDP, Xp, Xsl, valid, nullptr, tid);
        __syncthreads();
        const float* Gp = G + ((b * nchunks + c) * ngroups + g) * (int64_t)(kQ * kQ);
        {
            floatx16 pa[1][2];
            acc_zero(pa);
            float rsum[16], csum[2];
#pragma unroll
            for (int v = 0; v < 16; ++v) rsum[v] = 0.f;
            csum[0] = csum[1] = 0.f;
            if (cb0 <= rb) {
                wave_mma<1, 2>(pa, sA + rb * 32 * LDP, LDP, sT + cb0 * 32 * LDP, LDP, 0, P);
#pragma unroll
                for (int jb = 0; jb < 2; ++jb) {
                    if (cb0 + jb > rb) continue;
                    const int j = (cb0 + jb) * 32 + acc_col(lane);
                    const float lj = s_l[j], dtj = s_dt[j];
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int i = rb * 32 + acc_row(lane, v);
                        if (i >= j) {
                            const float dgh = __expf(s_l[i] - lj) * dtj * pa[0][jb][v];
                            dG[0][jb][v] += dgh;
                            const float pr = dgh * Gp[i * kQ + j];
                            rsum[v] += pr;
                            csum[jb] += pr;
                        }
                    }
                }
            }
            // row sums: over the 32 lanes of a half wave (columns) -> slot (wave & 1) of row i
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float r = half_wave_sum(rsum[v]);
                if ((lane & 31) == 0) s_rs[(wave & 1) * kQ + rb * 32 + acc_row(lane, v)] = r;
            }
            // column sums: over this lane's 16 rows, then the other half wave -> slot rb of column j
#pragma unroll
            for (int jb = 0; jb < 2; ++jb) {
                const float cs = csum[jb] + __shfl_xor(csum[jb], 32, 64);
                if (lane < 32) s_cs[rb * kQ + (cb0 + jb) * 32 + lane] = cs;
            }
        }
        __syncthreads();

        // ---- B: dC[i][n] += e^{l_i} sum_p dy[i][p] S_prev[p][n]     (dy tile still in sA; row scale applied in fp32)
        stage_transposed<T, P, N, 512, false>(sT, LDP, Sprev + tile, N, P, nullptr, tid);
        __syncthreads();
        {
            floatx16 tc[1][NB];
            acc_zero(tc);
            wave_mma<1, NB>(tc, sA + rb * 32 * LDP, LDP, sT + nb0 * 32 * LDP, LDP, 0, P);
            const T* Cg = Cm + b * Csb + t0 * Csl + g * Csg;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int i = rb * 32 + acc_row(lane, v);
                const float sc = s_e[i];
                float r = 0.f;
#pragma unroll
                for (int jn = 0; jn < NB; ++jn) {
                    const float t = tc[0][jn][v] * sc;
                    dC[0][jn][v] += t;
                    if (i < valid) r += t * to_f32(Cg[(int64_t)i * Csl + (nb0 + jn) * 32 + acc_col(lane)]);
                }
                r = half_wave_sum(r);
                if ((lane & 31) == 0) s_rc[(wave & 1) * kQ + i] = r;
            }
        }
        __syncthreads();

        // ---- C: dB[j][n] += dt_j e^{Lam-l_j} sum_p x[j][p] dS[p][n]
        stage_rows<T, kQ, P, 512, false>(sA, LDP, Xp, Xsl, valid, nullptr, tid);
        stage_transposed<T, P, N, 512, false>(sT, LDP, dprev + tile, N, P, nullptr, tid);
        __syncthreads();
        {
            floatx16 tb[1][NB];
            acc_zero(tb);
            wave_mma<1, NB>(tb, sA + rb * 32 * LDP, LDP, sT + nb0 * 32 * LDP, LDP, 0, P);
            const T* Bg = Bm + b * Bsb + t0 * Bsl + g * Bsg;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int j = rb * 32 + acc_row(lane, v);
                const float sc = s_d[j];
                float r = 0.f;
#pragma unroll
                for (int jn = 0; jn < NB; ++jn) {
                    const float t = tb[0][jn][v] * sc;
                    dB[0][jn][v] += t;
                    if (j < valid) r += t * to_f32(Bg[(int64_t)j * Bsl + (nb0 + jn) * 32 + acc_col(lane)]);
                }
                r = half_wave_sum(r);
                if ((lane & 31) == 0) s_rb[(wave & 1) * kQ + j] = r;
            }
        }
        __syncthreads();
        // dl_t for this head: row role minus column role
        if (tid < kQ) {
            const float rs = s_rs[tid] + s_rs[kQ + tid];
            const float cs = s_cs[tid] + s_cs[kQ + tid] + s_cs[2 * kQ + tid] + s_cs[3 * kQ + tid];
            const float rc = s_rc[tid] + s_rc[kQ + tid];
            const float rbv = s_rb[tid] + s_rb[kQ + tid];
            dl[((b * nheads + h) * nchunks + c) * kQ + tid] = rs - cs + rc - rbv;
        }
    }

    const T* Bp = Bm + b * Bsb + t0 * Bsl + g * Bsg;
    const T* Cp = Cm + b * Csb + t0 * Csl + g * Csg;

    // The head-summed dG is rounded to the operand type only here.  For bf16 it is split into
    // hi + lo (two MFMA passes) so that the group-level contractions see it at ~2^-17 relative.
    constexpr int NPASS = sizeof(T) == 2 ? 2 : 1;

    // ---- F1: dC[i][n] += sum_{j<=i} dG[i][j] B[j][n]
    stage_transposed<T, kQ, N, 512, false>(sT2, LDQ, Bp, Bsl, valid, nullptr, tid);
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
#pragma unroll
        for (int jb = 0; jb < 2; ++jb)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int i = rb * 32 + acc_row(lane, v), j = (cb0 + jb) * 32 + acc_col(lane);
                const float full = dG[0][jb][v];
                const T hi = from_f32<T>(full);
                sA2[i * LDQ + j] = pass == 0 ? hi : from_f32<T>(full - to_f32(hi));
            }
        __syncthreads();
        wave_mma<1, NB>(dC, sA2 + rb * 32 * LDQ, LDQ, sT2 + nb0 * 32 * LDQ, LDQ, 0, (rb + 1) * 32);
        __syncthreads();
    }

    // ---- F2: dB[j][n] += sum_{i>=j} dG[i][j] C[i][n]
    stage_transposed<T, kQ, N, 512, false>(sT2, LDQ, Cp, Csl, valid, nullptr, tid);
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
#pragma unroll
        for (int jb = 0; jb < 2; ++jb)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int i = rb * 32 + acc_row(lane, v), j = (cb0 + jb) * 32 + acc_col(lane);
                const float full = dG[0][jb][v];
                const T hi = from_f32<T>(full);
                sA2[j * LDQ + i] = pass == 0 ? hi : from_f32<T>(full - to_f32(hi));
            }
        __syncthreads();
        wave_mma<1, NB>(dB, sA2 + rb * 32 * LDQ, LDQ, sT2 + nb0 * 32 * LDQ, LDQ, rb * 32, kQ);
        __syncthreads();
    }

    // ---- store partials [b][c][g][slice][Q][N]
    const int64_t pt = (((b * nchunks + c) * ngroups + g) * nslices + slice) * (int64_t)(kQ * N);
#pragma unroll
    for (int jn = 0; jn < NB; ++jn)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = rb * 32 + acc_row(lane, v), col = (nb0 + jn) * 32 + acc_col(lane);
            dCp[pt + row * N + col] = dC[0][jn][v];
            dBp[pt + row * N + col] = dB[0][jn][v];
        }
}

// dB / dC = sum over head slices of the partials, cast to the activation type.  One thread per 4 state columns.
template <typename T>
__global__ void __launch_bounds__(256)
bc_reduce_kernel(const float* __restrict__ dBp, const float* __restrict__ dCp, T* __restrict__ dB, T* __restrict__ dC,
                 int64_t nb, int64_t seqlen, int64_t ngroups, int64_t nchunks, int64_t nslices, int N,
                 int64_t dBsb, int64_t dBsl, int64_t dBsg, int64_t dCsb, int64_t dCsl, int64_t dCsg) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int n4s = N / 4;
    const int64_t total = nb * seqlen * ngroups * n4s;
    if (idx >= total) return;
    const int n4 = (int)(idx % n4s) * 4;
    const int64_t g = (idx / n4s) % ngroups;
    const int64_t t = (idx / n4s / ngroups) % seqlen;
    const int64_t b = idx / n4s / ngroups / seqlen;
    const int64_t c = t / kQ, i = t % kQ;
    const int64_t base = (((b * nchunks + c) * ngroups + g) * nslices) * (int64_t)(kQ * N) + i * N + n4;
    floatx4 sb = {0.f, 0.f, 0.f, 0.f}, sc = {0.f, 0.f, 0.f, 0.f};
    for (int64_t s = 0; s < nslices; ++s) {
        sb += *reinterpret_cast<const floatx4*>(dBp + base + s * (int64_t)(kQ * N));
        sc += *reinterpret_cast<const floatx4*>(dCp + base + s * (int64_t)(kQ * N));
    }
    T* ob = dB + b * dBsb + t * dBsl + g * dBsg + n4;
    T* oc = dC + b * dCsb + t * dCsl + g * dCsg + n4;
#pragma unroll
    for (int q = 0; q < 4; ++q) { ob[q] = from_f32<T>(sb[q]); oc[q] = from_f32<T>(sc[q]); }
}

// dA[h] = sum_{b,c} dAp[b][h][c], dD likewise.  One block per head.
__global__ void __launch_bounds__(256)
ad_reduce_kernel(const float* __restrict__ dAp, const float* __restrict__ dDp, float* __restrict__ dA, float* __restrict__ dD,
                 int64_t nb, int64_t nheads, int64_t nchunks) {
    __shared__ float red[2][4];
    const int64_t h = blockIdx.x;
    float sa = 0.f, sd = 0.f;
    for (int64_t e = threadIdx.x; e < nb * nchunks; e += 256) {
        const int64_t b = e / nchunks, c = e % nchunks;
        sa += dAp[(b * nheads + h) * nchunks + c];
        sd += dDp[(b * nheads + h) * nchunks + c];
    }
    sa = warp_sum(sa); sd = warp_sum(sd);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) { red[0][wave] = sa; red[1][wave] = sd; }
    __syncthreads();
    if (threadIdx.x == 0) {
        dA[h] = red[0][0] + red[0][1] + red[0][2] + red[0][3];
        if (dD) dD[h] = red[1][0] + red[1][1] + red[1][2] + red[1][3];
    }
}

__global__ void zero_f32_kernel(float* __restrict__ p, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.f;
}
__global__ void copy_f32_kernel(const float* __restrict__ src, float* __restrict__ dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src ? src[i] : 0.f;
}

template <typename T, int P, int N>
size_t dx_smem() {
    const size_t a = (size_t)(kQ + P) * lds_ld<T>(N), b = (size_t)(kQ + P) * lds_ld<T>(kQ);
    return (4 * kQ + 12) * sizeof(float) + (a > b ? a : b) * sizeof(T);
}
template <typename T, int P, int N>
size_t gg_smem() {
    size_t a = (size_t)2 * kQ * lds_ld<T>(P), b = (size_t)(kQ + N) * lds_ld<T>(kQ), c = (size_t)(kQ + N) * lds_ld<T>(P);
    size_t m = a > b ? a : b;
    m = m > c ? m : c;
    return (14 * kQ + 4) * sizeof(float) + m * sizeof(T);
}

template <typename T, int P, int N>
int ssd_bwd_impl(const m2_ssd_params* p, hipStream_t st) {
    const int64_t nc = ceil_div(p->seqlen, (int64_t)kQ);
    const SsdWorkspace w = ssd_carve(p, p->workspace, true);
    const int dt_f32 = p->dt_dtype == M2_F32;
    const T* x = static_cast<const T*>(p->x);
    const T* Bm = static_cast<const T*>(p->B);
    const T* Cm = static_cast<const T*>(p->C);
    const T* dy = static_cast<const T*>(p->dy);
    int rc;
    // recompute G, S_prev, final state
    if ((rc = ssd_launch_states<T, P, N>(p, w, w.sfinal, st))) return rc;
    // local dS contributions (reuses the `local` region) and the reverse recurrence
    {
        auto k = chunk_state_kernel<T, P, N, true>;
        const size_t sm = state_smem<T, P, N>();
        if ((rc = allow_smem(k, sm))) return rc;
        k<<<dim3((unsigned)nc, (unsigned)p->nheads, (unsigned)p->batch), 256, sm, st>>>(
            dy, p->dt, dt_f32, p->A, Cm, w.local, nullptr, p->seqlen, p->nheads, p->ngroups, nc,
            p->dy_stride_b, p->dy_stride_l, p->dy_stride_h, p->dt_stride_b, p->dt_stride_l,
            p->C_stride_b, p->C_stride_l, p->C_stride_g);
        if ((rc = check_launch("ssd chunk_state_kernel<dstate>"))) return rc;
        state_scan_kernel<T, P * N, true><<<dim3((unsigned)p->nheads, (unsigned)p->batch), 256, 0, st>>>(
            w.local, w.lam, p->d_final_state, static_cast<T*>(w.dprev), p->d_initial_state,
            static_cast<const T*>(w.prev), w.sfinal, w.dlam, p->nheads, nc);
        if ((rc = check_launch("ssd state_scan_kernel<reverse>"))) return rc;
    }
    {
        auto k = group_grad_kernel<T, P, N>;
        const size_t sm = gg_smem<T, P, N>();
        if ((rc = allow_smem(k, sm))) return rc;
        M2_REQUIRE(p->ngroups * w.nslices <= 65535, M2_ERR_SHAPE, "ssd_bwd: too many group slices");
        k<<<dim3((unsigned)nc, (unsigned)(p->ngroups * w.nslices), (unsigned)p->batch), 512, sm, st>>>(
            x, p->dt, dt_f32, p->A, Bm, Cm, dy, static_cast<const T*>(w.prev), static_cast<const T*>(w.dprev), w.G, w.dBp, w.dCp, w.dl,
            p->seqlen, p->nheads, p->ngroups, nc, w.nslices, w.heads_per_slice,
            p->x_stride_b, p->x_stride_l, p->x_stride_h, p->dt_stride_b, p->dt_stride_l,
            p->B_stride_b, p->B_stride_l, p->B_stride_g, p->C_stride_b, p->C_stride_l, p->C_stride_g,
            p->dy_stride_b, p->dy_stride_l, p->dy_stride_h);
        if ((rc = check_launch("ssd group_grad_kernel"))) return rc;
    }
    {
        auto k = dx_kernel<T, P, N>;
        const size_t sm = dx_smem<T, P, N>();
        if ((rc = allow_smem(k, sm))) return rc;
        k<<<dim3((unsigned)nc, (unsigned)p->nheads, (unsigned)p->batch), 256, sm, st>>>(
            x, p->dt, dt_f32, p->A, Bm, p->D, w.G, w.dl, dy, static_cast<const T*>(w.dprev), w.dlam,
            static_cast<T*>(p->dx), p->ddt, w.dAp, w.dDp, p->seqlen, p->nheads, p->ngroups, nc,
            p->x_stride_b, p->x_stride_l, p->x_stride_h, p->dt_stride_b, p->dt_stride_l,
            p->B_stride_b, p->B_stride_l, p->B_stride_g,
            p->dy_stride_b, p->dy_stride_l, p->dy_stride_h, p->dx_stride_b, p->dx_stride_l, p->dx_stride_h,
            p->ddt_stride_b, p->ddt_stride_l);
        if ((rc = check_launch("ssd dx_kernel"))) return rc;
    }
    {
        const int64_t total = p->batch * p->seqlen * p->ngroups * (N / 4);
        bc_reduce_kernel<T><<<(unsigned)ceil_div(total, (int64_t)256), 256, 0, st>>>(
            w.dBp, w.dCp, static_cast<T*>(p->dB), static_cast<T*>(p->dC), p->batch, p->seqlen, p->ngroups, nc, w.nslices, N,
            p->dB_stride_b, p->dB_stride_l, p->dB_stride_g, p->dC_stride_b, p->dC_stride_l, p->dC_stride_g);
        if ((rc = check_launch("ssd bc_reduce_kernel"))) return rc;
        ad_reduce_kernel<<<(unsigned)p->nheads, 256, 0, st>>>(w.dAp, w.dDp, p->dA, p->D ? p->dD : nullptr, p->batch, p->nheads, nc);
        if ((rc = check_launch("ssd ad_reduce_kernel"))) return rc;
    }
    return M2_OK;
}

}  // namespace
}  // namespace m2

extern "C" size_t m2_ssd_bwd_workspace_bytes(const m2_ssd_params* p) {
    if (!p || p->batch <= 0 || p->seqlen <= 0 || p->nheads <= 0) return 256;
    return m2::ssd_carve(p, nullptr, true).bytes;
}

extern "C" int m2_ssd_bwd(const m2_ssd_params* p, void* stream) {
    using namespace m2;
    int rc = ssd_check(p, "ssd_bwd");
    if (rc) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (p->nheads == 0) return M2_OK;
    M2_REQUIRE(p->dA, M2_ERR_NULL, "ssd_bwd: dA is required");
    M2_REQUIRE(!p->D || p->dD, M2_ERR_NULL, "ssd_bwd: dD is required when D is given");
    if (p->batch == 0 || p->seqlen == 0) {
        // empty reductions: parameter gradients are zero; the state gradient passes straight through
        zero_f32_kernel<<<(unsigned)ceil_div(p->nheads, (int64_t)256), 256, 0, st>>>(p->dA, p->nheads);
        if (p->dD) zero_f32_kernel<<<(unsigned)ceil_div(p->nheads, (int64_t)256), 256, 0, st>>>(p->dD, p->nheads);
        if (p->d_initial_state && p->batch > 0) {
            const int64_t n = p->batch * p->nheads * p->headdim * p->dstate;
            copy_f32_kernel<<<(unsigned)ceil_div(n, (int64_t)256), 256, 0, st>>>(p->d_final_state, p->d_initial_state, n);
        }
        return check_launch("ssd_bwd (empty)");
    }
    M2_REQUIRE(p->x && p->dt && p->A && p->B && p->C && p->dy, M2_ERR_NULL, "ssd_bwd: x, dt, A, B, C, dy are required");
    M2_REQUIRE(p->dx && p->ddt && p->dB && p->dC, M2_ERR_NULL, "ssd_bwd: dx, ddt, dB, dC are required");
    const int V = p->dtype == M2_F32 ? 4 : 8;
    M2_REQUIRE(p->dy_stride_b % V == 0 && p->dy_stride_l % V == 0 && p->dy_stride_h % V == 0 && aligned16(p->dy), M2_ERR_ALIGN,
               "ssd_bwd: dy must be 16-byte aligned with strides that are multiples of %d elements", V);
    const size_t need = m2_ssd_bwd_workspace_bytes(p);
    M2_REQUIRE(p->workspace && p->workspace_bytes >= need, M2_ERR_WORKSPACE, "ssd_bwd: workspace %zu bytes < %zu needed",
               p->workspace_bytes, need);
    M2_REQUIRE((reinterpret_cast<uintptr_t>(p->workspace) & 255u) == 0, M2_ERR_ALIGN, "ssd_bwd: workspace must be 256-byte aligned");
    M2_DISPATCH_DTYPE(p->dtype, T, M2_DISPATCH_PN(p, P, N, return (ssd_bwd_impl<T, P, N>(p, st))));
    return M2_OK;
}
