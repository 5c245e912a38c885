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
// cancellation once D x dominates y.)  The state term is evaluated in the equivalent form
//   <dS, S_new> - sum_{i>=j} (B_i . dBoff_i^h)  =  e^{Lam} <dS, S_prev> + sum_{i<j} (B_i . dBoff_i^h)
// (a prefix instead of a suffix of the per-token terms), which avoids subtracting two large numbers that were
// rounded differently.  Everything is exact per chunk, so rounding does not accumulate along the sequence as it
// would with a global reverse cumulative sum (:459-461).
//
// Launch sequence (16-bit operands; fp32 operands take the kernels named in brackets):
//   prep_kernel, state_pass16_kernel [chunk_state + state_scan]   recompute G, tables, S_prev (skipped if the caller kept them)
//   state_pass16_kernel<REVERSE> [chunk_state<DSTATE> + state_scan<REVERSE>]
//                                                              dS per chunk, d initial state (and e^{Lam} <dS, S_prev> when
//                                                              ssd_bwd16_kernel does not run)
//   dg16_kernel [dg_kernel]   per (b, chunk, group, head slice)  partial dG (heads reduced in registers), dl_diag per head
//   ssd_bwd16_kernel [off_kernel<C>, <B>, diag_off_kernel<bwd>]
//                             per (b, chunk, group, head slice)  dx, per-token decay-gradient terms, e^{Lam} <dS, S_prev>,
//                                                                dD partials, partial state parts of dB / dC
//   tail1_kernel              da_body: ddt, dA partials per (b, head, chunk);  slice_sum_body: partials over the head slices
//   tail2_kernel              bc_final16_body [bc_final_body] per (b, chunk, group): dC = dG B + dCoff, dB = dG^T C + dBoff;
//                             ad_reduce_body per head: dA, dD (fixed order, no atomics)
#include "ssd_host.hpp"

namespace m2 {
namespace {

// ------------------------------------------------------------------------------------------
// dG partial and the diagonal part of the decay gradient.
// grid (nchunks, ngroups * nslices, batch), 512 threads (8 waves).  Wave w owns the 32x32 blocks of the
// [kQ][kQ] tile with block-row rb = w >> 1 and block-columns cb0 = 2 (w & 1), cb0 + 1.
//   per head:  P = dY X^T  (MFMA, K = headdim);   dG^h[i][j] = e^{l_i - l_j} dt_j P[i][j]   (i >= j)
//              dG += dG^h;    pr = dG^h o G;   dl_diag[i] = sum_j pr[i][j] - sum_i' pr[i'][i]
// Row and column sums come from the same fp32 products, so pairs inside a suffix cancel exactly.
template <typename T, int P>
constexpr bool dg_g_in_lds() { return (size_t)14 * kQ * sizeof(float) + ((size_t)2 * kQ * lds_ld<T>(P) + (size_t)kQ * lds_ld<T>(kQ)) * sizeof(T) <= 150 * 1024; }

template <typename T, int P>
__global__ void __launch_bounds__(512, 2)
dg_kernel(const T* __restrict__ X, const float* __restrict__ ldtab,
          const T* __restrict__ dY, const T* __restrict__ Gm, float* __restrict__ dGp, float* __restrict__ dl_diag,
          int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t nchunks, int64_t nslices, int64_t hps,
          int64_t Xsb, int64_t Xsl, int64_t Xsh, int64_t dYsb, int64_t dYsl, int64_t dYsh) {
    constexpr int LDP = lds_ld<T>(P);
    constexpr int LDQ = lds_ld<T>(kQ);
    extern __shared__ __align__(16) unsigned char smem_raw[];
    float* wtab = reinterpret_cast<float*>(smem_raw);      // [8 waves][kQ]  l (wave-private)
    float* s_rs = wtab + 8 * kQ;                           // [2][kQ]
    float* s_cs = s_rs + 2 * kQ;                           // [4][kQ]
    T* sA = reinterpret_cast<T*>(s_cs + 4 * kQ);           // dY [kQ][LDP]
    T* sT = sA + kQ * LDP;                                 // X  [kQ][LDP]
    T* sG = sT + kQ * LDP;                                 // G  [kQ][LDQ]  (blocks above the diagonal are never read)

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31;
    const int64_t c = blockIdx.x, b = blockIdx.z;
    const int64_t g = blockIdx.y / nslices, slice = blockIdx.y % nslices;
    const int64_t hpg = nheads / ngroups;
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    const int rb = wave >> 1, cb0 = (wave & 1) * 2;
    const bool active = cb0 <= rb;
    float* wl = wtab + wave * kQ;

    // causal-masked G of this (chunk, group), shared by all heads: staged once
    constexpr bool G_LDS = dg_g_in_lds<T, P>();
    const T* Gg = Gm + ((b * nchunks + c) * ngroups + g) * (int64_t)(kQ * kQ);
    if (G_LDS) stage_rows<T, kQ, kQ, 512, false>(sG, LDQ, Gg, kQ, kQ, nullptr, tid);
    floatx16 dG[1][2];
    acc_zero(dG);

    // the next head's dY and X tiles travel global -> registers while the current head is computed
    constexpr int V = VecTraits<T>::kVec;
    constexpr int VPR = P / V;                     // 16-byte vectors per token row
    constexpr int NV = kQ * VPR / 512;             // vectors per thread per tile
    static_assert((kQ * VPR) % 512 == 0, "tile does not divide over the workgroup");
    uint4 pdy[NV], pxx[NV];
    auto prefetch = [&](int64_t h) {
        const T* gy = dY + b * dYsb + t0 * dYsl + h * dYsh;
        const T* gx = X + b * Xsb + t0 * Xsl + h * Xsh;
#pragma unroll
        for (int it = 0; it < NV; ++it) {
            const int e = it * 512 + tid, rr = e / VPR, cv = e % VPR;
            const bool ok = rr < valid;
            pdy[it] = ok ? *reinterpret_cast<const uint4*>(gy + (int64_t)rr * dYsl + cv * V) : uint4{0u, 0u, 0u, 0u};
            pxx[it] = ok ? *reinterpret_cast<const uint4*>(gx + (int64_t)rr * Xsl + cv * V) : uint4{0u, 0u, 0u, 0u};
        }
    };
    prefetch(g * hpg + slice * hps);

    for (int64_t hh = 0; hh < hps; ++hh) {
        const int64_t h = g * hpg + slice * hps + hh;
        float l0, l1, d0, d1;
        wave_ld_load(ldtab, (b * nheads + h) * nchunks + c, l0, l1, d0, d1);
        wl[lane] = l0; wl[lane + 64] = l1;
        const float l_first = rb < 2 ? __shfl(l0, rb * 32, 64) : __shfl(l1, rb * 32 - 64, 64);
        const float l_last = rb < 2 ? __shfl(l0, rb * 32 + 31, 64) : __shfl(l1, rb * 32 + 31 - 64, 64);
        const bool fast = (l_first - l_last) < kMaxRange;
        // column-side values of this lane's two columns j = (cb0 + jb) * 32 + r
        float lj[2], dtj[2], vj[2];
#pragma unroll
        for (int jb = 0; jb < 2; ++jb) {
            const int src = jb * 32 + r;
            lj[jb] = cb0 == 0 ? __shfl(l0, src, 64) : __shfl(l1, src, 64);
            dtj[jb] = cb0 == 0 ? __shfl(d0, src, 64) : __shfl(d1, src, 64);
            vj[jb] = (cb0 + jb <= rb) ? __expf(fminf(l_first - lj[jb], kMaxRange)) * dtj[jb] : 0.f;
        }

        __syncthreads();      // previous head: tiles consumed, s_rs / s_cs consumed
#pragma unroll
        for (int it = 0; it < NV; ++it) {
            const int e = it * 512 + tid, rr = e / VPR, cv = e % VPR;
            *reinterpret_cast<uint4*>(sA + rr * LDP + cv * V) = pdy[it];
            *reinterpret_cast<uint4*>(sT + rr * LDP + cv * V) = pxx[it];
        }
        __syncthreads();
        if (hh + 1 < hps) prefetch(h + 1);

        float rsum[16], csum[2] = {0.f, 0.f};
#pragma unroll
        for (int v = 0; v < 16; ++v) rsum[v] = 0.f;
        if (active) {
#pragma unroll
            for (int jb = 0; jb < 2; ++jb) {
                if (cb0 + jb > rb) continue;
                floatx16 pa[1][1];
                acc_zero(pa);
                wave_mma<1, 1>(pa, sA + rb * 32 * LDP, LDP, sT + (cb0 + jb) * 32 * LDP, LDP, 0, P);
                const int j = (cb0 + jb) * 32 + r;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int i = rb * 32 + acc_row(lane, v);
                    float w;
                    if (fast) w = __expf(wl[i] - l_first) * vj[jb];            // u_i * v_j
                    else w = __expf(fminf(wl[i] - lj[jb], 0.f)) * dtj[jb];
                    const float dgh = (i >= j) ? w * pa[0][0][v] : 0.f;
                    dG[0][jb][v] += dgh;
                    const float pr = dgh * to_f32(G_LDS ? sG[i * LDQ + j] : Gg[i * kQ + j]);
                    rsum[v] += pr;
                    csum[jb] += pr;
                }
            }
        }
        int ri;
        const float rtot = half_wave_reduce16(rsum, &ri);
        if ((lane & 1) == 0) s_rs[(wave & 1) * kQ + rb * 32 + acc_row(lane, ri)] = rtot;
#pragma unroll
        for (int jb = 0; jb < 2; ++jb) {
            const float cs = lane_xor_add<32>(csum[jb]);
            if (lane < 32) s_cs[rb * kQ + (cb0 + jb) * 32 + lane] = cs;
        }
        __syncthreads();
        if (tid < kQ) {
            const float rs = s_rs[tid] + s_rs[kQ + tid];
            const float cs = s_cs[tid] + s_cs[kQ + tid] + s_cs[2 * kQ + tid] + s_cs[3 * kQ + tid];
            dl_diag[((b * nheads + h) * nchunks + c) * kQ + tid] = rs - cs;
        }
    }
    if (!active) return;
    float* out = dGp + (((b * nchunks + c) * ngroups + g) * nslices + slice) * (int64_t)(kQ * kQ);
#pragma unroll
    for (int jb = 0; jb < 2; ++jb) {
        if (cb0 + jb > rb) continue;
#pragma unroll
        for (int v = 0; v < 16; ++v)
            out[(rb * 32 + acc_row(lane, v)) * kQ + (cb0 + jb) * 32 + r] = dG[0][jb][v];
    }
}

// ------------------------------------------------------------------------------------------
// Off-diagonal (state) parts of dC and dB, heads of a slice reduced in registers.
// grid (nchunks, ngroups * nslices, batch), 512 threads.  Wave w owns rows rb = w >> 1 and state-column blocks
// nb0 = (w & 1) * NB .. + NB - 1 of the [kQ][N] tile.
//   SIDE_C:  dC[i][n] += e^{l_i} sum_p dy[i][p] S_prev[p][n];   dl_c[i] = C_i . (that head's contribution)
//   SIDE_B:  dB[j][n] += dt_j e^{Lam - l_j} sum_p x[j][p] dS[p][n]
// The row scale is applied in fp32 after the MFMA, so both operands are exact copies of the inputs.
template <typename T, int P, int N>
constexpr bool off_c_in_lds() { return (size_t)10 * kQ * sizeof(float) + ((size_t)(kQ + N) * lds_ld<T>(P) + (size_t)kQ * lds_ld<T>(N)) * sizeof(T) <= 150 * 1024; }

template <typename T, int P, int N, bool SIDE_C>
__global__ void __launch_bounds__(512, SIDE_C ? 2 : 4)
off_kernel(const T* __restrict__ Arow, int64_t Asb, int64_t Asl, int64_t Ash,      // dY (C side) or X (B side)
           const float* __restrict__ ldtab,
           const T* __restrict__ St,                                               // S_prev (C side) or dS (B side): [b][c][h][P][N]
           const T* __restrict__ Cm, int64_t Csb, int64_t Csl, int64_t Csg,        // C side only
           float* __restrict__ outp, float* __restrict__ dl_c,
           int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t nchunks, int64_t nslices, int64_t hps) {
    constexpr int LDP = lds_ld<T>(P);
    constexpr int NB = N / 64;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    float* wtab = reinterpret_cast<float*>(smem_raw);      // [8 waves][kQ]  row scale (wave-private)
    float* s_rc = wtab + 8 * kQ;                           // [2][kQ]
    T* sA = reinterpret_cast<T*>(s_rc + 2 * kQ);           // [kQ][LDP]
    T* sT = sA + kQ * LDP;                                 // [N][LDP]   state tile transposed

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31;
    const int64_t c = blockIdx.x, b = blockIdx.z;
    const int64_t g = blockIdx.y / nslices, slice = blockIdx.y % nslices;
    const int64_t hpg = nheads / ngroups;
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    const int rb = wave >> 1, nb0 = (wave & 1) * NB;
    float* ws = wtab + wave * kQ;

    constexpr int LDN = lds_ld<T>(N);
    T* sC = sT + N * LDP;                                  // C side: C [kQ][LDN], staged once for all heads
    constexpr bool C_LDS = off_c_in_lds<T, P, N>();
    const T* Cgl = SIDE_C ? Cm + b * Csb + t0 * Csl + g * Csg : nullptr;
    if (SIDE_C && C_LDS) stage_rows<T, kQ, N, 512, false>(sC, LDN, Cgl, Csl, valid, nullptr, tid);
    floatx16 acc[1][NB];
    acc_zero(acc);

    // the next head's row tile and state tile travel global -> registers while the current head is computed
    constexpr int V = VecTraits<T>::kVec;
    constexpr int VPR = P / V, NVA = kQ * VPR / 512;      // row tile: vectors per token row / per thread
    constexpr int VPS = N / V, NVS = P * VPS / 512;       // state tile [P][N]: vectors per row / per thread
    static_assert((kQ * VPR) % 512 == 0 && (P * VPS) % 512 == 0, "tile does not divide over the workgroup");
    uint4 pa[NVA], ps[NVS];
    auto prefetch = [&](int64_t h) {
        const T* ga = Arow + b * Asb + t0 * Asl + h * Ash;
#pragma unroll
        for (int it = 0; it < NVA; ++it) {
            const int e = it * 512 + tid, rr = e / VPR, cv = e % VPR;
            pa[it] = rr < valid ? *reinterpret_cast<const uint4*>(ga + (int64_t)rr * Asl + cv * V) : uint4{0u, 0u, 0u, 0u};
        }
        const T* gs = St + ((b * nchunks + c) * nheads + h) * (int64_t)(P * N);
#pragma unroll
        for (int it = 0; it < NVS; ++it) {
            // consecutive threads take consecutive state rows p of the same 16-byte column vector (see stage_transposed)
            const int e = it * 512 + tid, cv = e / P, pr = e % P;
            ps[it] = *reinterpret_cast<const uint4*>(gs + (int64_t)pr * N + cv * V);
        }
    };
    constexpr bool PREFETCH = SIDE_C;
    if (PREFETCH) prefetch(g * hpg + slice * hps);

    for (int64_t hh = 0; hh < hps; ++hh) {
        const int64_t h = g * hpg + slice * hps + hh;
        float l0, l1, d0, d1;
        wave_ld_load(ldtab, (b * nheads + h) * nchunks + c, l0, l1, d0, d1);
        if (SIDE_C) { ws[lane] = __expf(l0); ws[lane + 64] = __expf(l1); }
        else {
            const float Lam = __shfl(l1, 63, 64);
            ws[lane] = d0 * __expf(Lam - l0); ws[lane + 64] = d1 * __expf(Lam - l1);
        }
        __syncthreads();
        if (!PREFETCH) prefetch(h);
#pragma unroll
        for (int it = 0; it < NVA; ++it) {
            const int e = it * 512 + tid, rr = e / VPR, cv = e % VPR;
            *reinterpret_cast<uint4*>(sA + rr * LDP + cv * V) = pa[it];
        }
#pragma unroll
        for (int it = 0; it < NVS; ++it) {
            const int e = it * 512 + tid, cv = e / P, pr = e % P;
            const T* el = reinterpret_cast<const T*>(&ps[it]);
#pragma unroll
            for (int i = 0; i < V; ++i) sT[(cv * V + i) * LDP + pr] = el[i];
        }
        __syncthreads();
        if (PREFETCH && hh + 1 < hps) prefetch(h + 1);
        float rcv[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) rcv[v] = 0.f;
#pragma unroll
        for (int jn = 0; jn < NB; ++jn) {
            floatx16 tc[1][1];
            acc_zero(tc);
            wave_mma<1, 1>(tc, sA + rb * 32 * LDP, LDP, sT + (nb0 + jn) * 32 * LDP, LDP, 0, P);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float t = tc[0][0][v] * ws[rb * 32 + acc_row(lane, v)];
                acc[0][jn][v] += t;
                if (SIDE_C) {
                    const int i = rb * 32 + acc_row(lane, v), n = (nb0 + jn) * 32 + r;
                    const T cval = C_LDS ? sC[i * LDN + n] : (i < valid ? Cgl[(int64_t)i * Csl + n] : (T)0.f);
                    rcv[v] += t * to_f32(cval);
                }
            }
        }
        if (SIDE_C) {
            int ri;
            const float tot = half_wave_reduce16(rcv, &ri);
            if ((lane & 1) == 0) s_rc[(wave & 1) * kQ + rb * 32 + acc_row(lane, ri)] = tot;
            __syncthreads();
            if (tid < kQ) dl_c[((b * nheads + h) * nchunks + c) * kQ + tid] = s_rc[tid] + s_rc[kQ + tid];
        }
    }
    float* out = outp + (((b * nchunks + c) * ngroups + g) * nslices + slice) * (int64_t)(kQ * N);
#pragma unroll
    for (int jn = 0; jn < NB; ++jn)
#pragma unroll
        for (int v = 0; v < 16; ++v)
            out[(rb * 32 + acc_row(lane, v)) * N + (nb0 + jn) * 32 + r] = acc[0][jn][v];
}

// Sum of the per-slice partials (fixed order) of up to three arrays in one launch.  One thread per float4;
// `tile` floats per (group, slice) tile; segment k covers threads [first_k, first_{k+1}).
struct SliceSumSeg { const float* part; float* out; int64_t nslices, tile, first; };
struct SliceSumArgs { SliceSumSeg seg[3]; int nseg; int64_t total; };
template <int THREADS>
__device__ __forceinline__ void slice_sum_body(const SliceSumArgs& a, int64_t blk) {
    const int64_t idx = blk * THREADS + threadIdx.x;
    if (idx >= a.total) return;
    int k = 0;
    if (a.nseg > 1 && idx >= a.seg[1].first) k = 1;
    if (a.nseg > 2 && idx >= a.seg[2].first) k = 2;
    const SliceSumSeg sg = a.seg[k];
    const int64_t per = sg.tile / 4, loc = idx - sg.first;
    const int64_t grp = loc / per, e = (loc % per) * 4;
    floatx4 s = {0.f, 0.f, 0.f, 0.f};
    for (int64_t sl = 0; sl < sg.nslices; ++sl) s += *reinterpret_cast<const floatx4*>(sg.part + (grp * sg.nslices + sl) * sg.tile + e);
    *reinterpret_cast<floatx4*>(sg.out + grp * sg.tile + e) = s;
}
__global__ void __launch_bounds__(256)
slice_sum_kernel(const SliceSumArgs a) { slice_sum_body<256>(a, blockIdx.x); }
// The slice sums and the per-chunk decay-gradient scan (da_body) in one launch: they are independent, and both are short.
template <typename T>
__global__ void __launch_bounds__(kDaHeads * 64)
tail1_kernel(const DaArgs d, const int64_t n_da, const SliceSumArgs a) {
    const int64_t blk = blockIdx.x;
    if (blk < n_da) da_body<T>(d, blk);
    else slice_sum_body<kDaHeads * 64>(a, blk - n_da);
}

// ------------------------------------------------------------------------------------------
// Group-level finish for fp32 operands, one side per workgroup of 512 threads:  dC = dG B + sum dCoff  or
// dB = dG^T C + sum dBoff  (dG and the off parts already summed over the head slices).
template <typename T, int N>
__device__ __forceinline__ void
bc_final_body(const float* __restrict__ dGp, const float* __restrict__ dCp, const float* __restrict__ dBp,
              const T* __restrict__ Bt, const T* __restrict__ Ct, T* __restrict__ dB, T* __restrict__ dC,
              int64_t seqlen, int64_t ngroups, int64_t nchunks,
              int64_t dBsb, int64_t dBsl, int64_t dBsg, int64_t dCsb, int64_t dCsl, int64_t dCsg, int64_t c, int64_t g, int64_t b,
              const bool side_b) {
    static_assert(sizeof(T) == 4, "16-bit operands take bc_final16_body");
    constexpr int LDQ = lds_ld<T>(kQ);
    constexpr int NB = N / 64;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* sA2 = reinterpret_cast<T*>(smem_raw);       // [kQ][LDQ]  dG (dC side) or its transpose (dB side)
    T* sT2 = sA2 + kQ * LDQ;                       // [N][LDQ]   Bt or Ct
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31;
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    const int rb = wave >> 1, cb0 = (wave & 1) * 2, nb0 = (wave & 1) * NB;
    const int64_t grp = (b * nchunks + c) * ngroups + g;

    // inputs are already summed over the head slices (slice_sum_body)
    floatx16 dG[1][2], acc[1][NB];
    acc_zero(dG);
    {
        const float* gp = dGp + grp * (int64_t)(kQ * kQ);
        const float* op = (side_b ? dBp : dCp) + grp * (int64_t)(kQ * N);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = rb * 32 + acc_row(lane, v);
#pragma unroll
            for (int jb = 0; jb < 2; ++jb)
                if (cb0 + jb <= rb) dG[0][jb][v] = gp[row * kQ + (cb0 + jb) * 32 + r];
#pragma unroll
            for (int jn = 0; jn < NB; ++jn) acc[0][jn][v] = op[row * N + (nb0 + jn) * 32 + r];
        }
    }
    //   dC[i][n] += sum_{j<=i} dG[i][j] B[j][n]      (A = dG,   k = j in [0, 32 (rb + 1)) )
    //   dB[j][n] += sum_{i>=j} dG[i][j] C[i][n]      (A = dG^T, k = i in [32 rb, kQ) )
    const T* tile = (side_b ? Ct : Bt) + grp * (int64_t)(N * kQ);
    stage_rows<T, N, kQ, 512, false>(sT2, LDQ, tile, kQ, N, nullptr, tid);
    const int k0 = side_b ? rb * 32 : 0, k1 = side_b ? kQ : (rb + 1) * 32;
#pragma unroll
    for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int i = rb * 32 + acc_row(lane, v), j = (cb0 + jb) * 32 + r;
            sA2[side_b ? j * LDQ + i : i * LDQ + j] = dG[0][jb][v];
        }
    __syncthreads();
    wave_mma<1, NB>(acc, sA2 + rb * 32 * LDQ, LDQ, sT2 + nb0 * 32 * LDQ, LDQ, k0, k1);
    T* out = side_b ? dB + b * dBsb + t0 * dBsl + g * dBsg : dC + b * dCsb + t0 * dCsl + g * dCsg;
    const int64_t osl = side_b ? dBsl : dCsl;
#pragma unroll
    for (int jn = 0; jn < NB; ++jn)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = rb * 32 + acc_row(lane, v), col = (nb0 + jn) * 32 + r;
            if (row < valid) out[(int64_t)row * osl + col] = from_f32<T>(acc[0][jn][v]);
        }
}

// Group-level finish for 16-bit operands, both sides in one workgroup of 8 waves, so that the head-summed dG is read once:
//   waves 0-3 (row block w):      dC[i][n] = sum_{j<=i} dG[i][j] B[j][n] + dCoff[i][n]
//   waves 4-7 (row block w - 4):  dB[j][n] = sum_{i>=j} dG[i][j] C[i][n] + dBoff[j][n]
// (wave w and wave w + 4 share a SIMD: 2w + 2 and 8 - 2w k blocks, ten on every SIMD).  dG is split into hi + lo
// operand-type tiles in LDS (row-major, 16-byte slots swizzled as everywhere), so the contractions see it at ~2^-17
// relative: the dC side reads its fragments row-wise, the dB side, which needs dG^T, through LDS transpose reads.  B^T / C^T
// fragments come straight from the operand-order tiles (one contiguous KiB per fragment), the MFMAs are issued with swapped
// operands, so a lane owns one token: the accumulators start from 16-byte loads of the summed state parts and leave as
// 16-byte stores after one lane-pair swap per 4-column group.  One barrier, no pass of the results through LDS.
// With few (batch, chunk, group) triples the launch is latency-bound and more, shorter workgroups win: BOTH = false runs
// one side per workgroup (`side_b`), wave w and w + 4 taking the two halves of the state columns of row block w & 3, with
// all B^T / C^T fragments requested before the barrier.
template <typename T, int N, bool BOTH>
__device__ __forceinline__ void
bc_final16_body(const float* __restrict__ dGs, const float* __restrict__ dCs, const float* __restrict__ dBs,
                const T* __restrict__ Bt, const T* __restrict__ Ct, T* __restrict__ dB, T* __restrict__ dC,
                int64_t seqlen, int64_t ngroups, int64_t nchunks,
                int64_t dBsb, int64_t dBsl, int64_t dBsg, int64_t dCsb, int64_t dCsl, int64_t dCsg, int64_t c, int64_t g, int64_t b,
                const bool wg_side_b) {
    static_assert(sizeof(T) == 2, "16-bit operands only");
    constexpr int NBN = BOTH ? N / 32 : N / 64, SPR = kQ / 8;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* sH = reinterpret_cast<T*>(smem_raw);      // [kQ][kQ] hi part of dG
    T* sL = sH + kQ * kQ;                        // [kQ][kQ] lo part
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31, half = lane >> 5;
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    const int64_t grp = (b * nchunks + c) * ngroups + g;
    {
        const float* gp = dGs + grp * (int64_t)(kQ * kQ);
#pragma unroll
        for (int it = 0; it < kQ * kQ / 4 / 512; ++it) {
            const int e = it * 512 + tid, i = e / (kQ / 4), j4 = (e % (kQ / 4)) * 4;
            floatx4 v = floatx4{0.f, 0.f, 0.f, 0.f};
            if ((j4 >> 5) <= (i >> 5)) v = *reinterpret_cast<const floatx4*>(gp + i * kQ + j4);      // blocks above the diagonal are never written
            const T h0 = from_f32<T>(v[0]), h1 = from_f32<T>(v[1]), h2 = from_f32<T>(v[2]), h3 = from_f32<T>(v[3]);
            const uint2 hw = {pack2<T>(to_f32(h0), to_f32(h1)), pack2<T>(to_f32(h2), to_f32(h3))};
            const uint2 lw = {pack2<T>(v[0] - to_f32(h0), v[1] - to_f32(h1)), pack2<T>(v[2] - to_f32(h2), v[3] - to_f32(h3))};
            const int at = (i * SPR + ((j4 >> 3) ^ tile_swz<SPR>(i))) * 8 + (j4 & 7);
            *reinterpret_cast<uint2*>(sH + at) = hw;
            *reinterpret_cast<uint2*>(sL + at) = lw;
        }
    }
    const bool side_b = BOTH ? wave >= 4 : wg_side_b;
    const int rb = wave & 3, tok = rb * 32 + r;
    const int n0 = BOTH ? 0 : (wave >> 2) * (N / 2);      // first state column of this wave
    floatx16 acc[NBN];
    {
        const float* op = (side_b ? dBs : dCs) + grp * (int64_t)(kQ * N) + (int64_t)tok * N + n0;
#pragma unroll
        for (int nb = 0; nb < NBN; ++nb)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const floatx4 v = *reinterpret_cast<const floatx4*>(op + nb * 32 + 8 * q + 4 * half);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[nb][4 * q + e] = v[e];
            }
    }
    const char* tile = reinterpret_cast<const char*>((side_b ? Ct : Bt) + grp * (int64_t)(N * kQ)) + (n0 / 32) * (8 * 1024);
    const int ks0 = side_b ? 2 * rb : 0, ks1 = side_b ? 8 : 2 * rb + 2;      // 16-wide k blocks of this wave
    Frag<T> xpre[BOTH ? 1 : 8][NBN];
    if constexpr (!BOTH) {
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
            if (ks >= ks0 && ks < ks1) {
#pragma unroll
                for (int nb = 0; nb < NBN; ++nb)
                    xpre[ks][nb].v = *reinterpret_cast<const bf16x8*>(tile + ((uint32_t)lane * 16u + (uint32_t)((nb * 8 + ks) * 1024)));
            }
    }
    __syncthreads();
    const int tr_tok = 8 * half + ((lane >> 2) & 3), tr_col = rb * 32 + ((lane >> 4) & 1) * 16 + 4 * (lane & 3);
    typedef T tvec4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
        if (ks < ks0 || ks >= ks1) continue;      // wave-uniform
        Frag<T> yh, yl;
        if (!side_b) {
            const int at = (tok * SPR + ((ks * 2 + half) ^ tile_swz<SPR>(tok))) * 8;
            yh = load_frag(sH + at);
            yl = load_frag(sL + at);
        } else {
            const int ta = ks * 16 + tr_tok, tb = ta + 4;
            const int aa = (ta * SPR + ((tr_col >> 3) ^ tile_swz<SPR>(ta))) * 8 + (tr_col & 7);
            const int ab = (tb * SPR + ((tr_col >> 3) ^ tile_swz<SPR>(tb))) * 8 + (tr_col & 7);
            const tvec4 h0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((M2_LDS tvec4*)(sH + aa));
            const tvec4 h1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((M2_LDS tvec4*)(sH + ab));
            const tvec4 l0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((M2_LDS tvec4*)(sL + aa));
            const tvec4 l1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((M2_LDS tvec4*)(sL + ab));
#pragma unroll
            for (int e = 0; e < 4; ++e) { yh.v[e] = h0[e]; yh.v[4 + e] = h1[e]; yl.v[e] = l0[e]; yl.v[4 + e] = l1[e]; }
        }
#pragma unroll
        for (int nb = 0; nb < NBN; ++nb) {
            Frag<T> xf;      // see mt_offset
            if constexpr (BOTH) xf.v = *reinterpret_cast<const bf16x8*>(tile + ((uint32_t)lane * 16u + (uint32_t)((nb * 8 + ks) * 1024)));
            else xf = xpre[ks][nb];
            mma_frag(acc[nb], xf, yh);
            mma_frag(acc[nb], xf, yl);
        }
    }
    T* out = (side_b ? dB + b * dBsb + t0 * dBsl + g * dBsg : dC + b * dCsb + t0 * dCsl + g * dCsg) + (int64_t)tok * (side_b ? dBsl : dCsl) + n0;
#pragma unroll
    for (int nb = 0; nb < NBN; ++nb)
#pragma unroll
        for (int qp = 0; qp < 2; ++qp) {
            float g8[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) pair_swap(acc[nb][8 * qp + e], acc[nb][8 * qp + 4 + e], g8[e], g8[4 + e]);
            const uint4 o = {pack2<T>(g8[0], g8[1]), pack2<T>(g8[2], g8[3]), pack2<T>(g8[4], g8[5]), pack2<T>(g8[6], g8[7])};
            if (tok < valid) *reinterpret_cast<uint4*>(out + nb * 32 + 8 * (2 * qp + half)) = o;
        }
}

// dA[h] = sum_{b,c} dAp[b][h][c], dD likewise (fixed order, no atomics).  One workgroup of 512 threads per head.
__device__ __forceinline__ void ad_reduce_body(const float* __restrict__ dAp, const float* __restrict__ dDp, const float* __restrict__ dbp,
                                               float* __restrict__ dA, float* __restrict__ dD, float* __restrict__ dbias,
                                               int64_t nb, int64_t nheads, int64_t nchunks, int64_t h) {
    __shared__ float red[3][8];
    float sa = 0.f, sd = 0.f, sb = 0.f;
    for (int64_t e = threadIdx.x; e < nb * nchunks; e += 512) {
        const int64_t b = e / nchunks, c = e % nchunks;
        sa += dAp[(b * nheads + h) * nchunks + c];
        sd += dDp[(b * nheads + h) * nchunks + c];
        if (dbias) sb += dbp[(b * nheads + h) * nchunks + c];
    }
    sa = warp_sum(sa); sd = warp_sum(sd); sb = warp_sum(sb);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) { red[0][wave] = sa; red[1][wave] = sd; red[2][wave] = sb; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float ta = 0.f, td = 0.f, tb = 0.f;
#pragma unroll
        for (int q = 0; q < 8; ++q) { ta += red[0][q]; td += red[1][q]; tb += red[2][q]; }
        dA[h] = ta;
        if (dD) dD[h] = td;
        if (dbias) dbias[h] = tb;
    }
}

// The group-level finish and the per-head reductions in one launch: the first workgroups run the group finish for
// ([side,] chunk, group, batch) = the index split in that order (fp32 operands: side 0 dC, side 1 dB, one workgroup each;
// 16-bit operands with BOTH: both sides in one workgroup), the others ad_reduce_body for one head each.
constexpr int64_t kTail2BothFrom = 256;      // (batch, chunk, group) triples from which a workgroup takes both sides: one per CU
struct Tail2Args {
    const float* dGp; const float* dCp; const float* dBp; const void* Bt; const void* Ct; void* dB; void* dC;
    int64_t dBsb, dBsl, dBsg, dCsb, dCsl, dCsg;
    const float* dAp; const float* dDp; const float* dbp; float* dA; float* dD; float* dbias;
    int64_t seqlen, ngroups, nchunks, batch, nheads, n_bc;
};
template <typename T, int N, bool BOTH>
__global__ void __launch_bounds__(512)
tail2_kernel(const Tail2Args a) {
    const int64_t blk = blockIdx.x;
    constexpr int SIDES = BOTH ? 1 : 2;
    static_assert(!BOTH || sizeof(T) == 2, "both sides in one workgroup: 16-bit operands only");
    if (blk < SIDES * a.n_bc) {
        const int64_t q = blk / SIDES;
        const int64_t c = q % a.nchunks, g = (q / a.nchunks) % a.ngroups, b = q / (a.nchunks * a.ngroups);
        if constexpr (sizeof(T) == 2) {
            bc_final16_body<T, N, BOTH>(a.dGp, a.dCp, a.dBp, static_cast<const T*>(a.Bt), static_cast<const T*>(a.Ct), static_cast<T*>(a.dB),
                                        static_cast<T*>(a.dC), a.seqlen, a.ngroups, a.nchunks, a.dBsb, a.dBsl, a.dBsg, a.dCsb, a.dCsl, a.dCsg, c, g,
                                        b, (blk & 1) != 0);
        } else {
            bc_final_body<T, N>(a.dGp, a.dCp, a.dBp, static_cast<const T*>(a.Bt), static_cast<const T*>(a.Ct), static_cast<T*>(a.dB),
                                static_cast<T*>(a.dC), a.seqlen, a.ngroups, a.nchunks, a.dBsb, a.dBsl, a.dBsg, a.dCsb, a.dCsl, a.dCsg, c, g, b,
                                (blk & 1) != 0);
        }
    } else {
        ad_reduce_body(a.dAp, a.dDp, a.dbp, a.dA, a.dD, a.dbias, a.batch, a.nheads, a.nchunks, blk - SIDES * a.n_bc);
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

template <typename T, int P>
size_t dg_smem() { return (size_t)(8 * kQ + 2 * kQ + 4 * kQ) * sizeof(float) + ((size_t)2 * kQ * lds_ld<T>(P) + (dg_g_in_lds<T, P>() ? (size_t)kQ * lds_ld<T>(kQ) : 0)) * sizeof(T); }
template <typename T, int P, int N>
size_t off_smem(bool side_c) { return (size_t)(8 * kQ + 2 * kQ) * sizeof(float) + ((size_t)(kQ + N) * lds_ld<T>(P) + ((side_c && off_c_in_lds<T, P, N>()) ? (size_t)kQ * lds_ld<T>(N) : 0)) * sizeof(T); }
template <typename T, int N>
size_t bcf_smem() { return sizeof(T) == 2 ? (size_t)2 * kQ * kQ * sizeof(T) : (size_t)(kQ + N) * lds_ld<T>(kQ) * sizeof(T); }

template <typename T, int P, int N>
int ssd_bwd_impl(const m2_ssd_params* p, hipStream_t st) {
    const int64_t nc = ceil_div(p->seqlen, (int64_t)kQ);
    const SsdWorkspace w = ssd_carve(p, p->workspace, true);
    const int dt_f32 = p->dt_dtype == M2_F32;
    const T* x = static_cast<const T*>(p->x);
    const T* Cm = static_cast<const T*>(p->C);
    const T* dy = static_cast<const T*>(p->dy);
    const dim3 grid_g((unsigned)nc, (unsigned)(p->ngroups * w.ns_g), (unsigned)p->batch);
    const dim3 grid_c((unsigned)nc, (unsigned)(p->ngroups * w.ns_c), (unsigned)p->batch);
    const dim3 grid_b((unsigned)nc, (unsigned)(p->ngroups * w.ns_b), (unsigned)p->batch);
    M2_REQUIRE(p->nheads <= 65535, M2_ERR_SHAPE, "ssd_bwd: too many group slices");
    int rc;
    // decay tables, G (+ operand tiles) and the state entering each chunk, unless the caller kept the forward's
    if (!p->chunk_states && (rc = ssd_launch_states<T, P, N>(p, w, nullptr, st))) return rc;
    // gradient of the state leaving each chunk (reverse recurrence over the chunks' own contributions)
    if constexpr (sizeof(T) == 2) {
        // the main backward kernel forms dlam itself when it runs; otherwise this pass does (and reads the forward states for it)
        constexpr int SPLIT = kStatePassSplit;
        auto k = state_pass16_kernel<T, P, N, true, !bwd16_ok<T, P, N>(), false, SPLIT>;
        const size_t sm = state_pass_smem<P, N, false, SPLIT>();
        if ((rc = allow_smem(k, sm))) return rc;
        StatePassArgs sa;
        sa.X = dy; sa.X_sb = p->dy_stride_b; sa.X_sl = p->dy_stride_l; sa.X_sh = p->dy_stride_h;
        sa.ldtab = w.ldtab; sa.Mt = w.Ct; sa.init = p->d_final_state; sa.prev = w.dprev; sa.final_out = p->d_initial_state;
        sa.sprev = w.prev; sa.dlam = w.dlam;
        sa.seqlen = p->seqlen; sa.nheads = p->nheads; sa.ngroups = p->ngroups; sa.nchunks = nc;
        k<<<dim3((unsigned)(p->nheads * SPLIT), (unsigned)p->batch), state_pass_threads<N>(), sm, st>>>(sa);
        if ((rc = check_launch("ssd state_pass16_kernel<reverse>"))) return rc;
    } else
    {   // fp32: local dS contributions (reuses the `local` region), then the reverse recurrence
        auto k = chunk_state_kernel<T, P, N, true>;
        const size_t sm = state_smem<T, P, N>();
        if ((rc = allow_smem(k, sm))) return rc;
        int64_t ns, hps;
        ssd_slicing(p, kWgsChunkState, &ns, &hps);
        k<<<dim3((unsigned)nc, (unsigned)(p->ngroups * ns), (unsigned)p->batch), 256, sm, st>>>(
            dy, w.ldtab, static_cast<const T*>(w.Ct), w.local, p->seqlen, p->nheads, p->ngroups, nc, ns, hps,
            p->dy_stride_b, p->dy_stride_l, p->dy_stride_h);
        if ((rc = check_launch("ssd chunk_state_kernel<dstate>"))) return rc;
        state_scan_kernel<T, P * N, true><<<dim3((unsigned)p->nheads, (unsigned)p->batch, kScanSplit), 256, 0, st>>>(
            w.local, w.lam, p->d_final_state, static_cast<T*>(w.dprev), p->d_initial_state,
            static_cast<const T*>(w.prev), w.dlam, p->nheads, nc);
        if ((rc = check_launch("ssd state_scan_kernel<reverse>"))) return rc;
    }
    {
        if constexpr (sizeof(T) == 2 && dg16_smem<P>() <= 160 * 1024) {
            auto k = dg16_kernel<T, P>;
            const size_t sm = dg16_smem<P>();
            if ((rc = allow_smem(k, sm))) return rc;
            k<<<grid_g, kDgWaves * 64, sm, st>>>(x, w.ldtab, dy, w.G, w.dGp, w.dl,
                                       p->seqlen, p->nheads, p->ngroups, nc, w.ns_g, w.hps_g,
                                       p->x_stride_b, p->x_stride_l, p->x_stride_h,
                                       p->dy_stride_b, p->dy_stride_l, p->dy_stride_h);
        } else {
            auto k = dg_kernel<T, P>;
            const size_t sm = dg_smem<T, P>();
            if ((rc = allow_smem(k, sm))) return rc;
            k<<<grid_g, 512, sm, st>>>(x, w.ldtab, dy, static_cast<const T*>(w.Gm), w.dGp, w.dl,
                                       p->seqlen, p->nheads, p->ngroups, nc, w.ns_g, w.hps_g,
                                       p->x_stride_b, p->x_stride_l, p->x_stride_h,
                                       p->dy_stride_b, p->dy_stride_l, p->dy_stride_h);
        }
        if ((rc = check_launch("ssd dg_kernel"))) return rc;
    }
    DaArgs da{};
    bool have_da = false;
    {
        if constexpr (!bwd16_ok<T, P, N>()) {
        auto kc = off_kernel<T, P, N, true>;
        auto kb = off_kernel<T, P, N, false>;
        const size_t smc = off_smem<T, P, N>(true), sm = off_smem<T, P, N>(false);
        if ((rc = allow_smem(kc, smc))) return rc;
        if ((rc = allow_smem(kb, sm))) return rc;
        kc<<<grid_c, 512, smc, st>>>(dy, p->dy_stride_b, p->dy_stride_l, p->dy_stride_h, w.ldtab,
                                    static_cast<const T*>(w.prev), Cm, p->C_stride_b, p->C_stride_l, p->C_stride_g,
                                    w.dCp, w.dlc, p->seqlen, p->nheads, p->ngroups, nc, w.ns_c, w.hps_c);
        if ((rc = check_launch("ssd off_kernel<C>"))) return rc;
        kb<<<grid_b, 512, sm, st>>>(x, p->x_stride_b, p->x_stride_l, p->x_stride_h, w.ldtab,
                                    static_cast<const T*>(w.dprev), nullptr, 0, 0, 0,
                                    w.dBp, nullptr, p->seqlen, p->nheads, p->ngroups, nc, w.ns_b, w.hps_b);
        if ((rc = check_launch("ssd off_kernel<B>"))) return rc;
        }
    }
    {
        DiagArgs a{};
        a.dt = p->dt; a.dt_f32 = dt_f32; a.A = p->A; a.D = p->D;
        a.Aoff = p->B; a.Ao_sb = p->B_stride_b; a.Ao_sl = p->B_stride_l; a.Ao_sg = p->B_stride_g;
        a.Gd = w.Gmt; a.S = w.dprev;
        a.Z = p->dy; a.Z_sb = p->dy_stride_b; a.Z_sl = p->dy_stride_l; a.Z_sh = p->dy_stride_h;
        a.dt_sb = p->dt_stride_b; a.dt_sl = p->dt_stride_l;
        a.seqlen = p->seqlen; a.nheads = p->nheads; a.ngroups = p->ngroups; a.nchunks = nc;
        ssd_slicing(p, 2, &a.nslices, &a.hps);
        a.X = p->x; a.X_sb = p->x_stride_b; a.X_sl = p->x_stride_l; a.X_sh = p->x_stride_h;
        a.dX = p->dx; a.dX_sb = p->dx_stride_b; a.dX_sl = p->dx_stride_l; a.dX_sh = p->dx_stride_h;
        a.ddt = p->ddt; a.ddt_sb = p->ddt_stride_b; a.ddt_sl = p->ddt_stride_l;
        a.ldtab = w.ldtab;
        a.dl_diag = w.dl; a.dl_c = w.dlc; a.dlam = w.dlam; a.dAp = w.dAp; a.dDp = w.dDp;
        a.dbp = p->dt_bias ? w.dbp : nullptr;
        const dim3 grid((unsigned)nc, (unsigned)(p->ngroups * a.nslices), (unsigned)p->batch);
        if constexpr (bwd16_ok<T, P, N>()) {
            Bwd16Args m{};
            m.ldtab = w.ldtab; m.D = p->D;
            m.Bm = p->B; m.B_sb = p->B_stride_b; m.B_sl = p->B_stride_l; m.B_sg = p->B_stride_g;
            m.Cm = p->C; m.C_sb = p->C_stride_b; m.C_sl = p->C_stride_l; m.C_sg = p->C_stride_g;
            m.Gmt = w.Gmt; m.dS = w.dprev; m.Sprev = w.prev;
            m.dy = p->dy; m.dy_sb = p->dy_stride_b; m.dy_sl = p->dy_stride_l; m.dy_sh = p->dy_stride_h;
            m.x = p->x; m.x_sb = p->x_stride_b; m.x_sl = p->x_stride_l; m.x_sh = p->x_stride_h;
            m.dx = p->dx; m.dx_sb = p->dx_stride_b; m.dx_sl = p->dx_stride_l; m.dx_sh = p->dx_stride_h;
            m.dirp = w.dirp; m.rbp = w.rbp; m.dlc = w.dlc; m.dDp8 = w.dDp8; m.dlam = w.dlam; m.dBp = w.dBp; m.dCp = w.dCp;
            m.seqlen = p->seqlen; m.nheads = p->nheads; m.ngroups = p->ngroups; m.nchunks = nc;
            m.nslices = w.ns_b; m.hps = w.hps_b;
            auto k = ssd_bwd16_kernel<T, P, N>;
            const size_t sm = bwd16_smem<P, N>();
            if ((rc = allow_smem(k, sm))) return rc;
            k<<<grid_b, 512, sm, st>>>(m);
            if ((rc = check_launch("ssd_bwd16_kernel"))) return rc;
            // the per-chunk scan that turns these per-token terms into ddt and dA partials runs with the slice sums below
            have_da = true;
            da.ldtab = w.ldtab; da.A = p->A; da.dl_diag = w.dl; da.dl_c = w.dlc; da.dlam = w.dlam;
            da.dirp = w.dirp; da.rbp = w.rbp; da.dDp8 = w.dDp8;
            da.ddt = p->ddt; da.dt_f32 = dt_f32; da.ddt_sb = p->ddt_stride_b; da.ddt_sl = p->ddt_stride_l; da.dAp = w.dAp; da.dDp = w.dDp;
            da.dbp = p->dt_bias ? w.dbp : nullptr;
            da.seqlen = p->seqlen; da.nheads = p->nheads; da.nchunks = nc; da.batch = p->batch;
        } else {
            auto k = diag_off_kernel<T, P, N, true>;
            const size_t sm = diag_smem<T, P, N, true>();
            if ((rc = allow_smem(k, sm))) return rc;
            k<<<grid, 256, sm, st>>>(a);
        }
        if ((rc = check_launch("ssd diag_off_kernel<bwd>"))) return rc;
    }
    {
        const int64_t ngrp = p->batch * nc * p->ngroups;
        const float *gs = w.dGp, *cs = w.dCp, *bs = w.dBp;
        {
            SliceSumArgs sa{};
            int64_t first = 0;
            auto add = [&](const float* part, float* out, int64_t ns, int64_t tile, const float** use) {
                if (ns <= 1) return;
                sa.seg[sa.nseg++] = SliceSumSeg{part, out, ns, tile, first};
                first += ngrp * tile / 4;
                *use = out;
            };
            add(w.dGp, w.dGs, w.ns_g, (int64_t)kQ * kQ, &gs);
            add(w.dCp, w.dCs, w.ns_c, (int64_t)kQ * N, &cs);
            add(w.dBp, w.dBs, w.ns_b, (int64_t)kQ * N, &bs);
            sa.total = first;
            if (have_da) {
                const int64_t n_da = da_blocks(da), n_ss = ceil_div(first, (int64_t)(kDaHeads * 64));
                tail1_kernel<T><<<(unsigned)(n_da + n_ss), kDaHeads * 64, 0, st>>>(da, n_da, sa);
            } else if (first > 0) {
                slice_sum_kernel<<<(unsigned)ceil_div(first, (int64_t)256), 256, 0, st>>>(sa);
            }
        }
        if ((rc = check_launch("ssd tail1_kernel"))) return rc;
        // 16-bit operands: one workgroup per (batch, chunk, group) once those alone fill the chip, one per side below that
        const bool both = sizeof(T) == 2 && ngrp >= kTail2BothFrom;
        auto k = tail2_kernel<T, N, false>;
        if constexpr (sizeof(T) == 2) { if (both) k = tail2_kernel<T, N, true>; }
        const size_t sm = bcf_smem<T, N>();
        if ((rc = allow_smem(k, sm))) return rc;
        Tail2Args ta;
        ta.dGp = gs; ta.dCp = cs; ta.dBp = bs; ta.Bt = w.Bt; ta.Ct = w.Ct; ta.dB = p->dB; ta.dC = p->dC;
        ta.dBsb = p->dB_stride_b; ta.dBsl = p->dB_stride_l; ta.dBsg = p->dB_stride_g;
        ta.dCsb = p->dC_stride_b; ta.dCsl = p->dC_stride_l; ta.dCsg = p->dC_stride_g;
        ta.dAp = w.dAp; ta.dDp = w.dDp; ta.dbp = w.dbp; ta.dA = p->dA; ta.dD = p->D ? p->dD : nullptr;
        ta.dbias = p->dt_bias ? p->d_dt_bias : nullptr;
        ta.seqlen = p->seqlen; ta.ngroups = p->ngroups; ta.nchunks = nc; ta.batch = p->batch; ta.nheads = p->nheads; ta.n_bc = ngrp;
        k<<<(unsigned)((both ? 1 : 2) * ngrp + p->nheads), 512, sm, st>>>(ta);
        if ((rc = check_launch("ssd tail2_kernel"))) return rc;
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
    M2_REQUIRE(!p->dt_bias || p->d_dt_bias, M2_ERR_NULL, "ssd_bwd: d_dt_bias is required when dt_bias is given");
    if (p->batch == 0 || p->seqlen == 0) {
        // empty reductions: parameter gradients are zero; the state gradient passes straight through
        zero_f32_kernel<<<(unsigned)ceil_div(p->nheads, (int64_t)256), 256, 0, st>>>(p->dA, p->nheads);
        if (p->dD) zero_f32_kernel<<<(unsigned)ceil_div(p->nheads, (int64_t)256), 256, 0, st>>>(p->dD, p->nheads);
        if (p->dt_bias) zero_f32_kernel<<<(unsigned)ceil_div(p->nheads, (int64_t)256), 256, 0, st>>>(p->d_dt_bias, p->nheads);
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
    // the gradients leave as 16-byte row stores
    M2_REQUIRE(p->dx_stride_b % V == 0 && p->dx_stride_l % V == 0 && p->dx_stride_h % V == 0 && aligned16(p->dx) &&
               p->dB_stride_b % V == 0 && p->dB_stride_l % V == 0 && p->dB_stride_g % V == 0 && aligned16(p->dB) &&
               p->dC_stride_b % V == 0 && p->dC_stride_l % V == 0 && p->dC_stride_g % V == 0 && aligned16(p->dC), M2_ERR_ALIGN,
               "ssd_bwd: dx, dB, dC must be 16-byte aligned with strides that are multiples of %d elements", V);
    const size_t need = m2_ssd_bwd_workspace_bytes(p);
    M2_REQUIRE(p->workspace && p->workspace_bytes >= need, M2_ERR_WORKSPACE, "ssd_bwd: workspace %zu bytes < %zu needed",
               p->workspace_bytes, need);
    M2_REQUIRE((reinterpret_cast<uintptr_t>(p->workspace) & 255u) == 0, M2_ERR_ALIGN, "ssd_bwd: workspace must be 256-byte aligned");
    M2_DISPATCH_DTYPE(p->dtype, T, M2_DISPATCH_PN(p, P, N, return (ssd_bwd_impl<T, P, N>(p, st))));
    return M2_OK;
}
