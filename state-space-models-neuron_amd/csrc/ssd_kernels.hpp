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
// The last two serve fp32 operands; for 16-bit operands ssd_states16.hpp does both in one pass.
#pragma once
#include "mma.hpp"

namespace m2 {


// ------------------------------------------------------------------------------------------
// Per (batch, chunk, group): G = C B^T and the head-independent operand tiles every other kernel reuses.
//   Gf  [kQ][kQ] fp32            G[i][j] (all blocks with block-row >= block-col)
//   Gm  [kQ][kQ] T               causal G:  G[i][j] for i >= j, else 0         (forward diagonal term, rows i)
//   Gmt [kQ][kQ] T               its transpose: Gmt[j][i] = G[i][j] for i >= j (backward dx term, rows j)
//   Bt, Ct N x kQ T              B and C transposed (tokens contiguous), laid out by mt_offset: MFMA operands of the
//                                chunk-state products
// kCbParts workgroups of 256 threads per (chunk, group, batch), see cb_body.  The upper-right 64x64 quadrant of G is
// never consumed and is neither computed nor written.
// Element offset of the 8 tokens s0 .. s0 + 7 (s0 a multiple of 8) of state column n inside a transposed B / C tile.
//   fp32   : [N][kQ], tokens contiguous (rows staged into LDS by chunk_state_kernel);
//   16-bit : MFMA operand order [N / 32][kQ / 16][64 lanes][8]: the B-operand fragment of a wave for column block n / 32
//            and k-step s0 / 16 is one contiguous KiB, lane = 32 ((s0 / 8) & 1) + n % 32 (read by state_pass16_kernel
//            straight into registers, eight full cache lines per load instruction).
template <typename T>
__device__ __forceinline__ int64_t mt_offset(int n, int s0) {
    if (sizeof(T) == 2) return ((int64_t)((n >> 5) * (kQ / 16) + (s0 >> 4)) * 64 + ((s0 >> 3) & 1) * 32 + (n & 31)) * 8;
    return (int64_t)n * kQ + s0;
}

// Workgroups per (chunk, group, batch): three for the 64x64 quadrants of G on and below the diagonal, four for the
// transposed tiles (32 tokens each) -- seven short independent pieces rather than two long ones.
constexpr int kCbParts = 7;
template <typename T, int N>
__device__ __forceinline__ void
cb_body(const T* __restrict__ Bm, const T* __restrict__ Cm, float* __restrict__ Gf, T* __restrict__ Gm, T* __restrict__ Gmt,
        T* __restrict__ Bt, T* __restrict__ Ct,
        int64_t seqlen, int64_t ngroups, int64_t nchunks,
        int64_t Bsb, int64_t Bsl, int64_t Bsg, int64_t Csb, int64_t Csl, int64_t Csg, int64_t c, int64_t g, int64_t b,
        const int part) {
    constexpr int LD = lds_ld<T>(N);      // the whole contraction length at once: one staging phase, one barrier
    constexpr int V = VecTraits<T>::kVec;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* sC = reinterpret_cast<T*>(smem_raw);      // [64][LD]
    T* sB = sC + 64 * LD;                        // [64][LD]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    const T* Bp = Bm + b * Bsb + t0 * Bsl + g * Bsg;
    const T* Cp = Cm + b * Csb + t0 * Csl + g * Csg;
    const int64_t grp = (b * nchunks + c) * ngroups + g;
    if (part >= 3) {
        // transposed copies of tokens [tk0, tk0 + 32): thread -> (state column n, group of V tokens)
        const int tk0 = (part - 3) * 32;
        T* Btp = Bt + grp * (int64_t)(N * kQ);
        T* Ctp = Ct + grp * (int64_t)(N * kQ);
        stage_rows<T, 32, N, 256, false>(sC, LD, Cp + (int64_t)tk0 * Csl, Csl, valid - tk0, nullptr, tid);
        stage_rows<T, 32, N, 256, false>(sB, LD, Bp + (int64_t)tk0 * Bsl, Bsl, valid - tk0, nullptr, tid);
        __syncthreads();
        for (int e = tid; e < N * (32 / V); e += 256) {
            const int n = e % N, s0 = (e / N) * V;
            T vb[V], vc[V];
#pragma unroll
            for (int q = 0; q < V; ++q) { vb[q] = sB[(s0 + q) * LD + n]; vc[q] = sC[(s0 + q) * LD + n]; }
            *reinterpret_cast<uint4*>(Btp + mt_offset<T>(n, tk0 + s0)) = *reinterpret_cast<const uint4*>(vb);
            *reinterpret_cast<uint4*>(Ctp + mt_offset<T>(n, tk0 + s0)) = *reinterpret_cast<const uint4*>(vc);
        }
        return;
    }
    // quadrant (wm, wn) of G = C B^T; wave (wi, wj) takes one 32x32 block of it
    const int wm = part == 0 ? 0 : 1, wn = part == 2 ? 1 : 0;
    const int wi = wave >> 1, wj = wave & 1;
    stage_rows<T, 64, N, 256, false>(sC, LD, Cp + (int64_t)(wm * 64) * Csl, Csl, valid - wm * 64, nullptr, tid);
    stage_rows<T, 64, N, 256, false>(sB, LD, Bp + (int64_t)(wn * 64) * Bsl, Bsl, valid - wn * 64, nullptr, tid);
    __syncthreads();
    if (wm * 2 + wi < wn * 2 + wj) return;          // block above the diagonal
    floatx16 acc[1][1];
    acc_zero(acc);
    wave_mma<1, 1>(acc, sC + wi * 32 * LD, LD, sB + wj * 32 * LD, LD, 0, N);
    float* Gfp = Gf + grp * (int64_t)(kQ * kQ);
    T* Gmp = Gm + grp * (int64_t)(kQ * kQ);
    T* Gmtp = Gmt + grp * (int64_t)(kQ * kQ);
    const int col = wn * 64 + wj * 32 + acc_col(lane);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int rowq = wm * 64 + wi * 32 + 8 * q + 4 * (lane >> 5);
        T mt[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = rowq + e;
            const float gv = acc[0][0][4 * q + e];
            const float gm = row >= col ? gv : 0.f;
            Gfp[row * kQ + col] = gv;
            Gmp[row * kQ + col] = from_f32<T>(gm);
            mt[e] = from_f32<T>(gm);
        }
        *reinterpret_cast<RawVec<T, 4>*>(Gmtp + col * kQ + rowq) = *reinterpret_cast<const RawVec<T, 4>*>(mt);
    }
}

// ------------------------------------------------------------------------------------------
// Cumulative log-decay table: one wave per (batch, head, chunk); ldtab[bhc] = [ l[0..kQ) | dt[0..kQ) ] in fp32,
// l = inclusive cumsum of A_h dt within the chunk, lam[bhc] = l[kQ-1].  Every other kernel reads this table instead
// of gathering dt (stride = nheads elements) and scanning it again per head.  The four waves of a workgroup take four
// consecutive heads of one (batch, chunk): dt is [b][l][h], so a token's four values are 8 (fp32: 16) consecutive bytes
// and are fetched by one thread per token and handed to the waves through LDS, instead of 128 two-byte gathers per wave.
constexpr int kLdHeads = 4;
inline int64_t ld_table_blocks(int64_t batch, int64_t nheads, int64_t nchunks) { return batch * nchunks * ((nheads + kLdHeads - 1) / kLdHeads); }
template <typename T>
__device__ __forceinline__ void
ld_table_body(const void* __restrict__ dt, int dt_f32, const float* __restrict__ dt_bias, const float* __restrict__ A, float* __restrict__ ldtab,
              float* __restrict__ lam, int64_t seqlen, int64_t nheads, int64_t nchunks,
              int64_t dtsb, int64_t dtsl, int64_t blk) {
    __shared__ float sdt[kLdHeads][kQ];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t hgroups = (nheads + kLdHeads - 1) / kLdHeads;
    const int64_t hg = blk % hgroups, c = (blk / hgroups) % nchunks, b = blk / (hgroups * nchunks);
    const int64_t h0 = hg * kLdHeads, h = h0 + wave;
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    const int hc = (int)(nheads - h0 < kLdHeads ? nheads - h0 : kLdHeads);
    if (threadIdx.x < kQ) {
        const int t = threadIdx.x;
        float v[kLdHeads] = {0.f, 0.f, 0.f, 0.f};      // tokens past the end of the sequence behave as dt = 0
        if (t < valid) {
            const int64_t off = b * dtsb + (t0 + t) * dtsl + h0;
            if (dt_f32) {
                const float* p = static_cast<const float*>(dt) + off;
                if (hc == kLdHeads && (reinterpret_cast<uintptr_t>(p) & 15) == 0) {
                    const floatx4 q = *reinterpret_cast<const floatx4*>(p);
#pragma unroll
                    for (int k = 0; k < kLdHeads; ++k) v[k] = q[k];
                } else {
                    for (int k = 0; k < hc; ++k) v[k] = p[k];
                }
            } else {
                const T* p = static_cast<const T*>(dt) + off;
                if (hc == kLdHeads && (reinterpret_cast<uintptr_t>(p) & (kLdHeads * sizeof(T) - 1)) == 0) {
                    const RawVec<T, kLdHeads> q = *reinterpret_cast<const RawVec<T, kLdHeads>*>(p);
                    const T* e = reinterpret_cast<const T*>(&q);
#pragma unroll
                    for (int k = 0; k < kLdHeads; ++k) v[k] = to_f32(e[k]);
                } else {
                    for (int k = 0; k < hc; ++k) v[k] = to_f32(p[k]);
                }
            }
        }
#pragma unroll
        for (int k = 0; k < kLdHeads; ++k) sdt[k][t] = v[k];
    }
    __syncthreads();
    if (h >= nheads) return;      // wave-uniform, behind the only barrier
    const int64_t bhc = (b * nheads + h) * nchunks + c;
    float l0, l1, d0 = sdt[wave][lane], d1 = sdt[wave][lane + 64];
    if (dt_bias) {
        // dt holds the raw projection: the step size is softplus(dt + dt_bias) (0 stays 0 past the end of the sequence)
        const float bh = dt_bias[h];
        if (lane < valid) d0 = softplus_f(d0 + bh);
        if (lane + 64 < valid) d1 = softplus_f(d1 + bh);
    }
    wave_cumsum_from(A[h], d0, d1, l0, l1);
    float* p = ldtab + bhc * (2 * kQ);
    p[lane] = l0; p[lane + 64] = l1; p[kQ + lane] = d0; p[kQ + lane + 64] = d1;
    if (lane == 63) lam[bhc] = l1;
}

// Both preparations in one launch (they are independent, and either alone leaves most of the GPU idle): the first
// kCbParts n_cb workgroups run cb_body for (part, chunk, group, batch) = the index split in that order, the others ld_table_body.
struct PrepArgs {
    const void* Bm; const void* Cm; float* Gf; void* Gm; void* Gmt; void* Bt; void* Ct;
    int64_t Bsb, Bsl, Bsg, Csb, Csl, Csg;
    const void* dt; int dt_f32; const float* dt_bias; const float* A; float* ldtab; float* lam; int64_t dtsb, dtsl;
    int64_t seqlen, nheads, ngroups, nchunks, n_cb;
};
template <typename T, int N>
__global__ void __launch_bounds__(256)
prep_kernel(const PrepArgs a) {
    const int64_t blk = blockIdx.x;
    if (blk < kCbParts * a.n_cb) {
        const int64_t q = blk / kCbParts;
        const int64_t c = q % a.nchunks, g = (q / a.nchunks) % a.ngroups, b = q / (a.nchunks * a.ngroups);
        cb_body<T, N>(static_cast<const T*>(a.Bm), static_cast<const T*>(a.Cm), a.Gf, static_cast<T*>(a.Gm), static_cast<T*>(a.Gmt),
                      static_cast<T*>(a.Bt), static_cast<T*>(a.Ct), a.seqlen, a.ngroups, a.nchunks,
                      a.Bsb, a.Bsl, a.Bsg, a.Csb, a.Csl, a.Csg, c, g, b, (int)(blk % kCbParts));
    } else {
        ld_table_body<T>(a.dt, a.dt_f32, a.dt_bias, a.A, a.ldtab, a.lam, a.seqlen, a.nheads, a.nchunks, a.dtsb, a.dtsl, blk - kCbParts * a.n_cb);
    }
}

// ------------------------------------------------------------------------------------------
// Local chunk state.  grid (nchunks, ngroups * nslices, batch), 256 threads; a workgroup loops over `hps` heads.
//   DSTATE == false:  out[p][n] = sum_j (dt_j e^{Lam-l_j}) x[j][p] * B[j][n]      (forward)
//   DSTATE == true :  out[p][n] = sum_i e^{l_i} dy[i][p] * C[i][n]                (backward)
// Used for fp32 operands (16-bit operands take state_pass16_kernel, which fuses this with the recurrence); `out` is fp32.
// `X` is x or dy; `Mt` is the group's B or C tile already transposed to [N][kQ] (tokens contiguous) by cb_body (prep_kernel),
// staged into LDS once per workgroup.  Per head only the x tile moves: it is loaded 16 bytes at a time, scaled in
// fp32 and written transposed; the next head's tile is prefetched into registers while the MFMAs run.
template <typename T, int P, int N, bool DSTATE>
__global__ void __launch_bounds__(256)
chunk_state_kernel(const T* __restrict__ X, const float* __restrict__ ldtab,
                   const T* __restrict__ Mt, float* __restrict__ out,
                   int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t nchunks, int64_t nslices, int64_t hps,
                   int64_t Xsb, int64_t Xsl, int64_t Xsh) {
    constexpr int LD = lds_ld<T>(kQ);
    constexpr int V = VecTraits<T>::kVec;
    constexpr int NIT = (P / V) / 2;              // 16-byte vectors per thread per head (thread <-> fixed token)
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* sX = reinterpret_cast<T*>(smem_raw);        // [P][LD]   x^T scaled
    T* sM = sX + P * LD;                           // [N][LD]   B^T or C^T
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int64_t c = blockIdx.x, b = blockIdx.z;
    const int64_t g = blockIdx.y / nslices, slice = blockIdx.y % nslices;
    const int64_t hpg = nheads / ngroups;
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    const int tok = tid & (kQ - 1), cvh = tid >> 7;       // this thread's token and channel-vector parity

    stage_rows<T, N, kQ, 256, false>(sM, LD, Mt + ((b * nchunks + c) * ngroups + g) * (int64_t)(N * kQ), kQ, N, nullptr, tid);

    constexpr int BM = P / 64, BN = N / 64;
    const int wm = wave >> 1, wn = wave & 1;
    uint4 pre[NIT];
    auto prefetch = [&](int64_t h) {
        const T* xp = X + b * Xsb + (t0 + tok) * Xsl + h * Xsh;
#pragma unroll
        for (int it = 0; it < NIT; ++it)
            pre[it] = tok < valid ? *reinterpret_cast<const uint4*>(xp + (it * 2 + cvh) * V) : uint4{0u, 0u, 0u, 0u};
    };
    prefetch(g * hpg + slice * hps);

    for (int64_t hh = 0; hh < hps; ++hh) {
        const int64_t h = g * hpg + slice * hps + hh;
        float l0, l1, d0, d1;
        wave_ld_load(ldtab, (b * nheads + h) * nchunks + c, l0, l1, d0, d1);
        const float Lam = __shfl(l1, 63, 64);
        // scale of this thread's token (token = lane + 64 * (wave & 1))
        const float lt = (wave & 1) ? l1 : l0, dtt = (wave & 1) ? d1 : d0;
        const float sc = DSTATE ? __expf(lt) : dtt * __expf(Lam - lt);
        __syncthreads();                     // previous head's MFMAs are done with sX
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const T* el = reinterpret_cast<const T*>(&pre[it]);
#pragma unroll
            for (int i = 0; i < V; ++i) sX[((it * 2 + cvh) * V + i) * LD + tok] = from_f32<T>(to_f32(el[i]) * sc);
        }
        __syncthreads();
        if (hh + 1 < hps) prefetch(h + 1);

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
    }
}

// ------------------------------------------------------------------------------------------
// Inter-chunk recurrence.  grid (nheads, batch, kScanSplit), 256 threads; a workgroup owns 1/kScanSplit of the
// [p][n] state of one (batch, head), each thread EPT float4 slices of it, and walks the chunks with the running
// state in registers (fp32).  The split only exists to put enough waves on the GPU to hide memory latency.
//
// forward (REVERSE == false):
//     run = init;  for c = 0..nc-1:  prev[c] = T(run);  run = e^{lam_c} run + local[c];  final = run
// reverse (REVERSE == true), the gradient recurrence:
//     run = dfinal;  for c = nc-1..0:  prev[c] = T(run)   (= dL/dS_new(c));
//                                      dlam[c][split] = e^{lam_c} <run, sprev[c]> over this workgroup's part
//                                      (sprev[c] = the forward state entering chunk c);
//                                      run = e^{lam_c} run + local[c]
//     dinit = run.
// dlam is the part of dL/dLam_c that flows through the carried state only.  The part through the chunk's own
// tokens is added by the consumer as a PREFIX sum of per-token terms; forming it here as <run, S_new(c)> and
// subtracting a suffix sum there would cancel two large numbers rounded differently (operand-type copies of
// the states), leaving an error that is constant over the chunk and accumulates in dA.
constexpr int kScanSplit = 4;
constexpr int kDlamParts = 8;     // partial sums of dlam per (batch, head, chunk): every producer fills all of them

template <typename T, int PN, bool REVERSE>
__global__ void __launch_bounds__(256)
state_scan_kernel(const float* __restrict__ local, const float* __restrict__ lam, const float* __restrict__ init,
                  T* __restrict__ prev, float* __restrict__ final_out,
                  const T* __restrict__ sprev, float* __restrict__ dlam,
                  int64_t nheads, int64_t nchunks) {
    constexpr int EPT = PN / 4 / 256 / kScanSplit;
    static_assert(PN % (1024 * kScanSplit) == 0, "state size must be a multiple of 4096 elements");
    const int part0 = blockIdx.z * (PN / kScanSplit);      // first element of this workgroup's part
    constexpr int kRedBatch = 64;
    __shared__ float red[kRedBatch * 4];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int64_t h = blockIdx.x, b = blockIdx.y;
    const int64_t bh = b * nheads + h;
    floatx4 run[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
        if (init) run[e] = *reinterpret_cast<const floatx4*>(init + bh * PN + part0 + (e * 256 + tid) * 4);
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
            const int off = part0 + (e * 256 + tid) * 4;
            float loc[4];
            loadv<float, 4>(local + tile + off, loc);
            // store the state entering (forward) / the gradient leaving (reverse) this chunk
            T o[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) o[q] = from_f32<T>(run[e][q]);
            if (sizeof(T) == 2) *reinterpret_cast<uint2*>(prev + tile + off) = *reinterpret_cast<const uint2*>(o);
            else *reinterpret_cast<uint4*>(prev + tile + off) = *reinterpret_cast<const uint4*>(o);
            if (REVERSE) {
                // state that ENTERED this chunk in the forward pass (operand type, as the other kernels consume it)
                T tv[4];
                if (sizeof(T) == 2) *reinterpret_cast<uint2*>(tv) = *reinterpret_cast<const uint2*>(sprev + tile + off);
                else *reinterpret_cast<uint4*>(tv) = *reinterpret_cast<const uint4*>(sprev + tile + off);
#pragma unroll
                for (int q = 0; q < 4; ++q) dot += run[e][q] * to_f32(tv[q]);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) run[e][q] = dec * run[e][q] + loc[q];
        }
        if (REVERSE) {
            // per-wave partial of e^{Lam} <dS, S_prev>; the four partials are combined once per kRedBatch chunks so
            // the streaming loop has no barrier
            dot = warp_sum(dot) * dec;
            if (lane == 0) red[(cc % kRedBatch) * 4 + wave] = dot;
            if ((cc % kRedBatch) == kRedBatch - 1 || cc == nchunks - 1) {
                __syncthreads();
                const int64_t first = cc - (cc % kRedBatch);
                if (tid <= cc - first) {
                    const int64_t c2 = REVERSE ? nchunks - 1 - (first + tid) : first + tid;
                    {
                        dlam[(bh * nchunks + c2) * kDlamParts + blockIdx.z] = red[tid * 4] + red[tid * 4 + 1] + red[tid * 4 + 2] + red[tid * 4 + 3];
                        dlam[(bh * nchunks + c2) * kDlamParts + kScanSplit + blockIdx.z] = 0.f;
                    }
                }
                __syncthreads();
            }
        }
    }
    if (final_out) {
#pragma unroll
        for (int e = 0; e < EPT; ++e)
            *reinterpret_cast<floatx4*>(final_out + bh * PN + part0 + (e * 256 + tid) * 4) = run[e];
    }
}

}  // namespace m2
