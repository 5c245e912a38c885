// dG partial and the diagonal part of the decay gradient, for 16-bit operands, with asynchronous tile copies.
//
//   per head:  Pm = dY X^T  (MFMA, K = headdim);   dG^h[i][j] = e^{l_i - l_j} dt_j Pm[i][j]   (i >= j)
//              dG += dG^h;    pr = dG^h o G;   dl_diag[i] = sum_j pr[i][j] - sum_i' pr[i'][i]
// Row and column sums come from the same fp32 products, so pairs inside a suffix cancel exactly.
//
// grid (nchunks, ngroups * nslices, batch), 8 waves.  Wave w owns the 32x32 blocks of the [kQ][kQ] tile with
// block-row rb = w >> 1 and block-columns cb0 = 2 (w & 1), cb0 + 1 (blocks above the diagonal do not exist).
// Both operands are token rows with k = channel contiguous, i.e. the tiles as they lie in global memory: they are
// copied global -> LDS asynchronously up to three heads ahead into a ring of buffers (one barrier per head; enough
// bytes in flight per CU to cover the HBM latency), slots
// XOR-swizzled inside each row.  The fp32 G values at this lane's accumulator positions are head-independent
// and stay in registers.  The row/column sums of head k are combined and written after the barrier of head k + 1.
#pragma once
#include "ssd_y.hpp"

namespace m2 {

template <int P>
constexpr int dg16_ring() { return (size_t)4 * (2 * kQ * P * 2 + 1024) + 6 * 1024 <= 160 * 1024 ? 4 : 2; }    // tile buffers
template <int P>
constexpr size_t dg16_smem() { return (size_t)dg16_ring<P>() * (2 * kQ * P * 2 + 2 * kQ * sizeof(float)) + (size_t)(2 * 6 * kQ) * sizeof(float); }

template <typename T, int P>
__global__ void __launch_bounds__(512, 2)
dg16_kernel(const T* __restrict__ X, const float* __restrict__ ldtab,
            const T* __restrict__ dY, const float* __restrict__ Gf, float* __restrict__ dGp, float* __restrict__ dl_diag,
            int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t nchunks, int64_t nslices, int64_t hps,
            int64_t Xsb, int64_t Xsl, int64_t Xsh, int64_t dYsb, int64_t dYsl, int64_t dYsh) {
    static_assert(sizeof(T) == 2, "16-bit operands only");
    constexpr int SPR = P / 8;                    // 16-byte slots per tile row
    constexpr int NX = kQ * SPR / 512;            // async copies per lane per tile
    constexpr int KS = P / 16;
    constexpr int TILE = kQ * P;
    constexpr int RING = dg16_ring<P>();
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* tiles = reinterpret_cast<T*>(smem_raw);                         // [RING][ dY | X ]
    float* sLD = reinterpret_cast<float*>(tiles + RING * 2 * TILE);    // [RING][ l kQ | dt kQ ]
    float* s_sum = sLD + RING * 2 * kQ;                                // [2 parities][ rs 2 x kQ | cs 4 x kQ ]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31, half = lane >> 5;
    const int64_t c = blockIdx.x, b = blockIdx.z;
    const int64_t g = blockIdx.y / nslices, slice = blockIdx.y % nslices;
    const int64_t hpg = nheads / ngroups;
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    const int rb = wave >> 1, cb0 = (wave & 1) * 2;
    const bool active = cb0 <= rb;

    const uint32_t wave_u = uniform(wave), lds_T = uniform(lds_addr_of(tiles)), lds_LD = uniform(lds_addr_of(sLD));
    uint32_t offY[NX], offX[NX];      // per-lane source byte offsets (head-independent)
#pragma unroll
    for (int it = 0; it < NX; ++it) {
        const int s = (wave * NX + it) * 64 + lane;
        const int row = s / SPR, cs = (s % SPR) ^ (row & (SPR - 1));
        const int grow = row < valid ? row : valid - 1;     // rows past the end: finite stand-ins, masked below
        offY[it] = (uint32_t)(grow * dYsl + cs * 8) * 2u;
        offX[it] = (uint32_t)(grow * Xsl + cs * 8) * 2u;
    }
    auto issue_tiles = [&](int64_t h, int buf) {
        const T* gy = dY + b * dYsb + t0 * dYsl + h * dYsh;
        const T* gx = X + b * Xsb + t0 * Xsl + h * Xsh;
        const uint32_t dst = lds_T + (uint32_t)(buf * 2 * TILE * 2);
#pragma unroll
        for (int it = 0; it < NX; ++it) {
            async_copy16(gy, offY[it], dst + (wave_u * NX + it) * 1024u);
            async_copy16(gx, offX[it], dst + (uint32_t)(TILE * 2) + (wave_u * NX + it) * 1024u);
        }
        async_copy_ldtab(ldtab, (b * nheads + h) * nchunks + c, lds_LD + (uint32_t)(buf * 2 * kQ * 4));
    };
    const int64_t h_first = g * hpg + slice * hps;
#pragma unroll
    for (int j = 0; j < RING - 1; ++j)
        if (j < hps) issue_tiles(h_first + j, j);

    // fp32 G at this lane's accumulator positions (head-independent)
    float gq[2][16];
    {
        const float* Gg = Gf + ((b * nchunks + c) * ngroups + g) * (int64_t)(kQ * kQ);
#pragma unroll
        for (int jb = 0; jb < 2; ++jb)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int i = rb * 32 + acc_row(lane, v), j = (cb0 + jb) * 32 + r;
                gq[jb][v] = (cb0 + jb <= rb && i >= j) ? Gg[i * kQ + j] : 0.f;
            }
    }
    floatx16 dG[1][2];
    acc_zero(dG);

    auto flush_sums = [&](int64_t h, int par) {
        if (tid < kQ) {
            const float* rs = s_sum + par * 6 * kQ;
            const float* cs = rs + 2 * kQ;
            dl_diag[((b * nheads + h) * nchunks + c) * kQ + tid] =
                (rs[tid] + rs[kQ + tid]) - (cs[tid] + cs[kQ + tid] + cs[2 * kQ + tid] + cs[3 * kQ + tid]);
        }
    };

    for (int64_t hh = 0; hh < hps; ++hh) {
        const int64_t h = h_first + hh;
        const int buf = (int)(hh % RING), par = (int)(hh & 1);
        {
            // the tiles of the heads after this one may stay in flight
            const int64_t younger = hps - 1 - hh;
            wait_vmem_keep<2 * NX + 1>((int)(younger < RING - 2 ? younger : RING - 2));
        }
        const float* sl = sLD + buf * 2 * kQ;
        const float* sd = sl + kQ;
        const float l_first = sl[rb * 32], l_last = sl[rb * 32 + 31];
        const bool fast = (l_first - l_last) < kMaxRange;
        // column-side values of this lane's two columns j = (cb0 + jb) * 32 + r, row-side values of its 16 rows
        float lj[2], dtj[2], vj[2], ui[16];
#pragma unroll
        for (int jb = 0; jb < 2; ++jb) {
            const int j = (cb0 + jb) * 32 + r;
            lj[jb] = sl[j];
            dtj[jb] = sd[j];
            vj[jb] = (cb0 + jb <= rb) ? __expf(fminf(l_first - lj[jb], kMaxRange)) * dtj[jb] : 0.f;
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) ui[v] = sl[rb * 32 + acc_row(lane, v)];
        if (fast) {
#pragma unroll
            for (int v = 0; v < 16; ++v) ui[v] = __expf(ui[v] - l_first);
        }
        __syncthreads();          // tiles of head hh are in LDS; the sums of head hh-1 are complete; buffer of hh-1 is free
        if (hh + RING - 1 < hps) issue_tiles(h + RING - 1, (int)((hh + RING - 1) % RING));
        if (hh > 0) flush_sums(h - 1, par ^ 1);
        const T* cA = tiles + buf * 2 * TILE;
        const T* cT = cA + TILE;
        float* s_rs = s_sum + par * 6 * kQ;
        float* s_cs = s_rs + 2 * kQ;

        float rsum[16], csum[2] = {0.f, 0.f};
#pragma unroll
        for (int v = 0; v < 16; ++v) rsum[v] = 0.f;
        if (active) {
            floatx16 pa[1][2];
            acc_zero(pa);
            const int ra = rb * 32 + r;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const Frag<T> af = load_frag(cA + (ra * SPR + ((ks * 2 + half) ^ (ra & (SPR - 1)))) * 8);
#pragma unroll
                for (int jb = 0; jb < 2; ++jb) {
                    if (cb0 + jb > rb) continue;
                    const int rt = (cb0 + jb) * 32 + r;
                    const Frag<T> bf = load_frag(cT + (rt * SPR + ((ks * 2 + half) ^ (rt & (SPR - 1)))) * 8);
                    mma_frag(pa[0][jb], af, bf);
                }
            }
#pragma unroll
            for (int jb = 0; jb < 2; ++jb) {
                if (cb0 + jb > rb) continue;
                const int j = (cb0 + jb) * 32 + r;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int i = rb * 32 + acc_row(lane, v);
                    float w;
                    if (fast) w = ui[v] * vj[jb];                              // u_i * v_j
                    else w = __expf(fminf(ui[v] - lj[jb], 0.f)) * dtj[jb];
                    // rows i >= valid hold stand-in data: G is zero there but dG itself must be masked
                    const float dgh = (i >= j && i < valid) ? w * pa[0][jb][v] : 0.f;
                    dG[0][jb][v] += dgh;
                    const float pr = dgh * gq[jb][v];
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
            const float cs = csum[jb] + __shfl_xor(csum[jb], 32, 64);
            if (lane < 32) s_cs[rb * kQ + (cb0 + jb) * 32 + lane] = cs;
        }
    }
    __syncthreads();
    flush_sums(h_first + hps - 1, (int)((hps - 1) & 1));
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

}  // namespace m2
