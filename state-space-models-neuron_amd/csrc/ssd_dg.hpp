// dG partial and the diagonal part of the decay gradient, for 16-bit operands, with asynchronous tile copies.
//
//   per head:  Pm = dY X^T  (MFMA, K = headdim);   dG^h[i][j] = e^{l_i - l_j} dt_j Pm[i][j]   (i >= j)
//              dG += dG^h;    pr = dG^h o G;   dl_diag[i] = sum_j pr[i][j] - sum_i' pr[i'][i]
// Row and column sums come from the same fp32 products, so pairs inside a suffix cancel exactly.
//
// grid (nchunks, ngroups * nslices, batch), 10 waves: one per 32x32 block of the lower triangle of the [kQ][kQ] tile
// (blocks above the diagonal do not exist).  Waves w, w + 4, w + 8 share a SIMD, so the SIMDs carry 3, 3, 2, 2 blocks;
// the diagonal blocks, which carry the i >= j mask, go to the SIMDs with two.
// Both operands are token rows with k = channel contiguous, i.e. the tiles as they lie in global memory: they are
// copied global -> LDS asynchronously (by waves 0-7) up to three heads ahead into a ring of buffers (one barrier per
// head), slots XOR-swizzled inside each row.  The fp32 G values at this lane's accumulator positions are
// head-independent and stay in registers.  The row/column sums of head k are combined and written after the barrier
// of head k + 1.
#pragma once
#include "ssd_y.hpp"

namespace m2 {

constexpr int kDgWaves = 10;
template <int P>
constexpr int dg16_ring() { return (size_t)4 * (2 * kQ * P * 2 + 1024) + 8 * 1024 <= 160 * 1024 ? 4 : 2; }    // tile buffers
template <int P>
constexpr size_t dg16_smem() { return (size_t)dg16_ring<P>() * (2 * kQ * P * 2 + 2 * kQ * sizeof(float)) + (size_t)(2 * 8 * kQ + kDgWaves * 32) * sizeof(float); }

template <typename T, int P>
__global__ void __launch_bounds__(kDgWaves * 64)
dg16_kernel(const T* __restrict__ X, const float* __restrict__ ldtab,
            const T* __restrict__ dY, const float* __restrict__ Gf, float* __restrict__ dGp, float* __restrict__ dl_diag,
            int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t nchunks, int64_t nslices, int64_t hps,
            int64_t Xsb, int64_t Xsl, int64_t Xsh, int64_t dYsb, int64_t dYsl, int64_t dYsh) {
    static_assert(sizeof(T) == 2, "16-bit operands only");
    constexpr int SPR = P / 8;                    // 16-byte slots per tile row
    constexpr int NX = kQ * SPR / 512;            // async copies per lane per tile (copying waves)
    constexpr int KS = P / 16;
    constexpr int TILE = kQ * P;
    constexpr int RING = dg16_ring<P>();
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* tiles = reinterpret_cast<T*>(smem_raw);                         // [RING][ dY | X ]
    float* sLD = reinterpret_cast<float*>(tiles + RING * 2 * TILE);    // [RING][ l kQ | dt kQ ]
    float* s_sum = sLD + RING * 2 * kQ;                                // [2 parities][ rs 4 x kQ | cs 4 x kQ ]
    float* su = s_sum + 2 * 8 * kQ + (threadIdx.x >> 6) * 32;          // [waves][32]: row factors of this wave's block

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31, half = lane >> 5;
    const int64_t c = blockIdx.x, b = blockIdx.z;
    const int64_t g = blockIdx.y / nslices, slice = blockIdx.y % nslices;
    const int64_t hpg = nheads / ngroups;
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    // block (rb, cb) of this wave (one nibble per wave): the four diagonal blocks sit on waves 2, 3, 6, 7, i.e. on the two
    // SIMDs that carry two waves; the six blocks below the diagonal on the two SIMDs that carry three
    //   wave   0     1     2     3     4     5     6     7     8     9
    //   block (1,0) (2,0) (0,0) (1,1) (2,1) (3,0) (2,2) (3,3) (3,1) (3,2)
    const int rb = (int)((0x3332321021ull >> (4 * wave)) & 15);
    const int cb = (int)((0x2132011000ull >> (4 * wave)) & 15);
    const bool masked = (rb == cb) || valid < kQ;      // wave-uniform
    const bool copier = wave < 8;

    const uint32_t wave_u = uniform(wave), lds_T = uniform(lds_addr_of(tiles)), lds_LD = uniform(lds_addr_of(sLD));
    uint32_t offY[NX], offX[NX];      // per-lane source byte offsets (head-independent)
#pragma unroll
    for (int it = 0; it < NX; ++it) {
        const int s = ((wave & 7) * NX + it) * 64 + lane;
        const int row = s / SPR, cs = (s % SPR) ^ tile_swz<SPR>(row);
        const int grow = row < valid ? row : valid - 1;     // rows past the end: finite stand-ins, masked below
        offY[it] = (uint32_t)(grow * dYsl + cs * 8) * 2u;
        offX[it] = (uint32_t)(grow * Xsl + cs * 8) * 2u;
    }
    auto issue_tiles = [&](int64_t h, int buf) {
        if (copier) {
            const T* gy = dY + b * dYsb + t0 * dYsl + h * dYsh;
            const T* gx = X + b * Xsb + t0 * Xsl + h * Xsh;
            const uint32_t dst = lds_T + (uint32_t)(buf * 2 * TILE * 2);
#pragma unroll
            for (int it = 0; it < NX; ++it) {
                async_copy16(gy, offY[it], dst + (wave_u * NX + it) * 1024u);
                async_copy16(gx, offX[it], dst + (uint32_t)(TILE * 2) + (wave_u * NX + it) * 1024u);
            }
        }
        async_copy_ldtab(ldtab, (b * nheads + h) * nchunks + c, lds_LD + (uint32_t)(buf * 2 * kQ * 4));
    };
    const int64_t h_first = g * hpg + slice * hps;
#pragma unroll
    for (int j = 0; j < RING - 1; ++j)
        if (j < hps) issue_tiles(h_first + j, j);

    // fp32 G at this lane's accumulator positions (head-independent); zero where i < j
    float gq[16];
    {
        const float* Gg = Gf + ((b * nchunks + c) * ngroups + g) * (int64_t)(kQ * kQ);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int i = rb * 32 + acc_row(lane, v), j = cb * 32 + r;
            gq[v] = i >= j ? Gg[i * kQ + j] : 0.f;
        }
    }
    floatx16 dG = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // row sums of block (rb, cb) go to rs[cb], column sums to cs[rb]; token t collects rs[0 .. t/32] and cs[t/32 .. 3]
    // (done by waves 2 and 3, which sit on the SIMDs that carry two waves; all eight values are read and the unwanted
    // ones dropped by a select: a branch per term costs more than the reads)
    auto flush_sums = [&](int64_t h, int par) {
        const int t = tid - 2 * 64;
        if (t >= 0 && t < kQ) {
            const float* rs = s_sum + par * 8 * kQ;
            const float* cs = rs + 4 * kQ;
            const int tb = t >> 5;
            float acc = 0.f;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float rv = rs[q * kQ + t], cv = cs[q * kQ + t];
                acc += (q <= tb ? rv : 0.f) - (q >= tb ? cv : 0.f);
            }
            dl_diag[((b * nheads + h) * nchunks + c) * kQ + t] = acc;
        }
    };

    for (int64_t hh = 0; hh < hps; ++hh) {
        const int64_t h = h_first + hh;
        const int buf = (int)(hh % RING), par = (int)(hh & 1);
        {
            // the tiles of the heads after this one may stay in flight
            const int64_t younger = hps - 1 - hh;
            const int keep = (int)(younger < RING - 2 ? younger : RING - 2);
            if (copier) wait_vmem_keep<2 * NX + 1>(keep); else wait_vmem_keep<1>(keep);
        }
        const float* sl = sLD + buf * 2 * kQ;
        const float* sd = sl + kQ;
        const float l_first = sl[rb * 32], l_last = sl[rb * 32 + 31];
        const bool fast = (l_first - l_last) < kMaxRange;
        // column-side values of this lane's column j = cb * 32 + r, row-side values of its 16 rows
        const int j = cb * 32 + r;
        const float lj = sl[j], dtj = sd[j];
        const float vj = __expf(fminf(l_first - lj, kMaxRange)) * dtj;
        // row factors: one exponential per row of the block (32 lanes), read back as four consecutive table entries per
        // group of accumulator rows 8 q + 4 half + 0..3 -- not 16 exponentials per lane
        if (lane < 32) su[lane] = fast ? __expf(sl[rb * 32 + lane] - l_first) : sl[rb * 32 + lane];
        wave_lds_sync();
        float ui[16];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const floatx4 u4 = *reinterpret_cast<const floatx4*>(su + 8 * q + 4 * half);
#pragma unroll
            for (int e = 0; e < 4; ++e) ui[4 * q + e] = u4[e];
        }
        if (fast) {
#pragma unroll
            for (int v = 0; v < 16; ++v) ui[v] *= vj;      // u_i * v_j
        } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) ui[v] = __expf(fminf(ui[v] - lj, 0.f)) * dtj;
        }
        __syncthreads();          // tiles of head hh are in LDS; the sums of head hh-1 are complete; buffer of hh-1 is free
        if (hh + RING - 1 < hps) issue_tiles(h + RING - 1, (int)((hh + RING - 1) % RING));
        if (hh > 0) flush_sums(h - 1, par ^ 1);
        const T* cA = tiles + buf * 2 * TILE;
        const T* cT = cA + TILE;
        float* s_rs = s_sum + par * 8 * kQ;
        float* s_cs = s_rs + 4 * kQ;

        floatx16 pa = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const int ra = rb * 32 + r, rt = cb * 32 + r;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const Frag<T> af = load_frag(cA + (ra * SPR + ((ks * 2 + half) ^ tile_swz<SPR>(ra))) * 8);
            const Frag<T> bf = load_frag(cT + (rt * SPR + ((ks * 2 + half) ^ tile_swz<SPR>(rt))) * 8);
            mma_frag(pa, af, bf);
        }
        float rsum[16], csum = 0.f;
        if (masked) {
            // diagonal block, or a chunk that runs past the end of the sequence (rows i >= valid hold stand-in data:
            // G is zero there but dG itself must be masked)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int i = rb * 32 + acc_row(lane, v);
                const float dgh = (i >= j && i < valid) ? ui[v] * pa[v] : 0.f;
                dG[v] += dgh;
                rsum[v] = dgh * gq[v];
                csum += rsum[v];
            }
        } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float dgh = ui[v] * pa[v];
                dG[v] += dgh;
                rsum[v] = dgh * gq[v];
                csum += rsum[v];
            }
        }
        int ri;
        const float rtot = half_wave_reduce16(rsum, &ri);
        if ((lane & 1) == 0) s_rs[cb * kQ + rb * 32 + acc_row(lane, ri)] = rtot;
        csum = lane_xor_add<32>(csum);
        if (lane < 32) s_cs[rb * kQ + cb * 32 + lane] = csum;
    }
    __syncthreads();
    flush_sums(h_first + hps - 1, (int)((hps - 1) & 1));
    float* out = dGp + (((b * nchunks + c) * ngroups + g) * nslices + slice) * (int64_t)(kQ * kQ);
#pragma unroll
    for (int v = 0; v < 16; ++v)
        out[(rb * 32 + acc_row(lane, v)) * kQ + cb * 32 + r] = dG[v];
}

}  // namespace m2
