// SSD backward dx kernel for 16-bit operands (same pipeline as ssd_y.hpp) and the per-token decay-gradient assembly.
//
//     dxd[j][p] = u_j * ( e^{Lam-l_ref} sum_n B[j][n] dS[p][n]  +  sum_{i>=j} (G[i][j] v_i) dy[i][p] )
//     dx = dt_j dxd + D dy            dir_j = sum_p dxd[j][p] x[j][p]          rb_j = dt_j sum_p (off part)[j][p] x[j][p]
//
// (factorised decay per 32-token row block around its LAST token: v_i = e^{l_i - l_ref}, u_j = e^{l_ref - l_j} <= 1;
// exact per-element fallback when the block's range exceeds kMaxRange).
//
// A workgroup of 8 waves handles one chunk of one group and loops over `hps` heads; wave w owns token rows
// 32 (w >> 1) .. + 31 and the channel half (w & 1).  Per head three tiles -- dS [P][N], dy [128][P], x [128][P] --
// are copied global -> LDS asynchronously, one head ahead, into one of two buffers (one barrier per head).  The
// B row fragments and the transposed causal C B^T fragments stay in registers.  dy reaches the MFMA through LDS
// transpose reads; the epilogue goes through a wave-private fp32 tile and reads x and dy row-wise from the same
// LDS tiles, so dx leaves in 16-byte row stores.
//
// The per-token results that need a scan over the chunk (ddt, dA) are left to da_kernel: this kernel writes the
// two channel-half partials of dir and rb, and per-wave partials of dD.
#pragma once
#include "ssd_y.hpp"

namespace m2 {

template <int P, int N>
constexpr size_t dx16_smem() {
    return (size_t)2 * ((P * N + 2 * kQ * P) * 2 + 2 * kQ * sizeof(float)) + (size_t)8 * (kQ + 32) * sizeof(float) + (size_t)8 * 16 * (P / 2) * sizeof(float);
}
template <typename T, int P, int N>
constexpr bool dx16_ok() { return sizeof(T) == 2 && dx16_smem<P, N>() <= 160 * 1024; }

struct Dx16Out {
    float* dirp;     // [b][h][c][2][kQ]
    float* rbp;      // [b][h][c][2][kQ]
    float* dDp8;     // [b][h][c][8]
};

template <typename T, int P, int N>
__global__ void __launch_bounds__(512, 1)
ssd_dx16_kernel(const DiagArgs a, const Dx16Out o) {
    static_assert(sizeof(T) == 2, "16-bit operands only");
    constexpr int PW = P / 2;                    // channels per wave
    constexpr int BN = PW / 32, KSN = N / 16;
    constexpr int SPR_S = N / 8, SPR_X = P / 8;
    constexpr int NS = P * SPR_S / 512, NX = kQ * SPR_X / 512;
    constexpr int TAB = kQ + 32;
    constexpr int TILES = P * N + 2 * kQ * P;    // elements per buffer
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* tiles = reinterpret_cast<T*>(smem_raw);                       // [2][ dS | dy | x ]
    float* sLD = reinterpret_cast<float*>(tiles + 2 * TILES);        // [2][ l kQ | dt kQ ]
    float* wt_all = sLD + 2 * 2 * kQ;                                // [8 waves][wv kQ | wu 32]
    float* sY = wt_all + 8 * TAB;                                    // [8 waves][16][PW]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31, half = lane >> 5;
    const int rbk = wave >> 1, ch = wave & 1;
    const int64_t c = blockIdx.x, b = blockIdx.z;
    const int64_t g = blockIdx.y / a.nslices, slice = blockIdx.y % a.nslices;
    const int64_t hpg = a.nheads / a.ngroups;
    const int64_t t0 = c * kQ;
    const int valid = (int)((a.seqlen - t0) < kQ ? (a.seqlen - t0) : kQ);
    const int row0 = rbk * 32, col0 = ch * PW;
    float* wv = wt_all + wave * TAB;
    float* wu = wv + kQ;
    float* sYw = sY + wave * 16 * PW;

    auto issue_tiles = [&](int64_t h, int buf) {
        T* dS = tiles + buf * TILES;
        T* dY = dS + P * N;
        T* dXt = dY + kQ * P;
        const T* Sp = static_cast<const T*>(a.S) + ((b * a.nchunks + c) * a.nheads + h) * (int64_t)(P * N);
#pragma unroll
        for (int it = 0; it < NS; ++it) {
            const int s0 = (wave * NS + it) * 64, s = s0 + lane;
            const int row = s / SPR_S, cs = (s % SPR_S) ^ swz_s<SPR_S>(row);
            async_copy16(Sp + row * N + cs * 8, dS + s0 * 8);
        }
        const T* Yp = static_cast<const T*>(a.Z) + b * a.Z_sb + t0 * a.Z_sl + h * a.Z_sh;
        const T* Xp = static_cast<const T*>(a.X) + b * a.X_sb + t0 * a.X_sl + h * a.X_sh;
#pragma unroll
        for (int it = 0; it < NX; ++it) {
            const int s0 = (wave * NX + it) * 64, s = s0 + lane;
            const int row = s / SPR_X, cs = (s % SPR_X) ^ swz_x(row);
            const int grow = row < valid ? row : valid - 1;       // rows past the end only ever meet zeros / are not stored
            async_copy16(Yp + (int64_t)grow * a.Z_sl + cs * 8, dY + s0 * 8);
            async_copy16(Xp + (int64_t)grow * a.X_sl + cs * 8, dXt + s0 * 8);
        }
        async_copy_ldtab(a.ldtab, (b * a.nheads + h) * a.nchunks + c, sLD + buf * 2 * kQ);
    };

    const int64_t h_first = g * hpg + slice * a.hps;
    issue_tiles(h_first, 0);

    // ---- head-independent operands, resident in registers: B rows and (causal C B^T)^T rows of this wave's tokens
    Frag<T> fd[8], fo[KSN];
    {
        const T* Gp = static_cast<const T*>(a.Gd) + ((b * a.nchunks + c) * a.ngroups + g) * (int64_t)(kQ * kQ) + (row0 + r) * kQ;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
            if (ks >= 2 * rbk) fd[ks] = load_frag(Gp + ks * 16 + half * 8);
        const T* Bp = static_cast<const T*>(a.Aoff) + b * a.Ao_sb + (t0 + row0 + r) * a.Ao_sl + g * a.Ao_sg;
        const bool b_ok = row0 + r < valid;
#pragma unroll
        for (int ks = 0; ks < KSN; ++ks) {
            if (b_ok) fo[ks] = load_frag(Bp + ks * 16 + half * 8);
            else {
#pragma unroll
                for (int e = 0; e < 8; ++e) fo[ks].v[e] = (T)0.f;
            }
        }
    }
    // transpose-read lane roles (see ssd_y.hpp)
    const int tr_tok = (lane >> 2) & 3;
    const int tr_col = ((lane >> 4) & 1) * 16 + 4 * (lane & 3);
    typedef T tvec4 __attribute__((ext_vector_type(4)));

    for (int64_t hh = 0; hh < a.hps; ++hh) {
        const int64_t h = h_first + hh;
        const int buf = (int)(hh & 1);
        const int64_t bhc = (b * a.nheads + h) * a.nchunks + c;
        const float Dh = a.D ? a.D[h] : 0.f;

        wait_vmem_all();          // this wave's share of the tiles of head hh, and the whole [ l | dt ] table, have landed
        // ---- wave-private decay tables from the shared [ l | dt ] table
        const float* sl = sLD + buf * 2 * kQ;
        const float* sd = sl + kQ;
        const float l_first = sl[row0], l_last = sl[row0 + 31], Lam = sl[kQ - 1];
        const bool fast = (l_first - l_last) < kMaxRange;
        const float lref = l_last;
        wv[lane] = lane >= row0 ? __expf(sl[lane] - lref) : 0.f;
        wv[lane + 64] = lane + 64 >= row0 ? __expf(sl[lane + 64] - lref) : 0.f;
        if (lane < 32) wu[lane] = __expf(fminf(lref - sl[row0 + lane], 0.f));
        __syncthreads();
        if (hh + 1 < a.hps) issue_tiles(h + 1, buf ^ 1);
        const T* cS = tiles + buf * TILES;
        const T* cY = cS + P * N;
        const T* cX = cY + kQ * P;

        const float off_fast = __expf(Lam - lref);
        auto off_scale = [&](int v) -> float { return fast ? off_fast : __expf(Lam - sl[row0 + acc_row(lane, v)]); };
        auto fin_scale = [&](int v) -> float { return fast ? wu[acc_row(lane, v)] : 1.f; };

        // ---- off-diagonal term: B rows (registers) x dS (LDS, natural layout)
        floatx16 acc[1][BN];
        acc_zero(acc);
#pragma unroll
        for (int ks = 0; ks < KSN; ++ks) {
#pragma unroll
            for (int j = 0; j < BN; ++j) {
                const int row = col0 + j * 32 + r;
                const Frag<T> bf = load_frag(cS + (row * SPR_S + ((ks * 2 + half) ^ swz_s<SPR_S>(row))) * 8);
                mma_frag(acc[0][j], fo[ks], bf);
            }
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float os = off_scale(v);
#pragma unroll
            for (int j = 0; j < BN; ++j) acc[0][j][v] *= os;
        }

        // ---- rb_j = dt_j sum_p x[j][p] * (off part, final scale applied): x at the accumulator positions by transpose reads
        {
            float rbv[16];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float s4[4] = {0.f, 0.f, 0.f, 0.f};
                const int tok = row0 + 8 * q + 4 * half + tr_tok;
#pragma unroll
                for (int j = 0; j < BN; ++j) {
                    const int col = col0 + j * 32 + tr_col;
                    const tvec4 xv = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
                        (M2_LDS tvec4*)(cX + (tok * SPR_X + ((col >> 3) ^ swz_x(tok))) * 8 + (col & 7)));
#pragma unroll
                    for (int e = 0; e < 4; ++e) s4[e] += acc[0][j][4 * q + e] * to_f32(xv[e]);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) rbv[4 * q + e] = s4[e] * fin_scale(4 * q + e);
            }
            int ri;
            const float tot = half_wave_reduce16(rbv, &ri);
            const int row = row0 + acc_row(lane, ri);
            if ((lane & 1) == 0) o.rbp[(bhc * 2 + ch) * kQ + row] = tot * sd[row];
        }

        // ---- diagonal term: transposed causal C B^T fragment scaled along k = i; dy through transpose reads
        const int jrow = row0 + r;
        const float l_row = sl[jrow];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            if (ks < 2 * rbk) continue;
            float f[8];
            if (fast) {
                const floatx4 fa = *reinterpret_cast<const floatx4*>(wv + ks * 16 + half * 8);
                const floatx4 fb = *reinterpret_cast<const floatx4*>(wv + ks * 16 + half * 8 + 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) { f[e] = fa[e]; f[4 + e] = fb[e]; }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int k = ks * 16 + half * 8 + e;
                    f[e] = (k >= jrow) ? __expf(sl[k] - l_row) : 0.f;
                }
            }
            const Frag<T> af = scale_frag(fd[ks], f);
#pragma unroll
            for (int j = 0; j < BN; ++j) {
                const int col = col0 + j * 32 + tr_col;
                const int ta = ks * 16 + 8 * half + tr_tok, tb = ta + 4;
                const tvec4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
                    (M2_LDS tvec4*)(cY + (ta * SPR_X + ((col >> 3) ^ swz_x(ta))) * 8 + (col & 7)));
                const tvec4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
                    (M2_LDS tvec4*)(cY + (tb * SPR_X + ((col >> 3) ^ swz_x(tb))) * 8 + (col & 7)));
                Frag<T> bf;
#pragma unroll
                for (int e = 0; e < 4; ++e) { bf.v[e] = lo[e]; bf.v[4 + e] = hi[e]; }
                mma_frag(acc[0][j], af, bf);
            }
        }

        // ---- epilogue, 16 token rows at a time
        constexpr int LPR = PW / 8;              // lanes per output row (this wave's channel half)
        constexpr int RPP = 64 / LPR;            // rows per pass
        static_assert(RPP <= 16 && 16 % RPP == 0, "row passes");
        T* dXp = static_cast<T*>(a.dX) + b * a.dX_sb + t0 * a.dX_sl + h * a.dX_sh;
        float dD_loc = 0.f;
#pragma unroll
        for (int qq = 0; qq < 2; ++qq) {
#pragma unroll
            for (int q2 = 0; q2 < 2; ++q2)
#pragma unroll
                for (int j = 0; j < BN; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int v = 4 * (2 * qq + q2) + e;
                        sYw[(8 * q2 + 4 * half + e) * PW + j * 32 + r] = acc[0][j][v] * fin_scale(v);
                    }
            wave_lds_sync();
#pragma unroll
            for (int ps = 0; ps < 16 / RPP; ++ps) {
                const int rl = ps * RPP + lane / LPR, cv = lane % LPR;
                const int tok = row0 + 16 * qq + rl;
                const floatx4 ya = *reinterpret_cast<const floatx4*>(sYw + rl * PW + cv * 8);
                const floatx4 yb = *reinterpret_cast<const floatx4*>(sYw + rl * PW + cv * 8 + 4);
                const int slot = ((col0 >> 3) + cv) ^ swz_x(tok);
                const uint4 xr = *reinterpret_cast<const uint4*>(cX + (tok * SPR_X + slot) * 8);
                const uint4 gr = *reinterpret_cast<const uint4*>(cY + (tok * SPR_X + slot) * 8);
                const T* xe = reinterpret_cast<const T*>(&xr);
                const T* ge = reinterpret_cast<const T*>(&gr);
                const float dtt = sd[tok];
                uint4 ov;
                T* oe = reinterpret_cast<T*>(&ov);
                float dir = 0.f, dd = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float dxd = e < 4 ? ya[e] : yb[e - 4];
                    const float x_ = to_f32(xe[e]), gy = to_f32(ge[e]);
                    oe[e] = from_f32<T>(dtt * dxd + Dh * gy);
                    dir += dxd * x_;
                    dd += gy * x_;
                }
                if (tok < valid) {
                    *reinterpret_cast<uint4*>(dXp + (int64_t)tok * a.dX_sl + col0 + cv * 8) = ov;
                    dD_loc += dd;
                }
                // sum over the LPR lanes that share the row
#pragma unroll
                for (int m = 1; m < LPR; m <<= 1) dir += __shfl_xor(dir, m, 64);
                if (cv == 0) o.dirp[(bhc * 2 + ch) * kQ + tok] = dir;
            }
            wave_lds_sync();
        }
        dD_loc = warp_sum(dD_loc);
        if (lane == 0) o.dDp8[bhc * 8 + wave] = dD_loc;
    }
}

// Per (batch, head, chunk): da_t = sum_{i>=t} (dl_diag_i + dl_c_i) + sum_{j<t} rb_j + dlam,  ddt_t = A da_t + dir_t,
// dA partial = sum_t da_t dt_t, dD partial = sum of the eight per-wave partials.  One wave per (b, h, c), four per workgroup; lanes hold
// the tokens in reverse order (127 - lane, 63 - lane), so the suffix over tokens is an inclusive prefix over lanes and
// the exclusive prefix over tokens an exclusive suffix over lanes.
template <typename T>
__global__ void __launch_bounds__(256)
da_kernel(const void* __restrict__ dt, int dt_f32, int64_t dt_sb, int64_t dt_sl, const float* __restrict__ A,
          const float* __restrict__ dl_diag, const float* __restrict__ dl_c, const float* __restrict__ dlam,
          const float* __restrict__ dirp, const float* __restrict__ rbp, const float* __restrict__ dDp8,
          void* __restrict__ ddt, int64_t ddt_sb, int64_t ddt_sl, float* __restrict__ dAp, float* __restrict__ dDp,
          int64_t seqlen, int64_t nheads, int64_t nchunks, int64_t total) {
    const int lane = threadIdx.x & 63;
    const int64_t bhc = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (bhc >= total) return;
    const int64_t c = bhc % nchunks, h = (bhc / nchunks) % nheads, b = bhc / (nchunks * nheads);
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    const int ta = kQ - 1 - lane, tb = 63 - lane;
    const float Ah = A[h];
    float xa = dl_diag[bhc * kQ + ta] + dl_c[bhc * kQ + ta];
    float xb = dl_diag[bhc * kQ + tb] + dl_c[bhc * kQ + tb];
    const float ra = rbp[(bhc * 2) * kQ + ta] + rbp[(bhc * 2 + 1) * kQ + ta];
    const float rbv = rbp[(bhc * 2) * kQ + tb] + rbp[(bhc * 2 + 1) * kQ + tb];
    const float dira = dirp[(bhc * 2) * kQ + ta] + dirp[(bhc * 2 + 1) * kQ + ta];
    const float dirb = dirp[(bhc * 2) * kQ + tb] + dirp[(bhc * 2 + 1) * kQ + tb];
    float dta = 0.f, dtb = 0.f;
    {
        const int64_t oa = b * dt_sb + (t0 + ta) * dt_sl + h, ob = b * dt_sb + (t0 + tb) * dt_sl + h;
        if (ta < valid) dta = dt_f32 ? static_cast<const float*>(dt)[oa] : to_f32(static_cast<const T*>(dt)[oa]);
        if (tb < valid) dtb = dt_f32 ? static_cast<const float*>(dt)[ob] : to_f32(static_cast<const T*>(dt)[ob]);
    }
    float ya = ra, yb = rbv;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float na = __shfl_up(xa, o, 64), nb = __shfl_up(xb, o, 64);
        const float ma = __shfl_down(ya, o, 64), mb = __shfl_down(yb, o, 64);
        if (lane >= o) { xa += na; xb += nb; }
        if (lane + o < 64) { ya += ma; yb += mb; }
    }
    xb += __shfl(xa, 63, 64);
    xa += (ya - ra) + __shfl(yb, 0, 64);
    xb += yb - rbv;
    float dlm = 0.f;
#pragma unroll
    for (int sp = 0; sp < kScanSplit; ++sp) dlm += dlam[bhc * kScanSplit + sp];
    const float da_a = xa + dlm, da_b = xb + dlm;
    float dAl = 0.f;
    if (ta < valid) {
        const float val = Ah * da_a + dira;
        const int64_t oo = b * ddt_sb + (t0 + ta) * ddt_sl + h;
        if (dt_f32) static_cast<float*>(ddt)[oo] = val; else static_cast<T*>(ddt)[oo] = from_f32<T>(val);
        dAl += da_a * dta;
    }
    if (tb < valid) {
        const float val = Ah * da_b + dirb;
        const int64_t oo = b * ddt_sb + (t0 + tb) * ddt_sl + h;
        if (dt_f32) static_cast<float*>(ddt)[oo] = val; else static_cast<T*>(ddt)[oo] = from_f32<T>(val);
        dAl += da_b * dtb;
    }
    dAl = warp_sum(dAl);
    if (lane == 0) {
        dAp[bhc] = dAl;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < 8; ++w) s += dDp8[bhc * 8 + w];
        dDp[bhc] = s;
    }
}

}  // namespace m2
