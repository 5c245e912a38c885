// The two "diagonal + off-diagonal" SSD kernels (forward output, backward dx/ddt) share one structure.
//
// Per (batch, chunk, head) the result is a [kQ tokens][P] tile
//     OUT[r][p] = final_r * ( off_r * sum_n Aoff[r][n] * S[p][n]   +   sum_k (Gd[r][k] * tab_w[k]) * Z[k][p] )
//   forward : Aoff = C,  S = state entering the chunk,  Gd = causal C B^T (rows i, k = j <= i),  Z = x
//             y = OUT + D x
//   backward: Aoff = B,  S = gradient of the state leaving the chunk,  Gd = (causal C B^T)^T (rows j, k = i >= j),
//             Z = dy;    dxd = OUT,  dx = dt dxd + D dy,  ddt = A da + dxd . x
//
// A workgroup owns one chunk of one group and loops over `hps` heads of that group.  What does not depend on the
// head -- the MFMA A-operand fragments of C (or B) and of the masked C B^T tile -- is loaded ONCE into registers;
// per head only S (natural layout) and Z (transposed, so that tokens are the contiguous k index) go through LDS.
//
// Decay.  e^{l_i - l_j} is factorised per 32-token row block around a reference token inside the block:
//   forward  (ref = first token of the block):  e^{l_i-l_j} dt_j = u_i * v_j,   u_i = e^{l_i-l_ref} <= 1,
//             v_j = e^{l_ref-l_j} dt_j;   for j inside the block v_j <= e^{R}, R = l_first - l_last of the block
//   backward (ref = last token of the block):   e^{l_i-l_j} = v_i * u_j,        u_j = e^{l_ref-l_j} <= 1, v_i = e^{l_i-l_ref}
// so the decay costs ONE multiply per operand element (v, applied to the register fragment) plus one per output
// row (u) instead of an exp per element.  R <= 32 * max|A dt| (51 for A = -16, dt = 0.1); if a block's range
// exceeds kMaxRange the wave falls back to evaluating e^{l_i-l_j} on the difference, element by element,
// which cannot overflow (the reference always does that, mamba2/mamba2_kernel.py:32-33).
#pragma once
#include "ssd_kernels.hpp"

namespace m2 {

constexpr float kMaxRange = 80.f;

struct DiagArgs {
    // common
    const void* dt; int dt_f32; const float* A; const float* D;
    const float* ldtab;         // [b][h][c][ l kQ | dt kQ ]
    const void* Aoff;           // C (fwd) or B (bwd): [b][l][g][N]
    int64_t Ao_sb, Ao_sl, Ao_sg;
    const void* Gd;             // masked CB^T (fwd) or its transpose (bwd): [b][c][g][kQ][kQ]
    const void* S;              // [b][c][h][P][N]
    const void* Z;              // x (fwd) or dy (bwd): [b][l][h][P]
    int64_t Z_sb, Z_sl, Z_sh;
    int64_t dt_sb, dt_sl;
    int64_t seqlen, nheads, ngroups, nchunks, nslices, hps;
    // forward
    void* Y; int64_t Y_sb, Y_sl, Y_sh;
    // backward
    const void* X; int64_t X_sb, X_sl, X_sh;
    void* dX; int64_t dX_sb, dX_sl, dX_sh;
    void* ddt; int64_t ddt_sb, ddt_sl;
    const float* dl_diag; const float* dl_c; const float* dlam;   // [b][h][c][kQ], [b][h][c][kQ], [b][h][c]
    float* dAp; float* dDp;                                       // [b][h][c]
    float* dbp;            // softplus folded into the scan: [b][h][c] partials of d_dt_bias (ddt is then w.r.t. the raw dt), else null
};

// The backward keeps a transposed copy of x in LDS for its epilogue when that fits (always for bf16);
// otherwise it reads x from global memory there.
template <typename T, int P, int N>
constexpr bool diag_xt_in_lds() {
    return (size_t)(4 * 4 * kQ + 2 * kQ + 8) * sizeof(float) + ((size_t)P * lds_ld<T>(N) + (size_t)2 * P * lds_ld<T>(kQ)) * sizeof(T) <= 150 * 1024;
}
template <typename T, int P, int N, bool BWD>
constexpr size_t diag_smem() {
    return (size_t)(4 * 4 * kQ + (BWD ? 2 * kQ + 8 : 0)) * sizeof(float) +
           ((size_t)P * lds_ld<T>(N) + (size_t)((BWD && diag_xt_in_lds<T, P, N>()) ? 2 : 1) * P * lds_ld<T>(kQ)) * sizeof(T);
}

template <typename T, int P, int N, bool BWD>
__global__ void __launch_bounds__(256, 2)
diag_off_kernel(const DiagArgs a) {
    constexpr int LDN = lds_ld<T>(N), LDQ = lds_ld<T>(kQ);
    constexpr int BN = P / 32, KSN = N / 16;
    constexpr bool XT = BWD && diag_xt_in_lds<T, P, N>();
    extern __shared__ __align__(16) unsigned char smem_raw[];
    float* wt_all = reinterpret_cast<float*>(smem_raw);              // [4 waves][4 tables][kQ]
    float* s_dir = wt_all + 4 * 4 * kQ;                              // BWD: [kQ] dxd . x
    float* s_rb = s_dir + (BWD ? kQ : 0);                            // BWD: [kQ] B . dBoff
    float* s_red = s_rb + (BWD ? kQ : 0);                            // BWD: [8]
    T* sS = reinterpret_cast<T*>(s_red + (BWD ? 8 : 0));             // [P][LDN]
    T* sZt = sS + P * LDN;                                           // [P][LDQ]
    T* sXt = sZt + P * LDQ;                                          // BWD: [P][LDQ]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31, half = lane >> 5, kh8 = half * 8;
    const int64_t c = blockIdx.x, b = blockIdx.z;
    const int64_t g = blockIdx.y / a.nslices, slice = blockIdx.y % a.nslices;
    const int64_t hpg = a.nheads / a.ngroups;
    const int64_t t0 = c * kQ;
    const int valid = (int)((a.seqlen - t0) < kQ ? (a.seqlen - t0) : kQ);
    const int row0 = wave * 32;
    float* wl = wt_all + (wave * 4 + 0) * kQ;
    float* wd = wt_all + (wave * 4 + 1) * kQ;
    float* wv = wt_all + (wave * 4 + 2) * kQ;
    float* wu = wt_all + (wave * 4 + 3) * kQ;

    // ---- head-independent A-operand fragments of the masked CB^T tile: kept in registers in the forward; the
    //      backward (more live state) re-reads them from global memory (L2-resident) for each head
    constexpr bool FD_RES = !BWD;
    Frag<T> fd[FD_RES ? 8 : 1];
    const T* Gp = static_cast<const T*>(a.Gd) + ((b * a.nchunks + c) * a.ngroups + g) * (int64_t)(kQ * kQ) + (row0 + r) * kQ;
    const T* Ao = static_cast<const T*>(a.Aoff) + b * a.Ao_sb + (t0 + row0 + r) * a.Ao_sl + g * a.Ao_sg;
    const bool ao_ok = row0 + r < valid;
    if (FD_RES) {
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const bool used = BWD ? (ks >= 2 * wave) : (ks <= 2 * wave + 1);
            if (used) fd[FD_RES ? ks : 0] = load_frag(Gp + ks * 16 + kh8);
        }
    }

    for (int64_t hh = 0; hh < a.hps; ++hh) {
        const int64_t h = g * hpg + slice * a.hps + hh;
        const float Ah = a.A[h];
        const float Dh = a.D ? a.D[h] : 0.f;

        // ---- wave-private cumulative sum and decay tables
        float l0, l1, d0, d1;
        wave_ld_load(a.ldtab, (b * a.nheads + h) * a.nchunks + c, l0, l1, d0, d1);
        // l at the first / last token of this wave's row block (tokens 32w, 32w+31) and at the chunk end
        const float l_first = wave < 2 ? __shfl(l0, row0, 64) : __shfl(l1, row0 - 64, 64);
        const float l_last = wave < 2 ? __shfl(l0, row0 + 31, 64) : __shfl(l1, row0 + 31 - 64, 64);
        const float Lam = __shfl(l1, 63, 64);
        const bool fast = (l_first - l_last) < kMaxRange;
        const float lref = BWD ? l_last : l_first;
        wl[lane] = l0; wl[lane + 64] = l1; wd[lane] = d0; wd[lane + 64] = d1;
        {
            // k-side table v (only the k range this wave contracts over is meaningful) and row table u
            const int k0i = lane, k1i = lane + 64;
            float v0, v1, u0, u1;
            if (!BWD) {
                v0 = k0i < row0 + 32 ? __expf(lref - l0) * d0 : 0.f;
                v1 = k1i < row0 + 32 ? __expf(lref - l1) * d1 : 0.f;
                u0 = __expf(fminf(l0 - lref, 0.f));
                u1 = __expf(fminf(l1 - lref, 0.f));
            } else {
                v0 = k0i >= row0 ? __expf(l0 - lref) : 0.f;
                v1 = k1i >= row0 ? __expf(l1 - lref) : 0.f;
                u0 = __expf(fminf(lref - l0, 0.f));
                u1 = __expf(fminf(lref - l1, 0.f));
            }
            wv[lane] = v0; wv[lane + 64] = v1; wu[lane] = u0; wu[lane + 64] = u1;
        }

        // ---- shared tiles for this head
        const int64_t tile = ((b * a.nchunks + c) * a.nheads + h) * (int64_t)(P * N);
        __syncthreads();          // every wave is done with the previous head's tiles
        stage_rows<T, P, N, 256, false>(sS, LDN, static_cast<const T*>(a.S) + tile, N, P, nullptr, tid);
        stage_transposed<T, kQ, P, 256, false>(sZt, LDQ, static_cast<const T*>(a.Z) + b * a.Z_sb + t0 * a.Z_sl + h * a.Z_sh, a.Z_sl,
                                               valid, nullptr, tid);
        if (XT)
            stage_transposed<T, kQ, P, 256, false>(sXt, LDQ, static_cast<const T*>(a.X) + b * a.X_sb + t0 * a.X_sl + h * a.X_sh,
                                                   a.X_sl, valid, nullptr, tid);
        __syncthreads();
        const T* Xg = BWD ? static_cast<const T*>(a.X) + b * a.X_sb + t0 * a.X_sl + h * a.X_sh : nullptr;
        // x[row0 + 8q + 4 half + e][col], e = 0..3, at this lane's accumulator positions
        auto load_x4 = [&](int q, int col, T (&xv)[4]) {
            if (XT) *reinterpret_cast<RawVec<T, 4>*>(xv) = *reinterpret_cast<const RawVec<T, 4>*>(sXt + col * LDQ + row0 + 8 * q + 4 * half);
            else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int row = row0 + 8 * q + 4 * half + e;
                    xv[e] = row < valid ? Xg[(int64_t)row * a.X_sl + col] : (T)0.f;
                }
            }
        };

        // per-row scales: off-diagonal prescale and final row scale (recomputed where used to keep registers free)
        const float off_fast = BWD ? __expf(Lam - lref) : __expf(lref);
        auto off_scale = [&](int v) -> float {
            if (fast) return off_fast;
            const float lr = wl[row0 + acc_row(lane, v)];
            return BWD ? __expf(Lam - lr) : __expf(lr);
        };
        auto fin_scale = [&](int v) -> float { return fast ? wu[row0 + acc_row(lane, v)] : 1.f; };

        // ---- off-diagonal term
        floatx16 acc[1][BN];
        acc_zero(acc);
#pragma unroll
        for (int ks = 0; ks < KSN; ++ks) {
            Frag<T> fo;                      // C (fwd) / B (bwd) row fragment straight from global memory (L2-resident)
            if (ao_ok) fo = load_frag(Ao + ks * 16 + kh8);
            else {
#pragma unroll
                for (int e = 0; e < 8; ++e) fo.v[e] = (T)0.f;
            }
#pragma unroll
            for (int j = 0; j < BN; ++j) {
                const Frag<T> bf = load_frag(sS + (j * 32 + r) * LDN + ks * 16 + kh8);
                mma_frag(acc[0][j], fo, bf);
            }
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float os = off_scale(v);
#pragma unroll
            for (int j = 0; j < BN; ++j) acc[0][j][v] *= os;
        }

        if (BWD) {
            // B_j . dBoff_j = dt_j x_j . dxd_off_j  (the column-role off-diagonal term of the decay gradient)
            float rbv[16];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < BN; ++j) {
                    const int col = j * 32 + r;
                    T xv[4];
                    load_x4(q, col, xv);
#pragma unroll
                    for (int e = 0; e < 4; ++e) s4[e] += acc[0][j][4 * q + e] * to_f32(xv[e]);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) rbv[4 * q + e] = s4[e] * fin_scale(4 * q + e);
            }
            int ri;
            const float tot = half_wave_reduce16(rbv, &ri);
            const int row = row0 + acc_row(lane, ri);
            if ((lane & 1) == 0) s_rb[row] = tot * wd[row];
        }

        // ---- diagonal term: A fragment = masked CB^T fragment scaled by the decay table along k
        const int jrow = row0 + r;            // this lane's A row (token index inside the chunk)
        const float l_row = wl[jrow];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const bool used = BWD ? (ks >= 2 * wave) : (ks <= 2 * wave + 1);
            if (!used) continue;
            float f[8];
            if (fast) {
                const floatx4 fa = *reinterpret_cast<const floatx4*>(wv + ks * 16 + kh8);
                const floatx4 fb = *reinterpret_cast<const floatx4*>(wv + ks * 16 + kh8 + 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) { f[e] = fa[e]; f[4 + e] = fb[e]; }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int k = ks * 16 + kh8 + e;
                    if (!BWD) f[e] = (k <= jrow) ? __expf(l_row - wl[k]) * wd[k] : 0.f;
                    else f[e] = (k >= jrow) ? __expf(wl[k] - l_row) : 0.f;
                }
            }
            const Frag<T> af = scale_frag(FD_RES ? fd[FD_RES ? ks : 0] : load_frag(Gp + ks * 16 + kh8), f);
#pragma unroll
            for (int j = 0; j < BN; ++j) {
                const Frag<T> bf = load_frag(sZt + (j * 32 + r) * LDQ + ks * 16 + kh8);
                mma_frag(acc[0][j], af, bf);
            }
        }

        // ---- epilogue
        if (!BWD) {
            T* Yp = static_cast<T*>(a.Y) + b * a.Y_sb + t0 * a.Y_sl + h * a.Y_sh;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
#pragma unroll
                for (int j = 0; j < BN; ++j) {
                    const int col = j * 32 + r;
                    T xv[4];
                    *reinterpret_cast<RawVec<T, 4>*>(xv) = *reinterpret_cast<const RawVec<T, 4>*>(sZt + col * LDQ + row0 + 8 * q + 4 * half);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int row = row0 + 8 * q + 4 * half + e;
                        if (row < valid)
                            Yp[(int64_t)row * a.Y_sl + col] = from_f32<T>(acc[0][j][4 * q + e] * fin_scale(4 * q + e) + Dh * to_f32(xv[e]));
                    }
                }
            }
        } else {
            T* dXp = static_cast<T*>(a.dX) + b * a.dX_sb + t0 * a.dX_sl + h * a.dX_sh;
            float dirv[16];
            float dD_loc = 0.f;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < BN; ++j) {
                    const int col = j * 32 + r;
                    T xv[4], gv[4];
                    load_x4(q, col, xv);
                    *reinterpret_cast<RawVec<T, 4>*>(gv) = *reinterpret_cast<const RawVec<T, 4>*>(sZt + col * LDQ + row0 + 8 * q + 4 * half);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int row = row0 + 8 * q + 4 * half + e;
                        const float dxd = acc[0][j][4 * q + e] * fin_scale(4 * q + e);
                        const float x_ = to_f32(xv[e]), gy = to_f32(gv[e]);
                        if (row < valid) dXp[(int64_t)row * a.dX_sl + col] = from_f32<T>(wd[row] * dxd + Dh * gy);
                        s4[e] += dxd * x_;
                        dD_loc += gy * x_;
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) dirv[4 * q + e] = s4[e];
            }
            int ri;
            const float tot = half_wave_reduce16(dirv, &ri);
            if ((lane & 1) == 0) s_dir[row0 + acc_row(lane, ri)] = tot;
            dD_loc = warp_sum(dD_loc);
            if (lane == 0) s_red[wave] = dD_loc;
            __syncthreads();      // s_dir, s_rb, s_red complete; also the "tiles are free" barrier for the next head
            if (wave == 0) {
                // da_t = sum_{i>=t} (dl_diag_i + dl_c_i) + sum_{j<t} rb_j + dlam;  lanes hold the tokens in reverse
                // order (127-lane, 63-lane), so the suffix over tokens is an inclusive prefix over lanes and the
                // exclusive prefix over tokens an exclusive suffix over lanes.
                const int64_t bhc = (b * a.nheads + h) * a.nchunks + c;
                const int ta = kQ - 1 - lane, tb = 63 - lane;
                float xa = a.dl_diag[bhc * kQ + ta] + a.dl_c[bhc * kQ + ta];
                float xb = a.dl_diag[bhc * kQ + tb] + a.dl_c[bhc * kQ + tb];
                const float ra = s_rb[ta], rbv = s_rb[tb];
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
                for (int sp = 0; sp < kDlamParts; ++sp) dlm += a.dlam[bhc * kDlamParts + sp];
                const float da_a = xa + dlm, da_b = xb + dlm;
                float dAl = 0.f, dbl = 0.f;
                if (ta < valid) {
                    float val = Ah * da_a + s_dir[ta];
                    if (a.dbp) { val *= softplus_grad_of_value(wd[ta]); dbl += val; }      // wd = softplus(raw dt + bias)
                    const int64_t o = b * a.ddt_sb + (t0 + ta) * a.ddt_sl + h;
                    if (a.dt_f32) static_cast<float*>(a.ddt)[o] = val; else static_cast<T*>(a.ddt)[o] = from_f32<T>(val);
                    dAl += da_a * wd[ta];
                }
                if (tb < valid) {
                    float val = Ah * da_b + s_dir[tb];
                    if (a.dbp) { val *= softplus_grad_of_value(wd[tb]); dbl += val; }
                    const int64_t o = b * a.ddt_sb + (t0 + tb) * a.ddt_sl + h;
                    if (a.dt_f32) static_cast<float*>(a.ddt)[o] = val; else static_cast<T*>(a.ddt)[o] = from_f32<T>(val);
                    dAl += da_b * wd[tb];
                }
                dAl = warp_sum(dAl);
                if (a.dbp) dbl = warp_sum(dbl);
                if (lane == 0) {
                    if (a.dbp) a.dbp[bhc] = dbl;
                    a.dAp[bhc] = dAl;
                    a.dDp[bhc] = s_red[0] + s_red[1] + s_red[2] + s_red[3];
                }
            }
        }
    }
}

}  // namespace m2
