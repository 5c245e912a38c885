// SSD backward main kernel for 16-bit operands: dx, the per-token decay-gradient terms, and the state parts of dB and
// dC, from ONE pass over dy, x, dS (gradient of the state leaving the chunk) and S_prev (state entering it).
//
// A workgroup of 8 waves handles one chunk of one group and loops over `hps` heads.  Per head the four tiles --
// dS [P][N], S_prev [P][N], dy [128][P], x [128][P] -- and the [ l | dt ] table are copied global -> LDS
// asynchronously, one head ahead, into one of two buffers (one barrier per head); all tiles keep their global layout
// (slots XOR-swizzled inside each row) and reach the MFMA either row-wise or through LDS transpose reads.
//
// The waves are specialised by role, two per 32-token row block (so that each role's long-lived registers are its own):
//   role A (waves 0-3): dxd[j][p] = u_j ( e^{Lam-l_ref} sum_n B[j][n] dS[p][n] + sum_{i>=j} (G[i][j] v_i) dy[i][p] )
//            dx = dt_j dxd + D dy,   dir_j = sum_p dxd x,   rb_j = dt_j sum_p (state part of dxd) x,   dD partial = sum dy x
//            (B rows and the transposed causal C B^T rows of its tokens stay in registers).
//   role B (waves 4-7):  dB_off[j][n] += dt_j e^{Lam-l_j} sum_p x[j][p] dS[p][n]
//                        dC_off[i][n] += e^{l_i}          sum_p dy[i][p] S_prev[p][n]
//            accumulated over the workgroup's heads in registers (row scale applied in fp32 after the MFMA, so both
//            operands are exact copies of the inputs) and written once at the end; and, from the same product before
//            it is accumulated,   dl_c[i] = e^{l_i} sum_n C[i][n] (sum_p dy[i][p] S_prev[p][n])
//            (the C row of the lane's token stays in registers).
// Every MFMA is issued with its operands swapped, so a lane's accumulators belong to ONE token: row scales and row dot
// products are lane-local (plus one exchange with the partner lane), and dx leaves in 16-byte stores after one
// lane-pair swap per 4-channel group, without a pass through LDS.
// All eight waves also form   dlam[c] = e^{Lam_c} <dS, S_prev>   (the part of dL/dLam_c that flows through the carried
// state) from the two tiles as they lie in LDS, one partial per wave.
// The decay is factorised per row block around its LAST token (see ssd_diag.hpp), with the exact per-element
// fallback when the block's range exceeds kMaxRange.  ddt and dA need a scan over the chunk and are left to da_body (tail1_kernel).
#pragma once
#include "ssd_y.hpp"

namespace m2 {

// of the N / 32 column blocks of a role-B lane's C row, this many are parked in LDS instead of registers
template <int N> constexpr int bwd16_clds() { return N / 32 > 2 ? N / 64 : 0; }
template <int P, int N>
constexpr size_t bwd16_smem() {
    return (size_t)2 * ((2 * P * N + 2 * kQ * P) * 2 + 2 * kQ * sizeof(float)) + (size_t)4 * (kQ + 32) * sizeof(float) +
           (size_t)4 * bwd16_clds<N>() * 4 * 64 * sizeof(uint2);
}
template <typename T, int P, int N>
constexpr bool bwd16_ok() { return sizeof(T) == 2 && bwd16_smem<P, N>() <= 160 * 1024; }

struct Bwd16Args {
    const float* ldtab;                                   // [b][h][c][ l kQ | dt kQ ]
    const float* D;
    const void* Bm; int64_t B_sb, B_sl, B_sg;             // B, C: [b][l][g][N]
    const void* Cm; int64_t C_sb, C_sl, C_sg;
    const void* Gmt;                                      // (causal C B^T)^T: [b][c][g][kQ][kQ]
    const void* dS; const void* Sprev;                    // [b][c][h][P][N]
    const void* dy; int64_t dy_sb, dy_sl, dy_sh;
    const void* x; int64_t x_sb, x_sl, x_sh;
    void* dx; int64_t dx_sb, dx_sl, dx_sh;
    float* dirp; float* rbp; float* dlc;                  // [b][h][c][kQ]
    float* dDp8;                                          // [b][h][c][8]
    float* dlam;                                          // [b][h][c][kDlamParts]
    float* dBp; float* dCp;                               // [b][c][g][slice][kQ][N]
    int64_t seqlen, nheads, ngroups, nchunks, nslices, hps;
};

template <typename T, int P, int N>
__global__ void __launch_bounds__(512, 1)
ssd_bwd16_kernel(const Bwd16Args a) {
    static_assert(sizeof(T) == 2, "16-bit operands only");
    constexpr int BN = P / 32, KSN = N / 16, KSP = P / 16, NBN = N / 32;
    static_assert(kDlamParts == 8 && (P * N) % (512 * 8) == 0, "one dlam partial per wave");
    constexpr int SPR_S = N / 8, SPR_X = P / 8;
    constexpr int NS = P * SPR_S / 512, NX = kQ * SPR_X / 512;
    constexpr int TAB = kQ + 32;
    constexpr int TILES = 2 * P * N + 2 * kQ * P;    // elements per buffer
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* tiles = reinterpret_cast<T*>(smem_raw);                       // [2][ dS | S_prev | dy | x ]
    float* sLD = reinterpret_cast<float*>(tiles + 2 * TILES);        // [2][ l kQ | dt kQ ]
    float* wt_all = sLD + 2 * 2 * kQ;                                // [4 role-A waves][wv kQ | wu 32]
    constexpr int JCL = bwd16_clds<N>(), JCR = NBN - JCL;            // C-row column blocks in LDS / in registers
    uint2* sCw_all = reinterpret_cast<uint2*>(wt_all + 4 * TAB);     // [4 role-B waves][JCL][4][64 lanes]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31, half = lane >> 5;
    const int rbk = wave & 3, role = wave >> 2;      // waves w and w + 4 share a SIMD: one of each role per SIMD
    const int64_t c = blockIdx.x, b = blockIdx.z;
    const int64_t g = blockIdx.y / a.nslices, slice = blockIdx.y % a.nslices;
    const int64_t hpg = a.nheads / a.ngroups;
    const int64_t t0 = c * kQ;
    const int valid = (int)((a.seqlen - t0) < kQ ? (a.seqlen - t0) : kQ);
    const int row0 = rbk * 32;
    const int64_t h_first = g * hpg + slice * a.hps;
    // transpose-read lane roles: the 16 lanes of a group fetch a [4 rows][16 columns] block; lane (i0 = bits 3:2, i1 = bits 1:0)
    // supplies the address of row i0, columns 4 i1 .. 4 i1 + 3 and receives column (lane & 15) of rows 0..3
    const int tr_row = (lane >> 2) & 3;
    const int tr_col = ((lane >> 4) & 1) * 16 + 4 * (lane & 3);
    typedef T tvec4 __attribute__((ext_vector_type(4)));

    const uint32_t wave_u = uniform(wave), lds_T = uniform(lds_addr_of(tiles)), lds_LD = uniform(lds_addr_of(sLD));
    auto issue_tiles = [&](int64_t h, int buf) {
        const int64_t tile = ((b * a.nchunks + c) * a.nheads + h) * (int64_t)(P * N);
        const T* Sp = static_cast<const T*>(a.dS) + tile;
        const T* Pp = static_cast<const T*>(a.Sprev) + tile;
        const uint32_t dst = lds_T + (uint32_t)(buf * TILES * 2);
        // the per-lane source offsets are rebuilt for every head on purpose: kept in registers across the head loop they are
        // the first thing the register allocator spills, and a spill reload in the middle of this sequence waits for all
        // copies issued so far.  Rebuilding is cheap because the swizzle splits into a lane part, formed once here, and a
        // chunk part that is wave-uniform (copy_lane_slot / copy_chunk_swz); the row products are 24-bit multiply-adds.
        uint32_t ln = (uint32_t)lane;
        asm volatile("" : "+v"(ln));
        constexpr int RPC_S = 64 / SPR_S, RPC_X = 64 / SPR_X;       // tile rows per 64-slot chunk
        const uint32_t sS = copy_lane_slot<SPR_S>(ln), sX = copy_lane_slot<SPR_X>(ln);
        const uint32_t lrS = ln / (uint32_t)SPR_S, lrX = ln / (uint32_t)SPR_X;
        const uint32_t baseS = lrS * (uint32_t)(N * 2) + (sS << 4);                 // row and slot fields do not overlap
#pragma unroll
        for (int it = 0; it < NS; ++it) {
            const uint32_t ch = wave_u * NS + it;
            const uint32_t off = ch * (uint32_t)(RPC_S * N * 2) + (baseS ^ (copy_chunk_swz<SPR_S>(ch) << 4));
            async_copy16(Sp, off, dst + ch * 1024u);
            async_copy16(Pp, off, dst + (uint32_t)(P * N * 2) + ch * 1024u);
        }
        const T* Yp = static_cast<const T*>(a.dy) + b * a.dy_sb + t0 * a.dy_sl + h * a.dy_sh;
        const T* Xp = static_cast<const T*>(a.x) + b * a.x_sb + t0 * a.x_sl + h * a.x_sh;
        const uint32_t ypitch = uniform((uint32_t)a.dy_sl * 2u), xpitch = uniform((uint32_t)a.x_sl * 2u), last = (uint32_t)(valid - 1);
#pragma unroll
        for (int it = 0; it < NX; ++it) {
            const uint32_t ch = wave_u * NX + it;
            const uint32_t row = ch * RPC_X + lrX;
            const uint32_t grow = row < last ? row : last;       // rows past the end: finite stand-ins, masked by zero scales
            const uint32_t cs16 = (sX ^ copy_chunk_swz<SPR_X>(ch)) << 4;
            async_copy16(Yp, __umul24(grow, ypitch) + cs16, dst + (uint32_t)(2 * P * N * 2) + ch * 1024u);
            async_copy16(Xp, __umul24(grow, xpitch) + cs16, dst + (uint32_t)((2 * P * N + kQ * P) * 2) + ch * 1024u);
        }
        async_copy_ldtab(a.ldtab, (b * a.nheads + h) * a.nchunks + c, lds_LD + (uint32_t)(buf * 2 * kQ * 4));
    };
    // this wave's share of <dS, S_prev> over the two tiles of buffer `buf` (same slot order in both, so any order will do)
    auto tiles_dot = [&](int buf, int64_t bhc, float Lam) {
        const T* cS = tiles + buf * TILES;
        const T* cP = cS + P * N;
        int t = tid;
        asm volatile("" : "+v"(t));
        float dot = 0.f;
#pragma unroll
        for (int it = 0; it < P * N / (512 * 8); ++it) {
            const uint4 u = *reinterpret_cast<const uint4*>(cS + (it * 512 + t) * 8);
            const uint4 v = *reinterpret_cast<const uint4*>(cP + (it * 512 + t) * 8);
            const uint32_t uw[4] = {u.x, u.y, u.z, u.w}, vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int q = 0; q < 4; ++q) dot = dot2_acc<T>(uw[q], vw[q], dot);
        }
        dot = warp_sum(dot);
        if (lane == 0) a.dlam[bhc * kDlamParts + wave] = __expf(Lam) * dot;
    };
    issue_tiles(h_first, 0);

    if (role == 0) {
        // role A is the longer of the two: its waves go first whenever both waves of a SIMD are ready
        __builtin_amdgcn_s_setprio(2);
        // =============================================================== role A: dx, dir, rb, dl_c, dD
        float* wv = wt_all + rbk * TAB;
        float* wu = wv + kQ;
        Frag<T> fd[8], foB[KSN];
        {
            const T* Gp = static_cast<const T*>(a.Gmt) + ((b * a.nchunks + c) * a.ngroups + g) * (int64_t)(kQ * kQ) + (row0 + r) * kQ;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks)
                if (ks >= 2 * rbk) fd[ks] = load_frag(Gp + ks * 16 + half * 8);
            const T* Bp = static_cast<const T*>(a.Bm) + b * a.B_sb + (t0 + row0 + r) * a.B_sl + g * a.B_sg;
            const bool ok = row0 + r < valid;
#pragma unroll
            for (int ks = 0; ks < KSN; ++ks) {
                if (ok) foB[ks] = load_frag(Bp + ks * 16 + half * 8);
                else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) foB[ks].v[e] = (T)0.f;
                }
            }
        }
        for (int64_t hh = 0; hh < a.hps; ++hh) {
            const int64_t h = h_first + hh;
            const int buf = (int)(hh & 1);
            const int64_t bhc = (b * a.nheads + h) * a.nchunks + c;
            const float Dh = a.D ? a.D[h] : 0.f;

            wait_vmem_all();          // this wave's share of the tiles of head hh, and the whole [ l | dt ] table, have landed
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
            tiles_dot(buf, bhc, Lam);
            const T* cS = tiles + buf * TILES;
            const T* cP = cS + P * N;
            const T* cY = cP + P * N;
            const T* cX = cY + kQ * P;

            // All products below are issued with the MFMA operands swapped (the two operand register layouts are the same),
            // so the accumulators hold TRANSPOSED output blocks: lane (r, half) owns token row0 + r and, per 32-channel
            // block j, the channels 32 j + 8 q + 4 half + 0..3 (q = 0..3).  Row scales, row dot products, the D dy term and
            // the stores are then lane-local (plus one exchange with the partner lane l ^ 32).
            const int tok = row0 + r;
            const float off_sc = fast ? __expf(Lam - lref) : __expf(Lam - sl[tok]);
            const float fin_sc = fast ? wu[r] : 1.f;
            // sum over this lane's channels of t[channel] * Z[tok][channel] (Z: row-major tile of token rows), both lanes of the pair
            auto row_dot = [&](const floatx16 (&t)[1][BN], const T* Z) -> float {
                float s = 0.f;
#pragma unroll
                for (int j = 0; j < BN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int p0 = j * 32 + 8 * q;
                        const uint2 zr = *reinterpret_cast<const uint2*>(Z + (tok * SPR_X + ((p0 >> 3) ^ tile_swz<SPR_X>(tok))) * 8 + 4 * half);
                        s += t[0][j][4 * q + 0] * unpack_lo<T>(zr.x) + t[0][j][4 * q + 1] * unpack_hi<T>(zr.x) +
                             t[0][j][4 * q + 2] * unpack_lo<T>(zr.y) + t[0][j][4 * q + 3] * unpack_hi<T>(zr.y);
                    }
                return lane_xor_add<32>(s);
            };

            // ---- state part of dxd: dS (LDS, natural layout) x B rows (registers)
            floatx16 acc[1][BN];
            acc_zero(acc);
#pragma unroll
            for (int ks = 0; ks < KSN; ++ks) {
#pragma unroll
                for (int j = 0; j < BN; ++j) {
                    const int row = j * 32 + r;
                    const Frag<T> bf = load_frag(cS + (row * SPR_S + ((ks * 2 + half) ^ tile_swz<SPR_S>(row))) * 8);
                    mma_frag(acc[0][j], bf, foB[ks]);
                }
            }
#pragma unroll
            for (int j = 0; j < BN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[0][j][v] *= off_sc;
            __builtin_amdgcn_sched_barrier(0);
            // ---- rb_j = dt_j sum_p x[j][p] * (state part, final scale applied)
            {
                const float tot = row_dot(acc, cX);
                if (half == 0) a.rbp[bhc * kQ + tok] = tot * fin_sc * sd[tok];
            }

            __builtin_amdgcn_sched_barrier(0);
            // ---- diagonal part: transposed causal C B^T fragment scaled along k = i; dy through transpose reads
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
                keep_packed(fd[ks]);
                const Frag<T> af = scale_frag(fd[ks], f);
#pragma unroll
                for (int j = 0; j < BN; ++j) {
                    const int col = j * 32 + tr_col;
                    const int ta = ks * 16 + 8 * half + tr_row, tb = ta + 4;
                    const tvec4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
                        (M2_LDS tvec4*)(cY + (ta * SPR_X + ((col >> 3) ^ tile_swz<SPR_X>(ta))) * 8 + (col & 7)));
                    const tvec4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
                        (M2_LDS tvec4*)(cY + (tb * SPR_X + ((col >> 3) ^ tile_swz<SPR_X>(tb))) * 8 + (col & 7)));
                    Frag<T> bf;
#pragma unroll
                    for (int e = 0; e < 4; ++e) { bf.v[e] = lo[e]; bf.v[4 + e] = hi[e]; }
                    mma_frag(acc[0][j], bf, af);
                }
            }

            __builtin_amdgcn_sched_barrier(0);
            // ---- epilogue: dx = dt_j dxd + D dy, dir_j = sum_p dxd x, dD partial = sum dy x.  One lane-pair swap per
            //      4-channel group leaves every lane with whole groups of 8 consecutive channels of its token: 16-byte
            //      reads of x and dy, 16-byte stores of dx, no pass through LDS
            T* dXp = static_cast<T*>(a.dx) + b * a.dx_sb + t0 * a.dx_sl + h * a.dx_sh + (int64_t)tok * a.dx_sl;
            const float dts = sd[tok] * fin_sc;      // the block's final scale rides on dt here and on the finished row sum below
            float dir = 0.f, dd = 0.f;
#pragma unroll
            for (int j = 0; j < BN; ++j) {
#pragma unroll
                for (int qp = 0; qp < 2; ++qp) {
                    float g8[8];
#pragma unroll
                    for (int e = 0; e < 4; ++e) pair_swap(acc[0][j][8 * qp + e], acc[0][j][8 * qp + 4 + e], g8[e], g8[4 + e]);
                    const int p0 = j * 32 + 8 * (2 * qp + half);
                    const int slot = (p0 >> 3) ^ tile_swz<SPR_X>(tok);
                    const uint4 xr = *reinterpret_cast<const uint4*>(cX + (tok * SPR_X + slot) * 8);
                    const uint4 gr = *reinterpret_cast<const uint4*>(cY + (tok * SPR_X + slot) * 8);
                    const uint32_t xw[4] = {xr.x, xr.y, xr.z, xr.w}, gw[4] = {gr.x, gr.y, gr.z, gr.w};
                    uint32_t ow[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float d0 = g8[2 * e], d1 = g8[2 * e + 1];
                        const float x0 = unpack_lo<T>(xw[e]), x1 = unpack_hi<T>(xw[e]);
                        const float y0 = unpack_lo<T>(gw[e]), y1 = unpack_hi<T>(gw[e]);
                        ow[e] = pack2<T>(dts * d0 + Dh * y0, dts * d1 + Dh * y1);
                        dir += d0 * x0 + d1 * x1;
                        dd = dot2_acc<T>(gw[e], xw[e], dd);
                    }
                    if (tok < valid) *reinterpret_cast<uint4*>(dXp + p0) = uint4{ow[0], ow[1], ow[2], ow[3]};
                }
            }
            dir = lane_xor_add<32>(dir);
            if (half == 0) a.dirp[bhc * kQ + tok] = dir * fin_sc;
            float dD_loc = warp_sum(tok < valid ? dd : 0.f);
            if (lane == 0) { a.dDp8[bhc * 8 + wave] = dD_loc; a.dDp8[bhc * 8 + wave + 4] = 0.f; }
        }
    } else {
        // =============================================================== role B: state parts of dB and dC, and dl_c
        // Operands swapped here too: lane (r, half) owns token row0 + r and, per 32-column block jn, the state columns
        // 32 jn + 8 q + 4 half + 0..3, so the row scales are two scalars per lane.
        floatx16 accB[1][NBN], accC[1][NBN];
        acc_zero(accB);
        acc_zero(accC);
        const int tok = row0 + r;
        // C row of this lane's token in accumulator order (the same for every head of the group)
        uint32_t cw[JCR][4][2];
        uint2* sCw = sCw_all + rbk * (JCL * 4 * 64);                 // written and read back by the same lane only
        {
            const T* Cp = static_cast<const T*>(a.Cm) + b * a.C_sb + (t0 + tok) * a.C_sl + g * a.C_sg;
#pragma unroll
            for (int jn = 0; jn < NBN; ++jn)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    uint2 v = uint2{0u, 0u};
                    if (tok < valid) v = *reinterpret_cast<const uint2*>(Cp + jn * 32 + 8 * q + 4 * half);
                    if (jn < JCR) { cw[jn < JCR ? jn : 0][q][0] = v.x; cw[jn < JCR ? jn : 0][q][1] = v.y; }
                    else sCw[((jn - JCR) * 4 + q) * 64 + lane] = v;
                }
        }
        for (int64_t hh = 0; hh < a.hps; ++hh) {
            const int64_t h = h_first + hh;
            const int buf = (int)(hh & 1);
            wait_vmem_all();
            const float* sl = sLD + buf * 2 * kQ;
            const float* sd = sl + kQ;
            __syncthreads();
            if (hh + 1 < a.hps) issue_tiles(h + 1, buf ^ 1);
            // lane-dependent LDS offsets are rebuilt from the lane number for every head (a few integer instructions):
            // carried across the head loop they are spilled, and every reload waits for the tile copies in flight
            int ln = lane;
            asm volatile("" : "+v"(ln));
            const int r = ln & 31, half = ln >> 5, tok = row0 + r;
            const int tr_row = (ln >> 2) & 3, tr_col = ((ln >> 4) & 1) * 16 + 4 * (ln & 3);
            tiles_dot(buf, (b * a.nheads + h) * a.nchunks + c, sl[kQ - 1]);
            // lane parts of the transpose-read addresses into a [P][N] state tile (byte offsets; see rows_times_state)
            const uint32_t c3 = (uint32_t)(tr_col >> 3);
            const uint32_t LA = (uint32_t)(8 * half + tr_row) * 256u + ((c3 ^ (uint32_t)(2 * half)) << 4) + (uint32_t)(tr_col & 7) * 2u;
            const uint32_t LB = (LA ^ 16u) + 1024u, trs = (uint32_t)tr_row << 6;
            // row scales of this lane's token: dt_j e^{Lam - l_j} (dB side) and e^{l_i} (dC side and dl_c; 0 past the end)
            const float lr = sl[tok];
            const float ws_b = sd[tok] * __expf(sl[kQ - 1] - lr);
            const float ws_c = tok < valid ? __expf(lr) : 0.f;
            const T* cS = tiles + buf * TILES;
            const T* cP = cS + P * N;
            const T* cY = cP + P * N;
            const T* cX = cY + kQ * P;
            float dlc = 0.f;
            // t[tok][n] = sum_p Rows[tok][p] * St[p][n]: the state tile through transpose reads, the rows as they lie
            auto rows_times_state = [&](const T* Rows, const T* St, const float ws, bool with_c, floatx16 (&accum)[1][NBN]) {
                Frag<T> af[KSP];
#pragma unroll
                for (int ks = 0; ks < KSP; ++ks) af[ks] = load_frag(Rows + (tok * SPR_X + ((ks * 2 + half) ^ tile_swz<SPR_X>(tok))) * 8);
                const uint32_t sbase = lds_addr_of(St);
#pragma unroll
                for (int jn = 0; jn < NBN; ++jn) {
                    floatx16 t = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                    const int col = jn * 32 + tr_col;
                    // 256-byte state rows: tile_swz of the rows this lane addresses (ks 16 + 8 half + tr_row, and 4 further) does
                    // not depend on ks, and jn enters the slot only through an XOR with tr_row, so the 16 addresses of a
                    // column block are two lane values plus compile-time offsets
                    const uint32_t xj = ((uint32_t)jn << 6) ^ trs;
                    const uint32_t aA = sbase + LA + xj, aB = sbase + LB + xj;
#pragma unroll
                    for (int ks = 0; ks < KSP; ++ks) {
                        const int pa = ks * 16 + 8 * half + tr_row, pb = pa + 4;
                        tvec4 lo, hi;
                        if constexpr (SPR_S == 16) {
                            lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((M2_LDS tvec4*)(uintptr_t)(aA + (uint32_t)(ks * 16 * 256)));
                            hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((M2_LDS tvec4*)(uintptr_t)(aB + (uint32_t)(ks * 16 * 256)));
                        } else {
                            lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
                                (M2_LDS tvec4*)(St + (pa * SPR_S + ((col >> 3) ^ tile_swz<SPR_S>(pa))) * 8 + (col & 7)));
                            hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
                                (M2_LDS tvec4*)(St + (pb * SPR_S + ((col >> 3) ^ tile_swz<SPR_S>(pb))) * 8 + (col & 7)));
                        }
                        Frag<T> bf;
#pragma unroll
                        for (int e = 0; e < 4; ++e) { bf.v[e] = lo[e]; bf.v[4 + e] = hi[e]; }
                        mma_frag(t, bf, af[ks]);
                    }
#pragma unroll
                    for (int v = 0; v < 16; ++v) accum[0][jn][v] += t[v] * ws;
                    asm volatile("" : "+v"(accum[0][jn]));      // the scaled sum is formed here, not after the last block
                    if (with_c) {
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            uint2 cv;
                            if (jn < JCR) cv = uint2{cw[jn < JCR ? jn : 0][q][0], cw[jn < JCR ? jn : 0][q][1]};
                            else cv = sCw[((jn - JCR) * 4 + q) * 64 + ln];
                            dlc += t[4 * q + 0] * unpack_lo<T>(cv.x) + t[4 * q + 1] * unpack_hi<T>(cv.x) +
                                   t[4 * q + 2] * unpack_lo<T>(cv.y) + t[4 * q + 3] * unpack_hi<T>(cv.y);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);      // keep the next block's operand reads from being hoisted up here
                }
            };
            rows_times_state(cX, cS, ws_b, false, accB);
            rows_times_state(cY, cP, ws_c, true, accC);
            // dl_c[i] = e^{l_i} sum_n C[i][n] (sum_p dy[i][p] S_prev[p][n])
            dlc = lane_xor_add<32>(dlc);
            if (half == 0) a.dlc[((b * a.nheads + h) * a.nchunks + c) * kQ + tok] = dlc * ws_c;
        }
        const int64_t part = (((b * a.nchunks + c) * a.ngroups + g) * a.nslices + slice) * (int64_t)(kQ * N) + (int64_t)tok * N;
#pragma unroll
        for (int jn = 0; jn < NBN; ++jn)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int64_t o = part + jn * 32 + 8 * q + 4 * half;
                *reinterpret_cast<floatx4*>(a.dBp + o) = floatx4{accB[0][jn][4 * q], accB[0][jn][4 * q + 1], accB[0][jn][4 * q + 2], accB[0][jn][4 * q + 3]};
                *reinterpret_cast<floatx4*>(a.dCp + o) = floatx4{accC[0][jn][4 * q], accC[0][jn][4 * q + 1], accC[0][jn][4 * q + 2], accC[0][jn][4 * q + 3]};
            }
    }
}

// Per (batch, head, chunk): da_t = sum_{i>=t} (dl_diag_i + dl_c_i) + sum_{j<t} rb_j + dlam,  ddt_t = A da_t + dir_t,
// dA partial = sum_t da_t dt_t, dD partial = sum of the per-wave partials.  One wave per (b, h, c); lanes hold the tokens in
// reverse order (127 - lane, 63 - lane), so the suffix over tokens is an inclusive prefix over lanes and the exclusive prefix
// over tokens an exclusive suffix over lanes.  The kDaHeads waves of a workgroup (workgroup `blk` of tail1_kernel) take
// consecutive heads of one (batch, chunk): ddt is [b][l][h], so their results for a token are neighbours in memory and
// leave through LDS as one 16-byte (operand type) or two 16-byte (fp32) stores per token instead of one 2- or 4-byte
// store per token and head.
constexpr int kDaHeads = 8;
struct DaArgs {
    const float* ldtab; const float* A; const float* dl_diag; const float* dl_c; const float* dlam;
    const float* dirp; const float* rbp; const float* dDp8;
    void* ddt; int dt_f32; int64_t ddt_sb, ddt_sl; float* dAp; float* dDp;
    float* dbp;            // with softplus folded into the scan: [b][h][c] partials of d_dt_bias, and ddt is w.r.t. the raw dt; else null
    int64_t seqlen, nheads, nchunks, batch;
};
inline int64_t da_blocks(const DaArgs& q) { return q.batch * q.nchunks * ((q.nheads + kDaHeads - 1) / kDaHeads); }
template <typename T>
__device__ __forceinline__ void da_body(const DaArgs& q, int64_t blk) {
    const float* __restrict__ ldtab = q.ldtab; const float* __restrict__ A = q.A;
    const float* __restrict__ dl_diag = q.dl_diag; const float* __restrict__ dl_c = q.dl_c; const float* __restrict__ dlam = q.dlam;
    const float* __restrict__ dirp = q.dirp; const float* __restrict__ rbp = q.rbp; const float* __restrict__ dDp8 = q.dDp8;
    const int dt_f32 = q.dt_f32; const int64_t ddt_sb = q.ddt_sb, ddt_sl = q.ddt_sl;
    float* __restrict__ dAp = q.dAp; float* __restrict__ dDp = q.dDp; float* __restrict__ dbp = q.dbp;
    const int64_t seqlen = q.seqlen, nheads = q.nheads, nchunks = q.nchunks;
    __shared__ float sv[kDaHeads][kQ];      // ddt of the workgroup's heads, [head][token]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t hgroups = (nheads + kDaHeads - 1) / kDaHeads;
    const int64_t hg = blk % hgroups, c = (blk / hgroups) % nchunks, b = blk / (hgroups * nchunks);
    const int64_t h0 = hg * kDaHeads, h = h0 + wave;
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);
    const int ta = kQ - 1 - lane, tb = 63 - lane;
    if (h < nheads) {      // wave-uniform
        const int64_t bhc = (b * nheads + h) * nchunks + c;
        const float Ah = A[h];
        float xa = dl_diag[bhc * kQ + ta] + dl_c[bhc * kQ + ta];
        float xb = dl_diag[bhc * kQ + tb] + dl_c[bhc * kQ + tb];
        const float ra = rbp[bhc * kQ + ta], rbv = rbp[bhc * kQ + tb];
        const float dira = dirp[bhc * kQ + ta], dirb = dirp[bhc * kQ + tb];
        const float dta = ldtab[bhc * 2 * kQ + kQ + ta], dtb = ldtab[bhc * 2 * kQ + kQ + tb];     // 0 past the end of the sequence
        float dlm = 0.f;
#pragma unroll
        for (int sp = 0; sp < kDlamParts; ++sp) dlm += dlam[bhc * kDlamParts + sp];
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
        const float da_a = xa + dlm, da_b = xb + dlm;
        float dAl = 0.f, dbl = 0.f;
        float va = 0.f, vb = 0.f;
        if (ta < valid) {
            va = Ah * da_a + dira;
            if (dbp) { va *= softplus_grad_of_value(dta); dbl += va; }      // dta = softplus(raw dt + bias)
            dAl += da_a * dta;
        }
        if (tb < valid) {
            vb = Ah * da_b + dirb;
            if (dbp) { vb *= softplus_grad_of_value(dtb); dbl += vb; }
            dAl += da_b * dtb;
        }
        sv[wave][ta] = va;
        sv[wave][tb] = vb;
        dAl = warp_sum(dAl);
        if (dbp) dbl = warp_sum(dbl);
        if (lane == 0) {
            dAp[bhc] = dAl;
            if (dbp) dbp[bhc] = dbl;
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < 8; ++w) s += dDp8[bhc * 8 + w];
            dDp[bhc] = s;
        }
    }
    __syncthreads();
    // one token per thread: its kDaHeads (fewer in the last head group) values are consecutive in ddt
    const int t = threadIdx.x;
    if (t < valid) {
        const int hc = (int)(nheads - h0 < kDaHeads ? nheads - h0 : kDaHeads);
        const int64_t oo = b * ddt_sb + (t0 + t) * ddt_sl + h0;
        if (dt_f32) {
            float* o = static_cast<float*>(q.ddt) + oo;
            if (hc == kDaHeads && (reinterpret_cast<uintptr_t>(o) & 15) == 0) {
                *reinterpret_cast<floatx4*>(o) = floatx4{sv[0][t], sv[1][t], sv[2][t], sv[3][t]};
                *reinterpret_cast<floatx4*>(o + 4) = floatx4{sv[4][t], sv[5][t], sv[6][t], sv[7][t]};
            } else {
                for (int k = 0; k < hc; ++k) o[k] = sv[k][t];
            }
        } else {
            T* o = static_cast<T*>(q.ddt) + oo;
            if (hc == kDaHeads && (reinterpret_cast<uintptr_t>(o) & 15) == 0) {
                T e[kDaHeads];
#pragma unroll
                for (int k = 0; k < kDaHeads; ++k) e[k] = from_f32<T>(sv[k][t]);
                *reinterpret_cast<uint4*>(o) = *reinterpret_cast<const uint4*>(e);
            } else {
                for (int k = 0; k < hc; ++k) o[k] = from_f32<T>(sv[k][t]);
            }
        }
    }
}

}  // namespace m2
