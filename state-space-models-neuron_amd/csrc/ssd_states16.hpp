// Chunk states for 16-bit operands in ONE pass: the per-chunk contributions and the recurrence over the chunks fused,
// with the running state in registers (fp32), so that no per-chunk contribution is ever written to memory.
//
//   forward:  S = init;   for c = 0 .. nc-1:   prev[c] = T(S);   S = e^{Lam_c} S + sum_j (dt_j e^{Lam_c - l_j}) x_j (x) B_j;   final = S
//   reverse:  R = dfinal; for c = nc-1 .. 0:   prev[c] = T(R);   dlam[c] = e^{Lam_c} <T(R), sprev[c]>;
//                                              R = e^{Lam_c} R + sum_i e^{l_i} dy_i (x) C_i;   dinit = R
// (dlam is the part of dL/dLam_c that flows through the carried state; sprev[c] = the forward state entering chunk c.
//  With DLAM == false the reverse pass leaves dlam to ssd_bwd16_kernel, which has both tiles in LDS anyway, and does
//  not read sprev at all.)
//
// grid (nheads * 2, batch), N / 32 waves; a workgroup owns one half of the ROWS of the [P][N] state (P / 2 head channels, all
// N columns), wave w the columns [32 w, +32) of them, as 32x32 MFMA accumulator blocks: only that half of the x / dy columns
// is loaded, scaled and staged, so the two workgroups of a head share no work.  Per chunk the MFMA computes
// X_scaled^T [P/2 x kQ] * M [kQ x N]:
//   * M (B or C of the group) comes from the transposed tiles that prep_kernel wrote in MFMA operand order: a wave's
//     B-operand fragment is one contiguous KiB of global memory, loaded straight into registers at the top of the
//     chunk's iteration (the tile is shared by all heads of the group and stays in L2);
//   * x / dy rows are loaded two chunks ahead into registers, scaled per token in fp32, rounded once and written
//     row-major into one of two LDS buffers (one barrier per chunk); the A-operand fragments (k = token contiguous)
//     come out of it through LDS transpose reads.
// The state leaves through an LDS tile of the workgroup's whole slab (one per chunk parity), written before the chunk's barrier
// and read behind it, so that a wave stores whole state rows: its share of the slab is one contiguous piece of memory.
#pragma once
#include "ssd_y.hpp"

namespace m2 {

struct StatePassArgs {
    const void* X; int64_t X_sb, X_sl, X_sh;      // x (forward) / dy (reverse): [b][l][h][P]
    const float* ldtab;                            // [b][h][c][ l kQ | dt kQ ]
    const void* Mt;                                // B^T (forward) / C^T (reverse) tiles: [b][c][g][N x kQ in operand order]
    const float* init;                             // fp32 [b][h][P][N]: initial state / gradient of the final state, or null
    void* prev;                                    // out [b][c][h][P][N], operand type
    float* final_out;                              // out fp32 [b][h][P][N]: final state / gradient of the initial state, or null
    const void* sprev;                             // reverse: [b][c][h][P][N] forward states entering the chunks
    float* dlam;                                   // reverse: out [b][h][c][kDlamParts]
    int64_t seqlen, nheads, ngroups, nchunks;
};

// workgroups per (batch, head): each takes half of the state rows (more, smaller workgroups: the chunk loop is a chain of
// dependent memory round trips, and only other resident waves can fill its gaps).  One workgroup per head (SPLIT = 1: whole
// 128-byte x rows, each operand fragment feeding two products, half the fragment traffic) is slower: reverse pass 52 -> 57 us,
// forward pass with the two-tile operands 56 -> 79 us at b4 l2048 h80.
constexpr int kStatePassSplit = 2;
// one wave per 32 state columns
template <int N> constexpr int state_pass_threads() { return (N / 32) * 64; }
template <int P, int N, bool HILO = false, int SPLIT = kStatePassSplit>
constexpr size_t state_pass_smem() {
    return (size_t)(HILO ? 2 : 1) * 2 * kQ * (P / SPLIT) * 2 + (size_t)2 * (P / SPLIT) * (N + 8) * 2;
}

// HILO: the scaled rows are staged as TWO 16-bit tiles, the rounded value and the rounded remainder, and each k step takes
// two products, so that the fp32 scale dt e^{Lam - l} reaches the accumulators with 16 significand bits instead of 8 (the
// final state is an fp32 output; with one tile its error is that of the operand rounding, 2^-9 of every term).
template <typename T, int P, int N, bool REVERSE, bool DLAM = REVERSE, bool HILO = false, int SPLIT = kStatePassSplit>
__global__ void __launch_bounds__(state_pass_threads<N>(), (SPLIT == 1 ? (P == 64 ? 2 : 1) : (P == 64 ? (DLAM ? 2 : 3) : (DLAM ? 1 : 2))))
state_pass16_kernel(const StatePassArgs a) {
    static_assert(sizeof(T) == 2, "16-bit operands only");
    constexpr int NWAVES = N / 32, THREADS = state_pass_threads<N>();
    constexpr int PH = P / SPLIT;                      // state rows (head channels) of this workgroup
    constexpr int NW = 32;                             // state columns per wave
    static_assert(SPLIT * NWAVES <= kDlamParts, "dlam slots");
    constexpr int PBW = PH / 32, NBW = 1;              // 32x32 blocks per wave
    constexpr int SPR_X = PH / 8;                      // 16-byte slots per staged x row
    constexpr int NXR = kQ * SPR_X / THREADS;              // x pieces per thread per chunk
    constexpr int LDO = N + 8;
    constexpr int LPR = N / 8;                         // lanes per state row (8 elements each)
    constexpr int RPP = 64 / LPR;                      // rows per store pass
    constexpr int RW = PH / NWAVES;                    // rows a wave stores: the workgroup's slab leaves as whole rows
    constexpr int NSP = RW / RPP;                      // store passes
    static_assert(RW % RPP == 0, "whole store passes");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    constexpr int XT = HILO ? 2 : 1;                   // staged tiles per chunk
    T* sX = reinterpret_cast<T*>(smem_raw);                                 // [2][XT][kQ][P / 2], slots swizzled inside each row
    T* sO = sX + 2 * XT * kQ * PH;                                          // [2][P / 2][LDO]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31, half = lane >> 5;
    const int pw = (int)(blockIdx.x / a.nheads);       // which half of the rows
    // the workgroups of one head are nheads apart in the grid: with a head count that is a multiple of 8 they land on the
    // same XCD and share the head's rows in its L2
    const int64_t h = blockIdx.x % a.nheads, b = blockIdx.y;
    const int n0 = wave * NW;                          // first state column of this wave
    const int64_t g = h / (a.nheads / a.ngroups);
    const int64_t bh = b * a.nheads + h;
    const int64_t nc = a.nchunks;
    const int tr_tok = 8 * half + ((lane >> 2) & 3);
    const int tr_col = ((lane >> 4) & 1) * 16 + 4 * (lane & 3);
    typedef T tvec4 __attribute__((ext_vector_type(4)));

    // The MFMAs are issued with swapped operands: acc[i][j][v] is the state at row pw P/2 + 32 i + r, column
    // n0 + 32 j + acc_row(lane, v), i.e. a lane holds groups of 4 consecutive columns of ONE row (8-byte staging writes).
    floatx16 acc[PBW][NBW];
#pragma unroll
    for (int i = 0; i < PBW; ++i)
#pragma unroll
        for (int j = 0; j < NBW; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = pw * PH + i * 32 + r, col = n0 + j * 32 + acc_row(lane, v);
                acc[i][j][v] = a.init ? a.init[bh * (P * N) + row * N + col] : 0.f;
            }

    // two chunks ahead in registers, in two sets used alternately: the x / dy pieces with their token's l and dt, and
    // the chunk's Lam.  The values of chunk cc are consumed before the barrier of its iteration; behind it the same set
    // is loaded with chunk cc + 2, so that a load has two iterations to land.
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    struct Ahead { u32x4 x[NXR]; float l[NXR], d[NXR], lam; };
    auto chunk_of = [&](int64_t cc) -> int64_t {       // cc-th chunk in processing order, clamped to the last one
        const int64_t k = cc < nc ? cc : nc - 1;
        return REVERSE ? nc - 1 - k : k;
    };
    // Addresses are a wave-uniform base (scalar registers) plus a 32-bit per-lane byte offset, recomputed from the thread
    // index where it is cheap: 64-bit per-lane pointers kept alive across the chunk loop cost more registers than the data.
    const uint32_t row_t = (uint32_t)tid / SPR_X, slot_t = (uint32_t)tid % SPR_X;      // piece `it` of this thread: row_t + it * RSTEP
    constexpr int RSTEP = THREADS / SPR_X;
    const uint32_t x_row_bytes = (uint32_t)(a.X_sl * 2);
    auto load_ahead = [&](int64_t c, Ahead& s) {
        const int64_t t0 = c * kQ;
        const uint32_t last = (uint32_t)(((a.seqlen - t0) < kQ ? (a.seqlen - t0) : kQ) - 1);      // last valid row
        const char* xp = reinterpret_cast<const char*>(static_cast<const T*>(a.X) + b * a.X_sb + t0 * a.X_sl + h * a.X_sh + pw * PH);
        const float* tab = a.ldtab + (bh * nc + c) * (2 * kQ);
        s.lam = tab[kQ - 1];
#pragma unroll
        for (int it = 0; it < NXR; ++it) {
            const uint32_t row = row_t + it * RSTEP;
            const uint32_t grow = row < last ? row : last;      // rows past the end: finite stand-ins, scaled by zero
            s.x[it] = *reinterpret_cast<const u32x4*>(xp + (grow * x_row_bytes + slot_t * 16u));
            s.l[it] = tab[row];
            s.d[it] = REVERSE ? (row <= last ? 1.f : 0.f) : tab[kQ + row];      // dt is 0 past the end of the sequence
        }
    };
    // loaded at the top of the iteration that consumes them (so that the wait in front of their use can be counted
    // exactly and leaves the next chunk's rows, issued behind them, in flight): the group's B^T / C^T fragments (L2) and,
    // for the reverse pass, this lane's pieces of the forward state
    Frag<T> bf[NBW][8];
    static_assert(REVERSE || !DLAM, "dlam belongs to the reverse pass");
    u32x4 spr[DLAM ? NSP : 1];
    const uint32_t st_off = (uint32_t)(((pw * PH + wave * RW + lane / LPR) * N + (lane % LPR) * 8) * 2);      // pass ps: + ps * RPP * N * 2
    auto load_same = [&](int64_t c) {
        const char* mp = reinterpret_cast<const char*>(static_cast<const T*>(a.Mt) + ((b * nc + c) * a.ngroups + g) * (int64_t)(N * kQ));
#pragma unroll
        for (int j = 0; j < NBW; ++j)
#pragma unroll
            for (int ks = 0; ks < 8; ++ks)      // see mt_offset
                bf[j][ks].v = *reinterpret_cast<const bf16x8*>(mp + ((uint32_t)lane * 16u + (uint32_t)((((n0 >> 5) + j) * 8 + ks) * 1024)));
        if (DLAM) {
            const char* sp = reinterpret_cast<const char*>(static_cast<const T*>(a.sprev) + ((b * nc + c) * a.nheads + h) * (int64_t)(P * N));
#pragma unroll
            for (int ps = 0; ps < NSP; ++ps) spr[ps] = *reinterpret_cast<const u32x4*>(sp + (st_off + (uint32_t)(ps * RPP * N * 2)));
        }
    };

    auto step = [&](int64_t cc, Ahead& s) {
        const int64_t c = chunk_of(cc);
        const int buf = (int)(cc & 1);
        // Issue priority falls as the workgroup advances, so that of the workgroups sharing a CU the one furthest behind
        // goes first: the hardware otherwise prefers the oldest waves, and the last workgroup placed on a CU that holds
        // one more than its neighbours finishes long after everybody else.
        switch ((int)(cc * 4 / nc)) {
            case 0: __builtin_amdgcn_s_setprio(3); break;
            case 1: __builtin_amdgcn_s_setprio(2); break;
            case 2: __builtin_amdgcn_s_setprio(1); break;
            default: __builtin_amdgcn_s_setprio(0); break;
        }
        T* cX = sX + buf * (XT * kQ * PH);
        __builtin_amdgcn_sched_barrier(0);      // keep this chunk's loads out of the previous chunk's MFMA phase (registers)
        load_same(c);
        // the values loaded one chunk ahead become visible to the optimiser here and no earlier: otherwise their
        // unpacking is scheduled right behind the loads, which then wait for the data a whole chunk too early
#pragma unroll
        for (int it = 0; it < NXR; ++it)
            asm volatile("" : "+v"(s.x[it]), "+v"(s.l[it]), "+v"(s.d[it]));      // whole 128-bit vectors: no re-packing
        asm volatile("" : "+v"(s.lam));
        // ---- scaled rows into LDS
#pragma unroll
        for (int it = 0; it < NXR; ++it) {
            const int row = (int)row_t + it * RSTEP, slot = (int)slot_t;
            const float sc = REVERSE ? s.d[it] * __expf(s.l[it]) : s.d[it] * __expf(s.lam - s.l[it]);
            // word-wise (two elements per 32-bit word), so that the loaded vectors stay four whole registers until here
            u32x4 o;
            if constexpr (HILO) {
                u32x4 o2;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float v0 = unpack_lo<T>(s.x[it][q]) * sc, v1 = unpack_hi<T>(s.x[it][q]) * sc;
                    o[q] = pack2<T>(v0, v1);
                    o2[q] = pack2<T>(v0 - unpack_lo<T>(o[q]), v1 - unpack_hi<T>(o[q]));
                }
                *reinterpret_cast<u32x4*>(cX + kQ * PH + (row * SPR_X + (slot ^ tile_swz<SPR_X>(row))) * 8) = o2;
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q) o[q] = pack2<T>(unpack_lo<T>(s.x[it][q]) * sc, unpack_hi<T>(s.x[it][q]) * sc);
            }
            *reinterpret_cast<u32x4*>(cX + (row * SPR_X + (slot ^ tile_swz<SPR_X>(row))) * 8) = o;
        }
        const float dec = __expf(s.lam);
        // the state as it enters this chunk goes into the slab tile of this parity (the other one may still be read by a
        // wave that is behind: it was filled one barrier ago)
        T* cO = sO + buf * (PH * LDO);
#pragma unroll
        for (int i = 0; i < PBW; ++i)
#pragma unroll
            for (int j = 0; j < NBW; ++j)
#pragma unroll
                for (int qp = 0; qp < 2; ++qp) {
                    // a lane and its partner (lane ^ 32) hold the two halves of every 8-column group: one exchange of the packed
                    // words leaves each with a whole group, written as 16 bytes (8-byte writes of 32 rows at this pitch would
                    // meet pairwise in the same banks)
                    const int q0 = 2 * qp, q1 = q0 + 1;
                    uint32_t o0, o1, o2, o3;
                    pair_swap(pack2<T>(acc[i][j][4 * q0], acc[i][j][4 * q0 + 1]), pack2<T>(acc[i][j][4 * q1], acc[i][j][4 * q1 + 1]), o0, o2);
                    pair_swap(pack2<T>(acc[i][j][4 * q0 + 2], acc[i][j][4 * q0 + 3]), pack2<T>(acc[i][j][4 * q1 + 2], acc[i][j][4 * q1 + 3]), o1, o3);
                    *reinterpret_cast<u32x4*>(cO + (i * 32 + r) * LDO + n0 + j * 32 + 8 * (q0 + half)) = u32x4{o0, o1, o2, o3};
                }
        __syncthreads();          // both tiles are complete; every wave is done with the other buffers
        // the rows two chunks on (past the end: the last chunk once more, rather than branching around the loads)
        load_ahead(chunk_of(cc + 2), s);

        // ---- the state entering (forward) / the gradient leaving (reverse) this chunk: whole rows of the workgroup's slab
        char* op = reinterpret_cast<char*>(static_cast<T*>(a.prev) + ((b * nc + c) * a.nheads + h) * (int64_t)(P * N));
        float dot = 0.f;
#pragma unroll
        for (int ps = 0; ps < NSP; ++ps) {
            const int rl = wave * RW + ps * RPP + lane / LPR, cv = lane % LPR;
            const u32x4 o = *reinterpret_cast<const u32x4*>(cO + rl * LDO + cv * 8);
            *reinterpret_cast<u32x4*>(op + (st_off + (uint32_t)(ps * RPP * N * 2))) = o;
            if (DLAM) {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    dot = dot2_acc<T>(o[q], spr[ps][q], dot);
            }
        }
        if (DLAM) {
            dot = warp_sum(dot);
            if (lane == 0) {
                const int slot = pw * NWAVES + wave;
                a.dlam[(bh * nc + c) * kDlamParts + slot] = dec * dot;
                for (int s2 = slot + SPLIT * NWAVES; s2 < kDlamParts; s2 += SPLIT * NWAVES) a.dlam[(bh * nc + c) * kDlamParts + s2] = 0.f;
            }
        }

        // ---- S = e^{Lam} S + X_scaled^T M  (accumulated as its transpose M^T X_scaled)
#pragma unroll
        for (int i = 0; i < PBW; ++i)
#pragma unroll
            for (int j = 0; j < NBW; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] *= dec;
        // all A-operand fragments of the chunk are read from LDS first: the eight products form one dependent chain, and a
        // read issued next to its product would put an LDS round trip between any two of them
#pragma unroll
        for (int xt = 0; xt < XT; ++xt) {
            const T* tX = cX + xt * (kQ * PH);
            Frag<T> af[PBW][8];
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                const int ta = ks * 16 + tr_tok, tb = ta + 4;
#pragma unroll
                for (int i = 0; i < PBW; ++i) {
                    const int col = i * 32 + tr_col;
                    const tvec4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
                        (M2_LDS tvec4*)(tX + (ta * SPR_X + ((col >> 3) ^ tile_swz<SPR_X>(ta))) * 8 + (col & 7)));
                    const tvec4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
                        (M2_LDS tvec4*)(tX + (tb * SPR_X + ((col >> 3) ^ tile_swz<SPR_X>(tb))) * 8 + (col & 7)));
#pragma unroll
                    for (int e = 0; e < 4; ++e) { af[i][ks].v[e] = lo[e]; af[i][ks].v[4 + e] = hi[e]; }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int ks = 0; ks < 8; ++ks)
#pragma unroll
                for (int i = 0; i < PBW; ++i)
#pragma unroll
                    for (int j = 0; j < NBW; ++j) mma_frag(acc[i][j], bf[j][ks], af[i][ks]);
            if (XT > 1) __builtin_amdgcn_sched_barrier(0);
        }
    };

    // Chunks are taken two per loop iteration (one per register set); an odd first chunk is peeled off in front so that
    // the loop body is free of conditionals (a branch around loads costs register copies, and with them early waits).
    Ahead s0, s1;
    int64_t cc = 0;
    if (nc & 1) {
        load_ahead(chunk_of(0), s1);
        load_ahead(chunk_of(1), s0);
        step(0, s1);
        cc = 1;
    } else {
        load_ahead(chunk_of(0), s0);
        load_ahead(chunk_of(1), s1);
    }
#pragma unroll 1
    for (; cc < nc; cc += 2) {
        step(cc, s0);
        step(cc + 1, s1);
    }
    if (a.final_out) {
#pragma unroll
        for (int i = 0; i < PBW; ++i)
#pragma unroll
            for (int j = 0; j < NBW; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = pw * PH + i * 32 + r, col = n0 + j * 32 + acc_row(lane, v);
                    a.final_out[bh * (P * N) + row * N + col] = acc[i][j][v];
                }
    }
}

}  // namespace m2
