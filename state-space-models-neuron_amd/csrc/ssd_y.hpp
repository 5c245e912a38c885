// SSD forward output kernel for 16-bit operands, software-pipelined over the heads of a group.
//
//     y[i][p] = u_i * ( e^{l_ref} sum_n C[i][n] S_prev[p][n]  +  sum_{j<=i} (G[i][j] v_j) x[j][p] )  +  D x[i][p]
//
// (same factorised decay as ssd_diag.hpp: u_i = e^{l_i - l_ref}, v_j = e^{l_ref - l_j} dt_j per 32-token row block,
// exact per-element fallback when a block's range exceeds kMaxRange).
//
// A workgroup (4 waves, wave w owns token rows 32w..32w+31) handles one chunk of one group and loops over `hps`
// heads.  The two tiles a head needs -- S_prev [P][N] and x [128][P] -- are copied global -> LDS by the
// asynchronous direct-to-LDS loads of gfx950 (no registers involved) into one of two buffers, ONE HEAD AHEAD:
// the copy for head k+1 is issued right after the barrier that opens head k and flies while head k's MFMAs and
// epilogue run.  There is one barrier per head.  Both tiles keep their natural (global) layout in LDS:
//   * S_prev rows are the MFMA B operand as they are (k = n contiguous);
//   * x is needed with k = token contiguous; the LDS transpose read (ds_read_b64_tr_b16) delivers exactly that
//     from the row-major tile, and the epilogue reads the same tile row-wise for the D x term.
// A direct-to-LDS load writes the 64 lanes' 16-byte pieces to 64 CONSECUTIVE LDS slots, so padding rows is not
// possible; bank conflicts are avoided by an XOR swizzle of the slot index inside each row instead (each lane
// simply fetches the global piece that belongs in its slot).
// The head-independent operands stay in registers for the whole loop: the causal C B^T fragments and the C row
// fragments.  The MFMAs are issued with swapped operands, so a lane's accumulators belong to ONE token (transposed
// output block): decay scales and the D x term are lane-local, and after one lane-pair swap per 4-channel group
// (v_permlane32_swap) y leaves in 16-byte row-contiguous stores, rounded once, without a pass through LDS.
#pragma once
#include "ssd_diag.hpp"

namespace m2 {

#define M2_LDS __attribute__((address_space(3)))
#define M2_GLB __attribute__((address_space(1)))

// wait until this wave's outstanding vector-memory operations (including direct-to-LDS loads) are done;
// the export and LDS/scalar counters are left alone.  gfx9 encoding: vmcnt = simm16[15:14,3:0], expcnt [6:4],
// lgkmcnt [11:8].
// A compiler-level memory fence follows, so that no read of the copied data is scheduled before the wait.
__device__ __forceinline__ void wait_vmem_all() {
    __builtin_amdgcn_s_waitcnt(0x0F70);
    asm volatile("" ::: "memory");
}
// ... until at most `groups` * PER of them are still outstanding (vector-memory operations retire in issue order, so
// this leaves the youngest ones in flight).  `groups` must be wave-uniform.  Operations the caller did not count
// (the compiler's own loads and stores) only make the wait longer, never too short.
template <int PER>
__device__ __forceinline__ void wait_vmem_keep(int groups) {
    static_assert(3 * PER < 64, "vmcnt is a 6-bit counter");
    constexpr int n1 = PER, n2 = 2 * PER, n3 = 3 * PER;
    if (groups <= 0) __builtin_amdgcn_s_waitcnt(0x0F70);
    else if (groups == 1) __builtin_amdgcn_s_waitcnt(0x0F70 | (n1 & 0xF) | ((n1 >> 4) << 14));
    else if (groups == 2) __builtin_amdgcn_s_waitcnt(0x0F70 | (n2 & 0xF) | ((n2 >> 4) << 14));
    else __builtin_amdgcn_s_waitcnt(0x0F70 | (n3 & 0xF) | ((n3 >> 4) << 14));
    asm volatile("" ::: "memory");
}

// Asynchronous 16-byte-per-lane copy global -> LDS: lane i reads 16 bytes at  gbase + voff_i  (gbase wave-uniform, voff a
// per-lane BYTE offset) and they land at LDS byte address  lds_addr + 16 i  (lds_addr wave-uniform).
// Written as inline assembly on purpose: for the compiler's own direct-to-LDS builtin the wait-count pass
// makes every later LDS store (and transpose read) wait for ALL outstanding vector-memory operations, which
// serialises exactly the copy/compute overlap this is for.  Completion is awaited explicitly (wait_vmem_all) before
// the barrier that publishes the tile; operations the compiler does not know about can only make its own
// vmcnt waits more conservative, never too short (vmcnt retires in order).
__device__ __forceinline__ void async_copy16(const void* gbase, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(gbase), "s"(lds_addr) : "memory");
}
// LDS byte address of a pointer into shared memory / a value the compiler may keep in a scalar register
__device__ __forceinline__ uint32_t lds_addr_of(const void* p) { return (uint32_t)(uintptr_t)(M2_LDS const void*)p; }
__device__ __forceinline__ uint32_t uniform(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }

// One float at a wave-uniform address through the scalar cache.  The head loops use it for per-head parameters: an ordinary
// load there is a vector-memory operation that the compiler counts on its own, without knowing of the direct-to-LDS copies
// around it, so the wait it puts in front of the value's first use is a vmcnt(0) -- a wait for the NEXT head's tiles in
// front of this head's arithmetic.
__device__ __forceinline__ float load_uniform_f32(const float* p) {
    float v;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(p) : "memory");
    return v;
}

// The [ l | dt ] table of one (batch, head, chunk): 2 kQ floats = 64 lanes x 16 bytes, one wave-wide copy.  Every
// wave of the workgroup issues it (same source, same destination, same data), so each wave may read the table as
// soon as ITS OWN copies have landed, and all waves issue the same number of vector-memory operations per head.
__device__ __forceinline__ void async_copy_ldtab(const float* __restrict__ ldtab, int64_t bhc, uint32_t lds_addr) {
    async_copy16(ldtab + bhc * (2 * kQ), (threadIdx.x & 63) * 16u, lds_addr);
}

// 16-byte slot s of row `row` lives at slot (s ^ tile_swz(row)) of that row: the XOR applied to the slot index
// inside a tile row of SPR slots.  The LDS serves 64 banks x 4 bytes per clock,
// i.e. 16 lanes of a 16-byte read or 32 lanes of an 8-byte transpose read, and both access patterns of these tiles
// must spread over all banks:
//   row-wise fragments : 16 consecutive rows, one slot each          -> 16 different (row parity, slot) bank groups
//   transpose reads    : 4 consecutive rows (aligned), 4 slots each   -> the rows' 4-slot groups must differ
// which a bit permutation of the row index gives (256-byte rows: swap the two low bit pairs; 128-byte rows: bit 0
// already selects the bank half, bits 1..3 go to slot bits 2, 0, 1; 64-byte rows: four consecutive rows are 256 contiguous
// bytes, which is what either access covers, so no permutation is needed).
template <int SPR> __device__ __forceinline__ int tile_swz(int row) {
    static_assert(SPR == 4 || SPR == 8 || SPR == 16, "tile rows of 64, 128 or 256 bytes");
    if (SPR == 4) return 0;
    if (SPR == 16) return ((row & 3) << 2) | ((row >> 2) & 3);
    return (((row >> 1) & 1) << 2) | (((row >> 3) & 1) << 1) | ((row >> 2) & 1);
}

// The same swizzle split for the direct-to-LDS copies: lane `ln` of 64-slot chunk `ch` of a tile fills slot ln % SPR of row
// ch * (64 / SPR) + ln / SPR, and tile_swz of that row is the XOR of a part that depends on the lane alone and a part that
// depends on the (wave-uniform) chunk alone, so the per-lane work of a copy is one XOR on a value computed once per head.
template <int SPR> __device__ __forceinline__ uint32_t copy_lane_slot(uint32_t ln) {      // (ln % SPR) ^ lane part of tile_swz
    static_assert(SPR == 8 || SPR == 16, "tile rows of 128 or 256 bytes");
    if (SPR == 16) return (ln & 15u) ^ ((ln >> 4) << 2);
    const uint32_t lr = ln >> 3;
    return (ln & 7u) ^ ((((lr >> 1) & 1u) << 2) | ((lr >> 2) & 1u));
}
template <int SPR> __device__ __forceinline__ uint32_t copy_chunk_swz(uint32_t ch) {      // chunk part of tile_swz
    return SPR == 16 ? (ch & 3u) : ((ch & 1u) << 1);
}

template <int P, int N>
constexpr size_t y16_smem() {
    return (size_t)2 * ((P * N + kQ * P) * 2 + 2 * kQ * sizeof(float)) + (size_t)4 * (kQ + 32) * sizeof(float);
}

template <typename T, int P, int N>
__global__ void __launch_bounds__(256, (y16_smem<P, N>() <= 80 * 1024 ? 2 : 1))
ssd_y16_kernel(const DiagArgs a) {
    static_assert(sizeof(T) == 2, "16-bit operands only");
    constexpr int BN = P / 32, KSN = N / 16;
    constexpr int SPR_S = N / 8, SPR_X = P / 8;            // 16-byte slots per row
    constexpr int NS = P * SPR_S / 256, NX = kQ * SPR_X / 256;   // direct-to-LDS loads per lane per tile
    constexpr int TAB = kQ + 32;
    // y stores a wave issues per head in a full chunk: a lane stores its half of the 8-channel groups of its token, 16 bytes each.  The
    // epilogue's loops run over exactly these bounds and the tile wait below leaves exactly this many operations in
    // flight, so the two cannot drift apart.
    constexpr int QPAIRS = 2, kStoresPerHead = BN * QPAIRS;
    static_assert(kStoresPerHead * 16 == P, "a token row is stored by a lane pair, 8 channels per store");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* sS = reinterpret_cast<T*>(smem_raw);                       // [2][P][N]     swizzled slots
    T* sX = sS + 2 * P * N;                                       // [2][kQ][P]    swizzled slots
    float* sLD = reinterpret_cast<float*>(sX + 2 * kQ * P);       // [2][ l kQ | dt kQ ]
    float* wt_all = sLD + 2 * 2 * kQ;                             // [4 waves][wv kQ | wu 32]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 31, half = lane >> 5;
    const int64_t c = blockIdx.x, b = blockIdx.z;
    const int64_t g = blockIdx.y / a.nslices, slice = blockIdx.y % a.nslices;
    const int64_t hpg = a.nheads / a.ngroups;
    const int64_t t0 = c * kQ;
    const int valid = (int)((a.seqlen - t0) < kQ ? (a.seqlen - t0) : kQ);
    const int row0 = wave * 32;
    float* wv = wt_all + wave * TAB;
    float* wu = wv + kQ;          // [32]: rows row0 .. row0 + 31

    // ---- asynchronous tile copy of one head into buffer `buf`; the per-lane source offsets do not depend on the head
    const uint32_t wave_u = uniform(wave), lds_S = uniform(lds_addr_of(sS)), lds_X = uniform(lds_addr_of(sX)), lds_LD = uniform(lds_addr_of(sLD));
    uint32_t offS[NS], offX[NX];
#pragma unroll
    for (int it = 0; it < NS; ++it) {
        const int s = (wave * NS + it) * 64 + lane;
        const int row = s / SPR_S, cs = (s % SPR_S) ^ tile_swz<SPR_S>(row);
        offS[it] = (uint32_t)(row * N + cs * 8) * 2u;
    }
#pragma unroll
    for (int it = 0; it < NX; ++it) {
        const int s = (wave * NX + it) * 64 + lane;
        const int row = s / SPR_X, cs = (s % SPR_X) ^ tile_swz<SPR_X>(row);
        // rows past the end of the sequence re-read the last valid row: their dt is 0, so they only ever meet zeros
        const int grow = row < valid ? row : valid - 1;
        offX[it] = (uint32_t)(grow * a.Z_sl + cs * 8) * 2u;
    }
    auto issue_tiles = [&](int64_t h, int buf) {
        const T* Sp = static_cast<const T*>(a.S) + ((b * a.nchunks + c) * a.nheads + h) * (int64_t)(P * N);
#pragma unroll
        for (int it = 0; it < NS; ++it) async_copy16(Sp, offS[it], lds_S + (uint32_t)(buf * (P * N) * 2) + (wave_u * NS + it) * 1024u);
        const T* Xp = static_cast<const T*>(a.Z) + b * a.Z_sb + t0 * a.Z_sl + h * a.Z_sh;
#pragma unroll
        for (int it = 0; it < NX; ++it) async_copy16(Xp, offX[it], lds_X + (uint32_t)(buf * (kQ * P) * 2) + (wave_u * NX + it) * 1024u);
        async_copy_ldtab(a.ldtab, (b * a.nheads + h) * a.nchunks + c, lds_LD + (uint32_t)(buf * 2 * kQ * 4));
    };

    const int64_t h_first = g * hpg + slice * a.hps;
    issue_tiles(h_first, 0);

    // ---- head-independent operands, resident in registers
    Frag<T> fd[8], fo[KSN];
    {
        const T* Gp = static_cast<const T*>(a.Gd) + ((b * a.nchunks + c) * a.ngroups + g) * (int64_t)(kQ * kQ) + (row0 + r) * kQ;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
            if (ks <= 2 * wave + 1) fd[ks] = load_frag(Gp + ks * 16 + half * 8);
        const T* Cp = static_cast<const T*>(a.Aoff) + b * a.Ao_sb + (t0 + row0 + r) * a.Ao_sl + g * a.Ao_sg;
        const bool c_ok = row0 + r < valid;
#pragma unroll
        for (int ks = 0; ks < KSN; ++ks) {
            if (c_ok) fo[ks] = load_frag(Cp + ks * 16 + half * 8);
            else {
#pragma unroll
                for (int e = 0; e < 8; ++e) fo[ks].v[e] = (T)0.f;
            }
        }
    }

    for (int64_t hh = 0; hh < a.hps; ++hh) {
        const int64_t h = h_first + hh;
        const int buf = (int)(hh & 1);
        const float Dh = a.D ? load_uniform_f32(a.D + h) : 0.f;

        // this wave's share of the tiles of head hh, and the whole [ l | dt ] table, have landed.  The y stores of the head
        // before were issued behind these copies and vector-memory operations retire in issue order, so in a full chunk
        // (every lane stores, kStoresPerHead instructions per head) they may stay in flight across the wait
        if (hh > 0 && valid == kQ) wait_vmem_keep<kStoresPerHead>(1); else wait_vmem_all();
        // ---- wave-private decay tables from the shared [ l | dt ] table
        const float* sl = sLD + buf * 2 * kQ;
        const float* sd = sl + kQ;
        const float l_first = sl[row0], l_last = sl[row0 + 31];
        const bool fast = (l_first - l_last) < kMaxRange;
        const float lref = l_first;
        wv[lane] = lane < row0 + 32 ? __expf(lref - sl[lane]) * sd[lane] : 0.f;
        wv[lane + 64] = lane + 64 < row0 + 32 ? __expf(lref - sl[lane + 64]) * sd[lane + 64] : 0.f;
        if (lane < 32) wu[lane] = __expf(fminf(sl[row0 + lane] - lref, 0.f));
        __syncthreads();          // everyone's share has landed; every wave is also done with head hh-1 (the other buffer)
        if (hh + 1 < a.hps) issue_tiles(h + 1, buf ^ 1);
        const T* cS = sS + buf * (P * N);
        const T* cX = sX + buf * (kQ * P);

        // Both products are issued with the operands swapped (the two operand register layouts are the same), so the
        // accumulators hold the TRANSPOSED output block: lane (r, half) owns token row0 + r and, per 32-channel block j,
        // the channels 32 j + 8 q + 4 half + 0..3 (q = 0..3).  Every row-wise quantity (decay scales, the D x term, the
        // stores) is then lane-local.
        const float off_sc = fast ? __expf(lref) : __expf(sl[row0 + r]);

        // ---- off-diagonal term: S_prev (LDS, natural layout) x C rows (registers)
        floatx16 acc[1][BN];
        acc_zero(acc);
#pragma unroll
        for (int ks = 0; ks < KSN; ++ks) {
#pragma unroll
            for (int j = 0; j < BN; ++j) {
                const int row = j * 32 + r;
                const Frag<T> bf = load_frag(cS + (row * SPR_S + ((ks * 2 + half) ^ tile_swz<SPR_S>(row))) * 8);
                mma_frag(acc[0][j], bf, fo[ks]);
            }
        }
#pragma unroll
        for (int j = 0; j < BN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[0][j][v] *= off_sc;

        // ---- diagonal term: causal C B^T fragment scaled by the decay table along k; x through transpose reads
        const int jrow = row0 + r;
        const float l_row = sl[jrow];
        // transpose read: the 16 lanes of a group fetch a [4 tokens][16 channels] block; lane (i0 = bits 3:2, i1 = bits 1:0)
        // supplies the address of token i0, channels 4 i1 .. 4 i1 + 3 and receives channel (lane & 15) of tokens 0..3
        const int tr_tok = 8 * half + ((lane >> 2) & 3);
        const int tr_col = ((lane >> 4) & 1) * 16 + 4 * (lane & 3);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            if (ks > 2 * wave + 1) continue;
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
                    f[e] = (k <= jrow) ? __expf(l_row - sl[k]) * sd[k] : 0.f;
                }
            }
            keep_packed(fd[ks]);
            const Frag<T> af = scale_frag(fd[ks], f);
#pragma unroll
            for (int j = 0; j < BN; ++j) {
                const int col = j * 32 + tr_col;
                const int ta = ks * 16 + tr_tok, tb = ta + 4;
                typedef T tvec4 __attribute__((ext_vector_type(4)));
                const tvec4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
                    (M2_LDS tvec4*)(cX + (ta * SPR_X + ((col >> 3) ^ tile_swz<SPR_X>(ta))) * 8 + (col & 7)));
                const tvec4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
                    (M2_LDS tvec4*)(cX + (tb * SPR_X + ((col >> 3) ^ tile_swz<SPR_X>(tb))) * 8 + (col & 7)));
                Frag<T> bf;
#pragma unroll
                for (int e = 0; e < 4; ++e) { bf.v[e] = lo[e]; bf.v[4 + e] = hi[e]; }
                mma_frag(acc[0][j], bf, af);
            }
        }

        // ---- epilogue: y = u * acc + D x.  A lane and its partner (lane ^ 32) hold the two halves of each group of 8
        //      channels of their token; swapping one 4-channel group per pair (v_permlane32_swap) leaves every lane with
        //      whole groups of 8 consecutive channels: 16-byte stores without a pass through LDS
        const int tok = row0 + r;
        const float fs = fast ? wu[r] : 1.f;
        T* Yp = static_cast<T*>(a.Y) + b * a.Y_sb + t0 * a.Y_sl + h * a.Y_sh + (int64_t)tok * a.Y_sl;
#pragma unroll
        for (int j = 0; j < BN; ++j) {
#pragma unroll
            for (int qp = 0; qp < QPAIRS; ++qp) {
                float g8[8];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    pair_swap(acc[0][j][8 * qp + e], acc[0][j][8 * qp + 4 + e], g8[e], g8[4 + e]);
                }
                const int p0 = j * 32 + 8 * (2 * qp + half);
                const uint4 xr = *reinterpret_cast<const uint4*>(cX + (tok * SPR_X + ((p0 >> 3) ^ tile_swz<SPR_X>(tok))) * 8);
                const T* xe = reinterpret_cast<const T*>(&xr);
                uint4 o;
                T* oe = reinterpret_cast<T*>(&o);
#pragma unroll
                for (int e = 0; e < 8; ++e) oe[e] = from_f32<T>(fs * g8[e] + Dh * to_f32(xe[e]));
                if (tok < valid) *reinterpret_cast<uint4*>(Yp + p0) = o;
            }
        }
    }
}

}  // namespace m2
