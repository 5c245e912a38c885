// MFMA tile helpers for gfx950 (CDNA4, 64-lane wavefronts).
//
// All SSD contractions are expressed as  OUT[m][n] += sum_k A[m][k] * Bt[n][k]  with BOTH
// operands staged in LDS with k contiguous, so every lane fetches its MFMA fragment with one
// 16-byte ds_read (bf16) and the two operands use the same code path.
//
//   bf16: v_mfma_f32_32x32x16_bf16   lane -> row (lane & 31), k = 8 * (lane >> 5) + 0..7
//   fp32: v_mfma_f32_32x32x2_f32     eight steps per 16 k, same lane -> (row, k) assignment (see Frag)
//   accumulator (both): 16 floats per lane; register v of lane holds
//        column  (lane & 31),   row  8 * (v >> 2) + 4 * (lane >> 5) + (v & 3)
#pragma once
#include "common.hpp"

namespace m2 {

constexpr int kQ = M2_CHUNK;   // 128 tokens per chunk

template <typename T> struct MmaTraits;
template <> struct MmaTraits<bf16_t> { static constexpr int kPad = 8; };
template <> struct MmaTraits<float> { static constexpr int kPad = 4; };

// leading dimension (elements) of an LDS tile with `k` contiguous columns; the pad keeps
// 16-byte alignment of every row and spreads rows over banks.
template <typename T> __host__ __device__ constexpr int lds_ld(int k) { return k + MmaTraits<T>::kPad; }

__device__ __forceinline__ int acc_row(int lane, int v) { return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3); }
__device__ __forceinline__ int acc_col(int lane) { return lane & 31; }

template <int BM, int BN>
__device__ __forceinline__ void acc_zero(floatx16 (&acc)[BM][BN]) {
#pragma unroll
    for (int i = 0; i < BM; ++i)
#pragma unroll
        for (int j = 0; j < BN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
}

// A fragment is the slice of an MFMA operand one lane owns for a 16-wide k step: 8 CONSECUTIVE k values,
// k = k0 + 8 * (lane >> 5) + 0..7, of row (lane & 31).  For bf16 this is the register layout of
// v_mfma_f32_32x32x16_bf16.  For fp32 the same 8 values are fed to eight v_mfma_f32_32x32x2_f32 (element s of
// both operands in step s); the hardware would pair k = 2s + (lane >> 5), but a contraction does not care in
// which order k is visited as long as A and B agree, and the contiguous form needs two 16-byte reads
// instead of eight scalar ones.
template <typename T> struct Frag;
template <> struct Frag<bf16_t> { bf16x8 v; };
template <> struct Frag<float> { float v[8]; };

__device__ __forceinline__ Frag<bf16_t> load_frag(const bf16_t* __restrict__ p) {
    Frag<bf16_t> f;
    f.v = *reinterpret_cast<const bf16x8*>(p);
    return f;
}
__device__ __forceinline__ Frag<float> load_frag(const float* __restrict__ p) {
    Frag<float> f;
    const floatx4 a = *reinterpret_cast<const floatx4*>(p), b = *reinterpret_cast<const floatx4*>(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) { f.v[i] = a[i]; f.v[4 + i] = b[i]; }
    return f;
}
__device__ __forceinline__ void mma_frag(floatx16& acc, const Frag<bf16_t>& a, const Frag<bf16_t>& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, acc, 0, 0, 0);
}
__device__ __forceinline__ void mma_frag(floatx16& acc, const Frag<float>& a, const Frag<float>& b) {
#pragma unroll
    for (int s = 0; s < 8; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[s], b.v[s], acc, 0, 0, 0);
}
// element-wise scale of a fragment by 8 fp32 factors (one per k), result rounded to the operand type
__device__ __forceinline__ Frag<bf16_t> scale_frag(const Frag<bf16_t>& a, const float (&f)[8]) {
    Frag<bf16_t> r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r.v[i] = (bf16_t)((float)a.v[i] * f[i]);
    return r;
}
__device__ __forceinline__ Frag<float> scale_frag(const Frag<float>& a, const float (&f)[8]) {
    Frag<float> r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r.v[i] = a.v[i] * f[i];
    return r;
}

// the two 16-bit elements of a 32-bit word as fp32, and back (round to nearest even)
template <typename T> __device__ __forceinline__ float unpack_lo(uint32_t w);
template <typename T> __device__ __forceinline__ float unpack_hi(uint32_t w);
template <> __device__ __forceinline__ float unpack_lo<bf16_t>(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
template <> __device__ __forceinline__ float unpack_hi<bf16_t>(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
// c + a.lo * b.lo + a.hi * b.hi for two words of 16-bit pairs in one instruction (v_dot2c_f32_bf16): the products of two
// 8-bit significands are exact in fp32, so this is the same sum as two FMAs on unpacked values, without the four unpacks
template <typename T> __device__ __forceinline__ float dot2_acc(uint32_t a, uint32_t b, float c);
template <> __device__ __forceinline__ float dot2_acc<bf16_t>(uint32_t a, uint32_t b, float c) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf2, a), __builtin_bit_cast(bf2, b), c, false);
}
template <typename T> __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef T tvec2 __attribute__((ext_vector_type(2)));
    const tvec2 v = {from_f32<T>(lo), from_f32<T>(hi)};
    return __builtin_bit_cast(uint32_t, v);
}

// Lane-pair exchange (lanes l and l + 32): lo = { own a | partner's b }, hi = { partner's a | own b } for the lower | upper
// half of the wave (v_permlane32_swap).  With the transposed 32x32 accumulator layout (a lane and its partner hold the two
// halves of each 8-element group of one row) this leaves every lane with whole groups of 8 consecutive elements.
// (The scalars are passed by value on purpose: a bit cast applied directly to a vector element reads element 0.)
__device__ __forceinline__ void pair_swap(uint32_t a, uint32_t b, uint32_t& lo, uint32_t& hi) {
    const auto sw = __builtin_amdgcn_permlane32_swap(a, b, false, false);
    lo = sw[0];
    hi = sw[1];
}
__device__ __forceinline__ void pair_swap(float a, float b, float& lo, float& hi) {
    const uint32_t ua = __builtin_bit_cast(uint32_t, a), ub = __builtin_bit_cast(uint32_t, b);
    const auto sw = __builtin_amdgcn_permlane32_swap(ua, ub, false, false);
    const uint32_t r0 = sw[0], r1 = sw[1];
    lo = __builtin_bit_cast(float, r0);
    hi = __builtin_bit_cast(float, r1);
}

// Makes a fragment opaque to the optimiser at this point (no instruction is emitted).  Used on loop-invariant
// fragments that are re-scaled inside a loop: without it the bf16 -> fp32 unpacking of the fragment is hoisted out of
// the loop and the fragment then occupies eight fp32 registers instead of four packed ones for the whole loop.
__device__ __forceinline__ void keep_packed(Frag<bf16_t>& f) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    u32x4 raw = __builtin_bit_cast(u32x4, f.v);
    asm volatile("" : "+v"(raw));
    f.v = __builtin_bit_cast(bf16x8, raw);
}
__device__ __forceinline__ void keep_packed(Frag<float>&) {}

// One wave: acc[i][j] (32x32 blocks) += A[rows i*32.., k0:k1] * Bt[rows j*32.., k0:k1]^T, operands in LDS.
// A points at the first of this wave's BM*32 rows, Bt at the first of its BN*32 rows.  k0, k1 multiples of 16.
template <int BM, int BN, typename T>
__device__ __forceinline__ void wave_mma(floatx16 (&acc)[BM][BN], const T* __restrict__ A, int lda,
                                         const T* __restrict__ Bt, int ldb, int k0, int k1) {
    const int lane = threadIdx.x & 63;
    const int r = lane & 31, kh = (lane >> 5) * 8;
    for (int k = k0; k < k1; k += 16) {
        Frag<T> a[BM], b[BN];
#pragma unroll
        for (int i = 0; i < BM; ++i) a[i] = load_frag(A + (i * 32 + r) * lda + k + kh);
#pragma unroll
        for (int j = 0; j < BN; ++j) b[j] = load_frag(Bt + (j * 32 + r) * ldb + k + kh);
#pragma unroll
        for (int i = 0; i < BM; ++i)
#pragma unroll
            for (int j = 0; j < BN; ++j) mma_frag(acc[i][j], a[i], b[j]);
    }
}

// ------------------------------------------------------------------------------------------
// Cooperative staging, global -> LDS.  NT threads; `tid` in [0, NT).
//
// stage_rows: global tile [ROWS][COLS] (COLS contiguous, row stride gstride) -> LDS [ROWS][ld].
// Rows >= valid are zero-filled.  If SCALE, row r is multiplied by rowscale[r] (fp32) first.
template <typename T, int ROWS, int COLS, int NT, bool SCALE>
__device__ __forceinline__ void stage_rows(T* __restrict__ s, int ld, const T* __restrict__ g, int64_t gstride,
                                           int valid, const float* __restrict__ rowscale, int tid) {
    constexpr int V = VecTraits<T>::kVec;
    constexpr int VPR = COLS / V;
    constexpr int TOTAL = ROWS * VPR;
    static_assert(COLS % V == 0, "tile width must be a multiple of the vector width");
    if (!SCALE) {
        // plain copy: 16 bytes stay 16 bytes, no conversion
#pragma unroll 4
        for (int e = tid; e < TOTAL; e += NT) {
            const int r = e / VPR, cv = e % VPR;
            uint4 raw = uint4{0u, 0u, 0u, 0u};
            if (r < valid) raw = *reinterpret_cast<const uint4*>(g + (int64_t)r * gstride + cv * V);
            *reinterpret_cast<uint4*>(s + r * ld + cv * V) = raw;
        }
        return;
    }
#pragma unroll 4
    for (int e = tid; e < TOTAL; e += NT) {
        const int r = e / VPR, cv = e % VPR;
        float v[V];
        if (r < valid) load16(g + (int64_t)r * gstride + cv * V, v);
        else {
#pragma unroll
            for (int i = 0; i < V; ++i) v[i] = 0.f;
        }
        if (SCALE) {
            const float sc = rowscale[r];
#pragma unroll
            for (int i = 0; i < V; ++i) v[i] *= sc;
        }
        store16(s + r * ld + cv * V, v);
    }
}

// stage_transposed: global tile [ROWS][COLS] (COLS contiguous) -> LDS [COLS][ld], element (c, r).
// Global reads stay 16-byte and coalesced; the transpose happens in the (2- or 4-byte) LDS writes.
template <typename T, int ROWS, int COLS, int NT, bool SCALE>
__device__ __forceinline__ void stage_transposed(T* __restrict__ s, int ld, const T* __restrict__ g, int64_t gstride,
                                                 int valid, const float* __restrict__ rowscale, int tid) {
    constexpr int V = VecTraits<T>::kVec;
    constexpr int VPR = COLS / V;
    constexpr int TOTAL = ROWS * VPR;
    static_assert(COLS % V == 0, "tile width must be a multiple of the vector width");
    if (!SCALE) {
#pragma unroll 4
        for (int e = tid; e < TOTAL; e += NT) {
            const int cv = e / ROWS, r = e % ROWS;
            uint4 raw = uint4{0u, 0u, 0u, 0u};
            if (r < valid) raw = *reinterpret_cast<const uint4*>(g + (int64_t)r * gstride + cv * V);
            const T* el = reinterpret_cast<const T*>(&raw);
#pragma unroll
            for (int i = 0; i < V; ++i) s[(cv * V + i) * ld + r] = el[i];
        }
        return;
    }
#pragma unroll 4
    for (int e = tid; e < TOTAL; e += NT) {
        // consecutive threads take consecutive tokens of the same channel vector: the LDS writes of a
        // wave then fall into consecutive addresses of V rows (few bank conflicts), while the global
        // reads of a wave are 64 rows x 16 bytes.
        const int cv = e / ROWS, r = e % ROWS;
        float v[V];
        if (r < valid) load16(g + (int64_t)r * gstride + cv * V, v);
        else {
#pragma unroll
            for (int i = 0; i < V; ++i) v[i] = 0.f;
        }
        const float sc = SCALE ? rowscale[r] : 1.f;
#pragma unroll
        for (int i = 0; i < V; ++i) s[(cv * V + i) * ld + r] = from_f32<T>(SCALE ? v[i] * sc : v[i]);
    }
}

// Sum of v over the 32 lanes that share (lane >> 5), for 16 values at once (the 16 accumulator rows of a lane),
// by a butterfly reduce-scatter: 16 cross-lane moves instead of 80.  On return every lane holds ONE total:
// that of register index  r = 8*b4 + 4*b3 + 2*b2 + b1  (b_k = bit k of lane), i.e. of accumulator row
// acc_row(lane, r); lanes differing only in bit 0 hold the same total.
__device__ __forceinline__ float half_wave_reduce16(float (&v)[16], int* reg_index) {
    const int lane = threadIdx.x & 63;
    const bool b4 = lane & 16, b3 = lane & 8, b2 = lane & 4, b1 = lane & 2;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const float keep = b4 ? v[k + 8] : v[k], send = b4 ? v[k] : v[k + 8];
        v[k] = keep + lane_xor<16>(send);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float keep = b3 ? v[k + 4] : v[k], send = b3 ? v[k] : v[k + 4];
        v[k] = keep + lane_xor<8>(send);
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const float keep = b2 ? v[k + 2] : v[k], send = b2 ? v[k] : v[k + 2];
        v[k] = keep + lane_xor<4>(send);
    }
    {
        const float keep = b1 ? v[1] : v[0], send = b1 ? v[0] : v[1];
        v[0] = keep + lane_xor<2>(send);
    }
    v[0] = lane_xor_add<1>(v[0]);
    *reg_index = (b4 ? 8 : 0) + (b3 ? 4 : 0) + (b2 ? 2 : 0) + (b1 ? 1 : 0);
    return v[0];
}

// Wave-private chunk cumulative sum: every wave computes l for all 128 tokens by itself (lane holds tokens
// `lane` and `lane + 64`), so no block barrier is needed.  Tokens >= valid behave as dt = 0.
// Split in two so that the loads of the next head's dt can be issued long before they are needed.
template <typename T>
__device__ __forceinline__ void wave_dt_load(const void* __restrict__ dt, int dt_f32, int64_t off, int64_t stride_l,
                                             int valid, float& d0, float& d1) {
    const int lane = threadIdx.x & 63;
    d0 = 0.f; d1 = 0.f;
    if (dt_f32) {
        const float* p = static_cast<const float*>(dt) + off;
        if (lane < valid) d0 = p[(int64_t)lane * stride_l];
        if (lane + 64 < valid) d1 = p[(int64_t)(lane + 64) * stride_l];
    } else {
        const T* p = static_cast<const T*>(dt) + off;
        if (lane < valid) d0 = to_f32(p[(int64_t)lane * stride_l]);
        if (lane + 64 < valid) d1 = to_f32(p[(int64_t)(lane + 64) * stride_l]);
    }
}
// The same loads without conversion or divergent branches (addresses of tokens >= valid are clamped), so that
// nothing forces a wait for them where they are issued; wave_dt_cvt turns them into dt values where they are used.
template <typename T>
__device__ __forceinline__ void wave_dt_load_raw(const void* __restrict__ dt, int dt_f32, int64_t off, int64_t stride_l,
                                                 int valid, uint32_t& r0, uint32_t& r1) {
    const int lane = threadIdx.x & 63;
    const int t0 = lane < valid ? lane : valid - 1, t1 = lane + 64 < valid ? lane + 64 : valid - 1;
    if (dt_f32) {
        const uint32_t* p = static_cast<const uint32_t*>(dt) + off;
        r0 = p[(int64_t)t0 * stride_l]; r1 = p[(int64_t)t1 * stride_l];
    } else {
        static_assert(sizeof(T) == 2 || sizeof(T) == 4, "dt element size");
        if (sizeof(T) == 2) {
            const uint16_t* p = static_cast<const uint16_t*>(dt) + off;
            r0 = p[(int64_t)t0 * stride_l]; r1 = p[(int64_t)t1 * stride_l];
        } else {
            const uint32_t* p = static_cast<const uint32_t*>(dt) + off;
            r0 = p[(int64_t)t0 * stride_l]; r1 = p[(int64_t)t1 * stride_l];
        }
    }
}
template <typename T>
__device__ __forceinline__ void wave_dt_cvt(int dt_f32, int valid, uint32_t r0, uint32_t r1, float& d0, float& d1) {
    const int lane = threadIdx.x & 63;
    if (dt_f32 || sizeof(T) == 4) { d0 = __uint_as_float(r0); d1 = __uint_as_float(r1); }
    else { d0 = __uint_as_float(r0 << 16); d1 = __uint_as_float(r1 << 16); }      // bf16 bits -> fp32
    if (lane >= valid) d0 = 0.f;
    if (lane + 64 >= valid) d1 = 0.f;
}
__device__ __forceinline__ void wave_cumsum_from(float A, float d0, float d1, float& l0, float& l1) {
    const int lane = threadIdx.x & 63;
    l0 = A * d0; l1 = A * d1;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float n0 = __shfl_up(l0, o, 64), n1 = __shfl_up(l1, o, 64);
        if (lane >= o) { l0 += n0; l1 += n1; }
    }
    l1 += __shfl(l0, 63, 64);
}
template <typename T>
__device__ __forceinline__ void wave_chunk_cumsum(const void* __restrict__ dt, int dt_f32, int64_t off, int64_t stride_l,
                                                  int valid, float A, float& l0, float& l1, float& d0, float& d1) {
    wave_dt_load<T>(dt, dt_f32, off, stride_l, valid, d0, d1);
    wave_cumsum_from(A, d0, d1, l0, l1);
}

// Per (batch, head, chunk) the cumulative log-decay and dt are computed once (ld_table_body, prep_kernel) into a table of
// 2 * kQ floats, [ l[0..kQ) | dt[0..kQ) ], tokens past the end of the sequence holding dt = 0 and the last l.
// Lane holds tokens `lane` and `lane + 64`.
__device__ __forceinline__ void wave_ld_load(const float* __restrict__ ldtab, int64_t bhc, float& l0, float& l1, float& d0, float& d1) {
    const int lane = threadIdx.x & 63;
    const float* p = ldtab + bhc * (2 * kQ);
    l0 = p[lane]; l1 = p[lane + 64]; d0 = p[kQ + lane]; d1 = p[kQ + lane + 64];
}

// Orders this wave's LDS writes before its later LDS reads of what OTHER lanes of the same wave wrote
// (wave-private staging buffers).  The hardware executes one wave's LDS operations in order; the fences
// keep the compiler from reordering them.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Inclusive cumulative sum l[t] = sum_{s<=t} A * dt[s] over one chunk (kQ = 128 tokens), in fp32.
// Tokens >= valid behave as dt = 0 (no decay, no input).  Results in LDS: s_l[kQ], s_dt[kQ].
// Must be called by all threads of the block (contains barriers); blockDim.x >= 128.
template <typename DT>
__device__ __forceinline__ void chunk_cumsum(const DT* __restrict__ dt, int64_t stride_l, int valid, float A,
                                             float* __restrict__ s_l, float* __restrict__ s_dt,
                                             float* __restrict__ s_tmp, int tid) {
    float a = 0.f, d = 0.f;
    if (tid < kQ) {
        if (tid < valid) d = to_f32(dt[(int64_t)tid * stride_l]);
        a = A * d;
        const int lane = tid & 63;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const float nb = __shfl_up(a, off, 64);
            if (lane >= off) a += nb;
        }
        if (tid == 63) s_tmp[0] = a;
    }
    __syncthreads();
    if (tid < kQ) {
        if (tid >= 64) a += s_tmp[0];
        s_l[tid] = a;
        s_dt[tid] = d;
    }
    __syncthreads();
}

// dt is stored either as fp32 or in the activation type T; `off` is the element offset of token 0.
template <typename T>
__device__ __forceinline__ void chunk_cumsum_any(const void* __restrict__ dt, int dt_f32, int64_t off, int64_t stride_l,
                                                 int valid, float A, float* __restrict__ s_l, float* __restrict__ s_dt,
                                                 float* __restrict__ s_tmp, int tid) {
    if (dt_f32) chunk_cumsum<float>(static_cast<const float*>(dt) + off, stride_l, valid, A, s_l, s_dt, s_tmp, tid);
    else chunk_cumsum<T>(static_cast<const T*>(dt) + off, stride_l, valid, A, s_l, s_dt, s_tmp, tid);
}

}  // namespace m2
