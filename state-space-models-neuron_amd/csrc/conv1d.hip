// Causal depthwise conv1d (+activation), forward and backward, for gfx950.
//
// Replaces the reference's NKI kernels conv1d_with_transpose (mamba2/conv1d_grouped.py:66-125),
// conv1d_with_transpose_bwd (:129-194) and conv1d_grouped_kernel_grad (:198-262).
//
// The op is HBM-bandwidth bound (8 FLOP + one SiLU per element), so the fast path is a
// streaming kernel on the channels-last (b, l, C) layout the mixer uses: one thread owns
// one 16-byte channel vector and walks TL consecutive tokens with the k-1 token history in
// registers, so every element is loaded once (plus a (k-1)/TL halo) and all global accesses
// are 16-byte, lane-contiguous along channels.  No transposes (the reference needs two per
// tile because its engine wants channels on partitions).
//
// The backward recomputes the pre-activation, forms g = dy * act'(z) and emits dx with a
// k-1 token lag, so the cross-segment halo is exact (the reference zero-pads g per tile and
// loses that contribution).  dw/db are reduced in fp32: registers -> LDS per block ->
// per-block partials in the workspace -> one small second-stage kernel.  No float atomics.
//
// A generic path (any strides, k <= 8, any C) covers the channel-major (b, C, l) layout of
// ConvNKI and unaligned shapes with one thread per output element.
#include "common.hpp"

namespace m2 {
namespace {

constexpr int kMaxK = 8;
#ifndef M2_CONV_TLF
#define M2_CONV_TLF 16
#endif
#ifndef M2_CONV_TLB
#define M2_CONV_TLB 32
#endif
#ifndef M2_CONV_UNR
#define M2_CONV_UNR 4
#endif
#ifndef M2_CONV_VF
#define M2_CONV_VF 8
#endif
#ifndef M2_CONV_VB
#define M2_CONV_VB 4
#endif
// Tokens per thread in the fast path, and bytes of channels per thread (VF forward, VB backward; at least two channels).
// Both directions are short on loads in flight, so they take short segments (many threads).  The backward carries five
// sums, two 3-token windows and the taps per channel: with two channels per thread it needs 96 registers (five waves per
// SIMD), with four 160 (three waves), and the narrower form is the faster one although its loads are 4-byte ones.
constexpr int kTLF = M2_CONV_TLF;
constexpr int kTLB = M2_CONV_TLB;
constexpr int kUNR = M2_CONV_UNR;    // tokens whose loads are in flight together
#ifndef M2_CONV_CVT
#define M2_CONV_CVT 64
#endif
#ifndef M2_CONV_SEG
#define M2_CONV_SEG 4
#endif
#ifndef M2_CONV_NT
#define M2_CONV_NT 1
#endif
constexpr int kCVT = M2_CONV_CVT;    // channel vectors per block (x dimension)
constexpr int kSEG = M2_CONV_SEG;    // token segments per block (y dimension)
static_assert(kTLF % kUNR == 0 && kTLB % kUNR == 0 && kUNR >= 3, "segments are whole load groups; the dx lag fits one group");

// streaming loads/stores of the activations (optionally non-temporal: nothing is re-read soon enough to be worth caching)
template <int BYTES> struct StreamVec;
template <> struct StreamVec<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };
template <> struct StreamVec<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <> struct StreamVec<4> { typedef uint32_t type; };
template <typename T, int V>
__device__ __forceinline__ RawVec<T, V> ld_stream(const T* __restrict__ p) {
    using S = typename StreamVec<V * (int)sizeof(T)>::type;
    RawVec<T, V> r;
    const S v = M2_CONV_NT ? __builtin_nontemporal_load(reinterpret_cast<const S*>(p)) : *reinterpret_cast<const S*>(p);
    *reinterpret_cast<S*>(&r) = v;
    return r;
}
template <typename T, int V>
__device__ __forceinline__ void st_stream(T* __restrict__ p, const float (&in)[V]) {
    using S = typename StreamVec<V * (int)sizeof(T)>::type;
    S raw;
    T* e = reinterpret_cast<T*>(&raw);
#pragma unroll
    for (int i = 0; i < V; ++i) e[i] = from_f32<T>(in[i]);
    if (M2_CONV_NT) __builtin_nontemporal_store(raw, reinterpret_cast<S*>(p)); else *reinterpret_cast<S*>(p) = raw;
}

__device__ __forceinline__ float ld_param(const void* p, int pd, int64_t i) {
    return pd == M2_F32 ? reinterpret_cast<const float*>(p)[i] : to_f32(reinterpret_cast<const bf16_t*>(p)[i]);
}
__device__ __forceinline__ void st_param(void* p, int pd, int64_t i, float v) {
    if (pd == M2_F32) reinterpret_cast<float*>(p)[i] = v;
    else reinterpret_cast<bf16_t*>(p)[i] = from_f32<bf16_t>(v);
}

// The 4 taps and the bias of V consecutive channels with 16-byte loads, all in flight together (w is (C, 4) contiguous).
template <typename WT, int V>
__device__ __forceinline__ void load_taps(const void* __restrict__ w, const void* __restrict__ bias, int64_t c0,
                                          float (&wv)[4][V], float (&bv)[V]) {
    constexpr int TV = (V * 4 * (int)sizeof(WT)) < 16 ? V * 4 : 16 / (int)sizeof(WT);     // elements per tap load (<= 16 bytes)
    constexpr int PER = 16 / (int)sizeof(WT);
    static_assert((V * 4) % TV == 0, "taps of one thread must fill whole vectors");
    const WT* wp = static_cast<const WT*>(w) + c0 * 4;
    float flat[V * 4];
#pragma unroll
    for (int i = 0; i < V * 4 / TV; ++i) {
        float tmp[TV];
        loadv<WT, TV>(wp + i * TV, tmp);
#pragma unroll
        for (int e = 0; e < TV; ++e) flat[i * TV + e] = tmp[e];
    }
#pragma unroll
    for (int j = 0; j < V; ++j) {
#pragma unroll
        for (int i = 0; i < 4; ++i) wv[i][j] = flat[j * 4 + i];
        bv[j] = 0.f;
    }
    if (bias) {
        constexpr int BV = V < PER ? V : PER;      // at most 16 bytes per load
#pragma unroll
        for (int i = 0; i < V / BV; ++i) {
            float tmp[BV];
            loadv<WT, BV>(static_cast<const WT*>(bias) + c0 + i * BV, tmp);
#pragma unroll
            for (int e = 0; e < BV; ++e) bv[i * BV + e] = tmp[e];
        }
    }
}

// ------------------------------------------------------------------------------------------
// Fast path, channels-last, k == 4.
// grid: x = ceil(CV / kCVT), y = ceil(nseg / kSEG), z = batch; block (kCVT, kSEG).
template <typename T, typename WT, int V, int ACT>
__global__ void __launch_bounds__(kCVT * kSEG)
conv_fwd_cl_kernel(const T* __restrict__ x, const void* __restrict__ w, const void* __restrict__ bias,
                   T* __restrict__ y, int64_t l, int64_t C, int64_t xsb, int64_t xsl, int64_t ysb, int64_t ysl) {
    const int64_t cv = (int64_t)blockIdx.x * kCVT + threadIdx.x;
    const int64_t seg = (int64_t)blockIdx.y * kSEG + threadIdx.y;
    const int64_t b = blockIdx.z;
    const int64_t c0 = cv * V;
    const int64_t t0 = seg * kTLF;
    if (c0 >= C || t0 >= l) return;

    float wv[4][V], bv[V];
    load_taps<WT, V>(w, bias, c0, wv, bv);
    const T* xp = x + b * xsb + c0;
    T* yp = y + b * ysb + c0;
    float h0[V], h1[V], h2[V];   // x[t-3], x[t-2], x[t-1]
#pragma unroll
    for (int j = 0; j < V; ++j) h0[j] = h1[j] = h2[j] = 0.f;
    if (t0 - 3 >= 0) loadv<T, V>(xp + (t0 - 3) * xsl, h0);
    if (t0 - 2 >= 0) loadv<T, V>(xp + (t0 - 2) * xsl, h1);
    if (t0 - 1 >= 0) loadv<T, V>(xp + (t0 - 1) * xsl, h2);
    auto step = [&](const RawVec<T, V>& r, T* __restrict__ yq) {
        float out[V], cur[V];
        cvtv<T, V>(r, cur);
#pragma unroll
        for (int j = 0; j < V; ++j) {
            float z = bv[j] + wv[0][j] * h0[j] + wv[1][j] * h1[j] + wv[2][j] * h2[j] + wv[3][j] * cur[j];
            out[j] = act_f<ACT>(z);
            h0[j] = h1[j]; h1[j] = h2[j]; h2[j] = cur[j];
        }
        st_stream<T, V>(yq, out);
    };
    // software pipeline: the loads of group g+1 are issued before group g is computed and stored
    RawVec<T, V> nxt[kUNR];
    if (t0 + kTLF <= l) {
        // whole segment inside the sequence: no per-token predicates, so the wait before a group's compute can leave
        // the previous group's stores in flight
        const T* xq = xp + t0 * xsl;
        T* yq = yp + t0 * ysl;
#pragma unroll
        for (int u = 0; u < kUNR; ++u) nxt[u] = ld_stream<T, V>(xq + u * xsl);
        for (int g = 0; g < kTLF / kUNR - 1; ++g) {
            RawVec<T, V> raw[kUNR];
            xq += kUNR * xsl;
#pragma unroll
            for (int u = 0; u < kUNR; ++u) { raw[u] = nxt[u]; nxt[u] = ld_stream<T, V>(xq + u * xsl); }
#pragma unroll
            for (int u = 0; u < kUNR; ++u) step(raw[u], yq + u * ysl);
            yq += kUNR * ysl;
        }
#pragma unroll
        for (int u = 0; u < kUNR; ++u) step(nxt[u], yq + u * ysl);
        return;
    }
    const int64_t t1 = l;
#pragma unroll
    for (int u = 0; u < kUNR; ++u)
        if (t0 + u < t1) nxt[u] = ld_stream<T, V>(xp + (t0 + u) * xsl);
    for (int64_t tg = t0; tg < t1; tg += kUNR) {
        RawVec<T, V> raw[kUNR];
#pragma unroll
        for (int u = 0; u < kUNR; ++u) raw[u] = nxt[u];
#pragma unroll
        for (int u = 0; u < kUNR; ++u)
            if (tg + kUNR + u < t1) nxt[u] = ld_stream<T, V>(xp + (tg + kUNR + u) * xsl);
#pragma unroll
        for (int u = 0; u < kUNR; ++u)
            if (tg + u < t1) step(raw[u], yp + (tg + u) * ysl);
    }
}

// Backward fast path.  Each thread marches t over [t0, t0+TL+3): at step t it forms g[t] and
// emits dx[t-3] = w3 g[t-3] + w2 g[t-2] + w1 g[t-1] + w0 g[t]  (dx[s] = sum_i w[i] g[s+3-i]).
// Partials: part[(blockIdx.z * gridDim.y + blockIdx.y)][c][0..4] = (dw0..dw3, db).
template <typename T, typename WT, int V, int ACT>
__global__ void __launch_bounds__(kCVT * kSEG)
conv_bwd_cl_kernel(const T* __restrict__ x, const void* __restrict__ w, const void* __restrict__ bias,
                   const T* __restrict__ dy, T* __restrict__ dx, float* __restrict__ part,
                   int64_t l, int64_t C, int64_t xsb, int64_t xsl, int64_t gsb, int64_t gsl,
                   int64_t dsb, int64_t dsl) {
    __shared__ float red[kSEG][5][kCVT * V + 1];
    const int64_t cv = (int64_t)blockIdx.x * kCVT + threadIdx.x;
    const int64_t seg = (int64_t)blockIdx.y * kSEG + threadIdx.y;
    const int64_t b = blockIdx.z;
    const int64_t c0 = cv * V;
    const int64_t t0 = seg * kTLB;
    const bool active = (c0 < C) && (t0 < l);

    float acc[5][V];
#pragma unroll
    for (int i = 0; i < 5; ++i)
#pragma unroll
        for (int j = 0; j < V; ++j) acc[i][j] = 0.f;

    if (active) {
        float wv[4][V], bv[V];
        load_taps<WT, V>(w, bias, c0, wv, bv);
        const T* xp = x + b * xsb + c0;
        const T* gp = dy + b * gsb + c0;
        T* dp = dx + b * dsb + c0;
        float h0[V], h1[V], h2[V];   // x[t-3..t-1]
        float g0[V], g1[V], g2[V];   // g[t-3..t-1]
#pragma unroll
        for (int j = 0; j < V; ++j) h0[j] = h1[j] = h2[j] = g0[j] = g1[j] = g2[j] = 0.f;
        if (t0 - 3 >= 0) loadv<T, V>(xp + (t0 - 3) * xsl, h0);
        if (t0 - 2 >= 0) loadv<T, V>(xp + (t0 - 2) * xsl, h1);
        if (t0 - 1 >= 0) loadv<T, V>(xp + (t0 - 1) * xsl, h2);
        // one token: g[t] from x[t-3..t] and dy[t]; the weight/bias sums if the token is this thread's own; dx[t-3] to dq if emit
        auto step = [&](const RawVec<T, V>& rx, const RawVec<T, V>& rg, bool own, bool emit, T* __restrict__ dq) {
            float g[V], cur[V], gy[V];
            cvtv<T, V>(rx, cur);
            cvtv<T, V>(rg, gy);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                float z = bv[j] + wv[0][j] * h0[j] + wv[1][j] * h1[j] + wv[2][j] * h2[j] + wv[3][j] * cur[j];
                g[j] = gy[j] * act_grad_f<ACT>(z);     // gy == 0 beyond the sequence end
                if (own) {
                    acc[0][j] += h0[j] * g[j];
                    acc[1][j] += h1[j] * g[j];
                    acc[2][j] += h2[j] * g[j];
                    acc[3][j] += cur[j] * g[j];
                    acc[4][j] += g[j];
                }
            }
            if (emit) {
                float o[V];
#pragma unroll
                for (int j = 0; j < V; ++j)
                    o[j] = wv[3][j] * g0[j] + wv[2][j] * g1[j] + wv[1][j] * g2[j] + wv[0][j] * g[j];
                st_stream<T, V>(dq, o);
            }
#pragma unroll
            for (int j = 0; j < V; ++j) {
                h0[j] = h1[j]; h1[j] = h2[j]; h2[j] = cur[j];
                g0[j] = g1[j]; g1[j] = g2[j]; g2[j] = g[j];
            }
        };
        // software pipeline: the loads of group g+1 are issued before group g is computed and stored
        RawVec<T, V> nx[kUNR], ng[kUNR];
        if (t0 + kTLB + kUNR <= l) {
            // the segment and its 3 lag tokens lie inside the sequence: no per-token predicates
            const T* xq = xp + t0 * xsl;
            const T* gq = gp + t0 * gsl;
            T* dq = dp + (t0 - 3) * dsl;
#pragma unroll
            for (int u = 0; u < kUNR; ++u) { nx[u] = ld_stream<T, V>(xq + u * xsl); ng[u] = ld_stream<T, V>(gq + u * gsl); }
            for (int grp = 0; grp < kTLB / kUNR; ++grp) {
                RawVec<T, V> rawx[kUNR], rawg[kUNR];
                xq += kUNR * xsl;
                gq += kUNR * gsl;
#pragma unroll
                for (int u = 0; u < kUNR; ++u) {
                    rawx[u] = nx[u]; rawg[u] = ng[u];
                    nx[u] = ld_stream<T, V>(xq + u * xsl); ng[u] = ld_stream<T, V>(gq + u * gsl);
                }
#pragma unroll
                for (int u = 0; u < kUNR; ++u) step(rawx[u], rawg[u], true, grp > 0 || u >= 3, dq + u * dsl);
                dq += kUNR * dsl;
            }
#pragma unroll
            for (int u = 0; u < 3; ++u) step(nx[u], ng[u], false, true, dq + u * dsl);
        } else {
            const int64_t tseg = (t0 + kTLB < l) ? t0 + kTLB : l;      // end of this thread's own tokens
            const int64_t tend = tseg + 3;                            // march 3 further for the dx lag
#pragma unroll
            for (int u = 0; u < kUNR; ++u) {
                const int64_t t = t0 + u;
                if (t < tend && t < l) { nx[u] = ld_stream<T, V>(xp + t * xsl); ng[u] = ld_stream<T, V>(gp + t * gsl); }
                else { nx[u] = RawVec<T, V>{}; ng[u] = RawVec<T, V>{}; }
            }
            for (int64_t tg = t0; tg < tend; tg += kUNR) {
                RawVec<T, V> rawx[kUNR], rawg[kUNR];
#pragma unroll
                for (int u = 0; u < kUNR; ++u) { rawx[u] = nx[u]; rawg[u] = ng[u]; }
#pragma unroll
                for (int u = 0; u < kUNR; ++u) {
                    const int64_t t = tg + kUNR + u;
                    if (t < tend && t < l) { nx[u] = ld_stream<T, V>(xp + t * xsl); ng[u] = ld_stream<T, V>(gp + t * gsl); }
                    else { nx[u] = RawVec<T, V>{}; ng[u] = RawVec<T, V>{}; }
                }
#pragma unroll
                for (int u = 0; u < kUNR; ++u) {
                    const int64_t t = tg + u;
                    if (t < tend) step(rawx[u], rawg[u], t < tseg, t - 3 >= t0, dp + (t - 3) * dsl);
                }
            }
        }
    }
    // block reduction over the kSEG token segments
#pragma unroll
    for (int i = 0; i < 5; ++i)
#pragma unroll
        for (int j = 0; j < V; ++j) red[threadIdx.y][i][threadIdx.x * V + j] = acc[i][j];
    __syncthreads();
    const int tid = threadIdx.y * kCVT + threadIdx.x;
    const int64_t pslot = (int64_t)blockIdx.z * gridDim.y + blockIdx.y;
    for (int e = tid; e < 5 * kCVT * V; e += kCVT * kSEG) {
        const int i = e / (kCVT * V), cc = e % (kCVT * V);
        const int64_t c = (int64_t)blockIdx.x * kCVT * V + cc;
        if (c < C) {
            float s = 0.f;
#pragma unroll
            for (int r = 0; r < kSEG; ++r) s += red[r][i][cc];
            part[(pslot * C + c) * 5 + i] = s;
        }
    }
}

// Zero fill (a kernel rather than a memset node, so that a caller may capture the call in a graph).
__global__ void conv_zero_kernel(uint16_t* __restrict__ p, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

// Second stage: sum the per-block partials.  Four adjacent lanes per (channel, tap-or-bias), each a quarter of the
// slots (fixed order), combined by two shuffles.
__global__ void __launch_bounds__(256)
conv_reduce_partials_kernel(const float* __restrict__ part, int64_t nslots, int64_t C, int k,
                            void* __restrict__ dw, void* __restrict__ db, int pd) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t e = t >> 2;
    const int q = (int)(t & 3);
    const int kk = k + 1;
    const bool live = e < C * kk;
    const int64_t c = live ? e / kk : 0;
    const int i = live ? (int)(e % kk) : 0;
    float s = 0.f;
    if (live) {
#pragma unroll 4
        for (int64_t r = q; r < nslots; r += 4) s += part[(r * C + c) * kk + i];
    }
    s = lane_xor_add<1>(s);
    s = lane_xor_add<2>(s);
    if (!live || q != 0) return;
    if (i < k) st_param(dw, pd, c * k + i, s);
    else if (db) st_param(db, pd, c, s);
}

// ------------------------------------------------------------------------------------------
// Generic path: any strides / layout, k <= 8, one thread per output element.
template <typename T>
__global__ void conv_fwd_generic_kernel(const T* __restrict__ x, const void* __restrict__ w, const void* __restrict__ bias,
                                        T* __restrict__ y, int64_t nb, int64_t l, int64_t C, int k,
                                        int64_t xsb, int64_t xsl, int64_t xsc, int64_t ysb, int64_t ysl, int64_t ysc,
                                        int pd, int act, int t_fastest) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= nb * l * C) return;
    int64_t b, t, c;
    if (t_fastest) { t = idx % l; c = (idx / l) % C; b = idx / (l * C); }
    else { c = idx % C; t = (idx / C) % l; b = idx / (l * C); }
    float z = bias ? ld_param(bias, pd, c) : 0.f;
    for (int i = 0; i < k; ++i) {
        const int64_t tt = t - (k - 1) + i;
        if (tt >= 0) z += ld_param(w, pd, c * k + i) * to_f32(x[b * xsb + tt * xsl + c * xsc]);
    }
    const float o = act == M2_ACT_SILU ? silu_f(z) : (act == M2_ACT_RELU ? (z > 0.f ? z : 0.f) : z);
    y[b * ysb + t * ysl + c * ysc] = from_f32<T>(o);
}

template <typename T>
__device__ __forceinline__ float conv_g_at(const T* __restrict__ x, const void* __restrict__ w, const void* __restrict__ bias,
                                           const T* __restrict__ dy, int64_t b, int64_t t, int64_t c, int k,
                                           int64_t xsb, int64_t xsl, int64_t xsc, int64_t gsb, int64_t gsl, int64_t gsc,
                                           int pd, int act) {
    float z = bias ? ld_param(bias, pd, c) : 0.f;
    for (int i = 0; i < k; ++i) {
        const int64_t tt = t - (k - 1) + i;
        if (tt >= 0) z += ld_param(w, pd, c * k + i) * to_f32(x[b * xsb + tt * xsl + c * xsc]);
    }
    const float d = act == M2_ACT_SILU ? silu_grad_f(z) : (act == M2_ACT_RELU ? (z > 0.f ? 1.f : 0.f) : 1.f);
    return to_f32(dy[b * gsb + t * gsl + c * gsc]) * d;
}

template <typename T>
__global__ void conv_bwd_dx_generic_kernel(const T* __restrict__ x, const void* __restrict__ w, const void* __restrict__ bias,
                                           const T* __restrict__ dy, T* __restrict__ dx, int64_t nb, int64_t l, int64_t C, int k,
                                           int64_t xsb, int64_t xsl, int64_t xsc, int64_t gsb, int64_t gsl, int64_t gsc,
                                           int64_t dsb, int64_t dsl, int64_t dsc, int pd, int act, int t_fastest) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= nb * l * C) return;
    int64_t b, t, c;
    if (t_fastest) { t = idx % l; c = (idx / l) % C; b = idx / (l * C); }
    else { c = idx % C; t = (idx / C) % l; b = idx / (l * C); }
    float s = 0.f;
    for (int i = 0; i < k; ++i) {
        const int64_t tt = t + (k - 1) - i;
        if (tt < l) s += ld_param(w, pd, c * k + i) * conv_g_at(x, w, bias, dy, b, tt, c, k, xsb, xsl, xsc, gsb, gsl, gsc, pd, act);
    }
    dx[b * dsb + t * dsl + c * dsc] = from_f32<T>(s);
}

// one block per channel; threads stride over (b, t)
template <typename T>
__global__ void __launch_bounds__(256)
conv_bwd_dw_generic_kernel(const T* __restrict__ x, const void* __restrict__ w, const void* __restrict__ bias,
                           const T* __restrict__ dy, void* __restrict__ dw, void* __restrict__ db,
                           int64_t nb, int64_t l, int k, int64_t xsb, int64_t xsl, int64_t xsc,
                           int64_t gsb, int64_t gsl, int64_t gsc, int pd, int act) {
    __shared__ float red[4][kMaxK + 1];
    const int64_t c = blockIdx.x;
    float acc[kMaxK + 1];
#pragma unroll
    for (int i = 0; i <= kMaxK; ++i) acc[i] = 0.f;
    for (int64_t e = threadIdx.x; e < nb * l; e += blockDim.x) {
        const int64_t b = e / l, t = e % l;
        const float g = conv_g_at(x, w, bias, dy, b, t, c, k, xsb, xsl, xsc, gsb, gsl, gsc, pd, act);
#pragma unroll
        for (int i = 0; i < kMaxK; ++i) {
            if (i < k) {
                const int64_t tt = t - (k - 1) + i;
                if (tt >= 0) acc[i] += to_f32(x[b * xsb + tt * xsl + c * xsc]) * g;
            }
        }
        acc[kMaxK] += g;
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int i = 0; i <= kMaxK; ++i) {
        const float s = warp_sum(acc[i]);
        if (lane == 0) red[wave][i] = s;
    }
    __syncthreads();
    if (threadIdx.x <= kMaxK) {
        const int i = threadIdx.x;
        const float s = red[0][i] + red[1][i] + red[2][i] + red[3][i];
        if (i < k) st_param(dw, pd, c * k + i, s);
        else if (i == kMaxK && db) st_param(db, pd, c, s);
    }
}

// elements per thread: 16-byte vectors forward, 8-byte vectors backward (the backward carries twice the
// per-channel state in registers; halving the vector keeps its occupancy up)
template <typename T> constexpr int conv_vec(bool bwd) {
    const int v = (int)((bwd ? M2_CONV_VB : M2_CONV_VF) / sizeof(T));
    return v < 2 ? 2 : v;
}

template <typename T, int V>
bool fast_path_ok(const m2_conv1d_params* p, bool bwd) {
    if (p->k != 4 || p->x_stride_c != 1 || p->y_stride_c != 1) return false;
    if (p->channels % V) return false;
    if (p->x_stride_b % V || p->x_stride_l % V || p->y_stride_b % V || p->y_stride_l % V) return false;
    auto al = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) % (V * sizeof(T))) == 0; };
    if (!al(p->x)) return false;
    if (reinterpret_cast<uintptr_t>(p->w) % 16 || reinterpret_cast<uintptr_t>(p->bias) % 16) return false;   // vector tap loads
    if (!bwd && !al(p->y)) return false;
    if (bwd) {
        if (p->dx_stride_c != 1 || p->dx_stride_b % V || p->dx_stride_l % V) return false;
        if (!al(p->dy) || !al(p->dx)) return false;
    }
    return true;
}

int check_common(const m2_conv1d_params* p) {
    M2_REQUIRE(p, M2_ERR_NULL, "conv1d: params is NULL");
    M2_REQUIRE(p->batch >= 0 && p->seqlen >= 0 && p->channels >= 0, M2_ERR_SHAPE, "conv1d: negative dimension");
    M2_REQUIRE(p->k >= 1 && p->k <= kMaxK, M2_ERR_SHAPE, "conv1d: kernel size %d not in [1, %d]", p->k, kMaxK);
    M2_REQUIRE(p->dtype == M2_F32 || p->dtype == M2_BF16, M2_ERR_DTYPE, "conv1d: bad dtype %d", p->dtype);
    M2_REQUIRE(p->param_dtype == M2_F32 || p->param_dtype == M2_BF16, M2_ERR_DTYPE, "conv1d: bad param dtype %d", p->param_dtype);
    M2_REQUIRE(p->activation >= M2_ACT_NONE && p->activation <= M2_ACT_RELU, M2_ERR_SHAPE, "conv1d: bad activation %d", p->activation);
    M2_REQUIRE(p->batch <= 65535, M2_ERR_SHAPE, "conv1d: batch %lld > 65535", (long long)p->batch);
    return M2_OK;
}

template <typename T>
int launch_fwd(const m2_conv1d_params* p, hipStream_t st) {
    const int64_t nb = p->batch, l = p->seqlen, C = p->channels;
    const T* x = static_cast<const T*>(p->x);
    T* y = static_cast<T*>(p->y);
    constexpr int V = conv_vec<T>(false);
    if (fast_path_ok<T, V>(p, false) && p->activation != M2_ACT_RELU) {
        const int64_t CV = C / V, nseg = ceil_div(l, kTLF);
        dim3 grid((unsigned)ceil_div(CV, kCVT), (unsigned)ceil_div(nseg, kSEG), (unsigned)nb), block(kCVT, kSEG);
        M2_REQUIRE(grid.y <= 65535, M2_ERR_SHAPE, "conv1d: sequence too long for the grid");
        auto go = [&](auto kern) {
            kern<<<grid, block, 0, st>>>(x, p->w, p->bias, y, l, C, p->x_stride_b, p->x_stride_l, p->y_stride_b, p->y_stride_l);
        };
        const bool silu = p->activation == M2_ACT_SILU;
        if (p->param_dtype == M2_F32) {
            if (silu) go(conv_fwd_cl_kernel<T, float, V, M2_ACT_SILU>); else go(conv_fwd_cl_kernel<T, float, V, M2_ACT_NONE>);
        } else {
            if (silu) go(conv_fwd_cl_kernel<T, bf16_t, V, M2_ACT_SILU>); else go(conv_fwd_cl_kernel<T, bf16_t, V, M2_ACT_NONE>);
        }
    } else {
        const int64_t total = nb * l * C;
        const int tf = (p->x_stride_l == 1 && p->x_stride_c != 1) ? 1 : 0;
        conv_fwd_generic_kernel<T><<<(unsigned)ceil_div(total, 256), 256, 0, st>>>(
            x, p->w, p->bias, y, nb, l, C, p->k, p->x_stride_b, p->x_stride_l, p->x_stride_c,
            p->y_stride_b, p->y_stride_l, p->y_stride_c, p->param_dtype, p->activation, tf);
    }
    return check_launch("conv1d_fwd");
}

template <typename T>
int launch_bwd(const m2_conv1d_params* p, hipStream_t st) {
    const int64_t nb = p->batch, l = p->seqlen, C = p->channels;
    const T* x = static_cast<const T*>(p->x);
    const T* dy = static_cast<const T*>(p->dy);
    T* dx = static_cast<T*>(p->dx);
    constexpr int V = conv_vec<T>(true);
    if (fast_path_ok<T, V>(p, true) && p->activation != M2_ACT_RELU) {
        const int64_t CV = C / V, nseg = ceil_div(l, kTLB);
        dim3 grid((unsigned)ceil_div(CV, kCVT), (unsigned)ceil_div(nseg, kSEG), (unsigned)nb), block(kCVT, kSEG);
        M2_REQUIRE(grid.y <= 65535, M2_ERR_SHAPE, "conv1d: sequence too long for the grid");
        const int64_t nslots = (int64_t)grid.y * grid.z;
        const size_t need = (size_t)nslots * C * 5 * sizeof(float);
        M2_REQUIRE(p->workspace && p->workspace_bytes >= need, M2_ERR_WORKSPACE,
                   "conv1d_bwd: workspace %zu bytes < %zu needed", p->workspace_bytes, need);
        float* part = static_cast<float*>(p->workspace);
        auto go = [&](auto kern) {
            kern<<<grid, block, 0, st>>>(x, p->w, p->bias, dy, dx, part, l, C, p->x_stride_b, p->x_stride_l, p->y_stride_b, p->y_stride_l,
                                         p->dx_stride_b, p->dx_stride_l);
        };
        const bool silu = p->activation == M2_ACT_SILU;
        if (p->param_dtype == M2_F32) {
            if (silu) go(conv_bwd_cl_kernel<T, float, V, M2_ACT_SILU>); else go(conv_bwd_cl_kernel<T, float, V, M2_ACT_NONE>);
        } else {
            if (silu) go(conv_bwd_cl_kernel<T, bf16_t, V, M2_ACT_SILU>); else go(conv_bwd_cl_kernel<T, bf16_t, V, M2_ACT_NONE>);
        }
        int rc = check_launch("conv1d_bwd");
        if (rc) return rc;
        conv_reduce_partials_kernel<<<(unsigned)ceil_div(C * 5 * 4, (int64_t)256), 256, 0, st>>>(part, nslots, C, 4, p->dw, p->db, p->param_dtype);
        return check_launch("conv1d_bwd_reduce");
    }
    const int64_t total = nb * l * C;
    const int tf = (p->x_stride_l == 1 && p->x_stride_c != 1) ? 1 : 0;
    conv_bwd_dx_generic_kernel<T><<<(unsigned)ceil_div(total, 256), 256, 0, st>>>(
        x, p->w, p->bias, dy, dx, nb, l, C, p->k, p->x_stride_b, p->x_stride_l, p->x_stride_c,
        p->y_stride_b, p->y_stride_l, p->y_stride_c, p->dx_stride_b, p->dx_stride_l, p->dx_stride_c,
        p->param_dtype, p->activation, tf);
    int rc = check_launch("conv1d_bwd_dx");
    if (rc) return rc;
    conv_bwd_dw_generic_kernel<T><<<(unsigned)C, 256, 0, st>>>(x, p->w, p->bias, dy, p->dw, p->db, nb, l, p->k,
                                                                p->x_stride_b, p->x_stride_l, p->x_stride_c,
                                                                p->y_stride_b, p->y_stride_l, p->y_stride_c, p->param_dtype, p->activation);
    return check_launch("conv1d_bwd_dw");
}

}  // namespace
}  // namespace m2

extern "C" int m2_conv1d_fwd(const m2_conv1d_params* p, void* stream) {
    using namespace m2;
    int rc = check_common(p);
    if (rc) return rc;
    if (p->batch == 0 || p->seqlen == 0 || p->channels == 0) return M2_OK;
    M2_REQUIRE(p->x && p->w && p->y, M2_ERR_NULL, "conv1d_fwd: x, w and y are required");
    M2_DISPATCH_DTYPE(p->dtype, T, return launch_fwd<T>(p, static_cast<hipStream_t>(stream)));
    return M2_OK;
}

extern "C" size_t m2_conv1d_bwd_workspace_bytes(int64_t batch, int64_t seqlen, int64_t channels, int32_t k) {
    using namespace m2;
    (void)k;
    const int64_t nseg = ceil_div(seqlen, kTLB);
    return (size_t)(ceil_div(nseg, kSEG) * batch * channels * 5) * sizeof(float) + 16;
}

extern "C" int m2_conv1d_bwd(const m2_conv1d_params* p, void* stream) {
    using namespace m2;
    int rc = check_common(p);
    if (rc) return rc;
    M2_REQUIRE(p->dw, M2_ERR_NULL, "conv1d_bwd: dw is required");
    if (p->channels == 0) return M2_OK;
    if (p->batch == 0 || p->seqlen == 0) {
        // empty reduction: gradients of the parameters are zero
        hipStream_t st = static_cast<hipStream_t>(stream);
        const size_t esz = p->param_dtype == M2_F32 ? 4 : 2;
        const int64_t nw = p->channels * p->k * (int64_t)(esz / 2), nb = p->channels * (int64_t)(esz / 2);     // 16-bit words
        conv_zero_kernel<<<(unsigned)ceil_div(nw, (int64_t)256), 256, 0, st>>>(static_cast<uint16_t*>(p->dw), nw);
        if (p->db) conv_zero_kernel<<<(unsigned)ceil_div(nb, (int64_t)256), 256, 0, st>>>(static_cast<uint16_t*>(p->db), nb);
        return check_launch("conv1d_bwd_zero");
    }
    M2_REQUIRE(p->x && p->w && p->dy && p->dx, M2_ERR_NULL, "conv1d_bwd: x, w, dy, dx are required");
    M2_DISPATCH_DTYPE(p->dtype, T, return launch_bwd<T>(p, static_cast<hipStream_t>(stream)));
    return M2_OK;
}
