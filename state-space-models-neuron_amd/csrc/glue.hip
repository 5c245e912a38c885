// Elementwise glue of the mixer core as HBM-bound kernels: softplus(dt + dt_bias) and the gated, grouped RMSNorm,
// forward and backward (mamba2/fused_kernel.py:33-73 softplus_with_bias(_bwd), :76-175 rmsnorm(_bwd); torch twins
// mamba2/mamba2_mixer.py:36-38, 88-105).  Every tensor is read once and written once; all arithmetic is fp32.
//
//   softplus:  out = v < 10 ? log(1 + e^v) : v,  v = dt + bias[h]              (threshold form, mamba2_mixer.py:36-38)
//              d_in = d_out * (v < 10 ? sigmoid(v) : 1),   d_bias[h] = sum over rows of d_in
//   rmsnorm:   h = x * silu(z);   out = w * h * rsqrt(mean_group(h^2) + eps)    per group of d / n_groups channels
//              backward (fused_kernel.py:159-171):  var = mean(h^2) + eps, r = rsqrt(var), gw = g w,
//              cf = mean(h gw) / var,  d_h = r (gw - cf h),  dx = d_h silu(z),  dz = d_h x silu'(z),  dw = sum_rows g h r
//
// A (row, group) is handled by one wave (groups of up to 2048 channels) or by the four waves of a workgroup (up to
// 8192), its channels in registers as 16-byte vectors; a workgroup walks a block of rows, so the per-channel weight
// and -- in the backward -- the dw accumulators stay in registers across rows.  dw and d_bias leave as per-block
// partials in a caller-owned workspace and are summed in a fixed order by a second small kernel (no atomics).
#include "common.hpp"

namespace m2 {
namespace {

// ------------------------------------------------------------------------------------------ softplus
template <typename T>
__global__ void __launch_bounds__(256)
softplus_fwd_kernel(const T* __restrict__ dt, int64_t dt_sr, const float* __restrict__ bias, T* __restrict__ out, int64_t out_sr,
                    int64_t rows, int64_t nheads) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows * nheads) return;
    const int64_t row = idx / nheads, h = idx % nheads;
    const float v = to_f32(dt[row * dt_sr + h]) + bias[h];
    out[row * out_sr + h] = from_f32<T>(softplus_f(v));
}

constexpr int kSpRows = 16;      // rows per workgroup of the softplus backward
// 256 threads = 4 row phases x 64 heads; a workgroup walks kSpRows rows and leaves one partial row of d_bias
template <typename T>
__global__ void __launch_bounds__(256)
softplus_bwd_kernel(const T* __restrict__ dt, int64_t dt_sr, const float* __restrict__ bias, const T* __restrict__ d_out, int64_t do_sr,
                    T* __restrict__ d_in, int64_t di_sr, float* __restrict__ partial, int64_t rows, int64_t nheads) {
    __shared__ float red[4][64];
    const int hl = threadIdx.x & 63, ph = threadIdx.x >> 6;
    const int64_t r0 = (int64_t)blockIdx.x * kSpRows;
    const int64_t r1 = r0 + kSpRows < rows ? r0 + kSpRows : rows;
    for (int64_t h0 = 0; h0 < nheads; h0 += 64) {
        const int64_t h = h0 + hl;
        float acc = 0.f;
        if (h < nheads) {
            const float bh = bias[h];
#pragma unroll 4
            for (int64_t r = r0 + ph; r < r1; r += 4) {
                const float v = to_f32(dt[r * dt_sr + h]) + bh;
                const float g = to_f32(d_out[r * do_sr + h]) * (v < kSoftplusThreshold ? sigmoid_f(v) : 1.f);
                d_in[r * di_sr + h] = from_f32<T>(g);
                acc += g;
            }
        }
        red[ph][hl] = acc;
        __syncthreads();
        if (ph == 0 && h < nheads) partial[(int64_t)blockIdx.x * nheads + h] = (red[0][hl] + red[1][hl]) + (red[2][hl] + red[3][hl]);
        __syncthreads();
    }
}

// out[c] = sum over the partial rows of partial[row][c] in a fixed order: 16 row phases per channel (1024 threads), 64
// channels per workgroup, the phases added pairwise.
__global__ void __launch_bounds__(1024)
column_sum_kernel(const float* __restrict__ partial, float* __restrict__ out, int64_t nrows, int64_t ncols) {
    __shared__ float red[16][64];
    const int c = threadIdx.x & 63, ph = threadIdx.x >> 6;
    const int64_t col = (int64_t)blockIdx.x * 64 + c;
    float s = 0.f;
    if (col < ncols) {
#pragma unroll 4
        for (int64_t r = ph; r < nrows; r += 16) s += partial[r * ncols + col];
    }
    red[ph][c] = s;
    __syncthreads();
    if (ph == 0 && col < ncols) {
        float t[16];
#pragma unroll
        for (int q = 0; q < 16; ++q) t[q] = red[q][c];
#pragma unroll
        for (int w = 8; w >= 1; w >>= 1)
#pragma unroll
            for (int q = 0; q < w; ++q) t[q] += t[q + w];
        out[col] = t[0];
    }
}

// ------------------------------------------------------------------------------------------ gated RMSNorm
struct NormArgs {
    const void* x; int64_t x_sr;            // [rows][d], channels contiguous
    const void* z; int64_t z_sr;            // gate, or null
    const float* w;                         // [d]
    void* out; int64_t out_sr; int out_f32; // forward output
    const void* g; int64_t g_sr;            // backward: d_out
    void* dx; int64_t dx_sr;
    void* dz; int64_t dz_sr;
    float* partial;                         // backward: [partial rows][d]
    int64_t rows, d, gw, rows_per_block;    // gw = channels per group
    float eps;
};

template <typename T> struct GlueVec;
template <> struct GlueVec<bf16_t> { static constexpr int V = 8; };
template <> struct GlueVec<float> { static constexpr int V = 4; };

template <typename T>
__device__ __forceinline__ void unpack_vec(const uint4 raw, float (&v)[GlueVec<T>::V]) {
    if constexpr (sizeof(T) == 2) {
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            v[2 * q] = __builtin_bit_cast(float, w[q] << 16);
            v[2 * q + 1] = __builtin_bit_cast(float, w[q] & 0xffff0000u);
        }
    } else {
        v[0] = __builtin_bit_cast(float, raw.x); v[1] = __builtin_bit_cast(float, raw.y);
        v[2] = __builtin_bit_cast(float, raw.z); v[3] = __builtin_bit_cast(float, raw.w);
    }
}
template <typename T>
__device__ __forceinline__ void store_vec(T* p, const float (&v)[GlueVec<T>::V]) {
    if constexpr (sizeof(T) == 2) {
        T e[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) e[q] = from_f32<T>(v[q]);
        *reinterpret_cast<uint4*>(p) = *reinterpret_cast<const uint4*>(e);
    } else {
        *reinterpret_cast<floatx4*>(p) = floatx4{v[0], v[1], v[2], v[3]};
    }
}

// sum over the WPG waves that share a (row, group); `slot` alternates between two LDS rows so that one barrier per
// reduction is enough
template <int WPG>
__device__ __forceinline__ void group_sum2(float& a, float& b, float (*red)[2][16], int slot) {
    a = warp_sum(a); b = warp_sum(b);
    if constexpr (WPG > 1) {
        const int wave = threadIdx.x >> 6;
        if ((threadIdx.x & 63) == 0) { red[slot][0][wave] = a; red[slot][1][wave] = b; }
        __syncthreads();
        a = red[slot][0][0]; b = red[slot][1][0];
#pragma unroll
        for (int q = 1; q < WPG; ++q) { a += red[slot][0][q]; b += red[slot][1][q]; }      // fixed order
    }
}

// grid (row blocks, groups).  WPG = waves per (row, group): 1 (256 threads, each wave its own rows) or 4 or 5 (the whole
// workgroup of WPG waves shares a row).  NV = vectors per lane.  GATED: z given.  EXACT: the group is exactly WPG x 64 x NV
// vectors wide, so no lane is idle and nothing is masked (5120 channels of a 16-bit type = 5 waves x 2 vectors).
template <typename T, int WPG, int NV, bool BWD, bool GATED, bool EXACT>
__global__ void __launch_bounds__(WPG == 1 ? 256 : WPG * 64)
rmsnorm_gated_kernel(const NormArgs a) {
    constexpr int V = GlueVec<T>::V;
    constexpr int TPG = WPG * 64;                 // threads per (row, group)
    __shared__ float red[2][2][16];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int tl = WPG > 1 ? tid : lane;          // index inside the (row, group)
    const int64_t grp = blockIdx.y;
    const int64_t c0 = grp * a.gw;                // first channel of the group
    const int nvec = (int)(a.gw / V);
    const float inv_n = 1.f / (float)a.gw;

    float w[NV][V], dw[BWD ? NV : 1][V];
#pragma unroll
    for (int it = 0; it < NV; ++it) {
        const int vi = it * TPG + tl;
#pragma unroll
        for (int e = 0; e < V; ++e) {
            w[it][e] = (EXACT || vi < nvec) ? a.w[c0 + (int64_t)vi * V + e] : 0.f;
            if (BWD) dw[it][e] = 0.f;
        }
    }
    // Rows are dealt out round-robin: workgroup i (WPG > 1; wave 4 i + w for WPG == 1) takes rows i, i + G, i + 2 G, ... with G
    // the number of workgroups (waves), so that at any moment the rows in flight over the whole chip are neighbours in
    // memory and every memory channel is in use.  (A contiguous block of rows per workgroup puts all workgroups a fixed
    // power-of-two-rich distance apart, and they then walk through the same channels together: 3.6 TB/s for the loads alone.)
    const int64_t r1 = a.rows;
    const int64_t RSTEP = WPG > 1 ? (int64_t)gridDim.x : (int64_t)gridDim.x * 4;
    int slot = 0;
    // WPG > 1: every wave takes every row of the workgroup (uniform trip count, barriers inside); WPG == 1: each wave its own rows.
    // the raw vectors of the next row are loaded before this row is reduced (the row after the last: the first once more)
    constexpr bool gated = GATED;
    // Two register sets, a row loaded a whole iteration before it is used: the forward always; the backward where the
    // workgroup is alone on its compute unit anyway (five waves: up to 256 registers each).  Otherwise the backward loads
    // the next row behind the first pass over the current one.
    constexpr bool TWO = !BWD || WPG == 5;
    struct RowRegs { uint4 x[NV], z[NV], g[BWD ? NV : 1]; };
    RowRegs ra, rb;
    const int64_t rfirst = WPG > 1 ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * 4 + wave;
    auto load_row = [&](int64_t r, RowRegs& q) {
        uint4 (&rx)[NV] = q.x; uint4 (&rz)[NV] = q.z; uint4 (&rg)[BWD ? NV : 1] = q.g;
        const int64_t rr = r < r1 ? r : rfirst;
        const T* xr = static_cast<const T*>(a.x) + rr * a.x_sr + c0;
        const T* zr = gated ? static_cast<const T*>(a.z) + rr * a.z_sr + c0 : xr;
        const T* gr = BWD ? static_cast<const T*>(a.g) + rr * a.g_sr + c0 : xr;
#pragma unroll
        for (int it = 0; it < NV; ++it) {
            const int vi = it * TPG + tl;
            const int64_t off = (int64_t)((EXACT || vi < nvec) ? vi : 0) * V;      // idle lanes read the first vector and ignore it
            rx[it] = *reinterpret_cast<const uint4*>(xr + off);
            if (gated) rz[it] = *reinterpret_cast<const uint4*>(zr + off);
            if (BWD) rg[it] = *reinterpret_cast<const uint4*>(gr + off);
        }
    };
    if (rfirst < r1) load_row(rfirst, ra);
    auto do_row = [&](int64_t r, RowRegs& q) {
        uint4 (&rx)[NV] = q.x; uint4 (&rz)[NV] = q.z; uint4 (&rg)[BWD ? NV : 1] = q.g;
        const bool zr = gated;
        float h[NV][V], xs[BWD ? NV : 1][V], zs[BWD ? NV : 1][V], gs[BWD ? NV : 1][V];
        float ss = 0.f, dot = 0.f;
#pragma unroll
        for (int it = 0; it < NV; ++it) {
            const int vi = it * TPG + tl;
            float xv[V], zv[V], gv[V];
            // an idle lane's x is zeroed as a raw vector (four selects): h, and with it every sum, is then zero there
            uint4 rxv = rx[it];
            if (!EXACT && vi >= nvec) rxv = uint4{0u, 0u, 0u, 0u};
            unpack_vec<T>(rxv, xv);
            if (gated) unpack_vec<T>(rz[it], zv);
            if (BWD) unpack_vec<T>(rg[it], gv);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const float gate = zr ? silu_f(zv[e]) : 1.f;
                h[it][e] = xv[e] * gate;
                ss += h[it][e] * h[it][e];
                if (BWD) {
                    xs[it][e] = xv[e]; zs[it][e] = zr ? zv[e] : 0.f; gs[it][e] = gv[e];
                    dot += h[it][e] * gv[e] * w[it][e];
                }
            }
        }
        if (!TWO) load_row(r + RSTEP, q);
        group_sum2<WPG>(ss, dot, red, slot);
        slot ^= 1;
        const float var = ss * inv_n + a.eps;
        const float rinv = __builtin_amdgcn_rsqf(var);
        if (!BWD) {
#pragma unroll
            for (int it = 0; it < NV; ++it) {
                const int vi = it * TPG + tl;
                if (!EXACT && vi >= nvec) continue;
                float o[V];
#pragma unroll
                for (int e = 0; e < V; ++e) o[e] = w[it][e] * (h[it][e] * rinv);
                if (a.out_f32) {
                    float* op = static_cast<float*>(a.out) + r * a.out_sr + c0 + (int64_t)vi * V;
#pragma unroll
                    for (int q = 0; q < V / 4; ++q) *reinterpret_cast<floatx4*>(op + 4 * q) = floatx4{o[4 * q], o[4 * q + 1], o[4 * q + 2], o[4 * q + 3]};
                } else {
                    store_vec<T>(static_cast<T*>(a.out) + r * a.out_sr + c0 + (int64_t)vi * V, o);
                }
            }
        } else {
            const float cf = dot * inv_n / var;
#pragma unroll
            for (int it = 0; it < NV; ++it) {
                const int vi = it * TPG + tl;
                if (!EXACT && vi >= nvec) continue;
                float ox[V], oz[V];
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    const float gwv = gs[it][e] * w[it][e];
                    const float dh = rinv * (gwv - cf * h[it][e]);
                    if (zr) {
                        const float z = zs[it][e];
                        const float s = sigmoid_f(z);
                        ox[e] = dh * (z * s);
                        oz[e] = dh * xs[it][e] * (s * (1.f + z * (1.f - s)));
                    } else {
                        ox[e] = dh; oz[e] = 0.f;
                    }
                    dw[it][e] += gs[it][e] * (h[it][e] * rinv);
                }
                store_vec<T>(static_cast<T*>(a.dx) + r * a.dx_sr + c0 + (int64_t)vi * V, ox);
                if (zr && a.dz) store_vec<T>(static_cast<T*>(a.dz) + r * a.dz_sr + c0 + (int64_t)vi * V, oz);
            }
        }
    };
    if constexpr (!TWO) {
        for (int64_t r = rfirst; r < r1; r += RSTEP) do_row(r, ra);
    } else {
        // rows in pairs, one per register set; a row's loads are issued before the row in front of it is processed
        for (int64_t r = rfirst; r < r1; r += 2 * RSTEP) {
            load_row(r + RSTEP, rb);
            do_row(r, ra);
            if (r + RSTEP < r1) {      // uniform over the workgroup when it shares its rows (WPG > 1)
                load_row(r + 2 * RSTEP, ra);
                do_row(r + RSTEP, rb);
            }
        }
    }
    if (BWD) {
        // one partial row per workgroup (WPG > 1: each lane owns its channels) or per wave (WPG == 1)
        const int64_t prow = WPG > 1 ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * 4 + wave;
        float* pp = a.partial + prow * a.d + c0;
#pragma unroll
        for (int it = 0; it < NV; ++it) {
            const int vi = it * TPG + tl;
            if (!EXACT && vi >= nvec) continue;
#pragma unroll
            for (int q = 0; q < V / 4; ++q)
                *reinterpret_cast<floatx4*>(pp + (int64_t)vi * V + 4 * q) = floatx4{dw[it][4 * q], dw[it][4 * q + 1], dw[it][4 * q + 2], dw[it][4 * q + 3]};
        }
    }
}

// rows per workgroup: about 512 workgroups in all for the backward (each leaves a partial row of dw), about 2048 for
// the forward, at least 4 rows each
int64_t norm_rows_per_block(int64_t rows, int64_t groups, bool bwd) {
    int64_t rb = rows * groups / (bwd ? 512 : 1024);
    if (rb < 4) rb = 4;
    return (rb + 3) / 4 * 4;
}
// The backward with a whole workgroup per (row, group): one workgroup per compute unit as well (it is alone there by its
// register count anyway; 256 workgroups 77 us, 512 -> 80, 768 -> 95 at 8192 rows of 5120 channels).
int64_t norm_rows_per_block_bwd(int64_t rows, int64_t groups, int64_t nvec) {
    if (nvec > 256 && rows * groups >= 4096) return ceil_div(rows * groups, device_cus());
    return norm_rows_per_block(rows, groups, true);
}
// The forward with a whole workgroup per (row, group): few rows (a decode step) are spread one per workgroup; many rows go
// to exactly ONE workgroup per compute unit (measured at 8192 rows of 5120 channels, rows dealt round-robin: 256 workgroups
// 46 us, 192 -> 55, 320 -> 57, 512 -> 52, 1024 -> 54: more resident waves only disturb the three streams).
int64_t norm_rows_per_block_fwd(int64_t rows, int64_t groups, int64_t nvec) {
    if (nvec > 256) {
        if (rows * groups < 4096) return 1;
        return ceil_div(rows * groups, device_cus());
    }
    return norm_rows_per_block(rows, groups, false);
}
// waves per (row, group) and vectors per lane for a group of `nvec` 16-byte vectors; false if it does not fit
bool norm_shape(int64_t nvec, int vec_elems, int* wpg, int* nv) {
    if (nvec <= 0) return false;
    if (nvec <= 256) { *wpg = 1; *nv = (int)((nvec + 63) / 64); return true; }
    // a group that five waves cover with no idle lane (5120 channels: the 2.7B width) takes five
    if (nvec % 320 == 0 && (nvec / 320 == 2 || nvec / 320 == 4) && nvec * vec_elems <= 8192) { *wpg = 5; *nv = (int)(nvec / 320); return true; }
    // up to 8192 channels per group in either type: 4 vectors of 8 per lane (16-bit), 8 vectors of 4 (fp32)
    if (nvec * vec_elems <= 8192) { *wpg = 4; *nv = (int)((nvec + 255) / 256); return true; }
    return false;
}

template <typename T, bool BWD>
int launch_norm(const NormArgs& a, int64_t groups, hipStream_t st) {
    constexpr int V = GlueVec<T>::V;
    int wpg = 0, nv = 0;
    if (!norm_shape(a.gw / V, V, &wpg, &nv))
        return fail(M2_ERR_SHAPE, "rmsnorm_gated: %lld channels per group exceed the supported 8192", (long long)a.gw);
    const dim3 grid((unsigned)ceil_div(a.rows, a.rows_per_block), (unsigned)groups);
    const bool exact = (int64_t)wpg * 64 * nv == a.gw / V, gated = a.z != nullptr;
#define M2_NORM_LAUNCH(W, N, G, E) { rmsnorm_gated_kernel<T, W, N, BWD, G, E><<<grid, (W == 1 ? 256 : W * 64), 0, st>>>(a); return check_launch("rmsnorm_gated_kernel"); }
#define M2_NORM_CASE(W, N) if (wpg == W && nv == N) { \
        if (gated) { if (exact) M2_NORM_LAUNCH(W, N, true, true) else M2_NORM_LAUNCH(W, N, true, false) } \
        else { if (exact) M2_NORM_LAUNCH(W, N, false, true) else M2_NORM_LAUNCH(W, N, false, false) } }
    M2_NORM_CASE(1, 1) M2_NORM_CASE(1, 2) M2_NORM_CASE(1, 3) M2_NORM_CASE(1, 4)
    M2_NORM_CASE(4, 2) M2_NORM_CASE(4, 3) M2_NORM_CASE(4, 4)
    M2_NORM_CASE(5, 2) M2_NORM_CASE(5, 4)
    if constexpr (sizeof(T) == 4) { M2_NORM_CASE(4, 5) M2_NORM_CASE(4, 6) M2_NORM_CASE(4, 7) M2_NORM_CASE(4, 8) }
#undef M2_NORM_CASE
#undef M2_NORM_LAUNCH
    return fail(M2_ERR_SHAPE, "rmsnorm_gated: no kernel for %d waves x %d vectors", wpg, nv);
}

// Block boundary of a decode step: residual += delta; out = weight * residual * rsqrt(mean(residual^2) + eps).
// One workgroup per row, the row (up to 8192 channels) stays in registers between the sum of squares and the output.
template <typename T>
__global__ void __launch_bounds__(256)
add_rmsnorm_kernel(float* __restrict__ res, int64_t res_sr, const T* __restrict__ delta, int64_t delta_sr, const float* __restrict__ w,
                   T* __restrict__ out, int64_t out_sr, int d, float eps) {
    constexpr int NV = 8;
    __shared__ float red[4];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    float* rr = res + row * res_sr;
    const T* dr = delta ? delta + row * delta_sr : nullptr;
    T* orow = out + row * out_sr;
    const int nvec = d / 4;
    floatx4 v[NV];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < NV; ++it) {
        const int vi = it * 256 + tid;
        v[it] = floatx4{0.f, 0.f, 0.f, 0.f};
        if (vi < nvec) {
            floatx4 r = *reinterpret_cast<const floatx4*>(rr + vi * 4);
            if (dr) {
                if constexpr (sizeof(T) == 2) {
                    const uint2 raw = *reinterpret_cast<const uint2*>(dr + vi * 4);
                    r[0] += __builtin_bit_cast(float, raw.x << 16); r[1] += __builtin_bit_cast(float, raw.x & 0xffff0000u);
                    r[2] += __builtin_bit_cast(float, raw.y << 16); r[3] += __builtin_bit_cast(float, raw.y & 0xffff0000u);
                } else {
                    const floatx4 dv = *reinterpret_cast<const floatx4*>(dr + vi * 4);
                    r[0] += dv[0]; r[1] += dv[1]; r[2] += dv[2]; r[3] += dv[3];
                }
                *reinterpret_cast<floatx4*>(rr + vi * 4) = r;
            }
            v[it] = r;
            ss += (r[0] * r[0] + r[1] * r[1]) + (r[2] * r[2] + r[3] * r[3]);
        }
    }
    ss = warp_sum(ss);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    const float rinv = rsqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)d + eps);
#pragma unroll
    for (int it = 0; it < NV; ++it) {
        const int vi = it * 256 + tid;
        if (vi < nvec) {
            const floatx4 wv = *reinterpret_cast<const floatx4*>(w + vi * 4);
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = wv[e] * (v[it][e] * rinv);
            if constexpr (sizeof(T) == 2) {
                T e4[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) e4[e] = from_f32<T>(o[e]);
                *reinterpret_cast<uint2*>(orow + vi * 4) = *reinterpret_cast<const uint2*>(e4);
            } else {
                *reinterpret_cast<floatx4*>(orow + vi * 4) = floatx4{o[0], o[1], o[2], o[3]};
            }
        }
    }
}

int check_norm_common(const m2_rmsnorm_params* p, const char* what) {
    M2_REQUIRE(p, M2_ERR_NULL, "%s: NULL params", what);
    M2_REQUIRE(p->rows >= 0 && p->channels > 0 && p->n_groups > 0 && p->channels % p->n_groups == 0, M2_ERR_SHAPE,
               "%s: rows %lld, channels %lld, groups %d", what, (long long)p->rows, (long long)p->channels, (int)p->n_groups);
    M2_REQUIRE(p->dtype == M2_F32 || p->dtype == M2_BF16, M2_ERR_DTYPE, "%s: unsupported dtype %d", what, (int)p->dtype);
    const int V = p->dtype == M2_F32 ? 4 : 8;
    M2_REQUIRE((p->channels / p->n_groups) % V == 0, M2_ERR_SHAPE, "%s: channels per group must be a multiple of %d", what, V);
    return M2_OK;
}

}  // namespace
}  // namespace m2

extern "C" int m2_softplus_bias_fwd(const void* dt, int64_t dt_stride_row, const float* dt_bias, void* out, int64_t out_stride_row,
                                    int64_t rows, int64_t nheads, int32_t dtype, void* stream) {
    using namespace m2;
    M2_REQUIRE(rows >= 0 && nheads > 0, M2_ERR_SHAPE, "softplus_bias_fwd: rows %lld, heads %lld", (long long)rows, (long long)nheads);
    if (rows == 0) return M2_OK;
    M2_REQUIRE(dt && dt_bias && out, M2_ERR_NULL, "softplus_bias_fwd: dt, dt_bias and out are required");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const unsigned blocks = (unsigned)ceil_div(rows * nheads, (int64_t)256);
    M2_DISPATCH_DTYPE(dtype, T, (softplus_fwd_kernel<T><<<blocks, 256, 0, st>>>(static_cast<const T*>(dt), dt_stride_row, dt_bias,
                                                                                 static_cast<T*>(out), out_stride_row, rows, nheads)));
    return check_launch("softplus_fwd_kernel");
}

extern "C" size_t m2_softplus_bias_bwd_workspace_bytes(int64_t rows, int64_t nheads) {
    if (rows <= 0 || nheads <= 0) return 256;
    return m2::align_up((size_t)m2::ceil_div(rows, (int64_t)m2::kSpRows) * (size_t)nheads * sizeof(float), 256);
}

extern "C" int m2_softplus_bias_bwd(const void* dt, int64_t dt_stride_row, const float* dt_bias, const void* d_out, int64_t d_out_stride_row,
                                    void* d_in, int64_t d_in_stride_row, float* d_bias, void* workspace, size_t workspace_bytes,
                                    int64_t rows, int64_t nheads, int32_t dtype, void* stream) {
    using namespace m2;
    M2_REQUIRE(rows >= 0 && nheads > 0, M2_ERR_SHAPE, "softplus_bias_bwd: rows %lld, heads %lld", (long long)rows, (long long)nheads);
    M2_REQUIRE(d_bias, M2_ERR_NULL, "softplus_bias_bwd: d_bias is required");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t nblk = ceil_div(rows, (int64_t)kSpRows);
    if (rows > 0) {
        M2_REQUIRE(dt && dt_bias && d_out && d_in, M2_ERR_NULL, "softplus_bias_bwd: dt, dt_bias, d_out and d_in are required");
        M2_REQUIRE(workspace && workspace_bytes >= m2_softplus_bias_bwd_workspace_bytes(rows, nheads), M2_ERR_WORKSPACE,
                   "softplus_bias_bwd: workspace %zu bytes < %zu needed", workspace_bytes, m2_softplus_bias_bwd_workspace_bytes(rows, nheads));
        float* partial = static_cast<float*>(workspace);
        M2_DISPATCH_DTYPE(dtype, T, (softplus_bwd_kernel<T><<<(unsigned)nblk, 256, 0, st>>>(
                                         static_cast<const T*>(dt), dt_stride_row, dt_bias, static_cast<const T*>(d_out), d_out_stride_row,
                                         static_cast<T*>(d_in), d_in_stride_row, partial, rows, nheads)));
        int rc = check_launch("softplus_bwd_kernel");
        if (rc) return rc;
    }
    // with no rows the sum is empty: column_sum_kernel writes zeros
    column_sum_kernel<<<(unsigned)ceil_div(nheads, (int64_t)64), 1024, 0, st>>>(static_cast<const float*>(workspace), d_bias, nblk, nheads);
    return check_launch("column_sum_kernel");
}

extern "C" int m2_rmsnorm_gated_fwd(const m2_rmsnorm_params* p, void* stream) {
    using namespace m2;
    int rc = check_norm_common(p, "rmsnorm_gated_fwd");
    if (rc) return rc;
    if (p->rows == 0) return M2_OK;
    M2_REQUIRE(p->x && p->weight && p->out, M2_ERR_NULL, "rmsnorm_gated_fwd: x, weight and out are required");
    const int V = p->dtype == M2_F32 ? 4 : 8;
    M2_REQUIRE(aligned16(p->x) && aligned16(p->out) && (!p->z || aligned16(p->z)) && p->x_stride_row % V == 0 && p->out_stride_row % 4 == 0 &&
                   (p->out_f32 || p->out_stride_row % V == 0) && (!p->z || p->z_stride_row % V == 0),
               M2_ERR_ALIGN, "rmsnorm_gated_fwd: pointers must be 16-byte aligned and row strides multiples of %d elements", V);
    NormArgs a{};
    a.x = p->x; a.x_sr = p->x_stride_row; a.z = p->z; a.z_sr = p->z_stride_row; a.w = p->weight;
    a.out = p->out; a.out_sr = p->out_stride_row; a.out_f32 = p->out_f32 || p->dtype == M2_F32;
    a.rows = p->rows; a.d = p->channels; a.gw = p->channels / p->n_groups; a.eps = p->eps;
    a.rows_per_block = norm_rows_per_block_fwd(p->rows, p->n_groups, a.gw / V);
    hipStream_t st = static_cast<hipStream_t>(stream);
    M2_DISPATCH_DTYPE(p->dtype, T, return (launch_norm<T, false>(a, p->n_groups, st)));
    return M2_OK;
}

extern "C" size_t m2_rmsnorm_gated_bwd_workspace_bytes(int64_t rows, int64_t channels, int32_t n_groups, int32_t dtype) {
    if (rows <= 0 || channels <= 0 || n_groups <= 0) return 256;
    const int64_t nvec = channels / n_groups / (dtype == M2_F32 ? 4 : 8);
    const int64_t nrb = m2::ceil_div(rows, m2::norm_rows_per_block_bwd(rows, n_groups, nvec));
    return m2::align_up((size_t)nrb * 4 * (size_t)channels * sizeof(float), 256);      // up to one partial row per wave
}

extern "C" int m2_rmsnorm_gated_bwd(const m2_rmsnorm_params* p, void* stream) {
    using namespace m2;
    int rc = check_norm_common(p, "rmsnorm_gated_bwd");
    if (rc) return rc;
    M2_REQUIRE(p->d_weight, M2_ERR_NULL, "rmsnorm_gated_bwd: d_weight is required");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int V = p->dtype == M2_F32 ? 4 : 8;
    int64_t prows = 0;
    if (p->rows > 0) {
        M2_REQUIRE(p->x && p->weight && p->d_out && p->dx, M2_ERR_NULL, "rmsnorm_gated_bwd: x, weight, d_out and dx are required");
        M2_REQUIRE(!p->z || p->dz, M2_ERR_NULL, "rmsnorm_gated_bwd: dz is required when z is given");
        M2_REQUIRE(aligned16(p->x) && aligned16(p->d_out) && aligned16(p->dx) && (!p->z || (aligned16(p->z) && aligned16(p->dz))) &&
                       p->x_stride_row % V == 0 && p->d_out_stride_row % V == 0 && p->dx_stride_row % V == 0 &&
                       (!p->z || (p->z_stride_row % V == 0 && p->dz_stride_row % V == 0)),
                   M2_ERR_ALIGN, "rmsnorm_gated_bwd: pointers must be 16-byte aligned and row strides multiples of %d elements", V);
        const size_t need = m2_rmsnorm_gated_bwd_workspace_bytes(p->rows, p->channels, p->n_groups, p->dtype);
        M2_REQUIRE(p->workspace && p->workspace_bytes >= need, M2_ERR_WORKSPACE, "rmsnorm_gated_bwd: workspace %zu bytes < %zu needed",
                   p->workspace_bytes, need);
        M2_REQUIRE((reinterpret_cast<uintptr_t>(p->workspace) & 15u) == 0, M2_ERR_ALIGN, "rmsnorm_gated_bwd: workspace must be 16-byte aligned");
        NormArgs a{};
        a.x = p->x; a.x_sr = p->x_stride_row; a.z = p->z; a.z_sr = p->z_stride_row; a.w = p->weight;
        a.g = p->d_out; a.g_sr = p->d_out_stride_row; a.dx = p->dx; a.dx_sr = p->dx_stride_row; a.dz = p->dz; a.dz_sr = p->dz_stride_row;
        a.partial = static_cast<float*>(p->workspace);
        a.rows = p->rows; a.d = p->channels; a.gw = p->channels / p->n_groups; a.eps = p->eps;
        a.rows_per_block = norm_rows_per_block_bwd(p->rows, p->n_groups, a.gw / V);
        int wpg = 0, nv = 0;
        if (!norm_shape(a.gw / V, V, &wpg, &nv))
            return fail(M2_ERR_SHAPE, "rmsnorm_gated_bwd: %lld channels per group exceed the supported 8192", (long long)a.gw);
        prows = ceil_div(p->rows, a.rows_per_block) * (wpg > 1 ? 1 : 4);
        M2_DISPATCH_DTYPE(p->dtype, T, rc = (launch_norm<T, true>(a, p->n_groups, st)));
        if (rc) return rc;
    }
    column_sum_kernel<<<(unsigned)ceil_div(p->channels, (int64_t)64), 1024, 0, st>>>(static_cast<const float*>(p->workspace), p->d_weight,
                                                                                     prows, p->channels);
    return check_launch("column_sum_kernel");
}

extern "C" int m2_add_rmsnorm(float* residual, int64_t residual_stride_row, const void* delta, int64_t delta_stride_row,
                              const float* weight, void* out, int64_t out_stride_row, int64_t rows, int64_t channels, float eps,
                              int32_t dtype, void* stream) {
    using namespace m2;
    M2_REQUIRE(rows >= 0 && channels > 0, M2_ERR_SHAPE, "add_rmsnorm: rows %lld, channels %lld", (long long)rows, (long long)channels);
    M2_REQUIRE(channels % 4 == 0 && channels <= 8192, M2_ERR_SHAPE, "add_rmsnorm: channels %lld must be a multiple of 4, at most 8192",
               (long long)channels);
    M2_REQUIRE(dtype == M2_F32 || dtype == M2_BF16, M2_ERR_DTYPE, "add_rmsnorm: unsupported dtype %d", (int)dtype);
    if (rows == 0) return M2_OK;
    M2_REQUIRE(residual && weight && out, M2_ERR_NULL, "add_rmsnorm: residual, weight and out are required");
    const size_t es = dtype == M2_F32 ? 4 : 2;
    M2_REQUIRE(aligned16(residual) && aligned16(weight) && residual_stride_row % 4 == 0 && (uintptr_t)out % (4 * es) == 0 &&
                   out_stride_row % 4 == 0 && (!delta || ((uintptr_t)delta % (4 * es) == 0 && delta_stride_row % 4 == 0)),
               M2_ERR_ALIGN, "add_rmsnorm: rows must start on 4-element boundaries (residual and weight on 16 bytes)");
    M2_REQUIRE(rows <= 0x7fffffff, M2_ERR_SHAPE, "add_rmsnorm: too many rows");
    hipStream_t st = static_cast<hipStream_t>(stream);
    M2_DISPATCH_DTYPE(dtype, T, (add_rmsnorm_kernel<T><<<(unsigned)rows, 256, 0, st>>>(residual, residual_stride_row, static_cast<const T*>(delta),
                                                                                     delta_stride_row, weight, static_cast<T*>(out),
                                                                                     out_stride_row, (int)channels, eps)));
    return check_launch("add_rmsnorm_kernel");
}
