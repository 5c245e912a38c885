// SSD chunked-scan forward for gfx950.
//
// Replaces the reference's NKI kernel mamba_kernel_ (mamba2/mamba2_kernel.py:67-170), which walks
// the chunks of one (batch, head) sequentially with the state on chip.  Here the work is split so
// that every (batch, head, chunk) tile is an independent workgroup (thousands of them for 256 CUs)
// and only a cheap elementwise recurrence is sequential in the chunk index:
//
//   1. cb_kernel           G = C B^T                         per (b, chunk, group)   MFMA
//   2. chunk_state_kernel  local state B^T (decay o dt o X)  per (b, chunk, head)    MFMA
//   3. state_scan_kernel   S_prev(c), final state            per (b, head)           fp32 FMA
//   4. chunk_scan_kernel   Y = (L o G)(dt o X) + e^l C S_prev + D X   per (b, chunk, head)   MFMA
//
// Extensions over the reference kernel: optional initial state, final-state output, any batch,
// ragged sequence length (tokens past the end behave as dt = 0 and are never written).
#include "ssd_host.hpp"
#include "ssd_y.hpp"

namespace m2 {
namespace {

// ------------------------------------------------------------------------------------------
// grid (nchunks, nheads, batch), 256 threads (4 waves; wave w owns output rows 32w..32w+31).
template <typename T, int P, int N>
__global__ void __launch_bounds__(256)
chunk_scan_kernel(const T* __restrict__ X, const void* __restrict__ dt, int dt_f32, const float* __restrict__ A,
                  const T* __restrict__ Cm, const float* __restrict__ D, const float* __restrict__ G,
                  const T* __restrict__ Sprev, T* __restrict__ Y,
                  int64_t seqlen, int64_t nheads, int64_t ngroups, int64_t nchunks,
                  int64_t Xsb, int64_t Xsl, int64_t Xsh, int64_t dtsb, int64_t dtsl,
                  int64_t Csb, int64_t Csl, int64_t Csg, int64_t Ysb, int64_t Ysl, int64_t Ysh) {
    constexpr int LDN = lds_ld<T>(N);      // tiles with N (state) columns
    constexpr int LDQ = lds_ld<T>(kQ);     // tiles with Q (token) columns
    constexpr int BN = P / 32;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    float* s_l = reinterpret_cast<float*>(smem_raw);
    float* s_dt = s_l + kQ;
    float* s_tmp = s_dt + kQ;                       // 4 floats
    T* buf = reinterpret_cast<T*>(s_tmp + 4);
    // phase 1: sC [kQ][LDN], sS [P][LDN];   phase 2: sM [kQ][LDQ], sXt [P][LDQ]   (same memory)
    T* sC = buf;
    T* sS = buf + kQ * LDN;
    T* sM = buf;
    T* sXt = buf + kQ * LDQ;

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int64_t c = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int64_t g = h / (nheads / ngroups);
    const int64_t t0 = c * kQ;
    const int valid = (int)((seqlen - t0) < kQ ? (seqlen - t0) : kQ);

    chunk_cumsum_any<T>(dt, dt_f32, b * dtsb + t0 * dtsl + h, dtsl, valid, A[h], s_l, s_dt, s_tmp, tid);

    // ---- phase 1: off-diagonal term  acc[t][p] = e^{l_t} * sum_n C[t][n] S_prev[p][n]
    const int64_t tile = ((b * nchunks + c) * nheads + h) * (int64_t)(P * N);
    stage_rows<T, kQ, N, 256, false>(sC, LDN, Cm + b * Csb + t0 * Csl + g * Csg, Csl, valid, nullptr, tid);
    stage_rows<T, P, N, 256, false>(sS, LDN, Sprev + tile, N, P, nullptr, tid);
    __syncthreads();
    floatx16 acc[1][BN];
    acc_zero(acc);
    wave_mma<1, BN>(acc, sC + wave * 32 * LDN, LDN, sS, LDN, 0, N);
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const float e = __expf(s_l[wave * 32 + acc_row(lane, v)]);
#pragma unroll
        for (int j = 0; j < BN; ++j) acc[0][j][v] *= e;
    }
    __syncthreads();     // everyone done reading sC / sS

    // ---- phase 2: diagonal term  acc[t][p] += sum_{s<=t} (e^{l_t-l_s} dt_s G[t][s]) x[s][p]
    const float* Gp = G + ((b * nchunks + c) * ngroups + g) * (int64_t)(kQ * kQ);
    for (int e = tid; e < kQ * (kQ / 4); e += 256) {
        const int t = e / (kQ / 4), s4 = (e % (kQ / 4)) * 4;
        if ((s4 >> 5) > (t >> 5)) continue;           // 32x32 block above the diagonal: never read
        const floatx4 g4 = *reinterpret_cast<const floatx4*>(Gp + t * kQ + s4);
        const float lt = s_l[t];
        T o[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int s = s4 + q;
            const float m = (s <= t) ? __expf(lt - s_l[s]) * s_dt[s] * g4[q] : 0.f;
            o[q] = from_f32<T>(m);
        }
        if (sizeof(T) == 2) *reinterpret_cast<uint2*>(sM + t * LDQ + s4) = *reinterpret_cast<const uint2*>(o);
        else *reinterpret_cast<uint4*>(sM + t * LDQ + s4) = *reinterpret_cast<const uint4*>(o);
    }
    const T* Xp = X + b * Xsb + t0 * Xsl + h * Xsh;
    stage_transposed<T, kQ, P, 256, false>(sXt, LDQ, Xp, Xsl, valid, nullptr, tid);
    __syncthreads();
    wave_mma<1, BN>(acc, sM + wave * 32 * LDQ, LDQ, sXt, LDQ, 0, (wave + 1) * 32);

    // ---- epilogue: + D x, store
    const float Dh = D ? D[h] : 0.f;
    T* Yp = Y + b * Ysb + t0 * Ysl + h * Ysh;
#pragma unroll
    for (int j = 0; j < BN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = wave * 32 + acc_row(lane, v);
            const int col = j * 32 + acc_col(lane);
            if (row < valid) {
                const float xv = to_f32(sXt[col * LDQ + row]);
                Yp[(int64_t)row * Ysl + col] = from_f32<T>(acc[0][j][v] + Dh * xv);
            }
        }
}

template <typename T, int P, int N>
size_t scan_smem() {
    const size_t a = (size_t)(kQ + P) * lds_ld<T>(N), b = (size_t)(kQ + P) * lds_ld<T>(kQ);
    return (2 * kQ + 4) * sizeof(float) + (a > b ? a : b) * sizeof(T);
}

// zero-length sequence: y is empty; the final state is the initial state (or zero)
__global__ void copy_or_zero_kernel(const float* __restrict__ src, float* __restrict__ dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src ? src[i] : 0.f;
}

template <typename T, int P, int N>
int ssd_fwd_impl(const m2_ssd_params* p, hipStream_t st) {
    const int64_t nc = ceil_div(p->seqlen, (int64_t)kQ);
    const SsdWorkspace w = ssd_carve(p, p->workspace, false);
    int rc;
    if ((rc = ssd_launch_states<T, P, N>(p, w, p->final_state, st))) return rc;
    DiagArgs a{};
    a.dt = p->dt; a.dt_f32 = p->dt_dtype == M2_F32; a.A = p->A; a.D = p->D;
    a.Aoff = p->C; a.Ao_sb = p->C_stride_b; a.Ao_sl = p->C_stride_l; a.Ao_sg = p->C_stride_g;
    a.Gd = w.Gm; a.S = w.prev; a.ldtab = w.ldtab;
    a.Z = p->x; a.Z_sb = p->x_stride_b; a.Z_sl = p->x_stride_l; a.Z_sh = p->x_stride_h;
    a.dt_sb = p->dt_stride_b; a.dt_sl = p->dt_stride_l;
    a.seqlen = p->seqlen; a.nheads = p->nheads; a.ngroups = p->ngroups; a.nchunks = nc;
    ssd_slicing(p, kWgsY, &a.nslices, &a.hps);
    a.Y = p->y; a.Y_sb = p->y_stride_b; a.Y_sl = p->y_stride_l; a.Y_sh = p->y_stride_h;
    M2_REQUIRE(p->ngroups * a.nslices <= 65535, M2_ERR_SHAPE, "ssd_fwd: too many group slices");
    const dim3 grid((unsigned)nc, (unsigned)(p->ngroups * a.nslices), (unsigned)p->batch);
    if constexpr (sizeof(T) == 2 && y16_smem<P, N>() <= 160 * 1024) {
        auto k = ssd_y16_kernel<T, P, N>;
        const size_t sm = y16_smem<P, N>();
        if ((rc = allow_smem(k, sm))) return rc;
        k<<<grid, 256, sm, st>>>(a);
        return check_launch("ssd_y16_kernel");
    }
    auto k = diag_off_kernel<T, P, N, false>;
    const size_t sm = diag_smem<T, P, N, false>();
    if ((rc = allow_smem(k, sm))) return rc;
    k<<<grid, 256, sm, st>>>(a);
    return check_launch("ssd diag_off_kernel<fwd>");
}

}  // namespace
}  // namespace m2

extern "C" size_t m2_ssd_chunk_states_bytes(const m2_ssd_params* p) {
    if (!p || p->batch <= 0 || p->seqlen <= 0 || p->nheads <= 0) return 0;
    return m2::ssd_carve(p, nullptr, false, true).kept_bytes;
}

extern "C" size_t m2_ssd_fwd_workspace_bytes(const m2_ssd_params* p) {
    if (!p || p->batch <= 0 || p->seqlen <= 0 || p->nheads <= 0) return 256;
    return m2::ssd_carve(p, nullptr, false).bytes;
}

extern "C" int m2_ssd_fwd(const m2_ssd_params* p, void* stream) {
    using namespace m2;
    int rc = ssd_check(p, "ssd_fwd");
    if (rc) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (p->batch == 0 || p->nheads == 0) return M2_OK;
    if (p->seqlen == 0) {
        if (p->final_state) {
            const int64_t n = p->batch * p->nheads * p->headdim * p->dstate;
            copy_or_zero_kernel<<<(unsigned)ceil_div(n, (int64_t)256), 256, 0, st>>>(p->initial_state, p->final_state, n);
            return check_launch("ssd copy_or_zero_kernel");
        }
        return M2_OK;
    }
    M2_REQUIRE(p->x && p->dt && p->A && p->B && p->C && p->y, M2_ERR_NULL, "ssd_fwd: x, dt, A, B, C, y are required");
    {
        const int V = p->dtype == M2_F32 ? 4 : 8;
        M2_REQUIRE(aligned16(p->y) && p->y_stride_b % V == 0 && p->y_stride_l % V == 0 && p->y_stride_h % V == 0, M2_ERR_ALIGN,
                   "ssd_fwd: y and its strides must be 16-byte aligned (multiples of %d elements)", V);
    }
    const size_t need = m2_ssd_fwd_workspace_bytes(p);
    M2_REQUIRE(p->workspace && p->workspace_bytes >= need, M2_ERR_WORKSPACE, "ssd_fwd: workspace %zu bytes < %zu needed",
               p->workspace_bytes, need);
    M2_REQUIRE((reinterpret_cast<uintptr_t>(p->workspace) & 255u) == 0, M2_ERR_ALIGN, "ssd_fwd: workspace must be 256-byte aligned");
    M2_DISPATCH_DTYPE(p->dtype, T, M2_DISPATCH_PN(p, P, N, return (ssd_fwd_impl<T, P, N>(p, st))));
    return M2_OK;
}
