// SSD chunked-scan forward for gfx950.
//
// Replaces the reference's NKI kernel mamba_kernel_ (mamba2/mamba2_kernel.py:67-170), which walks
// the chunks of one (batch, head) sequentially with the state on chip.  Here only the state recurrence
// is sequential in the chunk index; everything else is one independent workgroup per (batch, chunk,
// group) that loops over a slice of the group's heads:
//
//   1. prep_kernel         l = cumsum(A dt) per (b, head, chunk);  G = C B^T (+ operand tiles) per (b, chunk, group)
//   2. states entering the chunks, final state
//        16-bit: state_pass16_kernel   contributions B^T (decay o dt o X) and recurrence fused, per (b, head)
//        fp32  : chunk_state_kernel + state_scan_kernel
//   3. ssd_y16_kernel (16-bit) / diag_off_kernel<false>      Y = (L o G)(dt o X) + e^l C S_prev + D X   MFMA
//
// Extensions over the reference kernel: optional initial state, final-state output, any batch,
// ragged sequence length (tokens past the end behave as dt = 0 and are never written).
#include "ssd_host.hpp"
#include "ssd_y.hpp"

namespace m2 {
namespace {

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
