// Host-side helpers shared by the SSD forward and backward launchers.
#pragma once
#include "ssd_kernels.hpp"
#include "ssd_diag.hpp"
#include "ssd_bwd_main.hpp"
#include "ssd_dg.hpp"
#include "ssd_states16.hpp"

namespace m2 {

// Workspace regions.  Forward uses G, local, prev, lam.  Backward additionally uses
// dprev (gradient w.r.t. the state leaving each chunk, operand type), dlam, dl (per-token gradient of the in-chunk cumulative
// sum, per head), per-(b,h,chunk) partials of dA and dD, and
// per-(b,chunk,group,head-slice) fp32 partials of dB and dC.
struct SsdWorkspace {
    float* G = nullptr; float* local = nullptr; void* prev = nullptr; float* lam = nullptr;
    void* Gm = nullptr; void* Gmt = nullptr; void* Bt = nullptr; void* Ct = nullptr;
    float* ldtab = nullptr;             // [b][h][c][ l kQ | dt kQ ]
    void* dprev = nullptr; float* dlam = nullptr;
    float* dbp = nullptr;                                               // per (b, h, chunk) partials of d_dt_bias
    float* dAp = nullptr; float* dDp = nullptr; float* dBp = nullptr; float* dCp = nullptr; float* dl = nullptr; float* dlc = nullptr; float* dGp = nullptr;
    float* dGs = nullptr; float* dBs = nullptr; float* dCs = nullptr;   // partials summed over the head slices
    float* dirp = nullptr; float* rbp = nullptr; float* dDp8 = nullptr; // per channel-half / per-wave partials of the dx kernel
    int64_t ns_g = 1, hps_g = 1, ns_c = 1, hps_c = 1, ns_b = 1, hps_b = 1;   // head slicing of the dg / off<C> / off<B> kernels
    size_t bytes = 0;
    size_t kept_bytes = 0;              // size of the forward -> backward carry-over (chunk_states buffer)
};

// A workgroup owns one chunk of one group and loops over a slice of that group's heads (operands shared by the
// group stay on chip, group-level reductions happen in registers).  The slice count is the smallest divisor of
// heads-per-group that gives at least `wgs_per_cu` workgroups per compute unit: the grid then fills the GPU in one
// round of long-running workgroups (measured: fewer, longer workgroups beat more, shorter ones for every kernel).
inline void ssd_slicing(const m2_ssd_params* p, int wgs_per_cu, int64_t* nslices, int64_t* hps) {
    const int64_t nc = ceil_div(p->seqlen, (int64_t)kQ);
    const int64_t hpg = p->nheads / p->ngroups;
    const int64_t base = p->batch * nc * p->ngroups;
    const int64_t target = device_cus() * wgs_per_cu;
    int64_t best = 1;
    for (int64_t s = 1; s <= hpg; ++s) {
        if (hpg % s) continue;
        best = s;
        if (base * s >= target) break;
    }
    *nslices = best;
    *hps = hpg / best;
}
constexpr int kWgsChunkState = 2, kWgsY = 2, kWgsDx = 1, kWgsDg = 1, kWgsOffC = 1, kWgsOffB = 2;

inline SsdWorkspace ssd_carve(const m2_ssd_params* p, void* base, bool bwd, bool kept_only = false) {
    const int64_t nc = ceil_div(p->seqlen, (int64_t)kQ);
    const size_t esz = p->dtype == M2_F32 ? 4 : 2;
    const size_t tiles = (size_t)p->batch * nc * p->nheads * p->headdim * p->dstate;
    const size_t bhc = (size_t)p->batch * p->nheads * nc;
    size_t off = 0;
    SsdWorkspace w;
    unsigned char* b8 = static_cast<unsigned char*>(base);
    auto take = [&](size_t n) { unsigned char* r = b8 ? b8 + off : nullptr; off += align_up(n, 256); return r; };
    // per-chunk state contributions: only the fp32 path materialises them (16-bit operands take the fused state pass)
    if (p->dtype == M2_F32) w.local = reinterpret_cast<float*>(take(tiles * 4));
    // What the backward reuses from the forward: the state entering each chunk, the decay tables and the
    // per-(chunk, group) operand tiles.  They live in the caller's chunk_states buffer when one is given
    // (forward writes, backward reads), otherwise in the workspace (backward recomputes them).
    {
        size_t koff = 0;
        unsigned char* k8 = static_cast<unsigned char*>(p->chunk_states);
        auto keep = [&](size_t n) -> unsigned char* {
            if (!p->chunk_states && !kept_only) return take(n);
            unsigned char* r = k8 ? k8 + koff : nullptr;
            koff += align_up(n, 256);
            return r;
        };
        const size_t grp = (size_t)p->batch * nc * p->ngroups;
        w.prev = keep(tiles * esz);
        w.lam = reinterpret_cast<float*>(keep(bhc * 4));
        w.ldtab = reinterpret_cast<float*>(keep(bhc * 2 * kQ * 4));
        w.G = reinterpret_cast<float*>(keep(grp * kQ * kQ * 4));
        w.Gm = keep(grp * kQ * kQ * esz);
        w.Gmt = keep(grp * kQ * kQ * esz);
        w.Bt = keep(grp * p->dstate * kQ * esz);
        w.Ct = keep(grp * p->dstate * kQ * esz);
        w.kept_bytes = koff;
    }
    if (bwd) {
        ssd_slicing(p, kWgsDg, &w.ns_g, &w.hps_g);
        ssd_slicing(p, kWgsOffC, &w.ns_c, &w.hps_c);
        ssd_slicing(p, kWgsOffB, &w.ns_b, &w.hps_b);
        if (p->dtype != M2_F32 && p->headdim == 64) {       // the main backward kernel produces both state parts there
            ssd_slicing(p, kWgsDx, &w.ns_b, &w.hps_b);
            w.ns_c = w.ns_b; w.hps_c = w.hps_b;
        }
        w.dprev = take(tiles * esz);
        w.dlam = reinterpret_cast<float*>(take(bhc * 4 * kDlamParts));
        w.dAp = reinterpret_cast<float*>(take(bhc * 4));
        w.dDp = reinterpret_cast<float*>(take(bhc * 4));
        w.dbp = reinterpret_cast<float*>(take(bhc * 4));
        w.dl = reinterpret_cast<float*>(take(bhc * kQ * 4));
        w.dlc = reinterpret_cast<float*>(take(bhc * kQ * 4));
        w.dirp = reinterpret_cast<float*>(take(bhc * 2 * kQ * 4));
        w.rbp = reinterpret_cast<float*>(take(bhc * 2 * kQ * 4));
        w.dDp8 = reinterpret_cast<float*>(take(bhc * 8 * 4));
        w.dGp = reinterpret_cast<float*>(take((size_t)p->batch * nc * p->ngroups * w.ns_g * kQ * kQ * 4));
        const size_t part = (size_t)p->batch * nc * p->ngroups * kQ * p->dstate * 4;
        w.dBp = reinterpret_cast<float*>(take(part * w.ns_b));
        w.dCp = reinterpret_cast<float*>(take(part * w.ns_c));
        w.dGs = reinterpret_cast<float*>(take((size_t)p->batch * nc * p->ngroups * kQ * kQ * 4));
        w.dBs = reinterpret_cast<float*>(take((size_t)p->batch * nc * p->ngroups * kQ * p->dstate * 4));
        w.dCs = reinterpret_cast<float*>(take((size_t)p->batch * nc * p->ngroups * kQ * p->dstate * 4));
    }
    w.bytes = off + 256;
    return w;
}

inline int ssd_check(const m2_ssd_params* p, const char* who) {
    M2_REQUIRE(p, M2_ERR_NULL, "%s: params is NULL", who);
    M2_REQUIRE(p->dtype == M2_F32 || p->dtype == M2_BF16, M2_ERR_DTYPE, "%s: bad dtype %d", who, p->dtype);
    M2_REQUIRE(p->dt_dtype == M2_F32 || p->dt_dtype == p->dtype, M2_ERR_DTYPE,
               "%s: dt dtype %d must be fp32 or the activation dtype", who, p->dt_dtype);
    M2_REQUIRE(p->batch >= 0 && p->seqlen >= 0 && p->nheads >= 0, M2_ERR_SHAPE, "%s: negative dimension", who);
    M2_REQUIRE(p->headdim == 64 || p->headdim == 128, M2_ERR_SHAPE, "%s: headdim %lld not in {64,128}", who, (long long)p->headdim);
    M2_REQUIRE(p->dstate == 64 || p->dstate == 128, M2_ERR_SHAPE, "%s: dstate %lld not in {64,128}", who, (long long)p->dstate);
    M2_REQUIRE(p->ngroups >= 1 && p->nheads % p->ngroups == 0, M2_ERR_SHAPE, "%s: nheads %lld not divisible by ngroups %lld", who,
               (long long)p->nheads, (long long)p->ngroups);
    M2_REQUIRE(p->batch <= 65535 && p->nheads <= 65535, M2_ERR_SHAPE, "%s: batch/nheads exceed the grid limit 65535", who);
    const int V = p->dtype == M2_F32 ? 4 : 8;
    M2_REQUIRE(p->x_stride_b % V == 0 && p->x_stride_l % V == 0 && p->x_stride_h % V == 0 &&
               p->B_stride_b % V == 0 && p->B_stride_l % V == 0 && p->B_stride_g % V == 0 &&
               p->C_stride_b % V == 0 && p->C_stride_l % V == 0 && p->C_stride_g % V == 0,
               M2_ERR_ALIGN, "%s: x/B/C strides must be multiples of %d elements (16 bytes)", who, V);
    M2_REQUIRE(aligned16(p->x) && aligned16(p->B) && aligned16(p->C), M2_ERR_ALIGN, "%s: x/B/C must be 16-byte aligned", who);
    {
        // the kernels address the rows of a chunk with 32-bit byte offsets formed by 24-bit multiplies
        const int64_t lim = (int64_t)1 << 21;
        auto ok = [&](int64_t s) { return s >= 0 && s < lim; };
        M2_REQUIRE(ok(p->x_stride_l) && ok(p->B_stride_l) && ok(p->C_stride_l) && ok(p->dt_stride_l) && (!p->y || ok(p->y_stride_l)),
                   M2_ERR_SHAPE, "%s: token strides must lie in [0, 2^21) elements", who);
        M2_REQUIRE(!p->dy || (ok(p->dy_stride_l) && ok(p->dx_stride_l) && ok(p->dB_stride_l) && ok(p->dC_stride_l) && ok(p->ddt_stride_l)),
                   M2_ERR_SHAPE, "%s: token strides of the gradients must lie in [0, 2^21) elements", who);
    }
    M2_REQUIRE(aligned16(p->chunk_states), M2_ERR_ALIGN, "%s: chunk_states must be 16-byte aligned", who);
    return M2_OK;
}

template <typename K>
inline int allow_smem(K kernel, size_t bytes) {
    if (bytes > 160 * 1024) return fail(M2_ERR_SHAPE, "kernel needs %zu bytes of LDS (> 160 KiB)", bytes);
    if (bytes > 48 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess)
            return fail(M2_ERR_LAUNCH, "hipFuncSetAttribute(%zu bytes of LDS) failed: %s", bytes, hipGetErrorString(hipGetLastError()));
    }
    return M2_OK;
}

template <typename T, int P, int N>
inline size_t state_smem() { return (size_t)(P + N) * lds_ld<T>(kQ) * sizeof(T); }
template <typename T>
inline size_t cb_smem(int n) { return (size_t)2 * 64 * lds_ld<T>(n) * sizeof(T); }

// Decay tables, G = C B^T (+ operand tiles), local chunk states, forward state scan.  Used by the forward and, when the
// caller did not keep the forward's chunk_states buffer, by the backward (recompute).
template <typename T, int P, int N>
inline int ssd_launch_states(const m2_ssd_params* p, const SsdWorkspace& w, float* final_out, hipStream_t st) {
    const int64_t nc = ceil_div(p->seqlen, (int64_t)kQ);
    const T* x = static_cast<const T*>(p->x);
    const T* Bm = static_cast<const T*>(p->B);
    const T* Cm = static_cast<const T*>(p->C);
    const int dt_f32 = p->dt_dtype == M2_F32;
    int rc;
    {
        // decay tables and G = C B^T (+ operand tiles), one launch
        auto k = prep_kernel<T, N>;
        const size_t sm = cb_smem<T>(N);
        if ((rc = allow_smem(k, sm))) return rc;
        PrepArgs pa;
        pa.Bm = Bm; pa.Cm = Cm; pa.Gf = w.G; pa.Gm = w.Gm; pa.Gmt = w.Gmt; pa.Bt = w.Bt; pa.Ct = w.Ct;
        pa.Bsb = p->B_stride_b; pa.Bsl = p->B_stride_l; pa.Bsg = p->B_stride_g;
        pa.Csb = p->C_stride_b; pa.Csl = p->C_stride_l; pa.Csg = p->C_stride_g;
        pa.dt = p->dt; pa.dt_f32 = dt_f32; pa.dt_bias = p->dt_bias; pa.A = p->A; pa.ldtab = w.ldtab; pa.lam = w.lam;
        pa.dtsb = p->dt_stride_b; pa.dtsl = p->dt_stride_l;
        pa.seqlen = p->seqlen; pa.nheads = p->nheads; pa.ngroups = p->ngroups; pa.nchunks = nc;
        pa.n_cb = nc * p->ngroups * p->batch;
        const int64_t blocks = kCbParts * pa.n_cb + ld_table_blocks(p->batch, p->nheads, nc);
        M2_REQUIRE(blocks < ((int64_t)1 << 31), M2_ERR_SHAPE, "ssd: too many workgroups");
        k<<<(unsigned)blocks, 256, sm, st>>>(pa);
        if ((rc = check_launch("ssd prep_kernel"))) return rc;
    }
    if constexpr (sizeof(T) == 2) {
        // 16-bit operands: contributions and recurrence in one pass, running state in registers
        // a caller that wants the final state (an fp32 output) gets the two-tile form, whose operand rounding is 2^-17
        // (3.7 us more per pass at b4 l2048 h80; the states entering the chunks come out of the same accumulators, so y
        // differs from the one-tile form in the last bit here and there)
        const bool hilo = final_out != nullptr;
        constexpr int SPLIT = kStatePassSplit;
        auto k = hilo ? state_pass16_kernel<T, P, N, false, false, true, SPLIT> : state_pass16_kernel<T, P, N, false, false, false, SPLIT>;
        const size_t sm = hilo ? state_pass_smem<P, N, true, SPLIT>() : state_pass_smem<P, N, false, SPLIT>();
        if ((rc = allow_smem(k, sm))) return rc;
        StatePassArgs sa;
        sa.X = x; sa.X_sb = p->x_stride_b; sa.X_sl = p->x_stride_l; sa.X_sh = p->x_stride_h;
        sa.ldtab = w.ldtab; sa.Mt = w.Bt; sa.init = p->initial_state; sa.prev = w.prev; sa.final_out = final_out;
        sa.sprev = nullptr; sa.dlam = nullptr;
        sa.seqlen = p->seqlen; sa.nheads = p->nheads; sa.ngroups = p->ngroups; sa.nchunks = nc;
        k<<<dim3((unsigned)(p->nheads * SPLIT), (unsigned)p->batch), state_pass_threads<N>(), sm, st>>>(sa);
        return check_launch("ssd state_pass16_kernel");
    } else {
        // fp32 operands: per-chunk contributions (fp32, workspace), then the recurrence over the chunks
        auto k = chunk_state_kernel<T, P, N, false>;
        const size_t sm = state_smem<T, P, N>();
        if ((rc = allow_smem(k, sm))) return rc;
        int64_t ns, hps;
        ssd_slicing(p, kWgsChunkState, &ns, &hps);
        M2_REQUIRE(p->ngroups * ns <= 65535, M2_ERR_SHAPE, "ssd: too many group slices");
        k<<<dim3((unsigned)nc, (unsigned)(p->ngroups * ns), (unsigned)p->batch), 256, sm, st>>>(
            x, w.ldtab, static_cast<const T*>(w.Bt), w.local, p->seqlen, p->nheads, p->ngroups, nc, ns, hps,
            p->x_stride_b, p->x_stride_l, p->x_stride_h);
        if ((rc = check_launch("ssd chunk_state_kernel"))) return rc;
        state_scan_kernel<T, P * N, false><<<dim3((unsigned)p->nheads, (unsigned)p->batch, kScanSplit), 256, 0, st>>>(
            w.local, w.lam, p->initial_state, static_cast<T*>(w.prev), final_out, nullptr, nullptr, p->nheads, nc);
        if ((rc = check_launch("ssd state_scan_kernel"))) return rc;
        return M2_OK;
    }
}

#define M2_DISPATCH_PN(p, P, N, ...)                                                     \
    do {                                                                                 \
        if ((p)->headdim == 64 && (p)->dstate == 64) { constexpr int P = 64, N = 64; __VA_ARGS__; }        \
        else if ((p)->headdim == 64 && (p)->dstate == 128) { constexpr int P = 64, N = 128; __VA_ARGS__; } \
        else if ((p)->headdim == 128 && (p)->dstate == 64) { constexpr int P = 128, N = 64; __VA_ARGS__; } \
        else { constexpr int P = 128, N = 128; __VA_ARGS__; }                            \
    } while (0)

}  // namespace m2
