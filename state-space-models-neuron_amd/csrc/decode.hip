// Single-token recurrent decode step for gfx950.
//
// Replaces the reference's NKI kernel mamba_inference_kernel_ (mamba2/mamba2_kernel_inference.py:27-104):
//   conv state shift + 1-token depthwise conv + SiLU on all of [x | B | C]     (:13-23)
//   S' = S * exp(A dt) + (dt x) (x) B                                          (:81,95-97)
//   y  = S' . C + D x                                                          (:101-102)
//
// The step is a pure streaming problem: per layer the fp32 state (b,h,p,n) is read once and written
// once, in place (the reference writes fresh copies, doubling the footprint).  Two launches:
//   decode_conv_kernel   one thread per (batch, channel): shifts the conv state in place and writes the
//                        activated [x | B | C] row as fp32 into the workspace.  It must finish before any
//                        state workgroup reads B/C, because every head of a group needs the same B/C
//                        channels whose history is being overwritten in place.
//   decode_ssm_kernel    one workgroup per (head, batch); a group of lanes owns one state row p and walks
//                        n with 16-byte accesses, so a wave issues whole 128-byte-or-wider lines and every
//                        state element is touched by exactly one thread (in-place update is race free).
#include <mutex>

#include "common.hpp"

namespace m2 {
namespace {

constexpr int kUP = 8;     // state rows a lane keeps in flight in the fast path

__device__ __forceinline__ float ld_any(const void* p, int dt, int64_t i) {
    return dt == M2_F32 ? reinterpret_cast<const float*>(p)[i] : to_f32(reinterpret_cast<const bf16_t*>(p)[i]);
}

template <typename T>
__global__ void __launch_bounds__(256)
decode_conv_kernel(const T* __restrict__ xBC, T* __restrict__ conv_state, const void* __restrict__ w, const void* __restrict__ bias,
                   float* __restrict__ act, int64_t nb, int64_t Cx, int k, int W, int64_t xsb, int pd, int activation) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= nb * Cx) return;
    const int64_t b = idx / Cx, c = idx % Cx;
    T* cs = conv_state + idx * W;
    float hist[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) hist[i] = 0.f;
    T raw[8];
    for (int i = 0; i < W; ++i) raw[i] = cs[i];
    const T xin = xBC[b * xsb + c];
    // taps: the last k-1 OLD columns, then the new input
    float z = bias ? ld_any(bias, pd, c) : 0.f;
    for (int i = 0; i < k - 1; ++i) z += ld_any(w, pd, c * k + i) * to_f32(raw[W - (k - 1) + i]);
    z += ld_any(w, pd, c * k + (k - 1)) * to_f32(xin);
    // shift left by one, append the input
    for (int i = 0; i + 1 < W; ++i) cs[i] = raw[i + 1];
    if (W > 0) cs[W - 1] = xin;
    act[idx] = activation == M2_ACT_SILU ? silu_f(z) : (activation == M2_ACT_RELU ? (z > 0.f ? z : 0.f) : z);
    (void)hist;
}

// bf16, k == 4, W in {3, 4}, Cx % 8 == 0: one thread owns 8 consecutive channels, whose W-column histories are
// W*16 contiguous bytes; every access is a 16-byte vector, the 32 taps and 8 biases of the thread included (all loads
// are issued before any is used).
template <int W, typename WT>
__global__ void __launch_bounds__(256)
decode_conv_vec_kernel(const bf16_t* __restrict__ xBC, bf16_t* __restrict__ conv_state, const WT* __restrict__ w,
                       const WT* __restrict__ bias, float* __restrict__ act, int64_t nb, int64_t Cx, int64_t xsb, int activation) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;      // (b, c8)
    const int64_t C8 = Cx / 8;
    if (idx >= nb * C8) return;
    const int64_t b = idx / C8, c0 = (idx % C8) * 8;
    bf16_t* cs = conv_state + (b * Cx + c0) * W;
    uint4 raw[W];
#pragma unroll
    for (int i = 0; i < W; ++i) raw[i] = reinterpret_cast<const uint4*>(cs)[i];
    const uint4 xr = *reinterpret_cast<const uint4*>(xBC + b * xsb + c0);
    constexpr int PER = 16 / (int)sizeof(WT);            // parameters per 16-byte vector
    float wv[32], bv[8];
#pragma unroll
    for (int i = 0; i < 32 / PER; ++i) {
        float tmp[PER];
        load16<WT>(w + c0 * 4 + i * PER, tmp);
#pragma unroll
        for (int e = 0; e < PER; ++e) wv[i * PER + e] = tmp[e];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) bv[j] = 0.f;
    if (bias) {
#pragma unroll
        for (int i = 0; i < 8 / PER; ++i) {
            float tmp[PER];
            load16<WT>(bias + c0 + i * PER, tmp);
#pragma unroll
            for (int e = 0; e < PER; ++e) bv[i * PER + e] = tmp[e];
        }
    }
    const bf16_t* old = reinterpret_cast<const bf16_t*>(raw);                // [8 channels][W]
    const bf16_t* xin = reinterpret_cast<const bf16_t*>(&xr);
    uint4 nw[W];
    bf16_t* nst = reinterpret_cast<bf16_t*>(nw);
    float out[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        float z = bv[j];
#pragma unroll
        for (int i = 0; i < 3; ++i) z += wv[j * 4 + i] * to_f32(old[j * W + (W - 3) + i]);
        z += wv[j * 4 + 3] * to_f32(xin[j]);
#pragma unroll
        for (int i = 0; i + 1 < W; ++i) nst[j * W + i] = old[j * W + i + 1];
        nst[j * W + W - 1] = xin[j];
        out[j] = activation == M2_ACT_SILU ? silu_f(z) : (activation == M2_ACT_RELU ? (z > 0.f ? z : 0.f) : z);
    }
#pragma unroll
    for (int i = 0; i < W; ++i) reinterpret_cast<uint4*>(cs)[i] = nw[i];
    float* ap = act + b * Cx + c0;
    *reinterpret_cast<floatx4*>(ap) = floatx4{out[0], out[1], out[2], out[3]};
    *reinterpret_cast<floatx4*>(ap + 4) = floatx4{out[4], out[5], out[6], out[7]};
}

// VEC = 4: n % 4 == 0, float4 accesses; VEC = 1: any n.
// GL lanes (a power of two <= 64) share one state row; rows per pass = 256 / GL.
// sum over each group of GL adjacent lanes (GL a power of two, wave-uniform; all lanes active)
__device__ __forceinline__ float group_sum(float v, int GL) {
    if (GL > 32) v = lane_xor_add<32>(v);
    if (GL > 16) v = lane_xor_add<16>(v);
    if (GL > 8) v = lane_xor_add<8>(v);
    if (GL > 4) v = lane_xor_add<4>(v);
    if (GL > 2) v = lane_xor_add<2>(v);
    if (GL > 1) v = lane_xor_add<1>(v);
    return v;
}

template <typename T, int VEC>
__global__ void __launch_bounds__(256)
decode_ssm_kernel(float* __restrict__ S, const float* __restrict__ act, const T* __restrict__ dt, const float* __restrict__ A,
                  const float* __restrict__ D, const float* __restrict__ dt_bias, T* __restrict__ y, int64_t nheads, int P, int N,
                  int64_t ngroups, int64_t Cx, int64_t dtsb, int64_t ysb, int GL) {
    const int tid = threadIdx.x;
    const int64_t h = blockIdx.x, b = blockIdx.y;
    const int64_t g = h / (nheads / ngroups);
    const int64_t d_inner = nheads * P;
    const float* xa = act + b * Cx + h * P;
    const float* Ba = act + b * Cx + d_inner + g * N;
    const float* Ca = act + b * Cx + d_inner + ngroups * N + g * N;
    // with dt_bias, dt is the raw projection output and the step size is softplus(dt + dt_bias)  (mamba2_mixer.py:268)
    float dtv = to_f32(dt[b * dtsb + h]);
    if (dt_bias) dtv = softplus_f(dtv + dt_bias[h]);
    const float dA = __expf(A[h] * dtv);
    const float Dh = D ? D[h] : 0.f;
    float* Sp = S + (b * nheads + h) * (int64_t)P * N;
    const int sub = tid % GL, rowi = tid / GL, rows_per_pass = 256 / GL;
    const int nv = N / VEC;
    if (VEC == 4 && nv == GL && P % (rows_per_pass * kUP) == 0) {
        // fast path (n = 4 * GL): each lane owns one float4 per row; kUP rows are loaded before any is used
        const floatx4 bv = *reinterpret_cast<const floatx4*>(Ba + sub * 4);
        const floatx4 cv = *reinterpret_cast<const floatx4*>(Ca + sub * 4);
        for (int p0 = 0; p0 < P; p0 += rows_per_pass * kUP) {
            floatx4 sv[kUP];
            float xv[kUP];
#pragma unroll
            for (int u = 0; u < kUP; ++u) {
                const int pp = p0 + u * rows_per_pass + rowi;
                sv[u] = __builtin_nontemporal_load(reinterpret_cast<const floatx4*>(Sp + (int64_t)pp * N + sub * 4));
                xv[u] = xa[pp];
            }
#pragma unroll
            for (int u = 0; u < kUP; ++u) {
                const int pp = p0 + u * rows_per_pass + rowi;
                const float dx = dtv * xv[u];
                float part = 0.f;
#pragma unroll
                for (int q = 0; q < 4; ++q) { sv[u][q] = sv[u][q] * dA + dx * bv[q]; part += sv[u][q] * cv[q]; }
                __builtin_nontemporal_store(sv[u], reinterpret_cast<floatx4*>(Sp + (int64_t)pp * N + sub * 4));
                part = group_sum(part, GL);
                if (sub == 0) y[b * ysb + h * P + pp] = from_f32<T>(part + Dh * xv[u]);
            }
        }
        return;
    }
    for (int p0 = 0; p0 < P; p0 += rows_per_pass) {
        const int pp = p0 + rowi;
        float part = 0.f, xv = 0.f;
        if (pp < P) {
            xv = xa[pp];
            const float dx = dtv * xv;
            for (int j = sub; j < nv; j += GL) {
                if (VEC == 4) {
                    floatx4 s = *reinterpret_cast<const floatx4*>(Sp + (int64_t)pp * N + j * 4);
                    const floatx4 bv = *reinterpret_cast<const floatx4*>(Ba + j * 4);
                    const floatx4 cv = *reinterpret_cast<const floatx4*>(Ca + j * 4);
#pragma unroll
                    for (int q = 0; q < 4; ++q) { s[q] = s[q] * dA + dx * bv[q]; part += s[q] * cv[q]; }
                    *reinterpret_cast<floatx4*>(Sp + (int64_t)pp * N + j * 4) = s;
                } else {
                    float s = Sp[(int64_t)pp * N + j];
                    s = s * dA + dx * Ba[j];
                    part += s * Ca[j];
                    Sp[(int64_t)pp * N + j] = s;
                }
            }
        }
        part = group_sum(part, GL);
        if (pp < P && sub == 0) y[b * ysb + h * P + pp] = from_f32<T>(part + Dh * xv);
    }
}

}  // namespace
}  // namespace m2

extern "C" size_t m2_decode_workspace_bytes(int64_t batch, int64_t nheads, int64_t headdim, int64_t dstate, int64_t ngroups) {
    return (size_t)(batch * (nheads * headdim + 2 * ngroups * dstate)) * sizeof(float) + 16;
}

namespace m2 {
namespace {

// Scratch of the entry point that allocates nothing: the activated conv output of one step, held in the library's own
// device image (every GPU the library runs on holds its own copy until the process ends).
constexpr size_t kStaticScratchFloats = (size_t)1 << 20;          // 4 MiB: batch x conv channels <= 1 048 576
static __device__ __align__(256) float scratch[kStaticScratchFloats];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
float* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the CURRENT device, looked up once per device (the array's name is only a host-side
// handle: kernels and copies get this pointer).
int static_scratch(float** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return fail(M2_ERR_LAUNCH, "decode_step_static: hipGetDevice failed or device index %d out of range", dev);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            return fail(M2_ERR_LAUNCH, "decode_step_static: hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = static_cast<float*>(ptr);
    }
    *out = g_scratch_ptr[dev];
    return M2_OK;
}

int decode_step_impl(const m2_decode_params* p, float* act, size_t act_bytes, const char* who, void* stream);

}  // namespace
}  // namespace m2

extern "C" int m2_decode_step(const m2_decode_params* p, void* stream) {
    using namespace m2;
    M2_REQUIRE(p, M2_ERR_NULL, "decode_step: params is NULL");
    return decode_step_impl(p, static_cast<float*>(p->workspace), p->workspace_bytes, "decode_step", stream);
}

extern "C" int m2_decode_step_static(const m2_decode_params* p, void* stream) {
    using namespace m2;
    M2_REQUIRE(p, M2_ERR_NULL, "decode_step_static: params is NULL");
    // each factor is bounded by the scratch size before the channel count is formed, so that the products cannot overflow;
    // negative or zero dimensions fall through to the shared checks below
    const int64_t lim = (int64_t)kStaticScratchFloats;
    const bool sane = p->nheads >= 0 && p->headdim >= 0 && p->ngroups >= 0 && p->dstate >= 0 && p->batch >= 0;
    M2_REQUIRE(!sane || (p->nheads <= lim && p->headdim <= lim && p->ngroups <= lim && p->dstate <= lim && p->batch <= lim),
               M2_ERR_WORKSPACE, "decode_step_static: a dimension exceeds the built-in scratch of %zu floats; use m2_decode_step with a workspace",
               kStaticScratchFloats);
    const int64_t Cx = sane ? p->nheads * p->headdim + 2 * p->ngroups * p->dstate : 0;
    // sizes beyond the built-in scratch are refused here; every other check is the shared one below
    M2_REQUIRE(p->batch <= 0 || Cx <= 0 || (uint64_t)Cx <= kStaticScratchFloats / (uint64_t)p->batch, M2_ERR_WORKSPACE,
               "decode_step_static: batch %lld x %lld conv channels exceed the built-in scratch of %zu floats; use m2_decode_step with a workspace",
               (long long)p->batch, (long long)Cx, kStaticScratchFloats);
    float* act = nullptr;
    const int rc = static_scratch(&act);
    if (rc) return rc;
    return decode_step_impl(p, act, kStaticScratchFloats * sizeof(float), "decode_step_static", stream);
}

namespace m2 {
namespace {

int decode_step_impl(const m2_decode_params* p, float* act, size_t act_bytes, const char* who, void* stream) {
    M2_REQUIRE(p->dtype == M2_F32 || p->dtype == M2_BF16, M2_ERR_DTYPE, "%s: bad dtype %d", who, p->dtype);
    M2_REQUIRE(p->param_dtype == M2_F32 || p->param_dtype == M2_BF16, M2_ERR_DTYPE, "%s: bad param dtype %d", who, p->param_dtype);
    M2_REQUIRE(p->batch >= 0 && p->nheads >= 0 && p->headdim >= 1 && p->dstate >= 1, M2_ERR_SHAPE, "%s: bad dimension", who);
    M2_REQUIRE(p->ngroups >= 1 && p->nheads % p->ngroups == 0, M2_ERR_SHAPE, "decode_step: nheads %lld not divisible by ngroups %lld",
               (long long)p->nheads, (long long)p->ngroups);
    M2_REQUIRE(p->k >= 1 && p->k <= 8, M2_ERR_SHAPE, "%s: conv kernel size %d not in [1,8]", who, p->k);
    M2_REQUIRE(p->W >= p->k - 1 && p->W <= 8, M2_ERR_SHAPE, "%s: conv state width %d must be in [k-1, 8]", who, p->W);
    M2_REQUIRE(p->batch <= 65535, M2_ERR_SHAPE, "%s: batch exceeds the grid limit 65535", who);
    if (p->batch == 0 || p->nheads == 0) return M2_OK;
    M2_REQUIRE(p->xBC && p->conv_w && p->S && p->dt && p->A && p->y, M2_ERR_NULL, "%s: xBC, conv_w, S, dt, A, y are required", who);
    M2_REQUIRE(p->W == 0 || p->conv_state, M2_ERR_NULL, "%s: conv_state is required", who);
    const int64_t Cx = p->nheads * p->headdim + 2 * p->ngroups * p->dstate;
    const size_t need = (size_t)(p->batch * Cx) * sizeof(float);
    M2_REQUIRE(act && act_bytes >= need, M2_ERR_WORKSPACE, "%s: workspace %zu bytes < %zu needed", who, act_bytes, need);
    M2_REQUIRE(aligned16(act) && aligned16(p->S), M2_ERR_ALIGN, "%s: workspace and S must be 16-byte aligned", who);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int vec = (p->dstate % 4 == 0 && (p->nheads * p->headdim) % 4 == 0 && Cx % 4 == 0) ? 4 : 1;
    int GL = 1;
    while (GL < 64 && GL < p->dstate / vec) GL <<= 1;
    const bool vec_conv = p->dtype == M2_BF16 && p->k == 4 && (p->W == 3 || p->W == 4) && Cx % 8 == 0 &&
                          p->xBC_stride_b % 8 == 0 && aligned16(p->xBC) && aligned16(p->conv_state) && aligned16(p->conv_w) &&
                          aligned16(p->conv_b);
    if (vec_conv) {
        const unsigned blocks = (unsigned)ceil_div(p->batch * (Cx / 8), (int64_t)256);
        const bf16_t* xb = static_cast<const bf16_t*>(p->xBC);
        bf16_t* csb = static_cast<bf16_t*>(p->conv_state);
        auto go = [&](auto kern, auto wt_tag) {
            using WT = decltype(wt_tag);
            kern<<<blocks, 256, 0, st>>>(xb, csb, static_cast<const WT*>(p->conv_w), static_cast<const WT*>(p->conv_b), act, p->batch, Cx,
                                         p->xBC_stride_b, p->activation);
        };
        if (p->param_dtype == M2_F32) {
            if (p->W == 3) go(decode_conv_vec_kernel<3, float>, float{}); else go(decode_conv_vec_kernel<4, float>, float{});
        } else {
            if (p->W == 3) go(decode_conv_vec_kernel<3, bf16_t>, bf16_t{}); else go(decode_conv_vec_kernel<4, bf16_t>, bf16_t{});
        }
        int rc = check_launch("decode_conv_vec_kernel");
        if (rc) return rc;
    }
    M2_DISPATCH_DTYPE(p->dtype, T, {
        if (!vec_conv) decode_conv_kernel<T><<<(unsigned)ceil_div(p->batch * Cx, (int64_t)256), 256, 0, st>>>(
            static_cast<const T*>(p->xBC), static_cast<T*>(p->conv_state), p->conv_w, p->conv_b, act, p->batch, Cx, p->k, p->W,
            p->xBC_stride_b, p->param_dtype, p->activation);
        int rc2 = check_launch("decode_conv_kernel");
        if (rc2) return rc2;
        dim3 grid((unsigned)p->nheads, (unsigned)p->batch);
        if (vec == 4)
            decode_ssm_kernel<T, 4><<<grid, 256, 0, st>>>(p->S, act, static_cast<const T*>(p->dt), p->A, p->D, p->dt_bias, static_cast<T*>(p->y),
                                                          p->nheads, (int)p->headdim, (int)p->dstate, p->ngroups, Cx, p->dt_stride_b, p->y_stride_b, GL);
        else
            decode_ssm_kernel<T, 1><<<grid, 256, 0, st>>>(p->S, act, static_cast<const T*>(p->dt), p->A, p->D, p->dt_bias, static_cast<T*>(p->y),
                                                          p->nheads, (int)p->headdim, (int)p->dstate, p->ngroups, Cx, p->dt_stride_b, p->y_stride_b, GL);
        return check_launch("decode_ssm_kernel");
    });
    return M2_OK;
}

}  // namespace
}  // namespace m2
