/*
 * mamba2_hip.h -- C ABI of the MI355X (gfx950) Mamba-2 mixer hot path.
 *
 * One shared library, libmamba2_hip.so, exports the entry points below.  They
 * replace the device kernels of awslabs/state-space-models-neuron (NKI kernels
 * behind torch.autograd.Function wrappers; the reference has no FFI of its own,
 * so the "binding" a maintainer adds is a ctypes call from those wrappers):
 *
 *   m2_conv1d_fwd / m2_conv1d_bwd      <- mamba2/conv1d_grouped.py:66-125 (conv1d_with_transpose),
 *                                         :129-194 (conv1d_with_transpose_bwd), :198-262
 *                                         (conv1d_grouped_kernel_grad); wrappers :265-334
 *   m2_ssd_fwd / m2_ssd_bwd            <- mamba2/mamba2_kernel.py:67-170 (mamba_kernel_),
 *                                         :277-485 (mamba_kernel_bwd_); wrapper :488-519
 *   m2_decode_step                     <- mamba2/mamba2_kernel_inference.py:27-104
 *                                         (mamba_inference_kernel_); wrapper :107-122
 *   m2_softplus_bias_* / m2_rmsnorm_gated_*  <- mamba2/fused_kernel.py:33-175 (glue kernels of the
 *                                         fused mixer core)
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer owned by the caller (inputs, outputs and
 *     workspace).  The library never allocates, frees or synchronises.
 *   - Work is enqueued on `stream` (a hipStream_t; NULL = the default stream),
 *     asynchronously and stream-ordered.
 *   - Return value: M2_OK or a negative M2_ERR_* code; m2_last_error() returns a
 *     thread-local message for the last failing call on this thread.
 *   - Element strides are in ELEMENTS, the innermost dimension is contiguous
 *     unless a stride for it is given.  x, B, C may be views into a packed
 *     [x | B | C] or [z | x | B | C | dt] buffer (the reference packs them,
 *     mamba2_kernel.py:71,109-115).
 *   - Accumulation, cumulative sums, decays and SSM states are always fp32.
 */
#ifndef MAMBA2_HIP_H
#define MAMBA2_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define M2_OK 0
#define M2_ERR_SHAPE (-1)       /* a dimension is out of the supported set            */
#define M2_ERR_DTYPE (-2)       /* unknown / unsupported element type                 */
#define M2_ERR_ALIGN (-3)       /* pointer or stride not aligned for the vector path  */
#define M2_ERR_WORKSPACE (-4)   /* workspace missing or too small                     */
#define M2_ERR_LAUNCH (-5)      /* hipGetLastError() after a launch                   */
#define M2_ERR_NULL (-6)        /* a required pointer is NULL                         */

#define M2_F32 0
#define M2_BF16 1

#define M2_ACT_NONE 0
#define M2_ACT_SILU 1
#define M2_ACT_RELU 2

#define M2_CHUNK 128            /* SSD chunk length (block_size = 128, mamba2_kernel.py:78) */

/* ABI version of this header; bumped on any incompatible change. */
int m2_abi_version(void);
const char* m2_last_error(void);
/* Layout of a parameter structure as THIS library was compiled: out[0] = sizeof, out[1..] = offsetof each field in
 * declaration order.  which: 0 m2_conv1d_params, 1 m2_ssd_params, 2 m2_decode_params, 3 m2_rmsnorm_params.  Returns the
 * number of entries (only the first `capacity` are written); a binding compares them with its own mirror of the structs. */
int m2_struct_layout(int32_t which, int64_t* out, int32_t capacity);

/* ------------------------------------------------------------------ conv1d
 * y[b,t,c] = act(bias[c] + sum_{i<k} w[c,i] * x[b,t-(k-1)+i,c]),  x[t<0] = 0.
 * Either layout is a stride choice: channels-last (b,l,C): stride_c == 1;
 * channel-major (b,C,l) (ConvNKI's layout, conv1d_grouped.py:300-306): stride_l == 1.
 * k in [1, 8].  w is (C, k) contiguous (the (C,1,k) parameter), bias (C) or NULL.
 */
typedef struct m2_conv1d_params {
    const void* x; const void* w; const void* bias;   /* inputs                       */
    const void* dy;                                    /* bwd only                     */
    void* y;                                           /* fwd only                     */
    void* dx; void* dw; void* db;                      /* bwd only; db may be NULL     */
    void* workspace; size_t workspace_bytes;           /* bwd only                     */
    int64_t batch, seqlen, channels; int32_t k;
    int64_t x_stride_b, x_stride_l, x_stride_c;
    int64_t y_stride_b, y_stride_l, y_stride_c;        /* y (fwd) / dy (bwd)           */
    int64_t dx_stride_b, dx_stride_l, dx_stride_c;
    int32_t dtype;                                     /* x, y, dy, dx                 */
    int32_t param_dtype;                               /* w, bias, dw, db              */
    int32_t activation;
} m2_conv1d_params;

int m2_conv1d_fwd(const m2_conv1d_params* p, void* stream);
size_t m2_conv1d_bwd_workspace_bytes(int64_t batch, int64_t seqlen, int64_t channels, int32_t k);
int m2_conv1d_bwd(const m2_conv1d_params* p, void* stream);

/* ------------------------------------------------------------------ SSD scan
 * dt (b,l,h), A (h) fp32, x (b,l,h,p), B,C (b,l,g,n), D (h) fp32 or NULL,
 * initial_state / final_state (b,h,p,n) fp32 contiguous or NULL, y (b,l,h,p).
 * Supported: p in {64,128}, n in {64,128}, h % g == 0, any l >= 0, any b >= 0.
 * Alignment and strides (both dtypes; refused with M2_ERR_ALIGN / M2_ERR_SHAPE, never copied):
 *   - x, B, C, y and, in the backward, dy, dx, dB, dC: base pointer 16-byte aligned and every
 *     stride a multiple of 16 bytes (8 elements of bf16, 4 of fp32): rows are read and written as
 *     16-byte vectors, the gradients too (so a slice of a packed gradient buffer must start at a
 *     column that is a multiple of 8 / 4);
 *   - token strides (x, B, C, dt, y, dy, dx, dB, dC, ddt) in [0, 2^21) elements: row offsets inside
 *     a chunk are 32-bit sums of 24-bit products;
 *   - workspace 256-byte aligned, chunk_states 16-byte aligned; batch, nheads <= 65535.
 * Backward takes the same inputs plus dy (y is unused) and writes
 * dx, ddt, dB, dC in the dtype of the matching input and dA (h), dD (h) in fp32,
 * already summed over the batch (the reference sums them in its wrapper,
 * mamba2_kernel.py:514).
 * chunk_states (optional): an opaque buffer of m2_ssd_chunk_states_bytes() bytes, 16-byte aligned,
 * that carries what the backward can reuse from the forward: first the SSM state entering each
 * chunk, (b, ceil(l/128), h, p, n) elements of `dtype`, then the per-chunk decay tables and the
 * per-(chunk, group) C B^T operand tiles.  Forward: if non-NULL it is written there (otherwise
 * into the workspace).  Backward: if non-NULL it must hold what the forward wrote for the same
 * inputs and is read instead of being recomputed; with NULL the backward recomputes all of it
 * from the inputs, as the reference does (mamba2_kernel.py:363-367).
 * dt_bias (optional, (h) fp32): when given, `dt` holds the RAW projection output and the step
 * size is softplus(dt + dt_bias[h]) (threshold form, x for x >= 10), applied where the decay
 * tables are built -- the fused mixer core's softplus_with_bias (fused_kernel.py:33-47, called at
 * :273) without a pass of its own.  The backward then returns ddt w.r.t. the raw dt and
 * d_dt_bias (h) fp32 summed over batch and tokens (softplus_with_bias_bwd, :50-73).
 */
typedef struct m2_ssd_params {
    const void* x; const void* dt; const float* A; const void* B; const void* C; const float* D;
    const float* initial_state; float* final_state;
    void* chunk_states;                                 /* optional, see above          */
    void* y;                                            /* fwd: out; unused by bwd      */
    /* backward only */
    const void* dy; const float* d_final_state;
    void* dx; void* ddt; float* dA; void* dB; void* dC; float* dD; float* d_initial_state;
    void* workspace; size_t workspace_bytes;
    int64_t batch, seqlen, nheads, headdim, dstate, ngroups;
    int64_t x_stride_b, x_stride_l, x_stride_h;         /* x; innermost (p) contiguous  */
    int64_t dt_stride_b, dt_stride_l;                   /* dt; innermost (h) contiguous */
    int64_t B_stride_b, B_stride_l, B_stride_g;
    int64_t C_stride_b, C_stride_l, C_stride_g;
    int64_t y_stride_b, y_stride_l, y_stride_h;
    int64_t dy_stride_b, dy_stride_l, dy_stride_h;
    int64_t dx_stride_b, dx_stride_l, dx_stride_h;
    int64_t ddt_stride_b, ddt_stride_l;
    int64_t dB_stride_b, dB_stride_l, dB_stride_g;
    int64_t dC_stride_b, dC_stride_l, dC_stride_g;
    int32_t dtype;                                      /* x, B, C, y, dy, dx, dB, dC   */
    int32_t dt_dtype;                                   /* dt, ddt                      */
    const float* dt_bias;                               /* optional (h): see below      */
    float* d_dt_bias;                                   /* backward, with dt_bias: (h)  */
} m2_ssd_params;

size_t m2_ssd_chunk_states_bytes(const m2_ssd_params* p);
size_t m2_ssd_fwd_workspace_bytes(const m2_ssd_params* p);
int m2_ssd_fwd(const m2_ssd_params* p, void* stream);
size_t m2_ssd_bwd_workspace_bytes(const m2_ssd_params* p);
int m2_ssd_bwd(const m2_ssd_params* p, void* stream);

/* ------------------------------------------------------------------ decode step
 * One token per batch row; conv_state (b,Cx,W) and S (b,h,p,n) fp32 are updated
 * IN PLACE (the reference writes fresh copies and the caller re-binds them,
 * mamba2_mixer.py:275-276).  W is k-1 or k columns.  SiLU is applied to all of
 * [x | B | C] after the conv (mamba2_kernel_inference.py:14,69-90).
 * workspace: b*Cx floats (activated conv output).
 */
typedef struct m2_decode_params {
    const void* xBC; void* conv_state; const void* conv_w; const void* conv_b;
    float* S; const void* dt; const float* A; const float* D; void* y;
    void* workspace; size_t workspace_bytes;
    int64_t batch, nheads, headdim, dstate, ngroups; int32_t k, W;
    int64_t xBC_stride_b, dt_stride_b, y_stride_b;
    int32_t dtype;                                      /* xBC, conv_state, dt, y       */
    int32_t param_dtype;                                /* conv_w, conv_b               */
    int32_t activation;
    const float* dt_bias;                               /* (h) or NULL.  Given: dt holds the raw projection output and the
                                                           step size is softplus(dt + dt_bias), threshold form
                                                           (mamba2/mamba2_mixer.py:268), applied inside in fp32            */
} m2_decode_params;

size_t m2_decode_workspace_bytes(int64_t batch, int64_t nheads, int64_t headdim, int64_t dstate, int64_t ngroups);
int m2_decode_step(const m2_decode_params* p, void* stream);

/* m2_decode_step for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc): the same kernels, same inputs and outputs, but the step's scratch -- the activated conv output,
 * batch x (nheads*headdim + 2*ngroups*dstate) floats -- lives in a 4 MiB array inside the library's device image
 * instead of a caller workspace; p->workspace and p->workspace_bytes are ignored.  No counterpart in the reference
 * (its decode kernel allocates fresh outputs per call, mamba2_kernel_inference.py:114-116).
 *   - limit: batch x conv channels <= 1 048 576 (batch 195 at the 2.7B width); beyond it M2_ERR_WORKSPACE.
 *   - allocates nothing; the array's device address is looked up on the first call per device (make that first call
 *     outside a graph capture).  The CURRENT device (hipGetDevice) must be the one `stream` belongs to: the address is
 *     kept per current-device index.  Each GPU holds its own 4 MiB copy until the process ends.
 *   - all calls on one GPU share that array: calls that overlap on one GPU (two streams, two threads) race; calls on
 *     one stream, or otherwise ordered, are safe.  Nothing in it has to start at zero (every call overwrites what it reads). */
int m2_decode_step_static(const m2_decode_params* p, void* stream);

/* ------------------------------------------------------------------ mixer glue
 * The elementwise passes between the conv, the scan and the output projection
 * (mamba2/fused_kernel.py:33-47 softplus_with_bias, :50-73 softplus_with_bias_bwd,
 * :76-103 rmsnorm, :127-175 rmsnorm_bwd; torch twins mamba2/mamba2_mixer.py:36-38, 88-105).
 * Rows are (batch x token) pairs; the channel dimension is contiguous, rows may be strided
 * (columns of the packed [z | xBC | dt] projection output and of its gradient).
 *
 * softplus:  out = softplus(dt + dt_bias[h]) in the threshold form (x for x >= 10);
 *            d_in = d_out * sigmoid(dt + dt_bias) (1 above the threshold), d_bias[h] = sum over rows, fp32.
 * rmsnorm:   h = x * silu(z) (h = x without z);  out = weight * h * rsqrt(mean(h^2) + eps) with the mean
 *            taken inside each of n_groups groups of channels / n_groups contiguous channels.
 *            Backward: dx, dz (same type as x) and d_weight (fp32, summed over the rows).
 *            Channels per group: a multiple of 8 (bf16) / 4 (fp32), at most 8192.
 * dt_bias, weight, d_bias, d_weight are fp32.  The backward entry points take a workspace of
 * m2_*_bwd_workspace_bytes() bytes (per-block partial sums, added in a fixed order: no atomics).
 */
int m2_softplus_bias_fwd(const void* dt, int64_t dt_stride_row, const float* dt_bias, void* out, int64_t out_stride_row,
                         int64_t rows, int64_t nheads, int32_t dtype, void* stream);
size_t m2_softplus_bias_bwd_workspace_bytes(int64_t rows, int64_t nheads);
int m2_softplus_bias_bwd(const void* dt, int64_t dt_stride_row, const float* dt_bias, const void* d_out, int64_t d_out_stride_row,
                         void* d_in, int64_t d_in_stride_row, float* d_bias, void* workspace, size_t workspace_bytes,
                         int64_t rows, int64_t nheads, int32_t dtype, void* stream);

typedef struct m2_rmsnorm_params {
    const void* x; const void* z;                       /* (rows, channels); z may be NULL (no gate)   */
    const float* weight;                                /* (channels)                                   */
    void* out;                                          /* forward: (rows, channels)                    */
    const void* d_out; void* dx; void* dz;              /* backward; dz required when z is given        */
    float* d_weight;                                    /* backward: (channels) fp32                    */
    void* workspace; size_t workspace_bytes;            /* backward only                                */
    int64_t rows, channels;
    int64_t x_stride_row, z_stride_row, out_stride_row, d_out_stride_row, dx_stride_row, dz_stride_row;
    int32_t n_groups;
    int32_t dtype;                                      /* x, z, d_out, dx, dz (and out unless out_f32) */
    int32_t out_f32;                                    /* forward output in fp32 (mamba2_mixer.py:104-105) */
    float eps;
} m2_rmsnorm_params;

int m2_rmsnorm_gated_fwd(const m2_rmsnorm_params* p, void* stream);
size_t m2_rmsnorm_gated_bwd_workspace_bytes(int64_t rows, int64_t channels, int32_t n_groups, int32_t dtype);
int m2_rmsnorm_gated_bwd(const m2_rmsnorm_params* p, void* stream);

/* Block boundary of the token-by-token loop (mamba2/modeling_mamba2.py:133-140 Mamba2Block.step's residual add,
 * followed by the next block's -- or the final -- Mamba2RMSNorm, :94-103), in one pass over the rows:
 *   residual += delta;   out = weight * residual * rsqrt(mean(residual^2) + eps)
 * residual (rows, channels) fp32, updated in place (the fp32 residual stream, residual_in_fp32);
 * delta (rows, channels) in `dtype`, or NULL (nothing to add: first block); out (rows, channels) in `dtype`; weight fp32.
 * channels: a multiple of 4, at most 8192.  Inference only (no backward). */
int m2_add_rmsnorm(float* residual, int64_t residual_stride_row, const void* delta, int64_t delta_stride_row,
                   const float* weight, void* out, int64_t out_stride_row, int64_t rows, int64_t channels, float eps,
                   int32_t dtype, void* stream);

/* ------------------------------------------------------------------ self tests / probes
 * m2_mfma_selftest: C (M x N fp32, row-major) = A (M x K) * Bt (N x K)^T through the same
 * LDS-staged MFMA tile code the SSD kernels use.  M, N multiples of 128; K multiple of 32.
 * m2_stream_copy: plain copy kernel of `bytes` bytes (multiple of 16), for calibrating
 * bandwidth counters and the achievable-HBM figure.
 * m2_tile_walk: the access pattern of the SSD kernels without their arithmetic.  src is a (batch, rows, row_bytes)
 * array; it is read as tiles of 128 rows x piece_bytes (64, 128, 256 or 512: half a head, a head, two, four heads of a
 * (b, l, h, p) tensor with 128-byte heads) and tile (b, t, u) is written as one contiguous block at
 * dst + ((b * rows / 128 + t) * (row_bytes / piece_bytes) + u) * 128 * piece_bytes.  in_order != 0: one workgroup per
 * (b, u) takes its tiles in order, two loads ahead (the state passes' shape); 0: one workgroup per tile.  rows a multiple
 * of 128, row_bytes a multiple of piece_bytes; dst has the size of src.  Neither has a counterpart in the reference:
 * they give the rate that the memory system allows a kernel with these streams.
 */
int m2_mfma_selftest(const void* A, const void* Bt, float* C, int64_t M, int64_t N, int64_t K, int32_t dtype, void* stream);
int m2_stream_copy(const void* src, void* dst, size_t bytes, void* stream);
int m2_tile_walk(const void* src, void* dst, int64_t batch, int64_t rows, int64_t row_bytes, int64_t piece_bytes,
                 int32_t in_order, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MAMBA2_HIP_H */
