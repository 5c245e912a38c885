// Error handling, ABI version and small probe kernels of libmamba2_hip.so.
#include "mma.hpp"

namespace m2 {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(M2_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return M2_OK;
}

namespace {

// C[M][N] = A[M][K] * Bt[N][K]^T through stage_rows + wave_mma; block = one 128x128 tile, 256 threads.
template <typename T>
__global__ void __launch_bounds__(256)
mfma_selftest_kernel(const T* __restrict__ A, const T* __restrict__ Bt, float* __restrict__ C, int64_t N, int64_t K) {
    constexpr int KB = 32;
    constexpr int LD = lds_ld<T>(KB);
    __shared__ __align__(16) T sA[128 * LD];
    __shared__ __align__(16) T sB[128 * LD];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t m0 = (int64_t)blockIdx.y * 128, n0 = (int64_t)blockIdx.x * 128;
    floatx16 acc[2][2];
    acc_zero(acc);
    for (int64_t k0 = 0; k0 < K; k0 += KB) {
        stage_rows<T, 128, KB, 256, false>(sA, LD, A + m0 * K + k0, K, 128, nullptr, tid);
        stage_rows<T, 128, KB, 256, false>(sB, LD, Bt + n0 * K + k0, K, 128, nullptr, tid);
        __syncthreads();
        wave_mma<2, 2>(acc, sA + wm * 64 * LD, LD, sB + wn * 64 * LD, LD, 0, KB);
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int64_t row = m0 + wm * 64 + i * 32 + acc_row(lane, v);
                const int64_t col = n0 + wn * 64 + j * 32 + acc_col(lane);
                C[row * N + col] = acc[i][j][v];
            }
}

// The HBM streams of the SSD kernels without their arithmetic: a (batch, rows, row_bytes) array is read as tiles of 128
// rows x `16 PPR` bytes (the rows of one head, or of half a head or of two, of a (b, l, h, p) tensor: short pieces a whole
// row apart) and every tile is written out as one contiguous block.  IN_ORDER: one workgroup per (batch, column of
// tiles) takes its tiles one after the other, loading two tiles ahead, as the state passes do; otherwise one workgroup
// per tile, as in the chunk-parallel kernels.
template <int PPR, bool IN_ORDER>
__global__ void __launch_bounds__(256) tile_walk_kernel(const char* __restrict__ src, char* __restrict__ dst, int tiles_down, int64_t row_bytes) {
    constexpr int ROWS = 128, NX = ROWS * PPR / 256;      // 16-byte pieces per thread per tile
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const int u = blockIdx.x, units = gridDim.x, tid = threadIdx.x;
    const int64_t b = IN_ORDER ? blockIdx.y : blockIdx.y / tiles_down;
    const int first = IN_ORDER ? 0 : (int)(blockIdx.y % tiles_down), count = IN_ORDER ? tiles_down : 1;
    const char* base = src + b * tiles_down * ROWS * row_bytes + (int64_t)u * (PPR * 16);
    auto load = [&](int t, u32x4* v) {
        if (t >= first + count) return;
#pragma unroll
        for (int i = 0; i < NX; ++i) {
            const int piece = tid + i * 256, row = piece / PPR, slot = piece % PPR;
            v[i] = *reinterpret_cast<const u32x4*>(base + ((int64_t)t * ROWS + row) * row_bytes + slot * 16);
        }
    };
    auto store = [&](int t, const u32x4* v) {
        char* o = dst + ((b * tiles_down + t) * units + u) * (int64_t)(ROWS * PPR * 16);
#pragma unroll
        for (int i = 0; i < NX; ++i) *reinterpret_cast<u32x4*>(o + (tid + i * 256) * 16) = v[i];
    };
    u32x4 s0[NX], s1[NX];
    load(first, s0);
    if (count > 1) load(first + 1, s1);
    for (int t = first; t < first + count; t += 2) {
        store(t, s0);
        load(t + 2, s0);
        if (t + 1 < first + count) {
            store(t + 1, s1);
            load(t + 3, s1);
        }
    }
}

// A workgroup copies blocks of 256 x 4 vectors: four 16-byte loads in flight per lane, each a whole 4 KiB run per wave
// pair, streamed past the caches on both sides (nothing is read twice).
__global__ void __launch_bounds__(256) stream_copy_kernel(const floatx4* __restrict__ src, floatx4* __restrict__ dst, size_t n) {
    constexpr size_t kBlock = 256 * 4;
    const size_t nblk = n / kBlock;
    for (size_t b = blockIdx.x; b < nblk; b += gridDim.x) {
        const floatx4* s = src + b * kBlock + threadIdx.x;
        floatx4* d = dst + b * kBlock + threadIdx.x;
        floatx4 v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = __builtin_nontemporal_load(s + q * 256);
#pragma unroll
        for (int q = 0; q < 4; ++q) __builtin_nontemporal_store(v[q], d + q * 256);
    }
    if (blockIdx.x == 0)
        for (size_t i = nblk * kBlock + threadIdx.x; i < n; i += 256) dst[i] = src[i];
}

#define M2_OFF(s, f) (int64_t)offsetof(s, f)
static const int64_t k_layout_0[] = {(int64_t)sizeof(m2_conv1d_params),
    M2_OFF(m2_conv1d_params, x), M2_OFF(m2_conv1d_params, w), M2_OFF(m2_conv1d_params, bias), M2_OFF(m2_conv1d_params, dy),
    M2_OFF(m2_conv1d_params, y), M2_OFF(m2_conv1d_params, dx), M2_OFF(m2_conv1d_params, dw), M2_OFF(m2_conv1d_params, db),
    M2_OFF(m2_conv1d_params, workspace), M2_OFF(m2_conv1d_params, workspace_bytes), M2_OFF(m2_conv1d_params, batch),
    M2_OFF(m2_conv1d_params, seqlen), M2_OFF(m2_conv1d_params, channels), M2_OFF(m2_conv1d_params, k),
    M2_OFF(m2_conv1d_params, x_stride_b), M2_OFF(m2_conv1d_params, x_stride_l), M2_OFF(m2_conv1d_params, x_stride_c),
    M2_OFF(m2_conv1d_params, y_stride_b), M2_OFF(m2_conv1d_params, y_stride_l), M2_OFF(m2_conv1d_params, y_stride_c),
    M2_OFF(m2_conv1d_params, dx_stride_b), M2_OFF(m2_conv1d_params, dx_stride_l), M2_OFF(m2_conv1d_params, dx_stride_c),
    M2_OFF(m2_conv1d_params, dtype), M2_OFF(m2_conv1d_params, param_dtype), M2_OFF(m2_conv1d_params, activation),};
static const int64_t k_layout_1[] = {(int64_t)sizeof(m2_ssd_params),
    M2_OFF(m2_ssd_params, x), M2_OFF(m2_ssd_params, dt), M2_OFF(m2_ssd_params, A), M2_OFF(m2_ssd_params, B),
    M2_OFF(m2_ssd_params, C), M2_OFF(m2_ssd_params, D), M2_OFF(m2_ssd_params, initial_state), M2_OFF(m2_ssd_params, final_state),
    M2_OFF(m2_ssd_params, chunk_states), M2_OFF(m2_ssd_params, y), M2_OFF(m2_ssd_params, dy),
    M2_OFF(m2_ssd_params, d_final_state), M2_OFF(m2_ssd_params, dx), M2_OFF(m2_ssd_params, ddt), M2_OFF(m2_ssd_params, dA),
    M2_OFF(m2_ssd_params, dB), M2_OFF(m2_ssd_params, dC), M2_OFF(m2_ssd_params, dD), M2_OFF(m2_ssd_params, d_initial_state),
    M2_OFF(m2_ssd_params, workspace), M2_OFF(m2_ssd_params, workspace_bytes), M2_OFF(m2_ssd_params, batch),
    M2_OFF(m2_ssd_params, seqlen), M2_OFF(m2_ssd_params, nheads), M2_OFF(m2_ssd_params, headdim), M2_OFF(m2_ssd_params, dstate),
    M2_OFF(m2_ssd_params, ngroups), M2_OFF(m2_ssd_params, x_stride_b), M2_OFF(m2_ssd_params, x_stride_l),
    M2_OFF(m2_ssd_params, x_stride_h), M2_OFF(m2_ssd_params, dt_stride_b), M2_OFF(m2_ssd_params, dt_stride_l),
    M2_OFF(m2_ssd_params, B_stride_b), M2_OFF(m2_ssd_params, B_stride_l), M2_OFF(m2_ssd_params, B_stride_g),
    M2_OFF(m2_ssd_params, C_stride_b), M2_OFF(m2_ssd_params, C_stride_l), M2_OFF(m2_ssd_params, C_stride_g),
    M2_OFF(m2_ssd_params, y_stride_b), M2_OFF(m2_ssd_params, y_stride_l), M2_OFF(m2_ssd_params, y_stride_h),
    M2_OFF(m2_ssd_params, dy_stride_b), M2_OFF(m2_ssd_params, dy_stride_l), M2_OFF(m2_ssd_params, dy_stride_h),
    M2_OFF(m2_ssd_params, dx_stride_b), M2_OFF(m2_ssd_params, dx_stride_l), M2_OFF(m2_ssd_params, dx_stride_h),
    M2_OFF(m2_ssd_params, ddt_stride_b), M2_OFF(m2_ssd_params, ddt_stride_l), M2_OFF(m2_ssd_params, dB_stride_b),
    M2_OFF(m2_ssd_params, dB_stride_l), M2_OFF(m2_ssd_params, dB_stride_g), M2_OFF(m2_ssd_params, dC_stride_b),
    M2_OFF(m2_ssd_params, dC_stride_l), M2_OFF(m2_ssd_params, dC_stride_g), M2_OFF(m2_ssd_params, dtype),
    M2_OFF(m2_ssd_params, dt_dtype), M2_OFF(m2_ssd_params, dt_bias), M2_OFF(m2_ssd_params, d_dt_bias),};
static const int64_t k_layout_2[] = {(int64_t)sizeof(m2_decode_params),
    M2_OFF(m2_decode_params, xBC), M2_OFF(m2_decode_params, conv_state), M2_OFF(m2_decode_params, conv_w),
    M2_OFF(m2_decode_params, conv_b), M2_OFF(m2_decode_params, S), M2_OFF(m2_decode_params, dt), M2_OFF(m2_decode_params, A),
    M2_OFF(m2_decode_params, D), M2_OFF(m2_decode_params, y), M2_OFF(m2_decode_params, workspace),
    M2_OFF(m2_decode_params, workspace_bytes), M2_OFF(m2_decode_params, batch), M2_OFF(m2_decode_params, nheads),
    M2_OFF(m2_decode_params, headdim), M2_OFF(m2_decode_params, dstate), M2_OFF(m2_decode_params, ngroups),
    M2_OFF(m2_decode_params, k), M2_OFF(m2_decode_params, W), M2_OFF(m2_decode_params, xBC_stride_b),
    M2_OFF(m2_decode_params, dt_stride_b), M2_OFF(m2_decode_params, y_stride_b), M2_OFF(m2_decode_params, dtype),
    M2_OFF(m2_decode_params, param_dtype), M2_OFF(m2_decode_params, activation), M2_OFF(m2_decode_params, dt_bias),};
static const int64_t k_layout_3[] = {(int64_t)sizeof(m2_rmsnorm_params),
    M2_OFF(m2_rmsnorm_params, x), M2_OFF(m2_rmsnorm_params, z), M2_OFF(m2_rmsnorm_params, weight),
    M2_OFF(m2_rmsnorm_params, out), M2_OFF(m2_rmsnorm_params, d_out), M2_OFF(m2_rmsnorm_params, dx),
    M2_OFF(m2_rmsnorm_params, dz), M2_OFF(m2_rmsnorm_params, d_weight), M2_OFF(m2_rmsnorm_params, workspace),
    M2_OFF(m2_rmsnorm_params, workspace_bytes), M2_OFF(m2_rmsnorm_params, rows), M2_OFF(m2_rmsnorm_params, channels),
    M2_OFF(m2_rmsnorm_params, x_stride_row), M2_OFF(m2_rmsnorm_params, z_stride_row), M2_OFF(m2_rmsnorm_params, out_stride_row),
    M2_OFF(m2_rmsnorm_params, d_out_stride_row), M2_OFF(m2_rmsnorm_params, dx_stride_row),
    M2_OFF(m2_rmsnorm_params, dz_stride_row), M2_OFF(m2_rmsnorm_params, n_groups), M2_OFF(m2_rmsnorm_params, dtype),
    M2_OFF(m2_rmsnorm_params, out_f32), M2_OFF(m2_rmsnorm_params, eps),};
#undef M2_OFF

}  // namespace
}  // namespace m2

extern "C" int m2_abi_version(void) { return 4; }

extern "C" int m2_struct_layout(int32_t which, int64_t* out, int32_t capacity) {
    using namespace m2;
    const int64_t* tab = nullptr;
    int n = 0;
    switch (which) {
        case 0: tab = k_layout_0; n = (int)(sizeof(k_layout_0) / sizeof(int64_t)); break;
        case 1: tab = k_layout_1; n = (int)(sizeof(k_layout_1) / sizeof(int64_t)); break;
        case 2: tab = k_layout_2; n = (int)(sizeof(k_layout_2) / sizeof(int64_t)); break;
        case 3: tab = k_layout_3; n = (int)(sizeof(k_layout_3) / sizeof(int64_t)); break;
        default: return fail(M2_ERR_SHAPE, "struct_layout: unknown structure %d", (int)which);
    }
    for (int i = 0; i < n && i < capacity; ++i) out[i] = tab[i];
    return n;
}
extern "C" const char* m2_last_error(void) { return m2::g_err; }

extern "C" int m2_mfma_selftest(const void* A, const void* Bt, float* C, int64_t M, int64_t N, int64_t K, int32_t dtype, void* stream) {
    using namespace m2;
    M2_REQUIRE(A && Bt && C, M2_ERR_NULL, "mfma_selftest: NULL pointer");
    M2_REQUIRE(M > 0 && N > 0 && K > 0 && M % 128 == 0 && N % 128 == 0 && K % 32 == 0, M2_ERR_SHAPE,
               "mfma_selftest: M, N must be multiples of 128 and K of 32");
    M2_REQUIRE(aligned16(A) && aligned16(Bt), M2_ERR_ALIGN, "mfma_selftest: operands must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    dim3 grid((unsigned)(N / 128), (unsigned)(M / 128));
    if (dtype == M2_F32) mfma_selftest_kernel<float><<<grid, 256, 0, st>>>(static_cast<const float*>(A), static_cast<const float*>(Bt), C, N, K);
    else if (dtype == M2_BF16) mfma_selftest_kernel<bf16_t><<<grid, 256, 0, st>>>(static_cast<const bf16_t*>(A), static_cast<const bf16_t*>(Bt), C, N, K);
    else return fail(M2_ERR_DTYPE, "mfma_selftest: bad dtype %d", dtype);
    return check_launch("mfma_selftest");
}

extern "C" int m2_stream_copy(const void* src, void* dst, size_t bytes, void* stream) {
    using namespace m2;
    M2_REQUIRE(src && dst, M2_ERR_NULL, "stream_copy: NULL pointer");
    M2_REQUIRE(bytes % 16 == 0 && aligned16(src) && aligned16(dst), M2_ERR_ALIGN, "stream_copy: size and pointers must be multiples of 16 bytes");
    if (bytes == 0) return M2_OK;
    const size_t n = bytes / 16;
    size_t blocks = (n + 1023) / 1024;
    if (blocks > 256 * 32) blocks = 256 * 32;
    stream_copy_kernel<<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<const floatx4*>(src), static_cast<floatx4*>(dst), n);
    return check_launch("stream_copy");
}

extern "C" int m2_tile_walk(const void* src, void* dst, int64_t batch, int64_t rows, int64_t row_bytes, int64_t piece_bytes,
                            int32_t in_order, void* stream) {
    using namespace m2;
    M2_REQUIRE(src && dst, M2_ERR_NULL, "tile_walk: NULL pointer");
    M2_REQUIRE(aligned16(src) && aligned16(dst), M2_ERR_ALIGN, "tile_walk: pointers must be multiples of 16 bytes");
    M2_REQUIRE(batch >= 1 && rows >= 128 && rows % 128 == 0 && row_bytes >= piece_bytes && row_bytes % piece_bytes == 0, M2_ERR_SHAPE,
               "tile_walk: rows must be a multiple of 128 and row_bytes a multiple of piece_bytes (got rows %lld, row_bytes %lld, piece_bytes %lld)",
               (long long)rows, (long long)row_bytes, (long long)piece_bytes);
    const int64_t tiles_down = rows / 128, units = row_bytes / piece_bytes, gy = in_order ? batch : batch * tiles_down;
    M2_REQUIRE(units <= 0x7fffffff && gy <= 65535 && tiles_down <= 0x7fffffff, M2_ERR_SHAPE, "tile_walk: grid too large");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)units, (unsigned)gy);
    const char* s = static_cast<const char*>(src);
    char* d = static_cast<char*>(dst);
#define M2_WALK(PPR) \
    do { if (in_order) tile_walk_kernel<PPR, true><<<grid, 256, 0, st>>>(s, d, (int)tiles_down, row_bytes); \
         else tile_walk_kernel<PPR, false><<<grid, 256, 0, st>>>(s, d, (int)tiles_down, row_bytes); } while (0)
    switch (piece_bytes) {
        case 64: M2_WALK(4); break;
        case 128: M2_WALK(8); break;
        case 256: M2_WALK(16); break;
        case 512: M2_WALK(32); break;
        default: return fail(M2_ERR_SHAPE, "tile_walk: piece_bytes must be 64, 128, 256 or 512 (got %lld)", (long long)piece_bytes);
    }
#undef M2_WALK
    return check_launch("tile_walk");
}
