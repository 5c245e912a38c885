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

__global__ void __launch_bounds__(256) stream_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

}  // namespace
}  // namespace m2

extern "C" int m2_abi_version(void) { return 3; }
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
    size_t blocks = (n + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    stream_copy_kernel<<<(unsigned)blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<const uint4*>(src), static_cast<uint4*>(dst), n);
    return check_launch("stream_copy");
}
