// Generic matrix product out[M][N] = a[M][K] . w[N][K]^T (+ bias) in float32 arithmetic.
// It serves the true 32-bit path (float32 operands, plain FMA, no reduced-precision matrix
// mode) and every operand mix the fast kernels do not take. Each output element is summed
// over k = 0..K-1 in order by one thread, so its value does not depend on M or on which
// tile it falls in. The reference's prefill GEMM has the same shape: a 64x64 tile, 4x4
// outputs per thread, k-step 16 (native/include/flyweight_v2_native_kernels.hpp:233-311).
#include "fw_common.h"
#include "fw_kernels.h"

#define GT 64   // tile edge
#define GK 16   // k step

template <typename TA, typename TW, typename TO, int MODE>
__global__ __launch_bounds__(256) void gemm_generic_kernel(
    const TA* __restrict__ a, const TW* __restrict__ w, const float* __restrict__ bias,
    TO* __restrict__ out, int M, int N, int K) {
    __shared__ float tile_a[GK][GT + 1];
    __shared__ float tile_w[GK][GT + 1];
    const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;   // 16 x 16 threads, 4 x 4 outputs each
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += GK) {
        // 64 rows x 16 k per operand = 1024 elements, 4 per thread
        for (int e = threadIdx.x; e < GT * GK; e += 256) {
            const int r = e / GK, kk = e % GK;
            const int k = k0 + kk;
            tile_a[kk][r] = (m0 + r < M && k < K) ? load_as_float(a, (size_t)(m0 + r) * K + k) : 0.0f;
            tile_w[kk][r] = (n0 + r < N && k < K) ? load_as_float(w, (size_t)(n0 + r) * K + k) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GK; ++kk) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = tile_a[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = tile_w[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float value = acc[i][j];
            if (bias) value += bias[n];
            const size_t at = (size_t)m * N + n;
            if (MODE == 1) value += load_as_float(out, at);
            store_from_float(out, at, value);
        }
    }
}

template <typename TA, typename TW>
static int launch(const void* a, const void* w, const float* bias, void* out, int out_dtype, int out_mode,
                  int M, int N, int K, hipStream_t stream) {
    dim3 grid(fw_ceil_div(N, GT), fw_ceil_div(M, GT));
    if (out_mode == 1) {
        gemm_generic_kernel<TA, TW, float, 1><<<grid, 256, 0, stream>>>((const TA*)a, (const TW*)w, bias, (float*)out, M, N, K);
    } else if (out_dtype == FW_F32) {
        gemm_generic_kernel<TA, TW, float, 0><<<grid, 256, 0, stream>>>((const TA*)a, (const TW*)w, bias, (float*)out, M, N, K);
    } else {
        gemm_generic_kernel<TA, TW, bf16_t, 0><<<grid, 256, 0, stream>>>((const TA*)a, (const TW*)w, bias, (bf16_t*)out, M, N, K);
    }
    return 0;
}

extern "C" int fw_gemm_generic(const void* a, int a_dtype, const void* w, int w_dtype, const float* bias,
                               void* out, int out_dtype, int out_mode, int M, int N, int K, void* stream) {
    FW_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    FW_REQUIRE(out_mode == 0 || out_mode == 1, "gemm: unknown out mode %d", out_mode);
    FW_REQUIRE(out_mode == 0 || out_dtype == FW_F32, "gemm: accumulation needs a float32 destination");
    FW_REQUIRE(out_dtype == FW_F32 || out_dtype == FW_BF16, "gemm: unknown out dtype %d", out_dtype);
    FW_REQUIRE(fw_ceil_div(M, GT) <= 65535, "gemm: too many rows (%d)", M);
    if (M == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (a_dtype == FW_F32 && w_dtype == FW_F32) launch<float, float>(a, w, bias, out, out_dtype, out_mode, M, N, K, s);
    else if (a_dtype == FW_BF16 && w_dtype == FW_BF16) launch<bf16_t, bf16_t>(a, w, bias, out, out_dtype, out_mode, M, N, K, s);
    else if (a_dtype == FW_BF16 && w_dtype == FW_F32) launch<bf16_t, float>(a, w, bias, out, out_dtype, out_mode, M, N, K, s);
    else if (a_dtype == FW_F32 && w_dtype == FW_BF16) launch<float, bf16_t>(a, w, bias, out, out_dtype, out_mode, M, N, K, s);
    else FW_REQUIRE(false, "gemm: unknown operand dtypes %d, %d", a_dtype, w_dtype);
    FW_LAUNCH_CHECK("gemm_generic");
    return 0;
}
