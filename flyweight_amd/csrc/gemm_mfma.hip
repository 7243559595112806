// Tiled matrix product for prompts: out[M][N] = a[M][K] . w[N][K]^T, bfloat16 operands,
// float32 accumulation on the matrix cores (v_mfma_f32_32x32x16_bf16).
//
// A workgroup of four waves computes a 128 x 128 tile; each wave a 64 x 64 quarter as 2 x 2
// MFMA tiles. Both operands are k-contiguous, so a 128 x 64 slab of each is copied per
// iteration: global -> registers (issued before the multiply of the current slab) -> LDS
// (after it), two LDS buffers, one barrier per iteration. LDS rows are padded from 128 to
// 144 bytes so that the 16-byte operand reads of 16 consecutive rows fall into different
// banks. Workgroups are numbered so that each XCD (every eighth workgroup id) works on a
// compact group of tiles and finds its operands in its own L2.
//
// Epilogues: store (bfloat16 or float32), add into the float32 residual stream, or SwiGLU
// (w = gate rows then up rows; a workgroup takes 64 features of each, every wave holds gate
// and up of the same element in one lane, and silu(gate) * up is stored as bfloat16).
// The reference's prompt GEMM is a 64x64 tile of plain FMAs without tensor cores
// (native/include/flyweight_v2_native_kernels.hpp:233-311).
#include "fw_common.h"
#include "fw_kernels.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

#define TM 128
#define TN 128
#define TK 64
#define ROW_BYTES 144           // 64 bf16 + 16 bytes of padding
#define SLAB_BYTES (TM * ROW_BYTES)
#define GROUP_M 8

enum { MF_STORE = 0, MF_ACCUMULATE = 1, MF_SWIGLU = 2 };

__device__ __forceinline__ float silu_fast(float g) {
    if (g >= 0.0f) return g / (1.0f + __expf(-g));
    const float e = __expf(g);
    return g * e / (1.0f + e);
}

template <int MODE, typename TO>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(
    const uint16_t* __restrict__ a, const uint16_t* __restrict__ w, const float* __restrict__ bias,
    TO* __restrict__ out, int M, int N, int K, int tiles_m, int tiles_n, int per_xcd, int up_offset) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    // [buffer][operand][row][ROW_BYTES]
    const int total = tiles_m * tiles_n;
    const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (logical >= total) return;
    const int width = GROUP_M * tiles_n;
    const int group = logical / width;
    const int first_m = group * GROUP_M;
    const int group_size = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
    const int pid_m = first_m + (logical % width) % group_size;
    const int pid_n = (logical % width) / group_size;
    const int features = MODE == MF_SWIGLU ? TN / 2 : TN;
    const int m0 = pid_m * TM, n0 = pid_n * features;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // what this thread copies: chunks tid, tid + 256, ... of 1024 per operand; chunk c is
    // 16 bytes at (row c / 8, k 8 * (c % 8))
    const uint16_t* a_src[4];
    const uint16_t* w_src[4];
    int lds_at[4];
    const int kc = (tid & 7) * 8;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = (tid >> 3) + 32 * i;
        int am = m0 + row;
        am = am < M ? am : M - 1;                       // rows past the end are computed and dropped
        int wr;
        if (MODE == MF_SWIGLU) wr = row < 64 ? n0 + row : up_offset + n0 + row - 64;
        else wr = n0 + row;
        const int limit = MODE == MF_SWIGLU ? (row < 64 ? N : up_offset + N) : N;
        wr = wr < limit ? wr : limit - 1;
        a_src[i] = a + (size_t)am * K + kc;
        w_src[i] = w + (size_t)wr * K + kc;
        lds_at[i] = row * ROW_BYTES + (tid & 7) * 16;
    }

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    u32x4 ra[4], rw[4];
    const u32x4 zero = {0u, 0u, 0u, 0u};
    auto fetch = [&](int k0) {
        const bool ok = k0 + kc < K;                    // K is a multiple of 8
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            ra[i] = ok ? *reinterpret_cast<const u32x4*>(a_src[i] + k0) : zero;
            rw[i] = ok ? *reinterpret_cast<const u32x4*>(w_src[i] + k0) : zero;
        }
    };
    auto stash = [&](int buffer) {
        unsigned char* base = lds + buffer * 2 * SLAB_BYTES;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<u32x4*>(base + lds_at[i]) = ra[i];
            *reinterpret_cast<u32x4*>(base + SLAB_BYTES + lds_at[i]) = rw[i];
        }
    };

    const int a_row0 = wm * 64 + (lane & 31);
    int b_row[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
        b_row[j] = MODE == MF_SWIGLU ? j * 64 + wn * 32 + (lane & 31) : wn * 64 + j * 32 + (lane & 31);
    const int k_lane = (lane >> 5) * 16;                // byte offset of this lane's 8 k within a k16 step

    fetch(0);
    stash(0);
    __syncthreads();
    const int steps = (K + TK - 1) / TK;
    for (int step = 0; step < steps; ++step) {
        const int buffer = step & 1;
        if (step + 1 < steps) fetch((step + 1) * TK);
        const unsigned char* sa = lds + buffer * 2 * SLAB_BYTES;
        const unsigned char* sb = sa + SLAB_BYTES;
#pragma unroll
        for (int k16 = 0; k16 < TK / 16; ++k16) {
            bf16x8 fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                fa[i] = *reinterpret_cast<const bf16x8*>(sa + (a_row0 + 32 * i) * ROW_BYTES + k16 * 32 + k_lane);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                fb[j] = *reinterpret_cast<const bf16x8*>(sb + b_row[j] * ROW_BYTES + k16 * 32 + k_lane);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (step + 1 < steps) stash(buffer ^ 1);
        __syncthreads();
    }

    // D layout of the 32x32 product: lane holds column lane % 32; register r is row
    // 8 * (r / 4) + 4 * (lane / 32) + r % 4
    const int col = lane & 31, row_base = (lane >> 5) * 4;
    if (MODE == MF_SWIGLU) {
        const int n = n0 + wn * 32 + col;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + row_base + (r & 3);
                if (m < M && n < N)
                    store_from_float(out, (size_t)m * N + n, silu_fast(acc[i][0][r]) * acc[i][1][r]);
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int n = n0 + wn * 64 + j * 32 + col;
            if (n >= N) continue;
            const float b = bias ? bias[n] : 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + row_base + (r & 3);
                if (m >= M) continue;
                const size_t at = (size_t)m * N + n;
                float value = acc[i][j][r] + b;
                if (MODE == MF_ACCUMULATE) value += load_as_float(out, at);
                store_from_float(out, at, value);
            }
        }
}

template <int MODE, typename TO>
static int launch(const void* a, const void* w, const float* bias, void* out, int M, int N, int K, hipStream_t stream) {
    const int features = MODE == MF_SWIGLU ? TN / 2 : TN;
    const int tiles_m = fw_ceil_div(M, TM), tiles_n = fw_ceil_div(N, features);
    const int per_xcd = fw_ceil_div((long long)tiles_m * tiles_n, 8);
    const int lds_bytes = 2 * 2 * SLAB_BYTES;
    static bool configured = false;     // per instantiation
    if (!configured) {
        hipError_t status = hipFuncSetAttribute((const void*)gemm_mfma_kernel<MODE, TO>,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (status != hipSuccess) {
            fw_set_error("gemm_mfma: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(status));
            return -1;
        }
        configured = true;
    }
    gemm_mfma_kernel<MODE, TO><<<per_xcd * 8, 256, lds_bytes, stream>>>(
        (const uint16_t*)a, (const uint16_t*)w, bias, (TO*)out, M, N, K, tiles_m, tiles_n, per_xcd, N);
    return 0;
}

// mode 0: out = a . w^T (+ bias) stored as out_dtype; 1: out (float32) += a . w^T (+ bias);
// 2: w is [2 * N][K] (gate rows, then up rows); out [M][N] bfloat16 = silu(gate) * up.
extern "C" int fw_gemm_mfma(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                            int M, int N, int K, void* stream) {
    FW_REQUIRE(M >= 1 && N > 0 && K > 0 && K % 8 == 0, "gemm_mfma: K (%d) must be a positive multiple of 8; M=%d N=%d", K, M, N);
    FW_REQUIRE(mode >= 0 && mode <= 2, "gemm_mfma: unknown mode %d", mode);
    FW_REQUIRE(mode != MF_ACCUMULATE || out_dtype == FW_F32, "gemm_mfma: accumulation needs a float32 destination");
    FW_REQUIRE(mode != MF_SWIGLU || (out_dtype == FW_BF16 && bias == nullptr), "gemm_mfma: SwiGLU stores bfloat16 and takes no bias");
    FW_REQUIRE(out_dtype == FW_F32 || out_dtype == FW_BF16, "gemm_mfma: unknown out dtype %d", out_dtype);
    FW_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_mfma: operands must be 16-byte aligned");
    FW_REQUIRE((long long)fw_ceil_div(M, TM) * fw_ceil_div(N, TN / 2) < (1ll << 30), "gemm_mfma: too many tiles");
    hipStream_t s = (hipStream_t)stream;
    int status;
    if (mode == MF_SWIGLU) status = launch<MF_SWIGLU, bf16_t>(a, w, nullptr, out, M, N, K, s);
    else if (mode == MF_ACCUMULATE) status = launch<MF_ACCUMULATE, float>(a, w, bias, out, M, N, K, s);
    else if (out_dtype == FW_F32) status = launch<MF_STORE, float>(a, w, bias, out, M, N, K, s);
    else status = launch<MF_STORE, bf16_t>(a, w, bias, out, M, N, K, s);
    if (status != 0) return status;
    FW_LAUNCH_CHECK("gemm_mfma");
    return 0;
}
