// Skinny matrix product for decode: out[M][N] = a[M][K] . w[N][K]^T with few rows (M <= 64),
// bfloat16 operands, float32 accumulation on the matrix cores. The step is bound by reading
// W once from HBM, so the kernel is shaped around that stream:
//
//  * a workgroup owns 16 * RT consecutive output features and ALL rows of a; its waves split
//    K between them in chunks of 128 and the partial sums meet in LDS, added in wave order
//    (a fixed order: the result does not depend on timing or on what else is in the batch);
//  * W goes from global memory straight into MFMA operand registers: for the 16x16x32
//    instruction lane (n, g) holds k = 8g..8g+7 of row n, so the four lanes of a row read 64
//    contiguous bytes per load and two consecutive loads finish a 128-byte line; the loads
//    of two chunks are issued before the first multiply;
//  * a (a few KB to 1 MB) is re-read from L2 by every workgroup.
//
// Epilogues: store (bfloat16 or float32), add into the float32 residual stream, or SwiGLU
// (W holds gate rows then up rows; the workgroup computes both for its features and stores
// silu(gate) * up, so the 2I-wide intermediate never exists).
// The reference's decode projections are one-warp-per-row vector kernels
// (native/include/flyweight_v2_qwen_kernels.hpp:855-941).
#include "fw_common.h"
#include "fw_kernels.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define SK_CHUNK 128    // k per wave per iteration

enum { SK_STORE = 0, SK_ACCUMULATE = 1, SK_SWIGLU = 2 };

__device__ __forceinline__ bf16x8 load8(const uint16_t* __restrict__ base, size_t offset, bool valid) {
    if (!valid) return bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    return *reinterpret_cast<const bf16x8*>(base + offset);
}

__device__ __forceinline__ float silu_f(float g) {
    if (g >= 0.0f) return g / (1.0f + __expf(-g));
    const float e = __expf(g);
    return g * e / (1.0f + e);
}

// MT: tiles of 16 rows of a; RT: tiles of 16 features per workgroup (for SwiGLU the second
// tile is the up-projection of the same features).
template <int MT, int RT, int SK_WAVES, int MODE, typename TO>
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_skinny_kernel(
    const uint16_t* __restrict__ a, const uint16_t* __restrict__ w, const float* __restrict__ bias,
    TO* __restrict__ out, int M, int N, int K, int up_offset /* rows between gate and up, SwiGLU only */) {
    __shared__ float partial[SK_WAVES][RT * MT][64][4];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;          // feature (for W) or row of a (for a) within a tile
    const int g = lane >> 4;            // k group
    const int features = MODE == SK_SWIGLU ? 16 : 16 * RT;
    const int n0 = blockIdx.x * features;

    f32x4 acc[RT][MT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    size_t w_row[RT];
    bool w_ok[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int n = MODE == SK_SWIGLU ? n0 + r16 + rt * up_offset : n0 + rt * 16 + r16;
        w_ok[rt] = MODE == SK_SWIGLU ? (n0 + r16 < N) : (n < N);
        w_row[rt] = (size_t)(w_ok[rt] ? n : 0) * K;
    }
    size_t a_row[MT];
    bool a_ok[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        a_ok[mt] = mt * 16 + r16 < M;
        a_row[mt] = (size_t)(a_ok[mt] ? mt * 16 + r16 : 0) * K;
    }

#pragma unroll 2
    for (int k0 = wave * SK_CHUNK; k0 < K; k0 += SK_WAVES * SK_CHUNK) {
        bf16x8 wf[RT][4], af[MT][4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + j * 32 + g * 8;
            const bool k_ok = k < K;        // K is a multiple of 8: a run of 8 is in or out as a whole
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) wf[rt][j] = load8(w, w_row[rt] + k, k_ok && w_ok[rt]);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) af[mt][j] = load8(a, a_row[mt] + k, k_ok && a_ok[mt]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[rt][j], af[mt][j], acc[rt][mt], 0, 0, 0);
    }
    fw_mfma_drain();     // the loop is left by a branch; the accumulators are read next

    // partial sums meet in LDS; wave `t % WAVES` finishes tile t
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int r = 0; r < 4; ++r) partial[wave][rt * MT + mt][lane][r] = acc[rt][mt][r];
    __syncthreads();

    // D layout of the 16x16 product: lane holds feature 4 * (lane / 16) + r of the tile for row lane % 16 of a
    const int tiles = MODE == SK_SWIGLU ? MT : RT * MT;
    for (int tile = wave; tile < tiles; tile += SK_WAVES) {
        const int rt = MODE == SK_SWIGLU ? 0 : tile / MT;
        const int mt = MODE == SK_SWIGLU ? tile : tile % MT;
        const int m = mt * 16 + r16;
        float total[4] = {0.f, 0.f, 0.f, 0.f}, second[4] = {0.f, 0.f, 0.f, 0.f};
        for (int v = 0; v < SK_WAVES; ++v)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                total[r] += partial[v][rt * MT + mt][lane][r];
                if (MODE == SK_SWIGLU) second[r] += partial[v][MT + mt][lane][r];
            }
        if (m >= M) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int n = n0 + rt * 16 + g * 4 + r;
            if (n >= N) continue;
            float value = total[r];
            if (MODE == SK_SWIGLU) {
                value = silu_f(value) * second[r];
            } else if (bias) {
                value += bias[n];
            }
            const size_t at = (size_t)m * N + n;
            if (MODE == SK_ACCUMULATE) value += load_as_float(out, at);
            store_from_float(out, at, value);
        }
    }
}

template <int MT, int RT, int WAVES>
static void launch_mode(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                        int M, int N, int K, int up_offset, hipStream_t stream) {
    const uint16_t* pa = (const uint16_t*)a;
    const uint16_t* pw = (const uint16_t*)w;
    const int threads = WAVES * 64;
    if (mode == SK_SWIGLU) {
        const int blocks = fw_ceil_div(N, 16);
        gemm_skinny_kernel<MT, 2, WAVES, SK_SWIGLU, bf16_t><<<blocks, threads, 0, stream>>>(pa, pw, nullptr, (bf16_t*)out, M, N, K, up_offset);
        return;
    }
    const int blocks = fw_ceil_div(N, 16 * RT);
    if (mode == SK_ACCUMULATE)
        gemm_skinny_kernel<MT, RT, WAVES, SK_ACCUMULATE, float><<<blocks, threads, 0, stream>>>(pa, pw, bias, (float*)out, M, N, K, 0);
    else if (out_dtype == FW_F32)
        gemm_skinny_kernel<MT, RT, WAVES, SK_STORE, float><<<blocks, threads, 0, stream>>>(pa, pw, bias, (float*)out, M, N, K, 0);
    else
        gemm_skinny_kernel<MT, RT, WAVES, SK_STORE, bf16_t><<<blocks, threads, 0, stream>>>(pa, pw, bias, (bf16_t*)out, M, N, K, 0);
}

template <int MT>
static void launch_rows(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                        int M, int N, int K, hipStream_t s) {
    // few features: one tile of 16 per workgroup so that enough workgroups stream W; a long
    // K beside few features: more waves per workgroup share it
    if (N > 4096) launch_mode<MT, 2, 8>(a, w, bias, out, out_dtype, mode, M, N, K, N, s);
    else if (K >= 4096) launch_mode<MT, 1, 16>(a, w, bias, out, out_dtype, mode, M, N, K, N, s);
    else launch_mode<MT, 1, 8>(a, w, bias, out, out_dtype, mode, M, N, K, N, s);
}

// mode 0: out = a . w^T (+ bias) stored as out_dtype; 1: out (float32) += a . w^T (+ bias);
// 2: w is [2 * N][K] (gate rows, then up rows); out [M][N] bfloat16 = silu(gate) * up.
extern "C" int fw_gemm_skinny(const void* a, const void* w, const float* bias, void* out, int out_dtype,
                              int mode, int M, int N, int K, void* stream) {
    FW_REQUIRE(M >= 1 && M <= 64, "gemm_skinny: takes 1..64 rows, got %d", M);
    FW_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "gemm_skinny: K (%d) must be a positive multiple of 8, N (%d) positive", K, N);
    FW_REQUIRE(mode >= 0 && mode <= 2, "gemm_skinny: unknown mode %d", mode);
    FW_REQUIRE(mode != SK_ACCUMULATE || out_dtype == FW_F32, "gemm_skinny: accumulation needs a float32 destination");
    FW_REQUIRE(mode != SK_SWIGLU || (out_dtype == FW_BF16 && bias == nullptr), "gemm_skinny: SwiGLU stores bfloat16 and takes no bias");
    FW_REQUIRE(out_dtype == FW_F32 || out_dtype == FW_BF16, "gemm_skinny: unknown out dtype %d", out_dtype);
    FW_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_skinny: operands must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    switch ((M + 15) / 16) {
        case 1: launch_rows<1>(a, w, bias, out, out_dtype, mode, M, N, K, s); break;
        case 2: launch_rows<2>(a, w, bias, out, out_dtype, mode, M, N, K, s); break;
        case 3: launch_rows<3>(a, w, bias, out, out_dtype, mode, M, N, K, s); break;
        default: launch_rows<4>(a, w, bias, out, out_dtype, mode, M, N, K, s); break;
    }
    FW_LAUNCH_CHECK("gemm_skinny");
    return 0;
}
