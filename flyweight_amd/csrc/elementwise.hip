// Row-wise kernels: embedding gather, RMS norm, SwiGLU, rotation tables, argmax/top-k.
// All reductions run in float32 in an order fixed by the row alone.
#include "fw_common.h"
#include "fw_kernels.h"

#include <stdarg.h>
#include <stdio.h>

// ---- error channel ---------------------------------------------------------------------
static thread_local char fw_error_text[1024] = "";

void fw_set_error(const char* format, ...) {
    va_list args;
    va_start(args, format);
    vsnprintf(fw_error_text, sizeof(fw_error_text), format, args);
    va_end(args);
}
extern "C" const char* fw_last_error(void) { return fw_error_text; }
extern "C" int fw_abi_version(void) { return 9; }

// ---- embedding -------------------------------------------------------------------------
// The reference gathers one row per token and widens it to float32
// (native/include/flyweight_v2_native_kernels.hpp:98-151).
// `scale` multiplies the row (architectures that scale their embeddings; 1 leaves it as stored).
template <typename W>
__global__ void embed_rows_kernel(const W* __restrict__ table, const int32_t* __restrict__ ids,
                                  float* __restrict__ out, int hidden, float scale) {
    const int row = blockIdx.y;
    const size_t base = (size_t)ids[row] * hidden;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < hidden; i += gridDim.x * blockDim.x)
        out[(size_t)row * hidden + i] = load_as_float(table, base + i) * scale;
}

extern "C" int fw_embed_rows(const void* table, int table_dtype, const int32_t* ids, float* out,
                             int rows, int hidden, int vocab, float scale, void* stream) {
    FW_REQUIRE(rows >= 0 && hidden > 0 && vocab > 0, "embed_rows: bad sizes rows=%d hidden=%d vocab=%d", rows, hidden, vocab);
    FW_REQUIRE(rows <= 65535, "embed_rows: at most 65535 rows per call, got %d", rows);
    if (rows == 0) return 0;
    dim3 grid(fw_ceil_div(hidden, 256) > 64 ? 64 : fw_ceil_div(hidden, 256), rows);
    if (table_dtype == FW_F32)
        embed_rows_kernel<float><<<grid, 256, 0, (hipStream_t)stream>>>((const float*)table, ids, out, hidden, scale);
    else if (table_dtype == FW_BF16)
        embed_rows_kernel<bf16_t><<<grid, 256, 0, (hipStream_t)stream>>>((const bf16_t*)table, ids, out, hidden, scale);
    else
        FW_REQUIRE(false, "embed_rows: unknown table dtype %d", table_dtype);
    FW_LAUNCH_CHECK("embed_rows");
    return 0;
}

// ---- RMS norm --------------------------------------------------------------------------
// y = x * rsqrt(mean(x^2) + eps) * w; the weight multiplies directly unless one_centered
// (native/include/flyweight_v2_qwen_kernels.hpp:425-447, rows variant :1180-1207).
template <typename T>
__global__ void rmsnorm_rows_kernel(const float* __restrict__ x, const float* __restrict__ weight,
                                    T* __restrict__ out, const int32_t* __restrict__ row_index,
                                    int hidden, float eps, int one_centered) {
    __shared__ float scratch[16];
    const int row = blockIdx.x;
    const size_t src = (size_t)(row_index ? row_index[row] : row) * hidden;
    float sum = 0.0f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float v = x[src + i];
        sum += v * v;
    }
    sum = block_sum(sum, scratch);
    const float inv = rsqrtf(sum / (float)hidden + eps);
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float w = one_centered ? 1.0f + weight[i] : weight[i];
        store_from_float(out, (size_t)row * hidden + i, x[src + i] * inv * w);
    }
}

// The same for a width that is a multiple of 4, four values a thread at a time: a row is read once
// in 16-byte pieces and kept in registers (up to 4 pieces a thread: 4,096 values), the result
// stored in pieces of four. The sum of a row is formed in an order of its own (per piece, then per
// thread, then over the block): still a function of the row alone.
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_rows4_kernel(const float* __restrict__ x, const float* __restrict__ weight,
                                                            T* __restrict__ out, const int32_t* __restrict__ row_index,
                                                            int hidden, float eps, int one_centered) {
    typedef __attribute__((ext_vector_type(4))) float f32x4;
    typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
    __shared__ float scratch[16];
    const int row = blockIdx.x;
    const f32x4* source = reinterpret_cast<const f32x4*>(x + (size_t)(row_index ? row_index[row] : row) * hidden);
    const int pieces = hidden / 4;
    f32x4 held[4], scale[4];
    float sum = 0.0f;
    // (the weight is asked for with the row, not behind the sum over the block. A wave per row, whose sum needs
    // neither LDS nor a barrier, was slower: 6.8 against 6.4 us for 2,048 rows of 2,048.)
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int piece = threadIdx.x + u * 256;
        held[u] = piece < pieces ? source[piece] : f32x4{0.f, 0.f, 0.f, 0.f};
        scale[u] = reinterpret_cast<const f32x4*>(weight)[piece < pieces ? piece : 0];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
        sum += (held[u][0] * held[u][0] + held[u][1] * held[u][1]) + (held[u][2] * held[u][2] + held[u][3] * held[u][3]);
    sum = block_sum(sum, scratch);
    const float inv = rsqrtf(sum / (float)hidden + eps);
    const float one = one_centered ? 1.0f : 0.0f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int piece = threadIdx.x + u * 256;
        if (piece >= pieces) break;
        const f32x4 w = scale[u];
        f32x4 y;
#pragma unroll
        for (int e = 0; e < 4; ++e) y[e] = held[u][e] * inv * (w[e] + one);
        if constexpr (sizeof(T) == 4) {
            reinterpret_cast<f32x4*>(out + (size_t)row * hidden)[piece] = y;
        } else {
            const u32x2 packed = {(uint32_t)float_to_bf16_bits(y[0]) | ((uint32_t)float_to_bf16_bits(y[1]) << 16),
                                  (uint32_t)float_to_bf16_bits(y[2]) | ((uint32_t)float_to_bf16_bits(y[3]) << 16)};
            reinterpret_cast<u32x2*>(out + (size_t)row * hidden)[piece] = packed;
        }
    }
}

extern "C" int fw_rmsnorm_rows(const float* x, const float* weight, void* out, int out_dtype,
                               const int32_t* row_index, int rows, int hidden, float eps,
                               int one_centered, void* stream) {
    FW_REQUIRE(rows >= 0 && hidden > 0, "rmsnorm_rows: bad sizes rows=%d hidden=%d", rows, hidden);
    FW_REQUIRE(eps > 0.0f, "rmsnorm_rows: eps must be positive");
    if (rows == 0) return 0;
    FW_REQUIRE(out_dtype == FW_F32 || out_dtype == FW_BF16, "rmsnorm_rows: unknown out dtype %d", out_dtype);
    const bool by_four = hidden % 4 == 0 && hidden <= 4096 && (uintptr_t)x % 16 == 0 && (uintptr_t)weight % 16 == 0 &&
                         (uintptr_t)out % 16 == 0;
    if (by_four && out_dtype == FW_F32)
        rmsnorm_rows4_kernel<float><<<rows, 256, 0, (hipStream_t)stream>>>(x, weight, (float*)out, row_index, hidden, eps, one_centered);
    else if (by_four)
        rmsnorm_rows4_kernel<bf16_t><<<rows, 256, 0, (hipStream_t)stream>>>(x, weight, (bf16_t*)out, row_index, hidden, eps, one_centered);
    else if (out_dtype == FW_F32)
        rmsnorm_rows_kernel<float><<<rows, 256, 0, (hipStream_t)stream>>>(x, weight, (float*)out, row_index, hidden, eps, one_centered);
    else
        rmsnorm_rows_kernel<bf16_t><<<rows, 256, 0, (hipStream_t)stream>>>(x, weight, (bf16_t*)out, row_index, hidden, eps, one_centered);
    FW_LAUNCH_CHECK("rmsnorm_rows");
    return 0;
}

// ---- SwiGLU ----------------------------------------------------------------------------
// silu(g) * u with a sigmoid that cannot overflow
// (native/include/flyweight_v2_qwen_kernels.hpp:1209-1223).
__device__ __forceinline__ float stable_sigmoid(float g) {
    if (g >= 0.0f) return 1.0f / (1.0f + expf(-g));
    const float e = expf(g);
    return e / (1.0f + e);
}

template <typename TI, typename TO>
__global__ void swiglu_kernel(const TI* __restrict__ gate_up, TO* __restrict__ out, int intermediate) {
    const int row = blockIdx.y;
    const TI* source = gate_up + (size_t)row * 2 * intermediate;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < intermediate; i += gridDim.x * blockDim.x) {
        const float g = load_as_float(source, i);
        const float u = load_as_float(source, (size_t)intermediate + i);
        store_from_float(out, (size_t)row * intermediate + i, g * stable_sigmoid(g) * u);
    }
}

extern "C" int fw_swiglu(const void* gate_up, int in_dtype, void* out, int out_dtype, int rows, int intermediate,
                         void* stream) {
    FW_REQUIRE(rows >= 0 && intermediate > 0, "swiglu: bad sizes rows=%d width=%d", rows, intermediate);
    FW_REQUIRE(rows <= 65535, "swiglu: at most 65535 rows per call, got %d", rows);
    if (rows == 0) return 0;
    int bx = fw_ceil_div(intermediate, 256);
    if (bx > 32) bx = 32;
    dim3 grid(bx, rows);
    hipStream_t s = (hipStream_t)stream;
    if (in_dtype == FW_F32 && out_dtype == FW_F32)
        swiglu_kernel<float, float><<<grid, 256, 0, s>>>((const float*)gate_up, (float*)out, intermediate);
    else if (in_dtype == FW_F32 && out_dtype == FW_BF16)
        swiglu_kernel<float, bf16_t><<<grid, 256, 0, s>>>((const float*)gate_up, (bf16_t*)out, intermediate);
    else if (in_dtype == FW_BF16 && out_dtype == FW_BF16)
        swiglu_kernel<bf16_t, bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)gate_up, (bf16_t*)out, intermediate);
    else
        FW_REQUIRE(false, "swiglu: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
    FW_LAUNCH_CHECK("swiglu");
    return 0;
}

// ---- rotation tables -------------------------------------------------------------------
// angle = position * theta^(-2i/d) (native/include/flyweight_v2_native_kernels.hpp:993-1008
// computes the same angle per element in float32). The product is formed in float64 so that
// a large position does not lose the low bits of the angle; cos and sin are float32.
__global__ void rope_table_kernel(const int32_t* __restrict__ positions, const double* __restrict__ inv_freq,
                                  float* __restrict__ cos_out, float* __restrict__ sin_out, int rows, int half) {
    const int index = blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= rows * half) return;
    const int row = index / half;
    const int pair = index - row * half;
    const double angle = (double)positions[row] * inv_freq[pair];
    cos_out[index] = (float)cos(angle);
    sin_out[index] = (float)sin(angle);
}

extern "C" int fw_rope_table(const int32_t* positions, const double* inv_freq, float* cos_out, float* sin_out,
                             int rows, int half, void* stream) {
    FW_REQUIRE(rows >= 0 && half > 0, "rope_table: bad sizes rows=%d half=%d", rows, half);
    if (rows == 0) return 0;
    const long long total = (long long)rows * half;
    rope_table_kernel<<<fw_ceil_div(total, 256), 256, 0, (hipStream_t)stream>>>(positions, inv_freq, cos_out, sin_out, rows, half);
    FW_LAUNCH_CHECK("rope_table");
    return 0;
}

// ---- argmax / top-k --------------------------------------------------------------------
// A candidate is ordered by (value descending, id ascending); NaN sorts last. The key packs
// both so that one 64-bit max finds the winner, as the reference's fused LM-head argmax
// does (native/include/flyweight_v2_qwen_kernels.hpp:2391-2405): ties go to the lowest id.
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        const unsigned long long other = __shfl_xor(v, offset, 64);
        v = other > v ? other : v;
    }
    return v;
}

__device__ __forceinline__ unsigned long long block_max_u64(unsigned long long v, unsigned long long* scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = (blockDim.x + 63) >> 6;
    v = wave_max_u64(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    unsigned long long best = 0;
    for (int i = 0; i < waves; ++i) best = scratch[i] > best ? scratch[i] : best;
    return best;
}

// Argmax in two steps, so that a few rows of a wide vocabulary still fill the chip: grid (parts,
// rows) finds the best key of each part of a row, then one wave per row finds the best of those.
// Keys order by value, then by the lower id, so the result does not depend on the cut.
#define ARGMAX_PARTS 64
__global__ __launch_bounds__(256) void argmax_parts_kernel(const float* __restrict__ logits,
                                                           unsigned long long* __restrict__ best_of_part, int vocab) {
    __shared__ unsigned long long scratch[16];
    const int part = blockIdx.x, row = blockIdx.y;
    const int per_part = (vocab + ARGMAX_PARTS - 1) / ARGMAX_PARTS;
    const int begin = part * per_part, end = begin + per_part < vocab ? begin + per_part : vocab;
    const float* source = logits + (size_t)row * vocab;
    unsigned long long best = 0;
    for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
        const unsigned long long key = candidate_key(source[i], i);
        if (key > best) best = key;
    }
    best = block_max_u64(best, scratch);
    if (threadIdx.x == 0) best_of_part[(size_t)row * ARGMAX_PARTS + part] = best;
}

__global__ __launch_bounds__(64) void argmax_finish_kernel(const unsigned long long* __restrict__ best_of_part,
                                                           int32_t* __restrict__ ids, int32_t* __restrict__ also,
                                                           int32_t* __restrict__ advance) {
    const int row = blockIdx.x;
    unsigned long long best = best_of_part[(size_t)row * ARGMAX_PARTS + threadIdx.x];     // 64 parts, 64 lanes
    best = wave_max_u64(best);
    if (threadIdx.x == 0) {
        const int id = (int)(0xffffffffu - (uint32_t)(best & 0xffffffffull));
        ids[row] = id;
        if (also) also[row] = id;
        if (advance) advance[row] += 1;
    }
}

// workspace: rows * 64 64-bit words (the best key of each part of each row). also: null, or a second
// place for the ids; advance: null, or a counter per row that goes up by one. (A decode step that
// follows at once takes its token ids and positions from these: nothing crosses to the host between.)
extern "C" int fw_argmax_rows(const float* logits, int32_t* ids, int32_t* also, int32_t* advance, void* workspace,
                              int rows, int vocab, void* stream) {
    FW_REQUIRE(rows >= 0 && rows <= 65535 && vocab > 0, "argmax_rows: bad sizes rows=%d vocab=%d", rows, vocab);
    if (rows == 0) return 0;
    FW_REQUIRE(workspace != nullptr && (uintptr_t)workspace % 8 == 0, "argmax_rows: needs an 8-byte aligned workspace");
    argmax_parts_kernel<<<dim3(ARGMAX_PARTS, rows), 256, 0, (hipStream_t)stream>>>(logits, (unsigned long long*)workspace, vocab);
    FW_LAUNCH_CHECK("argmax_rows (parts)");
    argmax_finish_kernel<<<rows, 64, 0, (hipStream_t)stream>>>((const unsigned long long*)workspace, ids, also, advance);
    FW_LAUNCH_CHECK("argmax_rows");
    return 0;
}

// ---- argmax for callers that cannot allocate ----------------------------------------------
// fw_argmax_rows without a workspace argument: the best keys of the parts live in a file-scope
// device array, of which every GPU holds its own copy at its own address until the process ends
// (FW_ARGMAX_STATIC_MAX_ROWS * 64 keys of 8 bytes = 512 KB). The array's name is only a stand-in
// on the host: its address on the current device is looked up once per device and kept, and that
// pointer is what the kernels get, as they get the workspace in fw_argmax_rows. Nothing has to
// start at zero (the first kernel writes all 64 keys of every row before the second reads them), so
// nothing is cleared; what the last call left is overwritten. Calls that overlap on one GPU (two
// streams, two threads) share the array and race.
#define FW_ARGMAX_STATIC_MAX_ROWS 1024
#define FW_ARGMAX_STATIC_MAX_DEVICES 64
static __device__ __align__(256) unsigned long long fw_argmax_static_scratch[FW_ARGMAX_STATIC_MAX_ROWS * ARGMAX_PARTS];
static unsigned long long* fw_argmax_static_address[FW_ARGMAX_STATIC_MAX_DEVICES];     // per device, null until looked up

extern "C" int fw_argmax_rows_static_max_rows(void) { return FW_ARGMAX_STATIC_MAX_ROWS; }

extern "C" int fw_argmax_rows_static(const float* logits, int32_t* ids, int32_t* also, int32_t* advance, int rows,
                                     int vocab, void* stream) {
    FW_REQUIRE(vocab > 0 && rows >= 0, "argmax_rows_static: bad sizes rows=%d vocab=%d", rows, vocab);
    FW_REQUIRE(rows <= FW_ARGMAX_STATIC_MAX_ROWS,
               "argmax_rows_static: %d rows, but the built-in scratch holds %d (use fw_argmax_rows with a workspace)", rows,
               FW_ARGMAX_STATIC_MAX_ROWS);
    if (rows == 0) return 0;
    FW_REQUIRE(logits != nullptr && ids != nullptr, "argmax_rows_static: logits and ids must be given");
    int device = -1;
    hipError_t status = hipGetDevice(&device);
    FW_REQUIRE(status == hipSuccess, "argmax_rows_static: hipGetDevice failed: %s", hipGetErrorString(status));
    FW_REQUIRE(device >= 0 && device < FW_ARGMAX_STATIC_MAX_DEVICES, "argmax_rows_static: device %d is beyond the %d this entry point keeps an address for",
               device, FW_ARGMAX_STATIC_MAX_DEVICES);
    unsigned long long* scratch = __atomic_load_n(&fw_argmax_static_address[device], __ATOMIC_ACQUIRE);
    if (scratch == nullptr) {       // first call on this device: two threads at once find the same address
        status = hipGetSymbolAddress((void**)&scratch, HIP_SYMBOL(fw_argmax_static_scratch));
        FW_REQUIRE(status == hipSuccess && scratch != nullptr, "argmax_rows_static: the scratch array's address on device %d: %s", device,
                   hipGetErrorString(status));
        __atomic_store_n(&fw_argmax_static_address[device], scratch, __ATOMIC_RELEASE);
    }
    argmax_parts_kernel<<<dim3(ARGMAX_PARTS, rows), 256, 0, (hipStream_t)stream>>>(logits, scratch, vocab);
    FW_LAUNCH_CHECK("argmax_rows_static (parts)");
    argmax_finish_kernel<<<rows, 64, 0, (hipStream_t)stream>>>(scratch, ids, also, advance);
    FW_LAUNCH_CHECK("argmax_rows_static");
    return 0;
}

// ---- logits: scale and soft cap ------------------------------------------------------------
// x <- x * scale, then, with a cap c > 0, x <- c * tanh(x / c): for architectures whose head has a
// logit scale or a soft cap. In place, float32.
__global__ void scale_softcap_kernel(float* __restrict__ x, long long count, float scale, float cap) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (long long)gridDim.x * blockDim.x) {
        float value = x[i] * scale;
        if (cap > 0.0f) value = cap * tanhf(value / cap);
        x[i] = value;
    }
}

extern "C" int fw_scale_softcap(float* x, long long count, float scale, float cap, void* stream) {
    FW_REQUIRE(count >= 0 && cap >= 0.0f, "scale_softcap: bad arguments count=%lld cap=%g", count, (double)cap);
    if (count == 0) return 0;
    long long blocks = (count + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    scale_softcap_kernel<<<(int)blocks, 256, 0, (hipStream_t)stream>>>(x, count, scale, cap);
    FW_LAUNCH_CHECK("scale_softcap");
    return 0;
}

// ---- fill ------------------------------------------------------------------------------
__global__ void fill_zero_kernel(uint32_t* __restrict__ ptr, long long words) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < words;
         i += (long long)gridDim.x * blockDim.x)
        ptr[i] = 0u;
}

__global__ void fill_zero_pieces_kernel(uint32_t* __restrict__ ptr, long long words_per_piece, long long stride_words) {
    uint32_t* piece = ptr + (size_t)blockIdx.y * stride_words;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < words_per_piece; i += (long long)gridDim.x * blockDim.x)
        piece[i] = 0u;
}

// `pieces` runs of `bytes` each, `stride_bytes` apart (a request's slot in the state of several layers
// that lie in one allocation), cleared in one launch.
extern "C" int fw_fill_zero_pieces(void* ptr, int pieces, long long bytes, long long stride_bytes, void* stream) {
    FW_REQUIRE(bytes >= 0 && bytes % 4 == 0 && stride_bytes % 4 == 0 && stride_bytes >= bytes,
               "fill_zero_pieces: %lld bytes every %lld bytes: both must be multiples of 4, the pieces apart", bytes, stride_bytes);
    FW_REQUIRE(pieces >= 0 && pieces <= 65535, "fill_zero_pieces: %d pieces (at most 65535)", pieces);
    if (bytes == 0 || pieces == 0) return 0;
    const long long words = bytes / 4;
    int blocks = fw_ceil_div(words, 256);
    if (blocks > 256) blocks = 256;
    fill_zero_pieces_kernel<<<dim3(blocks, pieces), 256, 0, (hipStream_t)stream>>>((uint32_t*)ptr, words, stride_bytes / 4);
    FW_LAUNCH_CHECK("fill_zero_pieces");
    return 0;
}

extern "C" int fw_fill_zero(void* ptr, long long bytes, void* stream) {
    FW_REQUIRE(bytes >= 0 && bytes % 4 == 0, "fill_zero: byte count %lld must be a multiple of 4", bytes);
    if (bytes == 0) return 0;
    const long long words = bytes / 4;
    int blocks = fw_ceil_div(words, 256);
    if (blocks > 2048) blocks = 2048;
    fill_zero_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((uint32_t*)ptr, words);
    FW_LAUNCH_CHECK("fill_zero");
    return 0;
}
