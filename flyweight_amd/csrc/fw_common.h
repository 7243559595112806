// Shared device helpers for the gfx950 kernels: storage types, conversions, wave64
// reductions, and the error channel behind the flat C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// dtype codes used across the C ABI
#define FW_F32 0
#define FW_BF16 1

// ---- error channel: every entry point returns 0 or -1 and leaves a message ---------
void fw_set_error(const char* format, ...);
// A workgroup barrier that orders LDS traffic only. __syncthreads() also waits for every global
// load in flight (its fence covers global memory), which empties a prefetch pipeline at each
// barrier; use this one where waves hand data to each other through LDS alone.
__device__ __forceinline__ void fw_lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Reductions over the four lanes l, l ^ 16, l ^ 32, l ^ 48 of a wave (every lane gets the result)
// with the row-swap instructions of gfx950 instead of two trips through the LDS crossbar
// (__shfl_xor). v_permlane16_swap exchanges rows 1 and 3 of its first register with rows 0 and 2
// of its second; v_permlane32_swap the upper half of the first with the lower half of the second.
// Given one value in two registers, the two results of a swap are the two partners of a lane.
// The second copy is made opaque: given one value twice the compiler may name one register
// twice, and the instruction then swaps rows inside that register. The results are taken as
// scalars before they are reinterpreted (a bit cast straight from the builtin's vector result
// lost its second element at compile time).
__device__ __forceinline__ void fw_quad_partners16(float x, float& mine, float& partner) {
    uint32_t u = __float_as_uint(x), copy = u;
    asm volatile("" : "+v"(copy));
    const auto swapped = __builtin_amdgcn_permlane16_swap(u, copy, false, false);
    const uint32_t first = swapped[0], second = swapped[1];
    mine = __uint_as_float(first);
    partner = __uint_as_float(second);
}
__device__ __forceinline__ void fw_quad_partners32(float x, float& mine, float& partner) {
    uint32_t u = __float_as_uint(x), copy = u;
    asm volatile("" : "+v"(copy));
    const auto swapped = __builtin_amdgcn_permlane32_swap(u, copy, false, false);
    const uint32_t first = swapped[0], second = swapped[1];
    mine = __uint_as_float(first);
    partner = __uint_as_float(second);
}
__device__ __forceinline__ float fw_quad_max(float x) {
    float a, b;
    fw_quad_partners16(x, a, b);
    fw_quad_partners32(fmaxf(a, b), a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float fw_quad_sum(float x) {
    float a, b;
    fw_quad_partners16(x, a, b);
    fw_quad_partners32(a + b, a, b);
    return a + b;
}

// Lets the matrix pipe finish what was issued before control goes on. Inside one basic block the
// compiler keeps a product and the first read of its result far enough apart; where the read is
// the target of a taken branch it has been seen one instruction behind the product, reading the
// registers the product writes last before they were written (seen in the attention kernel with
// head sizes below the template's: two of four components stale). Called once behind a loop of
// products, before branches that lead to code reading the accumulators. 24 wait states cover the
// longest product (16 passes).
__device__ __forceinline__ void fw_mfma_drain() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 15\n\ts_nop 7");
    __builtin_amdgcn_sched_barrier(0);
}

#define FW_REQUIRE(cond, ...)                    \
    do {                                         \
        if (!(cond)) {                           \
            fw_set_error(__VA_ARGS__);           \
            return -1;                           \
        }                                        \
    } while (0)
#define FW_LAUNCH_CHECK(name)                                                     \
    do {                                                                          \
        hipError_t fw_status__ = hipGetLastError();                               \
        if (fw_status__ != hipSuccess) {                                          \
            fw_set_error("%s: launch failed: %s", name, hipGetErrorString(fw_status__)); \
            return -1;                                                            \
        }                                                                         \
    } while (0)

// ---- bfloat16 as raw bits ----------------------------------------------------------
struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float bf16_to_float(bf16_t v) {
    return __uint_as_float(((uint32_t)v.bits) << 16);
}
__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits) {
    return __uint_as_float(bits << 16);
}
// round to nearest, ties to even; NaN stays NaN
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
    bf16_t r;
    r.bits = float_to_bf16_bits(f);
    return r;
}

template <typename T> __device__ __forceinline__ float load_as_float(const T* p, size_t i);
template <> __device__ __forceinline__ float load_as_float<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ __forceinline__ float load_as_float<bf16_t>(const bf16_t* p, size_t i) {
    return bf16_to_float(p[i]);
}
template <typename T> __device__ __forceinline__ void store_from_float(T* p, size_t i, float v);
template <> __device__ __forceinline__ void store_from_float<float>(float* p, size_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void store_from_float<bf16_t>(bf16_t* p, size_t i, float v) {
    p[i] = float_to_bf16(v);
}
// the value a store of this type would leave behind (used where a value is both kept
// in registers and written, so later reads from memory see the same number)
template <typename T> __device__ __forceinline__ float round_through(float v);
template <> __device__ __forceinline__ float round_through<float>(float v) { return v; }
template <> __device__ __forceinline__ float round_through<bf16_t>(float v) {
    return bf16_bits_to_float(float_to_bf16_bits(v));
}

// ---- wave64 reductions (fixed butterfly order: the result does not depend on
//      anything but the 64 inputs) -----------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, 64));
    return v;
}

// block-wide sum for blocks of up to 1024 threads; every thread gets the result
__device__ __forceinline__ float block_sum(float v, float* scratch /* >= 16 floats */) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int waves = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.0f;
    for (int i = 0; i < waves; ++i) total += scratch[i];
    return total;
}

static inline int fw_ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }

// Eight bfloat16 of a weight matrix that a decode step reads once: with `streamed` the load says
// so (nontemporal), which keeps a stream of weights from pushing the step's activations out of the
// caches and, on whole 1 KB pieces per wave, reads faster (a read-only kernel over 268 MB: 39.5 against
// 43.7 us). Weights in row-major order are loaded as they always were.
typedef __attribute__((ext_vector_type(8))) __bf16 fw_bf16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t fw_u32x4;
template <bool STREAMED>
__device__ __forceinline__ fw_bf16x8 fw_load_weights(const uint16_t* from) {
    const fw_u32x4* at = reinterpret_cast<const fw_u32x4*>(from);
    const fw_u32x4 v = STREAMED ? __builtin_nontemporal_load(at) : *at;
    return __builtin_bit_cast(fw_bf16x8, v);
}

// ---- candidates for the next token ----------------------------------------------------
// A candidate is ordered by (value descending, id ascending); NaN sorts last. The key packs both
// so that one 64-bit comparison orders two candidates (a greater key comes first) and ties go to
// the lowest id, as the reference's fused LM-head argmax does
// (native/include/flyweight_v2_qwen_kernels.hpp:2391-2405).
__device__ __forceinline__ unsigned long long candidate_key(float value, int id) {
    uint32_t bits = value == 0.0f ? 0u : __float_as_uint(value);        // -0 and +0 are one value: the lower id first
    uint32_t ordered;
    if (value != value) ordered = 0u;                                   // NaN: below everything
    else ordered = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u); // monotone in value
    return ((unsigned long long)ordered << 32) | (unsigned long long)(0xffffffffu - (uint32_t)id);
}
__device__ __forceinline__ int candidate_id(unsigned long long key) { return (int)(0xffffffffu - (uint32_t)(key & 0xffffffffull)); }

