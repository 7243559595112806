// Gated short convolution (the LFM2 conv mixer's middle): with (B | C | x) = in_proj(h),
//   bx = B * x;  y_t = sum_j taps[j] * bx_{t-(L-1)+j} (+ bias);  out = C * y
// tap L-1 multiplies the current token and tap 0 the oldest; before the sequence starts
// bx is zero. The per-request state is the last L-1 values of bx per channel, oldest first
// (native/include/flyweight_v2_native_kernels.hpp:1295-1345; the reference walks a chunk's
// rows serially per channel, here every (row, channel) is independent and the state is
// read where a row reaches back past the start of its segment).
//
// A batch holds segments of several sequences. The general variant is two launches: the
// outputs (state is only read), then the state update (one thread per segment and channel
// reads what it needs, then writes). A batch of single-token segments runs one fused launch.
#include "fw_common.h"
#include "fw_kernels.h"

#define CONV_MAX_KERNEL 16

template <typename T>
__device__ __forceinline__ float bx_at(const T* __restrict__ bcx, int row, int channel, int hidden) {
    const T* source = bcx + (size_t)row * 3 * hidden;
    return load_as_float(source, channel) * load_as_float(source, 2 * (size_t)hidden + channel);
}

template <typename T, typename TO>
__global__ void shortconv_rows_kernel(const T* __restrict__ bcx, TO* __restrict__ out,
                                      const float* __restrict__ taps, const float* __restrict__ conv_bias,
                                      const float* __restrict__ state, const int32_t* __restrict__ row_seg,
                                      const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot,
                                      int hidden, int kernel_size) {
    const int row = blockIdx.y;
    const int channel = blockIdx.x * blockDim.x + threadIdx.x;
    if (channel >= hidden) return;
    const int seg = row_seg[row];
    const int first = seg_row0[seg];
    const int history = kernel_size - 1;
    const float* channel_state = state + ((size_t)seg_slot[seg] * hidden + channel) * history;
    const float* channel_taps = taps + (size_t)channel * kernel_size;
    const int offset_in_segment = row - first;
    float y = 0.0f;
    for (int j = 0; j < kernel_size; ++j) {
        const int offset = offset_in_segment - history + j;
        const float bx = offset >= 0 ? bx_at(bcx, first + offset, channel, hidden)
                                     : channel_state[history + offset];
        y = fmaf(channel_taps[j], bx, y);
    }
    if (conv_bias) y += conv_bias[channel];
    const float gate = load_as_float(bcx, (size_t)row * 3 * hidden + hidden + channel);
    store_from_float(out, (size_t)row * hidden + channel, gate * y);
}

template <typename T>
__global__ void shortconv_state_kernel(const T* __restrict__ bcx, float* __restrict__ state,
                                       const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot,
                                       int hidden, int kernel_size) {
    const int seg = blockIdx.y;
    const int channel = blockIdx.x * blockDim.x + threadIdx.x;
    if (channel >= hidden) return;
    const int first = seg_row0[seg];
    const int count = seg_row0[seg + 1] - first;
    const int history = kernel_size - 1;
    float* channel_state = state + ((size_t)seg_slot[seg] * hidden + channel) * history;
    float next[CONV_MAX_KERNEL];
    for (int k = 0; k < history; ++k) {
        const int offset = count - history + k;     // position within the segment, may be negative
        next[k] = offset >= 0 ? bx_at(bcx, first + offset, channel, hidden) : channel_state[history + offset];
    }
    for (int k = 0; k < history; ++k) channel_state[k] = next[k];
}

// every segment is one row: output and state shift in one pass
template <typename T, typename TO>
__global__ void shortconv_decode_kernel(const T* __restrict__ bcx, TO* __restrict__ out,
                                        const float* __restrict__ taps, const float* __restrict__ conv_bias,
                                        float* __restrict__ state, const int32_t* __restrict__ seg_slot,
                                        int hidden, int kernel_size) {
    const int row = blockIdx.y;
    const int channel = blockIdx.x * blockDim.x + threadIdx.x;
    if (channel >= hidden) return;
    const int history = kernel_size - 1;
    float* channel_state = state + ((size_t)seg_slot[row] * hidden + channel) * history;
    const float* channel_taps = taps + (size_t)channel * kernel_size;
    float window[CONV_MAX_KERNEL];
    for (int k = 0; k < history; ++k) window[k] = channel_state[k];
    window[history] = bx_at(bcx, row, channel, hidden);
    float y = 0.0f;
    for (int j = 0; j < kernel_size; ++j) y = fmaf(channel_taps[j], window[j], y);
    if (conv_bias) y += conv_bias[channel];
    for (int k = 0; k < history; ++k) channel_state[k] = window[k + 1];
    const float gate = load_as_float(bcx, (size_t)row * 3 * hidden + hidden + channel);
    store_from_float(out, (size_t)row * hidden + channel, gate * y);
}

template <typename T, typename TO>
static void launch(const void* bcx, void* out, const float* taps, const float* conv_bias, float* state,
                   const int32_t* row_seg, const int32_t* seg_row0, const int32_t* seg_slot, int rows,
                   int segments, int hidden, int kernel_size, hipStream_t stream) {
    const int bx = fw_ceil_div(hidden, 256);
    if (rows == segments) {
        shortconv_decode_kernel<T, TO><<<dim3(bx, rows), 256, 0, stream>>>(
            (const T*)bcx, (TO*)out, taps, conv_bias, state, seg_slot, hidden, kernel_size);
        return;
    }
    shortconv_rows_kernel<T, TO><<<dim3(bx, rows), 256, 0, stream>>>(
        (const T*)bcx, (TO*)out, taps, conv_bias, state, row_seg, seg_row0, seg_slot, hidden, kernel_size);
    shortconv_state_kernel<T><<<dim3(bx, segments), 256, 0, stream>>>(
        (const T*)bcx, state, seg_row0, seg_slot, hidden, kernel_size);
}

extern "C" int fw_shortconv(const void* bcx, int in_dtype, void* out, int out_dtype, const float* taps,
                            const float* conv_bias, float* state, const int32_t* row_seg, const int32_t* seg_row0,
                            const int32_t* seg_slot, int rows, int segments, int hidden, int kernel_size,
                            int slots, void* stream) {
    FW_REQUIRE(rows >= 0 && segments >= 0 && hidden > 0, "shortconv: bad sizes rows=%d segments=%d hidden=%d", rows, segments, hidden);
    FW_REQUIRE(kernel_size >= 2 && kernel_size <= CONV_MAX_KERNEL, "shortconv: kernel size %d outside 2..%d", kernel_size, CONV_MAX_KERNEL);
    FW_REQUIRE(segments <= rows, "shortconv: %d segments but only %d rows", segments, rows);
    FW_REQUIRE(rows <= 65535 && segments <= slots, "shortconv: rows=%d (max 65535), segments=%d, slots=%d", rows, segments, slots);
    if (rows == 0) return 0;
    FW_REQUIRE(segments >= 1, "shortconv: rows without a segment");
    hipStream_t s = (hipStream_t)stream;
    if (in_dtype == FW_F32 && out_dtype == FW_F32) launch<float, float>(bcx, out, taps, conv_bias, state, row_seg, seg_row0, seg_slot, rows, segments, hidden, kernel_size, s);
    else if (in_dtype == FW_F32 && out_dtype == FW_BF16) launch<float, bf16_t>(bcx, out, taps, conv_bias, state, row_seg, seg_row0, seg_slot, rows, segments, hidden, kernel_size, s);
    else if (in_dtype == FW_BF16 && out_dtype == FW_BF16) launch<bf16_t, bf16_t>(bcx, out, taps, conv_bias, state, row_seg, seg_row0, seg_slot, rows, segments, hidden, kernel_size, s);
    else FW_REQUIRE(false, "shortconv: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
    FW_LAUNCH_CHECK("shortconv");
    return 0;
}
