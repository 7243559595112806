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

// The same for kernels of up to four taps, eight consecutive rows of a channel per thread: the
// products B * x of the rows and of the three before them are formed once and slide through
// the taps in registers (a row's product is otherwise read by as many threads as there are taps),
// and the chain of dependent loads in front (segment of the row, its first row, its slot) is paid
// once for eight rows: with a thread per (row, channel) a prompt's 16 thousand workgroups were
// bound by that chain. The taps are aligned to the end of a window of four: tap j of a kernel of L
// taps sits at place j + 4 - L; the places in front are skipped. Sums in the order of the taps, as above.
#define CONV_TILE_ROWS 8
#define CONV_TILE_HISTORY 3
// C: channels side by side per thread (2: loads and stores of twice the width, where the model's width is
// even and the input float32: 2,048 rows of 2,048 channels 19.4 -> 16.2 us; with 4, 19.2 us; a channel's
// arithmetic is the same either way).
template <typename T, typename TO, int C>
__global__ __launch_bounds__(256) void shortconv_rows8_kernel(const T* __restrict__ bcx, TO* __restrict__ out,
                                                              const float* __restrict__ taps, const float* __restrict__ conv_bias,
                                                              const float* __restrict__ state, const int32_t* __restrict__ row_seg,
                                                              const int32_t* __restrict__ seg_row0, const int32_t* __restrict__ seg_slot,
                                                              int rows, int hidden, int kernel_size) {
    constexpr int R = CONV_TILE_ROWS, H = CONV_TILE_HISTORY;
    const int r0 = blockIdx.y * R;
    const int channel = (blockIdx.x * blockDim.x + threadIdx.x) * C;
    if (channel >= hidden) return;
    const int history = kernel_size - 1, unused = H - history;      // places of the window in front of tap 0
    // every row's segment and place in it, asked for together and first (two dependent loads each)
    int seg_of[R], offset_of[R];
#pragma unroll
    for (int i = 0; i < R; ++i) seg_of[i] = row_seg[r0 + i < rows ? r0 + i : rows - 1];
#pragma unroll
    for (int i = 0; i < R; ++i) offset_of[i] = r0 + i - seg_row0[seg_of[i]];
    // C values that lie side by side, as one load
    const auto load_run = [&](const T* from, float (&values)[C]) {
        if (C == 2 && sizeof(T) == 4) {
            const float2 pair = *reinterpret_cast<const float2*>(from);
            values[0] = pair.x;
            values[C - 1] = pair.y;
        } else {
#pragma unroll
            for (int c = 0; c < C; ++c) values[c] = load_as_float(from, c);
        }
    };
    // the products of rows r0 - 3 .. r0 + 7 (0 where that is no row of this step)
    float product[R + H][C], gate[R][C];
#pragma unroll
    for (int p = 0; p < R + H; ++p) {
        const int row = r0 - H + p;
        const bool valid = row >= 0 && row < rows;
        const T* source = bcx + (size_t)(valid ? row : 0) * 3 * hidden;
        float b[C], x[C];
        load_run(source + channel, b);
        load_run(source + 2 * (size_t)hidden + channel, x);
#pragma unroll
        for (int c = 0; c < C; ++c) product[p][c] = valid ? b[c] * x[c] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < R; ++i) load_run(bcx + (size_t)(r0 + i < rows ? r0 + i : rows - 1) * 3 * hidden + hidden + channel, gate[i]);
    float tap[H + 1][C], bias[C];
#pragma unroll
    for (int c = 0; c < C; ++c) {
#pragma unroll
        for (int place = 0; place <= H; ++place)
            tap[place][c] = place >= unused ? taps[(size_t)(channel + c) * kernel_size + (place - unused)] : 0.0f;
        bias[c] = conv_bias ? conv_bias[channel + c] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int row = r0 + i;
        if (row >= rows) break;
        const int seg = seg_of[i], offset_in_segment = offset_of[i];
        float result[C];
#pragma unroll
        for (int c = 0; c < C; ++c) {
            float y = 0.0f;
#pragma unroll
            for (int place = 0; place <= H; ++place) {
                if (place < unused) continue;       // in front of tap 0: not this kernel's (and never multiplied, not even by 0)
                float value = product[i + place][c];
                const int offset = offset_in_segment - H + place;       // where in the segment this place lies
                if (offset < 0)                                         // in front of the segment: the request's state
                    value = state[((size_t)seg_slot[seg] * hidden + channel + c) * history + history + offset];
                y = fmaf(tap[place][c], value, y);
            }
            y += bias[c];
            result[c] = gate[i][c] * y;
        }
        if (C == 2 && sizeof(TO) == 2) {
            const uint32_t packed = (uint32_t)float_to_bf16_bits(result[0]) | ((uint32_t)float_to_bf16_bits(result[C - 1]) << 16);
            *reinterpret_cast<uint32_t*>(out + (size_t)row * hidden + channel) = packed;
        } else {
#pragma unroll
            for (int c = 0; c < C; ++c) store_from_float(out, (size_t)row * hidden + channel + c, result[c]);
        }
    }
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
    if (kernel_size <= CONV_TILE_HISTORY + 1 && rows >= 4 * CONV_TILE_ROWS) {
        if (hidden % 2 == 0 && sizeof(T) == 4)
            shortconv_rows8_kernel<T, TO, 2><<<dim3(fw_ceil_div(hidden / 2, 256), fw_ceil_div(rows, CONV_TILE_ROWS)), 256, 0, stream>>>(
                (const T*)bcx, (TO*)out, taps, conv_bias, state, row_seg, seg_row0, seg_slot, rows, hidden, kernel_size);
        else
            shortconv_rows8_kernel<T, TO, 1><<<dim3(bx, fw_ceil_div(rows, CONV_TILE_ROWS)), 256, 0, stream>>>(
                (const T*)bcx, (TO*)out, taps, conv_bias, state, row_seg, seg_row0, seg_slot, rows, hidden, kernel_size);
    } else
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
    // (segments may outnumber slots: rows that only fill a recorded step up share one spare slot)
    FW_REQUIRE(rows <= 65535 && slots >= 1, "shortconv: rows=%d (max 65535), segments=%d, slots=%d", rows, segments, slots);
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
