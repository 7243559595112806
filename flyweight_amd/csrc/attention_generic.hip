// Attention over the paged cache, generic variants in float32 arithmetic.
//
// Cache layout (one K and one V pool per cache entry, pages of P = 64 tokens, the width
// of a wavefront): K [page][kv_head][P][head_dim] keeps a key's channels together, which
// is the order QK^T reduces over; V [page][kv_head][head_dim][P] keeps a channel's tokens
// together, which is the order PV reduces over. A token at position t of a sequence lives
// in page block_table[t / P] at offset t % P. (The reference's unwired paging primitive
// uses the same P and a page-major layout, native/src/paged_kv.h:48-83.)
#include "fw_common.h"
#include "fw_kernels.h"

#define ATTN_PAGE 64
#define ATTN_MAX_HEAD_DIM 256

// One wave per (row, head-vector). Head-vectors 0..nh-1 are queries, nh..nh+nkv-1 keys,
// the rest values. Per-head RMS norm then half-split rotation: channel i pairs with
// i + rotary_dim/2; out[i] = a cos - b sin, out[i + half] = b cos + a sin
// (native/include/flyweight_v2_native_kernels.hpp:1015-1050). Values are stored untouched.
template <typename TI, typename T>
__global__ __launch_bounds__(64) void qk_norm_rope_kv_write_kernel(
    const TI* __restrict__ qkv, T* __restrict__ q_out, const float* __restrict__ q_norm_weight,
    const float* __restrict__ k_norm_weight, float eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int rotary_dim, T* __restrict__ k_pages, T* __restrict__ v_pages,
    const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ row_seg,
    const int32_t* __restrict__ row_pos, int num_heads, int num_kv_heads, int head_dim) {
    __shared__ float normed[ATTN_MAX_HEAD_DIM];
    const int row = blockIdx.x;
    const int vec = blockIdx.y;
    const int lane = threadIdx.x;
    const int width = (num_heads + 2 * num_kv_heads) * head_dim;
    const TI* source = qkv + (size_t)row * width + (size_t)vec * head_dim;
    const int pos = row_pos[row];
    const int page = block_table[(size_t)row_seg[row] * table_stride + pos / ATTN_PAGE];
    const int slot = pos % ATTN_PAGE;

    if (vec >= num_heads + num_kv_heads) {      // value head: transposed store
        const int kvh = vec - num_heads - num_kv_heads;
        T* dest = v_pages + ((size_t)page * num_kv_heads + kvh) * head_dim * ATTN_PAGE;
        for (int d = lane; d < head_dim; d += 64) store_from_float(dest, (size_t)d * ATTN_PAGE + slot, load_as_float(source, d));
        return;
    }
    const bool is_query = vec < num_heads;
    const float* weight = is_query ? q_norm_weight : k_norm_weight;
    float inv = 1.0f;
    if (weight) {
        float sum = 0.0f;
        for (int d = lane; d < head_dim; d += 64) {
            const float v = load_as_float(source, d);
            sum += v * v;
        }
        sum = wave_sum(sum);
        inv = rsqrtf(sum / (float)head_dim + eps);
    }
    for (int d = lane; d < head_dim; d += 64) {
        const float v = load_as_float(source, d);
        normed[d] = weight ? v * inv * weight[d] : v;
    }
    __syncthreads();
    const int half = rotary_dim / 2;
    T* dest = is_query ? q_out + ((size_t)row * num_heads + vec) * head_dim
                       : k_pages + (((size_t)page * num_kv_heads + (vec - num_heads)) * ATTN_PAGE + slot) * head_dim;
    for (int d = lane; d < head_dim; d += 64) {
        float value = normed[d];
        if (d < rotary_dim) {
            const int pair = d < half ? d : d - half;
            const float other = normed[d < half ? d + half : d - half];
            const float c = cos_table[(size_t)row * half + pair];
            const float s = sin_table[(size_t)row * half + pair];
            value = d < half ? value * c - other * s : value * c + other * s;
        }
        store_from_float(dest, d, value);
    }
}

// The same for heads of up to 64 channels (a channel per lane), eight rows of one head-vector per
// wave: what the wave reads for its eight rows is asked for together, so the chain of dependent
// loads in front (position and segment of the row, its page) is paid once for eight rows. A prompt
// of 2,048 rows has a hundred thousand (row, head-vector) pairs; as waves of one pair each they
// were bound by that chain. The rotation's partner channel comes from the partner lane. The same
// arithmetic in the same order as above.
#define QK_ROWS 8
template <typename TI, typename T>
__global__ __launch_bounds__(64) void qk_norm_rope_kv_write_rows_kernel(
    const TI* __restrict__ qkv, T* __restrict__ q_out, const float* __restrict__ q_norm_weight,
    const float* __restrict__ k_norm_weight, float eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int rotary_dim, T* __restrict__ k_pages, T* __restrict__ v_pages,
    const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ row_seg,
    const int32_t* __restrict__ row_pos, int num_heads, int num_kv_heads, int head_dim, int rows) {
    const int r0 = blockIdx.x * QK_ROWS;
    const int vec = blockIdx.y;
    const int lane = threadIdx.x;
    const int width = (num_heads + 2 * num_kv_heads) * head_dim;
    const bool active = lane < head_dim;
    const bool is_value = vec >= num_heads + num_kv_heads, is_query = vec < num_heads;
    const float* weight = is_value ? nullptr : (is_query ? q_norm_weight : k_norm_weight);
    const int half = rotary_dim / 2;
    const bool turned = !is_value && lane < rotary_dim;
    const int pair = lane < half ? lane : lane - half;
    int row_of[QK_ROWS], pos[QK_ROWS], page[QK_ROWS];
    float v[QK_ROWS], c[QK_ROWS], sn[QK_ROWS];
#pragma unroll
    for (int i = 0; i < QK_ROWS; ++i) {
        row_of[i] = r0 + i < rows ? r0 + i : rows - 1;
        pos[i] = row_pos[row_of[i]];
        page[i] = row_seg[row_of[i]];
    }
#pragma unroll
    for (int i = 0; i < QK_ROWS; ++i) {
        v[i] = load_as_float(qkv + (size_t)row_of[i] * width + (size_t)vec * head_dim, active ? lane : 0);
        c[i] = turned ? cos_table[(size_t)row_of[i] * half + pair] : 1.0f;
        sn[i] = turned ? sin_table[(size_t)row_of[i] * half + pair] : 0.0f;
    }
    const float w = (weight && active) ? weight[lane] : 1.0f;
#pragma unroll
    for (int i = 0; i < QK_ROWS; ++i) page[i] = block_table[(size_t)page[i] * table_stride + pos[i] / ATTN_PAGE];
    if (is_value && sizeof(T) == 2) {
        // Eight rows that follow each other in one page, the first at a slot that is a multiple of eight (a
        // prompt portion that begins at such a position): a channel's eight values are 16 bytes side by side
        // in the transposed page and leave as one store instead of eight of 2 bytes.
        bool together = r0 + QK_ROWS <= rows && pos[0] % 8 == 0;
#pragma unroll
        for (int i = 1; i < QK_ROWS; ++i) together = together && page[i] == page[0] && pos[i] == pos[0] + i;
        if (together) {
            const int kvh = vec - num_heads - num_kv_heads;
            T* dest = v_pages + ((size_t)page[0] * num_kv_heads + kvh) * head_dim * ATTN_PAGE;
            uint32_t packed[QK_ROWS / 2];
#pragma unroll
            for (int i = 0; i < QK_ROWS / 2; ++i)
                packed[i] = (uint32_t)float_to_bf16_bits(v[2 * i]) | ((uint32_t)float_to_bf16_bits(v[2 * i + 1]) << 16);
            if (active) {
                uint32_t* to = reinterpret_cast<uint32_t*>(dest + (size_t)lane * ATTN_PAGE + pos[0] % ATTN_PAGE);
                typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
                *reinterpret_cast<u32x4_t*>(to) = u32x4_t{packed[0], packed[1], packed[2], packed[3]};
            }
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < QK_ROWS; ++i) {
        if (r0 + i >= rows) break;
        const int slot = pos[i] % ATTN_PAGE;
        if (is_value) {      // value head: transposed store
            const int kvh = vec - num_heads - num_kv_heads;
            T* dest = v_pages + ((size_t)page[i] * num_kv_heads + kvh) * head_dim * ATTN_PAGE;
            if (active) store_from_float(dest, (size_t)lane * ATTN_PAGE + slot, v[i]);
            continue;
        }
        float value = active ? v[i] : 0.0f;
        if (weight) {
            const float sum = wave_sum(value * value);
            const float inv = rsqrtf(sum / (float)head_dim + eps);
            value = value * inv * w;
        }
        const float other = __shfl(value, lane < half ? lane + half : lane - half, 64);
        if (lane < rotary_dim) value = lane < half ? value * c[i] - other * sn[i] : value * c[i] + other * sn[i];
        T* dest = is_query ? q_out + ((size_t)row_of[i] * num_heads + vec) * head_dim
                           : k_pages + (((size_t)page[i] * num_kv_heads + (vec - num_heads)) * ATTN_PAGE + slot) * head_dim;
        if (active) store_from_float(dest, lane, value);
    }
}

extern "C" int fw_qk_norm_rope_kv_write(const void* qkv, int in_dtype, void* q_out, int dtype, const float* q_norm_weight,
                                        const float* k_norm_weight, float eps, const float* cos_table,
                                        const float* sin_table, int rotary_dim, void* k_pages, void* v_pages,
                                        const int32_t* block_table, int table_stride, const int32_t* row_seg,
                                        const int32_t* row_pos, int rows, int num_heads, int num_kv_heads,
                                        int head_dim, int page_size, int num_pages, int write_kv, void* stream) {
    FW_REQUIRE(rows >= 0 && num_heads > 0 && num_kv_heads > 0, "qk_norm_rope: bad sizes rows=%d heads=%d kv_heads=%d", rows, num_heads, num_kv_heads);
    FW_REQUIRE(head_dim > 0 && head_dim <= ATTN_MAX_HEAD_DIM, "qk_norm_rope: head_dim %d outside 1..%d", head_dim, ATTN_MAX_HEAD_DIM);
    FW_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0, "qk_norm_rope: rotary_dim %d must be even and at most head_dim %d", rotary_dim, head_dim);
    FW_REQUIRE(rotary_dim == 0 || (cos_table && sin_table), "qk_norm_rope: rotation asked for without tables");
    FW_REQUIRE(page_size == ATTN_PAGE, "qk_norm_rope: page size must be %d, got %d", ATTN_PAGE, page_size);
    FW_REQUIRE(num_pages > 0 && table_stride > 0, "qk_norm_rope: empty cache (pages=%d, table stride=%d)", num_pages, table_stride);
    FW_REQUIRE((q_norm_weight == nullptr) == (k_norm_weight == nullptr), "qk_norm_rope: q and k norm weights come together");
    FW_REQUIRE(rows <= 1 << 20, "qk_norm_rope: too many rows (%d)", rows);
    if (rows == 0) return 0;
    const int vectors = write_kv ? num_heads + 2 * num_kv_heads : num_heads;
    FW_REQUIRE(vectors <= 65535, "qk_norm_rope: too many heads (%d)", vectors);
    dim3 grid(rows, vectors);
    hipStream_t s = (hipStream_t)stream;
    if (head_dim <= 64 && rows >= 8 * QK_ROWS) {    // a prompt's rows, eight to a wave
        dim3 by_rows((rows + QK_ROWS - 1) / QK_ROWS, vectors);
#define FW_QK_ROWS_LAUNCH(TI, T)                                                                                     \
    qk_norm_rope_kv_write_rows_kernel<TI, T><<<by_rows, 64, 0, s>>>(                                                 \
        (const TI*)qkv, (T*)q_out, q_norm_weight, k_norm_weight, eps, cos_table, sin_table, rotary_dim, (T*)k_pages, \
        (T*)v_pages, block_table, table_stride, row_seg, row_pos, num_heads, num_kv_heads, head_dim, rows)
        if (in_dtype == FW_F32 && dtype == FW_F32) FW_QK_ROWS_LAUNCH(float, float);
        else if (in_dtype == FW_F32 && dtype == FW_BF16) FW_QK_ROWS_LAUNCH(float, bf16_t);
        else if (in_dtype == FW_BF16 && dtype == FW_BF16) FW_QK_ROWS_LAUNCH(bf16_t, bf16_t);
        else FW_REQUIRE(false, "qk_norm_rope: unsupported dtypes in=%d out=%d", in_dtype, dtype);
#undef FW_QK_ROWS_LAUNCH
        FW_LAUNCH_CHECK("qk_norm_rope_kv_write");
        return 0;
    }
#define FW_QK_LAUNCH(TI, T)                                                                                          \
    qk_norm_rope_kv_write_kernel<TI, T><<<grid, 64, 0, s>>>(                                                         \
        (const TI*)qkv, (T*)q_out, q_norm_weight, k_norm_weight, eps, cos_table, sin_table, rotary_dim, (T*)k_pages, \
        (T*)v_pages, block_table, table_stride, row_seg, row_pos, num_heads, num_kv_heads, head_dim)
    if (in_dtype == FW_F32 && dtype == FW_F32) FW_QK_LAUNCH(float, float);
    else if (in_dtype == FW_F32 && dtype == FW_BF16) FW_QK_LAUNCH(float, bf16_t);
    else if (in_dtype == FW_BF16 && dtype == FW_BF16) FW_QK_LAUNCH(bf16_t, bf16_t);
    else FW_REQUIRE(false, "qk_norm_rope: unsupported dtypes in=%d out=%d", in_dtype, dtype);
#undef FW_QK_LAUNCH
    FW_LAUNCH_CHECK("qk_norm_rope_kv_write");
    return 0;
}

// One wave per (row, head). Keys are visited page by page, one key per lane; softmax is
// the running-maximum form in float32 (scores, maximum, exponentials, sum and the weighted
// sum of values all float32), as the reference's decode fallback computes it in two
// passes (native/include/flyweight_v2_qwen_kernels.hpp:12570-12585,12664-12704). The order
// of every sum depends only on the row's position and the window, never on the batch.
template <typename T>
__global__ __launch_bounds__(64) void attention_generic_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ row_seg,
    const int32_t* __restrict__ row_pos, int num_heads, int num_kv_heads, int head_dim, float scale, int window) {
    __shared__ float qs[ATTN_MAX_HEAD_DIM];
    __shared__ float ps[ATTN_PAGE];
    const int row = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int kvh = head / (num_heads / num_kv_heads);
    const int pos = row_pos[row];
    const int32_t* table = block_table + (size_t)row_seg[row] * table_stride;
    const T* query = q + ((size_t)row * num_heads + head) * head_dim;
    for (int d = lane; d < head_dim; d += 64) qs[d] = load_as_float(query, d);
    __syncthreads();
    const int first = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
    float running_max = -INFINITY, running_sum = 0.0f;
    float acc[ATTN_MAX_HEAD_DIM / 64] = {};
    for (int tile = first / ATTN_PAGE; tile <= pos / ATTN_PAGE; ++tile) {
        const int page = table[tile];
        const int t = tile * ATTN_PAGE + lane;
        const bool valid = t >= first && t <= pos;
        float score = -INFINITY;
        if (valid) {
            const T* key = k_pages + (((size_t)page * num_kv_heads + kvh) * ATTN_PAGE + lane) * head_dim;
            float dot = 0.0f;
            for (int d = 0; d < head_dim; ++d) dot = fmaf(qs[d], load_as_float(key, d), dot);
            score = dot * scale;
        }
        const float new_max = fmaxf(running_max, wave_max(score));
        const float p = valid ? expf(score - new_max) : 0.0f;
        const float alpha = expf(running_max - new_max);
        running_sum = running_sum * alpha + wave_sum(p);
        running_max = new_max;
        ps[lane] = p;
        __syncthreads();
        const int lo = first - tile * ATTN_PAGE > 0 ? first - tile * ATTN_PAGE : 0;
        const int hi = pos - tile * ATTN_PAGE < ATTN_PAGE - 1 ? pos - tile * ATTN_PAGE : ATTN_PAGE - 1;
#pragma unroll
        for (int j = 0; j < ATTN_MAX_HEAD_DIM / 64; ++j) {
            const int d = lane + 64 * j;
            if (d < head_dim) {
                const T* value = v_pages + (((size_t)page * num_kv_heads + kvh) * head_dim + d) * ATTN_PAGE;
                float sum = 0.0f;
                for (int s = lo; s <= hi; ++s) sum = fmaf(ps[s], load_as_float(value, s), sum);
                acc[j] = acc[j] * alpha + sum;
            }
        }
        __syncthreads();
    }
    T* dest = out + ((size_t)row * num_heads + head) * head_dim;
#pragma unroll
    for (int j = 0; j < ATTN_MAX_HEAD_DIM / 64; ++j) {
        const int d = lane + 64 * j;
        if (d < head_dim) store_from_float(dest, d, acc[j] / running_sum);
    }
}

extern "C" int fw_attention_generic(const void* q, void* out, int dtype, const void* k_pages,
                                    const void* v_pages, const int32_t* block_table, int table_stride,
                                    const int32_t* row_seg, const int32_t* row_pos, int rows, int num_heads,
                                    int num_kv_heads, int head_dim, float scale, int window, int page_size,
                                    int num_pages, void* stream) {
    FW_REQUIRE(rows >= 0 && num_heads > 0 && num_kv_heads > 0 && num_heads % num_kv_heads == 0,
               "attention: heads %d must be a positive multiple of kv heads %d", num_heads, num_kv_heads);
    FW_REQUIRE(head_dim > 0 && head_dim <= ATTN_MAX_HEAD_DIM, "attention: head_dim %d outside 1..%d", head_dim, ATTN_MAX_HEAD_DIM);
    FW_REQUIRE(page_size == ATTN_PAGE, "attention: page size must be %d, got %d", ATTN_PAGE, page_size);
    FW_REQUIRE(window >= 0, "attention: window must be 0 (all keys) or positive, got %d", window);
    FW_REQUIRE(num_pages > 0 && table_stride > 0, "attention: empty cache (pages=%d, table stride=%d)", num_pages, table_stride);
    FW_REQUIRE(rows <= 1 << 20 && num_heads <= 65535, "attention: too many rows/heads (%d, %d)", rows, num_heads);
    if (rows == 0) return 0;
    dim3 grid(rows, num_heads);
    if (dtype == FW_F32)
        attention_generic_kernel<float><<<grid, 64, 0, (hipStream_t)stream>>>(
            (const float*)q, (float*)out, (const float*)k_pages, (const float*)v_pages, block_table, table_stride,
            row_seg, row_pos, num_heads, num_kv_heads, head_dim, scale, window);
    else if (dtype == FW_BF16)
        attention_generic_kernel<bf16_t><<<grid, 64, 0, (hipStream_t)stream>>>(
            (const bf16_t*)q, (bf16_t*)out, (const bf16_t*)k_pages, (const bf16_t*)v_pages, block_table, table_stride,
            row_seg, row_pos, num_heads, num_kv_heads, head_dim, scale, window);
    else
        FW_REQUIRE(false, "attention: unknown dtype %d", dtype);
    FW_LAUNCH_CHECK("attention_generic");
    return 0;
}
