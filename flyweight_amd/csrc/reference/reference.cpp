// Plain C++ references of the GPU kernels (see fw_reference.h).
#include "fw_reference.h"

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <limits>
#include <vector>

namespace {

thread_local char error_text[512] = "";

int fail(const char* format, ...) {
    va_list args;
    va_start(args, format);
    std::vsnprintf(error_text, sizeof(error_text), format, args);
    va_end(args);
    return -1;
}

// (value descending, id ascending), NaN below everything: the order of the engine's candidates
// (native/include/flyweight_v2_qwen_kernels.hpp:2391-2405 packs the same order into one key)
bool better(float a, int ia, float b, int ib) {
    const bool a_nan = std::isnan(a), b_nan = std::isnan(b);
    if (a_nan != b_nan) return b_nan;
    if (!a_nan && a != b) return a > b;
    return ia < ib;
}

double silu(double g) { return g / (1.0 + std::exp(-g)); }

}  // namespace

extern "C" {

const char* fwr_last_error(void) { return error_text; }

// native/include/flyweight_v2_native_kernels.hpp:98-151
int fwr_embed_rows(const float* table, const int32_t* ids, float* out, int rows, int hidden, int vocab, float scale) {
    for (int r = 0; r < rows; ++r) {
        if (ids[r] < 0 || ids[r] >= vocab) return fail("embed_rows: id %d of row %d is outside the table of %d", ids[r], r, vocab);
        for (int i = 0; i < hidden; ++i) out[(size_t)r * hidden + i] = table[(size_t)ids[r] * hidden + i] * scale;
    }
    return 0;
}

// native/include/flyweight_v2_qwen_kernels.hpp:425-447
int fwr_rmsnorm_rows(const float* x, const float* weight, float* out, const int32_t* row_index, int rows, int hidden,
                     float eps, int one_centered) {
    for (int r = 0; r < rows; ++r) {
        const float* row = x + (size_t)(row_index ? row_index[r] : r) * hidden;
        double squares = 0.0;
        for (int i = 0; i < hidden; ++i) squares += (double)row[i] * row[i];
        const double inv = 1.0 / std::sqrt(squares / hidden + (double)eps);
        for (int i = 0; i < hidden; ++i)
            out[(size_t)r * hidden + i] = (float)(row[i] * inv * ((one_centered ? 1.0 : 0.0) + weight[i]));
    }
    return 0;
}

// native/include/flyweight_v2_native_kernels.hpp:199-212 (out x rows, one dot product each)
int fwr_gemm(const float* a, const float* w, const float* bias, float* out, int M, int N, int K, int accumulate) {
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double sum = 0.0;
            for (int k = 0; k < K; ++k) sum += (double)a[(size_t)m * K + k] * w[(size_t)n * K + k];
            if (bias) sum += bias[n];
            float& target = out[(size_t)m * N + n];
            target = (float)((accumulate ? (double)target : 0.0) + sum);
        }
    return 0;
}

// native/src/v2_runtime.cpp:28797-28805 with silu_mul of native/include/flyweight_v2_qwen_kernels.hpp:1209-1223
int fwr_gemm_swiglu(const float* a, const float* w, float* out, int M, int N, int K) {
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double gate = 0.0, up = 0.0;
            for (int k = 0; k < K; ++k) {
                gate += (double)a[(size_t)m * K + k] * w[(size_t)n * K + k];
                up += (double)a[(size_t)m * K + k] * w[(size_t)(N + n) * K + k];
            }
            out[(size_t)m * N + n] = (float)(silu(gate) * up);
        }
    return 0;
}

int fwr_swiglu(const float* gate_up, float* out, int rows, int width) {
    for (int r = 0; r < rows; ++r)
        for (int i = 0; i < width; ++i)
            out[(size_t)r * width + i] = (float)(silu(gate_up[(size_t)r * 2 * width + i]) * gate_up[(size_t)r * 2 * width + width + i]);
    return 0;
}

// native/include/flyweight_v2_native_kernels.hpp:1302-1345: the ring of the last L - 1 values of B * x,
// oldest first; tap L - 1 multiplies the current token
int fwr_shortconv(const float* bcx, float* out, const float* taps, const float* conv_bias, float* state,
                  const int32_t* seg_row0, const int32_t* seg_slot, int segments, int hidden, int kernel_size, int slots) {
    if (kernel_size < 2) return fail("shortconv: kernel size %d must be at least 2", kernel_size);
    const int history = kernel_size - 1;
    std::vector<double> window(kernel_size);
    for (int seg = 0; seg < segments; ++seg) {
        const int slot = seg_slot[seg];
        if (slot < 0 || slot >= slots) return fail("shortconv: slot %d of segment %d is outside 0..%d", slot, seg, slots - 1);
        for (int c = 0; c < hidden; ++c) {
            float* ring = state + ((size_t)slot * hidden + c) * history;
            for (int row = seg_row0[seg]; row < seg_row0[seg + 1]; ++row) {
                const float* in = bcx + (size_t)row * 3 * hidden;
                const double newest = (double)in[c] * in[2 * hidden + c];       // B * x
                for (int j = 0; j < history; ++j) window[j] = ring[j];
                window[history] = newest;
                double y = 0.0;
                for (int j = 0; j < kernel_size; ++j) y += (double)taps[(size_t)c * kernel_size + j] * window[j];
                if (conv_bias) y += conv_bias[c];
                out[(size_t)row * hidden + c] = (float)(in[hidden + c] * y);    // C * y
                for (int j = 0; j + 1 < history; ++j) ring[j] = ring[j + 1];
                ring[history - 1] = (float)newest;
            }
        }
    }
    return 0;
}

// native/include/flyweight_v2_native_kernels.hpp:993-1008
int fwr_rope_table(const int32_t* positions, const double* inv_freq, float* cos_out, float* sin_out, int rows, int half) {
    for (int r = 0; r < rows; ++r)
        for (int i = 0; i < half; ++i) {
            const double angle = (double)positions[r] * inv_freq[i];
            cos_out[(size_t)r * half + i] = (float)std::cos(angle);
            sin_out[(size_t)r * half + i] = (float)std::sin(angle);
        }
    return 0;
}

// native/include/flyweight_v2_native_kernels.hpp:1015-1050 (norm, then rotation), store as
// native/include/flyweight_v2_qwen_kernels.hpp:11962-11975 but into pages
int fwr_qk_norm_rope_kv_write(const float* qkv, float* q_out, const float* q_norm_weight, const float* k_norm_weight,
                              float eps, const float* cos_table, const float* sin_table, int rotary_dim, float* k_pages,
                              float* v_pages, const int32_t* block_table, int table_stride, const int32_t* row_seg,
                              const int32_t* row_pos, int rows, int num_heads, int num_kv_heads, int head_dim,
                              int page_size, int num_pages, int write_kv) {
    if (rotary_dim % 2 || rotary_dim < 0 || rotary_dim > head_dim) return fail("qk_norm_rope: rotary_dim %d", rotary_dim);
    const int half = rotary_dim / 2, width = (num_heads + 2 * num_kv_heads) * head_dim;
    std::vector<double> head(head_dim);
    auto norm_and_rotate = [&](const float* in, const float* weight, int row) {
        double squares = 0.0;
        for (int d = 0; d < head_dim; ++d) squares += (double)in[d] * in[d];
        const double inv = weight ? 1.0 / std::sqrt(squares / head_dim + (double)eps) : 1.0;
        for (int d = 0; d < head_dim; ++d) head[d] = weight ? in[d] * inv * weight[d] : in[d];
        for (int i = 0; i < half; ++i) {
            const double c = cos_table[(size_t)row * half + i], s = sin_table[(size_t)row * half + i];
            const double a = head[i], b = head[i + half];
            head[i] = a * c - b * s;
            head[i + half] = b * c + a * s;
        }
    };
    for (int r = 0; r < rows; ++r) {
        const float* in = qkv + (size_t)r * width;
        for (int h = 0; h < num_heads; ++h) {
            norm_and_rotate(in + (size_t)h * head_dim, q_norm_weight, r);
            for (int d = 0; d < head_dim; ++d) q_out[((size_t)r * num_heads + h) * head_dim + d] = (float)head[d];
        }
        if (!write_kv) continue;
        const int pos = row_pos[r], page = block_table[(size_t)row_seg[r] * table_stride + pos / page_size];
        if (page < 0 || page >= num_pages) return fail("qk_norm_rope: row %d writes to page %d of %d", r, page, num_pages);
        const int slot = pos % page_size;
        for (int h = 0; h < num_kv_heads; ++h) {
            norm_and_rotate(in + (size_t)(num_heads + h) * head_dim, k_norm_weight, r);
            const float* v = in + (size_t)(num_heads + num_kv_heads + h) * head_dim;
            for (int d = 0; d < head_dim; ++d) {
                k_pages[(((size_t)page * num_kv_heads + h) * page_size + slot) * head_dim + d] = (float)head[d];
                v_pages[(((size_t)page * num_kv_heads + h) * head_dim + d) * page_size + slot] = v[d];
            }
        }
    }
    return 0;
}

// scores native/include/flyweight_v2_qwen_kernels.hpp:12570-12585, softmax and values :12664-12704,
// the causal rule native/include/flyweight_v2_native_kernels.hpp:4150-4176
int fwr_attention(const float* q, float* out, const float* k_pages, const float* v_pages, const int32_t* block_table,
                  int table_stride, const int32_t* row_seg, const int32_t* row_pos, int rows, int num_heads,
                  int num_kv_heads, int head_dim, float scale, int window, int page_size, int num_pages) {
    if (num_heads % num_kv_heads) return fail("attention: %d heads over %d kv heads", num_heads, num_kv_heads);
    const int group = num_heads / num_kv_heads;
    std::vector<double> scores, sum(head_dim);
    for (int r = 0; r < rows; ++r) {
        const int pos = row_pos[r];
        const int first = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
        const int32_t* table = block_table + (size_t)row_seg[r] * table_stride;
        for (int h = 0; h < num_heads; ++h) {
            const int kvh = h / group;
            const float* query = q + ((size_t)r * num_heads + h) * head_dim;
            scores.assign(pos - first + 1, 0.0);
            double highest = -std::numeric_limits<double>::infinity();
            for (int t = first; t <= pos; ++t) {
                const int page = table[t / page_size];
                if (page < 0 || page >= num_pages) return fail("attention: row %d reads page %d of %d", r, page, num_pages);
                const float* key = k_pages + (((size_t)page * num_kv_heads + kvh) * page_size + t % page_size) * head_dim;
                double dot = 0.0;
                for (int d = 0; d < head_dim; ++d) dot += (double)query[d] * key[d];
                scores[t - first] = dot * scale;
                highest = std::max(highest, scores[t - first]);
            }
            double total = 0.0;
            std::fill(sum.begin(), sum.end(), 0.0);
            for (int t = first; t <= pos; ++t) {
                const double p = std::exp(scores[t - first] - highest);
                total += p;
                const int page = table[t / page_size];
                const float* value = v_pages + ((size_t)page * num_kv_heads + kvh) * head_dim * page_size + t % page_size;
                for (int d = 0; d < head_dim; ++d) sum[d] += p * value[(size_t)d * page_size];
            }
            for (int d = 0; d < head_dim; ++d) out[((size_t)r * num_heads + h) * head_dim + d] = (float)(sum[d] / total);
        }
    }
    return 0;
}

int fwr_argmax_rows(const float* logits, int32_t* ids, int rows, int vocab) {
    for (int r = 0; r < rows; ++r) {
        const float* row = logits + (size_t)r * vocab;
        int best = 0;
        for (int i = 1; i < vocab; ++i)
            if (better(row[i], i, row[best], best)) best = i;
        ids[r] = best;
    }
    return 0;
}

// native/src/v2_runtime.cpp:29500-29566 (the candidates), 29686-29743 (the cuts and the draw),
// 29307-29314 (the generator): one row after the other, the whole row sorted, every sum in order
int fwr_sample_rows(const float* logits, const float* settings, unsigned long long* states, int32_t* ids, int rows, int vocab) {
    std::vector<int> order(vocab);
    std::vector<double> p(vocab);
    for (int r = 0; r < rows; ++r) {
        const float* row = logits + (size_t)r * vocab;
        const double temperature = settings[4 * r], top_p = settings[4 * r + 2], min_p = settings[4 * r + 3];
        const long long top_k = (long long)settings[4 * r + 1];
        for (int i = 0; i < vocab; ++i) order[i] = i;
        std::sort(order.begin(), order.end(), [&](int a, int b) { return better(row[a], a, row[b], b); });
        const int candidates = top_k > 0 && top_k < vocab ? (int)top_k : vocab;
        ids[r] = order[0];
        if (!(temperature > 0.0)) continue;       // (a single candidate is drawn like any list: the generator moves on)
        const double best = (double)row[order[0]] / temperature;
        double total = 0.0;
        for (int i = 0; i < candidates; ++i) {
            const double scaled = (double)row[order[i]] / temperature;
            p[i] = std::isfinite(scaled) ? std::exp(scaled - best) : 0.0;
            total += p[i];
        }
        if (!(total > 0.0) || !std::isfinite(total)) continue;
        int keep = candidates;
        if (top_p < 1.0) {
            double share = 0.0;
            for (int i = 0; i < candidates; ++i) {
                share += p[i] / total;
                if (share >= top_p) {
                    keep = i + 1;
                    break;
                }
            }
        }
        if (min_p > 0.0) {
            const double least = min_p * p[0];
            int kept = 1;
            while (kept < keep && p[kept] >= least) ++kept;
            keep = kept;
        }
        double kept_total = 0.0;
        for (int i = 0; i < keep; ++i) kept_total += p[i];
        unsigned long long x = states[r] ? states[r] : 0x9E3779B97F4A7C15ull;
        x ^= x >> 12;
        x ^= x << 25;
        x ^= x >> 27;
        states[r] = x;
        const double u = (double)((x * 2685821657736338717ull) >> 11) * (1.0 / 9007199254740992.0);
        const double threshold = u * kept_total;
        double running = 0.0;
        ids[r] = order[keep - 1];
        for (int i = 0; i < keep; ++i) {
            running += p[i];
            if (threshold <= running) {
                ids[r] = order[i];
                break;
            }
        }
    }
    return 0;
}

int fwr_scale_softcap(float* x, long long count, float scale, float cap) {
    for (long long i = 0; i < count; ++i) {
        double value = (double)x[i] * scale;
        if (cap > 0.0f) value = cap * std::tanh(value / cap);
        x[i] = (float)value;
    }
    return 0;
}

}  // extern "C"
