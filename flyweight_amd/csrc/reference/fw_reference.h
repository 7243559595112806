// A plain C++ reference beside every GPU kernel: the same operation on float32 arrays in host
// memory, written for reading, not for speed: one loop nest per formula, sums in double. It is the
// oracle that needs no GPU: the CPU tests hold it against the tests' numpy model, the GPU tests hold
// the kernels against it at sizes other than the engine's. Each function names the kernel it stands
// beside (csrc/*.hip) and where the reference engine computes the same thing. Nothing of the
// product path calls it. All functions return 0, or -1 with the reason in fwr_last_error().
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* fwr_last_error(void);

// elementwise.hip embed_rows: out[r][:] = table[ids[r]][:] * scale
int fwr_embed_rows(const float* table, const int32_t* ids, float* out, int rows, int hidden, int vocab, float scale);
// elementwise.hip rmsnorm_rows: out[r] = x[src] * rsqrt(mean(x[src]^2) + eps) * (w or 1 + w); src = row_index[r] or r
int fwr_rmsnorm_rows(const float* x, const float* weight, float* out, const int32_t* row_index, int rows, int hidden,
                     float eps, int one_centered);
// gemm_*.hip: out[m][n] = (accumulate ? out[m][n] : 0) + sum_k a[m][k] w[n][k] + bias[n]
int fwr_gemm(const float* a, const float* w, const float* bias, float* out, int M, int N, int K, int accumulate);
// the SwiGLU epilogue: w holds N gate rows, then N up rows; out[m][n] = silu(a . gate_n) * (a . up_n)
int fwr_gemm_swiglu(const float* a, const float* w, float* out, int M, int N, int K);
// elementwise.hip swiglu: gate_up [rows][2 * width] (gate, then up) -> out [rows][width]
int fwr_swiglu(const float* gate_up, float* out, int rows, int width);
// shortconv.hip: bcx [rows][3H] = (B, C, x); per segment the causal depthwise filter over B * x,
// continuing from and updating state [slots][H][L - 1] (oldest first); out = C * (y + bias)
int fwr_shortconv(const float* bcx, float* out, const float* taps, const float* conv_bias, float* state,
                  const int32_t* seg_row0, const int32_t* seg_slot, int segments, int hidden, int kernel_size, int slots);
// elementwise.hip rope_table: cos, sin [rows][half] of positions[r] * inv_freq[i] (the angle in double)
int fwr_rope_table(const int32_t* positions, const double* inv_freq, float* cos_out, float* sin_out, int rows, int half);
// attention_generic.hip qk_norm_rope_kv_write: qkv [rows][(nh + 2 nkv) hd]; per head RMS norm of q and k
// (weights [hd], null: none), half-split rotation of the first rotary_dim channels, k and v stored at
// (page of block_table[row_seg[r]][pos / page_size], pos % page_size); q_out [rows][nh * hd].
// K pages [pages][nkv][page_size][hd], V pages [pages][nkv][hd][page_size].
int fwr_qk_norm_rope_kv_write(const float* qkv, float* q_out, const float* q_norm_weight, const float* k_norm_weight,
                              float eps, const float* cos_table, const float* sin_table, int rotary_dim, float* k_pages,
                              float* v_pages, const int32_t* block_table, int table_stride, const int32_t* row_seg,
                              const int32_t* row_pos, int rows, int num_heads, int num_kv_heads, int head_dim,
                              int page_size, int num_pages, int write_kv);
// attention_generic.hip / attention_mfma.hip: row r at position p sees keys max(0, p - window + 1) .. p of its
// sequence (window 0: all); softmax with the maximum subtracted; head h reads kv head h / (nh / nkv)
int fwr_attention(const float* q, float* out, const float* k_pages, const float* v_pages, const int32_t* block_table,
                  int table_stride, const int32_t* row_seg, const int32_t* row_pos, int rows, int num_heads,
                  int num_kv_heads, int head_dim, float scale, int window, int page_size, int num_pages);
// elementwise.hip argmax / top-k: order by value descending, then id ascending; NaN last
int fwr_argmax_rows(const float* logits, int32_t* ids, int rows, int vocab);
// sampling.hip: settings [rows][4] = temperature (0: greedy), top_k (0: all), top_p, min_p; states: the
// rows' xorshift64* generators, moved on by the rows that draw
int fwr_sample_rows(const float* logits, const float* settings, unsigned long long* states, int32_t* ids, int rows, int vocab);
// elementwise.hip scale_softcap: x * scale, then with cap > 0 cap * tanh(x / cap)
int fwr_scale_softcap(float* x, long long count, float scale, float cap);

#ifdef __cplusplus
}
#endif
