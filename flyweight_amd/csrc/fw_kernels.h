// Flat C ABI of the gfx950 kernel library. Every pointer is a device pointer unless a
// comment says otherwise; `stream` is a hipStream_t. Every function returns 0 on success
// and -1 on failure, after which fw_last_error() describes what was refused. Shapes are
// checked on the host before anything is launched; a kernel never runs on operands it
// was not written for.
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* fw_last_error(void);
int fw_abi_version(void);

// out[r][:] = table[ids[r]][:] * scale  (float32 out: the residual stream)
int fw_embed_rows(const void* table, int table_dtype, const int32_t* ids, float* out,
                  int rows, int hidden, int vocab, float scale, void* stream);

// x <- x * scale, then with cap > 0: x <- cap * tanh(x / cap); float32, in place
int fw_scale_softcap(float* x, long long count, float scale, float cap, void* stream);

// RMS norm of float32 rows: out[r] = x[src] * rsqrt(mean(x[src]^2) + eps) * w, where
// src = row_index ? row_index[r] : r.  one_centered: multiply by (1 + w) instead of w.
int fw_rmsnorm_rows(const float* x, const float* weight, void* out, int out_dtype,
                    const int32_t* row_index, int rows, int hidden, float eps,
                    int one_centered, void* stream);

// out = a[M][K] . w[N][K]^T (+ bias[N]); out_mode 0: store in out_dtype,
// 1: out (float32) += result (the residual sum).
int fw_gemm_generic(const void* a, int a_dtype, const void* w, int w_dtype, const float* bias,
                    void* out, int out_dtype, int out_mode, int M, int N, int K, void* stream);

// bfloat16 matrix products on the matrix cores, float32 accumulation. a [M][K], w [N][K], K a
// multiple of 8. mode 0: out = a . w^T (+ bias) stored as out_dtype; mode 1: out (float32) +=
// a . w^T (+ bias); mode 2 (SwiGLU): w is [2N][K], gate rows then up rows, out [M][N] bfloat16 =
// silu(a . gate^T) * (a . up^T). fw_gemm_skinny streams w once for M <= 64 (decode);
// fw_gemm_mfma tiles both operands through LDS (prompts).
int fw_gemm_skinny(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                   int M, int N, int K, void* stream);
int fw_gemm_mfma(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                 int M, int N, int K, void* stream);
// The prompt product with large tiles (256 x 256 or 256 x 192; storing products also 128 rows by as many columns,
// where that fills the chip better), for shapes that give enough of them to fill the chip
// (fw_gemm_mfma_big_tiles says how many, fw_gemm_mfma_big_plan also which).
int fw_gemm_mfma_big(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                     int M, int N, int K, void* stream);
int fw_gemm_mfma_big_tiles(int mode, int M, int N, int K);     // 0: the kernel does not take the shape
int fw_gemm_mfma_big_plan(int mode, int M, int N, int K, int* rows, int* columns);     // the same, and the tile's edges
// The prompt product with tiles of 128 rows and `columns` (128 or 64) columns whose four waves split
// K (half the LDS traffic per flop of fw_gemm_mfma's tiles), for outputs too narrow for the
// 256 x 256 tiles to fill the chip. Modes 0 and 1; K a multiple of 64 (fw_gemm_mfma_deep_tiles says
// 0 for shapes it does not take, else the number of tiles).
int fw_gemm_mfma_deep(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                      int M, int N, int K, int columns, void* stream);
int fw_gemm_mfma_deep_tiles(int mode, int M, int N, int K, int columns);
// fw_gemm_mfma with K cut into slices for products with fewer tiles than compute units (a few
// hundred rows, a narrow output). fw_gemm_mfma_split_plan says what a shape needs: bytes of
// workspace and int32 counters that are zero before the first call and are left zero (both 0: the
// shape is not cut, use fw_gemm_mfma). Calls that overlap on one device need their own of both.
int fw_gemm_mfma_split_plan(int mode, int M, int N, int K, size_t* workspace_bytes, int* counters);
int fw_gemm_mfma_split(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                       int M, int N, int K, void* workspace, size_t workspace_bytes, int* counters,
                       int counters_len, void* stream);
// The same product for 1..64 rows with K split over workgroups, so that a is not re-read by every
// few features (decode steps of 17..64 requests). fw_gemm_medium_plan says what a shape needs:
// bytes of workspace (0: none) and int32 counters (0: none) that are zero before the first call;
// the kernel leaves them zero. Calls that overlap on one device need their own of both.
// The accumulating product can leave what the norm after it needs, as fw_gemm_decode does
// (next_activations [M][N] bfloat16, next_squares [squares_rows][16 for M <= 16, else 64]), and
// any mode takes such prepared activations as a, with squares / squares_rows / eps.
int fw_gemm_medium_plan(int M, int N, int K, int mode, size_t* workspace_bytes, int* counters, int* squares_rows);
int fw_gemm_medium(const void* a, const void* w, int w_tiled, const float* bias, void* out, int out_dtype, int mode,
                   int M, int N, int K, void* workspace, size_t workspace_bytes, int* counters,
                   int counters_len, const float* next_norm_weight, int next_one_centered,
                   void* next_activations, float* next_squares, const float* squares, int squares_rows,
                   float eps, void* stream);

// Fused product for decode steps of up to 16 rows. prologue 0: a is bfloat16 [M][K]; 1: a is
// float32 rows, RMS-normed with norm_weight/eps (rows gathered through row_index if given) inside
// the kernel. epilogue 0: store out_dtype [M][N]; 1: float32 out += ; 2: SwiGLU, w = [gate rows;
// up rows], out bfloat16 [M][N]; 3: gated short convolution of single-token segments, w = [B rows;
// C rows; x rows] of N channels each, state [slots][N][kernel_size - 1] read and shifted.
// fw_gemm_decode_fits says whether a shape is taken (1) or must go to separate kernels (0).
// The accumulating epilogue can also leave what the NEXT norm needs: next_activations bfloat16
// [M][N] = x_new * w_next and next_squares [fw_gemm_decode_accumulate_tiles(N)][16], per-tile sums
// of x_new^2 of every row. A later call takes them with prologue 2 (a = those activations,
// squares/squares_tiles = those sums, eps) and applies the row's scale in its epilogue.
// w_tiled (here and in fw_gemm_medium): w is not row-major [rows][K] but lies in operand tiles,
// [rows / 16][K / 32][4][16][8]: tile (i, j) holds rows 16 i .. 16 i + 15, columns 32 j .. 32 j + 31 as
// 1 KB in the order in which a wave loads a matrix-core operand (lane = 16 * (column / 8) + row), so
// that a wave reads whole contiguous kilobytes (rows padded with zeros to a multiple of 16; K a
// multiple of 32). The same sums in the same order: the results are bit for bit those of row-major w.
int fw_gemm_decode(int prologue, const void* a, const float* norm_weight, const int32_t* row_index, float eps,
                   int one_centered, const void* w, int w_tiled, const float* bias, void* out, int out_dtype, int epilogue,
                   int M, int N, int K, const float* taps, const float* conv_bias, float* state,
                   const int32_t* seg_slot, int kernel_size, const float* next_norm_weight,
                   int next_one_centered, void* next_activations, float* next_squares, const float* squares,
                   int squares_tiles, void* stream);
int fw_gemm_decode_fits(int M, int N, int K, int epilogue);
int fw_gemm_decode_accumulate_tiles(int N);

// out[r][i] = silu(gu[r][i]) * gu[r][I + i]; the input may be float32 beside a bfloat16 output
int fw_swiglu(const void* gate_up, int in_dtype, void* out, int out_dtype, int rows, int intermediate,
              void* stream);

// cos/sin of position * inv_freq for every row: tables [rows][half]
int fw_rope_table(const int32_t* positions, const double* inv_freq, float* cos_out, float* sin_out,
                  int rows, int half, void* stream);

// Gated short convolution over a mixed batch. bcx [rows][3H] = (B | C | x); taps [H][L]
// oldest first; conv_bias [H] or null; state [slots][H][L-1] float32, oldest first.
// Row r belongs to segment row_seg[r]; segment s covers rows seg_row0[s]..seg_row0[s+1]
// and continues the sequence whose state lives in slot seg_slot[s].
int fw_shortconv(const void* bcx, int in_dtype, void* out, int out_dtype, const float* taps,
                 const float* conv_bias, float* state, const int32_t* row_seg, const int32_t* seg_row0,
                 const int32_t* seg_slot, int rows, int segments, int hidden, int kernel_size,
                 int slots, void* stream);

// Per-head RMS norm of q and k (weights may be null: no norm), half-split rotation of the
// first rotary_dim channels by the row's angle, q out, k and v appended to the pages of
// the row's segment. qkv [rows][(nh + 2 nkv) hd]. k_pages [pages][nkv][P][hd];
// v_pages [pages][nkv][hd][P]. block_table [segments][table_stride].
int fw_qk_norm_rope_kv_write(const void* qkv, int in_dtype, void* q_out, int dtype, const float* q_norm_weight,
                             const float* k_norm_weight, float eps, const float* cos_table,
                             const float* sin_table, int rotary_dim, void* k_pages, void* v_pages,
                             const int32_t* block_table, int table_stride, const int32_t* row_seg,
                             const int32_t* row_pos, int rows, int num_heads, int num_kv_heads,
                             int head_dim, int page_size, int num_pages, int write_kv, void* stream);

// Causal attention of every row over the cached keys 0..row_pos[r] (or the last `window`
// of them) of its segment. out [rows][nh*hd].
int fw_attention_generic(const void* q, void* out, int dtype, const void* k_pages,
                         const void* v_pages, const int32_t* block_table, int table_stride,
                         const int32_t* row_seg, const int32_t* row_pos, int rows, int num_heads,
                         int num_kv_heads, int head_dim, float scale, int window, int page_size,
                         int num_pages, void* stream);

// The same attention on the matrix cores, bfloat16 only, head_dim a multiple of 16 up to 256.
// Prompt portions: rows are cut into tiles of up to 64 that never span two segments (tile_seg,
// tile_row0), in any order: workgroups start in the order of the tiles, so the caller lists those
// that see the most keys first. heads_together: how many query heads of a kv group one workgroup takes, reading
// the keys and values once for all of them (1, or 4 up to head_dim 64: 4 pays behind a long
// context, 1 evens out a short causal prompt); 0: chosen from the shape alone.
int fw_attention_prefill(const void* q, void* out, const void* k_pages, const void* v_pages,
                         const int32_t* block_table, int table_stride, const int32_t* tile_seg,
                         const int32_t* tile_row0, int tiles, const int32_t* seg_row0, const int32_t* row_pos,
                         int rows, int num_heads, int num_kv_heads, int head_dim, float scale, int window,
                         int page_size, int num_pages, int heads_together, void* stream);
// Decode (one row per request): the keys are split between workgroups in runs of 4 pages and
// merged in order by the workgroup that finishes last. partial: float32 workspace
// [rows][heads][max_splits][head_dim + 4]; max_context: an upper bound on position + 1 of every
// row, known to the caller; tickets: rows * kv_heads * ceil(heads / kv_heads / 16) int32 counters,
// zero before the first call and left zero. decode_work: null, or one int32 on the device, the runs
// of 4 pages that all the rows of the step see together; with it a workgroup takes as many runs as
// bring the step down to about 512 workgroups.
int fw_attention_decode(const void* q, void* out, float* partial, int max_splits, int max_context,
                        const int32_t* decode_work, int* tickets, int tickets_len, const void* k_pages, const void* v_pages, const int32_t* block_table, int table_stride,
                        const int32_t* row_seg, const int32_t* row_pos, int rows, int num_heads, int num_kv_heads,
                        int head_dim, float scale, int window, int page_size, int num_pages, void* stream);

// The same with the work of fw_qk_norm_rope_kv_write in front of it, in one kernel: qkv float32
// [rows][(heads + 2 kv_heads) * head_dim] are the step's raw projections; every workgroup norms and
// rotates the query heads it works on, and the one whose pages hold the row's own position stores
// the new key (normed, rotated) and value (write_kv 0: they are in the cache already).
int fw_attention_decode_fused(const float* qkv, const float* q_norm_weight, const float* k_norm_weight, float eps,
                              const float* cos_table, const float* sin_table, int rotary_dim, int write_kv, void* out,
                              float* partial, int max_splits, int max_context, const int32_t* decode_work, int* tickets,
                              int tickets_len, void* k_pages,
                              void* v_pages, const int32_t* block_table, int table_stride, const int32_t* row_seg,
                              const int32_t* row_pos, int rows, int num_heads, int num_kv_heads, int head_dim, float scale,
                              int window, int page_size, int num_pages, void* stream);

// ids[r] = argmax(logits[r]) with ties to the lowest id, also written to also[r] if that is not null;
// advance[r] += 1 if that is not null; workspace: rows * 64 64-bit words
int fw_argmax_rows(const float* logits, int32_t* ids, int32_t* also, int32_t* advance, void* workspace, int rows, int vocab,
                   void* stream);

// fw_argmax_rows for callers that cannot allocate device memory (code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc) and so have no workspace to bring. It has no
// counterpart in the reference. The keys of the parts go to an array built into the library, one
// copy per GPU (512 KB, held until the process ends); at most fw_argmax_rows_static_max_rows() rows
// (1,024), more is refused with an error. The call allocates and frees nothing. Every call on a GPU
// uses that GPU's one array: calls that overlap there (several streams or threads) race; calls that
// follow each other in one stream do not. Same results as fw_argmax_rows.
int fw_argmax_rows_static(const float* logits, int32_t* ids, int32_t* also, int32_t* advance, int rows, int vocab,
                          void* stream);
int fw_argmax_rows_static_max_rows(void);

// The next token of every row, drawn on the device: settings float32 [rows][4] = temperature (0:
// greedy, the best candidate, ties to the lowest id), top_k (0: all candidates), top_p, min_p;
// states [rows]: the rows' xorshift64* generators, moved on by the rows that draw. also / advance
// as in fw_argmax_rows. Candidates are taken in (value descending, id ascending) order; the sums of
// a list of up to 1,024 candidates are float64, in that order, those of a longer one whole numbers
// (parts in 2^-46 fixed point at 65,536 logits).
int fw_sample_rows(const float* logits, const float* settings, unsigned long long* states, int32_t* ids, int32_t* also,
                   int32_t* advance, int rows, int vocab, void* stream);

int fw_fill_zero(void* ptr, long long bytes, void* stream);
// `pieces` runs of `bytes` each, `stride_bytes` apart, cleared in one launch
int fw_fill_zero_pieces(void* ptr, int pieces, long long bytes, long long stride_bytes, void* stream);

#ifdef __cplusplus
}
#endif
