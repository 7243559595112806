// Fused matrix products for decode steps of up to 16 rows.
//
// A decode step of a small batch is a chain of short kernels, each of which costs a few
// microseconds to start and to drain whatever it computes, while the weights themselves
// stream in well under a millisecond. This kernel folds the neighbours of each matrix product
// into it, without putting anything in front of the stream of W:
//
//  prologue   none: a is bfloat16 [M][K];  or RMS norm of float32 rows x (optionally gathered
//             through row_index). The norm is not applied before the product: with
//             h = x * r * w (r the row's 1/rms, w the norm weight) the product is
//             r * sum_k bf16(x_k w_k) W_nk, so every wave turns its own slices of x into operands
//             as it goes (rounded to bfloat16 before the scale instead of after it: the same
//             relative rounding), adds up x^2 of what it reads, and the row's r multiplies the
//             sums in the epilogue;
//             or "pre-normed": the kernel that last added to the residual stream (the
//             accumulating epilogue below) also left bf16(x * w_next) and, per tile of features,
//             the sum of x^2 of every row; this kernel reads those as plain bfloat16 activations
//             and forms the row's r from the partial sums, so the norm costs almost nothing;
//  product    W streams once from global memory straight into v_mfma_f32_16x16x32_bf16
//             operands, K split over the waves of the workgroup in chunks of 128;
//  epilogue   store | add into the float32 residual stream (optionally leaving the pre-normed
//             activations for the next norm, see above) | SwiGLU (tiles: gate, up) |
//             gated short convolution for single-token segments (tiles: B, C, x of the same
//             channels; reads and shifts the request's state; see shortconv.hip).
//
// A workgroup owns 16 (or 8, so that narrow outputs still fill the chip) features per tile and
// may take several tiles in turn. Partial sums (and sums of squares) meet in LDS and are added
// in wave order: results do not depend on timing or on what else is in the batch.
#include "fw_common.h"
#include "fw_kernels.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

#define DG_CHUNK 128
#define DG_MAX_TAPS 16

enum { DG_STORE = 0, DG_ACCUMULATE = 1, DG_SWIGLU = 2, DG_CONV = 3 };

struct DecodeGemmArgs {
    const void* a;              // bfloat16 [M][K] (no prologue) or float32 rows (norm prologue)
    const float* norm_weight;   // [K], norm prologue only
    const int32_t* row_index;   // gather of x rows, or null
    float eps;
    int one_centered;
    const uint16_t* w;          // [tiles * tile_stride ...][K], or the same in operand tiles (w_tiled)
    int w_tiled;                // W lies in tiles of 16 rows x 32 columns, each 1 KB in the order of a wave's operand load
    const float* bias;          // per W row, or null
    void* out;
    int M, N, K;                // N: features per tile kind (output width)
    int tile_stride;            // W rows between the tiles of one feature (SwiGLU, conv); 0 otherwise
    // convolution epilogue
    const float* taps;          // [N][kernel_size]
    const float* conv_bias;     // [N] or null
    float* state;               // [slots][N][kernel_size - 1]
    const int32_t* seg_slot;    // [M]
    int kernel_size;
    // accumulating epilogue: what the next norm will need (all null: nothing is left)
    const float* next_norm_weight;  // [N]
    int next_one_centered;
    uint16_t* next_activations;     // bfloat16 [M][N] = x_new * (w_next or 1 + w_next)
    float* next_squares;            // [tiles][16]: sum over the tile's features of x_new^2 per row
    // pre-normed prologue
    const float* squares;           // [squares_tiles][16], left by the kernel above
    int squares_tiles;
};

__device__ __forceinline__ float dg_silu(float g) {
    if (g >= 0.0f) return g / (1.0f + __expf(-g));
    const float e = __expf(g);
    return g * e / (1.0f + e);
}

template <int RT, int WAVES, int ROWS, int PRO, int EPI, typename TO, bool WT>
__global__ __launch_bounds__(WAVES * 64) void decode_gemm_kernel(const DecodeGemmArgs p, const int num_tiles) {
    __shared__ float partial[WAVES][RT][64][4];
    __shared__ float squares[WAVES][16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r16 = lane & 15, g = lane >> 4;
    const int M = p.M, N = p.N, K = p.K;
    constexpr bool TILED = EPI == DG_SWIGLU || EPI == DG_CONV;    // the tiles of a workgroup are kinds of one feature

    const bool a_ok = r16 < M;
    const int a_index = a_ok ? (PRO == 1 && p.row_index ? p.row_index[r16] : r16) : 0;     // (pre-normed rows are never gathered)
    // pointers to the rows; the column (k + 8 g) is added at each load so that it can be clamped
    const uint16_t* a_bf16 = static_cast<const uint16_t*>(p.a) + (size_t)a_index * K;
    const float* a_f32 = static_cast<const float*>(p.a) + (size_t)a_index * K;
    const float* norm_w = p.norm_weight;
    const float one = p.one_centered ? 1.0f : 0.0f;

    // Pre-normed rows: this lane's share of the partial sums of x^2 that the rows' producer left
    // (the waves and the four lanes of a row split the tiles in a fixed order). The loads are
    // issued here, in front of the stream of W, and their values are first used behind the
    // product: a wave issues in order, so a sum formed here would hold W back by a round trip.
    constexpr int SQ_HELD = 8;
    float held[SQ_HELD];
    float prepared_square = 0.0f;
    bool prepared = false;
    if (PRO == 2) {
        const float* from = p.squares + r16;        // a row of 16 per tile: every lane's column exists
        const int last = p.squares_tiles - 1;
#pragma unroll
        for (int u = 0; u < SQ_HELD; ++u) {
            const int t = wave * 4 + g + u * WAVES * 4;
            held[u] = from[(size_t)(t < last ? t : last) * 16];
        }
    }
    // The convolution's request slot, asked for before anything else needs waiting for.
    int conv_slot = 0;
    if (EPI == DG_CONV) conv_slot = p.seg_slot[r16 < M ? r16 : 0];
    for (int tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
        const uint16_t* w_row[RT];
        bool w_ok[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const int feature = tile * ROWS + (ROWS == 16 ? r16 : (r16 & 7));
            const int n = TILED ? feature + rt * p.tile_stride : feature + rt * ROWS * num_tiles;
            w_ok[rt] = TILED ? feature < N : n < N;
            const int row = w_ok[rt] ? n : 0;
            // row-major: the row's start (the column is added at each load); in operand tiles: this lane's
            // 16 bytes of the tile row's first tile (a tile further along K lies 512 elements on)
            w_row[rt] = WT ? p.w + ((size_t)(row >> 4) * (size_t)(K >> 5) << 9) + (((g << 4) | (row & 15)) << 3)
                           : p.w + (size_t)row * K;
        }
        f32x4 acc[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) acc[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
        float square = 0.0f;
        // What the accumulating epilogue reads (the residual stream's old values, the next norm's
        // weight) is asked for here, so that it has arrived when the sums have: places that do
        // not exist are read from element 0 and dropped. One tile kind (RT 1): wave 0 finishes.
        float old_value[4] = {0.f, 0.f, 0.f, 0.f}, next_weight[4] = {0.f, 0.f, 0.f, 0.f};
        if (EPI == DG_ACCUMULATE) {
            const bool row_ok = r16 < M && !(ROWS == 8 && g >= 2);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int n = tile * ROWS + g * 4 + r;
                const bool ok = row_ok && n < N;
                old_value[r] = static_cast<const float*>(p.out)[ok ? (size_t)r16 * N + n : 0];
                if (p.next_norm_weight) next_weight[r] = p.next_norm_weight[ok ? n : 0];
            }
        }
#pragma unroll 2
        for (int k0 = wave * DG_CHUNK; k0 < K; k0 += WAVES * DG_CHUNK) {
            bf16x8 wf[RT][4], af[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // Every load is issued unconditionally (a run past the end of K, or of a row that
                // does not exist, is read from a valid place and dropped): a branch around a load
                // would make the compiler wait for all loads in flight at the next wait.
                const int k = k0 + j * 32;
                const bool ok = k + g * 8 < K;          // K is a multiple of 8: a run of 8 is in or out as a whole
                const int from = ok ? k + g * 8 : 0;    // columns 0..7 always exist
                const bf16x8 none = {0, 0, 0, 0, 0, 0, 0, 0};
                const size_t w_from = WT ? (ok ? (size_t)(k >> 5) << 9 : 0) : (size_t)from;
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    const bf16x8 v = fw_load_weights<WT>(w_row[rt] + w_from);
                    wf[rt][j] = (ok && w_ok[rt]) ? v : none;
                }
                if (PRO != 1) {
                    const bf16x8 v = *reinterpret_cast<const bf16x8*>(a_bf16 + from);
                    af[j] = (ok && a_ok) ? v : none;
                } else {
                    const f32x4 lo = *reinterpret_cast<const f32x4*>(a_f32 + from);
                    const f32x4 hi = *reinterpret_cast<const f32x4*>(a_f32 + from + 4);
                    const f32x4 wl = *reinterpret_cast<const f32x4*>(norm_w + from);
                    const f32x4 wh = *reinterpret_cast<const f32x4*>(norm_w + from + 4);
                    const float keep = (ok && a_ok) ? 1.0f : 0.0f;
                    u32x4 packed;
#pragma unroll
                    for (int e = 0; e < 4; ++e) square += keep * (lo[e] * lo[e] + hi[e] * hi[e]);
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        packed[e] = (uint32_t)float_to_bf16_bits(keep * lo[2 * e] * (one + wl[2 * e])) |
                                    ((uint32_t)float_to_bf16_bits(keep * lo[2 * e + 1] * (one + wl[2 * e + 1])) << 16);
                        packed[2 + e] = (uint32_t)float_to_bf16_bits(keep * hi[2 * e] * (one + wh[2 * e])) |
                                        ((uint32_t)float_to_bf16_bits(keep * hi[2 * e + 1] * (one + wh[2 * e + 1])) << 16);
                    }
                    af[j] = __builtin_bit_cast(bf16x8, packed);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                    acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[rt][j], af[j], acc[rt], 0, 0, 0);
        }
        fw_mfma_drain();     // the loop is left by a branch; the accumulators are read next

        // The convolution's state and taps of this lane's channels (kernels of up to four taps;
        // longer ones read them in the epilogue): asked for in front of the barrier, so that they
        // travel while the partial sums meet.
        float early_state[4][3], early_taps[4][4];
        const bool early = EPI == DG_CONV && p.kernel_size <= 4;
        if (EPI == DG_CONV && early && wave == 0) {
            const int history = p.kernel_size - 1;
            const bool row_ok = r16 < M && !(ROWS == 8 && g >= 2);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int n = tile * ROWS + g * 4 + r;
                const bool ok = row_ok && n < N;
                const float* channel_state = p.state + (ok ? ((size_t)conv_slot * N + n) * history : 0);
                const float* channel_taps = p.taps + (ok ? (size_t)n * p.kernel_size : 0);
#pragma unroll
                for (int k = 0; k < 3; ++k) early_state[r][k] = channel_state[k < history ? k : 0];
#pragma unroll
                for (int j = 0; j < 4; ++j) early_taps[r][j] = channel_taps[j < p.kernel_size ? j : 0];
            }
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int r = 0; r < 4; ++r) partial[wave][rt][lane][r] = acc[rt][r];
        if (PRO == 2) {
            if (!prepared) {
                float part[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int u = 0; u < SQ_HELD; ++u)
                    part[u & 3] += wave * 4 + g + u * WAVES * 4 < p.squares_tiles ? held[u] : 0.0f;
                const float* from = p.squares + r16;
                for (int t = wave * 4 + g + SQ_HELD * WAVES * 4; t < p.squares_tiles; t += WAVES * 4) part[0] += from[(size_t)t * 16];
                prepared_square = (part[0] + part[1]) + (part[2] + part[3]);
                prepared = true;
            }
            square = prepared_square;
        }
        if (PRO != 0) {
            // this wave's share of sum x^2 of row r16: over the four k groups
            square += __shfl_xor(square, 16, 64);
            square += __shfl_xor(square, 32, 64);
            if (g == 0) squares[wave][r16] = square;
        }
        __syncthreads();

        // D layout: lane holds W row 4 * (lane / 16) + r of the tile for row lane % 16 of a.
        // With 8 features per tile the rows 8..15 repeat rows 0..7 and are dropped.
        const int m = r16;
        const bool mine = m < M && !(ROWS == 8 && g >= 2);
        const int n0 = tile * ROWS;
        float inv = 1.0f;
        if (PRO != 0 && mine) {
            float total = 0.0f;
            for (int v = 0; v < WAVES; ++v) total += squares[v][m];
            inv = rsqrtf(total / (float)K + p.eps);
        }
        if (!TILED) {
            for (int rt = wave; rt < RT; rt += WAVES) {
                float total[4] = {0.f, 0.f, 0.f, 0.f};
                for (int v = 0; v < WAVES; ++v)
#pragma unroll
                    for (int r = 0; r < 4; ++r) total[r] += partial[v][rt][lane][r];
                float row_square = 0.0f;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int n = n0 + g * 4 + r + rt * ROWS * num_tiles;
                    if (!mine || n >= N) continue;
                    float value = total[r] * inv;
                    if (p.bias) value += p.bias[n];
                    TO* out = static_cast<TO*>(p.out);
                    const size_t at = (size_t)m * N + n;
                    if (EPI == DG_ACCUMULATE) value += old_value[r];
                    store_from_float(out, at, value);
                    if (EPI == DG_ACCUMULATE && p.next_activations) {
                        const float w = next_weight[r] + (p.next_one_centered ? 1.0f : 0.0f);
                        p.next_activations[at] = float_to_bf16_bits(value * w);
                        row_square += value * value;
                    }
                }
                if (EPI == DG_ACCUMULATE && p.next_squares) {       // RT is 1 here: wave 0, every lane
                    row_square += __shfl_xor(row_square, 16, 64);
                    row_square += __shfl_xor(row_square, 32, 64);
                    if (g == 0) p.next_squares[(size_t)tile * 16 + m] = m < M ? row_square : 0.0f;
                }
            }
        } else if (wave == 0 && mine) {
            float total[RT][4];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int r = 0; r < 4; ++r) total[rt][r] = 0.0f;
            for (int v = 0; v < WAVES; ++v)
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) total[rt][r] += partial[v][rt][lane][r];
            TO* out = static_cast<TO*>(p.out);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int n = n0 + g * 4 + r;
                if (n >= N) continue;
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    total[rt][r] *= inv;
                    if (p.bias) total[rt][r] += p.bias[n + rt * p.tile_stride];
                }
                if (EPI == DG_SWIGLU) {
                    store_from_float(out, (size_t)m * N + n, dg_silu(total[0][r]) * total[RT > 1 ? 1 : 0][r]);
                } else {        // DG_CONV: tiles are B, C, x of channel n; the row is a segment of one token
                    const int history = p.kernel_size - 1;
                    float* channel_state = p.state + ((size_t)conv_slot * N + n) * history;
                    const float newest = total[0][r] * total[RT > 2 ? 2 : 0][r];
                    float y = 0.0f;
                    if (early) {
                        // the same sum in the same order, over values that are already here
                        float window[4];
#pragma unroll
                        for (int k = 0; k < 3; ++k) window[k] = k < history ? early_state[r][k] : 0.0f;
                        window[3] = 0.0f;
#pragma unroll
                        for (int k = 0; k < 4; ++k)
                            if (k == history) window[k] = newest;
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (j < p.kernel_size) y = fmaf(early_taps[r][j], window[j], y);
                        if (p.conv_bias) y += p.conv_bias[n];
#pragma unroll
                        for (int k = 0; k < 3; ++k)
                            if (k < history) channel_state[k] = window[k + 1];
                    } else {
                        const float* channel_taps = p.taps + (size_t)n * p.kernel_size;
                        float window[DG_MAX_TAPS];
                        for (int k = 0; k < history; ++k) window[k] = channel_state[k];
                        window[history] = newest;
                        for (int j = 0; j < p.kernel_size; ++j) y = fmaf(channel_taps[j], window[j], y);
                        if (p.conv_bias) y += p.conv_bias[n];
                        for (int k = 0; k < history; ++k) channel_state[k] = window[k + 1];
                    }
                    store_from_float(out, (size_t)m * N + n, total[RT > 1 ? 1 : 0][r] * y);
                }
            }
        }
        if (tile + (int)gridDim.x < num_tiles) __syncthreads();       // the partial sums are free again
    }
}

#define DG_MAX_BLOCKS 1024
#define DG_NARROW_BELOW (192 * 16)

template <int RT, int WAVES, int ROWS, int PRO, int EPI, typename TO>
static int launch(const DecodeGemmArgs& args, hipStream_t stream) {
    const int tile_features = (EPI == DG_STORE || EPI == DG_ACCUMULATE) ? ROWS * RT : ROWS;
    const int num_tiles = fw_ceil_div(args.N, tile_features);
    const int blocks = num_tiles > DG_MAX_BLOCKS ? DG_MAX_BLOCKS : num_tiles;
    if (args.w_tiled) decode_gemm_kernel<RT, WAVES, ROWS, PRO, EPI, TO, true><<<blocks, WAVES * 64, 0, stream>>>(args, num_tiles);
    else decode_gemm_kernel<RT, WAVES, ROWS, PRO, EPI, TO, false><<<blocks, WAVES * 64, 0, stream>>>(args, num_tiles);
    return 0;
}

// prologue 0: a bfloat16 [M][K]; 1: RMS norm of float32 rows (norm_weight, eps, one_centered,
// optional row_index); 2: a bfloat16 [M][K] = x * w left by an accumulating call together with
// `squares` [squares_tiles][16], the row's scale is formed from those. epilogue 0: store out_dtype [M][N]; 1: float32 out += ; 2: SwiGLU, w =
// [gate rows; up rows], out bfloat16 [M][N]; 3: gated short convolution, w = [B rows; C rows; x
// rows] of N channels each, out_dtype [M][N], state updated. w_tiled: w is given in operand tiles
// (fw_tile_weights) instead of row-major; the results are bit for bit the same.
extern "C" int fw_gemm_decode(int prologue, const void* a, const float* norm_weight, const int32_t* row_index,
                              float eps, int one_centered, const void* w, int w_tiled, const float* bias, void* out,
                              int out_dtype, int epilogue, int M, int N, int K, const float* taps,
                              const float* conv_bias, float* state, const int32_t* seg_slot, int kernel_size,
                              const float* next_norm_weight, int next_one_centered, void* next_activations,
                              float* next_squares, const float* squares, int squares_tiles, void* stream) {
    FW_REQUIRE(M >= 1 && M <= 16, "gemm_decode: takes 1..16 rows, got %d", M);
    FW_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "gemm_decode: K (%d) must be a positive multiple of 8, N (%d) positive", K, N);
    FW_REQUIRE(prologue >= 0 && prologue <= 2, "gemm_decode: unknown prologue %d", prologue);
    FW_REQUIRE(!w_tiled || K % 32 == 0, "gemm_decode: weights in operand tiles need K (%d) to be a multiple of 32", K);
    FW_REQUIRE(prologue != 2 || (squares != nullptr && squares_tiles >= 1 && eps > 0.0f), "gemm_decode: the pre-normed prologue needs the partial sums of squares and eps");
    FW_REQUIRE((next_activations == nullptr) == (next_squares == nullptr) && (next_activations == nullptr) == (next_norm_weight == nullptr),
               "gemm_decode: the next norm's weight, activations and sums of squares come together");
    FW_REQUIRE(next_activations == nullptr || epilogue == DG_ACCUMULATE, "gemm_decode: only the accumulating product prepares the next norm");
    FW_REQUIRE(epilogue >= 0 && epilogue <= 3, "gemm_decode: unknown epilogue %d", epilogue);
    FW_REQUIRE(prologue != 1 || (norm_weight != nullptr && eps > 0.0f), "gemm_decode: the norm prologue needs its weight and eps");
    FW_REQUIRE(epilogue != DG_ACCUMULATE || out_dtype == FW_F32, "gemm_decode: accumulation needs a float32 destination");
    FW_REQUIRE(epilogue != DG_ACCUMULATE || prologue == 0, "gemm_decode: the accumulating product takes bfloat16 activations");
    FW_REQUIRE(epilogue != DG_SWIGLU || out_dtype == FW_BF16, "gemm_decode: SwiGLU stores bfloat16");
    FW_REQUIRE(out_dtype == FW_F32 || out_dtype == FW_BF16, "gemm_decode: unknown out dtype %d", out_dtype);
    FW_REQUIRE(epilogue != DG_CONV || (taps && state && seg_slot && kernel_size >= 2 && kernel_size <= DG_MAX_TAPS),
               "gemm_decode: the convolution epilogue needs taps, state, slots and a kernel size in 2..%d", DG_MAX_TAPS);
    FW_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0) && ((uintptr_t)norm_weight % 16 == 0),
               "gemm_decode: operands must be 16-byte aligned");
    DecodeGemmArgs args;
    args.a = a; args.norm_weight = norm_weight; args.row_index = row_index; args.eps = eps; args.one_centered = one_centered;
    args.w = (const uint16_t*)w; args.w_tiled = w_tiled ? 1 : 0; args.bias = bias; args.out = out; args.M = M; args.N = N; args.K = K;
    args.tile_stride = (epilogue == DG_SWIGLU || epilogue == DG_CONV) ? N : 0;
    args.taps = taps; args.conv_bias = conv_bias; args.state = state; args.seg_slot = seg_slot; args.kernel_size = kernel_size;
    args.next_norm_weight = next_norm_weight; args.next_one_centered = next_one_centered;
    args.next_activations = (uint16_t*)next_activations; args.next_squares = next_squares;
    args.squares = squares; args.squares_tiles = squares_tiles;
    hipStream_t s = (hipStream_t)stream;
    // Few features: tiles of 8, so that there are more workgroups (2,048 features: 256 instead of 128). From 192
    // tiles of 16 on the wider tile wins, whose waves read whole 1 KB pieces of W (3,072 features at 8 rows: 4.9
    // against 6.5 us).
    const bool narrow = N < DG_NARROW_BELOW;
    int status = -2;
#define DG_TRY(RT, WAVES, ROWS, PRO, EPI, TO) status = launch<RT, WAVES, ROWS, PRO, EPI, TO>(args, s)
    if (epilogue == DG_ACCUMULATE) {
        if (K >= 4096) { if (narrow) DG_TRY(1, 16, 8, 0, DG_ACCUMULATE, float); else DG_TRY(1, 16, 16, 0, DG_ACCUMULATE, float); }
        else { if (narrow) DG_TRY(1, 8, 8, 0, DG_ACCUMULATE, float); else DG_TRY(1, 8, 16, 0, DG_ACCUMULATE, float); }
    } else if (epilogue == DG_STORE) {
#define DG_STORE_CASE(RT, ROWS)                                                                     \
    if (prologue == 1) { if (out_dtype == FW_F32) DG_TRY(RT, 8, ROWS, 1, DG_STORE, float); else DG_TRY(RT, 8, ROWS, 1, DG_STORE, bf16_t); } \
    else if (prologue == 2) { if (out_dtype == FW_F32) DG_TRY(RT, 8, ROWS, 2, DG_STORE, float); else DG_TRY(RT, 8, ROWS, 2, DG_STORE, bf16_t); } \
    else { if (out_dtype == FW_F32) DG_TRY(RT, 8, ROWS, 0, DG_STORE, float); else DG_TRY(RT, 8, ROWS, 0, DG_STORE, bf16_t); }
        if (N >= 16384) { DG_STORE_CASE(2, 16) } else if (narrow) { DG_STORE_CASE(1, 8) } else { DG_STORE_CASE(1, 16) }
#undef DG_STORE_CASE
    } else if (epilogue == DG_SWIGLU) {
        if (prologue == 1) { if (narrow) DG_TRY(2, 8, 8, 1, DG_SWIGLU, bf16_t); else DG_TRY(2, 8, 16, 1, DG_SWIGLU, bf16_t); }
        else if (prologue == 2) { if (narrow) DG_TRY(2, 8, 8, 2, DG_SWIGLU, bf16_t); else DG_TRY(2, 8, 16, 2, DG_SWIGLU, bf16_t); }
        else { if (narrow) DG_TRY(2, 8, 8, 0, DG_SWIGLU, bf16_t); else DG_TRY(2, 8, 16, 0, DG_SWIGLU, bf16_t); }
    } else {
#define DG_CONV_CASE(ROWS)                                                                          \
    if (prologue == 1) { if (out_dtype == FW_F32) DG_TRY(3, 8, ROWS, 1, DG_CONV, float); else DG_TRY(3, 8, ROWS, 1, DG_CONV, bf16_t); } \
    else if (prologue == 2) { if (out_dtype == FW_F32) DG_TRY(3, 8, ROWS, 2, DG_CONV, float); else DG_TRY(3, 8, ROWS, 2, DG_CONV, bf16_t); } \
    else { if (out_dtype == FW_F32) DG_TRY(3, 8, ROWS, 0, DG_CONV, float); else DG_TRY(3, 8, ROWS, 0, DG_CONV, bf16_t); }
        if (narrow) { DG_CONV_CASE(8) } else { DG_CONV_CASE(16) }
#undef DG_CONV_CASE
    }
#undef DG_TRY
    if (status != 0) return -1;
    FW_LAUNCH_CHECK("gemm_decode");
    return 0;
}

// How many tiles of features the accumulating product of this shape uses (the first extent of
// the sums of squares it leaves for the next norm).
extern "C" int fw_gemm_decode_accumulate_tiles(int N) {
    const bool narrow = N < DG_NARROW_BELOW;
    return fw_ceil_div(N, narrow ? 8 : 16);
}

// Whether fw_gemm_decode takes this shape (the caller falls back to separate kernels if not).
extern "C" int fw_gemm_decode_fits(int M, int N, int K, int epilogue) {
    (void)epilogue;
    return (M >= 1 && M <= 16 && K > 0 && K % 8 == 0 && N > 0) ? 1 : 0;
}
