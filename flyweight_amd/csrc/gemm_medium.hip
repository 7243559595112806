// Matrix product for a few dozen rows: out[M][N] = a[M][K] . w[N][K]^T, M <= 64, bfloat16 operands,
// float32 accumulation on the matrix cores. This is the decode step of 17..64 requests (and any
// short batch): still bound by reading W once from HBM, but a is now large enough (up to 1 MB)
// that re-reading it from L2 in every workgroup of a few features would cost several times the
// traffic of W itself. So the work is cut the other way:
//
//  * a workgroup (4 waves) owns 64 or 32 consecutive features and a slice of K; with few
//    features the slices of K go to different workgroups (blockIdx.y) so that every compute unit
//    still streams its share of W;
//  * W goes from global memory straight into MFMA operand registers (lane (n, g) of the 16x16x32
//    instruction holds k = 8g..8g+7 of feature n), four chunks of 64 k in flight per wave;
//  * a is staged through LDS once per workgroup (two buffers, one barrier per chunk), also
//    four chunks ahead in registers, and read from there as MFMA operands by every wave;
//  * partial sums over K: inside a workgroup through LDS in wave order; between workgroups
//    through a float32 workspace that the LAST workgroup of a tile to arrive (a ticket from an
//    atomic counter) sums in slice order, so the result does not depend on timing. The counter
//    is left at zero again. Nobody waits for anybody.
//
// Every global load is unconditional (addresses clamped into the operands, a zeroed outside
// the slice on its way to LDS): a branch around a load, or arithmetic right behind it, makes
// the compiler wait for loads in flight. The barriers order LDS traffic only, for the same reason.
// Epilogues as in the other products: store, add into the float32 residual stream, SwiGLU.
// The reference has no counterpart for this batch size: its decode projections are
// one-warp-per-row vector kernels run per request (native/include/flyweight_v2_qwen_kernels.hpp:855-941).
#include "fw_common.h"
#include "fw_kernels.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define GM_THREADS 256
#define GM_DEPTH 4      // chunks in flight
#define GM_PAD 8        // bfloat16 elements between LDS rows: spreads the rows over the banks

enum { GM_STORE = 0, GM_ACCUMULATE = 1, GM_SWIGLU = 2 };

struct MediumArgs {
    const uint16_t* a;
    const uint16_t* w;
    int w_tiled;            // W lies in tiles of 16 rows x 32 columns, each 1 KB in the order of a wave's operand load
    const float* bias;
    void* out;
    int M, N, K;            // N: output features (for SwiGLU w has 2N rows: gate, then up)
    int k_per_split;        // a multiple of the workgroup's chunk
    int splits;
    float* partials;        // [splits][tiles][kinds * MT][FW][64][4]
    int* counters;          // [tiles], zero between calls
    // accumulating product of up to 16 rows: what the norm after it will need (all null: nothing)
    const float* next_norm_weight;  // [N]
    int next_one_centered;
    uint16_t* next_activations;     // bfloat16 [M][N] = x_new * (w_next or 1 + w_next)
    float* next_squares;            // [tiles * FW][row stride]: this wave's sum of x_new^2 per row (rows >= M: unspecified)
    // prepared activations: a = x * w of an RMS norm, left by an accumulating product together with
    // these sums; the rows' 1/rms is formed here and applied to the sums of the product
    const float* squares;           // [squares_rows][row stride]
    int squares_rows;
    float eps;
    int rotate;                     // workgroups start their walk over K at different chunks
};

// rows of the sums of squares are 16 wide for up to 16 rows of a (the fused decode product's
// layout), 64 wide beyond
__host__ __device__ inline int gm_square_stride(int M) { return M <= 16 ? 16 : 64; }

__device__ __forceinline__ float gm_silu(float g) {
    if (g >= 0.0f) return g / (1.0f + __expf(-g));
    const float e = __expf(g);
    return g * e / (1.0f + e);
}

// MT: tiles of 16 rows of a. FW: waves side by side over features (4: 64 features, no split of
// K inside the workgroup; 2: 32 features, the two halves of a 128-k chunk go to wave pairs).
template <int MT, int FW, int MODE, typename TO, bool ROTATE, bool WT>
__global__ __launch_bounds__(GM_THREADS) void gemm_medium_kernel(const MediumArgs p) {
    constexpr int KP = 4 / FW;                  // parts of K inside the workgroup
    constexpr int CHUNK = 64 * KP;              // k per iteration of the workgroup
    constexpr int KINDS = MODE == GM_SWIGLU ? 2 : 1;
    constexpr int SEG = CHUNK / 8;              // 16-byte pieces per row of a chunk of a
    constexpr int PIECES = MT * 16 * SEG;       // pieces per chunk of a
    constexpr int AP = (PIECES + GM_THREADS - 1) / GM_THREADS;
    constexpr int STRIDE = CHUNK + GM_PAD;
    __shared__ __attribute__((aligned(16))) uint16_t a_lds[2][MT * 16][STRIDE];
    __shared__ float k_parts[KP > 1 ? KP - 1 : 1][KP > 1 ? FW : 1][KP > 1 ? KINDS * MT : 1][KP > 1 ? 64 : 1][4];
    __shared__ int ticket_shared;
    __shared__ float square_parts[GM_THREADS], inv_rows[64];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r16 = lane & 15, g = lane >> 4;
    const int ft = wave % FW, kp = wave / FW;
    const int M = p.M, N = p.N, K = p.K;
    const int square_stride = gm_square_stride(M);
    const int tile = blockIdx.x, tiles = gridDim.x;
    const int n0 = tile * 16 * FW;
    const int k_begin = blockIdx.y * p.k_per_split;
    const int k_end = min(K, k_begin + p.k_per_split);
    const int chunks = (k_end - k_begin + CHUNK - 1) / CHUNK;
    const int iterations = (chunks + GM_DEPTH - 1) / GM_DEPTH * GM_DEPTH;

    const int feature = n0 + 16 * ft + r16;
    const uint16_t* w_row[KINDS];
#pragma unroll
    for (int kind = 0; kind < KINDS; ++kind) {
        const int row = (feature < N ? feature : 0) + kind * N;
        w_row[kind] = WT ? p.w + ((size_t)(row >> 4) * (size_t)(K >> 5) << 9) + (((g << 4) | (row & 15)) << 3)
                         : p.w + (size_t)row * K;
    }
    const uint16_t* a_piece[AP];
    int piece_row[AP], piece_k[AP];
#pragma unroll
    for (int i = 0; i < AP; ++i) {
        const int q = threadIdx.x + i * GM_THREADS;
        piece_row[i] = q / SEG;
        piece_k[i] = (q % SEG) * 8;
        a_piece[i] = p.a + (size_t)min(piece_row[i], M - 1) * K;
    }

    bf16x8 wf[GM_DEPTH][KINDS][2], areg[GM_DEPTH][AP];
    f32x4 acc[KINDS][MT];
#pragma unroll
    for (int kind = 0; kind < KINDS; ++kind)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[kind][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Nothing is done to a loaded value before the chunk is used (a select right behind a load
    // would wait for it at once): W comes from a clamped address as it is, and the rows of a are
    // zeroed outside the slice when they move to LDS, three chunks after their load.
    // Workgroups walk their slice of K from different chunks on (and around): all of them read the
    // same rows of a, and in step they would ask one cache line of it at a time from every compute
    // unit at once. Where a workgroup starts depends on its tile alone, so the order of its sum
    // over K does not depend on the batch or on timing. It pays for a large W that is not split over
    // workgroups (inside a decode step of 8 rows: gate|up 17.3 -> 16.5 us, the head 59.8 -> 50.3 us);
    // the smaller products and those whose slices meet through the workspace lose a little by it.
    const int rotate = ROTATE ? (int)((tile * 5u + blockIdx.y * 3u) % (unsigned)(chunks > 0 ? chunks : 1)) : 0;
    auto chunk_start = [&](const int c) {
        if (!ROTATE) return k_begin + c * CHUNK;
        if (c >= chunks) return k_end;                  // past the slice: nothing of it is inside
        const int turned = c + rotate;
        return k_begin + (turned < chunks ? turned : turned - chunks) * CHUNK;
    };
    auto load = [&](const int d, const int c) {
        const int k0 = chunk_start(c);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int k = k0 + kp * 64 + ks * 32 + g * 8;
            // (slices and chunks begin at multiples of 32, and K is one where W lies in tiles: a tile's columns are inside or outside together)
            const size_t from = k < k_end ? (WT ? (size_t)(k >> 5) << 9 : (size_t)k) : 0;
#pragma unroll
            for (int kind = 0; kind < KINDS; ++kind) wf[d][kind][ks] = fw_load_weights<WT>(w_row[kind] + from);
        }
#pragma unroll
        for (int i = 0; i < AP; ++i) {
            const int k = k0 + piece_k[i];
            areg[d][i] = *reinterpret_cast<const bf16x8*>(a_piece[i] + (k < k_end ? k : 0));
        }
    };
    auto stage = [&](const int d, const int buffer, const int c) {
        const bf16x8 none = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < AP; ++i)
            if (PIECES % GM_THREADS == 0 || piece_row[i] < MT * 16) {
                // K and the slices are multiples of 8: a run of 8 is inside or outside as a whole
                const bool inside = chunk_start(c) + piece_k[i] < k_end;
                *reinterpret_cast<bf16x8*>(&a_lds[buffer][piece_row[i]][piece_k[i]]) = inside ? areg[d][i] : none;
            }
    };
    auto multiply = [&](const int d, const int buffer) {
        bf16x8 af[2][MT];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                af[ks][mt] = *reinterpret_cast<const bf16x8*>(&a_lds[buffer][mt * 16 + r16][kp * 64 + ks * 32 + g * 8]);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int kind = 0; kind < KINDS; ++kind)
                    acc[kind][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[d][kind][ks], af[ks][mt], acc[kind][mt], 0, 0, 0);
    };

    // prepared activations: this thread's share of the sums of squares of one row is asked for
    // first and added up behind the first chunks of W (a wave issues in order: a sum formed here
    // would hold the stream of W back by a round trip)
    constexpr int SQ_HELD = 32;
    float held[SQ_HELD];
    if (p.squares) {
        const int row = threadIdx.x % square_stride, part = threadIdx.x / square_stride, parts = GM_THREADS / square_stride;
        const float* from = p.squares + row;
        const int last = p.squares_rows - 1;
#pragma unroll
        for (int u = 0; u < SQ_HELD; ++u) {
            const int e = part + u * parts;
            held[u] = from[(size_t)(e < last ? e : last) * square_stride];
        }
    }
#pragma unroll
    for (int d = 0; d < GM_DEPTH; ++d) load(d, d);
    // the shares of the sums of squares have been on their way since before W: they are the
    // oldest loads, so adding them up here waits for nothing that was asked for after them
    float square_share = 0.0f;
    if (p.squares) {
        const int row = threadIdx.x % square_stride, part = threadIdx.x / square_stride, parts = GM_THREADS / square_stride;
        float share[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < SQ_HELD; ++u) share[u & 3] += part + u * parts < p.squares_rows ? held[u] : 0.0f;
        const float* from = p.squares + row;
        for (int e = part + SQ_HELD * parts; e < p.squares_rows; e += parts) share[0] += from[(size_t)e * square_stride];
        square_share = (share[0] + share[1]) + (share[2] + share[3]);
    }
    stage(0, 0, 0);
    if (p.squares) square_parts[threadIdx.x] = square_share;
    fw_lds_barrier();
    if (p.squares && threadIdx.x < square_stride) {
        // the shares of a row meet in a fixed order; read in the epilogue, many barriers from here
        float total = 0.0f;
        for (int part = 0; part < GM_THREADS / square_stride; ++part) total += square_parts[part * square_stride + threadIdx.x];
        inv_rows[threadIdx.x] = rsqrtf(total / (float)K + p.eps);
    }
    for (int c0 = 0; c0 < iterations; c0 += GM_DEPTH) {
#pragma unroll
        for (int d = 0; d < GM_DEPTH; ++d) {
            // chunk c0 + d: its W is in register set d, its a in LDS buffer d % 2; the next chunk's a
            // waits in register set d + 1 and moves to the other buffer; set d is then refilled
            multiply(d, d & 1);
            stage((d + 1) % GM_DEPTH, (d + 1) & 1, c0 + d + 1);
            load(d, c0 + d + GM_DEPTH);
            fw_lds_barrier();       // LDS only: the loads just issued stay in flight
        }
    }
    fw_mfma_drain();     // branches follow that lead to code reading the accumulators

    // the parts of K inside the workgroup meet in LDS, in wave order
    if (KP > 1) {
        if (kp > 0)
#pragma unroll
            for (int kind = 0; kind < KINDS; ++kind)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) k_parts[kp > 0 ? kp - 1 : 0][ft][kind * MT + mt][lane][r] = acc[kind][mt][r];
        __syncthreads();
        if (kp == 0)
            for (int part = 0; part < KP - 1; ++part)
#pragma unroll
                for (int kind = 0; kind < KINDS; ++kind)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[kind][mt][r] += k_parts[part][ft][kind * MT + mt][lane][r];
    }

    // The slices of K of different workgroups meet in the workspace; the last to arrive sums them.
    // The partial sums are written and read with device-scope accesses, which go past the caches
    // that workgroups on different dies do not share, so no cache has to be written back or
    // dropped as a whole (what a device-wide fence does): a wave waits for its own stores to be
    // acknowledged, the workgroup meets, then one thread takes the ticket.
    // What the accumulating epilogue reads beside the sums (the residual stream's old values, the
    // next norm's weight) is asked for before the slices of the other workgroups are, so that one
    // round trip covers both.
    const int early_first = n0 + 16 * ft + 4 * g;
    const bool early_whole = early_first + 3 < N && (N & 3) == 0;
    f32x4 early_old[MT], early_weight = {0.f, 0.f, 0.f, 0.f};
    auto fetch_early = [&]() {
        if (MODE != GM_ACCUMULATE || sizeof(TO) != 4 || !early_whole) return;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + r16;
            early_old[mt] = *reinterpret_cast<const f32x4*>(reinterpret_cast<const float*>(p.out) + (size_t)(m < M ? m : 0) * N + early_first);
        }
        if (p.next_activations) early_weight = *reinterpret_cast<const f32x4*>(p.next_norm_weight + early_first);
    };
    if (p.splits <= 1 && kp == 0) fetch_early();
    if (p.splits > 1) {
        float* mine = p.partials + ((((size_t)blockIdx.y * tiles + tile) * (KINDS * MT) * FW + ft) * 64 + lane) * 4;
        if (kp == 0)
#pragma unroll
            for (int kind = 0; kind < KINDS; ++kind)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        __hip_atomic_store(mine + (size_t)(kind * MT + mt) * FW * 256 + r, acc[kind][mt][r], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (threadIdx.x == 0)
            ticket_shared = __hip_atomic_fetch_add(&p.counters[tile], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (ticket_shared != p.splits - 1) return;
        if (kp == 0) {
            fetch_early();
#pragma unroll
            for (int kind = 0; kind < KINDS; ++kind)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[kind][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
            for (int split = 0; split < p.splits; ++split) {
                const float* theirs = p.partials + ((((size_t)split * tiles + tile) * (KINDS * MT) * FW + ft) * 64 + lane) * 4;
                float v[KINDS * MT][4];
#pragma unroll
                for (int t = 0; t < KINDS * MT; ++t)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        v[t][r] = __hip_atomic_load(theirs + (size_t)t * FW * 256 + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int kind = 0; kind < KINDS; ++kind)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[kind][mt][r] += v[kind * MT + mt][r];
            }
        }
        if (threadIdx.x == 0) __hip_atomic_store(&p.counters[tile], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (kp != 0) return;

    // D layout of the 16x16 product: lane holds features 4 * (lane / 16) + r of the wave's tile
    // for row lane % 16 of a
    const int n_first = n0 + 16 * ft + 4 * g;
    const bool whole = n_first + 3 < N && (N & 3) == 0;     // four features in one aligned piece
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r16;
        const bool mine = m < M;
        const size_t at = (size_t)(mine ? m : 0) * N + n_first;
        float v[4];
        const float inv = p.squares ? inv_rows[mine ? m : 0] : 1.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int n = n_first + r;
            if (MODE == GM_SWIGLU) v[r] = gm_silu(acc[0][mt][r] * inv) * (acc[1][mt][r] * inv);
            else v[r] = acc[0][mt][r] * inv + ((p.bias && n < N) ? p.bias[n] : 0.0f);
        }
        if (mine) {
            if constexpr (sizeof(TO) == 4) {
                float* to = reinterpret_cast<float*>(p.out) + at;
                if (whole) {
                    f32x4 packed = {v[0], v[1], v[2], v[3]};
                    if (MODE == GM_ACCUMULATE) {
                        const f32x4 old = early_old[mt];
#pragma unroll
                        for (int r = 0; r < 4; ++r) packed[r] = v[r] = v[r] + old[r];
                    }
                    *reinterpret_cast<f32x4*>(to) = packed;
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (n_first + r >= N) continue;
                        if (MODE == GM_ACCUMULATE) v[r] += to[r];
                        to[r] = v[r];
                    }
                }
            } else {
                uint16_t* to = reinterpret_cast<uint16_t*>(p.out) + at;
                if (whole) {
                    uint2 packed;
                    packed.x = (uint32_t)float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
                    packed.y = (uint32_t)float_to_bf16_bits(v[2]) | ((uint32_t)float_to_bf16_bits(v[3]) << 16);
                    *reinterpret_cast<uint2*>(to) = packed;
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (n_first + r < N) to[r] = float_to_bf16_bits(v[r]);
                }
            }
        }
        // what the norm after this addition needs: x * w of that norm in bfloat16, and this wave's
        // sum of x^2 per row; the product that follows forms the row's 1/rms from those sums
        if (MODE == GM_ACCUMULATE && p.next_activations) {
            float row_square = 0.0f;
            if (mine) {
                const float one = p.next_one_centered ? 1.0f : 0.0f;
                if (whole) {
                    const f32x4 w = early_weight;
                    uint2 packed;
                    packed.x = (uint32_t)float_to_bf16_bits(v[0] * (w[0] + one)) | ((uint32_t)float_to_bf16_bits(v[1] * (w[1] + one)) << 16);
                    packed.y = (uint32_t)float_to_bf16_bits(v[2] * (w[2] + one)) | ((uint32_t)float_to_bf16_bits(v[3] * (w[3] + one)) << 16);
                    *reinterpret_cast<uint2*>(p.next_activations + at) = packed;
                    row_square = (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int n = n_first + r;
                        if (n >= N) continue;
                        p.next_activations[at + r] = float_to_bf16_bits(v[r] * (p.next_norm_weight[n] + one));
                        row_square += v[r] * v[r];
                    }
                }
            }
            row_square += __shfl_xor(row_square, 16, 64);
            row_square += __shfl_xor(row_square, 32, 64);
            if (g == 0) p.next_squares[((size_t)tile * FW + ft) * square_stride + m] = row_square;
        }
    }
}

// ----- host side ---------------------------------------------------------------------------

struct MediumPlan {
    int mt, fw, tiles, splits, k_per_split;
    size_t workspace_bytes;
};


static MediumPlan medium_plan(int M, int N, int K, int mode) {
    MediumPlan plan;
    plan.mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
    const int kinds = mode == GM_SWIGLU ? 2 : 1;
    if (fw_ceil_div(N, 64) >= 384) {            // enough tiles of 64 features for every compute unit
        plan.fw = 4;
        plan.tiles = fw_ceil_div(N, 64);
        plan.splits = 1;
        plan.k_per_split = fw_ceil_div(K, 64) * 64;
    } else {
        plan.fw = 2;
        plan.tiles = fw_ceil_div(N, 32);
        const int chunk = 128;
        int splits = (256 + plan.tiles / 2) / plan.tiles;           // about one workgroup per compute unit
        // A slice costs its workgroup a start (the first loads' way from memory) and an end (its sums
        // to the workspace, the ticket, the last one reading all of them: three trips to memory, 5-8 us)
        // whatever its length, so K is only cut where a slice keeps at least nine chunks: at 64 rows
        // and K 1,024 one slice against two or three 12.4 vs 21.1 us (gate|up of 4,608 features), 8.1 vs
        // 13.2 (3,072 features), 7.4 vs 10.4 (1,024); K 2,048, 2,048 features 10.9 vs 12.0 us; K 4,608,
        // 1,024 features 4 slices 14.1 vs 8 slices 15.7 us; K 8,192 stays at 4 slices (18.9 us; 1: 34.9).
        const int most = K / (9 * chunk) > 1 ? K / (9 * chunk) : 1;
        splits = splits < 1 ? 1 : (splits > most ? most : splits);
        if (splits > 16) splits = 16;
        plan.k_per_split = fw_ceil_div(fw_ceil_div(K, splits), chunk) * chunk;
        plan.splits = fw_ceil_div(K, plan.k_per_split);
    }
    plan.workspace_bytes = plan.splits > 1
        ? (size_t)plan.splits * plan.tiles * kinds * plan.mt * plan.fw * 64 * 4 * sizeof(float) : 0;
    return plan;
}

// What fw_gemm_medium needs for a shape: bytes of workspace (0: none), the number of int32
// counters (0: none; they must be zero before the first call and are left zero), and how many
// rows of 16 the sums of squares for the next norm take.
extern "C" int fw_gemm_medium_plan(int M, int N, int K, int mode, size_t* workspace_bytes, int* counters, int* squares_rows) {
    FW_REQUIRE(M >= 1 && M <= 64 && N > 0 && K > 0, "gemm_medium: takes 1..64 rows, got M %d N %d K %d", M, N, K);
    const MediumPlan plan = medium_plan(M, N, K, mode);
    *workspace_bytes = plan.workspace_bytes;
    *counters = plan.splits > 1 ? plan.tiles : 0;
    *squares_rows = plan.tiles * plan.fw;       // first extent of the sums of squares left for the next norm (the second: 16 for M <= 16, else 64)
    return 0;
}

template <int MT, int FW, bool ROTATE, bool WT>
static void medium_launch_as(const MediumArgs& args, int out_dtype, int mode, dim3 grid, hipStream_t stream) {
    if (mode == GM_SWIGLU) gemm_medium_kernel<MT, FW, GM_SWIGLU, bf16_t, ROTATE, WT><<<grid, GM_THREADS, 0, stream>>>(args);
    else if (mode == GM_ACCUMULATE) gemm_medium_kernel<MT, FW, GM_ACCUMULATE, float, ROTATE, WT><<<grid, GM_THREADS, 0, stream>>>(args);
    else if (out_dtype == FW_F32) gemm_medium_kernel<MT, FW, GM_STORE, float, ROTATE, WT><<<grid, GM_THREADS, 0, stream>>>(args);
    else gemm_medium_kernel<MT, FW, GM_STORE, bf16_t, ROTATE, WT><<<grid, GM_THREADS, 0, stream>>>(args);
}

template <int MT, int FW>
static void medium_launch(const MediumArgs& args, int out_dtype, int mode, dim3 grid, hipStream_t stream) {
    if (args.rotate) {
        if (args.w_tiled) medium_launch_as<MT, FW, true, true>(args, out_dtype, mode, grid, stream);
        else medium_launch_as<MT, FW, true, false>(args, out_dtype, mode, grid, stream);
    } else {
        if (args.w_tiled) medium_launch_as<MT, FW, false, true>(args, out_dtype, mode, grid, stream);
        else medium_launch_as<MT, FW, false, false>(args, out_dtype, mode, grid, stream);
    }
}

// mode 0: out = a . w^T (+ bias) stored as out_dtype; 1: out (float32) += a . w^T (+ bias);
// 2: w is [2 * N][K] (gate rows, then up rows); out [M][N] bfloat16 = silu(gate) * up.
// workspace / counters: as fw_gemm_medium_plan says for this shape. Calls that overlap on one
// device must not share counters or workspace.
extern "C" int fw_gemm_medium(const void* a, const void* w, int w_tiled, const float* bias, void* out, int out_dtype, int mode,
                              int M, int N, int K, void* workspace, size_t workspace_bytes, int* counters,
                              int counters_len, const float* next_norm_weight, int next_one_centered,
                              void* next_activations, float* next_squares, const float* squares, int squares_rows,
                              float eps, void* stream) {
    FW_REQUIRE(M >= 1 && M <= 64, "gemm_medium: takes 1..64 rows, got %d", M);
    FW_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "gemm_medium: K (%d) must be a positive multiple of 8, N (%d) positive", K, N);
    FW_REQUIRE(mode >= 0 && mode <= 2, "gemm_medium: unknown mode %d", mode);
    FW_REQUIRE(!w_tiled || K % 32 == 0, "gemm_medium: weights in operand tiles need K (%d) to be a multiple of 32", K);
    FW_REQUIRE(mode != GM_ACCUMULATE || out_dtype == FW_F32, "gemm_medium: accumulation needs a float32 destination");
    FW_REQUIRE(mode != GM_SWIGLU || (out_dtype == FW_BF16 && bias == nullptr), "gemm_medium: SwiGLU stores bfloat16 and takes no bias");
    FW_REQUIRE(out_dtype == FW_F32 || out_dtype == FW_BF16, "gemm_medium: unknown out dtype %d", out_dtype);
    FW_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0) && ((uintptr_t)out % 16 == 0) && ((uintptr_t)workspace % 16 == 0),
               "gemm_medium: operands must be 16-byte aligned");
    FW_REQUIRE((next_activations == nullptr) == (next_squares == nullptr) && (next_activations == nullptr) == (next_norm_weight == nullptr),
               "gemm_medium: the next norm's weight, activations and sums of squares come together");
    FW_REQUIRE(next_activations == nullptr || mode == GM_ACCUMULATE, "gemm_medium: only the accumulating product prepares the next norm");
    FW_REQUIRE(squares == nullptr || (squares_rows >= 1 && eps > 0.0f), "gemm_medium: prepared activations come with their sums of squares and eps");
    const MediumPlan plan = medium_plan(M, N, K, mode);
    FW_REQUIRE(plan.splits == 1 || (workspace != nullptr && workspace_bytes >= plan.workspace_bytes && counters != nullptr &&
                                    counters_len >= plan.tiles),
               "gemm_medium: this shape needs %zu bytes of workspace and %d counters", plan.workspace_bytes, plan.tiles);
    FW_REQUIRE(plan.tiles <= 65535 * 16 && plan.splits <= 65535, "gemm_medium: too many tiles");
    MediumArgs args;
    args.a = (const uint16_t*)a; args.w = (const uint16_t*)w; args.w_tiled = w_tiled ? 1 : 0; args.bias = bias; args.out = out;
    args.M = M; args.N = N; args.K = K; args.k_per_split = plan.k_per_split; args.splits = plan.splits;
    args.partials = (float*)workspace; args.counters = counters;
    args.next_norm_weight = next_norm_weight; args.next_one_centered = next_one_centered;
    args.next_activations = (uint16_t*)next_activations; args.next_squares = next_squares;
    args.squares = squares; args.squares_rows = squares_rows; args.eps = eps;
    args.rotate = plan.splits == 1 && (long long)N * K * (mode == GM_SWIGLU ? 2 : 1) > (1ll << 24);
    const dim3 grid(plan.tiles, plan.splits);
    hipStream_t s = (hipStream_t)stream;
    if (plan.fw == 4) {
        if (plan.mt == 1) medium_launch<1, 4>(args, out_dtype, mode, grid, s);
        else if (plan.mt == 2) medium_launch<2, 4>(args, out_dtype, mode, grid, s);
        else medium_launch<4, 4>(args, out_dtype, mode, grid, s);
    } else {
        if (plan.mt == 1) medium_launch<1, 2>(args, out_dtype, mode, grid, s);
        else if (plan.mt == 2) medium_launch<2, 2>(args, out_dtype, mode, grid, s);
        else medium_launch<4, 2>(args, out_dtype, mode, grid, s);
    }
    FW_LAUNCH_CHECK("gemm_medium");
    return 0;
}
