// Tiled matrix product for long prompts and wide outputs: out[M][N] = a[M][K] . w[N][K]^T with
// 256 x 256 tiles. The 128 x 128 kernel beside this one moves 64 KB through a compute unit's
// vector memory path (64 bytes a clock) for every 1,024 clocks of MFMA work: at full MFMA rate
// the path would be busy all the time, and the kernel is bound by it at a third of the peak.
// Twice the tile edge halves the bytes per flop, in the memory path and in LDS alike:
//
//  * a workgroup of four waves computes 256 x 256; each wave a 128 x 128 quarter as 4 x 4 tiles of
//    v_mfma_f32_32x32x16_bf16, its 256 accumulators in the accumulation registers; one wave per
//    SIMD, so the overlap of loads, LDS reads and MFMAs is inside the wave;
//  * 256 x 32 slabs of both operands travel from global memory STRAIGHT into LDS
//    (global_load_lds_dwordx4: no staging registers, which the accumulators leave no room for),
//    three slabs ahead of the one being multiplied, four stages, one barrier per slab; rows are
//    not padded, their chunks are stored permuted against bank conflicts;
//  * workgroups are numbered so that each XCD works on a compact group of tiles.
//
// A product whose 256-row tiles would leave compute units idle takes tiles of 128 rows (each wave
// 64 rows): 2,048 rows by 3,072 features are 128 tiles of 256 x 192 but exactly 256 of 128 x 192.
// Such a tile moves more bytes per flop through LDS and the memory path, so it is used only where
// it fills the chip better.
//
// It needs enough tiles to fill the chip (the caller checks): 2,048 rows by 8,192 gated features
// are 512 tiles. Epilogues as the other products: store, add into the residual stream, SwiGLU
// (a tile holds 128 gate and the 128 up features of the same columns; a lane holds both of an
// element). The reference's prompt GEMM is a 64x64 tile of plain FMAs without tensor cores
// (native/include/flyweight_v2_native_kernels.hpp:233-311).
#include "fw_common.h"
#include "fw_kernels.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

#define BT 256                  // tile edge (rows: of the tall tiles)
#define BK 32                   // k per slab: an LDS row is 64 bytes, four 16-byte chunks
#define BSTAGES 4               // slabs in LDS: one is multiplied, three are on their way
#define BSLAB (BT * BK * 2)     // bytes of one operand's slab
#define BGROUP_M 4
#define B_LOADS 4               // most wave-wide loads (16 rows of 64 bytes) per wave per operand per slab

enum { MB_STORE = 0, MB_ACCUMULATE = 1, MB_SWIGLU = 2 };

__device__ __forceinline__ float silu_big(float g) {
    if (g >= 0.0f) return g / (1.0f + __expf(-g));
    const float e = __expf(g);
    return g * e / (1.0f + e);
}
// The same without a branch and with the hardware reciprocal (within an ulp or two of the above:
// far below the bfloat16 the result is rounded to). exp(-g) overflows to infinity for very
// negative g, whose reciprocal is 0: the result is -0, as it should be.
__device__ __forceinline__ float silu_quick(float g) { return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)); }
// two floats -> two bfloat16 in one word, round to nearest even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
// the value the neighbouring lane (lane ^ 1) holds
__device__ __forceinline__ float from_neighbour(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
}

template <int TM, int TN>
struct BigTile {
    static constexpr int ROWS = 2 * TM * 32;               // rows of a tile
    static constexpr int WIDE = 2 * TN * 32;               // columns of a tile
    static constexpr int A_LOADS = ROWS / 64;              // wave-wide loads per wave for a slab of a (16 rows each)
    static constexpr int W_LOADS = WIDE / 64;              // and for a slab of w
    static constexpr int SLAB_LOADS = A_LOADS + W_LOADS;   // and for a slab of both operands
};

// K must be a multiple of BK (the loads go straight to LDS: nothing can be zeroed on the way).
// TN: 32-column product tiles per wave, 4 (a 256 x 256 tile) or 3 (256 x 192: a width of 6,144
// features gives 192 tiles of 256 columns for 256 compute units, but exactly 256 tiles of 192).
// TM: 32-row product tiles per wave, 4 (256 rows a tile) or 2 (128 rows).
template <int MODE, typename TO, int TN, int TM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_mfma_big_kernel(
    const uint16_t* __restrict__ a, const uint16_t* __restrict__ w, const float* __restrict__ bias,
    TO* __restrict__ out, int M, int N, int K, int tiles_m, int tiles_n, int per_xcd, int up_offset) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];      // [stage][a slab | w slab]
    const int total = tiles_m * tiles_n;
    const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (logical >= total) return;
    const int width = BGROUP_M * tiles_n;
    const int group = logical / width;
    const int first_m = group * BGROUP_M;
    const int group_size = tiles_m - first_m < BGROUP_M ? tiles_m - first_m : BGROUP_M;
    const int pid_m = first_m + (logical % width) % group_size;
    const int pid_n = (logical % width) / group_size;
    static_assert((TN == 4 && TM == 4) || (MODE != MB_SWIGLU && (TN == 3 || TN == 4) && (TM == 2 || TM == 4)),
                  "narrower or lower tiles: store and accumulate only");
    constexpr int ROWS = BigTile<TM, TN>::ROWS, WIDE = BigTile<TM, TN>::WIDE;
    constexpr int A_LOADS = BigTile<TM, TN>::A_LOADS, W_LOADS = BigTile<TM, TN>::W_LOADS, SLAB_LOADS = BigTile<TM, TN>::SLAB_LOADS;
    const int features = MODE == MB_SWIGLU ? BT / 2 : WIDE;
    const int m0 = pid_m * ROWS, n0 = pid_n * features;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // The copy: a wave-wide load writes 1,024 contiguous bytes of LDS, lane l its 16 bytes at
    // l * 16: 16 rows of 64 bytes. Rows are not padded; instead the four chunks of a row are
    // stored permuted (chunk c of row r in slot c ^ ((r / 4) % 4)), so that the 16-byte operand
    // reads of 16 consecutive rows cover all 64 banks once (rows r, r + 4, r + 8, r + 12 would
    // otherwise share theirs). Lane l therefore ASKS for chunk (l % 4) ^ ((r / 4) % 4) of row
    // r = l / 4 of its 16 rows.
    const uint16_t* a_src[B_LOADS];
    const uint16_t* w_src[B_LOADS];     // W_LOADS of them are used (with w_src[W_LOADS] the host pass emitted no launch stub)
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        const int row = (wave * A_LOADS + i) * 16 + (lane >> 2);
        const int chunk = (lane & 3) ^ ((row >> 2) & 3);
        int am = m0 + row;
        am = am < M ? am : M - 1;                       // rows past the end are computed and dropped
        a_src[i] = a + (size_t)am * K + chunk * 8;
    }
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
        const int row = (wave * W_LOADS + i) * 16 + (lane >> 2);
        const int chunk = (lane & 3) ^ ((row >> 2) & 3);
        int wr;
        if (MODE == MB_SWIGLU) wr = row < BT / 2 ? n0 + row : up_offset + n0 + row - BT / 2;
        else wr = n0 + row;
        const int limit = MODE == MB_SWIGLU ? (row < BT / 2 ? N : up_offset + N) : N;
        wr = wr < limit ? wr : limit - 1;
        w_src[i] = w + (size_t)wr * K + chunk * 8;
    }
    auto request = [&](int slab) {
        unsigned char* stage = lds + (slab % BSTAGES) * 2 * BSLAB;
        const int k0 = slab * BK;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
            __builtin_amdgcn_global_load_lds(a_src[i] + k0, reinterpret_cast<uint32_t*>(stage + (wave * A_LOADS + i) * 1024), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i)
            __builtin_amdgcn_global_load_lds(w_src[i] + k0, reinterpret_cast<uint32_t*>(stage + BSLAB + (wave * W_LOADS + i) * 1024), 16, 0, 0);
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // this wave's rows of the a slab, and its rows of the w slab: for SwiGLU the columns of a wave
    // are 64 gate features (tiles 0, 1) and the 64 up features of the same columns (tiles 2, 3)
    const int a_row0 = wm * (TM * 32) + (lane & 31);
    int b_row[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
        b_row[j] = MODE == MB_SWIGLU ? (j >> 1) * (BT / 2) + wn * 64 + (j & 1) * 32 + (lane & 31) : wn * (TN * 32) + j * 32 + (lane & 31);
    // every row this lane reads is (lane % 32) plus a multiple of 32: one permutation for all
    const int swizzle = ((lane & 31) >> 2) & 3;
    int slot[BK / 16];
#pragma unroll
    for (int t = 0; t < BK / 16; ++t) slot[t] = ((2 * t + (lane >> 5)) ^ swizzle) * 16;

    // operand registers of one k16 step: the wave's row tiles of a and column tiles of w
    struct Operands {
        bf16x8 fa[TM], fb[TN];
    };
    auto read = [&](Operands& f, int slab, int t) {
        const unsigned char* sa = lds + (slab % BSTAGES) * 2 * BSLAB;
        const unsigned char* sb = sa + BSLAB;
#pragma unroll
        for (int i = 0; i < TM; ++i)
            f.fa[i] = *reinterpret_cast<const bf16x8*>(sa + (a_row0 + 32 * i) * (BK * 2) + slot[t]);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            f.fb[j] = *reinterpret_cast<const bf16x8*>(sb + b_row[j] * (BK * 2) + slot[t]);
    };
    auto multiply = [&](const Operands& f, int first_row_tile, int row_tiles) {
#pragma unroll
        for (int i = first_row_tile; i < first_row_tile + row_tiles; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.fa[i], f.fb[j], acc[i][j], 0, 0, 0);
    };
    // Asks the scheduler to issue `count` times: `mfmas` MFMAs, then one instruction of `kind`
    // (0x100 LDS read, 0x020 global load). A wave issues in order and an MFMA holds the matrix
    // pipe for 32 clocks, so whatever sits between two MFMAs costs nothing.
#define FW_INTERLEAVE(count, mfmas, kind)                          \
    _Pragma("unroll") for (int u = 0; u < (count); ++u) {          \
        __builtin_amdgcn_sched_group_barrier(0x008, (mfmas), 0);   \
        __builtin_amdgcn_sched_group_barrier((kind), 1, 0);        \
    }
    // Tells the compiler that these operands are needed HERE, so that it waits for their LDS reads
    // before the next reads are issued and not, for all reads together, in front of the MFMAs.
    auto arrived = [&](const Operands& f) {
        asm volatile("" ::"v"(f.fa[0]), "v"(f.fa[1]), "v"(f.fa[TM - 2]), "v"(f.fa[TM - 1]), "v"(f.fb[0]), "v"(f.fb[1]), "v"(f.fb[2]), "v"(f.fb[TN - 1]));
    };
    // waits until at most `slabs` of this wave's requested slabs are still on their way (SLAB_LOADS loads each)
    auto wait_for_all_but = [&](int slabs) {
        if (slabs >= 3) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * SLAB_LOADS) : "memory");
        else if (slabs == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * SLAB_LOADS) : "memory");
        else if (slabs == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(1 * SLAB_LOADS) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };

    // Four stages: while slab s is multiplied, slabs s + 1 .. s + 3 are in LDS or on their way.
    // The two k16 steps of a slab are software-pipelined by hand, because with one wave per SIMD
    // nothing else hides the latency of LDS: the operands of the next step are read between the
    // MFMAs of this step. In the middle of step 0 of slab s the wave makes sure that slab s + 1
    // has landed (its own loads: vmcnt; everybody's: the barrier), which also tells that every
    // wave has read the last of slab s, whose stage then takes slab s + 4.
    const int steps = K / BK;
    for (int s = 0; s < BSTAGES && s < steps; ++s) request(s);
    wait_for_all_but((steps < BSTAGES ? steps : BSTAGES) - 1);
    __builtin_amdgcn_s_barrier();
    Operands f0, f1;
    read(f0, 0, 0);
    int s = 0;
    // steady state: slab s + 4 exists, nothing is conditional, so that each part is one run of
    // instructions the scheduler can interleave
    for (; s + BSTAGES < steps; ++s) {
        // first half of step 0 of slab s, with the reads of step 1 between its MFMAs
        arrived(f0);
        read(f1, s, 1);
        multiply(f0, 0, TM / 2);
        FW_INTERLEAVE(TM / 2 * TN, 1, 0x100)    // (where the reads outnumber the MFMAs the rest is left to the scheduler)
        __builtin_amdgcn_sched_barrier(0);
        arrived(f1);                                        // slab s has been read
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * SLAB_LOADS) : "memory");   // slab s + 1 has landed; s + 2 and s + 3 may still fly
        __builtin_amdgcn_s_barrier();
        // second half, with the requests for slab s + 4 between its MFMAs
        request(s + BSTAGES);
        multiply(f0, TM / 2, TM / 2);
        FW_INTERLEAVE(TM / 2 * TN, 1, 0x020)
        __builtin_amdgcn_sched_barrier(0);
        // step 1, with the reads of step 0 of slab s + 1 between its MFMAs
        read(f0, s + 1, 0);
        multiply(f1, 0, TM);
        FW_INTERLEAVE(2 * TN, TM / 2, 0x100)
        __builtin_amdgcn_sched_barrier(0);
    }
    // the last slabs: nothing more to request
    for (; s < steps; ++s) {
        arrived(f0);
        read(f1, s, 1);
        multiply(f0, 0, TM);
        __builtin_amdgcn_sched_barrier(0);
        arrived(f1);
        if (s + 1 < steps) {
            wait_for_all_but(steps - 2 - s);                // slabs s + 2 .. may still fly
            __builtin_amdgcn_s_barrier();
            read(f0, s + 1, 0);
        }
        multiply(f1, 0, TM);
        __builtin_amdgcn_sched_barrier(0);
    }
#undef FW_INTERLEAVE
    fw_mfma_drain();     // branches follow that lead to code reading the accumulators

    // D layout of the 32x32 product: lane holds column lane % 32; register r is row
    // 8 * (r / 4) + 4 * (lane / 32) + r % 4
    const int col = lane & 31, row_base = (lane >> 5) * 4;
    // A tile that lies wholly inside the output (and an even N for the two-byte kinds) takes the
    // quick way: no bounds, no branches, pointers stepped by rows, and for bfloat16 two
    // neighbouring lanes swap one value each so that each stores a pair of columns as one word.
    // With one workgroup per compute unit nothing runs beside the epilogue, so its length counts.
    const bool inside = m0 + ROWS <= M && n0 + features <= N && (sizeof(TO) == 4 || (N & 1) == 0);
    const bool odd = lane & 1;
    if constexpr (MODE == MB_SWIGLU) {
        if (inside) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                uint16_t* pair = reinterpret_cast<uint16_t*>(out) + (size_t)(m0 + wm * (TM * 32) + row_base) * N +
                                 (n0 + wn * 64 + j * 32 + (col & ~1));
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const int r = 4 * q + 2 * h;        // rows 8 q + 2 h and the one below, of row tile i
                            const float upper = silu_quick(acc[i][j][r]) * acc[i][j + 2][r];
                            const float lower = silu_quick(acc[i][j][r + 1]) * acc[i][j + 2][r + 1];
                            const float got = from_neighbour(odd ? upper : lower);
                            const uint32_t word = odd ? pack_bf16x2(got, lower) : pack_bf16x2(upper, got);
                            const int row = i * 32 + 8 * q + 2 * h + (odd ? 1 : 0);
                            *reinterpret_cast<uint32_t*>(pair + (size_t)row * N) = word;
                        }
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int n = n0 + wn * 64 + j * 32 + col;
            if (n >= N) continue;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = m0 + wm * (TM * 32) + i * 32 + 8 * (r >> 2) + row_base + (r & 3);
                    if (m < M) store_from_float(out, (size_t)m * N + n, silu_quick(acc[i][j][r]) * acc[i][j + 2][r]);
                }
        }
        return;
    }
    if (inside) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn * (TN * 32) + j * 32 + col;
            const float b = bias ? bias[n] : 0.0f;
            if constexpr (sizeof(TO) == 4) {
                float* column = reinterpret_cast<float*>(out) + (size_t)(m0 + wm * (TM * 32) + row_base) * N + n;
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        float* to = column + (size_t)(i * 32 + 8 * (r >> 2) + (r & 3)) * N;
                        float value = acc[i][j][r] + b;
                        if (MODE == MB_ACCUMULATE) value += *to;
                        *to = value;
                    }
            } else {
                uint16_t* pair = reinterpret_cast<uint16_t*>(out) + (size_t)(m0 + wm * (TM * 32) + row_base) * N + (n & ~1);
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int q = 0; q < 4; ++q)
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const int r = 4 * q + 2 * h;
                            const float upper = acc[i][j][r] + b, lower = acc[i][j][r + 1] + b;
                            const float got = from_neighbour(odd ? upper : lower);
                            const uint32_t word = odd ? pack_bf16x2(got, lower) : pack_bf16x2(upper, got);
                            *reinterpret_cast<uint32_t*>(pair + (size_t)(i * 32 + 8 * q + 2 * h + (odd ? 1 : 0)) * N) = word;
                        }
            }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int n = n0 + wn * (TN * 32) + j * 32 + col;
        if (n >= N) continue;
        const float b = bias ? bias[n] : 0.0f;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * (TM * 32) + i * 32 + 8 * (r >> 2) + row_base + (r & 3);
                if (m >= M) continue;
                const size_t at = (size_t)m * N + n;
                float value = acc[i][j][r] + b;
                if (MODE == MB_ACCUMULATE) value += load_as_float(out, at);
                store_from_float(out, at, value);
            }
    }
}

template <int MODE, typename TO, int TN = 4, int TM = 4>
static int launch_big(const void* a, const void* w, const float* bias, void* out, int M, int N, int K, hipStream_t stream) {
    const int features = MODE == MB_SWIGLU ? BT / 2 : 2 * TN * 32;
    const int tiles_m = fw_ceil_div(M, 2 * TM * 32), tiles_n = fw_ceil_div(N, features);
    const int per_xcd = fw_ceil_div((long long)tiles_m * tiles_n, 8);
    const int lds_bytes = BSTAGES * 2 * BSLAB;
    static bool configured = false;     // per instantiation
    if (!configured) {
        hipError_t status = hipFuncSetAttribute((const void*)gemm_mfma_big_kernel<MODE, TO, TN, TM>,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (status != hipSuccess) {
            fw_set_error("gemm_mfma_big: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(status));
            return -1;
        }
        configured = true;
    }
    gemm_mfma_big_kernel<MODE, TO, TN, TM><<<per_xcd * 8, 256, lds_bytes, stream>>>(
        (const uint16_t*)a, (const uint16_t*)w, bias, (TO*)out, M, N, K, tiles_m, tiles_n, per_xcd, N);
    return 0;
}

// The tile a storing or accumulating product is cut into: 256 or 128 rows by 256 or 192 columns,
// whichever takes the least time by this count: rounds of tiles over the chip's 256 compute units
// times the tile's area, a tile of 128 rows counting a quarter more than its area (it moves more
// bytes per flop). Gated products (SwiGLU) keep 256 x 256, and accumulating ones 256 rows: their
// epilogue reads the old values where nothing hides the read, and twice the tiles for the same
// output pay that twice as often (2,048 x 3,072 x 2,048: storing 50.9 -> 35.6 us with tiles of
// 128 x 192, accumulating 51.6 -> 58.5 us).
struct BigPlan {
    int rows, columns, tiles;
};
static BigPlan big_plan(int mode, int M, int N) {
    if (mode == MB_SWIGLU) return {BT, BT / 2, fw_ceil_div(M, BT) * fw_ceil_div(N, BT / 2)};
    BigPlan best = {0, 0, 0};
    long long best_cost = 0;
    for (int rows = BT; rows >= (mode == MB_STORE ? BT / 2 : BT); rows /= 2)
        for (int columns = BT; columns >= 192; columns -= 64) {
            const long long tiles = (long long)fw_ceil_div(M, rows) * fw_ceil_div(N, columns);
            const long long cost = fw_ceil_div(tiles, 256) * (rows / 32) * (columns / 32) * (rows == BT ? 4 : 5);
            if (best.tiles == 0 || cost < best_cost) {
                best = {rows, columns, (int)(tiles < (1ll << 30) ? tiles : (1ll << 30))};
                best_cost = cost;
            }
        }
    return best;
}

// How many tiles the kernel cuts a shape into, by the tile it will choose (the caller decides
// whether that fills the chip); 0 if the kernel does not take the shape (K must be a multiple
// of 32).
extern "C" int fw_gemm_mfma_big_tiles(int mode, int M, int N, int K) {
    if (K <= 0 || K % BK || M < 1 || N < 1) return 0;
    return big_plan(mode, M, N).tiles;
}

// The same with the tile's edges: what the caller needs to tell how much of the tiles the output fills.
extern "C" int fw_gemm_mfma_big_plan(int mode, int M, int N, int K, int* rows, int* columns) {
    if (K <= 0 || K % BK || M < 1 || N < 1) return 0;
    const BigPlan plan = big_plan(mode, M, N);
    if (rows) *rows = plan.rows;
    if (columns) *columns = plan.columns;
    return plan.tiles;
}

template <int MODE, typename TO>
static int launch_planned(const BigPlan& plan, const void* a, const void* w, const float* bias, void* out, int M, int N, int K,
                          hipStream_t stream) {
    if (plan.rows == BT || MODE != MB_STORE)
        return plan.columns == BT ? launch_big<MODE, TO, 4, 4>(a, w, bias, out, M, N, K, stream)
                                  : launch_big<MODE, TO, 3, 4>(a, w, bias, out, M, N, K, stream);
    if constexpr (MODE == MB_STORE)
        return plan.columns == BT ? launch_big<MODE, TO, 4, 2>(a, w, bias, out, M, N, K, stream)
                                  : launch_big<MODE, TO, 3, 2>(a, w, bias, out, M, N, K, stream);
    return -1;
}

// Same contract as fw_gemm_mfma.
extern "C" int fw_gemm_mfma_big(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                                int M, int N, int K, void* stream) {
    FW_REQUIRE(M >= 1 && N > 0 && K > 0 && K % BK == 0, "gemm_mfma_big: K (%d) must be a positive multiple of %d; M=%d N=%d", K, BK, M, N);
    FW_REQUIRE(mode >= 0 && mode <= 2, "gemm_mfma_big: unknown mode %d", mode);
    FW_REQUIRE(mode != MB_ACCUMULATE || out_dtype == FW_F32, "gemm_mfma_big: accumulation needs a float32 destination");
    FW_REQUIRE(mode != MB_SWIGLU || (out_dtype == FW_BF16 && bias == nullptr), "gemm_mfma_big: SwiGLU stores bfloat16 and takes no bias");
    FW_REQUIRE(out_dtype == FW_F32 || out_dtype == FW_BF16, "gemm_mfma_big: unknown out dtype %d", out_dtype);
    FW_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_mfma_big: operands must be 16-byte aligned");
    FW_REQUIRE((long long)fw_ceil_div(M, BT / 2) * fw_ceil_div(N, BT / 2) < (1ll << 30), "gemm_mfma_big: too many tiles");
    hipStream_t s = (hipStream_t)stream;
    const BigPlan plan = big_plan(mode, M, N);
    int status;
    if (mode == MB_SWIGLU) status = launch_big<MB_SWIGLU, bf16_t>(a, w, nullptr, out, M, N, K, s);
    else if (mode == MB_ACCUMULATE) status = launch_planned<MB_ACCUMULATE, float>(plan, a, w, bias, out, M, N, K, s);
    else if (out_dtype == FW_F32) status = launch_planned<MB_STORE, float>(plan, a, w, bias, out, M, N, K, s);
    else status = launch_planned<MB_STORE, bf16_t>(plan, a, w, bias, out, M, N, K, s);
    if (status != 0) return status;
    FW_LAUNCH_CHECK("gemm_mfma_big");
    return 0;
}
