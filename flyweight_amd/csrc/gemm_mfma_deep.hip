// Tiled matrix product for prompts whose output is too narrow for the 256 x 256 tiles to fill the
// chip (2,048 rows x 2,048 features: 64 large tiles for 256 compute units): out[M][N] =
// a[M][K] . w[N][K]^T with 128 x 128 tiles in which the four waves split K, not the tile.
//
// With a 128 x 128 tile cut into four 64 x 64 quarters, one per wave, every k16 step of a wave
// reads four operands from LDS for four MFMAs: at full MFMA rate the four waves would ask LDS for
// 128 bytes a clock, all it has. Here every wave computes the WHOLE tile for a quarter of the k
// range of each slab (a slab is 64 k = four k16 steps, wave w takes step w): eight operand reads
// for sixteen MFMAs, half the LDS traffic per flop, as in the 256 x 256 kernel. The price is 256
// accumulators per wave and an exchange at the end: the four partial tiles meet in LDS, each wave
// finishes four of the sixteen 32 x 32 product tiles (the parts added in the order of the waves).
//
//  * slabs of 128 rows x 64 k of both operands travel from global memory straight into LDS
//    (global_load_lds_dwordx4), three slabs ahead of the one being multiplied, four stages of
//    32 KB; a row is 128 bytes, its eight 16-byte chunks stored permuted (chunk c of row r in slot
//    c ^ ((r / 2) % 8)) so that the operand reads of sixteen consecutive rows, two rows to 256
//    bytes, cover all 64 banks once (with c ^ (r % 8) rows r and r + 8 met in the same banks:
//    two conflict cycles per MFMA on the counters);
//  * one wave per SIMD: the operands of the next slab are read between the MFMAs of this one, and
//    the loads of the slab three ahead are issued there too; one barrier per slab;
//  * workgroups are numbered so that each XCD works on a compact group of tiles.
//
// K must be a multiple of 64 (nothing can be zeroed on the way to LDS). Epilogues: store, add
// into the float32 residual stream. The reference's prompt GEMM is a 64x64 tile of plain FMAs
// without tensor cores (native/include/flyweight_v2_native_kernels.hpp:233-311).
#include "fw_common.h"
#include "fw_kernels.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

#define DT 128                  // tile edge
#define DK 64                   // k per slab: an LDS row is 128 bytes, eight 16-byte chunks
#define DSTAGES 4               // slabs in LDS: one is multiplied, three are on their way
#define DSLAB (DT * DK * 2)     // bytes of one operand's slab (16 KB)
#define DGROUP_M 4
#define D_LOADS 4               // wave-wide loads (8 rows of 128 bytes) per wave per operand per slab

enum { MD_STORE = 0, MD_ACCUMULATE = 1 };

// TN: 32-column product tiles of a tile, 4 (128 x 128) or 2 (128 x 64: an output of 1,024 features
// gives 128 tiles of 128 columns for 256 compute units, but 256 of 64; six operand reads for eight
// MFMAs then).
template <int MODE, typename TO, int TN>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_mfma_deep_kernel(
    const uint16_t* __restrict__ a, const uint16_t* __restrict__ w, const float* __restrict__ bias,
    TO* __restrict__ out, int M, int N, int K, int tiles_m, int tiles_n, int per_xcd) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];      // [stage][a slab | w slab]
    const int total = tiles_m * tiles_n;
    const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (logical >= total) return;
    const int width = DGROUP_M * tiles_n;
    const int group = logical / width;
    const int first_m = group * DGROUP_M;
    const int group_size = tiles_m - first_m < DGROUP_M ? tiles_m - first_m : DGROUP_M;
    const int pid_m = first_m + (logical % width) % group_size;
    const int pid_n = (logical % width) / group_size;
    static_assert(TN == 4 || TN == 2, "128 or 64 columns");
    constexpr int W_LOADS = TN;             // wave-wide loads per wave for a slab of w: 32 * TN rows, 8 rows a load, 4 waves
    constexpr int SLAB_LOADS = D_LOADS + W_LOADS;
    const int m0 = pid_m * DT, n0 = pid_n * (32 * TN);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    // The copy: a wave-wide load writes 1,024 contiguous bytes of LDS, lane l its 16 bytes at
    // l * 16: 8 rows of 128 bytes. Lane l asks for chunk (l % 8) ^ ((r / 2) % 8) of row r = l / 8 of
    // its 8 rows (rows past the end of a or w are read from the last row and never stored).
    const uint16_t* a_src[D_LOADS];
    const uint16_t* w_src[D_LOADS];         // W_LOADS of them are used
#pragma unroll
    for (int i = 0; i < D_LOADS; ++i) {
        const int row = (wave * D_LOADS + i) * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ ((row >> 1) & 7);
        int am = m0 + row;
        am = am < M ? am : M - 1;
        a_src[i] = a + (size_t)am * K + chunk * 8;
    }
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
        const int row = (wave * W_LOADS + i) * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ ((row >> 1) & 7);
        int wr = n0 + row;
        wr = wr < N ? wr : N - 1;
        w_src[i] = w + (size_t)wr * K + chunk * 8;
    }
    auto request = [&](int slab) {
        unsigned char* stage = lds + (slab % DSTAGES) * 2 * DSLAB;
        const int k0 = slab * DK;
#pragma unroll
        for (int i = 0; i < D_LOADS; ++i)
            __builtin_amdgcn_global_load_lds(a_src[i] + k0, reinterpret_cast<uint32_t*>(stage + (wave * D_LOADS + i) * 1024), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i)
            __builtin_amdgcn_global_load_lds(w_src[i] + k0, reinterpret_cast<uint32_t*>(stage + DSLAB + (wave * W_LOADS + i) * 1024), 16, 0, 0);
    };

    f32x16 acc[4][TN];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // This wave's k16 step of every slab: chunks 2 * wave and 2 * wave + 1 of a row, the lower for
    // lanes 0..31, the upper for lanes 32..63. Every row a lane reads is (lane % 32) plus a
    // multiple of 32, so one permutation serves all of them.
    const int slot = ((2 * wave + (lane >> 5)) ^ ((lane >> 1) & 7)) * 16;
    const int row_offset = (lane & 31) * (DK * 2) + slot;
    struct Operands {
        bf16x8 fa[4], fb[TN];
    };
    auto read = [&](Operands& f, int slab) {
        const unsigned char* sa = lds + (slab % DSTAGES) * 2 * DSLAB + row_offset;
        const unsigned char* sb = sa + DSLAB;
#pragma unroll
        for (int i = 0; i < 4; ++i) f.fa[i] = *reinterpret_cast<const bf16x8*>(sa + 32 * i * (DK * 2));
#pragma unroll
        for (int j = 0; j < TN; ++j) f.fb[j] = *reinterpret_cast<const bf16x8*>(sb + 32 * j * (DK * 2));
    };
    auto multiply = [&](const Operands& f) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.fa[i], f.fb[j], acc[i][j], 0, 0, 0);
    };
    // Asks the scheduler to issue `count` times: `mfmas` MFMAs, then one instruction of `kind`
    // (0x100 LDS read, 0x020 global load).
#define FW_INTERLEAVE(count, mfmas, kind)                          \
    _Pragma("unroll") for (int u = 0; u < (count); ++u) {          \
        __builtin_amdgcn_sched_group_barrier(0x008, (mfmas), 0);   \
        __builtin_amdgcn_sched_group_barrier((kind), 1, 0);        \
    }
    auto arrived = [&](const Operands& f) {
        asm volatile("" ::"v"(f.fa[0]), "v"(f.fa[1]), "v"(f.fa[2]), "v"(f.fa[3]), "v"(f.fb[0]), "v"(f.fb[1]), "v"(f.fb[TN - 2]), "v"(f.fb[TN - 1]));
    };
    // waits until at most `slabs` of this wave's requested slabs are still on their way (SLAB_LOADS loads each)
    auto wait_for_all_but = [&](int slabs) {
        if (slabs >= 3) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * SLAB_LOADS) : "memory");
        else if (slabs == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * SLAB_LOADS) : "memory");
        else if (slabs == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(1 * SLAB_LOADS) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };

    // While slab s is multiplied, slabs s + 1 .. s + 3 are in LDS or on their way. Per slab: the
    // wave makes sure that slab s + 1 has landed (its own loads: vmcnt; everybody's: the barrier,
    // which also tells that every wave has read slab s, whose operands are in registers by then),
    // then reads the operands of slab s + 1 and asks for slab s + 4 (into the stage of slab s)
    // between the sixteen MFMAs of slab s.
    const int steps = K / DK;
    for (int s = 0; s < DSTAGES && s < steps; ++s) request(s);
    wait_for_all_but((steps < DSTAGES ? steps : DSTAGES) - 1);
    __builtin_amdgcn_s_barrier();
    Operands f0, f1;
    read(f0, 0);
    int s = 0;
    // steady state, two slabs per turn so that the operand sets keep their names
    for (; s + DSTAGES + 1 < steps; s += 2) {
        arrived(f0);                                        // slab s has been read
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * SLAB_LOADS) : "memory");   // slab s + 1 has landed; s + 2 and s + 3 may still fly
        __builtin_amdgcn_s_barrier();
        read(f1, s + 1);
        request(s + DSTAGES);
        multiply(f0);
        FW_INTERLEAVE(2 * TN, 1, 0x100)     // (with two column tiles: eight MFMAs for six reads and six loads,
        FW_INTERLEAVE(2 * TN, 1, 0x020)     //  four of each placed here, the rest left to the scheduler)
        __builtin_amdgcn_sched_barrier(0);
        arrived(f1);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * SLAB_LOADS) : "memory");
        __builtin_amdgcn_s_barrier();
        read(f0, s + 2);
        request(s + 1 + DSTAGES);
        multiply(f1);
        FW_INTERLEAVE(2 * TN, 1, 0x100)     // (with two column tiles: eight MFMAs for six reads and six loads,
        FW_INTERLEAVE(2 * TN, 1, 0x020)     //  four of each placed here, the rest left to the scheduler)
        __builtin_amdgcn_sched_barrier(0);
    }
    // the last slabs: one at a time, asking for what is left to ask for
    for (; s < steps; ++s) {
        arrived(f0);
        if (s + 1 < steps) {
            // slabs requested so far: min(steps, s + DSTAGES); those behind s + 1 may still fly
            const int requested = steps < s + DSTAGES ? steps : s + DSTAGES;
            wait_for_all_but(requested - (s + 2));
            __builtin_amdgcn_s_barrier();
            read(f1, s + 1);
            if (s + DSTAGES < steps) request(s + DSTAGES);
        }
        multiply(f0);
        __builtin_amdgcn_sched_barrier(0);
        if (s + 1 < steps) {
            arrived(f1);
            f0 = f1;
        }
    }
#undef FW_INTERLEAVE
    fw_mfma_drain();     // branches follow that lead to code reading the accumulators

    // The four partial tiles meet in LDS (free now: 128 KB), eight product tiles at a time (with
    // four column tiles: row tiles 0 and 1, then 2 and 3; with two: all at once): every wave leaves
    // its parts of the eight (4 KB each), then finishes two of them: the four parts added in the
    // order of the waves, whatever the timing, and sent through the epilogue. Which accumulators a
    // wave reads does not depend on the wave (only where it reads the parts from does), so they
    // stay where they are.
    constexpr int PASSES = TN / 2, PASS_ROWS = 8 / TN;     // passes of eight product tiles; row tiles in a pass
    f32x4* exchange = reinterpret_cast<f32x4*>(lds);       // [wave][tile of the pass][four rows][lane]
    // D layout of the 32x32 product: lane holds column lane % 32; register r is row
    // 8 * (r / 4) + 4 * (lane / 32) + r % 4
    const int col = lane & 31, row_base = (lane >> 5) * 4;
    // the accumulating epilogue's old values of the product tiles this wave will finish are asked
    // for now: they travel while the parts are exchanged (with one workgroup per compute unit
    // nothing else would hide that read)
    float old_value[PASSES][2][16];
    if (MODE == MD_ACCUMULATE) {
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int tile = wave * 2 + u, i = pass * PASS_ROWS + tile / TN, j = tile % TN;
                const int n = n0 + j * 32 + col;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = m0 + i * 32 + 8 * (r >> 2) + row_base + (r & 3);
                    old_value[pass][u][r] = load_as_float(out, (m < M && n < N) ? (size_t)m * N + n : 0);
                }
            }
    }
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
        __syncthreads();        // the operands (first pass) or the parts of the pass before have been read
#pragma unroll
        for (int i2 = 0; i2 < PASS_ROWS; ++i2)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                f32x4* to = exchange + (size_t)((wave * 8 + i2 * TN + j) * 4) * 64 + lane;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f32x16& t = acc[pass * PASS_ROWS + i2][j];
                    to[q * 64] = f32x4{t[4 * q], t[4 * q + 1], t[4 * q + 2], t[4 * q + 3]};
                }
            }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int tile = wave * 2 + u, i = pass * PASS_ROWS + tile / TN, j = tile % TN;
            const int n = n0 + j * 32 + col;
            const float b = (bias && n < N) ? bias[n] : 0.0f;
            const f32x4* from = exchange + (size_t)(tile * 4) * 64 + lane;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                f32x4 sum = from[q * 64];
#pragma unroll
                for (int part = 1; part < 4; ++part) sum += from[(size_t)(part * 8 * 4 + q) * 64];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int m = m0 + i * 32 + 8 * q + row_base + e;
                    if (m >= M || n >= N) continue;
                    const size_t at = (size_t)m * N + n;
                    float value = sum[e] + b;
                    if (MODE == MD_ACCUMULATE) value += old_value[pass][u][4 * q + e];
                    store_from_float(out, at, value);
                }
            }
        }
    }
}

template <int MODE, typename TO, int TN>
static int launch_deep(const void* a, const void* w, const float* bias, void* out, int M, int N, int K, hipStream_t stream) {
    const int tiles_m = fw_ceil_div(M, DT), tiles_n = fw_ceil_div(N, 32 * TN);
    const int per_xcd = fw_ceil_div((long long)tiles_m * tiles_n, 8);
    const int lds_bytes = DSTAGES * 2 * DSLAB;
    static bool configured = false;     // per instantiation
    if (!configured) {
        hipError_t status = hipFuncSetAttribute((const void*)gemm_mfma_deep_kernel<MODE, TO, TN>,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (status != hipSuccess) {
            fw_set_error("gemm_mfma_deep: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(status));
            return -1;
        }
        configured = true;
    }
    gemm_mfma_deep_kernel<MODE, TO, TN><<<per_xcd * 8, 256, lds_bytes, stream>>>(
        (const uint16_t*)a, (const uint16_t*)w, bias, (TO*)out, M, N, K, tiles_m, tiles_n, per_xcd);
    return 0;
}

// How many tiles a shape gives with tiles of `columns` (128 or 64) columns; 0 if the kernel does
// not take the shape (K must be a multiple of 64; SwiGLU is not served).
extern "C" int fw_gemm_mfma_deep_tiles(int mode, int M, int N, int K, int columns) {
    if (K <= 0 || K % DK || mode < 0 || mode > 1 || (columns != 128 && columns != 64)) return 0;
    return fw_ceil_div(M, DT) * fw_ceil_div(N, columns);
}

// fw_gemm_mfma's contract for modes 0 and 1, on tiles of 128 rows and `columns` (128 or 64) columns.
extern "C" int fw_gemm_mfma_deep(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                                 int M, int N, int K, int columns, void* stream) {
    FW_REQUIRE(M >= 1 && N > 0 && K > 0 && K % DK == 0, "gemm_mfma_deep: K (%d) must be a positive multiple of %d; M=%d N=%d", K, DK, M, N);
    FW_REQUIRE(mode == MD_STORE || mode == MD_ACCUMULATE, "gemm_mfma_deep: mode %d is not served", mode);
    FW_REQUIRE(columns == 128 || columns == 64, "gemm_mfma_deep: tiles have 128 or 64 columns, not %d", columns);
    FW_REQUIRE(mode != MD_ACCUMULATE || out_dtype == FW_F32, "gemm_mfma_deep: accumulation needs a float32 destination");
    FW_REQUIRE(out_dtype == FW_F32 || out_dtype == FW_BF16, "gemm_mfma_deep: unknown out dtype %d", out_dtype);
    FW_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_mfma_deep: operands must be 16-byte aligned");
    FW_REQUIRE((long long)fw_ceil_div(M, DT) * fw_ceil_div(N, 64) < (1ll << 30), "gemm_mfma_deep: too many tiles");
    hipStream_t s = (hipStream_t)stream;
    int status;
    if (columns == 128) {
        if (mode == MD_ACCUMULATE) status = launch_deep<MD_ACCUMULATE, float, 4>(a, w, bias, out, M, N, K, s);
        else if (out_dtype == FW_F32) status = launch_deep<MD_STORE, float, 4>(a, w, bias, out, M, N, K, s);
        else status = launch_deep<MD_STORE, bf16_t, 4>(a, w, bias, out, M, N, K, s);
    } else {
        if (mode == MD_ACCUMULATE) status = launch_deep<MD_ACCUMULATE, float, 2>(a, w, bias, out, M, N, K, s);
        else if (out_dtype == FW_F32) status = launch_deep<MD_STORE, float, 2>(a, w, bias, out, M, N, K, s);
        else status = launch_deep<MD_STORE, bf16_t, 2>(a, w, bias, out, M, N, K, s);
    }
    if (status != 0) return status;
    FW_LAUNCH_CHECK("gemm_mfma_deep");
    return 0;
}
