// Tiled matrix product for prompts: out[M][N] = a[M][K] . w[N][K]^T, bfloat16 operands,
// float32 accumulation on the matrix cores (v_mfma_f32_32x32x16_bf16).
//
// A workgroup of four waves computes a 128 x 128 tile; each wave a 64 x 64 quarter as 2 x 2
// MFMA tiles. Both operands are k-contiguous, so a 128 x 64 slab of each is copied per
// iteration: global -> registers (requested two slabs ahead of the one being multiplied) ->
// LDS (one slab ahead), two LDS buffers, one barrier per iteration. LDS rows are padded from 128 to
// 144 bytes so that the 16-byte operand reads of 16 consecutive rows fall into different
// banks. Workgroups are numbered so that each XCD (every eighth workgroup id) works on a
// compact group of tiles and finds its operands in its own L2.
//
// Epilogues: store (bfloat16 or float32), add into the float32 residual stream, or SwiGLU
// (w = gate rows then up rows; a workgroup takes 64 features of each, every wave holds gate
// and up of the same element in one lane, and silu(gate) * up is stored as bfloat16).
//
// A product of a few hundred rows with a narrow output has fewer tiles than the chip has compute
// units (128 rows x 2,048 features: 32). There K is cut into slices (blockIdx.y), each slice's
// workgroup leaves its float32 sums in a workspace, and the last workgroup of a tile to arrive (a
// ticket from an atomic counter) adds the slices in their order and runs the epilogue: the result
// does not depend on timing, nobody waits for anybody, and the counter is left at zero.
// The reference's prompt GEMM is a 64x64 tile of plain FMAs without tensor cores
// (native/include/flyweight_v2_native_kernels.hpp:233-311).
#include "fw_common.h"
#include "fw_kernels.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

#define TM 128
#define TN 128
#define TK 64
#define ROW_BYTES 144           // 64 bf16 + 16 bytes of padding
#define GROUP_M 8

enum { MF_STORE = 0, MF_ACCUMULATE = 1, MF_SWIGLU = 2 };

__device__ __forceinline__ float silu_fast(float g) {
    if (g >= 0.0f) return g / (1.0f + __expf(-g));
    const float e = __expf(g);
    return g * e / (1.0f + e);
}

// BN: features per workgroup tile (128, or 64 so that narrow outputs still give every compute
// unit two workgroups). Each wave computes 64 x (BN / 2) as 2 x (BN / 64) MFMA tiles.
// SPLIT: K is cut into slices of k_per_split (a multiple of TK), one per blockIdx.y.
template <int MODE, int BN, typename TO, bool SPLIT>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(
    const uint16_t* __restrict__ a, const uint16_t* __restrict__ w, const float* __restrict__ bias,
    TO* __restrict__ out, int M, int N, int K, int tiles_m, int tiles_n, int per_xcd, int up_offset,
    int k_per_split, float* partials, int* counters) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    constexpr int NJ = BN / 64;                     // MFMA tiles per wave along the features
    constexpr int W_CHUNKS = BN / 32;               // 16-byte runs of W per thread per slab
    constexpr int A_SLAB = TM * ROW_BYTES, W_SLAB = BN * ROW_BYTES;
    // [buffer][a slab | w slab]
    const int total = tiles_m * tiles_n;
    const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (logical >= total) return;
    const int width = GROUP_M * tiles_n;
    const int group = logical / width;
    const int first_m = group * GROUP_M;
    const int group_size = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
    const int pid_m = first_m + (logical % width) % group_size;
    const int pid_n = (logical % width) / group_size;
    const int features = MODE == MF_SWIGLU ? BN / 2 : BN;
    const int m0 = pid_m * TM, n0 = pid_n * features;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int k_first = SPLIT ? blockIdx.y * k_per_split : 0;
    const int k_limit = SPLIT ? (K < k_first + k_per_split ? K : k_first + k_per_split) : K;

    // what this thread copies: runs of 16 bytes at (row tid / 8 + 32 i, k 8 * (tid % 8)); the
    // pointers are to the rows, the column is added at each load so that it can be clamped
    const uint16_t* a_src[4];
    const uint16_t* w_src[W_CHUNKS];
    int lds_at[4];
    const int kc = (tid & 7) * 8;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = (tid >> 3) + 32 * i;
        int am = m0 + row;
        am = am < M ? am : M - 1;                       // rows past the end are computed and dropped
        a_src[i] = a + (size_t)am * K;
        lds_at[i] = row * ROW_BYTES + (tid & 7) * 16;
        if (i < W_CHUNKS) {
            int wr;
            if (MODE == MF_SWIGLU) wr = row < BN / 2 ? n0 + row : up_offset + n0 + row - BN / 2;
            else wr = n0 + row;
            const int limit = MODE == MF_SWIGLU ? (row < BN / 2 ? N : up_offset + N) : N;
            wr = wr < limit ? wr : limit - 1;
            w_src[i] = w + (size_t)wr * K;
        }
    }

    f32x16 acc[2][NJ];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // Two slabs are on their way from global memory while a third is multiplied: what limits
    // this kernel is the latency of those loads times the bytes in flight per compute unit.
    // The two register sets are named apart (not indexed) so that they stay in registers.
    u32x4 ra0[4], rw0[W_CHUNKS], ra1[4], rw1[W_CHUNKS];
    const u32x4 zero = {0u, 0u, 0u, 0u};
    auto fetch = [&](u32x4 (&ra)[4], u32x4 (&rw)[W_CHUNKS], int k0) {
        // Every load is issued unconditionally (past the end of K from column 0) and nothing
        // touches the value until it moves to LDS: a branch around a load, or arithmetic right
        // behind it, would make the compiler wait for loads in flight.
        const int from = k0 + kc < k_limit ? k0 + kc : 0;   // K is a multiple of 8: columns 0..7 always exist
#pragma unroll
        for (int i = 0; i < 4; ++i) ra[i] = *reinterpret_cast<const u32x4*>(a_src[i] + from);
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) rw[i] = *reinterpret_cast<const u32x4*>(w_src[i] + from);
    };
    auto stash = [&](const u32x4 (&ra)[4], const u32x4 (&rw)[W_CHUNKS], int buffer, int k0) {
        unsigned char* base = lds + buffer * (A_SLAB + W_SLAB);
        const bool ok = k0 + kc < k_limit;              // a past the end of the slice is zero; W may then be anything finite
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(base + lds_at[i]) = ok ? ra[i] : zero;
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) *reinterpret_cast<u32x4*>(base + A_SLAB + lds_at[i]) = rw[i];
    };

    const int a_row0 = wm * 64 + (lane & 31);
    int b_row[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
        b_row[j] = MODE == MF_SWIGLU ? j * (BN / 2) + wn * (BN / 4) + (lane & 31) : wn * (BN / 2) + j * 32 + (lane & 31);
    const int k_lane = (lane >> 5) * 16;                // byte offset of this lane's 8 k within a k16 step

    auto multiply = [&](int buffer) {
        const unsigned char* sa = lds + buffer * (A_SLAB + W_SLAB);
        const unsigned char* sb = sa + A_SLAB;
#pragma unroll
        for (int k16 = 0; k16 < TK / 16; ++k16) {
            bf16x8 fa[2], fb[NJ];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                fa[i] = *reinterpret_cast<const bf16x8*>(sa + (a_row0 + 32 * i) * ROW_BYTES + k16 * 32 + k_lane);
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                fb[j] = *reinterpret_cast<const bf16x8*>(sb + b_row[j] * ROW_BYTES + k16 * 32 + k_lane);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    };

    // slab s travels: global -> register set s % 2 (requested while slab s - 2 is multiplied)
    // -> LDS buffer s % 2 (stored while slab s - 1 is multiplied) -> multiplied. The steady
    // state has no branches, so the compiler can count exactly which loads it must wait for.
    const int steps = (k_limit - k_first + TK - 1) / TK;
    int step = 0;
    // The barriers order LDS traffic only: the loads just requested stay in flight across them.
    fetch(ra0, rw0, k_first);
    fetch(ra1, rw1, k_first + TK);                      // past the end: dropped when stored
    stash(ra0, rw0, 0, k_first);
    fw_lds_barrier();
    while (step + 3 < steps) {
        fetch(ra0, rw0, k_first + (step + 2) * TK);
        __builtin_amdgcn_sched_barrier(0);              // keep the requests ahead of the work they overlap
        multiply(0);
        stash(ra1, rw1, 1, k_first + (step + 1) * TK);
        fw_lds_barrier();
        fetch(ra1, rw1, k_first + (step + 3) * TK);
        __builtin_amdgcn_sched_barrier(0);
        multiply(1);
        stash(ra0, rw0, 0, k_first + (step + 2) * TK);
        fw_lds_barrier();
        step += 2;
    }
    // at most three slabs are left: slab `step` is in buffer 0, slab step + 1 in set 1
    if (step + 2 < steps) fetch(ra0, rw0, k_first + (step + 2) * TK);
    multiply(0);
    if (step + 1 < steps) {
        stash(ra1, rw1, 1, k_first + (step + 1) * TK);
        fw_lds_barrier();
        multiply(1);
        if (step + 2 < steps) {
            stash(ra0, rw0, 0, k_first + (step + 2) * TK);
            fw_lds_barrier();
            multiply(0);
        }
    }
    fw_mfma_drain();     // the branches below lead to code that reads the accumulators

    // The slices of K meet in the workspace: [slice][tile][accumulator register][thread]. The
    // sums are written and read with device-scope accesses (past the caches that workgroups on
    // different dies do not share); a wave waits for its own stores, the workgroup meets, one
    // thread takes the ticket, and the last workgroup of the tile adds the slices in their order.
    if (SPLIT && gridDim.y > 1) {
        constexpr int REGS = 2 * NJ * 16;
        __shared__ int ticket_shared;
        float* mine = partials + ((size_t)blockIdx.y * total + logical) * REGS * 256 + tid;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    __hip_atomic_store(mine + (size_t)((i * NJ + j) * 16 + r) * 256, acc[i][j][r], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) ticket_shared = __hip_atomic_fetch_add(&counters[logical], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (ticket_shared != (int)gridDim.y - 1) return;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
        // the sums of several slices are requested together (their latency is what this costs) and
        // added in slice order
        constexpr int AHEAD = NJ == 1 ? 4 : 2;
        const int slices = (int)gridDim.y;
        for (int slice = 0; slice < slices; slice += AHEAD) {
            float v[AHEAD][REGS];
#pragma unroll
            for (int u = 0; u < AHEAD; ++u) {
                const int from = slice + u < slices ? slice + u : slices - 1;
                const float* theirs = partials + ((size_t)from * total + logical) * REGS * 256 + tid;
#pragma unroll
                for (int r = 0; r < REGS; ++r)
                    v[u][r] = __hip_atomic_load(theirs + (size_t)r * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
            for (int u = 0; u < AHEAD; ++u)
                if (slice + u < slices)
#pragma unroll
                    for (int i = 0; i < 2; ++i)
#pragma unroll
                        for (int j = 0; j < NJ; ++j)
#pragma unroll
                            for (int r = 0; r < 16; ++r) acc[i][j][r] += v[u][(i * NJ + j) * 16 + r];
        }
        if (tid == 0) __hip_atomic_store(&counters[logical], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // D layout of the 32x32 product: lane holds column lane % 32; register r is row
    // 8 * (r / 4) + 4 * (lane / 32) + r % 4
    const int col = lane & 31, row_base = (lane >> 5) * 4;
    if (MODE == MF_SWIGLU) {
        static_assert(MODE != MF_SWIGLU || NJ == 2, "the SwiGLU tile holds gate and up side by side");
        const int n = n0 + wn * (BN / 4) + col;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + row_base + (r & 3);
                if (m < M && n < N)
                    store_from_float(out, (size_t)m * N + n, silu_fast(acc[i][0][r]) * acc[i][NJ - 1][r]);
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int n = n0 + wn * (BN / 2) + j * 32 + col;
            if (n >= N) continue;
            const float b = bias ? bias[n] : 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + row_base + (r & 3);
                if (m >= M) continue;
                const size_t at = (size_t)m * N + n;
                float value = acc[i][j][r] + b;
                if (MODE == MF_ACCUMULATE) value += load_as_float(out, at);
                store_from_float(out, at, value);
            }
        }
}

// slices == 0: K is not cut (and the kernel has no code for it)
template <int MODE, int BN, typename TO, bool SPLIT = false>
static int launch(const void* a, const void* w, const float* bias, void* out, int M, int N, int K, hipStream_t stream,
                  int slices = 0, int k_per_split = 0, float* partials = nullptr, int* counters = nullptr) {
    const int features = MODE == MF_SWIGLU ? BN / 2 : BN;
    const int tiles_m = fw_ceil_div(M, TM), tiles_n = fw_ceil_div(N, features);
    const int per_xcd = fw_ceil_div((long long)tiles_m * tiles_n, 8);
    const int lds_bytes = 2 * (TM + BN) * ROW_BYTES;
    static bool configured = false;     // per instantiation
    if (!configured) {
        hipError_t status = hipFuncSetAttribute((const void*)gemm_mfma_kernel<MODE, BN, TO, SPLIT>,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (status != hipSuccess) {
            fw_set_error("gemm_mfma: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(status));
            return -1;
        }
        configured = true;
    }
    gemm_mfma_kernel<MODE, BN, TO, SPLIT><<<dim3(per_xcd * 8, SPLIT ? slices : 1), 256, lds_bytes, stream>>>(
        (const uint16_t*)a, (const uint16_t*)w, bias, (TO*)out, M, N, K, tiles_m, tiles_n, per_xcd, N, k_per_split, partials,
        counters);
    return 0;
}

// Narrow outputs take 64-feature tiles when 128-feature ones would give at most one workgroup
// per compute unit (measured at 2,048 rows: 2048 features 42 vs 51 us, 3072 features 63 vs 49 us);
// with a long K and exactly one 128-feature tile per compute unit the wider tile wins again (less
// traffic per flop: 2,048 features, K 8,192: 111 vs 126 us).
template <int MODE, typename TO>
static int launch_by_width(const void* a, const void* w, const float* bias, void* out, int M, int N, int K, hipStream_t stream) {
    const long long tiles128 = (long long)fw_ceil_div(M, TM) * fw_ceil_div(N, TN);
    if (tiles128 < 256 || (tiles128 == 256 && K < 4096)) return launch<MODE, 64, TO>(a, w, bias, out, M, N, K, stream);
    return launch<MODE, 128, TO>(a, w, bias, out, M, N, K, stream);
}

// mode 0: out = a . w^T (+ bias) stored as out_dtype; 1: out (float32) += a . w^T (+ bias);
// 2: w is [2 * N][K] (gate rows, then up rows); out [M][N] bfloat16 = silu(gate) * up.
extern "C" int fw_gemm_mfma(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                            int M, int N, int K, void* stream) {
    FW_REQUIRE(M >= 1 && N > 0 && K > 0 && K % 8 == 0, "gemm_mfma: K (%d) must be a positive multiple of 8; M=%d N=%d", K, M, N);
    FW_REQUIRE(mode >= 0 && mode <= 2, "gemm_mfma: unknown mode %d", mode);
    FW_REQUIRE(mode != MF_ACCUMULATE || out_dtype == FW_F32, "gemm_mfma: accumulation needs a float32 destination");
    FW_REQUIRE(mode != MF_SWIGLU || (out_dtype == FW_BF16 && bias == nullptr), "gemm_mfma: SwiGLU stores bfloat16 and takes no bias");
    FW_REQUIRE(out_dtype == FW_F32 || out_dtype == FW_BF16, "gemm_mfma: unknown out dtype %d", out_dtype);
    FW_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_mfma: operands must be 16-byte aligned");
    FW_REQUIRE((long long)fw_ceil_div(M, TM) * fw_ceil_div(N, TN / 2) < (1ll << 30), "gemm_mfma: too many tiles");
    hipStream_t s = (hipStream_t)stream;
    int status;
    if (mode == MF_SWIGLU) status = launch<MF_SWIGLU, 128, bf16_t>(a, w, nullptr, out, M, N, K, s);
    else if (mode == MF_ACCUMULATE) status = launch_by_width<MF_ACCUMULATE, float>(a, w, bias, out, M, N, K, s);
    else if (out_dtype == FW_F32) status = launch_by_width<MF_STORE, float>(a, w, bias, out, M, N, K, s);
    else status = launch_by_width<MF_STORE, bf16_t>(a, w, bias, out, M, N, K, s);
    if (status != 0) return status;
    FW_LAUNCH_CHECK("gemm_mfma");
    return 0;
}

// ----- K cut into slices, for products with fewer tiles than compute units ---------------------
struct SplitPlan {
    int tiles, slices, k_per_split;
    size_t workspace_bytes;
};

static SplitPlan split_plan(int mode, int M, int N, int K) {
    SplitPlan plan;
    const int bn = mode == MF_SWIGLU ? 128 : 64;        // 64 features of the output either way
    plan.tiles = fw_ceil_div(M, TM) * fw_ceil_div(N, 64);
    int slices = 1;
    if (plan.tiles < 192) {
        slices = (256 + plan.tiles / 2) / plan.tiles;   // about one workgroup per compute unit (two gain nothing)
        const int most = K / (4 * TK);                  // at least four slabs per slice
        slices = slices > most ? most : slices;
        slices = slices > 8 ? 8 : slices;               // what the last workgroup of a tile has to add
        slices = slices < 1 ? 1 : slices;
    }
    plan.k_per_split = fw_ceil_div(fw_ceil_div(K, slices), TK) * TK;
    plan.slices = fw_ceil_div(K, plan.k_per_split);
    plan.workspace_bytes = plan.slices > 1 ? (size_t)plan.slices * plan.tiles * TM * bn * sizeof(float) : 0;
    return plan;
}

// What fw_gemm_mfma_split needs for a shape: bytes of float32 workspace and the number of int32
// counters (zero before the first call; left zero). Both 0: the product has tiles enough, use
// fw_gemm_mfma.
extern "C" int fw_gemm_mfma_split_plan(int mode, int M, int N, int K, size_t* workspace_bytes, int* counters) {
    FW_REQUIRE(M >= 1 && N > 0 && K > 0 && mode >= 0 && mode <= 2, "gemm_mfma_split: M %d N %d K %d mode %d", M, N, K, mode);
    FW_REQUIRE((long long)fw_ceil_div(M, TM) * fw_ceil_div(N, 64) < (1ll << 30), "gemm_mfma_split: too many tiles");
    const SplitPlan plan = split_plan(mode, M, N, K);
    *workspace_bytes = plan.workspace_bytes;
    *counters = plan.slices > 1 ? plan.tiles : 0;
    return 0;
}

// fw_gemm_mfma's contract with K cut into slices as fw_gemm_mfma_split_plan says. Calls that
// overlap on one device must not share counters or workspace.
extern "C" int fw_gemm_mfma_split(const void* a, const void* w, const float* bias, void* out, int out_dtype, int mode,
                                  int M, int N, int K, void* workspace, size_t workspace_bytes, int* counters,
                                  int counters_len, void* stream) {
    FW_REQUIRE(M >= 1 && N > 0 && K > 0 && K % 8 == 0, "gemm_mfma_split: K (%d) must be a positive multiple of 8; M=%d N=%d", K, M, N);
    FW_REQUIRE(mode >= 0 && mode <= 2, "gemm_mfma_split: unknown mode %d", mode);
    FW_REQUIRE(mode != MF_ACCUMULATE || out_dtype == FW_F32, "gemm_mfma_split: accumulation needs a float32 destination");
    FW_REQUIRE(mode != MF_SWIGLU || (out_dtype == FW_BF16 && bias == nullptr), "gemm_mfma_split: SwiGLU stores bfloat16 and takes no bias");
    FW_REQUIRE(out_dtype == FW_F32 || out_dtype == FW_BF16, "gemm_mfma_split: unknown out dtype %d", out_dtype);
    FW_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_mfma_split: operands must be 16-byte aligned");
    FW_REQUIRE((long long)fw_ceil_div(M, TM) * fw_ceil_div(N, 64) < (1ll << 30), "gemm_mfma_split: too many tiles");
    const SplitPlan plan = split_plan(mode, M, N, K);
    FW_REQUIRE(plan.slices > 1, "gemm_mfma_split: this shape (M %d N %d K %d) is not cut; use gemm_mfma", M, N, K);
    FW_REQUIRE(workspace != nullptr && workspace_bytes >= plan.workspace_bytes && counters != nullptr && counters_len >= plan.tiles &&
                   (uintptr_t)workspace % 16 == 0,
               "gemm_mfma_split: this shape needs %zu bytes of workspace and %d counters", plan.workspace_bytes, plan.tiles);
    FW_REQUIRE(plan.slices <= 65535, "gemm_mfma_split: too many slices");
    hipStream_t s = (hipStream_t)stream;
    float* partials = (float*)workspace;
    int status;
    if (mode == MF_SWIGLU) status = launch<MF_SWIGLU, 128, bf16_t, true>(a, w, nullptr, out, M, N, K, s, plan.slices, plan.k_per_split, partials, counters);
    else if (mode == MF_ACCUMULATE) status = launch<MF_ACCUMULATE, 64, float, true>(a, w, bias, out, M, N, K, s, plan.slices, plan.k_per_split, partials, counters);
    else if (out_dtype == FW_F32) status = launch<MF_STORE, 64, float, true>(a, w, bias, out, M, N, K, s, plan.slices, plan.k_per_split, partials, counters);
    else status = launch<MF_STORE, 64, bf16_t, true>(a, w, bias, out, M, N, K, s, plan.slices, plan.k_per_split, partials, counters);
    if (status != 0) return status;
    FW_LAUNCH_CHECK("gemm_mfma_split");
    return 0;
}
