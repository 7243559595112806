// Attention over the paged cache on the matrix cores (bfloat16 cache, float32 softmax).
//
// One wave works on 16 "columns" against the keys of one kv head. For a prompt portion a
// column is a query row (16 consecutive rows of one segment and one head per wave, four such
// waves per workgroup sharing the pages through LDS). For decode
// a column is one of the query heads that share the kv head, and the keys are split between
// workgroups in runs of SPLIT_PAGES pages whose partial results (running maximum, sum and
// unnormalised output) the workgroup that finishes last merges in the order of the keys.
//
// The products are formed transposed so that nothing has to change lanes between them:
//   S^T[key][col] = K[key][d] . Q^T[d][col]        (v_mfma_f32_16x16x32_bf16, k = d)
//   O^T[d][col]  += V^T[d][key] . P^T[key][col]    (k = key)
// Lane (col, g) receives the scores of keys 4g..4g+3 of each 16-key tile, which is exactly
// what it must supply as P^T for keys {4g..4g+3} of two tiles if the 32 keys of the second
// product are taken in that order; V^T is fetched in the same order, which its layout
// ([page][kv_head][head_dim][64 keys]: a channel's keys together) makes two 8-byte loads.
// K ([page][kv_head][64 keys][head_dim]) is fetched straight into operand registers too.
// Maximum, exponentials, sums and the rescaling of O are float32; P is rounded to bfloat16
// for the second product. The reference's fast decode tier has the same split-and-merge shape
// (native/src/split_kv.h:77-124, native/src/v2_runtime.cpp:24241-24267).
#include "fw_common.h"
#include "fw_kernels.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define PAGE 64
#define SPLIT_PAGES 4           // keys per decode split = 256, whatever the batch
#define NEG_BIG (-1.0e30f)
#define PART_STRIDE(head_dim) ((head_dim) + 4)   // unnormalised output, maximum, sum, two unused: rows stay 16-byte aligned

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    return (uint32_t)float_to_bf16_bits(lo) | ((uint32_t)float_to_bf16_bits(hi) << 16);
}
// the same in one instruction (v_cvt_pk_bf16_f32, round to nearest even)
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
__device__ __forceinline__ uint32_t pack_bf16_pair(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// State of one wave: 16 columns, HD channels (HD a multiple of 32; channels >= head_dim are zero).
template <int HD>
struct Columns {
    bf16x8 q[HD / 32];          // this lane's part of Q^T: column lane % 16, d = 32 c + 8 (lane / 16) ..
    f32x4 o[HD / 16];           // O^T: column lane % 16, d = 16 t + 4 (lane / 16) + r
    float m, l;                 // running maximum (in units of log2) and this lane's share of the sum
};

// One page of 64 keys against NH sets of columns that share the keys (query heads of one kv
// group over the same rows): the keys and values are read once for all of them. `lo`/`hi`: the
// keys of this page that this lane's column may see are those with lo <= key <= hi
// (page-relative; hi < 0: none). `last_written`: keys beyond it hold whatever an earlier owner of
// the page left, and are zeroed before they meet P = 0: here if CLEAN_V, else the caller has done
// it (the prompt kernel does when it copies a page to LDS). K_PADDED: a key's row holds HD channels,
// those past head_dim zero (the prompt kernel's LDS tile), so every lane loads; else the lanes past
// head_dim take zeros without loading.
//
// The softmax arithmetic (one exponential per score on the quarter-rate unit) takes more issue
// cycles than the matrix products take on their pipe, so the work is laid out in phases, each
// over all heads, with one short branch (the mask) that touches nothing but the scores: the
// compiler can then let the products of one head run behind the arithmetic of another, and the
// accumulators stay where they are (a join of two paths that both write them costs a register
// move per accumulator and page). A page of which every key counts for every column of the wave
// (all pages but those on the diagonal, at a window's edge, and a sequence's last) skips the
// mask. The scale is folded into the exponent's argument: the maximum is taken over the raw
// scores (the scale is positive) and kept scaled.
template <int HD, int NH, bool CLEAN_V, bool K_PADDED, bool EARLY_V = false>
__device__ __forceinline__ void attend_page(Columns<HD> (&c)[NH], const uint16_t* __restrict__ k_page,
                                            const uint16_t* __restrict__ v_page, int head_dim, float scale_log2,
                                            int lo, int hi, int last_written, int k_stride, int v_stride) {
    const int lane = threadIdx.x & 63;
    const int i16 = lane & 15, g = lane >> 4;
    // all key loads of the page are issued before the first product
    bf16x8 kf[4][HD / 32];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
        const uint16_t* key = k_page + (size_t)(kt * 16 + i16) * k_stride + g * 8;
#pragma unroll
        for (int dc = 0; dc < HD / 32; ++dc) {
            if (K_PADDED) {
                kf[kt][dc] = *reinterpret_cast<const bf16x8*>(key + dc * 32);
            } else {
                kf[kt][dc] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
                if (dc * 32 + g * 8 < head_dim) kf[kt][dc] = *reinterpret_cast<const bf16x8*>(key + dc * 32);
            }
        }
    }
    // EARLY_V (pages read from global memory, one page per wave): the values are asked for
    // together with the keys, so that they travel while the scores are formed, not after them.
    u32x2 early_a[EARLY_V ? 2 : 1][EARLY_V ? HD / 16 : 1], early_b[EARLY_V ? 2 : 1][EARLY_V ? HD / 16 : 1];
    if (EARLY_V) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int t = 0; t < HD / 16; ++t) {
                const int channel = t * 16 + i16 < head_dim ? t * 16 + i16 : head_dim - 1;
                const uint16_t* value = v_page + (size_t)channel * v_stride + kb * 32 + g * 4;
                early_a[kb][t] = *reinterpret_cast<const u32x2*>(value);
                early_b[kb][t] = *reinterpret_cast<const u32x2*>(value + 16);
            }
    }
    // scores of all heads
    f32x4 s[NH][4];
#pragma unroll
    for (int h = 0; h < NH; ++h)
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            s[h][kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int dc = 0; dc < HD / 32; ++dc)
                s[h][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[kt][dc], c[h].q[dc], s[h][kt], 0, 0, 0);
        }
    const bool full = __all(lo <= 0 && hi >= PAGE - 1) && last_written >= PAGE - 1;
    if (!full) {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = kt * 16 + g * 4 + r;
                const bool seen = key >= lo && key <= hi;
#pragma unroll
                for (int h = 0; h < NH; ++h) s[h][kt][r] = seen ? s[h][kt][r] : NEG_BIG;
            }
    }
    // the running maximum of each column: over this lane's 16 scores, then over the four lanes
    // that share the column
    float alpha[NH], shift[NH];
    bool rose = false;
#pragma unroll
    for (int h = 0; h < NH; ++h) {
        float page_max = NEG_BIG;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int r = 0; r < 4; ++r) page_max = fmaxf(page_max, s[h][kt][r]);
        page_max = fw_quad_max(page_max);
        // a column that has seen no key yet keeps NEG_BIG (the raw maximum times the scale would overflow)
        const bool any_key = page_max > 0.5f * NEG_BIG;
        const float new_max = fmaxf(c[h].m, any_key ? page_max * scale_log2 : NEG_BIG);
        // the hardware's 2^x: arguments are <= 0 here, and one far below (a first page, a masked key
        // against a real maximum) gives 0
        alpha[h] = __builtin_amdgcn_exp2f(c[h].m - new_max);
        rose |= alpha[h] != 1.0f;
        c[h].m = new_max;
        // a masked score (NEG_BIG) times the scale is far below any maximum: its exponential is 0.
        // A column without any key so far (maximum NEG_BIG) subtracts nothing, so that the same holds.
        shift[h] = new_max > 0.5f * NEG_BIG ? -new_max : 0.0f;
    }
    // One head of up to 64 channels whose output lies in ordinary registers: rescaling it always
    // (sixteen multiplications by a factor that is 1 after the first pages) costs less than the
    // register moves that joining two paths, of which one writes the output, costs per page.
    if (NH == 1 && HD <= 64) {
#pragma unroll
        for (int t = 0; t < HD / 16; ++t) c[0].o[t] *= alpha[0];
    } else if (__any(rose)) {   // the maximum of some column rose (seldom after the first pages)
#pragma unroll
        for (int h = 0; h < NH; ++h)
#pragma unroll
            for (int t = 0; t < HD / 16; ++t) c[h].o[t] *= alpha[h];
    }
    uint32_t p[NH][4][2];
#pragma unroll
    for (int h = 0; h < NH; ++h) {
        float sum = 0.0f;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            float e[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                e[r] = __builtin_amdgcn_exp2f(fmaf(s[h][kt][r], scale_log2, shift[h]));
                sum += e[r];
            }
            p[h][kt][0] = pack_bf16_pair(e[0], e[1]);
            p[h][kt][1] = pack_bf16_pair(e[2], e[3]);
        }
        c[h].l = c[h].l * alpha[h] + sum;
    }
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
        bf16x8 pf[NH];
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            u32x4 pw = {p[h][2 * kb][0], p[h][2 * kb][1], p[h][2 * kb + 1][0], p[h][2 * kb + 1][1]};
            pf[h] = __builtin_bit_cast(bf16x8, pw);
        }
        const int key_a = kb * 32 + g * 4, key_b = key_a + 16;
        // keys <= last_written are kept: two keys per 32-bit word, the low half first. Without branches:
        // one between the load of V and the product would put every product into a block of its own.
        auto kept = [&](int first_key) -> uint32_t {
            return first_key + 1 <= last_written ? 0xffffffffu : (first_key <= last_written ? 0xffffu : 0u);
        };
        const uint32_t keep_a0 = kept(key_a), keep_a1 = kept(key_a + 2), keep_b0 = kept(key_b), keep_b1 = kept(key_b + 2);
        // Every channel tile of the template is computed, those past head_dim from the last real
        // channel again (their output is never stored): a branch around a matrix product whose
        // result is read right behind the branch is not safe. The compiler spaces a product and
        // the first read of its result inside one block, but where the read was the target of
        // a taken branch it came one instruction after the product and saw the registers that
        // the product writes last still unwritten (head sizes below the template's, two of four
        // components stale).
#pragma unroll
        for (int t = 0; t < HD / 16; ++t) {
            const int channel = t * 16 + i16 < head_dim ? t * 16 + i16 : head_dim - 1;
            const uint16_t* value = v_page + (size_t)channel * v_stride;
            u32x2 va, vb;
            if (EARLY_V) {
                va = early_a[kb][t];
                vb = early_b[kb][t];
            } else {
                va = *reinterpret_cast<const u32x2*>(value + key_a);
                vb = *reinterpret_cast<const u32x2*>(value + key_b);
            }
            u32x4 vw = {va[0], va[1], vb[0], vb[1]};
            if (CLEAN_V) vw = u32x4{va[0] & keep_a0, va[1] & keep_a1, vb[0] & keep_b0, vb[1] & keep_b1};
            const bf16x8 vf = __builtin_bit_cast(bf16x8, vw);
#pragma unroll
            for (int h = 0; h < NH; ++h) c[h].o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[h], c[h].o[t], 0, 0, 0);
        }
    }
    // for the same reason the last products have left the pipe before control leaves this function
    fw_mfma_drain();
}

template <int HD>
__device__ __forceinline__ void load_query(Columns<HD>& c, const uint16_t* __restrict__ q_row, int head_dim, bool valid) {
    const int g = (threadIdx.x & 63) >> 4;
#pragma unroll
    for (int dc = 0; dc < HD / 32; ++dc) {
        c.q[dc] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
        if (valid && dc * 32 + g * 8 < head_dim) c.q[dc] = *reinterpret_cast<const bf16x8*>(q_row + dc * 32 + g * 8);
    }
#pragma unroll
    for (int t = 0; t < HD / 16; ++t) c.o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    c.m = NEG_BIG;
    c.l = 0.0f;
}

// ---- prompt portions ---------------------------------------------------------------------------
// A workgroup per (tile of 64 query rows, kv head, run of NH query heads of its group), numbered
// tile by tile in the order the caller lists the tiles (those that see the most keys first: the
// short ones then fill in behind, whatever head they belong to); four waves, 16
// rows each, every wave with the same NH heads: a page's keys and values are read once for all
// of them (from global memory and from LDS), which is what a long context is bound by. Fewer
// heads per workgroup give more and shorter workgroups, which evens out a short causal prompt.
// The pages of
// the kv head are copied global -> registers (two pages ahead) -> LDS (one page ahead of the
// one being worked on; two LDS buffers, one barrier per page), so that the copy hides behind the
// softmax arithmetic. tile_seg / tile_row0: the segment of each tile and its first row (a tile never
// spans two segments). LDS rows are padded by 16 bytes against bank conflicts.
#define KV_PAD 8
// Where the kernel needs no more than 256 registers a wave it says so (two waves per SIMD at
// least): the compiler then keeps the MFMA results in ordinary registers. Left with all 512 it puts
// them into the accumulation registers, and the softmax's rescaling of the output and the masks on
// the scores then cost a move out and a move back per value and page (112 + 80 of the ~560 vector
// instructions of two pages).
template <int HD, int NH>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((HD <= 64 && NH == 1) ? 2 : 1))) void attention_prefill_kernel(
    const uint16_t* __restrict__ q, uint16_t* __restrict__ out, const uint16_t* __restrict__ k_pages,
    const uint16_t* __restrict__ v_pages, const int32_t* __restrict__ block_table, int table_stride,
    const int32_t* __restrict__ tile_seg, const int32_t* __restrict__ tile_row0, const int32_t* __restrict__ seg_row0,
    const int32_t* __restrict__ row_pos, int num_heads, int num_kv_heads, int head_dim, float scale_log2, int window) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    // a key's row in LDS holds HD channels, those past head_dim zero: every lane loads its operand
    constexpr int k_stride = HD + KV_PAD;
    const int v_stride = PAGE + KV_PAD;
    const int k_elems = PAGE * k_stride, v_elems = head_dim * v_stride;
    uint16_t* lds = reinterpret_cast<uint16_t*>(lds_raw);      // [buffer][K tile | V tile]
    if (head_dim < HD) {
        const int runs_per_row = (HD - head_dim) / 8;          // head_dim is a multiple of 16
        for (int run = threadIdx.x; run < 2 * PAGE * runs_per_row; run += 256) {
            const int buffer = run / (PAGE * runs_per_row), row = run / runs_per_row % PAGE, at = run % runs_per_row;
            *reinterpret_cast<u32x4*>(lds + (size_t)buffer * (k_elems + v_elems) + row * k_stride + head_dim + at * 8) = u32x4{0u, 0u, 0u, 0u};
        }
    }

    const int group = num_heads / num_kv_heads, runs = (group + NH - 1) / NH;
    const int per_tile = num_kv_heads * runs;
    const int tile = blockIdx.x / per_tile, of_tile = blockIdx.x % per_tile;
    const int kvh = of_tile / runs, first_in_group = (of_tile % runs) * NH;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 15, g = lane >> 4;
    const int seg = tile_seg[tile];
    const int tile_first_row = tile_row0[tile];
    const int seg_end = seg_row0[seg + 1];
    const int tile_rows = seg_end - tile_first_row < 64 ? seg_end - tile_first_row : 64;
    const int row0 = tile_first_row + wave * 16;                        // this wave's rows
    const int rows = tile_rows - wave * 16 < 16 ? tile_rows - wave * 16 : 16;     // may be <= 0
    const bool valid = col < rows;
    const int my_row = valid ? row0 + col : tile_first_row;
    const int my_pos = row_pos[my_row];
    const int wave_hi = rows > 0 ? row_pos[row0 + rows - 1] : -1;       // last position of this wave
    const int pos_lo = row_pos[tile_first_row], pos_hi = row_pos[tile_first_row + tile_rows - 1];
    const int my_first = window > 0 && my_pos - window + 1 > 0 ? my_pos - window + 1 : 0;
    const int tile_first = window > 0 && pos_lo - window + 1 > 0 ? pos_lo - window + 1 : 0;

    // a head past the end of the group computes along on zeros and is not stored
    Columns<HD> c[NH];
#pragma unroll
    for (int h = 0; h < NH; ++h) {
        const bool head_there = first_in_group + h < group;
        const int head = kvh * group + (head_there ? first_in_group + h : 0);
        load_query<HD>(c[h], q + ((size_t)my_row * num_heads + head) * head_dim, head_dim, valid && head_there);
    }
    const int32_t* table = block_table + (size_t)seg * table_stride;
    const size_t page_elems = (size_t)PAGE * head_dim;

    // the copy: a page's K is 64 rows of head_dim, its V head_dim rows of 64; runs of 16 bytes.
    // Loads are unconditional (a run or a page past the end is read from a valid place again and
    // never used) and the barriers order LDS traffic only, so that the pages requested stay in
    // flight while the page before them is worked on.
    const int k_runs = PAGE * head_dim / 8;                                      // as many for V
    constexpr int MAX_RUNS = HD * PAGE / 8 / 256;                                // per thread, per operand
    const int first_block = tile_first / PAGE, last_block = pos_hi / PAGE;
    u32x4 hold_k0[MAX_RUNS], hold_v0[MAX_RUNS], hold_k1[MAX_RUNS], hold_v1[MAX_RUNS];
    // what a thread copies of every page: fixed offsets, so that a page's address is a scalar
    // base plus these (no vector arithmetic per page; the registers that receive a page are
    // otherwise borrowed for it, and giving them back means waiting for loads still in flight)
    uint32_t run_offset[MAX_RUNS];
#pragma unroll
    for (int u = 0; u < MAX_RUNS; ++u) run_offset[u] = (uint32_t)(tid + u * 256 < k_runs ? tid + u * 256 : 0) * 8u;
    auto fetch = [&](u32x4 (&hold_k)[MAX_RUNS], u32x4 (&hold_v)[MAX_RUNS], int block) {
        const int page = __builtin_amdgcn_readfirstlane(table[block < last_block ? block : last_block]);
        const size_t at = ((size_t)page * num_kv_heads + kvh) * page_elems;
        const uint16_t* k_from = k_pages + at;
        const uint16_t* v_from = v_pages + at;
#pragma unroll
        for (int u = 0; u < MAX_RUNS; ++u) {
            hold_k[u] = *reinterpret_cast<const u32x4*>(k_from + run_offset[u]);
            hold_v[u] = *reinterpret_cast<const u32x4*>(v_from + run_offset[u]);
        }
    };
    // The values of keys past the last one written (only in the tile's last page) are zeroed on
    // their way to LDS: whatever an earlier owner of the page left there must not meet P = 0.
    auto stash = [&](const u32x4 (&hold_k)[MAX_RUNS], const u32x4 (&hold_v)[MAX_RUNS], int buffer, int block) {
        uint16_t* kt = lds + (size_t)buffer * (k_elems + v_elems);
        uint16_t* vt = kt + k_elems;
        const int k_per_row = head_dim / 8;
        const int last_written = pos_hi - block * PAGE;         // < 0 for a page past the end: never attended
#pragma unroll
        for (int u = 0; u < MAX_RUNS; ++u) {
            const int run = tid + u * 256;
            if (run < k_runs) {
                *reinterpret_cast<u32x4*>(kt + (run / k_per_row) * k_stride + (run % k_per_row) * 8) = hold_k[u];
                u32x4 v = hold_v[u];
                if (last_written < PAGE - 1) {
                    const int key0 = (run % 8) * 8;             // this run: keys key0 .. key0 + 7 of one channel
#pragma unroll
                    for (int word = 0; word < 4; ++word) {
                        const int first_key = key0 + 2 * word;
                        v[word] &= first_key + 1 <= last_written ? 0xffffffffu : (first_key <= last_written ? 0xffffu : 0u);
                    }
                }
                *reinterpret_cast<u32x4*>(vt + (run / 8) * v_stride + (run % 8) * 8) = v;
            }
        }
    };
    auto attend = [&](int block, int buffer) {
        const int base = block * PAGE;
        if (rows > 0 && base <= wave_hi) {      // a wave whose rows all lie before this page has nothing to add
            const uint16_t* kt = lds + (size_t)buffer * (k_elems + v_elems);
            // a lane without a row computes along with the bounds of the tile's first row (nothing of
            // it is stored): a page that is whole for the rows is then whole for the wave
            attend_page<HD, NH, false, true>(c, kt, kt + k_elems, head_dim, scale_log2, my_first - base, my_pos - base, pos_hi - base,
                            k_stride, v_stride);
        }
    };

    // page b travels: global -> register set (b - first) % 2, requested two pages ahead -> LDS
    // buffer (b - first) % 2, stored while page b - 1 is worked on -> attended
    fetch(hold_k0, hold_v0, first_block);
    fetch(hold_k1, hold_v1, first_block + 1);
    stash(hold_k0, hold_v0, 0, first_block);
    fw_lds_barrier();
    for (int block = first_block; block <= last_block; block += 2) {
        fetch(hold_k0, hold_v0, block + 2);
        __builtin_amdgcn_sched_barrier(0);      // keep the requests ahead of the work they overlap
        attend(block, 0);
        stash(hold_k1, hold_v1, 1, block + 1);
        fw_lds_barrier();
        if (block + 1 > last_block) break;
        fetch(hold_k1, hold_v1, block + 3);
        __builtin_amdgcn_sched_barrier(0);
        attend(block + 1, 1);
        stash(hold_k0, hold_v0, 0, block + 2);
        fw_lds_barrier();
    }
#pragma unroll
    for (int h = 0; h < NH; ++h) {
        const float l = fw_quad_sum(c[h].l);
        if (!valid || first_in_group + h >= group) continue;
        const float inv = 1.0f / l;
        uint16_t* dest = out + ((size_t)my_row * num_heads + kvh * group + first_in_group + h) * head_dim;
#pragma unroll
        for (int t = 0; t < HD / 16; ++t) {
            if (t * 16 >= head_dim) break;
            u32x2 packed = {pack_bf16(c[h].o[t][0] * inv, c[h].o[t][1] * inv), pack_bf16(c[h].o[t][2] * inv, c[h].o[t][3] * inv)};
            *reinterpret_cast<u32x2*>(dest + t * 16 + g * 4) = packed;
        }
    }
}

// ---- decode ------------------------------------------------------------------------------------
#define DECODE_WORKGROUPS 512        // two per compute unit: beyond, longer splits serve better than more of them
// grid (rows, kv heads * head tiles, splits); four waves, each takes one page of the split's
// SPLIT_PAGES, and their results are merged in LDS in the order of the keys. Columns are the
// query heads of the kv group (16 per head tile). partial [rows][heads][max_splits][head_dim + 4]:
// unnormalised output, then maximum and sum; a split with nothing to do writes nothing and takes
// no ticket. The last workgroup of a (row, kv head, head tile) to arrive merges what the others
// left; the only workgroup of a short row writes the result at once.
// What the fused variant does in front of the attention: the step's raw projections (float32
// [rows][(heads + 2 kv heads) * head_dim]: queries, keys, values) get their per-head RMS norm and
// rotation here, as qk_norm_rope_kv_write does in a kernel of its own (the same arithmetic in the
// same order), so that a decode step needs no such kernel. Every workgroup norms and rotates the
// query heads it works on; the workgroup whose pages include the row's own position also norms and
// rotates the new key, stores it and the new value in their page, and reads them back from there
// with the rest of the page (its own stores, ordered by a workgroup barrier).
struct FusedProjections {
    const float* qkv;               // null: q holds finished bfloat16 queries and the cache is up to date
    const float* q_norm_weight;     // [head_dim] or null
    const float* k_norm_weight;
    float eps;
    const float* cos_table;         // [rows][rotary_dim / 2]
    const float* sin_table;
    int rotary_dim;
    int write_kv;                   // 0: another execution of the layer has stored this step's keys and values already
};

// One head-vector of head_dim channels by one wave: optional RMS norm, then the half-split rotation
// of the first rotary_dim channels; `store(d, value)` takes the results. scratch: head_dim floats of
// LDS of the wave's own. (native/include/flyweight_v2_native_kernels.hpp:1015-1050)
template <typename Store>
__device__ __forceinline__ void norm_rotate_vector(const float* __restrict__ source, const float* __restrict__ weight, float eps,
                                                   const float* __restrict__ cos_row, const float* __restrict__ sin_row,
                                                   int rotary_dim, int head_dim, float* scratch, Store store) {
    const int lane = threadIdx.x & 63;
    float inv = 1.0f;
    if (weight) {
        float sum = 0.0f;
        for (int d = lane; d < head_dim; d += 64) {
            const float v = source[d];
            sum += v * v;
        }
        sum = wave_sum(sum);
        inv = rsqrtf(sum / (float)head_dim + eps);
    }
    for (int d = lane; d < head_dim; d += 64) {
        const float v = source[d];
        scratch[d] = weight ? v * inv * weight[d] : v;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int half = rotary_dim / 2;
    for (int d = lane; d < head_dim; d += 64) {
        float value = scratch[d];
        if (d < rotary_dim) {
            const int pair = d < half ? d : d - half;
            const float other = scratch[d < half ? d + half : d - half];
            const float c = cos_row[pair], s = sin_row[pair];
            value = d < half ? value * c - other * s : value * c + other * s;
        }
        store(d, value);
    }
}

template <int HD, bool FUSED>
__global__ __launch_bounds__(64 * SPLIT_PAGES) __attribute__((amdgpu_waves_per_eu(HD <= 128 ? 2 : 1))) void attention_decode_split_kernel(
    const uint16_t* __restrict__ q, uint16_t* __restrict__ out, float* partial, int* tickets,
    uint16_t* k_pages, uint16_t* v_pages, const int32_t* __restrict__ block_table, int table_stride,
    const int32_t* __restrict__ row_seg, const int32_t* __restrict__ row_pos, int num_heads, int num_kv_heads,
    int head_dim, float scale_log2, int window, int max_splits, const int32_t* __restrict__ decode_work, const FusedProjections fused) {
    __shared__ f32x4 shared_o[SPLIT_PAGES][HD / 16][64];
    __shared__ float shared_m[SPLIT_PAGES][16], shared_l[SPLIT_PAGES][16];
    __shared__ int ticket_shared;
    __shared__ __attribute__((aligned(16))) uint16_t fused_q[FUSED ? 16 : 1][FUSED ? HD : 8];
    __shared__ float fused_scratch[FUSED ? SPLIT_PAGES : 1][FUSED ? HD : 1];
    const int row = blockIdx.x, split = blockIdx.z;
    const int group = num_heads / num_kv_heads;
    const int head_tiles = (group + 15) / 16;
    const int kvh = blockIdx.y / head_tiles, head_tile = blockIdx.y % head_tiles;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 15, g = lane >> 4;
    const int pos = row_pos[row];
    const int segment = row_seg[row];       // asked for together with the position, not behind the branch below
    const int first = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
    // Splits are counted from the first page that holds a visible key; a split is `rounds` runs of
    // SPLIT_PAGES pages. One run each serves while the step's runs (decode_work: over all its rows;
    // times the kv heads and head tiles) are no more than about two workgroups per compute unit;
    // beyond, fewer and longer workgroups read the cache faster, and a row has fewer parts to merge (one
    // workgroup for a whole row needs no merge at all). Counting the step's work, not the row's, gives
    // a long row among short ones its share of the chip.
    int rounds = 1;
    if (decode_work) {
        const long long workgroups = (long long)decode_work[0] * gridDim.y;
        rounds = (int)(workgroups / DECODE_WORKGROUPS);
        rounds = rounds < 1 ? 1 : rounds;
    }
    const int pages_per_split = SPLIT_PAGES * rounds;
    const int first_block = first / PAGE + split * pages_per_split;
    const int last_block = pos / PAGE;
    if (first_block > last_block) return;       // the whole workgroup
    const int in_group = head_tile * 16 + col;
    const bool valid = in_group < group;
    const int head = kvh * group + (valid ? in_group : 0);

    Columns<HD> columns_of_wave[1];
    Columns<HD>& c = columns_of_wave[0];
    if (FUSED) {
        const int width = (num_heads + 2 * num_kv_heads) * head_dim;
        const float* projections = fused.qkv + (size_t)row * width;
        const int half = fused.rotary_dim / 2;
        const float* cos_row = fused.cos_table + (size_t)row * half;
        const float* sin_row = fused.sin_table + (size_t)row * half;
        const int columns = group - head_tile * 16 < 16 ? group - head_tile * 16 : 16;
        // the vectors of this workgroup: its query heads, then (where the row's own position lies
        // in its pages) the new key and the new value; a wave takes every fourth
        const bool stores = fused.write_kv && last_block < first_block + pages_per_split;
        const int vectors = columns + (stores ? 2 : 0);
        const int slot = pos % PAGE;
        const int own_page = stores ? block_table[(size_t)segment * table_stride + last_block] : 0;
        for (int v = wave; v < vectors; v += SPLIT_PAGES) {
            if (v < columns) {
                uint16_t* dest = fused_q[v];
                norm_rotate_vector(projections + (size_t)(kvh * group + head_tile * 16 + v) * head_dim, fused.q_norm_weight, fused.eps,
                                   cos_row, sin_row, fused.rotary_dim, head_dim, fused_scratch[wave],
                                   [&](int d, float value) { dest[d] = float_to_bf16_bits(value); });
            } else if (v == columns) {
                uint16_t* dest = k_pages + (((size_t)own_page * num_kv_heads + kvh) * PAGE + slot) * head_dim;
                norm_rotate_vector(projections + (size_t)(num_heads + kvh) * head_dim, fused.k_norm_weight, fused.eps, cos_row, sin_row,
                                   fused.rotary_dim, head_dim, fused_scratch[wave],
                                   [&](int d, float value) { dest[d] = float_to_bf16_bits(value); });
            } else {
                const float* value = projections + (size_t)(num_heads + num_kv_heads + kvh) * head_dim;
                uint16_t* dest = v_pages + ((size_t)own_page * num_kv_heads + kvh) * head_dim * PAGE + slot;
                for (int d = lane; d < head_dim; d += 64) dest[(size_t)d * PAGE] = float_to_bf16_bits(value[d]);
            }
        }
        // the page is read below by this workgroup's own waves: its stores have to be done first
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        load_query<HD>(c, fused_q[valid ? col : 0], head_dim, valid);
    } else {
        load_query<HD>(c, q + ((size_t)row * num_heads + head) * head_dim, head_dim, valid);
    }
    for (int round = 0; round < rounds; ++round) {
        const int block = first_block + round * SPLIT_PAGES + wave;
        if (block > last_block) break;
        const int page = block_table[(size_t)segment * table_stride + block];
        const size_t at = ((size_t)page * num_kv_heads + kvh) * PAGE * head_dim;
        const int base = block * PAGE;
        // a lane without a head computes along (q = 0, nothing of it is stored)
        attend_page<HD, 1, true, false, (HD <= 128)>(columns_of_wave, k_pages + at, v_pages + at, head_dim, scale_log2, first - base, pos - base, pos - base,
                        head_dim, PAGE);
    }
    const float l = fw_quad_sum(c.l);
#pragma unroll
    for (int t = 0; t < HD / 16; ++t) shared_o[wave][t][lane] = c.o[t];
    if (g == 0) {
        shared_m[wave][col] = c.m;
        shared_l[wave][col] = l;
    }
    __syncthreads();
    // how many workgroups work on this row: those whose first page holds a visible key
    const int row_splits = (last_block - first / PAGE + 1 + pages_per_split - 1) / pages_per_split;
    const int stride = PART_STRIDE(head_dim);
    if (wave == 0 && valid) {
        float m = NEG_BIG;
#pragma unroll
        for (int w = 0; w < SPLIT_PAGES; ++w) m = fmaxf(m, shared_m[w][col]);
        float total = 0.0f, weight[SPLIT_PAGES];
#pragma unroll
        for (int w = 0; w < SPLIT_PAGES; ++w) {
            weight[w] = exp2f(shared_m[w][col] - m);        // a wave without a page has l = 0 and o = 0
            total += weight[w] * shared_l[w][col];
        }
        float* dest = partial + (((size_t)row * num_heads + head) * max_splits + split) * stride;
        uint16_t* final_dest = out + ((size_t)row * num_heads + head) * head_dim;
#pragma unroll
        for (int t = 0; t < HD / 16; ++t) {
            if (t * 16 >= head_dim) break;
            f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int w = 0; w < SPLIT_PAGES; ++w) sum += weight[w] * shared_o[w][t][lane];
            if (row_splits == 1) {
                // the only workgroup of its row: the result is final
                const float inv = 1.0f / total;
                u32x2 packed = {pack_bf16(sum[0] * inv, sum[1] * inv), pack_bf16(sum[2] * inv, sum[3] * inv)};
                *reinterpret_cast<u32x2*>(final_dest + t * 16 + g * 4) = packed;
            } else {
                // device-scope stores: they pass the caches that workgroups on other dies do not share
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    __hip_atomic_store(dest + t * 16 + g * 4 + r, sum[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        if (g == 0 && row_splits > 1) {
            __hip_atomic_store(dest + head_dim, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(dest + head_dim + 1, total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (row_splits == 1) return;
    // The workgroup of a (row, kv head) that arrives last merges the parts, in the order of the keys:
    // every wave waits for its own stores to be acknowledged, the workgroup meets, one thread
    // takes the ticket. Nobody waits for another workgroup. The ticket counter is left at zero.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    int* ticket = tickets + (size_t)row * gridDim.y + blockIdx.y;
    if (threadIdx.x == 0) ticket_shared = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (ticket_shared != row_splits - 1) return;
    if (threadIdx.x == 0) __hip_atomic_store(ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int columns = group - head_tile * 16 < 16 ? group - head_tile * 16 : 16;
    for (int item = threadIdx.x; item < columns * head_dim; item += 64 * SPLIT_PAGES) {
        const int merged_head = kvh * group + head_tile * 16 + item / head_dim, d = item % head_dim;
        const float* source = partial + ((size_t)row * num_heads + merged_head) * max_splits * stride;
        // Sixteen parts are requested at a time (past the last one: the last one again, not used),
        // maximum, weight and value together: one round trip for up to sixteen parts. The running
        // sums are rescaled when a later batch of parts raises the maximum.
        auto part_at = [&](int sp, int offset) {
            const int clamped = sp < row_splits ? sp : row_splits - 1;
            return __hip_atomic_load(source + (size_t)clamped * stride + offset, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        };
        constexpr int AT_ONCE = 16;
        float m = NEG_BIG, total = 0.0f, acc = 0.0f;
        for (int sp0 = 0; sp0 < row_splits; sp0 += AT_ONCE) {
            float ms[AT_ONCE], ls[AT_ONCE], vs[AT_ONCE];
#pragma unroll
            for (int u = 0; u < AT_ONCE; ++u) {
                ms[u] = part_at(sp0 + u, head_dim);
                ls[u] = part_at(sp0 + u, head_dim + 1);
                vs[u] = part_at(sp0 + u, d);
            }
            float highest = m;
#pragma unroll
            for (int u = 0; u < AT_ONCE; ++u) highest = fmaxf(highest, ms[u]);
            const float keep = exp2f(m - highest);      // 0 for the first batch, whose sums are 0 anyway
            total *= keep;
            acc *= keep;
            m = highest;
#pragma unroll
            for (int u = 0; u < AT_ONCE; ++u) {
                const float weight = sp0 + u < row_splits ? exp2f(ms[u] - m) : 0.0f;
                total += weight * ls[u];
                acc += weight * vs[u];
            }
        }
        out[((size_t)row * num_heads + merged_head) * head_dim + d] = float_to_bf16_bits(acc / total);
    }
}

static const float LOG2E = 1.4426950408889634f;

static int check_common(const char* name, int rows, int num_heads, int num_kv_heads, int head_dim, int page_size,
                        int window, int num_pages, int table_stride) {
    FW_REQUIRE(rows >= 0 && num_heads > 0 && num_kv_heads > 0 && num_heads % num_kv_heads == 0,
               "%s: heads %d must be a positive multiple of kv heads %d", name, num_heads, num_kv_heads);
    FW_REQUIRE(head_dim >= 16 && head_dim <= 256 && head_dim % 16 == 0, "%s: head_dim %d must be a multiple of 16 in 16..256", name, head_dim);
    FW_REQUIRE(page_size == PAGE, "%s: page size must be %d, got %d", name, PAGE, page_size);
    FW_REQUIRE(window >= 0, "%s: window must be 0 (all keys) or positive, got %d", name, window);
    FW_REQUIRE(num_pages > 0 && table_stride > 0, "%s: empty cache (pages=%d, table stride=%d)", name, num_pages, table_stride);
    return 0;
}

#define FW_BY_HEAD_DIM(head_dim, CALL)      \
    do {                                    \
        if (head_dim <= 32) { CALL(32); }   \
        else if (head_dim <= 64) { CALL(64); } \
        else if (head_dim <= 128) { CALL(128); } \
        else { CALL(256); }                 \
    } while (0)

// bfloat16 q [rows][heads * head_dim] -> out (same shape). tile_seg / tile_row0 [tiles]: tiles of
// up to 64 rows that never span two segments, in any order (workgroups start in that order: list
// the tiles that see the most keys first). heads_together: query heads of a kv group that one
// workgroup takes (1, or 4 up to head_dim 64). Four read a page once for four heads (1.09 vs
// 1.27 ms for 2,048 rows behind 30,720 tokens, 32 heads in 8 groups, head_dim 64), one gives four
// times as many workgroups to even out tiles of unequal length (58 vs 81 us for the same rows
// from position 0; equal behind 6,144 tokens). The caller, who knows the positions, says which;
// 0: chosen here from the shape alone: 4 where that still leaves every compute unit four workgroups.
extern "C" int fw_attention_prefill(const void* q, void* out, const void* k_pages, const void* v_pages,
                                    const int32_t* block_table, int table_stride, const int32_t* tile_seg,
                                    const int32_t* tile_row0, int tiles, const int32_t* seg_row0,
                                    const int32_t* row_pos, int rows, int num_heads, int num_kv_heads, int head_dim,
                                    float scale, int window, int page_size, int num_pages, int heads_together,
                                    void* stream) {
    if (check_common("attention_prefill", rows, num_heads, num_kv_heads, head_dim, page_size, window, num_pages, table_stride)) return -1;
    FW_REQUIRE(tiles >= 0 && tiles <= rows && num_heads <= 65535, "attention_prefill: %d tiles for %d rows", tiles, rows);
    const int most_together = head_dim <= 64 ? 4 : 1;
    FW_REQUIRE(heads_together == 0 || heads_together == 1 || (heads_together == 4 && most_together == 4),
               "attention_prefill: %d heads together with head_dim %d (1, or 4 up to head_dim 64)", heads_together, head_dim);
    if (rows == 0 || tiles == 0) return 0;
    const int group = num_heads / num_kv_heads;
    if (heads_together == 0)
        heads_together = most_together == 4 && group >= 4 && (long long)tiles * num_kv_heads * ((group + 3) / 4) >= 1024 ? 4 : 1;
    const long long blocks = (long long)tiles * num_kv_heads * ((group + heads_together - 1) / heads_together);
    FW_REQUIRE(blocks < (1ll << 31), "attention_prefill: too many tiles and heads");
    dim3 grid((unsigned)blocks);
#define LAUNCH(HD, NH)                                                                                             \
    {                                                                                                              \
        const int lds_bytes = 2 * (PAGE * (HD + KV_PAD) + head_dim * (PAGE + KV_PAD)) * 2;                         \
        static int configured = 0;                                                                                 \
        if (lds_bytes > configured) {                                                                              \
            hipError_t status = hipFuncSetAttribute((const void*)attention_prefill_kernel<HD, NH>,                 \
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);        \
            FW_REQUIRE(status == hipSuccess, "attention_prefill: cannot reserve %d bytes of LDS", lds_bytes);      \
            configured = lds_bytes;                                                                                \
        }                                                                                                          \
        attention_prefill_kernel<HD, NH><<<grid, 256, lds_bytes, (hipStream_t)stream>>>(                            \
            (const uint16_t*)q, (uint16_t*)out, (const uint16_t*)k_pages, (const uint16_t*)v_pages, block_table,    \
            table_stride, tile_seg, tile_row0, seg_row0, row_pos, num_heads, num_kv_heads, head_dim, scale * LOG2E, \
            window);                                                                                               \
    }
    if (head_dim <= 32) {
        if (heads_together == 4) LAUNCH(32, 4) else LAUNCH(32, 1)
    } else if (head_dim <= 64) {
        if (heads_together == 4) LAUNCH(64, 4) else LAUNCH(64, 1)
    } else if (head_dim <= 128) {
        LAUNCH(128, 1)
    } else {
        LAUNCH(256, 1)
    }
#undef LAUNCH
    FW_LAUNCH_CHECK("attention_prefill");
    return 0;
}

static int decode_check(int max_splits, int max_context, int* tickets, int tickets_len, int table_stride, int rows, int num_heads,
                        int num_kv_heads, int head_dim, int window, int page_size, int num_pages) {
    if (check_common("attention_decode", rows, num_heads, num_kv_heads, head_dim, page_size, window, num_pages, table_stride)) return -1;
    FW_REQUIRE(max_splits >= 1 && max_splits <= 65535, "attention_decode: max_splits %d outside 1..65535", max_splits);
    FW_REQUIRE(max_context >= 1, "attention_decode: max_context must be positive");
    int blocks = (max_context + PAGE - 1) / PAGE;
    if (window > 0 && (window + PAGE - 2) / PAGE + 1 < blocks) blocks = (window + PAGE - 2) / PAGE + 1;
    FW_REQUIRE(max_splits * SPLIT_PAGES >= blocks, "attention_decode: %d splits of %d pages do not cover %d pages of context",
               max_splits, SPLIT_PAGES, blocks);
    FW_REQUIRE((max_context + PAGE - 1) / PAGE <= table_stride, "attention_decode: a context of %d tokens exceeds the block table (%d pages)",
               max_context, table_stride);
    const int head_tiles = (num_heads / num_kv_heads + 15) / 16;
    FW_REQUIRE(rows <= 1 << 20 && num_kv_heads * head_tiles <= 65535 && num_heads <= 65535, "attention_decode: grid too large");
    FW_REQUIRE(rows == 0 || max_splits == 1 || (tickets != nullptr && (long long)tickets_len >= (long long)rows * num_kv_heads * head_tiles),
               "attention_decode: %d rows need %d ticket counters", rows, rows * num_kv_heads * head_tiles);
    return 0;
}

static int decode_launch(const void* q, void* out, float* partial, int max_splits, const int32_t* decode_work, int* tickets, void* k_pages, void* v_pages,
                         const int32_t* block_table, int table_stride, const int32_t* row_seg, const int32_t* row_pos, int rows,
                         int num_heads, int num_kv_heads, int head_dim, float scale, int window, const FusedProjections& fused,
                         void* stream) {
    if (rows == 0) return 0;
    const int head_tiles = (num_heads / num_kv_heads + 15) / 16;
    dim3 grid(rows, num_kv_heads * head_tiles, max_splits);

#define CALL(HD)                                                                                                              \
    if (fused.qkv)                                                                                                            \
        attention_decode_split_kernel<HD, true><<<grid, 64 * SPLIT_PAGES, 0, (hipStream_t)stream>>>(                          \
            (const uint16_t*)q, (uint16_t*)out, partial, tickets, (uint16_t*)k_pages, (uint16_t*)v_pages, block_table,        \
            table_stride, row_seg, row_pos, num_heads, num_kv_heads, head_dim, scale * LOG2E, window, max_splits, decode_work, fused); \
    else                                                                                                                      \
        attention_decode_split_kernel<HD, false><<<grid, 64 * SPLIT_PAGES, 0, (hipStream_t)stream>>>(                         \
            (const uint16_t*)q, (uint16_t*)out, partial, tickets, (uint16_t*)k_pages, (uint16_t*)v_pages, block_table,        \
            table_stride, row_seg, row_pos, num_heads, num_kv_heads, head_dim, scale * LOG2E, window, max_splits, decode_work, fused)
    FW_BY_HEAD_DIM(head_dim, CALL);
#undef CALL
    FW_LAUNCH_CHECK("attention_decode");
    return 0;
}

// One row per request. partial: float32 workspace of rows * heads * max_splits * (head_dim + 4).
// max_context: no row's position reaches it (the caller knows; the kernel cannot check);
// max_splits must cover the keys such a row sees, in runs of 4 pages. decode_work: null, or one
// int32 on the device: the runs of 4 pages that all the rows of the step see together (the sum over
// the rows of ceil((position + 1) / 256)); with it a workgroup takes as many runs as bring the step
// down to about 512 workgroups (it changes how the work is shared out, not what is computed). tickets: rows * kv heads *
// ceil(group / 16) int32 counters, zero before the first call and left zero; calls that overlap on
// one device need their own (and their own workspace).
extern "C" int fw_attention_decode(const void* q, void* out, float* partial, int max_splits, int max_context,
                                   const int32_t* decode_work, int* tickets, int tickets_len, const void* k_pages,
                                   const void* v_pages, const int32_t* block_table, int table_stride,
                                   const int32_t* row_seg, const int32_t* row_pos, int rows, int num_heads,
                                   int num_kv_heads, int head_dim, float scale, int window, int page_size,
                                   int num_pages, void* stream) {
    if (decode_check(max_splits, max_context, tickets, tickets_len, table_stride, rows, num_heads, num_kv_heads, head_dim, window,
                     page_size, num_pages)) return -1;
    return decode_launch(q, out, partial, max_splits, decode_work, tickets, const_cast<void*>(k_pages), const_cast<void*>(v_pages), block_table,
                         table_stride, row_seg, row_pos, rows, num_heads, num_kv_heads, head_dim, scale, window, FusedProjections{}, stream);
}

// fw_attention_decode with the work of fw_qk_norm_rope_kv_write in front of it, in the same kernel:
// qkv float32 [rows][(heads + 2 kv heads) * head_dim] are the step's raw projections; the new keys and
// values are stored in their pages (write_kv 0: they are there already and only the queries are
// formed). Norm weights float32 [head_dim] or null, rotation tables float32 [rows][rotary_dim / 2]
// (null with rotary_dim 0). Results as the two kernels one after the other give them.
extern "C" int fw_attention_decode_fused(const float* qkv, const float* q_norm_weight, const float* k_norm_weight, float eps,
                                         const float* cos_table, const float* sin_table, int rotary_dim, int write_kv, void* out,
                                         float* partial, int max_splits, int max_context, const int32_t* decode_work, int* tickets, int tickets_len,
                                         void* k_pages, void* v_pages, const int32_t* block_table, int table_stride,
                                         const int32_t* row_seg, const int32_t* row_pos, int rows, int num_heads,
                                         int num_kv_heads, int head_dim, float scale, int window, int page_size, int num_pages,
                                         void* stream) {
    if (decode_check(max_splits, max_context, tickets, tickets_len, table_stride, rows, num_heads, num_kv_heads, head_dim, window,
                     page_size, num_pages)) return -1;
    FW_REQUIRE(qkv != nullptr, "attention_decode_fused: the projections are missing");
    FW_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0, "attention_decode_fused: rotary_dim %d with head_dim %d",
               rotary_dim, head_dim);
    FW_REQUIRE(rotary_dim == 0 || (cos_table != nullptr && sin_table != nullptr), "attention_decode_fused: the rotation tables are missing");
    FW_REQUIRE((q_norm_weight == nullptr) == (k_norm_weight == nullptr), "attention_decode_fused: q and k are normed together or not at all");
    FusedProjections fused;
    fused.qkv = qkv; fused.q_norm_weight = q_norm_weight; fused.k_norm_weight = k_norm_weight; fused.eps = eps;
    fused.cos_table = cos_table; fused.sin_table = sin_table; fused.rotary_dim = rotary_dim; fused.write_kv = write_kv;
    return decode_launch(nullptr, out, partial, max_splits, decode_work, tickets, k_pages, v_pages, block_table, table_stride, row_seg, row_pos,
                         rows, num_heads, num_kv_heads, head_dim, scale, window, fused, stream);
}
