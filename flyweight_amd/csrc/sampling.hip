// Drawing the next token of every row on the device: greedy, temperature, top-k, top-p, min-p,
// each request with its own xorshift64* generator, in the reference's order of operations
// (native/src/v2_runtime.cpp:29500-29566, 29686-29743; generator :29307-29314):
//
//   candidates sorted by (value descending, id ascending), the first top_k of them (0: all);
//   p_i = exp((l_i - l_0) / T) in float64; total = sum of p; top_p keeps the shortest prefix
//   whose shares p_i / total add up to it; min_p ends the prefix before the first p_i < min_p;
//   u * (sum of the kept p) is walked down the prefix until the running sum reaches it.
//
// One workgroup of 1,024 threads per row. The sorted list is never made as a whole: candidates
// come in batches of up to 1,024, the best that are below the last batch's smallest (a radix
// select over the 64-bit keys: up to six passes over the row, counting in LDS), sorted in LDS,
// their p formed by all threads, thread i holding candidate i and the running sums up to it (a
// scan in a fixed order). With top_k up to 1,024 (the usual case) that is one batch, and up to 512
// it is gathered without a select: everything at or above the k-th of the threads' own best. A
// longer list (no top_k) begins with such a batch too, everything at or above the 512th of the
// threads' best, which stays in LDS for both walks: a peaked row ends both there (81 us at top_p
// 0.9 against 137 us when each walk selected its own first 1,024). A draw over the whole
// vocabulary of a flat distribution takes as many batches as it walks through.
// A row whose temperature is 0 takes the best candidate and leaves its generator alone, so
// greedy and sampled requests share one launch; a drawing row with a single candidate (top_k 1)
// moves its generator on like any other draw. Nothing is allocated; nothing crosses to the host.
#include "fw_common.h"
#include "fw_kernels.h"

#define SAMPLE_THREADS 1024
#define SAMPLE_BATCH 1024
#define SAMPLE_DIGIT_BITS 11
#define SAMPLE_BINS (1 << SAMPLE_DIGIT_BITS)

struct SampleShared {
    unsigned int histogram[SAMPLE_BINS];
    unsigned long long keys[SAMPLE_BATCH];
    double p[SAMPLE_BATCH];
    double running[SAMPLE_BATCH];   // the sum of p up to and including each candidate of the batch
    unsigned long long wave_keys[SAMPLE_THREADS / 64];
    double wave_sums[SAMPLE_THREADS / 64];
    unsigned long long prefix;      // of the key being selected, the digits found so far
    unsigned int wanted;            // how many candidates are still wanted inside the prefix
    unsigned int gathered;
    int exact;                      // the select has found its key before the last digit
    int wave_least[SAMPLE_THREADS / 64];
    // what the candidate at which a walk ends tells the others
    int keep_here;
    double kept_share;
};

__device__ __forceinline__ unsigned long long sample_wave_max(unsigned long long v) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        const unsigned long long other = __shfl_xor(v, offset, 64);
        v = other > v ? other : v;
    }
    return v;
}

// The sum of x over the threads up to and including this one (or, with `whole`, over all of them:
// every thread gets the same), added up in a fixed order: inside a wave by doubling steps, then the
// waves before this one in turn.
__device__ double sample_running_sum(double x, SampleShared& s, bool whole) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    double sum = x;
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
        const double other = __shfl_up(sum, offset, 64);
        if (lane >= offset) sum += other;
    }
    __syncthreads();
    if (lane == 63) s.wave_sums[wave] = sum;
    __syncthreads();
    double before = 0.0;
    const int waves = whole ? SAMPLE_THREADS / 64 : wave;
    for (int w = 0; w < waves; ++w) before += s.wave_sums[w];
    return whole ? before : before + sum;
}

// the least of the threads' values; every thread gets it
__device__ int sample_least(int value, SampleShared& s) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        const int other = __shfl_xor(value, offset, 64);
        value = other < value ? other : value;
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s.wave_least[threadIdx.x >> 6] = value;
    __syncthreads();
    int least = s.wave_least[0];
    for (int w = 1; w < SAMPLE_THREADS / 64; ++w) least = s.wave_least[w] < least ? s.wave_least[w] : least;
    return least;
}

// Calls visit(value, id) for this thread's share of a row, four neighbours at a time where the row
// allows 16-byte loads.
template <typename Visit>
__device__ __forceinline__ void sample_for_each(const float* __restrict__ row, int vocab, Visit visit) {
    if ((vocab & 3) == 0 && ((uintptr_t)row & 15) == 0) {
        const float4* quads = reinterpret_cast<const float4*>(row);
        for (int q = threadIdx.x; q < vocab / 4; q += SAMPLE_THREADS) {
            const float4 v = quads[q];
            visit(v.x, 4 * q);
            visit(v.y, 4 * q + 1);
            visit(v.z, 4 * q + 2);
            visit(v.w, 4 * q + 3);
        }
    } else {
        for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) visit(row[i], i);
    }
}

// Sorts the first `slots` (a power of two, at most 1,024) keys in LDS, greatest first (every thread
// calls; a barrier before and after).
__device__ void sample_sort(unsigned long long* keys, int slots) {
    __syncthreads();
    for (int size = 2; size <= slots; size <<= 1)
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            const int partner = threadIdx.x ^ stride;
            if (partner > (int)threadIdx.x && partner < slots) {
                const unsigned long long a = keys[threadIdx.x], b = keys[partner];
                const bool descending = (threadIdx.x & size) == 0;
                if (descending ? a < b : a > b) {
                    keys[threadIdx.x] = b;
                    keys[partner] = a;
                }
            }
            __syncthreads();
        }
}

// The key of the `count`-th best candidate among those with lower <= key < ceiling; every thread
// gets it. If fewer than `count` are there, `lower`: all of them are wanted. (`lower` is a bound
// the caller knows the wanted candidates to lie above: what is below it is not even counted, which
// keeps thousands of lanes from adding to the same few counters in the first pass.)
// each(visit) calls visit(key) for this thread's share of the keys that are searched.
template <typename Each>
__device__ unsigned long long sample_select(Each each, unsigned long long lower, unsigned long long ceiling, unsigned int count,
                                            SampleShared& s) {
    // a call may follow another directly: every wave must have read the last call's prefix, wanted
    // and exact before they are set anew
    __syncthreads();
    if (threadIdx.x == 0) {
        s.prefix = 0ull;
        s.wanted = count;
        s.exact = 0;
    }
    int shift = 64;
    for (int level = 0; level < 6; ++level) {
        const int bits = shift >= SAMPLE_DIGIT_BITS ? SAMPLE_DIGIT_BITS : shift;    // 11, 11, 11, 11, 11, 9
        shift -= bits;
        for (int i = threadIdx.x; i < SAMPLE_BINS; i += SAMPLE_THREADS) s.histogram[i] = 0u;
        __syncthreads();
        const unsigned long long prefix = s.prefix;
        const int above = shift + bits;             // the digits found so far are the key's bits from here up
        each([&](unsigned long long key) {
            if (key >= lower && key < ceiling && (above >= 64 || (key >> above) == prefix))
                atomicAdd(&s.histogram[(unsigned int)(key >> shift) & ((1u << bits) - 1u)], 1u);
        });
        __syncthreads();
        // the first wave finds the digit at which the count from the top reaches what is wanted
        if (threadIdx.x < 64) {
            const int lane = threadIdx.x, per_lane = SAMPLE_BINS / 64;
            // lane 0 holds the highest bins
            const int first = SAMPLE_BINS - 1 - lane * per_lane;
            unsigned int mine = 0u;
            for (int b = 0; b < per_lane; ++b) mine += s.histogram[first - b];
            unsigned int before = mine;                // inclusive scan over the lanes, highest bins first
#pragma unroll
            for (int offset = 1; offset < 64; offset <<= 1) {
                const unsigned int other = __shfl_up(before, offset, 64);
                if (lane >= offset) before += other;
            }
            const unsigned int wanted = s.wanted;
            const unsigned int all = __shfl(before, 63, 64);
            if (level == 0 && all < wanted) {
                if (lane == 0) s.wanted = 0u;           // fewer are left than wanted: all of them
            } else {
                const unsigned int ahead = before - mine;
                if (ahead < wanted && wanted <= before) {       // the digit is among this lane's bins
                    unsigned int passed = ahead;
                    int digit = first;
                    for (int b = 0; b < per_lane; ++b) {
                        const unsigned int here = s.histogram[first - b];
                        if (passed + here >= wanted) {
                            digit = first - b;
                            break;
                        }
                        passed += here;
                    }
                    s.prefix = (prefix << bits) | (unsigned long long)digit;
                    s.wanted = wanted - passed;
                    // everything in this digit's counter is wanted: the smallest key with these digits is the answer
                    if (passed + s.histogram[digit] == wanted) s.exact = 1;
                }
            }
        }
        __syncthreads();
        if (s.wanted == 0u) return lower;
        if (s.exact) {
            const unsigned long long found = shift > 0 ? s.prefix << shift : s.prefix;
            return found > lower ? found : lower;
        }
    }
    return s.prefix;
}

// Gathers the candidates with floor <= key < ceiling (at most SAMPLE_BATCH) and sorts them, best
// first; returns how many. Their p = exp((l - best) / T) are formed alongside.
__device__ int sample_batch(const float* __restrict__ row, int vocab, unsigned long long floor_key, unsigned long long ceiling,
                            double best_scaled, double temperature, SampleShared& s) {
    if (threadIdx.x == 0) s.gathered = 0u;
    s.keys[threadIdx.x] = 0ull;
    __syncthreads();
    sample_for_each(row, vocab, [&](float value, int id) {
        const unsigned long long key = candidate_key(value, id);
        if (key >= floor_key && key < ceiling) {
            const unsigned int slot = atomicAdd(&s.gathered, 1u);
            if (slot < SAMPLE_BATCH) s.keys[slot] = key;
        }
    });
    __syncthreads();
    const int count = s.gathered < SAMPLE_BATCH ? (int)s.gathered : SAMPLE_BATCH;
    int slots = 2;
    while (slots < count) slots <<= 1;
    // empty slots are 0 and end up last: a real key is never 0 (its low word is 0xffffffff - id, id < 2^31)
    sample_sort(s.keys, slots);
    if ((int)threadIdx.x < count) {
        const double scaled = (double)row[candidate_id(s.keys[threadIdx.x])] / temperature;
        const double p = exp(scaled - best_scaled);
        s.p[threadIdx.x] = __builtin_isfinite(scaled) ? p : 0.0;     // not finite: no share
    }
    __syncthreads();
    return count;
}

// the sum of exp((l - best) / T) over the candidates with key >= floor_key, in a fixed order
__device__ double sample_total(const float* __restrict__ row, int vocab, unsigned long long floor_key, double best_scaled,
                               double temperature, SampleShared& s) {
    double mine = 0.0;
    sample_for_each(row, vocab, [&](float value, int id) {
        if (candidate_key(value, id) >= floor_key) {
            const double scaled = (double)value / temperature;
            if (__builtin_isfinite(scaled)) mine += exp(scaled - best_scaled);
        }
    });
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) mine += __shfl_xor(mine, offset, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s.wave_sums[threadIdx.x >> 6] = mine;
    __syncthreads();
    double total = 0.0;
    for (int w = 0; w < SAMPLE_THREADS / 64; ++w) total += s.wave_sums[w];
    return total;
}

// settings: [rows][4] = temperature, top_k (a whole number), top_p, min_p. states: the rows'
// generators, read and moved on by the rows that draw.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(const float* __restrict__ logits,
                                                                     const float* __restrict__ settings,
                                                                     unsigned long long* __restrict__ states,
                                                                     int32_t* __restrict__ ids, int32_t* __restrict__ also,
                                                                     int32_t* __restrict__ advance, int vocab) {
    __shared__ SampleShared s;
    const int r = blockIdx.x;
    const float* row = logits + (size_t)r * vocab;
    const double temperature = (double)settings[4 * r + 0];
    const double top_p = (double)settings[4 * r + 2], min_p = (double)settings[4 * r + 3];
    long long top_k = (long long)settings[4 * r + 1];

    // every thread's best candidate; the best of those is the row's
    unsigned long long mine = 0ull;
    sample_for_each(row, vocab, [&](float value, int id) {
        const unsigned long long key = candidate_key(value, id);
        mine = key > mine ? key : mine;
    });
    unsigned long long best = sample_wave_max(mine);
    if ((threadIdx.x & 63) == 0) s.wave_keys[threadIdx.x >> 6] = best;
    __syncthreads();
    best = 0ull;
    for (int w = 0; w < SAMPLE_THREADS / 64; ++w) best = s.wave_keys[w] > best ? s.wave_keys[w] : best;
    const int best_id = candidate_id(best);
    auto leave = [&](int token) {
        if (threadIdx.x == 0) {
            ids[r] = token;
            if (also) also[r] = token;
            if (advance) advance[r] += 1;
        }
    };
    const long long candidates = (top_k > 0 && top_k < vocab) ? top_k : vocab;
    const double best_scaled = (double)row[best_id] / temperature;
    if (!(temperature > 0.0) || !__builtin_isfinite(best_scaled)) {
        leave(best_id);         // greedy, or a best value that is not finite (no share is): the generator rests
        return;
    }
    if (candidates == 1) {
        // one candidate is drawn like any list (native/src/v2_runtime.cpp:29722-29733): the generator moves on
        if (threadIdx.x == 0) {
            unsigned long long x = states[r] ? states[r] : 0x9E3779B97F4A7C15ull;
            x ^= x >> 12;
            x ^= x << 25;
            x ^= x >> 27;
            states[r] = x;
        }
        leave(best_id);
        return;
    }
    // The k-th best of the threads' best candidates (1,024 different ones) lies at or below the row's
    // k-th best: a bound for the first select over the row.
    s.keys[threadIdx.x] = mine;
    __syncthreads();
    const unsigned long long bound = sample_select([&](auto visit) { visit(s.keys[threadIdx.x]); }, 0ull, ~0ull,
                                                   (unsigned int)(candidates < SAMPLE_BATCH ? candidates : SAMPLE_BATCH), s);
    // (a longer list begins with what lies at or above the 512th of them: see below)
    unsigned long long half_bound = bound;
    if (candidates > SAMPLE_BATCH)
        half_bound = sample_select([&](auto visit) { visit(s.keys[threadIdx.x]); }, 0ull, ~0ull, SAMPLE_BATCH / 2, s);
    const auto over_row = [&](auto visit) {
        sample_for_each(row, vocab, [&](float value, int id) { visit(candidate_key(value, id)); });
    };

    // Up to 1,024 candidates are one batch. Everything at or above the bound is gathered at once; that
    // is the wanted candidates and usually few more (only a row with very many equal values gives more
    // than a batch holds: then the exact key of the last wanted candidate is selected first).
    bool first_batch_ready = false;
    int first_count = 0, first_asked = 0;       // asked: how many a batch was meant to hold (fewer came: nothing is left below)
    if (candidates <= SAMPLE_BATCH) {
        // (beyond half a batch the bound lies so low that what is above it seldom fits: 768 wanted of
        // 65,536 evenly spread values leave some 1,400 above the 768th of the threads' best)
        int count = 0;
        const bool at_once = candidates <= SAMPLE_BATCH / 2;
        if (at_once) count = sample_batch(row, vocab, bound, ~0ull, best_scaled, temperature, s);
        if (!at_once || s.gathered > SAMPLE_BATCH) {
            const unsigned long long floor_key = sample_select(over_row, bound, ~0ull, (unsigned int)candidates, s);
            count = sample_batch(row, vocab, floor_key, ~0ull, best_scaled, temperature, s);
        }
        first_count = count < candidates ? count : (int)candidates;
        first_batch_ready = true;
    } else {
        // The best of a longer list, gathered at once like a short list's: both walks begin with them,
        // and a peaked row ends both there. How many they are is not known beforehand (512 at least),
        // so this batch, unlike the selected ones, says nothing about what is left below it.
        first_count = sample_batch(row, vocab, half_bound, ~0ull, best_scaled, temperature, s);
        if (s.gathered > SAMPLE_BATCH) {
            const unsigned long long floor_key = sample_select(over_row, bound, ~0ull, SAMPLE_BATCH, s);
            first_count = sample_batch(row, vocab, floor_key, ~0ull, best_scaled, temperature, s);
            first_asked = SAMPLE_BATCH;
        }
        first_batch_ready = true;
    }
    // the sum over all candidates, which the shares of top_p are taken of
    double total = 1.0;
    if (top_p < 1.0) {
        if (candidates <= SAMPLE_BATCH) {
            total = sample_running_sum((int)threadIdx.x < first_count ? s.p[threadIdx.x] : 0.0, s, true);
        } else {
            const unsigned long long floor_key = candidates == vocab ? 0ull : sample_select(over_row, 0ull, ~0ull, (unsigned int)candidates, s);
            total = sample_total(row, vocab, floor_key, best_scaled, temperature, s);
        }
    }

    // First walk: where the kept prefix ends (top_p, min_p) and the sum of its p. Second walk: the
    // draw. Both go through the candidates in order, a batch at a time (with one batch it stays in
    // LDS); inside a batch thread i holds candidate i and the running sums up to it.
    double share_before = 0.0, mass_before = 0.0;       // of the batches walked so far
    long long keep = candidates;
    double threshold = 0.0;
    unsigned long long moved_on = 0ull;
    int token = best_id;
    // without cuts everything is kept: the kept sum is the sum over all candidates, and only the draw walks
    // (with one batch the first walk costs less than a sum over the row)
    const bool no_cuts = !(top_p < 1.0) && !(min_p > 0.0) && candidates > SAMPLE_BATCH;
    if (no_cuts) {
        unsigned long long floor_key = 0ull;
        if (candidates < vocab) floor_key = sample_select(over_row, 0ull, ~0ull, (unsigned int)candidates, s);
        mass_before = sample_total(row, vocab, floor_key, best_scaled, temperature, s);
    }
    for (int walk = no_cuts ? 1 : 0; walk < 2; ++walk) {
        unsigned long long ceiling = ~0ull;
        long long position = 0;
        const long long limit = walk == 0 ? candidates : keep;
        if (walk == 1) {
            // the draw (the generator moves on exactly once per drawn token; every thread forms the same numbers)
            unsigned long long x = states[r] ? states[r] : 0x9E3779B97F4A7C15ull;
            x ^= x >> 12;
            x ^= x << 25;
            x ^= x >> 27;
            moved_on = x;
            const double u = (double)((x * 2685821657736338717ull) >> 11) * (1.0 / 9007199254740992.0);
            threshold = u * mass_before;        // the sum of the kept p
            mass_before = 0.0;
        }
        bool stopped = false;
        while (position < limit && !stopped) {
            int count, asked;
            if (position == 0 && first_batch_ready) {
                count = first_count;        // still in LDS: made before the walks, and no later batch has taken its place
                asked = first_asked;
            } else {
                first_batch_ready = false;
                const long long left = limit - position;
                const unsigned int want = left < SAMPLE_BATCH ? (unsigned int)left : SAMPLE_BATCH;
                const unsigned long long floor_key = sample_select(over_row, position == 0 ? bound : 0ull, ceiling, want, s);
                count = sample_batch(row, vocab, floor_key, ceiling, best_scaled, temperature, s);
                asked = (int)want;
            }
            if (count == 0) break;
            const int here = limit - position < count ? (int)(limit - position) : count;
            const bool mine_counts = (int)threadIdx.x < here;
            const double p = mine_counts ? s.p[threadIdx.x] : 0.0;
            const double mass = mass_before + sample_running_sum(p, s, false);
            s.running[threadIdx.x] = mass;
            int first_stop = SAMPLE_BATCH;      // the first candidate of the batch at which the walk ends
            if (walk == 0) {
                const double share = top_p < 1.0 ? share_before + sample_running_sum(p / total, s, false) : 0.0;
                const bool below_min = min_p > 0.0 && position + threadIdx.x >= 1 && p < min_p;      // p of the best is 1
                const bool reaches_top = top_p < 1.0 && share >= top_p;
                if (mine_counts && (below_min || reaches_top)) first_stop = threadIdx.x;
                first_stop = sample_least(first_stop, s);
                if (first_stop < SAMPLE_BATCH) {
                    // the candidate at which it ends tells the others what is kept: up to it, without it if
                    // its p is below min_p (that is looked at first), with it if its share reaches top_p
                    if ((int)threadIdx.x == first_stop) s.keep_here = below_min ? first_stop : first_stop + 1;
                    __syncthreads();
                    keep = position + s.keep_here;
                    if (s.keep_here > 0) mass_before = s.running[s.keep_here - 1];
                    stopped = true;
                } else {
                    if ((int)threadIdx.x == here - 1) s.kept_share = share;
                    __syncthreads();
                    mass_before = s.running[here - 1];
                    share_before = s.kept_share;
                }
            } else {
                if (mine_counts && threshold <= mass) first_stop = threadIdx.x;
                first_stop = sample_least(first_stop, s);
                if (first_stop < SAMPLE_BATCH) {
                    token = candidate_id(s.keys[first_stop]);
                    stopped = true;
                } else {
                    token = candidate_id(s.keys[here - 1]);     // the last of the kept, should the sum never get there
                    __syncthreads();
                    mass_before = s.running[here - 1];
                }
            }
            __syncthreads();
            ceiling = s.keys[count - 1];
            position += count;
            if (count < asked) break;       // fewer than were asked for: nothing is left below
            __syncthreads();
        }
    }
    if (threadIdx.x == 0) states[r] = moved_on;
    leave(token);
}

// logits float32 [rows][vocab]; settings float32 [rows][4] (temperature, top_k, top_p, min_p; a
// temperature of 0 is greedy); states [rows] 64-bit generator states, moved on for the rows that
// draw; ids int32 [rows]. also / advance: as in fw_argmax_rows.
extern "C" int fw_sample_rows(const float* logits, const float* settings, unsigned long long* states, int32_t* ids,
                              int32_t* also, int32_t* advance, int rows, int vocab, void* stream) {
    FW_REQUIRE(rows >= 0 && rows <= 65535 && vocab > 0, "sample_rows: bad sizes rows=%d vocab=%d", rows, vocab);
    if (rows == 0) return 0;
    FW_REQUIRE(logits != nullptr && settings != nullptr && states != nullptr && ids != nullptr,
               "sample_rows: logits, settings, states and ids must be given");
    FW_REQUIRE((uintptr_t)states % 8 == 0, "sample_rows: the generator states must be 8-byte aligned");
    sample_rows_kernel<<<rows, SAMPLE_THREADS, 0, (hipStream_t)stream>>>(logits, settings, states, ids, also, advance, vocab);
    FW_LAUNCH_CHECK("sample_rows");
    return 0;
}
