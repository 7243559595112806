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
// 0.9 against 137 us when each walk selected its own first 1,024). A long list that this batch does
// not end (a flat distribution over the whole vocabulary) is not walked at all: the candidate at
// which a running sum reaches its target is searched digit by digit of its key, the row's mass
// added up per digit (sample_crossing), a dozen passes over the row whatever its shape.
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
    union {
        struct {
            unsigned long long keys[SAMPLE_BATCH];
            double p[SAMPLE_BATCH];
            double running[SAMPLE_BATCH];   // the sum of p up to and including each candidate of the batch
        };
        unsigned long long bin_mass[SAMPLE_BINS];   // the search for a crossing: each digit's mass in fixed point
    };
    unsigned long long bin_key[SAMPLE_BINS];        // and its greatest key
    unsigned long long above;                       // fixed-point mass of the keys above the digits found so far
    unsigned long long found_key;
    int found;                                      // 0: still searching, 1: the key is found, -1: the sums never get there
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

// the greatest of the threads' keys; every thread gets it
__device__ unsigned long long sample_block_max(unsigned long long v, SampleShared& s) {
    v = sample_wave_max(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s.wave_keys[threadIdx.x >> 6] = v;
    __syncthreads();
    unsigned long long best = 0ull;
    for (int w = 0; w < SAMPLE_THREADS / 64; ++w) best = s.wave_keys[w] > best ? s.wave_keys[w] : best;
    return best;
}

// exp((l - best) / T) / divisor of one logit (0 where the scaled logit is not finite)
__device__ __forceinline__ double sample_part(float value, double best_scaled, double temperature, double divisor) {
    const double scaled = (double)value / temperature;
    return __builtin_isfinite(scaled) ? exp(scaled - best_scaled) / divisor : 0.0;
}

// The sum of the parts of the candidates with key >= at_least and key > above, in a fixed order
// (each thread its own in the order of their ids, the threads of a wave by halving, the waves in turn).
__device__ double sample_mass(const float* __restrict__ row, int vocab, unsigned long long at_least, unsigned long long above,
                              double best_scaled, double temperature, double divisor, SampleShared& s) {
    double mine = 0.0;
    sample_for_each(row, vocab, [&](float value, int id) {
        const unsigned long long key = candidate_key(value, id);
        if (key >= at_least && key > above) mine += sample_part(value, best_scaled, temperature, divisor);
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

// A long list is not walked candidate by candidate. The candidate at which the running sum of the
// parts p / divisor, taken in the list's order (greatest key first) over the candidates with key >=
// floor_key, first reaches `target`: its key, or 0 if the sum never gets there. Found digit by digit
// of the key like the select above, with the mass of every digit instead of its count: each pass
// over the row adds the parts up per digit, in 64-bit fixed point (whole numbers add up to the same
// sum in any order, so the result does not depend on timing), and the digit in which the running
// sum passes the target is taken. A digit that holds one candidate ends the search. What fixed
// point rounds off (2^-47 of the greatest part per candidate) can misplace the answer by a
// neighbour where the target falls within that of a candidate's edge; the answer is therefore held
// against the sums in floating point, in the fixed order of sample_mass, and moved to a neighbour
// until it fits them (which it nearly always does at once). The fixed point is set so that a whole
// row of parts of 1 stays below 2^63 (2^46 for a vocabulary of 65,536).
__device__ unsigned long long sample_crossing(const float* __restrict__ row, int vocab, unsigned long long floor_key, double best_scaled,
                                              double temperature, double target, double divisor, SampleShared& s) {
    const double SAMPLE_FIXED = ldexp(1.0, 63 - (32 - __clz(vocab)));
    const double scaled_target = target * SAMPLE_FIXED;
    unsigned long long target_fixed = scaled_target >= 18446744073709549568.0 ? ~0ull : (unsigned long long)scaled_target;
    if (target_fixed == 0ull) target_fixed = 1ull;      // (the first candidate reaches any target that is not above its part)
    __syncthreads();
    if (threadIdx.x == 0) {
        s.prefix = 0ull;
        s.above = 0ull;
        s.found = 0;
    }
    int shift = 64;
    for (int level = 0; level < 6; ++level) {
        const int bits = shift >= SAMPLE_DIGIT_BITS ? SAMPLE_DIGIT_BITS : shift;
        shift -= bits;
        for (int i = threadIdx.x; i < SAMPLE_BINS; i += SAMPLE_THREADS) {
            s.histogram[i] = 0u;
            s.bin_mass[i] = 0ull;
            s.bin_key[i] = 0ull;
        }
        __syncthreads();
        const unsigned long long prefix = s.prefix;
        const int over = shift + bits;
        sample_for_each(row, vocab, [&](float value, int id) {
            const unsigned long long key = candidate_key(value, id);
            if (key >= floor_key && (over >= 64 || (key >> over) == prefix)) {
                const unsigned int digit = (unsigned int)(key >> shift) & ((1u << bits) - 1u);
                const double part = sample_part(value, best_scaled, temperature, divisor) * SAMPLE_FIXED;
                atomicAdd(&s.histogram[digit], 1u);
                atomicAdd(&s.bin_mass[digit], part >= 18446744073709549568.0 ? ~0ull : (unsigned long long)part);
                atomicMax(&s.bin_key[digit], key);
            }
        });
        __syncthreads();
        if (threadIdx.x < 64) {
            const int lane = threadIdx.x, per_lane = SAMPLE_BINS / 64;
            const int first = SAMPLE_BINS - 1 - lane * per_lane;    // lane 0 holds the highest digits
            unsigned long long mine = 0ull;
            for (int b = 0; b < per_lane; ++b) mine += s.bin_mass[first - b];
            unsigned long long before = mine;
#pragma unroll
            for (int offset = 1; offset < 64; offset <<= 1) {
                const unsigned long long other = __shfl_up(before, offset, 64);
                if (lane >= offset) before += other;
            }
            const unsigned long long start = s.above;
            const unsigned long long all = __shfl(before, 63, 64);
            if (start + all < target_fixed) {
                if (lane == 0) s.found = -1;
            } else {
                const unsigned long long ahead = start + (before - mine);
                if (ahead < target_fixed && target_fixed <= ahead + mine) {     // the digit is among this lane's
                    unsigned long long passed = ahead;
                    int digit = first;
                    for (int b = 0; b < per_lane; ++b) {
                        const unsigned long long here = s.bin_mass[first - b];
                        if (passed + here >= target_fixed) {
                            digit = first - b;
                            break;
                        }
                        passed += here;
                    }
                    s.prefix = (prefix << bits) | (unsigned long long)digit;
                    s.above = passed;
                    if (s.histogram[digit] == 1u) {
                        s.found_key = s.bin_key[digit];
                        s.found = 1;
                    }
                }
            }
        }
        __syncthreads();
        if (s.found != 0) break;
    }
    if (s.found < 0) return 0ull;
    unsigned long long key = s.found > 0 ? s.found_key : s.prefix;
    // held against the sums in floating point
    for (int tries = 0; tries < 8; ++tries) {
        const double before = sample_mass(row, vocab, floor_key, key, best_scaled, temperature, divisor, s);
        const double own = sample_part(row[candidate_id(key)], best_scaled, temperature, divisor);
        if (before >= target) {
            // reached before this candidate: the one before it in the list (the least key above)
            unsigned long long next = 0ull;
            sample_for_each(row, vocab, [&](float value, int id) {
                const unsigned long long k = candidate_key(value, id);
                if (k > key && ~k > next) next = ~k;
            });
            next = sample_block_max(next, s);
            if (next == 0ull) break;
            key = ~next;
        } else if (before + own < target) {
            // not yet reached with this candidate: the one behind it (the greatest key below, inside the list)
            unsigned long long next = 0ull;
            sample_for_each(row, vocab, [&](float value, int id) {
                const unsigned long long k = candidate_key(value, id);
                if (k < key && k >= floor_key && k > next) next = k;
            });
            next = sample_block_max(next, s);
            if (next == 0ull) return 0ull;      // the list ends here: the sums never get there
            key = next;
        } else {
            break;
        }
    }
    return key;
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
    // draw. Both go through the batch in LDS in order: thread i holds candidate i and the running
    // sums up to it.
    double mass_before = 0.0;       // the sum of the kept p, once the first walk has found where they end
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
    bool long_list = false;
    for (int walk = no_cuts ? 1 : 0; walk < 2 && !long_list; ++walk) {
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
        // the batch in LDS: made before the walks, the list's first candidates
        const int count = first_count;
        const int here = limit < count ? (int)limit : count;
        const bool mine_counts = (int)threadIdx.x < here;
        const double p = mine_counts ? s.p[threadIdx.x] : 0.0;
        const double mass = mass_before + sample_running_sum(p, s, false);
        s.running[threadIdx.x] = mass;
        int first_stop = SAMPLE_BATCH;      // the first candidate of the batch at which the walk ends
        bool stopped = false;
        if (walk == 0) {
            const double share = top_p < 1.0 ? sample_running_sum(p / total, s, false) : 0.0;
            const bool below_min = min_p > 0.0 && threadIdx.x >= 1 && p < min_p;      // p of the best is 1
            const bool reaches_top = top_p < 1.0 && share >= top_p;
            if (mine_counts && (below_min || reaches_top)) first_stop = threadIdx.x;
            first_stop = sample_least(first_stop, s);
            if (first_stop < SAMPLE_BATCH) {
                // the candidate at which it ends tells the others what is kept: up to it, without it if
                // its p is below min_p (that is looked at first), with it if its share reaches top_p
                if ((int)threadIdx.x == first_stop) s.keep_here = below_min ? first_stop : first_stop + 1;
                __syncthreads();
                keep = s.keep_here;
                if (s.keep_here > 0) mass_before = s.running[s.keep_here - 1];
                stopped = true;
            } else {
                __syncthreads();
                mass_before = s.running[here - 1];      // everything in the batch is kept
            }
        } else {
            if (mine_counts && threshold <= mass) first_stop = threadIdx.x;
            first_stop = sample_least(first_stop, s);
            stopped = first_stop < SAMPLE_BATCH;
            // (the last of the kept, should the sum never get there)
            token = candidate_id(s.keys[stopped ? first_stop : here - 1]);
        }
        __syncthreads();
        // The walk goes on behind the batch if the list does (a batch that was selected to hold 1,024 and
        // holds fewer has everything). A long list is not walked batch by batch: the search below.
        if (!stopped && here < limit && !(first_asked > 0 && count < first_asked)) long_list = true;
    }
    if (long_list) {
        // The kept candidates are those from some key up: the last of top_k, the candidate at which the
        // shares reach top_p, the least whose p is not below min_p (p falls along the list), whichever
        // is greatest. Then the draw: the candidate at which the running sum reaches u times the kept sum.
        __syncthreads();        // every wave has left the batch's arrays, which the search's bins lie over
        unsigned long long keep_key = 0ull;
        if (candidates < vocab) keep_key = sample_select(over_row, 0ull, ~0ull, (unsigned int)candidates, s);
        const unsigned long long list_floor = keep_key;
        if (top_p < 1.0) {
            const unsigned long long reached = sample_crossing(row, vocab, list_floor, best_scaled, temperature, top_p, total, s);
            keep_key = reached > keep_key ? reached : keep_key;
        }
        if (min_p > 0.0) {
            unsigned long long least = 0ull;        // of the complements: the least key whose p holds
            sample_for_each(row, vocab, [&](float value, int id) {
                const unsigned long long key = candidate_key(value, id);
                if (key >= list_floor && sample_part(value, best_scaled, temperature, 1.0) >= min_p && ~key > least) least = ~key;
            });
            least = sample_block_max(least, s);
            if (least != 0ull && ~least > keep_key) keep_key = ~least;
        }
        const double kept_mass = sample_mass(row, vocab, keep_key, 0ull, best_scaled, temperature, 1.0, s);
        unsigned long long x = states[r] ? states[r] : 0x9E3779B97F4A7C15ull;
        x ^= x >> 12;
        x ^= x << 25;
        x ^= x >> 27;
        moved_on = x;
        const double u = (double)((x * 2685821657736338717ull) >> 11) * (1.0 / 9007199254740992.0);
        unsigned long long drawn = sample_crossing(row, vocab, keep_key, best_scaled, temperature, u * kept_mass, 1.0, s);
        if (drawn == 0ull) {
            // the sum never got there: the last of the kept (the least key from keep_key up)
            unsigned long long least = 0ull;
            sample_for_each(row, vocab, [&](float value, int id) {
                const unsigned long long key = candidate_key(value, id);
                if (key >= keep_key && ~key > least) least = ~key;
            });
            drawn = ~sample_block_max(least, s);
        }
        token = candidate_id(drawn);
    }
    __syncthreads();        // (every thread has read the generator's state before it moves on)
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
