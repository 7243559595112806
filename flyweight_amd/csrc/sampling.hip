// Drawing the next token of every row on the device: greedy, temperature, top-k, top-p, min-p,
// each request with its own xorshift64* generator, in the reference's order of operations
// (native/src/v2_runtime.cpp:29500-29566, 29686-29743; generator :29307-29314):
//
//   candidates sorted by (value descending, id ascending), the first top_k of them (0: all);
//   p_i = exp((l_i - l_0) / T) in float64; total = sum of p; top_p keeps the shortest prefix
//   whose shares p_i / total add up to it; min_p ends the prefix before the first p_i < min_p;
//   u * (sum of the kept p) is walked down the prefix until the running sum reaches it.
//
// One workgroup of 1,024 threads per row. The sorted list is never made as a whole. With top_k up to
// 1,024 (the usual case) the candidates are one batch: selected (a radix select over the 64-bit keys:
// up to six passes over the row, counting in LDS), sorted in LDS, their p formed by all threads, thread
// i holding candidate i and the running sums up to it (a scan in a fixed order); up to 512 they are
// gathered without a select, everything at or above the k-th of the threads' own best. A longer list
// (no top_k) is not walked at all: one pass counts the row into 2,048 bins of the value with each
// bin's mass, and the candidate at which a running sum reaches its target (where top_p ends the list,
// where the draw lands) is found in the one bin where the bins' sums pass it, whose candidates are
// gathered and sorted like a short list; the answer is held against the sums in floating point in a
// fixed order, so that it does not depend on timing (sample_crossing_bins).
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
    union {
        struct {
            double p[SAMPLE_BATCH];
            double running[SAMPLE_BATCH];   // the sum of p up to and including each candidate of the batch
        };
        unsigned long long bin_key[SAMPLE_BINS];    // the search by the key's digits: each digit's greatest key
    };
    unsigned long long bin_mass[SAMPLE_BINS];       // a long list: each bin's mass in fixed point
    unsigned long long above;                       // fixed-point mass of the keys above the bin or digits found so far
    unsigned long long found_key;
    int found;                                      // 0: still searching, 1: found, -1: the sums never get there
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

// The sum of x over the threads up to and including this one, in whole numbers.
__device__ unsigned long long sample_running_fixed(unsigned long long x, SampleShared& s) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    unsigned long long sum = x;
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
        const unsigned long long other = __shfl_up(sum, offset, 64);
        if (lane >= offset) sum += other;
    }
    __syncthreads();
    if (lane == 63) s.wave_keys[wave] = sum;
    __syncthreads();
    unsigned long long before = 0ull;
    for (int w = 0; w < wave; ++w) before += s.wave_keys[w];
    return before + sum;
}

// Calls visit(value, id) for this thread's share of a row, four neighbours at a time where the row
// allows 16-byte loads, and eight such loads asked for before the first value is looked at: a pass over
// the row is one workgroup's, and with a load per turn of the loop it would wait out the memory's
// latency sixteen times over.
#define SAMPLE_AHEAD 8
template <int AHEAD = SAMPLE_AHEAD, typename Visit>
__device__ __forceinline__ void sample_for_each(const float* __restrict__ row, int vocab, Visit visit) {
    if ((vocab & 3) == 0 && ((uintptr_t)row & 15) == 0) {
        const float4* quads = reinterpret_cast<const float4*>(row);
        const int count = vocab / 4;
        for (int q0 = threadIdx.x; q0 < count; q0 += AHEAD * SAMPLE_THREADS) {
            float4 v[AHEAD];
#pragma unroll
            for (int u = 0; u < AHEAD; ++u) {
                const int q = q0 + u * SAMPLE_THREADS;
                v[u] = quads[q < count ? q : q0];
            }
#pragma unroll
            for (int u = 0; u < AHEAD; ++u) {
                const int q = q0 + u * SAMPLE_THREADS;
                if (q < count) {
                    visit(v[u].x, 4 * q);
                    visit(v[u].y, 4 * q + 1);
                    visit(v[u].z, 4 * q + 2);
                    visit(v[u].w, 4 * q + 3);
                }
            }
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

// ---- a long list (no top_k, or one above 1,024) --------------------------------------------------
// A long list is not walked candidate by candidate, and its sums are whole numbers: every candidate's
// part p = exp((l - best) / T) is taken in fixed point, round(p * 2^f) with f such that a whole row of
// parts of 1 stays below 2^63 (f = 46 for a vocabulary of 65,536, 50 at most), and a running sum is the
// sum of these numbers, the same in any order and on any number of threads: where the reference adds
// in float64 along the sorted list, this differs from it by up to 2^-47 of the greatest part per
// candidate (5e-10 of the total over 65,536 candidates), so a cut or a draw can fall on the
// neighbouring candidate where the target lies that close to the boundary between two.
//
// The candidates are counted once into 2,048 bins by their value's distance from the best,
// bin = (best - value) * 2,047 / span, span being what the row's finite values cover, or 48
// temperatures if that is less (what lies further down has parts below e^-48 and shares the last
// bin). The bin falls as the key rises, so the bins are the sorted list cut into pieces: the piece in
// which a running sum reaches its target is read off the bins' masses, its candidates, some hundred of
// 65,536, are gathered and sorted in LDS like a short list, and the candidate is the one at which the
// running sum inside the piece gets there. Both searches of a draw (where top_p ends the list, where
// u lands) use the same bins: two passes over the row and one per search. A piece that holds more
// than a batch (a row of equal values) is searched by the digits of the key instead.
__device__ __forceinline__ int sample_value_bin(float value, float best_value, float scale) {
    const float d = (best_value - value) * scale;       // >= 0; NaN for a NaN, inf for -inf: the last bin
    return d < (float)(SAMPLE_BINS - 1) ? (int)d : SAMPLE_BINS - 1;
}

// round(part) for 0 <= part <= 2^50: one addition (the sum's low bits are the number) instead of a
// conversion of a dozen instructions, once per logit
__device__ __forceinline__ unsigned long long sample_fixed(double part) {
    return (unsigned long long)(__double_as_longlong(part + 6755399441055744.0) - __double_as_longlong(6755399441055744.0));
}

// a target in fixed point: at least 1 (the first candidate reaches any target that is not above its part)
__device__ __forceinline__ unsigned long long sample_target(double fraction, unsigned long long of) {
    const double scaled = fraction * (double)of;
    const unsigned long long target = scaled >= 9223372036854775808.0 ? (1ull << 63) : (unsigned long long)scaled;
    return target == 0ull ? 1ull : (target > of ? of : target);
}

// the fixed-point part of one logit (0 where the scaled logit is not finite)
__device__ __forceinline__ unsigned long long sample_part(float value, double best_scaled, double temperature, double fixed_one) {
    const double scaled = (double)value / temperature;
    return __builtin_isfinite(scaled) ? sample_fixed(exp(scaled - best_scaled) * fixed_one) : 0ull;
}

// the sum of the threads' numbers; every thread gets it
__device__ unsigned long long sample_block_sum(unsigned long long v, SampleShared& s) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) s.wave_keys[threadIdx.x >> 6] = v;
    __syncthreads();
    unsigned long long total = 0ull;
    for (int w = 0; w < SAMPLE_THREADS / 64; ++w) total += s.wave_keys[w];
    return total;
}

// The search by the digits of the key, for a piece of the list that no batch holds: the candidate at
// which the running sum of the parts, in the list's order over the candidates with key >= floor_key,
// first reaches `target` (its key, and in *reached the sum up to and including it), or 0 if the sum
// never gets there. Digit by digit like the select above, with the mass of every digit instead of its
// count; a digit that holds one candidate ends the search. Up to six passes over the row, each forming
// every part again. Uses the bins' memory.
__device__ unsigned long long sample_crossing(const float* __restrict__ row, int vocab, unsigned long long floor_key, double best_scaled,
                                              double temperature, unsigned long long target, double fixed_one, unsigned long long* reached,
                                              SampleShared& s) {
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
                atomicAdd(&s.histogram[digit], 1u);
                atomicAdd(&s.bin_mass[digit], sample_part(value, best_scaled, temperature, fixed_one));
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
            if (start + all < target) {
                if (lane == 0) s.found = -1;
            } else {
                const unsigned long long ahead = start + (before - mine);
                if (ahead < target && target <= ahead + mine) {     // the digit is among this lane's
                    unsigned long long passed = ahead;
                    int digit = first;
                    for (int b = 0; b < per_lane; ++b) {
                        const unsigned long long here = s.bin_mass[first - b];
                        if (passed + here >= target) {
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
    const unsigned long long key = s.found > 0 ? s.found_key : s.prefix;
    *reached = s.above + sample_part(row[candidate_id(key)], best_scaled, temperature, fixed_one);
    __syncthreads();        // (every thread has read what the search left before a next one begins)
    return key;
}

// One pass: the bins' counts and masses over the candidates with key >= floor_key, and with min_p the
// complement of the least key whose p holds (0: none).
__device__ void sample_fill_bins(const float* __restrict__ row, int vocab, unsigned long long floor_key, float best_value, float scale,
                                 double best_scaled, double temperature, double min_p, double fixed_one, unsigned long long* holding,
                                 SampleShared& s) {
    __syncthreads();
    for (int i = threadIdx.x; i < SAMPLE_BINS; i += SAMPLE_THREADS) {
        s.histogram[i] = 0u;
        s.bin_mass[i] = 0ull;
    }
    __syncthreads();
    unsigned long long least = 0ull, tail_mass = 0ull;
    unsigned int tail_count = 0u;       // the last bin can hold most of a peaked row: each thread counts its own
    sample_for_each<2>(row, vocab, [&](float value, int id) {
        const unsigned long long key = candidate_key(value, id);
        if (key >= floor_key) {
            const double scaled = (double)value / temperature;
            const double p = __builtin_isfinite(scaled) ? exp(scaled - best_scaled) : 0.0;
            if (min_p > 0.0 && p >= min_p && ~key > least) least = ~key;
            const unsigned long long fixed = sample_fixed(p * fixed_one);
            const int bin = sample_value_bin(value, best_value, scale);
            if (bin == SAMPLE_BINS - 1) {
                tail_count += 1u;
                tail_mass += fixed;
            } else {
                atomicAdd(&s.histogram[bin], 1u);
                atomicAdd(&s.bin_mass[bin], fixed);
            }
        }
    });
    if (tail_count > 0u) {
        atomicAdd(&s.histogram[SAMPLE_BINS - 1], tail_count);
        atomicAdd(&s.bin_mass[SAMPLE_BINS - 1], tail_mass);
    }
    *holding = min_p > 0.0 ? sample_block_max(least, s) : 0ull;
    __syncthreads();
}

// the sum of all bins; every thread gets it
__device__ unsigned long long sample_bins_total(SampleShared& s) {
    unsigned long long mine = 0ull;
    for (int i = threadIdx.x; i < SAMPLE_BINS; i += SAMPLE_THREADS) mine += s.bin_mass[i];
    return sample_block_sum(mine, s);
}

// The candidate at which the running sum of the parts, in the list's order over the candidates with
// key >= floor_key, first reaches `target` (its key, and in *reached the sum up to and including it;
// 0 if it never does), from the bins that sample_fill_bins has left (made with a floor at or below
// this one). bins_valid: cleared if the search had to go by the key's digits, which uses the bins' memory.
__device__ unsigned long long sample_crossing_bins(const float* __restrict__ row, int vocab, unsigned long long floor_key, float best_value,
                                                   float scale, double best_scaled, double temperature, unsigned long long target,
                                                   double fixed_one, unsigned long long* reached, bool& bins_valid, SampleShared& s) {
    __syncthreads();
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x, per_lane = SAMPLE_BINS / 64;
        const int first = lane * per_lane;      // lane 0 holds the bins of the best values
        unsigned long long mine = 0ull;
        for (int b = 0; b < per_lane; ++b) mine += s.bin_mass[first + b];
        unsigned long long before = mine;
#pragma unroll
        for (int offset = 1; offset < 64; offset <<= 1) {
            const unsigned long long other = __shfl_up(before, offset, 64);
            if (lane >= offset) before += other;
        }
        const unsigned long long all = __shfl(before, 63, 64);
        if (lane == 0) s.found = all < target ? -1 : 0;
        const unsigned long long ahead = before - mine;
        if (all >= target && ahead < target && target <= before) {       // the bin is among this lane's
            unsigned long long passed = ahead;
            int bin = first + per_lane - 1;
            for (int b = 0; b < per_lane; ++b) {
                const unsigned long long here = s.bin_mass[first + b];
                if (passed + here >= target) {
                    bin = first + b;
                    break;
                }
                passed += here;
            }
            s.prefix = (unsigned long long)bin;
            s.above = passed;
        }
    }
    if (threadIdx.x == 0) s.gathered = 0u;
    s.keys[threadIdx.x] = 0ull;
    __syncthreads();
    if (s.found < 0) return 0ull;
    const int bin = (int)s.prefix;
    const unsigned long long start = s.above;
    if (s.histogram[bin] <= 4u * SAMPLE_BATCH)      // (the count includes what lies below this floor; far too many: not even tried)
        sample_for_each(row, vocab, [&](float value, int id) {
            const unsigned long long key = candidate_key(value, id);
            if (key >= floor_key && sample_value_bin(value, best_value, scale) == bin) {
                const unsigned int slot = atomicAdd(&s.gathered, 1u);
                if (slot < SAMPLE_BATCH) s.keys[slot] = key;
            }
        });
    else if (threadIdx.x == 0)
        s.gathered = SAMPLE_BATCH + 1u;
    __syncthreads();
    const unsigned int gathered = s.gathered;
    if (gathered > SAMPLE_BATCH) {
        // the digits search counts from the list's top: what it finds is the same candidate
        bins_valid = false;
        return sample_crossing(row, vocab, floor_key, best_scaled, temperature, target, fixed_one, reached, s);
    }
    if (gathered == 0u) return 0ull;    // (the floor lies above this bin: the list ends before the target)
    int slots = 2;
    while (slots < (int)gathered) slots <<= 1;
    sample_sort(s.keys, slots);
    unsigned long long fixed = 0ull;
    if (threadIdx.x < gathered) fixed = sample_part(row[candidate_id(s.keys[threadIdx.x])], best_scaled, temperature, fixed_one);
    const unsigned long long running = start + sample_running_fixed(fixed, s);
    s.bin_key[threadIdx.x] = running;       // (the batch's p and running sums are not in use: the same memory)
    int stop = (threadIdx.x < gathered && running >= target) ? (int)threadIdx.x : SAMPLE_BATCH;
    stop = sample_least(stop, s);
    unsigned long long key = 0ull;
    if (stop < SAMPLE_BATCH) {
        key = s.keys[stop];
        *reached = s.bin_key[stop];
    }
    __syncthreads();        // (every thread has read them before the next pass uses the batch's memory)
    return key;             // (0: the floor cut this bin short of the target)
}

// The fixed-point sum of the parts of the candidates with key >= from, from the bins and one pass over
// the row for the candidates of its own bin.
__device__ unsigned long long sample_mass_from(const float* __restrict__ row, int vocab, unsigned long long from, float best_value,
                                               float scale, double best_scaled, double temperature, double fixed_one, SampleShared& s) {
    const int bin = sample_value_bin(row[candidate_id(from)], best_value, scale);
    unsigned long long mine = 0ull;
    for (int i = threadIdx.x; i < bin; i += SAMPLE_THREADS) mine += s.bin_mass[i];
    sample_for_each(row, vocab, [&](float value, int id) {
        if (candidate_key(value, id) >= from && sample_value_bin(value, best_value, scale) == bin)
            mine += sample_part(value, best_scaled, temperature, fixed_one);
    });
    return sample_block_sum(mine, s);
}

// settings: [rows][4] = temperature, top_k (a whole number), top_p, min_p. states: the rows'
// generators, read and moved on by the rows that draw.
// Two kernels share the rows: LONG takes those that draw from more than 1,024 candidates, the other all
// the rest (each is compiled for its own path's registers; a workgroup whose row is the other's leaves
// at once).
template <bool LONG>
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(const float* __restrict__ logits,
                                                                     const float* __restrict__ settings,
                                                                     unsigned long long* __restrict__ states,
                                                                     int32_t* __restrict__ ids, int32_t* __restrict__ also,
                                                                     int32_t* __restrict__ advance, int vocab) {
    __shared__ SampleShared s;
    const int r = blockIdx.x;
    {
        const long long k = (long long)settings[4 * r + 1];
        const bool long_list = settings[4 * r + 0] > 0.0f && !(k > 0 && k <= SAMPLE_BATCH) && vocab > SAMPLE_BATCH;
        if (long_list != LONG) return;
    }
    const float* row = logits + (size_t)r * vocab;
    const double temperature = (double)settings[4 * r + 0];
    const double top_p = (double)settings[4 * r + 2], min_p = (double)settings[4 * r + 3];
    long long top_k = (long long)settings[4 * r + 1];

    // every thread's best candidate; the best of those is the row's (and the least finite value, for a long list's bins)
    unsigned long long mine = 0ull;
    float low = __builtin_inff();
    sample_for_each(row, vocab, [&](float value, int id) {
        const unsigned long long key = candidate_key(value, id);
        mine = key > mine ? key : mine;
        if (LONG && __builtin_isfinite(value)) low = fminf(low, value);
    });
    unsigned long long best = sample_wave_max(mine);
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) low = fminf(low, __shfl_xor(low, offset, 64));
    if ((threadIdx.x & 63) == 0) {
        s.wave_keys[threadIdx.x >> 6] = best;
        s.wave_sums[threadIdx.x >> 6] = (double)low;
    }
    __syncthreads();
    best = 0ull;
    for (int w = 0; w < SAMPLE_THREADS / 64; ++w) {
        best = s.wave_keys[w] > best ? s.wave_keys[w] : best;
        low = fminf(low, (float)s.wave_sums[w]);
    }
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
    // the draw's number (the generator moves on exactly once per drawn token; every thread forms the same numbers)
    unsigned long long moved_on = states[r] ? states[r] : 0x9E3779B97F4A7C15ull;
    moved_on ^= moved_on >> 12;
    moved_on ^= moved_on << 25;
    moved_on ^= moved_on >> 27;
    const double u = (double)((moved_on * 2685821657736338717ull) >> 11) * (1.0 / 9007199254740992.0);
    __syncthreads();        // (every thread has read the generator's state before it moves on)
    if (threadIdx.x == 0) states[r] = moved_on;
    if (candidates == 1) {
        // one candidate is drawn like any list (native/src/v2_runtime.cpp:29722-29733): the generator has moved on
        leave(best_id);
        return;
    }
    const auto over_row = [&](auto visit) {
        sample_for_each(row, vocab, [&](float value, int id) { visit(candidate_key(value, id)); });
    };

    if constexpr (LONG) {
        // A long list. The kept candidates are those from some key up: the last of top_k, the candidate at
        // which the shares reach top_p, the least whose p is not below min_p (p falls along the list),
        // whichever is greatest. Then the draw: the candidate at which the running sum reaches u times the kept sum.
        // fixed point: a whole row of parts of 1 stays below 2^63, and one part within what sample_fixed takes
        const int fixed_bits = 63 - (32 - __clz(vocab));
        const double fixed_one = ldexp(1.0, fixed_bits < 50 ? fixed_bits : 50);
        const unsigned long long floor_key = candidates < vocab ? sample_select(over_row, 0ull, ~0ull, (unsigned int)candidates, s) : 0ull;
        const float best_value = row[best_id];
        const float reach = (float)(temperature * 48.0);
        float span = best_value - low;
        if (!(span <= reach)) span = reach;
        const float scale = span > 0.0f ? (float)(SAMPLE_BINS - 1) / span : 0.0f;
        unsigned long long holding = 0ull;
        sample_fill_bins(row, vocab, floor_key, best_value, scale, best_scaled, temperature, min_p, fixed_one, &holding, s);
        bool bins_valid = true;
        unsigned long long keep_key = floor_key;
        unsigned long long kept_mass = sample_bins_total(s);
        if (top_p < 1.0) {
            unsigned long long reached_mass = 0ull;
            const unsigned long long reached = sample_crossing_bins(row, vocab, floor_key, best_value, scale, best_scaled, temperature,
                                                                    sample_target(top_p, kept_mass), fixed_one, &reached_mass, bins_valid, s);
            if (reached > keep_key) {
                keep_key = reached;
                kept_mass = reached_mass;
            }
        }
        if (!bins_valid) {
            unsigned long long unused = 0ull;
            sample_fill_bins(row, vocab, floor_key, best_value, scale, best_scaled, temperature, 0.0, fixed_one, &unused, s);
            bins_valid = true;
        }
        if (holding != 0ull && ~holding > keep_key) {
            keep_key = ~holding;
            kept_mass = sample_mass_from(row, vocab, keep_key, best_value, scale, best_scaled, temperature, fixed_one, s);
        }
        unsigned long long drawn_mass = 0ull;
        unsigned long long drawn = sample_crossing_bins(row, vocab, keep_key, best_value, scale, best_scaled, temperature,
                                                        sample_target(u, kept_mass), fixed_one, &drawn_mass, bins_valid, s);
        if (drawn == 0ull) {
            // (the sum never got there: the last of the kept, the least key from keep_key up)
            unsigned long long least = 0ull;
            sample_for_each(row, vocab, [&](float value, int id) {
                const unsigned long long key = candidate_key(value, id);
                if (key >= keep_key && ~key > least) least = ~key;
            });
            drawn = ~sample_block_max(least, s);
        }
        leave(candidate_id(drawn));
        return;
    } else {

    // Up to 1,024 candidates are one batch in LDS. The k-th best of the threads' best candidates (1,024
    // different ones) lies at or below the row's k-th best: a bound for a select over the row, and up to
    // 512 wanted everything at or above it is gathered without one; that is the wanted candidates and
    // usually few more (only a row with very many equal values gives more than a batch holds: then the
    // exact key of the last wanted candidate is selected first). Beyond half a batch the bound lies so
    // low that what is above it seldom fits: 768 wanted of 65,536 evenly spread values leave some 1,400
    // above the 768th of the threads' best.
    s.keys[threadIdx.x] = mine;
    __syncthreads();
    const unsigned long long bound = sample_select([&](auto visit) { visit(s.keys[threadIdx.x]); }, 0ull, ~0ull, (unsigned int)candidates, s);
    int count = 0;
    const bool at_once = candidates <= SAMPLE_BATCH / 2;
    if (at_once) count = sample_batch(row, vocab, bound, ~0ull, best_scaled, temperature, s);
    if (!at_once || s.gathered > SAMPLE_BATCH) {
        const unsigned long long floor_key = sample_select(over_row, bound, ~0ull, (unsigned int)candidates, s);
        count = sample_batch(row, vocab, floor_key, ~0ull, best_scaled, temperature, s);
    }
    const int listed = count < candidates ? count : (int)candidates;
    // the sum over all candidates, which the shares of top_p are taken of
    const double total = top_p < 1.0 ? sample_running_sum((int)threadIdx.x < listed ? s.p[threadIdx.x] : 0.0, s, true) : 1.0;

    // First walk: where the kept prefix ends (top_p, min_p) and the sum of its p. Second walk: the
    // draw. Both go through the batch in order: thread i holds candidate i and the running sums up to it.
    double mass_before = 0.0;       // the sum of the kept p, once the first walk has found where they end
    int keep = listed;
    int token = best_id;
    for (int walk = 0; walk < 2; ++walk) {
        const int here = walk == 0 ? listed : keep;
        const double threshold = u * mass_before;       // (the second walk's: of the sum of the kept p)
        const bool mine_counts = (int)threadIdx.x < here;
        const double p = mine_counts ? s.p[threadIdx.x] : 0.0;
        const double mass = sample_running_sum(p, s, false);
        s.running[threadIdx.x] = mass;
        int first_stop = SAMPLE_BATCH;      // the first candidate of the batch at which the walk ends
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
            } else {
                __syncthreads();    // everything in the batch is kept
            }
            mass_before = keep > 0 ? s.running[keep - 1] : 0.0;
        } else {
            if (mine_counts && threshold <= mass) first_stop = threadIdx.x;
            first_stop = sample_least(first_stop, s);
            // (the last of the kept, should the sum never get there)
            token = candidate_id(s.keys[first_stop < SAMPLE_BATCH ? first_stop : here - 1]);
        }
        __syncthreads();
    }
    leave(token);
    }
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
    sample_rows_kernel<false><<<rows, SAMPLE_THREADS, 0, (hipStream_t)stream>>>(logits, settings, states, ids, also, advance, vocab);
    FW_LAUNCH_CHECK("sample_rows");
    if (vocab > SAMPLE_BATCH) {
        sample_rows_kernel<true><<<rows, SAMPLE_THREADS, 0, (hipStream_t)stream>>>(logits, settings, states, ids, also, advance, vocab);
        FW_LAUNCH_CHECK("sample_rows (long lists)");
    }
    return 0;
}
