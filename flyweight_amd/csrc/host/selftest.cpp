// A self-test of the host library through its C entry points, meant to be built with the address
// and undefined-behaviour sanitizers (the package's tests build it so and run it): random request
// lifetimes over the cache (admit, reserve, commit, truncate, release), windowed groups, and the
// scheduler driven to completion under page pressure with cancelled and failed requests. Every
// answer is checked against a model kept here; exit status 0 means all of it held.
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "fw_host.h"

namespace {

int failures = 0;
#define EXPECT(cond)                                                              \
    do {                                                                          \
        if (!(cond)) {                                                            \
            std::fprintf(stderr, "selftest: line %d: %s\n", __LINE__, #cond);     \
            ++failures;                                                           \
        }                                                                         \
    } while (0)

struct Random {
    uint64_t state;
    explicit Random(uint64_t seed) : state(seed * 2654435761u + 1) {}
    uint32_t next() {
        state ^= state >> 12; state ^= state << 25; state ^= state >> 27;
        return (uint32_t)((state * 2685821657736338717ull) >> 33);
    }
    int below(int n) { return (int)(next() % (uint32_t)n); }
};

void pools() {
    void* pool = fwh_pool_create(3);
    EXPECT(fwh_pool_alloc(pool) == 0 && fwh_pool_alloc(pool) == 1 && fwh_pool_alloc(pool) == 2);
    EXPECT(fwh_pool_alloc(pool) == FWH_OUT_OF_PAGES);
    EXPECT(fwh_pool_free(pool, 1) == 0 && fwh_pool_free(pool, 1) == FWH_ERROR);
    EXPECT(fwh_pool_free(pool, 7) == FWH_ERROR && fwh_pool_free(pool, -1) == FWH_ERROR);
    EXPECT(fwh_pool_alloc(pool) == 1 && fwh_pool_peak(pool) == 3);
    fwh_pool_destroy(pool);
    EXPECT(fwh_pool_create(0) == nullptr && std::strlen(fwh_last_error()) > 0);
}

// Random lifetimes over a cache with one plain and one windowed group (on odd seeds the windowed
// group has a smaller pool of its own); a model of lengths is kept beside it and the library's
// own check runs after every change.
void cache_lifetimes(uint64_t seed) {
    const int pages = 24, slots = 5, page = 64, window = 100;
    const int windowed_pages = seed % 2 ? 9 : pages;
    const int windows[2] = {0, window};
    const int sizes[2] = {pages, windowed_pages};
    void* cache = seed % 2 ? fwh_cache_create_sized(2, windows, sizes, slots, page, 0) : fwh_cache_create(2, windows, pages, slots, page, 0);
    EXPECT(cache != nullptr);
    Random random(seed);
    std::map<int64_t, int> length;      // live request -> committed length
    int64_t next_id = 1;
    for (int step = 0; step < 4000; ++step) {
        const int what = random.below(10);
        if (what < 2 && (int)length.size() < slots) {
            const int slot = fwh_cache_admit(cache, next_id);
            EXPECT(slot >= 0 && slot < slots);
            EXPECT(fwh_cache_admit(cache, next_id) == FWH_ERROR);          // already live
            length[next_id++] = 0;
        } else if (what < 7 && !length.empty()) {
            auto it = length.begin();
            std::advance(it, random.below((int)length.size()));
            const int grown = it->second + 1 + random.below(150);
            const int status = fwh_cache_reserve(cache, it->first, grown);
            EXPECT(status == 0 || status == FWH_OUT_OF_PAGES);
            if (status == 0) {
                if (random.below(4) == 0) {             // the step does not run after all
                    EXPECT(fwh_cache_truncate(cache, it->first, it->second) == 0);
                } else {
                    EXPECT(fwh_cache_commit(cache, it->first, grown) == 0);
                    it->second = grown;
                }
            }
            EXPECT(fwh_cache_length_of(cache, it->first) == it->second);
        } else if (what < 8 && !length.empty()) {
            auto it = length.begin();
            std::advance(it, random.below((int)length.size()));
            // cutting back: fine while the windowed group still holds the keys it would need
            const int shorter = it->second - random.below(40);
            if (shorter >= 0) {
                const int status = fwh_cache_truncate(cache, it->first, shorter);
                EXPECT(status == 0 || status == FWH_ERROR);
                if (status == 0) it->second = std::min(it->second, shorter);
                EXPECT(fwh_cache_length_of(cache, it->first) == it->second);
            }
        } else if (!length.empty()) {
            auto it = length.begin();
            std::advance(it, random.below((int)length.size()));
            EXPECT(fwh_cache_release(cache, it->first) == 0);
            EXPECT(fwh_cache_release(cache, it->first) == FWH_ERROR);
            EXPECT(fwh_cache_is_live(cache, it->first) == 0);
            length.erase(it);
        }
        EXPECT(fwh_cache_check(cache) == 0);
        // block tables: as long as the sequence needs, nothing given back in the plain group
        for (const auto& entry : length) {
            int table[64];
            const int blocks = fwh_cache_table(cache, entry.first, 0, table, 64);
            EXPECT(blocks >= (entry.second + page - 1) / page && blocks <= 64);
            for (int b = 0; b < blocks && b < 64; ++b) EXPECT(table[b] >= 0 && table[b] < pages);
            const int windowed = fwh_cache_table(cache, entry.first, 1, table, 64);
            const int passed = entry.second - window + 1 > 0 ? (entry.second - window + 1) / page : 0;
            for (int b = 0; b < windowed && b < 64; ++b) EXPECT((table[b] == FWH_NO_PAGE) == (b < passed));
            for (int b = 0; b < windowed && b < 64; ++b) EXPECT(table[b] < windowed_pages);
        }
    }
    for (const auto& entry : length) EXPECT(fwh_cache_release(cache, entry.first) == 0);
    EXPECT(fwh_pool_free_count(fwh_cache_group_pool(cache, 0)) == pages);
    EXPECT(fwh_pool_free_count(fwh_cache_group_pool(cache, 1)) == windowed_pages);
    EXPECT(fwh_pool_free_count(fwh_cache_slot_pool(cache)) == slots);
    fwh_cache_destroy(cache);
}

int oracle(const std::vector<int>& tokens) {
    long long sum = 0;
    for (int t : tokens) sum += t;
    return (int)((sum * 31 + (long long)tokens.size()) % 97);
}

// The scheduler driven to the end with a fake model; some requests are cancelled, some fail in a
// step. Every other request must produce what it produces alone, and everything comes back.
void scheduler_runs(uint64_t seed) {
    Random random(seed);
    const int pages = 6 + random.below(6), slots = 2 + random.below(3);
    const int windows[1] = {0};
    void* cache = fwh_cache_create(1, windows, pages, slots, 64, 0);
    void* scheduler = fwh_scheduler_create(cache, 1024, 32 + random.below(100), 16 + random.below(64), 0, 256, 97);
    EXPECT(cache && scheduler);
    struct Seen { std::vector<int> prompt, tokens; int budget = 0; bool cancel = false, fail = false, ended = false, error = false; };
    std::map<int64_t, Seen> seen;
    const int requests = 8 + random.below(8);
    for (int i = 0; i < requests; ++i) {
        Seen s;
        s.prompt.resize(1 + random.below(150));
        for (int& t : s.prompt) t = random.below(97);
        s.budget = 1 + random.below(40);
        s.cancel = random.below(8) == 0;
        s.fail = !s.cancel && random.below(8) == 0;
        const int64_t id = fwh_scheduler_submit(scheduler, s.prompt.data(), (int)s.prompt.size(), s.budget, nullptr, 0);
        EXPECT(id > 0);
        seen[id] = s;
    }
    std::vector<int> bad(3, 97);
    EXPECT(fwh_scheduler_submit(scheduler, bad.data(), 3, 4, nullptr, 0) == FWH_ERROR);      // outside the vocabulary
    int steps = 0;
    while (fwh_scheduler_has_work(scheduler)) {
        int counts[7];
        EXPECT(fwh_scheduler_schedule(scheduler, counts) == 0);
        std::vector<int64_t> owners(counts[0] + 1);
        std::vector<int> lengths(counts[0] + 1), wants(counts[0] + 1), tokens(counts[1] + 1);
        fwh_plan_segments(scheduler, owners.data(), lengths.data(), wants.data(), tokens.data());
        std::vector<int64_t> drawn_for;
        std::vector<int> drawn;
        int at = 0, failed_now = 0;
        for (int i = 0; i < counts[0]; ++i) {
            Seen& s = seen[owners[i]];
            int info[9];
            EXPECT(fwh_request_info(scheduler, owners[i], info) == 0);
            // the segment brings the request's next tokens
            std::vector<int> all = s.prompt;
            all.insert(all.end(), s.tokens.begin(), s.tokens.end());
            for (int t = 0; t < lengths[i]; ++t) EXPECT(tokens[at + t] == all[info[0] + t]);
            at += lengths[i];
            if (s.fail && info[0] + lengths[i] > (int)s.prompt.size() / 2) {        // this step refuses it
                EXPECT(fwh_scheduler_fail(scheduler, owners[i], "refused by the selftest") == 1);
                EXPECT(fwh_scheduler_fail(scheduler, owners[i], "again") == 0);
                ++failed_now;
                continue;
            }
            if (wants[i]) {
                drawn_for.push_back(owners[i]);
                drawn.push_back(oracle(all));
            }
        }
        std::vector<int64_t> event_owner(2 * counts[0] + counts[3] + counts[5] + failed_now + 2);
        std::vector<int> event_value(event_owner.size()), event_kind(event_owner.size());
        const int made = fwh_scheduler_complete(scheduler, drawn_for.data(), drawn.data(), (int)drawn.size(), event_owner.data(),
                                                event_value.data(), event_kind.data(), (int)event_owner.size());
        EXPECT(made >= 0);
        for (int e = 0; e < made; ++e) {
            Seen& s = seen[event_owner[e]];
            if (event_kind[e] == FWH_EVENT_TOKEN) s.tokens.push_back(event_value[e]);
            if (event_kind[e] == FWH_EVENT_FINISHED) { EXPECT(!s.ended); s.ended = true; }
            if (event_kind[e] == FWH_EVENT_ERROR) {
                EXPECT(!s.ended);
                s.ended = s.error = true;
                EXPECT(std::strlen(fwh_request_error(scheduler, event_owner[e])) > 0);
            }
        }
        for (auto& entry : seen)
            if (entry.second.cancel && !entry.second.ended && (int)entry.second.tokens.size() >= entry.second.budget / 2)
                fwh_scheduler_cancel(scheduler, entry.first);
        EXPECT(fwh_cache_check(cache) == 0);
        EXPECT(++steps < 100000);
        if (steps >= 100000) break;
    }
    for (auto& entry : seen) {
        Seen& s = entry.second;
        EXPECT(s.ended);
        std::vector<int> all = s.prompt;
        for (size_t i = 0; i < s.tokens.size(); ++i) {        // every token is the one the request draws alone
            EXPECT(s.tokens[i] == oracle(all));
            all.push_back(s.tokens[i]);
        }
        if (!s.cancel && !s.error) EXPECT((int)s.tokens.size() == s.budget);
        EXPECT(fwh_scheduler_forget(scheduler, entry.first) == 1 && fwh_scheduler_forget(scheduler, entry.first) == 0);
    }
    EXPECT(fwh_pool_free_count(fwh_cache_group_pool(cache, 0)) == pages);
    EXPECT(fwh_pool_free_count(fwh_cache_slot_pool(cache)) == slots);
    fwh_scheduler_destroy(scheduler);
    fwh_cache_destroy(cache);
}

}  // namespace

int main() {
    EXPECT(fwh_abi_version() >= 2);
    pools();
    for (uint64_t seed = 1; seed <= 6; ++seed) cache_lifetimes(seed);
    for (uint64_t seed = 1; seed <= 40; ++seed) scheduler_runs(seed);
    if (failures) {
        std::fprintf(stderr, "selftest: %d checks failed\n", failures);
        return 1;
    }
    std::printf("selftest: ok\n");
    return 0;
}
