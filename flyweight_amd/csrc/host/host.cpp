// The flat C ABI over the host-side bookkeeping (see fw_host.h).
#include "fw_host.h"

#include <cstring>
#include <string>

#include "cache.hpp"
#include "scheduler.hpp"

namespace {

thread_local std::string last_error;

template <typename F>
int guarded(F&& body) {
    try {
        return body();
    } catch (const fwh::OutOfPages& e) {
        last_error = e.what();
        return FWH_OUT_OF_PAGES;
    } catch (const std::exception& e) {
        last_error = e.what();
        return FWH_ERROR;
    }
}

fwh::Pool* pool_of(void* p) { return static_cast<fwh::Pool*>(p); }
fwh::Cache* cache_of(void* p) { return static_cast<fwh::Cache*>(p); }
fwh::Scheduler* scheduler_of(void* p) { return static_cast<fwh::Scheduler*>(p); }

int copy_ids(const std::vector<fwh::Request*>& from, int64_t* to) {
    for (size_t i = 0; i < from.size(); ++i) to[i] = from[i]->id;
    return (int)from.size();
}

}  // namespace

extern "C" {

const char* fwh_last_error(void) { return last_error.c_str(); }
int fwh_abi_version(void) { return 5; }

// ---- pools ---------------------------------------------------------------------------------
void* fwh_pool_create(int size) {
    void* made = nullptr;
    guarded([&] { made = new fwh::Pool(size); return 0; });
    return made;
}
void fwh_pool_destroy(void* pool) { delete pool_of(pool); }
int fwh_pool_alloc(void* pool) { return guarded([&] { return pool_of(pool)->alloc(); }); }
int fwh_pool_free(void* pool, int id) { return guarded([&] { pool_of(pool)->free(id); return 0; }); }
int fwh_pool_size(void* pool) { return pool_of(pool)->size(); }
int fwh_pool_free_count(void* pool) { return pool_of(pool)->free_count(); }
int fwh_pool_peak(void* pool) { return pool_of(pool)->peak(); }
int fwh_pool_is_held(void* pool, int id) { return pool_of(pool)->is_held(id) ? 1 : 0; }

// ---- cache ---------------------------------------------------------------------------------
void* fwh_cache_create(int num_groups, const int* windows, int num_pages, int max_requests, int page_size,
                       int max_pages_per_request) {
    void* made = nullptr;
    guarded([&] {
        made = new fwh::Cache(std::vector<int>(windows, windows + num_groups), std::vector<int>{num_pages}, max_requests, page_size,
                              max_pages_per_request);
        return 0;
    });
    return made;
}
void* fwh_cache_create_sized(int num_groups, const int* windows, const int* pages, int max_requests, int page_size,
                             int max_pages_per_request) {
    void* made = nullptr;
    guarded([&] {
        if (num_groups < 1) throw std::invalid_argument("a cache sized per group needs at least one group");
        made = new fwh::Cache(std::vector<int>(windows, windows + num_groups), std::vector<int>(pages, pages + num_groups), max_requests,
                              page_size, max_pages_per_request);
        return 0;
    });
    return made;
}
void fwh_cache_destroy(void* cache) { delete cache_of(cache); }
void* fwh_cache_group_pool(void* cache, int group) {
    void* pool = nullptr;
    guarded([&] { pool = &cache_of(cache)->group(group).pool; return 0; });
    return pool;
}
void* fwh_cache_slot_pool(void* cache) { return &cache_of(cache)->slots(); }
int fwh_cache_admit(void* cache, int64_t request) { return guarded([&] { return cache_of(cache)->admit(request); }); }
int fwh_cache_reserve(void* cache, int64_t request, int new_length) {
    return guarded([&] { cache_of(cache)->reserve(request, new_length); return 0; });
}
int fwh_cache_commit(void* cache, int64_t request, int new_length) {
    return guarded([&] { cache_of(cache)->commit(request, new_length); return 0; });
}
int fwh_cache_truncate(void* cache, int64_t request, int token_count) {
    return guarded([&] { cache_of(cache)->truncate(request, token_count); return 0; });
}
int fwh_cache_truncate_batch(void* cache, const int64_t* requests, const int* token_counts, int count) {
    return guarded([&] {
        for (int i = 0; i < count; ++i) cache_of(cache)->truncate(requests[i], token_counts[i]);
        return 0;
    });
}
int fwh_cache_release(void* cache, int64_t request) { return guarded([&] { cache_of(cache)->release(request); return 0; }); }
int fwh_cache_is_live(void* cache, int64_t request) { return cache_of(cache)->is_live(request) ? 1 : 0; }
int fwh_cache_slot_of(void* cache, int64_t request) { return guarded([&] { return cache_of(cache)->of(request).slot; }); }
int fwh_cache_length_of(void* cache, int64_t request) { return guarded([&] { return cache_of(cache)->of(request).length; }); }
int fwh_cache_pages_missing(void* cache, int64_t request, int new_length, int* per_group) {
    return guarded([&] {
        fwh::Cache* c = cache_of(cache);
        for (int g = 0; g < c->num_groups(); ++g) per_group[g] = c->pages_missing(request, new_length, g);
        return c->num_groups();
    });
}
int fwh_cache_table(void* cache, int64_t request, int group, int* pages, int capacity) {
    return guarded([&] {
        const auto& tables = cache_of(cache)->group(group).tables;
        auto it = tables.find(request);
        if (it == tables.end()) throw std::out_of_range("request " + std::to_string(request) + " has no block table");
        const int n = (int)it->second.size();
        for (int i = 0; i < n && i < capacity; ++i) pages[i] = it->second[i];
        return n;
    });
}
int fwh_cache_fill_tables(void* cache, int group, const int64_t* requests, int count, int stride, int* rows) {
    return guarded([&] {
        const auto& tables = cache_of(cache)->group(group).tables;
        for (int i = 0; i < count; ++i) {
            auto it = tables.find(requests[i]);
            if (it == tables.end()) throw std::out_of_range("request " + std::to_string(requests[i]) + " has no block table");
            const std::vector<int>& table = it->second;
            if ((int)table.size() > stride) throw std::length_error("a block table is longer than the row it is copied to");
            int* row = rows + (size_t)i * stride;
            // a page that was given back is never read (the window has passed it); any valid id will do
            for (int b = 0; b < stride; ++b) row[b] = b < (int)table.size() && table[b] != fwh::NO_PAGE ? table[b] : 0;
        }
        return 0;
    });
}
int fwh_cache_longest_table(void* cache, int group, const int64_t* requests, int count) {
    return guarded([&] {
        const auto& tables = cache_of(cache)->group(group).tables;
        int longest = 0;
        for (int i = 0; i < count; ++i) {
            auto it = tables.find(requests[i]);
            if (it == tables.end()) throw std::out_of_range("request " + std::to_string(requests[i]) + " has no block table");
            longest = (int)it->second.size() > longest ? (int)it->second.size() : longest;
        }
        return longest;
    });
}
int fwh_cache_describe(void* cache, const int64_t* requests, int count, int* lengths, int* slots) {
    return guarded([&] {
        fwh::Cache* c = cache_of(cache);
        for (int i = 0; i < count; ++i) {
            const fwh::Live& live = c->of(requests[i]);
            lengths[i] = live.length;
            slots[i] = live.slot;
        }
        return 0;
    });
}
int fwh_cache_reserve_batch(void* cache, const int64_t* requests, const int* new_lengths, int count) {
    return guarded([&] {
        cache_of(cache)->reserve_batch(requests, new_lengths, count);
        return 0;
    });
}
int fwh_cache_commit_batch(void* cache, const int64_t* requests, const int* new_lengths, int count) {
    return guarded([&] {
        for (int i = 0; i < count; ++i) cache_of(cache)->commit(requests[i], new_lengths[i]);
        return 0;
    });
}
int fwh_cache_live(void* cache, int64_t* requests, int capacity) {
    int n = 0;
    for (const auto& entry : cache_of(cache)->live()) {
        if (n < capacity) requests[n] = entry.first;
        ++n;
    }
    return n;
}
int fwh_cache_check(void* cache) { return guarded([&] { cache_of(cache)->check(); return 0; }); }

// ---- scheduler -----------------------------------------------------------------------------
void* fwh_scheduler_create(void* cache, int max_positions, int max_batch_tokens, int chunk_size, int max_live, int max_queued,
                           int vocab_size) {
    void* made = nullptr;
    guarded([&] {
        made = new fwh::Scheduler(cache_of(cache), max_positions, max_batch_tokens, chunk_size, max_live, max_queued, vocab_size);
        return 0;
    });
    return made;
}
void fwh_scheduler_destroy(void* scheduler) { delete scheduler_of(scheduler); }
int64_t fwh_scheduler_submit(void* scheduler, const int* prompt, int prompt_len, int max_new_tokens, const int* stop_tokens,
                             int num_stop) {
    int64_t id = FWH_ERROR;
    guarded([&] { id = scheduler_of(scheduler)->submit(prompt, prompt_len, max_new_tokens, stop_tokens, num_stop)->id; return 0; });
    return id;
}
int fwh_scheduler_cancel(void* scheduler, int64_t request) { return scheduler_of(scheduler)->cancel(request) ? 1 : 0; }
int fwh_scheduler_fail(void* scheduler, int64_t request, const char* message) {
    return guarded([&] { return scheduler_of(scheduler)->fail_request(request, message ? message : "failed") ? 1 : 0; });
}
int fwh_scheduler_has_work(void* scheduler) { return scheduler_of(scheduler)->has_work() ? 1 : 0; }
int fwh_scheduler_preemptions(void* scheduler) { return scheduler_of(scheduler)->preemptions(); }
int fwh_scheduler_queue(void* scheduler, int which, int64_t* requests, int capacity) {
    fwh::Scheduler* s = scheduler_of(scheduler);
    int n = 0;
    auto put = [&](const fwh::Request* request) {
        if (n < capacity) requests[n] = request->id;
        ++n;
    };
    if (which == 0) for (const fwh::Request* request : s->waiting()) put(request);
    else for (const fwh::Request* request : s->running()) put(request);
    return n;
}
int fwh_scheduler_schedule(void* scheduler, int counts[7]) {
    return guarded([&] {
        fwh::Scheduler* s = scheduler_of(scheduler);
        const fwh::Plan& plan = s->schedule();
        fwh::Cache& cache = s->cache();
        int covered = 0;
        for (const fwh::Segment& segment : plan.segments) {
            covered = std::max(covered, segment.first + segment.count);
            for (int g = 0; g < cache.num_groups(); ++g)
                covered = std::max(covered, (int)cache.group(g).tables.at(segment.request->id).size() * cache.page_size());
        }
        counts[6] = covered;
        counts[0] = (int)plan.segments.size();
        counts[1] = plan.num_tokens;
        counts[2] = (int)plan.preempted.size();
        counts[3] = (int)plan.failed.size();
        counts[4] = (int)plan.admitted.size();
        counts[5] = (int)plan.cancelled.size();
        return 0;
    });
}
int fwh_plan_segments(void* scheduler, int64_t* requests, int* num_tokens, int* wants_logits, int* tokens) {
    const fwh::Plan& plan = scheduler_of(scheduler)->plan();
    int at = 0;
    for (size_t i = 0; i < plan.segments.size(); ++i) {
        const fwh::Segment& segment = plan.segments[i];
        requests[i] = segment.request->id;
        num_tokens[i] = segment.count;
        wants_logits[i] = segment.wants_logits ? 1 : 0;
        for (int t = 0; t < segment.count; ++t) tokens[at++] = segment.request->token_at(segment.first + t);
    }
    return (int)plan.segments.size();
}
int fwh_plan_list(void* scheduler, int which, int64_t* requests) {
    const fwh::Plan& plan = scheduler_of(scheduler)->plan();
    switch (which) {
        case 0: return copy_ids(plan.preempted, requests);
        case 1: return copy_ids(plan.failed, requests);
        case 2: return copy_ids(plan.admitted, requests);
        case 3: return copy_ids(plan.cancelled, requests);
    }
    last_error = "fwh_plan_list: unknown list";
    return FWH_ERROR;
}
int fwh_scheduler_complete(void* scheduler, const int64_t* requests, const int* tokens, int count, int64_t* event_requests,
                           int* event_values, int* event_kinds, int capacity) {
    return guarded([&] {
        std::unordered_map<int64_t, int> sampled;
        for (int i = 0; i < count; ++i) sampled[requests[i]] = tokens[i];
        const std::vector<fwh::Event> events = scheduler_of(scheduler)->complete(sampled);
        if ((int)events.size() > capacity) throw std::length_error("the event buffer is too small");
        for (size_t i = 0; i < events.size(); ++i) {
            event_requests[i] = events[i].request;
            event_values[i] = events[i].value;
            event_kinds[i] = events[i].kind;
        }
        return (int)events.size();
    });
}
int fwh_plan_fill_decode(void* scheduler, int capacity, int* tokens, int* positions, int* slots, int table_stride,
                         int* tables, int group_stride) {
    return guarded([&] {
        fwh::Scheduler* s = scheduler_of(scheduler);
        const fwh::Plan& plan = s->plan();
        if (plan.segments.empty() || !plan.preempted.empty() || !plan.failed.empty() || !plan.admitted.empty() ||
            !plan.cancelled.empty() || (int)plan.segments.size() > capacity)
            return FWH_NOT_DECODE_ONLY;
        for (const fwh::Segment& segment : plan.segments)
            if (segment.count != 1 || !segment.wants_logits) return FWH_NOT_DECODE_ONLY;
        fwh::Cache& cache = s->cache();
        const int rows = (int)plan.segments.size();
        for (int g = 0; g < cache.num_groups(); ++g)
            for (const fwh::Segment& segment : plan.segments)
                if ((int)cache.group(g).tables.at(segment.request->id).size() > table_stride)
                    throw std::length_error("a block table is longer than the row it is copied to");
        for (int i = 0; i < rows; ++i) {
            const fwh::Request* request = plan.segments[i].request;
            tokens[i] = request->token_at(plan.segments[i].first);
            positions[i] = plan.segments[i].first;
            slots[i] = cache.of(request->id).slot;
            for (int g = 0; g < cache.num_groups(); ++g) {
                const std::vector<int>& table = cache.group(g).tables.at(request->id);
                int* row = tables + (size_t)g * group_stride + (size_t)i * table_stride;
                // a page that was given back is never read (the window has passed it); any valid id will do
                for (int b = 0; b < table_stride; ++b) row[b] = b < (int)table.size() && table[b] != fwh::NO_PAGE ? table[b] : 0;
            }
        }
        return rows;
    });
}
int fwh_plan_steps_ahead(void* scheduler, int limit, int64_t* requests, int capacity) {
    return guarded([&] {
        fwh::Scheduler* s = scheduler_of(scheduler);
        const fwh::Plan& plan = s->plan();
        if (plan.segments.empty() || !plan.preempted.empty() || !plan.failed.empty() || !plan.admitted.empty() ||
            !plan.cancelled.empty() || s->place_for_admission() || plan.segments.size() != s->running().size())
            return 0;       // (a running request that this plan leaves out, for want of pages or budget, may be in the next)
        int ahead = limit, longest_budget = 0;
        for (const fwh::Segment& segment : plan.segments) {
            const fwh::Request* request = segment.request;
            if (segment.count != 1 || !segment.wants_logits || request->cancelled) return 0;
            const int budget = request->max_new_tokens - (int)request->generated.size() - 1;
            const int room = s->max_positions() - request->total() - 1;
            longest_budget = std::max(longest_budget, budget);
            ahead = std::min(ahead, room);
        }
        ahead = std::min(ahead, longest_budget);       // no step in which nobody is left
        if (ahead < 0) ahead = 0;
        if (requests)
            for (size_t i = 0; i < plan.segments.size() && (int)i < capacity; ++i) requests[i] = plan.segments[i].request->id;
        return ahead;
    });
}
int fwh_plan_budgets(void* scheduler, int* budgets, int capacity) {
    return guarded([&] {
        const fwh::Plan& plan = scheduler_of(scheduler)->plan();
        int rows = 0;
        for (const fwh::Segment& segment : plan.segments) {
            if (rows >= capacity) break;
            const fwh::Request* request = segment.request;
            const int budget = request->max_new_tokens - (int)request->generated.size() - (segment.wants_logits ? 1 : 0);
            budgets[rows++] = budget > 0 ? budget : 0;
        }
        return rows;
    });
}
int fwh_scheduler_complete_ordered(void* scheduler, const int* tokens, int count, int64_t* event_requests,
                                   int* event_values, int* event_kinds, int capacity) {
    return guarded([&] {
        fwh::Scheduler* s = scheduler_of(scheduler);
        std::unordered_map<int64_t, int> sampled;
        int given = 0;
        for (const fwh::Segment& segment : s->plan().segments)
            if (segment.wants_logits) {
                if (given >= count) throw fwh::SchedulerError("fewer tokens were handed over than the plan's segments want");
                sampled[segment.request->id] = tokens[given++];
            }
        if (given != count) throw fwh::SchedulerError("more tokens were handed over than the plan's segments want");
        const std::vector<fwh::Event> events = s->complete(sampled);
        if ((int)events.size() > capacity) throw std::length_error("the event buffer is too small");
        for (size_t i = 0; i < events.size(); ++i) {
            event_requests[i] = events[i].request;
            event_values[i] = events[i].value;
            event_kinds[i] = events[i].kind;
        }
        return (int)events.size();
    });
}
int fwh_request_info(void* scheduler, int64_t request, int info[9]) {
    return guarded([&] {
        const fwh::Request* r = scheduler_of(scheduler)->find(request);
        if (!r) throw std::out_of_range("unknown request " + std::to_string(request));
        info[0] = r->computed; info[1] = r->live; info[2] = r->finished; info[3] = r->cancelled; info[4] = r->admitted_at;
        info[5] = r->preemptions; info[6] = (int)r->prompt.size(); info[7] = (int)r->generated.size(); info[8] = r->max_new_tokens;
        return 0;
    });
}
int fwh_request_generated(void* scheduler, int64_t request, int* tokens, int capacity) {
    return guarded([&] {
        const fwh::Request* r = scheduler_of(scheduler)->find(request);
        if (!r) throw std::out_of_range("unknown request " + std::to_string(request));
        for (int i = 0; i < (int)r->generated.size() && i < capacity; ++i) tokens[i] = r->generated[i];
        return (int)r->generated.size();
    });
}
const char* fwh_request_error(void* scheduler, int64_t request) {
    const fwh::Request* r = scheduler_of(scheduler)->find(request);
    return r ? r->error.c_str() : "";
}
int fwh_scheduler_hold_admissions(void* scheduler, int plans) {
    scheduler_of(scheduler)->hold_admissions(plans);
    return 0;
}
int fwh_scheduler_forget(void* scheduler, int64_t request) { return scheduler_of(scheduler)->forget(request) ? 1 : 0; }

}  // extern "C"
