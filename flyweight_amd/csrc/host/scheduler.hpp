// Continuous batching: which requests run in the next step, and with which tokens.
//
// A step is one mixed batch: first every decoding request contributes its one row, then the
// rest of the token budget goes to portions of prompts (oldest first), then new requests are
// admitted while a slot and the pages of their first portion are there. Pages a step will
// write are reserved while the plan is made. When the pool cannot cover a decode row the most
// recently admitted request gives way: its pages and slot are freed and it returns to the front
// of the queue with what it has generated (recomputed later; the logits do not depend on how a
// sequence is cut, so the continuation is the same). The oldest request never gives way; a
// request that does not fit even alone ends with an error. Nobody is admitted in a step in
// which somebody gave way.
//
// The reference visits its tasks round-robin, one prompt chunk or one token of ONE task per
// step (native/src/v2_runtime.cpp:33699-33963), reserves a whole slot per task and so never
// runs out of pages; queue limit and validation follow its task submit (:32502-32599).
#pragma once
#include <algorithm>
#include <deque>
#include <memory>
#include <unordered_set>

#include "cache.hpp"

namespace fwh {

enum EventKind { EVENT_TOKEN = 0, EVENT_FINISHED = 1, EVENT_ERROR = 2, EVENT_PREFILL = 3 };

struct SchedulerError : std::invalid_argument {
    using std::invalid_argument::invalid_argument;
};

struct Request {
    int64_t id = 0;
    std::vector<int> prompt, generated, stop_tokens;
    int max_new_tokens = 0;
    int computed = 0;               // tokens whose keys / values / state are in the cache
    bool live = false, finished = false, cancelled = false;
    std::string error;
    int admitted_at = -1;           // admission counter: larger = more recent
    int preemptions = 0;

    int total() const { return (int)(prompt.size() + generated.size()); }
    int remaining() const { return total() - computed; }
    int token_at(int index) const {
        return index < (int)prompt.size() ? prompt[index] : generated[index - (int)prompt.size()];
    }
};

struct Segment {
    Request* request;
    int first, count;
    bool wants_logits;
};

struct Event {
    int64_t request;
    int value;
    int kind;
};

struct Plan {
    std::vector<Segment> segments;
    std::vector<Request*> preempted, failed, admitted, cancelled;
    int num_tokens = 0;
    std::unordered_set<int64_t> planned;

    void clear() { *this = Plan(); }
    void add(const Segment& segment) {
        segments.push_back(segment);
        num_tokens += segment.count;
        planned.insert(segment.request->id);
    }
    void drop(const Request* request) {
        if (!planned.count(request->id)) return;
        std::vector<Segment> kept;
        for (const Segment& segment : segments) {
            if (segment.request == request) num_tokens -= segment.count;
            else kept.push_back(segment);
        }
        segments.swap(kept);
        planned.erase(request->id);
    }
    bool has(const Request* request) const { return planned.count(request->id) != 0; }
};

class Scheduler {
public:
    // vocab_size 0: the vocabulary is not known and token ids are not looked at.
    Scheduler(Cache* cache, int max_positions, int max_batch_tokens, int chunk_size, int max_live, int max_queued,
              int vocab_size = 0)
        : cache_(cache), max_positions_(max_positions), max_batch_tokens_(max_batch_tokens), chunk_size_(chunk_size),
          max_queued_(max_queued), vocab_size_(vocab_size) {
        if (max_batch_tokens < 1 || chunk_size < 1) throw SchedulerError("max_batch_tokens and chunk_size must be positive");
        max_live_ = max_live > 0 && max_live < cache->max_requests() ? max_live : cache->max_requests();
    }

    // Validation as the reference's task submit: a prompt, room for prompt + output in the
    // context, a bounded queue; and what its decode refuses token by token
    // (native/src/v2_runtime.cpp:27529-27530), here before the request takes a place: every token
    // id inside the vocabulary, so that no step ever meets one that is not.
    Request* submit(const int* prompt, int prompt_len, int max_new_tokens, const int* stop, int num_stop) {
        if (prompt_len < 1) throw SchedulerError("the prompt is empty");
        if (max_new_tokens < 1) throw SchedulerError("max_tokens must be at least 1");
        if (vocab_size_ > 0) {
            for (int i = 0; i < prompt_len; ++i)
                if (prompt[i] < 0 || prompt[i] >= vocab_size_)
                    throw SchedulerError("token id " + std::to_string(prompt[i]) + " at place " + std::to_string(i) +
                                         " of the prompt is outside the vocabulary (0.." + std::to_string(vocab_size_ - 1) + ")");
            for (int i = 0; i < num_stop; ++i)
                if (stop[i] < 0 || stop[i] >= vocab_size_)
                    throw SchedulerError("stop token " + std::to_string(stop[i]) + " is outside the vocabulary (0.." +
                                         std::to_string(vocab_size_ - 1) + ")");
        }
        if (prompt_len + max_new_tokens > max_positions_)
            throw SchedulerError("prompt (" + std::to_string(prompt_len) + ") + max_tokens (" + std::to_string(max_new_tokens) +
                                 ") exceeds the context of " + std::to_string(max_positions_));
        if ((int)waiting_.size() >= max_queued_)
            throw SchedulerError("the queue holds " + std::to_string(max_queued_) + " requests already");
        auto request = std::make_unique<Request>();
        request->id = next_id_++;
        request->prompt.assign(prompt, prompt + prompt_len);
        request->stop_tokens.assign(stop, stop + num_stop);
        request->max_new_tokens = max_new_tokens;
        Request* raw = request.get();
        requests_[raw->id] = std::move(request);
        waiting_.push_back(raw);
        return raw;
    }
    bool cancel(int64_t id) {
        Request* request = find(id);
        if (!request || request->finished) return false;
        request->cancelled = true;
        return true;
    }
    // A request that cannot go on (the step refused its tokens, or failed while it ran them, so
    // that what the cache holds of it cannot be trusted): it ends with an error, whatever it holds
    // is given back, and it leaves the plan made last, whose other segments stand as they are;
    // its error event comes with that plan's completion. The reference isolates a task's failure
    // the same way (native/src/v2_runtime.cpp:33788-33797). False if it has ended already.
    bool fail_request(int64_t id, const std::string& message) {
        Request* request = find(id);
        if (!request || request->finished) return false;
        plan_.drop(request);
        auto queued = std::find(waiting_.begin(), waiting_.end(), request);
        if (queued != waiting_.end()) waiting_.erase(queued);
        auto listed = [&](std::vector<Request*>& list) {
            list.erase(std::remove(list.begin(), list.end(), request), list.end());
        };
        listed(plan_.preempted);
        listed(plan_.admitted);
        fail(request, message, plan_);
        return true;
    }
    bool has_work() const { return !waiting_.empty() || !running_.empty(); }
    // The next `plans` plans admit nobody: for a caller that has already run those steps on the
    // device, with the requests that were running when it began.
    void hold_admissions(int plans) { held_plans_ = plans > 0 ? plans : 0; }
    // whether a waiting request could be admitted now as far as places go (slots, live requests)
    bool place_for_admission() const {
        return !waiting_.empty() && (int)running_.size() < max_live_ && cache_->slots().free_count() > 0;
    }
    int preemptions() const { return preemptions_; }
    Request* find(int64_t id) {
        auto it = requests_.find(id);
        return it == requests_.end() ? nullptr : it->second.get();
    }
    bool forget(int64_t id) {
        Request* request = find(id);
        if (!request || !request->finished) return false;
        plan_.drop(request);        // the plan made last may still name it
        for (std::vector<Request*>* list : {&plan_.preempted, &plan_.failed, &plan_.admitted, &plan_.cancelled})
            list->erase(std::remove(list->begin(), list->end(), request), list->end());
        requests_.erase(id);
        return true;
    }
    const std::deque<Request*>& waiting() const { return waiting_; }
    const std::vector<Request*>& running() const { return running_; }
    const Plan& plan() const { return plan_; }
    Cache& cache() { return *cache_; }
    int max_positions() const { return max_positions_; }

    const Plan& schedule() {
        // endings whose events no completion has handed out yet (a request failed between two plans)
        std::vector<Request*> failed_before = plan_.failed, cancelled_before = plan_.cancelled;
        plan_.clear();
        Plan& plan = plan_;
        plan.failed = failed_before;
        plan.cancelled = cancelled_before;
        // cancelled requests leave first
        for (Request* request : std::vector<Request*>(running_))
            if (request->cancelled) {
                evict(request);
                request->finished = true;
                plan.cancelled.push_back(request);
            }
        for (Request* request : std::vector<Request*>(waiting_.begin(), waiting_.end()))
            if (request->cancelled) {
                waiting_.erase(std::find(waiting_.begin(), waiting_.end(), request));
                request->finished = true;
                plan.cancelled.push_back(request);
            }
        const bool admit = held_plans_ == 0;
        if (held_plans_ > 0) --held_plans_;
        while (true) {
            plan_once(plan, admit);
            if (!plan.segments.empty() || running_.empty()) return plan;
            // every running request waits for pages and none can move
            if (running_.size() == 1) fail(running_[0], "out of cache pages: the request does not fit even alone", plan);
            else preempt(running_.back(), plan);
        }
    }

    // After the step: `sampled` holds the token drawn from the logits of the last row of every
    // segment that wanted them.
    std::vector<Event> complete(const std::unordered_map<int64_t, int>& sampled) {
        std::vector<Event> events;
        Plan& plan = plan_;
        for (const Segment& segment : plan.segments)       // nothing changes unless every token is there
            if (segment.wants_logits && !sampled.count(segment.request->id))
                throw SchedulerError("no token was handed over for request " + std::to_string(segment.request->id));
        for (Request* request : plan.failed) events.push_back({request->id, 0, EVENT_ERROR});
        for (Request* request : plan.cancelled) events.push_back({request->id, (int)request->generated.size(), EVENT_FINISHED});
        for (const Segment& segment : plan.segments) {
            Request* request = segment.request;
            request->computed += segment.count;
            cache_->commit(request->id, request->computed);
            if (!segment.wants_logits) {
                events.push_back({request->id, request->computed, EVENT_PREFILL});
                continue;
            }
            const int token = sampled.find(request->id)->second;
            request->generated.push_back(token);
            events.push_back({request->id, token, EVENT_TOKEN});
            const bool stop = std::find(request->stop_tokens.begin(), request->stop_tokens.end(), token) != request->stop_tokens.end();
            if (stop || (int)request->generated.size() >= request->max_new_tokens || request->total() >= max_positions_) {
                evict(request);
                request->finished = true;
                events.push_back({request->id, (int)request->generated.size(), EVENT_FINISHED});
            }
        }
        plan.segments.clear();      // a plan is completed once
        plan.failed.clear();
        plan.cancelled.clear();
        return events;
    }

private:
    void evict(Request* request) {
        cache_->release(request->id);
        request->live = false;
        request->computed = 0;
        running_.erase(std::find(running_.begin(), running_.end(), request));
    }
    void fail(Request* request, const std::string& message, Plan& plan) {
        if (request->live) evict(request);
        request->error = message;
        request->finished = true;
        plan.failed.push_back(request);
    }
    void preempt(Request* victim, Plan& plan) {
        plan.drop(victim);
        evict(victim);
        victim->preemptions += 1;
        preemptions_ += 1;
        waiting_.push_front(victim);
        plan.preempted.push_back(victim);
    }

    void plan_once(Plan& plan, bool admit) {
        Cache& cache = *cache_;
        // 1. decode rows, oldest first; make room by preempting the newest
        for (Request* request : std::vector<Request*>(running_)) {
            if (!request->live || request->remaining() != 1 || plan.has(request)) continue;
            if (plan.num_tokens >= max_batch_tokens_) break;
            while (request->live && !cache.fits(request->id, request->computed + 1)) {
                if (running_.size() == 1) fail(request, "out of cache pages: the request does not fit even alone", plan);
                else preempt(running_.back(), plan);      // may be the request itself, if it is the newest
            }
            if (!request->live) continue;
            cache.reserve(request->id, request->computed + 1);
            plan.add({request, request->computed, 1, true});
        }
        // 2. portions of prompts of running requests, oldest first
        for (Request* request : std::vector<Request*>(running_)) {
            if (request->remaining() < 1 || plan.has(request)) continue;
            if (plan.num_tokens >= max_batch_tokens_) break;
            plan_portion(request, plan);
        }
        // 3. admissions, in queue order, while everything a first portion needs is there;
        //    none in a step in which somebody had to give way
        while (admit && !waiting_.empty() && plan.preempted.empty() && plan.num_tokens < max_batch_tokens_ &&
               (int)running_.size() < max_live_ && cache.slots().free_count() > 0) {
            Request* request = waiting_.front();
            const int total = (int)request->prompt.size() + request->max_new_tokens;
            const int limit = std::min(cache.max_pages_per_request(), cache.num_pages());
            if (cache.num_groups() > 0 && cache.pages_for(total) > limit) {
                waiting_.pop_front();
                fail(request, "the request needs " + std::to_string(cache.pages_for(total)) + " cache pages for " +
                                  std::to_string(total) + " tokens; the pool holds " + std::to_string(limit), plan);
                continue;
            }
            const int portion = std::min({request->remaining(), chunk_size_, max_batch_tokens_ - plan.num_tokens});
            bool room = true;
            for (int g = 0; g < cache.num_groups(); ++g)
                if (cache.group(g).pool.free_count() < cache.pages_for(portion)) room = false;
            if (!room) break;
            waiting_.pop_front();
            cache.admit(request->id);
            request->live = true;
            request->admitted_at = admissions_++;
            running_.push_back(request);
            plan.admitted.push_back(request);
            plan_portion(request, plan);
        }
    }

    void plan_portion(Request* request, Plan& plan) {
        Cache& cache = *cache_;
        int portion = std::min({request->remaining(), chunk_size_, max_batch_tokens_ - plan.num_tokens});
        // shrink to what the pool can hold right now; a portion may be cut anywhere
        while (portion >= 1 && !cache.fits(request->id, request->computed + portion)) {
            const int over = (request->computed + portion) % cache.page_size();
            portion -= over ? over : cache.page_size();
        }
        if (portion < 1) return;
        cache.reserve(request->id, request->computed + portion);
        plan.add({request, request->computed, portion, portion == request->remaining()});
    }

    Cache* cache_;
    int max_positions_, max_batch_tokens_, chunk_size_, max_live_, max_queued_, vocab_size_;
    int held_plans_ = 0;
    std::deque<Request*> waiting_;
    std::vector<Request*> running_;         // in admission order, oldest first
    std::unordered_map<int64_t, std::unique_ptr<Request>> requests_;
    Plan plan_;
    int64_t next_id_ = 1;
    int admissions_ = 0, preemptions_ = 0;
};

}  // namespace fwh
