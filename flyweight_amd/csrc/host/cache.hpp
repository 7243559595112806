// The cache's bookkeeping: LIFO pools, block tables per page group, state slots.
// Same operations as the reference's (unwired) paging primitive, native/src/paged_kv.h:133-204
// (pool, ensure / truncate / release), grown by page groups with a window and by slots.
#pragma once
#include <cstdint>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

namespace fwh {

struct OutOfPages : std::runtime_error {
    using std::runtime_error::runtime_error;
};
struct AccountingError : std::logic_error {
    using std::logic_error::logic_error;
};

class Pool {
public:
    explicit Pool(int size) : held_(size, 0) {
        if (size <= 0) throw std::invalid_argument("a pool needs at least one entry");
        free_.reserve(size);
        for (int id = size - 1; id >= 0; --id) free_.push_back(id);      // id 0 is handed out first
    }
    int size() const { return (int)held_.size(); }
    int free_count() const { return (int)free_.size(); }
    int in_use() const { return size() - free_count(); }
    int peak() const { return peak_; }
    bool is_held(int id) const { return id >= 0 && id < size() && held_[id]; }
    int alloc() {
        if (free_.empty()) throw OutOfPages("out of cache pages");
        const int id = free_.back();
        free_.pop_back();
        held_[id] = 1;
        if (in_use() > peak_) peak_ = in_use();
        return id;
    }
    void free(int id) {
        if (!is_held(id)) throw AccountingError("id " + std::to_string(id) + " is freed but not held");
        held_[id] = 0;
        free_.push_back(id);
    }

private:
    std::vector<int> free_;
    std::vector<char> held_;
    int peak_ = 0;
};

constexpr int NO_PAGE = -1;

struct Group {
    int window;                                             // 0: every key is kept
    Pool pool;
    std::unordered_map<int64_t, std::vector<int>> tables;   // request -> page per block (NO_PAGE once given back)
    Group(int window_, int pages) : window(window_), pool(pages) {}
};

struct Live {
    int slot;
    int length = 0;
};

class Cache {
public:
    // pages: one pool size for every group, or one per group (a group that keeps a window of keys
    // needs far fewer pages than one that keeps them all).
    Cache(const std::vector<int>& windows, const std::vector<int>& pages, int max_requests, int page_size, int max_pages_per_request)
        : page_size_(page_size), max_requests_(max_requests), slots_(max_requests) {
        if (pages.size() != 1 && pages.size() != windows.size())
            throw std::invalid_argument("page counts: one for all groups or one per group");
        groups_.reserve(windows.size());
        int largest = 0;
        num_pages_ = 0;
        for (size_t g = 0; g < windows.size() || g < 1; ++g) {
            const int count = pages[pages.size() == 1 ? 0 : g];
            if (page_size <= 0 || count <= 0) throw std::invalid_argument("page size and page count must be positive");
            largest = count > largest ? count : largest;
            // what bounds a sequence: the smallest pool among the groups that keep every key
            const bool keeps_all = g >= windows.size() || windows[g] <= 0;
            if (keeps_all && (num_pages_ == 0 || count < num_pages_)) num_pages_ = count;
            if (g < windows.size()) groups_.emplace_back(windows[g], count);
        }
        if (num_pages_ == 0) num_pages_ = largest;
        max_pages_per_request_ = max_pages_per_request > 0 ? max_pages_per_request : largest;
    }

    int page_size() const { return page_size_; }
    int num_pages() const { return num_pages_; }
    int max_requests() const { return max_requests_; }
    int max_pages_per_request() const { return max_pages_per_request_; }
    int num_groups() const { return (int)groups_.size(); }
    Group& group(int g) { return groups_.at(g); }
    Pool& slots() { return slots_; }
    const std::unordered_map<int64_t, Live>& live() const { return live_; }

    int pages_for(int tokens) const { return (tokens + page_size_ - 1) / page_size_; }

    // Blocks before this one hold only keys the window has passed once the sequence is
    // `length` tokens long (the next query sits at position `length`).
    int first_needed_block(const Group& group, int length) const {
        if (group.window <= 0) return 0;
        const int first_key = length - group.window + 1 > 0 ? length - group.window + 1 : 0;
        return first_key / page_size_;
    }

    bool is_live(int64_t request) const { return live_.count(request) != 0; }
    const Live& of(int64_t request) const {
        auto it = live_.find(request);
        if (it == live_.end()) throw std::out_of_range("request " + std::to_string(request) + " is not live");
        return it->second;
    }

    // pages a reservation up to new_length would take from group g
    int pages_missing(int64_t request, int new_length, int g) const {
        const Group& group = groups_[g];
        auto it = group.tables.find(request);
        const int have = it == group.tables.end() ? 0 : (int)it->second.size();
        const int blocks = pages_for(new_length);
        return blocks > have ? blocks - have : 0;
    }
    bool fits(int64_t request, int new_length) const {
        if (pages_for(new_length) > max_pages_per_request_) return false;
        for (int g = 0; g < num_groups(); ++g)
            if (groups_[g].pool.free_count() < pages_missing(request, new_length, g)) return false;
        return true;
    }
    // free pages of the tightest group
    int free_pages() const {
        int least = 1 << 30;
        for (const Group& group : groups_) least = group.pool.free_count() < least ? group.pool.free_count() : least;
        return least;
    }

    int admit(int64_t request) {
        if (is_live(request)) throw AccountingError("request " + std::to_string(request) + " is already live");
        if (slots_.free_count() == 0) throw OutOfPages("out of request slots");
        const int slot = slots_.alloc();
        live_[request] = Live{slot, 0};
        for (Group& group : groups_) group.tables[request] = {};
        return slot;
    }
    // Maps pages for positions < new_length in every group, or throws and changes nothing.
    void reserve(int64_t request, int new_length) {
        of(request);
        if (pages_for(new_length) > max_pages_per_request_)
            throw OutOfPages("request " + std::to_string(request) + " would need " + std::to_string(pages_for(new_length)) +
                             " pages; a block table holds " + std::to_string(max_pages_per_request_));
        for (int g = 0; g < num_groups(); ++g) {
            const int missing = pages_missing(request, new_length, g);
            if (groups_[g].pool.free_count() < missing)
                throw OutOfPages("out of cache pages: request " + std::to_string(request) + " needs " + std::to_string(missing) +
                                 " more, " + std::to_string(groups_[g].pool.free_count()) + " free");
        }
        for (int g = 0; g < num_groups(); ++g) {
            Group& group = groups_[g];
            std::vector<int>& table = group.tables[request];
            for (int missing = pages_missing(request, new_length, g); missing > 0; --missing) table.push_back(group.pool.alloc());
        }
    }
    // The reservations of a whole step: all of them, or OutOfPages and nothing changed.
    void reserve_batch(const int64_t* requests, const int* new_lengths, int count) {
        std::vector<int> needed(groups_.size(), 0);
        for (int i = 0; i < count; ++i) {
            of(requests[i]);
            if (pages_for(new_lengths[i]) > max_pages_per_request_)
                throw OutOfPages("request " + std::to_string(requests[i]) + " would need " + std::to_string(pages_for(new_lengths[i])) +
                                 " pages; a block table holds " + std::to_string(max_pages_per_request_));
            for (int g = 0; g < num_groups(); ++g) needed[g] += pages_missing(requests[i], new_lengths[i], g);
        }
        for (int g = 0; g < num_groups(); ++g)
            if (groups_[g].pool.free_count() < needed[g])
                throw OutOfPages("out of cache pages: the step needs " + std::to_string(needed[g]) + " more, " +
                                 std::to_string(groups_[g].pool.free_count()) + " free");
        for (int i = 0; i < count; ++i) reserve(requests[i], new_lengths[i]);
    }
    void commit(int64_t request, int new_length) {
        Live& state = live_.at(request);
        if (new_length < state.length) throw std::invalid_argument("a sequence does not shrink");
        state.length = new_length;
        for (Group& group : groups_) {
            std::vector<int>& table = group.tables[request];
            const int passed = first_needed_block(group, new_length);
            for (int block = 0; block < passed && block < (int)table.size(); ++block)
                if (table[block] != NO_PAGE) {
                    group.pool.free(table[block]);
                    table[block] = NO_PAGE;
                }
        }
    }
    // Gives back the pages behind the first token_count tokens in every group, as the reference's
    // truncate_tokens (native/src/paged_kv.h:180-187): reservations that were not used after all, or
    // a sequence cut back. The length becomes token_count if it was longer. A windowed group cannot
    // be cut back to where its window has passed pages already: those keys are gone.
    void truncate(int64_t request, int token_count) {
        Live& state = live_.at(request);
        if (token_count < 0) throw std::invalid_argument("a sequence has no negative length");
        const int keep = pages_for(token_count);
        if (token_count < state.length)
            for (const Group& group : groups_) {
                const std::vector<int>& table = group.tables.at(request);
                for (int block = first_needed_block(group, token_count); block < keep && block < (int)table.size(); ++block)
                    if (table[block] == NO_PAGE)
                        throw std::invalid_argument("request " + std::to_string(request) + " cannot be cut back to " +
                                                    std::to_string(token_count) + " tokens: its window has passed keys it would need");
            }
        for (Group& group : groups_) {
            std::vector<int>& table = group.tables[request];
            while ((int)table.size() > keep) {
                if (table.back() != NO_PAGE) group.pool.free(table.back());
                table.pop_back();
            }
        }
        if (token_count < state.length) state.length = token_count;
    }
    void release(int64_t request) {
        auto it = live_.find(request);
        if (it == live_.end()) throw AccountingError("request " + std::to_string(request) + " is released but not live");
        for (Group& group : groups_) {
            auto table = group.tables.find(request);
            for (int page : table->second)
                if (page != NO_PAGE) group.pool.free(page);
            group.tables.erase(table);
        }
        slots_.free(it->second.slot);
        live_.erase(it);
    }

    // No page lost, none held twice; slots likewise.
    void check() const {
        for (const Group& group : groups_) {
            std::vector<char> seen(group.pool.size(), 0);
            int held = 0;
            for (const auto& entry : group.tables) {
                if (!live_.count(entry.first)) throw AccountingError("block tables and live requests differ");
                for (int page : entry.second) {
                    if (page == NO_PAGE) continue;
                    if (seen[page]) throw AccountingError("a page is held by two block tables");
                    if (!group.pool.is_held(page)) throw AccountingError("a block table holds a page the pool believes free");
                    seen[page] = 1;
                    ++held;
                }
            }
            if (group.tables.size() != live_.size()) throw AccountingError("block tables and live requests differ");
            if (held != group.pool.in_use())
                throw AccountingError(std::to_string(group.pool.in_use()) + " pages are out of the pool but tables hold " +
                                      std::to_string(held));
        }
        std::vector<char> slot_seen(max_requests_, 0);
        for (const auto& entry : live_) {
            if (slot_seen[entry.second.slot] || !slots_.is_held(entry.second.slot)) throw AccountingError("slot accounting is off");
            slot_seen[entry.second.slot] = 1;
        }
        if ((int)live_.size() != slots_.in_use()) throw AccountingError("slot accounting is off");
    }

private:
    int page_size_, num_pages_, max_requests_, max_pages_per_request_;
    std::vector<Group> groups_;
    Pool slots_;
    std::unordered_map<int64_t, Live> live_;
};

}  // namespace fwh
