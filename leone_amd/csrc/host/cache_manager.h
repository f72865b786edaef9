// The cache manager: pages, block tables and state slots.  Host side only; it owns no device memory.
//
// The reference keeps a request's keys and values in growable segments and stages every append as a
// transaction: prepare_append reserves room, kernels write only there, commit_append makes it
// visible, any error rolls back exactly (crates/leone/src/kv.rs:326-370, 856-927).  The same
// contract is kept here over fixed-size pages:
//
//   * a group is a set of layers with the same cache need; it has its own pages, free list and one
//     block table per request (logical block -> page id, -1 where no page is mapped);
//   * reserve maps pages for the positions a step is about to write, in every group, all or
//     nothing; commit advances the request's length and, for a windowed group, hands back pages
//     that no later query can reach; rollback undoes an uncommitted reservation; release returns
//     everything a request holds, pages and state slot, at once;
//   * a state slot is an index into per-request storage of fixed size, handed out on admission
//     and returned on release;
//   * fork lets a new request share the full pages of another request's prefix (the reference's
//     fork shares committed, immutable segments and gives the writer a private tail,
//     crates/leone/src/kv.rs:307-324, 676-691): pages carry reference counts, a page goes back to
//     the free list when its last holder lets go, and a shared page is never written because
//     sharing stops at a page boundary; truncate cuts a request back (crates/leone/src/kv.rs:929-950).
#pragma once

#include <cstdint>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

namespace leone::host {

using RequestKey = std::int64_t;

struct GroupSpec {
    int num_pages;
    int page_tokens;
    int window;   // 0: every position is kept; otherwise only the last `window`
};

// A reservation needs more free pages than a group has; nothing was changed.
struct OutOfPages : std::runtime_error {
    OutOfPages(int group, int needed, int free);
    int group, needed, free;
};

// Every per-request state slot is taken.
struct OutOfSlots : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// The manager was used against its contract (unknown request, double free, ...).
struct CacheError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

class CacheManager {
public:
    CacheManager(std::vector<GroupSpec> groups, int max_requests, int max_context);

    // ---- queries
    int group_count() const { return static_cast<int>(groups_.size()); }
    const GroupSpec& group(int g) const { return groups_.at(g); }
    int max_requests() const { return max_requests_; }
    int max_context() const { return max_context_; }
    int max_blocks(int g) const;
    bool has(RequestKey request) const { return requests_.count(request) != 0; }
    std::vector<RequestKey> requests() const;   // every admitted request, ascending
    int length(RequestKey request) const { return get(request).length; }
    int pending(RequestKey request) const { return get(request).pending_tokens; }
    int slot(RequestKey request) const { return get(request).slot; }
    const std::vector<int>& table(RequestKey request, int g) const { return get(request).tables.at(g); }
    int free_pages(int g) const { return static_cast<int>(free_.at(g).size()); }
    const std::vector<int>& free_list(int g) const { return free_.at(g); }
    int free_slots() const { return static_cast<int>(free_slots_.size()); }
    const std::vector<int>& free_slot_list() const { return free_slots_; }
    int holders(int g, int page) const { return refs_.at(g).at(page); }
    int shared_pages(int g) const;
    int pages_high_water(int g) const { return high_water_.at(g); }
    // With the log switched on, every page whose last holder lets go is noted (whoever frees it: release,
    // a window that has passed, a rollback, a truncation); drain_freed hands the notes out and clears them.
    // For a caller that wants to overwrite what freed pages hold before anyone gets them again.
    void log_freed(bool on);
    std::vector<int> drain_freed(int g);
    long freed_count(int g) const;      // how many pages the next drain_freed will hand out

    // New pages each group must map to append `tokens` to `request` now.
    std::vector<int> pages_needed(RequestKey request, int tokens) const;

    // ---- life cycle
    int admit(RequestKey request);
    // Admits `child` holding the full pages of the first `tokens` tokens of `parent` (all it has
    // committed if negative).  Returns how many tokens the child holds: `tokens` rounded down to a
    // page boundary of every group; what lies beyond, the child computes for itself.
    int fork(RequestKey parent, RequestKey child, int tokens);
    // Cuts a request back to `position` tokens.  Pages wholly beyond go back; the page that holds
    // `position` stays and must be the request's own unless `position` is a page boundary.
    void truncate(RequestKey request, int position);
    // Maps pages so that positions [length, length + tokens) can be written.  All groups or none.
    void reserve(RequestKey request, int tokens);
    // The reserved positions now hold data (`tokens` negative: whatever was reserved).
    void commit(RequestKey request, int tokens);
    // Undoes an uncommitted reservation exactly.
    void rollback(RequestKey request);
    // Returns every page and the state slot of a request (finished, cancelled or preempted).
    void release(RequestKey request);

private:
    struct Request {
        int slot = 0;
        int length = 0;           // committed tokens
        int pending_tokens = 0;
        std::vector<std::vector<int>> tables;           // per group: block -> page, -1 unmapped
        std::vector<std::vector<int>> pending_blocks;   // per group: blocks mapped by the open reservation
    };

    const Request& get(RequestKey request) const;
    Request& get(RequestKey request);
    int take(int g);
    void drop(int g, int page);
    std::vector<int> blocks_to_map(const Request& state, int g, int start, int tokens) const;

    std::vector<GroupSpec> groups_;
    int max_requests_;
    int max_context_;
    std::vector<std::vector<int>> free_;    // LIFO: a page given back is the next one handed out
    std::vector<int> free_slots_;
    std::vector<std::vector<int>> refs_;    // holders of every page
    std::vector<int> high_water_;
    bool log_freed_ = false;
    std::vector<std::vector<int>> freed_log_;
    std::unordered_map<RequestKey, Request> requests_;
};

}  // namespace leone::host
