#include "cache_manager.h"

#include <algorithm>
#include <numeric>

namespace leone::host {

namespace {
std::string text(const char* what, RequestKey request) {
    return "request " + std::to_string(request) + " " + what;
}
}  // namespace

OutOfPages::OutOfPages(int group_, int needed_, int free_)
    : std::runtime_error("cache group " + std::to_string(group_) + " needs " + std::to_string(needed_) +
                         " free pages, has " + std::to_string(free_)),
      group(group_), needed(needed_), free(free_) {}

CacheManager::CacheManager(std::vector<GroupSpec> groups, int max_requests, int max_context)
    : groups_(std::move(groups)), max_requests_(max_requests), max_context_(max_context) {
    if (max_requests <= 0 || max_context <= 0) throw std::invalid_argument("max_requests and max_context must be positive");
    for (const GroupSpec& g : groups_)
        if (g.num_pages <= 0 || g.page_tokens <= 0 || g.window < 0) throw std::invalid_argument("invalid cache group");
    for (const GroupSpec& g : groups_) {
        std::vector<int> pages(g.num_pages);
        for (int i = 0; i < g.num_pages; ++i) pages[i] = g.num_pages - 1 - i;   // page 0 is handed out first
        free_.push_back(std::move(pages));
        refs_.emplace_back(g.num_pages, 0);
        high_water_.push_back(0);
    }
    free_slots_.resize(max_requests);
    for (int i = 0; i < max_requests; ++i) free_slots_[i] = max_requests - 1 - i;
}

int CacheManager::max_blocks(int g) const {
    const int pt = groups_.at(g).page_tokens;
    return (max_context_ + pt - 1) / pt;
}

std::vector<RequestKey> CacheManager::requests() const {
    std::vector<RequestKey> keys;
    for (const auto& kv : requests_) keys.push_back(kv.first);
    std::sort(keys.begin(), keys.end());
    return keys;
}

int CacheManager::shared_pages(int g) const {
    const std::vector<int>& refs = refs_.at(g);
    return static_cast<int>(std::count_if(refs.begin(), refs.end(), [](int r) { return r > 1; }));
}

const CacheManager::Request& CacheManager::get(RequestKey request) const {
    auto found = requests_.find(request);
    if (found == requests_.end()) throw CacheError(text("is not admitted", request));
    return found->second;
}

CacheManager::Request& CacheManager::get(RequestKey request) {
    return const_cast<Request&>(static_cast<const CacheManager*>(this)->get(request));
}

std::vector<int> CacheManager::blocks_to_map(const Request& state, int g, int start, int tokens) const {
    std::vector<int> blocks;
    if (tokens <= 0) return blocks;
    // Every position of the range is written, also in a windowed group: rows of the same step
    // read them.  Blocks that fall behind the window are handed back at commit.
    const int pt = groups_[g].page_tokens;
    const std::vector<int>& table = state.tables[g];
    const int first = start / pt, last = (start + tokens - 1) / pt;
    for (int b = first; b <= last; ++b)
        if (b >= static_cast<int>(table.size()) || table[b] < 0) blocks.push_back(b);
    return blocks;
}

std::vector<int> CacheManager::pages_needed(RequestKey request, int tokens) const {
    const Request& state = get(request);
    std::vector<int> needed(groups_.size());
    for (int g = 0; g < group_count(); ++g)
        needed[g] = static_cast<int>(blocks_to_map(state, g, state.length + state.pending_tokens, tokens).size());
    return needed;
}

int CacheManager::admit(RequestKey request) {
    if (has(request)) throw CacheError(text("is already admitted", request));
    if (free_slots_.empty()) throw OutOfSlots("all " + std::to_string(max_requests_) + " state slots are in use");
    Request state;
    state.slot = free_slots_.back();
    free_slots_.pop_back();
    state.tables.resize(groups_.size());
    state.pending_blocks.resize(groups_.size());
    const int slot = state.slot;
    requests_.emplace(request, std::move(state));
    return slot;
}

int CacheManager::take(int g) {
    const int page = free_[g].back();
    free_[g].pop_back();
    refs_[g][page] = 1;
    return page;
}

void CacheManager::drop(int g, int page) {
    if (refs_[g][page] <= 0)
        throw CacheError("group " + std::to_string(g) + ": page " + std::to_string(page) +
                         " is given back more often than it was taken");
    if (--refs_[g][page] == 0) {
        free_[g].push_back(page);
        if (log_freed_) freed_log_[g].push_back(page);
    }
}

void CacheManager::log_freed(bool on) {
    log_freed_ = on;
    freed_log_.assign(groups_.size(), {});
}

long CacheManager::freed_count(int g) const {
    if (g < 0 || g >= group_count()) throw CacheError("no cache group " + std::to_string(g));
    if (!log_freed_) return 0;
    std::vector<int> pages = freed_log_[g];                               // a page freed twice since is one page
    std::sort(pages.begin(), pages.end());
    return static_cast<long>(std::unique(pages.begin(), pages.end()) - pages.begin());
}

std::vector<int> CacheManager::drain_freed(int g) {
    if (g < 0 || g >= group_count()) throw CacheError("no cache group " + std::to_string(g));
    std::vector<int> out;
    if (log_freed_) out.swap(freed_log_[g]);
    std::sort(out.begin(), out.end());
    out.erase(std::unique(out.begin(), out.end()), out.end());      // a page freed twice since is one page
    return out;
}

int CacheManager::fork(RequestKey parent, RequestKey child, int tokens) {
    const Request& source = get(parent);
    if (source.pending_tokens) throw CacheError(text("has an uncommitted reservation", parent));
    if (has(child)) throw CacheError(text("is already admitted", child));
    const int limit = tokens < 0 ? source.length : std::min(tokens, source.length);
    long unit = 1;
    for (const GroupSpec& g : groups_) unit = std::lcm(unit, static_cast<long>(g.page_tokens));
    const int shared = static_cast<int>(limit / unit * unit);
    std::vector<std::vector<int>> plans;
    for (int gi = 0; gi < group_count(); ++gi) {
        const GroupSpec& g = groups_[gi];
        const int blocks = shared / g.page_tokens;
        const int first = g.window == 0 ? 0 : std::max(0, shared - (g.window - 1)) / g.page_tokens;
        const std::vector<int>& table = source.tables[gi];
        std::vector<int> pages(blocks, -1);
        for (int b = first; b < blocks; ++b) {
            if (b >= static_cast<int>(table.size()) || table[b] < 0)
                throw CacheError("group " + std::to_string(gi) + ": the parent's window has passed block " +
                                 std::to_string(b) + "; fork later tokens");
            pages[b] = table[b];
        }
        plans.push_back(std::move(pages));
    }
    admit(child);
    Request& state = requests_.at(child);
    for (int gi = 0; gi < group_count(); ++gi) {
        for (int page : plans[gi])
            if (page >= 0) ++refs_[gi][page];
        state.tables[gi] = std::move(plans[gi]);
    }
    state.length = shared;
    return shared;
}

void CacheManager::truncate(RequestKey request, int position) {
    Request& state = get(request);
    if (state.pending_tokens) throw CacheError(text("has an uncommitted reservation", request));
    if (position < 0 || position > state.length)
        throw CacheError("cannot truncate request " + std::to_string(request) + " of length " +
                         std::to_string(state.length) + " to " + std::to_string(position));
    for (int gi = 0; gi < group_count(); ++gi) {
        const GroupSpec& g = groups_[gi];
        const std::vector<int>& table = state.tables[gi];
        const int size = static_cast<int>(table.size());
        const int keep = (position + g.page_tokens - 1) / g.page_tokens;
        if (position % g.page_tokens && keep <= size && table[keep - 1] >= 0 && refs_[gi][table[keep - 1]] > 1)
            throw CacheError("group " + std::to_string(gi) + ": the page holding position " + std::to_string(position) +
                             " is shared; truncate to a multiple of " + std::to_string(g.page_tokens));
        if (g.window != 0) {
            const int reach = std::max(0, position - (g.window - 1)) / g.page_tokens;
            for (int b = reach; b < std::min(keep, size); ++b)
                if (table[b] < 0)
                    throw CacheError("group " + std::to_string(gi) + ": keys before position " + std::to_string(position) +
                                     " have left the window; they cannot be brought back by truncation");
        }
    }
    for (int gi = 0; gi < group_count(); ++gi) {
        const GroupSpec& g = groups_[gi];
        std::vector<int>& table = state.tables[gi];
        const int keep = (position + g.page_tokens - 1) / g.page_tokens;
        for (int b = keep; b < static_cast<int>(table.size()); ++b)
            if (table[b] >= 0) drop(gi, table[b]);
        if (keep < static_cast<int>(table.size())) table.resize(keep);
    }
    state.length = position;
}

void CacheManager::reserve(RequestKey request, int tokens) {
    Request& state = get(request);
    if (tokens <= 0) throw CacheError("a reservation must cover at least one token");
    if (state.pending_tokens) throw CacheError(text("already has an uncommitted reservation", request));
    const int start = state.length;
    if (static_cast<long>(start) + tokens > max_context_)
        throw CacheError("request " + std::to_string(request) + ": " + std::to_string(start) + " + " +
                         std::to_string(tokens) + " tokens exceed the context of " + std::to_string(max_context_));
    std::vector<std::vector<int>> plans;
    for (int g = 0; g < group_count(); ++g) {
        std::vector<int> blocks = blocks_to_map(state, g, start, tokens);
        if (static_cast<int>(blocks.size()) > free_pages(g))
            throw OutOfPages(g, static_cast<int>(blocks.size()), free_pages(g));
        plans.push_back(std::move(blocks));
    }
    for (int g = 0; g < group_count(); ++g) {
        std::vector<int>& table = state.tables[g];
        for (int b : plans[g]) {
            if (static_cast<int>(table.size()) <= b) table.resize(b + 1, -1);
            table[b] = take(g);
        }
        state.pending_blocks[g] = std::move(plans[g]);
        high_water_[g] = std::max(high_water_[g], groups_[g].num_pages - free_pages(g));
    }
    state.pending_tokens = tokens;
}

void CacheManager::commit(RequestKey request, int tokens) {
    Request& state = get(request);
    if (!state.pending_tokens) throw CacheError(text("has no reservation to commit", request));
    if (tokens >= 0 && tokens != state.pending_tokens)
        throw CacheError("commit of " + std::to_string(tokens) + " tokens does not match the reservation of " +
                         std::to_string(state.pending_tokens));
    state.length += state.pending_tokens;
    state.pending_tokens = 0;
    for (int gi = 0; gi < group_count(); ++gi) {
        const GroupSpec& g = groups_[gi];
        state.pending_blocks[gi].clear();
        if (g.window == 0) continue;
        // The next query sits at position `length` and reads keys >= length - window + 1.
        const int reach = state.length - (g.window - 1);
        std::vector<int>& table = state.tables[gi];
        const int end = std::min(static_cast<int>(table.size()), std::max(0, reach) / g.page_tokens);
        for (int b = 0; b < end; ++b)
            if (table[b] >= 0) {
                drop(gi, table[b]);
                table[b] = -1;
            }
    }
}

void CacheManager::rollback(RequestKey request) {
    Request& state = get(request);
    for (int g = 0; g < group_count(); ++g) {
        std::vector<int>& table = state.tables[g];
        std::vector<int>& blocks = state.pending_blocks[g];
        for (auto b = blocks.rbegin(); b != blocks.rend(); ++b) {
            drop(g, table[*b]);
            table[*b] = -1;
        }
        const int pt = groups_[g].page_tokens;
        const long covered = static_cast<long>((state.length + pt - 1) / pt) * pt;
        while (!table.empty() && table.back() < 0 && static_cast<long>(table.size()) * pt > covered) table.pop_back();
        blocks.clear();
    }
    state.pending_tokens = 0;
}

void CacheManager::release(RequestKey request) {
    auto found = requests_.find(request);
    if (found == requests_.end()) throw CacheError(text("is not admitted (released twice?)", request));
    Request state = std::move(found->second);
    requests_.erase(found);
    for (int g = 0; g < group_count(); ++g)
        for (int page : state.tables[g])
            if (page >= 0) drop(g, page);
    free_slots_.push_back(state.slot);
}

}  // namespace leone::host
