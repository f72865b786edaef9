#include "scheduler.h"

#include <algorithm>
#include <string>

namespace leone::host {

void SchedulerPolicy::validate() const {
    const std::pair<const char*, std::int64_t> fields[] = {
        {"max_live_requests", max_live_requests},   {"max_queued_requests", max_queued_requests},
        {"max_step_tokens", max_step_tokens},       {"prefill_chunk_tokens", prefill_chunk_tokens},
        {"max_prompt_tokens", max_prompt_tokens},   {"max_output_tokens", max_output_tokens}};
    for (const auto& f : fields)
        if (f.second <= 0) throw SchedulerError(std::string("policy: ") + f.first + " must be positive");
}

Scheduler::Scheduler(const SchedulerPolicy& policy, CacheManager& cache) : policy_(policy), cache_(cache) {
    policy_.validate();
}

// ---- admission

Reject Scheduler::submit(RequestKey request, const std::int32_t* prompt, int prompt_tokens,
                         std::int64_t max_new_tokens, bool has_eos, std::int32_t eos) {
    ++stats_.submitted;
    const Reject reason = reject_reason(request, prompt_tokens, max_new_tokens);
    if (reason != Reject::None) {
        ++stats_.rejected;
        events_.push_back({EventKind::Reject, request, static_cast<int>(reason), 0, 0});
        return reason;
    }
    auto state = std::make_shared<Live>();
    state->request = request;
    state->tokens.assign(prompt, prompt + prompt_tokens);
    state->prompt_len = prompt_tokens;
    state->max_new_tokens = max_new_tokens;
    state->has_eos = has_eos;
    state->eos = eos;
    state->order = ++order_;
    queue_.push_back(std::move(state));
    stats_.max_queue_depth = std::max<std::int64_t>(stats_.max_queue_depth, queue_.size());
    events_.push_back({EventKind::Submit, request, prompt_tokens,
                       static_cast<int>(std::min<std::int64_t>(max_new_tokens, 0x7fffffff)), 0});
    return Reject::None;
}

Reject Scheduler::reject_reason(RequestKey request, int prompt, std::int64_t out) const {
    if (live_.count(request)) return Reject::Duplicate;
    for (const LivePtr& q : queue_)
        if (q->request == request) return Reject::Duplicate;
    if (prompt <= 0 || prompt > policy_.max_prompt_tokens) return Reject::PromptLimit;
    if (out <= 0 || out > policy_.max_output_tokens) return Reject::OutputLimit;
    // The last generated token is never fed back, so the cache holds prompt + out - 1 tokens
    // (crates/leone/src/runtime.rs:3597-3615).
    const std::int64_t held = prompt + out - 1;
    if (held > cache_.max_context()) return Reject::ContextLimit;
    for (int gi = 0; gi < cache_.group_count(); ++gi) {
        const GroupSpec& g = cache_.group(gi);
        std::int64_t need;
        if (g.window == 0) {
            need = (held + g.page_tokens - 1) / g.page_tokens;
        } else {
            const std::int64_t portion = std::min(policy_.prefill_chunk_tokens, policy_.max_step_tokens);
            const std::int64_t span = std::min<std::int64_t>(held, g.window - 1 + portion);
            need = (span + g.page_tokens - 1) / g.page_tokens + 1;
        }
        if (need > g.num_pages) return Reject::KvCapacity;
    }
    if (static_cast<std::int64_t>(queue_.size()) >= policy_.max_queued_requests) return Reject::QueueLimit;
    return Reject::None;
}

bool Scheduler::cancel(RequestKey request) {
    for (auto it = queue_.begin(); it != queue_.end(); ++it)
        if ((*it)->request == request) {
            LivePtr state = *it;
            queue_.erase(it);
            finish(state, FinishReason::Cancelled, false);
            return true;
        }
    auto found = live_.find(request);
    if (found == live_.end()) return false;
    found->second->cancelled = true;
    return true;
}

// ---- planning

const std::vector<PlannedEntry>& Scheduler::plan() {
    if (planned_valid_) throw SchedulerError("the previous step was neither completed nor aborted");
    std::vector<LivePtr> gone;   // (a step planned ahead became the planned step when the one before it was completed)
    for (const auto& kv : live_)
        if (kv.second->cancelled) gone.push_back(kv.second);
    std::sort(gone.begin(), gone.end(), [](const LivePtr& a, const LivePtr& b) { return a->order < b->order; });
    for (const LivePtr& state : gone) finish(state, FinishReason::Cancelled, true);

    std::vector<PlannedEntry> entries;
    const std::size_t rounds = live_.size() + queue_.size() + 1;
    for (std::size_t round = 0; round < rounds; ++round) {
        entries = plan_once();
        if (!entries.empty() || live_.empty()) break;
        // Every live request waits for pages that only another live request could free.
        std::vector<PlannedEntry> none;
        preempt(newest(), none);
    }
    if (entries.empty() && has_work()) throw SchedulerError("no request can make progress");
    planned_ = std::move(entries);
    planned_valid_ = true;
    if (!planned_.empty()) {
        ++stats_.steps;
        std::int64_t rows = 0;
        for (const PlannedEntry& e : planned_) rows += e.count;
        stats_.max_step_rows = std::max(stats_.max_step_rows, rows);
        events_.push_back({EventKind::StepBegin, 0, static_cast<int>(planned_.size()), 0, 0});
        for (const PlannedEntry& e : planned_)
            events_.push_back({EventKind::StepEntry, e.request, e.start, e.count, e.sample ? 1 : 0});
    }
    return planned_;
}

const std::vector<PlannedEntry>& Scheduler::plan_ahead() {
    if (!planned_valid_) throw SchedulerError("no step is planned to look beyond");
    if (ahead_valid_) throw SchedulerError("a step ahead is planned already");
    ahead_.clear();
    if (planned_.empty() || planned_.size() != live_.size() ||
        static_cast<std::int64_t>(planned_.size()) > policy_.max_step_tokens)
        return ahead_;
    // somebody could be admitted into the next step: then it is not this step's rows once more
    if (!queue_.empty() && static_cast<std::int64_t>(live_.size()) < policy_.max_live_requests && cache_.free_slots() > 0)
        return ahead_;
    for (const PlannedEntry& entry : planned_) {
        const Live& state = *live_.at(entry.request);
        if (!entry.sample || state.cancelled) return ahead_;
        const std::int64_t generated = static_cast<std::int64_t>(state.tokens.size()) - state.prompt_len + 1;
        if (generated >= state.max_new_tokens) return ahead_;           // this step's token is its last
        if (cache_.length(entry.request) != entry.start + entry.count)
            throw SchedulerError("request " + std::to_string(entry.request) +
                                 ": the planned step has not run; there is nothing to look beyond yet");
    }
    std::vector<PlannedEntry> entries;
    for (const PlannedEntry& entry : planned_) {
        try {
            cache_.reserve(entry.request, 1);
        } catch (const std::runtime_error&) {    // no page (a preemption is the planned way's affair), or the context's end
            for (const PlannedEntry& held : entries) cache_.rollback(held.request);
            return ahead_;
        }
        entries.push_back({entry.request, entry.start + entry.count, 1, true});
    }
    ahead_ = std::move(entries);
    ahead_valid_ = true;
    ++stats_.steps;
    stats_.decode_rows += static_cast<std::int64_t>(ahead_.size());
    stats_.max_step_rows = std::max<std::int64_t>(stats_.max_step_rows, ahead_.size());
    events_.push_back({EventKind::StepAhead, 0, static_cast<int>(ahead_.size()), 0, 0});
    for (const PlannedEntry& e : ahead_) events_.push_back({EventKind::StepEntry, e.request, e.start, e.count, 1});
    return ahead_;
}

Scheduler::LivePtr Scheduler::newest() const {
    LivePtr best;
    for (const auto& kv : live_)
        if (!best || kv.second->order > best->order) best = kv.second;
    return best;
}

std::vector<PlannedEntry> Scheduler::plan_once() {
    std::vector<PlannedEntry> entries;
    std::int64_t budget = policy_.max_step_tokens;
    std::vector<LivePtr> by_age;
    for (const auto& kv : live_) by_age.push_back(kv.second);
    std::sort(by_age.begin(), by_age.end(), [](const LivePtr& a, const LivePtr& b) { return a->order < b->order; });

    // 1. one token for every request that is decoding, oldest first
    for (const LivePtr& state : by_age) {
        if (budget == 0) break;
        if (!live_.count(state->request)) continue;   // preempted a moment ago
        const int cached = cache_.length(state->request);
        if (static_cast<int>(state->tokens.size()) - cached != 1) continue;
        while (true) {
            try {
                cache_.reserve(state->request, 1);
            } catch (const OutOfPages&) {
                LivePtr victim = newest();
                preempt(victim, entries);
                if (victim == state) break;
                continue;
            }
            entries.push_back({state->request, cached, 1, true});
            --budget;
            ++stats_.decode_rows;
            break;
        }
    }
    // 2. prompt portions for the live requests that still have some, oldest first
    bool starved = false;
    for (const LivePtr& state : by_age) {
        if (budget == 0 || starved) break;
        if (!live_.count(state->request)) continue;
        const int cached = cache_.length(state->request);
        const int remaining = static_cast<int>(state->tokens.size()) - cached;
        if (remaining <= 1) continue;
        const int wanted = static_cast<int>(std::min<std::int64_t>({remaining, policy_.prefill_chunk_tokens, budget}));
        const int taken = reserve_portion(*state, wanted);
        if (taken == 0) {
            starved = true;   // younger requests must not take the pages an older one waits for
            break;
        }
        entries.push_back({state->request, cached, taken, taken == remaining});
        budget -= taken;
        ++stats_.prefill_portions;
        stats_.prefill_tokens += taken;
    }
    // 3. admit from the queue
    while (!queue_.empty() && !starved && budget > 0 &&
           static_cast<std::int64_t>(live_.size()) < policy_.max_live_requests && cache_.free_slots() > 0) {
        LivePtr state = queue_.front();
        const int remaining = static_cast<int>(state->tokens.size());
        // Admit only when the pages for everything the request already holds are free now, so that a
        // request just preempted is not taken back in only to be preempted again.
        if (!live_.empty() && !room_for(remaining)) break;
        cache_.admit(state->request);
        const int wanted = static_cast<int>(std::min<std::int64_t>({remaining, policy_.prefill_chunk_tokens, budget}));
        const int taken = reserve_portion(*state, wanted);
        if (taken == 0) {
            cache_.release(state->request);
            break;
        }
        queue_.pop_front();
        live_[state->request] = state;
        ++stats_.admitted;
        stats_.max_live = std::max<std::int64_t>(stats_.max_live, live_.size());
        events_.push_back({EventKind::Admit, state->request, 0, 0, 0});
        entries.push_back({state->request, 0, taken, taken == remaining});
        budget -= taken;
        if (remaining > 1 || taken > 1) {
            ++stats_.prefill_portions;
            stats_.prefill_tokens += taken;
        } else {
            ++stats_.decode_rows;
        }
    }
    return entries;
}

int Scheduler::reserve_portion(const Live& state, int wanted) {
    int n = wanted;
    while (n > 0) {
        try {
            cache_.reserve(state.request, n);
            return n;
        } catch (const OutOfPages&) {
            int lo = 0, hi = n - 1;   // the largest count whose pages are free
            while (lo < hi) {
                const int mid = (lo + hi + 1) / 2;
                if (fits(state.request, mid)) lo = mid; else hi = mid - 1;
            }
            n = lo;
        }
    }
    return 0;
}

bool Scheduler::room_for(int tokens) const {
    for (int gi = 0; gi < cache_.group_count(); ++gi) {
        const GroupSpec& g = cache_.group(gi);
        const std::int64_t span =
            g.window == 0 ? tokens : std::min<std::int64_t>(tokens, g.window - 1 + policy_.prefill_chunk_tokens);
        if ((span + g.page_tokens - 1) / g.page_tokens > cache_.free_pages(gi)) return false;
    }
    return true;
}

bool Scheduler::fits(RequestKey request, int tokens) const {
    if (tokens == 0) return true;
    const std::vector<int> needed = cache_.pages_needed(request, tokens);
    for (int g = 0; g < cache_.group_count(); ++g)
        if (needed[g] > cache_.free_pages(g)) return false;
    return true;
}

void Scheduler::preempt(const LivePtr& victim, std::vector<PlannedEntry>& planned) {
    const RequestKey request = victim->request;
    planned.erase(std::remove_if(planned.begin(), planned.end(),
                                 [request](const PlannedEntry& e) { return e.request == request; }),
                  planned.end());
    cache_.rollback(request);
    cache_.release(request);
    live_.erase(request);
    ++victim->preemptions;
    queue_.push_front(victim);
    ++stats_.preemptions;
    events_.push_back({EventKind::Preempt, request, static_cast<int>(victim->tokens.size()), 0, 0});
}

// ---- after the step

int Scheduler::complete(const std::unordered_map<RequestKey, std::int32_t>& sampled) {
    if (!planned_valid_) throw SchedulerError("no step is planned");
    // Check everything before anything changes, so that a refused call leaves the step planned.
    for (const PlannedEntry& entry : planned_) {
        const int held = cache_.length(entry.request);           // a step ahead that ran has added its one token
        if (held != entry.start + entry.count && !(ahead_valid_ && held == entry.start + entry.count + 1))
            throw SchedulerError("request " + std::to_string(entry.request) + ": the step was not committed to the cache");
        if (entry.sample && !sampled.count(entry.request))
            throw SchedulerError("request " + std::to_string(entry.request) + ": the step returned no token");
    }
    std::vector<PlannedEntry> planned = std::move(planned_);
    planned_.clear();
    planned_valid_ = false;
    int done = 0;
    for (const PlannedEntry& entry : planned) {
        if (!entry.sample) continue;
        LivePtr state = live_.at(entry.request);
        const std::int32_t token = sampled.at(entry.request);
        state->tokens.push_back(token);
        ++stats_.emitted_tokens;
        events_.push_back({EventKind::Token, entry.request, entry.start + entry.count - 1, token, 0});
        const std::int64_t generated = static_cast<std::int64_t>(state->tokens.size()) - state->prompt_len;
        if (state->has_eos && token == state->eos) {
            finish(state, FinishReason::Eos, true);
            ++done;
        } else if (generated >= state->max_new_tokens) {
            finish(state, FinishReason::Length, true);
            ++done;
        }
    }
    if (ahead_valid_) {
        // The step ahead is the planned step now; a request that has just ended is no longer in it (what its
        // row there wrote went back with everything else it held).
        for (const PlannedEntry& entry : ahead_)
            if (live_.count(entry.request)) planned_.push_back(entry);
        ahead_.clear();
        ahead_valid_ = false;
        planned_valid_ = !planned_.empty();
    }
    return done;
}

int Scheduler::abort() {
    if (!planned_valid_) throw SchedulerError("no step is planned");
    std::vector<PlannedEntry> planned = std::move(planned_);
    planned_.clear();
    planned_valid_ = false;
    ahead_.clear();                     // its requests are the planned step's: they go with them
    ahead_valid_ = false;
    for (const PlannedEntry& entry : planned) {
        LivePtr state = live_.at(entry.request);
        cache_.rollback(entry.request);
        finish(state, FinishReason::Aborted, true);
    }
    return static_cast<int>(planned.size());
}

void Scheduler::finish(const LivePtr& state, FinishReason reason, bool held) {
    if (held) {
        cache_.release(state->request);
        live_.erase(state->request);
    }
    Finished record;
    record.request = state->request;
    record.prompt.assign(state->tokens.begin(), state->tokens.begin() + state->prompt_len);
    record.tokens.assign(state->tokens.begin() + state->prompt_len, state->tokens.end());
    record.reason = reason;
    record.preemptions = state->preemptions;
    finished_.push_back(std::move(record));
    if (reason == FinishReason::Cancelled) ++stats_.cancelled;
    else if (reason == FinishReason::Aborted) ++stats_.aborted;
    else ++stats_.finished;
    events_.push_back({EventKind::Finish, state->request, static_cast<int>(reason), 0, 0});
}

// ---- views

std::vector<RequestKey> Scheduler::live_requests() const {
    std::vector<LivePtr> states;
    for (const auto& kv : live_) states.push_back(kv.second);
    std::sort(states.begin(), states.end(), [](const LivePtr& a, const LivePtr& b) { return a->order < b->order; });
    std::vector<RequestKey> keys;
    for (const LivePtr& s : states) keys.push_back(s->request);
    return keys;
}

std::vector<RequestKey> Scheduler::queued_requests() const {
    std::vector<RequestKey> keys;
    for (const LivePtr& s : queue_) keys.push_back(s->request);
    return keys;
}

const Scheduler::Live& Scheduler::find(RequestKey request) const {
    auto found = live_.find(request);
    if (found != live_.end()) return *found->second;
    for (const LivePtr& s : queue_)
        if (s->request == request) return *s;
    throw SchedulerError("request " + std::to_string(request) + " is neither live nor queued");
}

const std::vector<std::int32_t>& Scheduler::history(RequestKey request) const { return find(request).tokens; }
int Scheduler::prompt_tokens(RequestKey request) const { return find(request).prompt_len; }
int Scheduler::preemptions(RequestKey request) const { return find(request).preemptions; }

}  // namespace leone::host
