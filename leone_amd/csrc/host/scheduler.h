// The scheduler: admission, prompt portions under a token budget, continuous decoding, finishing.
//
// It decides; it runs nothing.  Each plan() yields the entries of one step with their pages already
// reserved; the caller runs them (which commits the cache) and reports the sampled tokens to
// complete().  It needs only the cache manager, so its decisions can be tested without a GPU.
//
// Kept from the reference's scheduler (crates/leone/src/scheduler.rs): typed admission rejects with
// nothing reserved on rejection (:99-110, :587-636); one budget per request and step, a prompt
// portion of at most prefill_chunk_tokens or one decoded token (:341-378); a request is finished on
// its end token or when its output budget is used up, and what it holds is released at once
// (:445-448, :1341-1343); cancellation of a queued request is immediate, of a running one at the
// next step boundary (:540-554); an executor error aborts the whole batch (:520-538,
// crates/leone/src/service.rs:270-297); counters (:171-192).
//
// What differs: the reference reserves a request's whole lifetime of cache at admission, so it never
// runs out in flight (:652-667).  Here pages are taken as tokens arrive.  When a decode row cannot
// get a page, the most recently admitted live request is preempted: everything it holds is released
// and it goes back to the head of the queue with its generated tokens appended to its prompt, to be
// recomputed (the reference's replay of a token checkpoint as prefill,
// crates/leone/src/runtime.rs:699-716).  Sampling draws are keyed by absolute position, so the
// continuation is unchanged.  A prompt portion that does not fit is shortened to the free pages or
// waits; it never preempts.
#pragma once

#include <cstdint>
#include <deque>
#include <memory>
#include <stdexcept>
#include <unordered_map>
#include <vector>

#include "cache_manager.h"

namespace leone::host {

enum class Reject : int {
    None = 0,
    PromptLimit,    // empty, or longer than the policy allows
    OutputLimit,    // zero, or more than the policy allows
    ContextLimit,   // prompt + output - 1 exceeds the model's context
    KvCapacity,     // could never fit the page pool, even alone
    QueueLimit,
    Duplicate,
};

enum class FinishReason : int { Eos = 0, Length, Cancelled, Aborted };

struct SchedulerError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct SchedulerPolicy {
    std::int64_t max_live_requests = 64;
    std::int64_t max_queued_requests = 1024;
    std::int64_t max_step_tokens = 2048;        // token budget of one step (decode rows + prompt portions)
    std::int64_t prefill_chunk_tokens = 512;    // longest prompt portion of one request in one step
    std::int64_t max_prompt_tokens = 1 << 30;
    std::int64_t max_output_tokens = 1 << 30;
    void validate() const;
};

struct PlannedEntry {
    RequestKey request;
    int start;      // absolute position of the first token
    int count;      // the tokens are the request's history [start, start + count)
    bool sample;    // the portion ends the known tokens: its last row's logits are wanted
};

struct Finished {
    RequestKey request;
    std::vector<std::int32_t> prompt;
    std::vector<std::int32_t> tokens;   // generated
    FinishReason reason;
    int preemptions;
};

struct SchedulerStats {
    std::int64_t submitted = 0, admitted = 0, rejected = 0, steps = 0, prefill_portions = 0, prefill_tokens = 0,
                 decode_rows = 0, emitted_tokens = 0, finished = 0, cancelled = 0, aborted = 0, preemptions = 0,
                 max_queue_depth = 0, max_step_rows = 0, max_live = 0;
};

// One record of the decision log.  A step is a StepBegin record (a = number of entries) followed by
// that many StepEntry records (a = start, b = count, c = sample).  Submit: a = prompt tokens, b = most new
// tokens; Reject: a = reason; Preempt: a = tokens known; Token: a = position of the row that gave it,
// b = token; Finish: a = reason.
// A StepAhead record is a StepBegin for a step planned beyond one whose tokens are not known yet.
enum class EventKind : int { Reject = 0, Submit, StepBegin, StepEntry, Admit, Preempt, Token, Finish, StepAhead };
struct Event {
    EventKind kind;
    RequestKey request;
    int a, b, c;
};

class Scheduler {
public:
    Scheduler(const SchedulerPolicy& policy, CacheManager& cache);

    // Queues a request, or says why not.  A rejected request holds nothing.
    Reject submit(RequestKey request, const std::int32_t* prompt, int prompt_tokens, std::int64_t max_new_tokens,
                  bool has_eos, std::int32_t eos);
    // A queued request goes at once; a live one at the next step boundary.
    bool cancel(RequestKey request);
    bool has_work() const { return !queue_.empty() || !live_.empty(); }
    // Decides the next step and reserves its pages.  Empty only if there is nothing to do.
    const std::vector<PlannedEntry>& plan();
    // One step beyond the planned one, before that one's tokens are known: every request of the planned step
    // once more, one row each at its next position, in the planned step's order, pages reserved.  The caller
    // feeds the rows the tokens the planned step is still choosing (they never leave the device) and so has
    // the next step running while it reads and reports the planned step's tokens.  Possible only where the
    // next step is known without those tokens: the planned step ran and is committed, every live request is
    // in it and gets a token from it, none of them uses up its output budget with that token, none is
    // cancelled, nobody waits in the queue for a place that is free, and every request finds its page.
    // Otherwise nothing is reserved and the answer is empty: complete the planned step first, as always.  A
    // request that ends on the planned step's token after all (its end token) simply drops out of the step
    // ahead: its row there is run for nothing and what it wrote goes back with everything else it holds.
    const std::vector<PlannedEntry>& plan_ahead();
    // The planned step ran and its cache writes are committed.  `sampled` holds a token for every entry
    // planned with `sample`.  Returns how many requests finished; they are the last of finished().  A step
    // planned ahead becomes the planned step (without the requests that have just finished).
    int complete(const std::unordered_map<RequestKey, std::int32_t>& sampled);
    // The planned step failed (or the one ahead of it): every request in them ends as aborted and gives back
    // what it holds.
    int abort();

    // The entries of the step that is planned and not yet completed or aborted (empty otherwise).
    const std::vector<PlannedEntry>& planned() const { return planned_; }
    // The entries of the step planned beyond it (empty if there is none).
    const std::vector<PlannedEntry>& ahead() const { return ahead_; }
    const std::vector<Finished>& finished() const { return finished_; }
    const std::vector<Event>& events() const { return events_; }
    const SchedulerStats& stats() const { return stats_; }
    const SchedulerPolicy& policy() const { return policy_; }
    std::vector<RequestKey> live_requests() const;      // oldest first
    std::vector<RequestKey> queued_requests() const;    // head of the queue first
    // The whole known history of a live or queued request: prompt, then generated tokens.
    const std::vector<std::int32_t>& history(RequestKey request) const;
    int prompt_tokens(RequestKey request) const;
    int preemptions(RequestKey request) const;

private:
    struct Live {
        RequestKey request;
        std::vector<std::int32_t> tokens;   // prompt, then generated tokens
        int prompt_len;
        std::int64_t max_new_tokens;
        bool has_eos;
        std::int32_t eos;
        std::int64_t order;
        bool cancelled = false;
        int preemptions = 0;
    };
    using LivePtr = std::shared_ptr<Live>;

    Reject reject_reason(RequestKey request, int prompt, std::int64_t out) const;
    std::vector<PlannedEntry> plan_once();
    int reserve_portion(const Live& state, int wanted);
    bool room_for(int tokens) const;
    bool fits(RequestKey request, int tokens) const;
    LivePtr newest() const;
    void preempt(const LivePtr& victim, std::vector<PlannedEntry>& planned);
    void finish(const LivePtr& state, FinishReason reason, bool held);
    const Live& find(RequestKey request) const;

    SchedulerPolicy policy_;
    CacheManager& cache_;
    std::deque<LivePtr> queue_;
    std::unordered_map<RequestKey, LivePtr> live_;
    std::vector<Finished> finished_;
    std::vector<Event> events_;
    SchedulerStats stats_;
    std::int64_t order_ = 0;
    bool planned_valid_ = false;
    std::vector<PlannedEntry> planned_;
    bool ahead_valid_ = false;
    std::vector<PlannedEntry> ahead_;
};

}  // namespace leone::host
