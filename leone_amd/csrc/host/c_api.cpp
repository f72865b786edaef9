#include "leone_host.h"

#include <algorithm>
#include <exception>
#include <string>
#include <unordered_map>

#include "cache_manager.h"
#include "sampler.h"
#include "scheduler.h"
#include "step_layout.h"

using namespace leone::host;

namespace {

thread_local std::string last_error;
thread_local int shortage[3] = {0, 0, 0};

// Runs `body`; maps what it throws to a code and keeps the message.
template <typename Body>
long guarded(Body&& body) {
    try {
        return body();
    } catch (const OutOfPages& e) {
        shortage[0] = e.group, shortage[1] = e.needed, shortage[2] = e.free;
        last_error = e.what();
        return LEONE_HOST_OUT_OF_PAGES;
    } catch (const OutOfSlots& e) {
        last_error = e.what();
        return LEONE_HOST_OUT_OF_SLOTS;
    } catch (const CacheError& e) {
        last_error = e.what();
        return LEONE_HOST_MISUSE;
    } catch (const SchedulerError& e) {
        last_error = e.what();
        return LEONE_HOST_SCHEDULER;
    } catch (const StepRefused& e) {
        last_error = e.what();
        return LEONE_HOST_STEP_REFUSED;
    } catch (const SamplerFault& e) {
        last_error = e.what();
        return LEONE_HOST_SAMPLER;
    } catch (const std::exception& e) {
        last_error = e.what();
        return LEONE_HOST_INVALID;
    }
}

CacheManager& cache_of(void* handle) {
    if (!handle) throw std::invalid_argument("null cache handle");
    return *static_cast<CacheManager*>(handle);
}
Scheduler& scheduler_of(void* handle) {
    if (!handle) throw std::invalid_argument("null scheduler handle");
    return *static_cast<Scheduler*>(handle);
}

template <typename T, typename U>
int copy_out(const std::vector<T>& from, U* out, int capacity) {
    const int n = static_cast<int>(from.size());
    if (out)
        for (int i = 0; i < std::min(n, capacity); ++i) out[i] = static_cast<U>(from[i]);
    return n;
}

}  // namespace

extern "C" {

const char* leone_host_last_error(void) { return last_error.c_str(); }

void* leone_cache_create(const int* groups, int n_groups, int max_requests, int max_context) {
    void* made = nullptr;
    guarded([&]() -> long {
        if (!groups || n_groups < 0) throw std::invalid_argument("cache groups are missing");
        std::vector<GroupSpec> specs;
        for (int g = 0; g < n_groups; ++g) specs.push_back({groups[3 * g], groups[3 * g + 1], groups[3 * g + 2]});
        made = new CacheManager(std::move(specs), max_requests, max_context);
        return 0;
    });
    return made;
}
void leone_cache_destroy(void* cache) { delete static_cast<CacheManager*>(cache); }

int leone_cache_admit(void* cache, int64_t request) {
    return guarded([&]() -> long { return cache_of(cache).admit(request); });
}
int leone_cache_fork(void* cache, int64_t parent, int64_t child, int tokens) {
    return guarded([&]() -> long { return cache_of(cache).fork(parent, child, tokens); });
}
int leone_cache_truncate(void* cache, int64_t request, int position) {
    return guarded([&]() -> long { cache_of(cache).truncate(request, position); return 0; });
}
int leone_cache_reserve(void* cache, int64_t request, int tokens) {
    return guarded([&]() -> long { cache_of(cache).reserve(request, tokens); return 0; });
}
int leone_cache_commit(void* cache, int64_t request, int tokens) {
    return guarded([&]() -> long { cache_of(cache).commit(request, tokens); return 0; });
}
int leone_cache_rollback(void* cache, int64_t request) {
    return guarded([&]() -> long { cache_of(cache).rollback(request); return 0; });
}
int leone_cache_release(void* cache, int64_t request) {
    return guarded([&]() -> long { cache_of(cache).release(request); return 0; });
}
int leone_cache_has(void* cache, int64_t request) {
    return guarded([&]() -> long { return cache_of(cache).has(request) ? 1 : 0; });
}
int leone_cache_requests(void* cache, int64_t* out, int capacity) {
    return guarded([&]() -> long { return copy_out(cache_of(cache).requests(), out, capacity); });
}
int leone_cache_length(void* cache, int64_t request) {
    return guarded([&]() -> long { return cache_of(cache).length(request); });
}
int leone_cache_pending(void* cache, int64_t request) {
    return guarded([&]() -> long { return cache_of(cache).pending(request); });
}
int leone_cache_slot(void* cache, int64_t request) {
    return guarded([&]() -> long { return cache_of(cache).slot(request); });
}
int leone_cache_table(void* cache, int64_t request, int group, int* out, int capacity) {
    return guarded([&]() -> long { return copy_out(cache_of(cache).table(request, group), out, capacity); });
}
int leone_cache_pages_needed(void* cache, int64_t request, int tokens, int* out) {
    return guarded([&]() -> long {
        const std::vector<int> needed = cache_of(cache).pages_needed(request, tokens);
        return copy_out(needed, out, static_cast<int>(needed.size()));
    });
}
int leone_cache_free_pages(void* cache, int group) {
    return guarded([&]() -> long { return cache_of(cache).free_pages(group); });
}
int leone_cache_free_list(void* cache, int group, int* out, int capacity) {
    return guarded([&]() -> long { return copy_out(cache_of(cache).free_list(group), out, capacity); });
}
int leone_cache_free_slots(void* cache) {
    return guarded([&]() -> long { return cache_of(cache).free_slots(); });
}
int leone_cache_free_slot_list(void* cache, int* out, int capacity) {
    return guarded([&]() -> long { return copy_out(cache_of(cache).free_slot_list(), out, capacity); });
}
int leone_cache_holders(void* cache, int group, int page) {
    return guarded([&]() -> long { return cache_of(cache).holders(group, page); });
}
int leone_cache_shared_pages(void* cache, int group) {
    return guarded([&]() -> long { return cache_of(cache).shared_pages(group); });
}
int leone_cache_high_water(void* cache, int group) {
    return guarded([&]() -> long { return cache_of(cache).pages_high_water(group); });
}
int leone_cache_log_freed(void* cache, int on) {
    return guarded([&]() -> long {
        cache_of(cache).log_freed(on != 0);
        return 0;
    });
}
int leone_cache_drain_freed(void* cache, int group, int* out, int capacity) {
    return guarded([&]() -> long {
        // nothing is taken off the log unless it fits: the size is asked for first, so a caller with too
        // little room loses no page and asks again
        CacheManager& manager = cache_of(cache);
        const long waiting = manager.freed_count(group);
        if (waiting > capacity || (!out && waiting > 0))
            throw CacheError("the freed pages of group " + std::to_string(group) + " need room for " +
                             std::to_string(waiting) + " entries");
        std::vector<int> pages = manager.drain_freed(group);
        for (size_t i = 0; i < pages.size(); ++i) out[i] = pages[i];
        return static_cast<long>(pages.size());
    });
}
int leone_cache_max_blocks(void* cache, int group) {
    return guarded([&]() -> long { return cache_of(cache).max_blocks(group); });
}
void leone_cache_shortage(int* group, int* needed, int* free) {
    if (group) *group = shortage[0];
    if (needed) *needed = shortage[1];
    if (free) *free = shortage[2];
}

void* leone_scheduler_create(void* cache, const int64_t* policy) {
    void* made = nullptr;
    guarded([&]() -> long {
        if (!policy) throw std::invalid_argument("the policy is missing");
        SchedulerPolicy p;
        p.max_live_requests = policy[0];
        p.max_queued_requests = policy[1];
        p.max_step_tokens = policy[2];
        p.prefill_chunk_tokens = policy[3];
        p.max_prompt_tokens = policy[4];
        p.max_output_tokens = policy[5];
        made = new Scheduler(p, cache_of(cache));
        return 0;
    });
    return made;
}
void leone_scheduler_destroy(void* scheduler) { delete static_cast<Scheduler*>(scheduler); }

int leone_scheduler_submit(void* scheduler, int64_t request, const int32_t* prompt, int prompt_tokens,
                           int64_t max_new_tokens, int eos) {
    return guarded([&]() -> long {
        if (prompt_tokens > 0 && !prompt) throw std::invalid_argument("the prompt is missing");
        return static_cast<int>(scheduler_of(scheduler).submit(request, prompt, std::max(prompt_tokens, 0),
                                                               max_new_tokens, eos >= 0, eos));
    });
}
int leone_scheduler_cancel(void* scheduler, int64_t request) {
    return guarded([&]() -> long { return scheduler_of(scheduler).cancel(request) ? 1 : 0; });
}
int leone_scheduler_has_work(void* scheduler) {
    return guarded([&]() -> long { return scheduler_of(scheduler).has_work() ? 1 : 0; });
}

int leone_scheduler_plan(void* scheduler) {
    return guarded([&]() -> long { return static_cast<long>(scheduler_of(scheduler).plan().size()); });
}
int leone_scheduler_planned(void* scheduler, int64_t* requests, int* starts, int* counts, int* samples, int capacity) {
    return guarded([&]() -> long {
        const std::vector<PlannedEntry>& last_plan = scheduler_of(scheduler).planned();
        const int n = static_cast<int>(last_plan.size());
        for (int i = 0; i < std::min(n, capacity); ++i) {
            requests[i] = last_plan[i].request;
            starts[i] = last_plan[i].start;
            counts[i] = last_plan[i].count;
            samples[i] = last_plan[i].sample ? 1 : 0;
        }
        return n;
    });
}
int leone_scheduler_plan_ahead(void* scheduler) {
    return guarded([&]() -> long { return static_cast<long>(scheduler_of(scheduler).plan_ahead().size()); });
}
int leone_scheduler_ahead(void* scheduler, int64_t* requests, int* starts, int* counts, int* samples, int capacity) {
    return guarded([&]() -> long {
        const std::vector<PlannedEntry>& entries = scheduler_of(scheduler).ahead();
        const int n = static_cast<int>(entries.size());
        for (int i = 0; i < std::min(n, capacity); ++i) {
            requests[i] = entries[i].request;
            starts[i] = entries[i].start;
            counts[i] = entries[i].count;
            samples[i] = entries[i].sample ? 1 : 0;
        }
        return n;
    });
}
int leone_scheduler_complete(void* scheduler, const int64_t* requests, const int32_t* tokens, int n) {
    return guarded([&]() -> long {
        std::unordered_map<RequestKey, std::int32_t> sampled;
        for (int i = 0; i < n; ++i) sampled[requests[i]] = tokens[i];
        return scheduler_of(scheduler).complete(sampled);
    });
}
int leone_scheduler_abort(void* scheduler) {
    return guarded([&]() -> long { return scheduler_of(scheduler).abort(); });
}
int leone_scheduler_history(void* scheduler, int64_t request, int32_t* out, int capacity) {
    return guarded([&]() -> long { return copy_out(scheduler_of(scheduler).history(request), out, capacity); });
}
int leone_scheduler_tokens(void* scheduler, int64_t request, int start, int count, int32_t* out) {
    return guarded([&]() -> long {
        const std::vector<std::int32_t>& history = scheduler_of(scheduler).history(request);
        if (start < 0 || count < 0 || static_cast<std::size_t>(start) + count > history.size())
            throw std::invalid_argument("token range out of bounds");
        std::copy(history.begin() + start, history.begin() + start + count, out);
        return count;
    });
}
int leone_scheduler_request_info(void* scheduler, int64_t request, int* prompt_tokens, int* preemptions) {
    return guarded([&]() -> long {
        Scheduler& s = scheduler_of(scheduler);
        if (prompt_tokens) *prompt_tokens = s.prompt_tokens(request);
        if (preemptions) *preemptions = s.preemptions(request);
        return 0;
    });
}
int leone_scheduler_live(void* scheduler, int64_t* out, int capacity) {
    return guarded([&]() -> long { return copy_out(scheduler_of(scheduler).live_requests(), out, capacity); });
}
int leone_scheduler_queued(void* scheduler, int64_t* out, int capacity) {
    return guarded([&]() -> long { return copy_out(scheduler_of(scheduler).queued_requests(), out, capacity); });
}
int leone_scheduler_finished_count(void* scheduler) {
    return guarded([&]() -> long { return static_cast<long>(scheduler_of(scheduler).finished().size()); });
}
int leone_scheduler_finished_info(void* scheduler, int index, int64_t* request, int* reason, int* preemptions,
                                  int* prompt_tokens, int* generated_tokens) {
    return guarded([&]() -> long {
        const Finished& f = scheduler_of(scheduler).finished().at(index);
        *request = f.request;
        *reason = static_cast<int>(f.reason);
        *preemptions = f.preemptions;
        *prompt_tokens = static_cast<int>(f.prompt.size());
        *generated_tokens = static_cast<int>(f.tokens.size());
        return 0;
    });
}
int leone_scheduler_finished_tokens(void* scheduler, int index, int32_t* prompt, int32_t* generated) {
    return guarded([&]() -> long {
        const Finished& f = scheduler_of(scheduler).finished().at(index);
        if (prompt) std::copy(f.prompt.begin(), f.prompt.end(), prompt);
        if (generated) std::copy(f.tokens.begin(), f.tokens.end(), generated);
        return 0;
    });
}
int leone_scheduler_event_count(void* scheduler) {
    return guarded([&]() -> long { return static_cast<long>(scheduler_of(scheduler).events().size()); });
}
int leone_scheduler_events(void* scheduler, int first, int count, int* kinds, int64_t* requests, int* a, int* b, int* c) {
    return guarded([&]() -> long {
        const std::vector<Event>& events = scheduler_of(scheduler).events();
        if (first < 0 || count < 0 || static_cast<std::size_t>(first) + count > events.size())
            throw std::invalid_argument("event range out of bounds");
        for (int i = 0; i < count; ++i) {
            const Event& e = events[first + i];
            kinds[i] = static_cast<int>(e.kind);
            requests[i] = e.request;
            a[i] = e.a, b[i] = e.b, c[i] = e.c;
        }
        return count;
    });
}
void leone_scheduler_stats(void* scheduler, int64_t* out) {
    guarded([&]() -> long {
        const SchedulerStats& s = scheduler_of(scheduler).stats();
        const int64_t values[15] = {s.submitted, s.admitted, s.rejected, s.steps, s.prefill_portions,
                                    s.prefill_tokens, s.decode_rows, s.emitted_tokens, s.finished, s.cancelled,
                                    s.aborted, s.preemptions, s.max_queue_depth, s.max_step_rows, s.max_live};
        std::copy(values, values + 15, out);
        return 0;
    });
}

long leone_step_pack(void* cache, int n_entries, const int64_t* requests, const int* counts, const int* want_counts,
                     const int32_t* tokens, const int32_t* wants, const int* shape, int32_t* out, long capacity,
                     long* sections, int* summary, int* placed) {
    return guarded([&]() -> long {
        const CacheManager& manager = cache_of(cache);
        if (n_entries < 0 || !requests || !counts || !want_counts || !shape || !sections)
            throw std::invalid_argument("step_pack: missing argument");
        std::vector<StepEntryView> entries(n_entries);
        long token_at = 0, want_at = 0;
        for (int i = 0; i < n_entries; ++i) {
            entries[i] = {requests[i], tokens + token_at, counts[i], wants + want_at, want_counts[i]};
            token_at += std::max(counts[i], 0);
            want_at += std::max(want_counts[i], 0);
        }
        // shape: vocabulary, all rows wanted, number of tilings, then (tile_rows, min_rows, group_tiles) of each
        StepShape step_shape{shape[0], shape[1] != 0, {}};
        if (shape[2] < 0 || shape[2] > 16) throw std::invalid_argument("step_pack: at most 16 tilings");
        for (int i = 0; i < shape[2]; ++i) {
            const RowTiling t{shape[3 + 3 * i], shape[4 + 3 * i], shape[5 + 3 * i]};
            if (t.tile_rows <= 0 || t.group_tiles <= 0 || t.min_rows <= 0)
                throw std::invalid_argument("step_pack: tile_rows, min_rows and group_tiles must be positive");
            step_shape.tilings.push_back(t);
        }
        const StepSections layout = step_sections(manager, entries, step_shape);
        std::copy(layout.offsets.begin(), layout.offsets.end(), sections);
        if (!out || capacity < layout.total()) return layout.total();
        std::vector<PlacedEntry> where;
        const StepSummary s = pack_step(manager, entries, step_shape, layout, out, where);
        if (summary) {   // rows, largest position, wanted rows, decode only, then (rows, tiles) of each tiling
            summary[0] = s.rows, summary[1] = s.max_position, summary[2] = s.wanted, summary[3] = s.decode_only ? 1 : 0;
            for (size_t i = 0; i < s.tiled.size(); ++i) summary[4 + 2 * i] = s.tiled[i].rows, summary[5 + 2 * i] = s.tiled[i].tiles;
        }
        if (placed)
            for (int i = 0; i < n_entries; ++i) {
                placed[5 * i] = where[i].given_index, placed[5 * i + 1] = where[i].slot;
                placed[5 * i + 2] = where[i].first_row, placed[5 * i + 3] = where[i].count;
                placed[5 * i + 4] = where[i].start;
            }
        return layout.total();
    });
}

int leone_sample_rows(const float* logits, int rows, int vocab, const double* temperature, const int* stage_counts,
                      const int* stage_kinds, const double* stage_values, const double* uniform, int* tokens) {
    return guarded([&]() -> long {
        if (!logits || !temperature || !stage_counts || !uniform || !tokens || rows <= 0 || vocab <= 0)
            throw std::invalid_argument("sample_rows: missing argument");
        int total = 0;
        for (int r = 0; r < rows; ++r) {
            if (stage_counts[r] < 0) throw std::invalid_argument("sample_rows: negative stage count");
            total += stage_counts[r];
        }
        if (total > 0 && (!stage_kinds || !stage_values)) throw std::invalid_argument("sample_rows: stages are missing");
        std::vector<StageSpec> stages(total);
        for (int i = 0; i < total; ++i) {
            if (stage_kinds[i] < 0 || stage_kinds[i] > 2) throw std::invalid_argument("sample_rows: unknown stage kind");
            stages[i] = {static_cast<Stage>(stage_kinds[i]), stage_values[i]};
        }
        sample_rows(logits, rows, vocab, temperature, stage_counts, stages.data(), uniform, tokens);
        return 0;
    });
}

}  // extern "C"
