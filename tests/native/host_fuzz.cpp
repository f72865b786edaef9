// Random workloads through the host library's C interface: requests are submitted, steps planned, laid
// out, committed, now and then aborted or cancelled, under few pages so that requests are preempted.
// Built with AddressSanitizer and UBSan by tests/test_host_native.py; it checks that everything a
// request held comes back and prints "ok".
#include <cassert>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <vector>
#include "leone_host.h"

int main() {
    std::mt19937 rng(12345);
    for (int round = 0; round < 200; ++round) {
        const int groups[6] = {8 + int(rng() % 40), 16, 0, 8 + int(rng() % 40), 8, 24};
        void* cache = leone_cache_create(groups, 2, 6, 400);
        assert(cache);
        int64_t policy[6] = {1 + int64_t(rng() % 6), 64, 16 + int64_t(rng() % 100), 8 + int64_t(rng() % 60), 1 << 20, 1 << 20};
        void* sched = leone_scheduler_create(cache, policy);
        assert(sched);
        int64_t next = 1;
        int submitted = 0;
        for (int i = 0; i < 12; ++i) {
            std::vector<int32_t> prompt(1 + rng() % 120);
            for (auto& t : prompt) t = int32_t(rng() % 1000);
            int rc = leone_scheduler_submit(sched, next++, prompt.data(), int(prompt.size()), 1 + rng() % 40, rng() % 3 == 0 ? int(rng() % 1000) : -1);
            assert(rc >= 0);
            if (rc == 0) ++submitted;
        }
        int steps = 0;
        while (leone_scheduler_has_work(sched) == 1) {
            int n = leone_scheduler_plan(sched);
            if (n < 0) { std::printf("plan failed: %s\n", leone_host_last_error()); return 1; }
            if (n == 0) continue;
            std::vector<int64_t> req(n); std::vector<int> st(n), ct(n), sm(n);
            leone_scheduler_planned(sched, req.data(), st.data(), ct.data(), sm.data(), n);
            if (rng() % 50 == 0) { leone_scheduler_abort(sched); continue; }
            // pack the step as the engine would
            std::vector<int> wc(n); std::vector<int32_t> toks, wants;
            for (int i = 0; i < n; ++i) {
                std::vector<int32_t> t(ct[i]);
                int got = leone_scheduler_tokens(sched, req[i], st[i], ct[i], t.data());
                assert(got == ct[i]);
                toks.insert(toks.end(), t.begin(), t.end());
                wc[i] = sm[i] ? 1 : 0;
                if (sm[i]) wants.push_back(ct[i] - 1);
            }
            wants.push_back(0); toks.push_back(0);
            int shape[9] = {1000, 0, 2, 32, 16, 4, 8, 5, 2};   // two row tilings
            long sections[16]; int summary[8]; std::vector<int> placed(5 * n + 5);
            long need = leone_step_pack(cache, n, req.data(), ct.data(), wc.data(), toks.data(), wants.data(), shape, nullptr, 0, sections, nullptr, nullptr);
            if (need <= 0) { std::printf("pack failed (%ld): %s n=%d\n", need, leone_host_last_error(), n); return 1; }
            std::vector<int32_t> out(need);
            long wrote = leone_step_pack(cache, n, req.data(), ct.data(), wc.data(), toks.data(), wants.data(), shape, out.data(), need, sections, summary, placed.data());
            assert(wrote == need);
            std::vector<int64_t> who; std::vector<int32_t> tok;
            for (int i = 0; i < n; ++i) {
                int rc = leone_cache_commit(cache, req[i], ct[i]);
                assert(rc == 0);
                if (sm[i]) { who.push_back(req[i]); tok.push_back(int32_t(rng() % 1000)); }
            }
            who.push_back(0); tok.push_back(0);
            int done = leone_scheduler_complete(sched, who.data(), tok.data(), int(who.size()) - 1);
            assert(done >= 0);
            if (rng() % 30 == 0 && n > 0) leone_scheduler_cancel(sched, req[rng() % n]);
            if (++steps > 100000) { std::printf("no end\n"); return 1; }
        }
        assert(leone_cache_free_slots(cache) == 6);
        assert(leone_cache_free_pages(cache, 0) == groups[0] && leone_cache_free_pages(cache, 1) == groups[3]);
        int events = leone_scheduler_event_count(sched);
        std::vector<int> kinds(events), a(events), b(events), c(events); std::vector<int64_t> rq(events);
        leone_scheduler_events(sched, 0, events, kinds.data(), rq.data(), a.data(), b.data(), c.data());
        int64_t stats[15]; leone_scheduler_stats(sched, stats);
        (void)submitted;
        leone_scheduler_destroy(sched);
        leone_cache_destroy(cache);
    }
    std::printf("ok\n");
    return 0;
}
