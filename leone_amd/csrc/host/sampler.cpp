#include "sampler.h"

#include <algorithm>
#include <cmath>
#include <thread>

namespace leone::host {

namespace {

struct Candidate {
    float logit;
    int id;
};

// The reference's order: higher logit first, the lower id on a tie.
inline bool before(const Candidate& a, const Candidate& b) {
    return a.logit > b.logit || (a.logit == b.logit && a.id < b.id);
}

// How many of the first `have` sorted candidates a stage keeps, or -1 if it has to see further than
// `have` (only possible while `have` < `size`, the number of candidates the distribution has).
// p[i] are probabilities under the distribution before the stage.
int stage_keeps(const StageSpec& stage, const std::vector<double>& p, int have, int size) {
    switch (stage.kind) {
        case Stage::TopK: {
            const double k = stage.value;
            const int wanted = k >= static_cast<double>(size) ? size : static_cast<int>(k);
            return wanted <= have ? wanted : -1;
        }
        case Stage::TopP: {
            double mass = 0.0;
            for (int i = 0; i < have; ++i) {
                mass += p[i];
                if (mass >= stage.value) return i + 1;
            }
            return have == size ? size : -1;
        }
        case Stage::MinP: {
            const double floor = stage.value * p[0];
            for (int i = 0; i < have; ++i)
                if (!(p[i] >= floor)) return i;
            return have == size ? size : -1;
        }
    }
    throw SamplerFault("unknown truncation stage");
}

}  // namespace

int sample_row(const float* logits, int vocab, double temperature, const std::vector<StageSpec>& stages, double u,
               int* kept_out) {
    if (vocab <= 0) throw SamplerFault("empty logits row");
    if (!(temperature > 0.0) || !std::isfinite(temperature)) throw SamplerFault("temperature must be finite and positive");
    for (const StageSpec& s : stages) {
        if (s.kind == Stage::TopK ? !(s.value >= 1.0) || s.value != std::floor(s.value)
                                  : !(s.value > 0.0 && s.value <= 1.0))
            throw SamplerFault("truncation value out of range");
    }
    // highest finite logit and the number of candidates
    int size = 0;
    float top = 0.f;
    for (int i = 0; i < vocab; ++i) {
        const float l = logits[i];
        if (!std::isfinite(l)) continue;
        if (size == 0 || l > top) top = l;
        ++size;
    }
    if (size == 0) return -1;
    const double shift = static_cast<double>(top) / temperature;
    auto weight = [&](float l) { return std::exp(static_cast<double>(l) / temperature - shift); };

    if (stages.empty()) {
        if (kept_out) *kept_out = size;
        // nothing is cut: the running sum goes over the ids as they come
        double total = 0.0, carry = 0.0;
        for (int i = 0; i < vocab; ++i)
            if (std::isfinite(logits[i])) {          // compensated: 150,000 terms of very different size
                const double y = weight(logits[i]) - carry, t = total + y;
                carry = (t - total) - y;
                total = t;
            }
        double running = 0.0;
        int last = -1;
        for (int i = 0; i < vocab; ++i) {
            if (!std::isfinite(logits[i])) continue;
            const double p = weight(logits[i]) / total;
            if (p <= 0.0) continue;
            last = i;
            running += p;
            if (u < running) return i;
        }
        return last;
    }

    // A first stage that keeps the k best whatever their probabilities are makes the sum over the whole
    // vocabulary cancel in the renormalisation that follows it: the weights then stand for themselves.
    const bool cut_first = stages[0].kind == Stage::TopK && stages[0].value < static_cast<double>(size);
    double total = 1.0;
    if (!cut_first) {
        double carry = 0.0;
        total = 0.0;
        for (int i = 0; i < vocab; ++i) {
            if (!std::isfinite(logits[i])) continue;
            const double y = weight(logits[i]) - carry, t = total + y;
            carry = (t - total) - y;
            total = t;
        }
    }

    // The best `have` candidates in order.  They are picked in one pass over the row that keeps the
    // best so far in a heap (nearly every logit loses against the heap's worst at once); if a stage has
    // to see further, the pass is repeated for eight times as many.
    int have = 0;
    std::vector<Candidate> pool;
    std::vector<double> p;
    auto grow = [&](int wanted) {
        wanted = std::min(wanted, size);
        auto worse = [](const Candidate& a, const Candidate& b) { return before(a, b); };   // heap top = the worst kept
        pool.clear();
        pool.reserve(wanted);
        for (int i = 0; i < vocab; ++i) {
            const float l = logits[i];
            if (!std::isfinite(l)) continue;
            const Candidate candidate{l, i};
            if (static_cast<int>(pool.size()) < wanted) {
                pool.push_back(candidate);
                std::push_heap(pool.begin(), pool.end(), worse);
            } else if (before(candidate, pool.front())) {
                std::pop_heap(pool.begin(), pool.end(), worse);
                pool.back() = candidate;
                std::push_heap(pool.begin(), pool.end(), worse);
            }
        }
        std::sort(pool.begin(), pool.end(), before);
        p.resize(wanted);
        for (int i = 0; i < wanted; ++i) p[i] = weight(pool[i].logit) / total;
        have = wanted;
    };
    int first_k = 1024;
    if (stages[0].kind == Stage::TopK && stages[0].value < 1e9) first_k = std::max(64, static_cast<int>(stages[0].value));
    grow(first_k);

    int kept = size;                                   // candidates of the present distribution
    for (const StageSpec& stage : stages) {
        int n;
        while ((n = stage_keeps(stage, p, std::min(have, kept), kept)) < 0) grow(have * 8);
        n = std::max(1, n);
        if (n < kept || kept > have) {
            // the kept prefix becomes the whole distribution: renormalise it
            if (n > have) grow(n);                     // top-k beyond what is sorted so far
            double mass = 0.0;
            for (int i = 0; i < n; ++i) mass += p[i];
            if (!(mass > 0.0) || !std::isfinite(mass)) throw SamplerFault("no finite logit");
            for (int i = 0; i < n; ++i) p[i] /= mass;
            kept = n;
        }
    }
    if (kept > have) grow(kept);
    if (kept_out) *kept_out = kept;

    // the draw, over the kept tokens in id order
    std::vector<std::pair<int, double>> by_id(kept);
    for (int i = 0; i < kept; ++i) by_id[i] = {pool[i].id, p[i]};
    std::sort(by_id.begin(), by_id.end());
    double running = 0.0;
    int last = -1;
    for (const auto& entry : by_id) {
        if (entry.second <= 0.0) continue;
        last = entry.first;
        running += entry.second;
        if (u < running) return entry.first;
    }
    return last;
}

void sample_rows(const float* logits, int rows, int vocab, const double* temperature, const int* stage_counts,
                 const StageSpec* stages, const double* uniform, int* tokens) {
    std::vector<int> first(rows + 1, 0);
    for (int r = 0; r < rows; ++r) first[r + 1] = first[r] + stage_counts[r];
    auto one = [&](int r) {
        const std::vector<StageSpec> mine(stages + first[r], stages + first[r + 1]);
        tokens[r] = sample_row(logits + static_cast<long>(r) * vocab, vocab, temperature[r], mine, uniform[r]);
    };
    const int workers = std::min(rows, 8);
    if (workers <= 1 || static_cast<long>(rows) * vocab < (1L << 16)) {
        for (int r = 0; r < rows; ++r) one(r);
        return;
    }
    std::vector<std::thread> pool;
    std::vector<std::exception_ptr> failed(workers);
    for (int w = 0; w < workers; ++w)
        pool.emplace_back([&, w]() {
            try {
                for (int r = w; r < rows; r += workers) one(r);
            } catch (...) {
                failed[w] = std::current_exception();
            }
        });
    for (std::thread& t : pool) t.join();
    for (const std::exception_ptr& e : failed)
        if (e) std::rethrow_exception(e);
}

}  // namespace leone::host
