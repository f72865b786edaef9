// Temperature sampling with the common truncation stages over a full-vocabulary row, in double.
//
// The rules are the reference's (crates/leone/src/sampler.rs): candidates are the finite logits in
// descending order, ties by the lower id; weights exp(l/t - l_max/t), normalised (:502-534); the
// stages run in the order given, each on the renormalised result of the one before, each keeping at
// least one token (:559-606): top-k keeps k, top-p the shortest prefix whose mass reaches p, min-p
// the tokens whose probability is at least p times the highest; the token is the first, in id
// order, whose cumulative probability exceeds the uniform value, the last eligible one if rounding
// leaves none (:843-858).
//
// What this routine adds is only economy: a row of 150,000 logits is not sorted as a whole.  The
// best M candidates are selected and sorted, and M grows only if a stage needs to look further.
#pragma once

#include <cstdint>
#include <stdexcept>
#include <vector>

namespace leone::host {

enum class Stage : int { TopK = 0, TopP = 1, MinP = 2 };

struct StageSpec {
    Stage kind;
    double value;
};

struct SamplerFault : std::runtime_error {
    using std::runtime_error::runtime_error;
};

// The token for one row; -1 if the row holds no finite logit.  `kept_out`, if given, receives the
// number of tokens left after the last stage.
int sample_row(const float* logits, int vocab, double temperature, const std::vector<StageSpec>& stages, double u,
               int* kept_out = nullptr);

// The same for `rows` rows of `vocab` logits each, row r with temperature[r], its own stages
// (stage_counts[r] of them, one after the other in `stages`) and uniform[r]; rows are shared out
// among a few threads.
void sample_rows(const float* logits, int rows, int vocab, const double* temperature, const int* stage_counts,
                 const StageSpec* stages, const double* uniform, int* tokens);

}  // namespace leone::host
