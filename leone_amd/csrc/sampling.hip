// Token selection on the device.
//
// argmax: the highest finite logit, the lowest index on a tie; NaN and
// infinities never win; a row without a finite value yields -1
// (crates/leone/src/sampler.rs:787-799, crates/leone/src/cpu.rs:1341-1362).
// temperature: weights exp(l/t - max/t) over the finite logits in double,
// the token is the first, in id order, whose running share exceeds the given
// uniform value; the last eligible token if rounding leaves none
// (crates/leone/src/sampler.rs:502-534, 843-858).
#include "common.h"
#include "leone_hip.h"

#include <math.h>
#include <mutex>

namespace leone {

constexpr int kSampleThreads = 1024;

struct Best {
    float value;
    int index;
};

__device__ inline Best better(Best a, Best b) {
    if (b.index < 0) return a;
    if (a.index < 0) return b;
    if (b.value > a.value || (b.value == a.value && b.index < a.index)) return b;
    return a;
}

__device__ inline Best block_best(Best mine, Best* scratch) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        Best other;
        other.value = __shfl_xor(mine.value, off, kWave);
        other.index = __shfl_xor(mine.index, off, kWave);
        mine = better(mine, other);
    }
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    __syncthreads();
    if (lane == 0) scratch[wave] = mine;
    __syncthreads();
    Best total = scratch[0];
    for (int w = 1; w < kSampleThreads / kWave; ++w) total = better(total, scratch[w]);
    return total;
}

// Two stages, as the reference's pair of kernels (crates/leone-cuda/cuda/ie_cuda.cu:4840, 4870): every
// workgroup finds the best of one chunk of a row, then one workgroup a row picks among the chunks.
// `better` prefers the lower index on equal values, so the result does not depend on the cut.
constexpr int kArgmaxChunk = 4096;

__global__ void __launch_bounds__(kSampleThreads)
argmax_partial_kernel(const float* __restrict__ logits, float* __restrict__ part_value,
                      int* __restrict__ part_index, int vocab, int chunks) {
    __shared__ Best scratch[kSampleThreads / kWave];
    const int chunk = blockIdx.x;
    const float* row = logits + static_cast<long>(blockIdx.y) * vocab;
    const int end = (chunk + 1) * kArgmaxChunk < vocab ? (chunk + 1) * kArgmaxChunk : vocab;
    Best mine{0.f, -1};
    for (int i = chunk * kArgmaxChunk + threadIdx.x; i < end; i += kSampleThreads) {
        const float v = row[i];
        if (!isfinite(v)) continue;
        if (mine.index < 0 || v > mine.value) mine = Best{v, i};
    }
    const Best total = block_best(mine, scratch);
    if (threadIdx.x == 0) {
        part_value[blockIdx.y * chunks + chunk] = total.value;
        part_index[blockIdx.y * chunks + chunk] = total.index;
    }
}

__global__ void __launch_bounds__(kSampleThreads)
argmax_final_kernel(const float* __restrict__ part_value, const int* __restrict__ part_index,
                    int* __restrict__ out, int chunks) {
    __shared__ Best scratch[kSampleThreads / kWave];
    Best mine{0.f, -1};
    for (int i = threadIdx.x; i < chunks; i += kSampleThreads)
        mine = better(mine, Best{part_value[blockIdx.x * chunks + i], part_index[blockIdx.x * chunks + i]});
    const Best total = block_best(mine, scratch);
    if (threadIdx.x == 0) out[blockIdx.x] = total.index;
}

// Temperature sampling, three steps: the row's highest logit (the two argmax kernels), then the sum of
// the weights of every chunk of 4096 ids (one workgroup a chunk), then one workgroup a row walks the chunk
// sums in id order to the chunk that holds the drawn value, and inside it the sums of its 16 waves, of the
// wave's 64 threads and the thread's 4 ids.  Sums are always taken in the same order (ids of a thread, threads
// of a wave, waves of a chunk, chunks of a row, each from the left), in both kernels, so that what the walk
// adds up is what was summed.  Where rounding lets the walk end without crossing the drawn value, the last
// token with a weight above zero is taken.
__device__ inline void chunk_weights(const float* row, int vocab, int chunk, double t, double highest, double w[4]) {
    const int base = chunk * kArgmaxChunk + 4 * static_cast<int>(threadIdx.x);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int id = base + i;
        const float v = id < vocab ? row[id] : NAN;
        w[i] = isfinite(v) ? exp(static_cast<double>(v) / t - highest) : 0.0;
    }
}

// thread_sum[t] = the weights of thread t's ids, wave_sum[v] = the thread sums of wave v from the left.
__device__ inline void chunk_sums_in_order(const double w[4], double* thread_sum, double* wave_sum) {
    thread_sum[threadIdx.x] = ((w[0] + w[1]) + w[2]) + w[3];
    __syncthreads();
    if (threadIdx.x % kWave == 0) {
        double sum = 0.0;
        for (int i = 0; i < kWave; ++i) sum += thread_sum[threadIdx.x + i];
        wave_sum[threadIdx.x / kWave] = sum;
    }
    __syncthreads();
}

__global__ void __launch_bounds__(kSampleThreads)
temperature_sums_kernel(const float* __restrict__ logits, const double* __restrict__ temperature,
                        const int* __restrict__ best, double* __restrict__ sums, int vocab, int chunks) {
    __shared__ double thread_sum[kSampleThreads];
    __shared__ double wave_sum[kSampleThreads / kWave];
    const int r = blockIdx.y, chunk = blockIdx.x;
    const float* row = logits + static_cast<long>(r) * vocab;
    const int top = best[r];
    if (top < 0) return;                                    // no finite logit: the row's answer is -1
    const double t = temperature[r];
    double w[4];
    chunk_weights(row, vocab, chunk, t, static_cast<double>(row[top]) / t, w);
    chunk_sums_in_order(w, thread_sum, wave_sum);
    if (threadIdx.x == 0) {
        double sum = 0.0;
        for (int v = 0; v < kSampleThreads / kWave; ++v) sum += wave_sum[v];
        sums[static_cast<long>(r) * chunks + chunk] = sum;
    }
}

// In `sum[0, n)`, walked from the left with `running` as the sum before: the first positive entry that takes
// the running sum above `target`, or the last positive entry; `running` ends as the sum before that entry.
__device__ inline int walk_to(const double* sum, int n, double target, double& running) {
    int at = -1;
    double before = running;
    for (int i = 0; i < n; ++i) {
        const double s = sum[i];
        if (!(s > 0.0)) continue;
        at = i;
        before = running;
        if (target < running + s) break;
        running += s;
    }
    running = before;
    return at;
}

__global__ void __launch_bounds__(kSampleThreads)
temperature_pick_kernel(const float* __restrict__ logits, const double* __restrict__ temperature,
                        const double* __restrict__ uniform, const int* __restrict__ best,
                        const double* __restrict__ sums, int* __restrict__ out, int vocab, int chunks) {
    __shared__ double thread_sum[kSampleThreads];
    __shared__ double wave_sum[kSampleThreads / kWave];
    __shared__ int chosen_chunk, chosen_thread;
    __shared__ double chosen_before, target;
    const int r = blockIdx.x;
    const float* row = logits + static_cast<long>(r) * vocab;
    const int top = best[r];
    if (top < 0) {
        if (threadIdx.x == 0) out[r] = -1;
        return;
    }
    const double* mine = sums + static_cast<long>(r) * chunks;
    if (threadIdx.x == 0) {
        double total = 0.0;
        for (int c = 0; c < chunks; ++c) total += mine[c];
        target = uniform[r] * total;
        double running = 0.0;
        chosen_chunk = walk_to(mine, chunks, target, running);   // the highest logit weighs 1: some chunk is positive
        chosen_before = running;
        if (chosen_chunk < 0) out[r] = top;                      // sums that are not numbers (a temperature the host let through)
    }
    __syncthreads();
    const int chunk = chosen_chunk;
    if (chunk < 0) return;
    const double t = temperature[r];
    double w[4];
    chunk_weights(row, vocab, chunk, t, static_cast<double>(row[top]) / t, w);
    chunk_sums_in_order(w, thread_sum, wave_sum);
    if (threadIdx.x == 0) {
        double running = chosen_before;
        const int wave = walk_to(wave_sum, kSampleThreads / kWave, target, running);
        const int lane = wave < 0 ? -1 : walk_to(thread_sum + wave * kWave, kWave, target, running);
        chosen_thread = lane < 0 ? -1 : wave * kWave + lane;
        chosen_before = running;
        if (lane < 0) out[r] = top;
    }
    __syncthreads();
    if (static_cast<int>(threadIdx.x) == chosen_thread) {
        double running = chosen_before;
        const int at = walk_to(w, 4, target, running);
        out[r] = at < 0 ? top : chunk * kArgmaxChunk + 4 * static_cast<int>(threadIdx.x) + at;
    }
}

// ---- the best k logits of a row ---------------------------------------------------------------------------
//
// The sampler's order (crates/leone/src/sampler.rs:502-534): finite logits only, the higher first, the
// lower id on a tie.  A logit and its id become one 64-bit key whose unsigned order is that order
// (0 for a value that is not finite, behind every finite one), so that selection is a matter of integers.
//
// One workgroup a row.  Every thread finds the best among the ids it owns (four neighbours out of every
// 4,096), four neighbouring threads make a cell; the k-th best of the 256 cells' keys is a bound that the
// row's k-th best key cannot lie behind.  A second walk collects every key not behind the bound (for
// k <= 256 and a vocabulary of 150,000 a few hundred), every collected key finds its place by counting the
// keys before it, and the first k places are the result.  A row whose collection would not fit (values
// arranged against the deal of ids to cells) is selected key by key instead.
constexpr int kCandidateMaxK = 256;
constexpr int kCandidateRoom = 4096;
constexpr int kCellThreads = 4;                              // threads whose ids make one cell

__device__ inline unsigned long long candidate_key(float v, int id) {
    v += 0.0f;                                              // -0 and +0 are one value
    const unsigned bits = __float_as_uint(v);
    if ((bits & 0x7f800000u) == 0x7f800000u) return 0ull;   // infinity or NaN
    const unsigned ordered = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    return (static_cast<unsigned long long>(ordered) << 32) | (0xffffffffu - static_cast<unsigned>(id));
}

__device__ inline int candidate_id(unsigned long long key) {
    return static_cast<int>(0xffffffffu - static_cast<unsigned>(key & 0xffffffffull));
}

// How many of keys[0, n) are greater than `key`: its place when the keys are put in falling order (the keys of
// finite logits are all different).  Every lane reads the same place at a time, which shared memory serves as one
// read; for the few hundred keys this is asked of it is much cheaper than a sort with a barrier a step.
__device__ inline int rank_among(const unsigned long long* keys, int n, unsigned long long key) {
    int greater = 0;
    int i = 0;
    for (; i + 2 <= n; i += 2) {
        const ulonglong2 two = *reinterpret_cast<const ulonglong2*>(keys + i);
        greater += (two.x > key) + (two.y > key);
    }
    if (i < n) greater += keys[i] > key;
    return greater;
}

// The greatest key of the workgroup, for every thread; `scratch` holds one place a wave.
__device__ inline unsigned long long block_max_key(unsigned long long mine, unsigned long long* scratch) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const unsigned long long other = __shfl_xor(mine, off, kWave);
        mine = other > mine ? other : mine;
    }
    __syncthreads();                                        // what the call before this one left has been read
    if (threadIdx.x % kWave == 0) scratch[threadIdx.x / kWave] = mine;
    __syncthreads();
    unsigned long long total = scratch[0];
    for (int w = 1; w < kSampleThreads / kWave; ++w) total = scratch[w] > total ? scratch[w] : total;
    return total;
}

struct Selection {
    int kept;   // keys[0, kept) are the row's best keys, the best first: min(k, size) of them
    int size;   // finite logits in the row
};

// Thread t owns the ids 4 q .. 4 q + 3 of every q with q % 1024 == t.  The four logits at ids 4 q .. 4 q + 3, NaN
// (which never counts) beyond the row's end; one 16-byte load where the row allows it.
__device__ inline float4 row_quad(const float* __restrict__ row, int q, int vocab, bool aligned) {
    const int id = 4 * q;
    if (aligned && id + 4 <= vocab) return *reinterpret_cast<const float4*>(row + id);
    float4 v;
    v.x = id < vocab ? row[id] : NAN;
    v.y = id + 1 < vocab ? row[id + 1] : NAN;
    v.z = id + 2 < vocab ? row[id + 2] : NAN;
    v.w = id + 3 < vocab ? row[id + 3] : NAN;
    return v;
}

// Calls use(value, id) for every id this thread owns, in rising order, eight quads' loads on their way at a time;
// beyond the row's end the value is NaN.
template <typename Use>
__device__ inline void for_own_ids(const float* __restrict__ row, int vocab, Use use) {
    const bool aligned = (reinterpret_cast<unsigned long long>(row) & 15ull) == 0ull;
    const int quads = (vocab + 3) / 4;
    constexpr int kAhead = 8;
    for (int q0 = threadIdx.x; q0 < quads; q0 += kAhead * kSampleThreads) {
        float4 v[kAhead];
#pragma unroll
        for (int a = 0; a < kAhead; ++a) {
            const int q = q0 + a * kSampleThreads;
            v[a] = q < quads ? row_quad(row, q, vocab, aligned) : float4{NAN, NAN, NAN, NAN};
        }
#pragma unroll
        for (int a = 0; a < kAhead; ++a) {
            const int id = 4 * (q0 + a * kSampleThreads);
            use(v[a].x, id);
            use(v[a].y, id + 1);
            use(v[a].z, id + 2);
            use(v[a].w, id + 3);
        }
    }
}

__device__ inline bool is_finite(float v) { return (__float_as_uint(v) & 0x7f800000u) != 0x7f800000u; }

// The selection described above; every thread of the workgroup calls it.  `keys` has kCandidateRoom places,
// `counters` two, `bound_at` one.  A row whose collection does not fit the room is selected the slow way instead,
// one key after the other, each the greatest that lies behind the one before: k walks over the row, for rows that
// are laid out against the deal of ids to cells and for no others.
//
// The walks compare logits as numbers (a greater value, or an equal one at a lower id, is the greater key) and
// make keys only of what they keep: the walks are bound by their arithmetic, not by memory.
__device__ inline Selection select_best(const float* __restrict__ row, int vocab, int k, unsigned long long* keys,
                                        int* counters, unsigned long long* bound_at) {
    static_assert(kSampleThreads / kCellThreads == kCandidateMaxK, "one cell for each candidate that may be asked for");
    float best_value = 0.f;
    int best_id = -1, finite = 0;
    for_own_ids(row, vocab, [&](float v, int id) {
        const bool counts = is_finite(v);
        finite += counts;
        if (counts && (best_id < 0 || v > best_value)) {      // ids come in rising order: of equal values the first stays
            best_value = v;
            best_id = id;
        }
    });
    // A cell is kCellThreads neighbouring threads; its best key goes to keys[cell].
    unsigned long long best = best_id < 0 ? 0ull : candidate_key(best_value, best_id);
#pragma unroll
    for (int off = 1; off < kCellThreads; off <<= 1) {
        const unsigned long long other = __shfl_xor(best, off, kWave);
        best = other > best ? other : best;
    }
    if (threadIdx.x % kCellThreads == 0) keys[threadIdx.x / kCellThreads] = best;
    if (threadIdx.x == 0) {
        counters[0] = counters[1] = 0;
        *bound_at = 0ull;
    }
    __syncthreads();
    // The k-th best of the cells' bests: 0 if fewer than k cells hold a finite value, then every finite value is
    // collected.
    if (threadIdx.x < kCandidateMaxK) {
        const unsigned long long mine = keys[threadIdx.x];
        if (mine != 0ull && rank_among(keys, kCandidateMaxK, mine) == k - 1) *bound_at = mine;
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) finite += __shfl_xor(finite, off, kWave);
    if (threadIdx.x % kWave == 0) atomicAdd(&counters[1], finite);
    __syncthreads();
    const unsigned long long bound = *bound_at;
    __syncthreads();                                        // the cells' bests have been read: their places are free

    const bool all = bound == 0ull;
    const int bound_id = candidate_id(bound);
    const float bound_value = all ? 0.f : row[bound_id];
    for_own_ids(row, vocab, [&](float v, int id) {
        if (is_finite(v) && (all || v > bound_value || (v == bound_value && id <= bound_id))) {
            const int at = atomicAdd(&counters[0], 1);
            if (at < kCandidateRoom) keys[at] = candidate_key(v, id);
        }
    });
    __syncthreads();
    const int found = counters[0], size = counters[1];
    if (found <= kCandidateRoom) {
        // every collected key finds its place by itself; the first k places are the result
        unsigned long long mine[kCandidateRoom / kSampleThreads];
        int place[kCandidateRoom / kSampleThreads];
#pragma unroll
        for (int n = 0; n < kCandidateRoom / kSampleThreads; ++n) {
            const int i = threadIdx.x + n * kSampleThreads;
            place[n] = k;
            if (i < found) {
                mine[n] = keys[i];
                place[n] = rank_among(keys, found, mine[n]);
            }
        }
        __syncthreads();
#pragma unroll
        for (int n = 0; n < kCandidateRoom / kSampleThreads; ++n)
            if (place[n] < k) keys[place[n]] = mine[n];
        __syncthreads();
        return Selection{found < k ? found : k, size};
    }
    unsigned long long* scratch = keys + kCandidateMaxK;
    unsigned long long behind = ~0ull;
    int kept = 0;
    for (; kept < k; ++kept) {
        unsigned long long mine = 0ull;
        for_own_ids(row, vocab, [&](float v, int id) {
            const unsigned long long key = candidate_key(v, id);
            if (key < behind && key > mine) mine = key;
        });
        mine = block_max_key(mine, scratch);
        if (mine == 0ull) break;
        if (threadIdx.x == 0) keys[kept] = mine;
        behind = mine;
    }
    __syncthreads();
    return Selection{kept, size};
}

__global__ void __launch_bounds__(kSampleThreads)
top_candidates_kernel(const float* __restrict__ logits, int k, float* __restrict__ out_values,
                      int* __restrict__ out_ids, int* __restrict__ out_count, int vocab) {
    __shared__ __align__(16) unsigned long long keys[kCandidateRoom];
    __shared__ int counters[2];
    __shared__ unsigned long long bound;
    const float* row = logits + static_cast<long>(blockIdx.x) * vocab;
    const Selection chosen = select_best(row, vocab, k, keys, counters, &bound);
    for (int i = threadIdx.x; i < chosen.kept; i += kSampleThreads) {
        const int id = candidate_id(keys[i]);
        out_ids[static_cast<long>(blockIdx.x) * kCandidateMaxK + i] = id;
        out_values[static_cast<long>(blockIdx.x) * kCandidateMaxK + i] = row[id];
    }
    if (threadIdx.x == 0) out_count[blockIdx.x] = chosen.kept;
}

// ---- temperature sampling with truncation stages, top-k first -------------------------------------------
//
// The host sampler's rules (csrc/host/sampler.cpp, after crates/leone/src/sampler.rs:502-606, 843-858) for the
// policies whose first stage keeps the k best logits, k at most kCandidateMaxK: those k are all the sampler
// ever looks at.  One workgroup a row selects them as above; the weights exp(l/t - l_max/t) are taken in
// double, one thread a candidate; one thread then walks the stages in the order given, each on the
// renormalised result of the one before, each keeping at least one token, with the sums taken from the left
// as the host takes them; the token is the first of the kept ones, in id order, whose running share exceeds
// the uniform value, the last with a share above zero if rounding leaves none.  A row without a finite logit
// gives -1.
//
// A row's parameters are kDrawParams doubles: temperature, uniform value, the number of stages (0: the row
// is not for this kernel and gets -1), then for each stage its kind (0 top-k, 1 top-p, 2 min-p) and value.
constexpr int kDrawStages = 8;
constexpr int kDrawParams = 3 + 2 * kDrawStages;

__global__ void __launch_bounds__(kSampleThreads)
sample_truncated_kernel(const float* __restrict__ logits, const double* __restrict__ params, int* __restrict__ out,
                        int vocab) {
    __shared__ __align__(16) unsigned long long keys[kCandidateRoom];
    __shared__ int counters[2];
    __shared__ unsigned long long bound;
    __shared__ int by_id[kCandidateMaxK];
    __shared__ double share[kCandidateMaxK];
    __shared__ double mass;
    __shared__ int keep;
    const float* row = logits + static_cast<long>(blockIdx.x) * vocab;
    const double* mine = params + static_cast<long>(blockIdx.x) * kDrawParams;
    // The caller checks the table before it uploads it; whatever the memory holds, the kernel stays in its arrays.
    const int stages = mine[2] >= 1.0 ? (mine[2] < kDrawStages ? static_cast<int>(mine[2]) : kDrawStages) : 0;
    const bool cut = stages > 0 && static_cast<int>(mine[3]) == 0 && mine[4] >= 1.0 && mine[4] <= kCandidateMaxK;
    if (!cut) {
        if (threadIdx.x == 0) out[blockIdx.x] = -1;
        return;
    }
    const int k = static_cast<int>(mine[4]);
    const Selection chosen = select_best(row, vocab, k, keys, counters, &bound);
    const int have = chosen.kept;
    if (have == 0) {
        if (threadIdx.x == 0) out[blockIdx.x] = -1;
        return;
    }
    const double t = mine[0];
    if (static_cast<int>(threadIdx.x) < have) {
        const double shift = static_cast<double>(row[candidate_id(keys[0])]) / t;
        share[threadIdx.x] = exp(static_cast<double>(row[candidate_id(keys[threadIdx.x])]) / t - shift);
    }
    // The candidates once more in id order: by_id[n] is the rank of the candidate with the n-th lowest id.  The
    // order of the draw, and of the whole row's sum.
    if (static_cast<int>(threadIdx.x) < have) {
        const unsigned my_id = static_cast<unsigned>(keys[threadIdx.x] & 0xffffffffull);   // the greater, the lower the id
        int lower = 0;
        for (int i = 0; i < have; ++i) lower += static_cast<unsigned>(keys[i] & 0xffffffffull) > my_id;
        by_id[lower] = threadIdx.x;
    }
    __syncthreads();

    // A first stage that cuts makes the sum over the whole row cancel in the renormalisation that follows: the
    // weights stand for themselves.  Otherwise every finite logit is a candidate and the sum is theirs, in id
    // order, compensated.
    if (threadIdx.x == 0) {
        double total = 1.0;
        if (!(k < chosen.size)) {
            double carry = 0.0;
            total = 0.0;
            for (int j = 0; j < have; ++j) {
                const double y = share[by_id[j]] - carry, sum = total + y;
                carry = (sum - total) - y;
                total = sum;
            }
        }
        mass = total;
    }
    __syncthreads();
    if (static_cast<int>(threadIdx.x) < have) share[threadIdx.x] /= mass;
    __syncthreads();

    int kept = chosen.size;                                 // tokens of the present distribution
    for (int s = 0; s < stages; ++s) {
        if (threadIdx.x == 0) {
            const int kind = static_cast<int>(mine[3 + 2 * s]);
            const double value = mine[4 + 2 * s];
            const int seen = kept < have ? kept : have;
            int n = seen;
            if (kind == 0) {
                n = value >= static_cast<double>(kept) ? kept : static_cast<int>(value);
            } else if (kind == 1) {
                double sum = 0.0;
                for (int i = 0; i < seen; ++i) {
                    sum += share[i];
                    if (sum >= value) {
                        n = i + 1;
                        break;
                    }
                }
            } else {
                const double floor = value * share[0];
                for (int i = 0; i < seen; ++i)
                    if (!(share[i] >= floor)) {
                        n = i;
                        break;
                    }
            }
            n = n < 1 ? 1 : n;
            n = n > have ? have : n;                        // the first stage has cut to what is held, or the row is held whole
            double sum = 0.0;
            for (int i = 0; i < n; ++i) sum += share[i];
            mass = sum;
            keep = n;
        }
        __syncthreads();
        const int n = keep;
        if (n < kept) {
            if (static_cast<int>(threadIdx.x) < n) share[threadIdx.x] /= mass;
            kept = n;
        }
        __syncthreads();
    }

    if (threadIdx.x == 0) {
        const double u = mine[1];
        double running = 0.0;
        int token = -1;
        for (int j = 0; j < have; ++j) {
            const int rank = by_id[j];
            if (rank >= kept) continue;
            const double p = share[rank];
            if (!(p > 0.0)) continue;
            token = candidate_id(keys[rank]);
            running += p;
            if (u < running) break;
        }
        out[blockIdx.x] = token;
    }
}

}  // namespace leone

using namespace leone;

extern "C" int leone_top_candidates_max() { return kCandidateMaxK; }

// For each row the `wanted` (1..leone_top_candidates_max()) best finite logits in the sampler's order,
// best first (so that the first j of them are the row's j best): out_values and out_ids hold
// leone_top_candidates_max() places a row, out_count[row] says how many are filled (fewer than wanted if
// the row has fewer finite logits).
extern "C" int leone_top_candidates(const float* logits, float* out_values, int* out_ids, int* out_count, int rows,
                                    int vocab, int wanted, hipStream_t stream) {
    LEONE_REQUIRE(logits && out_values && out_ids && out_count, "top_candidates: null pointer");
    LEONE_REQUIRE(rows > 0 && vocab > 0 && vocab <= (1 << 30), "top_candidates: rows %d vocab %d out of range", rows, vocab);
    LEONE_REQUIRE(wanted >= 1 && wanted <= kCandidateMaxK,
                  "top_candidates: %d wanted, at most %d can be selected", wanted, kCandidateMaxK);
    top_candidates_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, wanted, out_values, out_ids, out_count, vocab);
    LEONE_LAUNCH_CHECK("top_candidates");
    return 0;
}

extern "C" int leone_sample_truncated_stages() { return kDrawStages; }
extern "C" int leone_sample_truncated_params() { return kDrawParams; }

// One token a row by temperature sampling with truncation stages of which the first keeps the k best logits,
// k at most leone_top_candidates_max().  `params` holds leone_sample_truncated_params() doubles a row:
// temperature (above zero), the uniform value in [0, 1), the number of stages (1..leone_sample_truncated_stages();
// 0 marks a row that is not to be sampled and gets -1), then a (kind, value) pair for each stage: 0 top-k,
// 1 top-p, 2 min-p; the first stage's kind is 0.  out[row] is -1 for a row without a finite logit.
extern "C" int leone_sample_truncated(const float* logits, const double* params, int* out, int rows, int vocab,
                                      hipStream_t stream) {
    LEONE_REQUIRE(logits && params && out, "sample_truncated: null pointer");
    LEONE_REQUIRE(rows > 0 && vocab > 0 && vocab <= (1 << 30), "sample_truncated: rows %d vocab %d out of range", rows, vocab);
    sample_truncated_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, params, out, vocab);
    LEONE_LAUNCH_CHECK("sample_truncated");
    return 0;
}

extern "C" int leone_argmax_chunk() { return kArgmaxChunk; }

// part_value and part_index hold rows * ceil(vocab / leone_argmax_chunk()) entries each.
extern "C" int leone_argmax(const float* logits, int* out, float* part_value, int* part_index, int rows, int vocab,
                            hipStream_t stream) {
    LEONE_REQUIRE(logits && out && part_value && part_index, "argmax: null pointer");
    LEONE_REQUIRE(rows > 0 && rows <= 65535 && vocab > 0, "argmax: rows %d vocab %d out of range", rows, vocab);
    const int chunks = ceil_div(vocab, kArgmaxChunk);
    argmax_partial_kernel<<<dim3(chunks, rows), kSampleThreads, 0, stream>>>(logits, part_value, part_index, vocab, chunks);
    LEONE_LAUNCH_CHECK("argmax");
    argmax_final_kernel<<<rows, kSampleThreads, 0, stream>>>(part_value, part_index, out, chunks);
    LEONE_LAUNCH_CHECK("argmax");
    return 0;
}

// ---- argmax without a workspace argument and without any allocation --------------------------------
// For callers that cannot allocate device memory around the call (code under graph capture, tight serving
// loops, harnesses that forbid it).  The per-chunk candidates of leone_argmax live in a file-scope device
// array instead of a workspace the caller brings.  Each GPU holds its own copy of the array at its own
// address until the process ends; the address is asked for once per device and kept.
constexpr int kStaticArgmaxEntries = 16384;                         // rows * chunks at most: 128 KiB a GPU
constexpr int kStaticMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticArgmaxEntries * (sizeof(float) + sizeof(int))];

namespace leone {
static std::mutex g_scratch_lock;
static void* g_scratch_ptr[kStaticMaxDevices] = {};                 // device address of `scratch`, per device

// The address of this device's copy of the array (the array's name is only a stand-in in host code).
static int scratch_for_current_device(void** out) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess || device < 0 || device >= kStaticMaxDevices) {
        set_error("argmax_static: no usable current device (%s)", hipGetErrorString(e));
        return 1;
    }
    std::lock_guard<std::mutex> guard(g_scratch_lock);
    if (g_scratch_ptr[device] == nullptr) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) {
            set_error("argmax_static: the address of the scratch array on device %d was refused: %s", device,
                      hipGetErrorString(e));
            return 1;
        }
        g_scratch_ptr[device] = ptr;
    }
    *out = g_scratch_ptr[device];
    return 0;
}
}  // namespace leone

extern "C" int leone_argmax_static_max_entries() { return kStaticArgmaxEntries; }

// The same result as leone_argmax.  rows * ceil(vocab / leone_argmax_chunk()) may be at most
// leone_argmax_static_max_entries(); beyond that the call is refused.  Every entry of the array that the
// second kernel reads is written by the first kernel of the same call, so nothing has to start at zero;
// what an earlier call left is overwritten or never read.  All calls on one GPU share that GPU's array:
// two calls that overlap in time on one GPU (different streams, or threads) race and give wrong tokens.
extern "C" int leone_argmax_static(const float* logits, int* out, int rows, int vocab, hipStream_t stream) {
    LEONE_REQUIRE(logits && out, "argmax_static: null pointer");
    LEONE_REQUIRE(rows > 0 && rows <= 65535 && vocab > 0, "argmax_static: rows %d vocab %d out of range", rows, vocab);
    const int chunks = ceil_div(vocab, kArgmaxChunk);
    LEONE_REQUIRE(static_cast<long>(rows) * chunks <= kStaticArgmaxEntries,
                  "argmax_static: %d rows of %d chunks need %ld entries, the fixed scratch array holds %d",
                  rows, chunks, static_cast<long>(rows) * chunks, kStaticArgmaxEntries);
    void* base = nullptr;
    if (scratch_for_current_device(&base)) return 1;
    float* part_value = static_cast<float*>(base);
    int* part_index = reinterpret_cast<int*>(static_cast<unsigned char*>(base) + kStaticArgmaxEntries * sizeof(float));
    argmax_partial_kernel<<<dim3(chunks, rows), kSampleThreads, 0, stream>>>(logits, part_value, part_index, vocab, chunks);
    LEONE_LAUNCH_CHECK("argmax_static");
    argmax_final_kernel<<<rows, kSampleThreads, 0, stream>>>(part_value, part_index, out, chunks);
    LEONE_LAUNCH_CHECK("argmax_static");
    return 0;
}

// Workspace: part_value and part_index as for leone_argmax, best with one entry a row, sums with
// rows * ceil(vocab / leone_argmax_chunk()) doubles.
extern "C" int leone_sample_temperature(const float* logits, const double* temperature, const double* uniform,
                                        int* out, float* part_value, int* part_index, int* best, double* sums,
                                        int rows, int vocab, hipStream_t stream) {
    LEONE_REQUIRE(logits && temperature && uniform && out && part_value && part_index && best && sums,
                  "sample_temperature: null pointer");
    LEONE_REQUIRE(rows > 0 && rows <= 65535 && vocab > 0, "sample_temperature: rows %d vocab %d out of range", rows, vocab);
    const int chunks = ceil_div(vocab, kArgmaxChunk);
    argmax_partial_kernel<<<dim3(chunks, rows), kSampleThreads, 0, stream>>>(logits, part_value, part_index, vocab, chunks);
    LEONE_LAUNCH_CHECK("sample_temperature");
    argmax_final_kernel<<<rows, kSampleThreads, 0, stream>>>(part_value, part_index, best, chunks);
    LEONE_LAUNCH_CHECK("sample_temperature");
    temperature_sums_kernel<<<dim3(chunks, rows), kSampleThreads, 0, stream>>>(logits, temperature, best, sums, vocab, chunks);
    LEONE_LAUNCH_CHECK("sample_temperature");
    temperature_pick_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, temperature, uniform, best, sums, out, vocab, chunks);
    LEONE_LAUNCH_CHECK("sample_temperature");
    return 0;
}
