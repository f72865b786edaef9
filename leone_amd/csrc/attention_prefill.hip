// Causal attention of prompt portions over the paged cache on the matrix cores, bfloat16.
//
// A portion's rows are cut into tiles of 32 consecutive rows; a wave takes one tile and one query
// head, its rows as two 16-column operands.  A workgroup is four waves whose tiles belong to the
// same request (the host lists them: entry, first row, row count, four to a workgroup).  The
// workgroup walks the keys its tiles can see once, 64 at a time: the next 64 keys and values travel
// from the cache to shared memory while the waves work on the present 64 (by loads that write to
// shared memory themselves; a stage at the edge of the keys or across pages goes through registers,
// where it is masked), and every wave takes from shared memory the 32-key halves its own rows can see.  A wave keeps the
// running reference, sum and accumulator of the reference's recurrence
// (crates/leone/src/cpu.rs:2359-2421) per query in registers; nothing of size rows x keys is ever
// stored (the reference's prefill materialises the scores, crates/leone-cuda/cuda/ie_cuda.cu:5124-5220).
// Products and operand layouts are those of the decode kernel: S^T = K . Q^T and O^T += V^T . P^T
// with v_mfma_f32_16x16x32_bf16 on 16-byte runs of the packed cache layout.  Keys are stored in
// shared memory in the order the first product's operand wants them, so that neighbouring lanes
// read neighbouring runs.
//
// The recurrence is kept in base-2 units: t = score * scale * log2(e), p = 2^(t - m).  m is a
// reference, not always the maximum: it is raised (and sums and accumulators rescaled) only when
// a score exceeds it by more than 8, so that in the common case a pass needs no exchange between
// lanes; p stays below 2^8 and the quotient of accumulator and sum does not depend on m.  m is
// always a whole number (the maximum rounded up), so that the bfloat16 rounding of p gives the same
// significant bits whatever m is: the weights do not depend on how the keys are cut into passes,
// stages and ranges, and a raised reference rescales by an exact power of two.  The sum
// of a query's p is one more row of the second product (a row of ones in V^T), so that numerator
// and denominator are sums of the same rounded values.
//
// Few rows over many keys (a late portion of a long prompt) would leave most of the chip idle: then
// the keys of a workgroup are cut into `splits` ranges of whole 64-key stages, one workgroup a range
// (blockIdx.y), each writes its reference, sum and unnormalised accumulator per (row, head, range),
// and a second kernel merges the ranges in order.
#include "common.h"
#include "leone_hip.h"
#include "prefill_order.h"

#include <math.h>

namespace leone {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int kPrefillWaves = 4;
constexpr int kPrefillThreads = kPrefillWaves * kWave;
constexpr int kColsPerWave = 2;                                  // 16-query operands a wave carries
constexpr int kRowsPerWave = 16 * kColsPerWave;                  // rows of a tile
constexpr int kStageKeys = 64;                                   // keys copied to shared memory at a time
constexpr int kKeysPerPass = 32;                                 // keys of one pass of a wave
constexpr float kRaise = 8.0f;                                   // a score this far above the reference raises it

__device__ inline bf16x8 pf_bits(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

// Runs of 16 bytes one stage holds: keys [head_dim / 8][64], values [8][head_dim].
__host__ __device__ constexpr int stage_runs(int head_dim) { return (head_dim / 8) * kStageKeys + 8 * head_dim; }

// tiles: [n_groups][4][3] = (entry, first row of the tile in the step, rows in the tile); a tile has at
// most 32 rows, 0 rows marks an unused place; the tiles of a group belong to one entry.
template <int kD16>
__global__ void __launch_bounds__(kPrefillThreads, 2)
attention_prefill_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ k_pool,
                         const bf16_t* __restrict__ v_pool, const int* __restrict__ positions,
                         const int* __restrict__ tiles, int n_groups, const int* __restrict__ block_table,
                         int max_blocks, int q_heads, int kv_heads, int page_shift, float scale, int window,
                         float* __restrict__ part_acc, float* __restrict__ part_ml, int splits) {
    constexpr int kD = kD16 * 16;
    constexpr int kRuns = kD / 8;                      // 16-byte runs of one key
    constexpr int kSteps = (kD16 + 1) / 2;             // 32-element steps of the first product
    constexpr int kKeyRuns = kRuns * kStageKeys;       // runs of the keys of one stage; the values take as many
    constexpr int kStageRuns = stage_runs(kD);
    constexpr int kCopies = (kKeyRuns + kPrefillThreads - 1) / kPrefillThreads;   // runs a thread copies, keys and values each

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x % kWave;
    const int tid = threadIdx.x;
    const int c = lane & 15, g = lane >> 4;

    // Which head and tile group this workgroup takes (an order that suits the dies' caches: prefill_order.h).
    const PrefillWork work = prefill_work(static_cast<int>(blockIdx.x), q_heads, n_groups);
    const int head = work.head, group = work.group;
    const int kvh = head / (q_heads / kv_heads);
    const int page_tokens = 1 << page_shift, page_mask = page_tokens - 1;

    extern __shared__ uint4 shared[];
    int* pages = reinterpret_cast<int*>(shared + 2 * kStageRuns);
    __shared__ int wave_lo[kPrefillWaves], wave_hi[kPrefillWaves];
    __shared__ int unmapped_seen;

    // This wave's tile.
    const int* my_tile = tiles + 3 * (static_cast<long>(group) * kPrefillWaves + wave);
    const int entry = tiles[3 * static_cast<long>(group) * kPrefillWaves];
    const int tile_row0 = my_tile[1];
    const int wave_rows = my_tile[2];
    const int p0 = wave_rows > 0 ? positions[tile_row0] : 0;    // rows of a portion are consecutive positions
    const int p_last = p0 + wave_rows - 1;
    const int key_hi = wave_rows > 0 ? p_last + 1 : 0;          // keys the wave may read: [key_lo, key_hi)
    const int key_lo = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
    // A pass wholly inside [full_lo, full_hi) is visible to every row of the wave: no masks.
    const int full_hi = p0 + 1;
    const int full_lo = (window > 0 && p_last - window + 1 > 0) ? p_last - window + 1 : 0;
    if (lane == 0) {
        wave_lo[wave] = wave_rows > 0 ? key_lo : 0x7fffffff;
        wave_hi[wave] = key_hi;
    }
    if (tid == 0) unmapped_seen = 0;
    __syncthreads();
    int group_lo = 0x7fffffff, group_hi = 0;
#pragma unroll
    for (int w = 0; w < kPrefillWaves; ++w) {
        group_lo = wave_lo[w] < group_lo ? wave_lo[w] : group_lo;
        group_hi = wave_hi[w] > group_hi ? wave_hi[w] : group_hi;
    }
    if (group_hi <= group_lo) return;                            // a group without rows (every wave agrees)
    if (splits > 1) {
        // This workgroup's share of the group's stages; what is outside it is treated like keys outside
        // the group's range.
        const int s_begin = group_lo / kStageKeys, s_end = (group_hi + kStageKeys - 1) / kStageKeys;
        const int share = (s_end - s_begin + splits - 1) / splits;
        const int mine_lo = (s_begin + static_cast<int>(blockIdx.y) * share) * kStageKeys;
        const int mine_hi = mine_lo + share * kStageKeys;
        group_lo = mine_lo > group_lo ? mine_lo : group_lo;
        group_hi = mine_hi < group_hi ? mine_hi : group_hi;
        if (group_hi <= group_lo) {                              // more ranges than stages: this one is empty
            if (g == 0) {
#pragma unroll
                for (int j = 0; j < kColsPerWave; ++j) {
                    const int r = 16 * j + c;
                    if (r >= wave_rows) continue;
                    const long slot = (static_cast<long>(tile_row0 + r) * q_heads + head) * splits + blockIdx.y;
                    part_ml[2 * slot] = -INFINITY;
                    part_ml[2 * slot + 1] = 0.f;
                }
            }
            return;
        }
    }

    // The page ids of the keys the group reads go to shared memory first, so that no load of keys or
    // values waits on a read of the block table.
    const int first_page = group_lo >> page_shift;
    const int n_pages = ((group_hi - 1) >> page_shift) - first_page + 1;
    const int* table = block_table + static_cast<long>(entry) * max_blocks;
    for (int i = tid; i < n_pages; i += kPrefillThreads) pages[i] = table[first_page + i];
    __syncthreads();

    // Q^T operands and each column's own position.
    bf16x8 qreg[kColsPerWave][kSteps];
    int col_pos[kColsPerWave];
#pragma unroll
    for (int j = 0; j < kColsPerWave; ++j) {
        const int r = 16 * j + c;
        const bool ok = r < wave_rows;
        col_pos[j] = ok ? p0 + r : -1;                                          // -1: the column sees no key
        const bf16_t* qrow = q + (static_cast<long>(tile_row0 + (ok ? r : 0)) * q_heads + head) * kD;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const int d0 = 32 * s + 8 * g;
            qreg[j][s] = (ok && d0 < kD) ? pf_bits(*reinterpret_cast<const uint4*>(qrow + d0)) : pf_bits(uint4{0u, 0u, 0u, 0u});
        }
    }

    // Per column: the reference m (base-2 units), the accumulator, and the sum of p as one more
    // accumulator tile (every row of it holds the sum).
    float m_ref[kColsPerWave];
    floatx4 acc[kColsPerWave][kD16], acc_sum[kColsPerWave];
#pragma unroll
    for (int j = 0; j < kColsPerWave; ++j) {
        m_ref[j] = -INFINITY;
        acc_sum[j] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < kD16; ++dt) acc[j][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    const float to_log2 = scale * 1.44269504088896340736f;
    const bf16x8 ones = pf_bits(uint4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u});

    // ---- copying a stage: keys [64 t, 64 t + 64) from the cache into registers, then into shared memory.
    // Copy i of a thread is run `idx / 64` of key `idx % 64` and, of the values, element `idx % kD`
    // of the eight keys from `8 (idx / kD)`, with idx = i * threads + tid.
    const long page_elems = static_cast<long>(page_tokens) * kD;
    const long head_elems = static_cast<long>(kvh) * page_elems;
    const long pool_stride = static_cast<long>(kv_heads) * page_elems;
    uint4 held_k[kCopies], held_v[kCopies];
    // A stage that lies inside one page and inside the group's keys needs one page id and no masks: its
    // runs go from the cache straight into shared memory, no register in between.  Such a load puts the 64
    // runs of a wave one after the other from a place in shared memory that is the same for the wave, each
    // lane naming the address it reads: so the lane that fills place L of the stage reads the run that
    // belongs there (for the keys, the order the first product's operand wants, see `deposit`).
    constexpr int kGroups = kKeyRuns / kWave;                       // loads of 64 runs that make up the keys of a stage
    constexpr int kDirect = (kGroups + kPrefillWaves - 1) / kPrefillWaves;
    auto fetch_direct = [&](int key_base, int page, uint4* to) {
        const int in_page = key_base & page_mask;
        const bf16_t* kp = k_pool + page * pool_stride + head_elems + static_cast<long>(in_page) * 8;
        const bf16_t* vp = v_pool + page * pool_stride + head_elems + static_cast<long>(in_page >> 3) * kD * 8;
        // place -> key of the 32-key half: the inverse of `deposit`'s order
        const int place = lane & 31;
        const int kk = ((place >> 2) & 3) * 8 + (place >> 4) * 4 + (place & 3);
#pragma unroll
        for (int i = 0; i < kDirect; ++i) {
            const int group = i * kPrefillWaves + wave;               // the same for the whole wave
            if (kGroups % kPrefillWaves != 0 && group >= kGroups) continue;
            const int q = 2 * group + (lane >> 5);                    // (half, run) of this lane's place
            const int half = q / kRuns, run = q % kRuns;
            const bf16_t* k_from = kp + (static_cast<long>(run) * page_tokens + 32 * half + kk) * 8;
            const bf16_t* v_from = vp + (static_cast<long>(group) * kWave + lane) * 8;
            __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(k_from), to + group * kWave, 16, 0, 0);
            __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(v_from), to + kKeyRuns + group * kWave, 16, 0, 0);
        }
    };
    auto fetch_any = [&](int key_base) {
#pragma unroll
        for (int i = 0; i < kCopies; ++i) {
            const int idx = i * kPrefillThreads + tid;
            held_k[i] = uint4{0u, 0u, 0u, 0u};
            held_v[i] = uint4{0u, 0u, 0u, 0u};
            if (kKeyRuns % kPrefillThreads != 0 && idx >= kKeyRuns) continue;
            {
                const int run = idx / kStageKeys, key = key_base + idx % kStageKeys;
                if (key >= group_lo && key < group_hi) {
                    const int page = pages[(key >> page_shift) - first_page];
                    if (page < 0) {
                        unmapped_seen = 1;
                    } else {
                        held_k[i] = *reinterpret_cast<const uint4*>(
                            k_pool + page * pool_stride + head_elems + (static_cast<long>(run) * page_tokens + (key & page_mask)) * 8);
                    }
                }
            }
            {
                const int tg = idx / kD, d = idx % kD, key = key_base + 8 * tg;
                if (key < group_hi && key + 8 > group_lo) {
                    const int page = pages[(key >> page_shift) - first_page];
                    if (page < 0) {
                        unmapped_seen = 1;
                    } else {
                        uint4 raw = *reinterpret_cast<const uint4*>(
                            v_pool + page * pool_stride + head_elems + (static_cast<long>((key & page_mask) >> 3) * kD + d) * 8);
                        if (key < group_lo || key + 8 > group_hi) {   // slots outside the range can hold anything: clear them
                            unsigned* w = reinterpret_cast<unsigned*>(&raw);
#pragma unroll
                            for (int h = 0; h < 4; ++h) {
                                const int e0 = key + 2 * h, e1 = e0 + 1;
                                unsigned mask = 0u;
                                if (e0 >= group_lo && e0 < group_hi) mask |= 0x0000ffffu;
                                if (e1 >= group_lo && e1 < group_hi) mask |= 0xffff0000u;
                                w[h] &= mask;
                            }
                        }
                        held_v[i] = raw;
                    }
                }
            }
        }
    };
    // Starts bringing stage t to `to`.  True: the runs are on their way to shared memory by themselves and
    // only have to be waited for; false: they are on their way to registers and `deposit` has to follow.
    auto fetch = [&](int t, uint4* to) -> bool {
        const int key_base = t * kStageKeys;
        if (page_shift >= 6 && key_base >= group_lo && key_base + kStageKeys <= group_hi) {
            const int page = __builtin_amdgcn_readfirstlane(pages[(key_base >> page_shift) - first_page]);
            if (page >= 0) {
                fetch_direct(key_base, page, to);
                return true;
            }
        }
        fetch_any(key_base);
        return false;
    };
    auto arrived = [&]() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };
    auto deposit = [&](uint4* to) {
#pragma unroll
        for (int i = 0; i < kCopies; ++i) {
            const int idx = i * kPrefillThreads + tid;
            if (kKeyRuns % kPrefillThreads != 0 && idx >= kKeyRuns) continue;
            // Key kk of a 32-key half sits where the first product's operand row reads it: rows 0..15 are
            // keys 8 (r / 4) + r % 4, rows 16..31 the keys four further on.
            const int run = idx / kStageKeys, kl = idx % kStageKeys;
            const int half = kl >> 5, kk = kl & 31;
            const int place = ((kk >> 2) & 1) * 16 + 4 * (kk >> 3) + (kk & 3);
            to[(half * kRuns + run) * 32 + place] = held_k[i];
            to[kKeyRuns + idx] = held_v[i];
        }
    };

    // ---- one pass of a wave: 32 keys against its 32 rows
    auto pass = [&](const uint4* from, int key0, int half, bool full) {
        const int run0 = key0 + 8 * g;                         // the lane's eight keys in the second product
        bf16x8 xa[kSteps], xb[kSteps];
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const bool in_head = 4 * s + g < kRuns;
            const uint4* row = from + (half * kRuns + 4 * s + g) * 32;
            xa[s] = in_head ? pf_bits(row[c]) : pf_bits(uint4{0u, 0u, 0u, 0u});
            xb[s] = in_head ? pf_bits(row[16 + c]) : pf_bits(uint4{0u, 0u, 0u, 0u});
        }
        float sc[kColsPerWave][8];
        float top[kColsPerWave];
#pragma unroll
        for (int j = 0; j < kColsPerWave; ++j) {
            floatx4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < kSteps; ++s) {
                sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[s], qreg[j][s], sa, 0, 0, 0);
                sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xb[s], qreg[j][s], sb, 0, 0, 0);
            }
            // lane (g, c): scores of keys run0 .. run0+7 for the query of column c
#pragma unroll
            for (int i = 0; i < 8; ++i) sc[j][i] = i < 4 ? sa[i & 3] : sb[i & 3];
        }
        if (!full) {                                           // the same for the whole wave
#pragma unroll
            for (int j = 0; j < kColsPerWave; ++j) {
                const int p = col_pos[j];
                const int p_lo = (window > 0) ? p - window + 1 : 0;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int key = run0 + i;
                    sc[j][i] = (key <= p && key >= p_lo) ? sc[j][i] : -INFINITY;
                }
            }
        }
        bool raise = false;
#pragma unroll
        for (int j = 0; j < kColsPerWave; ++j) {
            top[j] = fmaxf(fmaxf(fmaxf(sc[j][0], sc[j][1]), fmaxf(sc[j][2], sc[j][3])),
                           fmaxf(fmaxf(sc[j][4], sc[j][5]), fmaxf(sc[j][6], sc[j][7]))) * to_log2;
            raise = raise || top[j] > m_ref[j] + kRaise;       // -inf + 8 is -inf: the first scores always raise
        }
        if (__any(raise)) {
            // Some score outgrew its reference: every column takes its true maximum so far as the new one.
#pragma unroll
            for (int j = 0; j < kColsPerWave; ++j) {
                float col_top = fmaxf(top[j], __shfl_xor(top[j], 16, kWave));
                col_top = fmaxf(col_top, __shfl_xor(col_top, 32, kWave));
                const float m_new = fmaxf(m_ref[j], ceilf(col_top));     // a whole number: see the rounding of the weights below
                const float alpha = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_ref[j] - m_new);   // 2^-inf = 0
                m_ref[j] = m_new;
#pragma unroll
                for (int r = 0; r < 4; ++r) acc_sum[j][r] *= alpha;
#pragma unroll
                for (int dt = 0; dt < kD16; ++dt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[j][dt][r] *= alpha;
            }
        }
        bf16x8 pt[kColsPerWave];
#pragma unroll
        for (int j = 0; j < kColsPerWave; ++j) {
            const float shift = m_ref[j] == -INFINITY ? 0.f : -m_ref[j];   // a column that has seen no key yet
#pragma unroll
            for (int i = 0; i < 8; ++i)
                pt[j][i] = static_cast<__bf16>(__builtin_amdgcn_exp2f(fmaf(sc[j][i], to_log2, shift)));
            acc_sum[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pt[j], acc_sum[j], 0, 0, 0);
        }
#pragma unroll
        for (int dt = 0; dt < kD16; ++dt) {
            const bf16x8 xv = pf_bits(from[kKeyRuns + (4 * half + g) * kD + 16 * dt + c]);
#pragma unroll
            for (int j = 0; j < kColsPerWave; ++j)
                acc[j][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xv, pt[j], acc[j][dt], 0, 0, 0);
        }
    };

    const int t_begin = group_lo / kStageKeys, t_end = (group_hi + kStageKeys - 1) / kStageKeys;
    if (!fetch(t_begin, shared)) deposit(shared);
    arrived();
    __syncthreads();
    // One round: start bringing the next stage to `writing`, work on the present one in `reading`.  The two
    // are told apart for the compiler (they never overlap), so that it does not wait for the runs on their way
    // to `writing` before it reads `reading`.
    auto round = [&](const uint4* __restrict__ reading, uint4* __restrict__ writing, int t, bool more) {
        // `writing` was last read before the barrier that ended the round before: it is free.  The next
        // stage is sent for between the two halves (measured: better than before the first half, where its
        // arrival in shared memory gets in the way of the reads of both halves).
        bool direct = false;
#pragma unroll
        for (int half = 0; half < kStageKeys / kKeysPerPass; ++half) {
            const int key0 = t * kStageKeys + half * kKeysPerPass;
            if (half == kStageKeys / kKeysPerPass - 1) direct = more && fetch(t + 1, writing);
            if (key0 >= key_hi || key0 + kKeysPerPass <= key_lo) continue;      // nothing of it for this wave
            pass(reading, key0, half, key0 >= full_lo && key0 + kKeysPerPass <= full_hi);
        }
        if (more && !direct) deposit(writing);
    };
    int cur = 0;
    for (int t = t_begin; t < t_end; ++t) {
        round(shared + cur * kStageRuns, shared + (cur ^ 1) * kStageRuns, t, t + 1 < t_end);
        arrived();
        __syncthreads();
        cur ^= 1;
    }

    const bool poisoned = unmapped_seen != 0;                    // every write to it came before the last barrier
    if (splits > 1) {
#pragma unroll
        for (int j = 0; j < kColsPerWave; ++j) {
            const int r = 16 * j + c;
            if (r >= wave_rows) continue;
            const long slot = (static_cast<long>(tile_row0 + r) * q_heads + head) * splits + blockIdx.y;
            if (g == 0) {
                part_ml[2 * slot] = m_ref[j];
                part_ml[2 * slot + 1] = poisoned ? __builtin_nanf("") : acc_sum[j][0];
            }
            if (m_ref[j] == -INFINITY) continue;                 // no key of this range for the row: nothing to merge
#pragma unroll
            for (int dt = 0; dt < kD16; ++dt)
                *reinterpret_cast<floatx4*>(part_acc + slot * kD + 16 * dt + 4 * g) = acc[j][dt];
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < kColsPerWave; ++j) {
        const int r = 16 * j + c;
        if (r >= wave_rows) continue;
        const float inv = poisoned ? __builtin_nanf("") : 1.0f / acc_sum[j][0];
        bf16_t* orow = out + (static_cast<long>(tile_row0 + r) * q_heads + head) * kD;
#pragma unroll
        for (int dt = 0; dt < kD16; ++dt) {
            // lane (g, c) holds elements 16dt + 4g .. +3 of query column c
            uint2 packed;
            packed.x = bf16_bits_from_float(acc[j][dt][0] * inv) |
                       (static_cast<uint32_t>(bf16_bits_from_float(acc[j][dt][1] * inv)) << 16);
            packed.y = bf16_bits_from_float(acc[j][dt][2] * inv) |
                       (static_cast<uint32_t>(bf16_bits_from_float(acc[j][dt][3] * inv)) << 16);
            *reinterpret_cast<uint2*>(orow + 16 * dt + 4 * g) = packed;
        }
    }
}

// Merges the key ranges of one row and query head: out = sum_s acc_s 2^(m_s - M) / sum_s l_s 2^(m_s - M),
// the sums taken in range order; a range that held no key for the row (m_s = -inf) counts as nothing,
// whatever its accumulator holds.  One wave a (row, head): lane s takes the reference and sum of range s,
// then all lanes walk the accumulators together.  blockIdx.x is a tile and a quarter of its rows.
constexpr int kMergeWaves = 4;
constexpr int kMergeThreads = kMergeWaves * kWave;
constexpr int kMergeBlocksPerTile = kRowsPerWave / kMergeWaves / 2;   // a wave takes two rows, one after the other
constexpr int kMaxPrefillSplits = 32;

__global__ void __launch_bounds__(kMergeThreads)
attention_prefill_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                               bf16_t* __restrict__ out, const int* __restrict__ tiles, int q_heads, int head_dim,
                               int splits) {
    const int* tile = tiles + 3 * static_cast<long>(blockIdx.x / kMergeBlocksPerTile);
    const int row0 = tile[1], rows = tile[2], head = blockIdx.y;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    for (int r = (blockIdx.x % kMergeBlocksPerTile) * kMergeWaves + wave; r < rows; r += kMergeWaves * kMergeBlocksPerTile) {
        const long rh = static_cast<long>(row0 + r) * q_heads + head;
        const float2 ml = lane < splits ? reinterpret_cast<const float2*>(part_ml)[rh * splits + lane]
                                        : float2{-INFINITY, 0.f};
        const float top = wave_max(ml.x);
        const bool counts = ml.x != -INFINITY;
        const float my_weight = counts ? __builtin_amdgcn_exp2f(ml.x - top) : 0.f;
        // A range without keys for this row has sum 0; a sum that is NaN (a key without a page) still shows.
        const float my_share = counts || ml.y != ml.y ? ml.y * (counts ? my_weight : 1.f) : 0.f;
        float den = 0.f;
        float num[4] = {0.f, 0.f, 0.f, 0.f};                     // head_dim <= 256: at most four elements a lane
        const float* acc = part_acc + rh * splits * head_dim;
        for (int s = 0; s < splits; ++s) {
            const float weight = __shfl(my_weight, s, kWave);
            den += __shfl(my_share, s, kWave);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int d = lane + kWave * i;
                if (d < head_dim) {
                    const float value = acc[static_cast<long>(s) * head_dim + d];   // may be anything where weight is 0
                    num[i] += weight != 0.f ? value * weight : 0.f;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int d = lane + kWave * i;
            if (d < head_dim) out[rh * head_dim + d] = from_float<bf16_t>(num[i] / den);
        }
    }
}

template <int kD16>
static int launch_prefill(const void* q, void* out, const void* k_pool, const void* v_pool, const int* positions,
                          const int* tiles, int n_groups, const int* block_table, int max_blocks, int q_heads,
                          int kv_heads, int page_shift, float scale, int window, float* part_acc, float* part_ml,
                          int splits, hipStream_t stream) {
    const size_t shared = 2 * static_cast<size_t>(stage_runs(16 * kD16)) * sizeof(uint4) + static_cast<size_t>(max_blocks) * sizeof(int);
    static size_t allowed = 48 * 1024;                 // what a kernel may use without asking
    if (shared > allowed) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_prefill_kernel<kD16>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(shared));
        if (e != hipSuccess) {
            set_error("attention_prefill: %zu bytes of shared memory were refused: %s", shared, hipGetErrorString(e));
            return 1;
        }
        allowed = shared;
    }
    attention_prefill_kernel<kD16><<<dim3(n_groups * q_heads, splits), kPrefillThreads, shared, stream>>>(
        static_cast<const bf16_t*>(q), static_cast<bf16_t*>(out), static_cast<const bf16_t*>(k_pool),
        static_cast<const bf16_t*>(v_pool), positions, tiles, n_groups, block_table, max_blocks, q_heads, kv_heads,
        page_shift, scale, window, part_acc, part_ml, splits);
    return 0;
}

}  // namespace leone

using namespace leone;

extern "C" int leone_attention_prefill_tile_rows() { return kRowsPerWave; }
extern "C" int leone_attention_prefill_group_tiles() { return kPrefillWaves; }

extern "C" int leone_attention_prefill_max_splits() { return kMaxPrefillSplits; }

// tiles holds n_groups * leone_attention_prefill_group_tiles() entries of (entry, first row, rows).
// splits > 1 cuts every workgroup's keys into that many ranges and needs the workspace: part_acc of
// rows * q_heads * splits * head_dim floats and part_ml of rows * q_heads * splits * 2, `rows` being one
// more than the last row any tile names; with splits == 1 both may be null.
extern "C" int leone_attention_prefill(const void* q, void* out, const void* k_pool, const void* v_pool,
                                       const int* positions, const int* tiles, int n_groups, const int* block_table,
                                       int max_blocks, int q_heads, int kv_heads, int head_dim, int page_tokens,
                                       float scale, int window, float* part_acc, float* part_ml, int splits,
                                       hipStream_t stream) {
    LEONE_REQUIRE(q && out && k_pool && v_pool && positions && tiles && block_table, "attention_prefill: null pointer");
    LEONE_REQUIRE(n_groups > 0 && q_heads > 0 && kv_heads > 0 && q_heads % kv_heads == 0,
                  "attention_prefill: %d tile groups, %d query heads over %d kv heads", n_groups, q_heads, kv_heads);
    LEONE_REQUIRE(static_cast<long>(n_groups) * q_heads <= 0x7fffffffL, "attention_prefill: too many tile groups");
    LEONE_REQUIRE(head_dim % 16 == 0 && head_dim >= 16 && head_dim <= 128,
                  "attention_prefill: head_dim %d must be a multiple of 16 in 16..128", head_dim);
    LEONE_REQUIRE(page_tokens >= 16 && (page_tokens & (page_tokens - 1)) == 0,
                  "attention_prefill: page_tokens %d must be a power of two, at least 16", page_tokens);
    LEONE_REQUIRE(window >= 0 && max_blocks > 0, "attention_prefill: bad window or block table");
    LEONE_REQUIRE(scale > 0.f, "attention_prefill: the score scale must be positive");
    LEONE_REQUIRE(splits >= 1 && splits <= kMaxPrefillSplits, "attention_prefill: splits %d must be in 1..%d", splits,
                  kMaxPrefillSplits);
    LEONE_REQUIRE(splits == 1 || (part_acc && part_ml), "attention_prefill: %d key ranges need the workspace", splits);
    LEONE_REQUIRE(q_heads <= 65535, "attention_prefill: too many heads for one launch");
    LEONE_REQUIRE(static_cast<size_t>(max_blocks) * sizeof(int) <= 16 * 1024,
                  "attention_prefill: a block table of %d entries does not fit shared memory", max_blocks);
    int page_shift = 0;
    while ((1 << page_shift) < page_tokens) ++page_shift;
    int status = 0;
#define LEONE_PREFILL_CASE(N)                                                                                      \
    case N:                                                                                                        \
        status = launch_prefill<N>(q, out, k_pool, v_pool, positions, tiles, n_groups, block_table, max_blocks,    \
                                   q_heads, kv_heads, page_shift, scale, window, part_acc, part_ml, splits,        \
                                   stream);                                                                        \
        break;
    switch (head_dim / 16) {
        LEONE_PREFILL_CASE(1) LEONE_PREFILL_CASE(2) LEONE_PREFILL_CASE(3) LEONE_PREFILL_CASE(4)
        LEONE_PREFILL_CASE(5) LEONE_PREFILL_CASE(6) LEONE_PREFILL_CASE(7) LEONE_PREFILL_CASE(8)
        default:
            set_error("attention_prefill: head_dim %d is not supported", head_dim);
            return 1;
    }
#undef LEONE_PREFILL_CASE
    if (status) return status;
    LEONE_LAUNCH_CHECK("attention_prefill");
    if (splits > 1) {
        attention_prefill_merge_kernel<<<dim3(n_groups * kPrefillWaves * kMergeBlocksPerTile, q_heads), kMergeThreads, 0,
                                         stream>>>(
            part_acc, part_ml, static_cast<bf16_t*>(out), tiles, q_heads, head_dim, splits);
        LEONE_LAUNCH_CHECK("attention_prefill_merge");
    }
    return 0;
}
