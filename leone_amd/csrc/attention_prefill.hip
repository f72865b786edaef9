// Causal attention of prompt portions over the paged cache on the matrix cores, bfloat16.
//
// A portion's rows are cut into tiles of 32 consecutive rows; a wave takes one tile and one query
// head, its rows as one 32-column operand.  A workgroup is four waves whose tiles belong to the
// same request (the host lists them: entry, first row, row count, four to a workgroup).  The
// workgroup walks the keys its tiles can see once, 64 at a time: the next 64 keys and values travel
// from the cache to shared memory while the waves work on the present 64 (by loads that write to
// shared memory themselves; a stage at the edge of the keys or across pages goes through registers,
// where it is masked), and every wave takes from shared memory the 32-key halves its own rows can see.  A wave keeps the
// running reference, sum and accumulator of the reference's recurrence
// (crates/leone/src/cpu.rs:2359-2421) per query in registers; nothing of size rows x keys is ever
// stored (the reference's prefill materialises the scores, crates/leone-cuda/cuda/ie_cuda.cu:5124-5220).
// The products are those of the decode kernel, S^T = K . Q^T and O^T += V^T . P^T, on 16-byte runs of the
// packed cache layout, but with v_mfma_f32_32x32x16_bf16: 32 keys against 32 rows an instruction.  That
// instruction does twice the work of the 16 x 16 x 32 one for the same operand registers, and operand
// reads are what holds the small one back (measured in a register loop: 2.45 against 1.4-1.6 PFLOP/s).
// Lane L gives row L % 32 of the first operand and column L % 32 of the second, elements 8 (L / 32) .. + 7 of
// the 16 that are summed over, and gets column L % 32 of the result, rows 8 (v / 4) + 4 (L / 32) + v % 4
// in register v.  Keys are stored in shared memory in the order in which the first product's rows want
// them, chosen so that a lane's scores are those of 8 + 8 neighbouring keys: they go into the second
// product as they are.
//
// The recurrence is kept in base-2 units: t = score * scale * log2(e), p = 2^(t - m).  m is a
// reference, not always the maximum: it is raised (and sums and accumulators rescaled) only when
// a score exceeds it by more than 8, so that in the common case a pass needs no exchange between
// lanes; p stays below 2^8 and the quotient of accumulator and sum does not depend on m.  m is
// always a whole number (the maximum rounded up), so that the bfloat16 rounding of p gives the same
// significant bits whatever m is: the weights do not depend on how the keys are cut into passes,
// stages and ranges, and a raised reference rescales by an exact power of two.  The sum
// of a query's p is taken over the rounded values, key by key, so that numerator and denominator are
// sums of the same numbers.
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
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;

constexpr int kPrefillWaves = 4;
constexpr int kPrefillThreads = kPrefillWaves * kWave;
constexpr int kRowsPerWave = 32;                                 // rows of a tile: one operand of the matrix instruction
constexpr int kStageKeys = 64;                                   // keys copied to shared memory at a time
constexpr int kKeysPerPass = 32;                                 // keys of one pass of a wave
constexpr float kRaise = 8.0f;                                   // a score this far above the reference raises it

__device__ inline bf16x8 pf_bits(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

// Which key of a 32-key pass sits in row r of the first product's operand, and in which row key k sits: the
// same swap of two bits either way.  Rows 8 b + 4 h + i (b 0..3, i 0..3) are what lane half h gets of the
// result; with this order they are keys 8 h + 0..7 (b 0, 1) and 16 + 8 h + 0..7 (b 2, 3).
__device__ inline int pass_key_or_row(int x) { return (x & 0x13) | ((x & 4) << 1) | ((x & 8) >> 1); }

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
    constexpr int kDT = (kD + 31) / 32;                // 32-row tiles of the second product's result
    constexpr int kKeyRuns = kRuns * kStageKeys;       // runs of the keys of one stage; the values take as many
    constexpr int kStageRuns = stage_runs(kD);
    constexpr int kCopies = (kKeyRuns + kPrefillThreads - 1) / kPrefillThreads;   // runs a thread copies, keys and values each

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x % kWave;
    const int tid = threadIdx.x;
    const int j = lane & 31, h = lane >> 5;            // this lane's row of the tile, and which half of the summed-over elements

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
            if (h == 0 && j < wave_rows) {
                const long slot = (static_cast<long>(tile_row0 + j) * q_heads + head) * splits + blockIdx.y;
                part_ml[2 * slot] = -INFINITY;
                part_ml[2 * slot + 1] = 0.f;
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

    // The Q^T operand and the row's own position.
    const bool row_ok = j < wave_rows;
    const int row_pos = row_ok ? p0 + j : -1;                                   // -1: the row sees no key
    bf16x8 qreg[kD16];
    {
        const bf16_t* qrow = q + (static_cast<long>(tile_row0 + (row_ok ? j : 0)) * q_heads + head) * kD;
#pragma unroll
        for (int s = 0; s < kD16; ++s)
            qreg[s] = row_ok ? pf_bits(*reinterpret_cast<const uint4*>(qrow + 16 * s + 8 * h)) : pf_bits(uint4{0u, 0u, 0u, 0u});
    }

    // Per row: the reference m (base-2 units), the sum of p over this lane's half of the keys, and the
    // accumulator (register v of tile dt: element 32 dt + 8 (v / 4) + 4 h + v % 4 of the row's result).
    float m_ref = -INFINITY, l_run = 0.f;
    floatx16 acc[kDT];
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[dt][v] = 0.f;
    const float to_log2 = scale * 1.44269504088896340736f;

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
        // place -> key of the 32-key half, as in `deposit`
        const int kk = pass_key_or_row(lane & 31);
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
            // Key kk of a 32-key half sits where the first product's operand row reads it.
            const int run = idx / kStageKeys, kl = idx % kStageKeys;
            const int half = kl >> 5, kk = kl & 31;
            const int place = pass_key_or_row(kk);
            to[(half * kRuns + run) * 32 + place] = held_k[i];
            to[kKeyRuns + idx] = held_v[i];
        }
    };

    // ---- one pass of a wave: 32 keys against its 32 rows
    auto pass = [&](const uint4* from, int key0, int half, bool full) {
        // Two sums, over the even and the odd steps, so that no instruction waits for the one before.
        floatx16 sc, sc_odd;
#pragma unroll
        for (int v = 0; v < 16; ++v) sc[v] = sc_odd[v] = 0.f;
        // All of the pass's keys are asked for from shared memory at once and the values right after the first
        // product's instructions, so that the way out of shared memory is waited for once a pass and the
        // values come while the weights are made.  (Left to the compiler the reads come in pairs right before
        // the instruction that needs them, a wait each, which a wave that has its SIMD to itself sits out.)
        bf16x8 xk[kD16];
#pragma unroll
        for (int s = 0; s < kD16; ++s) {
            // operand row j is key pass_key_or_row(j); this lane's elements 16 s + 8 h .. + 7 are run 2 s + h
            xk[s] = pf_bits(from[(half * kRuns + 2 * s + h) * 32 + j]);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < kD16; ++s) {
            if (s % 2 == 0) sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xk[s], qreg[s], sc, 0, 0, 0);
            else sc_odd = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xk[s], qreg[s], sc_odd, 0, 0, 0);
        }
        bf16x8 xv[2][kDT];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int dt = 0; dt < kDT; ++dt) {
                const int d = 32 * dt + j;                     // operand row j of tile dt is element d of the values
                // this lane's keys 16 ks + 8 h .. + 7 of the pass are one run of the values' layout
                xv[ks][dt] = (kD % 32 == 0 || d < kD) ? pf_bits(from[kKeyRuns + (4 * half + 2 * ks + h) * kD + d])
                                                      : pf_bits(uint4{0u, 0u, 0u, 0u});
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (kD16 > 1) {
#pragma unroll
            for (int v = 0; v < 16; ++v) sc[v] += sc_odd[v];
        }
        // lane (j, h): sc[v] is row j's score of key key0 + 8 h + v (v < 8) or key0 + 16 + 8 h + v - 8
        if (!full) {                                           // the same for the whole wave
            const int p_lo = (window > 0) ? row_pos - window + 1 : 0;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int key = key0 + 8 * h + (v & 7) + 16 * (v >> 3);
                sc[v] = (key <= row_pos && key >= p_lo) ? sc[v] : -INFINITY;
            }
        }
        float top = sc[0];
#pragma unroll
        for (int v = 1; v < 16; ++v) top = fmaxf(top, sc[v]);
        top *= to_log2;
        if (__any(top > m_ref + kRaise)) {                     // -inf + 8 is -inf: the first scores always raise
            // Some score outgrew its reference: every row takes its true maximum so far as the new one.
            const float row_top = fmaxf(top, __shfl_xor(top, 32, kWave));
            const float m_new = fmaxf(m_ref, ceilf(row_top));           // a whole number: see the rounding of the weights below
            const float alpha = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m_ref - m_new);   // 2^-inf = 0
            m_ref = m_new;
            l_run *= alpha;
#pragma unroll
            for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[dt][v] *= alpha;
        }
        const float shift = m_ref == -INFINITY ? 0.f : -m_ref;         // a row that has seen no key yet
        bf16x8 pt[2];
#pragma unroll
        for (int v = 0; v < 16; ++v)
            pt[v >> 3][v & 7] = static_cast<__bf16>(__builtin_amdgcn_exp2f(fmaf(sc[v], to_log2, shift)));
        // the sum of what the second product sees: the rounded values, two to an instruction (p . 1 + p' . 1 + sum)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const uint4 packed = __builtin_bit_cast(uint4, pt[ks]);
            const unsigned pairs[4] = {packed.x, packed.y, packed.z, packed.w};
#pragma unroll
            for (int i = 0; i < 4; ++i)
                l_run = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pairs[i]), __builtin_bit_cast(bf16x2, 0x3f803f80u),
                                                        l_run, false);
        }
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int dt = 0; dt < kDT; ++dt) acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xv[ks][dt], pt[ks], acc[dt], 0, 0, 0);
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
    const float l_row = l_run + __shfl_xor(l_run, 32, kWave);    // both halves of the keys
    if (splits > 1) {
        if (!row_ok) return;
        const long slot = (static_cast<long>(tile_row0 + j) * q_heads + head) * splits + blockIdx.y;
        if (h == 0) {
            part_ml[2 * slot] = m_ref;
            part_ml[2 * slot + 1] = poisoned ? __builtin_nanf("") : l_row;
        }
        if (m_ref == -INFINITY) return;                          // no key of this range for the row: nothing to merge
#pragma unroll
        for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int d0 = 32 * dt + 8 * b + 4 * h;
                if (kD % 32 == 0 || d0 < kD)
                    *reinterpret_cast<floatx4*>(part_acc + slot * kD + d0) =
                        floatx4{acc[dt][4 * b], acc[dt][4 * b + 1], acc[dt][4 * b + 2], acc[dt][4 * b + 3]};
            }
        return;
    }
    if (!row_ok) return;
    const float inv = poisoned ? __builtin_nanf("") : 1.0f / l_row;
    bf16_t* orow = out + (static_cast<long>(tile_row0 + j) * q_heads + head) * kD;
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int d0 = 32 * dt + 8 * b + 4 * h;              // registers 4 b .. 4 b + 3 are elements d0 .. d0 + 3
            if (kD % 32 != 0 && d0 >= kD) continue;
            uint2 packed;
            packed.x = bf16_bits_from_float(acc[dt][4 * b] * inv) |
                       (static_cast<uint32_t>(bf16_bits_from_float(acc[dt][4 * b + 1] * inv)) << 16);
            packed.y = bf16_bits_from_float(acc[dt][4 * b + 2] * inv) |
                       (static_cast<uint32_t>(bf16_bits_from_float(acc[dt][4 * b + 3] * inv)) << 16);
            *reinterpret_cast<uint2*>(orow + d0) = packed;
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
