// Split-KV attention over the paged cache on the matrix cores, bfloat16.
//
// One workgroup takes (query row, kv head, up to 16 of its query heads, one
// split of the keys); its four waves walk 32-key tiles of the split.  For a
// tile a wave computes S^T = K . Q^T (keys x heads) with
// v_mfma_f32_16x16x32_bf16, runs the running-maximum softmax of the reference
// (crates/leone/src/cpu.rs:2299-2357) in float on the accumulator registers,
// and adds O^T += V^T . P^T with the same instruction.  The softmax works in
// powers of two against a reference that is a whole number (the running
// maximum rounded up): the weights 2^(s - reference) that are rounded to
// bfloat16 for the second product then have the same significant bits
// whatever the reference, so they do not depend on how the keys are cut
// into tiles, waves and splits, and changes of the reference rescale the
// sums by exact powers of two.  The row sum is taken over the rounded
// weights, the ones the values are weighted with.  The cache packs keys
// as [element / 8][token][8] and values as [token / 8][element][8], so that
// both operands are 16-byte loads straight from the cache with the 16 lanes of
// a quarter wave on neighbouring runs, a key or value being read once for all
// query heads of its group.  The waves' partial results are
// merged in shared memory, the splits' by a second kernel, both in a fixed
// order (the reference's partial + reduce pair:
// crates/leone-cuda/cuda/ie_cuda.cu:4465, 4769).  (Letting the workgroup that
// finishes last do the merge was measured: the device-wide fences it needs
// cost far more than the second launch, 8.8 against 6.0 ms a step.)
//
// A step in which every row is another request (single decoded tokens) can leave the work on the new token's
// heads to this kernel (`FromProjection`): it takes the fused q/k/v projection as it comes, normalises and
// rotates the query heads it needs in registers (per-head RMSNorm, half-split rotation:
// crates/leone/src/backend.rs:2182-2208, crates/leone/src/cpu.rs:1721-1779), and the workgroup whose keys
// end with the row's own position does the same for the new key, writes it and the new value into the cache
// and only then walks its tiles.  One launch fewer a layer; the values are those of the separate kernel
// (rowwise.hip).  Head sizes that are multiples of 64 only: there a lane holds both halves of its pairs.
//
// Operand layouts of the 16x16x32 instruction (lane l, c = l % 16, g = l / 16):
//   A: row c,    k-slots 8g .. 8g+7        B: column c, k-slots 8g .. 8g+7
//   C/D: column c, rows 4g .. 4g+3
// Which key or element a k-slot stands for is free as long as A and B agree.
// For S^T the two 16-key halves of a tile are laid out so that lane (g, c)
// ends up with the scores of keys 8g .. 8g+7 of the tile: exactly the k-slots
// it has to supply as P^T for the second product.
#include "common.h"
#include "leone_hip.h"

#include <math.h>
#include <type_traits>

namespace leone {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int kDecodeWaves = 4;
constexpr int kDecodeThreads = kDecodeWaves * kWave;
constexpr int kTileKeys = 32;

__device__ inline bf16x8 load8(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}
__device__ inline bf16x8 load8_streamed(const bf16_t* p) {   // keys and values: read once a step
    return __builtin_bit_cast(bf16x8, load_streamed16(p));
}
__device__ inline bf16x8 zero8() {
    uint4 z = {0u, 0u, 0u, 0u};
    return __builtin_bit_cast(bf16x8, z);
}

// The fused q/k/v projection of the step's rows and what turns it into queries, keys and values.
struct FromProjection {
    const void* qkv;        // [rows, (q_heads + 2 kv_heads) * head_dim], bfloat16, or float32 in `planes` planes
    int is_float;
    int planes;
    long plane;
    AnyVec q_gain, k_gain;  // null pointers: no norm
    float eps;
    const float* cos_table; // [table_positions, head_dim / 2], or null: no rotation
    const float* sin_table;
    int table_positions;
    bf16_t* k_out;          // the pools, for the new token; null: this run writes no cache
    bf16_t* v_out;
};

// Eight elements of the projection from element offset `at` of row `row`: planes added in order, then rounded
// to bfloat16 as a stored projection would be.
__device__ inline void load_projection8(const FromProjection& f, long row_width, long row, long at, float out[8]) {
    if (!f.is_float) {
        const uint4 raw = *reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(f.qkv) + row * row_width + at);
        const unsigned w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[2 * i] = __uint_as_float(w[i] << 16);
            out[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
        return;
    }
    // The planes are asked for four at a time before any is added (a plane beyond the last is the last one again
    // and is not added): one trip to memory for up to five planes instead of one a plane.  Added in their order.
    const float* src = static_cast<const float*>(f.qkv) + row * row_width + at;
    const float4 a0 = *reinterpret_cast<const float4*>(src), b0 = *reinterpret_cast<const float4*>(src + 4);
    out[0] = a0.x; out[1] = a0.y; out[2] = a0.z; out[3] = a0.w;
    out[4] = b0.x; out[5] = b0.y; out[6] = b0.z; out[7] = b0.w;
    for (int p0 = 1; p0 < f.planes; p0 += 4) {
        float4 lo[4], hi[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float* from = src + (p0 + q < f.planes ? p0 + q : f.planes - 1) * f.plane;
            lo[q] = *reinterpret_cast<const float4*>(from);
            hi[q] = *reinterpret_cast<const float4*>(from + 4);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (p0 + q < f.planes) {
                out[0] += lo[q].x; out[1] += lo[q].y; out[2] += lo[q].z; out[3] += lo[q].w;
                out[4] += hi[q].x; out[5] += hi[q].y; out[6] += hi[q].z; out[7] += hi[q].w;
            }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = to_float(from_float<bf16_t>(out[i]));
}

// kD16 = head_dim / 16.
// Two tiles of keys and values are held at a time (one on its way, one being worked on): up to a head size of
// 64 that fits three waves a SIMD, up to 128 two; larger heads need all registers.
template <int kD16, bool kFused>
__global__ void __launch_bounds__(kDecodeThreads, kD16 <= 4 ? 3 : kD16 <= 8 ? 2 : 1)
attention_decode_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pool,
                        const bf16_t* __restrict__ v_pool, const int* __restrict__ positions,
                        const int* __restrict__ row_entry, const int* __restrict__ block_table, int max_blocks,
                        float* __restrict__ part_acc, float* __restrict__ part_ml, bf16_t* __restrict__ out,
                        int q_heads, int kv_heads, int page_shift, float to_log2, int window, int splits,
                        FromProjection from) {
    constexpr int kD = kD16 * 16;
    constexpr int kSteps = (kD16 + 1) / 2;           // 32-element steps of the q.k product
    extern __shared__ float smem[];                   // [waves][columns][kD] accumulators, then m and l

    const int group = q_heads / kv_heads;
    const int col_tiles = (group + 15) / 16;
    const int row = blockIdx.x;
    const int kvh = blockIdx.y / col_tiles;
    const int col0 = (blockIdx.y % col_tiles) * 16;
    const int cols = group - col0 < 16 ? group - col0 : 16;   // query heads handled here
    const int split = blockIdx.z;
    const int wave = threadIdx.x / kWave;
    const int lane = threadIdx.x % kWave;
    const int c = lane & 15, g = lane >> 4;
    const int page_tokens = 1 << page_shift;
    const int page_mask = page_tokens - 1;

    const int n = positions[row] + 1;                                    // keys 0 .. n-1 exist
    const int lo = (window > 0 && n - window > 0) ? n - window : 0;      // first key in reach
    const int* table = block_table + static_cast<long>(row_entry[row]) * max_blocks;
    const int t_begin = lo / kTileKeys, t_end = (n + kTileKeys - 1) / kTileKeys;
    const int per_split = (t_end - t_begin + splits - 1) / splits;
    const int my_begin = t_begin + split * per_split;
    const int my_end = my_begin + per_split < t_end ? my_begin + per_split : t_end;

    // The page ids of this split's keys go to shared memory first: no load of keys or values then
    // waits on a read of the block table.
    int* pages = reinterpret_cast<int*>(smem + kDecodeWaves * cols * (kD + 2));
    const int first_page = (my_begin * kTileKeys) >> page_shift;
    {
        const int last_key = (my_end * kTileKeys < n ? my_end * kTileKeys : n) - 1;
        const int n_pages = my_begin < my_end ? (last_key >> page_shift) - first_page + 1 : 0;
        for (int i = threadIdx.x; i < n_pages; i += kDecodeThreads) pages[i] = table[first_page + i];
    }
    if constexpr (kFused) {
        // The workgroup whose keys end with the row's own position makes that position's key and value and
        // writes them into the cache; its waves read them from there after the barrier.  (With more than 16
        // query heads a kv head several workgroups do, each for itself: the same bytes.)
        if (from.k_out != nullptr && my_begin < my_end && my_end == t_end) {
            const long width = static_cast<long>(q_heads + 2 * kv_heads) * kD;
            const int pos = n - 1;
            const int page = table[pos >> page_shift];
            if (page >= 0) {                              // the host reserves the page before the launch
                const long base = (static_cast<long>(page) * kv_heads + kvh) * page_tokens * kD;
                const int token = pos & page_mask;
                constexpr int kHalfRuns = kD16;           // runs of 8 elements in half a head
                if (wave == 0) {
                    // lane L < kHalfRuns: elements 8L .. 8L+7 and their partners in the other half
                    const bool mine = lane < kHalfRuns;
                    float a[8], b[8];
                    float ss = 0.f;
                    // gains and angles are asked for together with the projection, not after the sum of squares
                    float ga[8], gb[8], cs[8], sn[8];
                    if (mine) {
                        if (from.k_gain.ptr) {
                            load_any8(from.k_gain, 8 * lane, ga);
                            load_any8(from.k_gain, kD / 2 + 8 * lane, gb);
                        }
                        if (from.cos_table != nullptr) {
                            const int tpos = pos < from.table_positions ? pos : from.table_positions - 1;
                            load_any8(AnyVec{from.cos_table, kF32}, static_cast<long>(tpos) * (kD / 2) + 8 * lane, cs);
                            load_any8(AnyVec{from.sin_table, kF32}, static_cast<long>(tpos) * (kD / 2) + 8 * lane, sn);
                        }
                        load_projection8(from, width, row, static_cast<long>(q_heads + kvh) * kD + 8 * lane, a);
                        load_projection8(from, width, row, static_cast<long>(q_heads + kvh) * kD + kD / 2 + 8 * lane, b);
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            ss = fmaf(a[i], a[i], ss);
                            ss = fmaf(b[i], b[i], ss);
                        }
                    }
                    ss = wave_sum(ss);
                    if (mine) {
                        if (from.k_gain.ptr) {
                            const float inv = 1.0f / sqrtf(ss / static_cast<float>(kD) + from.eps);
#pragma unroll
                            for (int i = 0; i < 8; ++i) {
                                a[i] = (a[i] * ga[i]) * inv;
                                b[i] = (b[i] * gb[i]) * inv;
                            }
                        }
                        if (from.cos_table != nullptr) {
#pragma unroll
                            for (int i = 0; i < 8; ++i) {
                                const float ru = a[i] * cs[i] - b[i] * sn[i];
                                const float rv = a[i] * sn[i] + b[i] * cs[i];
                                a[i] = ru;
                                b[i] = rv;
                            }
                        }
                        uint4 lo, hi;
                        unsigned* wl = reinterpret_cast<unsigned*>(&lo);
                        unsigned* wh = reinterpret_cast<unsigned*>(&hi);
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            wl[i] = bf16_bits_from_float(a[2 * i]) | (static_cast<unsigned>(bf16_bits_from_float(a[2 * i + 1])) << 16);
                            wh[i] = bf16_bits_from_float(b[2 * i]) | (static_cast<unsigned>(bf16_bits_from_float(b[2 * i + 1])) << 16);
                        }
                        *reinterpret_cast<uint4*>(from.k_out + base + key_offset(token, 8 * lane, page_tokens)) = lo;
                        *reinterpret_cast<uint4*>(from.k_out + base + key_offset(token, kD / 2 + 8 * lane, page_tokens)) = hi;
                    }
                } else if (wave == 1) {
                    // values are copied as they are, one element of one token at a time
                    const long value_at = static_cast<long>(q_heads + kv_heads + kvh) * kD;
                    for (int e = 8 * lane; e < kD; e += 8 * kWave) {
                        float v[8];
                        load_projection8(from, width, row, value_at + e, v);
#pragma unroll
                        for (int i = 0; i < 8; ++i)
                            from.v_out[base + value_offset(token, e + i, kD)] = from_float<bf16_t>(v[i]);
                    }
                }
            }
            __threadfence_block();                         // the waves of this workgroup read what was written
        }
    }
    __syncthreads();

    // One 32-key tile in two steps: `issue` asks for its keys and values, `finish` does the arithmetic.  The
    // next tile of the wave is asked for before the present one is finished, so that a wave always has loads
    // in flight (with a row or two and a few thousand keys a wave has only a handful of tiles, and without
    // this each of them waited out the memory's latency by itself).  Every call of `issue` gives the same
    // number of load instructions whatever the tile: lanes with nothing to read (keys outside [lo, n), a key
    // without a page, no further tile) read the pool's first bytes instead and the result is cleared in
    // `finish`; the compiler counts loads in flight and would wait for all of them after a load that may or may
    // not have been issued.  `full` tiles lie wholly inside [lo, n) and need no masks; at most the first and
    // the last tile of a row are not.
    struct Tile {
        bf16x8 xa[kSteps], xb[kSteps], xv[kD16];
    };
    auto issue = [&](int t, bool exists, Tile& r) {
        const int key0 = t * kTileKeys;
        // A-operand row c of half a is key 8*(c/4) + c%4, of half b four keys further
        const int ka = key0 + 8 * (c >> 2) + (c & 3);
        const int run0 = key0 + 8 * g;                   // this lane's eight keys for the second product
        const bool near = exists && ka + 4 >= lo && ka < n;   // ka or kb = ka + 4 in reach: they share a page (pages hold multiples of 8 keys)
        const bool any = exists && run0 < n && run0 + 8 > lo;
        const int page_k = near ? pages[(ka >> page_shift) - first_page] : -1;
        const int page_v = any ? pages[(run0 >> page_shift) - first_page] : -1;
        const bf16_t* pk = page_k < 0 ? k_pool
                                      : k_pool + (static_cast<long>(page_k) * kv_heads + kvh) * page_tokens * kD + (ka & page_mask) * 8;
        const bf16_t* pv = page_v < 0 ? v_pool
                                      : v_pool + (static_cast<long>(page_v) * kv_heads + kvh) * page_tokens * kD +
                                            static_cast<long>((run0 & page_mask) >> 3) * kD * 8;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const bool in_head = 32 * s + 8 * g < kD;
            const long run = in_head ? static_cast<long>(4 * s + g) * page_tokens * 8 : 0;   // elements 32s+8g .. +7 of the key
            r.xa[s] = load8_streamed(pk + run);
            r.xb[s] = load8_streamed(pk + run + 32);           // four keys further
        }
#pragma unroll
        for (int dt = 0; dt < kD16; ++dt) r.xv[dt] = load8_streamed(pv + (16 * dt + c) * 8);
    };
    // The wave's first tile is asked for before the queries are made: neither waits for the other.
    Tile one, two;
    if (my_begin + wave < my_end) issue(my_begin + wave, true, one);

    // Q^T operand: column c is query head kvh*group + col0 + c.
    bf16x8 qreg[kSteps];
    if constexpr (kFused) {
        // Lane (c, g) holds elements 32s + 8g .. + 7 of head c for every step s; with a head size that is a
        // multiple of 64 the partner of such a run in the other half of the head is the same lane's run of
        // step s + kSteps / 2.
        static_assert(!kFused || kD16 % 4 == 0, "the fused query path needs a head size that is a multiple of 64");
        constexpr int kHalfSteps = kSteps / 2;
        const bool head_ok = c < cols;
        const long width = static_cast<long>(q_heads + 2 * kv_heads) * kD;
        const long head_at = static_cast<long>(kvh * group + col0 + (head_ok ? c : 0)) * kD;
        // everything is asked for first (heads, gains, angles), 16 or 32 bytes at a time, then worked on
        float v[kSteps][8], gain[kSteps][8], cs[kHalfSteps][8], sn[kHalfSteps][8];
        const int tpos = n - 1 < from.table_positions ? n - 1 : from.table_positions - 1;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            load_projection8(from, width, row, head_at + 32 * s + 8 * g, v[s]);
            if (from.q_gain.ptr) load_any8(from.q_gain, 32 * s + 8 * g, gain[s]);
        }
        if (from.cos_table != nullptr) {
#pragma unroll
            for (int s = 0; s < kHalfSteps; ++s) {
                load_any8(AnyVec{from.cos_table, kF32}, static_cast<long>(tpos) * (kD / 2) + 32 * s + 8 * g, cs[s]);
                load_any8(AnyVec{from.sin_table, kF32}, static_cast<long>(tpos) * (kD / 2) + 32 * s + 8 * g, sn[s]);
            }
        }
        float ss = 0.f;
#pragma unroll
        for (int s = 0; s < kSteps; ++s)
#pragma unroll
            for (int i = 0; i < 8; ++i) ss = fmaf(v[s][i], v[s][i], ss);
        ss += __shfl_xor(ss, 16, kWave);                  // the four lanes that share head c
        ss += __shfl_xor(ss, 32, kWave);
        if (from.q_gain.ptr) {
            const float inv = 1.0f / sqrtf(ss / static_cast<float>(kD) + from.eps);
#pragma unroll
            for (int s = 0; s < kSteps; ++s)
#pragma unroll
                for (int i = 0; i < 8; ++i) v[s][i] = (v[s][i] * gain[s][i]) * inv;
        }
        if (from.cos_table != nullptr) {
#pragma unroll
            for (int s = 0; s < kHalfSteps; ++s) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float a = v[s][i], b = v[s + kHalfSteps][i];
                    v[s][i] = a * cs[s][i] - b * sn[s][i];
                    v[s + kHalfSteps][i] = a * sn[s][i] + b * cs[s][i];
                }
            }
        }
#pragma unroll
        for (int s = 0; s < kSteps; ++s)
#pragma unroll
            for (int i = 0; i < 8; ++i) qreg[s][i] = head_ok ? static_cast<__bf16>(v[s][i]) : static_cast<__bf16>(0.0f);
    } else {
        const bool head_ok = c < cols;
        const bf16_t* qrow = q + (static_cast<long>(row) * q_heads + kvh * group + col0 + (head_ok ? c : 0)) * kD;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const int d0 = 32 * s + 8 * g;
            qreg[s] = (head_ok && d0 < kD) ? load8(qrow + d0) : zero8();
        }
    }

    float m_run = -INFINITY, l_run = 0.f;
    bool unmapped = false;
    floatx4 acc[kD16];
#pragma unroll
    for (int dt = 0; dt < kD16; ++dt) acc[dt] = floatx4{0.f, 0.f, 0.f, 0.f};

    auto finish = [&](int t, Tile& r) {
        const int key0 = t * kTileKeys;
        const bool full = key0 >= lo && key0 + kTileKeys <= n;      // the same for the whole wave
        const int ka = key0 + 8 * (c >> 2) + (c & 3);
        const int kb = ka + 4;
        const int run0 = key0 + 8 * g;
        bool va = ka >= lo && ka < n, vb = kb >= lo && kb < n, any = run0 < n && run0 + 8 > lo;
        if ((va || vb) && pages[(ka >> page_shift) - first_page] < 0) {
            unmapped = true;                              // never read outside the pool; the result is poisoned below
            va = vb = false;
        }
        if (any && pages[(run0 >> page_shift) - first_page] < 0) {
            unmapped = true;
            any = false;
        }
        if (!full || kD16 % 2 != 0 || __any(unmapped)) {
            // what was read in place of nothing counts as zero
#pragma unroll
            for (int s = 0; s < kSteps; ++s) {
                const bool in_head = 32 * s + 8 * g < kD;
                if (!(va && in_head)) r.xa[s] = zero8();
                if (!(vb && in_head)) r.xb[s] = zero8();
            }
            const bool whole = run0 >= lo && run0 + 8 <= n;
#pragma unroll
            for (int dt = 0; dt < kD16; ++dt) {
                if (!any) {
                    r.xv[dt] = zero8();
                } else if (!whole) {
                    // slots outside [lo, n) may hold anything, even NaN: clear them, a zero weight is not enough
                    uint4 raw = __builtin_bit_cast(uint4, r.xv[dt]);
                    unsigned* w = reinterpret_cast<unsigned*>(&raw);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int e0 = run0 + 2 * i, e1 = e0 + 1;
                        unsigned mask = 0u;
                        if (e0 >= lo && e0 < n) mask |= 0x0000ffffu;
                        if (e1 >= lo && e1 < n) mask |= 0xffff0000u;
                        w[i] &= mask;
                    }
                    r.xv[dt] = __builtin_bit_cast(bf16x8, raw);
                }
            }
        }

        // ---- S^T = K . Q^T for the two 16-key halves --------------------------------------------
        floatx4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(r.xa[s], qreg[s], sa, 0, 0, 0);
            sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(r.xb[s], qreg[s], sb, 0, 0, 0);
        }
        // lane (g, c) now holds, for query column c, the scores of keys key0 + 8g + j, j = 0..7
        float sc[8];
        float tile_max = -INFINITY;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int key = run0 + j;
            const float raw = j < 4 ? sa[j & 3] : sb[j & 3];
            sc[j] = (full || (key >= lo && key < n)) ? raw * to_log2 : -INFINITY;
            tile_max = fmaxf(tile_max, sc[j]);
        }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, kWave));
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, kWave));
        const float m_new = fmaxf(m_run, ceilf(tile_max));   // finite: every tile of the range holds a key in reach
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);   // an exact power of two (0 from -inf)
        float psum = 0.f;
        bf16x8 pt;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            pt[j] = static_cast<__bf16>(__builtin_amdgcn_exp2f(sc[j] - m_new));
            psum += static_cast<float>(pt[j]);
        }
        psum += __shfl_xor(psum, 16, kWave);
        psum += __shfl_xor(psum, 32, kWave);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        // ---- O^T += V^T . P^T ------------------------------------------------------------------
#pragma unroll
        for (int dt = 0; dt < kD16; ++dt) {
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) acc[dt][r4] *= alpha;
            acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(r.xv[dt], pt, acc[dt], 0, 0, 0);
        }
    };

    // Two tiles in turn: while one is finished the other is on its way.  After its last tile the wave asks
    // for a tile that does not exist (see `issue`).
    if constexpr (kD16 > 8) {                           // two tiles of such heads do not fit the registers
        for (int t = my_begin + wave; t < my_end; t += kDecodeWaves) {
            if (t != my_begin + wave) issue(t, true, one);
            finish(t, one);
        }
    } else {
        int t = my_begin + wave;
        if (t < my_end) {
            while (true) {
                const int t1 = t + kDecodeWaves;
                issue(t1, t1 < my_end, two);
                finish(t, one);
                if (t1 >= my_end) break;
                const int t2 = t1 + kDecodeWaves;
                issue(t2, t2 < my_end, one);
                finish(t1, two);
                if (t2 >= my_end) break;
                t = t2;
            }
        }
    }

    // ---- merge the four waves --------------------------------------------------------------------
    float* sm_acc = smem;                                         // [waves][cols][kD]
    float* sm_m = smem + kDecodeWaves * cols * kD;                // [waves][cols]
    float* sm_l = sm_m + kDecodeWaves * cols;
    if (__any(unmapped)) l_run = __builtin_nanf("");   // a key in reach had no page: say so in the result
    if (g == 0 && c < cols) {
        sm_m[wave * cols + c] = m_run;
        sm_l[wave * cols + c] = l_run;
    }
    if (c < cols) {
#pragma unroll
        for (int dt = 0; dt < kD16; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) sm_acc[(wave * cols + c) * kD + 16 * dt + 4 * g + r] = acc[dt][r];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < cols * kD; i += kDecodeThreads) {
        const int col = i / kD, d = i % kD;
        float top = -INFINITY;
#pragma unroll
        for (int w = 0; w < kDecodeWaves; ++w) top = fmaxf(top, sm_m[w * cols + col]);
        float num = 0.f, den = 0.f;
        if (top != -INFINITY) {
#pragma unroll
            for (int w = 0; w < kDecodeWaves; ++w) {
                const float mw = sm_m[w * cols + col];
                const float wgt = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - top);
                num += sm_acc[(w * cols + col) * kD + d] * wgt;
                den += sm_l[w * cols + col] * wgt;
            }
        }
        const long rh = static_cast<long>(row) * q_heads + kvh * group + col0 + col;
        if (splits == 1) {                            // nothing to merge with: this is the result
            out[rh * kD + d] = from_float<bf16_t>(num / den);
            continue;
        }
        const long slot = rh * splits + split;
        part_acc[slot * kD + d] = num;
        if (d == 0) {
            part_ml[slot * 2] = top;
            part_ml[slot * 2 + 1] = den;
        }
    }
}

// Merges the splits of one (row, query head): out = sum_s acc_s 2^(m_s - M) / sum_s l_s 2^(m_s - M),
// the sums taken in split order.  The weights 2^(m_s - M) are computed once, one thread a split.
constexpr int kReduceThreads = 128;
constexpr int kMaxSplits = 256;

__global__ void __launch_bounds__(kReduceThreads)
attention_reduce_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                        bf16_t* __restrict__ out, int head_dim, int splits) {
    __shared__ float weight[kMaxSplits];
    __shared__ float wave_top[kReduceThreads / kWave];
    const long rh = blockIdx.x;                      // row * q_heads + head
    const float* ml = part_ml + rh * splits * 2;
    float top = -INFINITY;
    for (int s = threadIdx.x; s < splits; s += kReduceThreads) top = fmaxf(top, ml[2 * s]);
    top = wave_max(top);
    if (threadIdx.x % kWave == 0) wave_top[threadIdx.x / kWave] = top;
    __syncthreads();
    top = fmaxf(wave_top[0], wave_top[1]);
    for (int s = threadIdx.x; s < splits; s += kReduceThreads)
        weight[s] = ml[2 * s] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ml[2 * s] - top);
    __syncthreads();
    float den = 0.f;
    for (int s = 0; s < splits; ++s) den += ml[2 * s + 1] * weight[s];
    for (int d = threadIdx.x; d < head_dim; d += kReduceThreads) {
        float num = 0.f;
        for (int s = 0; s < splits; ++s) num += part_acc[(rh * splits + s) * head_dim + d] * weight[s];
        out[rh * head_dim + d] = from_float<bf16_t>(num / den);
    }
}

// The four waves' partial results, and the page ids of a split (at most the whole block table).
static size_t decode_smem_bytes(int head_dim, int group, int max_blocks) {
    const int cols = group < 16 ? group : 16;
    return (static_cast<size_t>(kDecodeWaves) * cols * head_dim + 2 * kDecodeWaves * cols) * sizeof(float) +
           static_cast<size_t>(max_blocks) * sizeof(int);
}

template <int kD16>
static void launch_decode(const void* q, const void* k_pool, const void* v_pool, const int* positions,
                          const int* row_entry, const int* block_table, int max_blocks, float* part_acc,
                          float* part_ml, void* out, int rows, int q_heads, int kv_heads, int page_shift, float scale,
                          int window, int splits, const FromProjection* from, hipStream_t stream) {
    const int group = q_heads / kv_heads;
    dim3 grid(rows, kv_heads * ((group + 15) / 16), splits);
    const size_t smem = decode_smem_bytes(kD16 * 16, group, max_blocks);
    const float to_log2 = scale * 1.4426950408889634f;
    if constexpr (kD16 % 4 == 0) {
        if (from != nullptr) {
            attention_decode_kernel<kD16, true><<<grid, kDecodeThreads, smem, stream>>>(
                nullptr, static_cast<const bf16_t*>(k_pool), static_cast<const bf16_t*>(v_pool), positions, row_entry,
                block_table, max_blocks, part_acc, part_ml, static_cast<bf16_t*>(out), q_heads, kv_heads, page_shift,
                to_log2, window, splits, *from);
            return;
        }
    }
    attention_decode_kernel<kD16, false><<<grid, kDecodeThreads, smem, stream>>>(
        static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_pool), static_cast<const bf16_t*>(v_pool),
        positions, row_entry, block_table, max_blocks, part_acc, part_ml, static_cast<bf16_t*>(out), q_heads, kv_heads,
        page_shift, to_log2, window, splits, FromProjection{});
}

static int decode_checked(const void* q, void* out, const void* k_pool, const void* v_pool, const int* positions,
                          const int* row_entry, const int* block_table, int max_blocks, float* part_acc,
                          float* part_ml, int rows, int q_heads, int kv_heads, int head_dim, int page_tokens,
                          float scale, int window, int splits, const FromProjection* from, hipStream_t stream) {
    LEONE_REQUIRE((q || from) && out && k_pool && v_pool && positions && row_entry && block_table,
                  "attention_decode: null pointer");
    LEONE_REQUIRE(splits == 1 || (part_acc && part_ml), "attention_decode: %d splits need the workspace", splits);
    LEONE_REQUIRE(rows > 0 && q_heads > 0 && kv_heads > 0 && q_heads % kv_heads == 0,
                  "attention_decode: rows %d, %d query heads over %d kv heads", rows, q_heads, kv_heads);
    LEONE_REQUIRE(head_dim % 16 == 0 && head_dim >= 16 && head_dim <= 256,
                  "attention_decode: head_dim %d must be a multiple of 16 in 16..256", head_dim);
    LEONE_REQUIRE(!from || head_dim % 64 == 0, "attention_decode: the projection is taken only at head sizes that are "
                  "multiples of 64, not %d", head_dim);
    LEONE_REQUIRE(page_tokens >= 16 && (page_tokens & (page_tokens - 1)) == 0,
                  "attention_decode: page_tokens %d must be a power of two, at least 16", page_tokens);
    LEONE_REQUIRE(decode_smem_bytes(head_dim, q_heads / kv_heads, max_blocks) <= 64 * 1024,
                  "attention_decode: head_dim %d needs more shared memory than a workgroup may have", head_dim);
    LEONE_REQUIRE(splits >= 1 && splits <= kMaxSplits, "attention_decode: splits %d must be in 1..%d", splits, kMaxSplits);
    LEONE_REQUIRE(window >= 0 && max_blocks > 0, "attention_decode: bad window or block table");
    const long grid_y = static_cast<long>(kv_heads) * ((q_heads / kv_heads + 15) / 16);
    LEONE_REQUIRE(grid_y <= 65535, "attention_decode: too many heads for one launch");
    int page_shift = 0;
    while ((1 << page_shift) < page_tokens) ++page_shift;
#define LEONE_DECODE_CASE(N)                                                                                      \
    case N:                                                                                                       \
        launch_decode<N>(q, k_pool, v_pool, positions, row_entry, block_table, max_blocks, part_acc, part_ml,     \
                         out, rows, q_heads, kv_heads, page_shift, scale, window, splits, from, stream);          \
        break;
    switch (head_dim / 16) {
        LEONE_DECODE_CASE(1) LEONE_DECODE_CASE(2) LEONE_DECODE_CASE(3) LEONE_DECODE_CASE(4)
        LEONE_DECODE_CASE(5) LEONE_DECODE_CASE(6) LEONE_DECODE_CASE(7) LEONE_DECODE_CASE(8)
        LEONE_DECODE_CASE(9) LEONE_DECODE_CASE(10) LEONE_DECODE_CASE(11) LEONE_DECODE_CASE(12)
        LEONE_DECODE_CASE(13) LEONE_DECODE_CASE(14) LEONE_DECODE_CASE(15) LEONE_DECODE_CASE(16)
        default:
            set_error("attention_decode: head_dim %d is not supported", head_dim);
            return 1;
    }
#undef LEONE_DECODE_CASE
    LEONE_LAUNCH_CHECK("attention_decode");
    if (splits > 1) {                                 // a single split has written the result itself
        attention_reduce_kernel<<<rows * q_heads, kReduceThreads, 0, stream>>>(
            part_acc, part_ml, static_cast<bf16_t*>(out), head_dim, splits);
        LEONE_LAUNCH_CHECK("attention_reduce");
    }
    return 0;
}

}  // namespace leone

using namespace leone;

// Workspace for splits > 1: part_acc holds rows*q_heads*splits*head_dim floats, part_ml rows*q_heads*splits*2.
extern "C" int leone_attention_decode(const void* q, void* out, const void* k_pool, const void* v_pool,
                                      const int* positions, const int* row_entry, const int* block_table,
                                      int max_blocks, float* part_acc, float* part_ml, int rows, int q_heads,
                                      int kv_heads, int head_dim, int page_tokens, float scale, int window,
                                      int splits, hipStream_t stream) {
    return decode_checked(q, out, k_pool, v_pool, positions, row_entry, block_table, max_blocks, part_acc, part_ml, rows,
                          q_heads, kv_heads, head_dim, page_tokens, scale, window, splits, nullptr, stream);
}

// The same for a step in which every row is another request, taking the fused q/k/v projection instead of
// finished queries: per-head RMSNorm (gains may be null) and half-split rotation (tables may be null) of the
// query heads, and with write_cache of the new key too, which goes into the cache with the new value before the
// keys are read.  qkv is bfloat16 [rows, (q_heads + 2 kv_heads) * head_dim], or float32 in qkv_planes planes
// (qkv_plane elements apart) that are added up in order.  head_dim a multiple of 64.
extern "C" int leone_attention_decode_projected(const void* qkv, int qkv_dtype, int qkv_planes, long qkv_plane,
                                                const void* q_gain, const void* k_gain, int gain_dtype, float eps,
                                                const float* cos_table, const float* sin_table, int table_positions,
                                                int rotary_dim, int pairing, void* out, void* k_pool, void* v_pool, int write_cache,
                                                const int* positions, const int* row_entry, const int* block_table,
                                                int max_blocks, float* part_acc, float* part_ml, int rows, int q_heads,
                                                int kv_heads, int head_dim, int page_tokens, float scale, int window,
                                                int splits, hipStream_t stream) {
    LEONE_REQUIRE(qkv && (qkv_dtype == kBF16 || qkv_dtype == kF32), "attention_decode: the projection is bfloat16 or float32");
    LEONE_REQUIRE(qkv_planes >= 1 && qkv_planes <= 64 && (qkv_dtype == kF32 || qkv_planes == 1),
                  "attention_decode: %d planes of the projection", qkv_planes);
    LEONE_REQUIRE((q_gain == nullptr) == (k_gain == nullptr), "attention_decode: q and k gains come together");
    LEONE_REQUIRE(!q_gain || ((gain_dtype == kF32 || gain_dtype == kBF16) && eps > 0.f),
                  "attention_decode: the head norms need gains of a known type and a positive eps");
    LEONE_REQUIRE((cos_table == nullptr) == (sin_table == nullptr), "attention_decode: cos and sin tables come together");
    LEONE_REQUIRE(!cos_table || table_positions > 0, "attention_decode: empty rotary table");
    LEONE_REQUIRE(!cos_table || (rotary_dim == head_dim && pairing == 0),
                  "attention_decode: the kernel that takes the projection rotates whole heads in half-split pairs, not "
                  "%d of %d elements with pairing %d", rotary_dim, head_dim, pairing);
    LEONE_REQUIRE(reinterpret_cast<uintptr_t>(qkv) % 32 == 0 &&
                      (!cos_table || (reinterpret_cast<uintptr_t>(cos_table) % 32 == 0 && reinterpret_cast<uintptr_t>(sin_table) % 32 == 0)) &&
                      (!q_gain || (reinterpret_cast<uintptr_t>(q_gain) % 32 == 0 && reinterpret_cast<uintptr_t>(k_gain) % 32 == 0)),
                  "attention_decode: the projection, the gains and the rotary tables must be aligned to 32 bytes");
    FromProjection from{qkv, qkv_dtype == kF32 ? 1 : 0, qkv_planes, qkv_plane, AnyVec{q_gain, gain_dtype},
                        AnyVec{k_gain, gain_dtype}, eps, cos_table, sin_table, table_positions,
                        write_cache ? static_cast<bf16_t*>(k_pool) : nullptr,
                        write_cache ? static_cast<bf16_t*>(v_pool) : nullptr};
    return decode_checked(nullptr, out, k_pool, v_pool, positions, row_entry, block_table, max_blocks, part_acc, part_ml,
                          rows, q_heads, kv_heads, head_dim, page_tokens, scale, window, splits, &from, stream);
}
