// Causal attention of prompt portions over the paged cache on the matrix cores, bfloat16.
//
// A portion's rows are cut into tiles of 32 consecutive rows (the host lists them: entry, first
// row, row count); a wave takes one tile and one query head, its rows as two 16-column operands;
// a workgroup is one to four such waves.  A wave walks the 32-key tiles its rows can see, from the cache, and
// keeps the running maximum, sum and accumulator of the reference's recurrence
// (crates/leone/src/cpu.rs:2359-2421) per query in registers; nothing of size rows x keys is ever
// stored (the reference's prefill materialises the scores, crates/leone-cuda/cuda/ie_cuda.cu:5124-5220).
// Products and operand layouts are those of the decode kernel: S^T = K . Q^T and O^T += V^T . P^T with
// v_mfma_f32_16x16x32_bf16, keys and values read as 16-byte runs of the packed cache layout, a tile of
// keys and values loaded once for both column operands.  Waves do not share data, so no barrier is
// needed; the four waves of a workgroup read the same keys, which the caches serve.
#include "common.h"
#include "leone_hip.h"

#include <math.h>
#include <type_traits>

namespace leone {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int kPrefillWaves = 4;
constexpr int kPrefillThreads = kPrefillWaves * kWave;
constexpr int kColsPerWave = 2;                                  // 16-query operands a wave carries
constexpr int kRowsPerWave = 16 * kColsPerWave;                  // rows of a tile
constexpr int kKeysPerTile = 32;

__device__ inline bf16x8 pf_load8(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}
__device__ inline bf16x8 pf_zero8() {
    uint4 z = {0u, 0u, 0u, 0u};
    return __builtin_bit_cast(bf16x8, z);
}

// tiles: [n_tiles][3] = (entry, first row of the tile in the step, rows in the tile), at most 32 rows a
// tile.  Wave w of workgroup b takes tile b * waves + w; waves share nothing but the launch, so tiles of
// different requests may sit in one workgroup.
template <int kD16>
__global__ void __launch_bounds__(kPrefillThreads, 2)
attention_prefill_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ out, const bf16_t* __restrict__ k_pool,
                         const bf16_t* __restrict__ v_pool, const int* __restrict__ positions,
                         const int* __restrict__ tiles, int n_tiles, const int* __restrict__ block_table,
                         int max_blocks, int q_heads, int kv_heads, int page_shift, float scale, int window) {
    constexpr int kD = kD16 * 16;
    constexpr int kSteps = (kD16 + 1) / 2;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x % kWave;
    const int tile = blockIdx.x * (blockDim.x / kWave) + wave;
    const bool has_tile = tile < n_tiles;
    const int entry = has_tile ? tiles[3 * tile] : 0;
    const int tile_row0 = has_tile ? tiles[3 * tile + 1] : 0;
    const int wave_rows = has_tile ? tiles[3 * tile + 2] : 0;
    const int head = blockIdx.y;
    const int kvh = head / (q_heads / kv_heads);
    const int c = lane & 15, g = lane >> 4;
    const int page_tokens = 1 << page_shift, page_mask = page_tokens - 1;
    const int wave_row0 = 0;
    const int* table = block_table + static_cast<long>(entry) * max_blocks;

    // The page ids of the keys a wave reads go to its part of shared memory first, so that no load of
    // keys or values waits on a read of the block table.
    extern __shared__ int all_pages[];
    int* pages = all_pages + wave * max_blocks;
    int first_page = 0;
    if (has_tile) {
        const int tile_p0 = positions[tile_row0];
        const int tile_lo = (window > 0 && tile_p0 - window + 1 > 0) ? tile_p0 - window + 1 : 0;
        first_page = tile_lo >> page_shift;
        const int n_pages = ((tile_p0 + wave_rows - 1) >> page_shift) - first_page + 1;
        for (int i = lane; i < n_pages; i += kWave) pages[i] = table[first_page + i];
    }
    __syncthreads();
    if (!has_tile) return;                                     // after the workgroup's only barrier

    // Rows of a portion are consecutive positions: row r of the wave sits at p0 + r.
    const int p0 = positions[tile_row0 + wave_row0];
    const int p_last = p0 + wave_rows - 1;
    const int key_hi = p_last + 1;                                              // keys the wave may read: [key_lo, key_hi)
    const int key_lo = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
    // A tile wholly inside [full_lo, full_hi) is visible to every row of the wave: no masks.
    const int full_hi = p0 + 1;
    const int full_lo = (window > 0 && p_last - window + 1 > 0) ? p_last - window + 1 : 0;

    // Q^T operands and each column's own position.
    bf16x8 qreg[kColsPerWave][kSteps];
    int col_pos[kColsPerWave];
#pragma unroll
    for (int j = 0; j < kColsPerWave; ++j) {
        const int r = 16 * j + c;
        const bool ok = r < wave_rows;
        col_pos[j] = ok ? p0 + r : -1;                                          // -1: the column sees no key
        const bf16_t* qrow = q + (static_cast<long>(tile_row0 + wave_row0 + (ok ? r : 0)) * q_heads + head) * kD;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const int d0 = 32 * s + 8 * g;
            qreg[j][s] = (ok && d0 < kD) ? pf_load8(qrow + d0) : pf_zero8();
        }
    }

    float m_run[kColsPerWave], l_run[kColsPerWave];
    floatx4 acc[kColsPerWave][kD16];
#pragma unroll
    for (int j = 0; j < kColsPerWave; ++j) {
        m_run[j] = -INFINITY;
        l_run[j] = 0.f;
#pragma unroll
        for (int dt = 0; dt < kD16; ++dt) acc[j][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    bool unmapped = false;

    auto do_tile = [&](int t, auto full_tag) {
        constexpr bool kFull = decltype(full_tag)::value;
        const int key0 = t * kKeysPerTile;
        const int ka = key0 + 8 * (c >> 2) + (c & 3);          // A-operand row c of half a; half b is four keys on
        const int kb = ka + 4;
        const int run0 = key0 + 8 * g;                         // the lane's eight keys in the second product
        bool va = true, vb = true, any = true, whole = true;
        if constexpr (!kFull) {
            va = ka >= key_lo && ka < key_hi;
            vb = kb >= key_lo && kb < key_hi;
            any = run0 < key_hi && run0 + 8 > key_lo;
            whole = run0 >= key_lo && run0 + 8 <= key_hi;
        }
        const bf16_t* pk = k_pool;
        const bf16_t* pv = v_pool;
        if (va || vb) {
            const int page = pages[(ka >> page_shift) - first_page];
            if (page < 0) {
                unmapped = true;
                va = vb = false;
            }
            pk = k_pool + (static_cast<long>(page) * kv_heads + kvh) * page_tokens * kD + (ka & page_mask) * 8;
        }
        if (any) {
            const int page = pages[(run0 >> page_shift) - first_page];
            if (page < 0) {
                unmapped = true;
                any = false;
            }
            pv = v_pool + (static_cast<long>(page) * kv_heads + kvh) * page_tokens * kD +
                 static_cast<long>((run0 & page_mask) >> 3) * kD * 8;
        }
        bf16x8 xa[kSteps], xb[kSteps], xv[kD16];
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const bool in_head = 32 * s + 8 * g < kD;
            const long run = static_cast<long>(4 * s + g) * page_tokens * 8;
            xa[s] = (va && in_head) ? pf_load8(pk + run) : pf_zero8();
            xb[s] = (vb && in_head) ? pf_load8(pk + run + 32) : pf_zero8();
        }
#pragma unroll
        for (int dt = 0; dt < kD16; ++dt) {
            xv[dt] = any ? pf_load8(pv + (16 * dt + c) * 8) : pf_zero8();
            if constexpr (!kFull) {
                if (any && !whole) {   // slots the wave may not read can hold anything: clear them
                    uint4 raw = __builtin_bit_cast(uint4, xv[dt]);
                    unsigned* w = reinterpret_cast<unsigned*>(&raw);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int e0 = run0 + 2 * i, e1 = e0 + 1;
                        unsigned mask = 0u;
                        if (e0 >= key_lo && e0 < key_hi) mask |= 0x0000ffffu;
                        if (e1 >= key_lo && e1 < key_hi) mask |= 0xffff0000u;
                        w[i] &= mask;
                    }
                    xv[dt] = __builtin_bit_cast(bf16x8, raw);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < kColsPerWave; ++j) {
            floatx4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < kSteps; ++s) {
                sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[s], qreg[j][s], sa, 0, 0, 0);
                sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xb[s], qreg[j][s], sb, 0, 0, 0);
            }
            // lane (g, c): scores of keys run0 .. run0+7 for the query of column c
            const int p = col_pos[j];
            const int p_lo = (window > 0) ? p - window + 1 : 0;
            float sc[8];
            float tile_max = -INFINITY;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int key = run0 + i;
                const float raw = i < 4 ? sa[i & 3] : sb[i & 3];
                sc[i] = (kFull || (key <= p && key >= p_lo)) ? raw * scale : -INFINITY;
                tile_max = fmaxf(tile_max, sc[i]);
            }
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, kWave));
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, kWave));
            const float m_new = fmaxf(m_run[j], tile_max);
            const float m_safe = m_new == -INFINITY ? 0.f : m_new;   // a column that has seen no key yet
            const float alpha = __expf(m_run[j] - m_safe);
            float psum = 0.f;
            bf16x8 pt;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float e = __expf(sc[i] - m_safe);
                psum += e;
                pt[i] = static_cast<__bf16>(e);
            }
            psum += __shfl_xor(psum, 16, kWave);
            psum += __shfl_xor(psum, 32, kWave);
            l_run[j] = l_run[j] * alpha + psum;
            m_run[j] = m_new;
            if (__any(alpha != 1.0f)) {       // after the first tiles the running maximum seldom moves
#pragma unroll
                for (int dt = 0; dt < kD16; ++dt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[j][dt][r] *= alpha;
            }
#pragma unroll
            for (int dt = 0; dt < kD16; ++dt)
                acc[j][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xv[dt], pt, acc[j][dt], 0, 0, 0);
        }
    };

    const int t_begin = key_lo / kKeysPerTile, t_end = (key_hi + kKeysPerTile - 1) / kKeysPerTile;
    for (int t = t_begin; t < t_end; ++t) {
        const int key0 = t * kKeysPerTile;
        if (key0 >= full_lo && key0 + kKeysPerTile <= full_hi)
            do_tile(t, std::true_type{});
        else
            do_tile(t, std::false_type{});
    }

    const bool poisoned = __any(unmapped);
#pragma unroll
    for (int j = 0; j < kColsPerWave; ++j) {
        const int r = 16 * j + c;
        if (r >= wave_rows) continue;
        const float inv = poisoned ? __builtin_nanf("") : 1.0f / l_run[j];
        bf16_t* orow = out + (static_cast<long>(tile_row0 + wave_row0 + r) * q_heads + head) * kD;
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

template <int kD16>
static void launch_prefill(const void* q, void* out, const void* k_pool, const void* v_pool, const int* positions,
                           const int* tiles, int n_tiles, const int* block_table, int max_blocks, int q_heads,
                           int kv_heads, int page_shift, float scale, int window, hipStream_t stream) {
    // Four tiles a workgroup when there are plenty (their waves read the same keys, which the caches
    // then serve once), fewer when the chip would otherwise stay half empty.
    const long wave_tiles = static_cast<long>(n_tiles) * q_heads;
    const int waves = wave_tiles >= 2048 ? 4 : wave_tiles >= 1024 ? 2 : 1;
    dim3 grid(ceil_div(n_tiles, waves), q_heads);
    attention_prefill_kernel<kD16><<<grid, waves * kWave, static_cast<size_t>(waves) * max_blocks * sizeof(int), stream>>>(
        static_cast<const bf16_t*>(q), static_cast<bf16_t*>(out), static_cast<const bf16_t*>(k_pool),
        static_cast<const bf16_t*>(v_pool), positions, tiles, n_tiles, block_table, max_blocks, q_heads, kv_heads,
        page_shift, scale, window);
}

}  // namespace leone

using namespace leone;

extern "C" int leone_attention_prefill_tile_rows() { return kRowsPerWave; }

extern "C" int leone_attention_prefill(const void* q, void* out, const void* k_pool, const void* v_pool,
                                       const int* positions, const int* tiles, int n_tiles, const int* block_table,
                                       int max_blocks, int q_heads, int kv_heads, int head_dim, int page_tokens,
                                       float scale, int window, hipStream_t stream) {
    LEONE_REQUIRE(q && out && k_pool && v_pool && positions && tiles && block_table, "attention_prefill: null pointer");
    LEONE_REQUIRE(n_tiles > 0 && q_heads > 0 && kv_heads > 0 && q_heads % kv_heads == 0,
                  "attention_prefill: %d tiles, %d query heads over %d kv heads", n_tiles, q_heads, kv_heads);
    LEONE_REQUIRE(q_heads <= 65535, "attention_prefill: at most 65535 query heads");
    LEONE_REQUIRE(head_dim % 16 == 0 && head_dim >= 16 && head_dim <= 128,
                  "attention_prefill: head_dim %d must be a multiple of 16 in 16..128", head_dim);
    LEONE_REQUIRE(page_tokens >= 16 && (page_tokens & (page_tokens - 1)) == 0,
                  "attention_prefill: page_tokens %d must be a power of two, at least 16", page_tokens);
    LEONE_REQUIRE(window >= 0 && max_blocks > 0, "attention_prefill: bad window or block table");
    LEONE_REQUIRE(static_cast<size_t>(kPrefillWaves) * max_blocks * sizeof(int) <= 64 * 1024,
                  "attention_prefill: a block table of %d entries does not fit shared memory", max_blocks);
    int page_shift = 0;
    while ((1 << page_shift) < page_tokens) ++page_shift;
#define LEONE_PREFILL_CASE(N)                                                                                     \
    case N:                                                                                                       \
        launch_prefill<N>(q, out, k_pool, v_pool, positions, tiles, n_tiles, block_table, max_blocks, q_heads,    \
                          kv_heads, page_shift, scale, window, stream);                                           \
        break;
    switch (head_dim / 16) {
        LEONE_PREFILL_CASE(1) LEONE_PREFILL_CASE(2) LEONE_PREFILL_CASE(3) LEONE_PREFILL_CASE(4)
        LEONE_PREFILL_CASE(5) LEONE_PREFILL_CASE(6) LEONE_PREFILL_CASE(7) LEONE_PREFILL_CASE(8)
        default:
            set_error("attention_prefill: head_dim %d is not supported", head_dim);
            return 1;
    }
#undef LEONE_PREFILL_CASE
    LEONE_LAUNCH_CHECK("attention_prefill");
    return 0;
}
