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
__device__ inline bf16x8 zero8() {
    uint4 z = {0u, 0u, 0u, 0u};
    return __builtin_bit_cast(bf16x8, z);
}

// kD16 = head_dim / 16.
// Up to a head size of 128 the kernel fits three waves a SIMD without spilling if the compiler is asked to
// (a little faster than two, measured); larger heads need their registers.
template <int kD16>
__global__ void __launch_bounds__(kDecodeThreads, kD16 <= 8 ? 3 : 1)
attention_decode_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pool,
                        const bf16_t* __restrict__ v_pool, const int* __restrict__ positions,
                        const int* __restrict__ row_entry, const int* __restrict__ block_table, int max_blocks,
                        float* __restrict__ part_acc, float* __restrict__ part_ml, bf16_t* __restrict__ out,
                        int q_heads, int kv_heads, int page_shift, float to_log2, int window, int splits) {
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
    __syncthreads();

    // Q^T operand: column c is query head kvh*group + col0 + c.
    bf16x8 qreg[kSteps];
    {
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

    // One 32-key tile.  `full` tiles lie wholly inside [lo, n) and need no masks; at most the first
    // and the last tile of a row are not.  All loads of a tile, keys and values, are issued before
    // the first product, so that they are in flight together.
    auto do_tile = [&](int t, auto full_tag) {
        constexpr bool kFull = decltype(full_tag)::value;
        const int key0 = t * kTileKeys;
        // A-operand row c of half a is key 8*(c/4) + c%4, of half b four keys further
        const int ka = key0 + 8 * (c >> 2) + (c & 3);
        const int kb = ka + 4;
        const int run0 = key0 + 8 * g;                   // this lane's eight keys for the second product
        bool va = true, vb = true, any = true, whole = true;
        if constexpr (!kFull) {
            va = ka >= lo && ka < n;
            vb = kb >= lo && kb < n;
            any = run0 < n && run0 + 8 > lo;
            whole = run0 >= lo && run0 + 8 <= n;
        }
        const bf16_t* pk = k_pool;
        const bf16_t* pv = v_pool;
        if (va || vb) {                                   // ka and kb share a page: pages hold multiples of 8 keys
            const int page = pages[(ka >> page_shift) - first_page];
            if (page < 0) {
                unmapped = true;                          // never read outside the pool; the result is poisoned below
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
            const long run = static_cast<long>(4 * s + g) * page_tokens * 8;   // elements 32s+8g .. +7 of the key
            xa[s] = (va && in_head) ? load8(pk + run) : zero8();
            xb[s] = (vb && in_head) ? load8(pk + run + 32) : zero8();           // four keys further
        }
#pragma unroll
        for (int dt = 0; dt < kD16; ++dt) xv[dt] = any ? load8(pv + (16 * dt + c) * 8) : zero8();

        // ---- S^T = K . Q^T for the two 16-key halves --------------------------------------------
        floatx4 sa = {0.f, 0.f, 0.f, 0.f}, sb = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            sa = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[s], qreg[s], sa, 0, 0, 0);
            sb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xb[s], qreg[s], sb, 0, 0, 0);
        }
        // lane (g, c) now holds, for query column c, the scores of keys key0 + 8g + j, j = 0..7
        float sc[8];
        float tile_max = -INFINITY;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int key = run0 + j;
            const float raw = j < 4 ? sa[j & 3] : sb[j & 3];
            sc[j] = (kFull || (key >= lo && key < n)) ? raw * to_log2 : -INFINITY;
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
            if constexpr (!kFull) {
                if (any && !whole) {
                    // slots outside [lo, n) may hold anything, even NaN: clear them, a zero weight is not enough
                    uint4 raw = __builtin_bit_cast(uint4, xv[dt]);
                    unsigned* w = reinterpret_cast<unsigned*>(&raw);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int e0 = run0 + 2 * i, e1 = e0 + 1;
                        unsigned mask = 0u;
                        if (e0 >= lo && e0 < n) mask |= 0x0000ffffu;
                        if (e1 >= lo && e1 < n) mask |= 0xffff0000u;
                        w[i] &= mask;
                    }
                    xv[dt] = __builtin_bit_cast(bf16x8, raw);
                }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[dt][r] *= alpha;
            acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xv[dt], pt, acc[dt], 0, 0, 0);
        }
    };

    for (int t = my_begin + wave; t < my_end; t += kDecodeWaves) {
        const int key0 = t * kTileKeys;
        if (key0 >= lo && key0 + kTileKeys <= n)
            do_tile(t, std::true_type{});
        else
            do_tile(t, std::false_type{});
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
                          int window, int splits, hipStream_t stream) {
    const int group = q_heads / kv_heads;
    dim3 grid(rows, kv_heads * ((group + 15) / 16), splits);
    const size_t smem = decode_smem_bytes(kD16 * 16, group, max_blocks);
    attention_decode_kernel<kD16><<<grid, kDecodeThreads, smem, stream>>>(
        static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_pool), static_cast<const bf16_t*>(v_pool),
        positions, row_entry, block_table, max_blocks, part_acc, part_ml, static_cast<bf16_t*>(out), q_heads, kv_heads,
        page_shift, scale * 1.4426950408889634f, window, splits);
}

}  // namespace leone

using namespace leone;

// Workspace for splits > 1: part_acc holds rows*q_heads*splits*head_dim floats, part_ml rows*q_heads*splits*2.
extern "C" int leone_attention_decode(const void* q, void* out, const void* k_pool, const void* v_pool,
                                      const int* positions, const int* row_entry, const int* block_table,
                                      int max_blocks, float* part_acc, float* part_ml, int rows, int q_heads,
                                      int kv_heads, int head_dim, int page_tokens, float scale, int window,
                                      int splits, hipStream_t stream) {
    LEONE_REQUIRE(q && out && k_pool && v_pool && positions && row_entry && block_table,
                  "attention_decode: null pointer");
    LEONE_REQUIRE(splits == 1 || (part_acc && part_ml), "attention_decode: %d splits need the workspace", splits);
    LEONE_REQUIRE(rows > 0 && q_heads > 0 && kv_heads > 0 && q_heads % kv_heads == 0,
                  "attention_decode: rows %d, %d query heads over %d kv heads", rows, q_heads, kv_heads);
    LEONE_REQUIRE(head_dim % 16 == 0 && head_dim >= 16 && head_dim <= 256,
                  "attention_decode: head_dim %d must be a multiple of 16 in 16..256", head_dim);
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
                         out, rows, q_heads, kv_heads, page_shift, scale, window, splits, stream);                \
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
