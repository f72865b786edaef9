// Attention over the paged cache.
//
// For a query row at absolute position `pos` of its request and query head h,
// with kv head h / (q_heads / kv_heads): scores s_j = (q . K[j]) * scale for
// keys j in [first, pos], first = 0 or pos - window + 1 for a windowed layer;
// softmax over them; out = sum_j p_j V[j].  This is the reference's recurrence
// (crates/leone/src/cpu.rs:2299-2421: scale after the dot, running maximum,
// rescaled sum and accumulator), with the keys found through the request's block
// table instead of its segment list.  Scores, maxima, sums and the accumulator
// are float whatever the cache's storage type.
//
// Cache layout of one layer: [page][kv head] blocks of page_tokens * head_dim
// elements, packed inside as key_offset() and value_offset() say.
#include "common.h"
#include "leone_hip.h"

#include <math.h>

namespace leone {

constexpr int kRowThreads = 256;
constexpr int kRowWaves = kRowThreads / kWave;
constexpr int kRowDimsPerLane = 4;                      // head_dim up to 256
constexpr int kRowMaxHeadDim = kWave * kRowDimsPerLane;

// One block per (row, query head).  Wave w takes keys first + w, first + w + 4,
// ...; lanes split the head's elements.  The four partial results are merged
// in a fixed order, so a launch repeats bit for bit.
template <typename T>
__global__ void attention_rows_kernel(const T* __restrict__ q, T* __restrict__ out,
                                      const T* __restrict__ k_pool, const T* __restrict__ v_pool,
                                      const int* __restrict__ positions, const int* __restrict__ row_entry,
                                      const int* __restrict__ block_table, int max_blocks, int q_heads,
                                      int kv_heads, int head_dim, int page_tokens, float scale, int window) {
    __shared__ float sm_m[kRowWaves];
    __shared__ float sm_l[kRowWaves];
    __shared__ float sm_acc[kRowWaves][kRowMaxHeadDim];

    const int row = blockIdx.x;
    const int head = blockIdx.y;
    const int wave = threadIdx.x / kWave;
    const int lane = threadIdx.x % kWave;
    const int kvh = head / (q_heads / kv_heads);
    const int pos = positions[row];
    const int* table = block_table + static_cast<long>(row_entry[row]) * max_blocks;
    const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

    const T* qr = q + (static_cast<long>(row) * q_heads + head) * head_dim;
    float qv[kRowDimsPerLane];
#pragma unroll
    for (int i = 0; i < kRowDimsPerLane; ++i) {
        const int d = lane + i * kWave;
        qv[i] = d < head_dim ? to_float(qr[d]) : 0.f;
    }

    float m = -INFINITY, l = 0.f;
    float acc[kRowDimsPerLane] = {0.f, 0.f, 0.f, 0.f};
    for (int j = first + wave; j <= pos; j += kRowWaves) {
        const int page = table[j / page_tokens];
        if (page < 0) {  // an unmapped block: poison the result instead of reading outside the pool
            l = __builtin_nanf("");
            continue;
        }
        const long head_base = (static_cast<long>(page) * kv_heads + kvh) * page_tokens * head_dim;
        const T* kr = k_pool + head_base;
        const T* vr = v_pool + head_base;
        const int token = j % page_tokens;
        float partial = 0.f;
        float vv[kRowDimsPerLane];
#pragma unroll
        for (int i = 0; i < kRowDimsPerLane; ++i) {
            const int d = lane + i * kWave;
            if (d < head_dim) {
                partial = fmaf(qv[i], to_float(kr[key_offset(token, d, page_tokens)]), partial);
                vv[i] = to_float(vr[value_offset(token, d, head_dim)]);
            } else {
                vv[i] = 0.f;
            }
        }
        const float s = wave_sum(partial) * scale;
        const float m_new = fmaxf(m, s);
        const float alpha = expf(m - m_new);
        const float beta = expf(s - m_new);
        l = l * alpha + beta;
#pragma unroll
        for (int i = 0; i < kRowDimsPerLane; ++i) acc[i] = acc[i] * alpha + beta * vv[i];
        m = m_new;
    }
    if (lane == 0) {
        sm_m[wave] = m;
        sm_l[wave] = l;
    }
#pragma unroll
    for (int i = 0; i < kRowDimsPerLane; ++i) sm_acc[wave][lane + i * kWave] = acc[i];
    __syncthreads();

    T* orow = out + (static_cast<long>(row) * q_heads + head) * head_dim;
    for (int d = threadIdx.x; d < head_dim; d += kRowThreads) {
        float top = sm_m[0];
#pragma unroll
        for (int w = 1; w < kRowWaves; ++w) top = fmaxf(top, sm_m[w]);
        float denom = 0.f, num = 0.f;
#pragma unroll
        for (int w = 0; w < kRowWaves; ++w) {
            // A wave that saw no key has m = -inf and contributes nothing.
            const float wgt = sm_m[w] == -INFINITY ? 0.f : expf(sm_m[w] - top);
            denom += sm_l[w] * wgt;
            num += sm_acc[w][d] * wgt;
        }
        orow[d] = from_float<T>(num / denom);
    }
}

}  // namespace leone

using namespace leone;

extern "C" int leone_attention_rows(const void* q, void* out, const void* k_pool, const void* v_pool, int dtype,
                                    const int* positions, const int* row_entry, const int* block_table,
                                    int max_blocks, int rows, int q_heads, int kv_heads, int head_dim,
                                    int page_tokens, float scale, int window, hipStream_t stream) {
    LEONE_REQUIRE(dtype == kF32 || dtype == kBF16, "attention_rows: unknown element type %d", dtype);
    LEONE_REQUIRE(q && out && k_pool && v_pool && positions && row_entry && block_table, "attention_rows: null pointer");
    LEONE_REQUIRE(rows > 0 && q_heads > 0 && kv_heads > 0 && q_heads % kv_heads == 0,
                  "attention_rows: rows %d, %d query heads over %d kv heads", rows, q_heads, kv_heads);
    LEONE_REQUIRE(q_heads <= 65535, "attention_rows: at most 65535 query heads");
    LEONE_REQUIRE(head_dim > 0 && head_dim <= kRowMaxHeadDim, "attention_rows: head_dim %d must be in 1..%d", head_dim, kRowMaxHeadDim);
    LEONE_REQUIRE(page_tokens > 0 && max_blocks > 0, "attention_rows: page_tokens %d and max_blocks %d must be positive", page_tokens, max_blocks);
    LEONE_REQUIRE(head_dim % 8 == 0 && page_tokens % 8 == 0,
                  "attention_rows: head_dim %d and page_tokens %d must be multiples of 8", head_dim, page_tokens);
    LEONE_REQUIRE(window >= 0, "attention_rows: window %d must not be negative", window);
    dim3 grid(rows, q_heads);
    if (dtype == kF32)
        attention_rows_kernel<float><<<grid, kRowThreads, 0, stream>>>(
            static_cast<const float*>(q), static_cast<float*>(out), static_cast<const float*>(k_pool),
            static_cast<const float*>(v_pool), positions, row_entry, block_table, max_blocks, q_heads, kv_heads,
            head_dim, page_tokens, scale, window);
    else
        attention_rows_kernel<bf16_t><<<grid, kRowThreads, 0, stream>>>(
            static_cast<const bf16_t*>(q), static_cast<bf16_t*>(out), static_cast<const bf16_t*>(k_pool),
            static_cast<const bf16_t*>(v_pool), positions, row_entry, block_table, max_blocks, q_heads, kv_heads,
            head_dim, page_tokens, scale, window);
    LEONE_LAUNCH_CHECK("attention_rows");
    return 0;
}
