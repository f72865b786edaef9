// Row-wise kernels: embedding gather, residual-add + RMSNorm, SwiGLU, the
// rotary table, and the fused per-head norm + rotation + cache write.
//
// Formulas follow the reference's scalar backend: RMSNorm
// y = (x * w) * rsqrt(mean(x^2) + eps) (crates/leone/src/cpu.rs:1642-1663),
// half-split rotary pairs (i, i + D/2) with inverse frequency theta^(-2i/D)
// (crates/leone/src/cpu.rs:1721-1779), SwiGLU g / (1 + exp(-g)) * u
// (crates/leone/src/cpu.rs:892-907).  Sums of squares, gains and rotations are
// computed in float whatever the storage type; rotary angles in double.
#include "common.h"

#include <type_traits>
#include "leone_hip.h"

namespace leone {

// ---- embedding -------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ tokens,
                             float* __restrict__ out, int hidden, int vocab, float scale) {
    const int row = blockIdx.x;
    const int token = tokens[row];
    float* dst = out + static_cast<long>(row) * hidden;
    if (token < 0 || token >= vocab) {
        // The host rejects such ids before the launch; never read outside the table.
        for (int c = threadIdx.x; c < hidden; c += blockDim.x) dst[c] = __builtin_nanf("");
        return;
    }
    const T* src = table + static_cast<long>(token) * hidden;
    for (int c = threadIdx.x; c < hidden; c += blockDim.x) dst[c] = to_float(src[c]) * scale;
}

// ---- a soft cap on logits -----------------------------------------------------
// x = cap * tanh(x / cap), in place: what some architectures put between the head and the sampler.
__global__ void __launch_bounds__(256) soft_cap_kernel(float* __restrict__ x, long n, float cap) {
    const long stride = static_cast<long>(gridDim.x) * blockDim.x;
    for (long i = static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) x[i] = cap * tanhf(x[i] / cap);
}

// ---- residual add + RMSNorm -------------------------------------------------
// One block per output row.  With `rows` == nullptr row r of `x` is updated in
// place (x += delta) and normalised into y[r].  With `rows` given, output row r
// reads x[rows[r]] (+ delta[rows[r]]) and x is left untouched.  `delta` may come in
// several planes, `plane` elements apart, whose sum (taken in order) is meant: the
// parts of a product whose inner dimension was cut.
template <typename TD, typename TY, int kThreads>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const TD* __restrict__ delta, int planes, long plane,
                                   AnyVec gain, float eps, TY* __restrict__ y,
                                   const int* __restrict__ rows, int hidden, float* __restrict__ squares_out) {
    __shared__ float scratch[kThreads / kWave];
    const int out_row = blockIdx.x;
    const long in_row = rows ? rows[out_row] : out_row;
    float* xr = x + in_row * hidden;
    const TD* dr = delta ? delta + in_row * hidden : nullptr;
    TY* yr = y + static_cast<long>(out_row) * hidden;
    float ss = 0.f;
    for (int c = threadIdx.x; c < hidden; c += kThreads) {
        float v = xr[c];
        if (dr) {
            for (int p = 0; p < planes; ++p) v += to_float(dr[p * plane + c]);
            if (!rows) xr[c] = v;
        }
        ss = fmaf(v, v, ss);
    }
    const float total = block_sum<kThreads>(ss, scratch);
    const float inv = squares_out ? 1.0f : 1.0f / sqrtf(total / static_cast<float>(hidden) + eps);
    if (squares_out) {                                 // the row's sum first, zeros for the other parts
        const int parts = (hidden + 15) / 16;
        for (int i = threadIdx.x; i < parts; i += kThreads) squares_out[static_cast<long>(out_row) * parts + i] = i == 0 ? total : 0.f;
    }
    for (int c = threadIdx.x; c < hidden; c += kThreads) {
        float v = xr[c];
        if (dr && rows)
            for (int p = 0; p < planes; ++p) v += to_float(dr[p * plane + c]);
        yr[c] = from_float<TY>((v * load_any(gain, c)) * inv);
    }
}

// The same for rows whose length is a multiple of 4 and at most 4 * kThreads * kChunks: every
// thread keeps its elements in registers, so the row is read once, with 16-byte loads, and the
// gains are fetched together with it.
__device__ inline void load4(const float* p, float v[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ inline void load4(const bf16_t* p, float v[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}
__device__ inline void store4(float* p, const float v[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ inline void store4(bf16_t* p, const float v[4]) {
    uint2 t;
    t.x = bf16_bits_from_float(v[0]) | (static_cast<uint32_t>(bf16_bits_from_float(v[1])) << 16);
    t.y = bf16_bits_from_float(v[2]) | (static_cast<uint32_t>(bf16_bits_from_float(v[3])) << 16);
    *reinterpret_cast<uint2*>(p) = t;
}

template <typename TD, typename TG, typename TY, int kThreads, int kChunks>
__global__ void __launch_bounds__(kThreads)
add_rmsnorm_vec_kernel(float* __restrict__ x, const TD* __restrict__ delta, int planes, long plane,
                       const TG* __restrict__ gain, float eps, TY* __restrict__ y, const int* __restrict__ rows,
                       int hidden, float* __restrict__ squares_out) {
    __shared__ float scratch[kThreads / kWave];
    const int out_row = blockIdx.x;
    const long in_row = rows ? rows[out_row] : out_row;
    float* xr = x + in_row * hidden;
    const TD* dr = delta ? delta + in_row * hidden : nullptr;
    TY* yr = y + static_cast<long>(out_row) * hidden;
    float v[kChunks][4], gv[kChunks][4];
    float ss = 0.f;
    // Everything a thread needs is asked for before anything is added: the row, the gains, and the planes four
    // at a time (a plane beyond the last is the last one again and is not added), so that the trips to memory
    // overlap instead of following one another plane by plane.  The planes are added in their order.
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
        const int c = 4 * (threadIdx.x + i * kThreads);
        if (c < hidden) {
            load4(xr + c, v[i]);
            load4(gain + c, gv[i]);
        }
    }
    if (dr) {
        for (int p0 = 0; p0 < planes; p0 += 4) {
            float d[kChunks][4][4];
#pragma unroll
            for (int i = 0; i < kChunks; ++i) {
                const int c = 4 * (threadIdx.x + i * kThreads);
                if (c < hidden) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) load4(dr + (p0 + q < planes ? p0 + q : planes - 1) * plane + c, d[i][q]);
                }
            }
#pragma unroll
            for (int i = 0; i < kChunks; ++i) {
                const int c = 4 * (threadIdx.x + i * kThreads);
                if (c < hidden) {
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        if (p0 + q < planes) {
#pragma unroll
                            for (int j = 0; j < 4; ++j) v[i][j] += d[i][q][j];
                        }
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
        const int c = 4 * (threadIdx.x + i * kThreads);
        if (c < hidden) {
            if (dr && !rows) store4(xr + c, v[i]);
#pragma unroll
            for (int j = 0; j < 4; ++j) ss = fmaf(v[i][j], v[i][j], ss);
        }
    }
    const float total = block_sum<kThreads>(ss, scratch);
    const float inv = squares_out ? 1.0f : 1.0f / sqrtf(total / static_cast<float>(hidden) + eps);
    if (squares_out) {                                 // the row's sum first, zeros for the other parts
        const int parts = (hidden + 15) / 16;
        for (int i = threadIdx.x; i < parts; i += kThreads) squares_out[static_cast<long>(out_row) * parts + i] = i == 0 ? total : 0.f;
    }
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
        const int c = 4 * (threadIdx.x + i * kThreads);
        if (c < hidden) {
            float o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = (v[i][j] * gv[i][j]) * inv;
            store4(yr + c, o);
        }
    }
}

// ---- SwiGLU -------------------------------------------------------------------
// in: [rows, 2F]; every block of 16 columns holds 8 gate values, then the 8 up values that belong to
// them (the order in which the fused gate/up weight keeps its rows).
// A thread takes one block of 16 columns: two loads of 8 values, one store of 8 results.
template <typename T>
struct alignas(8 * sizeof(T)) Run8 {
    T v[8];
};
template <typename T>
__global__ void __launch_bounds__(256)
swiglu_kernel(const T* __restrict__ gate_up, T* __restrict__ out, long rows, int ffn) {
    const int groups = ffn / 8;
    const int group = blockIdx.x * blockDim.x + threadIdx.x;
    if (group >= groups) return;
    for (long r = blockIdx.y; r < rows; r += gridDim.y) {
        const T* in = gate_up + r * 2 * ffn + 16 * static_cast<long>(group);
        const Run8<T> gate = *reinterpret_cast<const Run8<T>*>(in);
        const Run8<T> up = *reinterpret_cast<const Run8<T>*>(in + 8);
        Run8<T> y;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float g = to_float(gate.v[i]);
            y.v[i] = from_float<T>((g / (1.0f + expf(-g))) * to_float(up.v[i]));
        }
        *reinterpret_cast<Run8<T>*>(out + r * ffn + 8 * static_cast<long>(group)) = y;
    }
}

// ---- rotary table ----------------------------------------------------------------
// cos/sin of pos * theta^(-2i/D), evaluated in double and stored as float
// (the reference's device table, crates/leone-cuda/cuda/ie_cuda.cu:2383-2401).
__global__ void rope_table_kernel(float* __restrict__ cos_out, float* __restrict__ sin_out,
                                  double theta, int pairs, int rotary_dim, int positions) {
    const long total = static_cast<long>(positions) * pairs;
    for (long i = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; i < total;
         i += static_cast<long>(gridDim.x) * blockDim.x) {
        const int pos = static_cast<int>(i / pairs);
        const int p = static_cast<int>(i % pairs);
        const double inv = pow(theta, -2.0 * static_cast<double>(p) / static_cast<double>(rotary_dim));
        const double angle = static_cast<double>(pos) * inv;
        cos_out[i] = static_cast<float>(cos(angle));
        sin_out[i] = static_cast<float>(sin(angle));
    }
}

// ---- per-head norm + rotation + cache write ------------------------------------------
// One wave per (row, head) of the fused projection output
// qkv[row] = [q heads | k heads | v heads], each head of D elements.
//   q heads: optional RMSNorm over D, optional rotation, written to q_out.
//   k heads: the same, written into the request's page at `position`.
//   v heads: copied into the page unchanged.
// Keys and values go into the page in the packed layouts of key_offset() and value_offset().
// A lane owns pairs p = lane, lane + 64, ... (p < D/2).  Which two elements pair p is, and whether it is
// rotated, is the position encoding's affair (crates/leone/src/cpu.rs:1765-1774 keeps the pairing a switch): of
// the head's first `rotary_dim` = 2 * rotary_half elements, pair p < rotary_half is (p, p + rotary_half) for
// the half-split pairing and (2p, 2p + 1) for the adjacent one and is rotated by the table's angle p; what
// lies beyond rotary_dim is normalised but not rotated (pairs (2p, 2p + 1) either way).
// When `write_cache` is 0 the k and v heads are skipped (a layer that reads
// another layer's cache).
constexpr int kMaxPairsPerLane = 4;  // head_dim up to 512
enum RopePairing : int { kPairHalfSplit = 0, kPairAdjacent = 1 };

template <typename TIn, typename T>
__global__ void qk_norm_rope_write_kernel(
    const TIn* __restrict__ qkv, int planes, long plane, T* __restrict__ q_out, T* __restrict__ k_pool, T* __restrict__ v_pool,
    AnyVec q_gain, AnyVec k_gain, float eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int table_positions, const int* __restrict__ positions,
    const int* __restrict__ row_entry, const int* __restrict__ block_table, int max_blocks,
    int q_heads, int kv_heads, int head_dim, int page_tokens, int write_cache, int rotary_half, int pairing) {
    const int row = blockIdx.x;
    const int head = blockIdx.y * (blockDim.x / kWave) + threadIdx.x / kWave;
    const int lane = threadIdx.x % kWave;
    const int heads_total = q_heads + (write_cache ? 2 * kv_heads : 0);
    if (head >= heads_total) return;
    const int half = head_dim / 2;
    const int qkv_width = (q_heads + 2 * kv_heads) * head_dim;
    const TIn* src = qkv + static_cast<long>(row) * qkv_width + static_cast<long>(head) * head_dim;
    const int pos = positions[row];

    const bool is_q = head < q_heads;
    const bool is_k = !is_q && head < q_heads + kv_heads;
    // Where element d of this head goes: q rows are plain; keys and values use the cache's packed layout.
    T* dst;
    int kind = 0;  // 0 plain, 1 key page, 2 value page
    int token = 0;
    if (is_q) {
        dst = q_out + (static_cast<long>(row) * q_heads + head) * head_dim;
    } else {
        const int kvh = is_k ? head - q_heads : head - q_heads - kv_heads;
        const int page = block_table[static_cast<long>(row_entry[row]) * max_blocks + pos / page_tokens];
        if (page < 0) return;  // host reserves pages before the launch
        dst = (is_k ? k_pool : v_pool) + (static_cast<long>(page) * kv_heads + kvh) * page_tokens * head_dim;
        kind = is_k ? 1 : 2;
        token = pos % page_tokens;
    }
    auto place = [&](int d) -> long {
        return kind == 0 ? d : kind == 1 ? key_offset(token, d, page_tokens) : value_offset(token, d, head_dim);
    };

    // the two elements of pair p
    auto first = [&](int p) { return pairing == kPairHalfSplit && p < rotary_half ? p : 2 * p; };
    auto second = [&](int p) { return pairing == kPairHalfSplit && p < rotary_half ? p + rotary_half : 2 * p + 1; };
    float a[kMaxPairsPerLane], b[kMaxPairsPerLane];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxPairsPerLane; ++i) {
        const int p = lane + i * kWave;
        if (p < half) {
            a[i] = to_float(src[first(p)]);
            b[i] = to_float(src[second(p)]);
            for (int s = 1; s < planes; ++s) {       // planes of a product cut along K: added in order
                a[i] += to_float(src[s * plane + first(p)]);
                b[i] += to_float(src[s * plane + second(p)]);
            }
            // rounded as a product stored in the outputs' type would be: the same bits whichever way it came
            a[i] = to_float(from_float<T>(a[i]));
            b[i] = to_float(from_float<T>(b[i]));
            ss = fmaf(a[i], a[i], ss);
            ss = fmaf(b[i], b[i], ss);
        }
    }
    if (!is_q && !is_k) {  // value head: plain copy
#pragma unroll
        for (int i = 0; i < kMaxPairsPerLane; ++i) {
            const int p = lane + i * kWave;
            if (p < half) {
                dst[place(first(p))] = from_float<T>(a[i]);
                dst[place(second(p))] = from_float<T>(b[i]);
            }
        }
        return;
    }
    const AnyVec gain = is_q ? q_gain : k_gain;
    float inv = 1.f;
    if (gain.ptr) {
        ss = wave_sum(ss);
        inv = 1.0f / sqrtf(ss / static_cast<float>(head_dim) + eps);
    }
    const bool rotate = cos_table != nullptr;
    const int tpos = pos < table_positions ? pos : table_positions - 1;  // host checks the bound
#pragma unroll
    for (int i = 0; i < kMaxPairsPerLane; ++i) {
        const int p = lane + i * kWave;
        if (p < half) {
            float u = a[i], v = b[i];
            if (gain.ptr) {
                u = (u * load_any(gain, first(p))) * inv;
                v = (v * load_any(gain, second(p))) * inv;
            }
            if (rotate && p < rotary_half) {
                const float c = cos_table[static_cast<long>(tpos) * rotary_half + p];
                const float s = sin_table[static_cast<long>(tpos) * rotary_half + p];
                const float ru = u * c - v * s;
                const float rv = u * s + v * c;
                u = ru;
                v = rv;
            }
            dst[place(first(p))] = from_float<T>(u);
            dst[place(second(p))] = from_float<T>(v);
        }
    }
}

// The same work for head sizes that are multiples of 16, in runs of 8 elements: a head is shared by
// head_dim / 16 neighbouring lanes, lane j of them owns elements 8j .. 8j+7 and their partners in the
// other half, so a lane reads two runs, writes two runs of q or two runs of the key layout (a run of
// the key layout is eight elements of one token), and the sum of squares crosses at most eight lanes.
template <typename T>
struct alignas(8 * sizeof(T)) HeadRun {
    T v[8];
};

// Eight elements of a gain vector, from an offset that is a multiple of 8.
__device__ inline void load_run(const AnyVec& v, int at, float out[8]) {
    if (v.dtype == kF32) {
        const HeadRun<float> r = *reinterpret_cast<const HeadRun<float>*>(static_cast<const float*>(v.ptr) + at);
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = r.v[i];
    } else {
        const HeadRun<bf16_t> r = *reinterpret_cast<const HeadRun<bf16_t>*>(static_cast<const bf16_t*>(v.ptr) + at);
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = to_float(r.v[i]);
    }
}

template <typename T>
__device__ inline void value_write_block(T* turned, int row_block, int kvh, const T* __restrict__ qkv, T* __restrict__ v_pool,
                                         const int* __restrict__ positions, const int* __restrict__ row_entry,
                                         const int* __restrict__ block_table, int max_blocks, int rows, int q_heads,
                                         int kv_heads, int head_dim, int page_tokens);

template <typename TIn, typename T, int kD16>
__global__ void __launch_bounds__(256)
qk_norm_rope_write_runs_kernel(
    const TIn* __restrict__ qkv, int planes, long plane, T* __restrict__ q_out, T* __restrict__ k_pool, T* __restrict__ v_pool,
    AnyVec q_gain, AnyVec k_gain, float eps, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int table_positions, const int* __restrict__ positions,
    const int* __restrict__ row_entry, const int* __restrict__ block_table, int max_blocks,
    int rows, int q_heads, int kv_heads, int page_tokens, int write_cache, int write_values, int value_blocks) {
    constexpr int kD = 16 * kD16;
    constexpr int kHalf = kD / 2;
    // The last `value_blocks` workgroups write the values of many rows in whole runs (value_write_block: eight
    // rows and one kv head each), in the same launch as the heads.
    if (static_cast<int>(gridDim.x - blockIdx.x) <= value_blocks) {
        if constexpr (std::is_same<TIn, T>::value) {
            extern __shared__ __align__(32) unsigned char turned_raw[];
            const int at = value_blocks - static_cast<int>(gridDim.x - blockIdx.x);
            value_write_block<T>(reinterpret_cast<T*>(turned_raw), at / kv_heads, at % kv_heads, qkv, v_pool, positions, row_entry,
                                 block_table, max_blocks, rows, q_heads, kv_heads, kD, page_tokens);
        }
        return;
    }
    constexpr int kShare = kD16 <= 1 ? 1 : kD16 <= 2 ? 2 : kD16 <= 4 ? 4 : 8;   // lanes a head takes (a power of two)
    const int heads_total = q_heads + (write_cache ? (write_values ? 2 : 1) * kv_heads : 0);
    const long item = (static_cast<long>(blockIdx.x) * blockDim.x + threadIdx.x) / kShare;
    const int j = threadIdx.x % kShare;
    const bool mine = item < static_cast<long>(rows) * heads_total && j < kD16;
    // Lanes without work still take part in the exchange below, with zeros.
    const int row = mine ? static_cast<int>(item / heads_total) : 0;
    const int head = mine ? static_cast<int>(item % heads_total) : 0;
    const int qkv_width = (q_heads + 2 * kv_heads) * kD;
    const TIn* src = qkv + static_cast<long>(row) * qkv_width + static_cast<long>(head) * kD + 8 * j;
    const bool is_q = head < q_heads;
    const bool is_k = !is_q && head < q_heads + kv_heads;

    float a[8], b[8];
    float ss = 0.f;
    if (mine) {
        const HeadRun<TIn> lo = *reinterpret_cast<const HeadRun<TIn>*>(src);
        const HeadRun<TIn> hi = *reinterpret_cast<const HeadRun<TIn>*>(src + kHalf);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            a[i] = to_float(lo.v[i]);
            b[i] = to_float(hi.v[i]);
        }
        for (int s = 1; s < planes; ++s) {           // planes of a product cut along K: added in order
            const HeadRun<TIn> lo_s = *reinterpret_cast<const HeadRun<TIn>*>(src + s * plane);
            const HeadRun<TIn> hi_s = *reinterpret_cast<const HeadRun<TIn>*>(src + s * plane + kHalf);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                a[i] += to_float(lo_s.v[i]);
                b[i] += to_float(hi_s.v[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            // rounded as a product stored in the outputs' type would be: the same bits whichever way it came
            a[i] = to_float(from_float<T>(a[i]));
            b[i] = to_float(from_float<T>(b[i]));
            ss = fmaf(a[i], a[i], ss);
            ss = fmaf(b[i], b[i], ss);
        }
    }
#pragma unroll
    for (int off = kShare / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, kWave);
    if (!mine) return;

    const int pos = positions[row];
    T* page_base = nullptr;
    int token = 0;
    if (!is_q) {
        const int kvh = is_k ? head - q_heads : head - q_heads - kv_heads;
        const int page = block_table[static_cast<long>(row_entry[row]) * max_blocks + pos / page_tokens];
        if (page < 0) return;  // host reserves pages before the launch
        page_base = (is_k ? k_pool : v_pool) + (static_cast<long>(page) * kv_heads + kvh) * page_tokens * kD;
        token = pos % page_tokens;
    }
    if (!is_q && !is_k) {      // value head: copied as it is; eight elements of one token lie 16 bytes apart
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            page_base[value_offset(token, 8 * j + i, kD)] = from_float<T>(a[i]);
            page_base[value_offset(token, kHalf + 8 * j + i, kD)] = from_float<T>(b[i]);
        }
        return;
    }
    const AnyVec gain = is_q ? q_gain : k_gain;
    if (gain.ptr) {
        const float inv = 1.0f / sqrtf(ss / static_cast<float>(kD) + eps);
        float ga[8], gb[8];
        load_run(gain, 8 * j, ga);
        load_run(gain, kHalf + 8 * j, gb);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            a[i] = (a[i] * ga[i]) * inv;
            b[i] = (b[i] * gb[i]) * inv;
        }
    }
    if (cos_table != nullptr) {
        const int tpos = pos < table_positions ? pos : table_positions - 1;  // host checks the bound
        const HeadRun<float> cs = *reinterpret_cast<const HeadRun<float>*>(cos_table + static_cast<long>(tpos) * kHalf + 8 * j);
        const HeadRun<float> sn = *reinterpret_cast<const HeadRun<float>*>(sin_table + static_cast<long>(tpos) * kHalf + 8 * j);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float ru = a[i] * cs.v[i] - b[i] * sn.v[i];
            const float rv = a[i] * sn.v[i] + b[i] * cs.v[i];
            a[i] = ru;
            b[i] = rv;
        }
    }
    HeadRun<T> lo, hi;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        lo.v[i] = from_float<T>(a[i]);
        hi.v[i] = from_float<T>(b[i]);
    }
    if (is_q) {
        T* dst = q_out + (static_cast<long>(row) * q_heads + head) * kD + 8 * j;
        *reinterpret_cast<HeadRun<T>*>(dst) = lo;
        *reinterpret_cast<HeadRun<T>*>(dst + kHalf) = hi;
    } else {
        *reinterpret_cast<HeadRun<T>*>(page_base + key_offset(token, 8 * j, page_tokens)) = lo;
        *reinterpret_cast<HeadRun<T>*>(page_base + key_offset(token, kHalf + 8 * j, page_tokens)) = hi;
    }
}

// Values of many rows at once.  A run of the value layout is one element of eight consecutive tokens,
// so eight rows that are the consecutive positions 8n .. 8n+7 of one request fill whole runs: a
// workgroup takes eight rows of the step and one kv head, reads the rows in runs of eight elements,
// turns them in shared memory and writes head_dim runs that lie side by side.  Rows that do not line
// up like that (the first and last rows of a portion, single decoded tokens) are written one element
// at a time.  One thread an element of the head.
template <typename T>
__device__ inline void value_write_block(T* turned, int row_block, int kvh, const T* __restrict__ qkv, T* __restrict__ v_pool,
                                         const int* __restrict__ positions, const int* __restrict__ row_entry,
                                         const int* __restrict__ block_table, int max_blocks, int rows, int q_heads,
                                         int kv_heads, int head_dim, int page_tokens) {
    const int row0 = row_block * 8;
    const int d = threadIdx.x;                                          // blockDim.x >= head_dim; threads beyond it only copy
    const int qkv_width = (q_heads + 2 * kv_heads) * head_dim;
    const long head_at = static_cast<long>(q_heads + kv_heads + kvh) * head_dim;
    const int n = rows - row0 < 8 ? rows - row0 : 8;
    const int p0 = positions[row0], e0 = row_entry[row0];
    bool lined_up = n == 8 && (p0 & 7) == 0;
    for (int i = 1; i < n && lined_up; ++i) lined_up = positions[row0 + i] == p0 + i && row_entry[row0 + i] == e0;
    // rows in, a run of eight elements a thread
    for (int idx = threadIdx.x; idx < n * (head_dim / 8); idx += blockDim.x) {
        const int r = idx / (head_dim / 8), chunk = idx % (head_dim / 8);
        *reinterpret_cast<HeadRun<T>*>(turned + r * head_dim + 8 * chunk) =
            *reinterpret_cast<const HeadRun<T>*>(qkv + static_cast<long>(row0 + r) * qkv_width + head_at + 8 * chunk);
    }
    __syncthreads();
    if (d >= head_dim) return;
    if (lined_up) {
        const int page = block_table[static_cast<long>(e0) * max_blocks + p0 / page_tokens];
        if (page < 0) return;  // host reserves pages before the launch
        HeadRun<T> run;
#pragma unroll
        for (int i = 0; i < 8; ++i) run.v[i] = turned[i * head_dim + d];
        T* base = v_pool + (static_cast<long>(page) * kv_heads + kvh) * page_tokens * head_dim;
        *reinterpret_cast<HeadRun<T>*>(base + value_offset(p0 % page_tokens, d, head_dim)) = run;
        return;
    }
    for (int i = 0; i < n; ++i) {
        const int pos = positions[row0 + i];
        const int page = block_table[static_cast<long>(row_entry[row0 + i]) * max_blocks + pos / page_tokens];
        if (page < 0) continue;
        T* base = v_pool + (static_cast<long>(page) * kv_heads + kvh) * page_tokens * head_dim;
        base[value_offset(pos % page_tokens, d, head_dim)] = turned[i * head_dim + d];
    }
}

template <typename T>
__global__ void __launch_bounds__(512)
value_write_kernel(const T* __restrict__ qkv, T* __restrict__ v_pool, const int* __restrict__ positions,
                   const int* __restrict__ row_entry, const int* __restrict__ block_table, int max_blocks,
                   int rows, int q_heads, int kv_heads, int head_dim, int page_tokens) {
    extern __shared__ __align__(32) unsigned char turned_raw[];
    value_write_block<T>(reinterpret_cast<T*>(turned_raw), blockIdx.x, blockIdx.y, qkv, v_pool, positions, row_entry, block_table,
                         max_blocks, rows, q_heads, kv_heads, head_dim, page_tokens);
}

template <typename TIn, typename T, int kD16>
static void launch_runs(const void* qkv, int planes, long plane, void* q_out, void* k_pool, void* v_pool, AnyVec qg, AnyVec kg, float eps,
                        const float* cos_table, const float* sin_table, int table_positions, const int* positions,
                        const int* row_entry, const int* block_table, int max_blocks, int rows, int q_heads,
                        int kv_heads, int page_tokens, int write_cache, hipStream_t stream) {
    constexpr int kShare = kD16 <= 1 ? 1 : kD16 <= 2 ? 2 : kD16 <= 4 ? 4 : 8;
    // Many rows are mostly prompt portions: their values go through the kernel that writes whole runs.
    const bool values_apart = write_cache && rows >= 64 && ceil_div(rows, 8) <= 0x7fffffff && kv_heads <= 65535 &&
                              std::is_same<TIn, T>::value && planes == 1;
    const long items = static_cast<long>(rows) * (q_heads + (write_cache ? (values_apart ? 1 : 2) * kv_heads : 0));
    const int blocks = ceil_div(items * kShare, 256);
    constexpr int kD = 16 * kD16;
    const long value_blocks = values_apart ? static_cast<long>(ceil_div(rows, 8)) * kv_heads : 0;
    if (blocks + value_blocks > 0x7fffffffL) {          // too many for one launch: the values by themselves
        qk_norm_rope_write_runs_kernel<TIn, T, kD16><<<blocks, 256, 0, stream>>>(
            static_cast<const TIn*>(qkv), planes, plane, static_cast<T*>(q_out), static_cast<T*>(k_pool), static_cast<T*>(v_pool), qg, kg, eps,
            cos_table, sin_table, table_positions, positions, row_entry, block_table, max_blocks, rows, q_heads, kv_heads,
            page_tokens, write_cache, 0, 0);
        value_write_kernel<T><<<dim3(ceil_div(rows, 8), kv_heads), kD, 8 * kD * sizeof(T), stream>>>(
            reinterpret_cast<const T*>(qkv), static_cast<T*>(v_pool), positions, row_entry, block_table, max_blocks, rows,
            q_heads, kv_heads, kD, page_tokens);
        return;
    }
    qk_norm_rope_write_runs_kernel<TIn, T, kD16><<<static_cast<int>(blocks + value_blocks), 256, values_apart ? 8 * kD * sizeof(T) : 0, stream>>>(
        static_cast<const TIn*>(qkv), planes, plane, static_cast<T*>(q_out), static_cast<T*>(k_pool), static_cast<T*>(v_pool), qg, kg, eps,
        cos_table, sin_table, table_positions, positions, row_entry, block_table, max_blocks, rows, q_heads, kv_heads,
        page_tokens, write_cache, values_apart ? 0 : 1, static_cast<int>(value_blocks));
}

static int check_dtype(int dtype, const char* what) {
    if (dtype != kF32 && dtype != kBF16) {
        set_error("%s: unknown element type %d", what, dtype);
        return 1;
    }
    return 0;
}

}  // namespace leone

using namespace leone;

extern "C" int leone_soft_cap(float* x, long n, float cap, hipStream_t stream) {
    LEONE_REQUIRE(x && n > 0 && cap > 0.f, "soft_cap: needs values and a positive cap");
    const long blocks = (n + 255) / 256;
    soft_cap_kernel<<<static_cast<int>(blocks < 4096 ? blocks : 4096), 256, 0, stream>>>(x, n, cap);
    LEONE_LAUNCH_CHECK("soft_cap");
    return 0;
}

extern "C" int leone_embed(const void* table, int dtype, const int* tokens, float* out, int rows,
                           int hidden, int vocab, float scale, hipStream_t stream) {
    if (check_dtype(dtype, "embed")) return 1;
    LEONE_REQUIRE(table && tokens && out, "embed: null pointer");
    LEONE_REQUIRE(rows > 0 && hidden > 0 && vocab > 0, "embed: rows %d hidden %d vocab %d must be positive", rows, hidden, vocab);
    const int threads = hidden >= 1024 ? 256 : 64;
    if (dtype == kF32)
        embed_kernel<float><<<rows, threads, 0, stream>>>(static_cast<const float*>(table), tokens, out, hidden, vocab, scale);
    else
        embed_kernel<bf16_t><<<rows, threads, 0, stream>>>(static_cast<const bf16_t*>(table), tokens, out, hidden, vocab, scale);
    LEONE_LAUNCH_CHECK("embed");
    return 0;
}

template <typename TD, typename TG, typename TY>
static void launch_add_rmsnorm_vec(float* x, const void* delta, int planes, long plane, const void* gain, float eps,
                                   void* y, const int* rows, int n_rows, int hidden, float* squares, hipStream_t stream) {
    const TD* d = static_cast<const TD*>(delta);
    const TG* g = static_cast<const TG*>(gain);
    TY* out = static_cast<TY*>(y);
    if (hidden <= 4 * 64 * 2)
        add_rmsnorm_vec_kernel<TD, TG, TY, 64, 2><<<n_rows, 64, 0, stream>>>(x, d, planes, plane, g, eps, out, rows, hidden, squares);
    else if (hidden <= 4 * 256 * 2)
        add_rmsnorm_vec_kernel<TD, TG, TY, 256, 2><<<n_rows, 256, 0, stream>>>(x, d, planes, plane, g, eps, out, rows, hidden, squares);
    else if (hidden <= 4 * 256 * 4)
        add_rmsnorm_vec_kernel<TD, TG, TY, 256, 4><<<n_rows, 256, 0, stream>>>(x, d, planes, plane, g, eps, out, rows, hidden, squares);
    else
        add_rmsnorm_vec_kernel<TD, TG, TY, 256, 8><<<n_rows, 256, 0, stream>>>(x, d, planes, plane, g, eps, out, rows, hidden, squares);
}

template <typename TD, typename TY>
static void launch_add_rmsnorm(float* x, const void* delta, int planes, long plane, AnyVec gain, float eps, void* y,
                               const int* rows, int n_rows, int hidden, float* squares, hipStream_t stream) {
    if (hidden % 4 == 0 && hidden <= 4 * 256 * 8) {
        if (gain.dtype == kF32)
            launch_add_rmsnorm_vec<TD, float, TY>(x, delta, planes, plane, gain.ptr, eps, y, rows, n_rows, hidden, squares, stream);
        else
            launch_add_rmsnorm_vec<TD, bf16_t, TY>(x, delta, planes, plane, gain.ptr, eps, y, rows, n_rows, hidden, squares, stream);
        return;
    }
    if (hidden > 512)
        add_rmsnorm_kernel<TD, TY, 256><<<n_rows, 256, 0, stream>>>(x, static_cast<const TD*>(delta), planes, plane, gain, eps, static_cast<TY*>(y), rows, hidden, squares);
    else
        add_rmsnorm_kernel<TD, TY, 64><<<n_rows, 64, 0, stream>>>(x, static_cast<const TD*>(delta), planes, plane, gain, eps, static_cast<TY*>(y), rows, hidden, squares);
}

extern "C" int leone_add_rmsnorm(float* x, const void* delta, int delta_dtype, int delta_planes, long delta_plane,
                                 const void* gain, int gain_dtype, float eps, void* y, int y_dtype, const int* rows,
                                 int n_rows, int hidden, float* squares_out, hipStream_t stream) {
    if (check_dtype(delta_dtype, "add_rmsnorm delta") || check_dtype(gain_dtype, "add_rmsnorm gain") ||
        check_dtype(y_dtype, "add_rmsnorm output"))
        return 1;
    LEONE_REQUIRE(x && gain && y, "add_rmsnorm: null pointer");
    LEONE_REQUIRE(n_rows > 0 && hidden > 0, "add_rmsnorm: rows %d hidden %d must be positive", n_rows, hidden);
    LEONE_REQUIRE(eps > 0.f && eps == eps, "add_rmsnorm: eps must be positive");
    LEONE_REQUIRE(!delta || (delta_planes >= 1 && delta_planes <= 16 && delta_plane >= 0),
                  "add_rmsnorm: %d planes of what is to be added", delta_planes);
    const int planes = delta_planes;
    const long plane = delta_plane;
    AnyVec g{gain, gain_dtype};
    if (delta_dtype == kF32 && y_dtype == kF32)
        launch_add_rmsnorm<float, float>(x, delta, planes, plane, g, eps, y, rows, n_rows, hidden, squares_out, stream);
    else if (delta_dtype == kBF16 && y_dtype == kBF16)
        launch_add_rmsnorm<bf16_t, bf16_t>(x, delta, planes, plane, g, eps, y, rows, n_rows, hidden, squares_out, stream);
    else if (delta_dtype == kF32 && y_dtype == kBF16)
        launch_add_rmsnorm<float, bf16_t>(x, delta, planes, plane, g, eps, y, rows, n_rows, hidden, squares_out, stream);
    else
        launch_add_rmsnorm<bf16_t, float>(x, delta, planes, plane, g, eps, y, rows, n_rows, hidden, squares_out, stream);
    LEONE_LAUNCH_CHECK("add_rmsnorm");
    return 0;
}

extern "C" int leone_swiglu(const void* gate_up, void* out, int dtype, int rows, int ffn, hipStream_t stream) {
    if (check_dtype(dtype, "swiglu")) return 1;
    LEONE_REQUIRE(gate_up && out, "swiglu: null pointer");
    LEONE_REQUIRE(rows > 0 && ffn > 0 && ffn % 8 == 0, "swiglu: rows %d, width %d: the width must be a positive multiple of 8", rows, ffn);
    const uintptr_t run = 8 * (dtype == kF32 ? sizeof(float) : sizeof(bf16_t));
    LEONE_REQUIRE(reinterpret_cast<uintptr_t>(gate_up) % run == 0 && reinterpret_cast<uintptr_t>(out) % run == 0,
                  "swiglu: input and output must be aligned to %d bytes", static_cast<int>(run));
    const dim3 grid(ceil_div(ffn / 8, 256), rows < 32768 ? rows : 32768);
    if (dtype == kF32)
        swiglu_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(gate_up), static_cast<float*>(out), rows, ffn);
    else
        swiglu_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<const bf16_t*>(gate_up), static_cast<bf16_t*>(out), rows, ffn);
    LEONE_LAUNCH_CHECK("swiglu");
    return 0;
}

extern "C" int leone_rope_table(float* cos_out, float* sin_out, double theta, int rotary_dim,
                                int positions, hipStream_t stream) {
    LEONE_REQUIRE(cos_out && sin_out, "rope_table: null pointer");
    LEONE_REQUIRE(rotary_dim > 0 && rotary_dim % 2 == 0, "rope_table: rotary dim %d must be even and positive", rotary_dim);
    LEONE_REQUIRE(positions > 0, "rope_table: positions %d must be positive", positions);
    LEONE_REQUIRE(theta > 0.0 && theta == theta, "rope_table: theta must be positive");
    const int pairs = rotary_dim / 2;
    const long total = static_cast<long>(positions) * pairs;
    long blocks = (total + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    rope_table_kernel<<<static_cast<int>(blocks), 256, 0, stream>>>(cos_out, sin_out, theta, pairs, rotary_dim, positions);
    LEONE_LAUNCH_CHECK("rope_table");
    return 0;
}

extern "C" int leone_qk_norm_rope_write(const void* qkv, int qkv_dtype, int qkv_planes, long qkv_plane, void* q_out,
                                        void* k_pool, void* v_pool, int dtype,
                                        const void* q_gain, const void* k_gain, int gain_dtype, float eps,
                                        const float* cos_table, const float* sin_table, int table_positions,
                                        int rotary_dim, int pairing,
                                        const int* positions, const int* row_entry, const int* block_table,
                                        int max_blocks, int rows, int q_heads, int kv_heads, int head_dim,
                                        int page_tokens, int write_cache, hipStream_t stream) {
    if (check_dtype(dtype, "qk_norm_rope_write") || check_dtype(gain_dtype, "qk_norm_rope_write gain") ||
        check_dtype(qkv_dtype, "qk_norm_rope_write input"))
        return 1;
    LEONE_REQUIRE(qkv && q_out && positions, "qk_norm_rope_write: null pointer");
    LEONE_REQUIRE(qkv_dtype == dtype || qkv_dtype == kF32, "qk_norm_rope_write: the input is of the output's type or float32");
    LEONE_REQUIRE(qkv_planes >= 1 && qkv_planes <= 64 && (qkv_planes == 1 || qkv_plane % 8 == 0),
                  "qk_norm_rope_write: %d planes of input", qkv_planes);
    LEONE_REQUIRE(!write_cache || (k_pool && v_pool && row_entry && block_table && max_blocks > 0 && page_tokens > 0),
                  "qk_norm_rope_write: cache write needs pools, row map and block table");
    LEONE_REQUIRE((q_gain == nullptr) == (k_gain == nullptr), "qk_norm_rope_write: q and k gains come together");
    LEONE_REQUIRE((cos_table == nullptr) == (sin_table == nullptr), "qk_norm_rope_write: cos and sin tables come together");
    LEONE_REQUIRE(!cos_table || table_positions > 0, "qk_norm_rope_write: empty rotary table");
    LEONE_REQUIRE(!cos_table || (rotary_dim > 0 && rotary_dim % 2 == 0 && rotary_dim <= head_dim),
                  "qk_norm_rope_write: rotary_dim %d must be even, positive and at most head_dim %d", rotary_dim, head_dim);
    LEONE_REQUIRE(pairing == kPairHalfSplit || pairing == kPairAdjacent, "qk_norm_rope_write: unknown pairing %d", pairing);
    // the kernel in runs of 8 is built for the half-split rotation of the whole head (or none)
    const bool whole_head = !cos_table || (rotary_dim == head_dim && pairing == kPairHalfSplit);
    LEONE_REQUIRE(rows > 0 && q_heads > 0 && kv_heads > 0, "qk_norm_rope_write: rows %d heads %d/%d must be positive", rows, q_heads, kv_heads);
    LEONE_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && head_dim <= 2 * kWave * kMaxPairsPerLane,
                  "qk_norm_rope_write: head_dim %d must be even and at most %d", head_dim, 2 * kWave * kMaxPairsPerLane);
    LEONE_REQUIRE(!write_cache || (head_dim % 8 == 0 && page_tokens % 8 == 0),
                  "qk_norm_rope_write: the cache needs head_dim %d and page_tokens %d to be multiples of 8", head_dim, page_tokens);
    AnyVec qg{q_gain, gain_dtype}, kg{k_gain, gain_dtype};
    const uintptr_t run_bytes = 8 * (dtype == kF32 ? sizeof(float) : sizeof(bf16_t));
    const uintptr_t in_run_bytes = 8 * (qkv_dtype == kF32 ? sizeof(float) : sizeof(bf16_t));
    const bool aligned = reinterpret_cast<uintptr_t>(qkv) % in_run_bytes == 0 && reinterpret_cast<uintptr_t>(q_out) % run_bytes == 0 &&
                         (!write_cache || (reinterpret_cast<uintptr_t>(k_pool) % run_bytes == 0 && page_tokens % 8 == 0));
    const bool tables_aligned = (!q_gain || (reinterpret_cast<uintptr_t>(q_gain) % 32 == 0 && reinterpret_cast<uintptr_t>(k_gain) % 32 == 0)) &&
                                (!cos_table || (reinterpret_cast<uintptr_t>(cos_table) % 32 == 0 && reinterpret_cast<uintptr_t>(sin_table) % 32 == 0));
    if (whole_head && head_dim % 16 == 0 && head_dim <= 128 && aligned && tables_aligned && static_cast<long>(rows) * (q_heads + 2 * kv_heads) * 8 < 0x7fffffffL * 256) {
#define LEONE_RUNS_ARGS                                                                                             \
    qkv, qkv_planes, qkv_plane, q_out, k_pool, v_pool, qg, kg, eps, cos_table, sin_table, table_positions, positions, \
        row_entry, block_table, max_blocks, rows, q_heads, kv_heads, page_tokens, write_cache, stream
#define LEONE_RUNS_CASE(N)                                                     \
    case N:                                                                    \
        if (dtype == kF32) launch_runs<float, float, N>(LEONE_RUNS_ARGS);      \
        else if (qkv_dtype == kF32) launch_runs<float, bf16_t, N>(LEONE_RUNS_ARGS); \
        else launch_runs<bf16_t, bf16_t, N>(LEONE_RUNS_ARGS);                  \
        break;
        switch (head_dim / 16) {
            LEONE_RUNS_CASE(1) LEONE_RUNS_CASE(2) LEONE_RUNS_CASE(3) LEONE_RUNS_CASE(4)
            LEONE_RUNS_CASE(5) LEONE_RUNS_CASE(6) LEONE_RUNS_CASE(7) LEONE_RUNS_CASE(8)
        }
#undef LEONE_RUNS_CASE
#undef LEONE_RUNS_ARGS
        LEONE_LAUNCH_CHECK("qk_norm_rope_write");
        return 0;
    }
    const int heads_total = q_heads + (write_cache ? 2 * kv_heads : 0);
    const int waves_per_block = 4;
    dim3 grid(rows, ceil_div(heads_total, waves_per_block));
#define LEONE_QK_ANY(TIN, T)                                                                                        \
    qk_norm_rope_write_kernel<TIN, T><<<grid, waves_per_block * kWave, 0, stream>>>(                                \
        static_cast<const TIN*>(qkv), qkv_planes, qkv_plane, static_cast<T*>(q_out), static_cast<T*>(k_pool),       \
        static_cast<T*>(v_pool), qg, kg, eps, cos_table, sin_table, table_positions, positions, row_entry,          \
        block_table, max_blocks, q_heads, kv_heads, head_dim, page_tokens, write_cache, cos_table ? rotary_dim / 2 : 0, pairing)
    if (dtype == kF32) LEONE_QK_ANY(float, float);
    else if (qkv_dtype == kF32) LEONE_QK_ANY(float, bf16_t);
    else LEONE_QK_ANY(bf16_t, bf16_t);
#undef LEONE_QK_ANY
    LEONE_LAUNCH_CHECK("qk_norm_rope_write");
    return 0;
}
