// The weight-streaming matrix product for 1 to 128 rows of X: Y[M,N] = X[M,K] . W[N,K]^T, bfloat16 operands,
// float accumulation.  This is the product of a decode step with many requests, where the reference runs its
// own multi-row matrix-vector kernels with folded epilogues (crates/leone/src/runtime.rs:7865-7906,
// crates/leone-cuda/cuda/ie_cuda.cu:1932, 2011, 6208): W is read from memory exactly once, X is small.
//
// A workgroup owns 4, 6 or 8 tiles of 16 rows of W and a range of K; the ranges of K (blockIdx.y,
// `splits` of them) exist so that matrices with few rows still give every compute unit a workgroup (the
// kernel is fastest with exactly one workgroup a compute unit: the caller picks waves and splits for that).
// A tile of W belongs to one wave, or (more than 64 rows of X) to two waves that share out the 32-element
// units of every chunk between them and add their sums up through shared memory at the end, in a fixed order:
// the workgroup then has two waves a SIMD instead of one, so that one wave's wait for shared memory, for a
// barrier or for its weights is the other's time on the matrix cores, and twice the weights are on their way.
// What W costs in memory traffic X must not cost again in cache traffic: every wave needs all of X, so X
// goes through shared memory, one chunk of K at a time (256 elements, 128 for more than 64 rows), copied
// there once per workgroup with 16-byte loads that run along the rows, while the waves work on the chunk
// before; W goes from memory straight into registers, one chunk ahead: a register that a matrix
// instruction has used is filled again at once.  A row of the chunk in shared memory is 32 (16) runs of 16
// bytes; run s of row r sits at place s ^ (r % 16), so that the sixteen lanes that read the same run of
// sixteen rows hit sixteen different banks.
//
// The products are v_mfma_f32_16x16x32_bf16 with W as the first operand: in a step of 64 elements lane
// (c, g) holds elements 16g .. 16g+15 of weight row c (32 contiguous bytes, so four lanes take a row's
// whole 128-byte line) and the same elements of X row c; both operands use the same assignment of elements
// to the instruction's k-slots, which is all it needs.  Afterwards lane (c, g) holds Y[row c][4g .. 4g+3]
// of each 16 x 16 tile.
//
// Outputs: store (bfloat16 or float), add into the float32 stream, or silu(gate) * up for a weight that
// interleaves 8 gate rows with their 8 up rows (crates/leone/src/cpu.rs:892-907).  With splits > 1 every
// range of K writes its own float plane [M,N], `plane` elements apart, and whoever reads them adds them
// up in order; sums are taken in a fixed order everywhere, so a launch repeats bit for bit, and a row of X
// gives the same bits whatever the other rows are.
#include "common.h"
#include "leone_hip.h"

#include <math.h>

namespace leone {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

enum RowsOut : int { kRowsStore = 0, kRowsResidual = 1, kRowsGated = 2, kRowsPlanes = 3 };

struct RowsArgs {
    const bf16_t* x;   // [M,K]
    const bf16_t* w;   // [N,K], or its tiled copy
    void* y;
    long plane;        // elements between two planes of y (kRowsPlanes)
    int m, n, k;
    int chunks_per_split;
};


__device__ inline uint4 rld(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ inline uint4 wld(const bf16_t* p) { return load_streamed16(p); }   // weights: read once

// kMT: tiles of 16 rows of X; kWaves: tiles of 16 rows of W a workgroup; kWays: waves that share a tile of W
// (each takes kUnits / kWays units of every chunk); kSteps: steps of 64 elements a chunk; kDepth: chunks the
// weights are asked for ahead.
template <int kMT, int kWaves, int kWays, int kSteps, int kDepth, int kOut, typename TOut, bool kTiled>
__global__ void __launch_bounds__(kWaves * kWays * kWave)
gemm_rows_kernel(RowsArgs a) {
    constexpr int kChunk = 64 * kSteps;              // elements of K a chunk
    constexpr int kRuns = kChunk / 8;                // 16-byte runs of a row of the chunk
    constexpr int kXRows = 16 * kMT;
    constexpr int kThreads = kWaves * kWays * kWave;
    constexpr int kCopies = (kXRows * kRuns + kThreads - 1) / kThreads;   // runs of X a thread copies per chunk
    constexpr bool kEven = kXRows * kRuns % kThreads == 0;
    constexpr int kChunkUnits = 2 * kSteps;          // 32-element units of a chunk
    static_assert(kChunkUnits % kWays == 0, "the units of a chunk must share out evenly");
    constexpr int kUnits = kChunkUnits / kWays;      // units of a chunk this wave takes: matrix instructions per tile of X
    extern __shared__ uint4 lds[];                   // two chunks of X: [2][kXRows][kRuns]; at the end the waves' sums

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x % kWave;
    const int tid = threadIdx.x;
    const int c = lane & 15, g = lane >> 4;
    const int m = a.m, n = a.n, k = a.k;
    const int way = wave / kWaves;                   // which share of every chunk's units
    const int unit0 = way * kUnits;                  // its first unit in a chunk

    // This wave's weight rows; rows past the end are clamped and their results never stored.
    const long tile = static_cast<long>(blockIdx.x) * kWaves + wave % kWaves;
    const long wr = 16 * tile + c;
    const bf16_t* wrow = a.w + (wr < n ? wr : n - 1) * k;
    // Tiled weights: the 16 bytes of lane L for half h of step S of a tile lie at ((S * 2 + h) * 64 + L) * 16 in
    // the tile, so that every load of a wave is 1 KB in one piece; K is a multiple of 64 there.
    const int all_steps = k / 64;
    const long tiles_n = (n + 15) / 16;
    const bf16_t* wtile = a.w + (tile < tiles_n ? tile : tiles_n - 1) * all_steps * 1024 + lane * 8;
    // The runs of X this thread copies: copy i is run (i * threads + tid) % kRuns of row (i * threads + tid) / kRuns.
    const bf16_t* xsrc[kCopies];
    int xdst[kCopies], xcol[kCopies];
#pragma unroll
    for (int i = 0; i < kCopies; ++i) {
        const int idx = i * kThreads + tid;
        const int row = (idx / kRuns) % kXRows, run = idx % kRuns;   // a copy past the end repeats an earlier one
        xsrc[i] = a.x + static_cast<long>(row < m ? row : m - 1) * k;
        xdst[i] = row * kRuns + (run ^ (row & 15));
        xcol[i] = 8 * run;
    }

    const int chunks = (k + kChunk - 1) / kChunk;
    const int ch_begin = blockIdx.y * a.chunks_per_split;
    const int ch_end = ch_begin + a.chunks_per_split < chunks ? ch_begin + a.chunks_per_split : chunks;

    floatx4 acc[kMT];
#pragma unroll
    for (int t = 0; t < kMT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

    // Loads of one chunk, X first: what waits for X to put it into shared memory leaves the weights, which
    // were asked for later, on their way.  A load that would start beyond the end of K starts at the row's
    // last run instead; X is cleared there, and so the weights read twice meet zeros.  No branches: the
    // compiler counts loads in flight along every path and would wait for all of them where paths join.
    auto fetch_x = [&](int ch, uint4 (&xn)[kCopies]) {
        const int k0 = ch * kChunk;
#pragma unroll
        for (int i = 0; i < kCopies; ++i) {
            const int at = k0 + xcol[i];
            xn[i] = rld(xsrc[i] + (at + 8 <= k ? at : k - 8));
        }
    };
    auto w_at = [&](int ch, int mine) {
        const int u = unit0 + mine;
        if constexpr (kTiled) {
            const int step = ch * kSteps + (u >> 1);
            return load_streamed16(wtile + static_cast<long>(step < all_steps ? step : all_steps - 1) * 1024 + 512 * (u & 1));
        } else {
            const int at = ch * kChunk + 16 * g + 64 * (u >> 1) + 8 * (u & 1);
            return rld(wrow + (at + 8 <= k ? at : k - 8));
        }
    };
    // Weights beyond the end of K count as zero themselves (not only through the zeros of X: a weight that is
    // not finite would turn 0 into NaN).  The load is made all the same, from the row's end, and cleared when
    // it is used: a select right behind the load would wait for it.
    auto w_inside = [&](int ch, int mine) {
        const int u = unit0 + mine;
        if constexpr (kTiled) return ch * kSteps + (u >> 1) < all_steps;
        else return ch * kChunk + 16 * g + 64 * (u >> 1) + 8 * (u & 1) + 8 <= k;
    };
    auto deposit = [&](uint4* to, const uint4 (&xn)[kCopies], int ch) {
        const int k0 = ch * kChunk;
#pragma unroll
        for (int i = 0; i < kCopies; ++i) {
            const bool inside = k0 + xcol[i] + 8 <= k;
            const uint4 v = xn[i];
            if (kEven || i + 1 < kCopies || (kCopies - 1) * kThreads + tid < kXRows * kRuns)
                to[xdst[i]] = uint4{inside ? v.x : 0u, inside ? v.y : 0u, inside ? v.z : 0u, inside ? v.w : 0u};
        }
    };
    // The matrix instructions of one chunk.  The operands from shared memory are asked for one group of
    // instructions ahead, so that their way out of shared memory is covered by the group before; a weight
    // register that has been used is filled again at once, from the next chunk.
    uint4 wreg[kDepth][kUnits];
    auto compute = [&](const uint4* from, uint4 (&wreg)[kUnits], int present, int next) {
        bf16x8 xb[2][kMT];
        auto read_x = [&](int mine, bf16x8 (&to)[kMT]) {
            const int u = unit0 + mine;
            const int run = (4 * u + 2 * g - 3 * (u & 1)) ^ c;          // 8 (u / 2) + 2 g + u % 2
#pragma unroll
            for (int t = 0; t < kMT; ++t) to[t] = __builtin_bit_cast(bf16x8, from[(16 * t + c) * kRuns + run]);
        };
        read_x(0, xb[0]);
#pragma unroll
        for (int u = 0; u < kUnits; ++u) {
            if (u + 1 < kUnits) read_x(u + 1, xb[(u + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);       // the reads stay ahead of the instructions they are not for
            const bool inside = w_inside(present, u);
            const uint4 held = wreg[u];
            const bf16x8 wa = __builtin_bit_cast(bf16x8, uint4{inside ? held.x : 0u, inside ? held.y : 0u,
                                                               inside ? held.z : 0u, inside ? held.w : 0u});
#pragma unroll
            for (int t = 0; t < kMT; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xb[u & 1][t], acc[t], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            wreg[u] = w_at(next, u);
        }
    };

    // Workgroups start at different chunks of their range and go round it, so that at any moment they ask
    // for different parts of X: the rows of X lie a power of two apart, and every workgroup asking for the
    // same columns of all rows at once would crowd a few channels of the cache.  The order of the sum over K
    // thus depends on the workgroup (on the columns of Y), never on the rows of X or on the launch.
    const int count = ch_end - ch_begin;
    const int rot = count <= 0 ? 0 : static_cast<int>(blockIdx.x % count);
    auto chunk_at = [&](int i) { const int r = i + rot; return ch_begin + (r >= count ? r - count : r); };
    uint4 xn[kCopies];
    auto chunk_or_last = [&](int i) { return chunk_at(i < count ? i : count - 1); };
    if (count > 0) {
        fetch_x(chunk_at(0), xn);
#pragma unroll
        for (int d = 0; d < kDepth; ++d)
#pragma unroll
            for (int u = 0; u < kUnits; ++u) wreg[d][u] = w_at(chunk_or_last(d), u);
        deposit(lds, xn, chunk_at(0));
    }
    __syncthreads();
    // The weights are asked for kDepth chunks ahead, X one chunk ahead, always (after the last chunk: the
    // last chunk again, unused).
    constexpr int kHalf = kXRows * kRuns;
    int cur = 0;
    for (int i = 0; i < count; i += kDepth) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            if (d > 0 && i + d >= count) break;
            const int next = chunk_or_last(i + d + 1);
            fetch_x(next, xn);
            compute(lds + cur * kHalf, wreg[d], chunk_at(i + d), chunk_or_last(i + d + kDepth));
            cur ^= 1;
            __builtin_amdgcn_sched_barrier(0);
            deposit(lds + cur * kHalf, xn, next);
            __syncthreads();
        }
    }

    // The waves that shared a tile of W add up: every wave but the tile's first leaves its sums in shared
    // memory (the chunks of X are done with), the first adds them in the order of the shares.
    if constexpr (kWays > 1) {
        floatx4* sums = reinterpret_cast<floatx4*>(lds);   // [kWays - 1][kWaves][kMT][64]
        if (way > 0) {
#pragma unroll
            for (int t = 0; t < kMT; ++t) sums[(((way - 1) * kWaves + wave % kWaves) * kMT + t) * kWave + lane] = acc[t];
        }
        __syncthreads();
        if (way > 0) return;
#pragma unroll
        for (int other = 1; other < kWays; ++other)
#pragma unroll
            for (int t = 0; t < kMT; ++t) {
                const floatx4 part = sums[(((other - 1) * kWaves + wave) * kMT + t) * kWave + lane];
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[t][r] += part[r];
            }
    }

    // Lane (c, g) holds, for tile t, Y[16t + c][16 tile + 4g .. + 3].
    const long col = 16 * tile + 4 * g;
#pragma unroll
    for (int t = 0; t < kMT; ++t) {
        const int row = 16 * t + c;
        if (kOut == kRowsGated) {
            // local rows 0..7 of a tile are gate rows, 8..15 the up rows that belong to them: lanes
            // g = 0, 1 hold gates, lanes g + 2 the matching ups
            floatx4 up;
#pragma unroll
            for (int r = 0; r < 4; ++r) up[r] = __shfl_xor(acc[t][r], 32, kWave);
            if (g < 2 && row < m && col < n) {
                bf16_t* out = static_cast<bf16_t*>(a.y) + static_cast<long>(row) * (n / 2) + 8 * tile + 4 * g;
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float gate = acc[t][r];
                    v[r] = (gate / (1.0f + expf(-gate))) * up[r];
                }
                uint2 packed;
                packed.x = bf16_bits_from_float(v[0]) | (static_cast<uint32_t>(bf16_bits_from_float(v[1])) << 16);
                packed.y = bf16_bits_from_float(v[2]) | (static_cast<uint32_t>(bf16_bits_from_float(v[3])) << 16);
                *reinterpret_cast<uint2*>(out) = packed;
            }
            continue;
        }
        if (row >= m || col >= n) continue;
        if (kOut == kRowsResidual) {
            float* out = static_cast<float*>(a.y) + static_cast<long>(row) * n + col;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (col + r < n) out[r] += acc[t][r];
        } else if (kOut == kRowsPlanes) {
            float* out = static_cast<float*>(a.y) + blockIdx.y * a.plane + static_cast<long>(row) * n + col;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (col + r < n) out[r] = acc[t][r];
        } else {
            TOut* out = static_cast<TOut*>(a.y) + static_cast<long>(row) * n + col;
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (col + r < n) out[r] = from_float<TOut>(acc[t][r]);
        }
    }
}

template <int kMT, int kWaves, int kWays, int kOut, typename TOut, bool kTiled>
static int launch_rows_laid(const RowsArgs& a, int splits, hipStream_t stream) {
    constexpr int kSteps = kMT <= 4 ? 4 : 2;
    constexpr int kDepth = kWays;                      // a wave keeps a whole chunk's worth of its weights on the way
    const size_t chunks_of_x = 2 * static_cast<size_t>(16 * kMT) * (64 * kSteps / 8) * sizeof(uint4);
    const size_t sums = static_cast<size_t>(kWays - 1) * kWaves * kMT * kWave * sizeof(floatx4);
    const size_t shared = chunks_of_x > sums ? chunks_of_x : sums;
    static size_t allowed = 48 * 1024;                 // what a kernel may use without asking
    if (shared > allowed) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_rows_kernel<kMT, kWaves, kWays, kSteps, kDepth, kOut, TOut, kTiled>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(shared));
        if (e != hipSuccess) {
            set_error("gemm_rows: %zu bytes of shared memory were refused: %s", shared, hipGetErrorString(e));
            return 1;
        }
        allowed = shared;
    }
    const int groups = ceil_div(a.n, 16 * kWaves);
    gemm_rows_kernel<kMT, kWaves, kWays, kSteps, kDepth, kOut, TOut, kTiled><<<dim3(groups, splits), kWaves * kWays * kWave, shared, stream>>>(a);
    return 0;
}

template <int kMT, int kWaves, int kWays, int kOut, typename TOut>
static int launch_rows(const RowsArgs& a, int splits, bool tiled, hipStream_t stream) {
    return tiled ? launch_rows_laid<kMT, kWaves, kWays, kOut, TOut, true>(a, splits, stream)
                 : launch_rows_laid<kMT, kWaves, kWays, kOut, TOut, false>(a, splits, stream);
}

template <int kMT, int kWaves, int kWays>
static int launch_rows_out(const RowsArgs& a, int out_mode, int out_dtype, int splits, bool tiled, hipStream_t stream) {
    switch (out_mode) {
        case kRowsStore:
            return out_dtype == kF32 ? launch_rows<kMT, kWaves, kWays, kRowsStore, float>(a, splits, tiled, stream)
                                     : launch_rows<kMT, kWaves, kWays, kRowsStore, bf16_t>(a, splits, tiled, stream);
        case kRowsResidual: return launch_rows<kMT, kWaves, kWays, kRowsResidual, float>(a, splits, tiled, stream);
        case kRowsGated: return launch_rows<kMT, kWaves, kWays, kRowsGated, bf16_t>(a, splits, tiled, stream);
        default: return launch_rows<kMT, kWaves, kWays, kRowsPlanes, float>(a, splits, tiled, stream);
    }
}

// Which (tiles, shares) a workgroup may have.  Two waves a tile are built where they were measured to gain:
// more than 64 rows of X (a wave then has twice the matrix instructions and reads of shared memory a unit of
// K, and a second wave on its SIMD fills its waits: 6,144 x 4,096 at 128 rows 21.3 against 23.9 us, 4,096 x
// 12,288 31.9 against 33.1); up to 64 rows they were level or 1 us slower, and four waves a tile no better.
constexpr bool rows_shape_built(int mt, int waves, int ways) {
    return ways == 1 || (ways == 2 && mt >= 6 && waves <= 6);
}

template <int kMT, int kWaves, int kWays>
static int launch_rows_if_built(const RowsArgs& a, int out_mode, int out_dtype, int splits, bool tiled, hipStream_t stream) {
    if constexpr (rows_shape_built(kMT, kWaves, kWays)) {
        return launch_rows_out<kMT, kWaves, kWays>(a, out_mode, out_dtype, splits, tiled, stream);
    } else {
        set_error("gemm_rows: %d tiles of W shared by %d waves each are not built for %d rows", kWaves, kWays, a.m);
        return 1;
    }
}

template <int kMT>
static int launch_rows_waves(const RowsArgs& a, int out_mode, int out_dtype, int splits, int waves, int ways, bool tiled,
                             hipStream_t stream) {
#define LEONE_ROWS_SHAPE(W, S) \
    if (waves == W && ways == S) return launch_rows_if_built<kMT, W, S>(a, out_mode, out_dtype, splits, tiled, stream);
    LEONE_ROWS_SHAPE(4, 1) LEONE_ROWS_SHAPE(6, 1) LEONE_ROWS_SHAPE(8, 1)
    LEONE_ROWS_SHAPE(4, 2) LEONE_ROWS_SHAPE(6, 2)
#undef LEONE_ROWS_SHAPE
    set_error("gemm_rows: %d tiles of W a workgroup, %d waves a tile", waves, ways);
    return 1;
}

}  // namespace leone

using namespace leone;

extern "C" int leone_gemm_rows_max_rows() { return 128; }
extern "C" int leone_gemm_rows_chunk(int m) { return m <= 64 ? 256 : 128; }

// x bfloat16 [m,k], w bfloat16 [n,k] (or, with w_tiled, what leone_weight_tiles made of it; k a multiple of 64
// then), m in 1..128, k a multiple of 8.  out_mode 0: y[m,n] of out_dtype;
// 1: y float32 [m,n] += product; 2: w interleaves 8 gate rows with their 8 up rows (n a multiple of 16),
// y bfloat16 [m,n/2] = silu(gate) * up; 3: y float32 [splits][m,n], `plane` elements apart, the product over
// the s-th range of k in plane s (every plane is written whole).  splits must be 1 unless out_mode is 3; the
// ranges are whole chunks of k and none may be empty.  waves (4, 6 or 8): 16 * waves rows of w a
// workgroup; ways (1 or 2, what leone_gemm_rows_shape_built allows): waves that share each of those tiles;
// tuning choices both: the result does not depend on them beyond the order of the sum over k.
extern "C" int leone_gemm_rows_shape_built(int m, int waves, int ways) {
    const int tiles = ceil_div(m, 16);
    const int mt = tiles <= 4 ? tiles : tiles <= 6 ? 6 : 8;
    return (waves == 4 || waves == 6 || waves == 8) && (ways == 1 || ways == 2) && rows_shape_built(mt, waves, ways);
}

extern "C" int leone_gemm_rows_bf16(const void* x, const void* w, int w_tiled, void* y, int out_mode, int out_dtype,
                                    int m, int n, int k, int splits, long plane, int waves, int ways, hipStream_t stream) {
    LEONE_REQUIRE(x && w && y, "gemm_rows: null pointer");
    LEONE_REQUIRE(!w_tiled || (k % 64 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0),
                  "gemm_rows: tiled weights need K %d to be a multiple of 64", k);
    LEONE_REQUIRE(m > 0 && m <= 128, "gemm_rows: rows %d must be in 1..128", m);
    LEONE_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_rows: sizes %d x %d: K must be a positive multiple of 8", n, k);
    LEONE_REQUIRE(out_mode >= kRowsStore && out_mode <= kRowsPlanes, "gemm_rows: unknown output mode %d", out_mode);
    LEONE_REQUIRE(out_mode != kRowsGated || n % 16 == 0, "gemm_rows: gated output needs N %d to be a multiple of 16", n);
    LEONE_REQUIRE(out_mode != kRowsStore || out_dtype == kF32 || out_dtype == kBF16, "gemm_rows: unknown output type");
    LEONE_REQUIRE(waves == 4 || waves == 6 || waves == 8, "gemm_rows: %d tiles of W a workgroup", waves);
    LEONE_REQUIRE(leone_gemm_rows_shape_built(m, waves, ways), "gemm_rows: %d waves a tile of W are not built for %d tiles and %d rows",
                  ways, waves, m);
    const int chunk = leone_gemm_rows_chunk(m);
    const int chunks = ceil_div(k, chunk);
    LEONE_REQUIRE(splits >= 1 && splits <= chunks && splits <= 65535, "gemm_rows: %d ranges of K for %d chunks", splits, chunks);
    LEONE_REQUIRE(splits == 1 || out_mode == kRowsPlanes, "gemm_rows: ranges of K need the planes output");
    const int per = ceil_div(chunks, splits);
    LEONE_REQUIRE(per * (splits - 1) < chunks, "gemm_rows: %d ranges of K would leave one empty (%d chunks)", splits, chunks);
    LEONE_REQUIRE(out_mode != kRowsPlanes || plane >= static_cast<long>(m) * n, "gemm_rows: planes overlap");
    RowsArgs a{static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), y, plane, m, n, k, per};
    int status = 0;
#define LEONE_ROWS_CASE(MT) \
    case MT: status = launch_rows_waves<MT>(a, out_mode, out_dtype, splits, waves, ways, w_tiled != 0, stream); break;
    const int tiles = ceil_div(m, 16);
    switch (tiles <= 4 ? tiles : tiles <= 6 ? 6 : 8) {
        LEONE_ROWS_CASE(1) LEONE_ROWS_CASE(2) LEONE_ROWS_CASE(3) LEONE_ROWS_CASE(4) LEONE_ROWS_CASE(6) LEONE_ROWS_CASE(8)
        default:
            set_error("gemm_rows: %d rows are not supported", m);
            return 1;
    }
#undef LEONE_ROWS_CASE
    if (status) return status;
    LEONE_LAUNCH_CHECK("gemm_rows");
    return 0;
}
