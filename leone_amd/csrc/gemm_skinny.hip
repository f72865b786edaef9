// Matrix product for few rows on the matrix cores: Y[M,N] = X[M,K] . W[N,K]^T,
// bfloat16 in, float accumulation, for M up to 64 (decode batches, logits of
// the wanted rows).  The weight matrix is streamed once; this is the place of
// the reference's row-per-block matrix-vector kernels
// (crates/leone-cuda/cuda/ie_cuda.cu:1719, launch shape :6178-6205).
//
// A workgroup of four waves owns 16 rows of W and splits K between its waves in
// steps of 64 elements; a wave computes Y^T tiles (16 rows of W x 16 rows of X)
// with v_mfma_f32_16x16x32_bf16, W as the A operand, X as the B operand.  Lane
// (c, g) reads 32 contiguous bytes of weight row c per step (elements 16g ..
// 16g+15 of the step), so a row's four lanes take a whole 128-byte line; both
// operands use the same assignment of elements to k-slots, which is all the
// instruction needs.  The four partial tiles are added in wave order in shared
// memory, so a launch repeats bit for bit.
#include "common.h"
#include "leone_hip.h"

namespace leone {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;


__device__ inline bf16x8 ld8(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}
__device__ inline bf16x8 z8() {
    uint4 z = {0u, 0u, 0u, 0u};
    return __builtin_bit_cast(bf16x8, z);
}

template <typename T>
__device__ inline void store4(T* p, floatx4 v);
template <>
__device__ inline void store4<float>(float* p, floatx4 v) {
    p[0] = v[0]; p[1] = v[1]; p[2] = v[2]; p[3] = v[3];
}
template <>
__device__ inline void store4<bf16_t>(bf16_t* p, floatx4 v) {
#pragma unroll
    for (int r = 0; r < 4; ++r) p[r] = from_float<bf16_t>(v[r]);
}

// kMT: 16-row tiles of X (M <= 16 * kMT).  kTail: K is not a multiple of 64.  kSkinnyWaves: waves of a
// workgroup, which split K between them (more for matrices with few rows, so that the chip is filled).
template <int kMT, bool kTail, int kSkinnyWaves, typename TOut>
__global__ void __launch_bounds__(kSkinnyWaves * kWave)
gemm_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, TOut* __restrict__ y, int m, int n,
                   int k) {
    __shared__ float partial[kSkinnyWaves][kMT][kWave][4];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);   // uniform: loops on it are scalar
    const int lane = threadIdx.x % kWave;
    const int c = lane & 15, g = lane >> 4;
    const long n0 = static_cast<long>(blockIdx.x) * 16;
    // Rows past the end are clamped: they only feed output rows and columns that are never stored.
    const long wr = n0 + c < n ? n0 + c : n - 1;
    const bf16_t* wrow = w + wr * k + 16 * g;
    const bf16_t* xrow[kMT];
#pragma unroll
    for (int t = 0; t < kMT; ++t) {
        const int xr = 16 * t + c < m ? 16 * t + c : m - 1;
        xrow[t] = x + static_cast<long>(xr) * k + 16 * g;
    }
    floatx4 acc[kMT];
#pragma unroll
    for (int t = 0; t < kMT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

    // One step: 64 elements of K.  `left` is how many elements of this lane's 16-element run exist.
    auto step = [&](int s, bf16x8 a0, bf16x8 a1, bool tail) {
        const int at = 64 * s;
        const int left = tail ? k - (at + 16 * g) : 16;
#pragma unroll
        for (int t = 0; t < kMT; ++t) {
            const bf16x8 b0 = left >= 8 ? ld8(xrow[t] + at) : z8();
            const bf16x8 b1 = left >= 16 ? ld8(xrow[t] + at + 8) : z8();
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b1, acc[t], 0, 0, 0);
        }
    };

    // Each wave takes a contiguous share of K, so that it reads long runs of every weight row.
    const int whole = k / 64;                        // steps of 64 elements without a tail
    const int share = (whole + kSkinnyWaves - 1) / kSkinnyWaves;
    const int s_end = (wave + 1) * share < whole ? (wave + 1) * share : whole;
    constexpr int kUnroll = 4;                       // weight loads of four steps are in flight together
    int s = wave * share;
    for (; s + kUnroll <= s_end; s += kUnroll) {
        bf16x8 a[kUnroll][2];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            a[u][0] = ld8(wrow + 64 * (s + u));
            a[u][1] = ld8(wrow + 64 * (s + u) + 8);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) step(s + u, a[u][0], a[u][1], false);
    }
    for (; s < s_end; ++s) step(s, ld8(wrow + 64 * s), ld8(wrow + 64 * s + 8), false);
    if (kTail && wave == kSkinnyWaves - 1) {                 // the last wave also takes the step that holds the end of K
        const int left = k - (64 * whole + 16 * g);
        step(whole, left >= 8 ? ld8(wrow + 64 * whole) : z8(), left >= 16 ? ld8(wrow + 64 * whole + 8) : z8(), true);
    }
#pragma unroll
    for (int t = 0; t < kMT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) partial[wave][t][lane][r] = acc[t][r];
    __syncthreads();
    // Wave t adds the four partial tiles of X tile t, in wave order.  Lane (c, g) holds
    // output rows (of W) n0 + 4g .. 4g+3 for X row 16t + c.
    for (int t = wave; t < kMT; t += kSkinnyWaves) {
        floatx4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int v = 0; v < kSkinnyWaves; ++v)
#pragma unroll
            for (int r = 0; r < 4; ++r) sum[r] += partial[v][t][lane][r];
        const int row = 16 * t + c;
        const long col = n0 + 4 * g;
        if (row < m) {
            TOut* out = y + static_cast<long>(row) * n + col;
            if (col + 4 <= n) {
                store4<TOut>(out, sum);
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (col + r < n) out[r] = from_float<TOut>(sum[r]);
            }
        }
    }
}

template <int kMT, int kWaves, typename TOut>
static void launch_skinny_waves(const void* x, const void* w, void* y, int m, int n, int k, hipStream_t stream) {
    const int blocks = ceil_div(n, 16);
    if (k % 64 == 0)
        gemm_skinny_kernel<kMT, false, kWaves, TOut><<<blocks, kWaves * kWave, 0, stream>>>(
            static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<TOut*>(y), m, n, k);
    else
        gemm_skinny_kernel<kMT, true, kWaves, TOut><<<blocks, kWaves * kWave, 0, stream>>>(
            static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<TOut*>(y), m, n, k);
}

// Enough waves to fill 256 CUs with several waves a SIMD: matrices with few rows split K further.
// The choice does not depend on the number of rows of X, so a row's result has the same bits
// whatever batch it is part of.
template <int kMT, typename TOut>
static void launch_skinny(const void* x, const void* w, void* y, int m, int n, int k, hipStream_t stream) {
    const int tiles = ceil_div(n, 16);
    const int steps = ceil_div(k, 64);
    if (tiles * 4 >= 4096 || steps < 16)
        launch_skinny_waves<kMT, 4, TOut>(x, w, y, m, n, k, stream);
    else
        launch_skinny_waves<kMT, 8, TOut>(x, w, y, m, n, k, stream);
}

template <typename TOut>
static int dispatch_skinny(const void* x, const void* w, void* y, int m, int n, int k, hipStream_t stream) {
    switch ((m + 15) / 16) {
        case 1: launch_skinny<1, TOut>(x, w, y, m, n, k, stream); break;
        case 2: launch_skinny<2, TOut>(x, w, y, m, n, k, stream); break;
        case 3: launch_skinny<3, TOut>(x, w, y, m, n, k, stream); break;
        case 4: launch_skinny<4, TOut>(x, w, y, m, n, k, stream); break;
        default: set_error("gemm_skinny: %d rows exceed 64", m); return 1;
    }
    return 0;
}

}  // namespace leone

using namespace leone;

extern "C" int leone_gemm_skinny_bf16(const void* x, const void* w, void* y, int out_dtype, int m, int n, int k,
                                      hipStream_t stream) {
    LEONE_REQUIRE(x && w && y, "gemm_skinny: null pointer");
    LEONE_REQUIRE(m > 0 && m <= 64, "gemm_skinny: rows %d must be in 1..64", m);
    LEONE_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_skinny: sizes %d x %d: K must be a positive multiple of 8", n, k);
    LEONE_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "gemm_skinny: unknown output type %d", out_dtype);
    const int status = out_dtype == kF32 ? dispatch_skinny<float>(x, w, y, m, n, k, stream)
                                         : dispatch_skinny<bf16_t>(x, w, y, m, n, k, stream);
    if (status) return status;
    LEONE_LAUNCH_CHECK("gemm_skinny");
    return 0;
}
