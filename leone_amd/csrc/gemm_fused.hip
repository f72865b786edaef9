// The weight-streaming matrix product for at most 16 rows with the neighbouring row-wise work
// folded in, so that a decode step needs one kernel where it had two or three:
//
//   input   plain : X is bfloat16 [M,K]
//           norm  : X is the float32 residual stream; the operand is bf16(x * gain) and the result is
//                   scaled by 1/sqrt(mean(x^2) + eps) per row afterwards, which is the same RMSNorm
//                   (crates/leone/src/cpu.rs:1642-1663) because that factor is constant along a row
//           prepared : X is bfloat16 [M,K] = bf16(x * gain), written by a product before (see `prepare`
//                   below) together with partial sums of x^2, one for every 16 columns of a row; the
//                   result is scaled by 1/sqrt(sum / K + eps) as for `norm`, and no kernel runs in between
//   output  store    : Y[M,N] in bfloat16 or float32
//           residual : Y is the float32 stream, Y += product (the reference's fused
//                      matrix-vector + residual, crates/leone/src/runtime.rs:9151-9157, 9311)
//           prepare  : as residual, and from the new stream values the operand of the norm that comes
//                      next: T[M,N] = bf16(y * next_gain) and, for this workgroup's 16 columns, the
//                      sum of y^2 of every row (the reference's fused norm + residual store,
//                      crates/leone/src/backend.rs:2371-2390)
//           gated    : W holds, in every block of 16 rows, 8 gate rows then the 8 up rows that belong to
//                      them; Y[M,N/2] = silu(gate) * up (crates/leone/src/cpu.rs:892-907)
//
// The weight matrix is streamed once; this is the place of the reference's row-per-block matrix-vector
// kernels (crates/leone-cuda/cuda/ie_cuda.cu:1719, launch shape :6178-6205).  A workgroup owns 16 rows of W
// and splits K between its waves in steps of 64 elements; a wave computes Y^T tiles (16 rows of W x 16 rows
// of X) with v_mfma_f32_16x16x32_bf16, W as the A operand, X as the B operand.  Lane (c, g) reads 32
// contiguous bytes of weight row c per step (elements 16g .. 16g+15 of the step), so a row's four lanes take
// a whole 128-byte line; both operands use the same assignment of elements to k-slots, which is all the
// instruction needs.  The partial tiles are added in wave order in shared memory, so a launch repeats bit
// for bit.
#include "common.h"
#include "leone_hip.h"

#include <math.h>

namespace leone {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

enum FusedIn : int { kInPlain = 0, kInNorm = 1, kInPrepared = 2 };
enum FusedOut : int { kOutStore = 0, kOutResidual = 1, kOutGated = 2, kOutPrepare = 3 };

struct FusedArgs {
    const void* x;       // plain: bfloat16 [M,K]; norm: float [*, K]
    const int* rows;     // norm: row r of the product reads stream row rows[r] (nullptr: r)
    const void* gain;    // norm: [K]
    int gain_dtype;
    float eps;
    const bf16_t* w;     // [N,K]
    void* y;
    int m, n, k;
    const float* squares_in;   // prepared: [M, ceil(K / 16)] partial sums of squares
    bf16_t* operand_out;       // prepare: [M,N]
    float* squares_out;        // prepare: [M, ceil(N / 16)]
    const void* next_gain;     // prepare: [N]
    int next_gain_dtype;
};

__device__ inline bf16x8 fz8() {
    uint4 z = {0u, 0u, 0u, 0u};
    return __builtin_bit_cast(bf16x8, z);
}
__device__ inline bf16x8 fld8(const bf16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}
__device__ inline void gain8(const void* gain, int dtype, int at, float out[8]) {
    if (dtype == kF32) {
        const float4 a = *reinterpret_cast<const float4*>(static_cast<const float*>(gain) + at);
        const float4 b = *reinterpret_cast<const float4*>(static_cast<const float*>(gain) + at + 4);
        out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
        out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
    } else {
        const uint4 t = *reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(gain) + at);
        const unsigned w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[2 * i] = __uint_as_float(w[i] << 16);
            out[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
}

template <int kIn, int kOut, bool kTail, int kWaves, typename TOut, bool kTiled>
__global__ void __launch_bounds__(kWaves * kWave)
gemm_fused_kernel(FusedArgs a) {
    __shared__ float partial[kWaves][kWave][4];
    __shared__ float squares[kWaves][16];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x % kWave;
    const int c = lane & 15, g = lane >> 4;
    const int m = a.m, n = a.n, k = a.k;
    const long n0 = static_cast<long>(blockIdx.x) * 16;
    // Rows past the end are clamped: they only feed output rows and columns that are never stored.
    const long wr = n0 + c < n ? n0 + c : n - 1;
    // Row-major weights: this lane's 32 bytes of step s lie at 64 s + 16 g of its row.  Tiled weights: the 16
    // bytes of lane L for half h of step s lie at ((s * 2 + h) * 64 + L) * 16 in the tile, so that every load of
    // a wave is 1 KB in one piece; such loads may carry the non-temporal hint.
    const bf16_t* wrow = kTiled ? a.w + static_cast<long>(blockIdx.x) * (k / 64) * 1024 + lane * 8 : a.w + wr * k + 16 * g;
    constexpr int kStepStride = kTiled ? 1024 : 64, kHalfStride = kTiled ? 512 : 8;
    auto wld = [&](int s, int h) {
        const bf16_t* p = wrow + static_cast<long>(s) * kStepStride + h * kHalfStride;
        return kTiled ? __builtin_bit_cast(bf16x8, load_streamed16(p)) : fld8(p);
    };
    float ss = 0.f;
    const int xr = c < m ? c : m - 1;
    const long xrow_index = (kIn == kInNorm && a.rows) ? a.rows[xr] : xr;
    // Prepared input: the rows' partial sums of squares ([m][k / 16] floats, k a multiple of 64) go to shared
    // memory after the walk over K, all threads side by side in 16-byte loads, and wave 0 adds each row's up
    // in index order.  (Asked for before the walk and kept in registers they cost the kernel a third of the
    // waves a compute unit holds, and with them the loads in flight that it lives on.)
    constexpr int kQuads = 8;                        // 16-byte loads a thread takes; the entry point checks that they suffice
    extern __shared__ float4 sums_of_squares[];      // [m * k / 64]
    const int quads = kIn == kInPrepared ? m * (k / 64) : 0;
    const bf16_t* xb = static_cast<const bf16_t*>(a.x) + xrow_index * k + 16 * g;   // plain
    const float* xf = static_cast<const float*>(a.x) + xrow_index * k + 16 * g;     // norm
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};

    // One step: 64 elements of K; this lane's run is elements at + 16g .. + 15, `left` of which exist.
    auto step = [&](int s, bf16x8 a0, bf16x8 a1, bool tail) {
        const int at = 64 * s;
        const int left = tail ? k - (at + 16 * g) : 16;
        bf16x8 b[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (left < 8 * (h + 1)) {
                b[h] = fz8();
            } else if (kIn != kInNorm) {
                b[h] = fld8(xb + at + 8 * h);
            } else {
                const float4 lo = *reinterpret_cast<const float4*>(xf + at + 8 * h);
                const float4 hi = *reinterpret_cast<const float4*>(xf + at + 8 * h + 4);
                const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                float gv[8];
                gain8(a.gain, a.gain_dtype, at + 16 * g + 8 * h, gv);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    ss = fmaf(v[i], v[i], ss);
                    b[h][i] = static_cast<__bf16>(v[i] * gv[i]);
                }
            }
        }
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b[0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b[1], acc, 0, 0, 0);
    };

    // Wave 0, which writes the result, asks for what the epilogue adds to (the stream's values, the next
    // norm's gains) before the walk over K: after it they would cost one more trip to memory.
    float stream_before[4] = {0.f, 0.f, 0.f, 0.f}, gain_after[4] = {0.f, 0.f, 0.f, 0.f};
    if ((kOut == kOutPrepare || kOut == kOutResidual) && wave == 0) {
        const long col = n0 + 4 * g;
        const float* out = static_cast<const float*>(a.y) + static_cast<long>(c) * n + col;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            if (c < m && col + r < n) {
                stream_before[r] = out[r];
                if (kOut == kOutPrepare) gain_after[r] = load_any(AnyVec{a.next_gain, a.next_gain_dtype}, col + r);
            }
        }
    }

    // Each wave takes a contiguous share of K, so that it reads long runs of every weight row.
    const int whole = k / 64;                        // steps of 64 elements without a tail
    const int share = (whole + kWaves - 1) / kWaves;
    const int s_end = (wave + 1) * share < whole ? (wave + 1) * share : whole;
    constexpr int kUnroll = 4;                       // weight loads of four steps are in flight together
    int s = wave * share;
    for (; s + kUnroll <= s_end; s += kUnroll) {
        bf16x8 wa[kUnroll][2];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            wa[u][0] = wld(s + u, 0);
            wa[u][1] = wld(s + u, 1);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) step(s + u, wa[u][0], wa[u][1], false);
    }
    for (; s < s_end; ++s) step(s, wld(s, 0), wld(s, 1), false);
    if (kTail && wave == kWaves - 1) {                 // the last wave also takes the step that holds the end of K
        const int left = k - (64 * whole + 16 * g);
        step(whole, left >= 8 ? wld(whole, 0) : fz8(), left >= 16 ? wld(whole, 1) : fz8(), true);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) partial[wave][lane][r] = acc[r];
    if (kIn == kInPrepared) {
        float4 held[kQuads];
#pragma unroll
        for (int i = 0; i < kQuads; ++i) {
            const int at = i * kWaves * kWave + static_cast<int>(threadIdx.x);
            held[i] = at < quads ? reinterpret_cast<const float4*>(a.squares_in)[at] : float4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int i = 0; i < kQuads; ++i) {
            const int at = i * kWaves * kWave + static_cast<int>(threadIdx.x);
            if (at < quads) sums_of_squares[at] = held[i];
        }
    }
    if (kIn == kInNorm) {
        ss += __shfl_xor(ss, 16, kWave);             // the four lanes that share X row c
        ss += __shfl_xor(ss, 32, kWave);
        if (g == 0) squares[wave][c] = ss;
    }
    __syncthreads();
    if (wave != 0) return;
    // Wave 0 adds the partial tiles in wave order.  Lane (c, g) holds the product of X row c with
    // weight rows n0 + 4g .. 4g+3.
    floatx4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int v = 0; v < kWaves; ++v)
#pragma unroll
        for (int r = 0; r < 4; ++r) sum[r] += partial[v][lane][r];
    if (kIn != kInPlain) {
        float total = 0.f;
        if (kIn == kInPrepared) {
            // lane (c, g) adds the g-th quarter of row c's partial sums, then the four quarters meet
            const int per = k / 64;                  // 16-byte runs of a quarter: k / 16 sums a row
            const float4* from = sums_of_squares + static_cast<long>(xr) * per;
            const int begin = g * (per / 4) + (g < per % 4 ? g : per % 4), end = begin + per / 4 + (g < per % 4 ? 1 : 0);
            for (int i = begin; i < end; i += 8) {       // eight reads on their way at a time
                float4 v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) v[u] = i + u < end ? from[i + u] : float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int u = 0; u < 8; ++u) total += (v[u].x + v[u].y) + (v[u].z + v[u].w);
            }
            total += __shfl_xor(total, 16, kWave);
            total += __shfl_xor(total, 32, kWave);
        } else {
#pragma unroll
            for (int v = 0; v < kWaves; ++v) total += squares[v][c];
        }
        const float inv = 1.0f / sqrtf(total / static_cast<float>(k) + a.eps);
#pragma unroll
        for (int r = 0; r < 4; ++r) sum[r] *= inv;
    }
    const int row = c;
    if (kOut == kOutGated) {
        // local rows 0..7 are gate rows, 8..15 the up rows that belong to them: lanes g = 0, 1 hold
        // gates, lanes g + 2 the matching ups
        floatx4 up;
#pragma unroll
        for (int r = 0; r < 4; ++r) up[r] = __shfl_xor(sum[r], 32, kWave);
        if (g < 2 && row < m) {
            bf16_t* out = static_cast<bf16_t*>(a.y) + static_cast<long>(row) * (n / 2) + n0 / 2 + 4 * g;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float gate = sum[r];
                out[r] = from_float<bf16_t>((gate / (1.0f + expf(-gate))) * up[r]);
            }
        }
        return;
    }
    const long col = n0 + 4 * g;
    if (kOut == kOutPrepare) {
        // every lane takes part in the exchange; rows and columns past the end count as zero
        float* out = static_cast<float*>(a.y) + static_cast<long>(row) * n + col;
        float squares = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            if (row < m && col + r < n) {
                const float v = stream_before[r] + sum[r];
                out[r] = v;
                squares = fmaf(v, v, squares);
                a.operand_out[static_cast<long>(row) * n + col + r] = from_float<bf16_t>(v * gain_after[r]);
            }
        }
        squares += __shfl_xor(squares, 16, kWave);
        squares += __shfl_xor(squares, 32, kWave);
        if (g == 0 && row < m) a.squares_out[static_cast<long>(row) * gridDim.x + blockIdx.x] = squares;
        return;
    }
    if (row >= m) return;
    if (kOut == kOutResidual) {
        float* out = static_cast<float*>(a.y) + static_cast<long>(row) * n + col;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (col + r < n) out[r] = stream_before[r] + sum[r];
    } else {
        TOut* out = static_cast<TOut*>(a.y) + static_cast<long>(row) * n + col;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (col + r < n) out[r] = from_float<TOut>(sum[r]);
    }
}

template <int kIn, int kOut, typename TOut>
static void launch_fused(const FusedArgs& a, bool tiled, hipStream_t stream) {
    const int tiles = ceil_div(a.n, 16);
    const int steps = ceil_div(a.k, 64);
    const bool tail = a.k % 64 != 0;
    const size_t shared = kIn == kInPrepared ? static_cast<size_t>(a.m) * (a.k / 16) * sizeof(float) : 0;
#define LEONE_FUSED(TAIL, WAVES)                                                                                  \
    do {                                                                                                          \
        if (tiled) gemm_fused_kernel<kIn, kOut, false, WAVES, TOut, true><<<tiles, WAVES * kWave, shared, stream>>>(a); \
        else gemm_fused_kernel<kIn, kOut, TAIL, WAVES, TOut, false><<<tiles, WAVES * kWave, shared, stream>>>(a);  \
    } while (0)
    // How many waves share a workgroup's walk over K.  Measured in whole decode steps of 1 and 8 rows at the
    // layer sizes of the 8B, 14B and 32B models, one engine, the choices in turn (a product timed alone, without
    // the norms and the residual folded in, says otherwise and misleads: 16 waves for gate/up look 1 % better
    // there and cost a step 8 %):
    //   up to one workgroup a compute unit and a long K (4,096 x 4,096 and x 12,288): 16 waves, or too few
    //     loads are in flight;
    //   up to four a unit (q/k/v everywhere, the output and down projections of the 14B and 32B sizes): 4 waves,
    //     fewer and longer streams (against 8: 14B 7.90 : 8.08 ms a step of 8 rows, 32B 15.98 : 16.33, 8B 4.93 : 4.98);
    //   more: 8 waves (4 or 16 for the head, 4 for gate/up: level; 16 for gate/up: 5.37 : 4.98).
    // With little of K to share (under 16 steps of 64) four waves are plenty.
    static int units = 0;
    if (units == 0) {
        int device = 0, count = 0;
        if (hipGetDevice(&device) != hipSuccess ||
            hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count <= 0)
            count = 256;
        units = count;
    }
    if (tiles <= units && steps >= 64) {
        if (tail) LEONE_FUSED(true, 16); else LEONE_FUSED(false, 16);
    } else if (steps < 16 || (tiles > units && tiles <= 4 * units)) {
        if (tail) LEONE_FUSED(true, 4); else LEONE_FUSED(false, 4);
    } else {
        if (tail) LEONE_FUSED(true, 8); else LEONE_FUSED(false, 8);
    }
#undef LEONE_FUSED
}

}  // namespace leone

using namespace leone;

// in_mode: 0 plain (x bfloat16 [m,k]), 1 norm (x float32 stream, optional rows, gain, eps), 2 prepared (x bfloat16
// [m,k] and squares_in float32 [m, ceil(k / 16)] as an earlier call's out_mode 3 wrote them, eps).
// out_mode: 0 store (y of out_dtype [m,n]), 1 residual (y float32 [m,n] += product), 2 gated (y bfloat16 [m,n/2]),
// 3 prepare (as 1, and operand_out bfloat16 [m,n] = bf16(y * next_gain), squares_out float32 [m, ceil(n / 16)]).
extern "C" int leone_gemm_fused_bf16(const void* x, int in_mode, const int* rows, const void* gain, int gain_dtype,
                                     float eps, const void* w, int w_tiled, void* y, int out_mode, int out_dtype, int m, int n,
                                     int k, const float* squares_in, void* operand_out, float* squares_out,
                                     const void* next_gain, int next_gain_dtype, hipStream_t stream) {
    LEONE_REQUIRE(x && w && y, "gemm_fused: null pointer");
    LEONE_REQUIRE(!w_tiled || (k % 64 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0),
                  "gemm_fused: tiled weights need K %d to be a multiple of 64", k);
    LEONE_REQUIRE(m > 0 && m <= 16, "gemm_fused: rows %d must be in 1..16", m);
    LEONE_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_fused: sizes %d x %d: K must be a positive multiple of 8", n, k);
    LEONE_REQUIRE(in_mode >= kInPlain && in_mode <= kInPrepared, "gemm_fused: unknown input mode %d", in_mode);
    LEONE_REQUIRE(in_mode != kInNorm || (gain && eps > 0.f && (gain_dtype == kF32 || gain_dtype == kBF16)),
                  "gemm_fused: the norm input needs a gain and a positive eps");
    LEONE_REQUIRE(in_mode != kInPrepared || (squares_in && eps > 0.f),
                  "gemm_fused: the prepared input needs the sums of squares and a positive eps");
    // the sums travel as 16-byte runs, eight to a thread of the smallest workgroup (256 threads)
    LEONE_REQUIRE(in_mode != kInPrepared || (k % 64 == 0 && static_cast<long>(m) * (k / 64) <= 8 * 256 &&
                                             reinterpret_cast<uintptr_t>(squares_in) % 16 == 0),
                  "gemm_fused: the prepared input takes K %d a multiple of 64 with rows x K / 64 up to 2048", k);
    LEONE_REQUIRE(out_mode >= kOutStore && out_mode <= kOutPrepare, "gemm_fused: unknown output mode %d", out_mode);
    LEONE_REQUIRE(out_mode != kOutGated || n % 16 == 0, "gemm_fused: gated output needs N %d to be a multiple of 16", n);
    LEONE_REQUIRE(out_mode != kOutStore || out_dtype == kF32 || out_dtype == kBF16, "gemm_fused: unknown output type");
    LEONE_REQUIRE(out_mode != kOutPrepare || (operand_out && squares_out && next_gain &&
                                              (next_gain_dtype == kF32 || next_gain_dtype == kBF16)),
                  "gemm_fused: the prepare output needs room for the operand and the sums, and the next gain");
    FusedArgs a{x, rows, gain, gain_dtype, eps, static_cast<const bf16_t*>(w), y, m, n, k,
                squares_in, static_cast<bf16_t*>(operand_out), squares_out, next_gain, next_gain_dtype};
#define LEONE_FUSED_OUT(IN)                                                                  \
    switch (out_mode) {                                                                      \
        case kOutStore:                                                                      \
            if (out_dtype == kF32) launch_fused<IN, kOutStore, float>(a, w_tiled != 0, stream);            \
            else launch_fused<IN, kOutStore, bf16_t>(a, w_tiled != 0, stream);                             \
            break;                                                                           \
        case kOutResidual: launch_fused<IN, kOutResidual, float>(a, w_tiled != 0, stream); break;          \
        case kOutPrepare: launch_fused<IN, kOutPrepare, float>(a, w_tiled != 0, stream); break;            \
        default: launch_fused<IN, kOutGated, bf16_t>(a, w_tiled != 0, stream); break;                      \
    }
    if (in_mode == kInPlain) {
        LEONE_FUSED_OUT(kInPlain)
    } else if (in_mode == kInNorm) {
        LEONE_FUSED_OUT(kInNorm)
    } else {
        LEONE_FUSED_OUT(kInPrepared)
    }
#undef LEONE_FUSED_OUT
    LEONE_LAUNCH_CHECK("gemm_fused");
    return 0;
}
