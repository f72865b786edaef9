// Micro-benchmarks of what this GPU's memory and matrix cores give when nothing else is asked of them: a
// read of a large buffer, a copy, and a loop of v_mfma_f32_16x16x32_bf16 on registers.  The bench reports its
// figures against these next to the nominal peaks, as the reference's bench reports against a measured
// stream rate (crates/leone-cli/src/main.rs:79, 4655-4802).
#include "common.h"
#include "leone_hip.h"

namespace leone {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

constexpr int kPeakThreads = 256;
constexpr int kPeakUnroll = 8;

// Every thread reads runs of 16 bytes, kPeakUnroll of them in flight, a workgroup's reads side by side: every
// instruction covers whole lines, and the loads carry the non-temporal hint (a tenth faster than plain loads for
// data that is read once; measured 7.0-7.1 TB/s with one or two workgroups a compute unit, 6.1-6.4 without the
// hint, 5.1 with eight workgroups a unit).
__global__ void __launch_bounds__(kPeakThreads)
peak_read_kernel(const uint4* __restrict__ src, long runs, unsigned* __restrict__ sink) {
    const long stride = static_cast<long>(gridDim.x) * kPeakThreads;
    unsigned seen = 0u;
    long at = static_cast<long>(blockIdx.x) * kPeakThreads + threadIdx.x;
    for (; at + (kPeakUnroll - 1) * stride < runs; at += kPeakUnroll * stride) {
        uint4 v[kPeakUnroll];
#pragma unroll
        for (int u = 0; u < kPeakUnroll; ++u) v[u] = load_streamed16(src + at + u * stride);
#pragma unroll
        for (int u = 0; u < kPeakUnroll; ++u) seen ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; at < runs; at += stride) {
        const uint4 v = src[at];
        seen ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (seen == 0x9e3779b9u) sink[0] = seen;      // keeps the reads; practically never true
}

__global__ void __launch_bounds__(kPeakThreads)
peak_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, long runs) {
    const long stride = static_cast<long>(gridDim.x) * kPeakThreads;
    long at = static_cast<long>(blockIdx.x) * kPeakThreads + threadIdx.x;
    for (; at + (kPeakUnroll - 1) * stride < runs; at += kPeakUnroll * stride) {
        uint4 v[kPeakUnroll];
#pragma unroll
        for (int u = 0; u < kPeakUnroll; ++u) v[u] = load_streamed16(src + at + u * stride);
#pragma unroll
        for (int u = 0; u < kPeakUnroll; ++u) dst[at + u * stride] = v[u];
    }
    for (; at < runs; at += stride) dst[at] = src[at];
}

// Independent accumulator tiles a wave, so that no instruction waits for the one before: eight of 16 x 16 or
// four of 32 x 32 (the same registers).  Which instruction shape runs faster is the chip's affair; the bench
// takes the better.
constexpr int kPeakTiles = 8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

template <bool kWide>
__global__ void __launch_bounds__(kPeakThreads)
peak_mfma_kernel(int iterations, float* __restrict__ sink) {
    const unsigned seed = 0x3f803f80u + (threadIdx.x & 7u);            // small bfloat16 values
    const bf16x8 a = __builtin_bit_cast(bf16x8, uint4{seed, seed, seed, seed});
    const bf16x8 b = __builtin_bit_cast(bf16x8, uint4{0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u});
    float total = 0.f;
    if constexpr (kWide) {
        floatx16 acc[kPeakTiles / 2];
#pragma unroll
        for (int t = 0; t < kPeakTiles / 2; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
        for (int i = 0; i < iterations; ++i) {
#pragma unroll
            for (int t = 0; t < kPeakTiles / 2; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[t], 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < kPeakTiles / 2; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) total += acc[t][r];
    } else {
        floatx4 acc[kPeakTiles];
#pragma unroll
        for (int t = 0; t < kPeakTiles; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
        for (int i = 0; i < iterations; ++i) {
#pragma unroll
            for (int t = 0; t < kPeakTiles; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[t], 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < kPeakTiles; ++t) total += acc[t][0] + acc[t][1] + acc[t][2] + acc[t][3];
    }
    if (total == -1.0f) sink[0] = total;          // keeps the loop; never true for these operands
}

}  // namespace leone

using namespace leone;

// Reads `bytes` (a multiple of 16) from src once.  sink: one word that is practically never written.
extern "C" int leone_peak_read(const void* src, long bytes, void* sink, int blocks, hipStream_t stream) {
    LEONE_REQUIRE(src && sink && bytes > 0 && bytes % 16 == 0 && blocks > 0, "peak_read: bad arguments");
    LEONE_REQUIRE(reinterpret_cast<uintptr_t>(src) % 16 == 0, "peak_read: the buffer must be aligned to 16 bytes");
    peak_read_kernel<<<blocks, kPeakThreads, 0, stream>>>(static_cast<const uint4*>(src), bytes / 16,
                                                         static_cast<unsigned*>(sink));
    LEONE_LAUNCH_CHECK("peak_read");
    return 0;
}

extern "C" int leone_peak_copy(const void* src, void* dst, long bytes, int blocks, hipStream_t stream) {
    LEONE_REQUIRE(src && dst && bytes > 0 && bytes % 16 == 0 && blocks > 0, "peak_copy: bad arguments");
    LEONE_REQUIRE(reinterpret_cast<uintptr_t>(src) % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0,
                  "peak_copy: the buffers must be aligned to 16 bytes");
    peak_copy_kernel<<<blocks, kPeakThreads, 0, stream>>>(static_cast<const uint4*>(src), static_cast<uint4*>(dst), bytes / 16);
    LEONE_LAUNCH_CHECK("peak_copy");
    return 0;
}

// blocks workgroups of four waves run `iterations` rounds of eight 16 x 16 x 32 matrix instructions each, or
// (wide) of four 32 x 32 x 16 ones, the same work: leone_peak_mfma_flops(blocks, iterations) floating-point
// operations in all.
extern "C" double leone_peak_mfma_flops(int blocks, int iterations) {
    return static_cast<double>(blocks) * (kPeakThreads / kWave) * iterations * kPeakTiles * (2.0 * 16 * 16 * 32);
}

extern "C" int leone_peak_mfma(int blocks, int iterations, int wide, void* sink, hipStream_t stream) {
    LEONE_REQUIRE(sink && blocks > 0 && iterations > 0, "peak_mfma: bad arguments");
    if (wide) peak_mfma_kernel<true><<<blocks, kPeakThreads, 0, stream>>>(iterations, static_cast<float*>(sink));
    else peak_mfma_kernel<false><<<blocks, kPeakThreads, 0, stream>>>(iterations, static_cast<float*>(sink));
    LEONE_LAUNCH_CHECK("peak_mfma");
    return 0;
}
