// Shared helpers for the gfx950 kernels: storage types, conversions, wave
// reductions and the error channel of the C entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

namespace leone {

// Element types as passed over the C boundary.
enum DType : int { kF32 = 0, kBF16 = 1 };

constexpr int kWave = 64;

// bfloat16 is carried as its 16 bits; all arithmetic is done in float.
struct bf16_t {
    uint16_t bits;
};

__host__ __device__ inline float to_float(float v) { return v; }
__host__ __device__ inline float to_float(bf16_t v) {
    union {
        uint32_t u;
        float f;
    } c;
    c.u = static_cast<uint32_t>(v.bits) << 16;
    return c.f;
}

// Round to nearest even; NaN stays NaN.
__host__ __device__ inline uint16_t bf16_bits_from_float(float f) {
    union {
        uint32_t u;
        float f;
    } c;
    c.f = f;
    uint32_t u = c.u;
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

template <typename T>
__host__ __device__ inline T from_float(float f);
template <>
__host__ __device__ inline float from_float<float>(float f) {
    return f;
}
template <>
__host__ __device__ inline bf16_t from_float<bf16_t>(float f) {
    bf16_t r;
    r.bits = bf16_bits_from_float(f);
    return r;
}

// A gain or table vector that may be stored in either type.
struct AnyVec {
    const void* ptr;
    int dtype;
};
__device__ inline float load_any(const AnyVec& v, long i) {
    return v.dtype == kF32 ? static_cast<const float*>(v.ptr)[i]
                           : to_float(static_cast<const bf16_t*>(v.ptr)[i]);
}

// Sixteen bytes that are read once and not again (weights, a request's keys and values): the load carries the
// non-temporal hint, so that the line does not push reusable ones out of the caches.  A stream of such reads
// measures about a tenth faster than plain loads.
typedef unsigned streamed16_t __attribute__((ext_vector_type(4)));
__device__ inline uint4 load_streamed16(const void* p) {
    const streamed16_t v = __builtin_nontemporal_load(static_cast<const streamed16_t*>(p));
    return uint4{v.x, v.y, v.z, v.w};
}

// Eight elements of such a vector from an offset that is a multiple of 8 (the vector aligned to 32 bytes).
__device__ inline void load_any8(const AnyVec& v, long at, float out[8]) {
    if (v.dtype == kF32) {
        const float4 a = *reinterpret_cast<const float4*>(static_cast<const float*>(v.ptr) + at);
        const float4 b = *reinterpret_cast<const float4*>(static_cast<const float*>(v.ptr) + at + 4);
        out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
        out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
    } else {
        const uint4 t = *reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(v.ptr) + at);
        const unsigned w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            union { uint32_t u; float f; } lo, hi;
            lo.u = w[i] << 16;
            hi.u = w[i] & 0xffff0000u;
            out[2 * i] = lo.f;
            out[2 * i + 1] = hi.f;
        }
    }
}

__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// Sum over a block of kThreads (a multiple of 64, at most 1024); every thread
// gets the result.  `scratch` holds at least kThreads/64 floats.  The order of
// the additions is fixed, so a launch repeats bit for bit.
template <int kThreads>
__device__ inline float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int wave = threadIdx.x / kWave;
    const int lane = threadIdx.x % kWave;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < kThreads / kWave; ++w) total += scratch[w];
    return total;
}

// ---- cache layout ----------------------------------------------------------
// One page of one kv head holds page_tokens * head_dim elements.  Both tensors
// are packed in runs of 8 elements (16 bytes of bfloat16) so that the matrix
// core kernels read whole runs with neighbouring lanes on neighbouring runs:
//   keys   [head_dim / 8][token][8 elements]   (run = 8 elements of one token)
//   values [token / 8][head_dim][8 tokens]     (run = one element of 8 tokens)
// head_dim and page_tokens are multiples of 8.
__host__ __device__ inline long key_offset(int token, int element, int page_tokens) {
    return (static_cast<long>(element >> 3) * page_tokens + token) * 8 + (element & 7);
}
__host__ __device__ inline long value_offset(int token, int element, int head_dim) {
    return (static_cast<long>(token >> 3) * head_dim + element) * 8 + (token & 7);
}

// ---- error channel -------------------------------------------------------
// Every entry point returns 0 on success.  On failure it returns nonzero and
// leaves a message that leone_last_error() hands out.
void set_error(const char* fmt, ...);

#define LEONE_REQUIRE(cond, ...)          \
    do {                                  \
        if (!(cond)) {                    \
            leone::set_error(__VA_ARGS__); \
            return 1;                     \
        }                                 \
    } while (0)

#define LEONE_LAUNCH_CHECK(name)                                                      \
    do {                                                                              \
        hipError_t e_ = hipGetLastError();                                            \
        if (e_ != hipSuccess) {                                                       \
            leone::set_error("%s: launch failed: %s", name, hipGetErrorString(e_));   \
            return 2;                                                                 \
        }                                                                             \
    } while (0)

inline int ceil_div(long a, long b) { return static_cast<int>((a + b - 1) / b); }

}  // namespace leone
