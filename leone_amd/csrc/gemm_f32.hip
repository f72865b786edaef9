// Single-precision matrix product for the true 32-bit path:
// C[M,N] = A[M,K] . B[N,K]^T, every product and sum in float (fused multiply-add,
// k ascending), no reduced-precision matrix mode.  The reference's scalar
// backend folds each output left to right in float the same way
// (crates/leone/src/cpu.rs:1379-1405, 1622-1640).
#include "common.h"
#include "leone_hip.h"

namespace leone {

constexpr int kTile = 64;   // output tile edge
constexpr int kDepth = 16;  // k elements per stage

__global__ void __launch_bounds__(256)
gemm_f32_kernel(const float* __restrict__ a, const float* __restrict__ b, float* __restrict__ c,
                int m, int n, int k) {
    __shared__ float as[kDepth][kTile + 4];
    __shared__ float bs[kDepth][kTile + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const long m0 = static_cast<long>(blockIdx.y) * kTile;
    const long n0 = static_cast<long>(blockIdx.x) * kTile;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < k; k0 += kDepth) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = tid + i * 256;
            const int r = idx / kDepth, kk = idx % kDepth;
            const long gm = m0 + r, gn = n0 + r;
            const int gk = k0 + kk;
            as[kk][r] = (gm < m && gk < k) ? a[gm * k + gk] : 0.f;
            bs[kk][r] = (gn < n && gk < k) ? b[gn * k + gk] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < kDepth; ++kk) {
            float av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                av[i] = as[kk][ty * 4 + i];
                bv[i] = bs[kk][tx * 4 + i];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const long gm = m0 + ty * 4 + i;
        if (gm >= m) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const long gn = n0 + tx * 4 + j;
            if (gn < n) c[gm * n + gn] = acc[i][j];
        }
    }
}

}  // namespace leone

using namespace leone;

extern "C" int leone_gemm_f32(const float* a, const float* b, float* c, int m, int n, int k, hipStream_t stream) {
    LEONE_REQUIRE(a && b && c, "gemm_f32: null pointer");
    LEONE_REQUIRE(m > 0 && n > 0 && k > 0, "gemm_f32: sizes %d x %d x %d must be positive", m, n, k);
    const int grid_y = ceil_div(m, kTile);
    LEONE_REQUIRE(grid_y <= 65535, "gemm_f32: %d rows exceed the launch limit", m);
    dim3 grid(ceil_div(n, kTile), grid_y);
    gemm_f32_kernel<<<grid, 256, 0, stream>>>(a, b, c, m, n, k);
    LEONE_LAUNCH_CHECK("gemm_f32");
    return 0;
}
