// True 32-bit linear layer: y[n, m] = sum_k x[n, k] * W[m, k] + bias[m].
//
// Weight layout [out, in] row-major as the reference's op_linear
// (v1/tensortype/hip_tensor.cpp:479-539, shape check v1/tensortype/tensortype.cpp:222-229).
// No matrix-core instruction and no reduced-precision mode is used: every
// product and sum is an fp32 fused multiply-add, and each output adds its
// products in the order k = 0, 1, 2, ...  whatever the number of rows, so a
// token's result does not depend on what else is in the batch.
#include "vt_common.h"

VT_DEFINE_LAST_ERROR()

#define BM 64
#define BK 16

template <int BN>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                      const float* __restrict__ bias, float* __restrict__ y, int N,
                                                      int M, int K) {
    constexpr int TN = BN / 16;
    __shared__ float xs[BK][BN + 1];
    __shared__ float ws[BK][BM + 1];
    int tid = threadIdx.x;
    int tx = tid & 15, ty = tid >> 4;
    int m0 = blockIdx.x * BM, n0 = blockIdx.y * BN;
    float acc[TN][4];
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int e = 0; e < (BN * BK) / 256; ++e) {
            int idx = tid + e * 256;
            int r = idx >> 4, kk = idx & 15;
            int n = n0 + r, k = k0 + kk;
            xs[kk][r] = (n < N && k < K) ? x[(size_t)n * K + k] : 0.f;
        }
#pragma unroll
        for (int e = 0; e < (BM * BK) / 256; ++e) {
            int idx = tid + e * 256;
            int r = idx >> 4, kk = idx & 15;
            int m = m0 + r, k = k0 + kk;
            ws[kk][r] = (m < M && k < K) ? w[(size_t)m * K + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float xv[TN], wv[4];
#pragma unroll
            for (int i = 0; i < TN; ++i) xv[i] = xs[kk][ty * TN + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < TN; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(xv[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TN; ++i) {
        int n = n0 + ty * TN + i;
        if (n >= N) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int m = m0 + tx * 4 + j;
            if (m < M) y[(size_t)n * M + m] = acc[i][j] + (bias ? bias[m] : 0.f);
        }
    }
}

extern "C" int vt_linear_f32(const float* x, const float* w, const float* bias, float* y, int N, int M, int K,
                             hipStream_t stream) {
    VT_REQUIRE(N >= 0 && M > 0 && K > 0, "vt_linear_f32: bad sizes N=%d M=%d K=%d", N, M, K);
    if (N == 0) return 0;
    if (N <= 16) {
        dim3 grid((M + BM - 1) / BM, (N + 15) / 16);
        gemm_f32_kernel<16><<<grid, 256, 0, stream>>>(x, w, bias, y, N, M, K);
    } else {
        dim3 grid((M + BM - 1) / BM, (N + 63) / 64);
        VT_REQUIRE(grid.y <= 65535, "vt_linear_f32: too many rows (%d)", N);
        gemm_f32_kernel<64><<<grid, 256, 0, stream>>>(x, w, bias, y, N, M, K);
    }
    VT_CHECK_LAUNCH("vt_linear_f32");
    return 0;
}
