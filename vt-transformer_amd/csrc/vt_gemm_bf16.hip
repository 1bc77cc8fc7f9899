// bfloat16 linear layers on the gfx950 matrix cores, for few rows (decoding
// and short portions): y[n, m] = sum_k x[n, k] * W[m, k] (+ bias[m]), fp32
// accumulation, fp32 or bf16 output; and the same with the SiLU gate fused:
// y[n, i] = silu(x.W[i]) * (x.W[I + i]).
//
// The reference calls hipblasGemmEx for each projection, rounds the result
// to 16 bits and then adds the bias in a second kernel
// (v1/tensortype/hip_tensor.cpp:514-535, v1/tensortype/hip_kernels/add_bias.cpp:8-17),
// and runs up, gate and the gating as three launches
// (v1/models/qwen2-7b/inference_fp16.dag:333-336).  Here the bias and the gate
// are applied to the fp32 accumulator.
//
// With few rows the time goes to reading W once from HBM, so the work is
// laid out for that: a wave owns 16 rows of W and a slice of k, reads its
// slice with 32 contiguous bytes per lane and feeds it to
// v_mfma_f32_16x16x32_bf16 as the A operand; the tokens are the B operand.
// The waves of a block split k and add their partial sums through LDS in wave
// order.  How k is split depends on the shape of W only, never on the number
// of rows, so a token's result does not change with the batch around it.
#include "vt_common.h"

VT_DEFINE_LAST_ERROR()

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

union Frag {
    uint4 u;
    bf16x8_t v;
};

__device__ __forceinline__ bf16x8_t load_frag(const bf16_t* p, bool ok) {
    Frag f;
    if (ok) f.u = *(const uint4*)p;
    else f.u = make_uint4(0, 0, 0, 0);
    return f.v;
}

// One "step" is 64 values of k: lane group g = lane/16 reads k in [64 s + 16 g, 64 s + 16 g + 16),
// the first 8 for one matrix instruction and the next 8 for a second one.
//
// A wave owns R tiles of 16 rows of W (rows m0 + 16 j + r) and NT tiles of 16 tokens: every fragment of x it
// reads serves R row tiles, so the traffic for x (from L2) stays at NT/R of the traffic for W (from HBM).
template <int NT, int R, int WPB, bool SWIGLU, typename TO>
__global__ __launch_bounds__(WPB * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ x,
                                                              const bf16_t* __restrict__ w,
                                                              const float* __restrict__ bias, TO* __restrict__ y,
                                                              int N, int Mout, int K) {
    constexpr int NW = SWIGLU ? 2 : 1;
    constexpr int RW = R * NW;                      // W fragments per k position
    constexpr int U = (RW >= 4) ? 2 : 4;            // fragments of 8 k values in flight per row (1 or 2 steps)
    __shared__ float red[RW][WPB][256];
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
    const int r = lane & 15, g = lane >> 4;
    const int m0 = blockIdx.x * (16 * R), n0 = blockIdx.y * (16 * NT);

    const int S = (K + 63) >> 6;
    const int s_begin = (int)(((long long)wv * S) / WPB), s_end = (int)(((long long)(wv + 1) * S) / WPB);

    const bf16_t* wrow[RW];
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const int mc = min(m0 + 16 * j + r, Mout - 1);
        wrow[j] = w + (size_t)mc * K;
        if (SWIGLU) wrow[R + j] = w + ((size_t)Mout + mc) * K;
    }
    const bf16_t* xrow[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) xrow[i] = x + (size_t)min(n0 + i * 16 + r, N - 1) * K;

    f32x4_t acc[RW][NT];
#pragma unroll
    for (int a = 0; a < RW; ++a)
#pragma unroll
        for (int i = 0; i < NT; ++i) acc[a][i] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

    // k position of fragment u of the group starting at step s: 64 s + 16 g + 8 u for u = 0, 1 and the same one
    // step later for u = 2, 3
    int s = s_begin;
    constexpr int SPI = U / 2;                      // steps per iteration
    for (; s + SPI <= s_end; s += SPI) {
        bf16x8_t wa[RW][U], xa[NT][U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = (s + (u >> 1)) * 64 + g * 16 + (u & 1) * 8;
            const bool ok = k < K;
#pragma unroll
            for (int a = 0; a < RW; ++a) wa[a][u] = load_frag(wrow[a] + k, ok);
#pragma unroll
            for (int i = 0; i < NT; ++i) xa[i][u] = load_frag(xrow[i] + k, ok);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int a = 0; a < RW; ++a)
#pragma unroll
                for (int i = 0; i < NT; ++i)
                    acc[a][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[a][u], xa[i][u], acc[a][i], 0, 0, 0);
    }
    for (; s < s_end; ++s) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int k = s * 64 + g * 16 + u * 8;
            const bool ok = k < K;
            bf16x8_t wa[RW], xa[NT];
#pragma unroll
            for (int a = 0; a < RW; ++a) wa[a] = load_frag(wrow[a] + k, ok);
#pragma unroll
            for (int i = 0; i < NT; ++i) xa[i] = load_frag(xrow[i] + k, ok);
#pragma unroll
            for (int a = 0; a < RW; ++a)
#pragma unroll
                for (int i = 0; i < NT; ++i)
                    acc[a][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[a], xa[i], acc[a][i], 0, 0, 0);
        }
    }

    // acc[j][i][e] is feature m0 + 16 j + 4 g + e of token n0 + 16 i + r.  Sum the waves in wave order.
#pragma unroll
    for (int i = 0; i < NT; ++i) {
#pragma unroll
        for (int a = 0; a < RW; ++a)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[a][wv][lane * 4 + e] = acc[a][i][e];
        __syncthreads();
        for (int idx = tid; idx < R * 256; idx += WPB * 64) {
            const int j = idx >> 8, c = idx & 255;
            const int ln = c >> 2, e = c & 3;
            const int m = m0 + 16 * j + 4 * (ln >> 4) + e, n = n0 + i * 16 + (ln & 15);
            float v = 0.f, u = 0.f;
            for (int q = 0; q < WPB; ++q) v += red[j][q][c];
            if (SWIGLU)
                for (int q = 0; q < WPB; ++q) u += red[(NW - 1) * R + j][q][c];
            if (m < Mout && n < N) {
                if (SWIGLU) v = v / (1.f + expf(-v)) * u;
                else if (bias) v += bias[m];
                store_f32<TO>(y, (size_t)n * Mout + m, v);
            }
        }
        __syncthreads();
    }
}

// Any shape (k not a multiple of 8): one thread per output, plain loop.
template <bool SWIGLU, typename TO>
__global__ void gemm_plain_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                  const float* __restrict__ bias, TO* __restrict__ y, int N, int Mout, int K) {
    int m = blockIdx.x * blockDim.x + threadIdx.x, n = blockIdx.y;
    if (m >= Mout) return;
    const bf16_t* xr = x + (size_t)n * K;
    const bf16_t* wr = w + (size_t)m * K;
    float v = 0.f, u = 0.f;
    for (int k = 0; k < K; ++k) v = fmaf(bf16_to_f32(xr[k]), bf16_to_f32(wr[k]), v);
    if (SWIGLU) {
        const bf16_t* wu = w + ((size_t)Mout + m) * K;
        for (int k = 0; k < K; ++k) u = fmaf(bf16_to_f32(xr[k]), bf16_to_f32(wu[k]), u);
        v = v / (1.f + expf(-v)) * u;
    } else if (bias) {
        v += bias[m];
    }
    store_f32<TO>(y, (size_t)n * Mout + m, v);
}

// the partial sums of a block pass through R * (SWIGLU ? 2 : 1) * WPB KB of LDS: at most 32 KB
template <int NT, int R, int WPB, bool SWIGLU, typename TO>
static int launch_one(dim3 grid, const bf16_t* x, const bf16_t* w, const float* bias, TO* y, int N, int Mout, int K,
                      hipStream_t stream) {
    if constexpr (R * (SWIGLU ? 2 : 1) * WPB <= 32) {
        gemm_skinny_kernel<NT, R, WPB, SWIGLU, TO><<<grid, WPB * 64, 0, stream>>>(x, w, bias, y, N, Mout, K);
        return 0;
    } else {
        return vt_fail("vt_linear_bf16: no kernel for %d row tiles with %d waves", R, WPB);
    }
}

template <int NT, int R, bool SWIGLU, typename TO>
static int launch_skinny(int wpb, dim3 grid, const bf16_t* x, const bf16_t* w, const float* bias, TO* y, int N,
                         int Mout, int K, hipStream_t stream) {
    if (wpb == 4) return launch_one<NT, R, 4, SWIGLU, TO>(grid, x, w, bias, y, N, Mout, K, stream);
    if (wpb == 8) return launch_one<NT, R, 8, SWIGLU, TO>(grid, x, w, bias, y, N, Mout, K, stream);
    return launch_one<NT, R, 16, SWIGLU, TO>(grid, x, w, bias, y, N, Mout, K, stream);
}

template <bool SWIGLU, typename TO>
static int linear_bf16(const bf16_t* x, const bf16_t* w, const float* bias, TO* y, int N, int Mout, int K,
                       hipStream_t stream) {
    if (N == 0) return 0;
    if (K % 8 != 0 || ((uintptr_t)x & 15) || ((uintptr_t)w & 15)) {
        VT_REQUIRE(N <= 65535, "vt_linear_bf16: too many rows (%d) for the any-shape kernel", N);
        gemm_plain_kernel<SWIGLU, TO><<<dim3((Mout + 255) / 256, N), 256, 0, stream>>>(x, w, bias, y, N, Mout, K);
        VT_CHECK_LAUNCH("vt_linear_bf16(plain)");
        return 0;
    }
    // How k is split over the waves of a block depends on the shape of W only, so that a token's sums are added
    // in the same order whatever the number of rows; the number of row tiles per wave does not change that order.
    const int tiles16 = (Mout + 15) / 16;
    const int wpb = tiles16 >= 1024 ? 4 : (tiles16 >= 512 ? 8 : 16);
    const int nt = N <= 16 ? 1 : (N <= 32 ? 2 : 4);
    // row tiles per wave: as many as token tiles (x is then read no more often than W), two even for one token
    // tile when W has rows to spare; bounded by the LDS that the sum over the waves needs
    const int want = nt == 1 ? (tiles16 >= 2048 ? 2 : 1) : nt;
    const int cap = 32 / (wpb * (SWIGLU ? 2 : 1));
    const int rr = want <= cap ? want : (cap >= 2 ? 2 : 1);
    dim3 grid((Mout + 16 * rr - 1) / (16 * rr), (N + 16 * nt - 1) / (16 * nt));
    VT_REQUIRE(grid.y <= 65535, "vt_linear_bf16: too many rows (%d)", N);
    int rc;
#define VT_GO(NT_, R_) rc = launch_skinny<NT_, R_, SWIGLU, TO>(wpb, grid, x, w, bias, y, N, Mout, K, stream)
    if (nt == 1 && rr == 1) VT_GO(1, 1);
    else if (nt == 1) VT_GO(1, 2);
    else if (nt == 2 && rr == 1) VT_GO(2, 1);
    else if (nt == 2) VT_GO(2, 2);
    else if (rr == 1) VT_GO(4, 1);
    else if (rr == 2) VT_GO(4, 2);
    else VT_GO(4, 4);
#undef VT_GO
    if (rc) return rc;
    VT_CHECK_LAUNCH("vt_linear_bf16");
    return 0;
}

// y[N, M] = x[N, K] . W[M, K]^T + bias
extern "C" int vt_linear_bf16(const void* x, const void* w, const float* bias, void* y, int out_dtype, int N, int M,
                              int K, hipStream_t stream) {
    VT_REQUIRE(N >= 0 && M > 0 && K > 0, "vt_linear_bf16: bad sizes N=%d M=%d K=%d", N, M, K);
    if (out_dtype == VT_F32) return linear_bf16<false, float>((const bf16_t*)x, (const bf16_t*)w, bias, (float*)y, N, M, K, stream);
    if (out_dtype == VT_BF16) return linear_bf16<false, bf16_t>((const bf16_t*)x, (const bf16_t*)w, bias, (bf16_t*)y, N, M, K, stream);
    return vt_fail("vt_linear_bf16: unknown out dtype %d", out_dtype);
}

// y[N, I] = silu(x . Wg^T) * (x . Wu^T),  W = [Wg; Wu] of shape [2 I, K]
extern "C" int vt_gated_linear_bf16(const void* x, const void* w, void* y, int out_dtype, int N, int I, int K,
                                    hipStream_t stream) {
    VT_REQUIRE(N >= 0 && I > 0 && K > 0, "vt_gated_linear_bf16: bad sizes N=%d I=%d K=%d", N, I, K);
    if (out_dtype == VT_F32) return linear_bf16<true, float>((const bf16_t*)x, (const bf16_t*)w, nullptr, (float*)y, N, I, K, stream);
    if (out_dtype == VT_BF16) return linear_bf16<true, bf16_t>((const bf16_t*)x, (const bf16_t*)w, nullptr, (bf16_t*)y, N, I, K, stream);
    return vt_fail("vt_gated_linear_bf16: unknown out dtype %d", out_dtype);
}
