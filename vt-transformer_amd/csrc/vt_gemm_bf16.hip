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
template <int NT, int WPB, bool SWIGLU, typename TO>
__global__ __launch_bounds__(WPB * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ x,
                                                              const bf16_t* __restrict__ w,
                                                              const float* __restrict__ bias, TO* __restrict__ y,
                                                              int N, int Mout, int K) {
    constexpr int NW = SWIGLU ? 2 : 1;
    __shared__ float red[NW][WPB][256];
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
    const int r = lane & 15, g = lane >> 4;
    const int m0 = blockIdx.x * 16, n0 = blockIdx.y * (16 * NT);

    const int S = (K + 63) >> 6;
    const int s_begin = (int)(((long long)wv * S) / WPB), s_end = (int)(((long long)(wv + 1) * S) / WPB);

    const int mc = min(m0 + r, Mout - 1);
    const bf16_t* wrow[NW];
    wrow[0] = w + (size_t)mc * K;
    if (SWIGLU) wrow[NW - 1] = w + ((size_t)Mout + mc) * K;
    const bf16_t* xrow[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) xrow[i] = x + (size_t)min(n0 + i * 16 + r, N - 1) * K;

    f32x4_t acc[NW][NT];
#pragma unroll
    for (int a = 0; a < NW; ++a)
#pragma unroll
        for (int i = 0; i < NT; ++i) acc[a][i] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

    int s = s_begin;
    // two steps at a time: 4 loads of W per lane in flight before the first matrix instruction
    for (; s + 2 <= s_end; s += 2) {
        bf16x8_t wa[NW][4], xa[NT][4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            int k = (s + (u >> 1)) * 64 + g * 16 + (u & 1) * 8;
            bool ok = k < K;
#pragma unroll
            for (int a = 0; a < NW; ++a) wa[a][u] = load_frag(wrow[a] + k, ok);
#pragma unroll
            for (int i = 0; i < NT; ++i) xa[i][u] = load_frag(xrow[i] + k, ok);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int a = 0; a < NW; ++a)
#pragma unroll
                for (int i = 0; i < NT; ++i)
                    acc[a][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[a][u], xa[i][u], acc[a][i], 0, 0, 0);
    }
    for (; s < s_end; ++s) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            int k = s * 64 + g * 16 + u * 8;
            bool ok = k < K;
            bf16x8_t wa[NW], xa[NT];
#pragma unroll
            for (int a = 0; a < NW; ++a) wa[a] = load_frag(wrow[a] + k, ok);
#pragma unroll
            for (int i = 0; i < NT; ++i) xa[i] = load_frag(xrow[i] + k, ok);
#pragma unroll
            for (int a = 0; a < NW; ++a)
#pragma unroll
                for (int i = 0; i < NT; ++i)
                    acc[a][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[a], xa[i], acc[a][i], 0, 0, 0);
        }
    }

    // acc[.][i][j] is feature m0 + 4 g + j of token n0 + 16 i + r.  Sum the waves in order.
#pragma unroll
    for (int i = 0; i < NT; ++i) {
#pragma unroll
        for (int a = 0; a < NW; ++a)
#pragma unroll
            for (int j = 0; j < 4; ++j) red[a][wv][lane * 4 + j] = acc[a][i][j];
        __syncthreads();
        if (tid < 256) {
            int ln = tid >> 2, j = tid & 3;
            int m = m0 + 4 * (ln >> 4) + j, n = n0 + i * 16 + (ln & 15);
            float v = 0.f, u = 0.f;
            for (int q = 0; q < WPB; ++q) v += red[0][q][tid];
            if (SWIGLU)
                for (int q = 0; q < WPB; ++q) u += red[NW - 1][q][tid];
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

template <int NT, bool SWIGLU, typename TO>
static void launch_skinny(int wpb, dim3 grid, const bf16_t* x, const bf16_t* w, const float* bias, TO* y, int N,
                          int Mout, int K, hipStream_t stream) {
    if (wpb == 4) gemm_skinny_kernel<NT, 4, SWIGLU, TO><<<grid, 256, 0, stream>>>(x, w, bias, y, N, Mout, K);
    else if (wpb == 8) gemm_skinny_kernel<NT, 8, SWIGLU, TO><<<grid, 512, 0, stream>>>(x, w, bias, y, N, Mout, K);
    else gemm_skinny_kernel<NT, 16, SWIGLU, TO><<<grid, 1024, 0, stream>>>(x, w, bias, y, N, Mout, K);
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
    int tiles_m = (Mout + 15) / 16;
    int wpb = tiles_m >= 1024 ? 4 : (tiles_m >= 512 ? 8 : 16);  // from the shape of W only
    int nt = N <= 16 ? 1 : (N <= 32 ? 2 : 4);
    dim3 grid(tiles_m, (N + 16 * nt - 1) / (16 * nt));
    VT_REQUIRE(grid.y <= 65535, "vt_linear_bf16: too many rows (%d)", N);
    if (nt == 1) launch_skinny<1, SWIGLU, TO>(wpb, grid, x, w, bias, y, N, Mout, K, stream);
    else if (nt == 2) launch_skinny<2, SWIGLU, TO>(wpb, grid, x, w, bias, y, N, Mout, K, stream);
    else launch_skinny<4, SWIGLU, TO>(wpb, grid, x, w, bias, y, N, Mout, K, stream);
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
