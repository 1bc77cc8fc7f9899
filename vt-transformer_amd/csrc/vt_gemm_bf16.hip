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

// ---------------------------------------------------------------------------
// 17 to 128 rows (a large decoding batch, a short portion): a block of 4 waves takes 64*R rows of W and 64
// tokens.  The tokens' values pass through LDS once per block (coalesced loads, two buffers), so they cost a
// fraction of W's traffic instead of a multiple; each wave streams its own 16*R rows of W from memory into
// registers one stage ahead.  For matrices with few rows the k range is split over blockIdx.z and the partial
// sums (fp32, [split][N][M]) are added by vt_sum_partials in split order.
// ---------------------------------------------------------------------------
#ifndef MID_BK
#define MID_BK 128                 // k values per stage (a multiple of 64)
#endif
#define MID_XROW (MID_BK + 8)
#define MID_KU (MID_BK / 32)       // matrix instructions along k per stage
#define MID_XP (MID_BK / 32)       // 16-byte pieces of x per thread and stage (64 tokens * MID_BK / 8 / 256)

template <int R, bool SWIGLU, typename TO>
__global__ __launch_bounds__(256) void gemm_mid_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                      const float* __restrict__ bias, TO* __restrict__ y,
                                                      float* __restrict__ partial, int N, int Mout, int K,
                                                      int k_per_split) {
    constexpr int NW = SWIGLU ? 2 : 1;
    constexpr int RW = R * NW;
    __shared__ __attribute__((aligned(16))) bf16_t xs[2][64][MID_XROW];
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
    const int r = lane & 15, g = lane >> 4;
    const int m0 = blockIdx.x * (64 * R) + wv * (16 * R), n0 = blockIdx.y * 64;
    const int k_begin = blockIdx.z * k_per_split, k_end = min(K, k_begin + k_per_split);

    const bf16_t* wrow[RW];
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const int mc = min(m0 + 16 * j + r, Mout - 1);
        wrow[j] = w + (size_t)mc * K;
        if (SWIGLU) wrow[R + j] = w + ((size_t)Mout + mc) * K;
    }
    // this thread's 16-byte pieces of a stage of x: a token's MID_BK values are MID_BK/8 consecutive pieces
    const bf16_t* xsrc[MID_XP];
    int xtok[MID_XP], xcol[MID_XP];
#pragma unroll
    for (int q = 0; q < MID_XP; ++q) {
        const int pidx = tid + 256 * q;
        xtok[q] = pidx / (MID_BK / 8);
        xcol[q] = (pidx % (MID_BK / 8)) * 8;
        xsrc[q] = x + (size_t)min(n0 + xtok[q], N - 1) * K + xcol[q];
    }
    f32x4_t acc[RW][4];
#pragma unroll
    for (int a = 0; a < RW; ++a)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[a][i] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

    uint4 xreg[MID_XP];
    bf16x8_t wcur[RW][MID_KU], wnxt[RW][MID_KU];
    auto fetch_x = [&](int k0) {
#pragma unroll
        for (int q = 0; q < MID_XP; ++q) {
            Frag f;
            f.v = load_frag(xsrc[q] + k0, k0 + xcol[q] < k_end);
            xreg[q] = f.u;
        }
    };
    auto park_x = [&](int buf) {
#pragma unroll
        for (int q = 0; q < MID_XP; ++q) *(uint4*)&xs[buf][xtok[q]][xcol[q]] = xreg[q];
    };
    // fragment u of a stage: k = k0 + 64 (u/2) + 16 g + 8 (u%2), so a lane reads 32 contiguous bytes per 64 k
    auto fetch_w = [&](bf16x8_t (&dst)[RW][MID_KU], int k0) {
#pragma unroll
        for (int u = 0; u < MID_KU; ++u) {
            const int k = k0 + (u >> 1) * 64 + g * 16 + (u & 1) * 8;
#pragma unroll
            for (int a = 0; a < RW; ++a) dst[a][u] = load_frag(wrow[a] + k, k < k_end);
        }
    };
    auto multiply = [&](const bf16x8_t (&wf)[RW][MID_KU], int buf) {
#pragma unroll
        for (int u = 0; u < MID_KU; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                Frag xf;
                xf.u = *(const uint4*)&xs[buf][i * 16 + r][(u >> 1) * 64 + g * 16 + (u & 1) * 8];
#pragma unroll
                for (int a = 0; a < RW; ++a)
                    acc[a][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[a][u], xf.v, acc[a][i], 0, 0, 0);
            }
    };

    if (k_begin < k_end) {
        fetch_x(k_begin);
        fetch_w(wcur, k_begin);
        park_x(0);
        __syncthreads();
        // two stages per turn so that the register buffers alternate without copies
        for (int k0 = k_begin; k0 < k_end; k0 += 2 * MID_BK) {
            const int k1 = k0 + MID_BK, k2 = k0 + 2 * MID_BK;
            if (k1 < k_end) { fetch_x(k1); fetch_w(wnxt, k1); }
            multiply(wcur, 0);
            if (k1 < k_end) park_x(1);
            __syncthreads();
            if (k1 >= k_end) break;
            if (k2 < k_end) { fetch_x(k2); fetch_w(wcur, k2); }
            multiply(wnxt, 1);
            if (k2 < k_end) park_x(0);
            __syncthreads();
        }
    }

    // acc[a][i][e] is feature m0 + 16 j + 4 g + e (j = a mod R) of token n0 + 16 i + r
    const bool split = gridDim.z > 1;
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + i * 16 + r;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int m = m0 + 16 * j + 4 * g + e;
                if (m >= Mout || n >= N) continue;
                float v = acc[j][i][e];
                if (SWIGLU) {
                    const float u = acc[R + j][i][e];
                    v = v / (1.f + expf(-v)) * u;
                } else if (bias && blockIdx.z == 0) {
                    v += bias[m];
                }
                if (split) partial[((size_t)blockIdx.z * N + n) * Mout + m] = v;
                else store_f32<TO>(y, (size_t)n * Mout + m, v);
            }
        }
}

// y[i] = sum over splits of partial[s][i], added in split order
template <typename TO>
__global__ void sum_partials_kernel(const float* __restrict__ partial, TO* __restrict__ y, size_t n, int splits) {
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= n) return;
    if (i + 4 <= n) {
        float4 a = *(const float4*)(partial + i);
        for (int s = 1; s < splits; ++s) {
            float4 b = *(const float4*)(partial + (size_t)s * n + i);
            a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
        }
        store_f32<TO>(y, i, a.x); store_f32<TO>(y, i + 1, a.y); store_f32<TO>(y, i + 2, a.z); store_f32<TO>(y, i + 3, a.w);
    } else {
        for (size_t j = i; j < n; ++j) {
            float a = partial[j];
            for (int s = 1; s < splits; ++s) a += partial[(size_t)s * n + j];
            store_f32<TO>(y, j, a);
        }
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

// Number of k ranges for the 64-token kernel: from the shape of W only (so the order of additions does not depend
// on the batch), enough blocks to fill the GPU, every range a multiple of the stage length.
static int mid_splits(int Mout, int K, int rows_per_block) {
    const int row_blocks = (Mout + rows_per_block - 1) / rows_per_block;
    const int stages = (K + MID_BK - 1) / MID_BK;
    int splits = (512 + row_blocks - 1) / row_blocks;
    if (splits > 16) splits = 16;
    if (splits > stages / 4) splits = stages / 4 > 0 ? stages / 4 : 1;
    return splits < 1 ? 1 : splits;
}

extern "C" long long vt_linear_bf16_workspace(int N, int M, int K, int gated) {
    // floats of workspace that vt_linear_bf16 / vt_gated_linear_bf16 need for this shape (0: none)
    if (N <= 16 || K % 8 != 0 || gated) return 0;
    const int splits = mid_splits(M, K, 128);
    return splits > 1 ? (long long)splits * N * M : 0;
}

template <bool SWIGLU, typename TO>
static int linear_bf16(const bf16_t* x, const bf16_t* w, const float* bias, TO* y, float* workspace, int N, int Mout,
                       int K, hipStream_t stream) {
    if (N == 0) return 0;
    if (K % 8 != 0 || ((uintptr_t)x & 15) || ((uintptr_t)w & 15)) {
        VT_REQUIRE(N <= 65535, "vt_linear_bf16: too many rows (%d) for the any-shape kernel", N);
        gemm_plain_kernel<SWIGLU, TO><<<dim3((Mout + 255) / 256, N), 256, 0, stream>>>(x, w, bias, y, N, Mout, K);
        VT_CHECK_LAUNCH("vt_linear_bf16(plain)");
        return 0;
    }
    if (N > 16) {
        // 64 tokens per block through LDS; two row tiles per wave (one for the gated product, which has two
        // matrices' rows per wave already)
        constexpr int RR = SWIGLU ? 1 : 2;
        const int splits = SWIGLU ? 1 : mid_splits(Mout, K, 64 * RR);
        VT_REQUIRE(splits == 1 || workspace, "vt_linear_bf16: this shape needs a workspace (vt_linear_bf16_workspace)");
        int kps = ((K + splits - 1) / splits + MID_BK - 1) / MID_BK * MID_BK;
        dim3 grid((Mout + 64 * RR - 1) / (64 * RR), (N + 63) / 64, splits);
        VT_REQUIRE(grid.y <= 65535, "vt_linear_bf16: too many rows (%d)", N);
        gemm_mid_kernel<RR, SWIGLU, TO><<<grid, 256, 0, stream>>>(x, w, bias, y, workspace, N, Mout, K, kps);
        VT_CHECK_LAUNCH("vt_linear_bf16(64 tokens)");
        if (splits > 1) {
            const size_t n = (size_t)N * Mout;
            sum_partials_kernel<TO><<<(unsigned)((n / 4 + 255) / 256 + 1), 256, 0, stream>>>(workspace, y, n, splits);
            VT_CHECK_LAUNCH("vt_linear_bf16(sum)");
        }
        return 0;
    }
    // How k is split over the waves of a block depends on the shape of W only, so that a token's sums are added
    // in the same order whatever the number of rows.
    const int tiles16 = (Mout + 15) / 16;
    const int wpb = tiles16 >= 1024 ? 4 : (tiles16 >= 512 ? 8 : 16);
    dim3 grid(tiles16, 1);
    int rc = launch_skinny<1, 1, SWIGLU, TO>(wpb, grid, x, w, bias, y, N, Mout, K, stream);
    if (rc) return rc;
    VT_CHECK_LAUNCH("vt_linear_bf16");
    return 0;
}

// y[N, M] = x[N, K] . W[M, K]^T + bias
extern "C" int vt_linear_bf16(const void* x, const void* w, const float* bias, void* y, int out_dtype, float* workspace,
                              int N, int M, int K, hipStream_t stream) {
    VT_REQUIRE(N >= 0 && M > 0 && K > 0, "vt_linear_bf16: bad sizes N=%d M=%d K=%d", N, M, K);
    if (out_dtype == VT_F32) return linear_bf16<false, float>((const bf16_t*)x, (const bf16_t*)w, bias, (float*)y, workspace, N, M, K, stream);
    if (out_dtype == VT_BF16) return linear_bf16<false, bf16_t>((const bf16_t*)x, (const bf16_t*)w, bias, (bf16_t*)y, workspace, N, M, K, stream);
    return vt_fail("vt_linear_bf16: unknown out dtype %d", out_dtype);
}

// y[N, I] = silu(x . Wg^T) * (x . Wu^T),  W = [Wg; Wu] of shape [2 I, K]
extern "C" int vt_gated_linear_bf16(const void* x, const void* w, void* y, int out_dtype, int N, int I, int K,
                                    hipStream_t stream) {
    VT_REQUIRE(N >= 0 && I > 0 && K > 0, "vt_gated_linear_bf16: bad sizes N=%d I=%d K=%d", N, I, K);
    if (out_dtype == VT_F32) return linear_bf16<true, float>((const bf16_t*)x, (const bf16_t*)w, nullptr, (float*)y, nullptr, N, I, K, stream);
    if (out_dtype == VT_BF16) return linear_bf16<true, bf16_t>((const bf16_t*)x, (const bf16_t*)w, nullptr, (bf16_t*)y, nullptr, N, I, K, stream);
    return vt_fail("vt_gated_linear_bf16: unknown out dtype %d", out_dtype);
}
