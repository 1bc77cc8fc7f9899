// Next-token choice from fp32 logits: the largest logit of every row first, by SLICES blocks per row that
// each scan a slice; then one block per row.
//
// Greedy: the largest logit, the lowest index among equals.  The reference's
// easy_top1 (v1/tensortype/hip_kernels/sampling.cpp:138-165) leaves the order
// among equals to its shuffle reduction (v1/tensortype/block_reduce.hpp:127-169).
//
// Stochastic: p = softmax(logits / temperature) in fp32, optionally cut to
// the top_k most probable and then to the smallest set whose mass reaches
// top_p (names and meanings of sglfront/sglfront/core.py:6-16), then the
// inverse CDF in index order at u * (kept mass).  The reference's own
// stochastic kernel, easy_top3 (sampling.cpp:28-100), is the case top_k = 3;
// like it (v1/tensortype/hip_tensor.cpp:1033-1034) the uniform number comes
// from the host.  Entries that tie with the k-th probability are all kept.
#include "vt_common.h"
#include <math.h>

VT_DEFINE_LAST_ERROR()

#define ST 1024

__device__ __forceinline__ float block_sum_all(float v, float* red) { return block_sum(v, red); }

__device__ __forceinline__ int block_sum_int(int v, int* red) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    int t = 0;
    for (int i = 0; i < nw; ++i) t += red[i];
    return t;
}

#define SLICES 32

__device__ __forceinline__ void take_larger(float& bv, int& bi, float v, int i) {
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
}

// largest logit (lowest index among equals) of slice blockIdx.x of row blockIdx.y -> pval/pidx[row][slice]
__global__ __launch_bounds__(256) void argmax_slices_kernel(const float* __restrict__ logits, int V, float* __restrict__ pval,
                                                           int* __restrict__ pidx) {
    __shared__ float sval[4];
    __shared__ int sidx[4];
    const int row = blockIdx.y, tid = threadIdx.x;
    const float* lg = logits + (size_t)row * V;
    // slices of whole groups of four, so that an aligned row is read 16 bytes at a time
    const int per = ((V + SLICES - 1) / SLICES + 3) & ~3;
    const int b = blockIdx.x * per, e = min(V, b + per);
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    if ((((size_t)lg) & 15) == 0) {
        const int e4 = b + ((e - b) & ~3);
        for (int i = b + tid * 4; i < e4; i += 1024) {
            const float4 v = *(const float4*)(lg + i);
            take_larger(bv, bi, v.x, i); take_larger(bv, bi, v.y, i + 1);
            take_larger(bv, bi, v.z, i + 2); take_larger(bv, bi, v.w, i + 3);
        }
        for (int i = e4 + tid; i < e; i += 256) take_larger(bv, bi, lg[i], i);
    } else {
        for (int i = b + tid; i < e; i += 256) take_larger(bv, bi, lg[i], i);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) take_larger(bv, bi, __shfl_xor(bv, o, 64), __shfl_xor(bi, o, 64));
    if ((tid & 63) == 0) { sval[tid >> 6] = bv; sidx[tid >> 6] = bi; }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 4; ++w) take_larger(bv, bi, sval[w], sidx[w]);
        pval[row * SLICES + blockIdx.x] = bv;
        pidx[row * SLICES + blockIdx.x] = bi;
    }
}

__global__ __launch_bounds__(ST) void sample_kernel(const float* __restrict__ logits, int V,
                                                   const float* __restrict__ temperature, const int* __restrict__ top_k,
                                                   const float* __restrict__ top_p, const float* __restrict__ uniform,
                                                   const float* __restrict__ pval, const int* __restrict__ pidx,
                                                   float* __restrict__ work, int* __restrict__ out) {
    __shared__ float red[16];
    __shared__ int redi[16];
    __shared__ float seg[ST];
    const int row = blockIdx.x, tid = threadIdx.x;
    const float* lg = logits + (size_t)row * V;
    const float T = temperature[row];
    const int k = top_k[row];

    // ---- largest logit, lowest index among equals: the best of the slices ----
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int w = 0; w < SLICES; ++w) take_larger(bv, bi, pval[row * SLICES + w], pidx[row * SLICES + w]);
    if (!(T > 0.f) || k == 1) {
        if (tid == 0) out[row] = bi;
        return;
    }

    // ---- unnormalised probabilities ----
    float* p = work + (size_t)row * V;
    const float invT = 1.f / T;
    float sum = 0.f;
    for (int i = tid; i < V; i += ST) {
        float e = expf((lg[i] - bv) * invT);
        p[i] = e;
        sum += e;
    }
    float total = block_sum_all(sum, red);
    float thr = 0.f;  // keep p >= thr

    // ---- top_k: the largest threshold that still keeps at least k entries (search over the bits of a float) ----
    if (k > 0 && k < V) {
        unsigned lo = 0u, hi = 0x3f800000u;  // p in (0, 1]; count(p >= 1.0) >= 1 always
        // invariant: count(p >= lo) >= k
        while (lo < hi) {
            unsigned mid = lo + (hi - lo + 1) / 2;
            float t = __uint_as_float(mid);
            int c = 0;
            for (int i = tid; i < V; i += ST) c += p[i] >= t;
            c = block_sum_int(c, redi);
            if (c >= k) lo = mid; else hi = mid - 1;
        }
        thr = __uint_as_float(lo);
        float s2 = 0.f;
        for (int i = tid; i < V; i += ST) s2 += p[i] >= thr ? p[i] : 0.f;
        total = block_sum_all(s2, red);
    }
    // ---- top_p: the largest threshold whose kept mass still reaches top_p of the total ----
    const float tp = top_p[row];
    if (tp < 1.f) {
        const float need = tp * total;
        unsigned lo = __float_as_uint(thr), hi = 0x3f800000u;
        // invariant: mass(p >= lo) >= need
        while (lo < hi) {
            unsigned mid = lo + (hi - lo + 1) / 2;
            float t = __uint_as_float(mid);
            float s2 = 0.f;
            for (int i = tid; i < V; i += ST) s2 += p[i] >= t ? p[i] : 0.f;
            s2 = block_sum_all(s2, red);
            if (s2 >= need) lo = mid; else hi = mid - 1;
        }
        thr = __uint_as_float(lo);
        float s2 = 0.f;
        for (int i = tid; i < V; i += ST) s2 += p[i] >= thr ? p[i] : 0.f;
        total = block_sum_all(s2, red);
    }

    // ---- inverse CDF in index order ----
    const int per = (V + ST - 1) / ST;
    const int b = tid * per, e = min(V, b + per);
    float s3 = 0.f;
    for (int i = b; i < e; ++i) s3 += p[i] >= thr ? p[i] : 0.f;
    seg[tid] = s3;
    __syncthreads();
    if (tid == 0) {
        float target = uniform[row] * total;
        float cum = 0.f;
        int pick = -1, last_kept_seg = -1;
        for (int t = 0; t < ST && pick < 0; ++t) {
            if (seg[t] > 0.f) last_kept_seg = t;
            if (cum + seg[t] > target && seg[t] > 0.f) pick = t; else cum += seg[t];
        }
        if (pick < 0) { pick = last_kept_seg; cum = -INFINITY; }  // rounding left the target past the end: last kept entry
        int choice = bi;
        if (pick >= 0) {
            int pb = pick * per, pe = min(V, pb + per);
            int last = -1;
            bool found = false;
            for (int i = pb; i < pe; ++i) {
                if (p[i] >= thr) {
                    last = i;
                    cum += p[i];
                    if (cum > target) { choice = i; found = true; break; }
                }
            }
            if (!found && last >= 0) choice = last;
        }
        out[row] = choice;
    }
}

// partials: 2 * vt_sample_slices() floats per row, scratch
extern "C" int vt_sample_slices() { return SLICES; }

extern "C" int vt_sample(const float* logits, int rows, int V, const float* temperature, const int* top_k,
                         const float* top_p, const float* uniform, float* work, float* partials, int* out,
                         hipStream_t stream) {
    VT_REQUIRE(rows >= 0 && V > 0, "vt_sample: bad sizes rows=%d vocab=%d", rows, V);
    VT_REQUIRE(rows <= 65535, "vt_sample: %d rows (at most 65535)", rows);
    VT_REQUIRE(partials != nullptr, "vt_sample: no scratch for the slices' maxima");
    if (rows == 0) return 0;
    float* pval = partials;
    int* pidx = (int*)(partials + (size_t)rows * SLICES);
    argmax_slices_kernel<<<dim3(SLICES, rows), 256, 0, stream>>>(logits, V, pval, pidx);
    VT_CHECK_LAUNCH("vt_sample(slices)");
    sample_kernel<<<rows, ST, 0, stream>>>(logits, V, temperature, top_k, top_p, uniform, pval, pidx, work, out);
    VT_CHECK_LAUNCH("vt_sample");
    return 0;
}
