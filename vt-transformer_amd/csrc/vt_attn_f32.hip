// True 32-bit attention over paged keys and values, for prompts and for
// decoding alike: one block per (token, query head).
//
// What it computes is the reference's chain querykey -> add mask -> softmax
// -> attn (v1/models/qwen2-7b/inference_fp16.dag:307-318): scores
// (1/sqrt(D)) q.k (scale: v1/tensortype/hip_tensor.cpp:691), keys after the
// token's own position masked (v1/tensortype/hip_kernels/causal_mask.cpp:57-83),
// softmax in fp32 with the row maximum subtracted
// (v1/tensortype/hip_kernels/softmax.cpp:10-43), weighted sum of the values;
// query head h uses key/value head h / (heads / kv_heads)
// (v1/tensortype/hip_kernels/transpose_0213.cpp:89-103).  Masked keys are
// skipped rather than added as a large negative number, and the score matrix is
// never stored: keys are visited in chunks of 256 at absolute key indices,
// with a running maximum and sum, so a token's result depends only on its
// position and the keys, not on how its request was cut into steps.
//
// `window` > 0 keeps only the last `window` keys (the token's own included).
#include "vt_common.h"
#include <math.h>

VT_DEFINE_LAST_ERROR()

struct AttnF32Args {
    const float* q;
    const float* k_pages;
    const float* v_pages;
    const int* positions;
    const int* tok_entry;
    const int* block_table;
    float* out;
    int n_heads, n_kv, D, page_size, max_blocks, num_pages, window;
    float scale;
};

#define CHUNK 256

__global__ __launch_bounds__(CHUNK) void attn_f32_kernel(AttnF32Args a) {
    extern __shared__ float smem[];
    float* qs = smem;             // D
    float* sp = qs + a.D;         // CHUNK
    float* spart = sp + CHUNK;    // CHUNK
    __shared__ float red[16];

    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int D = a.D, ps = a.page_size;
    const int kvh = h / (a.n_heads / a.n_kv);
    const int pos = a.positions[t];
    const int* bt = a.block_table + (size_t)a.tok_entry[t] * a.max_blocks;
    const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;

    for (int d = tid; d < D; d += CHUNK) qs[d] = a.q[((size_t)t * a.n_heads + h) * D + d];
    __syncthreads();

    const int G = CHUNK / D;  // key groups for the weighted sum (D <= 256)
    const int d_own = tid % D, g_own = tid / D;
    const bool pv_active = g_own < G;

    float m = -INFINITY, l = 0.f, acc = 0.f;
    for (int c0 = (lo / CHUNK) * CHUNK; c0 <= pos; c0 += CHUNK) {
        int j = c0 + tid;
        bool valid = j >= lo && j <= pos;
        float s = -INFINITY;
        if (valid) {
            int blk = j / ps;
            int pg = bt[blk];
            if (pg >= 0 && pg < a.num_pages) {
                const float* kr = a.k_pages + (((size_t)pg * a.n_kv + kvh) * ps + (j - blk * ps)) * D;
                float dot = 0.f;
                for (int d = 0; d < D; ++d) dot = fmaf(qs[d], kr[d], dot);
                s = dot * a.scale;
            } else {
                s = __int_as_float(0x7fc00000);  // a missing page must show, not pass as a masked key
            }
        }
        float cmax = block_max(s, red);
        float m_new = fmaxf(m, cmax);
        float p = valid ? expf(s - m_new) : 0.f;
        sp[tid] = p;
        float csum = block_sum(p, red);  // its barriers also publish sp
        float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
        l = l * alpha + csum;

        float part = 0.f;
        if (pv_active) {
            for (int jj = g_own; jj < CHUNK; jj += G) {
                int jk = c0 + jj;
                if (jk < lo || jk > pos) continue;
                int blk = jk / ps;
                int pg = bt[blk];
                if (pg < 0 || pg >= a.num_pages) continue;
                part = fmaf(sp[jj], a.v_pages[(((size_t)pg * a.n_kv + kvh) * D + d_own) * ps + (jk - blk * ps)], part);
            }
        }
        spart[tid] = part;
        __syncthreads();
        if (tid < D) {
            float sum = 0.f;
            for (int g = 0; g < G; ++g) sum += spart[g * D + tid];
            acc = acc * alpha + sum;
        }
        __syncthreads();
        m = m_new;
    }
    if (tid < D) a.out[((size_t)t * a.n_heads + h) * D + tid] = acc / l;
}

extern "C" int vt_attn_f32(const float* q, const float* k_pages, const float* v_pages, const int* positions,
                           const int* tok_entry, const int* block_table, float* out, int n, int n_heads, int n_kv,
                           int D, int page_size, int max_blocks, int num_pages, int window, float scale,
                           hipStream_t stream) {
    VT_REQUIRE(n >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "vt_attn_f32: bad heads %d/%d", n_heads, n_kv);
    VT_REQUIRE(D > 0 && D <= 256, "vt_attn_f32: head size %d is not in 1..256", D);
    VT_REQUIRE(page_size > 0 && max_blocks > 0 && num_pages > 0, "vt_attn_f32: bad cache sizes");
    VT_REQUIRE(n_heads <= 65535, "vt_attn_f32: too many heads (%d)", n_heads);
    if (n == 0) return 0;
    AttnF32Args a;
    a.q = q; a.k_pages = k_pages; a.v_pages = v_pages; a.positions = positions; a.tok_entry = tok_entry;
    a.block_table = block_table; a.out = out; a.n_heads = n_heads; a.n_kv = n_kv; a.D = D; a.page_size = page_size;
    a.max_blocks = max_blocks; a.num_pages = num_pages; a.window = window; a.scale = scale;
    size_t shmem = (size_t)(D + 2 * CHUNK) * sizeof(float);
    attn_f32_kernel<<<dim3(n, n_heads), CHUNK, shmem, stream>>>(a);
    VT_CHECK_LAUNCH("vt_attn_f32");
    return 0;
}
