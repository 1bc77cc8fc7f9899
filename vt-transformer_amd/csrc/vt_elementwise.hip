// Embedding gather, fused residual-add + RMSNorm, SiLU gating, and rotary
// encoding fused with the write of keys and values into cache pages.
//
// Formulas are the reference's:
//   RMSNorm   v1/tensortype/hip_kernels/rmsnorm.cpp:7-44   out = (w*x) * rsqrt(sum(x^2)/dim + eps)
//   rotary    v1/tensortype/hip_kernels/rotary_embed.cpp:6-27  pairs (i, i+D/2)
//   SiLU gate v1/tensortype/hip_kernels/silu_product.cpp:8-16  a/(1+exp(-a)) * u
//   residual  v1/tensortype/hip_kernels/pointwise.cpp:51-57   (float)A + (float)B
//   embedding v1/tensortype/hip_kernels/embed.cpp:7-37        row copy
// Unlike the reference the residual stream stays in fp32 between kernels, and
// no size has to be a multiple of the block size.
#include "vt_common.h"

VT_DEFINE_LAST_ERROR()

// ---------------------------------------------------------------------------
// embedding: out[t, :] = table[ids[t], :] as fp32
// ---------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids, float* __restrict__ out,
                             int hidden, int vocab) {
    int t = blockIdx.x;
    int id = ids[t];
    bool ok = id >= 0 && id < vocab;
    const T* row = table + (size_t)(ok ? id : 0) * hidden;
    float* o = out + (size_t)t * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = ok ? load_f32<T>(row, i) : __int_as_float(0x7fc00000);
}

extern "C" int vt_embed(const void* table, int table_dtype, const int* ids, float* out, int n, int hidden, int vocab,
                        hipStream_t stream) {
    VT_REQUIRE(n >= 0 && hidden > 0 && vocab > 0, "vt_embed: bad sizes n=%d hidden=%d vocab=%d", n, hidden, vocab);
    if (n == 0) return 0;
    if (table_dtype == VT_F32)
        embed_kernel<float><<<n, 256, 0, stream>>>((const float*)table, ids, out, hidden, vocab);
    else if (table_dtype == VT_BF16)
        embed_kernel<bf16_t><<<n, 256, 0, stream>>>((const bf16_t*)table, ids, out, hidden, vocab);
    else
        return vt_fail("vt_embed: unknown table dtype %d", table_dtype);
    VT_CHECK_LAUNCH("vt_embed");
    return 0;
}

// ---------------------------------------------------------------------------
// x = h[row] (+ delta[row]);  if update: h[row] = x;  out[r] = (gain*x) / sqrt(mean(x^2)+eps)
// rows == nullptr: row = r.  One block per output row; sums in fp32.
// ---------------------------------------------------------------------------
template <typename TD, typename TO, bool HAS_DELTA>
__global__ void rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta, const float* __restrict__ gain,
                               TO* __restrict__ out, const int* __restrict__ rows, int hidden, float eps, int update) {
    __shared__ float red[16];
    int r = blockIdx.x;
    size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* hr = h + src * hidden;
    const TD* dr = HAS_DELTA ? delta + src * hidden : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float x = hr[i];
        if (HAS_DELTA) x += load_f32<TD>(dr, i);
        ss += x * x;
    }
    ss = block_sum(ss, red);
    float rinv = 1.0f / sqrtf(ss / (float)hidden + eps);
    TO* o = out + (size_t)r * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float x = hr[i];
        if (HAS_DELTA) {
            x += load_f32<TD>(dr, i);
            if (update) hr[i] = x;
        }
        store_f32<TO>(o, i, (gain[i] * x) * rinv);
    }
}

extern "C" int vt_rmsnorm(float* h, const void* delta, int delta_dtype, const float* gain, void* out, int out_dtype,
                          const int* rows, int n_out, int hidden, float eps, int update_h, hipStream_t stream) {
    VT_REQUIRE(n_out >= 0 && hidden > 0, "vt_rmsnorm: bad sizes n=%d hidden=%d", n_out, hidden);
    VT_REQUIRE(!(update_h && rows), "vt_rmsnorm: cannot update the residual through a row list");
    if (n_out == 0) return 0;
    int threads = hidden >= 2048 ? 512 : 256;
#define VT_RN(TD, TO, HD)                                                                                       \
    rmsnorm_kernel<TD, TO, HD><<<n_out, threads, 0, stream>>>(h, (const TD*)delta, gain, (TO*)out, rows, hidden, \
                                                              eps, update_h)
    if (!delta) {
        if (out_dtype == VT_F32) VT_RN(float, float, false);
        else if (out_dtype == VT_BF16) VT_RN(float, bf16_t, false);
        else return vt_fail("vt_rmsnorm: unknown out dtype %d", out_dtype);
    } else if (delta_dtype == VT_F32) {
        if (out_dtype == VT_F32) VT_RN(float, float, true);
        else if (out_dtype == VT_BF16) VT_RN(float, bf16_t, true);
        else return vt_fail("vt_rmsnorm: unknown out dtype %d", out_dtype);
    } else if (delta_dtype == VT_BF16) {
        if (out_dtype == VT_F32) VT_RN(bf16_t, float, true);
        else if (out_dtype == VT_BF16) VT_RN(bf16_t, bf16_t, true);
        else return vt_fail("vt_rmsnorm: unknown out dtype %d", out_dtype);
    } else {
        return vt_fail("vt_rmsnorm: unknown delta dtype %d", delta_dtype);
    }
#undef VT_RN
    VT_CHECK_LAUNCH("vt_rmsnorm");
    return 0;
}

// ---------------------------------------------------------------------------
// h += delta (fp32 sum), for a residual that no norm follows
// ---------------------------------------------------------------------------
template <typename TD>
__global__ void residual_add_kernel(float* __restrict__ h, const TD* __restrict__ delta, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) h[i] += load_f32<TD>(delta, i);
}

extern "C" int vt_residual_add(float* h, const void* delta, int delta_dtype, long long n, hipStream_t stream) {
    if (n <= 0) return 0;
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (delta_dtype == VT_F32) residual_add_kernel<float><<<blocks, 256, 0, stream>>>(h, (const float*)delta, (size_t)n);
    else if (delta_dtype == VT_BF16) residual_add_kernel<bf16_t><<<blocks, 256, 0, stream>>>(h, (const bf16_t*)delta, (size_t)n);
    else return vt_fail("vt_residual_add: unknown dtype %d", delta_dtype);
    VT_CHECK_LAUNCH("vt_residual_add");
    return 0;
}

// ---------------------------------------------------------------------------
// out[t, i] = silu(gu[t, i]) * gu[t, inter + i]
// ---------------------------------------------------------------------------
template <typename TI, typename TO>
__global__ void silu_mul_kernel(const TI* __restrict__ gu, TO* __restrict__ out, int inter) {
    int t = blockIdx.y;
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= inter) return;
    const TI* row = gu + (size_t)t * 2 * inter;
    float g = load_f32<TI>(row, i);
    float u = load_f32<TI>(row, (size_t)inter + i);
    store_f32<TO>(out + (size_t)t * inter, i, g / (1.f + expf(-g)) * u);
}

extern "C" int vt_silu_mul(const void* gu, int in_dtype, void* out, int out_dtype, int n, int inter, hipStream_t stream) {
    VT_REQUIRE(n >= 0 && inter > 0, "vt_silu_mul: bad sizes n=%d inter=%d", n, inter);
    if (n == 0) return 0;
    VT_REQUIRE(n <= 65535, "vt_silu_mul: more than 65535 rows (%d)", n);
    dim3 grid((inter + 255) / 256, n);
    if (in_dtype == VT_F32 && out_dtype == VT_F32)
        silu_mul_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)gu, (float*)out, inter);
    else if (in_dtype == VT_F32 && out_dtype == VT_BF16)
        silu_mul_kernel<float, bf16_t><<<grid, 256, 0, stream>>>((const float*)gu, (bf16_t*)out, inter);
    else if (in_dtype == VT_BF16 && out_dtype == VT_BF16)
        silu_mul_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, inter);
    else if (in_dtype == VT_BF16 && out_dtype == VT_F32)
        silu_mul_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((const bf16_t*)gu, (float*)out, inter);
    else
        return vt_fail("vt_silu_mul: unknown dtypes %d -> %d", in_dtype, out_dtype);
    VT_CHECK_LAUNCH("vt_silu_mul");
    return 0;
}

// ---------------------------------------------------------------------------
// Rotary encoding of queries and keys and the write of keys and values into
// cache pages, one block per (token, head).
//
// qkv row of a token: [n_heads*D queries | n_kv*D keys | n_kv*D values], row stride in_stride.
// Rotation of dims i and i+rot/2 (i < rot/2) by the angle of (position, i); dims from `rot` on pass through.
// Key pages:   [page][kv_head][slot][D]
// Value pages: [page][kv_head][D][slot]     (slot fastest, so attention reads 4 keys of one dim at once)
// ---------------------------------------------------------------------------
struct RopeStoreArgs {
    const void* qkv;
    const float* cos_t;
    const float* sin_t;
    const int* positions;
    const int* tok_entry;
    const int* block_table;
    void* q_out;
    void* k_pages;
    void* v_pages;
    long long in_stride;
    int rot, max_pos, max_blocks, page_size, num_pages;
    int n_heads, n_kv, D, write_kv;
};

template <typename TI, typename TO>
__global__ void rope_store_kernel(RopeStoreArgs a) {
    int t = blockIdx.x;
    int head = blockIdx.y;
    int D = a.D, half = a.rot >> 1;
    int pos = a.positions[t];
    const TI* in = (const TI*)a.qkv + (size_t)t * a.in_stride + (size_t)head * D;
    bool is_q = head < a.n_heads;
    bool is_v = head >= a.n_heads + a.n_kv;
    // the host sizes the table for every position it hands out; the clamp only keeps a bad call from faulting
    int tp = pos < a.max_pos ? (pos < 0 ? 0 : pos) : a.max_pos - 1;
    const float* c = a.cos_t + (size_t)tp * half;
    const float* s = a.sin_t + (size_t)tp * half;

    size_t page = 0;
    int slot = 0, kvh = 0;
    if (!is_q) {
        int e = a.tok_entry[t];
        int blk = pos / a.page_size;
        slot = pos - blk * a.page_size;
        int pg = (blk < a.max_blocks) ? a.block_table[(size_t)e * a.max_blocks + blk] : -1;
        if (pg < 0 || pg >= a.num_pages) return;  // no page: the host never asks for this
        page = (size_t)pg;
        kvh = is_v ? head - a.n_heads - a.n_kv : head - a.n_heads;
    }
    for (int i = threadIdx.x; i < D; i += blockDim.x) {
        float x = load_f32<TI>(in, i);
        float o = x;
        if (!is_v && i < a.rot) {
            if (i < half) {
                float y = load_f32<TI>(in, i + half);
                o = c[i] * x - s[i] * y;
            } else {
                float y = load_f32<TI>(in, i - half);
                o = c[i - half] * x + s[i - half] * y;
            }
        }
        if (is_q) {
            store_f32<TO>((TO*)a.q_out + ((size_t)t * a.n_heads + head) * D, i, o);
        } else if (!is_v) {
            store_f32<TO>((TO*)a.k_pages, ((page * a.n_kv + kvh) * a.page_size + slot) * D + i, o);
        } else {
            store_f32<TO>((TO*)a.v_pages, ((page * a.n_kv + kvh) * D + i) * a.page_size + slot, o);
        }
    }
}

extern "C" int vt_rope_store(const void* qkv, int in_dtype, long long in_stride, const float* cos_t, const float* sin_t,
                             int rot, int max_pos, const int* positions, const int* tok_entry, const int* block_table,
                             int max_blocks, void* q_out, void* k_pages, void* v_pages, int out_dtype, int page_size,
                             int num_pages, int n, int n_heads, int n_kv, int D, int write_kv, hipStream_t stream) {
    VT_REQUIRE(n >= 0 && n_heads > 0 && D > 0, "vt_rope_store: bad sizes n=%d heads=%d D=%d", n, n_heads, D);
    VT_REQUIRE(rot >= 0 && rot <= D && rot % 2 == 0, "vt_rope_store: rotary dims %d must be even and at most D=%d", rot, D);
    VT_REQUIRE(!write_kv || (n_kv > 0 && page_size > 0 && num_pages > 0 && max_blocks > 0),
               "vt_rope_store: bad cache sizes kv=%d page=%d pages=%d blocks=%d", n_kv, page_size, num_pages, max_blocks);
    VT_REQUIRE(rot == 0 || max_pos > 0, "vt_rope_store: empty rotary table");
    if (n == 0) return 0;
    RopeStoreArgs a;
    a.qkv = qkv; a.cos_t = cos_t; a.sin_t = sin_t; a.positions = positions; a.tok_entry = tok_entry;
    a.block_table = block_table; a.q_out = q_out; a.k_pages = k_pages; a.v_pages = v_pages;
    a.in_stride = in_stride; a.rot = rot; a.max_pos = max_pos; a.max_blocks = max_blocks;
    a.page_size = page_size; a.num_pages = num_pages; a.n_heads = n_heads; a.n_kv = n_kv; a.D = D; a.write_kv = write_kv;
    dim3 grid(n, n_heads + (write_kv ? 2 * n_kv : 0));
    VT_REQUIRE(grid.y <= 65535, "vt_rope_store: too many heads (%u)", grid.y);
    int threads = D <= 64 ? 64 : (D <= 128 ? 128 : 256);
    if (in_dtype == VT_F32 && out_dtype == VT_F32) rope_store_kernel<float, float><<<grid, threads, 0, stream>>>(a);
    else if (in_dtype == VT_F32 && out_dtype == VT_BF16) rope_store_kernel<float, bf16_t><<<grid, threads, 0, stream>>>(a);
    else if (in_dtype == VT_BF16 && out_dtype == VT_BF16) rope_store_kernel<bf16_t, bf16_t><<<grid, threads, 0, stream>>>(a);
    else return vt_fail("vt_rope_store: unsupported dtypes %d -> %d", in_dtype, out_dtype);
    VT_CHECK_LAUNCH("vt_rope_store");
    return 0;
}

// ---------------------------------------------------------------------------
// out[r, :] = (TO) in[rows[r], :]   (row gather with conversion)
// ---------------------------------------------------------------------------
template <typename TI, typename TO>
__global__ void gather_rows_kernel(const TI* __restrict__ in, const int* __restrict__ rows, TO* __restrict__ out, int width) {
    int r = blockIdx.x;
    size_t src = rows ? (size_t)rows[r] : (size_t)r;
    for (int i = threadIdx.x; i < width; i += blockDim.x)
        store_f32<TO>(out + (size_t)r * width, i, load_f32<TI>(in + src * width, i));
}

extern "C" int vt_gather_rows(const void* in, int in_dtype, const int* rows, void* out, int out_dtype, int n, int width,
                              hipStream_t stream) {
    VT_REQUIRE(n >= 0 && width > 0, "vt_gather_rows: bad sizes n=%d width=%d", n, width);
    if (n == 0) return 0;
    if (in_dtype == VT_F32 && out_dtype == VT_F32)
        gather_rows_kernel<float, float><<<n, 256, 0, stream>>>((const float*)in, rows, (float*)out, width);
    else if (in_dtype == VT_F32 && out_dtype == VT_BF16)
        gather_rows_kernel<float, bf16_t><<<n, 256, 0, stream>>>((const float*)in, rows, (bf16_t*)out, width);
    else if (in_dtype == VT_BF16 && out_dtype == VT_F32)
        gather_rows_kernel<bf16_t, float><<<n, 256, 0, stream>>>((const bf16_t*)in, rows, (float*)out, width);
    else if (in_dtype == VT_BF16 && out_dtype == VT_BF16)
        gather_rows_kernel<bf16_t, bf16_t><<<n, 256, 0, stream>>>((const bf16_t*)in, rows, (bf16_t*)out, width);
    else return vt_fail("vt_gather_rows: unknown dtypes %d -> %d", in_dtype, out_dtype);
    VT_CHECK_LAUNCH("vt_gather_rows");
    return 0;
}
