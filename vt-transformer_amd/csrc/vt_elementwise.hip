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

// The same, for widths that are a multiple of 4 and at most 256 * 4 * RMS_MAXV: every value is read once with
// 16-byte loads and kept in registers between the sum and the scaling.  The sum of squares is taken in the same
// order whatever the number of rows.
#define RMS_MAXV 16
__device__ __forceinline__ float4 load4(const float* p) { return *(const float4*)p; }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
    uint2 u = *(const uint2*)p;
    return make_float4(lowp_lo(u.x), lowp_hi(u.x), lowp_lo(u.y), lowp_hi(u.y));
}
__device__ __forceinline__ void store4(float* p, float4 v) { *(float4*)p = v; }
__device__ __forceinline__ void store4(bf16_t* p, float4 v) {
    uint2 u;
    u.x = (unsigned)f32_to_bf16(v.x) | ((unsigned)f32_to_bf16(v.y) << 16);
    u.y = (unsigned)f32_to_bf16(v.z) | ((unsigned)f32_to_bf16(v.w) << 16);
    *(uint2*)p = u;
}

template <typename TD, typename TO, bool HAS_DELTA, int NV>
__global__ __launch_bounds__(256) void rmsnorm_vec_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                                         const float* __restrict__ gain, TO* __restrict__ out,
                                                         const int* __restrict__ rows, int hidden, float eps, int update) {
    __shared__ float red[16];
    const int r = blockIdx.x, tid = threadIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* hr = h + src * hidden;
    const TD* dr = HAS_DELTA ? delta + src * hidden : nullptr;
    const int nq = hidden >> 2;
    float4 x[NV], gn[NV];
    float ss = 0.f;
    // the gains are asked for together with the values, not after the sum: one trip to memory instead of two
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int qi = tid + v * 256;
        if (qi < nq) gn[v] = load4(gain + 4 * qi);
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int qi = tid + v * 256;
        if (qi < nq) {
            x[v] = load4(hr + 4 * qi);
            if (HAS_DELTA) {
                float4 d = load4(dr + 4 * qi);
                x[v].x += d.x; x[v].y += d.y; x[v].z += d.z; x[v].w += d.w;
                if (update) store4(hr + 4 * qi, x[v]);
            }
            ss += x[v].x * x[v].x + x[v].y * x[v].y + x[v].z * x[v].z + x[v].w * x[v].w;
        }
    }
    ss = block_sum(ss, red);
    const float rinv = 1.0f / sqrtf(ss / (float)hidden + eps);
    TO* o = out + (size_t)r * hidden;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int qi = tid + v * 256;
        if (qi < nq) {
            const float4 g = gn[v];
            store4(o + 4 * qi, make_float4((g.x * x[v].x) * rinv, (g.y * x[v].y) * rinv, (g.z * x[v].z) * rinv,
                                           (g.w * x[v].w) * rinv));
        }
    }
}

template <typename TD, typename TO, bool HD>
static void launch_rmsnorm(float* h, const void* delta, const float* gain, void* out, const int* rows, int n_out,
                           int hidden, float eps, int update_h, hipStream_t stream) {
    const bool aligned = (hidden % 4 == 0) && !((uintptr_t)h & 15) && !((uintptr_t)gain & 15) && !((uintptr_t)out & 15) &&
                         !((uintptr_t)delta & 15);
    const int nq = hidden / 4;
#define VT_RNV(NV) rmsnorm_vec_kernel<TD, TO, HD, NV><<<n_out, 256, 0, stream>>>(h, (const TD*)delta, gain, (TO*)out, \
                                                                               rows, hidden, eps, update_h)
    if (aligned && nq <= 256 * 1) VT_RNV(1);
    else if (aligned && nq <= 256 * 2) VT_RNV(2);
    else if (aligned && nq <= 256 * 4) VT_RNV(4);
    else if (aligned && nq <= 256 * 8) VT_RNV(8);
    else if (aligned && nq <= 256 * RMS_MAXV) VT_RNV(RMS_MAXV);
    else {
        int threads = hidden >= 2048 ? 512 : 256;
        rmsnorm_kernel<TD, TO, HD><<<n_out, threads, 0, stream>>>(h, (const TD*)delta, gain, (TO*)out, rows, hidden, eps,
                                                                 update_h);
    }
#undef VT_RNV
}

extern "C" int vt_rmsnorm(float* h, const void* delta, int delta_dtype, const float* gain, void* out, int out_dtype,
                          const int* rows, int n_out, int hidden, float eps, int update_h, hipStream_t stream) {
    VT_REQUIRE(n_out >= 0 && hidden > 0, "vt_rmsnorm: bad sizes n=%d hidden=%d", n_out, hidden);
    VT_REQUIRE(!(update_h && rows), "vt_rmsnorm: cannot update the residual through a row list");
    if (n_out == 0) return 0;
#define VT_RN(TD, TO, HD) launch_rmsnorm<TD, TO, HD>(h, delta, gain, out, rows, n_out, hidden, eps, update_h, stream)
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

// Four values per access, four accesses of gate and of up in flight per thread before any is used: the kernel
// moves 3 values per result and lives on bytes in flight.  For widths that are a multiple of 4.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void silu_mul_vec_kernel(const TI* __restrict__ gu, TO* __restrict__ out, int inter,
                                                          int n) {
    const int qpr = inter >> 2;                                   // quads per row
    const long long total = (long long)qpr * n;
    const long long stride = (long long)gridDim.x * 256;
    for (long long base = (long long)blockIdx.x * 256 + threadIdx.x; base < total; base += 4 * stride) {
        float4 g[4], u[4];
        long long idx[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            idx[k] = base + k * stride;
            if (idx[k] < total) {
                const long long t = idx[k] / qpr;
                const int i = (int)(idx[k] - t * qpr) * 4;
                const TI* row = gu + (size_t)t * 2 * inter;
                g[k] = load4(row + i);
                u[k] = load4(row + inter + i);
            }
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            if (idx[k] < total) {
                const long long t = idx[k] / qpr;
                const int i = (int)(idx[k] - t * qpr) * 4;
                store4(out + (size_t)t * inter + i,
                       make_float4(g[k].x / (1.f + __expf(-g[k].x)) * u[k].x, g[k].y / (1.f + __expf(-g[k].y)) * u[k].y,
                                   g[k].z / (1.f + __expf(-g[k].z)) * u[k].z, g[k].w / (1.f + __expf(-g[k].w)) * u[k].w));
            }
        }
    }
}

// 16-bit in and out, widths that are a multiple of 8.  A thread takes one group of eight columns in four rows: eight
// 16-byte loads (gate and up of each row) are asked for before any is used, a wave's load is 1 KB of one row.  The
// loads are marked non-temporal: every byte passes once, and the memory delivers more to loads so marked.
// The gate's division is one reciprocal instruction (1 ulp, far below the 16-bit rounding of the result).
typedef unsigned ew_u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float silu_gate(float g, float u) { return g * __builtin_amdgcn_rcpf(1.f + __expf(-g)) * u; }
__device__ __forceinline__ unsigned silu_mul_pair(unsigned g, unsigned u) {
    return vt_pack2(silu_gate(lowp_lo(g), lowp_lo(u)), silu_gate(lowp_hi(g), lowp_hi(u)));
}
#define SILU_ROWS 4
__global__ __launch_bounds__(256) void silu_mul_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out,
                                                             int inter, int n) {
    const int c = (blockIdx.x * 256 + threadIdx.x) * 8;           // first of the thread's eight columns
    if (c >= inter) return;
    const int t0 = blockIdx.y * SILU_ROWS;
    ew_u32x4_t g[SILU_ROWS], u[SILU_ROWS];
#pragma unroll
    for (int k = 0; k < SILU_ROWS; ++k) {
        if (t0 + k < n) {
            const bf16_t* row = gu + (size_t)(t0 + k) * 2 * inter + c;
            g[k] = __builtin_nontemporal_load((const ew_u32x4_t*)row);
            u[k] = __builtin_nontemporal_load((const ew_u32x4_t*)(row + inter));
        }
    }
#pragma unroll
    for (int k = 0; k < SILU_ROWS; ++k) {
        if (t0 + k < n) {
            ew_u32x4_t o;
            o.x = silu_mul_pair(g[k].x, u[k].x); o.y = silu_mul_pair(g[k].y, u[k].y);
            o.z = silu_mul_pair(g[k].z, u[k].z); o.w = silu_mul_pair(g[k].w, u[k].w);
            // (stored plainly: the product behind reads it next, out of the memory-side cache if it is left there)
            *(ew_u32x4_t*)(out + (size_t)(t0 + k) * inter + c) = o;
        }
    }
}

template <typename TI, typename TO>
static void launch_silu_mul(const void* gu, void* out, int n, int inter, hipStream_t stream) {
    if constexpr (sizeof(TI) == 2 && sizeof(TO) == 2) {
        if (inter % 8 == 0 && !((uintptr_t)gu & 15) && !((uintptr_t)out & 15)) {
            const dim3 grid((inter / 8 + 255) / 256, (n + SILU_ROWS - 1) / SILU_ROWS);
            silu_mul_bf16x8_kernel<<<grid, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, inter, n);
            return;
        }
    }
    if (inter % 4 == 0 && !((uintptr_t)gu & 15) && !((uintptr_t)out & 15)) {
        const long long total = (long long)(inter / 4) * n;
        long long blocks = (total + 1023) / 1024;
        if (blocks > 8192) blocks = 8192;
        if (blocks < 1) blocks = 1;
        silu_mul_vec_kernel<TI, TO><<<(unsigned)blocks, 256, 0, stream>>>((const TI*)gu, (TO*)out, inter, n);
    } else {
        silu_mul_kernel<TI, TO><<<dim3((inter + 255) / 256, n), 256, 0, stream>>>((const TI*)gu, (TO*)out, inter);
    }
}

extern "C" int vt_silu_mul(const void* gu, int in_dtype, void* out, int out_dtype, int n, int inter, hipStream_t stream) {
    VT_REQUIRE(n >= 0 && inter > 0, "vt_silu_mul: bad sizes n=%d inter=%d", n, inter);
    if (n == 0) return 0;
    VT_REQUIRE(n <= 65535, "vt_silu_mul: more than 65535 rows (%d)", n);
    if (in_dtype == VT_F32 && out_dtype == VT_F32) launch_silu_mul<float, float>(gu, out, n, inter, stream);
    else if (in_dtype == VT_F32 && out_dtype == VT_BF16) launch_silu_mul<float, bf16_t>(gu, out, n, inter, stream);
    else if (in_dtype == VT_BF16 && out_dtype == VT_BF16) launch_silu_mul<bf16_t, bf16_t>(gu, out, n, inter, stream);
    else if (in_dtype == VT_BF16 && out_dtype == VT_F32) launch_silu_mul<bf16_t, float>(gu, out, n, inter, stream);
    else return vt_fail("vt_silu_mul: unknown dtypes %d -> %d", in_dtype, out_dtype);
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
                o = rotate_low(c[i], s[i], x, y);
            } else {
                float y = load_f32<TI>(in, i - half);
                o = rotate_high(c[i - half], s[i - half], x, y);
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

// Four dims per thread with 8- or 16-byte accesses, one block per token; for head sizes that are a multiple of 4
// and rotary dims that are a multiple of 8.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void rope_store_vec_kernel(RopeStoreArgs a) {
    const int t = blockIdx.x;
    const int D = a.D, half = a.rot >> 1, qd = D >> 2;
    const int pos = a.positions[t];
    const int tp = pos < a.max_pos ? (pos < 0 ? 0 : pos) : a.max_pos - 1;
    const float* c = a.cos_t + (size_t)tp * half;
    const float* s = a.sin_t + (size_t)tp * half;
    const int n_heads_all = a.n_heads + (a.write_kv ? 2 * a.n_kv : 0);
    const TI* in = (const TI*)a.qkv + (size_t)t * a.in_stride;
    long long page = -1;
    int slot = 0;
    if (a.write_kv) {
        const int e = a.tok_entry[t];
        const int blk = pos / a.page_size;
        slot = pos - blk * a.page_size;
        const int pg = (blk < a.max_blocks) ? a.block_table[(size_t)e * a.max_blocks + blk] : -1;
        if (pg >= 0 && pg < a.num_pages) page = pg;
    }
    for (int q = threadIdx.x; q < n_heads_all * qd; q += 256) {
        const int head = q / qd, i = (q - head * qd) * 4;
        const bool is_q = head < a.n_heads, is_v = head >= a.n_heads + a.n_kv;
        if (!is_q && page < 0) continue;   // no page: the host never asks for this
        const TI* hp = in + (size_t)head * D;
        float4 x = load4(hp + i), o = x;
        if (!is_v && i < a.rot) {
            if (i < half) {
                float4 y = load4(hp + i + half), cc = load4(c + i), sn = load4(s + i);
                o = make_float4(rotate_low(cc.x, sn.x, x.x, y.x), rotate_low(cc.y, sn.y, x.y, y.y), rotate_low(cc.z, sn.z, x.z, y.z),
                                rotate_low(cc.w, sn.w, x.w, y.w));
            } else {
                float4 y = load4(hp + i - half), cc = load4(c + i - half), sn = load4(s + i - half);
                o = make_float4(rotate_high(cc.x, sn.x, x.x, y.x), rotate_high(cc.y, sn.y, x.y, y.y), rotate_high(cc.z, sn.z, x.z, y.z),
                                rotate_high(cc.w, sn.w, x.w, y.w));
            }
        }
        if (is_q) {
            store4((TO*)a.q_out + ((size_t)t * a.n_heads + head) * D + i, o);
        } else if (!is_v) {
            const int kvh = head - a.n_heads;
            store4((TO*)a.k_pages + (((size_t)page * a.n_kv + kvh) * a.page_size + slot) * D + i, o);
        } else {
            const int kvh = head - a.n_heads - a.n_kv;
            TO* vp = (TO*)a.v_pages + (((size_t)page * a.n_kv + kvh) * D + i) * a.page_size + slot;
            store_f32<TO>(vp, 0, o.x);
            store_f32<TO>(vp, (size_t)a.page_size, o.y);
            store_f32<TO>(vp, (size_t)2 * a.page_size, o.z);
            store_f32<TO>(vp, (size_t)3 * a.page_size, o.w);
        }
    }
}

// Many tokens, 16-bit pages (a prompt portion): a block takes sixteen consecutive tokens of the step and either one
// kv head (its keys and its values) or RG_QH query heads.  The pages hold values transposed ([D][slot]), so a token
// alone writes its D values two bytes at a time, a page row apart; here the sixteen tokens' values meet in LDS
// ([D][token]) and a thread per dim writes the slots that are consecutive in one page with one store of up to 16 bytes
// (a whole page row when the sixteen tokens are a page's, as in a prompt cut at page edges).  Runs are found from
// the tokens' own pages and slots, so any mixture of entries and positions is written correctly, only less wide.
// Rows that are rotated go four pieces of four dims per thread at a time, all their loads asked for first.
#define RG_TOK 16
#define RG_PAD 18       // halfwords per tile row: a thread per row reads them without bank conflicts
#define RG_QH 4         // query heads of a block that rotates queries
#define RG_U 4          // pieces in flight per thread
template <typename TI>
__global__ __launch_bounds__(256) void rope_store_group_kernel(RopeStoreArgs a, int n) {
    extern __shared__ unsigned short rg_tile[];        // [D][RG_PAD]
    __shared__ int s_page[RG_TOK], s_slot[RG_TOK], s_pos[RG_TOK];
    const int tid = threadIdx.x;
    const int t0 = blockIdx.x * RG_TOK, cnt = min(RG_TOK, n - t0);
    const int D = a.D, half = a.rot >> 1, qd = D >> 2;
    const bool kv_block = (int)blockIdx.y < a.n_kv;
    const int kvh = blockIdx.y;                                         // (a kv block's head)
    const int head0 = kv_block ? a.n_heads + kvh : ((int)blockIdx.y - a.n_kv) * RG_QH;
    const int n_rot_heads = kv_block ? 1 : min(RG_QH, a.n_heads - head0);
    if (tid < RG_TOK) {
        int page = -1, slot = 0, pos = 0;
        if (tid < cnt) {
            pos = a.positions[t0 + tid];
            if (kv_block) {
                const int e = a.tok_entry[t0 + tid];
                const int blk = pos / a.page_size;
                slot = pos - blk * a.page_size;
                const int pg = (blk >= 0 && blk < a.max_blocks) ? a.block_table[(size_t)e * a.max_blocks + blk] : -1;
                if (pg >= 0 && pg < a.num_pages) page = pg;      // (no page: the host never asks for this)
            }
        }
        s_page[tid] = page; s_slot[tid] = slot; s_pos[tid] = pos;
    }
    __syncthreads();
    // the block's query heads, or its kv head's keys: rotated, a row of D at a time.  32 lanes along a row (four dims
    // each), 8 rows side by side; row r is head r % n_rot_heads of token r / n_rot_heads (a product and a shift: the
    // quotient of r < 64 by a number up to RG_QH), so that no piece costs an integer division.
    const int lane_q = tid & 31, lane_r = tid >> 5;
    const int n_rows = cnt * n_rot_heads;
    const unsigned inv = (65536u + n_rot_heads - 1) / n_rot_heads;
    for (int q0 = lane_q; q0 < qd; q0 += 32) {
        const int i = q0 * 4;
        const bool rotated = i < a.rot, low = i < half;
        const int ip = low ? i : i - half, iy = low ? i + half : i - half;
        for (int r0 = lane_r; r0 < n_rows; r0 += 8 * RG_U) {
            float4 x[RG_U], y[RG_U], cc[RG_U], sn[RG_U];
#pragma unroll
            for (int u = 0; u < RG_U; ++u) {
                const int r = r0 + 8 * u;
                if (r < n_rows) {
                    const int j = (int)((r * inv) >> 16), h = r - j * n_rot_heads;
                    const int pos = s_pos[j];
                    const int tp = pos < a.max_pos ? (pos < 0 ? 0 : pos) : a.max_pos - 1;
                    const TI* hp = (const TI*)a.qkv + (size_t)(t0 + j) * a.in_stride + (size_t)(head0 + h) * D;
                    x[u] = load4(hp + i);
                    if (rotated) {
                        y[u] = load4(hp + iy);
                        cc[u] = load4(a.cos_t + (size_t)tp * half + ip);
                        sn[u] = load4(a.sin_t + (size_t)tp * half + ip);
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < RG_U; ++u) {
                const int r = r0 + 8 * u;
                if (r >= n_rows) continue;
                const int j = (int)((r * inv) >> 16), h = r - j * n_rot_heads;
                float4 o = x[u];
                if (rotated)
                    o = make_float4(rotate_pair(cc[u].x, sn[u].x, x[u].x, y[u].x, low), rotate_pair(cc[u].y, sn[u].y, x[u].y, y[u].y, low),
                                    rotate_pair(cc[u].z, sn[u].z, x[u].z, y[u].z, low), rotate_pair(cc[u].w, sn[u].w, x[u].w, y[u].w, low));
                if (!kv_block) store4((bf16_t*)a.q_out + ((size_t)(t0 + j) * a.n_heads + head0 + h) * D + i, o);
                else if (s_page[j] >= 0)
                    store4((bf16_t*)a.k_pages + (((size_t)s_page[j] * a.n_kv + kvh) * a.page_size + s_slot[j]) * D + i, o);
            }
        }
    }
    if (!kv_block) return;
    // the head's values into the tile, a column per token
    for (int q0 = lane_q; q0 < qd; q0 += 32) {
        const int i = q0 * 4;
        for (int j = lane_r; j < cnt; j += 8) {
            const TI* hp = (const TI*)a.qkv + (size_t)(t0 + j) * a.in_stride + (size_t)(a.n_heads + a.n_kv + kvh) * D;
            const float4 x = load4(hp + i);
            rg_tile[(i + 0) * RG_PAD + j] = f32_to_bf16(x.x);
            rg_tile[(i + 1) * RG_PAD + j] = f32_to_bf16(x.y);
            rg_tile[(i + 2) * RG_PAD + j] = f32_to_bf16(x.z);
            rg_tile[(i + 3) * RG_PAD + j] = f32_to_bf16(x.w);
        }
    }
    __syncthreads();
    // a thread per dim: the runs of tokens whose slots follow each other in one page, each in the widest stores
    // that the slot's alignment allows (page rows start at multiples of 16 bytes: page sizes are multiples of 8)
    for (int d = tid; d < D; d += 256) {
        const unsigned short* src = rg_tile + d * RG_PAD;
        int j = 0;
        while (j < cnt) {
            const int page = s_page[j], slot = s_slot[j];
            int m = 1;
            while (j + m < cnt && s_page[j + m] == page && s_slot[j + m] == slot + m) ++m;
            if (page >= 0) {
                bf16_t* dst = (bf16_t*)a.v_pages + (((size_t)page * a.n_kv + kvh) * D + d) * a.page_size + slot;
                int k = 0;
                while (k < m) {
                    const int sl = slot + k, left = m - k;
                    const unsigned short* sp = src + j + k;
                    if (!(sl & 7) && left >= 8) {
                        uint4 v;
                        v.x = sp[0] | ((unsigned)sp[1] << 16); v.y = sp[2] | ((unsigned)sp[3] << 16);
                        v.z = sp[4] | ((unsigned)sp[5] << 16); v.w = sp[6] | ((unsigned)sp[7] << 16);
                        *(uint4*)(dst + k) = v;
                        k += 8;
                    } else if (!(sl & 3) && left >= 4) {
                        *(uint2*)(dst + k) = make_uint2(sp[0] | ((unsigned)sp[1] << 16), sp[2] | ((unsigned)sp[3] << 16));
                        k += 4;
                    } else if (!(sl & 1) && left >= 2) {
                        *(unsigned*)(dst + k) = sp[0] | ((unsigned)sp[1] << 16);
                        k += 2;
                    } else {
                        dst[k] = sp[0];
                        k += 1;
                    }
                }
            }
            j += m;
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
    const int isz = in_dtype == VT_F32 ? 4 : 2;
    const bool vec = (D % 4 == 0) && (rot % 8 == 0) && (in_stride % 4 == 0) && !((uintptr_t)qkv & 15) &&
                     !((uintptr_t)q_out & 15) && !((uintptr_t)k_pages & 15) && !((uintptr_t)cos_t & 15) &&
                     !((uintptr_t)sin_t & 15) && (((size_t)D * isz) % 8 == 0);
    dim3 grid(n, n_heads + (write_kv ? 2 * n_kv : 0));
    VT_REQUIRE(grid.y <= 65535, "vt_rope_store: too many heads (%u)", grid.y);
    int threads = D <= 64 ? 64 : (D <= 128 ? 128 : 256);
    // sixteen tokens and a kv head per block, the values through LDS: 16-bit pages, a portion of many tokens
    const bool grouped = vec && write_kv && out_dtype == VT_BF16 && n >= 4 * RG_TOK && page_size % 8 == 0 &&
                         n_kv + n_heads <= 65535 && !((uintptr_t)v_pages & 15);
    const dim3 ggrid((n + RG_TOK - 1) / RG_TOK, n_kv + (n_heads + RG_QH - 1) / RG_QH);
    const size_t glds = (size_t)D * RG_PAD * sizeof(unsigned short);
    VT_REQUIRE(!grouped || glds <= 48 * 1024, "vt_rope_store: head size %d is too large for the grouped kernel", D);
#define VT_RS(TI, TO)                                                                    \
    do {                                                                                 \
        if (grouped && sizeof(TO) == 2) rope_store_group_kernel<TI><<<ggrid, 256, glds, stream>>>(a, n); \
        else if (vec) rope_store_vec_kernel<TI, TO><<<n, 256, 0, stream>>>(a);           \
        else rope_store_kernel<TI, TO><<<grid, threads, 0, stream>>>(a);                 \
    } while (0)
    if (in_dtype == VT_F32 && out_dtype == VT_F32) VT_RS(float, float);
    else if (in_dtype == VT_F32 && out_dtype == VT_BF16) VT_RS(float, bf16_t);
    else if (in_dtype == VT_BF16 && out_dtype == VT_BF16) VT_RS(bf16_t, bf16_t);
    else return vt_fail("vt_rope_store: unsupported dtypes %d -> %d", in_dtype, out_dtype);
#undef VT_RS
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

// ---------------------------------------------------------------------------
// Streaming read: what the memory delivers to a kernel that only reads (the measured ceiling that the weight
// streaming kernels are compared with).  Every wave reads a contiguous share, 1 KB per load instruction and
// eight loads in flight, and leaves the XOR of its 32-bit words in sums[wave]; the words behind the last full
// share of all waves are read by the last wave one load at a time.  The loads are marked non-temporal, as the
// weight-streaming kernels mark theirs: read once, not to be kept in the caches (6.7 against 6.0 TB/s unmarked).
typedef unsigned stream_u32x4_t __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(1024) void stream_read_kernel(const uint4* __restrict__ p, size_t n16,
                                                          unsigned* __restrict__ sums) {
    constexpr int U = 8;
    const size_t waves = (size_t)gridDim.x * (blockDim.x >> 6);
    const size_t wave = (size_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const size_t per = n16 / (waves * 64 * U) * (64 * U);      // 16-byte pieces per wave, whole turns only
    const uint4* q = p + wave * per + lane;
    unsigned acc = 0;
    for (size_t i = 0; i < per; i += 64 * U) {
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const stream_u32x4_t t = __builtin_nontemporal_load((const stream_u32x4_t*)(q + i + 64 * u));
            v[u] = make_uint4(t.x, t.y, t.z, t.w);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (wave == waves - 1)
        for (size_t i = waves * per + lane; i < n16; i += 64) {
            const uint4 v = p[i];
            acc ^= v.x ^ v.y ^ v.z ^ v.w;
        }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc ^= __shfl_xor(acc, off);
    if (lane == 0) sums[wave] = acc;
}

// sums: blocks * 16 words; the XOR of all of them is the XOR of the buffer's 32-bit words (bytes a multiple of 16)
extern "C" int vt_stream_read(const void* p, long long bytes, unsigned* sums, int blocks, hipStream_t stream) {
    VT_REQUIRE(bytes >= 0 && bytes % 16 == 0 && (((uintptr_t)p) & 15) == 0,
               "vt_stream_read: %lld bytes at %p are not whole 16-byte pieces", bytes, p);
    VT_REQUIRE(blocks > 0 && blocks <= 65535, "vt_stream_read: %d blocks", blocks);
    stream_read_kernel<<<blocks, 1024, 0, stream>>>((const uint4*)p, (size_t)bytes / 16, sums);
    VT_CHECK_LAUNCH("vt_stream_read");
    return 0;
}

// ---------------------------------------------------------------------------
// Random weights whose bits do not depend on where they are made.  Element i of a tensor is a function of
// (key, i) alone: three words of the SplitMix64 stream that starts at `key` (counters 3 i + 1 .. 3 i + 3), cut
// into twelve 16-bit integers whose sum is close to normally distributed (mean 393,210, variance 2^32 - 1).  The
// sum is exact in integers; one float multiplication and one addition, each rounded on its own, make the value,
// so the host's twin of this kernel (weights/random_init.py) produces the same bits.  The reference has no such
// mode (nearest: the fixed mt19937(1979) of v1/tensortype/context.cpp:45).
__device__ __forceinline__ unsigned long long splitmix64_at(unsigned long long key, unsigned long long counter) {
    unsigned long long z = key + counter * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

template <typename TO>
__global__ void random_normal_kernel(TO* __restrict__ out, unsigned long long n, unsigned long long first,
                                     unsigned long long key, float scale, float mean) {
    const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
    for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const unsigned long long e = first + i;
        int s = 0;
#pragma unroll
        for (int j = 1; j <= 3; ++j) {
            const unsigned long long w = splitmix64_at(key, 3ull * e + j);
            s += (int)(w & 0xffffu) + (int)((w >> 16) & 0xffffu) + (int)((w >> 32) & 0xffffu) + (int)(w >> 48);
        }
        float v;
        {
            // the product and the sum each rounded on its own, as the host's twin does: never one fused operation
#pragma clang fp contract(off)
            const float prod = (float)(s - 393210) * scale;
            v = prod + mean;
        }
        store_f32<TO>(out, i, v);
    }
}

// out[i] = mean + scale * (sum of twelve 16-bit integers of element first + i  -  393,210), i < n
extern "C" int vt_random_normal(void* out, int out_dtype, long long n, long long first, unsigned long long key,
                                float scale, float mean, hipStream_t stream) {
    VT_REQUIRE(n >= 0 && first >= 0, "vt_random_normal: n=%lld first=%lld", n, first);
    if (n == 0) return 0;
    const unsigned blocks = (unsigned)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    if (out_dtype == VT_F32)
        random_normal_kernel<float><<<blocks, 256, 0, stream>>>((float*)out, (unsigned long long)n, (unsigned long long)first, key, scale, mean);
    else if (out_dtype == VT_BF16)
        random_normal_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (unsigned long long)n, (unsigned long long)first, key, scale, mean);
    else
        return vt_fail("vt_random_normal: unknown out dtype %d", out_dtype);
    VT_CHECK_LAUNCH("vt_random_normal");
    return 0;
}
