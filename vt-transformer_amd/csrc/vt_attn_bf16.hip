// bfloat16 attention over paged keys and values on the gfx950 matrix cores,
// for portions of prompts and for decoding, compiled for one head size
// (VT_HEAD_DIM, a multiple of 16 up to 256).
//
// It replaces the reference's chain of launches per layer
// (v1/models/qwen2-7b/inference_fp16.dag:299-318): repeat the key/value heads
// for their query heads (v1/tensortype/hip_kernels/transpose_0213.cpp:89-103),
// scores with scale 1/sqrt(D) (v1/tensortype/hip_tensor.cpp:691), additive
// causal mask (v1/tensortype/hip_kernels/causal_mask.cpp:57-83), softmax in
// fp32 (v1/tensortype/hip_kernels/softmax.cpp:10-43), weighted sum of values.
// Nothing is repeated or materialised here: the rows of a tile are
// (token, query head of one key/value group) pairs, so one read of a
// key/value head serves all of its query heads.
//
// One wave = one work item = 16 rows x a range of keys.  Both products are
// computed transposed so that the probabilities leave the first matrix
// instruction in the register layout the second one wants as its B operand:
//   S^T[key, row] = K[key, :] . Q[row, :]^T      A = 16 keys x k dims     B = k dims x 16 rows
//   O^T[dim, row] = V^T[dim, key] . P^T[key, row] A = 16 dims x 16 keys    B = 16 keys x 16 rows
// K pages are [page][kv head][slot][D]; V pages are [page][kv head][D][slot],
// so both A operands are contiguous reads per lane.  Softmax statistics are
// per row = per lane%16, kept in fp32 in the exp2 domain.
//
// An item either writes its rows' output, or (when the keys of a row tile
// are split over several items) an unnormalised partial result that
// vt_attn_bf16_combine merges.
#include "vt_common.h"
#include <math.h>

VT_DEFINE_LAST_ERROR()

#ifndef VT_HEAD_DIM
#error "compile with -DVT_HEAD_DIM=<head size>"
#endif
static_assert(VT_HEAD_DIM % 16 == 0 && VT_HEAD_DIM >= 16 && VT_HEAD_DIM <= 256, "head size must be 16..256 in steps of 16");

#define D VT_HEAD_DIM
#define ITEM_INTS 8  // entry, q_tok0, q_len, pos0, q_row0, key_lo, key_hi, part (-1: final)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) short bf16x4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

struct AttnArgs {
    const bf16_t* q;        // [N][n_heads][D]
    const bf16_t* k_pages;  // [pages][n_kv][page_size][D]
    const bf16_t* v_pages;  // [pages][n_kv][D][page_size]
    const int* block_table; // [entries][max_blocks]
    const int* items;       // [n_items][ITEM_INTS]
    bf16_t* out;            // [N][n_heads][D]
    float* part_o;          // [parts][n_kv][16][D]
    float* part_ml;         // [parts][n_kv][16][2]
    int n_items, n_heads, n_kv, page_size, max_blocks, num_pages, window;
    float scale_log2;       // scale * log2(e)
    // decode mode: one token per entry, items are computed here from the entries' positions
    const int* entry_pos0;  // [entries] position of each entry's token
    const int* dec_params;  // [0] = chunk: keys per item (a multiple of 16), read from memory so that a
                            //       captured launch can be replayed with another value
    int p_max;              // items per entry
};

union U8 { uint2 u; bf16x4_t v; };
union U16 { uint4 u; bf16x8_t v; };

__device__ __forceinline__ unsigned pack2(float a, float b) {
    return (unsigned)f32_to_bf16(a) | ((unsigned)f32_to_bf16(b) << 16);
}

template <bool DECODE>
__global__ __launch_bounds__(256) void attn_bf16_kernel(AttnArgs a) {
    const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int item = blockIdx.x * 4 + wv;
    if (item >= a.n_items) return;
    int entry, q_tok0, q_len, pos0, q_row0, key_lo, key_hi, part;
    if (DECODE) {
        // item = (entry, part p): keys [p*chunk, (p+1)*chunk) of the entry's one token
        const int chunk = a.dec_params[0];
        entry = item / a.p_max;
        const int pi = item - entry * a.p_max;
        q_tok0 = entry; q_len = 1; q_row0 = 0;
        pos0 = a.entry_pos0[entry];
        const int lo = a.window > 0 ? max(0, pos0 - a.window + 1) : 0;
        const int p_first = ((lo >> 4) << 4) / chunk, p_last = pos0 / chunk;
        if (pi < p_first || pi > p_last) return;
        key_lo = max((lo >> 4) << 4, pi * chunk);
        key_hi = min(pos0 + 1, (pi + 1) * chunk);
        part = (p_first == p_last) ? -1 : item;
    } else {
        const int* it = a.items + (size_t)item * ITEM_INTS;
        entry = it[0]; q_tok0 = it[1]; q_len = it[2]; pos0 = it[3]; q_row0 = it[4];
        key_lo = it[5]; key_hi = it[6]; part = it[7];
        if (entry < 0) return;
    }
    const int kvh = blockIdx.y;
    const int G = a.n_heads / a.n_kv;
    const int r = lane & 15, g = lane >> 4;
    const int ps = a.page_size;

    const int n_rows = q_len * G;
    const int row = q_row0 + r;
    const bool row_ok = row < n_rows;
    const int rowc = row_ok ? row : n_rows - 1;
    const int ti = rowc / G, head = kvh * G + (rowc - ti * G);
    const int p = pos0 + ti;                                  // this row's position
    const int p_lo = a.window > 0 ? p - a.window + 1 : 0;     // first key it sees

    // queries of this lane's row: the B operand of S^T, kept for the whole item
    const bf16_t* qrow = a.q + ((size_t)(q_tok0 + ti) * a.n_heads + head) * D;
    constexpr bool WIDE = (D % 32 == 0);
    constexpr int QSTEPS = WIDE ? D / 32 : D / 16;
    bf16x8_t q8[WIDE ? QSTEPS : 1];
    bf16x4_t q4[WIDE ? 1 : QSTEPS];
    if constexpr (WIDE) {
#pragma unroll
        for (int s = 0; s < QSTEPS; ++s) { U16 t; t.u = *(const uint4*)(qrow + s * 32 + g * 8); q8[s] = t.v; }
    } else {
#pragma unroll
        for (int s = 0; s < QSTEPS; ++s) { U8 t; t.u = *(const uint2*)(qrow + s * 16 + g * 4); q4[s] = t.v; }
    }

    f32x4_t o[D / 16];
#pragma unroll
    for (int t = 0; t < D / 16; ++t) o[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    const int* bt = a.block_table + (size_t)entry * a.max_blocks;
    for (int j0 = key_lo; j0 < key_hi; j0 += 16) {
        const int blk = j0 / ps;
        int pg = bt[blk];
        if (pg < 0 || pg >= a.num_pages) continue;  // a page the window has passed; its keys are masked for every row
        const int off = j0 - blk * ps;
        const bf16_t* kb = a.k_pages + (((size_t)pg * a.n_kv + kvh) * ps + off + r) * D;
        f32x4_t s = (f32x4_t){0.f, 0.f, 0.f, 0.f};
        if constexpr (WIDE) {
#pragma unroll
            for (int st = 0; st < QSTEPS; ++st) {
                U16 t; t.u = *(const uint4*)(kb + st * 32 + g * 8);
                s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(t.v, q8[st], s, 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int st = 0; st < QSTEPS; ++st) {
                U8 t; t.u = *(const uint2*)(kb + st * 16 + g * 4);
                s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(t.v, q4[st], s, 0, 0, 0);
            }
        }
        // s[i] is key j0 + 4 g + i against row r
        float sv[4];
        bool ok[4];
        float mb = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int j = j0 + 4 * g + i;
            ok[i] = (j <= p) && (j >= p_lo);
            sv[i] = s[i] * a.scale_log2;
            if (ok[i]) mb = fmaxf(mb, sv[i]);
        }
        mb = fmaxf(mb, __shfl_xor(mb, 16, 64));
        mb = fmaxf(mb, __shfl_xor(mb, 32, 64));
        const float m_new = fmaxf(m, mb);
        const float alpha = (m == -INFINITY) ? 0.f : exp2f(m - m_new);
        float pv[4], psum = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            pv[i] = ok[i] ? exp2f(sv[i] - m_new) : 0.f;
            psum += pv[i];
        }
        l = l * alpha + psum;
        m = m_new;
        U8 pf;
        pf.u.x = pack2(pv[0], pv[1]);
        pf.u.y = pack2(pv[2], pv[3]);
        const bf16_t* vb = a.v_pages + (((size_t)pg * a.n_kv + kvh) * D + r) * ps + off + 4 * g;
#pragma unroll
        for (int t = 0; t < D / 16; ++t) {
            U8 vf; vf.u = *(const uint2*)(vb + (size_t)t * 16 * ps);
            o[t] *= alpha;
            o[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf.v, pf.v, o[t], 0, 0, 0);
        }
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);

    if (part < 0) {
        if (!row_ok) return;
        const float inv = l > 0.f ? 1.f / l : 0.f;
        bf16_t* orow = a.out + ((size_t)(q_tok0 + ti) * a.n_heads + head) * D;
#pragma unroll
        for (int t = 0; t < D / 16; ++t) {
            uint2 w;
            w.x = pack2(o[t][0] * inv, o[t][1] * inv);
            w.y = pack2(o[t][2] * inv, o[t][3] * inv);
            *(uint2*)(orow + t * 16 + 4 * g) = w;
        }
    } else {
        if (!row_ok) return;
        const size_t slot = ((size_t)part * a.n_kv + kvh) * 16 + r;
        float* po = a.part_o + slot * D;
#pragma unroll
        for (int t = 0; t < D / 16; ++t) *(f32x4_t*)(po + t * 16 + 4 * g) = o[t];
        if (g == 0) {
            a.part_ml[slot * 2] = m;
            a.part_ml[slot * 2 + 1] = l;
        }
    }
}

// Merge the partial results of a row tile whose keys were split.
// citems: [n][6] = q_tok0, q_len, q_row0, part0, n_parts, unused.  One block per (tile, kv head), 16 rows x D.
template <bool DECODE>
__global__ void attn_combine_kernel(const int* __restrict__ citems, const float* __restrict__ part_o,
                                    const float* __restrict__ part_ml, bf16_t* __restrict__ out, int n_heads, int n_kv,
                                    const int* __restrict__ entry_pos0, const int* __restrict__ dec_params, int p_max,
                                    int window) {
    int q_tok0, q_len, q_row0, part0, n_parts;
    if (DECODE) {
        const int e = blockIdx.x, chunk = dec_params[0], pos0 = entry_pos0[e];
        const int lo = window > 0 ? max(0, pos0 - window + 1) : 0;
        const int p_first = ((lo >> 4) << 4) / chunk, p_last = pos0 / chunk;
        q_tok0 = e; q_len = 1; q_row0 = 0;
        part0 = e * p_max + p_first;
        n_parts = p_last - p_first + 1;
        if (n_parts <= 1) return;   // a single item wrote the output itself
    } else {
        const int* it = citems + (size_t)blockIdx.x * 6;
        q_tok0 = it[0]; q_len = it[1]; q_row0 = it[2]; part0 = it[3]; n_parts = it[4];
        if (n_parts <= 0) return;
    }
    const int kvh = blockIdx.y, G = n_heads / n_kv;
    for (int idx = threadIdx.x; idx < 16 * D; idx += blockDim.x) {
        int r = idx / D, d = idx - r * D;
        int row = q_row0 + r;
        if (row >= q_len * G) continue;
        float mx = -INFINITY;
        for (int pi = 0; pi < n_parts; ++pi)
            mx = fmaxf(mx, part_ml[((((size_t)(part0 + pi)) * n_kv + kvh) * 16 + r) * 2]);
        float num = 0.f, den = 0.f;
        for (int pi = 0; pi < n_parts; ++pi) {
            size_t slot = (((size_t)(part0 + pi)) * n_kv + kvh) * 16 + r;
            float mp = part_ml[slot * 2];
            float w = (mp == -INFINITY) ? 0.f : exp2f(mp - mx);
            num += w * part_o[slot * D + d];
            den += w * part_ml[slot * 2 + 1];
        }
        int ti = row / G, head = kvh * G + (row - ti * G);
        out[((size_t)(q_tok0 + ti) * n_heads + head) * D + d] = f32_to_bf16(den > 0.f ? num / den : 0.f);
    }
}

extern "C" int vt_attn_bf16_head_dim() { return D; }

extern "C" int vt_attn_bf16(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                            const int* items, int n_items, const int* citems, int n_citems, void* out, float* part_o,
                            float* part_ml, int n_heads, int n_kv, int page_size, int max_blocks, int num_pages,
                            int window, float scale, hipStream_t stream) {
    VT_REQUIRE(n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "vt_attn_bf16: bad heads %d/%d", n_heads, n_kv);
    VT_REQUIRE(page_size > 0 && page_size % 16 == 0, "vt_attn_bf16: page size %d is not a multiple of 16", page_size);
    VT_REQUIRE(max_blocks > 0 && num_pages > 0, "vt_attn_bf16: bad cache sizes");
    VT_REQUIRE(n_kv <= 65535, "vt_attn_bf16: too many kv heads (%d)", n_kv);
    VT_REQUIRE(n_citems == 0 || (part_o && part_ml), "vt_attn_bf16: split keys but no workspace");
    if (n_items <= 0) return 0;
    AttnArgs a;
    a.q = (const bf16_t*)q; a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
    a.block_table = block_table; a.items = items; a.out = (bf16_t*)out; a.part_o = part_o; a.part_ml = part_ml;
    a.n_items = n_items; a.n_heads = n_heads; a.n_kv = n_kv; a.page_size = page_size; a.max_blocks = max_blocks;
    a.num_pages = num_pages; a.window = window; a.scale_log2 = scale * 1.4426950408889634f;
    a.entry_pos0 = nullptr; a.dec_params = nullptr; a.p_max = 0;
    attn_bf16_kernel<false><<<dim3((n_items + 3) / 4, n_kv), 256, 0, stream>>>(a);
    VT_CHECK_LAUNCH("vt_attn_bf16");
    if (n_citems > 0) {
        attn_combine_kernel<false><<<dim3(n_citems, n_kv), 256, 0, stream>>>(citems, part_o, part_ml, (bf16_t*)out,
                                                                            n_heads, n_kv, nullptr, nullptr, 0, window);
        VT_CHECK_LAUNCH("vt_attn_bf16(combine)");
    }
    return 0;
}

// Decoding: one token per entry (token i belongs to entry i, at position entry_pos0[i]).  Every entry gets p_max
// items of dec_params[0] keys each; items beyond the entry's keys exit at once.  Nothing here depends on values
// that change between steps except through device memory, so the launches can be captured once and replayed.
// The workspace holds n_entries * p_max partial slots.
extern "C" int vt_attn_bf16_decode(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                                   const int* entry_pos0, const int* dec_params, int n_entries, int p_max, void* out,
                                   float* part_o, float* part_ml, int n_heads, int n_kv, int page_size, int max_blocks,
                                   int num_pages, int window, float scale, hipStream_t stream) {
    VT_REQUIRE(n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "vt_attn_bf16_decode: bad heads %d/%d", n_heads, n_kv);
    VT_REQUIRE(n_heads / n_kv <= 16, "vt_attn_bf16_decode: %d query heads per kv head do not fit one tile of 16 rows",
               n_heads / n_kv);
    VT_REQUIRE(page_size > 0 && page_size % 16 == 0, "vt_attn_bf16_decode: page size %d is not a multiple of 16", page_size);
    VT_REQUIRE(max_blocks > 0 && num_pages > 0 && p_max > 0, "vt_attn_bf16_decode: bad sizes");
    VT_REQUIRE(n_kv <= 65535, "vt_attn_bf16_decode: too many kv heads (%d)", n_kv);
    VT_REQUIRE(part_o && part_ml && entry_pos0 && dec_params, "vt_attn_bf16_decode: missing buffers");
    if (n_entries <= 0) return 0;
    AttnArgs a;
    a.q = (const bf16_t*)q; a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
    a.block_table = block_table; a.items = nullptr; a.out = (bf16_t*)out; a.part_o = part_o; a.part_ml = part_ml;
    a.n_items = n_entries * p_max; a.n_heads = n_heads; a.n_kv = n_kv; a.page_size = page_size; a.max_blocks = max_blocks;
    a.num_pages = num_pages; a.window = window; a.scale_log2 = scale * 1.4426950408889634f;
    a.entry_pos0 = entry_pos0; a.dec_params = dec_params; a.p_max = p_max;
    attn_bf16_kernel<true><<<dim3((a.n_items + 3) / 4, n_kv), 256, 0, stream>>>(a);
    VT_CHECK_LAUNCH("vt_attn_bf16_decode");
    attn_combine_kernel<true><<<dim3(n_entries, n_kv), 256, 0, stream>>>(nullptr, part_o, part_ml, (bf16_t*)out, n_heads,
                                                                        n_kv, entry_pos0, dec_params, p_max, window);
    VT_CHECK_LAUNCH("vt_attn_bf16_decode(combine)");
    return 0;
}
