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
    int ps_shift;           // log2(page_size) if it is a power of two, else -1
};

__device__ __forceinline__ int page_index(const AttnArgs& a, int j) {
    return a.ps_shift >= 0 ? (j >> a.ps_shift) : (j / a.page_size);
}

union U8 { uint2 u; bf16x4_t v; };
union U16 { uint4 u; bf16x8_t v; };

typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;

// two floats to two bf16 (round to nearest even) in one instruction
__device__ __forceinline__ unsigned pack2(float a, float b) {
    f32x2_t v = {a, b};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2_t));
}

// One step of the running softmax of a row over NK*4 scores held by this lane (s[kt][i] = raw dot product of key
// j0 + 16 kt + 4 g + i), shared with the three other lanes of the row.  `full`: every key of the block is visible
// to every row of the tile, so no score is tested.  Leaves the probabilities as bf16 pairs in pk, the factor for
// what was accumulated before in alpha.  Maxima are kept in the exp2 domain (scores times scale*log2 e).
template <int NK>
__device__ __forceinline__ void softmax_step(const f32x4_t (&s)[NK], int j0, int g, int p, int p_lo, bool full,
                                             float scale_log2, float& m, float& l, float& alpha, unsigned (&pk)[NK * 2]) {
    float mb = -INFINITY;
    if (full) {
#pragma unroll
        for (int kt = 0; kt < NK; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) mb = fmaxf(mb, s[kt][i]);
    } else {
#pragma unroll
        for (int kt = 0; kt < NK; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = j0 + 16 * kt + 4 * g + i;
                if (j <= p && j >= p_lo) mb = fmaxf(mb, s[kt][i]);
            }
    }
    mb *= scale_log2;
    mb = fmaxf(mb, __shfl_xor(mb, 16, 64));
    mb = fmaxf(mb, __shfl_xor(mb, 32, 64));
    const float m_new = fmaxf(m, mb);
    alpha = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - m_new);
    float pv[NK][4], psum = 0.f;
#pragma unroll
    for (int kt = 0; kt < NK; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int j = j0 + 16 * kt + 4 * g + i;
            const bool ok = full || (j <= p && j >= p_lo);   // a visible key makes m_new finite
            pv[kt][i] = ok ? __builtin_amdgcn_exp2f(fmaf(s[kt][i], scale_log2, -m_new)) : 0.f;
            psum += pv[kt][i];
        }
    l = l * alpha + psum;
    m = m_new;
#pragma unroll
    for (int kt = 0; kt < NK; ++kt) {
        pk[2 * kt] = pack2(pv[kt][0], pv[kt][1]);
        pk[2 * kt + 1] = pack2(pv[kt][2], pv[kt][3]);
    }
}


constexpr bool WIDE = (D % 32 == 0);           // 16x16x32 instruction for the scores when the head size allows
constexpr int QSTEPS = WIDE ? D / 32 : D / 16;
constexpr int DT = D / 16;

// Keys and values of one block of 16 keys as this lane needs them for the two A operands.
struct KVBlock {
    uint4 k8[WIDE ? QSTEPS : 1];
    uint2 k4[WIDE ? 1 : QSTEPS];
    uint2 v[DT];
    bool ok;
};

// `pg` is the page of the block (read from the block table ahead of time, so that the loads below do not wait for it)
__device__ __forceinline__ void load_block(KVBlock& b, const AttnArgs& a, int pg, int j0, int kvh, int r, int g) {
    const int ps = a.page_size;
    const int blk = page_index(a, j0);
    b.ok = pg >= 0 && pg < a.num_pages;   // a page the window has passed: its keys are masked for every row
    if (!b.ok) return;
    const int off = j0 - blk * ps;
    const bf16_t* kb = a.k_pages + (((size_t)pg * a.n_kv + kvh) * ps + off + r) * D;
    if constexpr (WIDE) {
#pragma unroll
        for (int st = 0; st < QSTEPS; ++st) b.k8[st] = *(const uint4*)(kb + st * 32 + g * 8);
    } else {
#pragma unroll
        for (int st = 0; st < QSTEPS; ++st) b.k4[st] = *(const uint2*)(kb + st * 16 + g * 4);
    }
    const bf16_t* vb = a.v_pages + (((size_t)pg * a.n_kv + kvh) * D + r) * ps + off + 4 * g;
#pragma unroll
    for (int t = 0; t < DT; ++t) b.v[t] = *(const uint2*)(vb + (size_t)t * 16 * ps);
}

// RT row tiles of 16 rows per wave share every key/value block they read.
template <bool DECODE, int RT>
__global__ __launch_bounds__(256) void attn_bf16_kernel(AttnArgs a) {
    const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // decoding: the four waves of a block share one item and take its key blocks in turn; otherwise one item per wave
    const int item = DECODE ? (int)blockIdx.x : (int)blockIdx.x * 4 + wv;
    if (item >= a.n_items) return;
    int entry, q_tok0, q_len, pos0, q_row0, key_lo, key_hi, part;
    if (DECODE) {
        // item = (entry, part p): keys [p*chunk, (p+1)*chunk) of the entry's one token
        const int chunk = a.dec_params[0];
        // Entries vary fastest: consecutive blocks go to different XCDs, and when every entry has one item the
        // blocks that have work are consecutive (with parts fastest they would all land on one XCD in eight).
        const int n_entries = a.n_items / a.p_max;
        const int pi = item / n_entries;
        entry = item - pi * n_entries;
        q_tok0 = entry; q_len = 1; q_row0 = 0;
        pos0 = a.entry_pos0[entry];
        const int lo = a.window > 0 ? max(0, pos0 - a.window + 1) : 0;
        const int p_first = ((lo >> 4) << 4) / chunk, p_last = pos0 / chunk;
        if (pi < p_first || pi > p_last) return;      // the whole block leaves together
        key_lo = max((lo >> 4) << 4, pi * chunk);
        key_hi = min(pos0 + 1, (pi + 1) * chunk);
        part = (p_first == p_last) ? -1 : entry * a.p_max + pi;
    } else {
        const int* it = a.items + (size_t)item * ITEM_INTS;
        entry = it[0]; q_tok0 = it[1]; q_len = it[2]; pos0 = it[3]; q_row0 = it[4];
        key_lo = it[5]; key_hi = it[6]; part = it[7];
        if (entry < 0) return;
    }
    const int kvh = blockIdx.y;
    const int G = a.n_heads / a.n_kv;
    const int r = lane & 15, g = lane >> 4;
    const int n_rows = q_len * G;

    bool row_ok[RT];
    int ti[RT], head[RT], p[RT], p_lo[RT], tile_hi[RT], tile_lo[RT], tile_first_p[RT], tile_last_lo[RT];
    bf16x8_t q8[RT][WIDE ? QSTEPS : 1];
    bf16x4_t q4[RT][WIDE ? 1 : QSTEPS];
    f32x4_t o[RT][DT];
    float m[RT], l[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int row = q_row0 + rt * 16 + r;
        row_ok[rt] = row < n_rows;
        const int rowc = row_ok[rt] ? row : n_rows - 1;
        ti[rt] = rowc / G;
        head[rt] = kvh * G + (rowc - ti[rt] * G);
        p[rt] = pos0 + ti[rt];                                   // this row's position
        p_lo[rt] = a.window > 0 ? p[rt] - a.window + 1 : 0;      // first key it sees
        // keys that any row of the tile may see (the same for every lane)
        const int last_row = min(n_rows - 1, q_row0 + rt * 16 + 15), first_row = min(n_rows - 1, q_row0 + rt * 16);
        tile_hi[rt] = (q_row0 + rt * 16 < n_rows) ? pos0 + last_row / G : -1;
        tile_lo[rt] = a.window > 0 ? pos0 + first_row / G - a.window + 1 : 0;
        // a block whose keys lie between these two is visible to every row of the tile
        tile_first_p[rt] = pos0 + first_row / G;
        tile_last_lo[rt] = a.window > 0 ? pos0 + last_row / G - a.window + 1 : 0;
        const bf16_t* qrow = a.q + ((size_t)(q_tok0 + ti[rt]) * a.n_heads + head[rt]) * D;
        if constexpr (WIDE) {
#pragma unroll
            for (int s = 0; s < QSTEPS; ++s) { U16 t; t.u = *(const uint4*)(qrow + s * 32 + g * 8); q8[rt][s] = t.v; }
        } else {
#pragma unroll
            for (int s = 0; s < QSTEPS; ++s) { U8 t; t.u = *(const uint2*)(qrow + s * 16 + g * 4); q4[rt][s] = t.v; }
        }
#pragma unroll
        for (int t = 0; t < DT; ++t) o[rt][t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
        m[rt] = -INFINITY;
        l[rt] = 0.f;
    }

    // Page ids of up to 64 pages at a time, one per lane: reading the table is then off the path of every block's
    // loads.  (The lane index of a read is the same for the whole wave.)
    const int* bt = a.block_table + (size_t)entry * a.max_blocks;
    const int ps = a.page_size;
    const int last_page = (key_hi - 1) / ps;
    int cache_base = key_lo / ps;
    int pg_lane = (cache_base + lane <= last_page) ? bt[cache_base + lane] : -1;
    auto page_of = [&](int j) {
        int blk = page_index(a, j);
        if (blk >= cache_base + 64) {
            cache_base = blk;
            pg_lane = (cache_base + lane <= last_page) ? bt[cache_base + lane] : -1;
        }
        return __builtin_amdgcn_readlane(pg_lane, __builtin_amdgcn_readfirstlane(blk - cache_base));
    };
    // one block of 16 keys against the RT row tiles of this wave
    auto multiply = [&](const KVBlock& cur, int j0) {
        if (!cur.ok) return;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            if (j0 > tile_hi[rt] || j0 + 15 < tile_lo[rt]) continue;   // every key masked for every row of the tile
            f32x4_t s = (f32x4_t){0.f, 0.f, 0.f, 0.f};
            if constexpr (WIDE) {
#pragma unroll
                for (int st = 0; st < QSTEPS; ++st) {
                    U16 t; t.u = cur.k8[st];
                    s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(t.v, q8[rt][st], s, 0, 0, 0);
                }
            } else {
#pragma unroll
                for (int st = 0; st < QSTEPS; ++st) {
                    U8 t; t.u = cur.k4[st];
                    s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(t.v, q4[rt][st], s, 0, 0, 0);
                }
            }
            // s[i] is key j0 + 4 g + i against row r of the tile
            const f32x4_t sc[1] = {s};
            const bool full = (j0 + 15 <= tile_first_p[rt]) && (j0 >= tile_last_lo[rt]);
            float alpha;
            unsigned pk[2];
            softmax_step<1>(sc, j0, g, p[rt], p_lo[rt], full, a.scale_log2, m[rt], l[rt], alpha, pk);
            U8 pf;
            pf.u.x = pk[0];
            pf.u.y = pk[1];
            const bool rescale = __any(alpha != 1.f);      // the maximum of some row moved
#pragma unroll
            for (int t = 0; t < DT; ++t) {
                U8 vf; vf.u = cur.v[t];
                if (rescale) o[rt][t] *= alpha;
                o[rt][t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf.v, pf.v, o[rt][t], 0, 0, 0);
            }
        }
    };
    // Two register buffers in turn: while one block is multiplied the other one is on its way from memory.
    KVBlock ba, bb;
    ba.ok = bb.ok = false;
    const int j_first = key_lo + (DECODE ? 16 * wv : 0), j_step = DECODE ? 64 : 16;
    if (j_first < key_hi) load_block(ba, a, page_of(j_first), j_first, kvh, r, g);
    for (int j0 = j_first; j0 < key_hi; j0 += 2 * j_step) {
        const int j1 = j0 + j_step, j2 = j0 + 2 * j_step;
        if (j1 < key_hi) load_block(bb, a, page_of(j1), j1, kvh, r, g);
        multiply(ba, j0);
        if (j2 < key_hi) load_block(ba, a, page_of(j2), j2, kvh, r, g);
        if (j1 < key_hi) multiply(bb, j1);
    }

    if constexpr (DECODE) {
        // The four waves hold partial results over disjoint keys of the same rows: merge them through LDS, half
        // of a large head at a time, and let all 256 threads write the result.
        constexpr int DH = (D > 128) ? D / 2 : D;
        __shared__ __attribute__((aligned(16))) float so[4][16][DH + 4];
        __shared__ float sm[4][16], sl[4][16];
        float lt = l[0];
        lt += __shfl_xor(lt, 16, 64);
        lt += __shfl_xor(lt, 32, 64);
        if (g == 0) { sm[wv][r] = m[0]; sl[wv][r] = lt; }
        const int n_valid = min(16, n_rows);
#pragma unroll
        for (int half = 0; half < D / DH; ++half) {
            if (half) __syncthreads();
#pragma unroll
            for (int t = 0; t < DH / 16; ++t) *(f32x4_t*)&so[wv][r][t * 16 + 4 * g] = o[0][half * (DH / 16) + t];
            __syncthreads();
            for (int idx = threadIdx.x; idx < n_valid * DH; idx += 256) {
                const int rr = idx / DH, dd = idx - rr * DH;
                const float mx = fmaxf(fmaxf(sm[0][rr], sm[1][rr]), fmaxf(sm[2][rr], sm[3][rr]));
                float num = 0.f, den = 0.f;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const float wt = (sm[w][rr] == -INFINITY) ? 0.f : exp2f(sm[w][rr] - mx);
                    num += wt * so[w][rr][dd];
                    den += wt * sl[w][rr];
                }
                const int d = half * DH + dd;
                if (part < 0) {
                    const int head_r = kvh * G + rr;      // one token per entry: row = head of the group
                    a.out[((size_t)q_tok0 * a.n_heads + head_r) * D + d] = f32_to_bf16(den > 0.f ? num / den : 0.f);
                } else {
                    const size_t slot = ((size_t)part * a.n_kv + kvh) * 16 + rr;
                    a.part_o[slot * D + d] = num;
                    if (d == 0) { a.part_ml[slot * 2] = mx; a.part_ml[slot * 2 + 1] = den; }
                }
            }
        }
        return;
    }

#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        float lt = l[rt];
        lt += __shfl_xor(lt, 16, 64);
        lt += __shfl_xor(lt, 32, 64);
        if (!row_ok[rt]) continue;
        if (part < 0) {
            const float inv = lt > 0.f ? 1.f / lt : 0.f;
            bf16_t* orow = a.out + ((size_t)(q_tok0 + ti[rt]) * a.n_heads + head[rt]) * D;
#pragma unroll
            for (int t = 0; t < DT; ++t) {
                uint2 w;
                w.x = pack2(o[rt][t][0] * inv, o[rt][t][1] * inv);
                w.y = pack2(o[rt][t][2] * inv, o[rt][t][3] * inv);
                *(uint2*)(orow + t * 16 + 4 * g) = w;
            }
        } else {
            // partial slots of an item: RT consecutive tiles of 16 rows
            const size_t slot = (((size_t)part * RT + rt) * a.n_kv + kvh) * 16 + r;
            float* po = a.part_o + slot * D;
#pragma unroll
            for (int t = 0; t < DT; ++t) *(f32x4_t*)(po + t * 16 + 4 * g) = o[rt][t];
            if (g == 0) {
                a.part_ml[slot * 2] = m[rt];
                a.part_ml[slot * 2 + 1] = lt;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Long portions of prompts: a block of 4 waves takes 64 * RT consecutive rows of one (entry, kv head) and walks
// their keys KB at a time.  Every key/value block is fetched from the pages once per block of waves, by all 256
// threads together with 16-byte loads, and parked in LDS (two buffers: the next block is on its way from memory
// while this one is multiplied); the four waves read their matrix operands from there.  Rows of an item that lie
// wholly above a key block skip it (the upper triangle of a causal portion costs nothing).
// ---------------------------------------------------------------------------
constexpr int KB = (D > 128) ? 16 : 32;        // keys per block
constexpr int KT = KB / 16;                    // score tiles per block
constexpr int KROW = D + 8;                    // padded rows: operand reads from LDS without bank conflicts
constexpr int VROW = KB + 8;
constexpr int KPIECES = KB * (D / 8);          // 16-byte pieces of a key block
constexpr int VPIECES = D * (KB / 8);
constexpr int KPT = (KPIECES + 255) / 256;     // pieces per thread
constexpr int VPT = (VPIECES + 255) / 256;
constexpr int PAGE_WINDOW = 256;               // page ids kept in LDS at a time

template <int RT>
__global__ __launch_bounds__(256) void attn_bf16_tile_kernel(AttnArgs a) {
    __shared__ __attribute__((aligned(16))) bf16_t k_lds[2][KB][KROW];
    __shared__ __attribute__((aligned(16))) bf16_t v_lds[2][D][VROW];
    __shared__ int s_pages[PAGE_WINDOW];
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
    const int* it = a.items + (size_t)blockIdx.x * ITEM_INTS;
    const int entry = it[0], q_tok0 = it[1], q_len = it[2], pos0 = it[3], q_row0 = it[4];
    const int key_lo = it[5], key_hi = it[6];
    if (entry < 0) return;
    const int kvh = blockIdx.y;
    const int G = a.n_heads / a.n_kv;
    const int r = lane & 15, g = lane >> 4;
    const int n_rows = q_len * G;
    const int ps = a.page_size;

    bool row_ok[RT];
    int ti[RT], head[RT], p[RT], p_lo[RT], tile_hi[RT], tile_lo[RT], tile_first_p[RT], tile_last_lo[RT];
    bf16x8_t q8[RT][WIDE ? QSTEPS : 1];
    bf16x4_t q4[RT][WIDE ? 1 : QSTEPS];
    f32x4_t o[RT][DT];
    float m[RT], l[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int row0 = q_row0 + (wv * RT + rt) * 16;
        const int row = row0 + r;
        row_ok[rt] = row < n_rows;
        const int rowc = row_ok[rt] ? row : n_rows - 1;
        ti[rt] = rowc / G;
        head[rt] = kvh * G + (rowc - ti[rt] * G);
        p[rt] = pos0 + ti[rt];
        p_lo[rt] = a.window > 0 ? p[rt] - a.window + 1 : 0;
        const int last_row = min(n_rows - 1, row0 + 15), first_row = min(n_rows - 1, row0);
        tile_hi[rt] = (row0 < n_rows) ? pos0 + last_row / G : -1;
        tile_lo[rt] = a.window > 0 ? pos0 + first_row / G - a.window + 1 : 0;
        tile_first_p[rt] = pos0 + first_row / G;
        tile_last_lo[rt] = a.window > 0 ? pos0 + last_row / G - a.window + 1 : 0;
        const bf16_t* qrow = a.q + ((size_t)(q_tok0 + ti[rt]) * a.n_heads + head[rt]) * D;
        if constexpr (WIDE) {
#pragma unroll
            for (int s = 0; s < QSTEPS; ++s) { U16 t; t.u = *(const uint4*)(qrow + s * 32 + g * 8); q8[rt][s] = t.v; }
        } else {
#pragma unroll
            for (int s = 0; s < QSTEPS; ++s) { U8 t; t.u = *(const uint2*)(qrow + s * 16 + g * 4); q4[rt][s] = t.v; }
        }
#pragma unroll
        for (int t = 0; t < DT; ++t) o[rt][t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
        m[rt] = -INFINITY;
        l[rt] = 0.f;
    }

    const int* bt = a.block_table + (size_t)entry * a.max_blocks;
    const int last_page = (key_hi - 1) / ps;
    int page_base = key_lo / ps;
    auto fill_pages = [&]() {   // all threads; callers put barriers around it
        const int pgi = page_base + tid;
        if (tid < PAGE_WINDOW) s_pages[tid] = (pgi <= last_page) ? bt[pgi] : -1;
    };
    struct Stage { uint4 k[KPT]; uint4 v[VPT]; };
    auto fetch = [&](Stage& st_, int j0) {   // this thread's pieces of keys [j0, j0 + KB) from the pages into registers
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            const int idx = tid + 256 * i;
            st_.k[i] = make_uint4(0, 0, 0, 0);
            if (idx < KPIECES) {
                const int key = idx / (D / 8), c = idx - key * (D / 8);
                const int j = j0 + key;
                const int blk = page_index(a, j);
                const int pg = (j < key_hi) ? s_pages[blk - page_base] : -1;
                if (pg >= 0 && pg < a.num_pages)
                    st_.k[i] = *(const uint4*)(a.k_pages + (((size_t)pg * a.n_kv + kvh) * ps + (j - blk * ps)) * D + c * 8);
            }
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int idx = tid + 256 * i;
            st_.v[i] = make_uint4(0, 0, 0, 0);
            if (idx < VPIECES) {
                const int d = idx / (KB / 8), kg = idx - d * (KB / 8);
                const int j = j0 + kg * 8;
                const int blk = page_index(a, j);
                const int pg = (j < key_hi) ? s_pages[blk - page_base] : -1;
                if (pg >= 0 && pg < a.num_pages)
                    st_.v[i] = *(const uint4*)(a.v_pages + (((size_t)pg * a.n_kv + kvh) * D + d) * ps + (j - blk * ps));
            }
        }
    };
    auto park = [&](const Stage& st_, int buf) {
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            const int idx = tid + 256 * i;
            if (idx < KPIECES) {
                const int key = idx / (D / 8), c = idx - key * (D / 8);
                *(uint4*)&k_lds[buf][key][c * 8] = st_.k[i];
            }
        }
#pragma unroll
        for (int i = 0; i < VPT; ++i) {
            const int idx = tid + 256 * i;
            if (idx < VPIECES) {
                const int d = idx / (KB / 8), kg = idx - d * (KB / 8);
                *(uint4*)&v_lds[buf][d][kg * 8] = st_.v[i];
            }
        }
    };

    // one key block (in LDS buffer `buf`, keys from j0) against the RT row tiles of this wave
    auto multiply = [&](int buf, int j0) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            if (j0 > tile_hi[rt] || j0 + KB - 1 < tile_lo[rt]) continue;   // every key masked for every row of the tile
            f32x4_t s[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                s[kt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
                const bf16_t* kr = &k_lds[buf][kt * 16 + r][0];
                if constexpr (WIDE) {
#pragma unroll
                    for (int st = 0; st < QSTEPS; ++st) {
                        U16 t; t.u = *(const uint4*)(kr + st * 32 + g * 8);
                        s[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(t.v, q8[rt][st], s[kt], 0, 0, 0);
                    }
                } else {
#pragma unroll
                    for (int st = 0; st < QSTEPS; ++st) {
                        U8 t; t.u = *(const uint2*)(kr + st * 16 + g * 4);
                        s[kt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(t.v, q4[rt][st], s[kt], 0, 0, 0);
                    }
                }
            }
            // s[kt][i] is key j0 + 16 kt + 4 g + i against row r of the tile
            const bool full = (j0 + KB - 1 <= tile_first_p[rt]) && (j0 >= tile_last_lo[rt]);
            float alpha;
            unsigned pk[KT * 2];
            softmax_step<KT>(s, j0, g, p[rt], p_lo[rt], full, a.scale_log2, m[rt], l[rt], alpha, pk);
            const bool rescale = __any(alpha != 1.f);      // the maximum of some row moved
            if constexpr (KT == 2) {
                // one 16x16x32 instruction per 16 dims: its 8 k slots of lane group g are keys 4g..4g+3 of the
                // first score tile and of the second
                U16 pf;
                pf.u = make_uint4(pk[0], pk[1], pk[2], pk[3]);
#pragma unroll
                for (int t = 0; t < DT; ++t) {
                    const bf16_t* vr = &v_lds[buf][t * 16 + r][4 * g];
                    U16 vf;
                    uint2 lo = *(const uint2*)vr, hi = *(const uint2*)(vr + 16);
                    vf.u = make_uint4(lo.x, lo.y, hi.x, hi.y);
                    if (rescale) o[rt][t] *= alpha;
                    o[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf.v, o[rt][t], 0, 0, 0);
                }
            } else {
                U8 pf;
                pf.u.x = pk[0]; pf.u.y = pk[1];
#pragma unroll
                for (int t = 0; t < DT; ++t) {
                    U8 vf; vf.u = *(const uint2*)&v_lds[buf][t * 16 + r][4 * g];
                    if (rescale) o[rt][t] *= alpha;
                    o[rt][t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf.v, pf.v, o[rt][t], 0, 0, 0);
                }
            }
        }
    };
    auto window_for = [&](int j) {   // make sure the page ids of block j are in LDS (the same decision in every thread)
        if (page_index(a, j + KB - 1) >= page_base + PAGE_WINDOW) {
            __syncthreads();
            page_base = page_index(a, j);
            fill_pages();
            __syncthreads();
        }
    };

    // Two sets of staging registers and two LDS buffers: a block is fetched two steps before it is multiplied, so
    // its loads have two multiplications' time to arrive.
    Stage sa, sb;
    fill_pages();
    __syncthreads();
    fetch(sa, key_lo);
    if (key_lo + KB < key_hi) { window_for(key_lo + KB); fetch(sb, key_lo + KB); }
    park(sa, 0);
    __syncthreads();
    for (int j0 = key_lo; j0 < key_hi; j0 += 2 * KB) {
        const int j1 = j0 + KB, j2 = j0 + 2 * KB, j3 = j0 + 3 * KB;
        if (j2 < key_hi) { window_for(j2); fetch(sa, j2); }
        multiply(0, j0);
        if (j1 < key_hi) park(sb, 1);
        __syncthreads();
        if (j1 >= key_hi) break;
        if (j3 < key_hi) { window_for(j3); fetch(sb, j3); }
        multiply(1, j1);
        if (j2 < key_hi) park(sa, 0);
        __syncthreads();
    }

#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        float lt = l[rt];
        lt += __shfl_xor(lt, 16, 64);
        lt += __shfl_xor(lt, 32, 64);
        if (!row_ok[rt]) continue;
        const float inv = lt > 0.f ? 1.f / lt : 0.f;
        bf16_t* orow = a.out + ((size_t)(q_tok0 + ti[rt]) * a.n_heads + head[rt]) * D;
#pragma unroll
        for (int t = 0; t < DT; ++t) {
            uint2 w;
            w.x = pack2(o[rt][t][0] * inv, o[rt][t][1] * inv);
            w.y = pack2(o[rt][t][2] * inv, o[rt][t][3] * inv);
            *(uint2*)(orow + t * 16 + 4 * g) = w;
        }
    }
}

// Merge the partial results of a tile of 16 rows whose keys were split over several items.
// citems: [n][6] = q_tok0, q_len, first row of the tile, first item's partial index, number of items, tile index
// within its items (each item holds `rt_per_item` tiles).  One block per (tile, kv head).
#define MAX_PARTS 128
template <bool DECODE>
__global__ __launch_bounds__(256) void attn_combine_kernel(const int* __restrict__ citems, const float* __restrict__ part_o,
                                                          const float* __restrict__ part_ml, bf16_t* __restrict__ out,
                                                          int n_heads, int n_kv, const int* __restrict__ entry_pos0,
                                                          const int* __restrict__ dec_params, int p_max, int window,
                                                          int rt_per_item) {
    __shared__ float sm[MAX_PARTS][16];   // m of (part, row), then the row's normalised weight of the part
    __shared__ float sl[MAX_PARTS][16];
    int q_tok0, q_len, q_row0, part0, n_parts, rt;
    if (DECODE) {
        const int e = blockIdx.x, chunk = dec_params[0], pos0 = entry_pos0[e];
        const int lo = window > 0 ? max(0, pos0 - window + 1) : 0;
        const int p_first = ((lo >> 4) << 4) / chunk, p_last = pos0 / chunk;
        q_tok0 = e; q_len = 1; q_row0 = 0; rt = 0;
        part0 = e * p_max + p_first;
        n_parts = p_last - p_first + 1;
        if (n_parts <= 1) return;   // a single item wrote the output itself
    } else {
        const int* it = citems + (size_t)blockIdx.x * 6;
        q_tok0 = it[0]; q_len = it[1]; q_row0 = it[2]; part0 = it[3]; n_parts = it[4]; rt = it[5];
        if (n_parts <= 0) return;
    }
    n_parts = min(n_parts, MAX_PARTS);   // the host never plans more
    const int kvh = blockIdx.y, G = n_heads / n_kv, tid = threadIdx.x;
    const int n_valid = min(16, q_len * G - q_row0);
    // slot of (part pi, row r) = (((part0 + pi) * rt_per_item + rt) * n_kv + kvh) * 16 + r
    const size_t slot0 = (((size_t)part0 * rt_per_item + rt) * n_kv + kvh) * 16;
    const size_t slot_step = (size_t)rt_per_item * n_kv * 16;
    for (int i = tid; i < n_parts * 16; i += 256) {
        const int pi = i >> 4, r = i & 15;
        const size_t sl_ = slot0 + pi * slot_step + r;
        const bool ok = r < n_valid;
        sm[pi][r] = ok ? part_ml[sl_ * 2] : -INFINITY;
        sl[pi][r] = ok ? part_ml[sl_ * 2 + 1] : 0.f;
    }
    __syncthreads();
    if (tid < 16) {
        float mx = -INFINITY;
        for (int pi = 0; pi < n_parts; ++pi) mx = fmaxf(mx, sm[pi][tid]);
        float den = 0.f;
        for (int pi = 0; pi < n_parts; ++pi) {
            const float w = (sm[pi][tid] == -INFINITY) ? 0.f : exp2f(sm[pi][tid] - mx);
            den += w * sl[pi][tid];
            sm[pi][tid] = w;
        }
        const float inv = den > 0.f ? 1.f / den : 0.f;
        for (int pi = 0; pi < n_parts; ++pi) sm[pi][tid] *= inv;
    }
    __syncthreads();
    for (int idx = tid; idx < n_valid * D; idx += 256) {
        const int r = idx / D, d = idx - r * D;
        const float* po = part_o + (slot0 + r) * D + d;
        float acc = 0.f;
#pragma unroll 4
        for (int pi = 0; pi < n_parts; ++pi) acc += sm[pi][r] * po[(size_t)pi * slot_step * D];
        const int row = q_row0 + r;
        const int ti = row / G, head = kvh * G + (row - ti * G);
        out[((size_t)(q_tok0 + ti) * n_heads + head) * D + d] = f32_to_bf16(acc);
    }
}

extern "C" int vt_attn_bf16_head_dim() { return D; }

static int shift_of(int v) {
    for (int sft = 0; sft < 31; ++sft)
        if ((1 << sft) == v) return sft;
    return -1;
}

static int check_common(const char* who, int n_heads, int n_kv, int page_size, int max_blocks, int num_pages) {
    VT_REQUIRE(n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "%s: bad heads %d/%d", who, n_heads, n_kv);
    VT_REQUIRE(page_size > 0 && page_size % 16 == 0, "%s: page size %d is not a multiple of 16", who, page_size);
    VT_REQUIRE(max_blocks > 0 && num_pages > 0, "%s: bad cache sizes", who);
    VT_REQUIRE(n_kv <= 65535, "%s: too many kv heads (%d)", who, n_kv);
    return 0;
}

// items: [n_items][8] = entry, q_tok0, q_len, pos0, first row, key_lo, key_hi, partial index (-1: writes the output).
// Each item covers 16 * rt rows (rt = 1 or 2).  The partial workspace holds (partial indices) * rt * n_kv * 16 rows.
extern "C" int vt_attn_bf16(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                            const int* items, int n_items, int rt, const int* citems, int n_citems, void* out,
                            float* part_o, float* part_ml, int n_heads, int n_kv, int page_size, int max_blocks,
                            int num_pages, int window, float scale, hipStream_t stream) {
    if (check_common("vt_attn_bf16", n_heads, n_kv, page_size, max_blocks, num_pages)) return -1;
    VT_REQUIRE(rt == 1 || rt == 2, "vt_attn_bf16: %d row tiles per item (1 or 2)", rt);
    VT_REQUIRE(n_citems == 0 || (part_o && part_ml), "vt_attn_bf16: split keys but no workspace");
    if (n_items <= 0) return 0;
    AttnArgs a;
    a.q = (const bf16_t*)q; a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
    a.block_table = block_table; a.items = items; a.out = (bf16_t*)out; a.part_o = part_o; a.part_ml = part_ml;
    a.n_items = n_items; a.n_heads = n_heads; a.n_kv = n_kv; a.page_size = page_size; a.max_blocks = max_blocks;
    a.num_pages = num_pages; a.window = window; a.scale_log2 = scale * 1.4426950408889634f;
    a.entry_pos0 = nullptr; a.dec_params = nullptr; a.p_max = 0; a.ps_shift = shift_of(page_size);
    dim3 grid((n_items + 3) / 4, n_kv);
    if (rt == 1) attn_bf16_kernel<false, 1><<<grid, 256, 0, stream>>>(a);
    else attn_bf16_kernel<false, 2><<<grid, 256, 0, stream>>>(a);
    VT_CHECK_LAUNCH("vt_attn_bf16");
    if (n_citems > 0) {
        attn_combine_kernel<false><<<dim3(n_citems, n_kv), 256, 0, stream>>>(citems, part_o, part_ml, (bf16_t*)out,
                                                                            n_heads, n_kv, nullptr, nullptr, 0, window, rt);
        VT_CHECK_LAUNCH("vt_attn_bf16(combine)");
    }
    return 0;
}

// Long portions: items [n][8] as above, each 64 * rt rows (rt = 1 or 2) of one entry with all the keys they may
// see (no split, the partial index is not used); one block of 4 waves per (item, kv head).
extern "C" int vt_attn_bf16_tiles(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                                  const int* items, int n_items, int rt, void* out, int n_heads, int n_kv, int page_size,
                                  int max_blocks, int num_pages, int window, float scale, hipStream_t stream) {
    if (check_common("vt_attn_bf16_tiles", n_heads, n_kv, page_size, max_blocks, num_pages)) return -1;
    VT_REQUIRE(rt == 1 || rt == 2, "vt_attn_bf16_tiles: %d row tiles per wave (1 or 2)", rt);
    if (n_items <= 0) return 0;
    AttnArgs a;
    a.q = (const bf16_t*)q; a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
    a.block_table = block_table; a.items = items; a.out = (bf16_t*)out; a.part_o = nullptr; a.part_ml = nullptr;
    a.n_items = n_items; a.n_heads = n_heads; a.n_kv = n_kv; a.page_size = page_size; a.max_blocks = max_blocks;
    a.num_pages = num_pages; a.window = window; a.scale_log2 = scale * 1.4426950408889634f;
    a.entry_pos0 = nullptr; a.dec_params = nullptr; a.p_max = 0; a.ps_shift = shift_of(page_size);
    dim3 grid(n_items, n_kv);
    if (rt == 1) attn_bf16_tile_kernel<1><<<grid, 256, 0, stream>>>(a);
    else attn_bf16_tile_kernel<2><<<grid, 256, 0, stream>>>(a);
    VT_CHECK_LAUNCH("vt_attn_bf16_tiles");
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
    if (check_common("vt_attn_bf16_decode", n_heads, n_kv, page_size, max_blocks, num_pages)) return -1;
    VT_REQUIRE(n_heads / n_kv <= 16, "vt_attn_bf16_decode: %d query heads per kv head do not fit one tile of 16 rows",
               n_heads / n_kv);
    VT_REQUIRE(p_max > 0 && p_max <= MAX_PARTS, "vt_attn_bf16_decode: %d items per entry (1..%d)", p_max, MAX_PARTS);
    VT_REQUIRE(part_o && part_ml && entry_pos0 && dec_params, "vt_attn_bf16_decode: missing buffers");
    if (n_entries <= 0) return 0;
    AttnArgs a;
    a.q = (const bf16_t*)q; a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
    a.block_table = block_table; a.items = nullptr; a.out = (bf16_t*)out; a.part_o = part_o; a.part_ml = part_ml;
    a.n_items = n_entries * p_max; a.n_heads = n_heads; a.n_kv = n_kv; a.page_size = page_size; a.max_blocks = max_blocks;
    a.num_pages = num_pages; a.window = window; a.scale_log2 = scale * 1.4426950408889634f;
    a.entry_pos0 = entry_pos0; a.dec_params = dec_params; a.p_max = p_max; a.ps_shift = shift_of(page_size);
    attn_bf16_kernel<true, 1><<<dim3(a.n_items, n_kv), 256, 0, stream>>>(a);
    VT_CHECK_LAUNCH("vt_attn_bf16_decode");
    attn_combine_kernel<true><<<dim3(n_entries, n_kv), 256, 0, stream>>>(nullptr, part_o, part_ml, (bf16_t*)out, n_heads,
                                                                        n_kv, entry_pos0, dec_params, p_max, window, 1);
    VT_CHECK_LAUNCH("vt_attn_bf16_decode(combine)");
    return 0;
}
