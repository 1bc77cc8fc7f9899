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

typedef vt_lowp8_t bf16x8_t;
typedef vt_lowp4_t bf16x4_t;
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
    // fused decode: the projections' output comes in unrotated and in fp32; the kernel rotates queries and the new
    // key itself and writes the new key and value into their page
    const float* qkv;       // [entries][qkv_stride]: queries of all heads, then keys, then values; or null
    long long qkv_stride;
    const float* cos_t;     // [max_pos][rot / 2]
    const float* sin_t;
    int rot, max_pos;       // rotated dims of a head (a multiple of 16, or 0)
};

__device__ __forceinline__ int page_index(const AttnArgs& a, int j) {
    return a.ps_shift >= 0 ? (j >> a.ps_shift) : (j / a.page_size);
}

union U8 { uint2 u; bf16x4_t v; };
union U16 { uint4 u; bf16x8_t v; };

// two floats to two 16-bit values (round to nearest even) in one instruction
__device__ __forceinline__ unsigned pack2(float a, float b) { return vt_pack2(a, b); }

// Maximum over the four lanes that share a row (lane % 16): two register swaps between rows of 16 and halves of 32
// lanes, which stay in the vector unit (a shuffle would go through the LDS crossbar).
typedef __attribute__((ext_vector_type(2))) unsigned u32x2_t;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4_t;
__device__ __forceinline__ float row_max4(float v) {
    const unsigned u = __float_as_uint(v);
    const u32x2_t a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const unsigned a0 = a.x, a1 = a.y;     // copies: a bit cast of a vector element reads the wrong one
    const unsigned x = __float_as_uint(fmaxf(__uint_as_float(a0), __uint_as_float(a1)));
    const u32x2_t b = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    const unsigned b0 = b.x, b1 = b.y;
    return fmaxf(__uint_as_float(b0), __uint_as_float(b1));
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
    mb = row_max4(mb * scale_log2);
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

// Keys and values of one block of 16 keys as they lie in their page: the keys are 16 D consecutive elements, the
// values 16 consecutive elements of each of D rows; lane l holds the 16-byte pieces l, l + 64, ... of each.  Read as
// the matrix instruction wants its operands (lane 16 g + r: key r or dim r, piece g) the four pieces of a row would
// sit in lanes 16 apart and every lane's load would be a cache access of its own; in this order a load of the wave
// is whole cache lines, and the pieces reach the lanes that need them through an LDS buffer of the wave
// (KV_LDS_ELEMS elements: keys [16][D + 8], values [D][24]).
constexpr int KVP = (2 * D + 63) / 64;            // pieces per lane, of the keys and of the values
constexpr int KL_ROW = D + 8, VL_ROW = 24;        // padded LDS rows: operand reads without bank conflicts

// With a head of 128 the key/value blocks go from the pages straight into LDS (global_load_lds, 16 bytes per lane):
// no registers hold them on the way and no thread stores them.  A wave's load writes 64 consecutive 16-byte slots
// of LDS, one per lane, and each lane chooses what it reads from memory, so the layout is made by the choice of
// addresses: a key row is 16 slots, and chunk c (8 dims) of LDS row p sits in slot c ^ (p % 16) of the row, so that
// the sixteen rows of a score tile are read from sixteen different slots modulo 16 (no bank conflicts, no padding);
// the values of a group of 16 keys are [tile of 16 dims][8 keys of 16][dim of the tile], 16 bytes each.
constexpr bool DIRECT = (D == 128);
// (direct: two buffers per wave of 16 keys and their values as they come, the next block but one is on its way
// while a block is multiplied)
constexpr int WAVE_BUFS = DIRECT ? 2 : 1;
constexpr int KV_BUF_ELEMS = DIRECT ? 2 * 16 * D : 16 * KL_ROW + D * VL_ROW;
constexpr int KV_LDS_ELEMS = WAVE_BUFS * KV_BUF_ELEMS;
struct KVBlock {
    u32x4_t k[KVP], v[KVP];
    bool ok;
};

// `pg` is the page of the block (read from the block table ahead of time, so that the loads below do not wait for
// it).  Nothing is tested before the loads: a block without a page (a window has passed it: its keys are masked for
// every row) reads `spare`, a page that exists, and is marked so that it is not multiplied.  Loads under a branch
// would make every later use wait for all the loads in flight.
// ONCE: no other wave of the launch reads this block (decoding: one wave takes all query heads of a kv head over a
// range of keys), so the loads are marked non-temporal, which the memory serves about a tenth faster.
template <bool ONCE>
__device__ __forceinline__ void load_block(KVBlock& b, const AttnArgs& a, int pg, int spare, int j0, int kvh, int lane) {
    const int ps = a.page_size;
    const int blk = page_index(a, j0);
    b.ok = pg >= 0 && pg < a.num_pages;
    const int pgc = b.ok ? pg : spare;
    const int off = j0 - blk * ps;
    const bf16_t* kb = a.k_pages + (((size_t)pgc * a.n_kv + kvh) * ps + off) * D;
    const bf16_t* vb = a.v_pages + ((size_t)pgc * a.n_kv + kvh) * D * ps + off;
#pragma unroll
    for (int i = 0; i < KVP; ++i) {
        const int x = min(lane + 64 * i, 2 * D - 1);
        if constexpr (ONCE) {
            b.k[i] = __builtin_nontemporal_load((const u32x4_t*)(kb + x * 8));
            b.v[i] = __builtin_nontemporal_load((const u32x4_t*)(vb + (size_t)(x >> 1) * ps + (x & 1) * 8));
        } else {
            b.k[i] = *(const u32x4_t*)(kb + x * 8);
            b.v[i] = *(const u32x4_t*)(vb + (size_t)(x >> 1) * ps + (x & 1) * 8);
        }
    }
}

// the pieces of a block into the wave's LDS buffer, where the operands are read from
__device__ __forceinline__ void park_block(const KVBlock& b, bf16_t* kl, int lane) {
    bf16_t* vl = kl + 16 * KL_ROW;
#pragma unroll
    for (int i = 0; i < KVP; ++i) {
        const int x = lane + 64 * i;
        if (2 * D % 64 == 0 || x < 2 * D) {
            const int key = x / (D / 8), c = x - key * (D / 8);
            *(u32x4_t*)(kl + key * KL_ROW + c * 8) = b.k[i];
            *(u32x4_t*)(vl + (x >> 1) * VL_ROW + (x & 1) * 8) = b.v[i];
        }
    }
}

// CH consecutive elements (from c, a multiple of CH) of a head as the projection left them in fp32, rotated: the
// pairs are (i, i + rot/2) for i < rot/2, elements from rot on pass through; rot is a multiple of 2 CH.  The same
// arithmetic as the separate rotation kernel (vt_rope_store).  In two steps (loads, then arithmetic), so that the
// loads of several chunks are in flight together: the compiler keeps a chunk's loads next to its arithmetic, and a
// row's chunks then wait for memory one after the other.
template <int CH>
struct RotIn {
    float4 x[CH / 4], y[CH / 4], c[CH / 4], s[CH / 4];
    bool in, low;
};
template <int CH>
__device__ __forceinline__ void rot_load(RotIn<CH>& r, const float* row, int c, int rot, const float* cos_t,
                                         const float* sin_t, int pos, int max_pos) {
    // nothing here sits under a test: a chunk outside the rotary dims (all of them if there are none) reads its own
    // elements again in place of a partner and of table entries, and drops them
    const int half = rot >> 1;
    r.in = c < rot;
    r.low = c < half;
    const int tp = pos < max_pos ? (pos < 0 ? 0 : pos) : max_pos - 1;
    const int ti = r.low ? c : c - half;
    const float* ct = r.in ? cos_t + (size_t)tp * half + ti : row + c;
    const float* st = r.in ? sin_t + (size_t)tp * half + ti : row + c;
    const float* other = row + (r.in ? (r.low ? c + half : c - half) : c);
#pragma unroll
    for (int i = 0; i < CH / 4; ++i) {
        r.x[i] = *(const float4*)(row + c + 4 * i);
        r.y[i] = *(const float4*)(other + 4 * i);
        r.c[i] = *(const float4*)(ct + 4 * i);
        r.s[i] = *(const float4*)(st + 4 * i);
    }
}
template <int CH>
__device__ __forceinline__ void rot_apply(float (&x)[CH], const RotIn<CH>& r) {
#pragma unroll
    for (int i = 0; i < CH / 4; ++i) {
        const float4 v = r.x[i], y = r.y[i], cc = r.c[i], sn = r.s[i];
        x[4 * i] = r.in ? rotate_pair(cc.x, sn.x, v.x, y.x, r.low) : v.x;
        x[4 * i + 1] = r.in ? rotate_pair(cc.y, sn.y, v.y, y.y, r.low) : v.y;
        x[4 * i + 2] = r.in ? rotate_pair(cc.z, sn.z, v.z, y.z, r.low) : v.z;
        x[4 * i + 3] = r.in ? rotate_pair(cc.w, sn.w, v.w, y.w, r.low) : v.w;
    }
}

// Merge the partial results of a tile of 16 rows whose keys were split over n_parts items; all 256 threads of a
// block.  sm and sl are [MAX_PARTS][16] floats of LDS.  Slot of (part pi, row r) = slot0 + pi * slot_step + r.
#define MAX_PARTS 128
__device__ __forceinline__ void merge_parts(float (*sm)[16], float (*sl)[16], const float* __restrict__ part_o,
                                            const float* __restrict__ part_ml, bf16_t* __restrict__ out, size_t slot0,
                                            size_t slot_step, int n_parts, int n_valid,
                                            int q_tok0, int q_row0, int G, int kvh, int n_heads) {
    const int tid = threadIdx.x;
    // With few rows and parts (decoding) a thread's share of the partial outputs is on its way from memory while
    // the weights of the parts are worked out, instead of being asked for only after them.
    constexpr int PRE = 16, Q = D / 4;
    const bool pre = n_valid * Q <= 256 && n_parts <= PRE;
    const int pr = tid / Q, pd = (tid - pr * Q) * 4;
    f32x4_t pv[PRE];
    if (pre && tid < n_valid * Q) {
        const float* po = part_o + (slot0 + pr) * D + pd;
#pragma unroll
        for (int pi = 0; pi < PRE; ++pi)
            if (pi < n_parts) pv[pi] = *(const f32x4_t*)(po + (size_t)pi * slot_step * D);
    }
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
    if (pre) {
        if (tid < n_valid * Q) {
            f32x4_t acc = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int pi = 0; pi < PRE; ++pi)
                if (pi < n_parts) acc += sm[pi][pr] * pv[pi];     // parts in order, as below
            const int row = q_row0 + pr;
            const int ti = row / G, head = kvh * G + (row - ti * G);
            uint2 w;
            w.x = pack2(acc[0], acc[1]);
            w.y = pack2(acc[2], acc[3]);
            *(uint2*)(out + ((size_t)(q_tok0 + ti) * n_heads + head) * D + pd) = w;
        }
        return;
    }
    // four elements of four dims per thread and turn, so that the loads of a turn are in flight together (one element
    // per turn made a chain of as many round trips as the row tile has elements per thread)
    for (int idx = tid * 4; idx < n_valid * D; idx += 256 * 4) {
        const int r = idx / D, d = idx - r * D;           // D is a multiple of 16: the four dims are of one row
        const float* po = part_o + (slot0 + r) * D + d;
        f32x4_t acc = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
        for (int pi = 0; pi < n_parts; ++pi) acc += sm[pi][r] * *(const f32x4_t*)(po + (size_t)pi * slot_step * D);
        const int row = q_row0 + r;
        const int ti = row / G, head = kvh * G + (row - ti * G);
        uint2 w;
        w.x = pack2(acc[0], acc[1]);
        w.y = pack2(acc[2], acc[3]);
        *(uint2*)(out + ((size_t)(q_tok0 + ti) * n_heads + head) * D + d) = w;
    }
}

// RT row tiles of 16 rows per wave share every key/value block they read.
template <bool DECODE, int RT>
__global__ __launch_bounds__(256, D > 128 ? 1 : (DECODE && !DIRECT ? 3 : 2)) void attn_bf16_kernel(AttnArgs a) {
    // the wave's index as a scalar: its item and everything read from it then stay in scalar registers, and the
    // tests on them are scalar branches
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    // decoding: the four waves of a block share one item and take its key blocks in turn; otherwise one item per wave
    const int item = DECODE ? (int)blockIdx.x : (int)blockIdx.x * 4 + wv;
    if (item >= a.n_items) return;
    int entry, q_tok0, q_len, pos0, q_row0, key_lo, key_hi, part;
    bool dec_writes = false;
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
        dec_writes = pi == p_last;                    // this item's keys include the token's own
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

    const int* bt = a.block_table + (size_t)entry * a.max_blocks;
    const int ps = a.page_size;
    const int last_page = (key_hi - 1) / ps;
    KVBlock cur;
    const int j_first = key_lo + (DECODE ? 16 * wv : 0), j_step = DECODE ? 64 : 16;
    // the last block this wave may read: the last one of its own, or for a wave without keys the item's first
    const int j_end = j_first < key_hi ? j_first + (key_hi - 1 - j_first) / j_step * j_step : key_lo;
    // (read through the constant address space: the kernel writes pages and results but never the block table,
    // and only so is this a scalar load, which neither counts among the vector loads in flight nor waits for them)
    typedef const __attribute__((address_space(4))) int* const_int_ptr;
    const const_int_ptr btc = (const_int_ptr)(uintptr_t)bt;
    auto page_at = [&](int j) __attribute__((always_inline)) { return btc[min(page_index(a, min(j, j_end)), last_page)]; };
    const int spare = min(max(btc[last_page], 0), a.num_pages - 1);
    // Direct loads: lane l brings piece l of a 1 KB run (four keys, or 32 dims of the 16 keys' values) to slot l.
    const unsigned dk_off = (unsigned)(lane >> 4) * (2 * D) + ((unsigned)((lane & 15) ^ (lane >> 4)) << 4);
    const unsigned dv_off = (unsigned)((lane & 15) + 16 * (lane >> 5)) * (unsigned)(2 * ps) + (unsigned)((lane >> 4) & 1) * 16u;
    extern __shared__ __attribute__((aligned(16))) bf16_t wave_lds[];
    const unsigned wave_lds0 = lds_address(wave_lds + wv * KV_LDS_ELEMS);
    bool buf_ok[2];
    auto issue = [&](int j, int pg, int buf) __attribute__((always_inline)) {     // keys j .. j + 15 -> buffer buf
        const int j0 = min(j, j_end);
        const int blk = page_index(a, j0);
        buf_ok[buf] = pg >= 0 && pg < a.num_pages;
        const int pgc = buf_ok[buf] ? pg : spare;
        const int off = j0 - blk * ps;
        const char* kb = (const char*)(a.k_pages + (((size_t)pgc * a.n_kv + kvh) * ps + off) * D);
        const char* vb = (const char*)(a.v_pages + ((size_t)pgc * a.n_kv + kvh) * D * ps + off);
        const unsigned dst = wave_lds0 + buf * (KV_BUF_ELEMS * 2);
#pragma unroll
        for (int i = 0; i < 4; ++i)      // (the slot of a chunk depends on its key: four keys on, bits 2 and 3 turn)
            load_to_lds16<DECODE>(kb + i * 1024, dk_off ^ (unsigned)(64 * i), dst + i * 1024);
#pragma unroll
        for (int u = 0; u < 4; ++u)
            load_to_lds16<DECODE>(vb + (size_t)(u * 32) * (2 * ps), dv_off, dst + 4096 + u * 1024);
    };
    // A decoding wave asks for its first blocks before it turns to the query, whose loads and rotation would
    // otherwise stand between the block table and the first keys: one round trip to memory less per launch.
    // Not a block that holds the token's own key and value, which are written below: the wave's first block
    // (late_first), or its second (late_second), is then asked for after that.
    const bool late_first = DECODE && a.qkv && dec_writes && min(j_first, j_end) + 16 > pos0;
    const bool late_second = DECODE && a.qkv && dec_writes && j_first + j_step + 16 > pos0;
    if constexpr (DIRECT) {
        // (every wave does, decoding or not: the loads of the rows below are then younger than these, and where the
        // compiler waits for them it waits for nothing that the first step does not need anyway)
        if (!late_first) {
            if (j_first < key_hi) issue(j_first, page_at(j_first), 0);
            if (j_first + j_step < key_hi && !late_second) issue(j_first + j_step, page_at(j_first + j_step), 1);
        }
    } else if (DECODE && a.qkv) {
        load_block<DECODE>(cur, a, page_at(j_first), spare, min(j_first, j_end), kvh, lane);
    }

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
        if (DECODE && a.qkv) {
            // the query as the projection left it: rotate its pairs (i, i + rot/2) by the angles of its position
            const float* qrow = a.qkv + (size_t)q_tok0 * a.qkv_stride + (size_t)head[rt] * D;
            constexpr int CH = WIDE ? 8 : 4, STEP = WIDE ? 32 : 16;
            constexpr int QB = (WIDE ? 4 : 8) < QSTEPS ? (WIDE ? 4 : 8) : QSTEPS;     // chunks whose loads fly together
#pragma unroll
            for (int s0 = 0; s0 < QSTEPS; s0 += QB) {
                RotIn<CH> rin[QB];
#pragma unroll
                for (int u = 0; u < QB; ++u)
                    if (s0 + u < QSTEPS)
                        rot_load<CH>(rin[u], qrow, (s0 + u) * STEP + g * CH, a.rot, a.cos_t, a.sin_t, pos0, a.max_pos);
                __builtin_amdgcn_sched_barrier(0);      // all of them asked for before the first is used
#pragma unroll
                for (int u = 0; u < QB; ++u) {
                    if (s0 + u >= QSTEPS) continue;
                    float x[CH];
                    rot_apply<CH>(x, rin[u]);
                    if constexpr (WIDE) {
                        U16 t; t.u = make_uint4(pack2(x[0], x[1]), pack2(x[2], x[3]), pack2(x[4], x[5]), pack2(x[6], x[7]));
                        q8[rt][s0 + u] = t.v;
                    } else {
                        U8 t; t.u = make_uint2(pack2(x[0], x[1]), pack2(x[2], x[3]));
                        q4[rt][s0 + u] = t.v;
                    }
                }
            }
        } else {
            const bf16_t* qrow = a.q + ((size_t)(q_tok0 + ti[rt]) * a.n_heads + head[rt]) * D;
            if constexpr (WIDE) {
#pragma unroll
                for (int s = 0; s < QSTEPS; ++s) { U16 t; t.u = *(const uint4*)(qrow + s * 32 + g * 8); q8[rt][s] = t.v; }
            } else {
#pragma unroll
                for (int s = 0; s < QSTEPS; ++s) { U8 t; t.u = *(const uint2*)(qrow + s * 16 + g * 4); q4[rt][s] = t.v; }
            }
            if constexpr (DIRECT) {
                // The compiler does not know of the loads into LDS and counts only its own.  Left to itself it waits
                // for these rows at their first use, inside the loop over the keys, with a count that is right for
                // its loads alone: in every turn that wait takes the block that was only just asked for with it, and
                // nothing is in flight while a block is multiplied.  So it is made to wait here, once: an empty
                // statement that "rewrites" the registers.
#pragma unroll
                for (int s = 0; s < QSTEPS; ++s) asm volatile("" : "+v"(q8[rt][s]));
            }
        }
#pragma unroll
        for (int t = 0; t < DT; ++t) o[rt][t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
        m[rt] = -INFINITY;
        l[rt] = 0.f;
    }

    if (DECODE && a.qkv && dec_writes) {
        // The token's own key (rotated) and value go into their page before this block reads it.  No other block
        // reads this slot: the other items of the entry end before it, other kv heads have pages of their own.
        const int ps_ = a.page_size;
        const int blk = pos0 / ps_, slot = pos0 - blk * ps_;
        const int pg = a.block_table[(size_t)entry * a.max_blocks + blk];
        if (pg >= 0 && pg < a.num_pages) {      // the host never leaves the token without a page
            const int tid = threadIdx.x;
            if (tid < D / 4) {
                float x[4];
                RotIn<4> rk;
                rot_load<4>(rk, a.qkv + (size_t)q_tok0 * a.qkv_stride + (size_t)(a.n_heads + kvh) * D, tid * 4, a.rot,
                            a.cos_t, a.sin_t, pos0, a.max_pos);
                rot_apply<4>(x, rk);
                bf16_t* kp = (bf16_t*)a.k_pages + (((size_t)pg * a.n_kv + kvh) * ps_ + slot) * D + tid * 4;
                *(uint2*)kp = make_uint2(pack2(x[0], x[1]), pack2(x[2], x[3]));
            } else if (tid >= 64 && tid < 64 + D / 4) {
                const int i = (tid - 64) * 4;
                const float4 v = *(const float4*)(a.qkv + (size_t)q_tok0 * a.qkv_stride + (size_t)(a.n_heads + a.n_kv + kvh) * D + i);
                bf16_t* vp = (bf16_t*)a.v_pages + (((size_t)pg * a.n_kv + kvh) * D + i) * ps_ + slot;
                vp[0] = f32_to_bf16(v.x);
                vp[(size_t)ps_] = f32_to_bf16(v.y);
                vp[(size_t)2 * ps_] = f32_to_bf16(v.z);
                vp[(size_t)3 * ps_] = f32_to_bf16(v.w);
            }
        }
        __syncthreads();
    }

    // one block of 16 keys (in the wave's buffer `buf`) against the RT row tiles of this wave
    bf16_t* const kl0 = wave_lds + wv * KV_LDS_ELEMS;     // this wave's buffers: keys, then values
    auto compute = [&](int j0, int buf) __attribute__((always_inline)) {
        bf16_t* const kl = kl0 + buf * KV_BUF_ELEMS;
        const bf16_t* const vl = kl + 16 * (DIRECT ? D : KL_ROW);
        wave_lds_order();
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            if (j0 > tile_hi[rt] || j0 + 15 < tile_lo[rt]) continue;   // every key masked for every row of the tile
            f32x4_t s = (f32x4_t){0.f, 0.f, 0.f, 0.f};
            if constexpr (WIDE) {
#pragma unroll
                for (int st = 0; st < QSTEPS; ++st) {
                    U16 t;
                    if constexpr (DIRECT) t.u = *(const uint4*)(kl + r * D + (((4 * st + g) ^ r) << 3));
                    else t.u = *(const uint4*)(kl + r * KL_ROW + st * 32 + g * 8);
                    s = VT_MFMA_16X16X32(t.v, q8[rt][st], s);
                }
            } else {
#pragma unroll
                for (int st = 0; st < QSTEPS; ++st) {
                    U8 t; t.u = *(const uint2*)(kl + r * KL_ROW + st * 16 + g * 4);
                    s = VT_MFMA_16X16X16(t.v, q4[rt][st], s);
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
                U8 vf;
                if constexpr (DIRECT) vf.u = *(const uint2*)(vl + ((2 * t + (g >> 1)) * 16 + r) * 8 + (g & 1) * 4);
                else vf.u = *(const uint2*)(vl + (t * 16 + r) * VL_ROW + 4 * g);
                if (rescale) o[rt][t] *= alpha;
                o[rt][t] = VT_MFMA_16X16X16(vf.v, pf.v, o[rt][t]);
            }
        }
        wave_lds_order();       // the next block is parked after these reads
    };
    // One register buffer: a block is parked in LDS as soon as it has arrived, the next one is asked for into the
    // same registers at once and is on its way while this one is multiplied; the page id of the one after comes
    // from the block table meanwhile (a scalar load).  Every turn loads, whether or not keys are left (then the
    // wave's last block again, which nobody multiplies), so that no load sits under a branch.  (Two and three
    // buffers were slower inside whole decoding steps.)
    if constexpr (DIRECT) {
        // Two blocks are on their way while keys are left: the one that is multiplied next, and the one after it,
        // which was asked for into the buffer that the last multiplication left.  (Nothing is tested around these
        // loads for the compiler's sake, which does not know of them: a block that the wave does not have is not
        // asked for, and the wait counts the loads that are.)
        if (late_first) {
            if (j_first < key_hi) issue(j_first, page_at(j_first), 0);
            if (j_first + j_step < key_hi) issue(j_first + j_step, page_at(j_first + j_step), 1);
        } else if (late_second && j_first + j_step < key_hi) {
            issue(j_first + j_step, page_at(j_first + j_step), 1);
        }
        int pg_next = page_at(j_first + 2 * j_step);
        int buf = 0;
        for (int j = j_first; j < key_hi; j += j_step) {
            if (j + j_step < key_hi) wait_loads<8>();       // the older of two blocks (eight loads each) has landed
            else wait_loads<0>();
            if (buf_ok[buf]) compute(j, buf);
            if (j + 2 * j_step < key_hi) issue(j + 2 * j_step, pg_next, buf);
            pg_next = page_at(j + 3 * j_step);
            buf ^= 1;
        }
    } else {
        if (!(DECODE && a.qkv)) {
            load_block<DECODE>(cur, a, page_at(j_first), spare, min(j_first, j_end), kvh, lane);
        } else if (late_first) {
            // the wave's first block holds the token's own key and value, which were written above: read it again
            load_block<DECODE>(cur, a, page_at(j_first), spare, min(j_first, j_end), kvh, lane);
        }
        int pg_next = page_at(j_first + j_step);      // page of the next block to load
        bf16_t* const kl = kl0;
        for (int j = j_first; j < key_hi; j += j_step) {
            const bool ok = cur.ok;
            if (ok) park_block(cur, kl, lane);
            load_block<DECODE>(cur, a, pg_next, spare, min(j + j_step, j_end), kvh, lane);
            pg_next = page_at(j + 2 * j_step);
            __builtin_amdgcn_sched_barrier(0);
            if (ok) compute(j, 0);
        }
    }

    if constexpr (DECODE) {
        // The four waves hold partial results over disjoint keys of the same rows: merge them through LDS, half
        // of a large head at a time, and let all 256 threads write the result.
        // (a large head in two passes of TH tiles of 16 dims; the second pass is a tile shorter when DT is odd)
        constexpr int TH = (D > 128) ? (DT + 1) / 2 : DT;
        constexpr int DH = TH * 16;
        __syncthreads();            // every wave is done with its key/value buffer: the merge takes the memory over
        float (*so)[16][DH + 4] = (float (*)[16][DH + 4])wave_lds;
        static_assert(4 * 16 * (DH + 4) * 4 <= 4 * KV_LDS_ELEMS * 2, "the merge fits where the waves' buffers were");
        __shared__ float sm[4][16], sl[4][16];
        float lt = l[0];
        lt += __shfl_xor(lt, 16, 64);
        lt += __shfl_xor(lt, 32, 64);
        if (g == 0) { sm[wv][r] = m[0]; sl[wv][r] = lt; }
        const int n_valid = min(16, n_rows);
#pragma unroll
        for (int half = 0; half * TH < DT; ++half) {
            if (half) __syncthreads();
            const int dims = min(DH, D - half * DH);      // dims of this pass
#pragma unroll
            for (int t = 0; t < TH; ++t)
                if (half * TH + t < DT) *(f32x4_t*)&so[wv][r][t * 16 + 4 * g] = o[0][half * TH + t];
            __syncthreads();
            for (int idx = threadIdx.x; idx < n_valid * dims; idx += 256) {
                const int rr = idx / dims, dd = idx - rr * dims;
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
// threads together with 16-byte loads, and parked in LDS (two buffers: the next block comes from memory into
// registers while this one is multiplied, and is parked in the other buffer afterwards; with a head of 128 it comes
// from memory straight into the other buffer, see DIRECT); the four waves read their
// matrix operands from there, each operand once for all RT row tiles of the wave.  Rows of an item that lie wholly
// above a key block skip it (the upper triangle of a causal portion costs nothing).
//
// A block of keys is KH halves of 32.  The 32 LDS rows of a half hold its key 8q + 4t + i at row 16t + 4q + i
// (t = 0, 1: the half's two score tiles), so that the eight scores a lane holds after the first product (four
// each from the two tiles) are eight consecutive keys 8g..8g+7: exactly the k slots of its B operand in the
// 16x16x32 product with the values, whose A operand is then one 16-byte read of the value rows in their natural
// key order.  The row sums of the probabilities come out of the matrix cores too: one more product per half
// against a tile of ones, which leaves every lane with the sum of its row.
// ---------------------------------------------------------------------------
constexpr int KB = (D > 128) ? 32 : 64;        // keys per block
constexpr int KH = KB / 32;                    // halves of 32 keys
constexpr int KT = KB / 16;                    // score tiles per block
constexpr int KROW = D + 8;                    // padded rows: operand reads from LDS without bank conflicts
constexpr int VROW = KB + 8;
constexpr int GP = 2 * D;                      // 16-byte pieces of 16 keys (and of their values)
constexpr int NP = (GP + 255) / 256;           // pieces per thread and group of 16 keys
// With a head of 128 the blocks go from the pages straight into LDS, in the layout described at DIRECT above.
constexpr int KBUF = DIRECT ? KB * D : KB * KROW;        // elements of a key buffer, of a value buffer
constexpr int VBUF = DIRECT ? D * KB : D * VROW;
constexpr int TILE_LDS_BYTES = 2 * (KBUF + VBUF) * (int)sizeof(bf16_t);

constexpr int AHEAD = 4;                       // LDS operands on their way before the products that use them
constexpr int SCHED_MFMA = 0x008, SCHED_LDS_READ = 0x100;      // instruction classes of sched_group_barrier

// key (relative to the block's first) of score tile kt, lane group g, register i
__device__ __forceinline__ int tile_key(int kt, int g, int i) { return 32 * (kt >> 1) + 8 * g + 4 * (kt & 1) + i; }

// Maximum of three floats in one instruction.  (fmaxf first makes each operand canonical, an instruction per
// operand, because a signalling NaN must become quiet; there is none here.)
__device__ __forceinline__ float max3(float x, float y, float z) {
    float d;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(x), "v"(y), "v"(z));
    return d;
}
__device__ __forceinline__ float max2(float x, float y) {
    float d;
    asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(x), "v"(y));
    return d;
}
__device__ __forceinline__ float row_max4_lean(float v) {
    const unsigned u = __float_as_uint(v);
    const u32x2_t a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const unsigned a0 = a.x, a1 = a.y;
    const unsigned x = __float_as_uint(max2(__uint_as_float(a0), __uint_as_float(a1)));
    const u32x2_t b = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    const unsigned b0 = b.x, b1 = b.y;
    return max2(__uint_as_float(b0), __uint_as_float(b1));
}

// softmax_step for the tiled kernel: the same arithmetic, the key order above, no row sum (the matrix cores add
// it).  FULL: every key of the block is visible to every row of the tile, nothing is tested.
template <bool FULL>
__device__ __forceinline__ void tile_softmax(const f32x4_t (&s)[KT], int j0, int g, int p, int p_lo,
                                             float scale_log2, float& m, float& alpha, unsigned (&pk)[KT * 2]) {
    bool ok[KT][4];
    float v[KT][4];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int j = j0 + tile_key(kt, g, i);
            ok[kt][i] = FULL || (j <= p && j >= p_lo);
            v[kt][i] = ok[kt][i] ? s[kt][i] : -INFINITY;
        }
    float mb = max2(max3(v[0][0], v[0][1], v[0][2]), v[0][3]);
#pragma unroll
    for (int kt = 1; kt < KT; ++kt) mb = max3(max3(mb, v[kt][0], v[kt][1]), v[kt][2], v[kt][3]);
    mb = row_max4_lean(mb * scale_log2);
    const float m_new = max2(m, mb);
    alpha = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - m_new);
    m = m_new;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        float pv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float e = __builtin_amdgcn_exp2f(fmaf(s[kt][i], scale_log2, -m_new));
            pv[i] = (FULL || ok[kt][i]) ? e : 0.f;      // a visible key makes m_new finite
        }
        pk[2 * kt] = pack2(pv[0], pv[1]);
        pk[2 * kt + 1] = pack2(pv[2], pv[3]);
    }
}

template <int RT>
__global__ __launch_bounds__(256, D > 128 ? 1 : 2) void attn_bf16_tile_kernel(AttnArgs a) {
    extern __shared__ __attribute__((aligned(16))) bf16_t tile_lds[];
    bf16_t* const k_lds = tile_lds;                       // [2][KBUF]
    bf16_t* const v_lds = tile_lds + 2 * KBUF;            // [2][VBUF]
    const int tid = threadIdx.x, lane = tid & 63;
    // the wave's index as a scalar: what depends only on it (which keys the wave's tiles see) then stays in scalar
    // registers and its tests are scalar branches
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int* it = a.items + (size_t)blockIdx.y * ITEM_INTS;
    const int entry = it[0], q_tok0 = it[1], q_len = it[2], pos0 = it[3], q_row0 = it[4];
    const int key_lo = it[5], key_hi = it[6], part = it[7];
    if (entry < 0) return;
    const int kvh = blockIdx.x;
    const int G = a.n_heads / a.n_kv;
    const int r = lane & 15, g = lane >> 4;
    const int n_rows = q_len * G;
    const int ps = a.page_size;

    bool row_ok[RT];
    int ti[RT], head[RT], p[RT], p_lo[RT], tile_first_p[RT], tile_last_lo[RT];
    bf16x8_t q8[RT][WIDE ? QSTEPS : 1];
    bf16x4_t q4[RT][WIDE ? 1 : QSTEPS];
    f32x4_t o[RT][DT], ol[RT];     // ol: the row sums, the same value in all four registers
    float m[RT];
    int wave_hi = -1, wave_lo = 0x7fffffff;   // keys that any row of the wave may see
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
        // a block whose keys lie between these two is visible to every row of the tile
        tile_first_p[rt] = pos0 + first_row / G;
        tile_last_lo[rt] = a.window > 0 ? pos0 + last_row / G - a.window + 1 : 0;
        if (row0 < n_rows) {
            wave_hi = max(wave_hi, pos0 + last_row / G);
            wave_lo = min(wave_lo, a.window > 0 ? pos0 + first_row / G - a.window + 1 : 0);
        }
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
        ol[rt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
        m[rt] = -INFINITY;
    }

    // This thread's pieces of a group of 16 keys: piece x of the keys is (key x / (D/8), dims 8 (x % (D/8))..),
    // piece x of the values is (dim x / 2, keys 8 (x % 2)..).  Byte offsets from the group's first element in the
    // pages, element offsets in an LDS buffer; fixed for the whole walk.
    unsigned k_src[NP], v_src[NP];
    int k_dst[KT][NP], v_dst[NP];
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int x = tid + 256 * i;
        const int key = x / (D / 8), c = x - key * (D / 8);
        k_src[i] = 2u * (unsigned)(key * D + c * 8);
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            const int jb = 16 * (kt & 1) + key;      // key within its half -> its LDS row
            const int row = 32 * (kt >> 1) + ((jb & 7) >> 2) * 16 + 4 * (jb >> 3) + (jb & 3);
            k_dst[kt][i] = row * KROW + c * 8;
        }
        const int d = x >> 1, h = x & 1;
        v_src[i] = 2u * (unsigned)(d * ps + 8 * h);
        v_dst[i] = d * VROW + 8 * h;
    }

    // The next fetch starts at offset f_off of the entry's page f_blk.  The page ids of that block's groups of 16
    // keys are read from the block table a step ahead; all of it is the same in every thread and lives in scalar
    // registers.  A group without a page (beyond the entry's keys, or passed by a window: every row masks its
    // keys) reads the entry's last page instead, whose contents are as harmless as the unused slots of any page.
    const int* bt = a.block_table + (size_t)entry * a.max_blocks;
    const int last_page = (key_hi - 1) / ps;
    const int pg_spare = min(max(bt[last_page], 0), a.num_pages - 1);
    int f_blk = key_lo / ps, f_off = key_lo - f_blk * ps;
    int pgn[KT];
    auto next_pages = [&]() __attribute__((always_inline)) {
        int blk = f_blk, off = f_off;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            pgn[kt] = bt[min(blk, last_page)];
            off += 16;
            const bool wrap = off == ps;
            off = wrap ? 0 : off;
            blk += wrap ? 1 : 0;
        }
    };
    const unsigned page_bytes = (unsigned)(a.n_kv * ps * D) * 2u;     // bytes per page, keys or values
    const char* const k_base = (const char*)(a.k_pages + (size_t)kvh * ps * D);
    const char* const v_base = (const char*)(a.v_pages + (size_t)kvh * ps * D);
    // (a native vector type: copies of HIP's uint4 struct become memcpy calls that keep the stage in scratch memory)
    u32x4_t st_k[KT][NP], st_v[KT][NP];
    // Direct path: wave w brings the block's keys 16 w .. 16 w + 15 and their values: one group of 16 keys, which
    // lies in one page, so a step costs the wave one page id and two addresses.  Its four key pieces (four keys
    // each, 1 KB) go to the LDS rows that the score tiles read them from (see tile_key); its four value pieces are
    // 32 dims each.  What differs from lane to lane and from piece to piece is fixed for the walk and kept in
    // registers; what changes from step to step is the same in every lane and kept in scalar registers.
    unsigned dma_k_off[4], dma_v_off[4];
    unsigned dma_k_lds[4], dma_v_lds[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int sw = (8 * (wv & 1) + 4 * (c >> 1) + (lane >> 4)) & 15;
        dma_k_off[c] = (unsigned)(4 * c + (lane >> 4)) * (2 * D) + ((unsigned)((lane & 15) ^ sw) << 4);
        dma_k_lds[c] = (unsigned)(8 * (wv >> 1) + 4 * (c & 1) + 2 * (wv & 1) + (c >> 1)) * 1024u;
        dma_v_off[c] = (unsigned)((lane & 15) + 16 * (lane >> 5) + 32 * c) * (unsigned)(2 * ps) + (unsigned)((lane >> 4) & 1) * 16u;
        dma_v_lds[c] = (unsigned)wv * 4096u + (unsigned)c * 1024u;
    }
    // The group's page and its offset there move on by KB keys per fetch without a division; the page id is read
    // from the block table a step ahead, through the constant address space (the kernel never writes the table):
    // only so is it a scalar load, which does not wait for the loads into LDS that are in flight.
    typedef const __attribute__((address_space(4))) int* const_int_ptr;
    const const_int_ptr btc = (const_int_ptr)(uintptr_t)bt;
    const unsigned lds_k0 = lds_address(k_lds), lds_v0 = lds_address(v_lds);
    const int adv_blk = KB / ps, adv_off = KB - adv_blk * ps;
    int g_blk, g_off, g_pg;
    {
        const int kp = key_lo + 16 * wv;
        g_blk = kp / ps;
        g_off = kp - g_blk * ps;
    }
    auto dma_pages = [&]() __attribute__((always_inline)) { g_pg = btc[min(g_blk, last_page)]; };
    auto fetch_dma = [&](int buf) __attribute__((always_inline)) {
        const unsigned kd = lds_k0 + buf * (KBUF * 2), vd = lds_v0 + buf * (VBUF * 2);     // byte addresses in LDS
        const int pg = ((unsigned)g_pg < (unsigned)a.num_pages) ? g_pg : pg_spare;
        const size_t pg_off = (size_t)(unsigned)pg * page_bytes;
        const char* ksrc = k_base + (pg_off + (unsigned)(g_off * (2 * D)));
        const char* vsrc = v_base + (pg_off + (unsigned)(g_off * 2));
#pragma unroll
        for (int c = 0; c < 4; ++c) load_to_lds16(ksrc, dma_k_off[c], kd + dma_k_lds[c]);
#pragma unroll
        for (int c = 0; c < 4; ++c) load_to_lds16(vsrc, dma_v_off[c], vd + dma_v_lds[c]);
        g_blk += adv_blk;
        g_off += adv_off;
        const bool wrap = g_off >= ps;
        g_off -= wrap ? ps : 0;
        g_blk += wrap ? 1 : 0;
        dma_pages();
    };
    auto fetch = [&]() __attribute__((always_inline)) {   // this thread's pieces of the next KB keys, pages -> registers
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            const int pg = (pgn[kt] >= 0 && pgn[kt] < a.num_pages) ? pgn[kt] : pg_spare;
            const size_t pg_off = (size_t)pg * page_bytes;
            const char* kb = k_base + (pg_off + (unsigned)(f_off * (2 * D)));
            const char* vb = v_base + (pg_off + (unsigned)(f_off * 2));
#pragma unroll
            for (int i = 0; i < NP; ++i) {
                if (GP % 256 == 0 || tid + 256 * i < GP) {
                    st_k[kt][i] = *(const u32x4_t*)(kb + k_src[i]);
                    st_v[kt][i] = *(const u32x4_t*)(vb + v_src[i]);
                }
            }
            f_off += 16;
            const bool wrap = f_off == ps;
            f_off = wrap ? 0 : f_off;
            f_blk += wrap ? 1 : 0;
        }
        next_pages();
    };
    auto park = [&](int buf) __attribute__((always_inline)) {
        bf16_t* const kd = k_lds + buf * KBUF;
        bf16_t* const vd = v_lds + buf * VBUF;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < NP; ++i)
                if (GP % 256 == 0 || tid + 256 * i < GP) {
                    *(u32x4_t*)(kd + k_dst[kt][i]) = st_k[kt][i];
                    *(u32x4_t*)(vd + v_dst[i] + 16 * kt) = st_v[kt][i];
                }
    };

    bf16x8_t ones8;
    { U16 t; t.u = make_uint4(VT_LOWP_ONE_PAIR, VT_LOWP_ONE_PAIR, VT_LOWP_ONE_PAIR, VT_LOWP_ONE_PAIR); ones8 = t.v; }
    // one key block (in LDS buffer `buf`, keys from j0) against the RT row tiles of this wave
    auto multiply = [&](int buf, int j0) __attribute__((always_inline)) {
        if (j0 > wave_hi || j0 + KB - 1 < wave_lo) return;   // every key masked for every row of the wave
        const bf16_t* const kd = k_lds + buf * KBUF;
        const bf16_t* const vd = v_lds + buf * VBUF;
        f32x4_t s[RT][KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) s[rt][kt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
            const bf16_t* kr = kd + (kt * 16 + r) * (DIRECT ? D : KROW);
            if constexpr (WIDE) {
#pragma unroll
                for (int st = 0; st < QSTEPS; ++st) {
                    U16 t;
                    if constexpr (DIRECT) t.u = *(const uint4*)(kr + (((4 * st + g) ^ r) << 3));
                    else t.u = *(const uint4*)(kr + st * 32 + g * 8);
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
                        s[rt][kt] = VT_MFMA_16X16X32(t.v, q8[rt][st], s[rt][kt]);
                }
            } else {
#pragma unroll
                for (int st = 0; st < QSTEPS; ++st) {
                    U8 t; t.u = *(const uint2*)(kr + st * 16 + g * 4);
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
                        s[rt][kt] = VT_MFMA_16X16X16(t.v, q4[rt][st], s[rt][kt]);
                }
            }
        }
        // The order the compiler gives these on its own is "read an operand, wait for it, multiply"; asked for
        // here: the reads of AHEAD operands first, then after every operand's products the read that is AHEAD
        // operands further on, so that an operand has been on its way for that many products when it is needed.
        // (Heads above 128, one block per compute unit: measured slower with it at one row tile.)
        if constexpr (WIDE && (D <= 128 || RT == 2)) {
#pragma unroll
            for (int n = 0; n < AHEAD; ++n) __builtin_amdgcn_sched_group_barrier(SCHED_LDS_READ, 1, 0);
#pragma unroll
            for (int n = 0; n < KT * QSTEPS; ++n) {
                __builtin_amdgcn_sched_group_barrier(SCHED_MFMA, RT, 0);
                if (n + AHEAD < KT * QSTEPS) __builtin_amdgcn_sched_group_barrier(SCHED_LDS_READ, 1, 0);
            }
        }
        // s[rt][kt][i] is key j0 + tile_key(kt, g, i) against row r of tile rt.  A tile with no visible key in
        // this block keeps its state: every probability is 0 and its factor 1.
        unsigned pk[RT][KT * 2];
        float alpha[RT];
        bool full = true;      // every key of the block is visible to every row of the wave
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) full = full && (j0 + KB - 1 <= tile_first_p[rt]) && (j0 >= tile_last_lo[rt]);
        if (full) {
            // (the tiles one after the other in one stretch of code: each one's chain of dependent operations
            // fills the other's waits)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) tile_softmax<true>(s[rt], j0, g, p[rt], p_lo[rt], a.scale_log2, m[rt], alpha[rt], pk[rt]);
        } else {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) tile_softmax<false>(s[rt], j0, g, p[rt], p_lo[rt], a.scale_log2, m[rt], alpha[rt], pk[rt]);
        }
        bool moved = false;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) moved = moved || (alpha[rt] != 1.f);
        if (__any(moved)) {      // the maximum of some row moved
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
                for (int t = 0; t < DT; ++t) o[rt][t] *= alpha[rt];
                ol[rt] *= alpha[rt];
            }
        }
#pragma unroll
        for (int h = 0; h < KH; ++h) {
            U16 pf[RT];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                pf[rt].u = make_uint4(pk[rt][4 * h], pk[rt][4 * h + 1], pk[rt][4 * h + 2], pk[rt][4 * h + 3]);
                ol[rt] = VT_MFMA_16X16X32(ones8, pf[rt].v, ol[rt]);
            }
#pragma unroll
            for (int t = 0; t < DT; ++t) {
                U16 vf;
                if constexpr (DIRECT) vf.u = *(const uint4*)(vd + (2 * h + (g >> 1)) * 2048 + ((2 * t + (g & 1)) * 16 + r) * 8);
                else vf.u = *(const uint4*)(vd + (t * 16 + r) * VROW + 32 * h + 8 * g);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                    o[rt][t] = VT_MFMA_16X16X32(vf.v, pf[rt].v, o[rt][t]);
            }
        }
        // (the same order for the value operands; a half's products begin with its row sums)
        if constexpr (D <= 128 || RT == 2) {
#pragma unroll
            for (int n = 0; n < AHEAD; ++n) __builtin_amdgcn_sched_group_barrier(SCHED_LDS_READ, 1, 0);
#pragma unroll
            for (int n = 0; n < KH * DT; ++n) {
                if (n % DT == 0) __builtin_amdgcn_sched_group_barrier(SCHED_MFMA, RT, 0);
                __builtin_amdgcn_sched_group_barrier(SCHED_MFMA, RT, 0);
                if (n + AHEAD < KH * DT) __builtin_amdgcn_sched_group_barrier(SCHED_LDS_READ, 1, 0);
            }
        }
    };

    int buf = 0;
    if constexpr (DIRECT) {
        dma_pages();
        fetch_dma(0);
        __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0): this wave's pieces are in LDS
        __syncthreads();
        for (int j0 = key_lo; j0 < key_hi; j0 += KB) {
            if (j0 + KB < key_hi) fetch_dma(buf ^ 1);     // the next block is on its way while this one is multiplied
            multiply(buf, j0);
            __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
            buf ^= 1;
        }
    } else {
        next_pages();
        fetch();
        park(0);
        __syncthreads();
        for (int j0 = key_lo; j0 < key_hi; j0 += KB) {
            const bool more = j0 + KB < key_hi;
            if (more) fetch();              // the next block is on its way while this one is multiplied
            multiply(buf, j0);
            if (more) park(buf ^ 1);
            __syncthreads();
            buf ^= 1;
        }
    }

#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (!row_ok[rt]) continue;
        const float lt = ol[rt][0];
        if (part >= 0) {
            // one of several items over the keys of these rows: the unnormalised sums, for the merge (the item's
            // 4 RT tiles of 16 rows lie one after the other, wave by wave)
            const size_t slot = (((size_t)part * (4 * RT) + (wv * RT + rt)) * a.n_kv + kvh) * 16 + r;
            float* po = a.part_o + slot * D;
#pragma unroll
            for (int t = 0; t < DT; ++t) *(f32x4_t*)(po + t * 16 + 4 * g) = o[rt][t];
            if (g == 0) {
                a.part_ml[slot * 2] = m[rt];
                a.part_ml[slot * 2 + 1] = lt;
            }
            continue;
        }
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

// citems: [n][6] = q_tok0, q_len, first row of the tile, first item's partial index, number of items, tile index
// within its items (each item holds `rt_per_item` tiles).  One block per (tile, kv head).
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
    const int kvh = blockIdx.y, G = n_heads / n_kv;
    const int n_valid = min(16, q_len * G - q_row0);
    const size_t slot0 = (((size_t)part0 * rt_per_item + rt) * n_kv + kvh) * 16;
    const size_t slot_step = (size_t)rt_per_item * n_kv * 16;
    merge_parts(sm, sl, part_o, part_ml, out, slot0, slot_step, n_parts, n_valid, q_tok0, q_row0, G, kvh, n_heads);
}

static int shift_of(int v) {
    for (int sft = 0; sft < 31; ++sft)
        if ((1 << sft) == v) return sft;
    return -1;
}

// LDS of the kernels whose waves hand key/value blocks to their lanes through buffers of their own: more than a
// kernel gets without asking when the head is large
constexpr int WAVE_LDS_BYTES = 4 * KV_LDS_ELEMS * (int)sizeof(bf16_t);
static int wave_kernels_lds() {
    static bool set = false;
    if (set) return 0;
    const void* fns[3] = {(const void*)attn_bf16_kernel<false, 1>, (const void*)attn_bf16_kernel<false, (D <= 128 ? 2 : 1)>,
                          (const void*)attn_bf16_kernel<true, 1>};
    for (const void* f : fns) {
        hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, WAVE_LDS_BYTES);
        VT_REQUIRE(e == hipSuccess, "attention: cannot get %d bytes of LDS: %s", WAVE_LDS_BYTES, hipGetErrorString(e));
    }
    set = true;
    return 0;
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
    VT_REQUIRE(rt == 1 || D <= 128, "vt_attn_bf16: two row tiles per item need a head size of at most 128 (this is %d)", D);
    VT_REQUIRE(n_citems == 0 || (part_o && part_ml), "vt_attn_bf16: split keys but no workspace");
    if (n_items <= 0) return 0;
    AttnArgs a;
    a.q = (const bf16_t*)q; a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
    a.block_table = block_table; a.items = items; a.out = (bf16_t*)out; a.part_o = part_o; a.part_ml = part_ml;
    a.n_items = n_items; a.n_heads = n_heads; a.n_kv = n_kv; a.page_size = page_size; a.max_blocks = max_blocks;
    a.num_pages = num_pages; a.window = window; a.scale_log2 = scale * 1.4426950408889634f;
    a.entry_pos0 = nullptr; a.dec_params = nullptr; a.p_max = 0; a.ps_shift = shift_of(page_size);
    a.qkv = nullptr; a.qkv_stride = 0; a.cos_t = a.sin_t = nullptr; a.rot = a.max_pos = 0;
    dim3 grid((n_items + 3) / 4, n_kv);
    if (wave_kernels_lds()) return -1;
    if (rt == 1) attn_bf16_kernel<false, 1><<<grid, 256, WAVE_LDS_BYTES, stream>>>(a);
    else attn_bf16_kernel<false, (D <= 128 ? 2 : 1)><<<grid, 256, WAVE_LDS_BYTES, stream>>>(a);
    VT_CHECK_LAUNCH("vt_attn_bf16");
    if (n_citems > 0) {
        attn_combine_kernel<false><<<dim3(n_citems, n_kv), 256, 0, stream>>>(citems, part_o, part_ml, (bf16_t*)out,
                                                                            n_heads, n_kv, nullptr, nullptr, 0, window, rt);
        VT_CHECK_LAUNCH("vt_attn_bf16(combine)");
    }
    return 0;
}

// Long portions: items [n][8] as above, each 64 * rt rows (rt = 1 or 2) of one entry; one block of 4 waves per
// (item, kv head).  An item holds all the keys its rows may see (partial index -1), or one of several ranges of them:
// then it leaves its partial result in workspace slot (partial index * 4 rt + tile) and the combine items [m][6]
// (one per 16-row tile, as above, with 4 rt tiles per item) merge the ranges.
// 1 if this head size's kernels load their key/value blocks straight into LDS (which decides how the host cuts
// their work), else 0
extern "C" int vt_attn_bf16_direct() { return DIRECT ? 1 : 0; }

extern "C" int vt_attn_bf16_tiles(const void* q, const void* k_pages, const void* v_pages, const int* block_table,
                                  const int* items, int n_items, int rt, const int* citems, int n_citems, void* out,
                                  float* part_o, float* part_ml, int n_heads, int n_kv, int page_size,
                                  int max_blocks, int num_pages, int window, float scale, hipStream_t stream) {
    if (check_common("vt_attn_bf16_tiles", n_heads, n_kv, page_size, max_blocks, num_pages)) return -1;
    VT_REQUIRE(rt == 1 || rt == 2, "vt_attn_bf16_tiles: %d row tiles per wave (1 or 2)", rt);
    VT_REQUIRE(n_citems == 0 || (citems && part_o && part_ml), "vt_attn_bf16_tiles: split keys but no workspace");
    if (n_items <= 0) return 0;
    AttnArgs a;
    a.q = (const bf16_t*)q; a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
    a.block_table = block_table; a.items = items; a.out = (bf16_t*)out; a.part_o = part_o; a.part_ml = part_ml;
    a.n_items = n_items; a.n_heads = n_heads; a.n_kv = n_kv; a.page_size = page_size; a.max_blocks = max_blocks;
    a.num_pages = num_pages; a.window = window; a.scale_log2 = scale * 1.4426950408889634f;
    a.entry_pos0 = nullptr; a.dec_params = nullptr; a.p_max = 0; a.ps_shift = shift_of(page_size);
    a.qkv = nullptr; a.qkv_stride = 0; a.cos_t = a.sin_t = nullptr; a.rot = a.max_pos = 0;
    // blocks start in the order of their index, x fastest: all kv heads of the first (longest) item, then the next
    // item's, so that the longest items of every head start first and the rest fill in as blocks finish
    dim3 grid(n_kv, n_items);
    VT_REQUIRE(grid.y <= 65535, "vt_attn_bf16_tiles: too many items (%d)", n_items);
    // more LDS than a kernel gets without asking
    static bool lds_set = false;
    if (!lds_set) {
        hipError_t e1 = hipFuncSetAttribute((const void*)attn_bf16_tile_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, TILE_LDS_BYTES);
        hipError_t e2 = hipFuncSetAttribute((const void*)attn_bf16_tile_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, TILE_LDS_BYTES);
        VT_REQUIRE(e1 == hipSuccess && e2 == hipSuccess, "vt_attn_bf16_tiles: cannot get %d bytes of LDS: %s", TILE_LDS_BYTES,
                   hipGetErrorString(e1 != hipSuccess ? e1 : e2));
        lds_set = true;
    }
    if (rt == 1) attn_bf16_tile_kernel<1><<<grid, 256, TILE_LDS_BYTES, stream>>>(a);
    else attn_bf16_tile_kernel<2><<<grid, 256, TILE_LDS_BYTES, stream>>>(a);
    VT_CHECK_LAUNCH("vt_attn_bf16_tiles");
    if (n_citems > 0) {
        attn_combine_kernel<false><<<dim3(n_citems, n_kv), 256, 0, stream>>>(citems, part_o, part_ml, (bf16_t*)out,
                                                                            n_heads, n_kv, nullptr, nullptr, 0, window, 4 * rt);
        VT_CHECK_LAUNCH("vt_attn_bf16_tiles(combine)");
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
    a.qkv = nullptr; a.qkv_stride = 0; a.cos_t = a.sin_t = nullptr; a.rot = a.max_pos = 0;
    if (wave_kernels_lds()) return -1;
    attn_bf16_kernel<true, 1><<<dim3(a.n_items, n_kv), 256, WAVE_LDS_BYTES, stream>>>(a);
    VT_CHECK_LAUNCH("vt_attn_bf16_decode");
    attn_combine_kernel<true><<<dim3(n_entries, n_kv), 256, 0, stream>>>(nullptr, part_o, part_ml, (bf16_t*)out, n_heads,
                                                                        n_kv, entry_pos0, dec_params, p_max, window, 1);
    VT_CHECK_LAUNCH("vt_attn_bf16_decode(combine)");
    return 0;
}

// Decoding, fused: as vt_attn_bf16_decode, but from the projections' fp32 output qkv [entries][qkv_stride] (queries
// of all heads, keys, values).  The attention kernel rotates the queries and the new key by the angles of the
// token's position (tables [max_pos][rot/2]; rot = 0: no rotation) and writes the new key and value into the
// token's page itself: two launches instead of three.  (Merging an entry's items in the same launch, by the item
// that finishes last, was measured too: the device-wide fences it needs cost more than the launch they save.)
extern "C" int vt_attn_bf16_decode_fused(const float* qkv, long long qkv_stride, const float* cos_t, const float* sin_t,
                                         int rot, int max_pos, void* k_pages, void* v_pages, const int* block_table,
                                         const int* entry_pos0, const int* dec_params, int n_entries, int p_max, void* out,
                                         float* part_o, float* part_ml, int n_heads, int n_kv, int page_size,
                                         int max_blocks, int num_pages, int window, float scale, hipStream_t stream) {
    if (check_common("vt_attn_bf16_decode_fused", n_heads, n_kv, page_size, max_blocks, num_pages)) return -1;
    VT_REQUIRE(n_heads / n_kv <= 16, "vt_attn_bf16_decode_fused: %d query heads per kv head do not fit one tile of 16 rows",
               n_heads / n_kv);
    VT_REQUIRE(p_max > 0 && p_max <= MAX_PARTS, "vt_attn_bf16_decode_fused: %d items per entry (1..%d)", p_max, MAX_PARTS);
    VT_REQUIRE(qkv && part_o && part_ml && entry_pos0 && dec_params, "vt_attn_bf16_decode_fused: missing buffers");
    VT_REQUIRE(qkv_stride >= (long long)(n_heads + 2 * n_kv) * D && qkv_stride % 4 == 0,
               "vt_attn_bf16_decode_fused: row stride %lld does not hold %d heads of %d", qkv_stride, n_heads + 2 * n_kv, D);
    VT_REQUIRE(rot >= 0 && rot <= D && rot % 16 == 0, "vt_attn_bf16_decode_fused: %d rotated dims (a multiple of 16 up to %d)", rot, D);
    VT_REQUIRE(rot == 0 || (cos_t && sin_t && max_pos > 0), "vt_attn_bf16_decode_fused: no rotary table");
    if (n_entries <= 0) return 0;
    AttnArgs a;
    a.q = nullptr; a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
    a.block_table = block_table; a.items = nullptr; a.out = (bf16_t*)out; a.part_o = part_o; a.part_ml = part_ml;
    a.n_items = n_entries * p_max; a.n_heads = n_heads; a.n_kv = n_kv; a.page_size = page_size; a.max_blocks = max_blocks;
    a.num_pages = num_pages; a.window = window; a.scale_log2 = scale * 1.4426950408889634f;
    a.entry_pos0 = entry_pos0; a.dec_params = dec_params; a.p_max = p_max; a.ps_shift = shift_of(page_size);
    a.qkv = qkv; a.qkv_stride = qkv_stride; a.cos_t = cos_t; a.sin_t = sin_t; a.rot = rot; a.max_pos = max_pos;
    if (wave_kernels_lds()) return -1;
    attn_bf16_kernel<true, 1><<<dim3(a.n_items, n_kv), 256, WAVE_LDS_BYTES, stream>>>(a);
    VT_CHECK_LAUNCH("vt_attn_bf16_decode_fused");
    attn_combine_kernel<true><<<dim3(n_entries, n_kv), 256, 0, stream>>>(nullptr, part_o, part_ml, (bf16_t*)out, n_heads,
                                                                        n_kv, entry_pos0, dec_params, p_max, window, 1);
    VT_CHECK_LAUNCH("vt_attn_bf16_decode_fused(combine)");
    return 0;
}
