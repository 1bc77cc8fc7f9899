// bfloat16 linear layers on the gfx950 matrix cores, for few rows (decoding
// and short portions): y[n, m] = sum_k x[n, k] * W[m, k] (+ bias[m]), fp32
// accumulation, fp32 or bf16 output; and the same with the SiLU gate fused:
// y[n, i] = silu(x.Wg[i]) * (x.Wu[i]).
//
// The reference calls hipblasGemmEx for each projection, rounds the result
// to 16 bits and then adds the bias in a second kernel
// (v1/tensortype/hip_tensor.cpp:514-535, v1/tensortype/hip_kernels/add_bias.cpp:8-17),
// and runs up, gate and the gating as three launches
// (v1/models/qwen2-7b/inference_fp16.dag:333-336).  Here the bias and the gate
// are applied to the fp32 accumulator.
//
// With few rows the time goes to reading W once from HBM, so the weights are
// kept in the order in which the matrix instruction wants them.  W [M, K] is
// cut into tiles of 16 rows x 32 k; a tile is stored as the 64 lanes' operand
// fragments one after the other (lane 16 g + r holds W[16 mt + r][32 kt + 8 g ..
// + 8]), 1 KB in all, and the tiles of a row of tiles follow each other along k:
//     packed[((mt * KT + kt) * 64 + lane) * 8 + j]
// with M padded to 16 and K to 128 by zeros (vt_pack_matrix_bf16).  A wave's load
// of a fragment is then 1 KB of consecutive memory, eight cache lines, where the
// same fragment from a row-major W touches 64 separate 16-byte pieces of 16 rows:
// the first-level cache handles a line per cycle, and with a piece per cycle the
// matrix could not be read faster than about 4.4 TB/s; in this order it is read
// at 5.3 to 5.6 TB/s.
//
// The waves of a block split k and add their partial sums through LDS in wave
// order.  How k is split depends on the shape of W only, never on the number
// of rows, so a token's result does not change with the batch around it.
#include "vt_common.h"
#include "vt_gemm_bf16.h"
#include <mutex>

VT_DEFINE_LAST_ERROR()

typedef vt_lowp8_t bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

union Frag {
    uint4 u;
    bf16x8_t v;
};

// A fragment of W from memory.  In a launch that reads every weight once (few tokens: one block of tokens) the loads
// are marked non-temporal: lines that nobody will ask for again do not push the tokens out of the caches, and the
// memory delivers about a tenth more to loads so marked (6.0 -> 6.7 TB/s to a kernel that only reads, measured).
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_w_once(const bf16_t* p) {
    const u32x4_t v = __builtin_nontemporal_load((const u32x4_t*)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

#define PK_TILE 512                 // elements of a packed tile
#define PK_KPAD 128                 // K is padded to a multiple of this

__host__ __device__ static inline int pk_rows(int M) { return (M + 15) & ~15; }
__host__ __device__ static inline int pk_cols(int K) { return (K + PK_KPAD - 1) / PK_KPAD * PK_KPAD; }

// ---------------------------------------------------------------------------
// Packing: one thread per 16-byte piece of the packed matrix.
// ---------------------------------------------------------------------------
__global__ void pack_matrix_kernel(const bf16_t* __restrict__ w, bf16_t* __restrict__ wp, int M, int K, int KT, size_t pieces) {
    const size_t p = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= pieces) return;
    const int lane = (int)(p & 63);
    const size_t tile = p >> 6;
    const int kt = (int)(tile % KT), mt = (int)(tile / KT);
    const int m = mt * 16 + (lane & 15), k = kt * 32 + (lane >> 4) * 8;
    uint32_t v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (m < M && k + j < K) ? w[(size_t)m * K + k + j] : 0u;
    uint4 o;
    o.x = v[0] | (v[1] << 16); o.y = v[2] | (v[3] << 16);
    o.z = v[4] | (v[5] << 16); o.w = v[6] | (v[7] << 16);
    *(uint4*)(wp + p * 8) = o;
}

extern "C" long long vt_packed_elems(int M, int K) { return (long long)pk_rows(M) * pk_cols(K); }

// wp must hold vt_packed_elems(M, K) elements
extern "C" int vt_pack_matrix_bf16(const void* w, void* wp, int M, int K, hipStream_t stream) {
    VT_REQUIRE(M > 0 && K > 0, "vt_pack_matrix_bf16: bad sizes M=%d K=%d", M, K);
    VT_REQUIRE((((uintptr_t)wp) & 15) == 0, "vt_pack_matrix_bf16: the packed matrix must be 16-byte aligned");
    const int KT = pk_cols(K) / 32;
    const size_t pieces = (size_t)(pk_rows(M) / 16) * KT * 64;
    pack_matrix_kernel<<<(unsigned)((pieces + 255) / 256), 256, 0, stream>>>((const bf16_t*)w, (bf16_t*)wp, M, K, KT, pieces);
    VT_CHECK_LAUNCH("vt_pack_matrix_bf16");
    return 0;
}

// The way back: one thread per 16-byte piece of the packed matrix writes its eight values into the row-major matrix.
// (A model that is kept packed only gets the row-major form of a matrix back for as long as a long portion's product
// through the GEMM library needs it.)
__global__ void unpack_matrix_kernel(const bf16_t* __restrict__ wp, bf16_t* __restrict__ w, int M, int K, int KT, size_t pieces) {
    const size_t p = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= pieces) return;
    const int lane = (int)(p & 63);
    const size_t tile = p >> 6;
    const int kt = (int)(tile % KT), mt = (int)(tile / KT);
    const int m = mt * 16 + (lane & 15), k = kt * 32 + (lane >> 4) * 8;
    if (m >= M || k >= K) return;
    const uint4 v = *(const uint4*)(wp + p * 8);
    bf16_t* dst = w + (size_t)m * K + k;
    if (k + 8 <= K && (((uintptr_t)dst) & 15) == 0) {
        *(uint4*)dst = v;
    } else {
        const uint32_t e[4] = {v.x, v.y, v.z, v.w};
        for (int j = 0; j < 8 && k + j < K; ++j) dst[j] = (bf16_t)(e[j >> 1] >> (16 * (j & 1)));
    }
}

// w [M, K] row-major from wp as vt_pack_matrix_bf16 made it
extern "C" int vt_unpack_matrix_bf16(const void* wp, void* w, int M, int K, hipStream_t stream) {
    VT_REQUIRE(M > 0 && K > 0, "vt_unpack_matrix_bf16: bad sizes M=%d K=%d", M, K);
    VT_REQUIRE((((uintptr_t)wp) & 15) == 0, "vt_unpack_matrix_bf16: the packed matrix must be 16-byte aligned");
    const int KT = pk_cols(K) / 32;
    const size_t pieces = (size_t)(pk_rows(M) / 16) * KT * 64;
    unpack_matrix_kernel<<<(unsigned)((pieces + 255) / 256), 256, 0, stream>>>((const bf16_t*)wp, (bf16_t*)w, M, K, KT, pieces);
    VT_CHECK_LAUNCH("vt_unpack_matrix_bf16");
    return 0;
}

__device__ __forceinline__ unsigned pack_bf16x2(float a, float b) { return vt_pack2(a, b); }

// x[row][k .. k + 8); beyond the end of the row its last eight values are read instead (W is zero there)
__device__ __forceinline__ bf16x8_t load_x(const bf16_t* row, int k, int K) {
    Frag f;
    f.u = *(const uint4*)(row + min(k, K - 8));
    return f.v;
}

// ---------------------------------------------------------------------------
// An RMSNorm handed from the product in front of it to the product behind it, so that it is no kernel of its own
// and the product behind it reads its tokens in bf16 like any other.
// The product in front (one that adds its result to the residual stream h) is the producer: beside h it writes
// xn = bf16(h * gain) for the norm's gains, and each of its blocks writes its features' share of every row's sum
// of h^2 to ssq_out[block][row].  The product behind is the consumer: its tokens are xn, it adds up the shares in
// block order and multiplies its sums by 1/sqrt(sum / width + eps), which is where the norm's division belongs
// since it is the same for a whole row.  The shares are added in a fixed order: the result does not depend on
// which block finished first.  Rows of ssq are SSQ_STRIDE(N) floats apart.
struct NormLink {
    bf16_t* xn_out;            // producer: [N][Mout], or null
    const float* gain_next;    //           [Mout]
    float* ssq_out;            //           [blocks][stride]
    const float* ssq_in;       // consumer: [n_ssq][stride], or null
    int n_ssq;
    float eps;
};
#define SSQ_STRIDE(N) ((N) <= 16 ? 16 : 64)

// Consumer of a NormLink at 17 to 64 rows (shares 64 floats apart): 1/sqrt(sum / K + eps) of every row into
// rinv[64], by all THREADS of the block.  Thread t adds rows 4 (t % 16) .. + 3 of shares t / 16, t / 16 + THREADS / 16,
// ... in that order (eight loads in flight at a time), the four lanes of a wave with the same rows add up, then the
// waves in wave order: a fixed order, whatever finished first.  part: [THREADS / 64][16]; ends with a barrier.
template <int THREADS>
__device__ __forceinline__ void link_row_scales(const NormLink& link, int K, float4 (*part)[16], float* rinv) {
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    float4 sh = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int b0 = tid >> 4; b0 < link.n_ssq; b0 += 8 * (THREADS / 16)) {
        float4 t4[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {       // eight loads asked for together, then added in order
            const int b = b0 + j * (THREADS / 16);
            t4[j] = b < link.n_ssq ? *(const float4*)(link.ssq_in + (size_t)b * 64 + (tid & 15) * 4)
                                   : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) { sh.x += t4[j].x; sh.y += t4[j].y; sh.z += t4[j].z; sh.w += t4[j].w; }
    }
#pragma unroll
    for (int o = 16; o < 64; o <<= 1) {
        sh.x += __shfl_xor(sh.x, o, 64); sh.y += __shfl_xor(sh.y, o, 64);
        sh.z += __shfl_xor(sh.z, o, 64); sh.w += __shfl_xor(sh.w, o, 64);
    }
    if (lane < 16) part[wv][lane] = sh;
    __syncthreads();
    if (tid < 64) {
        float tot = 0.f;
        for (int q = 0; q < THREADS / 64; ++q) tot += ((const float*)&part[q][0])[tid];
        rinv[tid] = 1.0f / sqrtf(tot / (float)K + link.eps);
    }
    __syncthreads();
}

// ---------------------------------------------------------------------------
// Up to 16 tokens: a block owns one tile row of W (16 features; two for the gated product) and all of k, which
// its WPB waves split; the tokens are the B operand.  U tiles are in flight per wave and matrix.
//
// The B fragment of a tile is 64 bytes of each of 16 token rows.  Read as the matrix instruction wants it (lane
// 16 g + r: row r, piece g) the four pieces of a row sit in lanes 16 apart and the cache sees 64 separate
// accesses; so lane l reads piece l % 4 of row l / 4 instead (the four lanes of a row are neighbours, 16 accesses
// of 64 bytes) and hands it through LDS to the lane that needs it.  The slots of a piece index are 17 apart, which
// keeps writes and reads off each other's banks; each wave has two such buffers of its own and no one else's, so
// nothing but the order of its own LDS operations keeps them consistent.
// ---------------------------------------------------------------------------
// NORM: the tokens come as the fp32 residual stream h [N][K] with the gains of an RMSNorm: the kernel reads h * gain
// (rounded to bf16) as its tokens, adds up h^2 on the way (every block walks all of k, so every block has the whole
// sum of every row) and multiplies the finished sums by 1/sqrt(mean(h^2) + eps): the norm costs no launch and no
// pass over h of its own.  resid: fp32 [N][Mout] that the result is added to (y may be resid itself).
// PARTS = 2: a block owns half a tile row, 8 features; the lanes of the other 8 rows load nothing and multiply zeros.
// Twice the blocks, for matrices with so few tile rows that whole ones would leave more than half of the compute
// units without a block (Qwen2-1.5B's q/k/v, output and down projections: 128, 96 and 96 tile rows; a decoding step at
// batch 8 1.42 -> 1.35 ms).  A tile's 16 rows x 32 k are packed as four stretches of 256 bytes, the first half of each
// being rows 0 to 7: a half block reads whole 128-byte lines, and no line that its other half reads.  (Quarters read
// half lines: 1.69 ms.  Halves for matrices of 224 and 288 tile rows, which fill the compute units unevenly: 3.05 ->
// 3.36 ms at Qwen2-7B's sizes.  Halves with 8 waves a block where whole tile rows take 16: 1.39 ms.)
template <int WPB, bool SWIGLU, bool NORM, typename TO, int PARTS = 1>
__global__ __launch_bounds__(WPB * 64) void gemm_skinny_kernel(const void* __restrict__ xin, const bf16_t* __restrict__ wp,
                                                              const float* __restrict__ bias, TO* __restrict__ y, int N,
                                                              int Mout, int K, int KT, int up_tiles,
                                                              const float* __restrict__ gain, float eps,
                                                              const float* resid, NormLink link) {
    constexpr int NW = SWIGLU ? 2 : 1;
    constexpr int U = NORM ? 2 : 4;     // tiles in flight (fp32 tokens take three times the registers: measured)
    __shared__ float red[NW][WPB][256];
    __shared__ uint4 xt[WPB][NORM ? 2 : 4][4 * 17];     // per wave: two exchange buffers of one tile (NORM) or of a pair
    __shared__ float ssq[NORM ? WPB : 1][16];
    __shared__ float4 ssq_part[WPB][4];                       // consumer of a NormLink: the waves' sums of shares
    const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63;
    const int r = lane & 15, g = lane >> 4;
    static_assert(!(PARTS > 1 && SWIGLU), "the gated product has tile rows enough");
    constexpr int RB = 16 / PARTS;                    // features of the block
    const int mt = blockIdx.x / PARTS, hb = blockIdx.x % PARTS;
    const bool w_on = PARTS == 1 || r / RB == hb;     // this lane's row of W is one of the block's
    auto load_w = [&](const bf16_t* p) __attribute__((always_inline)) { return w_on ? load_w_once(p) : make_uint4(0u, 0u, 0u, 0u); };
    // Consumer of a NormLink: thread t adds up rows 4 (t % 4) .. + 3 of shares t / 4, t / 4 + threads / 4, ...; the
    // first two loads are asked for here, ahead of everything, and used at the end.
    float4 sh0 = make_float4(0.f, 0.f, 0.f, 0.f), sh1 = sh0;
    if constexpr (!NORM) {
        if (link.ssq_in) {
            const int b0 = tid >> 2, b1 = b0 + WPB * 16;
            if (b0 < link.n_ssq) sh0 = *(const float4*)(link.ssq_in + (size_t)b0 * 16 + (tid & 3) * 4);
            if (b1 < link.n_ssq) sh1 = *(const float4*)(link.ssq_in + (size_t)b1 * 16 + (tid & 3) * 4);
        }
    }
    const int t_begin = (int)(((long long)wv * KT) / WPB), t_end = (int)(((long long)(wv + 1) * KT) / WPB);
    const bf16_t* wbase[NW];
    wbase[0] = wp + ((size_t)mt * KT * 64 + lane) * 8;
    if (SWIGLU) wbase[1] = wp + ((size_t)(mt + up_tiles) * KT * 64 + lane) * 8;
    // bf16 tokens: lane l reads piece l % 4 (8 values) of row l / 4 and writes one 16-byte slot.
    const bf16_t* xrow = (const bf16_t*)xin + (size_t)min(lane >> 2, N - 1) * K;
    const int xpiece = (lane & 3) * 8;
    const int wslot = (lane & 3) * 17 + (lane >> 2), rslot = g * 17 + r;
    // fp32 residual stream (NORM): a row's 32 values of a tile are 128 bytes, so lane l reads quarter-piece l % 8
    // (4 values) of rows l / 8 and l / 8 + 8, two loads of eight whole cache lines, and writes two 8-byte halves
    // of slots.
    const float* hrow_a = (const float*)xin + (size_t)min(lane >> 3, N - 1) * K;
    const float* hrow_b = (const float*)xin + (size_t)min((lane >> 3) + 8, N - 1) * K;
    const int hq = (lane & 7) * 4;
    uint2* const xt2 = (uint2*)&xt[wv][0][0];
    const int hslot_a = 2 * ((lane & 7) / 2 * 17 + (lane >> 3)) + (lane & 1), hslot_b = hslot_a + 16;
    // Lanes whose row is no token load nothing: the cache is asked for one line per row that exists, which is worth
    // a fifth of the gate/up product's time at 8 rows.  (For bf16 tokens the same costs more than it saves.)
    const bool has_a = (lane >> 3) < N, has_b = (lane >> 3) + 8 < N;
    float ss_a = 0.f, ss_b = 0.f;
    // A piece in two steps, its loads and (with the norm) its arithmetic, so that the loads of all the tiles of a turn
    // are asked for before the first tile's arithmetic; kept in one step, the compiler leaves a tile's arithmetic next
    // to its loads, and the tiles of a turn wait for memory one after the other (qkv at 7B sizes: 13.8 -> 12.1 us with
    // one token, 13.9 -> 13.0 with 8; a decoding step 3.46 -> 3.44 ms at batch 8, 3.22 -> 3.18 at batch 1).
    struct Piece { Frag f; uint2 a, b; float4 ha, hb, gg; };
    auto load_piece = [&](int t) __attribute__((always_inline)) {
        Piece p;
        if constexpr (NORM) {
            const int kc = min(t * 32 + hq, K - 4);
            p.ha = p.hb = p.gg = make_float4(0.f, 0.f, 0.f, 0.f);
            if (has_a) { p.ha = *(const float4*)(hrow_a + kc); p.gg = *(const float4*)(gain + kc); }
            if (has_b) p.hb = *(const float4*)(hrow_b + kc);
        } else {
            p.f.v = load_x(xrow, t * 32 + xpiece, K);
        }
        return p;
    };
    auto finish_piece = [&](Piece& p, int t) __attribute__((always_inline)) {
        if constexpr (NORM) {
            const float4 ha = p.ha, hb = p.hb, gg = p.gg;
            if (t * 32 + hq < K) {
                ss_a += (ha.x * ha.x + ha.y * ha.y) + (ha.z * ha.z + ha.w * ha.w);
                ss_b += (hb.x * hb.x + hb.y * hb.y) + (hb.z * hb.z + hb.w * hb.w);
            }
            p.a = make_uint2(pack_bf16x2(ha.x * gg.x, ha.y * gg.y), pack_bf16x2(ha.z * gg.z, ha.w * gg.w));
            p.b = make_uint2(pack_bf16x2(hb.x * gg.x, hb.y * gg.y), pack_bf16x2(hb.z * gg.z, hb.w * gg.w));
        }
    };
    // through the wave's LDS buffer `b` to the lane that needs it
    auto exchange = [&](Piece& p, int b) __attribute__((always_inline)) {
        if constexpr (NORM) {
            xt2[b * (2 * 4 * 17) + hslot_a] = p.a;
            xt2[b * (2 * 4 * 17) + hslot_b] = p.b;
        } else {
            xt[wv][b][wslot] = p.f.u;
        }
        wave_lds_order();
        p.f.u = xt[wv][b][rslot];
        wave_lds_order();       // and the next write to this buffer after these reads
    };
    f32x4_t acc[NW];
#pragma unroll
    for (int a = 0; a < NW; ++a) acc[a] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    int t = t_begin;
    if constexpr (!NORM) {
        // bf16 tokens by pairs of k tiles: a token's 64 values of a pair are one cache line, so lane l reads piece
        // l % 8 (8 values) of row l / 8 (and of row l / 8 + 8 if there are more than 8 tokens): eight accesses of a
        // whole line per load, where a tile at a time is sixteen of half a line, and it is the number of accesses
        // that the first-level cache limits.  The waves split k in pairs (KT is a multiple of 4).
        const int KP = KT >> 1;
        const int p_begin = (int)(((long long)wv * KP) / WPB), p_end = (int)(((long long)(wv + 1) * KP) / WPB);
        const bf16_t* xr_a = (const bf16_t*)xin + (size_t)min(lane >> 3, N - 1) * K;
        const bf16_t* xr_b = (const bf16_t*)xin + (size_t)min((lane >> 3) + 8, N - 1) * K;
        const int xpc = (lane & 7) * 8;
        const bool two = N > 8;
        uint4* const xw = &xt[wv][0][0];                // [2 buffers][2 tiles][4 * 17]
        const int ws = ((lane & 7) >> 2) * 68 + (lane & 3) * 17 + (lane >> 3);
        constexpr int UP = 2;                           // pairs in flight
        auto pair_exchange = [&](const Frag& xa, const Frag& xb, int b, Frag& f0, Frag& f1) __attribute__((always_inline)) {
            uint4* const buf = xw + b * 136;
            buf[ws] = xa.u;
            if (two) buf[ws + 8] = xb.u;                // (rows from the number of tokens on are never stored)
            wave_lds_order();
            f0.u = buf[rslot];
            f1.u = buf[68 + rslot];
            wave_lds_order();                           // and the next write to this buffer after these reads
        };
        int p = p_begin;
        for (; p + UP <= p_end; p += UP) {
            Frag wa[NW][2 * UP], xa[UP], xb[UP], xf[2 * UP];
#pragma unroll
            for (int up = 0; up < UP; ++up) {
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int a = 0; a < NW; ++a)
                        wa[a][2 * up + u].u = load_w(wbase[a] + (size_t)(2 * (p + up) + u) * PK_TILE);
                xa[up].v = load_x(xr_a, (p + up) * 64 + xpc, K);
                if (two) xb[up].v = load_x(xr_b, (p + up) * 64 + xpc, K);
            }
#pragma unroll
            for (int up = 0; up < UP; ++up) pair_exchange(xa[up], xb[up], up & 1, xf[2 * up], xf[2 * up + 1]);
#pragma unroll
            for (int u = 0; u < 2 * UP; ++u)
#pragma unroll
                for (int a = 0; a < NW; ++a)
                    acc[a] = VT_MFMA_16X16X32(wa[a][u].v, xf[u].v, acc[a]);
        }
        for (; p < p_end; ++p) {
            Frag wa[NW][2], xa, xb, xf[2];
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int a = 0; a < NW; ++a) wa[a][u].u = load_w(wbase[a] + (size_t)(2 * p + u) * PK_TILE);
            xa.v = load_x(xr_a, p * 64 + xpc, K);
            if (two) xb.v = load_x(xr_b, p * 64 + xpc, K);
            pair_exchange(xa, xb, 0, xf[0], xf[1]);
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int a = 0; a < NW; ++a)
                    acc[a] = VT_MFMA_16X16X32(wa[a][u].v, xf[u].v, acc[a]);
        }
        t = t_end;      // (nothing left for the loops below)
    }
    for (; t + U <= t_end; t += U) {
        Frag wa[NW][U];
        Piece xa[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int a = 0; a < NW; ++a) wa[a][u].u = load_w(wbase[a] + (size_t)(t + u) * PK_TILE);
            xa[u] = load_piece(t + u);
        }
        if constexpr (NORM) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            finish_piece(xa[u], t + u);
            exchange(xa[u], u & 1);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int a = 0; a < NW; ++a)
                acc[a] = VT_MFMA_16X16X32(wa[a][u].v, xa[u].f.v, acc[a]);
    }
    for (; t < t_end; ++t) {
        Piece xa = load_piece(t);
        finish_piece(xa, t);
        exchange(xa, 0);
#pragma unroll
        for (int a = 0; a < NW; ++a) {
            Frag wa;
            wa.u = load_w(wbase[a] + (size_t)t * PK_TILE);
            acc[a] = VT_MFMA_16X16X32(wa.v, xa.f.v, acc[a]);
        }
    }
    if constexpr (NORM) {
        // the eight lanes of a row hold its quarter-pieces: add them, then the waves' shares in wave order
#pragma unroll
        for (int o = 1; o < 8; o <<= 1) {
            ss_a += __shfl_xor(ss_a, o, 64);
            ss_b += __shfl_xor(ss_b, o, 64);
        }
        if ((lane & 7) == 0) { ssq[wv][lane >> 3] = ss_a; ssq[wv][(lane >> 3) + 8] = ss_b; }
    }
    // acc[a][e] is feature 16 mt + 4 g + e of token r.  Sum the waves in wave order.
#pragma unroll
    for (int a = 0; a < NW; ++a)
#pragma unroll
        for (int e = 0; e < 4; ++e) red[a][wv][lane * 4 + e] = acc[a][e];
    const bool consumes = !NORM && link.ssq_in != nullptr;
    if constexpr (!NORM) {
        if (consumes) {
            float4 sh = make_float4(sh0.x + sh1.x, sh0.y + sh1.y, sh0.z + sh1.z, sh0.w + sh1.w);
            for (int b = (tid >> 2) + 2 * WPB * 16; b < link.n_ssq; b += WPB * 16) {      // (more than 2 x threads / 4 shares)
                const float4 t4 = *(const float4*)(link.ssq_in + (size_t)b * 16 + (tid & 3) * 4);
                sh.x += t4.x; sh.y += t4.y; sh.z += t4.z; sh.w += t4.w;
            }
            // the 16 lanes of a wave that hold the same four rows; every lane ends with the same sum
#pragma unroll
            for (int o = 4; o < 64; o <<= 1) {
                sh.x += __shfl_xor(sh.x, o, 64); sh.y += __shfl_xor(sh.y, o, 64);
                sh.z += __shfl_xor(sh.z, o, 64); sh.w += __shfl_xor(sh.w, o, 64);
            }
            if (lane < 4) ssq_part[wv][lane] = sh;
        }
    }
    __syncthreads();
    for (int c = tid; c < 256; c += WPB * 64) {
        const int ln = c >> 2, e = c & 3;
        const int m = mt * 16 + 4 * (ln >> 4) + e, n = ln & 15;
        float v = 0.f, u = 0.f;
        for (int q = 0; q < WPB; ++q) v += red[0][q][c];
        if (SWIGLU)
            for (int q = 0; q < WPB; ++q) u += red[NW - 1][q][c];
        float sq = 0.f;
        if (m < Mout && n < N && (PARTS == 1 || (4 * (ln >> 4) + e) / RB == hb)) {
            if constexpr (NORM) {
                float tot = 0.f;
                for (int q = 0; q < WPB; ++q) tot += ssq[q][n];
                const float rinv = 1.0f / sqrtf(tot / (float)K + eps);
                v *= rinv;
                u *= rinv;
            } else if (consumes) {
                float tot = 0.f;
                const float* col = (const float*)&ssq_part[0][0] + n;       // [waves][16 rows]
                for (int q = 0; q < WPB; ++q) tot += col[q * 16];
                const float rinv = 1.0f / sqrtf(tot / (float)K + link.eps);
                v *= rinv;
                u *= rinv;
            }
            if (SWIGLU) v = v / (1.f + expf(-v)) * u;
            else if (bias) v += bias[m];
            if (resid) v += resid[(size_t)n * Mout + m];
            store_f32<TO>(y, (size_t)n * Mout + m, v);
            if (link.xn_out) {
                link.xn_out[(size_t)n * Mout + m] = f32_to_bf16(v * link.gain_next[m]);
                sq = v * v;
            }
        }
        if (link.xn_out) red[0][0][c] = sq;       // (this thread alone has read slot c)
    }
    if (link.xn_out) {
        // this block's share of the rows' sums of squares: 16 features per row, added in feature order
        __syncthreads();
        if (tid < 16) {
            float tot = 0.f;
            for (int gg = 0; gg < 4; ++gg)
                for (int e = 0; e < 4; ++e) tot += red[0][0][((gg * 16 + tid) << 2) + e];
            link.ssq_out[(size_t)blockIdx.x * 16 + tid] = tot;
        }
    }
}

// ---------------------------------------------------------------------------
// 17 to 64 tokens per block (a large decoding batch, a short portion): a block of WM waves takes 16*WM*R features
// and 64 tokens.  The tokens' values pass through LDS once per block, so they cost a fraction of W's traffic
// instead of a multiple; each wave streams the tiles of its own R tile rows of W from memory into registers,
// MID_WD stages (of 128 k, four tiles) ahead.  For matrices with few rows the k range is split over blockIdx.z and
// the partial sums (fp32, [split][N][M]) are added by sum_partials_kernel in split order.
//
// The tokens are brought by one more wave that does nothing else: it loads them from memory straight into LDS
// (global_load_lds, 16 bytes per lane, MID_XST - 1 stages ahead of the stage that is multiplied), so that neither a
// stage's tokens nor its rows of W have to come within the time of one stage, which is shorter than the way from
// memory.  A wave's load writes 64 consecutive 16-byte slots of LDS, one per lane, and each lane chooses what it
// reads, so the layout is made by the addresses: a token's 128 values of a stage are 16 slots, and chunk c sits in
// slot c ^ (token % 16), which keeps the sixteen rows of an operand tile on different banks without padding.
// Only that wave has such loads in flight; the others' waits for their rows of W count what they asked for.
// ---------------------------------------------------------------------------
#define MID_BK 128                 // k values per stage = PK_KPAD: a stage never leaves the packed matrix
#define MID_KU (MID_BK / 32)       // tiles along k per stage
#define MID_XST 3                  // stages of tokens in LDS
#define MID_WD 2                   // stages of W in registers (3 and 4: the same times)
// bytes of a stage of NTT token tiles in LDS, and of a block's stages
#define MID_STAGE_BYTES(NTT) ((NTT) * 16 * MID_BK * 2)
#define MID_LDS_BYTES(NTT) (MID_XST * MID_STAGE_BYTES(NTT))

// WM waves that multiply per block (and one that loads the tokens): the host picks it so that the blocks fill the
// compute units evenly.  NTT: token tiles of 16 per block, 4 (up to 64 tokens in a launch) or 8 (more: W is then
// read once per 128 tokens).
// ONCE: one block of tokens, so that no other block reads these rows of W again (see load_w_once).
template <int R, bool SWIGLU, int WM, typename TO, bool ONCE, int NTT>
__global__ __launch_bounds__((WM + 1) * 64) void gemm_mid_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wp,
                                                            const float* __restrict__ bias, TO* __restrict__ y,
                                                            float* __restrict__ partial, int N, int Mout, int K, int KT,
                                                            int up_tiles, int k_per_split, NormLink link) {
    constexpr int NW = SWIGLU ? 2 : 1;
    constexpr int RW = R * NW;
    extern __shared__ __attribute__((aligned(1024))) bf16_t xs[];      // [MID_XST][NTT * 16 * MID_BK]
    __shared__ float4 link_part[WM + 1][16];
    __shared__ float link_rinv[64];
    const int tid = threadIdx.x, wv = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int r = lane & 15, g = lane >> 4;
    // behind a norm that the product in front has prepared (up to 64 tokens): the rows' 1/sqrt(mean + eps)
    const bool consumes = link.ssq_in != nullptr;
    const int n0 = blockIdx.y * (NTT * 16);
    const int k_begin = blockIdx.z * k_per_split, k_end = min(pk_cols(K), k_begin + k_per_split);
    const int S = k_begin < k_end ? (k_end - k_begin + MID_BK - 1) / MID_BK : 0;      // stages of this block
    const bool loader = wv == WM;
    const int mw = loader ? 0 : wv;                       // (the loading wave's sums are never stored)
    const int mt0 = (blockIdx.x * WM + mw) * R;
    const int m_tiles = pk_rows(Mout) >> 4;
    f32x4_t acc[RW][NTT];
#pragma unroll
    for (int a = 0; a < RW; ++a)
#pragma unroll
        for (int i = 0; i < NTT; ++i) acc[a][i] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

    if (loader) {
        // A stage is 4 NTT loads of four tokens each: lane l brings chunk (l % 16) ^ (token % 16) of token 4 i + l / 16
        // to slot l.  Tokens beyond the last repeat it; k beyond the row reads the row's last chunk again (the
        // packed matrix is zero there).
        constexpr int NL = 4 * NTT;      // loads per stage
        static_assert(NL < 64, "the wait for a stage counts its loads in six bits");
        const unsigned lds0 = lds_address(xs);
        unsigned tok_off[NL];
        int chunk_k[4];
#pragma unroll
        for (int i = 0; i < NL; ++i) tok_off[i] = (unsigned)min(4 * i + (lane >> 4), N - 1 - n0) * (unsigned)K * 2u;
        const bf16_t* const xblk = x + (size_t)n0 * K;       // (32-bit offsets from the block's first token)
#pragma unroll
        for (int i = 0; i < 4; ++i) chunk_k[i] = 8 * ((lane & 15) ^ ((4 * i + (lane >> 4)) & 15));
        auto issue = [&](int st) __attribute__((always_inline)) {
            const int k0 = k_begin + st * MID_BK;
            const unsigned dst = lds0 + (unsigned)(st % MID_XST) * MID_STAGE_BYTES(NTT);
#pragma unroll
            for (int i = 0; i < NL; ++i)
                load_to_lds16(xblk, tok_off[i] + 2u * (unsigned)min(k0 + chunk_k[i & 3], K - 8), dst + i * 1024);
        };
#pragma unroll
        for (int st = 0; st < MID_XST - 1; ++st)
            if (st < S) issue(st);
        if (consumes) link_row_scales<(WM + 1) * 64>(link, K, link_part, link_rinv);
        for (int st = 0; st < S; ++st) {
            // stage st has landed when no more loads are in flight than those of the stages asked for after it
            static_assert(MID_XST == 3, "at most one stage is asked for behind the one that is waited for");
            const int later = min(st + MID_XST - 1, S) - (st + 1);
            if (later == 1) wait_loads<NL>();
            else wait_loads<0>();
            __syncthreads();
            // every wave has left stage st - 1, whose buffer the stage MID_XST - 1 ahead takes
            if (st + MID_XST - 1 < S) issue(st + MID_XST - 1);
        }
        return;
    }

    // this wave's tile rows; beyond the matrix the last one again (its results are not stored)
    const bf16_t* wbase[RW];
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const int mt = min(mt0 + j, m_tiles - 1);
        wbase[j] = wp + ((size_t)mt * KT * 64 + lane) * 8;
        if (SWIGLU) wbase[R + j] = wp + ((size_t)(mt + up_tiles) * KT * 64 + lane) * 8;
    }
    Frag wst[MID_WD][RW][MID_KU];
    auto fetch_w = [&](Frag (&dst)[RW][MID_KU], int st) __attribute__((always_inline)) {
        const size_t t0 = (size_t)((k_begin + st * MID_BK) >> 5) * PK_TILE;
#pragma unroll
        for (int u = 0; u < MID_KU; ++u)
#pragma unroll
            for (int a = 0; a < RW; ++a) {
                const bf16_t* src = wbase[a] + t0 + (size_t)u * PK_TILE;
                if constexpr (ONCE) dst[a][u].u = load_w_once(src);
                else dst[a][u].u = *(const uint4*)src;
            }
    };
    // token 16 i + r's chunk 4 u + g of stage buffer b
    const bf16_t* const xrd = xs + r * MID_BK;
    int xsw[MID_KU];
#pragma unroll
    for (int u = 0; u < MID_KU; ++u) xsw[u] = ((4 * u + g) ^ r) << 3;
    auto multiply = [&](const Frag (&wf)[RW][MID_KU], int st) __attribute__((always_inline)) {
        const bf16_t* const xb = xrd + (st % MID_XST) * (NTT * 16 * MID_BK);
        // 16 token operands are asked for together, ahead of their products: a wave is alone on its SIMD when a
        // block has a compute unit to itself, and read two at a time the way from LDS is waited for eight times
        constexpr int UB = 16 / NTT;     // k tiles whose operands are read together
#pragma unroll
        for (int u0 = 0; u0 < MID_KU; u0 += UB) {
            Frag xf[UB][NTT];
#pragma unroll
            for (int u = 0; u < UB; ++u)
#pragma unroll
                for (int i = 0; i < NTT; ++i) xf[u][i].u = *(const uint4*)(xb + i * 16 * MID_BK + xsw[u0 + u]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < UB; ++u)
#pragma unroll
                for (int i = 0; i < NTT; ++i)
#pragma unroll
                    for (int a = 0; a < RW; ++a)
                        acc[a][i] = VT_MFMA_16X16X32(wf[a][u0 + u].v, xf[u][i].v, acc[a][i]);
        }
    };
#pragma unroll
    for (int d = 0; d < MID_WD; ++d)
        if (d < S) fetch_w(wst[d], d);
    // (here, behind the first stages' loads, the shares' way from the second-level cache costs nothing)
    if (consumes) link_row_scales<(WM + 1) * 64>(link, K, link_part, link_rinv);
    // MID_WD stages per turn so that the register stages rotate without copies; one barrier per stage, which the
    // loading wave meets when the stage's tokens have landed
    for (int st = 0; st < S; st += MID_WD) {
#pragma unroll
        for (int d = 0; d < MID_WD; ++d) {
            if (st + d < S) {
                __syncthreads();
                multiply(wst[d], st + d);
                if (st + d + MID_WD < S) fetch_w(wst[d], st + d + MID_WD);
            }
        }
    }

    // acc[a][i][e] is feature 16 (mt0 + j) + 4 g + e (j = a mod R) of token n0 + 16 i + r
    const bool split = gridDim.z > 1;
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
        for (int i = 0; i < NTT; ++i) {
            const int n = n0 + i * 16 + r;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int m = (mt0 + j) * 16 + 4 * g + e;
                if (m >= Mout || n >= N) continue;
                float v = acc[j][i][e];
                if (consumes) v *= link_rinv[(i * 16 + r) & 63];      // (a norm is taken over with up to 64 tokens)
                if (SWIGLU) {
                    float u = acc[R + j][i][e];
                    if (consumes) u *= link_rinv[(i * 16 + r) & 63];
                    v = v / (1.f + expf(-v)) * u;
                } else if (bias && blockIdx.z == 0) {
                    v += bias[m];
                }
                if (split) partial[((size_t)blockIdx.z * N + n) * Mout + m] = v;
                else store_f32<TO>(y, (size_t)n * Mout + m, v);
            }
        }
}

// ---------------------------------------------------------------------------
// 17 to 64 tokens, k not split over blocks: as in the few-row kernel a block owns one tile row of W (16 features)
// and all of k, which its WPB waves split, and the waves' sums meet in LDS in wave order; each wave multiplies a
// tile of W with NT token tiles of 16 rows, whose pieces it reads row by row (16 accesses of 64 bytes per tile) and
// hands to their lanes through LDS of its own.  Every block reads all the tokens (64 x k values from the second-level
// cache, four times the bytes of its share of W); in exchange nothing is left to add up afterwards, so the result can
// take a residual with it, and a matrix of 224 tile rows fills the compute units without a split.
// ---------------------------------------------------------------------------
// slots (16 bytes) of one k tile of a wave's exchange buffer: NT token tiles of 4 pieces x 17 rows, and 8 more where
// that is a multiple of 16, so that the two tiles of a pair, which a wave writes together, lie 32 banks apart
template <int NT>
__host__ __device__ constexpr int rows_tile_slots() { return NT * 4 * 17 + ((NT * 4 * 17) % 16 == 0 ? 8 : 0); }

template <int WPB, int NT>
__host__ __device__ constexpr int rows_lds_bytes() {
    constexpr int exchange = WPB * 2 * rows_tile_slots<NT>() * 16, sums = WPB * NT * 256 * 4;
    return exchange > sums ? exchange : sums;
}

// (The exchange buffers leave room for two blocks of 8 waves per compute unit: four waves per SIMD.  Saying so keeps
// the compiler from giving up loads in flight for a fifth and sixth wave that can never come.)
template <int WPB, int NT, int R, typename TO>
__global__ __launch_bounds__(WPB * 64) __attribute__((amdgpu_waves_per_eu(2, 4))) void gemm_rows_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wp,
                                                            const float* __restrict__ bias, TO* __restrict__ y, int N,
                                                            int Mout, int K, int KT, const float* resid, NormLink link) {
    extern __shared__ __attribute__((aligned(16))) unsigned char rows_lds[];
    __shared__ float4 link_part[WPB][16];
    __shared__ float link_rinv[64];
    const int tid = threadIdx.x, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = tid & 63;
    const int r = lane & 15, g = lane >> 4;
    const int m_tiles = (Mout + 15) >> 4;
    const bool consumes = link.ssq_in != nullptr;
    if (consumes) link_row_scales<WPB * 64>(link, K, link_part, link_rinv);
    float ssq_acc = 0.f;        // producer: row tid's sum of squares over this block's features
    // the waves split k in pairs of tiles (KT is a multiple of 4): a token's 64 values of a pair are one cache line
    const int KP = KT >> 1;
    const int p_begin = (int)(((long long)wv * KP) / WPB), p_end = (int)(((long long)(wv + 1) * KP) / WPB);
    // this block's R tile rows; beyond the matrix the last one again (its results are not stored)
    const bf16_t* wbase[R];
#pragma unroll
    for (int j = 0; j < R; ++j) wbase[j] = wp + ((size_t)min((int)blockIdx.x * R + j, m_tiles - 1) * KT * 64 + lane) * 8;
    // Lane l reads piece l % 8 (8 values) of rows l / 8 and l / 8 + 8 of each token tile: eight lanes read a whole
    // cache line, a load is eight accesses (by 32 values, a tile at a time, it would be sixteen of half a line, and
    // it is the number of accesses that the first-level cache limits).  Pieces 0..3 belong to the pair's first tile.
    const bf16_t* xrow[NT][2];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
        xrow[i][0] = x + (size_t)min(16 * i + (lane >> 3), N - 1) * K;
        xrow[i][1] = x + (size_t)min(16 * i + (lane >> 3) + 8, N - 1) * K;
    }
    const int xpiece = (lane & 7) * 8;
    constexpr int TS = rows_tile_slots<NT>();
    uint4* const xt = (uint4*)rows_lds + (size_t)wv * 2 * TS;      // this wave's [2 tiles][NT][4 * 17] slots
    const int wslot = ((lane & 7) >> 2) * TS + (lane & 3) * 17 + (lane >> 3), rslot = g * 17 + r;
    f32x4_t acc[R][NT];
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
        for (int i = 0; i < NT; ++i) acc[j][i] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    // Blocks that start together would walk the tokens' lines in step and meet at the same channels of the
    // second-level cache: every block starts at another pair of its waves' ranges.
    const int p_len = p_end - p_begin;
    int p = p_begin + (p_len > 0 ? (int)(blockIdx.x % (unsigned)p_len) : 0);
    for (int q = 0; q < p_len; ++q, p = (p + 1 < p_end) ? p + 1 : p_begin) {
        Frag wa[2][R], xa[NT][2];
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int j = 0; j < R; ++j) wa[u][j].u = load_w_once(wbase[j] + (size_t)(2 * p + u) * PK_TILE);
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            xa[i][0].v = load_x(xrow[i][0], p * 64 + xpiece, K);
            xa[i][1].v = load_x(xrow[i][1], p * 64 + xpiece, K);
        }
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            xt[i * 4 * 17 + wslot] = xa[i][0].u;
            xt[i * 4 * 17 + wslot + 8] = xa[i][1].u;
        }
        wave_lds_order();
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int i = 0; i < NT; ++i) {
                Frag xf;
                xf.u = xt[u * TS + i * 4 * 17 + rslot];
#pragma unroll
                for (int j = 0; j < R; ++j)
                    acc[j][i] = VT_MFMA_16X16X32(wa[u][j].v, xf.v, acc[j][i]);
            }
        wave_lds_order();       // the next pair is written after these reads
    }
    // acc[j][i][e] is feature 16 (R blockIdx.x + j) + 4 g + e of token 16 i + r.  The waves' sums take the exchange
    // buffers' place, one tile row at a time.
    float* const red = (float*)rows_lds;            // [WPB][NT][256]
#pragma unroll
    for (int j = 0; j < R; ++j) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NT; ++i) *(f32x4_t*)&red[((size_t)wv * NT + i) * 256 + lane * 4] = acc[j][i];
        __syncthreads();
        const int mt = blockIdx.x * R + j;
        for (int c = tid; c < NT * 256; c += WPB * 64) {
            const int i = c >> 8, cc = c & 255, ln = cc >> 2, e = cc & 3;
            const int m = mt * 16 + 4 * (ln >> 4) + e, n = 16 * i + (ln & 15);
            float v = 0.f, sq = 0.f;
            for (int q = 0; q < WPB; ++q) v += red[((size_t)q * NT + i) * 256 + cc];
            if (m < Mout && n < N) {
                if (consumes) v *= link_rinv[n];
                if (bias) v += bias[m];
                if (resid) v += resid[(size_t)n * Mout + m];
                store_f32<TO>(y, (size_t)n * Mout + m, v);
                if (link.xn_out) {
                    link.xn_out[(size_t)n * Mout + m] = f32_to_bf16(v * link.gain_next[m]);
                    sq = v * v;
                }
            }
            if (link.xn_out) red[(size_t)i * 256 + cc] = sq;       // (this thread alone has read slot cc of tile i)
        }
        if (link.xn_out) {
            // this tile row's share of the rows' sums of squares: 16 features per row, added in feature order
            __syncthreads();
            if (tid < NT * 16) {
                const int i = tid >> 4, nn = tid & 15;
                for (int gg = 0; gg < 4; ++gg)
                    for (int e = 0; e < 4; ++e) ssq_acc += red[(size_t)i * 256 + (((gg * 16 + nn) << 2) + e)];
            }
        }
    }
    if (link.xn_out && tid < 64) link.ssq_out[(size_t)blockIdx.x * 64 + tid] = tid < NT * 16 ? ssq_acc : 0.f;
}

template <int WPB, int NT, int R, typename TO>
static int launch_rows(const bf16_t* x, const bf16_t* wp, const float* bias, TO* y, int N, int Mout, int K, int KT,
                       const float* resid, hipStream_t stream, const NormLink& link) {
    constexpr int lds = rows_lds_bytes<WPB, NT>();
    static bool set = false;
    if (!set) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_rows_kernel<WPB, NT, R, TO>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        VT_REQUIRE(e == hipSuccess, "vt_linear_bf16: cannot get %d bytes of LDS: %s", lds, hipGetErrorString(e));
        set = true;
    }
    const int m_tiles = (Mout + 15) / 16;
    gemm_rows_kernel<WPB, NT, R, TO><<<(m_tiles + R - 1) / R, WPB * 64, lds, stream>>>(x, wp, bias, y, N, Mout, K, KT, resid, link);
    VT_CHECK_LAUNCH("vt_linear_bf16(rows)");
    return 0;
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

// The same for up to 64 rows with a residual to add to, row by row: block (c, n) adds up columns 1024 c .. + 1023 of
// row n (four per thread), adds the residual, and as the producer of a NormLink writes bf16(y * gain) and the share
// c of row n's sum of squares (rows from N to 63: zero).
#define SUM_COLS 1024
__global__ __launch_bounds__(256) void sum_partials_rows_kernel(const float* __restrict__ partial, float* __restrict__ y,
                                                                const float* resid, int N, int M, int splits,
                                                                NormLink link) {
    __shared__ float red[4];
    const int n = blockIdx.y, tid = threadIdx.x, col = (blockIdx.x * 256 + tid) * 4;
    if (n >= N) {
        if (link.xn_out && tid == 0) link.ssq_out[(size_t)blockIdx.x * 64 + n] = 0.f;
        return;
    }
    float sq = 0.f;
    if (col < M) {          // (M is a multiple of 4)
        const size_t at = (size_t)n * M + col, all = (size_t)N * M;
        float4 a = *(const float4*)(partial + at);
        for (int s = 1; s < splits; ++s) {
            const float4 b = *(const float4*)(partial + (size_t)s * all + at);
            a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
        }
        if (resid) {
            const float4 h = *(const float4*)(resid + at);
            a.x += h.x; a.y += h.y; a.z += h.z; a.w += h.w;
        }
        *(float4*)(y + at) = a;
        if (link.xn_out) {
            const float4 gg = *(const float4*)(link.gain_next + col);
            *(uint2*)(link.xn_out + at) = make_uint2(pack_bf16x2(a.x * gg.x, a.y * gg.y), pack_bf16x2(a.z * gg.z, a.w * gg.w));
            sq = (a.x * a.x + a.y * a.y) + (a.z * a.z + a.w * a.w);
        }
    }
    if (link.xn_out) {
        sq = wave_sum(sq);
        if ((tid & 63) == 0) red[tid >> 6] = sq;
        __syncthreads();
        if (tid == 0) link.ssq_out[(size_t)blockIdx.x * 64 + n] = (red[0] + red[1]) + (red[2] + red[3]);
    }
}

// Any shape (k not a multiple of 8, or x not aligned): one thread per output, plain loop over the packed matrix.
__device__ __forceinline__ float packed_at(const bf16_t* wp, int KT, int m, int k) {
    return bf16_to_f32(wp[(((size_t)(m >> 4) * KT + (k >> 5)) * 64 + ((k & 31) >> 3) * 16 + (m & 15)) * 8 + (k & 7)]);
}
template <bool SWIGLU, typename TO>
__global__ void gemm_plain_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ wp,
                                  const float* __restrict__ bias, TO* __restrict__ y, int N, int Mout, int K, int KT,
                                  int up_tiles) {
    int m = blockIdx.x * blockDim.x + threadIdx.x, n = blockIdx.y;
    if (m >= Mout) return;
    const bf16_t* xr = x + (size_t)n * K;
    float v = 0.f, u = 0.f;
    for (int k = 0; k < K; ++k) v = fmaf(bf16_to_f32(xr[k]), packed_at(wp, KT, m, k), v);
    if (SWIGLU) {
        for (int k = 0; k < K; ++k) u = fmaf(bf16_to_f32(xr[k]), packed_at(wp, KT, up_tiles * 16 + m, k), u);
        v = v / (1.f + expf(-v)) * u;
    } else if (bias) {
        v += bias[m];
    }
    store_f32<TO>(y, (size_t)n * Mout + m, v);
}

#define ROWS_MAX 64                 // rows up to which a plain product keeps k inside a block (gemm_rows_kernel)

static int compute_units() {
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
    }
    return cus;
}

// Number of k ranges for the 64-token kernel: from the shape of W only (so the order of additions does not depend
// on the batch).  A launch lasts (rounds of blocks over the compute units) x (stages of a block); every further
// range costs half a stage for the launch that adds the partial sums, and their traffic: 64 tokens x 128 rows
// x 8 bytes per row block, where a stage reads 32 KB of W per block.
static int mid_splits(int Mout, int K, int rows_per_block) {
    const int row_blocks = (Mout + rows_per_block - 1) / rows_per_block;
    const int stages = pk_cols(K) / MID_BK, cus = compute_units();
    int best = 1;
    double best_cost = -1.;
    for (int s = 1; s <= 16 && s <= stages; ++s) {
        const long rounds = ((long)row_blocks * s + cus - 1) / cus;
        const double cost = (double)(rounds * ((stages + s - 1) / s)) + (s > 1 ? s * (0.5 + 2. * row_blocks / cus) : 0.);
        if (best_cost < 0. || cost < best_cost) { best = s; best_cost = cost; }
    }
    return best;
}

// Waves per block of the 64-token kernel when k is not split: the blocks of a launch all take the same time, so
// the launch lasts (rounds of blocks over the compute units) x (work of a block); pick the smallest product.
static int mid_waves(int Mout, int rows_per_wave, int token_blocks) {
    const int cus = compute_units();
    const int choices[5] = {3, 4, 5, 6, 8};
    int best = 4;
    long best_cost = -1;
    for (int c = 0; c < 5; ++c) {
        const int w = choices[c], rows = rows_per_wave * w;
        const long blocks = (long)((Mout + rows - 1) / rows) * token_blocks;
        const long cost = ((blocks + cus - 1) / cus) * w;
        if (best_cost < 0 || cost < best_cost) { best = w; best_cost = cost; }
    }
    return best;
}

// Up to 16 tokens: the parts of a tile row of W [Mout, .] that blocks take (gemm_skinny_kernel<PARTS>); by the shape of W
// alone, so that a token's sums do not depend on the number of rows.
static int skinny_parts(int Mout) {
    return 2 * ((Mout + 15) / 16) <= compute_units() ? 2 : 1;
}

// 17 to 64 rows: tile rows per block (1 or 2) if gemm_rows_kernel takes the product, 0 if the 64-token kernel does.
// The first lasts about 4 us + 0.026 us per k tile and token tile (every block takes in all the tokens, and that
// is what its time goes to, however many rows of W it has); the second about 14 us, the launch that adds its
// partial sums included, + 0.21 us per MB of W (measured at 7B and 1.5B layer sizes).  From the shape of W and
// whether the rows are more than 32 only.
static int rows_tile_rows(int N, int Mout, int K) {
    if (N <= 16 || N > ROWS_MAX || K % 8 != 0) return 0;
    const int tiles = (Mout + 15) / 16, cus = compute_units();
    const int rr = tiles <= cus ? 1 : 2;
    if ((tiles + rr - 1) / rr > cus) return 0;      // many rows: the 64-token kernel needs no split there
    const double rows_us = 4. + 0.026 * (pk_cols(K) / 32) * (N <= 32 ? 2 : 4);
    const double mid_us = 14. + 0.21 * 2e-6 * Mout * K;
    return rows_us < mid_us ? rr : 0;
}

// whether a plain product of N rows keeps all of k inside a block, so that it can add its result to a residual
extern "C" int vt_linear_bf16_adds_residual(int N, int M, int K) {
    if (N <= 0 || M <= 0 || K <= 0 || K % 8 != 0) return 0;
    if (N <= 16 || rows_tile_rows(N, M, K) > 0) return 1;
    // 17 to 64 rows with k split over blocks: the launch that adds the partial sums adds the residual too
    return N <= ROWS_MAX && M % 4 == 0 && mid_splits(M, K, 128) > 1;
}

extern "C" long long vt_linear_bf16_workspace(int N, int M, int K, int gated) {
    // floats of workspace that vt_linear_bf16 / vt_gated_linear_bf16 need for this shape (0: none)
    if (N <= 16 || K % 8 != 0 || gated) return 0;
    if (rows_tile_rows(N, M, K)) return 0;       // gemm_rows_kernel: nothing is split
    const int splits = mid_splits(M, K, 128);
    return splits > 1 ? (long long)splits * N * M : 0;
}

// gain != null: x is the fp32 residual stream and the RMSNorm (gain, eps) is part of the product (up to 16 tokens);
// resid != null: the result is added to it (up to 64 tokens).
static const NormLink NO_LINK = {nullptr, nullptr, nullptr, nullptr, 0, 0.f};

// shares of the rows' sums of squares that a producing product of this shape writes (0: it cannot produce)
extern "C" int vt_linear_bf16_link_shares(int N, int M, int K) {
    if (N <= 0 || N > ROWS_MAX || M <= 0 || K <= 0 || K % 8 != 0 || M % 8 != 0) return 0;
    const int tiles = (M + 15) / 16;
    if (N <= 16) return skinny_parts(M) * tiles;                       // a block per tile row, or per part of one
    const int rr = rows_tile_rows(N, M, K);
    if (rr) return (tiles + rr - 1) / rr;                               // a block per rr tile rows, whole k
    if (mid_splits(M, K, 128) > 1) return (M + SUM_COLS - 1) / SUM_COLS; // the launch that adds the partial sums
    return 0;
}

template <bool SWIGLU, typename TO>
static int linear_bf16(const void* xv, const bf16_t* wp, const float* bias, TO* y, float* workspace, int N, int Mout,
                       int K, const float* gain, float eps, const float* resid, hipStream_t stream,
                       const NormLink& link = NO_LINK) {
    if (N == 0) return 0;
    const bool linked = link.xn_out || link.ssq_in;
    VT_REQUIRE(!linked || (N <= ROWS_MAX && K % 8 == 0 && (((uintptr_t)xv) & 15) == 0 && !gain),
               "vt_linear_bf16: a norm is handed over between products of up to 64 rows with k a multiple of 8 (N=%d, K=%d)", N, K);
    VT_REQUIRE(!link.xn_out || (resid && vt_linear_bf16_link_shares(N, Mout, K) > 0 && link.gain_next && link.ssq_out),
               "vt_linear_bf16: a product that hands a norm on adds to a residual and has gains and room for the sums");
    VT_REQUIRE(!link.ssq_in || (link.n_ssq > 0 && (((uintptr_t)link.ssq_in) & 15) == 0),
               "vt_linear_bf16: the shares of the sums of squares are missing or not 16-byte aligned");
    const bf16_t* x = (const bf16_t*)xv;
    VT_REQUIRE(!gain || N <= 16, "vt_linear_bf16: the fused norm needs at most 16 rows (N=%d)", N);
    VT_REQUIRE((!gain && !resid) || (K % 8 == 0 && (((uintptr_t)xv) & 15) == 0),
               "vt_linear_bf16: the fused norm and residual need k a multiple of 8 and aligned tokens (K=%d)", K);
    VT_REQUIRE(!gain || (((uintptr_t)gain) & 15) == 0, "vt_linear_bf16: the norm's gains are not 16-byte aligned");
    const int KT = pk_cols(K) / 32, up_tiles = pk_rows(Mout) / 16;
    VT_REQUIRE((((uintptr_t)wp) & 15) == 0, "vt_linear_bf16: the packed matrix is not 16-byte aligned");
    if (K % 8 != 0 || ((uintptr_t)x & 15)) {
        VT_REQUIRE(N <= 65535, "vt_linear_bf16: too many rows (%d) for the any-shape kernel", N);
        gemm_plain_kernel<SWIGLU, TO><<<dim3((Mout + 255) / 256, N), 256, 0, stream>>>(x, wp, bias, y, N, Mout, K, KT, up_tiles);
        VT_CHECK_LAUNCH("vt_linear_bf16(plain)");
        return 0;
    }
    const int rows_rr = SWIGLU ? 0 : rows_tile_rows(N, Mout, K);
    VT_REQUIRE(!resid || vt_linear_bf16_adds_residual(N, Mout, K), "vt_linear_bf16: %d rows of [%d, %d] do not take a "
               "residual (vt_linear_bf16_adds_residual)", N, Mout, K);
    if constexpr (!SWIGLU) {
        // whole k in a block of 8 waves (gemm_rows_kernel)
#define VT_ROWS(NT, RR) launch_rows<8, NT, RR, TO>(x, wp, bias, y, N, Mout, K, KT, resid, stream, link)
        if (rows_rr == 1) return N <= 32 ? VT_ROWS(2, 1) : VT_ROWS(4, 1);
        if (rows_rr == 2) return N <= 32 ? VT_ROWS(2, 2) : VT_ROWS(4, 2);
#undef VT_ROWS
    }
    if (N > 16) {
        // 64 tokens per block through LDS; two tile rows per wave (one for the gated product, which has two
        // matrices' rows per wave already)
        constexpr int RR = SWIGLU ? 1 : 2;
        const int splits = SWIGLU ? 1 : mid_splits(Mout, K, 64 * RR);
        VT_REQUIRE(splits == 1 || workspace, "vt_linear_bf16: this shape needs a workspace (vt_linear_bf16_workspace)");
        int kps = ((pk_cols(K) + splits - 1) / splits + MID_BK - 1) / MID_BK * MID_BK;
        // more than 64 tokens: 128 per block, so that W is read once per 128
        const int tok = N > 64 ? 128 : 64, token_blocks = (N + tok - 1) / tok;
        const int wm = SWIGLU ? mid_waves(Mout, 16 * RR, token_blocks) : 4;
        dim3 grid((Mout + 16 * wm * RR - 1) / (16 * wm * RR), token_blocks, splits);
        VT_REQUIRE(grid.y <= 65535, "vt_linear_bf16: too many rows (%d)", N);
        VT_REQUIRE(!(resid || link.xn_out) || (splits > 1 && N <= ROWS_MAX && Mout % 4 == 0 && sizeof(TO) == 4),
                   "vt_linear_bf16: %d rows of [%d, %d] do not take a residual (vt_linear_bf16_adds_residual)", N, Mout, K);
        VT_REQUIRE(!link.ssq_in || grid.y == 1, "vt_linear_bf16: a prepared norm is taken with up to 64 rows (N=%d)", N);
        // the product takes the norm in front (link.ssq_in); the one behind is prepared where the sums are added up
        NormLink in = NO_LINK;
        in.ssq_in = link.ssq_in; in.n_ssq = link.n_ssq; in.eps = link.eps;
#define VT_MID__(W, O, T) do { \
            static bool lds_set = false; \
            if (!lds_set) { \
                hipError_t e = hipFuncSetAttribute((const void*)gemm_mid_kernel<RR, SWIGLU, W, TO, O, T>, hipFuncAttributeMaxDynamicSharedMemorySize, MID_LDS_BYTES(T)); \
                VT_REQUIRE(e == hipSuccess, "vt_linear_bf16: cannot get %d bytes of LDS: %s", MID_LDS_BYTES(T), hipGetErrorString(e)); \
                lds_set = true; \
            } \
            gemm_mid_kernel<RR, SWIGLU, W, TO, O, T><<<grid, (W + 1) * 64, MID_LDS_BYTES(T), stream>>>(x, wp, bias, y, workspace, N, Mout, K, KT, up_tiles, kps, in); \
        } while (0)
#define VT_MID_(W, O) do { if (tok == 64) VT_MID__(W, O, 4); else VT_MID__(W, O, 8); } while (0)
#define VT_MID(W) do { if (grid.y == 1) VT_MID_(W, true); else VT_MID_(W, false); } while (0)
        if (wm == 3) VT_MID(3);
        else if (wm == 4) VT_MID(4);
        else if (wm == 5) VT_MID(5);
        else if (wm == 6) VT_MID(6);
        else VT_MID(8);
#undef VT_MID
#undef VT_MID_
#undef VT_MID__
        VT_CHECK_LAUNCH("vt_linear_bf16(64 tokens)");
        if (splits > 1) {
            const size_t n = (size_t)N * Mout;
            if constexpr (sizeof(TO) == 4) {
                if (resid || link.xn_out) {
                    NormLink outl = NO_LINK;
                    outl.xn_out = link.xn_out; outl.gain_next = link.gain_next; outl.ssq_out = link.ssq_out;
                    sum_partials_rows_kernel<<<dim3((Mout + SUM_COLS - 1) / SUM_COLS, link.xn_out ? 64 : N), 256, 0, stream>>>(
                        workspace, (float*)y, resid, N, Mout, splits, outl);
                    VT_CHECK_LAUNCH("vt_linear_bf16(sum rows)");
                    return 0;
                }
            }
            sum_partials_kernel<TO><<<(unsigned)((n / 4 + 255) / 256 + 1), 256, 0, stream>>>(workspace, y, n, splits);
            VT_CHECK_LAUNCH("vt_linear_bf16(sum)");
        }
        return 0;
    }
    // How k is split over the waves of a block depends on the shape of W only, so that a token's sums are added
    // in the same order whatever the number of rows: 8 waves, 16 for matrices with few rows and a long k.
    const int tiles16 = (Mout + 15) / 16;
    const bool wide = tiles16 >= 512 || KT < 256;
#define VT_SKINNY(W, NRM) gemm_skinny_kernel<W, SWIGLU, NRM, TO><<<tiles16, W * 64, 0, stream>>>(x, wp, bias, y, N, Mout, K, KT, up_tiles, gain, eps, resid, link)
#define VT_SKINNY_PART(P, W, NRM) gemm_skinny_kernel<W, false, NRM, TO, P><<<P * tiles16, W * 64, 0, stream>>>(x, wp, bias, y, N, Mout, K, KT, up_tiles, gain, eps, resid, link)
    if constexpr (!SWIGLU) {
        if (skinny_parts(Mout) == 2) {
            if (gain) { if (wide) VT_SKINNY_PART(2, 8, true); else VT_SKINNY_PART(2, 16, true); }
            else { if (wide) VT_SKINNY_PART(2, 8, false); else VT_SKINNY_PART(2, 16, false); }
            VT_CHECK_LAUNCH("vt_linear_bf16(half tile rows)");
            return 0;
        }
    }
    if (gain) { if (wide) VT_SKINNY(8, true); else VT_SKINNY(16, true); }
    else { if (wide) VT_SKINNY(8, false); else VT_SKINNY(16, false); }
#undef VT_SKINNY
#undef VT_SKINNY_PART
    VT_CHECK_LAUNCH("vt_linear_bf16");
    return 0;
}

// y[N, M] = x[N, K] . W[M, K]^T + bias; wp = W packed by vt_pack_matrix_bf16
extern "C" int vt_linear_bf16(const void* x, const void* wp, const float* bias, void* y, int out_dtype, float* workspace,
                              int N, int M, int K, hipStream_t stream) {
    VT_REQUIRE(N >= 0 && M > 0 && K > 0, "vt_linear_bf16: bad sizes N=%d M=%d K=%d", N, M, K);
    if (out_dtype == VT_F32) return linear_bf16<false, float>(x, (const bf16_t*)wp, bias, (float*)y, workspace, N, M, K, nullptr, 0.f, nullptr, stream);
    if (out_dtype == VT_BF16) return linear_bf16<false, bf16_t>(x, (const bf16_t*)wp, bias, (bf16_t*)y, workspace, N, M, K, nullptr, 0.f, nullptr, stream);
    return vt_fail("vt_linear_bf16: unknown out dtype %d", out_dtype);
}

// ---------------------------------------------------------------------------
// The product without a workspace argument and without any allocation: the partial sums of a split k range go into
// an array that the code object itself brings, one copy per GPU.
// ---------------------------------------------------------------------------
static __device__ __align__(256) float vt_linear_scratch[VT_LINEAR_NOALLOC_MAX_FLOATS];

#define VT_MAX_DEVICES 64
// Where this GPU's copy of the array lies.  In host code the array's name is only a handle for the runtime, not an
// address that a kernel could use: the address is asked for once per device, with that device current.
static int noalloc_scratch(float** out) {
    static float* ptrs[VT_MAX_DEVICES] = {nullptr};
    static std::mutex lock;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return vt_fail("vt_linear_bf16_noalloc: hipGetDevice: %s", hipGetErrorString(e));
    VT_REQUIRE(dev >= 0 && dev < VT_MAX_DEVICES, "vt_linear_bf16_noalloc: device %d is beyond the %d that are kept track of",
               dev, VT_MAX_DEVICES);
    std::lock_guard<std::mutex> guard(lock);
    if (!ptrs[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(vt_linear_scratch));
        if (e != hipSuccess || !p)
            return vt_fail("vt_linear_bf16_noalloc: hipGetSymbolAddress on device %d: %s", dev, hipGetErrorString(e));
        ptrs[dev] = (float*)p;
    }
    *out = ptrs[dev];
    return 0;
}

extern "C" int vt_linear_bf16_noalloc(const void* x, const void* wp, const float* bias, void* y, int out_dtype,
                                      int N, int M, int K, hipStream_t stream) {
    VT_REQUIRE(N >= 0 && M > 0 && K > 0, "vt_linear_bf16_noalloc: bad sizes N=%d M=%d K=%d", N, M, K);
    const long long need = vt_linear_bf16_workspace(N, M, K, 0);
    VT_REQUIRE(need <= (long long)VT_LINEAR_NOALLOC_MAX_FLOATS,
               "vt_linear_bf16_noalloc: x [%d, %d] with W [%d, %d] needs %lld floats for its partial sums, the built-in "
               "array holds %d: use vt_linear_bf16 with a workspace", N, K, M, K, need, VT_LINEAR_NOALLOC_MAX_FLOATS);
    float* scratch = nullptr;
    if (need > 0 && noalloc_scratch(&scratch) != 0) return -1;
    if (out_dtype == VT_F32) return linear_bf16<false, float>(x, (const bf16_t*)wp, bias, (float*)y, scratch, N, M, K, nullptr, 0.f, nullptr, stream);
    if (out_dtype == VT_BF16) return linear_bf16<false, bf16_t>(x, (const bf16_t*)wp, bias, (bf16_t*)y, scratch, N, M, K, nullptr, 0.f, nullptr, stream);
    return vt_fail("vt_linear_bf16_noalloc: unknown out dtype %d", out_dtype);
}

// The same with an RMSNorm in front (up to 16 tokens) and a residual addition behind (up to 64), each optional:
// gain != null: h is the fp32 residual stream [N, K] and y = (rmsnorm(h; gain, eps) . W^T) + bias, else h is x in bf16;
// resid != null (fp32 [N, M], may be y): y = resid + that.  y is fp32.
// workspace: for shapes whose k range is split over blocks (vt_linear_bf16_workspace), else null.
extern "C" int vt_linear_bf16_fused(const void* h, const float* gain, float eps, const void* wp, const float* bias,
                                    const float* resid, float* y, float* workspace, int N, int M, int K, hipStream_t stream) {
    VT_REQUIRE(N >= 0 && M > 0 && K > 0, "vt_linear_bf16_fused: bad sizes N=%d M=%d K=%d", N, M, K);
    VT_REQUIRE(gain || resid, "vt_linear_bf16_fused: neither a norm nor a residual: use vt_linear_bf16");
    return linear_bf16<false, float>(h, (const bf16_t*)wp, bias, y, workspace, N, M, K, gain, eps, resid, stream);
}

// The product between two RMSNorms that are no kernels of their own (up to 64 rows; S = 16 floats up to 16 rows,
// else 64):
// ssq_in != null: x is xn = bf16(h * gain) as a producing product left it, ssq_in [n_ssq][S] its blocks' shares of the
// rows' sums of h^2, and the result is multiplied by 1/sqrt(sum / K + eps_in);
// xn_out != null (needs resid): beside y = resid + product, xn_out [N][M] = bf16(y * gain_next) and this product's
// shares ssq_out [vt_linear_bf16_link_shares(N, M, K)][S] are written for the product behind the next norm.
// workspace: as for vt_linear_bf16.
extern "C" int vt_linear_bf16_link(const void* x, const void* wp, const float* bias, const float* resid, float* y,
                                   float* workspace, int N, int M, int K, const float* ssq_in, int n_ssq, float eps_in,
                                   void* xn_out, const float* gain_next, float* ssq_out, hipStream_t stream) {
    VT_REQUIRE(N >= 0 && M > 0 && K > 0, "vt_linear_bf16_link: bad sizes N=%d M=%d K=%d", N, M, K);
    VT_REQUIRE(ssq_in || xn_out, "vt_linear_bf16_link: neither end of a norm: use vt_linear_bf16");
    const NormLink link = {(bf16_t*)xn_out, gain_next, ssq_out, ssq_in, n_ssq, eps_in};
    return linear_bf16<false, float>(x, (const bf16_t*)wp, bias, y, workspace, N, M, K, nullptr, 0.f, resid, stream, link);
}

// the gated product behind a norm that the product in front has prepared (x = xn, ssq_in, n_ssq, eps_in as above)
extern "C" int vt_gated_linear_bf16_link(const void* x, const void* wp, void* y, int out_dtype, int N, int I, int K,
                                         const float* ssq_in, int n_ssq, float eps_in, hipStream_t stream) {
    VT_REQUIRE(N >= 0 && I > 0 && K > 0, "vt_gated_linear_bf16_link: bad sizes N=%d I=%d K=%d", N, I, K);
    VT_REQUIRE(ssq_in, "vt_gated_linear_bf16_link: no sums of squares: use vt_gated_linear_bf16");
    const NormLink link = {nullptr, nullptr, nullptr, ssq_in, n_ssq, eps_in};
    if (out_dtype == VT_F32) return linear_bf16<true, float>(x, (const bf16_t*)wp, nullptr, (float*)y, nullptr, N, I, K, nullptr, 0.f, nullptr, stream, link);
    if (out_dtype == VT_BF16) return linear_bf16<true, bf16_t>(x, (const bf16_t*)wp, nullptr, (bf16_t*)y, nullptr, N, I, K, nullptr, 0.f, nullptr, stream, link);
    return vt_fail("vt_gated_linear_bf16_link: unknown out dtype %d", out_dtype);
}

// y[N, I] = silu(x . Wg^T) * (x . Wu^T); wp = Wg [I, K] packed, followed by Wu [I, K] packed.
// gain != null: x is the fp32 residual stream and rmsnorm(x; gain, eps) takes its place (up to 16 tokens).
extern "C" int vt_gated_linear_bf16(const void* x, const void* wp, void* y, int out_dtype, int N, int I, int K,
                                    const float* gain, float eps, hipStream_t stream) {
    VT_REQUIRE(N >= 0 && I > 0 && K > 0, "vt_gated_linear_bf16: bad sizes N=%d I=%d K=%d", N, I, K);
    if (out_dtype == VT_F32) return linear_bf16<true, float>(x, (const bf16_t*)wp, nullptr, (float*)y, nullptr, N, I, K, gain, eps, nullptr, stream);
    if (out_dtype == VT_BF16) return linear_bf16<true, bf16_t>(x, (const bf16_t*)wp, nullptr, (bf16_t*)y, nullptr, N, I, K, gain, eps, nullptr, stream);
    return vt_fail("vt_gated_linear_bf16: unknown out dtype %d", out_dtype);
}
