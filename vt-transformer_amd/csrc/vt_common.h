// Shared helpers of the gfx950 kernels: conversion of the 16-bit type, wave and block
// reductions for 64-wide wavefronts, launch checking.
//
// Every entry point is extern "C", takes raw device pointers and a stream,
// launches on that stream and returns 0, or a negative code after writing a
// message that vt_last_error() hands out.  Shapes are validated on the host
// before a launch; no kernel reads outside what its arguments describe.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#define VT_WAVE 64

// activation / weight element types
#define VT_F32 0
#define VT_BF16 1

typedef uint16_t bf16_t;  // raw bits

// One library = one translation unit, so the error text lives here.
static char vt_err_buf_[512] = "";
static int vt_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(vt_err_buf_, sizeof(vt_err_buf_), fmt, ap);
    va_end(ap);
    return -1;
}
// Each library's source file invokes this once.
#define VT_DEFINE_LAST_ERROR() \
    extern "C" const char* vt_last_error() { return vt_err_buf_; }

#define VT_CHECK_LAUNCH(name)                                              \
    do {                                                                   \
        hipError_t e_ = hipGetLastError();                                 \
        if (e_ != hipSuccess) return vt_fail("%s: launch failed: %s", name, hipGetErrorString(e_)); \
    } while (0)

#define VT_REQUIRE(cond, ...)                   \
    do {                                        \
        if (!(cond)) return vt_fail(__VA_ARGS__); \
    } while (0)

// The 16-bit type of a build is bfloat16, or IEEE half when the source is compiled with -DVT_LOWP_F16: the same
// kernels, another conversion and another matrix instruction of the same shape and rate.  A library is built once
// per 16-bit type and its file name says which; `bf16_t` is the raw 16 bits either way, and VT_BF16 the code of "the
// build's 16-bit type" in the entry points' dtype arguments.
typedef __attribute__((ext_vector_type(2))) float vt_f32x2_t;
#ifdef VT_LOWP_F16
typedef _Float16 vt_lowp_t;
typedef __attribute__((ext_vector_type(4))) _Float16 vt_lowp4_t;
#define VT_MFMA_16X16X32(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0)
#define VT_MFMA_16X16X16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0)
#define VT_LOWP_ONE_PAIR 0x3c003c00u       // two ones
__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return (float)__builtin_bit_cast(_Float16, v); }
// round to nearest even; NaN stays NaN, what is too large becomes infinity
__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return __builtin_bit_cast(bf16_t, (_Float16)f); }
// the two values of a 32-bit word
__device__ __forceinline__ float lowp_lo(unsigned u) { return bf16_to_f32((bf16_t)(u & 0xffffu)); }
__device__ __forceinline__ float lowp_hi(unsigned u) { return bf16_to_f32((bf16_t)(u >> 16)); }
#else
typedef __bf16 vt_lowp_t;
typedef __attribute__((ext_vector_type(4))) short vt_lowp4_t;
#define VT_MFMA_16X16X32(a, b, c) __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0)
#define VT_MFMA_16X16X16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0)
#define VT_LOWP_ONE_PAIR 0x3f803f80u
__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
    return __uint_as_float(((uint32_t)v) << 16);
}

// round to nearest even; NaN stays NaN
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}
__device__ __forceinline__ float lowp_lo(unsigned u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float lowp_hi(unsigned u) { return __uint_as_float(u & 0xffff0000u); }
#endif
typedef __attribute__((ext_vector_type(8))) vt_lowp_t vt_lowp8_t;
typedef __attribute__((ext_vector_type(2))) vt_lowp_t vt_lowp2_t;
// two floats to two 16-bit values (round to nearest even) in one instruction
__device__ __forceinline__ unsigned vt_pack2(float a, float b) {
    vt_f32x2_t v = {a, b};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, vt_lowp2_t));
}

template <typename T> __device__ __forceinline__ float load_f32(const T* p, size_t i);
template <> __device__ __forceinline__ float load_f32<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ __forceinline__ float load_f32<bf16_t>(const bf16_t* p, size_t i) { return bf16_to_f32(p[i]); }

template <typename T> __device__ __forceinline__ void store_f32(T* p, size_t i, float v);
template <> __device__ __forceinline__ void store_f32<float>(float* p, size_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void store_f32<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f32_to_bf16(v); }

// Between a wave's writes to an LDS buffer that only it uses and its reads of what its other lanes wrote: the LDS
// executes a wave's operations in order, so all this has to do is to keep the compiler from moving the reads up.
__device__ __forceinline__ void wave_lds_order() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---------------------------------------------------------------------------
// Loads from memory straight into LDS (global_load_lds_dwordx4, 16 bytes per lane).  A wave's load writes 64
// consecutive 16-byte slots of LDS, one per lane, and every lane chooses its own address in memory: lane l's 16
// bytes at base + off go to LDS bytes lds + 16 l .. + 15; `base` and `lds` are the same in every lane.  No register
// holds the data on its way and no thread stores it, and the layout in LDS is made by the choice of addresses.
// Written as assembly: when the compiler knows of such a load it makes every later read of LDS wait for it, since
// it cannot tell one buffer from another; the program waits itself (wait_loads) before it reads what has landed.
// The compiler's own waits for its own loads stay right: loads return in the order they were asked for, and these
// only add to the number that it counts.  ONCE: no other wave reads these bytes (a non-temporal load).
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void* vt_lds_void_ptr;
template <bool ONCE = false>
__device__ __forceinline__ void load_to_lds16(const void* base, unsigned off, unsigned lds) {
    if constexpr (ONCE)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                     :: "v"(off), "s"(base), "s"(lds) : "memory", "m0");
    else
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(off), "s"(base), "s"(lds) : "memory", "m0");
}
// the address in LDS of an object there, as the loads above want it
__device__ __forceinline__ unsigned lds_address(const void* p) { return (unsigned)(uintptr_t)(vt_lds_void_ptr)p; }
// wait until at most N of this wave's loads are in flight; no access to memory moves across it
template <int N>
__device__ __forceinline__ void wait_loads() {
    static_assert(N >= 0 && N < 64, "the counter has six bits");
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Block reductions for blockDim.x a multiple of 64, up to 1024.  `red` is
// shared memory of at least 16 floats.  The order of the additions depends
// only on blockDim.x, so a row's sum does not depend on what else is in the
// launch.
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += red[i];
    return t;
}
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    int w = threadIdx.x >> 6, nw = blockDim.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float t = red[0];
    for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
    return t;
}

// One pair of a rotary encoding, x with its partner y: the low element is c x - s y, the high one c x + s y.  Every
// kernel that rotates goes through these two, with the product and the fused multiply-add spelled out, so that
// all of them round alike whatever the compiler would contract on its own.
__device__ __forceinline__ float rotate_low(float c, float s, float x, float y) { return __fmaf_rn(c, x, -__fmul_rn(s, y)); }
__device__ __forceinline__ float rotate_high(float c, float s, float x, float y) { return __fmaf_rn(c, x, __fmul_rn(s, y)); }
// the one or the other by a flag, without a branch (the same bits: only the product's sign differs)
__device__ __forceinline__ float rotate_pair(float c, float s, float x, float y, bool low) {
    const float p = __fmul_rn(s, y);
    return __fmaf_rn(c, x, low ? -p : p);
}
