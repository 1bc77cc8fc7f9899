// Entry points of the bfloat16 few-row matrix products (vt_gemm_bf16.hip).  All return 0, or a negative code after
// leaving a message for vt_last_error().  Pointers are device pointers unless said otherwise; every launch goes to
// `stream`.
#pragma once
#include <hip/hip_runtime.h>

extern "C" {

const char* vt_last_error();

// elements of the packed form of W [M, K] (rows padded to 16, k to 128)
long long vt_packed_elems(int M, int K);
int vt_pack_matrix_bf16(const void* w, void* wp, int M, int K, hipStream_t stream);
int vt_unpack_matrix_bf16(const void* wp, void* w, int M, int K, hipStream_t stream);

// whether a plain product of N rows with W [M, K] can add its result to a residual in the same kernel
int vt_linear_bf16_adds_residual(int N, int M, int K);
// floats of workspace that vt_linear_bf16 needs for this shape (0: none)
long long vt_linear_bf16_workspace(int N, int M, int K, int gated);

// y[N, M] = x[N, K] . W[M, K]^T + bias; wp = W packed; out_dtype 0: float32, 1: bfloat16.  Shapes whose k range is
// split over blocks (vt_linear_bf16_workspace > 0) put their partial sums into `workspace`.
int vt_linear_bf16(const void* x, const void* wp, const float* bias, void* y, int out_dtype, float* workspace,
                   int N, int M, int K, hipStream_t stream);

// The same product for callers that cannot allocate device memory and have no workspace to bring: code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference
// (which allocates its products' outputs and leaves scratch memory to the GEMM library).  The partial sums go into
// a file-scope device array of VT_LINEAR_NOALLOC_MAX_FLOATS floats (16 MiB) that every GPU the library runs on holds
// from the first call on it until the process ends; a shape that needs more is refused with an error.  The call
// allocates nothing and frees nothing.  All calls on one GPU share that array: calls that overlap on one GPU (two
// streams, two threads) race; calls on one stream do not.  Nothing in the array has to start at zero: every partial
// sum that a call reads it has written first.  The first call on a GPU looks the array's address up
// (hipGetSymbolAddress) and should therefore happen outside a graph capture.
#define VT_LINEAR_NOALLOC_MAX_FLOATS (4 * 1024 * 1024)
int vt_linear_bf16_noalloc(const void* x, const void* wp, const float* bias, void* y, int out_dtype,
                           int N, int M, int K, hipStream_t stream);

int vt_linear_bf16_fused(const void* h, const float* gain, float eps, const void* wp, const float* bias,
                         const float* resid, float* y, float* workspace, int N, int M, int K, hipStream_t stream);
int vt_gated_linear_bf16(const void* x, const void* wp, void* y, int out_dtype, int N, int I, int K,
                         const float* gain, float eps, hipStream_t stream);

// An RMSNorm handed from the product in front of it (which adds to the residual stream and writes, beside it, the
// stream times the norm's gains in bfloat16 and its blocks' shares of the rows' sums of squares) to the product
// behind it (which reads those as its tokens and divides its sums by the norm's root): see vt_gemm_bf16.hip.
int vt_linear_bf16_link_shares(int N, int M, int K);
int vt_linear_bf16_link(const void* x, const void* wp, const float* bias, const float* resid, float* y,
                        float* workspace, int N, int M, int K, const float* ssq_in, int n_ssq, float eps_in,
                        void* xn_out, const float* gain_next, float* ssq_out, hipStream_t stream);
int vt_gated_linear_bf16_link(const void* x, const void* wp, void* y, int out_dtype, int N, int I, int K,
                              const float* ssq_in, int n_ssq, float eps_in, hipStream_t stream);

}
