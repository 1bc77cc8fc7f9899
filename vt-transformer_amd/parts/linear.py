"""y = x W^T + b with W stored [out, in], as the reference's op_linear
(v1/tensortype/hip_tensor.cpp:479-539; layout asserted in
v1/tensortype/tensortype.cpp:222-229).

float32: the hand-written fp32 kernel, always (no matrix-core mode).
bfloat16: the hand-written matrix-core kernel while the rows are few enough
that reading W dominates, on a copy of W in the matrix instruction's own order;
above that the GEMM library on the row-major W, which is where the reference's
engine uses a library too (hipblasGemmEx, hip_tensor.cpp:514-535).
"""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import NormedInput, Runtime

# up to this many rows W is streamed once per 64 rows by the skinny kernel
SKINNY_MAX_ROWS = 64
# ... and up to this many for a matrix with few rows and a long k (the down projection), where the GEMM library is
# at its worst: 59 against 99 us at 128 rows of 3,584 x 18,944, 86 against 125 us at 256 (measured)
LONG_K_MAX_ROWS = 256
# ... and up to this many for the gated pair of matrices (gate/up), 128 rows to a block: one launch that also
# applies the gate against the library's product and a gating kernel behind it
GATED_MAX_ROWS = 128


# A model that keeps the packed copy only: from this many rows on, a product unpacks its matrix into scratch memory
# and goes through the GEMM library (the unpacking costs about two passes over W, the few-row kernels one pass per 64
# rows, and the library is the faster multiplier by far)
UNPACK_MIN_ROWS = 256


def packed_kernel_rows(m: int, k: int) -> int:
    """Rows up to which the hand-written kernel on the packed matrix multiplies [rows, k] by W[m, k]."""
    return LONG_K_MAX_ROWS if k >= 4 * m else SKINNY_MAX_ROWS


# the few-row kernel applies an RMSNorm in front for up to this many rows
FUSE_MAX_ROWS = ops.NORM_MAX_ROWS


def norm_inside_products(rt: Runtime) -> bool:
    """Whether this runtime's products may apply an RMSNorm on their way (the norm in front of a few-row product, or
    handed from the product in front of it to the product behind it).  Those kernels round the stream times the
    norm's gains to 16 bits and divide by the root afterwards, on the fp32 sums.  bfloat16 has float32's range, so
    the order costs nothing there.  float16 does not: an un-normalised h * gain beyond 65,504 would become infinite and
    one below 6e-5 would lose bits, where the normalised value that the reference rounds ((w * x) * r,
    v1/tensortype/hip_kernels/rmsnorm.cpp:28-41) is harmless.  In float16 the norm therefore stays a kernel of its
    own, which rounds once, behind the scaling."""
    return rt.lowp and rt.dtype != torch.float16


def can_fuse(rt: Runtime, n: int) -> bool:
    """Whether a product of n rows can take the residual stream with its norm still to be applied."""
    return norm_inside_products(rt) and n <= FUSE_MAX_ROWS


def can_add_residual(rt: Runtime, n: int, m: int, k: int) -> bool:
    """Whether the product of n rows with W [m, k] can add its result to the residual stream itself: it can where
    no k range is split over blocks (up to 16 rows; 17 to 64 for matrices that the kernel for it suits)."""
    return rt.lowp and ops.linear_bf16_adds_residual(n, m, k)


def can_hand_norm_on(rt: Runtime, n: int, m: int, k: int) -> bool:
    """Whether the product of n rows with W [m, k], adding to the residual stream, can prepare the norm behind it."""
    return norm_inside_products(rt) and n <= ops.LINK_MAX_ROWS and ops.linear_bf16_link_shares(n, m, k) > 0


def takes_prepared_norm(rt: Runtime, n: int, k: int) -> bool:
    """Whether a product of n rows over k can take a norm that the product in front has prepared."""
    return norm_inside_products(rt) and n <= ops.LINK_MAX_ROWS and k % 8 == 0


def linear(rt: Runtime, x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], name: str,
           out_dtype: Optional[torch.dtype] = None, bias_lowp: Optional[torch.Tensor] = None,
           packed=None, residual: Optional[torch.Tensor] = None, hand_on=None):
    """x [N, K] in the runtime's dtype -> [N, M].  `name` keys the output's scratch buffer.
    Output dtype: float32 from the hand-written kernels unless `out_dtype` says otherwise; the
    library path returns the 16-bit type (its bias, if any, is `bias_lowp`, the same values in that type).
    packed: W as rt.pack(w) made it, for the few-row kernel (made on the spot if missing: slow).
    x may be a NormedInput (the norm then happens inside the few-row kernel, or before the product as a kernel of
    its own where that is not possible).  residual (float32 [N, M]): the product is added to it in place and
    `residual` is returned (by the product's kernel where `can_add_residual` says so, else by a kernel after it).
    hand_on (with residual): the norm that comes behind this product (`rms_fusable`); where the kernel can, it
    prepares that norm on its way and a prepared NormedInput is returned instead of `residual`."""
    n, k = x.shape
    m = w.shape[0] if w is not None else packed.rows * packed.halves   # (no row-major copy: the runtime keeps the packed one only)
    if residual is not None or isinstance(x, NormedInput):
        w_any = packed if packed is not None else w
        is_packed = isinstance(w_any, ops.PackedMatrix)
        if isinstance(x, NormedInput):
            ok = (takes_prepared_norm(rt, n, k) and is_packed) if x.prepared else (can_fuse(rt, n) and k % 8 == 0)
            if not ok:
                x = x.materialize()
        norm = x if isinstance(x, NormedInput) else None
        if norm is not None or can_add_residual(rt, n, m, k):
            out = residual if residual is not None else rt.buffer(name, (n, m), torch.float32)
            need = ops.linear_bf16_workspace(n, m, k) if n > 16 else 0
            work = rt.buffer("linear.partials", (need,), torch.float32) if need else None
            emits = (hand_on is not None and residual is not None and is_packed
                     and getattr(hand_on, "rms_fusable", False) and can_hand_norm_on(rt, n, m, k))
            if emits and norm is not None and not norm.prepared:
                x, norm = norm.materialize(), None     # (a product cannot take the norm in front both ways at once)
            if emits or (norm is not None and norm.prepared):
                xn = ssq = None
                if emits:
                    xn = rt.buffer(name + ".xn", (n, m), rt.dtype)
                    ssq = rt.buffer(name + ".ssq", (ops.linear_bf16_link_shares(n, m, k), ops.link_stride(n)), torch.float32)
                ops.linear_bf16_link(norm.xn if norm else x, w_any, bias, out, residual=residual,
                                     ssq_in=norm.ssq if norm else None, eps_in=norm.eps if norm else 0.0,
                                     xn_out=xn, gain_next=hand_on.gain if emits else None, ssq_out=ssq, workspace=work)
                return NormedInput(out, hand_on, xn, ssq) if emits else out
            return ops.linear_bf16(norm.h if norm else x, w_any, bias, out, work,
                                   norm_gain=norm.gain if norm else None, norm_eps=norm.eps if norm else 0.0,
                                   residual=residual)
        if residual is not None:
            # a shape the fused kernels do not take (k no multiple of 8): the product, then the addition
            return ops.residual_add(residual, linear(rt, x, w, bias, name, out_dtype, bias_lowp, packed))
    if rt.dtype == torch.float32:
        out = rt.buffer(name, (n, m), torch.float32)
        return ops.linear_f32(x, w, bias, out)
    if w is None and not rt.keep_row_major and n >= UNPACK_MIN_ROWS:
        # every product's matrix in turn in the same scratch memory (the largest one's size)
        w = ops.unpack_matrix_bf16(packed, rt.buffer("linear.unpacked", (packed.halves * packed.rows, packed.cols), rt.dtype))
    if w is None or n <= (packed_kernel_rows(m, k) if packed is not None else SKINNY_MAX_ROWS):
        out = rt.buffer(name, (n, m), out_dtype or torch.float32)
        need = ops.linear_bf16_workspace(n, m, k) if n > 16 else 0
        work = rt.buffer("linear.partials", (need,), torch.float32) if need else None
        return ops.linear_bf16(x, packed if packed is not None else w, bias, out, work)
    out = rt.buffer(name + ".lib", (n, m), rt.dtype)
    if bias is not None:
        if bias_lowp is None:
            bias_lowp = bias.to(rt.dtype)
        torch.addmm(bias_lowp, x, w.t(), out=out)
    else:
        torch.mm(x, w.t(), out=out)
    return out
