"""Python face of the HIP kernels.

Every function checks on the host that the operands are what the kernel and
its launch grid assume (device, dtype, contiguity, shapes) and raises
before anything is launched otherwise.  A missing or unloadable library is an
error, never a reason to compute some other way.
"""
from __future__ import annotations

import ctypes
import math
from typing import Optional

import torch

from . import build as _build
from .build import KernelBuildError, load_lib

F32, BF16 = 0, 1
# The 16-bit types.  A library that handles 16-bit values exists once for each (kernels.build.HALF_LIBS); BF16 is the
# code of "the library's 16-bit type" in the entry points' dtype arguments, whichever build is called.
LOWP = (torch.bfloat16, torch.float16)
_CODES = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: BF16}


class KernelError(RuntimeError):
    pass


def _code(t: torch.Tensor) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise KernelError(f"dtype {t.dtype} is not handled by the kernels (float32, bfloat16 and float16 are)") from None


def _half(*ts) -> bool:
    """Which build of a library a call needs: True if the 16-bit tensors among `ts` are float16.  The two 16-bit
    types do not meet in one call."""
    kinds = {t.dtype for t in ts if t is not None and t.dtype in LOWP}
    if len(kinds) > 1:
        raise KernelError("bfloat16 and float16 tensors in one call")
    return torch.float16 in kinds


def _any_build(name: str, head_dim: Optional[int] = None):
    """A library for a question whose answer is the same in both of its builds (launch shapes, sizes of scratch
    memory): the build that is loaded already, so that a float16 model does not compile the bfloat16 one for it."""
    for half in (False, True):
        lib = _build._loaded.get(_build.lib_spec(name, head_dim, half)[0])
        if lib is not None:
            return lib
    return load_lib(name, head_dim)


def _lowp(t: torch.Tensor, name: str) -> torch.dtype:
    """The 16-bit type of a call's leading tensor."""
    if t.dtype not in LOWP:
        raise KernelError(f"{name}: dtype {t.dtype}, expected bfloat16 or float16")
    return t.dtype


def _chk(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor is on {t.device}, the kernels run on the GPU only")
    if not t.is_contiguous():
        raise KernelError(f"{name}: tensor is not contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: dtype {t.dtype}, expected {dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _run(lib, fn: str, *args) -> None:
    rc = getattr(lib, fn)(*args)
    if rc != 0:
        raise KernelError(lib.vt_last_error().decode("utf-8", "replace"))


def _i(v) -> ctypes.c_int:
    return ctypes.c_int(int(v))


def _f(v) -> ctypes.c_float:
    return ctypes.c_float(float(v))


# ---------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    n = ids.numel()
    vocab, hidden = table.shape
    _chk(table, "embed.table")
    _chk(ids, "embed.ids", torch.int32)
    _chk(out, "embed.out", torch.float32, (n, hidden))
    _run(load_lib("vt_elementwise", half=_half(table)), "vt_embed", _ptr(table), _i(_code(table)), _ptr(ids), _ptr(out), _i(n), _i(hidden),
         _i(vocab), _stream())
    return out


def rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], gain: torch.Tensor, out: torch.Tensor, eps: float,
            rows: Optional[torch.Tensor] = None, update_h: bool = True) -> torch.Tensor:
    """out[r] = gain * x / sqrt(mean(x^2) + eps), x = h[row] + delta[row]; with update_h the sum is written back to h."""
    hidden = h.shape[-1]
    _chk(h, "rmsnorm.h", torch.float32)
    _chk(gain, "rmsnorm.gain", torch.float32, (hidden,))
    if delta is not None:
        _chk(delta, "rmsnorm.delta", None, h.shape)
    if rows is not None:
        _chk(rows, "rmsnorm.rows", torch.int32)
        n_out = rows.numel()
        update_h = False
    else:
        n_out = h.shape[0]
    _chk(out, "rmsnorm.out", None, (n_out, hidden))
    _run(load_lib("vt_elementwise", half=_half(delta, out)), "vt_rmsnorm", _ptr(h), _ptr(delta), _i(_code(delta) if delta is not None else -1),
         _ptr(gain), _ptr(out), _i(_code(out)), _ptr(rows), _i(n_out), _i(hidden), _f(eps),
         _i(1 if (update_h and delta is not None) else 0), _stream())
    return out


def residual_add(h: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    _chk(h, "residual_add.h", torch.float32)
    _chk(delta, "residual_add.delta", None, h.shape)
    _run(load_lib("vt_elementwise", half=_half(delta)), "vt_residual_add", _ptr(h), _ptr(delta), _i(_code(delta)),
         ctypes.c_longlong(h.numel()), _stream())
    return h


def silu_mul(gu: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    n, two_i = gu.shape
    _chk(gu, "silu_mul.gu")
    _chk(out, "silu_mul.out", None, (n, two_i // 2))
    if two_i % 2:
        raise KernelError(f"silu_mul: input width {two_i} is odd")
    _run(load_lib("vt_elementwise", half=_half(gu, out)), "vt_silu_mul", _ptr(gu), _i(_code(gu)), _ptr(out), _i(_code(out)), _i(n),
         _i(two_i // 2), _stream())
    return out


def gather_rows(x: torch.Tensor, rows: Optional[torch.Tensor], out: torch.Tensor) -> torch.Tensor:
    _chk(x, "gather_rows.x")
    n = rows.numel() if rows is not None else x.shape[0]
    if rows is not None:
        _chk(rows, "gather_rows.rows", torch.int32)
    _chk(out, "gather_rows.out", None, (n, x.shape[1]))
    _run(load_lib("vt_elementwise", half=_half(x, out)), "vt_gather_rows", _ptr(x), _i(_code(x)), _ptr(rows), _ptr(out), _i(_code(out)),
         _i(n), _i(x.shape[1]), _stream())
    return out


def stream_read(buf: torch.Tensor, sums: torch.Tensor, blocks: int = 256) -> torch.Tensor:
    """Read `buf` once with a kernel that does nothing else (the measured ceiling of weight streaming).
    sums: int32 [blocks * 16]; the XOR of its words is the XOR of the buffer's 32-bit words."""
    _chk(buf, "stream_read.buf")
    _chk(sums, "stream_read.sums", torch.int32, (blocks * 16,))
    nbytes = buf.numel() * buf.element_size()
    if nbytes % 16:
        raise KernelError(f"stream_read: {nbytes} bytes are not whole 16-byte pieces")
    _run(load_lib("vt_elementwise"), "vt_stream_read", _ptr(buf), ctypes.c_longlong(nbytes), _ptr(sums), _i(blocks), _stream())
    return sums


def random_normal(out: torch.Tensor, key: int, scale: float, mean: float, first: int = 0) -> torch.Tensor:
    """out.flat[i] = mean + scale * (twelve 16-bit integers of element first + i, summed and centred): close to
    N(mean, (65536 scale)^2), and the same bits as weights.random_init.counter_normal makes on the host."""
    _chk(out, "random_normal.out")
    _run(load_lib("vt_elementwise", half=_half(out)), "vt_random_normal", _ptr(out), _i(_code(out)), ctypes.c_longlong(out.numel()),
         ctypes.c_longlong(int(first)), ctypes.c_ulonglong(int(key) & 0xFFFFFFFFFFFFFFFF), _f(scale), _f(mean), _stream())
    return out


def rope_store(qkv: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], positions: torch.Tensor,
               tok_entry: torch.Tensor, block_table: Optional[torch.Tensor], q_out: torch.Tensor,
               k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], n_heads: int, n_kv: int, head_dim: int,
               write_kv: bool = True) -> None:
    """Rotate queries and keys by the tables' angles at `positions`, write the queries to q_out and, with
    write_kv, keys and values into their pages ([page][kv][slot][D] and [page][kv][D][slot])."""
    n = qkv.shape[0]
    width = (n_heads + (2 * n_kv if write_kv else 0)) * head_dim
    _chk(qkv, "rope_store.qkv")
    if qkv.shape[1] < width:
        raise KernelError(f"rope_store.qkv: {qkv.shape[1]} columns, need {width}")
    _chk(positions, "rope_store.positions", torch.int32, (n,))
    _chk(tok_entry, "rope_store.tok_entry", torch.int32, (n,))
    _chk(q_out, "rope_store.q_out", None, (n, n_heads * head_dim))
    rot = 0
    max_pos = 0
    if cos is not None:
        _chk(cos, "rope_store.cos", torch.float32)
        _chk(sin, "rope_store.sin", torch.float32, cos.shape)
        max_pos, half = cos.shape
        rot = 2 * half
    page_size = num_pages = max_blocks = 0
    if write_kv:
        num_pages, kvh, page_size, d = k_pages.shape
        if (kvh, d) != (n_kv, head_dim):
            raise KernelError(f"rope_store.k_pages: shape {tuple(k_pages.shape)} does not fit kv heads {n_kv} x {head_dim}")
        _chk(k_pages, "rope_store.k_pages", q_out.dtype)
        _chk(v_pages, "rope_store.v_pages", q_out.dtype, (num_pages, n_kv, head_dim, page_size))
        _chk(block_table, "rope_store.block_table", torch.int32)
        max_blocks = block_table.shape[1]
    _run(load_lib("vt_elementwise", half=_half(qkv, q_out, k_pages)), "vt_rope_store", _ptr(qkv), _i(_code(qkv)), ctypes.c_longlong(qkv.stride(0)),
         _ptr(cos), _ptr(sin), _i(rot), _i(max_pos), _ptr(positions), _ptr(tok_entry), _ptr(block_table),
         _i(max_blocks), _ptr(q_out), _ptr(k_pages), _ptr(v_pages), _i(_code(q_out)), _i(page_size), _i(num_pages),
         _i(n), _i(n_heads), _i(n_kv), _i(head_dim), _i(1 if write_kv else 0), _stream())


# ---------------------------------------------------------------------------
def linear_f32(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor) -> torch.Tensor:
    n, k = x.shape
    m = w.shape[0]
    _chk(x, "linear_f32.x", torch.float32)
    _chk(w, "linear_f32.w", torch.float32, (m, k))
    _chk(out, "linear_f32.out", torch.float32, (n, m))
    if bias is not None:
        _chk(bias, "linear_f32.bias", torch.float32, (m,))
    _run(load_lib("vt_gemm_f32"), "vt_linear_f32", _ptr(x), _ptr(w), _ptr(bias), _ptr(out), _i(n), _i(m), _i(k), _stream())
    return out


class PackedMatrix:
    """W [rows, cols] in bfloat16 in the order the matrix instruction reads it (vt_gemm_bf16.hip): tiles of
    16 rows x 32 columns, each stored as the 64 lanes' fragments; rows padded to 16 and columns to 128 by zeros.
    `halves` = 2: two matrices of `rows` rows each, packed one after the other (gate, then up)."""

    __slots__ = ("data", "rows", "cols", "halves")

    def __init__(self, data: torch.Tensor, rows: int, cols: int, halves: int = 1):
        self.data, self.rows, self.cols, self.halves = data, int(rows), int(cols), int(halves)

    def first_rows(self, n: int) -> "PackedMatrix":
        """The matrix of the first n rows (a multiple of 16): the packed rows of tiles are contiguous."""
        if self.halves != 1 or n % 16 or not 0 < n <= self.rows:
            raise KernelError(f"cannot take the first {n} rows of a packed matrix of {self.rows}")
        per_tile_row = self.data.numel() // ((self.rows + 15) // 16)
        return PackedMatrix(self.data[:(n // 16) * per_tile_row], n, self.cols)


def pack_matrix_bf16(w: torch.Tensor, halves: int = 1) -> PackedMatrix:
    """Pack W [rows, cols] (halves = 2: [2 * rows, cols], the two matrices stacked) for linear_bf16 /
    gated_linear_bf16."""
    lp = _lowp(w, "pack_matrix_bf16.w")
    _chk(w, "pack_matrix_bf16.w", lp)
    if w.dim() != 2 or w.shape[0] % halves:
        raise KernelError(f"pack_matrix_bf16: shape {tuple(w.shape)} is not {halves} stacked matrices")
    rows, cols = w.shape[0] // halves, w.shape[1]
    lib = load_lib("vt_gemm_bf16", half=_half(w))
    lib.vt_packed_elems.restype = ctypes.c_longlong
    per = int(lib.vt_packed_elems(_i(rows), _i(cols)))
    data = torch.empty(halves * per, dtype=lp, device=w.device)
    for h in range(halves):
        _run(lib, "vt_pack_matrix_bf16", _ptr(w[h * rows:(h + 1) * rows]), _ptr(data[h * per:(h + 1) * per]), _i(rows),
             _i(cols), _stream())
    return PackedMatrix(data, rows, cols, halves)


def unpack_matrix_bf16(packed: PackedMatrix, out: torch.Tensor) -> torch.Tensor:
    """The row-major matrix [halves * rows, cols] back from its packed form, into `out`."""
    lp = _lowp(packed.data, "unpack_matrix_bf16.packed")
    _chk(out, "unpack_matrix_bf16.out", lp, (packed.halves * packed.rows, packed.cols))
    lib = load_lib("vt_gemm_bf16", half=_half(packed.data))
    per = packed.data.numel() // packed.halves
    for h in range(packed.halves):
        _run(lib, "vt_unpack_matrix_bf16", _ptr(packed.data[h * per:(h + 1) * per]),
             _ptr(out[h * packed.rows:(h + 1) * packed.rows]), _i(packed.rows), _i(packed.cols), _stream())
    return out


def linear_bf16_workspace(n: int, m: int, k: int) -> int:
    """Floats of scratch memory that linear_bf16 needs for x [n, k], W [m, k] (0: none)."""
    lib = _any_build("vt_gemm_bf16")
    lib.vt_linear_bf16_workspace.restype = ctypes.c_longlong
    return int(lib.vt_linear_bf16_workspace(_i(n), _i(m), _i(k), _i(0)))


NORM_MAX_ROWS = 16         # rows up to which the few-row product applies an RMSNorm in front
LINK_MAX_ROWS = 64         # rows up to which a product takes a norm that the product in front has prepared
_adds_residual = {}


def linear_bf16_adds_residual(n: int, m: int, k: int) -> bool:
    """Whether linear_bf16 takes `residual` for x [n, k] and W [m, k]: up to 16 rows always (k a multiple of 8); 17
    to 64 rows where the kernel that keeps all of k inside a block is the faster one for this W, and where k is split
    over blocks (the launch that adds the partial sums then adds the residual too)."""
    key = (n, m, k)
    if key not in _adds_residual:
        _adds_residual[key] = bool(_any_build("vt_gemm_bf16").vt_linear_bf16_adds_residual(_i(n), _i(m), _i(k)))
    return _adds_residual[key]


def linear_bf16(x: torch.Tensor, w, bias: Optional[torch.Tensor], out: torch.Tensor,
                workspace: Optional[torch.Tensor] = None, norm_gain: Optional[torch.Tensor] = None,
                norm_eps: float = 0.0, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Few rows (decoding, short portions): W is read once per 64 rows.  w: a PackedMatrix (a plain [m, k] tensor
    is packed on the spot, which costs more than the product).  Shapes whose k range is split over blocks need
    `workspace` (float32, at least linear_bf16_workspace(n, m, k) elements).
    float32 output: with norm_gain (up to 16 rows), x is the float32 residual stream and rmsnorm(x; gain, eps) is
    what gets multiplied; with residual (where linear_bf16_adds_residual says so; float32 [n, m], may be `out`), out =
    residual + the product (17 to 64 rows of a shape whose k range is split: by the launch that adds the partial sums,
    which needs the workspace)."""
    n, k = x.shape
    lp = _lowp((w.data if isinstance(w, PackedMatrix) else w), "linear_bf16.w")
    if not isinstance(w, PackedMatrix):
        _chk(w, "linear_bf16.w", lp, (w.shape[0], k))
        w = pack_matrix_bf16(w)
    m = w.rows
    if w.cols != k or w.halves != 1:
        raise KernelError(f"linear_bf16: x [{n}, {k}] does not fit a packed matrix [{w.rows}, {w.cols}] x {w.halves}")
    fused = norm_gain is not None or residual is not None
    _chk(x, "linear_bf16.x", torch.float32 if norm_gain is not None else lp)
    _chk(w.data, "linear_bf16.w", lp)
    _chk(out, "linear_bf16.out", torch.float32 if fused else None, (n, m))
    if bias is not None:
        _chk(bias, "linear_bf16.bias", torch.float32, (m,))
    if fused:
        if k % 8 or (norm_gain is not None and n > NORM_MAX_ROWS):
            raise KernelError(f"linear_bf16: the fused norm takes at most {NORM_MAX_ROWS} rows and k a multiple of 8 "
                              f"(n={n}, k={k})")
        if residual is not None and not linear_bf16_adds_residual(n, m, k):
            raise KernelError(f"linear_bf16: {n} rows of [{m}, {k}] do not take a residual (linear_bf16_adds_residual)")
        if norm_gain is not None:
            _chk(norm_gain, "linear_bf16.norm_gain", torch.float32, (k,))
        if residual is not None:
            _chk(residual, "linear_bf16.residual", torch.float32, (n, m))
        need = linear_bf16_workspace(n, m, k) if n > 16 else 0
        if need and (workspace is None or workspace.numel() < need):
            raise KernelError(f"linear_bf16: x [{n}, {k}] with W [{m}, {k}] needs a workspace of {need} floats")
        if need:
            _chk(workspace, "linear_bf16.workspace", torch.float32)
        _run(load_lib("vt_gemm_bf16", half=_half(w.data, x, out)), "vt_linear_bf16_fused", _ptr(x), _ptr(norm_gain), _f(norm_eps), _ptr(w.data), _ptr(bias),
             _ptr(residual), _ptr(out), _ptr(workspace if need else None), _i(n), _i(m), _i(k), _stream())
        return out
    need = linear_bf16_workspace(n, m, k) if n > 16 else 0
    if need:
        if workspace is None:
            raise KernelError(f"linear_bf16: x [{n}, {k}] with W [{m}, {k}] needs a workspace of {need} floats")
        _chk(workspace, "linear_bf16.workspace", torch.float32)
        if workspace.numel() < need:
            raise KernelError(f"linear_bf16: workspace of {workspace.numel()} floats, need {need}")
    _run(load_lib("vt_gemm_bf16", half=_half(w.data, x, out)), "vt_linear_bf16", _ptr(x), _ptr(w.data), _ptr(bias), _ptr(out), _i(_code(out)),
         _ptr(workspace if need else None), _i(n), _i(m), _i(k), _stream())
    return out


_link_shares = {}


def linear_bf16_link_shares(n: int, m: int, k: int) -> int:
    """Blocks' shares of the rows' sums of squares that a product of this shape writes when it hands an RMSNorm on to
    the product behind it (linear_bf16_link with xn_out); 0: this shape cannot."""
    key = (n, m, k)
    if key not in _link_shares:
        _link_shares[key] = int(_any_build("vt_gemm_bf16").vt_linear_bf16_link_shares(_i(n), _i(m), _i(k)))
    return _link_shares[key]


def link_stride(n: int) -> int:
    """Floats between the shares of the rows' sums of squares that products of n rows write and read."""
    return 16 if n <= 16 else 64


def linear_bf16_link(x: torch.Tensor, w: PackedMatrix, bias: Optional[torch.Tensor], out: torch.Tensor,
                     residual: Optional[torch.Tensor] = None, ssq_in: Optional[torch.Tensor] = None, eps_in: float = 0.0,
                     xn_out: Optional[torch.Tensor] = None, gain_next: Optional[torch.Tensor] = None,
                     ssq_out: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The few-row product between RMSNorms that are no kernels of their own (up to 64 rows).
    ssq_in (float32 [shares, link_stride(n)]): x is bf16(h * gain) as the product in front left it, and the result
    is divided by the norm's root, which the shares of the rows' sums of squares give (eps_in: the norm's eps).
    xn_out (bfloat16 [n, m]; needs residual): beside out = residual + product, xn_out = bf16(out * gain_next) and this
    product's own shares ssq_out (float32 [linear_bf16_link_shares(n, m, k), link_stride(n)]) for the product behind
    the next norm.  workspace: as for linear_bf16."""
    n, k = x.shape
    lp = _lowp(w.data, "linear_bf16_link.w")
    m = w.rows
    if w.cols != k or w.halves != 1:
        raise KernelError(f"linear_bf16_link: x [{n}, {k}] does not fit a packed matrix [{w.rows}, {w.cols}] x {w.halves}")
    _chk(x, "linear_bf16_link.x", lp)
    _chk(w.data, "linear_bf16_link.w", lp)
    _chk(out, "linear_bf16_link.out", torch.float32, (n, m))
    if bias is not None:
        _chk(bias, "linear_bf16_link.bias", torch.float32, (m,))
    if residual is not None:
        _chk(residual, "linear_bf16_link.residual", torch.float32, (n, m))
        if not linear_bf16_adds_residual(n, m, k):
            raise KernelError(f"linear_bf16_link: {n} rows of [{m}, {k}] do not take a residual (linear_bf16_adds_residual)")
    n_ssq = 0
    if ssq_in is not None:
        _chk(ssq_in, "linear_bf16_link.ssq_in", torch.float32)
        if ssq_in.dim() != 2 or ssq_in.shape[1] != link_stride(n):
            raise KernelError(f"linear_bf16_link.ssq_in: shape {tuple(ssq_in.shape)}, expected [shares, {link_stride(n)}]")
        n_ssq = ssq_in.shape[0]
    if xn_out is not None:
        shares = linear_bf16_link_shares(n, m, k)
        if residual is None or shares == 0:
            raise KernelError(f"linear_bf16_link: {n} rows of [{m}, {k}] cannot hand a norm on (linear_bf16_link_shares)")
        _chk(xn_out, "linear_bf16_link.xn_out", lp, (n, m))
        _chk(gain_next, "linear_bf16_link.gain_next", torch.float32, (m,))
        _chk(ssq_out, "linear_bf16_link.ssq_out", torch.float32, (shares, link_stride(n)))
    need = linear_bf16_workspace(n, m, k) if n > 16 else 0
    if need:
        if workspace is None or workspace.numel() < need:
            raise KernelError(f"linear_bf16_link: x [{n}, {k}] with W [{m}, {k}] needs a workspace of {need} floats")
        _chk(workspace, "linear_bf16_link.workspace", torch.float32)
    _run(load_lib("vt_gemm_bf16", half=_half(w.data, x, out)), "vt_linear_bf16_link", _ptr(x), _ptr(w.data), _ptr(bias), _ptr(residual), _ptr(out),
         _ptr(workspace if need else None), _i(n), _i(m), _i(k), _ptr(ssq_in), _i(n_ssq), _f(eps_in), _ptr(xn_out),
         _ptr(gain_next), _ptr(ssq_out), _stream())
    return out


def gated_linear_bf16_link(x: torch.Tensor, w: PackedMatrix, out: torch.Tensor, ssq_in: torch.Tensor,
                           eps_in: float) -> torch.Tensor:
    """gated_linear_bf16 behind an RMSNorm that the product in front has prepared: x = bf16(h * gain), ssq_in its
    shares of the rows' sums of squares (up to 64 rows)."""
    n, k = x.shape
    lp = _lowp(w.data, "gated_linear_bf16_link.w")
    if w.cols != k or w.halves != 2:
        raise KernelError(f"gated_linear_bf16_link: x [{n}, {k}] does not fit a packed matrix [{w.rows}, {w.cols}] x {w.halves}")
    _chk(x, "gated_linear_bf16_link.x", lp)
    _chk(w.data, "gated_linear_bf16_link.w", lp)
    _chk(out, "gated_linear_bf16_link.out", None, (n, w.rows))
    _chk(ssq_in, "gated_linear_bf16_link.ssq_in", torch.float32)
    if n > 64 or ssq_in.dim() != 2 or ssq_in.shape[1] != link_stride(n):
        raise KernelError(f"gated_linear_bf16_link: {n} rows, ssq_in of shape {tuple(ssq_in.shape)}: up to 64 rows and "
                          f"[shares, {link_stride(n)}]")
    _run(load_lib("vt_gemm_bf16", half=_half(w.data, x, out)), "vt_gated_linear_bf16_link", _ptr(x), _ptr(w.data), _ptr(out), _i(_code(out)), _i(n),
         _i(w.rows), _i(k), _ptr(ssq_in), _i(ssq_in.shape[0]), _f(eps_in), _stream())
    return out


def gated_linear_bf16(x: torch.Tensor, w_gate_up, out: torch.Tensor, norm_gain: Optional[torch.Tensor] = None,
                      norm_eps: float = 0.0) -> torch.Tensor:
    """out = silu(x Wg^T) * (x Wu^T).  w_gate_up: a PackedMatrix of two halves (pack_matrix_bf16(w, halves=2)), or
    the stacked [2 I, k] tensor, which is packed on the spot.  With norm_gain (up to 16 rows), x is the float32
    residual stream and rmsnorm(x; gain, eps) is what gets multiplied."""
    n, k = x.shape
    lp = _lowp((w_gate_up.data if isinstance(w_gate_up, PackedMatrix) else w_gate_up), "gated_linear_bf16.w")
    if not isinstance(w_gate_up, PackedMatrix):
        _chk(w_gate_up, "gated_linear_bf16.w", lp, (w_gate_up.shape[0], k))
        w_gate_up = pack_matrix_bf16(w_gate_up, halves=2)
    w = w_gate_up
    if w.cols != k or w.halves != 2:
        raise KernelError(f"gated_linear_bf16: x [{n}, {k}] does not fit a packed matrix [{w.rows}, {w.cols}] x {w.halves}")
    _chk(x, "gated_linear_bf16.x", torch.float32 if norm_gain is not None else lp)
    _chk(w.data, "gated_linear_bf16.w", lp)
    _chk(out, "gated_linear_bf16.out", None, (n, w.rows))
    if norm_gain is not None:
        if n > 16 or k % 8:
            raise KernelError(f"gated_linear_bf16: the fused norm takes at most 16 rows and k a multiple of 8 (n={n}, k={k})")
        _chk(norm_gain, "gated_linear_bf16.norm_gain", torch.float32, (k,))
    _run(load_lib("vt_gemm_bf16", half=_half(w.data, x, out)), "vt_gated_linear_bf16", _ptr(x), _ptr(w.data), _ptr(out), _i(_code(out)), _i(n),
         _i(w.rows), _i(k), _ptr(norm_gain), _f(norm_eps), _stream())
    return out


# ---------------------------------------------------------------------------
def attention_f32(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, positions: torch.Tensor,
                  tok_entry: torch.Tensor, block_table: torch.Tensor, out: torch.Tensor, n_heads: int, n_kv: int,
                  head_dim: int, window: int, scale: float) -> torch.Tensor:
    n = q.shape[0]
    num_pages, kvh, page_size, d = k_pages.shape
    _chk(q, "attention_f32.q", torch.float32, (n, n_heads * head_dim))
    _chk(k_pages, "attention_f32.k_pages", torch.float32, (num_pages, n_kv, page_size, head_dim))
    _chk(v_pages, "attention_f32.v_pages", torch.float32, (num_pages, n_kv, head_dim, page_size))
    _chk(positions, "attention_f32.positions", torch.int32, (n,))
    _chk(tok_entry, "attention_f32.tok_entry", torch.int32, (n,))
    _chk(block_table, "attention_f32.block_table", torch.int32)
    _chk(out, "attention_f32.out", torch.float32, (n, n_heads * head_dim))
    _run(load_lib("vt_attn_f32"), "vt_attn_f32", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(positions), _ptr(tok_entry),
         _ptr(block_table), _ptr(out), _i(n), _i(n_heads), _i(n_kv), _i(head_dim), _i(page_size),
         _i(block_table.shape[1]), _i(num_pages), _i(window), _f(scale), _stream())
    return out


ATTN_F32_MAX_HEAD_DIM = 256     # the float32 attention kernel keeps a head's dims in a block's registers: up to this many
ATTN_ITEM_INTS = 8
ATTN_CITEM_INTS = 6


def attention_bf16(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                   items: torch.Tensor, n_items: int, citems: Optional[torch.Tensor], n_citems: int, out: torch.Tensor,
                   part_o: Optional[torch.Tensor], part_ml: Optional[torch.Tensor], n_heads: int, n_kv: int,
                   head_dim: int, window: int, scale: float, max_part: int = 0, rt: int = 1) -> torch.Tensor:
    """`items` [>=n_items, 8] int32: entry, q_tok0, q_len, pos0, first row, key_lo, key_hi, partial index (-1 = final);
    an item covers 16 * rt rows.  `citems` [>=n_citems, 6] int32: q_tok0, q_len, first row of a 16-row tile, first
    partial index, number of items, tile index within the item.  The planner (engine) makes them; `max_part` is the
    number of partial indices it used, checked against the workspace here."""
    n = q.shape[0]
    num_pages, kvh, page_size, d = k_pages.shape
    lp = _lowp(k_pages, "attention_bf16.k_pages")
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention_bf16: head size {head_dim} is not a multiple of 16 in 16..256")
    if rt not in (1, 2, 3):
        raise KernelError(f"attention_bf16: {rt} row tiles per item (1 or 2)")
    _chk(q, "attention_bf16.q", lp, (n, n_heads * head_dim))
    _chk(k_pages, "attention_bf16.k_pages", lp, (num_pages, n_kv, page_size, head_dim))
    _chk(v_pages, "attention_bf16.v_pages", lp, (num_pages, n_kv, head_dim, page_size))
    _chk(block_table, "attention_bf16.block_table", torch.int32)
    _chk(items, "attention_bf16.items", torch.int32)
    _chk(out, "attention_bf16.out", lp, (n, n_heads * head_dim))
    if items.numel() < n_items * ATTN_ITEM_INTS:
        raise KernelError("attention_bf16: item list shorter than n_items")
    if n_citems:
        _chk(citems, "attention_bf16.citems", torch.int32)
        _chk(part_o, "attention_bf16.part_o", torch.float32)
        _chk(part_ml, "attention_bf16.part_ml", torch.float32)
        if citems.numel() < n_citems * ATTN_CITEM_INTS:
            raise KernelError("attention_bf16: combine list shorter than n_citems")
        if part_o.numel() < max_part * rt * n_kv * 16 * head_dim or part_ml.numel() < max_part * rt * n_kv * 16 * 2:
            raise KernelError("attention_bf16: workspace for split keys is too small")
    lib = load_lib("vt_attn_bf16", head_dim, half=_half(k_pages, v_pages, out))
    _run(lib, "vt_attn_bf16", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(block_table), _ptr(items), _i(n_items), _i(rt),
         _ptr(citems), _i(n_citems), _ptr(out), _ptr(part_o), _ptr(part_ml), _i(n_heads), _i(n_kv), _i(page_size),
         _i(block_table.shape[1]), _i(num_pages), _i(window), _f(scale), _stream())
    return out


def attention_bf16_direct(head_dim: int) -> bool:
    """Whether the bfloat16 attention kernels of this head size load their key/value blocks straight into LDS; the
    host cuts their work differently then (parts.attention_plan)."""
    return bool(_any_build("vt_attn_bf16", head_dim).vt_attn_bf16_direct())


def attention_bf16_tiles(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                         items: torch.Tensor, n_items: int, out: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                         window: int, scale: float, rt: int = 1, citems: Optional[torch.Tensor] = None, n_citems: int = 0,
                         part_o: Optional[torch.Tensor] = None, part_ml: Optional[torch.Tensor] = None,
                         n_parts: int = 0) -> torch.Tensor:
    """Long portions: `items` as for attention_bf16, each 64 * rt rows of one entry against all the keys they may
    see, or (partial index >= 0) against one of several ranges of them; key and value blocks go through LDS once per
    block of four waves.  `citems` [>=n_citems, 6] as for attention_bf16, one per 16-row tile of every item whose keys
    were split (4 * rt tiles per item); part_o / part_ml: float32 workspaces of at least n_parts * 4 * rt * n_kv *
    16 * head_dim and n_parts * 4 * rt * n_kv * 32 elements."""
    n = q.shape[0]
    num_pages, kvh, page_size, d = k_pages.shape
    lp = _lowp(k_pages, "attention_bf16_tiles.k_pages")
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention_bf16_tiles: head size {head_dim} is not a multiple of 16 in 16..256")
    if rt not in (1, 2):
        raise KernelError(f"attention_bf16_tiles: {rt} row tiles per wave (1 or 2)")
    _chk(q, "attention_bf16_tiles.q", lp, (n, n_heads * head_dim))
    _chk(k_pages, "attention_bf16_tiles.k_pages", lp, (num_pages, n_kv, page_size, head_dim))
    _chk(v_pages, "attention_bf16_tiles.v_pages", lp, (num_pages, n_kv, head_dim, page_size))
    _chk(block_table, "attention_bf16_tiles.block_table", torch.int32)
    _chk(items, "attention_bf16_tiles.items", torch.int32)
    _chk(out, "attention_bf16_tiles.out", lp, (n, n_heads * head_dim))
    if items.numel() < n_items * ATTN_ITEM_INTS:
        raise KernelError("attention_bf16_tiles: item list shorter than n_items")
    if n_citems or n_parts:
        if citems is None or part_o is None or part_ml is None:
            raise KernelError("attention_bf16_tiles: split keys need citems and the two workspaces")
        _chk(citems, "attention_bf16_tiles.citems", torch.int32)
        _chk(part_o, "attention_bf16_tiles.part_o", torch.float32)
        _chk(part_ml, "attention_bf16_tiles.part_ml", torch.float32)
        if citems.numel() < n_citems * ATTN_CITEM_INTS:
            raise KernelError("attention_bf16_tiles: combine list shorter than n_citems")
        if part_o.numel() < n_parts * 4 * rt * n_kv * 16 * head_dim or part_ml.numel() < n_parts * 4 * rt * n_kv * 32:
            raise KernelError(f"attention_bf16_tiles: workspaces too small for {n_parts} partial results")
    _run(load_lib("vt_attn_bf16", head_dim, half=_half(k_pages, v_pages, out)), "vt_attn_bf16_tiles", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
         _ptr(items), _i(n_items), _i(rt), _ptr(citems if n_citems else None), _i(n_citems), _ptr(out),
         _ptr(part_o if n_citems else None), _ptr(part_ml if n_citems else None), _i(n_heads), _i(n_kv), _i(page_size),
         _i(block_table.shape[1]), _i(num_pages), _i(window), _f(scale), _stream())
    return out


def attention_bf16_decode(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                          entry_pos0: torch.Tensor, dec_params: torch.Tensor, p_max: int, out: torch.Tensor,
                          part_o: torch.Tensor, part_ml: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                          window: int, scale: float) -> torch.Tensor:
    """One token per entry (token i is entry i at position entry_pos0[i]); every entry's keys are cut into at most
    p_max items of dec_params[0] keys.  All that changes from step to step is read from device memory."""
    n = q.shape[0]
    num_pages, kvh, page_size, d = k_pages.shape
    lp = _lowp(k_pages, "attention_bf16_decode.k_pages")
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention_bf16_decode: head size {head_dim} is not a multiple of 16 in 16..256")
    _chk(q, "attention_bf16_decode.q", lp, (n, n_heads * head_dim))
    _chk(k_pages, "attention_bf16_decode.k_pages", lp, (num_pages, n_kv, page_size, head_dim))
    _chk(v_pages, "attention_bf16_decode.v_pages", lp, (num_pages, n_kv, head_dim, page_size))
    _chk(block_table, "attention_bf16_decode.block_table", torch.int32)
    if block_table.shape[0] < n:
        raise KernelError("attention_bf16_decode: fewer block table rows than entries")
    _chk(entry_pos0, "attention_bf16_decode.entry_pos0", torch.int32, (n,))
    _chk(dec_params, "attention_bf16_decode.dec_params", torch.int32)
    _chk(out, "attention_bf16_decode.out", lp, (n, n_heads * head_dim))
    _chk(part_o, "attention_bf16_decode.part_o", torch.float32)
    _chk(part_ml, "attention_bf16_decode.part_ml", torch.float32)
    if part_o.numel() < n * p_max * n_kv * 16 * head_dim or part_ml.numel() < n * p_max * n_kv * 32:
        raise KernelError("attention_bf16_decode: workspace too small")
    _run(load_lib("vt_attn_bf16", head_dim, half=_half(k_pages, v_pages, out)), "vt_attn_bf16_decode", _ptr(q), _ptr(k_pages), _ptr(v_pages),
         _ptr(block_table), _ptr(entry_pos0), _ptr(dec_params), _i(n), _i(p_max), _ptr(out), _ptr(part_o), _ptr(part_ml),
         _i(n_heads), _i(n_kv), _i(page_size), _i(block_table.shape[1]), _i(num_pages), _i(window), _f(scale), _stream())
    return out


def attention_bf16_decode_fused(qkv: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                                k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                                entry_pos0: torch.Tensor, dec_params: torch.Tensor, p_max: int, out: torch.Tensor,
                                part_o: torch.Tensor, part_ml: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                                window: int, scale: float) -> torch.Tensor:
    """attention_bf16_decode from the projections' fp32 output (queries, keys, values of token i = entry i in row i):
    the attention kernel rotates queries and the new key and writes key and value into the token's page itself."""
    n = qkv.shape[0]
    num_pages, kvh, page_size, d = k_pages.shape
    lp = _lowp(k_pages, "attention_bf16_decode_fused.k_pages")
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention_bf16_decode_fused: head size {head_dim} is not a multiple of 16 in 16..256")
    _chk(qkv, "attention_bf16_decode_fused.qkv", torch.float32)
    if qkv.dim() != 2 or qkv.shape[1] < (n_heads + 2 * n_kv) * head_dim or qkv.stride(1) != 1:
        raise KernelError(f"attention_bf16_decode_fused.qkv: shape {tuple(qkv.shape)} does not hold {n_heads}+2x{n_kv} heads of {head_dim}")
    rot = max_pos = 0
    if cos is not None:
        _chk(cos, "attention_bf16_decode_fused.cos", torch.float32)
        _chk(sin, "attention_bf16_decode_fused.sin", torch.float32, cos.shape)
        max_pos, half = cos.shape
        rot = 2 * half
        if rot % 16 or rot > head_dim:
            raise KernelError(f"attention_bf16_decode_fused: {rot} rotated dims (a multiple of 16 up to {head_dim})")
    _chk(k_pages, "attention_bf16_decode_fused.k_pages", lp, (num_pages, n_kv, page_size, head_dim))
    _chk(v_pages, "attention_bf16_decode_fused.v_pages", lp, (num_pages, n_kv, head_dim, page_size))
    _chk(block_table, "attention_bf16_decode_fused.block_table", torch.int32)
    if block_table.shape[0] < n:
        raise KernelError("attention_bf16_decode_fused: fewer block table rows than entries")
    _chk(entry_pos0, "attention_bf16_decode_fused.entry_pos0", torch.int32, (n,))
    _chk(dec_params, "attention_bf16_decode_fused.dec_params", torch.int32)
    _chk(out, "attention_bf16_decode_fused.out", lp, (n, n_heads * head_dim))
    _chk(part_o, "attention_bf16_decode_fused.part_o", torch.float32)
    _chk(part_ml, "attention_bf16_decode_fused.part_ml", torch.float32)
    if part_o.numel() < n * p_max * n_kv * 16 * head_dim or part_ml.numel() < n * p_max * n_kv * 32:
        raise KernelError("attention_bf16_decode_fused: workspace too small")
    _run(load_lib("vt_attn_bf16", head_dim, half=_half(k_pages, v_pages, out)), "vt_attn_bf16_decode_fused", _ptr(qkv), ctypes.c_longlong(qkv.stride(0)),
         _ptr(cos), _ptr(sin), _i(rot), _i(max_pos), _ptr(k_pages), _ptr(v_pages), _ptr(block_table), _ptr(entry_pos0),
         _ptr(dec_params), _i(n), _i(p_max), _ptr(out), _ptr(part_o), _ptr(part_ml), _i(n_heads), _i(n_kv),
         _i(page_size), _i(block_table.shape[1]), _i(num_pages), _i(window), _f(scale), _stream())
    return out


# ---------------------------------------------------------------------------
def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor, work: torch.Tensor, out: torch.Tensor,
           partials: Optional[torch.Tensor] = None) -> torch.Tensor:
    """partials: scratch of sample_partials_size(rows) floats (made here if not given)."""
    rows, vocab = logits.shape
    _chk(logits, "sample.logits", torch.float32)
    _chk(temperature, "sample.temperature", torch.float32, (rows,))
    _chk(top_k, "sample.top_k", torch.int32, (rows,))
    _chk(top_p, "sample.top_p", torch.float32, (rows,))
    _chk(uniform, "sample.uniform", torch.float32, (rows,))
    _chk(work, "sample.work", torch.float32)
    if work.numel() < rows * vocab:
        raise KernelError("sample: workspace smaller than the logits")
    _chk(out, "sample.out", torch.int32, (rows,))
    if partials is None:
        partials = torch.empty(sample_partials_size(rows), dtype=torch.float32, device=logits.device)
    _chk(partials, "sample.partials", torch.float32)
    if partials.numel() < sample_partials_size(rows):
        raise KernelError("sample: scratch for the slices' maxima is too small")
    _run(load_lib("vt_sampling"), "vt_sample", _ptr(logits), _i(rows), _i(vocab), _ptr(temperature), _ptr(top_k),
         _ptr(top_p), _ptr(uniform), _ptr(work), _ptr(partials), _ptr(out), _stream())
    return out


def sample_partials_size(rows: int) -> int:
    return 2 * max(1, rows) * int(load_lib("vt_sampling").vt_sample_slices())


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise KernelError("no GPU is visible: this engine has no CPU path")
    return torch.device("cuda", torch.cuda.current_device())
