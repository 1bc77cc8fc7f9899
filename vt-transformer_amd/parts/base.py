"""What a part is, and the registries that parts are chosen from.

A model is put together from parts of five roles.  Each part gets its sizes
and constants as constructor parameters (from a `PartSpec`), says which
tensors it needs, and computes on the tokens of one step.  No part knows
which model it is in, which layer it is, or what the other parts of its
layer are.

Interfaces (N = tokens of the step, H = model width):

  Norm            forward(h[N,H] fp32, delta[N,H] or None, rows=None) -> normed [N or R, H] in the runtime's dtype.
                  With `delta`, h += delta happens first (and is stored in h unless `rows` picks rows).
  PositionEncoding
                  rotary_tables(n_positions) -> (cos, sin) fp32 [n_positions, dims/2] or None if the
                  encoding is not a rotation that the fused kernel can apply;
                  apply(q, k, positions) -> (q, k) otherwise.
  Mixer           forward(x[N,H], ctx, cache, state) -> [N,H]; cache_need() / state_need() say what the cache
                  manager has to hold for it (keys and values in pages; fixed-size state per request).
                  Optional: prepare_step(ctx) -> {key: int32 array} or None, called on the host once per step
                  before the step's metadata goes to the device; what it returns is found in ctx.extra[key] on
                  the device when the part runs (work items of its kernels, lengths they read from memory).
  FeedForward     forward(x[N,H], ctx) -> [N,H]
  Embedding       forward(ids[N] int32) -> h[N,H] fp32; `name` and `table` say what it has loaded.
  Head            load(get, rt, shared) where `shared` maps tensor names to tensors that other parts have placed
                  on the device already (a tied head finds the embedding's table there); forward(x[R,H]) -> fp32
                  logits [R,V].
  Block           forward(h, delta, ctx, cache, state) -> (h, delta): arranges two norms, a mixer and a
                  feed-forward around the fp32 residual stream h.  `delta` is a layer output that has
                  not been added to h yet, so that the next norm can fuse the addition.

The reference's counterpart is the set of `op.*` words that a model program
strings together (v1/tensortype/nn_operators.cpp:530-576) and its user words
with stack parameters (v1/models/qwen2-7b/inference_fp16.dag:287-345).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional, Tuple

import torch

from ..config.base import ConfigError, PartSpec


@dataclass(frozen=True)
class TensorDecl:
    """A tensor that a part needs: its shape and what it is.

    role "matrix": kept in the runtime's dtype (bfloat16, float16 or float32);
    "gain", "bias": small vectors, kept in float32 (exact from bfloat16);
    "table": integers, kept as int32.  A tensor stored in 32-bit stays so."""

    shape: Tuple[int, ...]
    role: str
    optional: bool = False


@dataclass(frozen=True)
class PageTensor:
    """One tensor of a cache page, as the mixer that owns it lays it out: what it keeps per token (`token_shape`)
    and where the page's token slots lie among those axes (`slot_axis`: the index at which an axis of page_size
    slots is inserted).  Keys kept as [kv head][slot][D] are PageTensor("k", (kv_heads, D), 1); values kept
    transposed, [kv head][D][slot], are PageTensor("v", (kv_heads, D), 2); one latent vector per token is
    PageTensor("latent", (rank,), 0).  dtype None: the runtime's."""

    name: str
    token_shape: Tuple[int, ...]
    slot_axis: int = 0
    dtype: Optional[torch.dtype] = None

    def __post_init__(self):
        if not 0 <= self.slot_axis <= len(self.token_shape):
            raise ValueError(f"page tensor '{self.name}': slot axis {self.slot_axis} is outside its {len(self.token_shape)} axes")

    def page_shape(self, page_size: int) -> Tuple[int, ...]:
        s = [int(x) for x in self.token_shape]
        s.insert(self.slot_axis, int(page_size))
        return tuple(s)

    def token_elems(self) -> int:
        n = 1
        for x in self.token_shape:
            n *= int(x)
        return n


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer wants kept in pages: the tensors of a page (the layout is the mixer's own: the cache manager
    only allocates what is listed and hands the mixer a dict by name), how long a token's entry stays alive, and the
    page sizes that the mixer's kernels take.  Layers whose needs are equal share a group of pages (one pool, one
    block table per request)."""

    tensors: Tuple[PageTensor, ...]
    window: int = 0  # 0: every token stays; W: a token is dead once W later tokens exist
    page_multiple: int = 1  # the mixer's kernels take pages whose size is a multiple of this many tokens

    def group_key(self):
        return (self.tensors, self.window)

    def same_layout(self, other: "CacheNeed") -> bool:
        """Whether a mixer with this need can read pages that a mixer with the other need writes."""
        return self.tensors == other.tensors

    def bytes_per_token(self, runtime_dtype: torch.dtype) -> int:
        return sum(t.token_elems() * torch.empty((), dtype=t.dtype or runtime_dtype).element_size() for t in self.tensors)


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size that a mixer wants kept between steps."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class Runtime:
    """Device, dtype and scratch buffers shared by the parts of one model."""

    def __init__(self, device: torch.device, dtype: torch.dtype, keep_row_major: bool = True):
        if dtype not in (torch.bfloat16, torch.float16, torch.float32):
            raise ValueError(f"dtype {dtype} is not supported (bfloat16, float16 and float32 are)")
        self.device = device
        self.dtype = dtype
        # a 16-bit type (bfloat16, or float16, the reference's own: v1/tensortype/hip_tensor.cpp:514-535): the
        # matrix-core kernels; float32: the true 32-bit path
        self.lowp = dtype != torch.float32
        # a 16-bit model keeps every matrix twice: row-major for the GEMM library (long portions) and packed for the
        # few-row kernels.  False: the packed copy only, and long portions go through the few-row kernels 64 rows
        # at a time, which reads W once per 64 rows: several times slower on prompts, half the memory (a model
        # that fits the GPU once but not twice).
        self.keep_row_major = bool(keep_row_major) or not self.lowp
        self._buffers: Dict[str, torch.Tensor] = {}
        self._scope = ""

    def place(self, t: torch.Tensor, role: str) -> torch.Tensor:
        """A loaded tensor as the kernels want it, on the device."""
        if role == "matrix":
            if t.dtype in (torch.float32, torch.bfloat16, torch.float16, torch.float64):
                return t.to(device=self.device, dtype=self.dtype).contiguous()
            raise ValueError(f"matrix of dtype {t.dtype}")
        if role in ("gain", "bias"):
            return t.to(device=self.device, dtype=torch.float32).contiguous()
        if role == "table":
            return t.to(device=self.device, dtype=torch.int32).contiguous()
        raise ValueError(f"unknown tensor role {role!r}")

    def pack(self, w: torch.Tensor, halves: int = 1):
        """The 16-bit matrix once more in the order the few-row matrix kernels read it (None in float32).  The
        row-major matrix stays for the GEMM library, which long portions go through."""
        if not self.lowp:
            return None
        from ..kernels import ops
        return ops.pack_matrix_bf16(w, halves)

    def row_major(self, w: torch.Tensor, packed) -> Optional[torch.Tensor]:
        """The row-major matrix to keep beside its packed copy: `w`, or None where only the packed copy stays."""
        return w if (self.keep_row_major or packed is None) else None

    def buffer(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        """A scratch tensor that keeps its address between steps (grown when a step needs more)."""
        n = 1
        for s in shape:
            n *= int(s)
        name = self._scope + name
        buf = self._buffers.get(name)
        if buf is None or buf.dtype != dtype or buf.numel() < n:
            if self._scope and torch.cuda.is_current_stream_capturing():
                raise RuntimeError(f"scratch buffer '{name}' would be allocated while a graph is being captured")
            buf = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._buffers[name] = buf
        return buf[:n].view(*shape)

    def scoped(self, prefix: str):
        """Scratch buffers asked for inside this context are a set of their own: a captured graph keeps the
        addresses of its buffers, so they must never be regrown by steps of another shape."""
        rt = self

        class _Scope:
            def __enter__(self_inner):
                self_inner.prev = rt._scope
                rt._scope = prefix
                return rt

            def __exit__(self_inner, *exc):
                rt._scope = self_inner.prev
                return False
        return _Scope()


class NormedInput:
    """What a block hands to a mixer or feed-forward that says it `takes_normed_input`: the residual stream and the
    norm that is to be applied to it, not yet applied, so that the part's first matrix product can do it on the way
    (few rows in bfloat16).  `materialize()` is the norm as a kernel of its own, for whoever cannot.

    The product in front of the norm may have `prepared` it (a part that `hands_norm_on`): beside adding its result
    to the stream it has written `xn` = bfloat16(h * gain) and `ssq`, its blocks' shares of the rows' sums of squares,
    so that the product behind the norm reads bfloat16 tokens and only divides its sums by the norm's root."""

    def __init__(self, h: torch.Tensor, norm, xn: Optional[torch.Tensor] = None, ssq: Optional[torch.Tensor] = None):
        self.h, self.norm, self.xn, self.ssq = h, norm, xn, ssq

    @property
    def prepared(self) -> bool:
        return self.xn is not None

    @property
    def shape(self):
        return self.h.shape

    @property
    def gain(self) -> torch.Tensor:
        return self.norm.gain

    @property
    def eps(self) -> float:
        return self.norm.eps

    def materialize(self) -> torch.Tensor:
        return self.norm.forward(self.h, None)


class HostStaging:
    """Pinned host buffers in rotation for copies to the device that do not make the host wait: a buffer is
    written again only after the copy that last read it has run."""

    def __init__(self, dtype: torch.dtype, depth: int = 4):
        self.dtype = dtype
        self._slots = [[None, None] for _ in range(depth)]   # [pinned tensor, event of its last copy]
        self._next = 0

    def upload(self, host, dev: torch.Tensor) -> None:
        """host: a numpy array of the buffer's dtype; dev: a device tensor of the same size."""
        self.upload_pieces([(host, dev)])

    def upload_pieces(self, pieces) -> None:
        """Several (host array, device tensor of the same size) pairs through one pinned buffer: one wait for the
        buffer, one copy to the device per piece."""
        n = sum(int(h.size) for h, _ in pieces)
        slot = self._slots[self._next]
        self._next = (self._next + 1) % len(self._slots)
        if slot[1] is not None:
            slot[1].synchronize()
        if slot[0] is None or slot[0].numel() < n:
            slot[0] = torch.empty(max(n, 256), dtype=self.dtype, pin_memory=True)
        at = 0
        for host, dev in pieces:
            k = int(host.size)
            if k == 0:
                continue
            slot[0][at:at + k].numpy()[...] = host.reshape(-1)
            dev.view(-1).copy_(slot[0][at:at + k], non_blocking=True)
            at += k
        if slot[1] is None:
            slot[1] = torch.cuda.Event()
        slot[1].record()


class Part:
    """Base of all parts."""

    # True: a decoding step through this part can be recorded once and replayed, i.e. between one step and the
    # next only values in device memory change (token ids, positions, block tables), never the launches, their
    # sizes or host values baked into them.  The step function replays decoding steps only if every part of the
    # model says so; a part that does not know stays with the default and its model is run step by step.
    replayable = False

    def tensors(self) -> Dict[str, TensorDecl]:
        """Full tensor names this part loads, with their shapes."""
        return {}

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        """Take the tensors named by `tensors()` (get(name) -> CPU or device tensor) onto the device."""


class Registry:
    def __init__(self, role: str):
        self.role = role
        self._kinds: Dict[str, Any] = {}

    def register(self, kind: str, cls=None):
        if cls is None:
            def deco(c):
                self._kinds[kind] = c
                return c
            return deco
        self._kinds[kind] = cls
        return cls

    def kinds(self):
        return sorted(self._kinds)

    def build(self, spec: PartSpec, **context):
        if spec.kind not in self._kinds:
            raise ConfigError(f"no {self.role} of kind '{spec.kind}' is registered (known: {', '.join(self.kinds())})")
        return self._kinds[spec.kind](**context, **spec.params)


NORMS = Registry("norm")
POSITIONS = Registry("position encoding")
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
BLOCKS = Registry("block")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("head")
