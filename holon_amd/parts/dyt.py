"""Dynamic Tanh in place of a norm, and the block that is built around it.

`norm dyt`: y = tanh(alpha x) w + b with a scalar `alpha` and vectors `w`, `b`. Nothing is summed over a row, so the
norm is elementwise and any number of them fuse with the adds around them. Arithmetic is float32.

`block sandwich32`: a norm in front of and behind each sublayer, over a residual stream kept in float32:

    x += m post1(mixer(pre1(x)));   x += m post2(ffn(pre2(x)))

with `m` a constant of the model (`residual_mult`). A layer may lack the feed-forward. A block with `reentry` adds the
embedding's rows (`Stream.origin`) to x in front of every run of it but the first (a range of layers that runs several
times, fed the embedding again at each pass). Every add and the norms on both sides of it are one kernel
(`csrc/dyt.hip`): a sublayer's result travels as a `Scaled` term until the next norm reads the stream.
"""
from __future__ import annotations

import ctypes

import torch

from ..kernels.registry import KernelOp, register_kernel
from ..registry import register_part
from ..spec import PartRef
from .base import FLOAT32, Build, NormPart, Part, Stream

_P, _I, _L, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
_DT = {torch.float32: 0, torch.bfloat16: 1}


def _ptr(t):
    return None if t is None else t.data_ptr()


def _need(cond: bool, what: str) -> None:
    if not cond:
        raise ValueError(what)


def _dyt(x, params):
    alpha, w, b = params
    return torch.tanh(alpha.float() * x.float()) * w.float() + b.float()


def dyt_stream_plain(x, term, post, scale, extra, pre, out_dtype):
    """x [T, W] (float32: updated in place when there is anything to add; any dtype when there is not);
    `term` [T, W] with `post` = (alpha [], w [W], b [W]) float32: x += scale * (tanh(alpha term) w + b);
    `extra` [T, W] float32: x += extra, after the term; `pre`: returns tanh(alpha x) w + b in `out_dtype`, else None.
    float32 arithmetic, one rounding of what is returned."""
    if term is not None:
        x.add_(scale * _dyt(term, post))
    if extra is not None:
        x.add_(extra)
    return _dyt(x, pre).to(out_dtype) if pre is not None else None


def _dyt_stream_hip(launch, x, term, post, scale, extra, pre, out_dtype):
    _need(x.is_cuda and x.is_contiguous() and x.dim() == 2 and x.dtype in _DT, "dyt_stream: contiguous rows on the GPU")
    rows, dim = x.shape
    changes = term is not None or extra is not None
    _need(not changes or x.dtype == torch.float32, "dyt_stream: terms are added into float32 rows")
    _need((term is None) == (post is None), "dyt_stream: a term comes with the norm behind it")
    for t, what in ((term, "term"), (extra, "extra")):
        _need(t is None or (t.is_cuda and t.is_contiguous() and t.shape == x.shape and t.dtype in _DT),
              f"dyt_stream: {what} must be contiguous rows of the stream's shape")
    _need(extra is None or extra.dtype == torch.float32, "dyt_stream: extra rows are float32")
    for p in (post, pre):
        _need(p is None or (p[0].dtype == torch.float32 and p[0].numel() == 1 and all(
            v.dtype == torch.float32 and v.is_contiguous() and v.shape == (dim,) for v in p[1:])),
            "dyt_stream: a norm is (alpha [], w [W], b [W]) in float32")
    y = None
    if pre is not None:
        _need(out_dtype in _DT, "dyt_stream: float32 or bfloat16 out")
        y = torch.empty((rows, dim), dtype=out_dtype, device=x.device)
    if rows == 0 or (not changes and pre is None):
        return y
    po, pr = post or (None, None, None), pre or (None, None, None)
    launch(x.data_ptr(), _DT[x.dtype], _ptr(term), _DT[term.dtype] if term is not None else 0, _ptr(po[0]), _ptr(po[1]),
           _ptr(po[2]), float(scale), _ptr(extra), _ptr(pr[0]), _ptr(pr[1]), _ptr(pr[2]), _ptr(y),
           _DT[out_dtype] if y is not None else 0, rows, dim)
    return y


register_kernel(KernelOp("dyt_stream", dyt_stream_plain, "holon_dyt_stream",
                         [_P, _I, _P, _I, _P, _P, _P, _F, _P, _P, _P, _P, _P, _I, _L, _I], _dyt_stream_hip))


class Scaled:
    """A sublayer's result that is not yet in the stream: what is to be added is scale * norm(term)."""

    def __init__(self, term: torch.Tensor, norm: "DynamicTanh", scale: float) -> None:
        self.term, self.norm, self.scale = term, norm, scale

    def index_select(self, dim: int, index: torch.Tensor) -> "Scaled":
        if dim != 0:
            raise ValueError("Scaled.index_select: rows only (dim 0)")
        return Scaled(self.term.index_select(0, index), self.norm, self.scale)


@register_part("norm", "dyt")
class DynamicTanh(NormPart):
    """y = tanh(alpha x) weight + bias over rows of `dim` values; `eps` is accepted and unused (the norm takes no
    mean or variance). The parameters are kept in float32. The result is in the engine's dtype unless asked
    otherwise."""

    graph_safe = True

    def __init__(self, build: Build, *, dim: int, eps: float = 0.0) -> None:
        super().__init__(build)
        self.dim = dim
        self.declare("weight", (dim,), kind=FLOAT32, init="norm")
        self.declare("bias", (dim,), kind=FLOAT32, init="zero")
        self.declare("alpha", (), kind=FLOAT32, init="unit")

    def params(self) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        return self.alpha, self.weight, self.bias

    def forward(self, x: torch.Tensor, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        return self.kernels.dyt_stream(x, None, None, 0.0, None, self.params(), out_dtype or self.build.dtype)

    __call__ = forward

    def add(self, x, residual: torch.Tensor, extra: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        """(norm(residual + x [+ extra]), the sum): `residual` is float32 and takes the sum in place. `x`: None, a
        `Scaled` term, or a plain tensor (added as it is, by the elementwise add of torch)."""
        term = post = None
        scale = 0.0
        if isinstance(x, Scaled):
            term, post, scale = x.term, x.norm.params(), x.scale
        elif x is not None:
            residual.add_(x)
        return self.kernels.dyt_stream(residual, term, post, scale, extra, self.params(), self.build.dtype), residual


@register_part("block", "sandwich32")
class Sandwich32(Part):
    """x += m post1(mixer(pre1(x))); x += m post2(ffn(pre2(x))) over a float32 stream; see the module's text. The four
    norms are of the kind the layer names (`norm`), called `norm1`, `norm1b`, `norm2`, `norm2b`; that kind's `add`
    must take `Scaled` terms (the Dynamic Tanh does)."""

    graph_safe = True
    reads_origin = False

    def __init__(self, build: Build, *, layer: int, hidden: int, mixer: PartRef, ffn: PartRef | None, norm: PartRef,
                 scale: float = 1.0, reentry: bool = False) -> None:
        super().__init__(build)
        self.hidden, self.scale = hidden, float(scale)
        self.attach("norm1", build.make(norm, dim=hidden))
        self.attach("mixer", build.make(mixer, layer=layer, hidden=hidden))
        self.attach("norm1b", build.make(norm, dim=hidden))
        self.ffn = None
        if ffn is not None:
            self.attach("norm2", build.make(norm, dim=hidden))
            self.attach("ffn", build.make(ffn, layer=layer, hidden=hidden))
            self.attach("norm2b", build.make(norm, dim=hidden))
        self.reentry = bool(reentry)
        self.reads_origin = self.reentry

    def forward(self, stream: Stream, step, site) -> Stream:
        h = stream.h
        if h.dtype != torch.float32 or h is stream.origin:       # the stream becomes float32 rows of its own (the
            h = stream.h = h.to(torch.float32, copy=True)        # embedding's rows stay as they are)
        again = stream.origin if self.reentry and site.turn > 0 else None
        a = self.norm1.add(stream.delta, h, extra=again)[0]
        stream.delta = stream.stats = None
        mixed = Scaled(self.mixer(a, step, site), self.norm1b, self.scale)
        if self.ffn is None:
            stream.delta = mixed
            return stream
        x = self.norm2.add(mixed, h)[0]
        stream.delta = Scaled(self.ffn(x, step), self.norm2b, self.scale)
        return stream

    __call__ = forward
