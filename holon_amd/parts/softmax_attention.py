"""Softmax attention over the paged cache for heads whose keys and values may differ in width, with the options a
design may name: biases on the q/k/v projections, rotary positions in either pairing, a scale of its own, a sliding
window, and a sink (one trained scalar for each head whose exponential is added to the softmax's normaliser; nothing
is read from the cache for it).
Two mixers use it: `attention` (grouped queries) and `latent_attention` (keys and values rebuilt from a cached
low-rank latent, computed in the latent's space so that nothing but the latent is kept).

Pages are laid out as the sigmoid attention lays them out (`parts/sigmoid_attention.py`): keys `[Hkv, P, D]`, then
values `[Hkv, V, P]`; `head_prepare` writes them. HIP form: `csrc/softmax_attention.hip`.
"""
from __future__ import annotations

import ctypes

import torch

from ..kernels.registry import KernelOp, register_kernel
from ..registry import register_part
from ..spec import PartRef
from .base import FLOAT32, Build, PagedState, Part
from .linear import Linear

_P, _I, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
_DT = {torch.float32: 0, torch.bfloat16: 1}


def _ptr(t):
    return None if t is None else t.data_ptr()


def softmax_attention_plain(q, pages, table, rows, token_row, positions, kv_heads, vdim, page_size, sink, scale,
                            window):
    """q [T, H, D]; `pages` [pages, G P (D + V)] (keys [G, P, D], then values [G, V, P]); `table` [S, max_pages]
    int32; token t belongs to row token_row[t] (slot rows.slots[row]) and stands at positions[t]. Query at position p
    sees keys max(0, p - window + 1) .. p (window 0: 0 .. p). weights = exp(s_j - top) / (sum_j exp(s_j - top) +
    exp(sink[h] - top)) with s = q . k * scale, `sink` [H] float32 or None (then no such term). -> [T, H V] in q's
    dtype; scores, weights and sums in float32."""
    t, heads, dim = q.shape
    keys = pages[:, : kv_heads * page_size * dim].view(-1, kv_heads, page_size, dim)
    vals = pages[:, kv_heads * page_size * dim:].view(-1, kv_heads, vdim, page_size).transpose(2, 3)
    out = torch.zeros((t, heads, vdim), dtype=torch.float32, device=q.device)
    pos = positions.tolist()
    slot_of, row_of = rows.slots.tolist(), token_row.tolist()
    group = heads // kv_heads
    for i in range(t):
        first = max(0, pos[i] - window + 1) if window > 0 else 0
        js = torch.arange(first, pos[i] + 1, device=q.device)
        pg = table[slot_of[row_of[i]], (js // page_size)].long()
        off = js % page_size
        kk = keys[pg, :, off].float().repeat_interleave(group, dim=1)                  # [n, H, D]
        vv = vals[pg, :, off].float().repeat_interleave(group, dim=1)                  # [n, H, V]
        s = torch.einsum("hd,nhd->nh", q[i].float(), kk) * scale
        top = s.max(0).values
        if sink is not None:
            top = torch.maximum(top, sink.float())
        w = torch.exp(s - top)
        den = w.sum(0)
        if sink is not None:
            den = den + torch.exp(sink.float() - top)
        out[i] = torch.einsum("nh,nhv->hv", w, vv) / den[:, None]
    return out.view(t, heads * vdim).to(q.dtype)


def _softmax_attention_hip(launch, q, pages, table, rows, token_row, positions, kv_heads, vdim, page_size, sink,
                           scale, window):
    t, heads, dim = q.shape
    ok = q.is_cuda and q.is_contiguous() and q.dtype in _DT and pages.dtype == q.dtype and pages.is_contiguous() \
        and pages.dim() == 2 and pages.shape[1] == kv_heads * page_size * (dim + vdim) and table.dtype == torch.int32 \
        and table.is_contiguous() and heads % kv_heads == 0 and token_row.shape[0] >= t and positions.shape[0] >= t \
        and (sink is None or (sink.dtype == torch.float32 and sink.is_contiguous() and sink.shape == (heads,)))
    if not ok:
        raise ValueError(f"softmax_attention: q {tuple(q.shape)} {q.dtype}, pages {tuple(pages.shape)} do not fit "
                         f"{kv_heads} kv heads, values of {vdim}, page {page_size}")
    out = torch.empty((t, heads * vdim), dtype=q.dtype, device=q.device)
    launch(q.data_ptr(), out.data_ptr(), pages.data_ptr(), table.data_ptr(), table.shape[1], table.shape[0],
           rows.slots.data_ptr(), token_row.data_ptr(), positions.data_ptr(), t, heads, kv_heads, dim, vdim, page_size,
           pages.shape[0], _ptr(sink), float(scale), int(window), _DT[q.dtype])
    return out


def head_linear_plain(x, weight):
    """x [T, H, A], weight [H, B, A] -> [T, H, B]: every head's own small projection, sums in float32, the result in
    x's dtype."""
    return torch.einsum("tha,hba->thb", x, weight.to(x.dtype)).contiguous()


def _head_linear_hip(launch, x, weight):
    """Steps of up to 16 rows: this package's kernel (the weights stream once, no copy of the result); more rows: the
    vendor library's batched product."""
    t, heads, a = x.shape
    b = weight.shape[1]
    if not (x.is_cuda and x.is_contiguous() and weight.is_contiguous() and weight.dtype == x.dtype and x.dtype in _DT
            and tuple(weight.shape) == (heads, b, a)):
        raise ValueError(f"head_linear: rows {tuple(x.shape)} {x.dtype} do not fit weights {tuple(weight.shape)} {weight.dtype}")
    if not 1 <= t <= 16 or t * a * 4 > 48 * 1024:
        return head_linear_plain(x, weight)
    y = torch.empty((t, heads, b), dtype=x.dtype, device=x.device)
    launch(x.data_ptr(), weight.data_ptr(), y.data_ptr(), t, heads, a, b, _DT[x.dtype])
    return y


def latent_prepare_plain(both, q_rank, q_weight, c_weight, eps, pages, write_page, write_off, page_size):
    """both [T, q_rank + R] (the two latents' projections side by side): each x * rsqrt(mean(x^2) + eps) * weight,
    float32 inside, one rounding. Returns the first [T, q_rank]; the second goes into `pages` [pages, 2 P R] at
    (write_page[t], write_off[t]) twice: as a key (row of [P, R]) and as a value (column of [R, P])."""
    t, rank = both.shape[0], both.shape[1] - q_rank

    def norm(x, w):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(both.dtype)
    cq, c = norm(both[:, :q_rank], q_weight), norm(both[:, q_rank:], c_weight)
    keys = pages[:, : page_size * rank].view(-1, page_size, rank)
    vals = pages[:, page_size * rank:].view(-1, rank, page_size)
    keys[write_page.long(), write_off.long()] = c
    vals[write_page.long(), :, write_off.long()] = c
    return cq.contiguous()


def _latent_prepare_hip(launch, both, q_rank, q_weight, c_weight, eps, pages, write_page, write_off, page_size):
    t, rank = both.shape[0], both.shape[1] - q_rank
    ok = both.is_cuda and both.is_contiguous() and both.dtype in _DT and rank > 0 and pages.dtype == both.dtype \
        and pages.is_contiguous() and pages.dim() == 2 and pages.shape[1] == 2 * page_size * rank \
        and all(w.dtype == both.dtype and w.is_contiguous() for w in (q_weight, c_weight)) \
        and q_weight.shape == (q_rank,) and c_weight.shape == (rank,) and write_page.shape[0] >= t \
        and write_off.shape[0] >= t
    if not ok:
        raise ValueError(f"latent_prepare: rows {tuple(both.shape)} {both.dtype}, pages {tuple(pages.shape)} do not fit "
                         f"latents of {q_rank} and {rank}, page {page_size}")
    cq = torch.empty((t, q_rank), dtype=both.dtype, device=both.device)
    launch(both.data_ptr(), t, q_rank, rank, q_weight.data_ptr(), c_weight.data_ptr(), float(eps), cq.data_ptr(),
           pages.data_ptr(), write_page.data_ptr(), write_off.data_ptr(), page_size, pages.shape[0], _DT[both.dtype])
    return cq


register_kernel(KernelOp("softmax_attention", softmax_attention_plain, "holon_softmax_attention",
                         [_P, _P, _P, _P, _I, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _F, _I, _I],
                         _softmax_attention_hip))
register_kernel(KernelOp("head_linear", head_linear_plain, "holon_head_linear_rows", [_P, _P, _P, _I, _I, _I, _I, _I],
                         _head_linear_hip))
register_kernel(KernelOp("latent_prepare", latent_prepare_plain, "holon_latent_prepare",
                         [_P, _I, _I, _I, _P, _P, _F, _P, _P, _P, _P, _I, _I, _I], _latent_prepare_hip))


def attend(k, q, held, view, step, kv_heads, vdim, sink, scale, window):
    """The attention of both mixers: on the matrix cores where keys and values have one width that those kernels
    serve (the pages' layout is then theirs), else the general kernel. q [T, H, D] -> [T, H V]."""
    t, heads, dim = q.shape
    if dim == vdim and k.attention_on_cores(dim, view.page_size, q.dtype):
        pages = held.pages.view(-1, 2, kv_heads, view.page_size * dim)
        return k.paged_attention(q, pages, view.table, step.rows, view.page_size, scale, window, sink=sink).view(t, heads * vdim)
    return k.softmax_attention(q, held.pages, view.table, step.rows, step.token_row, step.positions, kv_heads, vdim,
                               view.page_size, sink, scale, window)


def to_half_split(rows_per_head: int, heads: int, rot: int) -> torch.Tensor:
    """The order of a projection's output rows that turns the interleaved pairing of rotary dimensions, (2i, 2i + 1),
    into the half-split one, (i, i + rot/2), head by head; rows from `rot` on stay. Queries and keys permuted alike
    keep every score."""
    one = list(range(0, rot, 2)) + list(range(1, rot, 2)) + list(range(rot, rows_per_head))
    return torch.tensor([h * rows_per_head + r for h in range(heads) for r in one], dtype=torch.long)


@register_part("mixer", "attention")
class SoftmaxAttention(Part):
    """Grouped-query softmax attention: q/k/v projections (one merged product) with optional biases (`qkv_bias`),
    optional rotary positions (`position`: any registered position part with a `table`; one that says `interleaved`
    has its pairing turned into the kernels' by reordering the projections' rows once), `scale`, an optional window
    and an optional sink per head (`sink`), output projection. Keys are `dim` wide, values `vdim`."""

    graph_safe = True

    def __init__(self, build: Build, *, heads: int, kv_heads: int, dim: int, vdim: int, hidden: int, layer: int,
                 scale: float | None = None, window: int = 0, qkv_bias: bool = False, sink: bool = False,
                 position: PartRef | None = None, name: str = "") -> None:
        super().__init__(build)
        if heads % kv_heads:
            raise ValueError(f"attention: {heads} heads are not a multiple of {kv_heads} kv heads")
        self.heads, self.kv_heads, self.dim, self.vdim, self.hidden = heads, kv_heads, dim, vdim, hidden
        self.window = int(window)
        self.scale = float(scale) if scale is not None else dim ** -0.5
        self.state_name = f"{name}.kv" if name else "kv"
        self.attach("q", Linear(build, inp=hidden, out=heads * dim))
        self.attach("k", Linear(build, inp=hidden, out=kv_heads * dim))
        self.attach("v", Linear(build, inp=hidden, out=kv_heads * vdim))
        self.attach("o", Linear(build, inp=heads * vdim, out=hidden))
        self.qkv_bias = bool(qkv_bias)
        if self.qkv_bias:
            self.declare("q_bias", (heads * dim,), kind=FLOAT32, init="zero")
            self.declare("k_bias", (kv_heads * dim,), kind=FLOAT32, init="zero")
            self.declare("v_bias", (kv_heads * vdim,), kind=FLOAT32, init="zero")
        self.has_sink = bool(sink)
        if self.has_sink:
            self.declare("sink", (heads,), kind=FLOAT32, init="zero")
        self.position = None
        if position is not None:
            self.attach("position", build.make(position, head_dim=dim))
        self.qkv: Linear | None = None
        self.bias: torch.Tensor | None = None

    def state(self):
        return [PagedState(self.state_name, elems=self.kv_heads * (self.dim + self.vdim), window=self.window)]

    def finalize(self) -> None:
        if self.q.weight is not None and getattr(self.position, "interleaved", False):
            rot = self.position.rotary_dim
            for proj, heads, bias in ((self.q, self.heads, "q_bias"), (self.k, self.kv_heads, "k_bias")):
                order = to_half_split(self.dim, heads, rot).to(proj.weight.device)
                proj.weight = proj.weight.index_select(0, order).contiguous()
                if self.qkv_bias:
                    setattr(self, bias, getattr(self, bias).index_select(0, order).contiguous())
        if self.qkv_bias and self.q_bias is not None:
            self.bias = torch.cat((self.q_bias, self.k_bias, self.v_bias)).contiguous()
        self.qkv = Linear.merge(self.build, self.q, self.k, self.v)
        for name in ("q", "k", "v"):
            self.drop(name)
        self._children["qkv"] = self.qkv

    def extra_tensors(self):
        return [self.bias] if self.bias is not None else []

    def forward(self, x: torch.Tensor, step, site) -> torch.Tensor:
        k = self.kernels
        held = site.paged[self.state_name]
        view = step.paged[held.group]
        table = getattr(self.position, "table", None)
        q = k.head_prepare(self.qkv(x), self.heads, self.kv_heads, self.dim, self.vdim, None, None, 0.0, table,
                           step.positions, held.pages, view.write_page, view.write_off, view.page_size, bias=self.bias)
        out = attend(k, q, held, view, step, self.kv_heads, self.vdim, self.sink if self.has_sink else None, self.scale,
                     self.window)
        return self.o(out)

    __call__ = forward


@register_part("mixer", "latent_attention")
class LatentAttention(Part):
    """Attention whose queries, keys and values come through low-rank latents, without positions:

        c_q = norm(W_dq x),  q_h = W_uq,h c_q;     c = norm(W_dkv x),  k_h = W_uk,h c,  v_h = W_uv,h c

    Only c [kv_rank] is cached per token. The scores q_h . k_h equal (W_uk,h^T q_h) . c, and the weighted sum of the
    v_h equals W_uv,h applied to the weighted sum of the c: the mixer attends in the latent's space, with one shared
    key/value head of width kv_rank whose keys and values are both c, and applies W_uk,h to the queries and W_uv,h to
    the results, head by head. `norm` is the kind of the two latents' norms (their `eps` comes with it); `window` 0
    sees everything before."""

    graph_safe = True

    def __init__(self, build: Build, *, heads: int, dim: int, vdim: int, q_rank: int, kv_rank: int, norm: PartRef,
                 hidden: int, layer: int, scale: float | None = None, window: int = 0, name: str = "") -> None:
        super().__init__(build)
        self.heads, self.dim, self.vdim, self.q_rank, self.kv_rank = heads, dim, vdim, q_rank, kv_rank
        self.window = int(window)
        self.scale = float(scale) if scale is not None else dim ** -0.5
        self.state_name = f"{name}.latent" if name else "latent"
        self.attach("dq", Linear(build, inp=hidden, out=q_rank))
        self.attach("dq_norm", build.make(norm, dim=q_rank))
        self.attach("uq", Linear(build, inp=q_rank, out=heads * dim))
        self.attach("dkv", Linear(build, inp=hidden, out=kv_rank))
        self.attach("dkv_norm", build.make(norm, dim=kv_rank))
        self.declare("uk", (heads * dim, kv_rank))
        self.declare("uv", (heads * vdim, kv_rank))
        self.attach("o", Linear(build, inp=heads * vdim, out=hidden))
        self.down: Linear | None = None
        self.uk_t = self.uv_h = None
        self._fused: float | None = None          # the norms' eps, when they are RMS norms of one eps: one kernel then
                                                  # norms both latents and writes the cache

    def state(self):
        return [PagedState(self.state_name, elems=2 * self.kv_rank, window=self.window)]

    def finalize(self) -> None:
        self.down = Linear.merge(self.build, self.dq, self.dkv)
        self.drop("dq")
        self.drop("dkv")
        self._children["down"] = self.down
        specs = [n.fusion() for n in (self.dq_norm, self.dkv_norm)]
        if all(sp is not None and sp.get("norm") == "rmsnorm" and sp["weight"] is not None for sp in specs) \
                and specs[0]["eps"] == specs[1]["eps"]:
            self._fused = float(specs[0]["eps"])
        if self.uk is not None:
            # [H, kv_rank, dim]: what turns a head's query into the latent's space; [H, vdim, kv_rank]: a head's values
            self.uk_t = self.uk.view(self.heads, self.dim, self.kv_rank).transpose(1, 2).contiguous()
            self.uv_h = self.uv.view(self.heads, self.vdim, self.kv_rank)

    def extra_tensors(self):
        return [self.uk_t] if self.uk_t is not None else []

    def forward(self, x: torch.Tensor, step, site) -> torch.Tensor:
        k = self.kernels
        t = x.shape[0]
        held = site.paged[self.state_name]
        view = step.paged[held.group]
        both = self.down(x)
        if self._fused is not None:               # both norms and the cache write in one kernel
            cq = k.latent_prepare(both, self.q_rank, self.dq_norm.weight, self.dkv_norm.weight, self._fused, held.pages,
                                  view.write_page, view.write_off, view.page_size)
        else:
            cq = self.dq_norm(both[:, : self.q_rank].contiguous())
            c = self.dkv_norm(both[:, self.q_rank:].contiguous()).view(t, 1, self.kv_rank)
            k.kv_write(c, c, held.pages.view(-1, 2, 1, view.page_size * self.kv_rank), view.write_page, view.write_off,
                       view.page_size)
        q = k.head_linear(self.uq(cq).view(t, self.heads, self.dim), self.uk_t)
        mixed = attend(k, q, held, view, step, 1, self.kv_rank, None, self.scale, self.window)
        out = k.head_linear(mixed.view(t, self.heads, self.kv_rank), self.uv_h)
        return self.o(out.view(t, self.heads * self.vdim))

    __call__ = forward
