"""Mixers that carry a matrix per head from token to token instead of a cache that grows: the gated delta rule and a
decayed key-value memory with token shift (the time mixing of RWKV-6 in shape). The matrices are float32
`SlotState`s; every quantity that enters a recurrence other than a projection's result (unit vectors, step sizes,
decays) is float32. HIP forms of the operations: `csrc/recurrent.hip`.

Both scans have one thread per value column: column j of a head's matrix S [D, V] never meets another column, so a
thread holds its D values in registers for the whole portion and reads the keys and queries the block shares."""
from __future__ import annotations

import ctypes

import torch

from ..kernels.registry import KernelOp, register_kernel
from ..registry import register_part
from .base import FLOAT32, Build, Part, SlotState
from .convs import CausalConv
from .linear import Linear

_P, _I, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
_DT = {torch.float32: 0, torch.bfloat16: 1}
MAX_KEY_DIM = 256             # the scans keep a column of D values in registers


def _ptr(t):
    return None if t is None else t.data_ptr()


def _need(cond: bool, what: str) -> None:
    if not cond:
        raise ValueError(what)


def _rows(slots, starts, query_start, n_rows):
    return slots.tolist()[:n_rows], starts.tolist()[:n_rows], query_start.tolist()[: n_rows + 1]


# -- gated delta rule -------------------------------------------------------------------------------------------------
def delta_prepare_plain(qkv, ab, a_log, dt_bias, heads, kv_heads, dim, vdim):
    """qkv [T, 2 G D + H V] (filtered q, k, v side by side), ab [T, 2 H] (the decay's and the step size's
    projections). -> float32: q / sqrt(sum q^2 + 1e-6) * D^-0.5 and k / sqrt(sum k^2 + 1e-6) per head [T, G, D] each,
    beta = sigmoid(b) [T, H], g = exp(-exp(a_log) * softplus(a + dt_bias)) [T, H]."""
    t = qkv.shape[0]
    q = qkv[:, : kv_heads * dim].float().view(t, kv_heads, dim)
    k = qkv[:, kv_heads * dim: 2 * kv_heads * dim].float().view(t, kv_heads, dim)
    qn = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    kn = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    a, b = ab[:, :heads].float(), ab[:, heads:].float()
    beta = torch.sigmoid(b)
    g = torch.exp(-torch.exp(a_log.float()) * torch.nn.functional.softplus(a + dt_bias.float()))
    return qn.contiguous(), kn.contiguous(), beta.contiguous(), g.contiguous()


def _delta_prepare_hip(launch, qkv, ab, a_log, dt_bias, heads, kv_heads, dim, vdim):
    t = qkv.shape[0]
    _need(qkv.is_cuda and qkv.is_contiguous() and qkv.dtype in _DT and qkv.shape[1] == 2 * kv_heads * dim + heads * vdim
          and ab.is_contiguous() and ab.dtype == qkv.dtype and tuple(ab.shape) == (t, 2 * heads)
          and a_log.dtype == torch.float32 and dt_bias.dtype == torch.float32 and a_log.shape == (heads,)
          and dt_bias.shape == (heads,), "delta_prepare: shapes do not fit the head counts")
    f32 = dict(dtype=torch.float32, device=qkv.device)
    qn, kn = torch.empty((t, kv_heads, dim), **f32), torch.empty((t, kv_heads, dim), **f32)
    beta, g = torch.empty((t, heads), **f32), torch.empty((t, heads), **f32)
    launch(qkv.data_ptr(), ab.data_ptr(), a_log.data_ptr(), dt_bias.data_ptr(), qn.data_ptr(), kn.data_ptr(),
           beta.data_ptr(), g.data_ptr(), t, heads, kv_heads, dim, vdim, _DT[qkv.dtype])
    return qn, kn, beta, g


def delta_scan_plain(qn, kn, qkv, beta, g, state, slots, starts, query_start, n_rows, heads, vdim, pieces=None):
    """Per row and head, along the row's tokens: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.
    qn, kn [T, G, D] float32; v is the last H V columns of qkv; state [slots, H, D, V] float32, read unless the row
    starts at position 0 and written back. -> o [T, H, V] float32. `pieces` as for `memory_scan`."""
    t, kv_heads, dim = qn.shape
    v = qkv[:, qkv.shape[1] - heads * vdim:].float().view(t, heads, vdim)
    out = torch.empty((t, heads, vdim), dtype=torch.float32, device=qn.device)
    group = heads // kv_heads
    slot_of, start_of, qs = _rows(slots, starts, query_start, n_rows)
    for b in range(n_rows):
        S = state[slot_of[b]].clone() if start_of[b] > 0 else torch.zeros_like(state[slot_of[b]])
        for i in range(qs[b], qs[b + 1]):
            kk = kn[i].repeat_interleave(group, dim=0)                 # [H, D]
            qq = qn[i].repeat_interleave(group, dim=0)
            S = S * g[i][:, None, None]
            u = beta[i][:, None] * (v[i] - torch.einsum("hdv,hd->hv", S, kk))
            S = S + kk[:, :, None] * u[:, None, :]
            out[i] = torch.einsum("hdv,hd->hv", S, qq)
        state[slot_of[b]] = S
    return out


def _delta_scan_hip(launch, qn, kn, qkv, beta, g, state, slots, starts, query_start, n_rows, heads, vdim, pieces=None):
    t, kv_heads, dim = qn.shape
    _need(qn.is_cuda and qn.dtype == torch.float32 and kn.dtype == torch.float32 and qn.is_contiguous()
          and kn.is_contiguous() and qkv.is_contiguous() and qkv.dtype in _DT and beta.is_contiguous()
          and g.is_contiguous() and state.dtype == torch.float32 and state.is_contiguous()
          and tuple(state.shape[1:]) == (heads, dim, vdim) and heads % kv_heads == 0,
          "delta_scan: shapes do not fit the head counts")
    _need(dim <= MAX_KEY_DIM and vdim <= 1024, f"delta_scan: key size {dim} (at most {MAX_KEY_DIM}), value size {vdim} "
          "(at most 1024)")
    out = torch.empty((t, heads, vdim), dtype=torch.float32, device=qn.device)
    extra = (0, 0, None, None, None)
    if pieces is not None:
        tokens, most, base, total = pieces
        ab = torch.empty((total, heads, dim, vdim + dim), dtype=torch.float32, device=qn.device)
        sin = torch.empty((total, heads, dim, vdim), dtype=torch.float32, device=qn.device)
        extra = (tokens, most, base.data_ptr(), ab.data_ptr(), sin.data_ptr())
    launch(qn.data_ptr(), kn.data_ptr(), qkv.data_ptr(), qkv.shape[1], qkv.shape[1] - heads * vdim, beta.data_ptr(),
           g.data_ptr(), state.data_ptr(), out.data_ptr(), slots.data_ptr(), starts.data_ptr(), query_start.data_ptr(),
           n_rows, heads, kv_heads, dim, vdim, state.shape[0], _DT[qkv.dtype], *extra)
    return out


def gated_out_plain(o, gate, weight, per_head_weight, eps, out_dtype, act="silu", den=None):
    """o [T, H, V] float32 -> [T, H V]: each head's o divided by its root mean square (eps inside the root), times
    `weight` ([V], shared by the heads, or [H V] with `per_head_weight`), times act(gate [T, H V]); `act` is "silu"
    or "sigmoid". The gates may be columns of a wider tensor (rows further apart than H V). `den` [T, H] float32 or
    None: every head's o is divided by it first."""
    t, heads, vdim = o.shape
    if den is not None:
        o = o / den[..., None]
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
    y = y * (weight.float().view(heads, vdim) if per_head_weight else weight.float())
    gf = gate.float().reshape(t, heads, vdim)
    return (y * (gf if act == "silu" else 1.0) * torch.sigmoid(gf)).view(t, heads * vdim).to(out_dtype)


def _gated_out_hip(launch, o, gate, weight, per_head_weight, eps, out_dtype, act="silu", den=None):
    t, heads, vdim = o.shape
    _need(o.is_cuda and o.is_contiguous() and o.dtype == torch.float32 and gate.dtype in _DT and gate.dim() == 2
          and tuple(gate.shape) == (t, heads * vdim) and gate.stride(1) == 1 and (t <= 1 or gate.stride(0) >= heads * vdim)
          and weight.is_contiguous() and weight.dtype == gate.dtype
          and weight.numel() == (heads * vdim if per_head_weight else vdim) and out_dtype == gate.dtype
          and act in ("silu", "sigmoid") and (den is None or (den.dtype == torch.float32 and den.is_contiguous()
                                                  and tuple(den.shape) == (t, heads))), "gated_out: shapes do not fit")
    y = torch.empty((t, heads * vdim), dtype=out_dtype, device=o.device)
    launch(o.data_ptr(), gate.data_ptr(), weight.data_ptr(), y.data_ptr(), t, heads, vdim, int(per_head_weight),
           float(eps), _DT[out_dtype], gate.stride(0) if t > 1 else heads * vdim, int(act == "sigmoid"), _ptr(den))
    return y


# -- decayed key-value memory -------------------------------------------------------------------------------------------
def shift_mix_plain(x, mu, state, slots, starts, query_start, token_row, n_rows, in_order=False):
    """x [T, W]; mu [n, W]; state [S, W]: the last row each request has seen (zeros before its first). ->
    [n, T, W], mix_s = x + (x' - x) * mu_s with x' the row of the token before (float32 inside, one rounding); the
    state takes each request's last row. `in_order`: every row has one token and token t is row t."""
    prev = torch.empty_like(x)
    slot_of, start_of, qs = _rows(slots, starts, query_start, n_rows)
    for b in range(n_rows):
        lo, hi = qs[b], qs[b + 1]
        prev[lo] = state[slot_of[b]] if start_of[b] > 0 else 0
        prev[lo + 1: hi] = x[lo: hi - 1]
        state[slot_of[b]] = x[hi - 1]
    xf, pf = x.float(), prev.float()
    return (xf[None] + (pf - xf)[None] * mu.float()[:, None, :]).to(x.dtype)


def _shift_mix_hip(launch, x, mu, state, slots, starts, query_start, token_row, n_rows, in_order=False):
    t, w = x.shape
    _need(x.is_cuda and x.is_contiguous() and x.dtype in _DT and mu.is_contiguous() and mu.dtype == x.dtype
          and mu.shape[1] == w and state.is_contiguous() and state.dtype == x.dtype and state.shape[1] == w,
          "shift_mix: shapes do not fit")
    y = torch.empty((mu.shape[0], t, w), dtype=x.dtype, device=x.device)
    launch(x.data_ptr(), mu.data_ptr(), state.data_ptr(), y.data_ptr(), slots.data_ptr(), starts.data_ptr(),
           query_start.data_ptr(), token_row.data_ptr(), t, n_rows, w, mu.shape[0], state.shape[0], _DT[x.dtype],
           int(bool(in_order) and t == n_rows))
    return y


def decay_lora_plain(a, w2t, w0):
    """a [T, R] float32 (the decay's first projection), w2t [R, C] (the second one, transposed), w0 [C] float32 ->
    exp(-exp(tanh(a) w2t + w0)) [T, C] float32."""
    return torch.exp(-torch.exp(torch.tanh(a.float()) @ w2t.float() + w0.float()))


def _decay_lora_hip(launch, a, w2t, w0):
    t, r = a.shape
    c = w2t.shape[1]
    _need(a.is_cuda and a.is_contiguous() and a.dtype == torch.float32 and w2t.is_contiguous() and w2t.dtype in _DT
          and w2t.shape[0] == r and w0.dtype == torch.float32 and w0.shape == (c,) and r <= 1024,
          "decay_lora: shapes do not fit (rank at most 1024)")
    y = torch.empty((t, c), dtype=torch.float32, device=a.device)
    launch(a.data_ptr(), w2t.data_ptr(), w0.data_ptr(), y.data_ptr(), t, c, r, _DT[w2t.dtype])
    return y


def memory_scan_plain(r, k, v, w, u, state, slots, starts, query_start, n_rows, heads, pieces=None):
    """Per row and head along the row's tokens: o = (S + diag(u) k v^T)^T r, then S <- diag(w) S + k v^T.
    r, k, v [T, H D]; w [T, H D] float32 (decay per key channel); u [H, D] float32; state [slots, H, D, D] float32.
    -> o [T, H, D] float32. `pieces` (what `scan_pieces` answers, or None) lets a kernel run long rows in pieces side
    by side; the result is the same but for the order of the sums."""
    t = r.shape[0]
    dim = r.shape[1] // heads
    rf, kf, vf = (x.float().view(t, heads, dim) for x in (r, k, v))
    wf = w.view(t, heads, dim)
    out = torch.empty((t, heads, dim), dtype=torch.float32, device=r.device)
    slot_of, start_of, qs = _rows(slots, starts, query_start, n_rows)
    for b in range(n_rows):
        S = state[slot_of[b]].clone() if start_of[b] > 0 else torch.zeros_like(state[slot_of[b]])
        for i in range(qs[b], qs[b + 1]):
            kv = kf[i][:, :, None] * vf[i][:, None, :]
            out[i] = torch.einsum("hdv,hd->hv", S + u.float()[:, :, None] * kv, rf[i])
            S = wf[i][:, :, None] * S + kv
        state[slot_of[b]] = S
    return out


def scan_pieces(step, tokens: int = 128, least: int = 256):
    """For a step with a row of `least` tokens or more (never a step replayed from a graph: those rows have one token):
    (tokens a piece, the most pieces a row has, the number of each row's first piece among all [rows] int32 on the
    device, pieces in all), made once a step and piece length from the host's row lengths; else None. (The delta
    rule takes pieces of 256 tokens: the ordered walk between its two passes multiplies matrices, and is the shorter
    the fewer pieces there are.)"""
    if step.rows.max_chunk_query < least:
        return None
    cache = step.__dict__.setdefault("_scan_pieces", {})
    if tokens not in cache:
        n = -(-step.h_counts // tokens)
        base = torch.from_numpy((n.cumsum() - n).astype("int32")).to(step.slots.device, non_blocking=True)
        cache[tokens] = (tokens, int(n.max()), base, int(n.sum()))
    return cache[tokens]


def _memory_scan_hip(launch, r, k, v, w, u, state, slots, starts, query_start, n_rows, heads, pieces=None):
    t = r.shape[0]
    dim = r.shape[1] // heads
    _need(r.is_cuda and all(x.is_contiguous() and x.dtype == r.dtype and x.shape == r.shape for x in (r, k, v))
          and r.dtype in _DT and w.dtype == torch.float32 and w.is_contiguous() and w.shape == r.shape
          and u.dtype == torch.float32 and u.is_contiguous() and tuple(u.shape) == (heads, dim)
          and state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (heads, dim, dim),
          "memory_scan: shapes do not fit")
    _need(dim <= MAX_KEY_DIM, f"memory_scan: head size {dim} (at most {MAX_KEY_DIM})")
    out = torch.empty((t, heads, dim), dtype=torch.float32, device=r.device)
    extra = (0, 0, None, None, None)
    if pieces is not None:
        tokens, most, base, total = pieces
        sloc = torch.empty((total, heads, dim, dim), dtype=torch.float32, device=r.device)
        pw = torch.empty((total, heads, dim), dtype=torch.float32, device=r.device)
        extra = (tokens, most, base.data_ptr(), sloc.data_ptr(), pw.data_ptr())
    launch(r.data_ptr(), k.data_ptr(), v.data_ptr(), w.data_ptr(), u.data_ptr(), state.data_ptr(), out.data_ptr(),
           slots.data_ptr(), starts.data_ptr(), query_start.data_ptr(), n_rows, heads, dim, state.shape[0],
           _DT[r.dtype], *extra)
    return out


register_kernel(KernelOp("delta_prepare", delta_prepare_plain, "holon_delta_prepare",
                         [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I], _delta_prepare_hip))
register_kernel(KernelOp("delta_scan", delta_scan_plain, "holon_delta_scan",
                         [_P, _P, _P, _I, _I, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P],
                         _delta_scan_hip))
register_kernel(KernelOp("gated_out", gated_out_plain, "holon_gated_out",
                         [_P, _P, _P, _P, _I, _I, _I, _I, _F, _I, ctypes.c_int64, _I, _P], _gated_out_hip))
register_kernel(KernelOp("shift_mix", shift_mix_plain, "holon_shift_mix",
                         [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I], _shift_mix_hip))
register_kernel(KernelOp("decay_lora", decay_lora_plain, "holon_decay_lora", [_P, _P, _P, _P, _I, _I, _I, _I],
                         _decay_lora_hip))
register_kernel(KernelOp("memory_scan", memory_scan_plain, "holon_memory_scan",
                         [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P, _P, _P],
                         _memory_scan_hip))


# -- parts ------------------------------------------------------------------------------------------------------------
@register_part("mixer", "gated_delta")
class GatedDelta(Part):
    """Gated delta rule: q and k with `kv_heads` heads of `dim`, v with `heads` heads of `vdim`, each through a short
    causal filter (`taps`) and silu; q and k as unit vectors (q also times dim^-0.5); per head a step size
    sigmoid(b x) and a decay exp(-exp(A_log) softplus(a x + dt_bias)); read-out after the write; each head's
    read-out divided by its root mean square (`eps`), times `norm` [vdim], times silu(g x); output projection."""

    graph_safe = True

    def __init__(self, build: Build, *, heads: int, kv_heads: int, dim: int, vdim: int, taps: int, eps: float,
                 hidden: int, layer: int, name: str = "") -> None:
        super().__init__(build)
        if heads % kv_heads:
            raise ValueError(f"gated_delta: {heads} heads are not a multiple of {kv_heads} key heads")
        if dim > MAX_KEY_DIM:
            raise ValueError(f"gated_delta: key size {dim} is above {MAX_KEY_DIM}")
        self.heads, self.kv_heads, self.dim, self.vdim, self.eps = heads, kv_heads, dim, vdim, float(eps)
        self.prefix = f"{name}." if name else ""
        for nm, out in (("q", kv_heads * dim), ("k", kv_heads * dim), ("v", heads * vdim)):
            self.attach(nm, Linear(build, inp=hidden, out=out))
            self.attach(f"{nm}_conv", CausalConv(build, channels=out, taps=taps, silu=True))
        self.attach("a", Linear(build, inp=hidden, out=heads))
        self.attach("b", Linear(build, inp=hidden, out=heads))
        self.attach("g", Linear(build, inp=hidden, out=heads * vdim))
        self.attach("o", Linear(build, inp=heads * vdim, out=hidden))
        self.declare("A_log", (heads,), kind=FLOAT32, init="zero")
        self.declare("dt_bias", (heads,), kind=FLOAT32, init="zero")
        self.declare("norm", (vdim,), init="norm")
        self.taps = int(taps)
        self.qkv = self.ab = self.conv = None

    def state(self):
        channels = 2 * self.kv_heads * self.dim + self.heads * self.vdim
        return [SlotState(self.prefix + "conv", (self.taps - 1, channels)),
                SlotState(self.prefix + "S", (self.heads, self.dim, self.vdim), torch.float32)]

    def finalize(self) -> None:
        """One product for q, k, v and one filter over all their channels; one product for a and b."""
        self.conv = CausalConv(self.build, channels=self.q.out + self.k.out + self.v.out, taps=self.taps, silu=True,
                               name=self.prefix + "conv")
        self.conv.weight = torch.cat([self.q_conv.weight, self.k_conv.weight, self.v_conv.weight], dim=0).contiguous()
        self.qkv = Linear.merge(self.build, self.q, self.k, self.v)
        self.ab = Linear.merge(self.build, self.a, self.b)
        for nm in ("q", "k", "v", "a", "b", "q_conv", "k_conv", "v_conv"):
            self.drop(nm)
        self._children.update(qkv=self.qkv, ab=self.ab, conv=self.conv)

    def forward(self, x: torch.Tensor, step, site) -> torch.Tensor:
        k = self.kernels
        qkv = self.conv(self.qkv(x), step, site)
        qn, kn, beta, g = k.delta_prepare(qkv, self.ab(x), self.A_log, self.dt_bias, self.heads, self.kv_heads,
                                          self.dim, self.vdim)
        o = k.delta_scan(qn, kn, qkv, beta, g, site.slot_state[self.prefix + "S"], step.slots, step.starts,
                         step.query_start, step.n_rows, self.heads, self.vdim, scan_pieces(step, 256, 512))
        return self.o(k.gated_out(o, self.g(x), self.norm, False, self.eps, self.build.dtype))

    __call__ = forward


@register_part("mixer", "decay_memory")
class DecayMemory(Part):
    """Token shift and a decayed key-value memory: each of r, k, v, g, w reads x + (x' - x) mu_s with x' the token
    before; per head and key channel a decay exp(-exp(w2 tanh(w1 mix_w) + w0)) (the rank of w1, w2 is `rank`, or the
    checkpoint's when None); the current token's own k v^T enters its read-out through the bonus `u` only; each
    head's read-out divided by its root mean square (`eps`), times `norm` [heads dim], times silu(g mix_g);
    output projection."""

    graph_safe = True
    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, build: Build, *, heads: int, dim: int, eps: float, hidden: int, layer: int,
                 rank: int | None = None, name: str = "") -> None:
        super().__init__(build)
        if dim > MAX_KEY_DIM:
            raise ValueError(f"decay_memory: head size {dim} is above {MAX_KEY_DIM}")
        self.heads, self.dim, self.eps, self.hidden = heads, dim, float(eps), hidden
        self.prefix = f"{name}." if name else ""
        for s in self.MIXES:
            self.declare(f"mu_{s}", (hidden,), init="unit")
        for nm in ("r", "k", "v", "g"):
            self.attach(nm, Linear(build, inp=hidden, out=heads * dim))
        self.attach("o", Linear(build, inp=heads * dim, out=hidden))
        self.declare("w1", (-1 if rank is None else rank, hidden))
        self.declare("w2", (heads * dim, -1 if rank is None else rank), init="tap")
        self.declare("w0", (heads * dim,), kind=FLOAT32, init="zero")
        self.declare("u", (heads, dim), kind=FLOAT32, init="zero")
        self.declare("norm", (heads * dim,), init="norm")
        self.mu = self.w2t = None

    def state(self):
        return [SlotState(self.prefix + "shift", (self.hidden,)),
                SlotState(self.prefix + "S", (self.heads, self.dim, self.dim), torch.float32)]

    def finalize(self) -> None:
        if self.w1 is not None and self.w1.shape[0] != self.w2.shape[1]:
            raise ValueError(f"decay_memory: the decay's two projections have ranks {self.w1.shape[0]} and "
                             f"{self.w2.shape[1]}")
        if self.mu_r is not None:
            self.mu = torch.stack([getattr(self, f"mu_{s}") for s in self.MIXES]).contiguous()
            self.w2t = self.w2.t().contiguous()       # [rank, channels]: what the decay's kernel streams

    def extra_tensors(self):
        return [self.mu, self.w2t] if self.mu is not None else []

    def forward(self, x: torch.Tensor, step, site) -> torch.Tensor:
        k = self.kernels
        rows = (step.slots, step.starts, step.query_start)
        mixes = k.shift_mix(x, self.mu, site.slot_state[self.prefix + "shift"], *rows, step.token_row, step.n_rows,
                            step.rows.in_order)
        r, kk, v, gate = (getattr(self, nm)(mixes[i]) for i, nm in enumerate(("r", "k", "v", "g")))
        lora = k.linear(mixes[4], self.w1, torch.float32)
        decay = k.decay_lora(lora, self.w2t, self.w0)
        o = k.memory_scan(r, kk, v, decay, self.u, site.slot_state[self.prefix + "S"], *rows, step.n_rows, self.heads,
                          scan_pieces(step))
        return self.o(k.gated_out(o, gate, self.norm, True, self.eps, self.build.dtype))

    __call__ = forward
