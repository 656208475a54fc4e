"""The matrix memory of xLSTM (mLSTM) as a mixer. Per head a matrix S [D, V], a vector n [D] and a running maximum
m, all float32 and part of the request's slot (n is kept as one more column of S: the column of a value that is
always 1); along a row's tokens, with log gates i and f:

    m' = max(f + m, i);   S' = exp(f + m - m') S + exp(i - m') k v^T;   n' likewise with k alone
    o = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)

S and n begin as zeros, and the running maximum begins at 0 as well, so a sequence's first token is already
compared with 0. The gates are capped, i = cap tanh(a_i / cap) and
f = logsigmoid(cap tanh(a_f / cap)), with a = W x + b; q is scaled by D^-0.5. Each head's o is divided by its root
mean square, multiplied by `norm` (a weight over all heads' values) and by sigmoid(W_g x), and projected out. One
product yields q, k, v, the output gate and both gates' pre-activations; gates, decays and the recurrence are float32.
HIP form: `csrc/mlstm.hip`."""
from __future__ import annotations

import ctypes

import torch

from ..kernels.registry import KernelOp, register_kernel
from ..registry import register_part
from .base import FLOAT32, Build, Part, SlotState
from .linear import Linear
from .recurrent import MAX_KEY_DIM, _rows, scan_pieces

_P, _I, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
_DT = {torch.float32: 0, torch.bfloat16: 1}


def state_copies(vdim: int) -> int:
    """Copies of m a head keeps: one for every 8 columns of S (the values' and n's)."""
    return -(-(vdim + 1) // 8)


def mlstm_scan_plain(proj, q_off, k_off, v_off, gate_off, gate_bias, cap, S, top, slots, starts, query_start,
                     n_rows, heads, dim, vdim, pieces=None):
    """proj [T, width]: q [H D] from column q_off, k [H D] from k_off, v [H V] from v_off, the gates' pre-activations
    [2 H] (input gates, then forget gates) from gate_off; gate_bias [2 H] float32. State per slot: S [H, D, V + 1]
    (the last column is n) and top [H, C], float32, read unless the row starts at position 0, written back;
    C = ceil((V + 1) / 8) equal copies (a kernel's blocks, one for every 8 columns, each keep their own).
    -> (numerators S^T q [T, H, V], denominators max(|n . q|, exp(-m)) + 1e-6 [T, H]), float32: o is their quotient.
    `pieces` (what `scan_pieces` answers, or None) lets a kernel run long rows in pieces side by side; the result is
    the same but for the order of the sums."""
    t = proj.shape[0]
    pf = proj.float()
    q = pf[:, q_off: q_off + heads * dim].view(t, heads, dim) * dim ** -0.5
    k = pf[:, k_off: k_off + heads * dim].view(t, heads, dim)
    v = pf[:, v_off: v_off + heads * vdim].view(t, heads, vdim)
    a = pf[:, gate_off: gate_off + 2 * heads] + gate_bias.float()
    gi = cap * torch.tanh(a[:, :heads] / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh(a[:, heads:] / cap))
    out = torch.empty((t, heads, vdim), dtype=torch.float32, device=proj.device)
    under = torch.empty((t, heads), dtype=torch.float32, device=proj.device)
    slot_of, start_of, qs = _rows(slots, starts, query_start, n_rows)
    for b in range(n_rows):
        s = slot_of[b]
        if start_of[b] > 0:
            Sb, nb, mb = S[s][..., :vdim].clone(), S[s][..., vdim].clone(), top[s][:, 0].clone()
        else:
            Sb, nb, mb = torch.zeros_like(S[s][..., :vdim]), torch.zeros_like(S[s][..., vdim]), torch.zeros_like(top[s][:, 0])
        for i in range(qs[b], qs[b + 1]):
            new = torch.maximum(gf[i] + mb, gi[i])
            keep, take = torch.exp(gf[i] + mb - new), torch.exp(gi[i] - new)
            Sb = keep[:, None, None] * Sb + take[:, None, None] * k[i][:, :, None] * v[i][:, None, :]
            nb = keep[:, None] * nb + take[:, None] * k[i]
            mb = new
            under[i] = torch.maximum((nb * q[i]).sum(-1).abs(), torch.exp(-mb)) + 1e-6
            out[i] = torch.einsum("hdv,hd->hv", Sb, q[i])
        S[s][..., :vdim], S[s][..., vdim], top[s] = Sb, nb, mb[:, None]
    return out, under


def _mlstm_scan_hip(launch, proj, q_off, k_off, v_off, gate_off, gate_bias, cap, S, top, slots, starts,
                    query_start, n_rows, heads, dim, vdim, pieces=None):
    t, width = proj.shape
    ok = proj.is_cuda and proj.is_contiguous() and proj.dtype in _DT and gate_bias.dtype == torch.float32 \
        and gate_bias.is_contiguous() and gate_bias.shape == (2 * heads,) \
        and all(x.dtype == torch.float32 and x.is_contiguous() for x in (S, top)) \
        and tuple(S.shape[1:]) == (heads, dim, vdim + 1) \
        and tuple(top.shape[1:]) == (heads, state_copies(vdim)) and S.shape[0] == top.shape[0] \
        and all(0 <= off and off + size <= width for off, size in
                ((q_off, heads * dim), (k_off, heads * dim), (v_off, heads * vdim), (gate_off, 2 * heads))) \
        and dim <= MAX_KEY_DIM and cap > 0
    if not ok:
        raise ValueError(f"mlstm_scan: rows {tuple(proj.shape)}, state {tuple(S.shape)} do not fit {heads} heads of "
                         f"{dim}/{vdim} (keys of at most {MAX_KEY_DIM})")
    f32 = dict(dtype=torch.float32, device=proj.device)
    out, under = torch.empty((t, heads, vdim), **f32), torch.empty((t, heads), **f32)
    extra = (0, 0, None, None, None, None)
    if pieces is not None:
        tokens, most, base, total = pieces
        work = (torch.empty((t, heads, 3), **f32), torch.empty((total, heads, dim, vdim + 1), **f32),
                torch.empty((total, heads), **f32))
        extra = (tokens, most, base.data_ptr(), *(w.data_ptr() for w in work))
    launch(proj.data_ptr(), width, q_off, k_off, v_off, gate_off, gate_bias.data_ptr(), float(cap), S.data_ptr(),
           top.data_ptr(), out.data_ptr(), under.data_ptr(), slots.data_ptr(), starts.data_ptr(), query_start.data_ptr(),
           n_rows, heads, dim, vdim, S.shape[0], _DT[proj.dtype], t, *extra)
    return out, under


register_kernel(KernelOp("mlstm_scan", mlstm_scan_plain, "holon_mlstm_scan",
                         [_P, _I, _I, _I, _I, _I, _P, _F, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P,
                          _P, _P],
                         _mlstm_scan_hip))


@register_part("mixer", "mlstm")
class MLSTM(Part):
    """See the module's text. `heads` heads with keys of `dim` and values of `vdim`; `gate_cap` caps both gates'
    pre-activations; `eps` is that of the per-head division by the root mean square."""

    graph_safe = True

    def __init__(self, build: Build, *, heads: int, dim: int, vdim: int, gate_cap: float, eps: float, hidden: int,
                 layer: int, name: str = "") -> None:
        super().__init__(build)
        if dim > MAX_KEY_DIM:
            raise ValueError(f"mlstm: key size {dim} is above {MAX_KEY_DIM}")
        if not gate_cap > 0:
            raise ValueError(f"mlstm: the gates' cap must be positive, got {gate_cap}")
        self.heads, self.dim, self.vdim, self.cap, self.eps = heads, dim, vdim, float(gate_cap), float(eps)
        self.prefix = f"{name}." if name else ""
        for nm, out in (("q", heads * dim), ("k", heads * dim), ("v", heads * vdim), ("g", heads * vdim), ("i", heads),
                        ("f", heads)):
            self.attach(nm, Linear(build, inp=hidden, out=out))
        self.attach("o", Linear(build, inp=heads * vdim, out=hidden))
        self.declare("i_bias", (heads,), kind=FLOAT32, init="zero")
        self.declare("f_bias", (heads,), kind=FLOAT32, init="zero")
        self.declare("norm", (heads * vdim,), init="norm")
        self.all: Linear | None = None
        self.gate_bias: torch.Tensor | None = None
        hd, hv = heads * dim, heads * vdim
        self.offsets = {"q": 0, "k": hd, "v": 2 * hd, "g": 2 * hd + hv, "gates": 2 * hd + 2 * hv}

    def state(self):
        return [SlotState(self.prefix + "S", (self.heads, self.dim, self.vdim + 1), torch.float32),
                SlotState(self.prefix + "top", (self.heads, state_copies(self.vdim)), torch.float32)]

    def finalize(self) -> None:
        """One product for q, k, v, the output gate and the two gates' pre-activations (rows padded with zeros to a
        multiple of 16, which the few-row products ask for)."""
        parts = [getattr(self, nm) for nm in ("q", "k", "v", "g", "i", "f")]
        rows = sum(p.out for p in parts)
        pad = -rows % 16
        merged = Linear(self.build, inp=parts[0].inp, out=rows + pad)
        weights = [p.weight for p in parts]
        if pad:
            weights.append(torch.zeros((pad, parts[0].inp), dtype=weights[0].dtype, device=weights[0].device))
        merged.weight = torch.cat(weights, dim=0).contiguous()
        for p in parts:
            p.weight = p.tiled = None
        merged.finalize()
        for nm in ("q", "k", "v", "g", "i", "f"):
            self.drop(nm)
        self.all = merged
        self._children["all"] = merged
        self.gate_bias = torch.cat((self.i_bias, self.f_bias)).contiguous()

    def extra_tensors(self):
        return [self.gate_bias] if self.gate_bias is not None else []

    def forward(self, x: torch.Tensor, step, site) -> torch.Tensor:
        k = self.kernels
        at, hv = self.offsets, self.heads * self.vdim
        proj = self.all(x)
        st = site.slot_state
        over, under = k.mlstm_scan(proj, at["q"], at["k"], at["v"], at["gates"], self.gate_bias, self.cap,
                                   st[self.prefix + "S"], st[self.prefix + "top"], step.slots, step.starts,
                                   step.query_start, step.n_rows, self.heads, self.dim, self.vdim, scan_pieces(step))
        y = k.gated_out(over, proj[:, at["g"]: at["g"] + hv], self.norm, True, self.eps, self.build.dtype, act="sigmoid",
                        den=under)
        return self.o(y)

    __call__ = forward
