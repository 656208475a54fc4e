"""Relanex, plainly: one function per mechanism, written from the design's equations, token by token where the design
is recurrent, with no cache, no batching and nothing shared with the engine. Everything runs in the dtype of the
tensors it is given (the tests pass float64).

    x0 = dyt(embed[token]);   a layer: x += m dyt(mixer(dyt(x)));  x += m dyt(ff(dyt(x)));   logits = head dyt(x)

A range of layers may run several times in a row with the same weights; before every pass after the first, x0 is
added to x."""
from __future__ import annotations

import math

import torch


def dyt(x, p, name):
    """tanh(alpha x) w + b: a norm without statistics."""
    return torch.tanh(p[name + ".alpha"] * x) * p[name] + p[name + ".b"]


def rms_div(x, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def yarn_frequencies(rot: dict, dtype=torch.float64):
    """(frequencies of the dims/2 pairs, the factor cos and sin are multiplied by)."""
    dims, base = rot["dims"], float(rot["base"])
    i = torch.arange(dims // 2, dtype=dtype)
    f = base ** (-2.0 * i / dims)
    s = rot.get("scaling")
    if not s:
        return f, 1.0
    factor, original = float(s["factor"]), float(s["original"])

    def dim_of(turns):
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(dim_of(float(s["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(s["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_interleaved(x, positions, rot: dict):
    """x [T, heads, dim]: dimensions (2i, 2i+1) of the first rot.dims turn by position * frequency_i."""
    dims = rot["dims"]
    f, gain = yarn_frequencies(rot, x.dtype)
    ang = positions.to(x.dtype)[:, None] * f[None, :]
    cos, sin = (ang.cos() * gain)[:, None, :], (ang.sin() * gain)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def attention(h, p, pre, m, eps):
    """Grouped-query softmax attention with biases on q, k, v, rotary positions and a sink in the denominator."""
    t = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ p[pre + "q"].T + p[pre + "q.b"]).view(t, H, D)
    k = (h @ p[pre + "k"].T + p[pre + "k.b"]).view(t, G, D)
    v = (h @ p[pre + "v"].T + p[pre + "v.b"]).view(t, G, V)
    if m.get("rot"):
        pos = torch.arange(t)
        q, k = rotate_interleaved(q, pos, m["rot"]), rotate_interleaved(k, pos, m["rot"])
    out = torch.zeros(t, H, V, dtype=h.dtype)
    for i in range(t):
        for hh in range(H):
            g = hh // (H // G)
            s = (k[: i + 1, g] @ q[i, hh]) * m["scale"]
            top = torch.maximum(s.max(), p[pre + "sink"][hh])
            w = torch.exp(s - top)
            out[i, hh] = (w[:, None] * v[: i + 1, g]).sum(0) / (w.sum() + torch.exp(p[pre + "sink"][hh] - top))
    return out.reshape(t, H * V) @ p[pre + "o"].T


def latent_attention(h, p, pre, m, eps):
    """Queries, keys and values through low-rank latents; a sliding window; no positions."""
    t = h.shape[0]
    H, D, V, W = m["heads"], m["dim"], m["vdim"], m["mask"]["size"]
    cq = rms_div(h @ p[pre + "dq"].T, eps) * p[pre + "dq.norm"]
    q = (cq @ p[pre + "uq"].T).view(t, H, D)
    c = rms_div(h @ p[pre + "dkv"].T, eps) * p[pre + "dkv.norm"]
    k = (c @ p[pre + "uk"].T).view(t, H, D)
    v = (c @ p[pre + "uv"].T).view(t, H, V)
    out = torch.zeros(t, H, V, dtype=h.dtype)
    for i in range(t):
        lo = max(0, i - W + 1)
        for hh in range(H):
            s = (k[lo: i + 1, hh] @ q[i, hh]) * m["scale"]
            w = torch.softmax(s, dim=0)
            out[i, hh] = (w[:, None] * v[lo: i + 1, hh]).sum(0)
    return out.reshape(t, H * V) @ p[pre + "o"].T


def mlstm(h, p, pre, m, eps):
    """A matrix memory per head with exponential input gates kept in range by a running maximum."""
    t = h.shape[0]
    H, D, V, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = (h @ p[pre + "q"].T).view(t, H, D) * D ** -0.5
    k = (h @ p[pre + "k"].T).view(t, H, D)
    v = (h @ p[pre + "v"].T).view(t, H, V)
    gi = cap * torch.tanh((h @ p[pre + "i"].T + p[pre + "i.b"]) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ p[pre + "f"].T + p[pre + "f.b"]) / cap))
    S = torch.zeros(H, D, V, dtype=h.dtype)
    n = torch.zeros(H, D, dtype=h.dtype)
    top = torch.zeros(H, dtype=h.dtype)
    out = torch.zeros(t, H, V, dtype=h.dtype)
    for i in range(t):
        new = torch.maximum(gf[i] + top, gi[i])
        keep, take = torch.exp(gf[i] + top - new), torch.exp(gi[i] - new)
        S = keep[:, None, None] * S + take[:, None, None] * k[i][:, :, None] * v[i][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[i]
        top = new
        num = torch.einsum("hdv,hd->hv", S, q[i])
        den = torch.maximum((n * q[i]).sum(-1).abs(), torch.exp(-top)) + 1e-6
        out[i] = num / den[:, None]
    y = rms_div(out, eps).reshape(t, H * V) * p[pre + "norm"]
    y = y * torch.sigmoid(h @ p[pre + "g"].T)
    return y @ p[pre + "o"].T


def dense_ff(h, p, pre):
    g = h @ p[pre + "gate"].T
    return (g * torch.sigmoid(g) * (h @ p[pre + "up"].T)) @ p[pre + "down"].T


MIXERS = {"attention": attention, "latent_attention": latent_attention, "mlstm": mlstm}


def run_order(config: dict) -> list[tuple[int, bool]]:
    """(layer, whether the embedding's output is added in front of it) for every layer run."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(start)]
    for turn in range(times):
        order += [(i, turn > 0 and i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, n)]


def forward(config: dict, tensors: dict, ids: list[int], dtype=torch.float64):
    """-> (logits [T, vocab], the stream after every layer run [runs, T, width])."""
    p = {k: v.to(dtype) for k, v in tensors.items()}
    eps, m = float(config["norm"]["eps"]), float(config["residual_mult"])
    x0 = dyt(p["embed"][torch.tensor(ids)], p, "embed.norm")
    x = x0.clone()
    after = []
    for i, again in run_order(config):
        layer, pre = config["layers"][i], f"l{i}."
        if again:
            x = x + x0
        y = MIXERS[layer["type"]](dyt(x, p, pre + "norm1"), p, pre + "mix.", layer["mixer"], eps)
        x = x + m * dyt(y, p, pre + "norm1b")
        if layer.get("mlp"):
            x = x + m * dyt(dense_ff(dyt(x, p, pre + "norm2"), p, pre + "mlp."), p, pre + "norm2b")
        after.append(x)
    return dyt(x, p, "final.norm") @ p["head"].T, torch.stack(after)
