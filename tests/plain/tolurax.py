"""The plain Tolurax model: one slow function per mechanism, written from the design's equations, token by token
where the design is a recurrence. It keeps no cache: a sequence is always computed whole, so it cannot share a fault of
the engine's state handling. It shares no code with `holon_amd`: it reads config.json as a dict and the checkpoint's
tensors by name.

Notation: x [T, W] the residual stream of one sequence, h the normed input of a mixer, t a position (from 0).
"""
from __future__ import annotations

import math

import torch


# -- small pieces ---------------------------------------------------------------------------------------------------
def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w with the biased variance; no bias term."""
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def rms_div(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z / (1 + torch.exp(-z))


def sigmoid(z):
    return 1 / (1 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def causal_conv(x, w):
    """x [T, C], w [C, taps]: y_t = sum_j w[:, j] x_(t - taps + 1 + j); what lies before the sequence is zero. The
    last column weighs the current token."""
    T, taps = x.shape[0], w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    return y


def rotary_frequencies(dims, base, scaling):
    """f_i = base^(-2i/dims), i < dims/2, then rescaled by wavelength bands when `scaling` is given: short waves
    (below original/high) stay, long ones (above original/low) are divided by `factor`, the band between is blended."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, orig = scaling["factor"], scaling["low"], scaling["high"], scaling["original"]
            wave = 2 * math.pi / f
            if wave < orig / high:
                pass
            elif wave > orig / low:
                f = f / factor
            else:
                s = (orig / wave - low) / (high - low)
                f = (1 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate(x, positions, dims, base, scaling):
    """x [T, heads, D]: dimension i < dims/2 pairs with i + dims/2; dimensions from `dims` on pass through."""
    freqs = torch.tensor(rotary_frequencies(dims, base, scaling), dtype=torch.float32)
    ang = positions.to(torch.float32)[:, None] * freqs[None, :]            # 32-bit angles, as the design asks
    cos, sin = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    half = dims // 2
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat((a * cos - b * sin, b * cos + a * sin, x[..., dims:]), dim=-1)


# -- mixers ---------------------------------------------------------------------------------------------------------
def windowed_sigmoid_attention(h, p, m, eps, get):
    """The left half of a parallel mixer. Weights of visible keys are sigmoid(score + bias of the head), not
    normalised over keys; query t sees keys t - size + 1 .. t."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ get(p + "q").T).view(T, H, D)
    k = (h @ get(p + "k").T).view(T, G, D)
    v = (h @ get(p + "v").T).view(T, G, V)
    q = rms_div(q, eps) * get(p + "q.norm")
    k = rms_div(k, eps) * get(p + "k.norm")
    pos = torch.arange(T)
    rot = m.get("rot")
    if rot:
        q = rotate(q, pos, rot["dims"], rot["base"], rot.get("scaling"))
        k = rotate(k, pos, rot["dims"], rot["base"], rot.get("scaling"))
    size = m["mask"]["size"]
    bias = get(p + "pb")
    out = torch.zeros(T, H, V, dtype=h.dtype)
    k, v = k.repeat_interleave(H // G, dim=1), v.repeat_interleave(H // G, dim=1)     # head hd reads kv head hd // (H/G)
    for t in range(T):
        first = max(0, t - size + 1)
        score = torch.einsum("hd,shd->sh", q[t], k[first: t + 1]) * m["scale"]     # [visible keys, H]
        out[t] = torch.einsum("sh,shv->hv", sigmoid(score + bias), v[first: t + 1])
    gate = sigmoid(h @ get(p + "g").T)
    return (out.reshape(T, H * V) * gate) @ get(p + "o").T


def decayed_outer_memory(h, p, m, eps, get):
    """The right half of a parallel mixer: per head a matrix S [D, D] that decays per key channel and takes k v^T
    every token; the current token's own k v^T enters the read-out through the bonus u only."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    prev = torch.cat((torch.zeros_like(h[:1]), h[:-1]), dim=0)

    def mixed(name):
        return h + (prev - h) * get(p + "mu." + name)
    r = (mixed("r") @ get(p + "r").T).view(T, H, D)
    k = (mixed("k") @ get(p + "k").T).view(T, H, D)
    v = (mixed("v") @ get(p + "v").T).view(T, H, D)
    gate = silu(mixed("g") @ get(p + "g").T)
    decay = torch.exp(-torch.exp(torch.tanh(mixed("w") @ get(p + "w1").T) @ get(p + "w2").T + get(p + "w0"))).view(T, H, D)
    u = get(p + "u")
    S = torch.zeros(H, D, D, dtype=h.dtype)
    out = torch.zeros(T, H, D, dtype=h.dtype)
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]                           # [H, D, D]: k v^T per head
        out[t] = torch.einsum("hdv,hd->hv", S + u[:, :, None] * kv, r[t])
        S = decay[t][:, :, None] * S + kv
    out = rms_div(out, eps).reshape(T, H * D) * get(p + "norm") * gate
    return out @ get(p + "o").T


def gated_delta(h, p, m, eps, get):
    """The delta mixer: per head a matrix S [D, V]; every token it decays by one number, is corrected towards
    storing v under key k (step size beta), and is read with q after the write."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ get(p + "q").T, get(p + "q.conv"))).view(T, G, D)
    k = silu(causal_conv(h @ get(p + "k").T, get(p + "k.conv"))).view(T, G, D)
    v = silu(causal_conv(h @ get(p + "v").T, get(p + "v.conv"))).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = sigmoid(h @ get(p + "b").T)
    g = torch.exp(-torch.exp(get(p + "A_log")) * softplus(h @ get(p + "a").T + get(p + "dt_bias")))
    S = torch.zeros(H, D, V, dtype=h.dtype)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)     # head hd reads q/k head hd // (H/G)
    for t in range(T):
        S = g[t][:, None, None] * S
        u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    out = rms_div(out, eps) * get(p + "norm")
    return (out.reshape(T, H * V) * silu(h @ get(p + "g").T)) @ get(p + "o").T


def gated_ffn(h, p, get):
    return (silu(h @ get(p + "gate").T) * (h @ get(p + "up").T)) @ get(p + "down").T


# -- the model ------------------------------------------------------------------------------------------------------
def run_order(config):
    """Layer numbers in the order they run; the layers of the loop's range `times` times in a row. With each entry:
    whether a pass of the loop starts there."""
    n, loop = len(config["layers"]), config.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    inside = list(range(loop["start"], loop["stop"]))
    order = [(i, False) for i in range(loop["start"])]
    for _ in range(loop["times"]):
        order += [(i, i == loop["start"]) for i in inside]
    return order + [(i, False) for i in range(loop["stop"], n)]


def forward(config, tensors, tokens, dtype=torch.float64):
    """-> (logits [T, vocab], the residual stream after every layer run [runs, T, W])."""
    def get(name):
        return tensors[name].to(dtype)
    eps = config["norm"]["eps"]
    x = get("embed")[torch.tensor(tokens)]
    x0 = x
    after = []
    for i, pass_start in run_order(config):
        layer, p = config["layers"][i], f"l{i}."
        if pass_start:
            x = torch.cat((x, x0), dim=-1) @ get("loop.in").T
        h = layer_norm(x, get(p + "norm1"), eps)
        if config.get("canon"):
            h = h + causal_conv(h, get(p + "canon1"))
        m = layer["mixer"]
        if layer["type"] == "delta":
            y = gated_delta(h, p + "mix.", m, eps, get)
        elif layer["type"] == "parallel":
            y = m["left_scale"] * windowed_sigmoid_attention(h, p + "mix.left.", m["left"], eps, get) \
                + m["right_scale"] * decayed_outer_memory(h, p + "mix.right.", m["right"], eps, get)
        else:
            raise ValueError(layer["type"])
        x = x + y
        if layer.get("mlp"):
            x = x + gated_ffn(layer_norm(x, get(p + "norm2"), eps), p + "mlp.", get)
        after.append(x)
    logits = layer_norm(x, get("final.norm"), eps) @ get("head").T
    cap = config.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    return logits, torch.stack(after)
