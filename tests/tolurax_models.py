"""Small Tolurax configurations and checkpoints for the tests, and the plain model behind one interface.

The tensors are drawn here, by checkpoint name, from laws that make faults visible: projections keep activations of
order one, filters and token-shift weights are far from zero, decays range from a few tokens to hundreds, and `sharp`
raises the q/k norm gains and lowers the head biases so that few keys carry most of the attention's weight."""
from __future__ import annotations

import copy
import functools
import json
import pathlib

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from tests.plain import tolurax as plain


def left(heads, kv_heads, dim, vdim, size, scale, rot=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size}, "scale": scale,
            **({"rot": rot} if rot is not None else {})}


def parallel(left_cfg, right_heads, right_dim, left_scale=0.8, right_scale=1.3, ff=None):
    return {"type": "parallel", "mlp": {"kind": "dense", "ff": ff} if ff else None,
            "mixer": {"left": left_cfg, "right": {"heads": right_heads, "dim": right_dim}, "left_scale": left_scale,
                      "right_scale": right_scale}}


def delta(heads, kv_heads, dim, vdim, conv, ff=None):
    return {"type": "delta", "mlp": {"kind": "dense", "ff": ff} if ff else None,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


SCALED = {"dims": 8, "base": 100.0, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}}

# X: a delta layer and a parallel layer, the first one looped three times; window 7 below the page sizes used.
CONFIG_X = {"architecture": "Tolurax", "width": 64, "vocab": 160, "norm": {"eps": 1e-5}, "canon": {"taps": 2},
            "logit_softcap": 5.0, "loop": {"start": 0, "stop": 1, "times": 3},
            "layers": [delta(4, 2, 16, 24, 3, ff=96), parallel(left(4, 2, 16, 8, 7, 0.3, SCALED), 2, 24)]}
# Y: no loop, no cap, four taps; windows of 33 (a page of 16 plus one beyond two pages) and 16 (exactly a page).
CONFIG_Y = {"architecture": "Tolurax", "width": 96, "vocab": 200, "norm": {"eps": 1e-6}, "canon": {"taps": 4},
            "layers": [parallel(left(3, 3, 32, 32, 33, 0.18, {"dims": 32, "base": 10000.0}), 3, 32, ff=128),
                       parallel(left(6, 2, 16, 24, 16, 0.25, {"dims": 4, "base": 50.0}), 2, 40, 1.0, 0.4),
                       delta(2, 2, 32, 16, 2, ff=64)]}
# Z: sizes that are 1 or equal: one head everywhere, a window of one token, one tap, a loop that runs once over the
# whole model, no rotation, no input filter.
CONFIG_Z = {"architecture": "Tolurax", "width": 32, "vocab": 50, "norm": {"eps": 1e-6},
            "loop": {"start": 0, "stop": 2, "times": 1},
            "layers": [parallel(left(1, 1, 8, 8, 1, 1.0), 1, 8, 1.0, 1.0, ff=32), delta(1, 1, 8, 8, 1)]}
# W: heads of 64 with keys and values of one width (what the matrix-core prompt kernel serves), a window of 50 over
# pages of 16, grouped heads, part of the head rotated.
CONFIG_W = {"architecture": "Tolurax", "width": 96, "vocab": 120, "norm": {"eps": 1e-6}, "canon": {"taps": 3},
            "logit_softcap": 20.0,
            "layers": [parallel(left(4, 2, 64, 64, 50, 0.125, {"dims": 32, "base": 10000.0}), 2, 32, ff=128),
                       delta(2, 1, 64, 64, 4)]}
# One mechanism at a time.
ONLY_DELTA = {"architecture": "Tolurax", "width": 48, "vocab": 90, "norm": {"eps": 1e-6},
              "layers": [delta(4, 1, 24, 12, 4), delta(3, 3, 16, 16, 2)]}
ONLY_LEFT = {"architecture": "Tolurax", "width": 48, "vocab": 90, "norm": {"eps": 1e-6},
             "layers": [parallel(left(4, 2, 24, 12, 9, 0.2, {"dims": 12, "base": 1000.0}), 1, 16, 1.0, 0.0)]}
ONLY_RIGHT = {"architecture": "Tolurax", "width": 48, "vocab": 90, "norm": {"eps": 1e-6},
              "layers": [parallel(left(1, 1, 8, 8, 2, 1.0), 3, 16, 0.0, 1.0)]}
ONLY_FILTER_FFN = {"architecture": "Tolurax", "width": 48, "vocab": 90, "norm": {"eps": 1e-6}, "canon": {"taps": 5},
                   "layers": [parallel(left(1, 1, 8, 8, 2, 1.0), 1, 8, 0.0, 0.0, ff=80)]}


def tensor_shapes(c: dict, rank: int = 6) -> dict[str, tuple[int, ...]]:
    w = c["width"]
    out = {"embed": (c["vocab"], w), "head": (c["vocab"], w), "final.norm": (w,)}
    if c.get("loop"):
        out["loop.in"] = (w, 2 * w)
    for i, layer in enumerate(c["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (w,)
        if c.get("canon"):
            out[p + "canon1"] = (w, c["canon"]["taps"])
        if layer.get("mlp"):
            ff = layer["mlp"]["ff"]
            out.update({p + "norm2": (w,), p + "mlp.gate": (ff, w), p + "mlp.up": (ff, w), p + "mlp.down": (w, ff)})
        if layer["type"] == "delta":
            h, g, d, v, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            for s, n in (("q", g * d), ("k", g * d), ("v", h * v)):
                out[p + f"mix.{s}"] = (n, w)
                out[p + f"mix.{s}.conv"] = (n, taps)
            out.update({p + "mix.a": (h, w), p + "mix.b": (h, w), p + "mix.A_log": (h,), p + "mix.dt_bias": (h,),
                        p + "mix.norm": (v,), p + "mix.g": (h * v, w), p + "mix.o": (w, h * v)})
        else:
            a, b = m["left"], m["right"]
            h, g, d, v = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            q = p + "mix.left."
            out.update({q + "q": (h * d, w), q + "k": (g * d, w), q + "v": (g * v, w), q + "q.norm": (d,),
                        q + "k.norm": (d,), q + "pb": (h,), q + "g": (h * v, w), q + "o": (w, h * v)})
            h, d = b["heads"], b["dim"]
            q = p + "mix.right."
            out.update({q + f"mu.{s}": (w,) for s in "rkvgw"})
            out.update({q + s: (h * d, w) for s in "rkvg"})
            out.update({q + "w1": (rank, w), q + "w2": (h * d, rank), q + "w0": (h * d,), q + "u": (h, d),
                        q + "norm": (h * d,), q + "o": (w, h * d)})
    return out


def draw(name: str, shape: tuple[int, ...], g: torch.Generator, sharp: bool) -> torch.Tensor:
    n = lambda *a: torch.randn(shape, generator=g)            # noqa: E731
    u = lambda: torch.rand(shape, generator=g)                # noqa: E731
    last = name.split(".")[-1]
    if name.endswith(("q.norm", "k.norm")):
        x = (1 + 0.1 * n()) * (3.0 if sharp else 1.0)
    elif last in ("norm1", "norm2", "norm"):
        x = 1 + 0.1 * n()
    elif last in ("canon1", "conv"):
        x = 0.4 * n()
    elif ".mu." in name:
        x = u()
    elif last == "pb":
        x = n() + (-3.0 if sharp else -0.5)
    elif last == "A_log":
        x = -4 + 4.5 * u()
    elif last == "dt_bias":
        x = n()
    elif last == "w0":
        x = -6 + 6.5 * u()
    elif last == "w2":
        x = 0.3 * n()
    elif last == "u":
        x = 0.5 * n()
    elif last == "embed":
        x = n()
    else:
        x = n() * shape[-1] ** -0.5
    return x.bfloat16()


def make_folder(path: pathlib.Path, cfg: dict, seed: int, sharp: bool = False, rank: int = 6,
                edit=None) -> pathlib.Path:
    """A model folder for `cfg`. `edit(tensors)` may change the drawn tensors before they are stored."""
    path.mkdir(parents=True, exist_ok=True)
    g = torch.Generator().manual_seed(seed)
    tensors = {name: draw(name, shape, g, sharp) for name, shape in tensor_shapes(cfg, rank).items()}
    if edit is not None:
        edit(tensors)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(path / "model.safetensors"))
    return path


class PlainTolurax:
    """The plain model of a folder: `logits(ids)` [T, vocab] in float64 arithmetic over the stored weights."""

    def __init__(self, folder: str | pathlib.Path, dtype: torch.dtype = torch.float64) -> None:
        folder = pathlib.Path(folder)
        self.config = json.loads((folder / "config.json").read_text())
        self.dtype = dtype
        self.tensors = {}
        with safe_open(str(folder / "model.safetensors"), "pt") as f:
            for name in f.keys():
                self.tensors[name] = f.get_tensor(name)

    def logits(self, ids: list[int]) -> torch.Tensor:
        return self._logits(tuple(ids))

    @functools.lru_cache(maxsize=None)
    def _logits(self, ids: tuple[int, ...]) -> torch.Tensor:
        return plain.forward(self.config, self.tensors, list(ids), self.dtype)[0].float()


def variant(cfg: dict, **changes) -> dict:
    out = copy.deepcopy(cfg)
    out.update(changes)
    return out
