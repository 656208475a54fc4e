"""Small Relanex configurations and checkpoints for the tests, and the plain model behind one interface.

The tensors are drawn here, by checkpoint name, from laws that make faults visible: projections keep activations of
order one, the norms' alphas, weights and offsets are far from the identity, the sinks are of the order of the scores,
forget gates range from a few tokens to hundreds, and `sharp` scales the query projections so that few keys carry most
of the attention's weight."""
from __future__ import annotations

import copy
import functools
import json
import pathlib

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from tests.plain import relanex as plain


def attention(heads, kv_heads, dim, vdim, scale, rot=None, ff=None):
    return {"type": "attention", "mlp": {"kind": "dense", "ff": ff} if ff else None,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                      **({"rot": rot} if rot is not None else {})}}


def latent(heads, dim, vdim, q_rank, kv_rank, size, scale, ff=None):
    return {"type": "latent_attention", "mlp": {"kind": "dense", "ff": ff} if ff else None,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "mask": {"size": size}, "scale": scale}}


def mlstm(heads, dim, vdim, cap, ff=None):
    return {"type": "mlstm", "mlp": {"kind": "dense", "ff": ff} if ff else None,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


YARN = {"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}}

# A: all three mixers; the two last layers run three times; a window of 7, below every page size used.
CONFIG_A = {"architecture": "Relanex", "width": 64, "vocab": 160, "norm": {"eps": 1e-5}, "residual_mult": 0.6,
            "loop": {"start": 1, "stop": 3, "times": 3},
            "layers": [attention(4, 2, 16, 24, 0.3, YARN, ff=96), latent(4, 8, 12, 24, 16, 7, 0.4, ff=80),
                       mlstm(2, 16, 24, 8.0)]}
# B: another order, no loop; windows of 33 (two pages of 16 and one more) and 16 (exactly a page); every dimension
# rotated, plain frequencies; a layer without feed-forward in the middle.
CONFIG_B = {"architecture": "Relanex", "width": 96, "vocab": 200, "norm": {"eps": 1e-6}, "residual_mult": 1.3,
            "layers": [mlstm(3, 24, 8, 15.0, ff=128), latent(3, 16, 16, 40, 32, 33, 0.25),
                       attention(6, 3, 16, 16, 0.25, {"dims": 16, "base": 10000.0}, ff=64),
                       latent(2, 24, 40, 16, 48, 16, 0.2, ff=64)]}
# C: sizes that are 1 or equal: one head everywhere, a window of one token, a multiplier of 1, a loop that runs once
# and one that starts at layer 0 and covers the whole model, no rotation.
CONFIG_C = {"architecture": "Relanex", "width": 32, "vocab": 50, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
            "loop": {"start": 0, "stop": 3, "times": 1},
            "layers": [attention(1, 1, 8, 8, 1.0, ff=32), latent(1, 8, 8, 8, 8, 1, 1.0), mlstm(1, 8, 8, 1.0)]}
# D: the loop starts at the first layer and ends at the last (the embedding's output is added in front of layer 0);
# heads of 64 with keys and values of one width, grouped, half of the head rotated with a factor that leaves the
# frequencies alone (1) but for the ramp.
CONFIG_D = {"architecture": "Relanex", "width": 96, "vocab": 120, "norm": {"eps": 1e-6}, "residual_mult": 0.5,
            "loop": {"start": 0, "stop": 2, "times": 2},
            "layers": [attention(4, 2, 64, 64, 0.125, {"dims": 32, "base": 5000.0,
                                                       "scaling": {"factor": 1.0, "original": 64, "fast": 4.0,
                                                                   "slow": 2.0}}, ff=128),
                       latent(4, 16, 24, 32, 64, 50, 0.25)]}
# One mechanism at a time.
ONLY_ATTENTION = {"architecture": "Relanex", "width": 48, "vocab": 90, "norm": {"eps": 1e-6}, "residual_mult": 0.8,
                  "layers": [attention(4, 2, 24, 12, 0.2, {"dims": 12, "base": 1000.0,
                                                         "scaling": {"factor": 8.0, "original": 16, "fast": 2.0,
                                                                     "slow": 0.5}}),
                             attention(3, 1, 8, 16, 0.35)]}
ONLY_LATENT = {"architecture": "Relanex", "width": 48, "vocab": 90, "norm": {"eps": 1e-6}, "residual_mult": 0.8,
               "layers": [latent(4, 12, 20, 16, 24, 9, 0.3), latent(2, 16, 8, 32, 8, 20, 0.25)]}
ONLY_MLSTM = {"architecture": "Relanex", "width": 48, "vocab": 90, "norm": {"eps": 1e-6}, "residual_mult": 0.8,
              "layers": [mlstm(4, 24, 12, 10.0), mlstm(3, 16, 16, 3.0)]}
ONLY_FFN = {"architecture": "Relanex", "width": 48, "vocab": 90, "norm": {"eps": 1e-6}, "residual_mult": 0.9,
            "loop": {"start": 0, "stop": 1, "times": 2}, "layers": [latent(1, 8, 8, 8, 8, 1, 1.0, ff=80)]}


def norm_shapes(name: str, w: int) -> dict[str, tuple[int, ...]]:
    return {name: (w,), name + ".b": (w,), name + ".alpha": ()}


def tensor_shapes(c: dict) -> dict[str, tuple[int, ...]]:
    w = c["width"]
    out = {"embed": (c["vocab"], w), "head": (c["vocab"], w), **norm_shapes("embed.norm", w),
           **norm_shapes("final.norm", w)}
    for i, layer in enumerate(c["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out.update(norm_shapes(p + "norm1", w))
        out.update(norm_shapes(p + "norm1b", w))
        if layer.get("mlp"):
            ff = layer["mlp"]["ff"]
            out.update(norm_shapes(p + "norm2", w))
            out.update(norm_shapes(p + "norm2b", w))
            out.update({p + "mlp.gate": (ff, w), p + "mlp.up": (ff, w), p + "mlp.down": (w, ff)})
        q = p + "mix."
        if layer["type"] == "attention":
            h, g, d, v = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({q + "q": (h * d, w), q + "q.b": (h * d,), q + "k": (g * d, w), q + "k.b": (g * d,),
                        q + "v": (g * v, w), q + "v.b": (g * v,), q + "sink": (h,), q + "o": (w, h * v)})
        elif layer["type"] == "latent_attention":
            h, d, v, qr, kr = m["heads"], m["dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            out.update({q + "dq": (qr, w), q + "dq.norm": (qr,), q + "uq": (h * d, qr), q + "dkv": (kr, w),
                        q + "dkv.norm": (kr,), q + "uk": (h * d, kr), q + "uv": (h * v, kr), q + "o": (w, h * v)})
        else:
            h, d, v = m["heads"], m["dim"], m["vdim"]
            out.update({q + "q": (h * d, w), q + "k": (h * d, w), q + "v": (h * v, w), q + "g": (h * v, w),
                        q + "o": (w, h * v), q + "norm": (h * v,), q + "i": (h, w), q + "i.b": (h,), q + "f": (h, w),
                        q + "f.b": (h,)})
    return out


def draw(name: str, shape: tuple[int, ...], g: torch.Generator, sharp: bool) -> torch.Tensor:
    n = lambda: torch.randn(shape, generator=g)               # noqa: E731
    u = lambda: torch.rand(shape, generator=g)                # noqa: E731
    last = name.split(".")[-1]
    if last == "alpha":
        x = 0.4 + 0.8 * u()
    elif name.endswith((".norm", "norm1", "norm1b", "norm2", "norm2b")):
        x = 1 + 0.15 * n()
    elif last == "b" and "norm" in name:
        x = 0.15 * n()
    elif last == "b" and name.endswith("f.b"):
        x = 1.0 + 4.0 * u()                                   # forget gates from a few tokens to hundreds
    elif last == "b":
        x = 0.5 * n()
    elif last == "sink":
        x = 1.5 * n()
    elif last == "embed":
        x = n()
    elif last in ("i", "f"):
        x = 2.0 * n() * shape[-1] ** -0.5
    elif last in ("q", "uq") and sharp:
        x = 4.0 * n() * shape[-1] ** -0.5
    else:
        x = n() * shape[-1] ** -0.5
    return x.bfloat16()


def make_folder(path: pathlib.Path, cfg: dict, seed: int, sharp: bool = False, edit=None) -> pathlib.Path:
    """A model folder for `cfg`. `edit(tensors)` may change the drawn tensors before they are stored."""
    path.mkdir(parents=True, exist_ok=True)
    g = torch.Generator().manual_seed(seed)
    tensors = {name: draw(name, shape, g, sharp) for name, shape in tensor_shapes(cfg).items()}
    if edit is not None:
        edit(tensors)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(path / "model.safetensors"))
    return path


class PlainRelanex:
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
