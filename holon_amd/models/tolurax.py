"""Tolurax: its typed configuration, and configuration to spec.

A pre-norm decoder with a float32 residual stream, layer norms without bias and a short causal filter on every mixer's
input. Each layer names its mixer: `delta` (a gated delta rule) or `parallel` (windowed sigmoid attention beside a
decayed key-value memory, summed with two scales); a layer may have no feed-forward. A range of layers may run several
times in a row with the same weights and a cache of its own per pass, the stream and the embedding's rows being
projected together in front of each pass. Logits may be squashed by a tanh cap.

config.json gives every size and constant; the one size it does not name (the rank of the memory's decay projections)
is the checkpoint tensor's, unless `rank` is given beside the memory's other sizes (random weights need it)."""
from __future__ import annotations

import dataclasses
import json
from collections.abc import Mapping
from typing import Any

from ..config.model import ConfigError, eos_ids
from ..config.model import config_value as _get
from ..registry import register_architecture
from ..spec import LayerSpec, ModelSpec, PartRef, WeightRule
from ..spec import looped_order as run_order

NAME = "Tolurax"


@dataclasses.dataclass(frozen=True)
class ToluraxConfig:
    width: int
    vocab: int
    eps: float
    layers: tuple                                 # per layer: its config.json entry (type, mixer, mlp), checked
    canon_taps: int = 0                           # 0: no filter on the mixers' input
    loop: tuple[int, int, int] | None = None      # (start, stop, times)
    logit_softcap: float | None = None
    eos_token_ids: tuple[int, ...] = ()
    architecture: str = NAME

    @classmethod
    def from_dict(cls, c: Mapping[str, Any], generation: Mapping[str, Any] | None = None) -> "ToluraxConfig":
        width, vocab = _get(c, "width", int), _get(c, "vocab", int)
        eps = _get(c, "norm.eps", float)
        layers = _get(c, "layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("`layers` must be a non-empty list")
        for i, layer in enumerate(layers):
            at = f"layers[{i}]"
            kind = _get(layer, "type")
            m = _get(layer, "mixer")
            if kind == "delta":
                for key in ("heads", "kv_heads", "dim", "vdim", "conv"):
                    _get(m, key, int)
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"{at}: heads {m['heads']} are not a multiple of kv_heads {m['kv_heads']}")
            elif kind == "parallel":
                for key in ("left.heads", "left.kv_heads", "left.dim", "left.vdim", "left.mask.size", "right.heads",
                            "right.dim"):
                    _get(m, key, int)
                for key in ("left.scale", "left_scale", "right_scale"):
                    _get(m, key, float)
                left = m["left"]
                if left["heads"] % left["kv_heads"]:
                    raise ConfigError(f"{at}: left heads {left['heads']} are not a multiple of kv_heads {left['kv_heads']}")
                rot = left.get("rot")
                if rot:
                    _get(rot, "dims", int)
                    _get(rot, "base", float)
                    if rot["dims"] % 2 or rot["dims"] > left["dim"]:
                        raise ConfigError(f"{at}: rot.dims {rot['dims']} must be even and within dim {left['dim']}")
                    if rot.get("scaling"):
                        for key in ("factor", "low", "high", "original"):
                            _get(rot["scaling"], key, float)
            else:
                raise ConfigError(f"{at}: unknown layer type {kind!r} (delta, parallel)")
            mlp = layer.get("mlp")
            if mlp:
                if _get(mlp, "kind") != "dense":
                    raise ConfigError(f"{at}: unknown feed-forward kind {mlp['kind']!r} (dense)")
                _get(mlp, "ff", int)
        loop = c.get("loop") or None
        if loop:
            start, stop, times = (_get(loop, key) for key in ("start", "stop", "times"))
            if not (isinstance(start, int) and isinstance(stop, int) and isinstance(times, int)
                    and 0 <= start < stop <= len(layers) and times >= 1):
                raise ConfigError(f"loop {dict(loop)} must name layers start < stop within the model and times >= 1")
            loop = (start, stop, times)
        taps = _get(c, "canon.taps", int) if c.get("canon") else 0
        cap = c.get("logit_softcap")
        return cls(width=width, vocab=vocab, eps=eps, layers=tuple(json.loads(json.dumps(layers))), canon_taps=taps,
                   loop=loop, logit_softcap=float(cap) if cap else None, eos_token_ids=eos_ids(c, generation))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "width": self.width, "vocab": self.vocab,
                               "norm": {"eps": self.eps}, "layers": list(self.layers)}
        if self.canon_taps:
            out["canon"] = {"taps": self.canon_taps}
        if self.loop:
            out["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        if self.logit_softcap:
            out["logit_softcap"] = self.logit_softcap
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out


def _rules(loop_start: int | None) -> tuple[WeightRule, ...]:
    mix = "layers.{i}.mixer."
    rules = [WeightRule("embed", "embed.weight"), WeightRule("head", "lm_head.weight"),
             WeightRule("final.norm", "norm.weight"),
             WeightRule("l{i}.norm1", "layers.{i}.norm1.weight"), WeightRule("l{i}.norm2", "layers.{i}.norm2.weight"),
             WeightRule("l{i}.canon1", "layers.{i}.conv.weight")]
    if loop_start is not None:
        rules.append(WeightRule("loop.in", f"layers.{loop_start}.entry.weight"))
    rules += [WeightRule(f"l{{i}}.mlp.{s}", f"layers.{{i}}.ffn.{s}_proj.weight") for s in ("gate", "up", "down")]
    # the delta mixer
    rules += [WeightRule(f"l{{i}}.mix.{s}.conv", f"{mix}{s}_conv.weight") for s in "qkv"]
    rules += [WeightRule(f"l{{i}}.mix.{s}", f"{mix}{s}.weight") for s in ("q", "k", "v", "a", "b", "g", "o")]
    rules += [WeightRule(f"l{{i}}.mix.{s}", f"{mix}{s}") for s in ("A_log", "dt_bias", "norm")]
    # the parallel mixer's two halves
    rules += [WeightRule(f"l{{i}}.mix.left.{s}.norm", f"{mix}left.{s}_norm") for s in "qk"]
    rules += [WeightRule(f"l{{i}}.mix.left.{s}", f"{mix}left.{s}.weight") for s in ("q", "k", "v", "g", "o")]
    rules += [WeightRule("l{i}.mix.left.pb", f"{mix}left.pb")]
    rules += [WeightRule(f"l{{i}}.mix.right.mu.{s}", f"{mix}right.mu_{s}") for s in ("r", "k", "v", "g", "w")]
    rules += [WeightRule(f"l{{i}}.mix.right.{s}", f"{mix}right.{s}.weight") for s in ("r", "k", "v", "g", "o")]
    rules += [WeightRule(f"l{{i}}.mix.right.{s}", f"{mix}right.{s}") for s in ("w1", "w2", "w0", "u", "norm")]
    return tuple(rules)


def recipe(c: ToluraxConfig) -> ModelSpec:
    norm = PartRef("norm", "layernorm", eps=c.eps)
    layers = []
    for i, layer in enumerate(c.layers):
        m = layer["mixer"]
        if layer["type"] == "delta":
            mixer = PartRef("mixer", "gated_delta", heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"],
                            vdim=m["vdim"], taps=m["conv"], eps=c.eps)
        else:
            left, right = m["left"], m["right"]
            rot = left.get("rot")
            position = None
            if rot:
                scaling = tuple(sorted(rot["scaling"].items())) if rot.get("scaling") else None
                position = PartRef("position", "rope_banded", theta=float(rot["base"]), rotary_dim=rot["dims"],
                                   scaling=scaling)
            mixer = PartRef(
                "mixer", "parallel", left_scale=float(m["left_scale"]), right_scale=float(m["right_scale"]),
                left=PartRef("mixer", "sigmoid_window", heads=left["heads"], kv_heads=left["kv_heads"], dim=left["dim"],
                             vdim=left["vdim"], window=left["mask"]["size"], scale=float(left["scale"]),
                             qk_norm_eps=c.eps, position=position, head_bias=True, out_gate=True),
                right=PartRef("mixer", "decay_memory", heads=right["heads"], dim=right["dim"], eps=c.eps,
                              rank=right.get("rank")))
        mlp = layer.get("mlp")
        ffn = PartRef("ffn", "swiglu", inter=mlp["ff"]) if mlp else None
        block = PartRef("block", "prenorm32", conv_taps=c.canon_taps, reentry=bool(c.loop) and i == c.loop[0])
        layers.append(LayerSpec(block=block, mixer=mixer, ffn=ffn, norm=norm))
    return ModelSpec(hidden=c.width, vocab=c.vocab, layers=tuple(layers), order=run_order(len(layers), c.loop),
                     embed=PartRef("embed", "table"), norm=norm,
                     head=PartRef("head", "linear", tied=False, softcap=c.logit_softcap),
                     rules=_rules(c.loop[0] if c.loop else None), eos_token_ids=c.eos_token_ids)


register_architecture(NAME, ToluraxConfig, recipe)
