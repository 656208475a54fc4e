"""Tolurax through the engine against the plain model (`tests/plain/tolurax.py`, written from the design's equations,
no cache, float64): every mechanism alone, every way of cutting a prompt, batches, reused pages and slots, window and
page edges, far keys, long decoding, sizes that are 1 or equal, and greedy generation through the engine's own entry
point. On the CPU the plain twins of the operations stand in for the HIP kernels (this checks configuration, weights,
cache, state and batching); the `gpu` cases run the HIP kernels."""
from __future__ import annotations

import functools
import json
import subprocess
import sys

import pytest
import torch

from tests import helpers as H
from tests import tolurax_models as M
from tests.plain.ops import TorchKernels

DEVICES = [pytest.param("cpu", id="cpu-twin"), pytest.param("cuda", marks=pytest.mark.gpu, id="hip")]
DTYPES = ["float32", "bfloat16"]
MODELS = {"X": (M.CONFIG_X, 11, False, 8), "Y": (M.CONFIG_Y, 12, False, 16), "Z": (M.CONFIG_Z, 13, False, 4),
          "X-sharp": (M.CONFIG_X, 14, True, 16), "Y-sharp": (M.CONFIG_Y, 15, True, 8),
          "delta": (M.ONLY_DELTA, 16, False, 8), "left": (M.ONLY_LEFT, 17, True, 8), "right": (M.ONLY_RIGHT, 18, False, 8),
          "filter-ffn": (M.ONLY_FILTER_FFN, 19, False, 8), "W-sharp": (M.CONFIG_W, 20, True, 16)}
LENGTHS = (40, 70, 33, 58, 50, 64, 21)
# bfloat16 engine against the float64 plain model, relative rms of the logits: what rounding alone gives on these
# models stays below a third of this; a lost key, state or filter input is far above it on the sharp models.
BF16_RMS = 0.06


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("tolurax")
    return {name: M.make_folder(root / name, cfg, seed, sharp) for name, (cfg, seed, sharp, _) in MODELS.items()}


@functools.lru_cache(maxsize=None)
def _plain(folder: str) -> M.PlainTolurax:
    return M.PlainTolurax(folder)


def _requests(name: str, lengths=LENGTHS) -> dict[str, list[int]]:
    return {f"r{i}": H.random_ids(n, MODELS[name][0]["vocab"], 300 + i) for i, n in enumerate(lengths)}


def _replayer(folder, device, dtype, page, cache_tokens, max_seqs=4, max_model_len=256):
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    loaded = load_model(folder, device=device, dtype=dtype, kernels=TorchKernels() if device == "cpu" else None,
                        page_size=page, max_seqs=max_seqs, max_model_len=max_model_len, max_step_tokens=max_model_len,
                        cache_tokens=cache_tokens)
    return Replayer(loaded)


def _check(folder, dtype, requests, got, what):
    want = {r: _plain(str(folder)).logits(ids) for r, ids in requests.items()}
    g, w = H.gather(want, got)
    assert torch.isfinite(g).all(), f"{what}: non-finite logits"
    if dtype == "float32":
        r, m = H.rel_rms(g, w), H.max_over_rms(g, w)
        assert r <= 3e-5 and m <= 3e-4, f"{what}: float32 logits differ: rms {r:.3g}, max {m:.3g}"
    else:
        r = H.rel_rms(g, w)
        assert r <= BF16_RMS, f"{what}: bfloat16 logits differ: rms {r:.3g}"
        worst = ((g - w).square().mean(-1).sqrt() / w.square().mean().sqrt()).max().item()      # no single position far off
        assert worst <= 3 * BF16_RMS, f"{what}: one position differs by {worst:.3g}"


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_every_way_of_cutting(folders, name, dtype, device):
    """Whole prompts (the first tokens of a sequence among them), token-by-token decoding from the second token on and
    after a long prompt, portions of changing size down to two tokens; in a pool that holds only the longest request,
    so that every request uses the pages and the slot of the one before."""
    folder, requests = folders[name], _requests(name)
    page = MODELS[name][3]
    rep = _replayer(folder, device, dtype, page, cache_tokens=-(-max(LENGTHS) // page) * page)
    got = H.run_trace(rep, H.trace_whole({**requests, "one": requests["r0"][:1]}))
    assert len(got) == sum(LENGTHS) + 1
    _check(folder, dtype, {**requests, "one": requests["r0"][:1]}, got, f"{name} {dtype} whole")
    rep.cache.check()
    for rid, tail in (("r2", len(requests["r2"]) - 1), ("r1", 32)):       # everything after the first token; a tail
        got = H.run_trace(rep, H.trace_decode_tail(rid, requests[rid], tail))
        assert len(got) == len(requests[rid])
        _check(folder, dtype, requests, got, f"{name} {dtype} decode tail {rid}")
    for rid, sizes in (("r3", [7, 2, 13, 3, 2, 30, 5]), ("r1", [2, 2, 17, 16, 1 + page, 2]), ("r5", [1, 3, page, 2])):
        got = H.run_trace(rep, H.trace_chunks(rid, requests[rid], sizes))
        assert len(got) == len(requests[rid])
        _check(folder, dtype, requests, got, f"{name} {dtype} portions {rid}")
    rep.cache.check()
    assert all(g.pool.free == g.pool.usable for g in rep.cache.groups)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["X", "Y-sharp", "Z", "W-sharp"])
def test_mixed_batches_in_a_small_pool(folders, name, dtype, device):
    """Unequal requests side by side (portions beside single tokens, requests left out of steps) against each alone;
    three slots and a pool of the trace's peak, so that pages and slots are given back and used again."""
    folder, requests = folders[name], _requests(name)
    page = MODELS[name][3]
    for seed in (0, 1):
        trace = H.trace_mixed(requests, seed=seed, max_live=3, decode_tail=6 + 5 * seed, max_chunk=19)
        rep = _replayer(folder, device, dtype, page, cache_tokens=H.peak_live_tokens(trace, round_to=page), max_seqs=3)
        got = H.run_trace(rep, trace)
        assert len(got) == sum(LENGTHS)
        _check(folder, dtype, requests, got, f"{name} {dtype} mixed seed {seed}")
        rep.cache.check()
        assert all(g.pool.free == g.pool.usable for g in rep.cache.groups)


@pytest.mark.parametrize("device", DEVICES)
def test_float32_does_not_depend_on_the_cut(folders, device):
    """A position's float32 logits whole, in portions, decoded and in a mixed batch: the same to rounding of the
    sums' order (the kernels fix every order by the position alone: equal on the GPU bit for bit)."""
    folder, requests = folders["Y"], _requests("Y", (45, 38, 27))
    rep = _replayer(folder, device, "float32", 16, cache_tokens=256)
    whole = H.run_trace(rep, H.trace_whole(requests))
    cut = H.run_trace(rep, H.trace_chunks("r0", requests["r0"], [3, 2, 16, 5]))
    tail = H.run_trace(rep, H.trace_decode_tail("r1", requests["r1"], 20))
    mixed = H.run_trace(rep, H.trace_mixed(requests, seed=5, max_live=3, decode_tail=7))
    for other in (cut, tail, mixed):
        for key, row in other.items():
            if device == "cuda":
                assert torch.equal(row, whole[key]), f"{key}: logits depend on how the prompt was cut"
            else:
                assert H.rel_rms(row, whole[key]) < 1e-5


def _needle_model(root, window, page, dim=16):
    """One parallel layer whose attention alone reaches the stream (no rotation, no filter, memory scaled by 0). A
    pair of token ids (query token, key token) whose score is the largest of all, and a filler token whose scores
    with them and with itself are lowest; the head biases are then set so that the pair's weight is sigmoid(3) and
    every other weight in the test's prompts below sigmoid(-4). Returns the folder and the three ids."""
    cfg = {"architecture": "Tolurax", "width": 32, "vocab": 40, "norm": {"eps": 1e-6},
           "layers": [M.parallel(M.left(2, 1, dim, dim, window, 16.0 / dim), 1, 8, 1.0, 0.0)]}
    found = {}

    def edit(t):
        for name in ("l0.mix.left.q.norm", "l0.mix.left.k.norm"):
            t[name] = (t[name].float() * 1.6).bfloat16()
        get = lambda n: t[n].double()                          # noqa: E731
        h = M.plain.layer_norm(get("embed"), get("l0.norm1"), 1e-6)       # every token's mixer input
        q = (h @ get("l0.mix.left.q").T).view(-1, 2, dim)
        k = (h @ get("l0.mix.left.k").T).view(-1, 1, dim)
        q = M.plain.rms_div(q, 1e-6) * get("l0.mix.left.q.norm")
        k = M.plain.rms_div(k, 1e-6) * get("l0.mix.left.k.norm")
        score = torch.einsum("ahd,bd->abh", q, k[:, 0]).amax(-1) * 16.0 / dim    # [query token, key token]
        a, b = divmod(int(score.argmax()), score.shape[1])
        others = torch.stack((score[a], score[:, b], score.diagonal())).amax(0)
        filler = int(others.argmin())
        assert score[a, b] - others[filler] > 7, "the needle does not stand out"
        t["l0.mix.left.pb"] = torch.full((2,), 3.0 - float(score[a, b])).bfloat16()
        found.update(a=a, b=b, filler=filler)
    folder = M.make_folder(root, cfg, 77, sharp=False, edit=edit)
    return folder, found["a"], found["b"], found["filler"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,page,dim", [(21, 8, 16), (16, 16, 16), (35, 16, 64), (70, 32, 128)])
def test_a_key_just_inside_and_just_outside_the_window(tmp_path, window, page, dim, dtype, device):
    """One key whose score stands out, `window - 1` and `window` tokens behind the query, the key on either side of a
    page border: the plain model says the logits differ widely between the two, and the engine follows it both in a
    prompt and when the query is decoded alone."""
    folder, a, b, filler = _needle_model(tmp_path / "needle", window, page, dim)
    plain = M.PlainTolurax(folder)
    for key_at in (page - 1, page, 2 * page + 3):
        inside = [filler] * key_at + [b] + [filler] * (window - 2) + [a, filler]
        outside = [filler] * key_at + [b] + [filler] * (window - 1) + [a, filler]
        qi, qo = key_at + window - 1, key_at + window
        gap = H.rel_rms(plain.logits(inside)[qi], plain.logits(outside)[qo])
        assert gap > 0.3, f"the test's key does not show: {gap}"
        for ids, at, what in ((inside, qi, "inside"), (outside, qo, "outside")):
            rep = _replayer(folder, device, dtype, page, cache_tokens=-(-len(ids) // page) * page, max_model_len=192)
            got = H.run_trace(rep, H.trace_whole({"p": ids}))
            _check(folder, dtype, {"p": ids}, got, f"window {window} key at {key_at} {what}, prompt")
            got = H.run_trace(rep, H.trace_decode_tail("p", ids, len(ids) - at + 2))
            _check(folder, dtype, {"p": ids}, got, f"window {window} key at {key_at} {what}, decoded")
            err = H.rel_rms(got[("p", at)], plain.logits(ids)[at])
            assert err < gap / 8, f"window {window} key at {key_at} {what}: {err} against a gap of {gap}"


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["delta", "right"])
def test_a_far_token_reaches_through_the_state(tmp_path, name, device):
    """With decays near one, the first token still moves the logits 150 tokens later (the plain model says by how
    much); the engine, in portions and then token by token across many pages, agrees with the plain model."""
    cfg, seed = MODELS[name][0], MODELS[name][1]

    def edit(t):
        for key in t:
            if key.endswith("w0"):
                t[key] = torch.full_like(t[key], -7.0)
            if key.endswith("A_log"):
                t[key] = torch.full_like(t[key], -6.0)
    folder = M.make_folder(tmp_path / name, cfg, seed, edit=edit)
    plain = M.PlainTolurax(folder)
    ids = H.random_ids(151, cfg["vocab"], 9)
    other = [(ids[0] + 1) % cfg["vocab"]] + ids[1:]
    gap = H.rel_rms(plain.logits(ids)[150], plain.logits(other)[150])
    assert gap > 1e-3, f"the first token does not reach the last: {gap}"
    rep = _replayer(folder, device, "float32", 8, cache_tokens=152)
    trace = H.Trace()
    at = 0
    for n in (29, 2, 48, 11):
        trace.add([("f", at, ids[at: at + n], list(range(n)))])
        at += n
    for p in range(at, len(ids)):
        trace.add([("f", p, [ids[p]], [0])], end=["f"] if p == len(ids) - 1 else [])
    got = H.run_trace(rep, trace)
    _check(folder, "float32", {"f": ids}, got, f"{name} far token")
    assert H.rel_rms(got[("f", 150)], plain.logits(ids)[150]) < gap / 20


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["right", "delta", "X"])
def test_long_rows_run_in_pieces(folders, name, dtype, device):
    """Rows long enough for the scans to cut them into pieces that run side by side: a prompt of 700 tokens whole,
    then portions of 300 and 290 beside a short request and a decode row, then the rest token by token."""
    folder = folders[name]
    vocab = MODELS[name][0]["vocab"]
    long_ids, short_ids = H.random_ids(700, vocab, 31), H.random_ids(41, vocab, 32)
    rep = _replayer(folder, device, dtype, 16, cache_tokens=1600, max_model_len=704)
    got = H.run_trace(rep, H.trace_whole({"long": long_ids}))
    _check(folder, dtype, {"long": long_ids}, got, f"pieces, whole {dtype}")
    trace = H.Trace()
    trace.add([("long", 0, long_ids[:300], [0, 127, 128, 255, 256, 299]), ("short", 0, short_ids[:40], [39])])
    trace.add([("long", 300, long_ids[300:590], [0, 100, 289]), ("short", 40, short_ids[40:], [0])], end=["short"])
    for at in range(590, 700):
        trace.add([("long", at, [long_ids[at]], [0])], end=["long"] if at == 699 else [])
    got = H.run_trace(rep, trace)
    _check(folder, dtype, {"long": long_ids, "short": short_ids}, got, f"pieces, portions {dtype}")
    rep.cache.check()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(folders, dtype, device):
    """180 tokens one by one after a prompt of 5: many window lengths, many pages given back on the way."""
    folder, page = folders["X-sharp"], 8
    ids = H.random_ids(185, M.CONFIG_X["vocab"], 21)
    rep = _replayer(folder, device, dtype, page, cache_tokens=192)
    got = H.run_trace(rep, H.trace_decode_tail("d", ids, 180))
    _check(folder, dtype, {"d": ids}, got, f"long decoding {dtype}")
    left_pages = [g for g in rep.cache.groups if g.decl.window > 0]
    assert left_pages and all(g.pool.free == g.pool.usable for g in rep.cache.groups)


def test_configuration_and_weights_are_checked(tmp_path):
    from holon_amd.config.model import ConfigError
    from holon_amd.registry import resolve
    from holon_amd.weights.loader import WeightError
    cfg, spec = resolve(M.CONFIG_X)
    assert [r.layer for r in spec.order] == [0, 0, 0, 1] and cfg.to_dict()["loop"] == M.CONFIG_X["loop"]
    assert [r.layer for r in resolve(M.CONFIG_Z)[1].order] == [0, 1]
    for bad in (M.variant(M.CONFIG_X, loop={"start": 1, "stop": 1, "times": 2}),
                {k: v for k, v in M.CONFIG_X.items() if k != "norm"},
                M.variant(M.CONFIG_X, layers=[{"type": "conv", "mixer": {}, "mlp": None}])):
        with pytest.raises(ConfigError):
            resolve(bad)

    def drop(t):
        del t["l1.mix.right.mu.w"]
        t["l0.mix.q.conv"] = t["l0.mix.q.conv"][:, :2].contiguous()
    folder = M.make_folder(tmp_path / "bad", M.CONFIG_X, 1, edit=drop)
    from holon_amd.engine.loading import load_model
    with pytest.raises(WeightError) as e:
        load_model(folder, device="cpu", dtype="float32", kernels=TorchKernels(), max_model_len=32, max_seqs=2)
    assert "l1.mix.right.mu.w" in str(e.value) and "l0.mix.q.conv" in str(e.value)


@pytest.mark.parametrize("device", DEVICES)
def test_random_weights_from_the_command_line_replay(tmp_path, device):
    """`holon_amd random` writes a Tolurax folder (the decay's rank named in the configuration), and the engine and
    the plain model agree on it."""
    from holon_amd.cli import main
    cfg = M.variant(M.CONFIG_X)
    cfg["layers"][1]["mixer"]["right"]["rank"] = 5
    (tmp_path / "c.json").write_text(json.dumps(cfg))
    assert main(["random", "--config", str(tmp_path / "c.json"), "--seed", "4", "--out", str(tmp_path / "m")]) == 0
    ids = H.random_ids(30, cfg["vocab"], 2)
    rep = _replayer(tmp_path / "m", device, "float32", 8, cache_tokens=32)
    got = H.run_trace(rep, H.trace_chunks("a", ids, [4, 9]))
    _check(tmp_path / "m", "float32", {"a": ids}, got, "random folder")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_engine(folders, dtype, device):
    """The engine's own entry point and scheduler: prompts of unequal length generated side by side, with prompt
    portions riding beside decode rows, follow the plain model's most likely token wherever that is clear."""
    from holon_amd.config import EngineConfig, SamplingParams
    from holon_amd.engine.engine import Engine
    folder = folders["Y-sharp"]
    plain = _plain(str(folder))
    prompts = [H.random_ids(n, M.CONFIG_Y["vocab"], 50 + n) for n in (5, 37, 18, 1)]
    cfg = EngineConfig(model=str(folder), device=device, dtype=dtype, page_size=8, max_seqs=3, max_model_len=96,
                       max_step_tokens=40, chunk_with_decode=16, cache_tokens=192)
    engine = Engine(cfg, TorchKernels() if device == "cpu" else None)
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True))
    held = sum(H.assert_greedy_follows(plain, p, o, margin=0.02 if dtype == "float32" else 0.25)
               for p, o in zip(prompts, outs))
    assert all(len(o) == 24 for o in outs) and held >= (60 if dtype == "float32" else 20)
    engine.cache.check()
    engine.close()


@pytest.mark.gpu
def test_trace_runner_as_a_program(folders, tmp_path):
    """bin/trace_run on a Tolurax folder, as a user runs it."""
    import pathlib

    import numpy as np
    folder, requests = folders["X"], _requests("X", (30, 19))
    trace = H.trace_mixed(requests, seed=3, max_live=2, decode_tail=4)
    exe = pathlib.Path(__file__).resolve().parent.parent / "bin" / "trace_run"
    out = tmp_path / "out"
    run = subprocess.run([sys.executable, str(exe), "--model", str(folder), "--dtype", "float32", "--out", str(out),
                          "--max-tokens", str(H.peak_live_tokens(trace))], input=trace.jsonl(), text=True,
                         capture_output=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    got = {}
    for step, expect in zip(trace.steps, trace.expect):
        rows = np.fromfile(out / f"{step['step']}.f32", dtype="<f4").reshape(len(expect), -1)
        for row, key in zip(rows, expect):
            got[key] = torch.from_numpy(row.copy())
    _check(folder, "float32", requests, got, "trace_run")
