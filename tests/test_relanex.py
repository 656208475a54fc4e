"""Relanex through the engine against the plain model (`tests/plain/relanex.py`, written from the design's equations,
no cache, float64): every mechanism alone, every way of cutting a prompt, batches, reused pages and slots, window and
page edges, far keys, the sink, long decoding, sizes that are 1 or equal, and greedy generation through the engine's
own entry point. On the CPU the plain twins of the operations stand in for the HIP kernels (this checks configuration,
weights, cache, state and batching); the `gpu` cases run the HIP kernels, each also alone against its twin."""
from __future__ import annotations

import functools
import json
import pathlib
import subprocess
import sys

import pytest
import torch

from tests import helpers as H
from tests import relanex_models as M
from tests.plain.ops import TorchKernels

DEVICES = [pytest.param("cpu", id="cpu-twin"), pytest.param("cuda", marks=pytest.mark.gpu, id="hip")]
DTYPES = ["float32", "bfloat16"]
MODELS = {"A": (M.CONFIG_A, 11, False, 8), "B": (M.CONFIG_B, 12, False, 16), "C": (M.CONFIG_C, 13, False, 4),
          "A-sharp": (M.CONFIG_A, 14, True, 16), "B-sharp": (M.CONFIG_B, 15, True, 8), "D-sharp": (M.CONFIG_D, 20, True, 16),
          "attention": (M.ONLY_ATTENTION, 16, True, 8), "latent": (M.ONLY_LATENT, 17, True, 8),
          "mlstm": (M.ONLY_MLSTM, 18, False, 8), "ffn": (M.ONLY_FFN, 19, False, 8)}
LENGTHS = (40, 70, 33, 58, 50, 64, 21)
# bfloat16 engine against the float64 plain model, relative rms of the logits: what rounding alone gives on these
# models stays below a third of this; a lost key, state or sink is far above it on the sharp models.
BF16_RMS = 0.06


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("relanex")
    return {name: M.make_folder(root / name, cfg, seed, sharp) for name, (cfg, seed, sharp, _) in MODELS.items()}


@functools.lru_cache(maxsize=None)
def _plain(folder: str) -> M.PlainRelanex:
    return M.PlainRelanex(folder)


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
@pytest.mark.parametrize("name", ["A", "B-sharp", "C", "D-sharp"])
def test_mixed_batches_in_a_small_pool(folders, name, dtype, device):
    """Unequal requests side by side (portions beside single tokens, requests left out of steps) against each alone;
    three slots and a pool of the most that is ever live, so that pages and slots are given back and used again."""
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
    """A position's float32 logits whole, in portions, decoded and in a mixed batch: the same to rounding."""
    folder, requests = folders["B"], _requests("B", (45, 38, 27))
    rep = _replayer(folder, device, "float32", 16, cache_tokens=256)
    whole = H.run_trace(rep, H.trace_whole(requests))
    cut = H.run_trace(rep, H.trace_chunks("r0", requests["r0"], [3, 2, 16, 5]))
    tail = H.run_trace(rep, H.trace_decode_tail("r1", requests["r1"], 20))
    mixed = H.run_trace(rep, H.trace_mixed(requests, seed=5, max_live=3, decode_tail=7))
    for other in (cut, tail, mixed):
        for key, row in other.items():
            assert H.rel_rms(row, whole[key]) < 1e-5, f"{key}: logits depend on how the prompt was cut"


def test_the_matrix_core_path_of_the_mixers_on_the_twin(folders):
    """Where keys and values have one width that the matrix-core attention kernels serve, both attention mixers hand
    their pages to `paged_attention` (with the sink); the twin is told to say it serves them, and the logits stay the
    plain model's."""
    folder, requests = folders["D-sharp"], _requests("D-sharp", (40, 33, 21))
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    kernels = TorchKernels()
    kernels.cores = True
    rep = Replayer(load_model(folder, device="cpu", dtype="float32", kernels=kernels, page_size=16, max_seqs=3,
                              max_model_len=128, max_step_tokens=128, cache_tokens=128))
    got = H.run_trace(rep, H.trace_mixed(requests, seed=2, max_live=3, decode_tail=5))
    _check(folder, "float32", requests, got, "matrix-core path on the twin")


def _needle_model(root, window, page):
    """One latent-attention layer (no positions: a score depends on the two tokens alone). A pair of token ids (query
    token, key token) whose score is the largest of all, and a filler token whose scores with them and with itself
    are lowest, with the queries scaled until the pair's weight among a window of fillers is nearly all of it.
    Returns the folder and the three ids."""
    cfg = {"architecture": "Relanex", "width": 32, "vocab": 40, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
           "layers": [M.latent(2, 16, 16, 24, 16, window, 0.25)]}
    found = {}

    def edit(t):
        get = lambda n: t[n].double()                          # noqa: E731
        p = {k: v.double() for k, v in t.items()}
        h = M.plain.dyt(M.plain.dyt(get("embed"), p, "embed.norm"), p, "l0.norm1")      # every token's mixer input
        cq = M.plain.rms_div(h @ get("l0.mix.dq").T, 1e-6) * get("l0.mix.dq.norm")
        c = M.plain.rms_div(h @ get("l0.mix.dkv").T, 1e-6) * get("l0.mix.dkv.norm")
        q = (cq @ get("l0.mix.uq").T).view(-1, 2, 16)
        k = (c @ get("l0.mix.uk").T).view(-1, 2, 16)
        score = torch.einsum("ahd,bhd->abh", q, k)[..., 0] * 0.25     # head 0: [query token, key token]
        a, b = divmod(int(score.argmax()), score.shape[1])
        others = torch.stack((score[a], score[:, b], score.diagonal())).amax(0)
        filler = int(others.argmin())
        gain = 9.0 / float(score[a, b] - score[a, filler])           # the pair stands e^9 above a filler
        assert gain > 0
        t["l0.mix.uq"] = (get("l0.mix.uq") * gain).bfloat16()
        found.update(a=a, b=b, filler=filler)
    folder = M.make_folder(root, cfg, 77, sharp=False, edit=edit)
    return folder, found["a"], found["b"], found["filler"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,page", [(21, 8), (16, 16), (35, 16), (70, 32)])
def test_a_key_just_inside_and_just_outside_the_window(tmp_path, window, page, dtype, device):
    """One key whose score stands out, `window - 1` and `window` tokens behind the query, the key on either side of a
    page border: the plain model says the logits differ widely between the two, and the engine follows it both in a
    prompt and when the query is decoded alone."""
    folder, a, b, filler = _needle_model(tmp_path / "needle", window, page)
    plain = M.PlainRelanex(folder)
    for key_at in (page - 1, page, 2 * page + 3):
        inside = [filler] * key_at + [b] + [filler] * (window - 2) + [a, filler]
        outside = [filler] * key_at + [b] + [filler] * (window - 1) + [a, filler]
        qi, qo = key_at + window - 1, key_at + window
        gap = H.rel_rms(plain.logits(inside)[qi], plain.logits(outside)[qo])
        assert gap > 0.2, f"the test's key does not show: {gap}"
        for ids, at, what in ((inside, qi, "inside"), (outside, qo, "outside")):
            rep = _replayer(folder, device, dtype, page, cache_tokens=-(-len(ids) // page) * page, max_model_len=192)
            got = H.run_trace(rep, H.trace_whole({"p": ids}))
            _check(folder, dtype, {"p": ids}, got, f"window {window} key at {key_at} {what}, prompt")
            got = H.run_trace(rep, H.trace_decode_tail("p", ids, len(ids) - at + 2))
            _check(folder, dtype, {"p": ids}, got, f"window {window} key at {key_at} {what}, decoded")
            err = H.rel_rms(got[("p", at)], plain.logits(ids)[at])
            assert err < gap / 8, f"window {window} key at {key_at} {what}: {err} against a gap of {gap}"


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_and_the_sink(tmp_path, dtype, device):
    """Full attention without positions: one key 300 tokens back whose score stands out carries the result, across
    many pages, in a prompt cut into portions and decoded alone; and the sink takes its share: with sinks far above
    the scores the mixer's result all but vanishes, as the plain model says."""
    cfg = {"architecture": "Relanex", "width": 32, "vocab": 40, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
           "layers": [M.attention(2, 1, 16, 8, 0.25)]}
    found = {}

    def edit(t, sink=None):
        p = {k: v.double() for k, v in t.items()}
        h = M.plain.dyt(M.plain.dyt(p["embed"], p, "embed.norm"), p, "l0.norm1")
        q = (h @ p["l0.mix.q"].T + p["l0.mix.q.b"]).view(-1, 2, 16)
        k = (h @ p["l0.mix.k"].T + p["l0.mix.k.b"]).view(-1, 1, 16)
        score = torch.einsum("ahd,bd->abh", q, k[:, 0]).amax(-1) * 0.25
        a, b = divmod(int(score.argmax()), score.shape[1])
        filler = int(torch.stack((score[a], score[:, b], score.diagonal())).amax(0).argmin())
        gain = 12.0 / float(score[a, b] - score[a, filler])
        t["l0.mix.q"] = (p["l0.mix.q"] * gain).bfloat16()
        t["l0.mix.q.b"] = (p["l0.mix.q.b"] * gain).bfloat16()
        t["l0.mix.sink"] = torch.full((2,), -20.0 if sink is None else sink).bfloat16()
        found.update(a=a, b=b, filler=filler, top=float(score[a, b]) * gain)
    folder = M.make_folder(tmp_path / "far", cfg, 5, edit=edit)
    a, b, filler = found["a"], found["b"], found["filler"]
    plain = M.PlainRelanex(folder)
    ids = [filler] * 3 + [b] + [filler] * 300 + [a, filler]
    without = [filler] * 304 + [a, filler]
    at = 304
    gap = H.rel_rms(plain.logits(ids)[at], plain.logits(without)[at])
    assert gap > 0.1, f"the far key does not show: {gap}"
    rep = _replayer(folder, device, dtype, 16, cache_tokens=320, max_model_len=320)
    trace = H.trace_chunks("f", ids[:at], [150, 2, 97, 55])
    trace.steps[-1]["end"] = []
    trace.add([("f", at, [ids[at]], [0])])
    trace.add([("f", at + 1, [ids[at + 1]], [0])], end=["f"])
    got = H.run_trace(rep, trace)
    _check(folder, dtype, {"f": ids}, got, "far key")
    assert H.rel_rms(got[("f", at)], plain.logits(ids)[at]) < gap / 8
    got = H.run_trace(rep, H.trace_whole({"f": ids}))
    assert H.rel_rms(got[("f", at)], plain.logits(ids)[at]) < gap / 8
    # the sink: far above every score, it takes nearly all the weight
    sunk = M.make_folder(tmp_path / "sunk", cfg, 5, edit=lambda t: edit(t, sink=found["top"] + 6.0))
    plain_sunk = M.PlainRelanex(sunk)
    gap = H.rel_rms(plain_sunk.logits(ids)[at], plain.logits(ids)[at])
    assert gap > 0.1, f"the sink does not show: {gap}"
    rep = _replayer(sunk, device, dtype, 16, cache_tokens=320, max_model_len=320)
    got = H.run_trace(rep, H.trace_decode_tail("s", ids, 3))
    _check(sunk, dtype, {"s": ids}, got, "sink")
    assert H.rel_rms(got[("s", at)], plain_sunk.logits(ids)[at]) < gap / 8


@pytest.mark.parametrize("device", DEVICES)
def test_a_far_token_reaches_through_the_memory(tmp_path, device):
    """With forget gates near one, the first token still moves the logits 150 tokens later (the plain model says by
    how much); the engine, in portions and then token by token, agrees with the plain model."""
    cfg, seed = M.ONLY_MLSTM, 18

    def edit(t):
        for key in t:
            if key.endswith("f.b"):
                t[key] = torch.full_like(t[key], 7.0)
    folder = M.make_folder(tmp_path / "mem", cfg, seed, edit=edit)
    plain = M.PlainRelanex(folder)
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
    _check(folder, "float32", {"f": ids}, got, "far token")
    assert H.rel_rms(got[("f", 150)], plain.logits(ids)[150]) < gap / 20


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mlstm", "A"])
def test_long_rows_run_in_pieces(folders, name, dtype, device):
    """Rows long enough for the memory's scan to cut them into pieces that run side by side: a prompt of 700 tokens
    whole, then portions of 300 and 290 beside a short request and a decode row, then the rest token by token."""
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
    folder, page = folders["A-sharp"], 8
    ids = H.random_ids(185, M.CONFIG_A["vocab"], 21)
    rep = _replayer(folder, device, dtype, page, cache_tokens=192)
    got = H.run_trace(rep, H.trace_decode_tail("d", ids, 180))
    _check(folder, dtype, {"d": ids}, got, f"long decoding {dtype}")
    windowed = [g for g in rep.cache.groups if g.decl.window > 0]
    assert windowed and all(g.pool.free == g.pool.usable for g in rep.cache.groups)


def test_configuration_and_weights_are_checked(tmp_path):
    from holon_amd.config.model import ConfigError
    from holon_amd.registry import resolve
    from holon_amd.weights.loader import WeightError
    cfg, spec = resolve(M.CONFIG_A)
    assert [r.layer for r in spec.order] == [0, 1, 2, 1, 2, 1, 2] and cfg.to_dict()["loop"] == M.CONFIG_A["loop"]
    assert [r.layer for r in resolve(M.CONFIG_C)[1].order] == [0, 1, 2]
    assert [r.layer for r in resolve(M.CONFIG_D)[1].order] == [0, 1, 0, 1]
    for bad in (M.variant(M.CONFIG_A, loop={"start": 1, "stop": 1, "times": 2}),
                {k: v for k, v in M.CONFIG_A.items() if k != "residual_mult"},
                M.variant(M.CONFIG_A, layers=[{"type": "conv", "mixer": {}, "mlp": None}]),
                M.variant(M.CONFIG_A, layers=[M.attention(3, 2, 8, 8, 1.0)])):
        with pytest.raises(ConfigError):
            resolve(bad)

    def drop(t):
        del t["l0.mix.sink"]
        t["l2.mix.i.b"] = torch.zeros(5).bfloat16()
    folder = M.make_folder(tmp_path / "bad", M.CONFIG_A, 1, edit=drop)
    from holon_amd.engine.loading import load_model
    with pytest.raises(WeightError) as e:
        load_model(folder, device="cpu", dtype="float32", kernels=TorchKernels(), max_model_len=32, max_seqs=2)
    assert "l0.mix.sink" in str(e.value) and "l2.mix.i.b" in str(e.value)


@pytest.mark.parametrize("device", DEVICES)
def test_random_weights_from_the_command_line_replay(tmp_path, device):
    """`holon_amd random` writes a Relanex folder, and the engine and the plain model agree on it."""
    from holon_amd.cli import main
    (tmp_path / "c.json").write_text(json.dumps(M.CONFIG_A))
    assert main(["random", "--config", str(tmp_path / "c.json"), "--seed", "4", "--out", str(tmp_path / "m")]) == 0
    ids = H.random_ids(30, M.CONFIG_A["vocab"], 2)
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
    folder = folders["B-sharp"]
    plain = _plain(str(folder))
    prompts = [H.random_ids(n, M.CONFIG_B["vocab"], 50 + n) for n in (5, 37, 18, 1)]
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
@pytest.mark.parametrize("name,dtype", [("A-sharp", "float32"), ("A-sharp", "bfloat16"), ("D-sharp", "float32")])
def test_graph_replays_equal_eager_steps(folders, name, dtype):
    """Decode steps replayed from HIP graphs give the tokens of eager steps, over many replays with the program's own
    eager work (prompt steps, sampling, host synchronisation) between them, while the batch shrinks through the
    buckets, pages are taken and given back and windows pass. (On the matrix-core attention path a replayed step cuts
    a row's keys over waves as its length bucket asks, an eager one as the row's length does, so the two differ by
    rounding: that path has the test below.)"""
    from holon_amd.config import EngineConfig, SamplingParams
    from holon_amd.engine.engine import Engine
    vocab = MODELS[name][0]["vocab"]
    prompts = [H.random_ids(n, vocab, 80 + n) for n in (3, 17, 8, 25, 40, 1)]
    outs = {}
    for graphs in (False, True):
        engine = Engine(EngineConfig(model=str(folders[name]), device="cuda", dtype=dtype, page_size=16, max_seqs=6,
                                     max_model_len=160, max_step_tokens=64, graphs=graphs, cache_tokens=960))
        rids = [engine.add(p, SamplingParams(temperature=0.0 if i % 2 else 0.7, seed=5, max_tokens=60 + 7 * i,
                                             ignore_eos=True)) for i, p in enumerate(prompts)]
        got = {r: [] for r in rids}
        while engine.has_work():
            for d in engine.step():
                got[d.rid].extend(d.token_ids)
        outs[graphs] = [got[r] for r in rids]
        engine.cache.check()
        if graphs:
            assert engine.runner.graph_replays > 20 and len(engine.runner.graphs) >= 3
        engine.close()
    assert outs[True] == outs[False]


@pytest.mark.gpu
def test_graph_replays_on_the_matrix_core_path(folders):
    """bfloat16 at head sizes the matrix-core kernels serve (the sink and the window among them): logits of decode
    steps replayed from graphs, two requests side by side and then one alone, against eager steps: as near the plain
    model as they are, and no further from each other than rounding puts them."""
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    folder = folders["D-sharp"]
    vocab = MODELS["D-sharp"][0]["vocab"]
    ids, other = H.random_ids(150, vocab, 7), H.random_ids(90, vocab, 8)
    want = _plain(str(folder)).logits(ids)[20:]
    outs = {}
    for graphs in (False, True):
        rep = Replayer(load_model(folder, device="cuda", dtype="bfloat16", page_size=16, max_seqs=6, max_model_len=160,
                                  max_step_tokens=64, cache_tokens=960, graphs=graphs))
        rep.step([{"id": "a", "tokens": ids[:20], "want": []}, {"id": "b", "tokens": other[:33], "want": []}])
        rows = []
        for p in range(20, 150):
            entries = [{"id": "a", "tokens": [ids[p]], "want": [0]}]
            if 13 + p < 90:
                entries.append({"id": "b", "tokens": [other[13 + p]], "want": [0]})
            rows.append(rep.step(entries)[0].float().cpu().clone())
        outs[graphs] = torch.stack(rows)
        assert rep.runner.graph_replays > 100 if graphs else rep.runner.graph_replays == 0
        assert H.rel_rms(outs[graphs], want) < 0.02
    apart = (outs[True] - outs[False]).square().mean(-1).sqrt() / outs[False].square().mean().sqrt()
    assert apart.max().item() < 0.03


# -- the HIP kernels alone, each against its plain form --------------------------------------------------------------
def _rel(a, b):
    return H.rel_rms(a.float(), b.float())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kernels_against_their_plain_forms(dtype):
    import holon_amd.parts  # noqa: F401  (registers the operations)
    from holon_amd.kernels import load_hip
    from holon_amd.kernels.api import AttnRows
    from holon_amd.kernels.registry import kernel_op
    k, dev = load_hip(), "cuda"
    g = torch.Generator(device=dev).manual_seed(3)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)      # noqa: E731
    tol = 2e-6 if dtype == torch.float32 else 1e-2
    for width in (352, 37):                                       # the norm with both adds; a width that is no multiple of 4
        x, term, extra = rn(19, width), rn(19, width).to(dtype), rn(19, width)
        post, pre = ((torch.rand((), device=dev) + 0.5, rn(width), rn(width)) for _ in range(2))
        x1, x2 = x.clone(), x.clone()
        y1 = k.dyt_stream(x1, term, post, 0.7, extra, pre, dtype)
        y2 = kernel_op("dyt_stream").plain(x2, term, post, 0.7, extra, pre, dtype)
        assert _rel(x1, x2) < 2e-6 and _rel(y1, y2) < tol
    lens, nq = [70, 33, 1, 17], [5, 33, 1, 1]
    for heads, kv, d, v, page, window, sunk in ((8, 2, 64, 40, 16, 0, True), (5, 1, 80, 80, 16, 40, False),
                                                (4, 2, 16, 24, 4, 7, True), (3, 3, 24, 8, 8, 0, False),
                                                (2, 1, 40, 40, 32, 33, True), (2, 2, 12, 20, 3, 5, True)):
        rows_n, most = len(lens), -(-max(lens) // page)
        pages = rn(rows_n * most + 1, kv * page * (d + v)).to(dtype)
        table = torch.full((rows_n + 1, most), rows_n * most, dtype=torch.int32)
        table[:rows_n] = torch.randperm(rows_n * most).view(rows_n, most).int()
        table = table.to(dev)
        qs = [0]
        for n in nq:
            qs.append(qs[-1] + n)
        as_i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)      # noqa: E731
        token_row = as_i32([b for b in range(rows_n) for _ in range(nq[b])])
        positions = as_i32([lens[b] - nq[b] + i for b in range(rows_n) for i in range(nq[b])])
        rows = AttnRows(slots=as_i32(list(range(rows_n))), lens=as_i32(lens), query_start=as_i32(qs), decode_rows=None,
                        chunk_rows=None, n_decode=0, n_chunk=0, max_decode_len=0, max_chunk_query=0, max_chunk_len=0)
        q = (rn(sum(nq), heads, d) * 1.5).to(dtype)
        sink = rn(heads) if sunk else None
        args = (q, pages, table, rows, token_row, positions, kv, v, page, sink, 0.3, window)
        assert _rel(k.softmax_attention(*args), kernel_op("softmax_attention").plain(*args)) < tol
    heads, kv, d, v, page, t = 4, 2, 16, 24, 8, 9                  # biases in the head preparation
    width = (heads + kv) * d + kv * v
    qkv, bias, tab = rn(t, width).to(dtype), rn(width), rn(64, 8)
    pos = torch.arange(t, dtype=torch.int32, device=dev)
    pg1 = torch.zeros(4, kv * page * (d + v), device=dev, dtype=dtype)
    pg2 = pg1.clone()
    q1 = k.head_prepare(qkv, heads, kv, d, v, None, None, 0.0, tab, pos, pg1, pos // page, pos % page, page, bias=bias)
    q2 = kernel_op("head_prepare").plain(qkv, heads, kv, d, v, None, None, 0.0, tab, pos, pg2, pos // page, pos % page,
                                         page, bias=bias)
    assert _rel(q1, q2) < tol and _rel(pg1, pg2) < tol
    for t, heads, a, b in ((1, 5, 40, 112), (8, 16, 128, 256), (16, 3, 96, 72), (5, 2, 24, 7), (40, 4, 64, 56)):
        x, w = rn(t, heads, a).to(dtype), (rn(heads, b, a) * a ** -0.5).to(dtype)      # every head's own projection
        assert _rel(k.head_linear(x, w), kernel_op("head_linear").plain(x.float(), w.float())) < tol
    for q_rank, rank, page in ((80, 112, 16), (24, 40, 8), (768, 256, 16), (7, 5, 4)):       # the two latents' norms
        t = 21
        both, qw, cw = rn(t, q_rank + rank).to(dtype), (1 + 0.1 * rn(q_rank)).to(dtype), (1 + 0.1 * rn(rank)).to(dtype)
        pos = torch.arange(t, dtype=torch.int32, device=dev)
        pg1 = torch.zeros((t + 3) // page + 1, 2 * page * rank, device=dev, dtype=dtype)      # every token's page exists
        pg2 = pg1.clone()
        wp, wo = (pos + 3) // page, (pos + 3) % page
        c1 = k.latent_prepare(both, q_rank, qw, cw, 1e-6, pg1, wp, wo, page)
        c2 = kernel_op("latent_prepare").plain(both, q_rank, qw, cw, 1e-6, pg2, wp, wo, page)
        assert _rel(c1, c2) < tol and _rel(pg1, pg2) < tol
    for heads, d, v in ((4, 40, 56), (2, 16, 40), (3, 64, 8), (1, 128, 20), (2, 200, 16)):     # the memory's scan
        hd, hv, copies = heads * d, heads * v, -(-(v + 1) // 8)
        width = -(-(2 * hd + 2 * hv + 2 * heads) // 16) * 16
        proj = rn(43, width).to(dtype)
        proj[:, 2 * hd + 2 * hv:] *= 3
        gb = rn(2 * heads)
        state = [rn(5, heads, d, v + 1), rn(5, heads, 1).expand(5, heads, copies).contiguous()]
        st1, st2 = [s.clone() for s in state], [s.clone() for s in state]
        rows = (torch.tensor([3, 0, 4], dtype=torch.int32, device=dev), torch.tensor([0, 9, 2], dtype=torch.int32, device=dev),
                torch.tensor([0, 37, 38, 43], dtype=torch.int32, device=dev))
        o1, u1 = k.mlstm_scan(proj, 0, hd, 2 * hd, 2 * hd + 2 * hv, gb, 12.0, *st1, *rows, 3, heads, d, v)
        o2, u2 = kernel_op("mlstm_scan").plain(proj, 0, hd, 2 * hd, 2 * hd + 2 * hv, gb, 12.0, *st2, *rows, 3, heads, d, v)
        assert _rel(o1, o2) < 1e-5 and _rel(u1, u2) < 1e-5 and all(_rel(a, b) < 1e-5 for a, b in zip(st1, st2))
        # long rows in pieces of 128 tokens: a row of 700 from a carried state, one of 300 from zero, a decode row
        long = rn(1001, width).to(dtype)
        long[:, 2 * hd + 2 * hv:] *= 3
        rows = (torch.tensor([1, 2, 0], dtype=torch.int32, device=dev), torch.tensor([5, 0, 77], dtype=torch.int32, device=dev),
                torch.tensor([0, 700, 1000, 1001], dtype=torch.int32, device=dev))
        cut = (128, 6, torch.tensor([0, 6, 9], dtype=torch.int32, device=dev), 10)
        st3, st4 = [s.clone() for s in state], [s.clone() for s in state]
        o3, u3 = k.mlstm_scan(long, 0, hd, 2 * hd, 2 * hd + 2 * hv, gb, 12.0, *st3, *rows, 3, heads, d, v, cut)
        o4, u4 = kernel_op("mlstm_scan").plain(long, 0, hd, 2 * hd, 2 * hd + 2 * hv, gb, 12.0, *st4, *rows, 3, heads, d, v)
        assert _rel(o3 / u3[..., None], o4 / u4[..., None]) < 2e-5 and all(_rel(a, b) < 2e-5 for a, b in zip(st3, st4))
        gate, wn = proj[:, 2 * hd + hv: 2 * hd + 2 * hv], rn(hv).to(dtype)
        assert _rel(k.gated_out(o1, gate, wn, True, 1e-6, dtype, act="sigmoid", den=u1),
                    kernel_op("gated_out").plain(o1, gate, wn, True, 1e-6, dtype, act="sigmoid", den=u1)) < tol


@pytest.mark.gpu
@pytest.mark.parametrize("d,heads,kv,window", [(64, 8, 2, 0), (128, 16, 4, 100), (128, 8, 8, 0), (256, 16, 1, 333),
                                               (64, 40, 1, 0)])
def test_the_sink_on_the_matrix_cores(d, heads, kv, window):
    """`paged_attention` with a sink in bfloat16 at the head sizes the matrix-core kernels serve: long and short
    prompt portions and decode rows of several lengths in one step, against the plain form."""
    from holon_amd.kernels import load_hip
    from holon_amd.kernels.api import AttnRows
    k, dev, page = load_hip(), "cuda", 16
    g = torch.Generator(device=dev).manual_seed(d + heads)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)      # noqa: E731
    lens, nq = [700, 40, 900, 33, 1], [300, 5, 1, 1, 1]
    most = -(-max(lens) // page)
    n_rows = len(lens)
    pages = rn(n_rows * most + 1, 2, kv, page * d).bfloat16()
    table = torch.full((n_rows + 1, most), n_rows * most, dtype=torch.int32)
    table[:n_rows] = torch.randperm(n_rows * most).view(n_rows, most).int()
    table = table.to(dev)
    qs = [0]
    for n in nq:
        qs.append(qs[-1] + n)
    as_i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)      # noqa: E731
    rows = AttnRows(slots=as_i32(list(range(n_rows))), lens=as_i32(lens), query_start=as_i32(qs),
                    decode_rows=as_i32([2, 3, 4]), chunk_rows=as_i32([0, 1]), n_decode=3, n_chunk=2, max_decode_len=900,
                    max_chunk_query=300, max_chunk_len=700)
    q = rn(sum(nq), heads, d).bfloat16()
    scale = 2.0 * d ** -0.5
    sink = 2.0 * rn(heads) + 2.0
    for with_sink in (sink, None):
        got = k.paged_attention(q, pages, table, rows, page, scale, window, sink=with_sink)
        want = TorchKernels().paged_attention(q.float(), pages.float(), table, rows, page, scale, window, sink=with_sink)
        assert H.rel_rms(got.float(), want) < 1e-2, (d, heads, kv, window, with_sink is not None)
    assert H.rel_rms(k.paged_attention(q, pages, table, rows, page, scale, window, sink=sink).float(),
                     k.paged_attention(q, pages, table, rows, page, scale, window).float()) > 0.05      # the sink shows


@pytest.mark.gpu
def test_trace_runner_as_a_program(folders, tmp_path):
    """bin/trace_run on a Relanex folder, as a user runs it."""
    import numpy as np
    folder, requests = folders["A"], _requests("A", (30, 19))
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
