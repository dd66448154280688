"""Dopirax through the engine against the plain model (`tests/plain/dopirax.py`, written from the design's equations,
no cache, float64): every mechanism alone, every way of cutting a prompt, batches, reused pages and slots, far keys and
keys at page borders, the first tokens of a sequence (where the one in the softmax's denominator weighs most), layers
that read another layer's keys and values, the router's choice, long decoding, sizes that are 1 or equal, and greedy
generation through the engine's own entry point. On the CPU the plain twins of the operations stand in for the HIP
kernels (this checks configuration, weights, cache, state and batching); the `gpu` cases run the HIP kernels, each also
alone against its twin."""
from __future__ import annotations

import functools
import json
import pathlib

import pytest
import torch

from tests import dopirax_models as M
from tests import helpers as H
from tests.plain import dopirax as plain
from tests.plain.ops import TorchKernels

DEVICES = [pytest.param("cpu", id="cpu-twin"), pytest.param("cuda", marks=pytest.mark.gpu, id="hip")]
DTYPES = ["float32", "bfloat16"]
MODELS = {"A": (M.CONFIG_A, 11, False, 8), "B": (M.CONFIG_B, 12, False, 16), "C": (M.CONFIG_C, 13, False, 4),
          "A-sharp": (M.CONFIG_A, 14, True, 16), "B-sharp": (M.CONFIG_B, 15, True, 8), "D-sharp": (M.CONFIG_D, 20, True, 16),
          "attention": (M.ONLY_ATTENTION, 16, True, 8), "diff": (M.ONLY_DIFF, 17, True, 8),
          "dense": (M.ONLY_DENSE, 18, False, 8), "moe": (M.ONLY_MOE, 19, False, 8)}
LENGTHS = (40, 70, 33, 58, 50, 64, 21)
# bfloat16 engine against the float64 plain model, relative rms of the logits: what rounding alone gives on these
# models stays well below this; a lost key, a missing sink, gate or expert is far above it on the sharp models.
BF16_RMS = 0.08


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("dopirax")
    return {name: M.make_folder(root / name, cfg, seed, sharp) for name, (cfg, seed, sharp, _) in MODELS.items()}


@functools.lru_cache(maxsize=None)
def _plain(folder: str) -> M.PlainDopirax:
    return M.PlainDopirax(folder)


def _requests(name: str, lengths=LENGTHS) -> dict[str, list[int]]:
    return {f"r{i}": H.random_ids(n, MODELS[name][0]["vocab"], 300 + i) for i, n in enumerate(lengths)}


def _replayer(folder, device, dtype, page, cache_tokens, max_seqs=4, max_model_len=256, kernels=None):
    from holon_amd.engine.loading import load_model
    from holon_amd.engine.replay import Replayer
    if kernels is None and device == "cpu":
        kernels = TorchKernels()
    loaded = load_model(folder, device=device, dtype=dtype, kernels=kernels, page_size=page, max_seqs=max_seqs,
                        max_model_len=max_model_len, max_step_tokens=max_model_len, cache_tokens=cache_tokens)
    return Replayer(loaded)


def _check(folder, dtype, requests, got, what):
    folder = pathlib.Path(folder)
    want = {r: _plain(str(folder)).logits(ids) for r, ids in requests.items()}
    g, w = H.gather(want, got)
    assert torch.isfinite(g).all(), f"{what}: non-finite logits"
    if dtype == "float32":
        r, m = H.rel_rms(g, w), H.max_over_rms(g, w)
        assert r <= 3e-5 and m <= 3e-4, f"{what}: float32 logits differ: rms {r:.3g}, max {m:.3g}"
    else:
        # In bfloat16 a router's close call may fall the other way (its input is rounded), and the position then has
        # another expert's output: the float32 runs hold the choice itself, and here the worst 4 % of positions are
        # set aside for every routed feed-forward a token passes. What a lost key or state does to one position is
        # held by the tests that place it, on models without experts.
        config = json.loads((folder / "config.json").read_text())
        routed = sum((layer.get("mlp") or {}).get("kind") == "moe" for layer in config["layers"])
        per = (g - w).square().mean(-1).sqrt() / w.square().mean().sqrt()
        if routed:
            per = per.sort().values[: len(per) - int(len(per) * min(0.04 * routed, 0.3)) - 1]
        r = per.square().mean().sqrt().item()
        assert r <= BF16_RMS, f"{what}: bfloat16 logits differ: rms {r:.3g}"
        assert per.max().item() <= 3 * BF16_RMS, f"{what}: one position differs by {per.max().item():.3g}"


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
    """Where keys and values have one width that the matrix-core attention kernels serve, both mixers hand their pages
    to `paged_attention` (the cap and the sink of one; the two maps over doubled values); the twin is told to say it
    serves them, and the logits stay the plain model's."""
    folder, requests = folders["D-sharp"], _requests("D-sharp", (70, 33, 58))
    kernels = TorchKernels()
    kernels.cores = True
    rep = _replayer(folder, "cpu", "float32", 16, cache_tokens=192, max_seqs=3, max_model_len=128, kernels=kernels)
    got = H.run_trace(rep, H.trace_mixed(requests, seed=2, max_live=3, decode_tail=5))
    _check(folder, "float32", requests, got, "matrix-core path on the twin")


@pytest.mark.parametrize("device", DEVICES)
def test_the_stream_after_every_layer(folders, device):
    """The residual stream after each layer, float32, against the plain model's: the block's pending terms added to
    its rows."""
    from holon_amd.engine.batch import StepRow
    from holon_amd.parts.base import Stream
    from holon_amd.parts.stream32 import _terms
    folder = folders["A"]
    ids = H.random_ids(37, M.CONFIG_A["vocab"], 3)
    rep = _replayer(folder, device, "float32", 8, cache_tokens=40)
    slot = rep.cache.admit()
    rep.cache.reserve(slot, len(ids))
    step, _ = rep.runner.prepare([StepRow(slot, 0, ids, [])])
    model = rep.loaded.model
    stream = Stream(model.embed(step.token_ids, step.token_take))
    want = _plain(str(folder)).streams(ids)
    assert len(want) == len(model.sites) == 5
    for site, ref in zip(model.sites, want):
        stream = model.blocks[site.layer](stream, step, site)
        x = stream.h.clone()
        for term, scale in _terms(stream.delta):
            x += scale * term.float()
        if stream.delta.row is not None:           # an output bias that waits for the same add
            x += stream.delta.row
        assert H.rel_rms(x.cpu(), ref) < 2e-5, f"layer {site.layer}"


def _needle(root, kind, dim, key_at, query_at, rot=None):
    """One layer of one mixer, no feed-forward. A pair of token ids (query token, key token) whose score, with the key
    at position `key_at` and the query at `query_at`, is the largest of all pairs', and a filler token whose scores
    with them and with itself are low; the query side is scaled until the pair's weight among hundreds of fillers is
    nearly all of it. Returns the folder and the three ids. (Heads of 64 with keys and values of one width take the
    matrix-core kernels in bfloat16 on the GPU.)"""
    rot = rot if rot is not None else dim // 2
    if kind == "attention":
        cfg = M.model(32, 40, [M.attention(2, 1, dim, 0.25, rot=rot, base=30.0)])
    else:
        cfg = M.model(32, 40, [M.attention_2(2, 1, dim, dim if dim == 64 else 8, 0.25, 0.3, rot=rot, base=30.0)])
    found = {}

    def edit(t):
        p = {k: v.double() for k, v in t.items()}
        a_in = plain.unit(p["embed"] * 2.0, 1e-6) * (1 + p["l0.norm1"])       # every token's mixer input
        n = a_in.shape[0]
        m = cfg["layers"][0]["mixer"]
        if kind == "attention":
            q = (a_in @ p["l0.mix.q"].T + p["l0.mix.q.b"]).view(n, 2, dim)[:, 0]
            k = (a_in @ p["l0.mix.k"].T + p["l0.mix.k.b"]).view(n, dim)
            turn = plain.turn_halves
        else:
            q = (plain.unit((a_in @ p["l0.mix.q"].T).view(n, 2, 2, dim), 1e-6) * p["l0.mix.q.norm"])[:, 0, 0]
            k = (plain.unit((a_in @ p["l0.mix.k"].T).view(n, 1, 2, dim), 1e-6) * p["l0.mix.k.norm"])[:, 0, 0]
            turn = plain.turn_neighbours
        # head 0 (its first map): every token's query at the query's place, every token's key at every place before it
        places = query_at + 1
        q_at = turn(q[None].expand(places, n, dim), 30.0, rot)[query_at]                       # [token, dim]
        k_at = turn(k[None].expand(places, n, dim), 30.0, rot)                                 # [place, token, dim]
        score = torch.einsum("ad,pbd->abp", q_at, k_at) * m["scale"]                           # [query token, key token, place]
        a, b = divmod(int(score[:, :, key_at].argmax()), n)
        worst = score[a].amax(-1)                       # a token's highest score with the query, wherever it stands
        worst[a] = worst[b] = float("inf")
        filler = int(worst.argmin())
        gain = 12.0 / max(float(score[a, b, key_at] - worst[filler]), 1e-3)      # the pair stands e^12 above any filler
        key = "l0.mix.q" if kind == "attention" else "l0.mix.q.norm"
        t[key] = (p[key] * gain).bfloat16()
        if kind == "attention":
            t["l0.mix.q.b"] = (p["l0.mix.q.b"] * gain).bfloat16()
            t["l0.mix.g"] = (p["l0.mix.g"] * 0.0).bfloat16()                     # every head passes half of its result
        found.update(a=a, b=b, filler=filler)
    folder = M.make_folder(root, cfg, 77, edit=edit)
    return folder, found["a"], found["b"], found["filler"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind,dim,page,key_at", [("attention", 16, 8, 7), ("attention", 16, 16, 16), ("attention", 64, 16, 35),
                                                  ("attention_2", 16, 8, 8), ("attention_2", 16, 16, 15),
                                                  ("attention_2", 64, 16, 32)])
def test_a_far_key_at_a_page_border(tmp_path, kind, dim, page, key_at, dtype, device):
    """One key 300 tokens behind the query, the last of a page, the first of one or inside one, whose score stands out
    among hundreds: it carries the result in a whole prompt, in a prompt cut into portions (down to two tokens, the
    query in one of them), and when the query is decoded alone; without it the logits are far away."""
    query_at = key_at + 300
    folder, a, b, filler = _needle(tmp_path / "needle", kind, dim, key_at, query_at)
    plain_model = M.PlainDopirax(folder)
    ids = [filler] * key_at + [b] + [filler] * (query_at - key_at - 1) + [a, filler]
    without = [filler] * query_at + [a, filler]
    gap = H.rel_rms(plain_model.logits(ids)[query_at], plain_model.logits(without)[query_at])
    assert gap > 0.1, f"the far key does not show: {gap}"
    rep = _replayer(folder, device, dtype, page, cache_tokens=-(-len(ids) // page) * page, max_model_len=352)
    tol = gap / 8
    got = H.run_trace(rep, H.trace_whole({"f": ids}))
    _check(folder, dtype, {"f": ids}, got, "far key, whole")
    assert H.rel_rms(got[("f", query_at)], plain_model.logits(ids)[query_at]) < tol
    got = H.run_trace(rep, H.trace_chunks("f", ids, [150, 2, 97, query_at - 249 - 1, 2]))
    assert H.rel_rms(got[("f", query_at)], plain_model.logits(ids)[query_at]) < tol, "a portion of two"
    got = H.run_trace(rep, H.trace_decode_tail("f", ids, 3))
    _check(folder, dtype, {"f": ids}, got, "far key, decoded")
    assert H.rel_rms(got[("f", query_at)], plain_model.logits(ids)[query_at]) < tol, "decoded alone"
    got = H.run_trace(rep, H.trace_whole({"g": without}))
    assert H.rel_rms(got[("g", query_at)], plain_model.logits(without)[query_at]) < tol
    rep.cache.check()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_the_one_in_the_denominator(folders, tmp_path, dtype, device):
    """The softmax whose denominator holds one more term, exp(0): on the first tokens of a sequence (where it weighs most) and
    behind scores pushed far below zero (where it takes nearly everything), the plain model with and without it are far
    apart and the engine follows the one with it."""
    cfg, seed, sharp, page = MODELS["attention"]

    def low(t):                                    # a key bias against the query bias: every score far below zero
        for i, layer in enumerate(cfg["layers"]):
            m = layer["mixer"]
            t[f"l{i}.mix.q.b"] = torch.full((m["heads"] * m["dim"],), 1.5).bfloat16()
            t[f"l{i}.mix.k.b"] = torch.full((m["kv_heads"] * m["dim"],), -1.5).bfloat16()
        for i in range(len(cfg["layers"])):
            rot = cfg["layers"][i]["mixer"]["rot"]["dims"]
            d = cfg["layers"][i]["mixer"]["dim"]
            for name, heads in (("q", cfg["layers"][i]["mixer"]["heads"]), ("k", cfg["layers"][i]["mixer"]["kv_heads"])):
                b = t[f"l{i}.mix.{name}.b"].view(heads, d).clone()
                b[:, :rot] = 0                     # the turned dimensions carry no bias: the scores stay low at any distance
                t[f"l{i}.mix.{name}.b"] = b.reshape(-1)
    for what, folder in (("first tokens", folders["attention"]),
                         ("low scores", M.make_folder(tmp_path / "low", cfg, seed, False, edit=low))):
        with_one, without = M.PlainDopirax(folder), M.PlainDopirax(folder, sink=False)
        ids = H.random_ids(6 if what == "first tokens" else 45, cfg["vocab"], 8)
        gap = H.rel_rms(without.logits(ids), with_one.logits(ids))
        assert gap > 0.05, f"{what}: the one in the denominator does not show: {gap}"
        rep = _replayer(folder, device, dtype, page, cache_tokens=64)
        for trace in (H.trace_whole({"s": ids}), H.trace_decode_tail("s", ids, len(ids) - 1)):
            got = H.run_trace(rep, trace)
            g, w = H.gather({"s": with_one.logits(ids)}, got)
            assert H.rel_rms(g, w) < (gap / 100 if dtype == "float32" else min(gap / 3, BF16_RMS)), what


@pytest.mark.parametrize("device", DEVICES)
def test_each_mechanism_shows(folders, tmp_path, device):
    """The cap, the gate, the biases, the rotation of either pairing, the vectors behind lam, the shared expert's gate
    and the router's bias each move the plain model's logits far more than the engine differs from it: a mechanism
    left out or mistaken would not pass the other tests."""
    ids = H.random_ids(60, 90, 4)
    flip = lambda t: t.flip(-1)                    # noqa: E731
    cases = [("attention", "l0.mix.g", lambda t: t * 0.0), ("attention", "l0.mix.o.b", lambda t: t * 0.0),
             ("attention", "l0.mix.k.b", lambda t: t * 0.0), ("attention", "l0.mix.q.b", lambda t: -t),
             ("diff", "l0.mix.lq1", lambda t: t + 0.5), ("diff", "l0.mix.lk2", lambda t: -t),
             ("diff", "l1.mix.q.norm", flip), ("diff", "l0.mix.k.norm", flip), ("diff", "l0.mix.v", lambda t: t.flip(0)),
             ("moe", "l0.mlp.shared.sg", lambda t: -t), ("moe", "l0.mlp.router.b", lambda t: t.flip(0))]
    for name, key, change in cases:
        base = _plain(str(folders[name]))
        cfg, seed, sharp, page = MODELS[name]

        def edit(t, key=key, change=change):
            t[key] = change(t[key].float()).bfloat16()
        other = M.PlainDopirax(M.make_folder(tmp_path / f"{name}-{key}", cfg, seed, sharp, edit=edit))
        gap = H.rel_rms(other.logits(ids), base.logits(ids))
        rep = _replayer(folders[name], device, "float32", page, cache_tokens=64)
        got = H.run_trace(rep, H.trace_chunks("x", ids, [23, 2, 9]))
        g, w = H.gather({"x": base.logits(ids)}, got)
        assert gap > 1e-2 and H.rel_rms(g, w) < gap / 100, f"{name} {key}: gap {gap}"
    for name, layer, key, value in (("attention", 0, "softcap", 400.0), ("attention", 0, "rot", {"dims": 2, "base": 10000.0}),
                                    ("diff", 2, "rot", {"dims": 2, "base": 10000.0}), ("diff", 0, "diff", 0.1)):
        changed = M.variant(MODELS[name][0])
        changed["layers"][layer]["mixer"][key] = value
        if name == "diff" and layer == 0:
            changed["layers"][1]["mixer"][key] = value
        other = M.PlainDopirax(M.make_folder(tmp_path / f"{name}-{key}-{layer}", changed, MODELS[name][1], True))
        assert H.rel_rms(other.logits(ids), _plain(str(folders[name])).logits(ids)) > 1e-2, (name, key)


@pytest.mark.parametrize("device", DEVICES)
def test_the_router_chooses_as_the_plain_model(device):
    """The router's weights on their own: the largest logits after the bias (which reorders them), equal logits to the
    lower index, weights the softmax over the chosen alone, and the shared expert's gate in the last column."""
    import holon_amd.parts  # noqa: F401
    from holon_amd.kernels.registry import kernel_op
    if device == "cuda":
        from holon_amd.kernels import load_hip
        router_top = load_hip().moe_router_top
    else:
        router_top = kernel_op("moe_router_top").plain
    g = torch.Generator().manual_seed(3)
    for experts, top, width, gated in ((8, 3, 64, True), (12, 4, 250, False), (6, 6, 32, True), (16, 1, 100, True), (1, 1, 8, True),
                                       (64, 6, 512, False), (130, 9, 48, True)):
        x = torch.randn(50, width, generator=g).to(device)
        router = (2.0 * torch.randn(experts + int(gated), width, generator=g) * width ** -0.5).to(device)
        router[1] = router[0]                      # two experts with equal logits (their biases are made equal below)
        bias = torch.randn(experts, generator=g).to(device) * 1.5
        if experts > 1:
            bias[1] = bias[0]
        got = router_top(x, router, bias, experts, top).cpu().double()
        z = x.double().cpu() @ router.double().cpu().T
        for t in range(50):
            want = torch.zeros(experts + int(gated), dtype=torch.float64)
            for e, weight in plain.route(z[t, :experts] + bias.double().cpu(), top):
                want[e] = weight
            if gated:
                want[experts] = torch.sigmoid(z[t, experts])
            close = sorted((z[t, :experts] + bias.double().cpu()).tolist(), reverse=True)
            if top < experts and experts > 2 and close[top - 1] - close[top] < 1e-5 and close[top - 1] != close[top]:
                continue                           # a call that float32 cannot make
            assert torch.allclose(got[t], want, atol=2e-6), (experts, top, t)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(folders, dtype, device):
    """180 tokens one by one after a prompt of 5, over many pages, through layers that write a cache and layers that
    read another's."""
    folder, page = folders["A-sharp"], 8
    ids = H.random_ids(185, M.CONFIG_A["vocab"], 21)
    rep = _replayer(folder, device, dtype, page, cache_tokens=192)
    trace = H.trace_decode_tail("d", ids, 180)
    trace.steps[-1]["end"] = []
    got = H.run_trace(rep, trace)
    _check(folder, dtype, {"d": ids}, got, f"long decoding {dtype}")
    assert len(rep.cache.groups) >= 1 and sum(len(d) for d in rep.loaded.model.state_decls()) == 3   # two layers keep none
    rep.cache.check()
    rep.step([], ["d"])
    assert all(g.pool.free == g.pool.usable for g in rep.cache.groups)


def test_configuration_and_weights_are_checked(tmp_path):
    from holon_amd.config.model import ConfigError
    from holon_amd.registry import resolve
    from holon_amd.weights.loader import WeightError
    cfg, spec = resolve(M.CONFIG_A)
    assert [(r.layer, r.reads) for r in spec.order] == [(0, None), (1, None), (2, 1), (3, None), (4, 1)]
    assert cfg.to_dict()["layers"] == M.CONFIG_A["layers"]
    bare = M.variant(M.CONFIG_A)                                # sizes a configuration may leave to the design
    del bare["layers"][0]["mixer"]["vdim"], bare["layers"][3]["mixer"]["kv_heads"]
    assert resolve(bare)[0].to_dict()["layers"] == M.CONFIG_A["layers"] and "vdim" not in bare["layers"][0]["mixer"]
    late = M.variant(M.CONFIG_A)
    late["layers"][2]["mixer"]["kv_from"] = 3                   # an attention layer, and not an earlier one
    chain = M.variant(M.CONFIG_A)
    chain["layers"][4]["mixer"]["kv_from"] = 2                  # a layer that has no keys of its own
    other_heads = M.variant(M.CONFIG_A)
    other_heads["layers"][2]["mixer"]["kv_heads"] = 1
    wide_values = M.variant(M.CONFIG_A)
    wide_values["layers"][0]["mixer"]["vdim"] = 24
    bad_rot = M.variant(M.CONFIG_A)
    bad_rot["layers"][0]["mixer"]["rot"]["dims"] = 7
    bad_top = M.variant(M.CONFIG_A)
    bad_top["layers"][0]["mlp"]["router"]["top"] = 9
    for bad in ({k: v for k, v in M.CONFIG_A.items() if k != "norm"},
                M.variant(M.CONFIG_A, layers=[{"type": "conv", "mixer": {}, "mlp": None}]),
                M.variant(M.CONFIG_A, layers=[M.attention(3, 2, 8, 1.0)]), late, chain, other_heads, wide_values, bad_rot,
                bad_top):
        with pytest.raises(ConfigError):
            resolve(bad)

    def drop(t):
        del t["l0.mix.g"]
        t["l0.mlp.router.b"] = torch.zeros(5).bfloat16()
        t["l2.mix.k"] = torch.zeros(32, 64).bfloat16()           # a layer that reads another's keys has none
    folder = M.make_folder(tmp_path / "bad", M.CONFIG_A, 1, edit=drop)
    from holon_amd.engine.loading import load_model
    with pytest.raises(WeightError) as e:
        load_model(folder, device="cpu", dtype="float32", kernels=TorchKernels(), max_model_len=32, max_seqs=2)
    assert "l0.mix.g" in str(e.value) and "l0.mlp.router.b" in str(e.value) and "l2.mix.k" in str(e.value)


@pytest.mark.parametrize("device", DEVICES)
def test_random_weights_from_the_command_line_replay(tmp_path, device):
    """`holon_amd random` writes a Dopirax folder, and the engine and the plain model agree on it."""
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
    plain_model = _plain(str(folder))
    prompts = [H.random_ids(n, M.CONFIG_B["vocab"], 50 + n) for n in (5, 37, 18, 1)]
    cfg = EngineConfig(model=str(folder), device=device, dtype=dtype, page_size=8, max_seqs=3, max_model_len=96,
                       max_step_tokens=40, chunk_with_decode=16, cache_tokens=192)
    engine = Engine(cfg, TorchKernels() if device == "cpu" else None)
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True))
    held = sum(H.assert_greedy_follows(plain_model, p, o, margin=0.02 if dtype == "float32" else 0.25)
               for p, o in zip(prompts, outs))
    assert all(len(o) == 24 for o in outs) and held >= (60 if dtype == "float32" else 20)
    engine.cache.check()
    engine.close()


@pytest.mark.gpu
@pytest.mark.parametrize("name,dtype", [("A-sharp", "float32"), ("A-sharp", "bfloat16"), ("D-sharp", "float32")])
def test_graph_replays_equal_eager_steps(folders, name, dtype):
    """Decode steps replayed from HIP graphs give the tokens of eager steps, over many replays with the program's own
    eager work (prompt steps, sampling, host synchronisation) between them, while the batch shrinks through the
    buckets and pages are taken and given back."""
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
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kernels_alone_against_their_plain_forms(dtype):
    """Every operation the design brought or changed, on the GPU, against its plain form in torch."""
    import holon_amd.parts  # noqa: F401
    from holon_amd.kernels import load_hip
    from holon_amd.kernels.registry import kernel_op
    from holon_amd.parts.positions import rope_table
    k, dev = load_hip(), "cuda"
    tol = 2e-6 if dtype == torch.float32 else 6e-3
    g = torch.Generator().manual_seed(0)

    def randn(*shape, to=dtype):
        return torch.randn(*shape, generator=g).to(dev).to(to)
    for dim in (96, 250, 1500):                    # the norm with a float32 weight and a result in the engine's dtype
        x, t1, t2 = randn(7, dim, to=torch.float32), randn(7, dim), randn(7, dim)
        w1 = 1 + 0.3 * randn(dim, to=torch.float32)
        xa, xb = x.clone(), x.clone()
        a = k.stream_rms(xa, [(t1, 1.0), (t2, 1.0)], None, w1, None, 1e-6, dtype)
        b = kernel_op("stream_rms").plain(xb, [(t1, 1.0), (t2, 1.0)], None, w1, None, 1e-6, dtype)
        assert H.rel_rms(xa, xb) < 1e-6 and H.rel_rms(a[0], b[0]) < tol and a[1] is None, dim
    for n in (5, 77 * 3, 4096 * 9):
        z = randn(n // 1 if n < 100 else n // 3, 1 if n < 100 else 3)
        assert H.rel_rms(k.relu2(z), kernel_op("relu2").plain(z)) < tol
    if dtype == torch.bfloat16:                    # the activation in the few-row product's epilogue
        for m, n, kk in ((1, 64, 256), (8, 320, 512), (16, 2048, 1024), (5, 48, 288)):
            x, w = randn(m, kk), randn(n, kk) * kk ** -0.5
            tiled = k.tile_weight(w)
            for copy in (None, tiled):
                fused = k.linear_relu2(x, w, copy)
                assert fused is not None and H.rel_rms(fused, k.relu2(k.linear(x, w, None, copy))) < 1e-6, (m, n, kk)
        assert k.linear_relu2(randn(17, 256), randn(64, 256), None) is None
    for heads, vdim, extra in ((4, 24, 16), (3, 64, 5), (16, 128, 0)):
        x, wide = randn(9, heads * vdim), randn(9, 40 + heads + extra)
        gates = wide[:, 40: 40 + heads]
        a, b = x.clone(), x.clone()
        k.head_gate(a, gates, heads)
        kernel_op("head_gate").plain(b, gates, heads)
        assert H.rel_rms(a, b) < tol, (heads, vdim)
    for dim in (33, 320, 5000):
        x, bias = randn(6, dim), randn(dim, to=torch.float32)
        a, b = x.clone(), x.clone()
        k.add_bias(a, bias)
        kernel_op("add_bias").plain(b, bias)
        assert H.rel_rms(a, b) < tol, dim
    for heads, groups, vdim in ((4, 2, 12), (3, 3, 64), (8, 1, 100), (1, 1, 2)):
        y = randn(11, 2 * heads * vdim)
        a = k.diff_combine(y, heads, groups, vdim, 0.37, 1e-6, 0.6)
        assert H.rel_rms(a, kernel_op("diff_combine").plain(y, heads, groups, vdim, 0.37, 1e-6, 0.6)) < tol, (heads, vdim)
    for experts, ff, shared in ((6, 24, 40), (3, 8, 16)):
        gate_up = randn(9, 2 * (experts * ff + shared))
        weights = kernel_op("moe_router_top").plain(randn(9, 32, to=torch.float32), randn(experts + 1, 32, to=torch.float32),
                                                    None, experts, 2)
        a = k.moe_gate(gate_up, weights, ff, shared, shared_weight=True)
        assert H.rel_rms(a, kernel_op("moe_gate").plain(gate_up, weights, ff, shared, shared_weight=True)) < tol
        a = k.moe_gate(gate_up, weights[:, :experts].contiguous(), ff, shared)
        assert H.rel_rms(a, kernel_op("moe_gate").plain(gate_up, weights[:, :experts].contiguous(), ff, shared)) < tol
    for experts, top, width, rows in ((8, 3, 256, 9), (12, 4, 250, 12), (64, 6, 2048, 65), (5, 1, 77, 5), (1, 1, 16, 2),
                                      (100, 7, 320, 101), (300, 2, 96, 300), (17, 17, 1024, 18)):
        x, router = randn(19, width), randn(rows, width, to=torch.float32) * 0.2
        bias = randn(experts, to=torch.float32) * 0.5
        got = k.moe_router_top(x, router, bias, experts, top)
        want = kernel_op("moe_router_top").plain(x, router, bias, experts, top)
        close = ((got != 0) != (want != 0)).any(1)            # rows whose choice fell the other way on a close call
        assert close.sum() <= 1 and torch.allclose(got[~close], want[~close], atol=2e-5), (experts, width)
    # a paged cache of three rows over scattered pages: every way `head_prepare` takes its values
    page, n_pages = 16, 40
    lens = [70, 33, 150]
    table = torch.full((4, 12), n_pages - 1, dtype=torch.int32)
    order, at = torch.randperm(n_pages - 1, generator=g).tolist(), 0
    for s, n in enumerate(lens):
        for i in range(-(-n // page)):
            table[s, i] = order[at]
            at += 1
    table = table.to(dev)
    token_row = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, n in enumerate(lens)]).to(dev)
    positions = torch.cat([torch.arange(n, dtype=torch.int32) for n in lens]).to(dev)
    write_page = table[token_row.long(), (positions // page).long()].contiguous()
    write_off = (positions % page).to(torch.int32)
    total = sum(lens)
    prepare = kernel_op("head_prepare").plain
    for heads, groups, dim, vdim, rot, values, share, extra, normed, biased in (
            (4, 2, 24, 24, 12, "keys", 1, 16, False, True), (6, 4, 16, 40, 8, "own", 2, 0, True, False),
            (4, 2, 64, 64, 64, "own", 2, 3, True, False), (3, 3, 8, 8, 0, "keys", 1, 0, False, False),
            (4, 4, 16, 12, 16, "own", 1, 0, True, True)):
        shared = groups // share if values == "own" else 0
        width = (heads + groups) * dim + shared * vdim
        qkv = randn(total, width + extra)
        tab = rope_table(256, rot, 1000.0).to(dev) if rot else None
        qw = (1 + 0.2 * randn(dim, to=torch.float32)).to(dtype) if normed else None
        kw = (1 + 0.2 * randn(dim, to=torch.float32)).to(dtype) if normed else None
        bias = randn(width, to=torch.float32) if biased else None
        pa = torch.zeros(n_pages, groups * page * dim + (shared or groups) * page * vdim, device=dev, dtype=dtype)
        pb = pa.clone()
        args = (heads, groups, dim, vdim, qw, kw, 1e-6, tab, positions)
        qa = k.head_prepare(qkv, *args, pa, write_page, write_off, page, bias=bias, values=values, value_share=share)
        qb = prepare(qkv, *args, pb, write_page, write_off, page, bias=bias, values=values, value_share=share)
        assert H.rel_rms(qa, qb) < tol and H.rel_rms(pa, pb) < tol, (heads, groups, dim, values)
        only_q = qkv[:, : heads * dim].contiguous()
        qa = k.head_prepare(only_q, heads, 0, dim, vdim, qw, kw, 1e-6, tab, positions, None, None, None, page,
                            bias=None if bias is None else bias[: heads * dim].contiguous())
        qc = prepare(only_q, heads, 0, dim, vdim, qw, kw, 1e-6, tab, positions, None, None, None, page,
                     bias=None if bias is None else bias[: heads * dim].contiguous())
        assert H.rel_rms(qa, qc) < tol and torch.equal(qc, qb), "queries alone"


@pytest.mark.parametrize("device", DEVICES)
def test_a_shared_prefix_through_the_engine(folders, device):
    """Every layer's state lies in pages without a window, so a request may start from the pages of an earlier one
    with the same first tokens, the layers that read another layer's cache included: the second request skips the
    shared pages and still generates what the plain model generates."""
    from holon_amd.config import EngineConfig, SamplingParams
    from holon_amd.engine.engine import Engine
    folder = folders["A-sharp"]
    plain_model = _plain(str(folder))
    head = H.random_ids(43, M.CONFIG_A["vocab"], 7)
    prompts = [head + H.random_ids(5, M.CONFIG_A["vocab"], 8), head + H.random_ids(9, M.CONFIG_A["vocab"], 9)]
    engine = Engine(EngineConfig(model=str(folder), device=device, dtype="float32", page_size=8, max_seqs=2,
                                 max_model_len=96, max_step_tokens=64, cache_tokens=192),
                    TorchKernels() if device == "cpu" else None)
    params = SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True)
    outs = [engine.generate([p], params)[0] for p in prompts]
    assert engine.stats()["prefix_tokens_saved"] >= 40
    held = sum(H.assert_greedy_follows(plain_model, p, o, margin=0.02) for p, o in zip(prompts, outs))
    assert held >= 18
    engine.cache.check()
    engine.close()


@pytest.mark.gpu
@pytest.mark.parametrize("dim", [64, 128, 256])
def test_the_cap_and_the_fixed_sink_on_the_matrix_cores(dim):
    """`paged_attention` as the attention mixer calls it (all keys before the query, a cap or none, a sink of 0 for
    every head, a gate a head or none), in bfloat16 at every head size the matrix cores serve, prompt portions beside decode rows over
    scattered pages, short rows among them (where the one in the denominator weighs most), against float64."""
    from holon_amd.kernels import load_hip
    from holon_amd.kernels.api import AttnRows
    k, dev, page, heads, groups = load_hip(), "cuda", 16, 8, 2
    g = torch.Generator().manual_seed(dim + 1)
    lens, counts = [300, 75, 190, 3, 129, 1, 40], [300, 1, 60, 3, 1, 1, 2]     # tokens a row holds, and brings in this step
    n_pages = sum(-(-n // page) for n in lens) + 1
    table = torch.full((len(lens) + 1, 24), n_pages - 1, dtype=torch.int32)
    order, at = torch.randperm(n_pages - 1, generator=g).tolist(), 0
    for s_, n in enumerate(lens):
        for i in range(-(-n // page)):
            table[s_, i] = order[at]
            at += 1
    pages = (torch.randn(n_pages, 2, groups, page * dim, generator=g) * 0.5).to(dev).bfloat16()
    qstart = [0]
    for c in counts:
        qstart.append(qstart[-1] + c)
    q = torch.randn(qstart[-1], heads, dim, generator=g).to(dev).bfloat16()
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)          # noqa: E731
    decode = [b for b, c in enumerate(counts) if c == 1]
    chunk = [b for b, c in enumerate(counts) if c > 1]
    rows = AttnRows(slots=i32(list(range(len(lens)))), lens=i32(lens), query_start=i32(qstart), decode_rows=i32(decode),
                    chunk_rows=i32(chunk), n_decode=len(decode), n_chunk=len(chunk),
                    max_decode_len=max(lens[b] for b in decode), max_chunk_query=max(counts),
                    max_chunk_len=max(lens[b] for b in chunk))
    sink = torch.zeros(heads, device=dev)
    twin = TorchKernels()
    gates = (2.0 * torch.randn(qstart[-1], heads + 7, generator=g)).to(dev).bfloat16()[:, 3: 3 + heads]    # columns of wider rows
    for scale, cap in ((2.0 * dim ** -0.5, 3.0), (dim ** -0.5, 30.0), (dim ** -0.5, 0.0), (0.05 * dim ** -0.5, 0.0)):
        for gate in (None, gates):                 # the gate a head in the kernels' last step
            got = k.paged_attention(q, pages, table.to(dev), rows, page, scale, 0, sink=sink, softcap=cap, head_gate=gate)
            want = twin.paged_attention(q.double(), pages.double(), table.to(dev), rows, page, scale, 0,
                                        sink=sink.double(), softcap=cap, head_gate=None if gate is None else gate.double())
            assert H.rel_rms(got, want) < 8e-3, (dim, scale, cap)
            per = ((got.double() - want).square().mean((1, 2)).sqrt() / want.square().mean().sqrt()).max().item()
            assert per < 4e-2, (dim, scale, cap, per)
        if cap == 0.0:                             # and without a sink: the kernels that stage keys through LDS
            got = k.paged_attention(q, pages, table.to(dev), rows, page, scale, 0, head_gate=gates)
            want = twin.paged_attention(q.double(), pages.double(), table.to(dev), rows, page, scale, 0,
                                        head_gate=gates.double())
            assert H.rel_rms(got, want) < 8e-3, (dim, scale, "gate alone")


@pytest.mark.gpu
@pytest.mark.parametrize("dim", [64, 128, 256])
def test_key_heads_that_share_value_heads_on_the_gpu(dim):
    """Pages that hold fewer value heads than key heads (two or three key heads read one value head): the matrix-core
    prompt and decode kernels in bfloat16 and the general kernel in both types, prompt portions beside decode rows over
    scattered pages, with and without a sink and a cap, against float64."""
    import holon_amd.parts  # noqa: F401
    from holon_amd.kernels import load_hip
    from holon_amd.kernels.api import AttnRows
    from holon_amd.kernels.registry import kernel_op
    k, dev, page = load_hip(), "cuda", 16
    g = torch.Generator().manual_seed(dim + 2)
    lens, counts = [300, 75, 190, 3, 129, 1, 40], [300, 1, 60, 3, 1, 1, 2]
    n_pages = sum(-(-n // page) for n in lens) + 1
    table = torch.full((len(lens) + 1, 24), n_pages - 1, dtype=torch.int32)
    order, at = torch.randperm(n_pages - 1, generator=g).tolist(), 0
    for s_, n in enumerate(lens):
        for i in range(-(-n // page)):
            table[s_, i] = order[at]
            at += 1
    qstart = [0]
    for c in counts:
        qstart.append(qstart[-1] + c)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)          # noqa: E731
    decode = [b for b, c in enumerate(counts) if c == 1]
    chunk = [b for b, c in enumerate(counts) if c > 1]
    rows = AttnRows(slots=i32(list(range(len(lens)))), lens=i32(lens), query_start=i32(qstart), decode_rows=i32(decode),
                    chunk_rows=i32(chunk), n_decode=len(decode), n_chunk=len(chunk),
                    max_decode_len=max(lens[b] for b in decode), max_chunk_query=max(counts),
                    max_chunk_len=max(lens[b] for b in chunk))
    token_row = torch.cat([torch.full((c,), b, dtype=torch.int32) for b, c in enumerate(counts)]).to(dev)
    positions = torch.cat([torch.arange(n - c, n, dtype=torch.int32) for n, c in zip(lens, counts)]).to(dev)
    twin, scale = TorchKernels(), 1.5 * dim ** -0.5
    for heads, groups, share in ((8, 4, 2), (6, 6, 3), (12, 2, 2)):
        pages = (torch.randn(n_pages, groups + groups // share, page * dim, generator=g) * 0.5).to(dev).bfloat16()
        q = torch.randn(qstart[-1], heads, dim, generator=g).to(dev).bfloat16()
        sink = torch.zeros(heads, device=dev)
        for sk, cap in ((None, 0.0), (sink, 0.0), (sink, 4.0)):
            want = twin.paged_attention(q.double(), pages.double(), table.to(dev), rows, page, scale, 0,
                                        sink=None if sk is None else sk.double(), softcap=cap, value_share=share)
            got = k.paged_attention(q, pages, table.to(dev), rows, page, scale, 0, sink=sk, softcap=cap, value_share=share)
            assert H.rel_rms(got, want) < 8e-3, (dim, heads, groups, share, cap)
            per = ((got.double() - want).square().mean((1, 2)).sqrt() / want.square().mean().sqrt()).max().item()
            assert per < 4e-2, (dim, heads, groups, share, cap, per)
            flat = pages.view(n_pages, -1)
            for dtype, tol in ((torch.bfloat16, 8e-3), (torch.float32, 2e-6)):
                ref = want if dtype == torch.bfloat16 else kernel_op("softmax_attention").plain(
                    q.double(), flat.double(), table.to(dev), rows, token_row, positions, groups, dim, page,
                    None if sk is None else sk.double(), scale, 0, softcap=cap, value_share=share).view(-1, heads, dim)
                general = k.softmax_attention(q.to(dtype), flat.to(dtype), table.to(dev), rows, token_row, positions,
                                              groups, dim, page, sk, scale, 0, softcap=cap, value_share=share)
                assert H.rel_rms(general.view(-1, heads, dim), ref) < tol, (dim, heads, groups, share, cap, dtype)
