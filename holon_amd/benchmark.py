"""Decode and prefill throughput of the engine at the Qwen3-8B shape with random weights, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--no-points]
    python -m holon_amd bench ...          (the same)

    python bench.py --workload mixed|long [--layers L]

One JSON line: decoded tokens a second at the given batch (default 8) with every request near a context of 4,096 tokens
(the far end of a 2,048-token prompt and 2,048 generated tokens: the requests are given prompts that leave just the
timed steps, `config.decode_prompt_len`), plus the prefill of one 2,048-token prompt (`prefill.ms` is the best of three
prompts, `prefill.ms_median` their median), the decode step's memory roofline, and `points`: decode at batch 1, 16, 32
and 64 at the same context and at batch 8 at a context of 32,768 (tokens a second, ms a step, the gigabytes a step
must read, the fraction of the memory roofline), and prompts of 512 and 8,192 tokens (tokens a second, best and median
ms, TFLOP, the fraction of the matrix peak; the longer one takes two steps under the step budget of 4,096 tokens).
`latency` holds the time to the first token of the 2,048-token prompt and the median time between two tokens of a
request, as the reference's driver reports them (bench/driver.py:102-134); `products` what every matrix product with
a choice of kernels took. A step is one decode step of the engine: scheduling, the model, sampling and the commit.
The engine is one process on one GPU; for --gpus > 1 a line says so and the exit code is 2.

--workload runs a whole job through the engine instead and prints its own line: `mixed` is 32 requests of 128 to 4,096
prompt tokens at the Qwen3-32B shape, portions of 512 tokens beside decode rows, 256 greedy tokens each; `long` is 8
prompts of 32,768 tokens at the Qwen3-4B shape, 512 tokens each at temperature 0.7.

--workload tolurax (or relanex, or nevodra) measures that design beside Qwen3 at equal sizes (width, layers, heads, head size,
feed-forward, vocabulary; random weights): a 2,048-token prompt and decode at batch 8 near a context of 2,048, at two
sizes (`--sizes`), one line with both models' figures and the bytes a decode step must read. `--only` runs one model
(for a profiler). --workload dopirax measures Dopirax the same way, beside Nevodra (the nearest design: both sublayers
on one float32 stream, a capped attention, experts) and Qwen3 (`--beside`).
"""
from __future__ import annotations

import argparse
import json
import sys
import time

HBM_GBS = 8000.0                 # MI355X published peaks
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}
QWEN3_8B = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 36, "hidden_size": 4096,
            "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 12288,
            "vocab_size": 151936, "rope_theta": 1e6, "rms_norm_eps": 1e-6, "tie_word_embeddings": False,
            "max_position_embeddings": 40960}
CONTEXT, PROMPT = 4096, 2048
LONG_CONTEXT = 32768            # the context of the long decode point (batch 8)
POINT_BATCHES = (1, 16, 32, 64)
POINT_PROMPTS = (512, 8192)
QWEN3_32B = dict(QWEN3_8B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, intermediate_size=25600)
QWEN3_4B = dict(QWEN3_8B, hidden_size=2560, intermediate_size=9728, tie_word_embeddings=True)


def workload(name: str, layers: int | None, dtype: str, products: str = "timed") -> int:
    """A whole job: every request added at once, stepped until all are finished."""
    import random

    import torch

    from .config import EngineConfig, SamplingParams
    from .engine.engine import Engine
    rng = random.Random(0)
    if name == "mixed":
        shape, model = QWEN3_32B, "Qwen3-32B shape"
        prompts = [[rng.randrange(shape["vocab_size"]) for _ in range(rng.randint(128, 4096))] for _ in range(32)]
        params = SamplingParams(temperature=0.0, max_tokens=256, ignore_eos=True)
        ecfg = dict(max_seqs=32, max_model_len=4096 + 256 + 16, max_step_tokens=1024, chunk_with_decode=512)
    else:
        shape, model = QWEN3_4B, "Qwen3-4B shape"
        prompts = [[rng.randrange(shape["vocab_size"]) for _ in range(32768)] for _ in range(8)]
        params = SamplingParams(temperature=0.7, seed=1, max_tokens=512, ignore_eos=True)
        ecfg = dict(max_seqs=8, max_model_len=40960, max_step_tokens=4096)
    cfg_json = dict(shape, num_hidden_layers=layers or shape["num_hidden_layers"])
    engine = Engine.from_random(cfg_json, seed=0, cfg=EngineConfig(
        model=f"random:{name}", device="cuda:0", dtype=dtype, page_size=16, products=products,
        cache_tokens=len(prompts) * (max(map(len, prompts)) + params.max_tokens + 64), **ecfg))
    for p in prompts:
        engine.add(p, params)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = steps = out_at = 0
    t_prompts = None
    while engine.has_work():
        out += sum(len(d.token_ids) for d in engine.step())
        steps += 1
        if t_prompts is None and not engine.sched.waiting and all(
                s.num_computed >= s.prompt_len for s in engine.sched.running):
            torch.cuda.synchronize()
            t_prompts, out_at = time.perf_counter() - t0, out
    torch.cuda.synchronize()
    total = time.perf_counter() - t0
    stats = engine.stats()
    prompt_tokens = sum(map(len, prompts))
    print(json.dumps({
        "metric": f"{name} workload, {model}: tokens/s over the whole job", "value": round((prompt_tokens + out) / total, 1),
        "unit": "tokens/s", "n_gpus": 1, "seconds": round(total, 3), "dtype": "bf16" if dtype == "bfloat16" else "fp32",
        "data": "synthetic (random weights, uniform random token ids)",
        "config": {"model": model, "layers": cfg_json["num_hidden_layers"], "layers_of_config": shape["num_hidden_layers"],
                   "requests": len(prompts), "prompt_tokens": prompt_tokens, "output_tokens": out, **ecfg},
        "until_prompts_done": {"seconds": round(t_prompts, 3), "prompt_tokens_per_s": round(prompt_tokens / t_prompts, 1)},
        "decode_tail": {"tokens_per_s": round((out - out_at) / max(total - t_prompts, 1e-9), 1)},
        "steps": steps, "mixed_steps": stats["mixed_steps"], "preemptions": stats["preemptions"],
        "products": {"mode": products, "took": stats["products"]}}), flush=True)
    return 0


DESIGN_SIZES = {     # width, layers, heads, kv heads, head size, feed-forward, vocabulary
    "2k": dict(width=2048, layers=8, heads=16, kv_heads=4, dim=128, ff=8192, vocab=32768),
    "4k": dict(width=4096, layers=4, heads=32, kv_heads=8, dim=128, ff=12288, vocab=32768)}


def tolurax_config(z: dict, window: int = 1024) -> dict:
    """A Tolurax model of a size's layers: three parallel layers (windowed sigmoid attention with the size's heads
    beside a decayed memory of heads of 64 over the same width) to every delta layer, a feed-forward in each."""
    def layer(i: int) -> dict:
        mlp = {"kind": "dense", "ff": z["ff"]}
        if i % 4 == 3:
            return {"type": "delta", "mlp": mlp, "mixer": {"heads": z["heads"], "kv_heads": z["heads"], "dim": z["dim"],
                                                          "vdim": z["dim"], "conv": 4}}
        left = {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["dim"],
                "mask": {"size": window}, "scale": z["dim"] ** -0.5,
                "rot": {"dims": z["dim"], "base": 10000.0,
                        "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}
        right = {"heads": z["width"] // 64, "dim": 64, "rank": 64}
        return {"type": "parallel", "mlp": mlp, "mixer": {"left": left, "right": right, "left_scale": 1.0,
                                                          "right_scale": 1.0}}
    return {"architecture": "Tolurax", "width": z["width"], "vocab": z["vocab"], "norm": {"eps": 1e-6},
            "canon": {"taps": 3}, "logit_softcap": 30.0, "layers": [layer(i) for i in range(z["layers"])]}


def relanex_config(z: dict, window: int = 1024) -> dict:
    """A Relanex model of a size's layers, in fours: softmax attention with the size's heads (half of each head
    rotated, YaRN), two latent-attention layers (the size's heads, latents of 768 and 256, a window), and a matrix
    memory with heads of 128, a feed-forward in each."""
    def layer(i: int) -> dict:
        mlp = {"kind": "dense", "ff": z["ff"]}
        if i % 4 == 0:
            return {"type": "attention", "mlp": mlp,
                    "mixer": {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["dim"],
                              "scale": z["dim"] ** -0.5,
                              "rot": {"dims": z["dim"] // 2, "base": 1e6,
                                      "scaling": {"factor": 8.0, "original": 4096, "fast": 16.0, "slow": 2.0}}}}
        if i % 4 == 3:
            return {"type": "mlstm", "mlp": mlp, "mixer": {"heads": z["width"] // 128, "dim": 128, "vdim": 128,
                                                          "gate_cap": 15.0}}
        return {"type": "latent_attention", "mlp": mlp,
                "mixer": {"heads": z["heads"], "dim": z["dim"], "vdim": z["dim"], "q_rank": 768, "kv_rank": 256,
                          "mask": {"size": window}, "scale": z["dim"] ** -0.5}}
    return {"architecture": "Relanex", "width": z["width"], "vocab": z["vocab"], "norm": {"eps": 1e-6},
            "residual_mult": 0.5, "layers": [layer(i) for i in range(z["layers"])]}


def nevodra_config(z: dict, window: int = 1024) -> dict:
    """A Nevodra model of a size's layers, in pairs: windowed attention with the size's heads (a tanh cap, a distance
    bias, four kept first tokens) over a dense PolyNorm feed-forward of the size's width, then latent attention (the
    size's heads, a latent of 192 and 64 rotated dimensions: cache entries of 256) over eight experts of a quarter of
    that width of which a token uses two, beside a shared one; filters of three taps on every sublayer's input."""
    def layer(i: int) -> dict:
        if i % 2 == 0:
            return {"type": "attention", "mlp": {"kind": "dense", "ff": z["ff"]},
                    "mixer": {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["dim"],
                              "scale": z["dim"] ** -0.5, "softcap": 30.0, "mask": {"size": window, "keep_first": 4}}}
        quarter = z["ff"] // 4
        return {"type": "latent_attention",
                "mlp": {"kind": "moe", "expert": {"ff": quarter}, "shared": {"ff": quarter},
                        "router": {"experts": 8, "top": 2, "scale": 1.5, "groups": {"count": 4, "keep": 2}}},
                "mixer": {"heads": z["heads"], "dim": z["dim"], "rot_dim": 64, "vdim": z["dim"], "kv_rank": 192,
                          "scale": (z["dim"] + 64) ** -0.5, "rot": {"dims": 64, "base": 1e6}}}
    return {"architecture": "Nevodra", "width": z["width"], "vocab": z["vocab"], "norm": {"eps": 1e-6},
            "embedding": {"scale": 1.0}, "canon": {"taps": 3}, "layers": [layer(i) for i in range(z["layers"])]}


def dopirax_config(z: dict) -> dict:
    """A Dopirax model of a size's layers, in fours: differential attention with half the size's heads (two maps a
    head, so as many score maps as the size has heads; keys and values of the size's head size, all of a map turned)
    over a dense feed-forward of the size's width; a second such layer that reads the first one's keys and values, over
    eight experts of a quarter of that width of which a token uses two, beside a gated shared one; then two layers of
    the attention whose values are its keys (the size's heads, half of a head turned, a cap of 30, a gate a head), one
    over the experts and one over the dense feed-forward."""
    quarter = z["ff"] // 4
    experts = {"kind": "moe", "expert": {"ff": quarter}, "shared": {"ff": quarter}, "router": {"experts": 8, "top": 2}}
    dense = {"kind": "dense", "ff": z["ff"]}

    def layer(i: int) -> dict:
        if i % 4 < 2:
            m = {"heads": z["heads"] // 2, "kv_heads": max(z["kv_heads"] // 2, 1), "dim": z["dim"], "vdim": z["dim"],
                 "scale": z["dim"] ** -0.5, "diff": 0.5, "rot": {"dims": z["dim"], "base": 1e6}}
            if i % 4 == 1:
                m["kv_from"] = i - 1
            return {"type": "attention_2", "mixer": m, "mlp": dense if i % 4 == 0 else experts}
        m = {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["dim"], "scale": z["dim"] ** -0.5,
             "softcap": 30.0, "rot": {"dims": z["dim"] // 2, "base": 1e6}}
        return {"type": "attention", "mixer": m, "mlp": experts if i % 4 == 2 else dense}
    return {"architecture": "Dopirax", "width": z["width"], "vocab": z["vocab"], "norm": {"eps": 1e-6},
            "embedding": {"scale": 1.0}, "layers": [layer(i) for i in range(z["layers"])]}


DESIGN_CONFIGS = {"tolurax": tolurax_config, "relanex": relanex_config, "nevodra": nevodra_config,
                  "dopirax": dopirax_config}


def design_cache_bytes(name: str, cfg_json: dict, z: dict, item: int, batch: int, context: int) -> int:
    """The bytes of paged cache a decode step of `batch` rows near `context` reads."""
    if name == "qwen3":
        return z["layers"] * 2 * z["kv_heads"] * z["dim"] * item * batch * context
    total = 0
    for layer in cfg_json["layers"]:
        m = layer["mixer"]
        if name == "dopirax":                       # every layer reads all of a cache, its own or another layer's
            maps = 2 if layer["type"] == "attention_2" else 1     # differential layers keep the keys of both maps
            total += m["kv_heads"] * (maps * m["dim"] + m["vdim"]) * item * batch * context
        elif layer["type"] == "parallel":             # the window's keys and values
            total += 2 * z["kv_heads"] * z["dim"] * item * batch * min(context, m["left"]["mask"]["size"])
        elif layer["type"] == "attention":
            seen = min(context, m["mask"]["size"] + m["mask"].get("keep_first", 0)) if m.get("mask") else context
            total += m["kv_heads"] * (m["dim"] + m["vdim"]) * item * batch * seen
        elif layer["type"] == "latent_attention":   # the cache entry, held as keys and as values
            seen = min(context, m["mask"]["size"]) if m.get("mask") else context
            total += 2 * (m["kv_rank"] + m.get("rot_dim", 0)) * item * batch * seen
    return total


def qwen3_config(z: dict) -> dict:
    return {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": z["layers"], "hidden_size": z["width"],
            "num_attention_heads": z["heads"], "num_key_value_heads": z["kv_heads"], "head_dim": z["dim"],
            "intermediate_size": z["ff"], "vocab_size": z["vocab"], "rope_theta": 1e6, "rms_norm_eps": 1e-6,
            "tie_word_embeddings": False, "max_position_embeddings": 8192}


def design(a) -> int:
    """A design (Tolurax or Relanex) beside Qwen3 at equal sizes: prompt and decode throughput, one line."""
    import gc

    import torch

    from .config import EngineConfig, SamplingParams
    from .engine.engine import Engine
    prompt, context, batch = 2048, 2048, 8
    g = torch.Generator().manual_seed(0)
    greedy = lambda n: SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True)      # noqa: E731
    out: dict = {}
    for size in a.sizes.split(","):
        z = DESIGN_SIZES[size]
        ours = DESIGN_CONFIGS[a.workload](z)
        others = [n for n in (a.beside or ("nevodra,qwen3" if a.workload == "dopirax" else "qwen3")).split(",") if n]
        beside = [(n, qwen3_config(z) if n == "qwen3" else DESIGN_CONFIGS[n](z)) for n in others if n != a.workload]
        for name, cfg_json in [(a.workload, ours)] + beside:
            if a.only and a.only != name:
                continue
            engine = Engine.from_random(cfg_json, seed=0, cfg=EngineConfig(
                model=f"random:{name}-{size}", device="cuda:0", dtype=a.dtype, page_size=16, max_seqs=batch,
                max_model_len=context + 64, max_step_tokens=4096, cache_tokens=batch * (context + 64),
                graphs=not a.no_graphs, products=a.products, prefix_cache=False))
            item = 2 if a.dtype == "bfloat16" else 4
            weights = sum(getattr(o, n).numel() * getattr(o, n).element_size()
                          for path, o, n, _ in engine.model.named_params() if not path.startswith("embed."))
            # what a request keeps in its slot (the recurrences' matrices, the filters' inputs): read and written a step
            state = sum(t[0].numel() * t.element_size() for _, _, t in engine.cache.slot_states)
            times = []
            for _ in range(3):
                engine.add(torch.randint(0, z["vocab"], (prompt,), generator=g).tolist(), greedy(1))
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                while engine.has_work():
                    engine.step()
                engine.drain()
                torch.cuda.synchronize()
                times.append((time.perf_counter() - t0) * 1e3)
            start = context - a.steps - a.warmup - 3
            for _ in range(batch):
                engine.add(torch.randint(0, z["vocab"], (start,), generator=g).tolist(), greedy(a.steps + a.warmup + 3))
            while engine.sched.waiting:
                engine.step()
            for _ in range(a.warmup):
                engine.step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(a.steps):
                engine.step()
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) * 1e3 / a.steps
            while engine.has_work():
                engine.step()
            kv = design_cache_bytes(name, cfg_json, z, item, batch, context)
            step_gb = (weights + kv + 2 * state * batch) / 1e9
            out.setdefault(size, {})[name] = {
                "prefill_tokens_per_s": round(prompt / (min(times) * 1e-3), 1), "prefill_ms": round(min(times), 3),
                "prefill_ms_median": round(sorted(times)[1], 3), "decode_tokens_per_s": round(batch / (ms * 1e-3), 1),
                "decode_ms_per_step": round(ms, 4), "decode_step_gb": round(step_gb, 3),
                "decode_frac_of_hbm": round(step_gb / (ms * 1e-3) / HBM_GBS, 4),
                "graphs": engine.runner.use_graphs}
            engine.close()
            del engine
            gc.collect()
            torch.cuda.empty_cache()
    print(json.dumps({"metric": f"{a.workload.capitalize()} beside {' and '.join(n.capitalize() for n in others)} at equal sizes: 2,048-token prompt, decode at batch 8 near "
                                "context 2,048",
                      "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
                      "dtype": "bf16" if a.dtype == "bfloat16" else "fp32",
                      "data": "synthetic (random weights, uniform random token ids)",
                      "sizes": {k: DESIGN_SIZES[k] for k in out}, "results": out}), flush=True)
    return 0


def main(argv: list[str] | None = None) -> int:
    ap = argparse.ArgumentParser(prog="bench", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=24,
                    help="untimed decode steps first (the first 15 or so after the prompts run 3%% slower)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=QWEN3_8B["num_hidden_layers"],
                    help="fewer layers than the configuration has (recorded in config)")
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    ap.add_argument("--no-points", action="store_true", help="skip the further decode and prefill points")
    ap.add_argument("--context", type=int, default=CONTEXT, help="the context the timed decode steps end at")
    ap.add_argument("--prompt", type=int, default=PROMPT, help="tokens of the timed prompt")
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--workload", choices=("decode", "mixed", "long", "tolurax", "relanex", "nevodra", "dopirax"),
                    default="decode")
    ap.add_argument("--sizes", default="2k,4k", help="--workload tolurax|relanex|nevodra|dopirax: which of its sizes (2k, 4k) to run")
    ap.add_argument("--only", choices=("tolurax", "relanex", "nevodra", "dopirax", "qwen3"), default=None,
                    help="--workload tolurax|relanex|nevodra|dopirax: one model only")
    ap.add_argument("--beside", default=None,
                    help="--workload of a design: the models it is measured beside, with commas (default: qwen3; for "
                         "dopirax: nevodra,qwen3)")
    ap.add_argument("--products", choices=("own", "vendor", "timed"), default="timed",
                    help="EngineConfig.products: which kernel products of 17 to 1,024 rows take (reported in the line)")
    a = ap.parse_args(argv)
    if a.gpus != 1:
        print(f"bench.py: this engine serves on one GPU; --gpus {a.gpus} is not a configuration it has", flush=True)
        return 2
    if a.workload != "decode":
        from .kernels import build as kernel_build
        if kernel_build.find_library() is None:
            kernel_build.build()
        if a.workload in DESIGN_CONFIGS:
            return design(a)
        return workload(a.workload, None if "--layers" not in (argv or sys.argv) else a.layers, a.dtype, a.products)

    import torch

    from .config import EngineConfig, SamplingParams
    from .engine.engine import Engine
    from .kernels import build as kernel_build

    if kernel_build.find_library() is None:
        kernel_build.build()
    cfg_json = dict(QWEN3_8B, num_hidden_layers=a.layers)
    max_batch = max(a.batch, 1 if a.no_points else max(POINT_BATCHES))
    longest = max(a.context, a.prompt, 0 if a.no_points else max(LONG_CONTEXT, max(POINT_PROMPTS)))
    engine = Engine.from_random(cfg_json, seed=0, cfg=EngineConfig(
        model="random:qwen3-8b", device="cuda:0", dtype=a.dtype, page_size=16, max_seqs=max_batch,
        max_model_len=longest + 16, max_step_tokens=4096,
        cache_tokens=max(max_batch * (CONTEXT + 16), a.batch * (a.context + 16), a.prompt + 16,
                         0 if a.no_points else 8 * (LONG_CONTEXT + 16)),
        graphs=not a.no_graphs, products=a.products))
    spec, c = engine.spec, cfg_json
    item = 2 if a.dtype == "bfloat16" else 4
    g = torch.Generator().manual_seed(0)
    greedy = lambda n: SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True)

    def decode(batch: int, steps: int, warmup: int, context: int = CONTEXT) -> tuple[float, float, float, int]:
        """(ms per decode step, mean context, median ms between two steps' ends, prompt length) for `batch` requests
        whose contexts end at `context`. The requests go on for two steps after the timed ones, so that the host's work
        for finished requests (not part of a decode step) falls outside the timed region."""
        after = 2
        start = context - steps - warmup - 1 - after
        for _ in range(batch):
            engine.add(torch.randint(0, c["vocab_size"], (start,), generator=g).tolist(),
                       greedy(steps + warmup + 1 + after))
        while engine.sched.waiting:                              # prompts, cut by the step budget
            engine.step()
        for _ in range(warmup):
            engine.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ends = []
        for _ in range(steps):
            engine.step()                      # returns when the step before has been committed: one step's time apart
            ends.append(time.perf_counter())
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        gaps = sorted(b - a for a, b in zip(ends, ends[1:])) or [ms * 1e-3]
        while engine.has_work():
            engine.step()
        return ms, start + 1 + warmup + steps / 2, gaps[len(gaps) // 2] * 1e3, start

    def prefill(tokens: int) -> tuple[float, float]:
        """(best, median) ms from adding a prompt of `tokens` to its first generated token on the host: one step, or as
        many as the step budget cuts the prompt into."""
        times = []
        for _ in range(3):                     # another prompt each time: nothing of it is in the prefix cache
            ids = torch.randint(0, c["vocab_size"], (tokens,), generator=g).tolist()
            engine.add(ids, greedy(1))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            while engine.has_work():
                engine.step()
            engine.drain()                     # the last step's one token on the host: the request is finished
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t0) * 1e3)
            assert not engine.has_work()
        return min(times), sorted(times)[1]

    h, hq, hkv, d, inter, v, layers = (c["hidden_size"], c["num_attention_heads"], c["num_key_value_heads"],
                                       c["head_dim"], c["intermediate_size"], c["vocab_size"], a.layers)
    layer_params = h * (hq + 2 * hkv) * d + hq * d * h + 3 * h * inter
    weight_bytes = (layers * (layer_params + 2 * h + 2 * d) + h + h * v) * item      # every weight a decode step reads
    kv_token_bytes = layers * 2 * hkv * d * item
    def prompt_flops(tokens: int) -> float:
        """Products of every layer over `tokens` rows, causal attention (half of the square), the head on one row."""
        return layers * (2 * tokens * layer_params + 2 * hq * d * tokens * tokens) + 2 * h * v

    pre_ms, ttft_ms = prefill(a.prompt)
    pre_flops = prompt_flops(a.prompt)
    ms, ctx, tpot_ms, decode_prompt = decode(a.batch, a.steps, a.warmup, a.context)
    step_bytes = weight_bytes + a.batch * ctx * kv_token_bytes
    achieved = step_bytes / (ms * 1e-3) / 1e9
    points = {}
    if not a.no_points:
        def decode_point(name: str, b: int, context: int) -> None:
            pms, pctx, _, _ = decode(b, a.steps, a.warmup, context)
            gb = (weight_bytes + b * pctx * kv_token_bytes) / 1e9
            points[name] = round(b / (pms * 1e-3), 1)
            points[f"{name}_ms"] = round(pms, 4)
            points[f"{name}_gb"] = round(gb, 2)
            points[f"{name}_frac"] = round(gb / (pms * 1e-3) / HBM_GBS, 4)
        for b in POINT_BATCHES:
            decode_point(f"decode_b{b}", b, CONTEXT)
        decode_point(f"decode_b8_ctx{LONG_CONTEXT}", 8, LONG_CONTEXT)
        for tokens in POINT_PROMPTS:
            best, median = prefill(tokens)
            points[f"prefill_{tokens}"] = round(tokens / (best * 1e-3), 1)
            points[f"prefill_{tokens}_ms"] = round(best, 3)
            points[f"prefill_{tokens}_ms_median"] = round(median, 3)
            points[f"prefill_{tokens}_tflop"] = round(prompt_flops(tokens) / 1e12, 2)
            points[f"prefill_{tokens}_frac"] = round(prompt_flops(tokens) / (best * 1e-3) / PEAK_FLOPS[a.dtype], 4)
    line = {
        "metric": f"decode tok/s at batch {a.batch} (context {a.context:,}), Qwen3-8B shape", "value": round(a.batch / (ms * 1e-3), 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if a.dtype == "bfloat16" else "fp32",
        "data": "synthetic (random weights, uniform random token ids)",
        "config": {"model": "Qwen3-8B shape", "layers": layers, "layers_of_config": QWEN3_8B["num_hidden_layers"],
                   "hidden": h, "heads": hq, "kv_heads": hkv, "head_dim": d, "intermediate": inter, "vocab": v,
                   "tied": False, "global_batch": a.batch, "seq_len": a.context, "prefill_tokens": a.prompt,
                   "decode_prompt_len": decode_prompt, "page_size": 16,
                   "parallelism": "single GPU", "graphs": not a.no_graphs, "mean_context": round(ctx, 1),
                   "products": a.products},
        "prefill": {"value": round(a.prompt / (pre_ms * 1e-3), 1), "tokens": a.prompt, "ms": round(pre_ms, 3),
                    "ms_is": "best of 3 prompts", "ms_median": round(ttft_ms, 3),
                    "frac": round(pre_flops / (pre_ms * 1e-3) / PEAK_FLOPS[a.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4)},
        "points": points,
        "products": engine.products(),
        "latency": {"ttft_ms_p50": round(ttft_ms, 3), "ttft_tokens": a.prompt, "tpot_ms_p50": round(tpot_ms, 4),
                    "tpot_batch": a.batch},
    }
    if engine.stats()["prefix_tokens_saved"]:
        raise RuntimeError("the prefix cache served part of a timed prompt: the figures above would count work not done")
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
