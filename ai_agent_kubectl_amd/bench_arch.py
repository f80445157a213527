"""Engine-level prefill and decode throughput of two model families at equal layer sizes.

`bench.py --arch-compare` runs this: for each size, a Vivepel configuration and the Llama configuration
with the same width, heads, head size, feed-forward width, vocabulary and depth (random weights), and with
`--arch-models ...,kafilorn` a Kafilorn of that width and depth (layers cycling mLSTM + dense, latent attention
+ experts, latent attention on the previous layer's cache + dense; latent ranks W/8 and 3W/8, 8 experts of
width ff/4 with 2 chosen plus a shared one, two residual streams), and with `...,suvapel` a Suvapel of that width and
depth (layers alternating a delta rule with attention beside a channel-decay delta rule, window = the chunk, four
taps, a 64-wide token input; its closest existing model is Kafilorn: recurrent state slots + windowed attention +
fp32 residual), and with `...,zibinex` a Zibinex of that width and depth (gated latent attention and sliding sigmoid
attention in turn, latent rank W/8 with a rotated part of half a head, the window = the chunk, the first layer's
feed-forward dense and clamped, the others 8 experts of width ff/4 with 2 chosen; its closest existing model is Kafilorn:
latent attention + experts + fp32 residual), go through the same engine path (`build_engine`, the scheduler, `ModelRunner.execute`, hipGraph decode):
B prompts of P tokens are prefilled (in steps of the engine's token budget), then N tokens are
decoded per sequence.  Reported per model: prefill tokens/s (prompt tokens / time in prefill steps)
and decode tokens/s (B x decode steps / time in decode steps), from the runner's own step timers.
"""
from __future__ import annotations

import json
import time

SIZES = {
    # name: (width, heads, kv heads, head size, ff, vocab, layers)
    "2k": (2048, 16, 4, 128, 8192, 32000, 8),
    "8b": (4096, 32, 8, 128, 14336, 128256, 8),
    "70b": (8192, 64, 8, 128, 28672, 128256, 4),
}


def _configs(size: str, chunk: int):
    import dataclasses

    from .models.config import PRESETS, ModelConfig, kafilorn_uniform, suvapel_uniform, vivepel_uniform, zibinex_uniform

    W, H, G, D, ff, V, L = SIZES[size]
    ll = ModelConfig(f"llama-{size}-{L}l", "llama", L, W, H, G, D, ff, V, 500000.0)
    vv = vivepel_uniform(f"vivepel-{size}-{L}l", L, W, H, G, D, ff, V, chunk=chunk)
    kk = kafilorn_uniform(f"kafilorn-{size}-{L}l", (L + 2) // 3, W, H, V, ff, experts=8, top=2, expert_ff=ff // 4,
                          window=chunk, streams=2, kv_rank=W // 8, q_rank=3 * W // 8, dim=D, rot_dim=D // 2)
    kk = dataclasses.replace(kk, layers=kk.layers[:L])
    ss = suvapel_uniform(f"suvapel-{size}-{L}l", L, W, H, G, D, ff, V, window=chunk)
    zz = zibinex_uniform(f"zibinex-{size}-{L}l", L, W, H, G, D, ff, V, window=chunk, kv_rank=W // 8, rot_dim=D // 2,
                         experts=8, top=2, expert_ff=ff // 4)
    for c in (ll, vv, kk, ss, zz):
        PRESETS[c.name] = c
    return ll, vv, kk, ss, zz


def run_one(model: str, batch: int, prompt: int, new_tokens: int, warmup: int = 1, device: str = "cuda") -> dict:
    import torch

    from .engine.builder import EngineOptions, build_engine
    from .engine.sequence import SamplingParams

    buckets = tuple(sorted({b for b in (1, 2, 4, 8, 16, 32, 64, 128, 256) if b <= batch} | {batch}))
    eng = build_engine(EngineOptions(model=model, device=device, max_batch=batch, graph_buckets=buckets,
                                     kv_cache_tokens=batch * (prompt + new_tokens + 32), max_model_len=prompt + new_tokens + 32,
                                     safe_decode=False, ignore_eos=True, prefix_caching=False))
    t0 = time.perf_counter()
    eng.runner.capture_graphs()
    t_cap = time.perf_counter() - t0
    g = torch.Generator().manual_seed(0)
    V = eng.runner.cfg.vocab_size
    params = SamplingParams(max_new_tokens=new_tokens, ignore_eos=True, safe_decode=False)
    out = {}
    for it in range(warmup + 1):
        prompts = torch.randint(0, V, (batch, prompt), generator=g).tolist()
        for k in eng.runner.stats:
            eng.runner.stats[k] = 0 if isinstance(eng.runner.stats[k], int) else 0.0
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.generate_blocking(prompts, params)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        st = dict(eng.runner.stats)
        out = {"model": model, "params_b": round(eng.runner.cfg.num_params() / 1e9, 3), "batch": batch, "prompt": prompt,
               "new_tokens": new_tokens,
               "prefill_tok_s": round(batch * prompt / max(st["prefill_ms"], 1e-9) * 1e3, 1),
               "decode_tok_s": round(batch * st["decode_steps"] / max(st["decode_ms"], 1e-9) * 1e3, 1),
               "prefill_ms": round(st["prefill_ms"], 2), "prefill_steps": st["prefill_steps"],
               "decode_ms_per_step": round(st["decode_ms"] / max(st["decode_steps"], 1), 3),
               "graph_replays": st["graph_replays"], "wall_s": round(wall, 3), "capture_s": round(t_cap, 1)}
    del eng
    torch.cuda.empty_cache()
    return out


def main(sizes=("2k", "8b"), batch: int = 32, prompt: int = 1024, new_tokens: int = 32, chunk: int = 1024,
         which=("llama", "vivepel")) -> dict:
    rows = []
    for size in sizes:
        ll, vv, kk, ss, zz = _configs(size, chunk)
        for cfg in [c for c, n in ((ll, "llama"), (vv, "vivepel"), (kk, "kafilorn"), (ss, "suvapel"), (zz, "zibinex")) if n in which]:
            r = run_one(cfg.name, batch, prompt, new_tokens)
            r["size"] = size
            rows.append(r)
            print("# " + json.dumps(r), flush=True)
    by = {(r["size"], r["model"].split("-")[0]): r for r in rows}
    ratio = {s: {k: round(by[(s, "vivepel")][k] / by[(s, "llama")][k], 3) for k in ("prefill_tok_s", "decode_tok_s")}
             for s in sizes if (s, "vivepel") in by and (s, "llama") in by}
    kratio = {s: {k: round(by[(s, "kafilorn")][k] / by[(s, "vivepel")][k], 3) for k in ("prefill_tok_s", "decode_tok_s")}
              for s in sizes if (s, "kafilorn") in by and (s, "vivepel") in by}
    out = {"metric": "arch_compare", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
           "chunk": chunk, "rows": rows, "vivepel_over_llama": ratio}
    if kratio:
        out["kafilorn_over_vivepel"] = kratio
    sratio = {s: {k: round(by[(s, "suvapel")][k] / by[(s, "kafilorn")][k], 3) for k in ("prefill_tok_s", "decode_tok_s")}
              for s in sizes if (s, "suvapel") in by and (s, "kafilorn") in by}
    if sratio:
        out["suvapel_over_kafilorn"] = sratio
    zratio = {s: {k: round(by[(s, "zibinex")][k] / by[(s, "kafilorn")][k], 3) for k in ("prefill_tok_s", "decode_tok_s")}
              for s in sizes if (s, "zibinex") in by and (s, "kafilorn") in by}
    if zratio:
        out["zibinex_over_kafilorn"] = zratio
    return out
