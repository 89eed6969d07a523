"""Prefill and decode throughput of Duguzen at layer sizes of a real model, beside Qwen3 (the closest existing model: dense
attention over paged K/V, SwiGLU feed-forward) at equal width, heads, feed-forward size and layer count.  Random weights,
bf16, one GPU.  `python bench.py --model duguzen [--dz-size mid]` prints one JSON line; the default bench workload is
untouched."""
import json
import time

import numpy as np

SIZES = {
    # width, heads, nope, rot, rank, vdim, dense ff, experts, expert ff, top, groups, keep, vocab
    "small": dict(width=1024, heads=8, nope=64, rot=32, rank=256, vdim=64, ff=4096, experts=16, eff=512, top=4, groups=4, keep=2, vocab=32768),
    "mid": dict(width=2048, heads=16, nope=128, rot=64, rank=512, vdim=128, ff=8192, experts=32, eff=1024, top=4, groups=4, keep=2, vocab=32768),
    "large": dict(width=4096, heads=32, nope=128, rot=64, rank=512, vdim=128, ff=12288, experts=32, eff=1536, top=6, groups=8, keep=4, vocab=65536),
}
LAYER_RUNS = 8   # dense, routed, then three times both again on the first two layers' weights


def duguzen_config(s):
    mx = {"heads": s["heads"], "dim": s["nope"], "rot_dim": s["rot"], "kv_rank": s["rank"], "vdim": s["vdim"],
          "rot": {"base": 10000.0, "dims": s["rot"]}, "scale": (s["nope"] + s["rot"]) ** -0.5}
    dense = {"kind": "dense", "ff": s["ff"]}
    moe = {"kind": "moe", "expert": {"ff": s["eff"]},
           "router": {"experts": s["experts"], "top": s["top"], "groups": {"count": s["groups"], "keep": s["keep"]}}}
    layers = []
    for i in range(LAYER_RUNS):
        l = {"type": "latent_attention", "mixer": mx, "mlp": dense if i % 2 == 0 else moe}
        if i >= 2:
            l["weights_of"] = i % 2
        layers.append(l)
    return {"architecture": "Duguzen", "width": s["width"], "vocab": s["vocab"], "norm": {"eps": 1e-5}, "layers": layers}


def qwen3_config(s):
    return dict(hidden_size=s["width"], num_hidden_layers=LAYER_RUNS, num_attention_heads=s["heads"],
                num_key_value_heads=max(1, s["heads"] // 4), head_dim=128, intermediate_size=s["ff"], vocab_size=s["vocab"],
                rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False, max_position_embeddings=8192)


def _timed(fn, iters):
    fn()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    return (time.perf_counter() - t0) / iters


def measure_duguzen(s, prompt_len, ctx, batches, iters):
    from .duguzen import DuguzenEngine
    eng = DuguzenEngine(duguzen_config(s), max_tokens=max(batches) * (ctx + 64) + prompt_len + 64, max_requests=max(batches),
                        dtype="bfloat16").fill_synthetic(seed=1, std=0.02)
    prompt = [(100 + i) % s["vocab"] for i in range(prompt_len)]
    out = {"weight_bytes": eng.weight_bytes()}

    def prefill():
        r = eng.new_request()
        eng.step([(r, prompt)], logits=False, tokens=True)
        eng.drop_request(r)
    out["prefill_tok_s"] = round(prompt_len / _timed(prefill, iters), 1)
    out["prefill_device_ms"] = round(eng.last_step_ms(), 3)
    for bs in batches:
        rids = [eng.new_request() for _ in range(bs)]
        eng.step([(r, prompt[:ctx]) for r in rids], logits=False, tokens=True)
        dt = _timed(lambda: eng.step([(r, [7]) for r in rids], logits=False, tokens=True), max(iters, 20))
        out["decode_bs%d_tok_s" % bs] = round(bs / dt, 1)
        out["decode_bs%d_device_ms" % bs] = round(eng.last_step_ms(), 3)
        for r in rids:
            eng.drop_request(r)
    eng.close()
    return out


def measure_qwen3(s, prompt_len, ctx, batches, iters):
    from .qwen3 import Qwen3Engine
    pages = max(batches) * ((ctx + 64) // 16 + 2) + prompt_len // 16 + 8
    eng = Qwen3Engine(qwen3_config(s), num_kv_pages=pages, max_batch_size=max(batches), enable_graph=True, decode_mode=1,
                      split_policy=1, max_positions=8192)
    eng.fill_synthetic(seed=1, std=0.02)
    prompt = [(100 + i) % s["vocab"] for i in range(prompt_len)]
    out = {}

    def prefill():
        r = eng.new_request()
        eng.prefill([r], [prompt])
        eng.drop_request(r)
    out["prefill_tok_s"] = round(prompt_len / _timed(prefill, iters), 1)
    for bs in batches:
        rids = [eng.new_request() for _ in range(bs)]
        eng.prefill(rids, [prompt[:ctx]] * bs)
        dt = _timed(lambda: eng.decode(rids, [7] * bs), max(iters, 20))
        out["decode_bs%d_tok_s" % bs] = round(bs / dt, 1)
        for r in rids:
            eng.drop_request(r)
    eng.close()
    return out


def run(args):
    sizes = [args.dz_size] if args.dz_size != "all" else list(SIZES)
    res = {}
    for name in sizes:
        s = SIZES[name]
        res[name] = {"duguzen": measure_duguzen(s, args.ctx, args.ctx, (1, 4), max(2, args.warmup)),
                     "qwen3_equal_size": measure_qwen3(s, args.ctx, args.ctx, (1, 4), max(2, args.warmup)),
                     "layer_runs": LAYER_RUNS, "sizes": s}
    print(json.dumps({"metric": "duguzen_vs_qwen3_layer_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
                      "n_gpus": 1, "prompt_len": args.ctx, "decode_ctx": args.ctx, "results": res}))
    return 0
