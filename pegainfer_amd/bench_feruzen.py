"""Prefill and decode throughput of Feruzen at layer sizes of a real model, beside Qwen3.5 (the closest existing model:
gated-delta-rule layers with short convolutions, every fourth layer softmax attention over paged K/V, gated feed-forward) at
equal width, head counts, head sizes, feed-forward size and layer count.  Random weights, bf16, one GPU.
`python bench.py --model feruzen [--fz-size mid]` prints one JSON line; the default bench workload is untouched."""
import json
import time

SIZES = {
    # width, delta: value heads / key heads x 128; attention: heads / kv heads x head_dim; matrix memory heads x dim x vdim;
    # dense ff; experts x expert ff, top, shared ff; vocab
    "small": dict(width=1024, lin_v=8, lin_k=4, heads=4, kv=1, head_dim=256, mm_heads=4, mm_dim=128, mm_vdim=128, ff=3072,
                  experts=16, eff=512, top=4, sff=1024, vocab=32768),
    "mid": dict(width=2560, lin_v=32, lin_k=16, heads=16, kv=4, head_dim=256, mm_heads=8, mm_dim=128, mm_vdim=256, ff=9216,
                experts=32, eff=1024, top=4, sff=2048, vocab=65536),
    "large": dict(width=4096, lin_v=32, lin_k=16, heads=16, kv=4, head_dim=256, mm_heads=16, mm_dim=128, mm_vdim=256, ff=12288,
                  experts=32, eff=1536, top=6, sff=3072, vocab=65536),
}
LAYERS = 8   # (delta + dense, delta + routed, delta + dense, parallel + routed) twice: Qwen3.5's three-to-one layer pattern


def feruzen_config(s):
    delta = {"heads": s["lin_v"], "kv_heads": s["lin_k"], "dim": 128, "vdim": 128, "conv": 4}
    par = {"left": {"heads": s["heads"], "kv_heads": s["kv"], "dim": s["head_dim"], "vdim": s["head_dim"],
                    "rot": {"base": 1e6, "dims": s["head_dim"] // 4}, "scale": s["head_dim"] ** -0.5},
           "right": {"heads": s["mm_heads"], "dim": s["mm_dim"], "vdim": s["mm_vdim"], "gate_cap": 15.0},
           "left_scale": 1.0, "right_scale": 1.0}
    dense = {"kind": "dense", "ff": s["ff"], "limit": 7.0}
    moe = {"kind": "moe", "expert": {"ff": s["eff"], "limit": 7.0}, "router": {"experts": s["experts"], "top": s["top"]},
           "shared": {"ff": s["sff"], "limit": 7.0}}
    layers = []
    for i in range(LAYERS):
        if i % 4 == 3:
            layers.append({"type": "parallel", "mixer": par, "mlp": moe})
        else:
            layers.append({"type": "delta", "mixer": delta, "mlp": dense if i % 2 == 0 else moe})
    return {"architecture": "Feruzen", "width": s["width"], "vocab": s["vocab"], "norm": {"eps": 1e-5, "groups": 4},
            "canon": {"taps": 4}, "layers": layers}


def qwen35_config(s):
    return dict(hidden_size=s["width"], intermediate_size=s["ff"], num_hidden_layers=LAYERS, vocab_size=s["vocab"],
                num_attention_heads=s["heads"], num_key_value_heads=s["kv"], head_dim=s["head_dim"],
                linear_num_key_heads=s["lin_k"], linear_num_value_heads=s["lin_v"], linear_key_head_dim=128,
                linear_value_head_dim=128, linear_conv_kernel_dim=4, rms_norm_eps=1e-6, rope_theta=1e7, partial_rotary_factor=0.25,
                layer_types=["full_attention" if i % 4 == 3 else "linear_attention" for i in range(LAYERS)])


def _timed(fn, iters):
    fn()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    return (time.perf_counter() - t0) / iters


def measure_feruzen(s, prompt_len, ctx, batches, iters):
    from .feruzen import FeruzenEngine
    eng = FeruzenEngine(feruzen_config(s), max_tokens=max(batches) * (ctx + 64) + prompt_len + 64, max_requests=max(batches),
                        dtype="bfloat16").fill_synthetic(seed=1, std=0.02)
    prompt = [(100 + i) % s["vocab"] for i in range(prompt_len)]
    out = {"weight_bytes": eng.weight_bytes(), "state_floats_per_request": eng.state_floats()}

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


def measure_qwen35(s, prompt_len, ctx, batches, iters):
    from .qwen35 import Qwen35Engine
    pages = max(batches) * ((ctx + 64) // 16 + 2) + prompt_len // 16 + 8
    eng = Qwen35Engine(qwen35_config(s), num_kv_pages=pages, max_batch_size=max(batches), enable_graph=True, max_positions=8192)
    eng.fill_synthetic(seed=1, std=0.02)
    prompt = [(100 + i) % s["vocab"] for i in range(prompt_len)]
    out = {}

    def prefill():
        r = eng.new_request()
        eng.prefill(r, prompt)
        eng.drop_request(r)
    out["prefill_tok_s"] = round(prompt_len / _timed(prefill, iters), 1)
    for bs in batches:
        rids = [eng.new_request() for _ in range(bs)]
        for r in rids:
            eng.prefill(r, prompt[:ctx])
        dt = _timed(lambda: eng.decode(rids, [7] * bs), max(iters, 20))
        out["decode_bs%d_tok_s" % bs] = round(bs / dt, 1)
        for r in rids:
            eng.drop_request(r)
    eng.close()
    return out


def run(args):
    sizes = [args.fz_size] if args.fz_size != "all" else list(SIZES)
    which = getattr(args, "fz_only", "both")
    res = {}
    for name in sizes:
        s = SIZES[name]
        res[name] = {"layers": LAYERS, "sizes": s}
        if which in ("both", "feruzen"):
            res[name]["feruzen"] = measure_feruzen(s, args.ctx, args.ctx, (1, 4), max(2, args.warmup))
        if which in ("both", "qwen35"):
            res[name]["qwen35_equal_size"] = measure_qwen35(s, args.ctx, args.ctx, (1, 4), max(2, args.warmup))
    print(json.dumps({"metric": "feruzen_vs_qwen35_layer_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
                      "n_gpus": 1, "prompt_len": args.ctx, "decode_ctx": args.ctx, "results": res}))
    return 0
