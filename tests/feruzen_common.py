"""Small Feruzen configurations with random weights for the tests.  Sizes are chosen so that values a real model tends to
make equal differ here (query / value sizes, taps of the input convolution and of the mixer's convolutions, the three
clamp limits, heads of the two halves of a parallel mixer), and so that the special cases are met: a rotation over part of
a head, one key/value head and several, more query heads per key/value head than one attention workgroup holds, a layer
without feed-forward, a router without shared expert, top 1, one norm group, one tap (no history at all)."""
import numpy as np
import torch

from oracle import feruzen_ref as R


def left(heads, kv, dim, vdim, dims, base=10000.0, scale=None):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "rot": {"base": base, "dims": dims},
            "scale": float(scale if scale is not None else dim ** -0.5)}


def right(heads, dim, vdim, cap):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def parallel(lf, rt, ls, rs, mlp):
    return {"type": "parallel", "mixer": {"left": lf, "right": rt, "left_scale": ls, "right_scale": rs}, "mlp": mlp}


def delta(heads, kv, dim, vdim, conv, mlp):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(ff, limit, experts, top, shared=None):
    d = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if shared:
        d["shared"] = {"ff": shared[0], "limit": shared[1]}
    return d


def base(width, vocab, groups, taps, layers, eps=1e-5):
    return {"architecture": "Feruzen", "width": width, "vocab": vocab, "norm": {"eps": eps, "groups": groups},
            "canon": {"taps": taps}, "layers": layers}


def config_a():
    return base(96, 131, 3, 3, [
        delta(4, 2, 24, 20, 2, moe(24, 1.25, 6, 2, shared=(40, 2.0))),
        parallel(left(6, 2, 16, 24, 8, base=1000.0, scale=0.3), right(3, 12, 28, 8.0), 0.7, 1.3, dense(72, 1.75)),
        parallel(left(2, 2, 40, 8, 40, base=50.0), right(1, 20, 16, 3.0), 1.5, 0.5, None),
        delta(3, 3, 8, 12, 5, dense(56, 0.9)),
    ])


def config_b():
    """one norm group, one tap everywhere (no history), top 1, no shared expert, a single attention head"""
    return base(64, 77, 1, 1, [
        parallel(left(1, 1, 32, 16, 0), right(2, 8, 8, 15.0), 1.0, 1.0, moe(16, 3.0, 5, 1)),
        delta(2, 1, 16, 32, 1, moe(40, 0.5, 4, 3, shared=(8, 1.0))),
        delta(1, 1, 12, 4, 3, None),
    ], eps=1e-6)


def config_odd():
    """nothing is a multiple of 8"""
    return base(50, 61, 5, 2, [
        parallel(left(3, 3, 10, 6, 4, base=30.0), right(3, 14, 7, 5.0), 0.9, 1.1, dense(30, 1.1)),
        delta(5, 1, 6, 11, 3, moe(10, 2.5, 6, 2, shared=(14, 1.3))),
    ])


def config_wide_heads():
    """more query heads per key/value head than an attention workgroup's 16 rows; memories wider than one column block
    (vdim > 64) and deeper than the smallest register layouts (dim > 64); attention values over more than 64 columns"""
    return base(128, 90, 2, 4, [
        parallel(left(20, 1, 8, 72, 6, base=200.0), right(2, 72, 80, 6.0), 1.0, 1.0, dense(64, 1.5)),
        delta(2, 1, 80, 72, 4, None),
        parallel(left(4, 2, 136, 16, 136, base=1e5, scale=0.05), right(1, 130, 12, 9.0), 0.6, 1.4, moe(32, 2.0, 4, 2)),
    ])


def config_real_heads():
    """head sizes of real models (128 and 256, equal for keys and values): in bf16 the attention of these layers runs on
    the matrix-core kernels that Qwen3 / Qwen3.5 use; the delta and memory layers get their widest register layouts"""
    return base(64, 70, 2, 4, [
        parallel(left(4, 2, 128, 128, 32, base=1e4), right(1, 128, 96, 12.0), 1.2, 0.8, dense(48, 2.0)),
        delta(2, 1, 128, 128, 4, moe(16, 1.5, 4, 2, shared=(24, 1.5))),
        parallel(left(2, 1, 256, 256, 64, base=1e6), right(2, 40, 24, 8.0), 0.9, 1.1, None),
    ])


def config_only_delta():
    """no attention anywhere (no cache part at all), seven layers deep: the depth-weighted sum runs over up to eight streams"""
    return base(40, 33, 2, 3, [delta(2, 1, 8, 12, 2 + i % 3, dense(24, 1.5) if i % 2 else None) for i in range(7)])


def config_only_parallel():
    """no delta layer anywhere"""
    return base(56, 45, 4, 2, [parallel(left(2, 1, 12, 20, 4), right(2, 10, 6, 4.0), 1.1, 0.9, moe(16, 1.0, 3, 3)),
                               parallel(left(3, 3, 8, 8, 8, base=77.0), right(1, 16, 24, 20.0), 0.5, 2.0, dense(40, 3.0))])


def config_tiny():
    return base(48, 50, 2, 2, [delta(2, 2, 8, 8, 2, dense(32, 1.5)),
                               parallel(left(2, 1, 8, 8, 8), right(2, 8, 8, 10.0), 1.0, 1.0, moe(16, 1.5, 4, 2, shared=(16, 1.5)))])


def bf16_round(a):
    return torch.as_tensor(np.asarray(a, dtype=np.float32)).bfloat16().float()


def random_weights(cfg, seed=0, gate_gain=6.0):
    """{name: float32 tensor holding bf16 values}.  gate_gain: size of the matrix memory's gate inputs; 6 drives them into
    the cap, which a bf16 run cannot follow: there the rounding of the gate inputs alone, summed over the log forget gates
    of a few dozen tokens, moves old entries against new ones by tens of percent (the restatement itself moves that much
    when its gate inputs are rounded to bf16), so bf16 runs take weights_for(), with gates a quarter that size (the delta rule's decay input scales along)."""
    g = torch.Generator().manual_seed(seed)
    D, V, K = cfg["width"], cfg["vocab"], cfg["canon"]["taps"]
    w = {}

    def lin(name, o, i, gain=1.0):
        w[name] = bf16_round(torch.randn(o, i, generator=g) * gain / i ** 0.5)

    def vec(name, n, mean=0.0, std=1.0):
        w[name] = bf16_round(mean + std * torch.randn(n, generator=g))

    def glu(p, f):
        lin(p + ".gate", f["ff"], D, 2.0)
        lin(p + ".up", f["ff"], D, 2.0)
        lin(p + ".down", D, f["ff"], 2.0)

    w["embed"] = bf16_round(torch.randn(V, D, generator=g))
    for i, l in enumerate(cfg["layers"]):
        p, m = "l%d" % i, l["mixer"]
        vec(p + ".norm1", D, 1.0, 0.2)
        w[p + ".canon1"] = bf16_round(0.4 * torch.randn(D, K, generator=g))
        coef = 0.3 * torch.randn(i + 2, generator=g)
        coef[-1] += 1.0
        w[p + ".dwa"] = bf16_round(coef)
        q = p + ".mix"
        if l["type"] == "delta":
            for n, rows in (("q", m["kv_heads"] * m["dim"]), ("k", m["kv_heads"] * m["dim"]), ("v", m["heads"] * m["vdim"])):
                lin("%s.%s" % (q, n), rows, D, 2.0)
                w["%s.%s.conv" % (q, n)] = bf16_round(0.5 * torch.randn(rows, m["conv"], generator=g))
            lin(q + ".b", m["heads"], D, 2.0)
            lin(q + ".a", m["heads"], D, gate_gain / 3.0)       # the decay's input: its rounding adds up over the tokens, too
            vec(q + ".A_log", m["heads"], -0.5, 0.7)
            vec(q + ".dt_bias", m["heads"], 0.0, 0.5)
            vec(q + ".norm", m["vdim"], 1.0, 0.2)
            lin(q + ".g", m["heads"] * m["vdim"], D, 2.0)
            lin(q + ".o", D, m["heads"] * m["vdim"], 2.0)
        else:
            a, r = m["left"], m["right"]
            lin(q + ".left.q", a["heads"] * a["dim"], D, 2.0)
            lin(q + ".left.k", a["kv_heads"] * a["dim"], D, 2.0)
            lin(q + ".left.v", a["kv_heads"] * a["vdim"], D, 2.0)
            vec(q + ".left.q.norm", a["dim"], 1.0, 0.3)
            vec(q + ".left.k.norm", a["dim"], 1.0, 0.3)
            lin(q + ".left.o", D, a["heads"] * a["vdim"], 2.0)
            lin(q + ".right.q", r["heads"] * r["dim"], D, 2.0)
            lin(q + ".right.k", r["heads"] * r["dim"], D, 2.0)
            lin(q + ".right.v", r["heads"] * r["vdim"], D, 2.0)
            lin(q + ".right.g", r["heads"] * r["vdim"], D, 2.0)
            lin(q + ".right.o", D, r["heads"] * r["vdim"], 2.0)
            vec(q + ".right.norm", r["heads"] * r["vdim"], 1.0, 0.2)
            lin(q + ".right.i", r["heads"], D, gate_gain)       # 6: large enough that the cap on the gates matters
            vec(q + ".right.i.b", r["heads"], 0.0, 1.0)
            lin(q + ".right.f", r["heads"], D, gate_gain)
            vec(q + ".right.f.b", r["heads"], 2.0, 1.0)
        f = l["mlp"]
        if not f:
            continue
        vec(p + ".norm2", D, 1.0, 0.2)
        if f["kind"] == "dense":
            glu(p + ".mlp", f)
        else:
            for e in range(f["router"]["experts"]):
                glu("%s.mlp.e%d" % (p, e), f["expert"])
            lin(p + ".mlp.router", f["router"]["experts"], D, 4.0)
            if f.get("shared"):
                glu(p + ".mlp.shared", f["shared"])
    vec("final.norm", D, 1.0, 0.2)
    return w


def weights_for(cfg, seed, dtype):
    return random_weights(cfg, seed, gate_gain=6.0 if dtype == "float32" else 1.5)


def engine_for(cfg, w, dtype, max_tokens=512, max_requests=4):
    from pegainfer_amd.feruzen import FeruzenEngine
    eng = FeruzenEngine(cfg, max_tokens=max_tokens, max_requests=max_requests, dtype=dtype)
    return eng.load_tensors({k: v.numpy() for k, v in w.items()})


def oracle_logits(cfg, w, tokens, hidden=False):
    out = R.forward(cfg, w, tokens, return_hidden=hidden)
    return (out[0].numpy(), out[1].numpy()) if hidden else out.numpy()


def row_err(got, ref):
    """per row: rms of the difference with its mean taken off, relative to the rms of the reference rows"""
    d = np.asarray(got, dtype=np.float64) - ref
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt(((ref - ref.mean(-1, keepdims=True)) ** 2).mean())


TOL = {"float32": 3e-5, "bfloat16": 8e-2}


def tokens_for(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], n).tolist()
