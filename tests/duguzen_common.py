"""Small Duguzen configurations with random weights for the tests: sizes chosen so that no two of them coincide (heads,
per-head sizes, latent rank, value size, expert counts, group sizes), layer kinds in mixed order, layers that borrow
another layer's weights, a layer without feed-forward, a rotation over part of the rotated dimensions."""
import numpy as np
import torch

from oracle import duguzen_ref as R


def mixer(heads, dim, rot_dim, rank, vdim, base=10000.0, dims=None, scale=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "kv_rank": rank, "vdim": vdim,
            "rot": {"base": base, "dims": rot_dim if dims is None else dims},
            "scale": float(scale if scale is not None else (dim + rot_dim) ** -0.5)}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, count=None, keep=None):
    rt = {"experts": experts, "top": top}
    if count is not None:
        rt["groups"] = {"count": count, "keep": keep}
    return {"kind": "moe", "expert": {"ff": ff}, "router": rt}


def layer(mx, mlp, weights_of=None):
    d = {"type": "latent_attention", "mixer": mx, "mlp": mlp}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def config_a():
    m0, m1, m3 = mixer(3, 24, 16, 40, 20, base=5000.0, dims=8), mixer(2, 16, 8, 24, 32), mixer(5, 8, 4, 16, 12, base=300.0)
    f0, f1 = moe(24, 6, 2, count=3, keep=2), dense(72)
    return {"architecture": "Duguzen", "width": 96, "vocab": 130, "norm": {"eps": 1e-5},
            "layers": [layer(m0, f0), layer(m1, f1), layer(m0, f0, 0), layer(m3, None), layer(m1, f1, 1)]}


def config_b():
    """a router without groups, one with single-expert groups that are all kept, one head, top 1"""
    m0, m1 = mixer(1, 32, 8, 12, 40, base=100.0), mixer(4, 8, 16, 48, 8, dims=16)
    return {"architecture": "Duguzen", "width": 64, "vocab": 77, "norm": {"eps": 1e-6},
            "layers": [layer(m0, moe(16, 5, 1)), layer(m1, moe(40, 4, 3, count=4, keep=4)), layer(m1, dense(20))]}


def config_odd():
    """nothing is a multiple of 8: every vector path and matrix-core form has to step aside for its scalar / plain twin"""
    m0, m1 = mixer(3, 10, 6, 14, 7, base=50.0, dims=4), mixer(5, 6, 2, 9, 11)
    return {"architecture": "Duguzen", "width": 50, "vocab": 61, "norm": {"eps": 1e-5},
            "layers": [layer(m0, dense(30)), layer(m1, moe(10, 6, 2, count=2, keep=1)), layer(m0, dense(30), 0)]}


def config_tiny():
    return {"architecture": "Duguzen", "width": 48, "vocab": 50, "norm": {"eps": 1e-5},
            "layers": [layer(mixer(2, 8, 8, 16, 8), dense(32)), layer(mixer(2, 8, 8, 16, 8), moe(16, 4, 2, count=2, keep=1))]}


def bf16_round(a):
    return torch.as_tensor(np.asarray(a, dtype=np.float32)).bfloat16().float()


def random_weights(cfg, seed=0, corr_scale=0.6):
    """{name: float32 tensor holding bf16 values}"""
    g = torch.Generator().manual_seed(seed)
    D, V = cfg["width"], cfg["vocab"]
    w = {}

    def lin(name, o, i, gain=1.0):
        w[name] = bf16_round(torch.randn(o, i, generator=g) * gain / i ** 0.5)

    def norm(name, d):
        w[name] = bf16_round(1.0 + 0.2 * torch.randn(d, generator=g))
        w[name + ".b"] = bf16_round(0.1 * torch.randn(d, generator=g))
        w[name + ".alpha"] = bf16_round(0.6 + 0.2 * torch.rand((), generator=g))

    w["embed"] = bf16_round(torch.randn(V, D, generator=g))
    for i, l in enumerate(cfg["layers"]):
        if "weights_of" in l:
            continue
        p, m = "l%d" % i, l["mixer"]
        norm(p + ".norm1", D)
        norm(p + ".norm1b", D)
        lin(p + ".mix.q", m["heads"] * (m["dim"] + m["rot_dim"]), D, 2.0)
        lin(p + ".mix.dkv", m["kv_rank"] + m["rot_dim"], D, 2.0)
        w[p + ".mix.dkv.norm"] = bf16_round(1.0 + 0.2 * torch.randn(m["kv_rank"], generator=g))
        lin(p + ".mix.uk", m["heads"] * m["dim"], m["kv_rank"], 2.0)
        lin(p + ".mix.uv", m["heads"] * m["vdim"], m["kv_rank"], 2.0)
        lin(p + ".mix.g", m["heads"], D, 2.0)
        lin(p + ".mix.o", D, m["heads"] * m["vdim"], 2.0)
        f = l["mlp"]
        if not f:
            continue
        norm(p + ".norm2", D)
        norm(p + ".norm2b", D)
        if f["kind"] == "dense":
            lin(p + ".mlp.up", f["ff"], D, 1.5)
            lin(p + ".mlp.down", D, f["ff"], 1.5)
        else:
            for e in range(f["router"]["experts"]):
                lin("%s.mlp.e%d.gate" % (p, e), f["expert"]["ff"], D, 2.0)
                lin("%s.mlp.e%d.up" % (p, e), f["expert"]["ff"], D, 2.0)
                lin("%s.mlp.e%d.down" % (p, e), D, f["expert"]["ff"], 2.0)
            lin(p + ".mlp.router", f["router"]["experts"], D, 3.0)
            # large enough that choice scores go negative and the correction changes who is chosen
            w[p + ".mlp.correction"] = bf16_round(corr_scale * torch.randn(f["router"]["experts"], generator=g) - 0.8)
    norm("final.norm", D)
    lin("head", V, D, 2.0)
    return w


def engine_for(cfg, w, dtype, max_tokens=512, max_requests=4):
    from pegainfer_amd.duguzen import DuguzenEngine
    eng = DuguzenEngine(cfg, max_tokens=max_tokens, max_requests=max_requests, dtype=dtype)
    return eng.load_tensors({k: v.numpy() for k, v in w.items()})


def oracle_logits(cfg, w, tokens, taps=None):
    return R.forward(cfg, w, tokens, taps).numpy()


def row_err(got, ref):
    """per row: rms of the difference with its mean taken off, relative to the rms of the reference rows"""
    d = np.asarray(got, dtype=np.float64) - ref
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt(((ref - ref.mean(-1, keepdims=True)) ** 2).mean())


TOL = {"float32": 3e-5, "bfloat16": 4e-2}


def tokens_for(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], n).tolist()
