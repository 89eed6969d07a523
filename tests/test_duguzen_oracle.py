"""CPU checks of the plain Duguzen restatement itself (oracle/duguzen_ref.py): properties each mechanism must have whatever
the weights are.  The product path is compared with this oracle in the GPU tests."""
import math

import numpy as np
import torch

import duguzen_common as C
from oracle import duguzen_ref as R


def test_rotation_is_relative_and_partial():
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(1, 12, generator=g, dtype=torch.float64), torch.randn(1, 12, generator=g, dtype=torch.float64)
    dots = []
    for pq, pk in ((5, 3), (105, 103), (1000, 998)):
        a = R.rope_half(q, torch.tensor([pq]), 700.0, 8)
        b = R.rope_half(k, torch.tensor([pk]), 700.0, 8)
        dots.append(float((a * b).sum()))
        assert torch.equal(a[:, 8:], q[:, 8:])          # dimensions beyond rot.dims pass through
    assert max(dots) - min(dots) < 1e-9                 # the score depends on the distance only
    assert torch.allclose(R.rope_half(q, torch.tensor([0]), 700.0, 8), q)


def test_rotation_pairs_i_with_i_plus_half():
    x = torch.zeros(1, 6, dtype=torch.float64)
    x[0, 1] = 1.0
    y = R.rope_half(x, torch.tensor([3]), 10.0, 6)[0]
    ang = 3 * 10.0 ** (-2.0 * 1 / 6)
    assert abs(y[1] - math.cos(ang)) < 1e-12 and abs(y[4] - math.sin(ang)) < 1e-12 and abs(y[0]) + abs(y[2]) < 1e-15


def test_router_groups_minus_infinity_not_zero():
    """all choice scores negative: an expert of a dropped group must not win because its score 'counts as 0'"""
    rt = {"experts": 4, "top": 2, "groups": {"count": 2, "keep": 1}}
    w = {"r.router": torch.zeros(4, 3), "r.correction": torch.tensor([-2.0, -3.0, -0.9, -5.0])}
    idx, wt = R.route(torch.ones(1, 3, dtype=torch.float64), w, "r", rt)
    # group scores: (-1.5 + -2.5) = -4 vs (-0.4 + -4.5) = -4.9 -> group 0 kept although expert 2 has the best single score
    assert sorted(idx[0].tolist()) == [0, 1]
    assert torch.allclose(wt, torch.full((1, 2), 0.5, dtype=torch.float64))     # weights are the plain sigmoid scores


def test_router_weights_are_not_renormalised_and_ignore_the_correction():
    cfg = C.config_a()
    w = C.random_weights(cfg, 3)
    h = torch.randn(7, cfg["width"], dtype=torch.float64)
    idx, wt = R.route(h, w, "l0.mlp", cfg["layers"][0]["mlp"]["router"])
    s = torch.sigmoid(h @ w["l0.mlp.router"].double().T)
    assert torch.allclose(wt, s.gather(1, idx))
    assert idx.shape == (7, 2) and all(len(set(r)) == 2 for r in idx.tolist())


def test_causality_and_borrowed_weights():
    cfg = C.config_a()
    w = C.random_weights(cfg, 5)
    toks = C.tokens_for(cfg, 19, 0)
    full = C.oracle_logits(cfg, w, toks)
    assert np.allclose(C.oracle_logits(cfg, w, toks[:11]), full[:11], atol=1e-9)      # a position sees j <= i only
    taps = []
    C.oracle_logits(cfg, w, toks, taps)
    assert len(taps) == len(cfg["layers"])
    assert not any(k.startswith("l2.") or k.startswith("l4.") for k in w)               # layers 2 and 4 own no tensors
    cfg2 = {**cfg, "layers": cfg["layers"][:2] + [cfg["layers"][0], cfg["layers"][3], cfg["layers"][1]]}
    w2 = {k.replace("l3.", "lX.").replace("l0.", "l2.") if k.startswith("l0.") else k: v for k, v in w.items()}
    w2.update({k: v for k, v in w.items() if k.startswith("l0.")})
    w2.update({k.replace("l1.", "l4."): v for k, v in w.items() if k.startswith("l1.")})
    assert np.allclose(C.oracle_logits(cfg2, w2, toks), full, atol=1e-9)               # own copies of the same tensors


def test_sigmoid_gate_and_squared_relu():
    cfg = C.config_tiny()
    w = C.random_weights(cfg, 2)
    h = torch.randn(5, cfg["width"], dtype=torch.float64)
    y = R.dense_ff(h, w, "l0.mlp")
    u = torch.relu(h @ w["l0.mlp.up"].double().T)
    assert torch.allclose(y, (u * u) @ w["l0.mlp.down"].double().T)
    w_closed = dict(w)
    w_closed["l0.mix.g"] = torch.zeros_like(w["l0.mix.g"])
    pos = torch.arange(5)
    a = R.latent_attention(h, w, "l0.mix", cfg["layers"][0]["mixer"], 1e-5, pos)
    b = R.latent_attention(h, w_closed, "l0.mix", cfg["layers"][0]["mixer"], 1e-5, pos)
    assert not torch.allclose(a, 2 * b) and torch.isfinite(a).all()      # gate 0.5 everywhere is one particular scaling


def test_borrowing_from_a_layer_that_borrows():
    cfg = C.config_a()
    w = C.random_weights(cfg, 6)
    toks = C.tokens_for(cfg, 9, 1)
    ref = C.oracle_logits(cfg, w, toks)
    chained = {**cfg, "layers": [dict(l) for l in cfg["layers"]]}
    chained["layers"][4]["weights_of"] = 1          # as before
    chained["layers"][2]["weights_of"] = 0
    chained["layers"].append({**cfg["layers"][2], "weights_of": 2})     # layer 5 borrows from 2, which borrows from 0
    direct = {**cfg, "layers": cfg["layers"] + [{**cfg["layers"][2], "weights_of": 0}]}
    assert R.owner(chained, 5) == 0
    assert np.allclose(C.oracle_logits(chained, w, toks), C.oracle_logits(direct, w, toks), atol=1e-12)
    assert not np.allclose(C.oracle_logits(direct, w, toks), ref, atol=1e-6)
