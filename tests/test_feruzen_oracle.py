"""CPU checks of the plain Feruzen restatement (oracle/feruzen_ref.py) against independent forms of the same equations, so
that the thing the GPU tests compare with is itself pinned: the recurrences against their unrolled sums, the convolution
against torch's, the grouped norm against a loop, the rotation against complex multiplication, causality and the reach of
the convolutions' history."""
import math

import numpy as np
import torch

import feruzen_common as C
from oracle import feruzen_ref as R

F = torch.float64


def test_time_convolution_matches_conv1d_and_last_column_is_the_current_token():
    g = torch.Generator().manual_seed(1)
    h, c = torch.randn(9, 5, generator=g, dtype=F), torch.randn(5, 4, generator=g, dtype=F)
    ref = torch.nn.functional.conv1d(torch.nn.functional.pad(h.T[None], (3, 0)), c[:, None, :], groups=5)[0].T
    assert torch.allclose(R.tconv(h, c), ref, atol=1e-12)
    only_now = torch.zeros(5, 4, dtype=F)
    only_now[:, -1] = 2.0
    assert torch.allclose(R.tconv(h, only_now), 2.0 * h)


def test_grouped_norm_is_a_norm_per_part():
    g = torch.Generator().manual_seed(2)
    y, w = torch.randn(4, 12, generator=g, dtype=F), torch.randn(12, generator=g, dtype=F)
    out = R.grms(y, w, 3, 1e-5)
    for r in range(4):
        for p in range(3):
            part = y[r, 4 * p:4 * p + 4]
            assert torch.allclose(out[r, 4 * p:4 * p + 4], part / torch.sqrt((part ** 2).mean() + 1e-5) * w[4 * p:4 * p + 4])


def test_pair_rotation_is_a_complex_multiplication_on_the_first_dims_only():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(6, 2, 10, generator=g, dtype=F)
    pos = torch.arange(6)
    out = R.rope_pairs(x, pos, 100.0, 6)
    assert torch.equal(out[..., 6:], x[..., 6:])
    for i in range(3):
        z = torch.complex(x[..., 2 * i], x[..., 2 * i + 1]) * torch.exp(1j * pos.to(F) * 100.0 ** (-2.0 * i / 6))[:, None]
        assert torch.allclose(out[..., 2 * i], z.real) and torch.allclose(out[..., 2 * i + 1], z.imag)


def test_delta_rule_state_equals_its_closed_form_for_orthogonal_keys():
    """with beta = 1, no decay and orthonormal keys the state after n tokens is sum_t k_t v_t^T (every write lands in an empty
    direction), and a key met again has its value REPLACED, not added"""
    d, dv = 6, 4
    S = torch.zeros(d, dv, dtype=F)
    keys = torch.eye(d, dtype=F)[[0, 1, 2, 1]]
    vals = torch.arange(16, dtype=F).reshape(4, 4)
    for k, v in zip(keys, vals):
        u = 1.0 * (v - S.T @ k)
        S = S + torch.outer(k, u)
    assert torch.allclose(S[0], vals[0]) and torch.allclose(S[2], vals[2]) and torch.allclose(S[1], vals[3])


def test_matrix_memory_equals_the_unstabilised_sum():
    """o_t = sum_s exp(i_s + sum_{r in (s, t]} f_r) (q_t . k_s) v_s / (max(|same with 1 for v|, 1) + 1e-6 e^{-m} ...): compare
    the stabilised recurrence with the direct sums in a range where nothing overflows"""
    cfg = C.config_tiny()
    m = cfg["layers"][1]["mixer"]["right"]
    w = C.random_weights(cfg, 4)
    g = torch.Generator().manual_seed(5)
    h = torch.randn(7, cfg["width"], generator=g, dtype=F)
    p = "l1.mix.right"
    got = R.matrix_memory(h, w, p, m, 1e-5)
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[p + ".q"].to(F).T).reshape(7, H, d) * d ** -0.5
    k = (h @ w[p + ".k"].to(F).T).reshape(7, H, d)
    v = (h @ w[p + ".v"].to(F).T).reshape(7, H, dv)
    ig = cap * torch.tanh((h @ w[p + ".i"].to(F).T + w[p + ".i.b"].to(F)) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ w[p + ".f"].to(F).T + w[p + ".f.b"].to(F)) / cap))
    out = torch.zeros(7, H, dv, dtype=F)
    for hh in range(H):
        mm = 0.0
        for t in range(7):
            mm = max(float(fg[t, hh]) + mm, float(ig[t, hh]))
            num, den = torch.zeros(dv, dtype=F), 0.0
            for s in range(t + 1):
                lw = float(ig[s, hh] + fg[s + 1:t + 1, hh].sum())
                a = math.exp(lw) * float(q[t, hh] @ k[s, hh])
                num += a * v[s, hh]
                den += a
            # the recurrence divides scaled sums: (num e^-m) / (max(|den e^-m|, e^-m) + 1e-6)
            out[t, hh] = num * math.exp(-mm) / (max(abs(den) * math.exp(-mm), math.exp(-mm)) + 1e-6)
    ref = R.rms(out, 1e-5).reshape(7, H * dv) * w[p + ".norm"].to(F) * torch.sigmoid(h @ w[p + ".g"].to(F).T)
    assert torch.allclose(got, ref @ w[p + ".o"].to(F).T, atol=1e-9)


def test_router_takes_the_largest_softmax_scores_unrenormalised():
    w = {"r.router": torch.tensor([[1.0, 0.0], [0.0, 1.0], [-1.0, 0.0], [0.5, 0.5]])}
    idx, val = R.router(torch.tensor([[2.0, 1.0]], dtype=F), w, "r", 2)
    s = torch.softmax(torch.tensor([2.0, 1.0, -2.0, 1.5], dtype=F), 0)
    assert idx.tolist() == [[0, 3]] and torch.allclose(val[0], s[[0, 3]]) and float(val.sum()) < 1.0


def test_the_model_is_causal_and_every_layer_kind_sees_the_past():
    cfg = C.config_a()
    w = C.random_weights(cfg, 6)
    toks = C.tokens_for(cfg, 14, 1)
    base = C.oracle_logits(cfg, w, toks)
    other = list(toks)
    other[9] = (other[9] + 1) % cfg["vocab"]
    moved = C.oracle_logits(cfg, w, other)
    assert np.abs(moved[:9] - base[:9]).max() == 0.0
    assert all(np.abs(moved[t] - base[t]).max() > 1e-6 for t in range(9, 14))


def test_clamp_glu_limits_gate_from_above_only_and_up_on_both_sides():
    w = {"f.gate": torch.tensor([[1.0]]), "f.up": torch.tensor([[1.0]]), "f.down": torch.tensor([[1.0]])}
    f = lambda z: float(R.clamp_glu(torch.tensor([[z]], dtype=F), w, "f", 2.0))  # noqa: E731
    assert abs(f(5.0) - 2.0 / (1 + math.exp(-1.702 * 2.0)) * 3.0) < 1e-12          # gate and up clamped at +2
    assert abs(f(-5.0) - (-5.0) / (1 + math.exp(1.702 * 5.0)) * (-1.0)) < 1e-12    # gate free below, up clamped at -2
