"""Plain, slow restatement of the Feruzen decoder (TEST INFRASTRUCTURE ONLY; nothing in pegainfer_amd/ imports it).

One function per mechanism, one whole sequence at a time, float64 on the CPU, no cache, no state carried between calls:
every recurrence is a Python loop over the tokens from position 0.

Notation (n tokens, residual width D, layer index i, X_0 = embedding rows):
  grms(y; w, G)   : y cut into G equal consecutive parts, each part / sqrt(mean(part^2) + eps), whole vector * w
  tconv(h; c)     : causal per-channel convolution over time, taps K: out_t = sum_j c[:, j] h_(t-K+1+j), zeros before 0
  layer           : h = x + tconv(x; canon1);  x <- x + grms(mixer(h); norm1);  x <- x + grms(ff(x); norm2)  (ff optional)
  depth average   : X_(i+1) = the layer's result; the next layer reads sum_(j <= i+1) dwa_i[j] X_j
  delta mixer     : q, k (kv_heads x dim), v (heads x vdim) = silu(tconv(W. h)); q, k -> unit length per head (q also
                    * dim^-1/2); beta = sigmoid(Wb h); g = exp(-exp(A_log) softplus(Wa h + dt_bias));
                    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;  out = rms(o) * w * silu(Wg h);  Wo
  parallel mixer  : left_scale * softmax attention (q/k RMS norm, interleaved partial rotation, grouped kv heads)
                    + right_scale * matrix memory (exponential input gate, sigmoid forget gate, both soft-capped,
                    stabilised by a running maximum m that starts at 0)
  clamp-GLU ff    : g = min(Wg x, L), u = clamp(Wu x, -L, L);  Wd (g sigmoid(1.702 g) (u + 1))
  routed ff       : s = softmax(Wr x); the `top` largest s choose experts, weights = those s (not renormalised);
                    plus a shared expert for every token
"""
import json
import math
import os

import torch
import torch.nn.functional as Fn

F = torch.float64


def read_config(path):
    with open(path if path.endswith(".json") else os.path.join(path, "config.json")) as f:
        return json.load(f)


def grms(y, weight, groups, eps):
    n, d = y.shape
    p = y.reshape(n, groups, d // groups)
    p = p / torch.sqrt((p * p).mean(-1, keepdim=True) + eps)
    return p.reshape(n, d) * weight


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def tconv(h, c):
    """h [n, C], c [C, K]; the last column of c multiplies the current token"""
    n, C = h.shape
    K = c.shape[1]
    pad = torch.cat([torch.zeros(K - 1, C, dtype=F), h], 0)
    out = torch.zeros(n, C, dtype=F)
    for j in range(K):
        out += pad[j:j + n] * c[:, j][None, :]
    return out


def rope_pairs(x, pos, base, dims):
    """x [n, heads, d]: neighbours (2i, 2i+1) of the first `dims` values are rotated by pos * base^(-2i/dims)"""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    ang = pos.to(F)[:, None] * f[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    rot = torch.stack([u * c - v * s, v * c + u * s], -1).reshape(x.shape[0], x.shape[1], dims)
    return torch.cat([rot, x[..., dims:]], -1)


def softmax_attention(h, w, p, m, eps):
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + ".q"].to(F).T).reshape(n, H, d)
    k = (h @ w[p + ".k"].to(F).T).reshape(n, G, d)
    v = (h @ w[p + ".v"].to(F).T).reshape(n, G, dv)
    q = rms(q, eps) * w[p + ".q.norm"].to(F)
    k = rms(k, eps) * w[p + ".k.norm"].to(F)
    pos = torch.arange(n)
    q = rope_pairs(q, pos, m["rot"]["base"], m["rot"]["dims"])
    k = rope_pairs(k, pos, m["rot"]["base"], m["rot"]["dims"])
    out = torch.zeros(n, H, dv, dtype=F)
    mask = torch.tril(torch.ones(n, n, dtype=torch.bool))
    for hh in range(H):
        g = hh // (H // G)
        sc = (q[:, hh] @ k[:, g].T) * m["scale"]
        sc = sc.masked_fill(~mask, -math.inf)
        out[:, hh] = torch.softmax(sc, -1) @ v[:, g]
    return out.reshape(n, H * dv) @ w[p + ".o"].to(F).T


def matrix_memory(h, w, p, m, eps):
    n = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[p + ".q"].to(F).T).reshape(n, H, d) * d ** -0.5
    k = (h @ w[p + ".k"].to(F).T).reshape(n, H, d)
    v = (h @ w[p + ".v"].to(F).T).reshape(n, H, dv)
    ig = cap * torch.tanh((h @ w[p + ".i"].to(F).T + w[p + ".i.b"].to(F)) / cap)
    fg = Fn.logsigmoid(cap * torch.tanh((h @ w[p + ".f"].to(F).T + w[p + ".f.b"].to(F)) / cap))
    out = torch.zeros(n, H, dv, dtype=F)
    for hh in range(H):
        S = torch.zeros(d, dv, dtype=F)
        nv = torch.zeros(d, dtype=F)
        mm = 0.0
        for t in range(n):
            i_t, f_t = float(ig[t, hh]), float(fg[t, hh])
            m_new = max(f_t + mm, i_t)
            a, b = math.exp(f_t + mm - m_new), math.exp(i_t - m_new)
            S = a * S + b * torch.outer(k[t, hh], v[t, hh])
            nv = a * nv + b * k[t, hh]
            mm = m_new
            den = max(abs(float(nv @ q[t, hh])), math.exp(-mm)) + 1e-6
            out[t, hh] = (S.T @ q[t, hh]) / den
    o = rms(out, eps).reshape(n, H * dv) * w[p + ".norm"].to(F)
    o = o * torch.sigmoid(h @ w[p + ".g"].to(F).T)
    return o @ w[p + ".o"].to(F).T


def parallel_mixer(h, w, p, m, eps):
    return (m["left_scale"] * softmax_attention(h, w, p + ".left", m["left"], eps)
            + m["right_scale"] * matrix_memory(h, w, p + ".right", m["right"], eps))


def delta_mixer(h, w, p, m, eps):
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = Fn.silu(tconv(h @ w[p + ".q"].to(F).T, w[p + ".q.conv"].to(F))).reshape(n, G, d)
    k = Fn.silu(tconv(h @ w[p + ".k"].to(F).T, w[p + ".k.conv"].to(F))).reshape(n, G, d)
    v = Fn.silu(tconv(h @ w[p + ".v"].to(F).T, w[p + ".v.conv"].to(F))).reshape(n, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + ".b"].to(F).T)
    decay = torch.exp(-torch.exp(w[p + ".A_log"].to(F)) * Fn.softplus(h @ w[p + ".a"].to(F).T + w[p + ".dt_bias"].to(F)))
    out = torch.zeros(n, H, dv, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(d, dv, dtype=F)
        for t in range(n):
            S = decay[t, hh] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, hh] = S.T @ q[t, g]
    o = rms(out, eps) * w[p + ".norm"].to(F)
    o = o.reshape(n, H * dv) * Fn.silu(h @ w[p + ".g"].to(F).T)
    return o @ w[p + ".o"].to(F).T


def clamp_glu(x, w, p, limit):
    g = torch.clamp(x @ w[p + ".gate"].to(F).T, max=limit)
    u = torch.clamp(x @ w[p + ".up"].to(F).T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + ".down"].to(F).T


def router(x, w, p, top):
    """(experts [n, top], weights [n, top]): softmax over all experts, the `top` largest, not renormalised"""
    s = torch.softmax(x @ w[p + ".router"].to(F).T, -1)
    val, idx = torch.topk(s, top, dim=-1)
    return idx, val


def routed_ff(x, w, p, mlp):
    idx, val = router(x, w, p, mlp["router"]["top"])
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for c in range(idx.shape[1]):
            e = int(idx[t, c])
            out[t] += val[t, c] * clamp_glu(x[t:t + 1], w, "%s.e%d" % (p, e), mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        out = out + clamp_glu(x, w, p + ".shared", mlp["shared"]["limit"])
    return out


def feed_forward(x, w, p, mlp):
    if mlp["kind"] == "dense":
        return clamp_glu(x, w, p, mlp["limit"])
    return routed_ff(x, w, p, mlp)


def mixer(h, w, p, layer, eps):
    if layer["type"] == "delta":
        return delta_mixer(h, w, p, layer["mixer"], eps)
    return parallel_mixer(h, w, p, layer["mixer"], eps)


def forward(cfg, w, tokens, return_hidden=False):
    """logits [n, vocab] (and the stream after every layer, [layers, n, D]) of one sequence"""
    eps, G = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x = w["embed"].to(F)[torch.as_tensor(tokens, dtype=torch.long)]
    stack, hidden = [x], []
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d" % i
        h = x + tconv(x, w[p + ".canon1"].to(F))
        x = x + grms(mixer(h, w, p + ".mix", layer, eps), w[p + ".norm1"].to(F), G, eps)
        if layer.get("mlp"):
            x = x + grms(feed_forward(x, w, p + ".mlp", layer["mlp"]), w[p + ".norm2"].to(F), G, eps)
        stack.append(x)
        dwa = w[p + ".dwa"].to(F)
        x = sum(dwa[j] * stack[j] for j in range(i + 2))
        hidden.append(x)
    logits = grms(x, w["final.norm"].to(F), G, eps) @ w["embed"].to(F).T
    return (logits, torch.stack(hidden)) if return_hidden else logits
