"""Plain, slow restatement of the Duguzen decoder (TEST INFRASTRUCTURE ONLY; nothing in pegainfer_amd/ imports it).

One function per mechanism, whole sequences at once, float64 on the CPU, no cache: every position is recomputed from
the full prefix, so a product path that keeps a latent cache, pages and batches can be compared with something that has
none of them.

Notation (one sequence of n tokens, residual width D):
  dyt(x; a, w, b)      = tanh(a x) * w + b                                  (no mean, no variance)
  layer                : x <- x + dyt_1b(mixer(dyt_1(x)));  x <- x + dyt_2b(ff(dyt_2(x)))   (second half only with an ff)
  latent attention     : q = Wq h, per head [dn | dr];  Wdkv h = [c_raw (r) | kr_raw (dr)];  c = rms(c_raw) * w_c
                         k_h = Wuk_h c, v_h = Wuv_h c;  score_ij = (qn_i . k_j + rope(qr_i) . rope(kr_j)) * scale, j <= i
                         out_h = softmax(score) v * sigmoid(Wg h)_h;  y = Wo concat(out_h)
  rope (rotate half)   : over the first R of the rotated dims, pair (i, i + R/2), angle p * base^(-2i/R)
  dense ff             : Wdown relu(Wup h)^2
  routed ff            : s = sigmoid(Wr h); choice = s + corr; groups of neighbours scored by their two largest choices,
                         only the best `keep` groups stay eligible; the `top` largest eligible choices are taken;
                         y = sum_e s_e * Wdown_e (silu(Wgate_e h) * Wup_e h)
"""
import json
import math
import os

import torch

F = torch.float64


def read_config(path):
    with open(path if path.endswith(".json") else os.path.join(path, "config.json")) as f:
        return json.load(f)


def owner(cfg, i):
    """index of the layer whose tensors layer i computes with"""
    for _ in range(len(cfg["layers"])):
        j = cfg["layers"][i].get("weights_of")
        if j is None or int(j) == i:
            return i
        i = int(j)
    raise ValueError("weights_of forms a cycle")


def dyt(x, w, name):
    return torch.tanh(w[name + ".alpha"].to(F) * x) * w[name].to(F) + w[name + ".b"].to(F)


def rms(x, weight, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def rope_half(x, pos, base, dims):
    """x [n, ..., d]; the first `dims` of d are rotated in (i, i + dims/2) pairs, the rest pass through"""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    ang = pos.to(F)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang).reshape(shape), torch.sin(ang).reshape(shape)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def latent_attention(h, w, p, mx, eps, pos):
    """h [n, D] -> [n, D]; p = tensor prefix '<layer>.mix', mx = the mixer's config"""
    n = h.shape[0]
    H, dn, dr, dv, r = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    base, rd = float(mx["rot"]["base"]), int(mx["rot"]["dims"])
    q = (h @ w[p + ".q"].to(F).T).reshape(n, H, dn + dr)
    dkv = h @ w[p + ".dkv"].to(F).T
    c = rms(dkv[:, :r], w[p + ".dkv.norm"].to(F), eps)
    kr = rope_half(dkv[:, r:], pos, base, rd)                     # [n, dr], shared by the heads
    qn, qr = q[..., :dn], rope_half(q[..., dn:], pos, base, rd)
    k = (c @ w[p + ".uk"].to(F).T).reshape(n, H, dn)
    v = (c @ w[p + ".uv"].to(F).T).reshape(n, H, dv)
    score = (torch.einsum("ihd,jhd->hij", qn, k) + torch.einsum("ihd,jd->hij", qr, kr)) * float(mx["scale"])
    mask = pos[None, :] > pos[:, None]
    score = score.masked_fill(mask[None], -math.inf)
    out = torch.einsum("hij,jhd->ihd", torch.softmax(score, -1), v)
    gate = torch.sigmoid(h @ w[p + ".g"].to(F).T)                  # [n, H]
    out = out * gate[..., None]
    return out.reshape(n, H * dv) @ w[p + ".o"].to(F).T


def dense_ff(h, w, p):
    return torch.relu(h @ w[p + ".up"].to(F).T) ** 2 @ w[p + ".down"].to(F).T


def route(h, w, p, rt):
    """-> (chosen expert ids [n, top], their weights [n, top])"""
    E, top = int(rt["experts"]), int(rt["top"])
    s = torch.sigmoid(h @ w[p + ".router"].to(F).T)
    choice = s + w[p + ".correction"].to(F) if (p + ".correction") in w else s.clone()
    g = rt.get("groups")
    if g and int(g["count"]) > 1:
        G, keep = int(g["count"]), int(g["keep"])
        per = choice.reshape(-1, G, E // G)
        gscore = per.topk(min(2, E // G), -1).values.sum(-1)
        kept = gscore.topk(keep, -1).indices
        ok = torch.zeros_like(gscore, dtype=torch.bool).scatter_(1, kept, True)
        choice = choice.masked_fill(~ok[..., None].expand_as(per).reshape(-1, E), -math.inf)
    idx = choice.topk(top, -1).indices
    return idx, s.gather(1, idx)


def routed_ff(h, w, p, mlp):
    idx, wt = route(h, w, p, mlp["router"])
    y = torch.zeros(h.shape[0], w[p + ".e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), wt[t]):
            pe = "%s.e%d" % (p, e)
            z = h[t] @ w[pe + ".gate"].to(F).T
            y[t] += a * ((z * torch.sigmoid(z)) * (h[t] @ w[pe + ".up"].to(F).T)) @ w[pe + ".down"].to(F).T
    return y


def forward(cfg, w, tokens, taps=None):
    """tokens: list of ids of ONE sequence -> logits [n, vocab] (float64); taps (a list) receives the residual stream
    after every layer run"""
    eps = float(cfg["norm"]["eps"])
    tok = torch.as_tensor(tokens, dtype=torch.long)
    pos = torch.arange(len(tokens))
    x = w["embed"].to(F)[tok]
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d" % owner(cfg, i)
        if layer["type"] != "latent_attention":
            raise ValueError("unknown mixer " + layer["type"])
        x = x + dyt(latent_attention(dyt(x, w, p + ".norm1"), w, p + ".mix", layer["mixer"], eps, pos), w, p + ".norm1b")
        mlp = layer.get("mlp")
        if mlp:
            hin = dyt(x, w, p + ".norm2")
            y = dense_ff(hin, w, p + ".mlp") if mlp["kind"] == "dense" else routed_ff(hin, w, p + ".mlp", mlp)
            x = x + dyt(y, w, p + ".norm2b")
        if taps is not None:
            taps.append(x.clone())
    return dyt(x, w, "final.norm") @ w["head"].to(F).T


def load_weights(path):
    """safetensors file or folder -> {name: torch tensor} (bf16 values widened to float32, int tables as int32)"""
    from safetensors import safe_open
    if os.path.isdir(path):
        path = os.path.join(path, "model.safetensors")
    out = {}
    with safe_open(path, "pt") as f:
        for k in f.keys():
            t = f.get_tensor(k)
            out[k] = t.float() if t.is_floating_point() else t
    return out
