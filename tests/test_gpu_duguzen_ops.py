"""Each Duguzen mechanism alone on the GPU against the plain restatement (oracle/duguzen_ref.py) or a direct torch fp32 /
fp64 formula: Dynamic-Tanh norms, the strided / batched / grouped GEMM, latent prep (RMS norm + rotation + cache write), the
latent attention (pages, key splits, crafted far keys), the grouped sigmoid router, expert sorting and combine."""
import math

import numpy as np
import pytest
import torch

import duguzen_common as C
from oracle import duguzen_ref as R

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dev(t, dtype=None):
    t = torch.as_tensor(t)
    return (t.to(dtype) if dtype else t).cuda().contiguous()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_dyt_norm_and_fused_boundary(dtype):
    from pegainfer_amd import ops_blocks as B
    g = torch.Generator().manual_seed(0)
    rows, d = 37, 52
    x = torch.randn(rows, d, generator=g) * 3
    y = C.bf16_round(torch.randn(rows, d, generator=g) * 2)
    P = [C.bf16_round(v) for v in (torch.tensor(0.7), 1 + 0.2 * torch.randn(d, generator=g), 0.1 * torch.randn(d, generator=g))]
    N = [C.bf16_round(v) for v in (torch.tensor(0.4), 1 + 0.2 * torch.randn(d, generator=g), 0.1 * torch.randn(d, generator=g))]
    td = DT[dtype]
    ref1 = torch.tanh(P[0].double() * x.double()) * P[1].double() + P[2].double()
    got1 = B.dyt_norm(dev(x), *[dev(v, td) for v in P]).float().cpu()
    tol = 1e-6 if dtype == "float32" else 1e-2
    assert (got1.double() - ref1).abs().max() < tol
    xs = dev(x)
    got2 = B.dyt_add_norm(xs, dev(y, td), [dev(v, td) for v in P], [dev(v, td) for v in N]).float().cpu()
    x2 = x.double() + torch.tanh(P[0].double() * y.double()) * P[1].double() + P[2].double()
    assert (xs.cpu().double() - x2).abs().max() < 2e-6            # the residual sum is fp32 in both instances
    ref2 = torch.tanh(N[0].double() * x2) * N[1].double() + N[2].double()
    assert (got2.double() - ref2).abs().max() < tol
    xs2 = dev(x)
    assert B.dyt_add_norm(xs2, dev(y, td), [dev(v, td) for v in P]) is None
    assert torch.equal(xs2, xs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_strided_gemm_dense_batched_transposed(dtype):
    from pegainfer_amd import ops_blocks as B
    g = torch.Generator().manual_seed(1)
    td = DT[dtype]
    for (T, M, K) in [(1, 5, 3), (70, 66, 50), (64, 64, 16), (130, 7, 129)]:
        x, w = C.bf16_round(torch.randn(T, K, generator=g)), C.bf16_round(torch.randn(M, K, generator=g))
        got = B.linear(dev(x, td), dev(w, td), out_dtype=torch.float32).cpu()
        assert (got.double() - x.double() @ w.double().T).abs().max() < 1e-4 * K
        sq = B.linear(dev(x, td), dev(w, td), out_dtype=torch.float32, epilogue=B.EPI_RELU_SQ).cpu()
        assert (sq.double() - torch.relu(x.double() @ w.double().T) ** 2).abs().max() < 1e-3 * K
    # per-head product over slices of a wider row with the weight read transposed, then one with a sigmoid gate
    T, H, dn, dr, r = 9, 3, 10, 6, 14
    row = C.bf16_round(torch.randn(T, H * (dn + dr) + 5, generator=g))
    uk = C.bf16_round(torch.randn(H * dn, r, generator=g))
    qc = torch.zeros(T, H, r + dr, device="cuda")
    xd, wd = dev(row, td), dev(uk, td)
    d = B.GemmDesc(x=xd.data_ptr(), w=wd.data_ptr(), y=qc.data_ptr(), x_dtype=B._dt(xd), w_dtype=B._dt(wd), y_dtype=1, m=r,
                   k=dn, rows=T, groups=H, x_row_stride=row.shape[1], x_group_stride=dn + dr, w_m_stride=1, w_k_stride=r,
                   w_group_stride=dn * r, y_row_stride=H * (r + dr), y_group_stride=r + dr)
    B.gemm_strided(d)
    q = row[:, :H * (dn + dr)].reshape(T, H, dn + dr)[..., :dn].double()
    ref = torch.einsum("thd,hdr->thr", q, uk.double().reshape(H, dn, r))
    assert (qc.cpu()[..., :r].double() - ref).abs().max() < 1e-4 and float(qc[..., r:].abs().max()) == 0.0
    gate = C.bf16_round(torch.randn(T, H + 2, generator=g))
    ol, uv = torch.randn(T, H, r, generator=g), C.bf16_round(torch.randn(H * 7, r, generator=g))
    out = torch.zeros(T, H * 7, device="cuda", dtype=td)
    old, uvd, gd = dev(ol), dev(uv, td), dev(gate, td)
    d = B.GemmDesc(x=old.data_ptr(), w=uvd.data_ptr(), y=out.data_ptr(), x_dtype=1, w_dtype=B._dt(uvd), y_dtype=B._dt(out), m=7,
                   k=r, rows=T, groups=H, x_row_stride=H * r, x_group_stride=r, w_m_stride=r, w_k_stride=1, w_group_stride=7 * r,
                   y_row_stride=H * 7, y_group_stride=7, epilogue=B.EPI_SIGMOID_GATE, gate=gd.data_ptr() + 2 * gd.element_size(),
                   gate_dtype=B._dt(gd), gate_row_stride=H + 2)
    B.gemm_strided(d)
    ref = torch.einsum("thr,hvr->thv", ol.double(), uv.double().reshape(H, 7, r)) * torch.sigmoid(gate[:, 2:].double())[..., None]
    assert (out.float().cpu().double().reshape(T, H, 7) - ref).abs().max() < (1e-4 if dtype == "float32" else 0.05)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_router_matches_the_plain_rule(dtype):
    from pegainfer_amd import ops_blocks as B
    td = DT[dtype]
    g = torch.Generator().manual_seed(2)
    cases = [(12, 4, 3, 4), (16, 4, 3, 4), (6, 3, 2, 2), (5, 1, 1, 1), (4, 4, 4, 3), (8, 8, 3, 2), (9, 3, 1, 3)]
    for (E, G, keep, top) in cases:
        d = 40
        h = C.bf16_round(torch.randn(33, d, generator=g))
        w = {"r.router": C.bf16_round(torch.randn(E, d, generator=g) * 0.5),
             "r.correction": C.bf16_round(torch.randn(E, generator=g) - 0.8)}
        rt = {"experts": E, "top": top, "groups": {"count": G, "keep": keep}}
        idx, wt = R.route(h.double(), w, "r", rt)
        e, ww = B.route(dev(h, td), dev(w["r.router"], td), dev(w["r.correction"], td), G, keep, top)
        assert torch.equal(e.cpu().long(), idx), (E, G, keep, top)
        assert (ww.cpu().double() - wt).abs().max() < 1e-5
        e2, _ = B.route(dev(h, td), dev(w["r.router"], td), None, G, keep, top)      # no correction: choose by the scores
        idx2, _ = R.route(h.double(), {"r.router": w["r.router"]}, "r", rt)
        assert torch.equal(e2.cpu().long(), idx2)


def test_expert_sort_grouped_gemm_and_combine():
    from pegainfer_amd import ops_blocks as B
    g = torch.Generator().manual_seed(3)
    rows, top, E, d, ff = 150, 3, 5, 24, 10          # expert 4 gets > 64 pairs (two tiles), expert 3 none
    expert = torch.randint(0, 3, (rows, top), generator=g, dtype=torch.int32)
    expert[:, 2] = 4
    pos_pair, pos_row, tg, t0, tr, nt, max_tiles = B.route_sort(expert.cuda(), E)
    n = int(nt.item())
    pp, tgc, t0c, trc = pos_pair.cpu(), tg.cpu()[:n], t0.cpu()[:n], tr.cpu()[:n]
    assert sorted(pp.tolist()) == list(range(rows * top)) and torch.equal(pos_row.cpu(), pp // top)
    assert int(trc.sum()) == rows * top and int(trc.max()) <= 64 and 3 not in tgc.tolist()
    for i in range(n):
        assert all(int(expert.reshape(-1)[pp[p]]) == int(tgc[i]) for p in range(int(t0c[i]), int(t0c[i] + trc[i])))
    x = C.bf16_round(torch.randn(rows, d, generator=g))
    w = C.bf16_round(torch.randn(E, ff, d, generator=g))
    y = torch.zeros(rows * top, ff, device="cuda")
    xd, wd = dev(x, torch.bfloat16), dev(w, torch.bfloat16)
    dsc = B.GemmDesc(x=xd.data_ptr(), w=wd.data_ptr(), y=y.data_ptr(), x_dtype=0, w_dtype=0, y_dtype=1, m=ff, k=d,
                     x_row_stride=d, w_m_stride=d, w_k_stride=1, w_group_stride=ff * d, y_row_stride=ff,
                     tile_group=tg.data_ptr(), tile_row0=t0.data_ptr(), tile_rows=tr.data_ptr(), n_tiles=nt.data_ptr(),
                     max_tiles=max_tiles, x_row_index=pos_row.data_ptr(), y_row_index=pos_pair.data_ptr())
    B.gemm_strided(dsc)
    ref = torch.einsum("pd,pfd->pf", x.double().repeat_interleave(top, 0), w.double()[expert.reshape(-1).long()])
    assert (y.cpu().double() - ref).abs().max() < 1e-4
    wt = torch.rand(rows, top, generator=g)
    out = B.route_combine(y, wt.cuda(), torch.float32).cpu()
    assert (out.double() - (ref.reshape(rows, top, ff) * wt.double()[..., None]).sum(1)).abs().max() < 1e-4


def _paged(entries, page_size, dtype, perm_seed=0):
    """entries [n, E] -> (cache tensor, page ids) with the pages in a scrambled order inside a larger pool"""
    n, E = entries.shape
    npages = (n + page_size - 1) // page_size
    pool = npages + 3
    order = np.random.default_rng(perm_seed).permutation(pool)[:npages]
    cache = torch.zeros(pool, page_size, E)
    for j in range(n):
        cache[order[j // page_size], j % page_size] = entries[j]
    return dev(cache, dtype), torch.tensor(order, dtype=torch.int32).cuda()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_latent_prep_norm_rotation_and_cache_write(dtype):
    from pegainfer_amd import ops_blocks as B
    td = DT[dtype]
    g = torch.Generator().manual_seed(4)
    H, dn, dr, r, rd, ps, base, eps = 3, 10, 12, 20, 8, 16, 777.0, 1e-5
    T, start = 21, 27                                   # positions 27 .. 47: the portion starts inside a page
    proj = C.bf16_round(torch.randn(T, H * (dn + dr) + r + dr + H, generator=g))
    cw = C.bf16_round(1 + 0.2 * torch.randn(r, generator=g))
    pos = torch.arange(start, start + T)
    E = r + dr
    cache, pages = _paged(torch.zeros(start + T, E), ps, td)
    inv = torch.tensor([base ** (-2.0 * i / rd) for i in range(rd // 2)], dtype=torch.float32).cuda()
    qc = torch.zeros(T, H, E, device="cuda")
    B.latent_prep(dev(proj, td), H * (dn + dr), dev(cw, td), eps, inv, rd, pos.int().cuda(), torch.zeros(T, dtype=torch.int32).cuda(),
                  torch.tensor([0, len(pages)], dtype=torch.int32).cuda(), pages, cache, ps * E, 0, ps, qc, H, dn, dr, r)
    dkv = proj[:, H * (dn + dr):H * (dn + dr) + E].double()
    c_ref = R.rms(dkv[:, :r], cw.double(), eps)
    kr_ref = R.rope_half(dkv[:, r:], pos, base, rd)
    q_ref = R.rope_half(proj[:, :H * (dn + dr)].double().reshape(T, H, dn + dr)[..., dn:], pos, base, rd)
    flat = cache.float().cpu()
    got = torch.stack([flat[int(pages[p // ps]), p % ps] for p in range(start, start + T)]).double()
    tol = 2e-5 if dtype == "float32" else 2e-2
    assert (got[:, :r] - c_ref).abs().max() < tol and (got[:, r:] - kr_ref).abs().max() < tol
    assert (qc.cpu()[..., r:].double() - q_ref).abs().max() < 2e-5          # the query side stays fp32
    untouched = torch.stack([flat[int(pages[p // ps]), p % ps] for p in range(start)])
    assert float(untouched.abs().max()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n_keys", [1, 17, 256, 257, 1024, 1025, 1300])
def test_latent_attention_matches_softmax(dtype, n_keys):
    from pegainfer_amd import ops_blocks as B
    td = DT[dtype]
    g = torch.Generator().manual_seed(n_keys)
    H, r, dr, ps = 3, 24, 8, 16
    E = r + dr
    entries = C.bf16_round(torch.randn(n_keys, E, generator=g))
    cache, pages = _paged(entries, ps, td, perm_seed=n_keys)
    rows = sorted({0, n_keys // 2, n_keys - 1})
    qc = torch.randn(len(rows), H, E, generator=g)
    o = B.latent_attention(dev(qc), cache, ps * E, 0, ps, torch.tensor(rows, dtype=torch.int32).cuda(),
                           torch.zeros(len(rows), dtype=torch.int32).cuda(), torch.tensor([0, len(pages)], dtype=torch.int32).cuda(),
                           pages, r, dr, 0.3, n_keys).cpu()
    for i, p in enumerate(rows):
        s = torch.einsum("he,je->hj", qc[i].double(), entries[:p + 1].double()) * 0.3
        ref = torch.softmax(s, -1) @ entries[:p + 1, :r].double()
        assert (o[i].double() - ref).abs().max() < 2e-5, (n_keys, p)


@pytest.mark.parametrize("far", [0, 15, 16, 255, 256, 1023, 1024, 1100])
def test_one_far_key_stands_out(far):
    """one key is made to dominate the softmax: the output must be that key's latent, wherever it sits - the first token,
    either side of a page border, of a round of keys and of a key split - and must ignore it when it is not yet visible"""
    from pegainfer_amd import ops_blocks as B
    g = torch.Generator().manual_seed(far)
    n, H, r, dr, ps = 1200, 2, 16, 8, 16
    E = r + dr
    entries = C.bf16_round(torch.randn(n, E, generator=g) * 0.2)
    probe = torch.zeros(E)
    probe[3], probe[r + 1] = 8.0, 8.0
    entries[far] = probe
    cache, pages = _paged(entries, ps, torch.float32, perm_seed=far)
    qc = torch.zeros(3, H, E)
    qc[:, :, 3] = qc[:, :, r + 1] = 4.0
    rows = [n - 1, far, max(far - 1, 0)]                # sees it from afar, sees it as its own position, does not see it
    o = B.latent_attention(dev(qc), cache, ps * E, 0, ps, torch.tensor(rows, dtype=torch.int32).cuda(),
                           torch.zeros(3, dtype=torch.int32).cuda(), torch.tensor([0, len(pages)], dtype=torch.int32).cuda(),
                           pages, r, dr, 1.0, n).cpu()
    assert (o[0] - probe[:r]).abs().max() < 1e-3 and (o[1] - probe[:r]).abs().max() < 1e-3
    if far > 0:
        assert float(o[2][:, 3].abs().max()) < 1.0


def test_latent_attention_rows_of_several_requests():
    from pegainfer_amd import ops_blocks as B
    g = torch.Generator().manual_seed(9)
    H, r, dr, ps = 2, 8, 4, 16
    E = r + dr
    lens = [40, 3, 17]
    ent = [C.bf16_round(torch.randn(n, E, generator=g)) for n in lens]
    pool = torch.zeros(12, ps, E)
    page_lists, nxt = [], 11
    for e in ent:                                        # pages handed out from the top, interleaved between requests
        pl = []
        for j in range(0, len(e), ps):
            pool[nxt, :len(e[j:j + ps])] = e[j:j + ps]
            pl.append(nxt)
            nxt -= 1
        page_lists.append(pl)
    indptr = np.cumsum([0] + [len(p) for p in page_lists]).astype(np.int32)
    rows = [(0, 39), (1, 0), (2, 16), (0, 15), (1, 2), (2, 15), (0, 16)]
    qc = torch.randn(len(rows), H, E, generator=g)
    o = B.latent_attention(dev(qc), dev(pool, torch.bfloat16), ps * E, 0, ps, torch.tensor([p for _, p in rows], dtype=torch.int32).cuda(),
                           torch.tensor([q for q, _ in rows], dtype=torch.int32).cuda(), torch.tensor(indptr).cuda(),
                           torch.tensor(sum(page_lists, []), dtype=torch.int32).cuda(), r, dr, 0.5, 40).cpu()
    for i, (q, p) in enumerate(rows):
        s = torch.einsum("he,je->hj", qc[i].double(), ent[q][:p + 1].double()) * 0.5
        assert (o[i].double() - torch.softmax(s, -1) @ ent[q][:p + 1, :r].double()).abs().max() < 2e-5


@pytest.mark.parametrize("split_keys", [0, 128])
@pytest.mark.parametrize("shape", [(3, 32, 8, [70, 1, 9]), (8, 64, 32, [300, 2]), (5, 16, 16, [13, 13, 1, 1]), (16, 128, 64, [5, 40])])
def test_latent_attention_matrix_core_form(shape, split_keys):
    """the tiled bf16 form against the direct softmax: several requests in one launch, portions that start deep inside a
    context, tiles that end inside an entry, key splits; q and the weights are rounded to bf16 inside, hence the tolerance"""
    from pegainfer_amd import ops_blocks as B
    H, r, dr, lens = shape
    g = torch.Generator().manual_seed(H * 100 + r)
    E, ps = r + dr, 16
    starts = [0 if i % 2 == 0 else 137 for i in range(len(lens))]          # odd entries continue a context of 137 tokens
    ctx = [s + n for s, n in zip(starts, lens)]
    ent = [C.bf16_round(torch.randn(n, E, generator=g) * 0.7) for n in ctx]
    npages = [(n + ps - 1) // ps for n in ctx]
    pool = torch.zeros(sum(npages) + 2, ps, E)
    order = np.random.default_rng(H).permutation(sum(npages) + 2)
    page_lists, at = [], 0
    for e, k in zip(ent, npages):
        pl = [int(x) for x in order[at:at + k]]
        at += k
        for j in range(len(e)):
            pool[pl[j // ps], j % ps] = e[j]
        page_lists.append(pl)
    indptr = np.cumsum([0] + npages).astype(np.int32)
    pos = [s + k for s, n in zip(starts, lens) for k in range(n)]
    req = [i for i, n in enumerate(lens) for _ in range(n)]
    T = len(pos)
    qc = torch.randn(T, H, E, generator=g)
    assert ffi_ok(B, r, dr, ps * E)
    args = (dev(pool, torch.bfloat16), ps * E, 0, ps, torch.tensor(pos, dtype=torch.int32).cuda(), torch.tensor(req, dtype=torch.int32).cuda(),
            torch.tensor(indptr).cuda(), torch.tensor(sum(page_lists, []), dtype=torch.int32).cuda(), r, dr, 0.25, max(ctx))
    o = B.latent_attention(dev(qc), *args, split_keys=split_keys, tiles=B.row_tiles(lens, H)).cpu()
    plain = B.latent_attention(dev(qc), *args, split_keys=split_keys).cpu()
    for i in range(T):
        e = ent[req[i]][:pos[i] + 1].double()
        ref = torch.softmax(torch.einsum("he,je->hj", qc[i].double(), e) * 0.25, -1) @ e[:, :r]
        assert (plain[i].double() - ref).abs().max() < 2e-5, i
        assert (o[i].double() - ref).abs().max() < 2.5e-2, (i, pos[i], float((o[i].double() - ref).abs().max()))
    assert float((o - plain).abs().mean()) < 2e-3


def ffi_ok(B, r, dr, page_stride):
    from pegainfer_amd import ffi
    return ffi.lib().pegainfer_latent_attention_tiled_ok(r, dr, page_stride, 0, 0) == 1


def test_matrix_core_form_sees_a_far_key_and_masks_an_unseen_one():
    from pegainfer_amd import ops_blocks as B
    for far in (0, 31, 32, 127, 128, 700):
        g = torch.Generator().manual_seed(far)
        n, H, r, dr, ps = 800, 8, 16, 16, 16
        E = r + dr
        entries = C.bf16_round(torch.randn(n, E, generator=g) * 0.2)
        probe = torch.zeros(E)
        probe[3], probe[r + 1] = 8.0, 8.0
        entries[far] = probe
        cache, pages = _paged(entries, ps, torch.bfloat16, perm_seed=far)
        lo = max(far - 1, 0)
        T = n - lo                                       # one portion: positions lo .. n-1
        qc = torch.zeros(T, H, E)
        qc[:, :, 3] = qc[:, :, r + 1] = 4.0
        o = B.latent_attention(dev(qc), cache, ps * E, 0, ps, torch.arange(lo, n, dtype=torch.int32).cuda(),
                               torch.zeros(T, dtype=torch.int32).cuda(), torch.tensor([0, len(pages)], dtype=torch.int32).cuda(),
                               pages, r, dr, 1.0, n, split_keys=128, tiles=B.row_tiles([T], H)).cpu()
        seen = o[far - lo:]
        assert (seen - probe[:r]).abs().max() < 2e-2, far
        if far > 0:
            assert float(o[0][:, 3].abs().max()) < 1.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_strided_gemm_forms_agree(dtype):
    """the few-rows form (<= 8 rows), the matrix-core tile form (bf16 weights) and the fp32-FMA tile form compute the same
    products of the stored values; only the order of the fp32 sums differs"""
    from pegainfer_amd import ops_blocks as B
    td = DT[dtype]
    g = torch.Generator().manual_seed(7)
    for (T, M, K) in [(1, 96, 128), (4, 33, 256), (7, 40, 64), (8, 200, 1024), (9, 40, 64), (70, 130, 192), (64, 64, 64), (200, 72, 320)]:
        x, w = C.bf16_round(torch.randn(T, K, generator=g)), C.bf16_round(torch.randn(M, K, generator=g))
        ref = x.double() @ w.double().T
        for epi in (B.EPI_NONE, B.EPI_RELU_SQ):
            want = ref if epi == B.EPI_NONE else torch.relu(ref) ** 2
            fast = B.linear(dev(x, td), dev(w, td), out_dtype=torch.float32, epilogue=epi).cpu()
            plain = B.linear(dev(x, td), dev(w, td), out_dtype=torch.float32, epilogue=epi, plain=True).cpu()
            tol = 2e-5 * K * (1 if epi == B.EPI_NONE else 10)
            assert (fast.double() - want).abs().max() < tol and (plain.double() - want).abs().max() < tol, (T, M, K, epi)
    # grouped rows with a small bound on the rows per tile: the few-rows form walks the same tile table
    rows, top, E, d, ff = 5, 2, 6, 64, 24
    expert = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(rows)]).int()
    pos_pair, pos_row, tg, t0, tr, nt, max_tiles = B.route_sort(expert.cuda(), E)
    x, w = C.bf16_round(torch.randn(rows, d, generator=g)), C.bf16_round(torch.randn(E, ff, d, generator=g))
    xd, wd = dev(x, td), dev(w, td)
    outs = []
    for plain in (0, 1):
        y = torch.zeros(rows * top, ff, device="cuda")
        B.gemm_strided(B.GemmDesc(x=xd.data_ptr(), w=wd.data_ptr(), y=y.data_ptr(), x_dtype=B._dt(xd), w_dtype=B._dt(wd), y_dtype=1,
                                  m=ff, k=d, x_row_stride=d, w_m_stride=d, w_k_stride=1, w_group_stride=ff * d, y_row_stride=ff,
                                  tile_group=tg.data_ptr(), tile_row0=t0.data_ptr(), tile_rows=tr.data_ptr(), n_tiles=nt.data_ptr(),
                                  max_tiles=max_tiles, x_row_index=pos_row.data_ptr(), y_row_index=pos_pair.data_ptr(),
                                  max_tile_rows=rows, plain=plain))
        outs.append(y.cpu())
    ref = torch.einsum("pd,pfd->pf", x.double().repeat_interleave(top, 0), w.double()[expert.reshape(-1).long()])
    assert (outs[0].double() - ref).abs().max() < 1e-4 and (outs[1].double() - ref).abs().max() < 1e-4


def test_grouped_gemm_over_128_row_tiles():
    from pegainfer_amd import ops_blocks as B
    g = torch.Generator().manual_seed(11)
    rows, top, E, d, ff = 400, 2, 3, 64, 136         # ~267 pairs per expert: two full 128-row tiles and a part of a third
    expert = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(rows)]).int()
    pos_pair, pos_row, tg, t0, tr, nt, max_tiles = B.route_sort(expert.cuda(), E, rows_per_tile=128)
    assert int(tr.cpu()[:int(nt.item())].max()) == 128
    x, w = C.bf16_round(torch.randn(rows, d, generator=g)), C.bf16_round(torch.randn(E, ff, d, generator=g))
    xd, wd = dev(x, torch.bfloat16), dev(w, torch.bfloat16)
    y = torch.zeros(rows * top, ff, device="cuda")
    B.gemm_strided(B.GemmDesc(x=xd.data_ptr(), w=wd.data_ptr(), y=y.data_ptr(), x_dtype=0, w_dtype=0, y_dtype=1, m=ff, k=d,
                              x_row_stride=d, w_m_stride=d, w_k_stride=1, w_group_stride=ff * d, y_row_stride=ff,
                              tile_group=tg.data_ptr(), tile_row0=t0.data_ptr(), tile_rows=tr.data_ptr(), n_tiles=nt.data_ptr(),
                              max_tiles=max_tiles, x_row_index=pos_row.data_ptr(), y_row_index=pos_pair.data_ptr(),
                              tile_rows_cap=128))
    ref = torch.einsum("pd,pfd->pf", x.double().repeat_interleave(top, 0), w.double()[expert.reshape(-1).long()])
    assert (y.cpu().double() - ref).abs().max() < 1e-4
    with pytest.raises(RuntimeError):                 # the 64-row fp32-FMA form refuses a table cut for 128-row tiles
        B.gemm_strided(B.GemmDesc(x=xd.data_ptr(), w=wd.data_ptr(), y=y.data_ptr(), x_dtype=0, w_dtype=0, y_dtype=1, m=ff, k=d,
                                  x_row_stride=d, w_m_stride=d, w_k_stride=1, w_group_stride=ff * d, y_row_stride=ff,
                                  tile_group=tg.data_ptr(), tile_row0=t0.data_ptr(), tile_rows=tr.data_ptr(),
                                  n_tiles=nt.data_ptr(), max_tiles=max_tiles, x_row_index=pos_row.data_ptr(),
                                  y_row_index=pos_pair.data_ptr(), tile_rows_cap=128, plain=1))
