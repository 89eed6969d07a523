"""Every Feruzen mechanism alone on the GPU (torch wrappers of pegainfer_amd/ops_blocks.py over the HIP blocks) against its
function in the plain restatement (oracle/feruzen_ref.py), in both storage types; and crafted inputs where random weights
would hide a fault: one far write among hundreds that a memory has to give back, one far key whose score stands out, keys
on both sides of page and key-tile borders, state regions used by another request before."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as Fn

import feruzen_common as C
from oracle import feruzen_ref as R

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F = torch.float64


def dev(t, dtype):
    return t.to(DT[dtype]).cuda().contiguous()


def close(got, ref, dtype, tol32=2e-5, tol16=3e-2):
    got, ref = got.detach().double().cpu(), ref.double()
    err = float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-9))
    assert err < (tol32 if dtype == "float32" else tol16), err


def B():
    from pegainfer_amd import ops_blocks
    return ops_blocks


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("taps", [1, 2, 5])
def test_time_convolution_carries_its_tail_through_portions_and_slots(dtype, taps):
    g = torch.Generator().manual_seed(taps)
    Cn = 70
    w = C.bf16_round(torch.randn(Cn, taps, generator=g))
    seqs = [C.bf16_round(torch.randn(n, Cn, generator=g)) for n in (23, 9)]
    refs = [x.double() + R.tconv(x.double(), w.double()) for x in seqs]
    state = torch.full((3, max(taps - 1, 1), Cn), 7.0, device="cuda")      # dirty: slots 2 and 0 are zeroed for the new requests
    state[2].zero_()
    state[0].zero_()
    plans = [[(0, 1), (1, 2)], [(0, 2), (1, 1)], [(0, 1), (1, 1)], [(0, 12)], [(0, 7), (1, 5)]]    # (sequence, rows) per step;
    # slots 2 and 0; the third step brings one row per entry: the decode form (output and tail in one launch)
    at, got = [0, 0], [[], []]
    for stp in plans:
        x = torch.cat([seqs[q][at[q]:at[q] + n] for q, n in stp])
        rg = B().Ragged([n for _, n in stp], slots=[2 if q == 0 else 0 for q, _ in stp])
        out = B().time_conv(dev(x, "float32"), dev(w, dtype), state if taps > 1 else state[:, :0], rg, residual=True,
                            out_dtype=torch.float32)
        off = 0
        for q, n in stp:
            got[q].append(out[off:off + n].cpu())
            at[q] += n
            off += n
    for q in range(2):
        close(torch.cat(got[q]), refs[q], "float32", tol32=1e-6)
    assert float(state[1].min()) == 7.0                                      # a slot no entry named is not touched
    x = dev(seqs[0], dtype)                                                  # the mixers' form: stored type in, silu, fp32 out
    state.zero_()
    out = B().time_conv(x, dev(w, dtype), state if taps > 1 else state[:, :0], B().Ragged([23]), silu=True, out_dtype=torch.float32)
    close(out, Fn.silu(R.tconv(seqs[0].double(), w.double())), "float32", tol32=1e-6)


@pytest.mark.parametrize("taps", [1, 3, 4, 7, 8, 9])
def test_time_convolution_over_long_portions(taps):
    """steps of a few hundred rows take the form with a sliding window in registers (up to 8 taps): entries that begin in the
    middle of a thread's walk, a tail carried into the second step, channels beyond a whole workgroup"""
    g = torch.Generator().manual_seed(taps)
    Cn = 300
    w = C.bf16_round(torch.randn(Cn, taps, generator=g))
    seqs = [C.bf16_round(torch.randn(n, Cn, generator=g)) for n in (333, 250, 40)]
    state = torch.zeros(3, max(taps - 1, 1), Cn, device="cuda")
    at, got = [0, 0, 0], [[], [], []]
    for stp in [[(0, 199), (1, 101), (2, 3)], [(2, 37), (0, 134), (1, 149)]]:
        x = torch.cat([seqs[q][at[q]:at[q] + n] for q, n in stp])
        rg = B().Ragged([n for _, n in stp], slots=[q for q, _ in stp])
        out = B().time_conv(dev(x, "bfloat16"), dev(w, "bfloat16"), state if taps > 1 else state[:, :0], rg, silu=True,
                            out_dtype=torch.float32)
        off = 0
        for q, n in stp:
            got[q].append(out[off:off + n].cpu())
            at[q] += n
            off += n
    for q in range(3):
        close(torch.cat(got[q]), Fn.silu(R.tconv(seqs[q].double(), w.double())), "float32", tol32=2e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mult", [1, 4])        # 4: rows and groups of whole fours take the vector form
@pytest.mark.parametrize("groups", [1, 3, 7])
def test_grouped_output_norm_residual_and_depth_sum(dtype, groups, mult):
    g = torch.Generator().manual_seed(groups)
    d, rows = mult * 42 * groups // math.gcd(42, groups), 9
    y, w = C.bf16_round(torch.randn(rows, d, generator=g) * 3), C.bf16_round(1 + 0.3 * torch.randn(d, generator=g))
    x = torch.randn(rows, d, generator=g)
    stack = torch.randn(3, rows, d, generator=g)
    coef = C.bf16_round(torch.randn(4, generator=g))
    r32, rb, mix = B().group_rms_add(dev(y, dtype), dev(w, dtype), groups, 1e-5, x=x.cuda(), stack=stack.cuda(), coef=dev(coef, dtype))
    ref = x.double() + R.grms(y.double(), w.double(), groups, 1e-5)
    close(r32, ref, "float32", tol32=2e-6)
    close(rb, ref, dtype)
    close(mix, sum(coef[j].double() * stack[j].double() for j in range(3)) + coef[3].double() * ref, "float32", tol32=2e-6)
    only, _, none = B().group_rms_add(dev(y, dtype), dev(w, dtype), groups, 1e-5)     # no residual, no sum: the final norm's form
    close(only, R.grms(y.double(), w.double(), groups, 1e-5), "float32", tol32=2e-6)
    assert none is None


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_clamp_glu(dtype):
    g = torch.Generator().manual_seed(1)
    gu = C.bf16_round(torch.randn(11, 2 * 37, generator=g) * 3)
    out = B().clamp_glu_rows(dev(gu, dtype), 1.25)
    ga, up = gu[:, :37].double().clamp(max=1.25), gu[:, 37:].double().clamp(-1.25, 1.25)
    close(out, ga * torch.sigmoid(1.702 * ga) * (up + 1), dtype)
    assert float(gu[:, :37].min()) < -1.25 and float(out.float().min()) < 0      # the gate is NOT clamped from below


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("experts,top", [(5, 1), (16, 3), (70, 4)])
def test_softmax_router(dtype, experts, top):
    g = torch.Generator().manual_seed(experts)
    h, wr = C.bf16_round(torch.randn(33, 48, generator=g)), C.bf16_round(torch.randn(experts, 48, generator=g) * 0.5)
    e, wt = B().route_topk(dev(h, dtype), dev(wr, dtype), top)
    idx, val = R.router(h.double(), {"r.router": wr}, "r", top)
    assert torch.equal(e.cpu().long().sort(-1).values, idx.sort(-1).values)
    close(wt.cpu().sort(-1).values, val.sort(-1).values, "float32", tol32=1e-5)
    assert float(wt.sum(-1).max()) < 1.0 or top == experts                       # the scores are not renormalised
    # the form the runtime uses: logits by a GEMM into fp32, then the selection alone
    logits = B().linear(dev(h, dtype), dev(wr, dtype), out_dtype=torch.float32)
    e2, w2 = B().route_from_logits(logits, top, dtype=DT[dtype])
    assert torch.equal(e2.cpu().long().sort(-1).values, idx.sort(-1).values)
    close(w2.cpu().sort(-1).values, val.sort(-1).values, "float32", tol32=1e-5)


def run_delta(cfg_m, w, p, h, dtype, lens_plan, eps=1e-5):
    """the delta mixer as the runtime strings it together, rows cut into steps by lens_plan (one request, slot 1)"""
    Bk = B()
    H, G, d, dv, taps = cfg_m["heads"], cfg_m["kv_heads"], cfg_m["dim"], cfg_m["vdim"], cfg_m["conv"]
    Wp = torch.cat([w[p + s] for s in (".q", ".k", ".v", ".g", ".b", ".a")])
    Wc = torch.cat([w[p + s] for s in (".q.conv", ".k.conv", ".v.conv")])
    Cn = 2 * G * d + H * dv
    conv_state = torch.zeros(2, max(taps - 1, 1), Cn, device="cuda")
    mem = torch.full((2, H, d, dv), 3.0, device="cuda")
    mem[1].zero_()
    outs, at = [], 0
    for n in lens_plan:
        rg = Bk.Ragged([n], slots=[1])
        proj = Bk.linear(dev(h[at:at + n], dtype), dev(Wp, dtype), plain=True)
        qkv = Bk.time_conv(proj, dev(Wc, dtype), conv_state if taps > 1 else conv_state[:, :0], rg, silu=True,
                           out_dtype=torch.float32, channels=Cn)
        o = Bk.delta_rule(qkv, proj, Cn + H * dv, Cn + H * dv + H, dev(w[p + ".A_log"], dtype), dev(w[p + ".dt_bias"], dtype), mem,
                          H, G, d, dv, rg)
        mixed = Bk.head_rms_gate(o, dev(w[p + ".norm"], dtype), proj[:, Cn:Cn + H * dv], "silu", 1.0, eps, H, dv)
        outs.append(Bk.linear(mixed, dev(w[p + ".o"], dtype), plain=True))
        at += n
    assert float(mem[0].min()) == 3.0
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("layer", [("a", 0), ("a", 3), ("wide", 1), ("odd", 1), ("b", 1)])
def test_delta_mixer_whole_and_in_portions(dtype, layer):
    cfg = {"a": C.config_a, "wide": C.config_wide_heads, "odd": C.config_odd, "b": C.config_b}[layer[0]]()
    w = C.random_weights(cfg, 3)
    p, m = "l%d.mix" % layer[1], cfg["layers"][layer[1]]["mixer"]
    h = C.bf16_round(torch.randn(45, cfg["width"], generator=torch.Generator().manual_seed(9)))
    ref = R.delta_mixer(h.double(), w, p, m, 1e-5)
    close(run_delta(m, w, p, h, dtype, [45]), ref, dtype, tol32=1e-4, tol16=6e-2)
    close(run_delta(m, w, p, h, dtype, [1, 2, 17, 1, 16, 8]), ref, dtype, tol32=1e-4, tol16=6e-2)


def test_delta_memory_gives_back_one_far_write_among_hundreds():
    """beta = 1 and no decay: token 3 writes value v* under key e0; 600 later tokens write under the other unit keys, again
    and again; the last token asks with e0 and must read v* (times dim^-1/2), across portions and the staging rounds"""
    Bk = B()
    d, dv, n = 8, 70, 604
    qkv = torch.zeros(n, 2 * d + dv)
    vals = torch.randn(n, dv, generator=torch.Generator().manual_seed(1))
    for t in range(n):
        key = 0 if t == 3 else 1 + (t % (d - 1))
        qkv[t, d + key] = 5.0 if t % 2 else 0.5          # keys of any length: the kernel makes them unit vectors
        qkv[t, key if t < n - 1 else 0] = 2.0
        qkv[t, 2 * d:] = vals[t]
    proj = torch.zeros(n, 2)
    proj[:, 0] = 30.0                                      # beta = sigmoid(30) = 1
    proj[:, 1] = -40.0                                     # softplus(-40) = 0: no decay
    zero = torch.zeros(1, device="cuda")
    for plan in ([n], [2, 1, 300, 1, 299, 1]):
        mem = torch.zeros(1, 1, d, dv, device="cuda")
        outs, at = [], 0
        for k in plan:
            outs.append(Bk.delta_rule(qkv[at:at + k].cuda().contiguous(), proj[at:at + k].cuda().contiguous(), 0, 1, zero, zero,
                                      mem, 1, 1, d, dv, Bk.Ragged([k])))
            at += k
        got = torch.cat(outs)[-1].cpu()
        assert float((got - vals[3] * d ** -0.5).abs().max()) < 1e-4 * float(vals[3].abs().max())


def run_parallel(cfg_m, w, p, h, dtype, plan, page_ids, eps=1e-5, page_size=16):
    """the parallel mixer as the runtime strings it together; plan: rows per step of ONE request whose pages are page_ids"""
    Bk = B()
    a, r = cfg_m["left"], cfg_m["right"]
    H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
    H2, d2, dv2 = r["heads"], r["dim"], r["vdim"]
    names = [".left.q", ".left.k", ".left.v", ".right.q", ".right.k", ".right.v", ".right.g", ".right.i", ".right.f"]
    Wp = torch.cat([w[p + s] for s in names])
    offs, at_ = [], 0
    for s in names:
        offs.append(at_)
        at_ += w[p + s].shape[0]
    Wo = torch.cat([w[p + ".left.o"], w[p + ".right.o"]], 1)
    half = a["rot"]["dims"] // 2
    inv_freq = torch.tensor([a["rot"]["base"] ** (-2.0 * i / a["rot"]["dims"]) for i in range(half)] or [0.0], dtype=torch.float32).cuda()
    n_pages = max(page_ids) + 2
    k_off, v_off = 5 * 16, 5 * 16 + page_size * G * d                          # the layer's part does not start the page
    page_stride = v_off + page_size * G * dv + 3
    cache = torch.full((n_pages * page_stride,), float("nan"), dtype=DT[dtype], device="cuda")
    mem = torch.zeros(1, H2 * (d2 * dv2 + d2 + 1), device="cuda")
    indptr = torch.tensor([0, len(page_ids)], dtype=torch.int32, device="cuda")
    pids = torch.tensor(page_ids, dtype=torch.int32, device="cuda")
    outs, at = [], 0
    for n in plan:
        rg = Bk.Ragged([n], starts=[at])
        proj = Bk.linear(dev(h[at:at + n], dtype), dev(Wp, dtype), plain=True)
        q = Bk.qk_norm_rope_paged(proj, offs[:3], H, G, d, dv, dev(w[p + ".left.q.norm"], dtype), dev(w[p + ".left.k.norm"], dtype),
                                  eps, inv_freq, a["rot"]["dims"], rg, indptr, pids, cache, page_stride, k_off, v_off, page_size)
        mix = torch.empty(n, H * dv + H2 * dv2, dtype=DT[dtype], device="cuda")
        mix[:, :H * dv] = Bk.paged_attention(q, cache, page_stride, k_off, v_off, page_size, rg, indptr, pids, G, dv, a["scale"],
                                             cfg_m["left_scale"])
        o = Bk.gated_matrix_memory(proj, offs[3:6] + offs[7:9], dev(w[p + ".right.i.b"], dtype), dev(w[p + ".right.f.b"], dtype),
                                   r["gate_cap"], mem, H2, d2, dv2, rg)
        Bk.head_rms_gate(o, dev(w[p + ".right.norm"], dtype), proj[:, offs[6]:offs[6] + H2 * dv2], "sigmoid", cfg_m["right_scale"],
                         eps, H2, dv2, out=mix[:, H * dv:])
        outs.append(Bk.linear(mix, dev(Wo, dtype), plain=True))
        at += n
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("layer", [("a", 1), ("a", 2), ("wide", 0), ("wide", 2), ("odd", 0), ("b", 0)])
def test_parallel_mixer_whole_and_in_portions_over_scattered_pages(dtype, layer):
    cfg = {"a": C.config_a, "wide": C.config_wide_heads, "odd": C.config_odd, "b": C.config_b}[layer[0]]()
    w = C.weights_for(cfg, 4, dtype)
    p, m = "l%d.mix" % layer[1], cfg["layers"][layer[1]]["mixer"]
    n = 150
    h = C.bf16_round(torch.randn(n, cfg["width"], generator=torch.Generator().manual_seed(8)))
    ref = R.parallel_mixer(h.double(), w, p, m, 1e-5)
    pages = [7, 2, 11, 0, 5, 9, 3, 12, 1, 10]                                   # ten pages of 16 tokens, in no order
    close(run_parallel(m, w, p, h, dtype, [n], pages), ref, dtype, tol32=1e-4, tol16=6e-2)
    # portions that end just before, at and just after page (16) and key tile (64) borders, then token by token over 127 / 128
    close(run_parallel(m, w, p, h, dtype, [15, 1, 1, 46, 2, 60] + [1] * 25, pages), ref, dtype, tol32=1e-4, tol16=6e-2)


def test_attention_finds_one_far_key_among_hundreds_and_stops_at_the_causal_edge():
    """all keys equal except position 5, whose key points along the last query; its score stands out, so the last row's
    output must be v_5; the row before the marked query has a key of its own kind AFTER it (position 5 + 1 ... are visible,
    the future is not): a second marked key at the very last position must not reach the row before it"""
    Bk = B()
    n, d, dv = 700, 16, 24
    g = torch.Generator().manual_seed(2)
    proj = torch.zeros(n, 2 * d + dv)
    base = torch.randn(d, generator=g)
    mark = torch.randn(d, generator=g)
    mark -= base * (mark @ base) / (base @ base)
    proj[:, :d] = base                               # every query and key looks along `base` ...
    proj[:, d:2 * d] = base
    proj[:, 2 * d:] = torch.randn(n, dv, generator=g)
    proj[5, d:2 * d] = mark * 3                      # ... but key 5 and key n - 1 look along `mark`
    proj[n - 1, d:2 * d] = mark * 3
    proj[n - 2, :d] = mark * 3                       # rows n - 2 and n - 1 ask along `mark`
    proj[n - 1, :d] = mark * 3
    ones = torch.ones(d, device="cuda")
    pages = list(range(44))[::-1]
    indptr = torch.tensor([0, 44], dtype=torch.int32, device="cuda")
    pids = torch.tensor(pages, dtype=torch.int32, device="cuda")
    page_stride = 16 * (d + dv)
    for plan in ([n], [5, 1, 58, 1, 634, 1]):
        cache = torch.zeros(45 * page_stride, device="cuda")
        rows, at = [], 0
        for k in plan:
            rg = Bk.Ragged([k], starts=[at])
            q = Bk.qk_norm_rope_paged(proj[at:at + k].cuda().contiguous(), [0, d, 2 * d], 1, 1, d, dv, ones, ones, 1e-6,
                                      torch.zeros(1, device="cuda"), 0, rg, indptr, pids, cache, page_stride, 0, 16 * d, 16)
            rows.append(Bk.paged_attention(q, cache, page_stride, 0, 16 * d, 16, rg, indptr, pids, 1, dv, 4.0))
            at += k
        out = torch.cat(rows).cpu()
        v = proj[:, 2 * d:]
        assert float((out[n - 2] - v[5]).abs().max()) < 1e-3          # the far key alone; key n - 1 is in this row's future
        assert float((out[n - 1] - 0.5 * (v[5] + v[n - 1])).abs().max()) < 1e-3
        assert float((out[3] - v[:4].mean(0)).abs().max()) < 1e-4     # the first tokens: equal scores, the mean of what is visible


def test_matrix_memory_keeps_a_far_strong_write_and_resets_with_its_slot():
    """token 4 is written with a large input gate, the forget gates stay open: 500 weak writes later its value still
    dominates the read-out; the same slot, zeroed and used by a second request, must not see any of it"""
    Bk = B()
    n, d, dv = 505, 12, 66
    g = torch.Generator().manual_seed(3)
    k = torch.randn(n, d, generator=g)
    v = torch.randn(n, dv, generator=g)
    proj = torch.zeros(n, 2 * d + dv + 2)
    proj[:, :d] = k[4]                               # every query asks for key 4
    proj[:, d:2 * d] = k
    proj[:, 2 * d:2 * d + dv] = v
    proj[:, 2 * d + dv] = -6.0                       # log input gate: weak writes ...
    proj[4, 2 * d + dv] = 9.0                        # ... one strong one
    proj[:, 2 * d + dv + 1] = 20.0                   # forget gate open (logsigmoid(cap tanh(20 / cap)) ~ 0)
    offs = [0, d, 2 * d, 2 * d + dv, 2 * d + dv + 1]
    zero = torch.zeros(1, device="cuda")
    mem = torch.zeros(1, d * dv + d + 1, device="cuda")
    outs, at = [], 0
    for kk in [3, 2, 250, 1, 249]:
        outs.append(Bk.gated_matrix_memory(proj[at:at + kk].cuda().contiguous(), offs, zero, zero, 15.0, mem, 1, d, dv, Bk.Ragged([kk])))
        at += kk
    got = torch.cat(outs)[-1].cpu()
    cos = float(Fn.cosine_similarity(got, v[4], dim=0))
    assert cos > 0.999, cos
    mem.zero_()
    again = Bk.gated_matrix_memory(proj[:3].cuda().contiguous(), offs, zero, zero, 15.0, mem, 1, d, dv, Bk.Ragged([3]))
    assert float((again.cpu() - torch.cat(outs)[:3].cpu()).abs().max()) == 0.0
