"""Torch-tensor wrappers over include/pegainfer_kernels_blocks.h: the model-independent blocks that exist in a bf16 and a
true-fp32 instance (Dynamic-Tanh norms over an fp32 stream, activations, the strided / batched / grouped GEMM, attention
over a paged latent cache, sigmoid-scored grouped routing).  Tensors are torch CUDA tensors used as device memory; the
storage type of a call (bf16 / fp32) is taken from the activation tensor.  Work is enqueued on torch's current stream.
No CPU fallback: without the HIP library every call raises ImportError.
"""
import ctypes

import torch

from . import ffi
from .ops import _chk, _p, _stream

EPI_NONE, EPI_RELU_SQ, EPI_SIGMOID_GATE = 0, 1, 2


def _dt(t):
    if t.dtype == torch.bfloat16:
        return 0
    if t.dtype == torch.float32:
        return 1
    raise TypeError("bf16 or fp32 tensors only")


class GemmDesc(ctypes.Structure):
    _fields_ = [("x", ctypes.c_void_p), ("w", ctypes.c_void_p), ("y", ctypes.c_void_p),
                ("x_dtype", ctypes.c_int32), ("w_dtype", ctypes.c_int32), ("y_dtype", ctypes.c_int32),
                ("m", ctypes.c_int32), ("k", ctypes.c_int32), ("rows", ctypes.c_int32), ("groups", ctypes.c_int32),
                ("x_row_stride", ctypes.c_int64), ("x_group_stride", ctypes.c_int64),
                ("w_m_stride", ctypes.c_int64), ("w_k_stride", ctypes.c_int64), ("w_group_stride", ctypes.c_int64),
                ("y_row_stride", ctypes.c_int64), ("y_group_stride", ctypes.c_int64),
                ("tile_group", ctypes.c_void_p), ("tile_row0", ctypes.c_void_p), ("tile_rows", ctypes.c_void_p),
                ("n_tiles", ctypes.c_void_p), ("max_tiles", ctypes.c_int32),
                ("x_row_index", ctypes.c_void_p), ("y_row_index", ctypes.c_void_p),
                ("epilogue", ctypes.c_int32), ("gate", ctypes.c_void_p), ("gate_dtype", ctypes.c_int32),
                ("gate_row_stride", ctypes.c_int64), ("max_tile_rows", ctypes.c_int32), ("tile_rows_cap", ctypes.c_int32),
                ("plain", ctypes.c_int32)]


def embed_f32(embed, token_ids_u32):
    out = torch.empty((token_ids_u32.numel(), embed.shape[1]), dtype=torch.float32, device=embed.device)
    _chk(ffi.lib().pegainfer_embed_f32(_p(embed), _p(token_ids_u32), _p(out), embed.shape[1], token_ids_u32.numel(),
                                       _dt(embed), _stream()), "embed_f32")
    return out


def dyt_norm(x_f32, alpha, w, b):
    """out = tanh(alpha x) w + b; x fp32 [rows, d]; alpha / w / b (and the result) in the storage type of w"""
    assert x_f32.dtype == torch.float32 and x_f32.is_contiguous()
    out = torch.empty(x_f32.shape, dtype=w.dtype, device=x_f32.device)
    _chk(ffi.lib().pegainfer_dyt_norm(_p(x_f32), _p(alpha), _p(w), _p(b), _p(out), x_f32.shape[-1],
                                      x_f32.numel() // x_f32.shape[-1], _dt(w), _stream()), "dyt_norm")
    return out


def dyt_add_norm(x_f32, y, post, nxt=None):
    """x += dyt(y; post) in place; returns dyt(x; nxt) when nxt = (alpha, w, b) is given"""
    assert x_f32.dtype == torch.float32 and x_f32.is_contiguous() and y.is_contiguous()
    out = torch.empty(y.shape, dtype=y.dtype, device=y.device) if nxt else None
    n = nxt or (None, None, None)
    _chk(ffi.lib().pegainfer_dyt_add_norm(_p(x_f32), _p(y), _p(post[0]), _p(post[1]), _p(post[2]), _p(n[0]), _p(n[1]), _p(n[2]),
                                          _p(out), y.shape[-1], y.numel() // y.shape[-1], _dt(y), _stream()), "dyt_add_norm")
    return out


def relu_sq(x):
    out = torch.empty_like(x)
    _chk(ffi.lib().pegainfer_relu_sq(_p(x), _p(out), x.numel(), _dt(x), _stream()), "relu_sq")
    return out


def silu_mul_rows(gate_up):
    rows, two_i = gate_up.shape
    out = torch.empty((rows, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    _chk(ffi.lib().pegainfer_silu_mul_rows(_p(gate_up), _p(out), two_i // 2, rows, _dt(gate_up), _stream()), "silu_mul_rows")
    return out


def gemm_strided(desc):
    _chk(ffi.lib().pegainfer_gemm_strided(ctypes.addressof(desc), _stream()), "gemm_strided")


def linear(x, w, out_dtype=None, epilogue=EPI_NONE, plain=False):
    """y[T, M] = x[T, K] w[M, K]^T through pegainfer_gemm_strided (any sizes, bf16 or fp32 operands, fp32 accumulation);
    plain = the fp32-FMA tile kernel whatever the shape"""
    T, K = x.shape
    M = w.shape[0]
    y = torch.empty((T, M), dtype=out_dtype or x.dtype, device=x.device)
    d = GemmDesc(x=_p(x), w=_p(w), y=_p(y), x_dtype=_dt(x), w_dtype=_dt(w), y_dtype=_dt(y), m=M, k=K, rows=T, groups=1,
                 x_row_stride=K, w_m_stride=K, w_k_stride=1, y_row_stride=M, epilogue=epilogue, plain=int(plain))
    gemm_strided(d)
    return y


def latent_prep(proj, dkv_offset, c_norm_w, eps, inv_freq, rot_dims, positions, token_req, page_indptr, page_ids, cache,
                page_stride, layer_off, page_size, qc, heads, nope, rot, rank):
    _chk(ffi.lib().pegainfer_latent_prep(_p(proj), proj.shape[1], dkv_offset, _p(c_norm_w), float(eps), _p(inv_freq), rot_dims,
                                         _p(positions), _p(token_req), _p(page_indptr), _p(page_ids), _p(cache), page_stride,
                                         layer_off, page_size, _p(qc), heads, nope, rot, rank, proj.shape[0], _dt(proj),
                                         _stream()), "latent_prep")


def row_tiles(lens, heads, device="cuda"):
    """the flattened (token, head) rows of a step with entries of `lens` tokens, cut into runs of <= 64 rows inside one entry"""
    row0, rows, at = [], [], 0
    for n in lens:
        for r in range(0, n * heads, 64):
            row0.append(at * heads + r)
            rows.append(min(64, n * heads - r))
        at += n
    return (torch.tensor(row0, dtype=torch.int32, device=device), torch.tensor(rows, dtype=torch.int32, device=device))


def latent_attention(qc, cache, page_stride, layer_off, page_size, positions, token_req, page_indptr, page_ids, rank, rot,
                     scale, max_kv_len, split_keys=0, tiles=None):
    """qc fp32 [T, heads, rank + rot] -> o_lat fp32 [T, heads, rank]; tiles = row_tiles(...) selects the matrix-core form"""
    T, H, E = qc.shape
    assert E == rank + rot and qc.dtype == torch.float32
    o = torch.empty((T, H, rank), dtype=torch.float32, device=qc.device)
    n = ffi.lib().pegainfer_latent_attention_workspace(T, H, rank, max_kv_len, split_keys)
    ws = torch.empty(max(int(n), 1), dtype=torch.float32, device=qc.device)
    t0, tr = tiles if tiles is not None else (None, None)
    _chk(ffi.lib().pegainfer_latent_attention(_p(qc), _p(o), _p(cache), page_stride, layer_off, page_size, _p(positions),
                                              _p(token_req), _p(page_indptr), _p(page_ids), H, rank, rot, float(scale), T,
                                              max_kv_len, split_keys, _p(ws), _p(t0), _p(tr), 0 if t0 is None else t0.numel(),
                                              _dt(cache), _stream()), "latent_attention")
    return o


def route(h, w_router, correction, n_groups, keep_groups, top):
    rows, d = h.shape
    e = torch.empty((rows, top), dtype=torch.int32, device=h.device)
    w = torch.empty((rows, top), dtype=torch.float32, device=h.device)
    _chk(ffi.lib().pegainfer_route_sigmoid_grouped(_p(h), _p(w_router), _p(correction), _p(e), _p(w), d, w_router.shape[0],
                                                   n_groups, keep_groups, top, rows, _dt(h), _stream()), "route")
    return e, w


def route_sort(expert, experts, rows_per_tile=64):
    """-> pos_pair, pos_row, tile_group, tile_row0, tile_rows, n_tiles (int32 device tensors), max_tiles"""
    rows, top = expert.shape
    P = rows * top
    max_tiles = (P + rows_per_tile - 1) // rows_per_tile + experts
    dev = expert.device
    pos_pair, pos_row = torch.empty(P, dtype=torch.int32, device=dev), torch.empty(P, dtype=torch.int32, device=dev)
    tg, t0, tr = (torch.zeros(max_tiles, dtype=torch.int32, device=dev) for _ in range(3))
    nt = torch.zeros(1, dtype=torch.int32, device=dev)
    _chk(ffi.lib().pegainfer_route_sort(_p(expert), P, top, experts, _p(pos_pair), _p(pos_row), _p(tg), _p(t0), _p(tr), _p(nt),
                                        max_tiles, rows_per_tile, _stream()), "route_sort")
    return pos_pair, pos_row, tg, t0, tr, nt, max_tiles


def route_combine(y_pairs, weight, out_dtype):
    rows, top = weight.shape
    d = y_pairs.shape[1]
    out = torch.empty((rows, d), dtype=out_dtype, device=y_pairs.device)
    _chk(ffi.lib().pegainfer_route_combine(_p(y_pairs), _p(weight), _p(out), d, top, rows, _dt(out), _stream()), "route_combine")
    return out
