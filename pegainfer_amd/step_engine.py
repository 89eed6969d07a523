"""Python driver shared by the host runtimes that serve a model through ONE batched step function (libpegainfer_qwen3.so:
include/pegainfer_duguzen.h, include/pegainfer_feruzen.h): prompts, portions of prompts and single decoded tokens of
several requests run as one batch.  No CPU fallback."""
import json
import os

import numpy as np

from . import ffi

DTYPES = {"bfloat16": 0, "bf16": 0, "float32": 1, "f32": 1}


class StepEngine:
    """Engine over a host runtime with ONE batched step function.  A subclass names its architecture and the prefix of its
    C entry points (include/pegainfer_<family>.h); everything else - weights, requests, the step, sampling, the per-layer
    tap - is the same call pattern."""
    architecture = None
    prefix = None

    def _fn(self, name):
        return getattr(self.lib, self.prefix + name)

    def __init__(self, config, max_tokens=4096, max_requests=8, dtype="bfloat16", device=0, _handle=None):
        self.lib = ffi.host_lib()
        self.cfg = config if isinstance(config, dict) else json.loads(config)
        self.dtype = dtype
        if _handle is None:
            text = json.dumps(self.cfg).encode()
            _handle = self._fn('create')(text, int(device), DTYPES[dtype], int(max_tokens), int(max_requests))
        self.h = _handle
        if not self.h:
            msg = self._fn('last_error')(None)
            raise RuntimeError(self.prefix + "create failed: " + (msg.decode() if msg else ""))
        self.vocab = self._fn('vocab_size')(self.h)
        self.width = self._fn('width')(self.h)
        self.layer_runs = self._fn('num_layer_runs')(self.h)
        self.page_size = self._fn('page_size')(self.h)

    @classmethod
    def from_pretrained(cls, model_dir, max_tokens=4096, max_requests=8, dtype="bfloat16", device=0):
        lib = ffi.host_lib()
        with open(os.path.join(model_dir, "config.json")) as f:
            cfg = json.load(f)
        h = getattr(lib, cls.prefix + 'from_pretrained')(os.fsencode(model_dir), int(device), DTYPES[dtype], int(max_tokens),
                                                  int(max_requests))
        if not h:
            msg = getattr(lib, cls.prefix + 'last_error')(None)
            raise RuntimeError("loading %s failed: %s" % (model_dir, msg.decode() if msg else ""))
        return cls(cfg, dtype=dtype, _handle=h)

    def _chk(self, rc, what):
        if rc != 0:
            msg = self._fn('last_error')(self.h)
            raise RuntimeError(f"{what} failed ({rc}): {msg.decode() if msg else ''}")

    # ---- weights ----
    def load_tensors(self, tensors):
        """tensors: {checkpoint name: array of bf16 bit patterns (uint16) or of floats (rounded to bf16 here)}"""
        for name, a in tensors.items():
            a = np.asarray(a)
            if a.dtype != np.uint16:
                u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
                a = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
            a = np.ascontiguousarray(a)
            self._chk(self._fn('load_tensor')(self.h, name.encode(), a.ctypes.data, int(a.size)), "load_tensor")
        self._chk(self._fn('finalize')(self.h), "finalize")
        return self

    def fill_synthetic(self, seed=0, std=0.02):
        self._chk(self._fn('fill_synthetic')(self.h, int(seed), float(std)), "fill_synthetic")
        self._chk(self._fn('finalize')(self.h), "finalize")
        return self

    def set_plain_kernels(self, on=True):
        self._fn('set_plain_kernels')(self.h, int(bool(on)))

    # ---- requests ----
    def new_request(self):
        r = self._fn('new_request')(self.h)
        if r < 0:
            self._chk(r, "new_request")
        return r

    def drop_request(self, rid):
        self._chk(self._fn('drop_request')(self.h, int(rid)), "drop_request")

    def seq_len(self, rid):
        return self._fn('request_seq_len')(self.h, int(rid))

    def available_pages(self):
        return self._fn('available_pages')(self.h)

    def capacity_pages(self):
        return self._fn('capacity_pages')(self.h)

    # ---- the step ----
    def step(self, entries, want=None, logits=True, tokens=False):
        """entries: [(request id, [token ids])]; want: rows of the concatenated tokens whose logits are computed (None = the
        last row of every entry).  Returns float32 logits [wanted, vocab] (and / or the greedy tokens of those rows)."""
        ids = np.ascontiguousarray([e[0] for e in entries], dtype=np.int32)
        lens = np.ascontiguousarray([len(e[1]) for e in entries], dtype=np.int32)
        toks = np.ascontiguousarray([t for e in entries for t in e[1]], dtype=np.uint32)
        if want is None:
            n_want, wp, rows = -1, None, len(entries)
        else:
            w = np.ascontiguousarray(want, dtype=np.int32)
            n_want, wp, rows = int(w.size), (w.ctypes.data if w.size else None), int(w.size)
        lg = np.zeros((rows, self.vocab), dtype=np.float32) if logits and rows else None
        tk = np.zeros(rows, dtype=np.int32) if tokens and rows else None
        self._chk(self._fn('step')(self.h, len(entries), ids.ctypes.data, lens.ctypes.data, toks.ctypes.data,
                                                  n_want, wp, lg.ctypes.data if lg is not None else None,
                                                  tk.ctypes.data if tk is not None else None), "step")
        if logits and tokens:
            return lg, tk
        return tk if tokens else lg

    def sample(self, row, temperature=0.0, top_k=-1, top_p=1.0, random_val=0.5):
        import ctypes
        out = ctypes.c_int32(0)
        self._chk(self._fn('sample')(self.h, int(row), float(temperature), int(top_k), float(top_p),
                                                    float(random_val), ctypes.addressof(out)), "sample")
        return out.value

    def debug_hidden_enable(self, on=True):
        self._chk(self._fn('debug_hidden_enable')(self.h, int(bool(on))), "debug_hidden_enable")

    def debug_hidden(self, rows):
        """float32 [layer runs, rows, width]: the residual stream after every layer run for the last step's token rows"""
        out = np.zeros((self.layer_runs, rows, self.width), dtype=np.float32)
        for li in range(self.layer_runs):
            n = self._fn('debug_hidden')(self.h, li, out[li].ctypes.data, rows)
            if n < 0:
                self._chk(n, "debug_hidden")
        return out

    def last_step_ms(self):
        return float(self._fn('last_step_ms')(self.h))

    def weight_bytes(self):
        return int(self._fn('weight_bytes')(self.h))

    def close(self):
        if getattr(self, "h", None):
            self._fn('destroy')(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # noqa: BLE001
            pass
