"""The kernels' plain C++ twins (exec-beholdd_amd/csrc/plain_twins.cpp) as Python calls on NumPy arrays,
for the tests that hold the twins to the plain implementation and the kernels to the twins."""

from __future__ import annotations

import ctypes

import numpy as np

F32, BF16 = 0, 1
PAGE = 64


def to_bf16_bits(x):
    """float32 array -> uint16 array of bfloat16 bits, rounded to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + (0x7FFF + ((u >> 16) & 1))) >> 16).astype(np.uint16)


def from_bf16_bits(b):
    return (b.astype(np.uint32) << 16).view(np.float32)


class Twins:
    def __init__(self, folder):
        from beholdd.kernels import build

        self.lib = ctypes.CDLL(build.build_plain_twins(str(folder)))
        assert self.lib.bhp_page_size() == PAGE

    @staticmethod
    def _p(array):
        return None if array is None else array.ctypes.data_as(ctypes.c_void_p)

    def _store(self, x, code):
        x = np.ascontiguousarray(x, dtype=np.float32)
        return x.copy() if code == F32 else to_bf16_bits(x)

    def _load(self, stored, code):
        return stored if code == F32 else from_bf16_bits(stored)

    def embed(self, tokens, table, code=F32):
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        stored = self._store(table, code)
        out = np.zeros((len(tokens), table.shape[1]), np.float32)
        status = self.lib.bhp_embed(self._p(tokens), self._p(stored), code, self._p(out), len(tokens), table.shape[1], table.shape[0])
        return status, out

    def rmsnorm(self, x, weight, eps, rows=None, w_code=F32, out_code=F32):
        x = np.ascontiguousarray(x, dtype=np.float32)
        n = len(rows) if rows is not None else x.shape[0]
        rows = None if rows is None else np.ascontiguousarray(rows, dtype=np.int32)
        w = None if weight is None else self._store(weight, w_code)
        out = np.zeros((n, x.shape[1]), np.float32 if out_code == F32 else np.uint16)
        assert self.lib.bhp_rmsnorm(self._p(x), self._p(rows), self._p(w), w_code, self._p(out), out_code, n, x.shape[1],
                                    ctypes.c_float(eps)) == 0
        return self._load(out, out_code)

    def gemm(self, a, w, code=F32, c=None):
        m, k = a.shape
        n = w.shape[0]
        sa, sw = self._store(a, code), self._store(w, code)
        out = np.zeros((m, n), np.float32) if c is None else np.ascontiguousarray(c, dtype=np.float32).copy()
        assert self.lib.bhp_gemm(self._p(sa), code, self._p(sw), code, self._p(out), F32, int(c is not None), m, n, k) == 0
        return out

    def swiglu(self, gate_up, code=F32):
        rows, two_f = gate_up.shape
        stored = self._store(gate_up, code)
        out = np.zeros((rows, two_f // 2), np.float32 if code == F32 else np.uint16)
        assert self.lib.bhp_swiglu(self._p(stored), self._p(out), code, rows, two_f // 2) == 0
        return self._load(out, code)

    def qk_norm_rope_cache(self, qkv, q_weight, k_weight, eps, cos, sin, positions, row_seq, page_table, n_pages, n_heads,
                           kv_heads, head_dim, kv_order, code=F32, write_kv=True, k_pages=None, v_pages=None):
        """Returns (q_out, k_pages, v_pages) as float32 arrays; the pages as flat [pages, kv_heads, 64 * head_dim] in the
        twin's own order (read them back with `key` / `value`)."""
        n_rows = qkv.shape[0]
        stored = self._store(qkv, code)
        kind = np.float32 if code == F32 else np.uint16
        q_out = np.zeros((n_rows, n_heads * head_dim), kind)
        k_pages = np.zeros((n_pages, kv_heads, PAGE * head_dim), kind) if k_pages is None else k_pages
        v_pages = np.zeros((n_pages, kv_heads, PAGE * head_dim), kind) if v_pages is None else v_pages
        qw = None if q_weight is None else np.ascontiguousarray(q_weight, dtype=np.float32)
        kw = None if k_weight is None else np.ascontiguousarray(k_weight, dtype=np.float32)
        cos = None if cos is None else np.ascontiguousarray(cos, dtype=np.float32)
        sin = None if sin is None else np.ascontiguousarray(sin, dtype=np.float32)
        positions = np.ascontiguousarray(positions, dtype=np.int32)
        row_seq = np.ascontiguousarray(row_seq, dtype=np.int32)
        table = np.ascontiguousarray(page_table, dtype=np.int32)
        status = self.lib.bhp_qk_norm_rope_cache(
            self._p(stored), code, self._p(q_out), self._p(qw), self._p(kw), F32, ctypes.c_float(eps), self._p(cos), self._p(sin),
            0 if cos is None else cos.shape[0], 0 if cos is None else 2 * cos.shape[1], self._p(positions), self._p(row_seq),
            self._p(k_pages), self._p(v_pages), self._p(table), table.shape[1], n_rows, n_heads, kv_heads, head_dim,
            int(write_kv), kv_order, n_pages)
        assert status == 0, status
        return self._load(q_out, code), k_pages, v_pages

    def attention(self, q, k_pages, v_pages, page_table, row_seq, positions, n_heads, kv_heads, head_dim, scale, window,
                  kv_order, code=F32):
        stored = self._store(q, code)
        out = np.zeros(q.shape, np.float32 if code == F32 else np.uint16)
        table = np.ascontiguousarray(page_table, dtype=np.int32)
        positions = np.ascontiguousarray(positions, dtype=np.int32)
        row_seq = np.ascontiguousarray(row_seq, dtype=np.int32)
        status = self.lib.bhp_attention(self._p(stored), self._p(out), code, self._p(k_pages), self._p(v_pages), self._p(table),
                                        table.shape[1], self._p(row_seq), self._p(positions), q.shape[0], n_heads, kv_heads,
                                        head_dim, ctypes.c_float(scale), window, kv_order, k_pages.shape[0])
        assert status == 0, status
        return self._load(out, code)

    def argmax(self, logits):
        logits = np.ascontiguousarray(logits, dtype=np.float32)
        tokens = np.zeros(logits.shape[0], np.int32)
        bad = np.zeros(logits.shape[0], np.int32)
        assert self.lib.bhp_argmax(self._p(logits), self._p(tokens), self._p(bad), logits.shape[0], logits.shape[1]) == 0
        return tokens, bad

    def sample(self, logits, temperature, uniform, top_k=None, top_p=None):
        """(tokens, bad, margin): margin is how far each draw lies from the nearer end of its token's interval, as a
        fraction of the kept mass."""
        logits = np.ascontiguousarray(logits, dtype=np.float32)
        n = logits.shape[0]
        tokens, bad, margin = np.zeros(n, np.int32), np.zeros(n, np.int32), np.zeros(n, np.float64)
        as_f32 = lambda v: None if v is None else np.ascontiguousarray(v, dtype=np.float32)
        temperature, uniform, top_p = as_f32(temperature), as_f32(uniform), as_f32(top_p)
        top_k = None if top_k is None else np.ascontiguousarray(top_k, dtype=np.int32)
        assert self.lib.bhp_sample(self._p(logits), self._p(temperature), self._p(top_k), self._p(top_p), self._p(uniform),
                                   self._p(tokens), self._p(bad), self._p(margin), n, logits.shape[1]) == 0
        return tokens, bad, margin

    def rows_index(self, block_rows, rows, width):
        """Where each element of a [rows, width] matrix lies when its rows are in blocks of `block_rows`."""
        self.lib.bhp_rows_index.restype = ctypes.c_long
        return np.array([[self.lib.bhp_rows_index(block_rows, r, c, width) for c in range(width)] for r in range(rows)])

    def key(self, k_pages, order, page, kv_head, token, head_dim, code=F32):
        """The key vector [head_dim] that lies at (page, kv_head, token)."""
        index = [self.lib.bhp_key_index(order, token, d, head_dim) for d in range(head_dim)]
        return self._load(k_pages[page, kv_head][index], code)

    def value(self, v_pages, order, page, kv_head, token, head_dim, code=F32):
        index = [self.lib.bhp_value_index(order, token, d, head_dim) for d in range(head_dim)]
        return self._load(v_pages[page, kv_head][index], code)
