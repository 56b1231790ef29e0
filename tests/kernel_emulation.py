"""A test double for the kernel library: the same calls, computed with torch on the CPU.

It exists so that the engine's own logic (step layout, paged cache, slots, generation loop)
can be tested where there is no GPU.  It is slow and lives under tests/: the product has no
CPU path, and nothing in the package imports this file.
"""

from __future__ import annotations

import torch

PAGE = 64


class TorchKernels:
    page_size = PAGE

    def __init__(self, device="cpu"):
        self.device = torch.device(device)
        self.calls = []

    def embed(self, tokens, table, out):
        self.calls.append("embed")
        out.copy_(table[tokens.long()].float())

    def rmsnorm(self, x, weight, eps, out, rows=None):
        self.calls.append("rmsnorm")
        src = x if rows is None else x[rows.long()]
        inv = 1.0 / torch.sqrt((src.double() ** 2).mean(-1, keepdim=True) + eps)
        y = src * inv.float()
        if weight is not None:
            y = y * weight.float()
        out.copy_(y.to(out.dtype))

    def gemm(self, a, w, out, accumulate=False, then_norm=None):
        self.calls.append("gemm")
        product = (a.double() @ w.double().t()).float()
        if accumulate:
            product = product + out.float()
        out.copy_(product.to(out.dtype))
        return None         # this double never prepares a following norm: the norm runs as a step of its own

    def qk_norm_rope_cache(self, qkv, q_out, q_weight, k_weight, eps, cos, sin, positions, row_seq,
                           k_pages, v_pages, page_table, n_heads, n_kv_heads, head_dim, write_kv, max_position):
        self.calls.append("qk_norm_rope_cache")
        n_rows = qkv.shape[0]
        q_width, kv_width = n_heads * head_dim, n_kv_heads * head_dim
        q = qkv[:, :q_width].float().reshape(n_rows, n_heads, head_dim)
        k = qkv[:, q_width:q_width + kv_width].float().reshape(n_rows, n_kv_heads, head_dim)
        v = qkv[:, q_width + kv_width:].reshape(n_rows, n_kv_heads, head_dim)

        def norm(x, w):
            if w is None:
                return x
            inv = 1.0 / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + eps)
            return x * inv.float() * w.float()

        def rotate(x):
            if cos is None:
                return x
            half = cos.shape[1]
            c = cos[positions.long()][:, None, :]
            s = sin[positions.long()][:, None, :]
            a, b, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
            return torch.cat([a * c - b * s, a * s + b * c, rest], dim=-1)

        q_out.copy_(rotate(norm(q, q_weight)).reshape(n_rows, q_width).to(q_out.dtype))
        if not write_kv:
            return
        k = rotate(norm(k, k_weight))
        for row in range(n_rows):
            pos = int(positions[row])
            page = int(page_table[int(row_seq[row]), pos // PAGE])
            k_pages[page, :, pos % PAGE, :] = k[row].to(k_pages.dtype)
            v_pages[page, :, :, pos % PAGE] = v[row].to(v_pages.dtype)

    def attention(self, q, out, k_pages, v_pages, page_table, row_seq, positions, n_heads, n_kv_heads, head_dim,
                  scale, window=0, layout=None):
        self.calls.append("attention")
        n_rows = q.shape[0]
        group = n_heads // n_kv_heads
        qh = q.float().reshape(n_rows, n_heads, head_dim)
        result = torch.empty_like(qh)
        for row in range(n_rows):
            pos, seq = int(positions[row]), int(row_seq[row])
            first = max(0, pos - window + 1) if window else 0
            index = torch.arange(first, pos + 1)
            pages = page_table[seq, index // PAGE].long()
            keys = k_pages[pages, :, index % PAGE, :].float()      # [n, kv_heads, head_dim]
            values = v_pages[pages, :, :, index % PAGE].float()
            for head in range(n_heads):
                kv = head // group
                scores = (keys[:, kv, :].double() @ qh[row, head].double()).float() * scale
                probs = torch.softmax(scores, dim=0)
                result[row, head] = (probs.double() @ values[:, kv, :].double()).float()
        out.copy_(result.reshape(n_rows, n_heads * head_dim).to(out.dtype))

    def pack_weight(self, w):
        return w

    def gemm_swiglu(self, a, w, out):
        self.calls.append("gemm_swiglu")
        both = torch.empty(a.shape[0], w.shape[0], dtype=a.dtype)
        self.gemm(a, w, both)
        self.swiglu(both, out)

    def swiglu(self, gate_up, out):
        self.calls.append("swiglu")
        width = out.shape[1]
        g, u = gate_up[:, :width].float(), gate_up[:, width:].float()
        out.copy_((g / (1 + torch.exp(-g)) * u).to(out.dtype))

    def sample(self, logits, tokens, bad, temperature=None, top_k=None, top_p=None, uniform=None):
        self.calls.append("sample")
        for row in range(logits.shape[0]):
            x = logits[row]
            if not torch.isfinite(x).all():
                tokens[row], bad[row] = -1, 1
                continue
            bad[row] = 0
            temp = float(temperature[row]) if temperature is not None else 0.0
            if temp <= 0:
                tokens[row] = int(torch.argmax(x))
                continue
            keep = torch.ones_like(x, dtype=torch.bool)
            k = int(top_k[row]) if top_k is not None else 0
            if 0 < k < x.numel():
                keep &= x >= torch.topk(x, k).values[-1]
            e = torch.where(keep, torch.exp((x - x.max()) / temp), torch.zeros_like(x)).double()
            p = float(top_p[row]) if top_p is not None else 1.0
            if 0 < p < 1:
                order = torch.argsort(e, descending=True)
                mass = torch.cumsum(e[order], 0)
                count = int(torch.searchsorted(mass, p * e.sum()).clamp(max=x.numel() - 1)) + 1
                keep &= e >= e[order][count - 1]
                e = torch.where(keep, e, torch.zeros_like(e))
            cdf = torch.cumsum(e, 0)
            target = float(uniform[row]) * float(cdf[-1])
            tokens[row] = int(torch.searchsorted(cdf, torch.tensor(target, dtype=cdf.dtype), right=True)
                              .clamp(max=x.numel() - 1))
