"""A slow torch stand-in for the kernel backend, for tests on a machine without a GPU.

It lets the engine's bookkeeping (block tables, slots, ragged batches, page reuse,
the scheduler) be exercised on the CPU.  It is test equipment: the product never
installs it, and the GPU tests never use it.  Arithmetic is done in float64 and
rounded to the output tensor's dtype.
"""
from __future__ import annotations


import torch

from easy_gpt.cpp_amd.kernels import KernelBackend

F64 = torch.float64


def _whole(t):
    """A product operand: a tensor, or float32 partial sums [splits, rows, cols] to be added up."""
    return t.sum(0) if t is not None and t.dim() == 3 else t


class EmulatedKernels(KernelBackend):
    name = "emulated"

    def product(self, x, w, unrounded=False, residual=None):
        out = torch.empty((x.shape[0], w.shape[0]), dtype=x.dtype)
        self.linear(x, w, None, out)
        return out

    def embed(self, token_ids, table, out):
        out.copy_(table[token_ids.long()].to(out.dtype))

    def add_rmsnorm(self, h, delta, weight, eps, out):
        delta = _whole(delta)
        if delta is not None:
            h.add_(delta.to(h.dtype))
        x = h.to(F64)
        inv = 1.0 / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
        out.copy_((x * inv * weight.to(F64)).to(out.dtype))

    def rows_add_rmsnorm(self, h, delta, rows, weight, eps, out):
        delta = _whole(delta)
        x = h[rows.long()].to(F64)
        if delta is not None:
            x = (h[rows.long()] + delta[rows.long()].to(h.dtype)).to(F64)
        inv = 1.0 / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
        out.copy_((x * inv * weight.to(F64)).to(out.dtype))

    def linear(self, x, w, bias, out):
        y = x.to(F64) @ w.to(F64).T
        if bias is not None:
            y = y + bias.to(F64)
        out.copy_(y.to(out.dtype))

    def qkv_rope_store(self, qkv, bias, positions, inv_freq, rotary_dim, slots, k_cache, v_cache, nq, nkv, hd,
                       page_size, out=None):
        src = _whole(qkv)
        qkv = src if out is None else out
        t = qkv.shape[0]
        x = src.to(F64)
        if bias is not None:
            x = x + bias.to(F64)
        heads = x.view(t, nq + 2 * nkv, hd).clone()
        if rotary_dim:
            half = rotary_dim // 2
            ang = (positions.to(torch.float32)[:, None] * inv_freq[None, :]).to(F64)
            cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            rot = heads[:, : nq + nkv, :rotary_dim]
            x1, x2 = rot[..., :half].clone(), rot[..., half:].clone()
            heads[:, : nq + nkv, :half] = x1 * cos - x2 * sin
            heads[:, : nq + nkv, half:rotary_dim] = x1 * sin + x2 * cos
        qkv.copy_(heads.view(t, -1).to(qkv.dtype))
        if slots is not None:
            page = (slots // page_size).long()
            off = (slots % page_size).long()
            k_new = qkv.view(t, nq + 2 * nkv, hd)[:, nq : nq + nkv]
            v_new = qkv.view(t, nq + 2 * nkv, hd)[:, nq + nkv :]
            for i in range(t):
                k_cache[page[i], :, off[i], :] = k_new[i]
                v_cache[page[i], :, :, off[i]] = v_new[i]
        return qkv

    def paged_attention(self, qkv, out, k_cache, v_cache, block_table, q_start, q_len, kv_len, nq, nkv, hd,
                        page_size, scale, window, max_q_len, max_kv_len, combine=True, singles=True):
        group = nq // nkv
        q_all = qkv.view(qkv.shape[0], nq + 2 * nkv, hd)[:, :nq].to(F64)
        for b in range(q_start.shape[0]):
            s, n, kv = int(q_start[b]), int(q_len[b]), int(kv_len[b])
            for i in range(n):
                p = kv - n + i
                lo = max(0, p - window + 1) if window else 0
                js = torch.arange(lo, p + 1)
                pages = block_table[b, (js // page_size)].long()
                assert (pages >= 0).all(), "attention would read a page that was given back"
                offs = (js % page_size).long()
                for h in range(nq):
                    kh = h // group
                    keys = k_cache[pages, kh, offs, :].to(F64)
                    vals = v_cache[pages, kh, :, offs].to(F64)
                    sc = (keys @ q_all[s + i, h]) * scale
                    pr = torch.softmax(sc, dim=0)
                    out[s + i, h * hd : (h + 1) * hd] = (pr @ vals).to(out.dtype)

    def swiglu(self, gate_up, out):
        gate_up = _whole(gate_up)
        i = out.shape[1]
        g, u = gate_up[:, :i].to(F64), gate_up[:, i:].to(F64)
        out.copy_((u * g / (1.0 + torch.exp(-g))).to(out.dtype))

    def argmax(self, logits, out):
        out.copy_(torch.argmax(logits, dim=-1).to(out.dtype))

    def sample(self, logits, temperature, top_k, top_p, uniform, out):
        for r in range(logits.shape[0]):
            t = float(temperature[r])
            if t <= 0:
                out[r] = int(torch.argmax(logits[r]))
                continue
            p = torch.softmax(logits[r].to(F64) / t, dim=-1)
            k, tp = int(top_k[r]), float(top_p[r])
            if 0 < k < p.numel():
                kth = torch.topk(p, k).values[-1]
                p = torch.where(p >= kth, p, torch.zeros_like(p))
                p = p / p.sum()
            if 0.0 < tp < 1.0:
                ps, order = torch.sort(p, descending=True, stable=True)
                cum = torch.cumsum(ps, 0)
                cut = int((cum >= tp).nonzero()[0]) + 1
                keep = torch.zeros_like(p)
                keep[order[:cut]] = ps[:cut]
                p = keep / keep.sum()
            cdf = torch.cumsum(p, 0)
            idx = int(torch.searchsorted(cdf, torch.tensor(float(uniform[r]) * float(cdf[-1]), dtype=F64)))
            out[r] = min(idx, p.numel() - 1)
