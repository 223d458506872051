"""The kernel backend: the one place from which parts reach device code.

`backend()` returns the object whose methods launch the hand-written HIP kernels
(`kernels.hip.HipKernels`).  There is no CPU implementation in the product: if
the compiled extension cannot be loaded on a machine with a GPU, `backend()`
raises.  `use_backend` lets a test put an object with the same methods in its
place (the tests' own slow emulation, to exercise the engine's bookkeeping on a
machine without a GPU).

Methods of a backend (T tokens, B requests, R rows, act = bfloat16 or float32):

  embed(token_ids i32[T], table act[V,H], out f32[T,H])
  add_rmsnorm(h f32[T,H], delta act[T,H]|None, weight act[H], eps, out act[T,H])
        h += delta in float32 (in place), out = h * rsqrt(mean(h^2) + eps) * weight
  rows_add_rmsnorm(h, delta|None, rows i32[R], weight, eps, out act[R,H])
        the same for rows `rows` only, h is not written
  linear(x act[T,K], w act[N,K], bias act[N]|None, out act|f32 [T,N])      out = x w^T + bias
  qkv_rope_store(qkv act[T,(nq+2nkv)*hd], bias|None, positions i32[T], inv_freq f32[rd/2]|None,
                 rotary_dim, slots i32[T]|None, k_cache, v_cache, nq, nkv, hd, page_size)
        adds bias, rotates the first rotary_dim features of every query and key head
        (pairs (i, i + rotary_dim/2), angle = position * inv_freq[i]) in place, and stores
        keys and values at `slots` (page * page_size + offset) of the caches, keys [P,nkv,page_size,hd],
        values [P,nkv,hd,page_size]
  paged_attention(qkv, out act[T,nq*hd], k_cache, v_cache, block_table i32[B,W], q_start i32[B],
                  q_len i32[B], kv_len i32[B], nq, nkv, hd, page_size, scale, window,
                  max_q_len, max_kv_len, combine=True, singles=True)
        query i of request b stands at position p = kv_len[b] - q_len[b] + i and reads keys
        j <= p (and j > p - window if window > 0) of that request through its block table
        (hints: singles=False says that no request brings exactly one token; combine=False lets the
        caller combine the parts of a split key range, which are then returned)
  swiglu(gate_up act[T,2I], out act[T,I])        out = silu(gate_up[:, :I]) * gate_up[:, I:]
  argmax(logits f32[R,V], out i32[R])            lowest index among equal maxima
  sample(logits f32[R,V], temperature f32[R], top_k i32[R], top_p f32[R], uniform f32[R], out i32[R])

Beside these, a backend has fused variants that fold neighbouring operations into one kernel.  They are part of
the contract too (`KernelBackend` below): each returns None (False for the decode attention) where it does not
cover a case, and the caller then takes the unfused way.
"""
from __future__ import annotations

import contextlib

_backend = None


class KernelBackend:
    """What parts may call on a backend beyond the operations listed above, with the answers of a backend that
    fuses nothing.  `kernels.hip.HipKernels` overrides them where its kernels cover the shapes."""

    name = "abstract"
    max_head_dim = 256      # the widest attention head the kernels take: a part refuses more when it is built
    fused_rows = 0          # products whose x operand is computed while it is staged take at most this many rows

    def pinned_stream(self):
        """Context manager within which every launch goes to the stream that is current on entry."""
        return contextlib.nullcontext()

    def residual_dtype(self, n_tokens, act_dtype):
        """The type of a step's residual stream: float32, or int64 (64-bit fixed point in units of 2^-32) where the
        backend's products can add themselves into the stream (`residual=`)."""
        import torch

        return torch.float32

    def residual_add(self, h, delta) -> None:
        """h += delta in place, for a residual stream of either kind: delta act [T, H] or float32 partial sums
        [S, T, H].  For norms other than the built-in one (whose kernel adds and normalises in one pass): plain
        tensor arithmetic, so that such a norm need not know how the stream is kept."""
        import torch

        d = delta.sum(0, dtype=torch.float32) if delta.dim() == 3 else delta.float()
        if h.dtype == torch.int64:
            h += torch.round(d.double() * 4294967296.0).to(torch.int64)
        else:
            h += d

    def residual_values(self, h):
        """The residual stream as a float32 tensor [T, H] (a copy if it is kept in fixed point)."""
        import torch

        return (h.double() * (1.0 / 4294967296.0)).float() if h.dtype == torch.int64 else h

    def product(self, x, w, unrounded=False, residual=None):
        """x w^T as act [m, n], or as float32 partial sums [splits, m, n] for a consumer that adds them up; or, given
        a residual stream in fixed point that the backend can add the product into, that stream."""
        raise NotImplementedError

    def product_normed(self, h, delta, norm_weight, w):
        """((h + delta) * norm_weight) w^T without the rows' 1/rms factor: (float32 partial sums [S, T, N], row sums
        of squares [S2, T], h + delta as a new tensor), or None."""
        return None

    def product_swiglu(self, gate_up, row_ss, hidden, eps, w, residual=None):
        """swiglu(scale * sum of the partial sums gate_up) w^T as float32 partial sums (or added into `residual`,
        which is then returned), or None."""
        return None

    def product_attention(self, part_o, part_ml, w, residual=None):
        """(the combined parts of a split attention) w^T as float32 partial sums (or added into `residual`, which is
        then returned), or None."""
        return None

    def gate_up_swiglu(self, x, w):
        """silu(x Wgate^T) * (x Wup^T) as act [T, I] in one kernel, or None."""
        return None

    def attention_decode_fused(self, *args, **kwargs):
        """Bias, rotation, cache store and attention for single decoded tokens straight from the QKV product's partial
        sums; False if not covered (nothing was done), else what paged_attention returns."""
        return False

    def combine_attention(self, part_o, part_ml, out):
        """out act [T, nq*hd] from the parts of a split attention."""
        raise NotImplementedError

    def rope_table(self, positions, inv_freq):
        """float32 [T, half, 2]: (cos, sin) of every token's angles, for the kernels that rotate; or None."""
        return None


class KernelsUnavailable(RuntimeError):
    pass


def backend():
    global _backend
    if _backend is None:
        from .hip import HipKernels  # raises KernelsUnavailable with the reason

        _backend = HipKernels()
    return _backend


def use_backend(obj) -> None:
    """Install `obj` as the backend (None restores the default).  For tests."""
    global _backend
    _backend = obj


_tuning_dir = None
library_tuning = False      # whether the library's bfloat16 products are chosen by measurement (tune_library_products)


def tune_library_products(enable: bool = True) -> None:
    """Let the library's matrix products (the many-row bfloat16 products, torch.mm) be chosen by measurement: the
    first time a shape is multiplied outside a graph capture, torch's TunableOp times the library's candidates for
    it (about a second per shape with the limits set here) and keeps the fastest for the life of the process; the
    library's own first choice is up to a third slower on some shapes (the 2,048 x 9,728 x 896 product: 53 us
    against 40).  Process-wide, off unless asked for: a step with new shapes waits for the measurement, and which
    candidate wins may differ from run to run, and with it the last bits of a result."""
    global _tuning_dir, library_tuning
    import torch.cuda.tunable as tunable

    if enable and _tuning_dir is None:
        import os
        import tempfile

        _tuning_dir = tempfile.TemporaryDirectory(prefix="egpt_tuning_")      # TunableOp writes its picks to a file
        tunable.set_filename(os.path.join(_tuning_dir.name, "picks.csv"))
        tunable.set_max_tuning_duration(30)
        tunable.set_max_tuning_iterations(20)
    tunable.enable(bool(enable))
    tunable.tuning_enable(bool(enable))
    library_tuning = bool(enable)
