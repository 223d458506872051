"""ctypes binding of the gfx950 kernel library: shape and dtype checks on the host, then the launch.

Every operand is checked against what the kernel and its grid assume before anything is
launched; a mismatch raises here instead of faulting on the device.  Launches go to torch's
current stream, so they order with torch's own work and can be captured into a graph.
"""
from __future__ import annotations

import ctypes

import torch

from . import KernelBackend, KernelsUnavailable

_F32, _BF16, _I32, _I64 = torch.float32, torch.bfloat16, torch.int32, torch.int64
_DT = {_F32: 0, _BF16: 1}


def _load_library() -> ctypes.CDLL:
    if not torch.cuda.is_available():
        raise KernelsUnavailable(
            "no GPU is visible to torch; this engine has no CPU path (its kernels are HIP code for gfx950)"
        )
    from ..csrc import build

    try:
        path = build.ensure_built()
        lib = ctypes.CDLL(path)
    except (build.BuildError, OSError) as e:
        raise KernelsUnavailable(f"the HIP kernel library could not be built or loaded: {e}") from e
    if lib.egpt_abi_version() != 16:
        raise KernelsUnavailable(f"{path} has an unexpected ABI version")
    return lib


class _FirstChoice:
    """Within it the library's products are its own first choice even where products are chosen by measurement:
    for the products with float32 output, which that measurement does not cover and which run another, slower
    way while it is on (the 2,048 x 1,152 x 896 product: 32 us against 12), and for products of a few dozen rows,
    where it gains nothing and errs now and then."""

    def __enter__(self):
        from . import library_tuning

        self.was_on = library_tuning
        if self.was_on:
            torch.cuda.tunable.enable(False)

    def __exit__(self, *exc):
        if self.was_on:
            torch.cuda.tunable.enable(True)
        return False


class _PinnedStream:
    def __init__(self, kernels):
        self.kernels = kernels

    def __enter__(self):
        self.before = self.kernels._pinned
        self.kernels._pinned = torch.cuda.current_stream().cuda_stream

    def __exit__(self, *exc):
        self.kernels._pinned = self.before
        return False


class HipKernels(KernelBackend):
    name = "hip-gfx950"

    def __init__(self):
        lib = _load_library()
        self.lib = lib
        self._pinned = None
        vp, i, f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        lib.egpt_error_string.restype = ctypes.c_char_p
        lib.egpt_error_string.argtypes = [i]
        sigs = {
            "egpt_embed": [vp, vp, vp, i, i, i, i, i, vp],
            "egpt_add_rmsnorm": [vp, i, vp, i, i, vp, vp, f, vp, i, i, i, vp],
            "egpt_swiglu": [vp, i, vp, i, i, f, vp, i, i, i, vp],
            "egpt_qkv_rope_store": [vp, i, vp, i, i, f, vp, vp, vp, vp, vp, i, vp, vp, vp, i, i, i, i, i, i, vp],
            "egpt_rope_table": [vp, vp, vp, i, i, vp],
            "egpt_gemm_skinny_norm": [vp, i, vp, vp, i, vp, vp, vp, vp, i, i, i, i, i, vp],
            "egpt_gemm_skinny_swiglu": [vp, i, vp, i, i, f, vp, vp, vp, i, i, i, i, i, vp],
            "egpt_gemm_skinny_attn": [vp, vp, i, i, i, vp, vp, vp, i, i, i, i, vp],
            "egpt_attention_combine": [vp, vp, vp, i, i, i, vp],
            "egpt_paged_attention_tiled": [vp, vp, vp, vp, vp, i, vp, vp, vp, i, i, i, i, i, i, f, i, i, i, vp, vp, i, i,
                                           i, vp],
            "egpt_paged_attention_decode": [vp, vp, vp, vp, vp, vp, vp, i, vp, vp, i, i, i, i, i, f, i, i, i, i, i, vp],
            "egpt_attention_decode_fused": [vp, i, vp, i, i, f, vp, vp, vp, vp, vp, vp, vp, vp, vp, i, vp, vp, i, i, i,
                                            i, i, f, i, i, i, i, i, vp],
            "egpt_linear": [vp, vp, vp, vp, i, i, i, i, i, vp],
            "egpt_gemm_f32": [vp, vp, vp, vp, i, i, i, i, vp],
            "egpt_gemm_skinny": [vp, vp, vp, vp, vp, vp, i, i, i, i, i, vp],
            "egpt_paged_attention": [vp, vp, vp, vp, vp, i, vp, vp, vp, i, i, i, i, i, i, f, i, i, vp],
            "egpt_paged_attention_mfma": [vp, vp, vp, vp, vp, vp, vp, i, vp, vp, vp, i, i, i, i, i, i, f, i, i, i, i, vp],
            "egpt_attention_any_tiled": [vp, vp, vp, vp, vp, i, vp, vp, vp, i, i, i, i, i, i, f, i, i, vp],
            "egpt_attention_any_decode": [vp, vp, vp, vp, vp, vp, vp, i, vp, vp, i, i, i, i, i, f, i, i, i, vp],
            "egpt_argmax": [vp, vp, vp, i, i, vp],
            "egpt_sample": [vp, vp, vp, vp, vp, vp, vp, i, i, vp],
            "egpt_sample_wide": [vp, vp, vp, vp, vp, vp, vp, i, i, vp],
            "egpt_gemm_gate_up_swiglu": [vp, vp, vp, i, i, i, i, vp],
        }
        lib.egpt_sample_workspace.restype = ctypes.c_size_t
        lib.egpt_sample_workspace.argtypes = [i, i]
        for name, argtypes in sigs.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = i

    # ------------------------------------------------------------------ helpers
    def _stream(self):
        """The stream to launch on: torch's current one.  Asking torch costs several microseconds, and a step
        launches a couple of hundred kernels, so a model's forward pass asks once (`pinned_stream`)."""
        return self._pinned if self._pinned is not None else torch.cuda.current_stream().cuda_stream

    def pinned_stream(self):
        """Context manager: within it every launch goes to the stream that is current on entry.  The caller
        promises not to change the current stream inside (graph capture changes it before the forward pass
        is entered, which is fine)."""
        return _PinnedStream(self)

    def _run(self, name: str, *args) -> None:
        code = getattr(self.lib, name)(*args)
        if code != 0:
            raise RuntimeError(f"{name}: {self.lib.egpt_error_string(code).decode()}")

    @staticmethod
    def _ptr(t: torch.Tensor | None):
        return None if t is None else t.data_ptr()

    @staticmethod
    def _need(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
        if not isinstance(t, torch.Tensor) or not t.is_cuda:
            raise TypeError(f"{name} must be a tensor on the GPU")
        if not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous")
        if dtype is not None and t.dtype != dtype:
            raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
        if shape is not None and tuple(t.shape) != tuple(shape):
            raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")

    @staticmethod
    def _act(t: torch.Tensor, name: str) -> int:
        if t.dtype not in _DT:
            raise TypeError(f"{name} must be float32 or bfloat16, got {t.dtype}")
        return _DT[t.dtype]

    def _caches(self, k_cache, v_cache, dtype, nkv: int, page_size: int, hd: int) -> None:
        self._need(k_cache, "k_cache", dtype)
        self._need(v_cache, "v_cache", dtype)
        if k_cache.dim() != 4 or tuple(k_cache.shape[1:]) != (nkv, page_size, hd):
            raise ValueError(f"k_cache must be [pages, {nkv}, {page_size}, {hd}], got {tuple(k_cache.shape)}")
        if v_cache.dim() != 4 or tuple(v_cache.shape[1:]) != (nkv, hd, page_size):
            raise ValueError(f"v_cache must be [pages, {nkv}, {hd}, {page_size}], got {tuple(v_cache.shape)}")
        if v_cache.shape[0] != k_cache.shape[0]:
            raise ValueError("k_cache and v_cache must have the same number of pages")

    def _product(self, t: torch.Tensor, name: str, act_dtype, rows: int, cols: int) -> int:
        """A product operand: act [rows, cols] (returns 0) or float32 partial sums [splits, rows, cols] (returns splits)."""
        if t.dim() == 3:
            self._need(t, name, _F32, (t.shape[0], rows, cols))
            return int(t.shape[0])
        self._need(t, name, act_dtype, (rows, cols))
        return 0

    # ------------------------------------------------------------------ kernels
    def embed(self, token_ids, table, out):
        dt = self._act(table, "table")
        v, h = table.shape
        t = token_ids.shape[0]
        self._need(token_ids, "token_ids", _I32, (t,))
        self._need(table, "table")
        self._need(out, "out", None, (t, h))
        self._run("egpt_embed", token_ids.data_ptr(), table.data_ptr(), out.data_ptr(), self._fixed(out, "out"), t, h, v,
                  dt, self._stream())

    # ------------------------------------------------------------------ the residual stream in fixed point
    fixed_residual_elements = 1 << 20    # splits x rows x columns of a product that is added with atomics, at most

    def residual_dtype(self, n_tokens: int, act_dtype) -> torch.dtype:
        """The type of the residual stream of a step: float32, or for few tokens in bfloat16 64-bit fixed point (int64
        in units of 2^-32).  Products whose k range is split over workgroups then add their parts straight into the
        stream with integer atomics (`residual=` below), which gives the same bits in any order, and the kernels
        that read the stream read one small tensor instead of every workgroup's partial sums."""
        return _I64 if (act_dtype == _BF16 and 0 < n_tokens <= self.fused_rows) else _F32

    @staticmethod
    def _fixed(t: torch.Tensor, name: str) -> int:
        if t.dtype not in (_F32, _I64):
            raise TypeError(f"{name} (a residual stream) must be float32 or int64 fixed point, got {t.dtype}")
        return 1 if t.dtype == _I64 else 0

    def _residual_target(self, residual, t: int, n: int, splits: int):
        """The stream to add a [t, n] product into, or None if it is to be returned as partial sums."""
        if residual is None or residual.dtype != _I64 or tuple(residual.shape) != (t, n):
            return None
        if splits * t * n > self.fixed_residual_elements:
            return None                  # so many atomics that partial sums and their reader are faster
        self._need(residual, "residual", _I64, (t, n))
        return residual

    def add_rmsnorm(self, h, delta, weight, eps, out):
        t, hid = h.shape
        dt = self._act(out, "out")
        self._need(h, "h")
        self._need(weight, "weight", out.dtype, (hid,))
        self._need(out, "out", None, (t, hid))
        splits = self._product(delta, "delta", out.dtype, t, hid) if delta is not None else 0
        self._run("egpt_add_rmsnorm", h.data_ptr(), self._fixed(h, "h"), self._ptr(delta), splits, t, None,
                  weight.data_ptr(), float(eps), out.data_ptr(), t, hid, dt, self._stream())

    def rows_add_rmsnorm(self, h, delta, rows, weight, eps, out):
        t, hid = h.shape
        r = rows.shape[0]
        dt = self._act(out, "out")
        self._need(h, "h")
        self._need(rows, "rows", _I32, (r,))
        self._need(weight, "weight", out.dtype, (hid,))
        self._need(out, "out", None, (r, hid))
        splits = self._product(delta, "delta", out.dtype, t, hid) if delta is not None else 0
        self._run("egpt_add_rmsnorm", h.data_ptr(), self._fixed(h, "h"), self._ptr(delta), splits, t, rows.data_ptr(),
                  weight.data_ptr(), float(eps), out.data_ptr(), r, hid, dt, self._stream())

    @staticmethod
    def _library_rows(m: int, n: int, k: int) -> bool:
        """Whether a bfloat16 product of m rows goes to the library (the reference uses cuBLAS for every linear
        layer).  Up to 16 rows never, beyond 64 always.  Between them the own kernels win where the k range
        has to be split over workgroups (an output narrower than k) and on small matrices, where a step is a
        chain of round trips to memory; the library wins on large ones, which it streams at 4 to 5 TB/s."""
        if m <= 16:
            return False
        if m > 64:
            return True
        if n < k:
            return False
        if m <= 32 and n >= 65536:
            # an output matrix over a whole vocabulary, up to 32 rows: the own kernel with four wavefronts (measured
            # on 151,936 x 896: 51 / 53 / 59 us at 17 / 24 / 32 rows against the library's 58 / 57 / 59; on 152,064 x
            # 3,584: 215 / 218 / 223 against 243 / 248 / 255; at 48 and 64 rows the library wins, 71 against 100 us and
            # 217 against 246, and workgroups of 8 or 16 wavefronts are slower than either)
            return False
        # (33 to 64 rows, measured with the weights coming from memory: 2,048 x 1,536 in 7.8 us against the library's 9.8,
        # 1,536 x 1,536 7.7 against 9.2, 2,560 x 2,048 8.9 against 12.0, 2,048 x 2,048 8.1 against 11.8; 4,608 x 3,584 18.9
        # either way, 3,584 x 3,584 14.2 against 13.7, 7,168 x 5,120 25.8 against 22.7)
        return n * k >= (6 << 20 if m > 32 else 16 << 20)

    def linear(self, x, w, bias, out):
        m, k = x.shape
        n = w.shape[0]
        dt = self._act(x, "x")
        self._need(x, "x")
        self._need(w, "w", x.dtype, (n, k))
        if bias is not None:
            self._need(bias, "bias", x.dtype, (n,))
        if out.dtype not in (x.dtype, _F32):
            raise TypeError(f"out must be {x.dtype} or float32, got {out.dtype}")
        self._need(out, "out", None, (m, n))
        if m == 0:
            return out
        if x.dtype == _BF16 and k % 8 == 0:
            to_f32 = out.dtype == _F32
            if not self._library_rows(m, n, k):
                # weight-streaming MFMA kernel
                self._run("egpt_gemm_skinny", x.data_ptr(), w.data_ptr(), self._ptr(bias),
                          out.data_ptr() if to_f32 else None, None if to_f32 else out.data_ptr(), None, m, n, k, 1,
                          4, self._stream())
                return out
            # many rows: the library's matrix product; float32 output (logits) unrounded
            if to_f32:
                with _FirstChoice():
                    torch.mm(x, w.t(), out_dtype=_F32, out=out)
                if bias is not None:
                    out += bias
            elif m <= 64 and n * k < 64 << 20:
                # a few dozen rows of a matrix that is not large: the library's first choice streams the weights well,
                # and a measurement of candidates that all take a few microseconds picks a poor one now and then (a
                # 64 x 17,920 x 1,536 product at 35 us instead of 18, once in a few runs); on 37,888 x 3,584 the
                # measured choice is the better one every time (51 us against 60)
                with _FirstChoice():
                    if bias is None:
                        torch.mm(x, w.t(), out=out)
                    else:
                        torch.addmm(bias, x, w.t(), out=out)
            elif bias is None:
                torch.mm(x, w.t(), out=out)
            else:
                torch.addmm(bias, x, w.t(), out=out)
            return out
        if x.dtype == _F32 and k % 4 == 0:
            # the float32 product on the matrix cores, the whole k range in one piece
            self._run("egpt_gemm_f32", x.data_ptr(), w.data_ptr(), self._ptr(bias), out.data_ptr(), m, n, k, 1,
                      self._stream())
            return out
        self._run("egpt_linear", x.data_ptr(), w.data_ptr(), self._ptr(bias), out.data_ptr(), m, n, k, dt,
                  1 if out.dtype == _F32 else 0, self._stream())
        return out

    @staticmethod
    def _f32_splits(n: int, k: int) -> int:
        """Into how many ranges the float32 product splits k: enough workgroups for a narrow result with few rows.
        The count depends on the matrix alone, never on the rows, so that a row's partial sums, and with them
        every value of the 32-bit path, are the same bits in whatever batch the row is computed."""
        steps = -(-k // 64)
        # at most 12 ranges: a step of few rows wants many workgroups, a prompt pays for every range with a float32
        # copy of its output (measured at the 0.5B sizes, decode step at batch 8 / 2,048-token prefill: 1.73 / 24.4 ms
        # with at most 8 ranges, 1.65 / 24.6 with 12, 1.58 / 26.5 with 16)
        s = min(steps, max(1, 512 // -(-n // 64)), 12)
        per = -(-steps // s)
        return -(-steps // per)

    @staticmethod
    def _n_splits(m: int, n: int, k: int) -> int:
        """How many workgroups share the k range of a skinny product: enough to fill the GPU when n is small,
        bounded so that the partial sums stay smaller than the weights they came from."""
        steps = -(-k // 128)
        n_blocks = -(-n // 64)
        # a long k range is worth more workgroups: each one's stream is a chain of steps, one load ahead
        most = 2048 if steps >= 14 else 1024
        # more than one tile of rows: x weighs as much as w in every workgroup and the partial sums more than with
        # few rows, so fewer, longer ranges (their x travels through registers a step ahead); a few more on a small
        # matrix (measured inside the model at 896 x 4,864: 1.291 -> 1.260 ms a step at batch 24 and 1.790 -> 1.771 at 64
        # with 13 ranges instead of 10, 1.853 with 19; at 1,536 x 8,960, 13 ranges cost 3 to 7 %)
        s = min(steps, max(1, most // n_blocks), max(1, k // (2 * m)), 20 if m <= 16 else 13 if n * k <= 8 << 20 else 10)
        if m > 16 and steps <= 16:
            # a short k range and more than one tile of rows: no more workgroups than CUs (measured at 64 rows: 2,048 x
            # 1,536 in 7.8 us with 6 ranges, 192 workgroups, against 9.0 with 12; 2,560 x 2,048 8.9 with 6 against 11.3 with
            # 8, 320 workgroups; 2,048 x 2,048 8.1 with 8, 256 workgroups; at 32 rows 5.6 against 6.3 and 7.0 against 7.9)
            s = min(s, max(1, 256 // n_blocks))
        per = -(-steps // s)
        return -(-steps // per)

    fused_rows = 16     # products with a computed x operand take at most this many rows
    normed_rows_cols = 400_000   # rows x columns beyond which the norm is not folded into a product

    # workgroups of the product with the norm folded in that the GPU holds at once, by wavefronts per workgroup: the
    # kernel's 128 to 136 registers a lane leave a SIMD three wavefronts, so a CU holds three workgroups of four
    # wavefronts or one wider one (seen in the kernels' own timestamps: of 504 workgroups of eight wavefronts, 280
    # start at once and the others when those have ended)
    _normed_resident = {4: 768, 8: 256, 16: 256}

    @classmethod
    def _normed_shape(cls, n: int, k: int) -> tuple[int, int]:
        """(splits of the k range, wavefronts per workgroup) of the product with the norm folded in.  Two steps of
        128 per workgroup are staged at once, which is the kernel's shortest chain of round trips; one step where
        the matrix is so small that this leaves the GPU short of workgroups.  Every workgroup computes its share
        of x again and waits for its first bytes once, so the workgroups should all be resident together: the
        width whose workgroups need the fewest rounds, and among those the narrowest (measured: 4,608 x 3,584 at
        8 rows takes 9.7 us with 252 workgroups of 16 wavefronts, 12.2 with 504 of 8; 17,920 x 1,536 is fastest
        with 420 of 16; the matrices of the 0.5B sizes fit in one round at any width and are fastest at 4)."""
        steps = -(-k // 128)
        per = max(2, -(-steps // 20))
        if -(-n // 64) * -(-steps // per) < 192:
            per = max(1, -(-steps // 20))
        s = -(-steps // per)
        rounds = {w: -(-(-(-n // (16 * w)) * s) // cls._normed_resident[w]) for w in (4, 8, 16)}
        waves = min((4, 8, 16), key=lambda w: (rounds[w], w))
        return s, waves

    def product_normed(self, h, delta, norm_weight, w, waves=None, splits=None):
        """((h + delta) * norm_weight) w^T without the rows' 1/rms factor, for few rows in bfloat16.
        Returns (float32 partial sums [S, T, N], row sums of squares [S, T], h + delta as a new tensor),
        or None if this case is not covered or not worth it (the caller then runs the norm by itself)."""
        t, k = h.shape
        n = w.shape[0]
        if w.dtype != _BF16 or not 0 < t <= self.fused_rows or k % 8 or not h.is_cuda:
            return None
        if splits is None and waves is None and (t * n > self.normed_rows_cols or n * k >= 64 << 20
                                                 or (n * k >= 16 << 20 and t * n > 150_000)):
            # every workgroup reads its k range of all rows of h and of delta's partial sums: on a matrix this large
            # (or with this many rows and columns) that costs more than a norm kernel of its own (measured on a
            # 37,888 x 3,584 product behind 14 partial sums: 80 us against 6 + 58; on a 17,920 x 1,536 one with 16 rows
            # 26 us against 5 + 13 when the norm still had 19 partial sums to add; with the stream in fixed point, which
            # it reads as it is, folding wins there up to 8 rows: 1.597 -> 1.552 ms a step of the 1.5B sizes, and loses
            # at 16: 1.819 -> 1.831; on 9,728 x 896 it always wins)
            return None
        if delta is not None and (delta.dim() != 3 or delta.dtype != _F32):
            return None
        fixed = self._fixed(h, "h")
        if fixed and delta is not None:
            return None                  # a stream in fixed point with something still to add: the norm's own kernel adds it
        self._need(h, "h")
        self._need(w, "w", _BF16, (n, k))
        self._need(norm_weight, "norm_weight", _BF16, (k,))
        d_splits = 0
        if delta is not None:
            d_splits = int(delta.shape[0])
            self._need(delta, "delta", _F32, (d_splits, t, k))
        auto_s, auto_w = self._normed_shape(n, k)
        s, waves = splits or auto_s, waves or auto_w
        out = torch.empty((s, t, n), dtype=_F32, device=h.device)
        ss = torch.empty((s, t), dtype=_F32, device=h.device)
        h_new = h if fixed else torch.empty_like(h)      # a stream in fixed point is complete: nothing is added here
        self._run("egpt_gemm_skinny_norm", h.data_ptr(), fixed, None if fixed else h_new.data_ptr(), self._ptr(delta),
                  d_splits, norm_weight.data_ptr(), w.data_ptr(), out.data_ptr(), ss.data_ptr(), t, n, k, s, waves,
                  self._stream())
        return out, ss, h_new

    def product_swiglu(self, gate_up, row_ss, hidden, eps, w, max_splits=20, waves=None, residual=None):
        """swiglu(scale * sum gate_up) w^T for float32 partial sums gate_up [S, T, 2I]; scale is the rows' 1/rms
        from row_ss [S2, T] (or 1).  Returns float32 partial sums [S3, T, N] or None if not covered; with a residual
        stream in fixed point [T, N] the product is added into it instead and the stream is returned."""
        if gate_up.dim() != 3 or gate_up.dtype != _F32 or w.dtype != _BF16:
            return None
        g_splits, t, two_i = gate_up.shape
        n, k = w.shape
        if two_i != 2 * k or not 0 < t <= self.fused_rows or k % 8:
            return None
        if waves is None and n >= 1536:
            # every workgroup computes its share of x from gate_up's partial sums, and with this many columns there
            # are dozens of workgroups per share: a SwiGLU kernel of its own and the plain product are faster
            # (measured inside the model at 8 rows: 15 us against 17 at 1,536 columns, 37 against 54 at 3,584)
            return None
        self._need(gate_up, "gate_up", _F32)
        self._need(w, "w", _BF16)
        ss_splits = 0
        if row_ss is not None:
            ss_splits = int(row_ss.shape[0])
            self._need(row_ss, "row_ss", _F32, (ss_splits, t))
        s = min(self._n_splits(t, n, k), max_splits)
        steps = -(-k // 128)
        s = -(-steps // -(-steps // s))
        if waves is None:
            # every workgroup computes its share of x from all of gate_up's partial sums: with few columns,
            # wider workgroups (which share the staged x) do that work fewer times
            waves = 8 if -(-n // 64) * s <= 512 else 4
        target = self._residual_target(residual, t, n, s)
        out = None if target is not None else torch.empty((s, t, n), dtype=_F32, device=w.device)
        self._run("egpt_gemm_skinny_swiglu", gate_up.data_ptr(), int(g_splits), self._ptr(row_ss), ss_splits, int(hidden),
                  float(eps), w.data_ptr(), self._ptr(out), self._ptr(target), t, n, k, s, waves, self._stream())
        return out if target is None else target

    def product_attention(self, part_o, part_ml, w, max_splits=None, waves=None, residual=None):
        """(combined attention output) w^T from the parts of a split attention: part_o [S, T, nq, hd],
        part_ml [S, T, nq, 2].  Returns float32 partial sums [S2, T, N] or None if not covered; with a residual
        stream in fixed point [T, N] the product is added into it instead and the stream is returned."""
        a_splits, t, nq, hd = part_o.shape
        n, k = w.shape
        if w.dtype != _BF16 or k != nq * hd or not 0 < t <= self.fused_rows or hd % 8 or a_splits > 64:
            return None
        if n * k > 16 << 20:
            # every workgroup combines the parts of its range of k before it has anything to multiply, and on a matrix
            # this large there are some 40 columns of workgroups that each do so: a kernel that combines the parts once
            # and the plain product are faster (measured, us for 8 rows: 5,120 x 5,120 28.3 against 18.2; 3,584 x 3,584
            # 11.7 against 11.8, 2,048 x 2,048 6.2 against 8.8, 896 x 896 4.1 against 6.6)
            return None
        self._need(part_o, "part_o", _F32)
        self._need(part_ml, "part_ml", _F32, (a_splits, t, nq, 2))
        self._need(w, "w", _BF16)
        # a short k range: few splits, whose partial sums the next product's prologue adds up in registers; a
        # long one: a step of 128 per workgroup, and workgroups of 8 wavefronts that share the combined x
        if max_splits is None:
            # (added into the residual stream, splits cost nobody a read: a step of 128 per workgroup; measured at the
            # 0.5B sizes, batch 8: 0.889 -> 0.874 ms a step with 7 splits instead of 4)
            max_splits = (8 if residual is not None and residual.dtype == _I64 else 4) if k <= 1024 else 14
        if waves is None:
            waves = 4 if k <= 1024 else 8
        s = min(self._n_splits(t, n, k), max_splits)
        steps = -(-k // 128)
        per = -(-steps // s)
        s = -(-steps // per)
        if -(-per * 128 // hd) + 1 > 8:
            return None
        target = self._residual_target(residual, t, n, s)
        out = None if target is not None else torch.empty((s, t, n), dtype=_F32, device=w.device)
        self._run("egpt_gemm_skinny_attn", part_o.data_ptr(), part_ml.data_ptr(), int(a_splits), int(nq), int(hd),
                  w.data_ptr(), self._ptr(out), self._ptr(target), t, n, s, waves, self._stream())
        return out if target is None else target

    def gate_up_swiglu(self, x, w, groups=None):
        """silu(x Wgate^T) * (x Wup^T) as act [T, I] for w = [Wgate; Wup] ([2I, k]), in one kernel: for 17 to 64
        rows in bfloat16.  Returns None where another way is faster or the case is not covered."""
        t, k = x.shape
        if x.dtype != _BF16 or w.dtype != _BF16 or not self.fused_rows < t <= 64 or k % 8 or w.shape[0] % 2:
            return None
        inter = w.shape[0] // 2
        if groups is None:
            if 2 * inter * k >= 16 << 20:
                # every workgroup reads all of x from L2, which on a large matrix costs more than the float32 product
                # and the SwiGLU kernel that this saves (measured at 64 rows: 12.8 us against 14.5 on 9,728 x 896,
                # 37 against 21 on 17,920 x 1,536)
                return None
            # two column groups per workgroup halve the reads of x; on small matrices one gives more workgroups
            groups = 2 if inter * k >= 1 << 20 else 1
        self._need(x, "x", _BF16)
        self._need(w, "w", _BF16, (2 * inter, k))
        out = torch.empty((t, inter), dtype=_BF16, device=x.device)
        self._run("egpt_gemm_gate_up_swiglu", x.data_ptr(), w.data_ptr(), out.data_ptr(), t, inter, k, groups,
                  self._stream())
        return out

    def combine_attention(self, part_o, part_ml, out):
        """out act [T, nq*hd] from the parts of a split attention (what paged_attention does with combine=True)."""
        a_splits, t, nq, hd = part_o.shape
        self._need(part_o, "part_o", _F32)
        self._need(part_ml, "part_ml", _F32, (a_splits, t, nq, 2))
        self._need(out, "out", _BF16, (t, nq * hd))
        self._run("egpt_attention_combine", part_o.data_ptr(), part_ml.data_ptr(), out.data_ptr(), t * nq, hd,
                  int(a_splits), self._stream())

    def product(self, x, w, unrounded=False, residual=None):
        """x w^T for a consumer that takes partial sums: returns act [m, n], or float32 [splits, m, n] whose sum
        over splits is the product (few rows in bfloat16: the k range is split over workgroups).  unrounded=True
        asks for float32 also from the many-row library product (as [1, m, n]): for consumers that go on computing
        with the values before they round, such as the bias and rotation of queries and keys, where a rounding
        in between is the largest single contribution to the bfloat16 error of the logits.  With a residual stream
        in fixed point [m, n], a product of few rows is added into it instead and the stream is returned."""
        m, k = x.shape
        n = w.shape[0]
        if x.dtype == _BF16 and m > 0 and k % 8 == 0 and not self._library_rows(m, n, k):
            self._need(x, "x")
            self._need(w, "w", x.dtype, (n, k))
            s = self._n_splits(m, n, k)
            target = self._residual_target(residual, m, n, s) if m <= self.fused_rows else None
            if m > 16 and n >= 4096:
                # more than one tile of rows and many columns: the kernel that keeps x in LDS for a k range of up
                # to 8 steps; as few splits as that allows (none at all for k <= 1024: no partial sums)
                steps = -(-k // 128)
                s = -(-steps // 8)
            out = None if target is not None else torch.empty((s, m, n), dtype=_F32, device=x.device)
            self._run("egpt_gemm_skinny", x.data_ptr(), w.data_ptr(), None, self._ptr(out), None, self._ptr(target),
                      m, n, k, s, 4, self._stream())
            return out if target is None else target
        if unrounded and x.dtype == _BF16 and m > 0 and k % 8 == 0:
            # many rows: the library's product (the reference uses cuBLAS for every linear layer), written out in
            # float32; it goes on as a single "partial sum" [1, m, n]
            self._need(x, "x")
            self._need(w, "w", x.dtype, (n, k))
            out = torch.empty((1, m, n), dtype=_F32, device=x.device)
            with _FirstChoice():
                torch.mm(x, w.t(), out_dtype=_F32, out=out[0])
            return out
        if x.dtype == _F32 and m > 0 and k % 4 == 0:
            self._need(x, "x")
            self._need(w, "w", _F32, (n, k))
            s = self._f32_splits(n, k)
            out = torch.empty((s, m, n), dtype=_F32, device=x.device)
            self._run("egpt_gemm_f32", x.data_ptr(), w.data_ptr(), None, out.data_ptr(), m, n, k, s, self._stream())
            return out
        out = torch.empty((m, n), dtype=x.dtype, device=x.device)
        return self.linear(x, w, None, out)

    def rope_table(self, positions, inv_freq):
        """float32 [T, half, 2]: (cos, sin) of float(positions[t]) * inv_freq[i].  A step's angles are the same in
        every layer; the kernels that rotate take this table in place of computing the values again."""
        t, half = positions.shape[0], inv_freq.shape[0]
        self._need(positions, "positions", _I32, (t,))
        self._need(inv_freq, "inv_freq", _F32, (half,))
        out = torch.empty((t, half, 2), dtype=_F32, device=positions.device)
        self._run("egpt_rope_table", positions.data_ptr(), inv_freq.data_ptr(), out.data_ptr(), t, half, self._stream())
        return out

    def qkv_rope_store(self, qkv, bias, positions, inv_freq, rotary_dim, slots, k_cache, v_cache, nq, nkv, hd,
                       page_size, out=None, row_ss=None, hidden=0, eps=0.0, cos_sin=None):
        """qkv: act [T, W] or float32 partial sums [S, T, W]; out: act [T, W] (default: qkv itself, in place).
        row_ss float32 [S2, T]: the product still lacks each row's factor 1/sqrt(sum_s row_ss[s] / hidden + eps).
        cos_sin: rope_table(positions, inv_freq), if the caller has it."""
        width = (nq + 2 * nkv) * hd
        t = qkv.shape[-2]
        if out is None:
            if qkv.dim() == 3:
                raise ValueError("partial sums need an output tensor")
            out = qkv
        dt = self._act(out, "out")
        self._need(out, "out", None, (t, width))
        splits = self._product(qkv, "qkv", out.dtype, t, width)
        self._need(positions, "positions", _I32, (t,))
        if bias is not None:
            self._need(bias, "bias", out.dtype, (width,))
        if rotary_dim:
            if rotary_dim % 2 or rotary_dim > hd:
                raise ValueError(f"rotary_dim {rotary_dim} must be even and <= head size {hd}")
            self._need(inv_freq, "inv_freq", _F32, (rotary_dim // 2,))
        if slots is not None:
            self._need(slots, "slots", _I32, (t,))
            self._caches(k_cache, v_cache, out.dtype, nkv, page_size, hd)
        ss_splits = 0
        if row_ss is not None:
            ss_splits = int(row_ss.shape[0])
            self._need(row_ss, "row_ss", _F32, (ss_splits, t))
        if cos_sin is not None:
            self._need(cos_sin, "cos_sin", _F32, (t, rotary_dim // 2, 2))
        self._run("egpt_qkv_rope_store", qkv.data_ptr(), splits, self._ptr(row_ss), ss_splits, int(hidden), float(eps),
                  out.data_ptr(), self._ptr(bias), positions.data_ptr(),
                  self._ptr(inv_freq) if rotary_dim else None, self._ptr(cos_sin) if rotary_dim else None,
                  int(rotary_dim), self._ptr(slots),
                  self._ptr(k_cache), self._ptr(v_cache), t, nq, nkv, hd, page_size, dt, self._stream())
        return out

    def paged_attention(self, qkv, out, k_cache, v_cache, block_table, q_start, q_len, kv_len, nq, nkv, hd, page_size,
                        scale, window, max_q_len, max_kv_len, combine=True, singles=True):
        """combine=False: when the kernel splits the key range, leave the parts to the caller and return
        (part_o [S, T, nq, hd], part_ml [S, T, nq, 2]); `out` is then not written.  Returns None otherwise.
        singles=False: no request brings exactly one token (a hint: the kernel that takes those apart is not launched)."""
        t = qkv.shape[0]
        b, width = block_table.shape
        dt = self._act(qkv, "qkv")
        self._need(qkv, "qkv", None, (t, (nq + 2 * nkv) * hd))
        self._need(out, "out", qkv.dtype, (t, nq * hd))
        self._caches(k_cache, v_cache, qkv.dtype, nkv, page_size, hd)
        self._need(block_table, "block_table", _I32)
        for name, v in (("q_start", q_start), ("q_len", q_len), ("kv_len", kv_len)):
            self._need(v, name, _I32, (b,))
        if max_kv_len > width * page_size:
            raise ValueError(f"block table of width {width} cannot hold {max_kv_len} tokens at page size {page_size}")
        if hd > 256:
            raise ValueError(f"head size {hd} is not supported by the attention kernels (at most 256)")
        if qkv.dtype == _BF16 and hd in (64, 128) and page_size % 16 == 0:
            # matrix-core kernel; the key range is split when there are too few (request, kv head) pairs to fill
            # the GPU, which is the case when only decoded tokens are in the batch
            if max_q_len == 1 and t == b and nq // nkv <= 16:
                # only decoded tokens: workgroups of several wavefronts per (request, kv head, key split)
                n_splits, n_waves, lean = self._decode_shape(b, nkv, hd, max_kv_len, combine)
                part_o = part_ml = None
                if n_splits > 1:
                    part_o = torch.empty((n_splits, t, nq, hd), dtype=_F32, device=qkv.device)
                    part_ml = torch.empty((n_splits, t, nq, 2), dtype=_F32, device=qkv.device)
                self._run("egpt_paged_attention_decode", qkv.data_ptr(), out.data_ptr(), self._ptr(part_o),
                          self._ptr(part_ml), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), width,
                          q_start.data_ptr(), kv_len.data_ptr(), b, nq, nkv, hd, page_size, float(scale), int(window),
                          n_splits, n_waves, 1 if combine else 0, lean, self._stream())
                return (part_o, part_ml) if (n_splits > 1 and not combine) else None
            if max_q_len > 1 and page_size & (page_size - 1) == 0:
                # prompt portions (and mixed batches): key/value tiles shared through LDS by the wavefronts of
                # a workgroup.  Few rows: small workgroups whose wavefronts split the keys, so that the GPU
                # has enough of them; many rows: 64 rows per workgroup, which read the keys fewer times.
                row_tiles = -(-t * (nq // nkv) // 16) * nkv
                # Measured (us for one layer's prompt on a GPU that is warm; row tiles of 16 rows; shape = row tiles x key
                # splits of a workgroup, 1xx the kernel of 32-row blocks, whose tiles of 64 keys must be whole pages):
                #   head size 64, 14 heads on 2:   448 tiles 24: 9.4, 44: 10.4 |  896 tiles 24: 16.9, 44: 14.7, 142: 16.4
                #     1,344 tiles 44: 20.0, 142: 21.3 | 1,792 tiles 44: 29.7, 142: 26.2 | 3,584 tiles 42: 76, 142: 53
                #     7,168 tiles (8,192 tokens) 42: 292, 142: 175 | 28,560 tiles (32,640 tokens) 42: 3,840, 142: 2,400
                #   head size 128, 12 heads on 2:  768 tiles 22: 31.0, 42: 26.1, 141: 27.8 | 1,536 tiles 42: 47.1, 141: 47.3
                #     3,072 tiles 42: 158, 141: 87;  28 heads on 4: 896 tiles 22: 28.8, 42: 16.3, 141: 19.3 | 1,792 tiles
                #     42: 40.7, 141: 30.0 | 7,168 tiles 42: 341, 141: 190;  40 heads on 8: 1,280 tiles 42: 23.2, 141: 19.6
                blocks_of_32 = page_size <= 64
                if hd == 64:
                    shape = 24 if row_tiles <= 512 else 44 if row_tiles <= 1536 or not blocks_of_32 else 142
                    if shape == 44 and row_tiles > 2048:
                        shape = 42
                else:
                    shape = 22 if row_tiles <= 192 else 42 if row_tiles <= 1024 or not blocks_of_32 else 141
                # Portions behind a prefix walk many keys per row and are few blocks of rows: the kernel of 32-row blocks
                # with 128 rows to a workgroup, and the tiles of keys of a block of rows dealt over as many workgroups
                # as give every CU one.  Measured (us, a layer; shape x workgroups that share the keys): head size 64,
                # 14 heads on 2, 512 tokens behind 4,096 / 8,192 / 32,768 keys 24x1: 35 / 70 / 257, 124x1: 32 / 59 / 196,
                # 142x1: 45 / 84 / 300, 142x4: 27 / 38 / 98; 256 tokens behind 32,768 124x1: 195, 124x4: 66, 142x8: 57; 64
                # tokens 124x1: 201, 142x16: 40; behind 2,048 keys nothing is gained (24x1: 24, 142x4: 23) and a prompt
                # without a prefix loses (2,048 tokens 142x1: 28, 142x2: 47); three portions of 512 behind 30,000 keys
                # 142x1: 283, 124x1: 397.  Head size 128, 12 heads on 2, 512 tokens behind 2,048 / 32,768 keys 42x1: 59 /
                # 643, 141x1: 59 / 665, 141x4: 30 / 185; 28 heads on 4: 141x1: 61 / 671, 141x2: 48 / 378; 40 heads on 8
                # (160 workgroups): 141x1: 103 / 679.
                key_splits = 1
                # (behind a prefix: the longest context is a few thousand tokens and at least twice the step's own)
                if (blocks_of_32 and max_kv_len >= 2 * t
                        and max_kv_len >= (self.prefix_keys if hd == 64 else self.prefix_keys // 2)):
                    shape = 142 if hd == 64 else 141
                    workgroups = -(-row_tiles // 8)
                    tiles = -(-max_kv_len // (64 * (shape % 10)))
                    key_splits = max(1, min(256 // workgroups, tiles // 4, 16))
                # Requests that bring one token (decoded tokens beside the portions) go to the decode kernel in a second
                # launch: here one workgroup would walk all of such a request's keys, 128 or 256 per iteration of some
                # 1.7 us, and the longest of them sets the launch's time
                part_o = part_ml = None
                n_splits = n_waves = lean = 0
                if singles and b > 1 and nq // nkv <= 16 and max_kv_len > self.singles_apart_beyond:
                    n_splits, n_waves, lean = self._decode_shape(b, nkv, hd, max_kv_len, True)
                parts_rows = max(n_splits * b if n_splits > 1 else 0, key_splits * t if key_splits > 1 else 0)
                if parts_rows:
                    part_o = torch.empty((parts_rows, nq, hd), dtype=_F32, device=qkv.device)
                    part_ml = torch.empty((parts_rows, nq, 2), dtype=_F32, device=qkv.device)
                self._run("egpt_paged_attention_tiled", qkv.data_ptr(), out.data_ptr(), k_cache.data_ptr(),
                          v_cache.data_ptr(), block_table.data_ptr(), width, q_start.data_ptr(), q_len.data_ptr(),
                          kv_len.data_ptr(), b, t, nq, nkv, hd, page_size, float(scale), int(window), shape, key_splits,
                          self._ptr(part_o), self._ptr(part_ml), n_splits, n_waves, lean, self._stream())
                return None
            n_splits = max(1, min(1024 // (b * nkv), -(-max_kv_len // 64), 64))
            part_o = part_ml = None
            if n_splits > 1:
                part_o = torch.empty((n_splits, t, nq, hd), dtype=_F32, device=qkv.device)
                part_ml = torch.empty((n_splits, t, nq, 2), dtype=_F32, device=qkv.device)
            self._run("egpt_paged_attention_mfma", qkv.data_ptr(), out.data_ptr(), self._ptr(part_o),
                      self._ptr(part_ml), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), width,
                      q_start.data_ptr(), q_len.data_ptr(), kv_len.data_ptr(), b, t, nq, nkv, hd, page_size,
                      float(scale), int(window), n_splits, 16, 1 if combine else 0,
                      self._stream())
            return (part_o, part_ml) if (n_splits > 1 and not combine) else None
        if hd % 16 == 0 and page_size % 16 == 0:
            # every other head size in steps of 16, and all of float32: the matrix-core kernels that take any of them
            if max_q_len == 1 and t == b:
                n_segments = -(-max_kv_len // self.attention_segment)
                part_o = torch.empty((n_segments, t, nq, hd), dtype=_F32, device=qkv.device)
                part_ml = torch.empty((n_segments, t, nq, 2), dtype=_F32, device=qkv.device)
                self._run("egpt_attention_any_decode", qkv.data_ptr(), out.data_ptr(), part_o.data_ptr(),
                          part_ml.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), width,
                          q_start.data_ptr(), kv_len.data_ptr(), b, nq, nkv, hd, page_size, float(scale), int(window),
                          n_segments, dt, self._stream())
                return None
            self._run("egpt_attention_any_tiled", qkv.data_ptr(), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                      block_table.data_ptr(), width, q_start.data_ptr(), q_len.data_ptr(), kv_len.data_ptr(), b, t,
                      nq, nkv, hd, page_size, float(scale), int(window), dt, self._stream())
            return None
        # head or page sizes that are no multiples of 16: the general kernel
        self._run("egpt_paged_attention", qkv.data_ptr(), out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                  block_table.data_ptr(), width, q_start.data_ptr(), q_len.data_ptr(), kv_len.data_ptr(), b, t,
                  nq, nkv, hd, page_size, float(scale), int(window), dt, self._stream())

    # A mixed step's requests of one token go to the decode kernel when the step's longest context is beyond this: the
    # second launch (and a third that combines key ranges) costs some 8 us, a workgroup of the tiled kernel that walks
    # 4,000 keys alone some 30.  Measured, us for one layer's attention of the 0.5B sizes, tiled kernel alone against
    # the two: one portion of 512 tokens beside 8 decoded tokens behind 600 keys each 11.0 against 18.3, behind 1,300
    # 16.2 against 18.6, behind 4,000 33.2 against 20.5, behind 16,000 122 against 32; four portions beside 24 decoded
    # tokens behind 1,300 keys 36.7 against 38.1, behind 4,000 61.6 against 43.5, behind 16,000 152 against 66
    singles_apart_beyond = 2048
    prefix_keys = 4096           # a step's longest context from which its portions are taken to lie behind a prefix
    attention_segment = 64       # keys per segment of the decode kernel for any head size (kSegment in attention_any.hip)

    @staticmethod
    def _decode_shape(b, nkv, hd, max_kv_len, combine):
        """(key splits, wavefronts per workgroup, lean variant or not) of the decode attention kernel.  The kernel is a chain of round
        trips to memory, and a wavefront takes one per round of 4 (head size 64) or 2 key blocks of 32 keys, so
        there should be enough wavefronts for one round each, and with few requests for one key block each.
        The key range is split over workgroups when the requests alone do not fill the GPU; parts that the
        output projection combines are read by every column of workgroups there, so they stay few."""
        key_blocks = -(-max_kv_len // 32)
        pairs = b * nkv
        self_most = 64                    # parts that the output projection (or the combining kernel) takes

        def splits_for(n_waves, blocks=None):
            per_round = n_waves * (1 if pairs * key_blocks <= 2048 else (blocks or (4 if hd == 64 else 2)))
            wanted = -(-key_blocks // per_round)
            # the output projection combines up to 8 parts in registers; more only behind contexts so long that 8
            # parts would leave every wavefront four rounds or more, and then up to some 512 workgroups in all: a CU
            # has only so many bytes on their way, so a long context wants many CUs more than it minds many parts
            # (measured at the 0.5B sizes with 32,000-token contexts: batch 1 takes 1.119 ms a step with 16 parts,
            # 0.991 with 32, 0.976 with 64; batch 8 takes 1.919 with 8, 1.588 with 16, 1.513 with 32, 1.673 with 64;
            # with 8,192-token contexts batch 1 takes 0.888 with 16 and 0.854 with 32, batch 8 is fastest with 8)
            most = max(8, min(self_most, 512 // pairs)) if wanted >= 32 else 8
            # as many workgroups as this at most (head size 64, 8,192-token contexts, batch 64: 2.821 ms a step with
            # 2,048 workgroups, 2.698 with 1,024).  Head size 128: at most two workgroups per CU, beyond which the
            # kernel's variant with fewer loads in flight runs (measured at the 1.5B sizes, 2,048-token contexts:
            # 2.42 ms a step with 512 workgroups at batch 32 against 2.63 with 576, 3.20 with 512 at batch 64 against
            # 3.48 with 1,152)
            room = 1024 if hd == 64 else 512
            return max(1, min(wanted, most, max(1, room // pairs)))

        n_splits = n_waves = 0
        if hd == 64 and pairs * key_blocks <= 8192:
            # a round of the variant that runs here is two key blocks; with few pairs, enough splits for one round
            # per wavefront (measured at 2,048-token contexts: 1.17 -> 1.13 ms a step at batch 16, 1.36 -> 1.33 at 24)
            n_splits, n_waves = splits_for(8, blocks=2), 8
            if pairs * n_splits > 256:
                n_splits = splits_for(8)
            # wide workgroups as long as each has a CU of its own: a few more than CUs, and those that share one set
            # the kernel's time (measured at 2,048-token contexts: 1.84 ms a step at batch 44 and 48 with 264 and 288
            # workgroups of eight wavefronts, 1.66 with 440 and 480 of four; 1.57 either way at batch 40)
            if pairs * n_splits > 256:
                n_waves = 0
        if not n_waves and 128 < 2 * pairs <= 256:
            # two key ranges of eight wavefronts while that gives every workgroup a CU of its own (measured at the 0.5B
            # sizes against the best shape of four wavefronts: batch 64 behind 2,048 tokens 1.727 ms a step against 1.765
            # (4 ranges; 1.811 with the 5 that the rule below gives), batch 56 1.680 against 1.725, batch 48 1.618 against
            # 1.626, batch 64 behind 3,584 tokens 1.923 against 1.962, behind 8,192 tokens 2.599 against 2.624; at the
            # 1.5B sizes, head size 128: batch 64 3.12 against 3.21, batch 48 3.02 against 3.04; folding the two parts'
            # combination into the output projection at these rows gave nothing: 1.752 against 1.728 at batch 64; behind
            # 32,000 tokens batch 64 takes 5.77 against 5.78 to 5.87 with 4 to 12 ranges of four wavefronts)
            n_splits, n_waves = 2, 8
        elif not n_waves and 128 < pairs <= 512 and key_blocks <= 288:
            # more pairs than half the CUs: no key ranges at all (and no combination of parts), eight wavefronts while
            # every workgroup has a CU of its own, four beyond (measured, ms a step against the rule below: batch 128
            # at the 0.5B sizes 2.44 against 2.52 behind 2,048 tokens and 4.04 against 4.21 behind 8,192, batch 256
            # 3.11 against 3.27; at the 1.5B sizes batch 128 4.03 against 4.20; at the 7B sizes, four kv heads, batch
            # 64 6.56 against 6.71 and batch 128 9.87 against 10.06)
            n_splits, n_waves = 1, 8 if pairs <= 256 else 4
        elif not n_waves and 32 < pairs <= 64 and key_blocks >= 64:
            # and with 33 to 64 pairs as many key ranges of eight wavefronts as give every workgroup a CU of its own
            # (measured, ms a step against the rule below, which takes 8 ranges of four wavefronts: at the 1.5B sizes
            # behind 2,048 tokens batch 32 2.31 against 2.42 and batch 24 2.21 against 2.27; at the 7B sizes behind 4,096
            # tokens batch 16 5.04 against 5.23; at the 14B sizes, eight kv heads, batch 8 9.00 against 9.50; at the 0.5B
            # sizes behind 8,192 tokens batch 32 1.82 against 1.87 and batch 24 1.63 against 1.67)
            n_splits, n_waves = 256 // pairs, 8
        if not n_waves:
            n_splits, n_waves = splits_for(4), 4
            # head size 128: eight wavefronts as well while every workgroup has a CU of its own (its 71 KB of LDS are
            # asked for at the first launch): a wavefront then has one round of keys, and the fused variant's nine
            # heads of 64 pairs are made in one pass (measured with 2,048- and 4,096-token contexts: 1.660 -> 1.600 ms
            # a step at batch 8 and 1.505 -> 1.443 at batch 1 at the 1.5B sizes, 3 % at the 7B sizes)
            # (with a key block per wavefront at least: 1.270 -> 1.243 ms a step of eight layers of the 7B sizes at batch 1)
            if hd == 128 and pairs * min(n_splits, -(-key_blocks // 8)) <= 256:
                n_splits, n_waves = min(n_splits, -(-key_blocks // 8)), 8
        # The kernel's variant with half the loads in flight per round and fewer registers.  Head size 64: always,
        # unless a wavefront walks so many key blocks that the rounds' depth counts (measured: 0.954 -> 0.933 ms a step
        # at batch 8 and 2,048-token contexts, 0.872 -> 0.853 at batch 1, 1.135 -> 1.102 at batch 8 and 8,192 tokens,
        # but 1.99 -> 2.03 at batch 8 and 32,000 tokens, 31 blocks per wavefront).  Head size 128: from one and a
        # half workgroups per CU on (fewer: 1 to 2% slower than the full variant).
        # (with more pairs than half the CUs also behind 8,192 tokens, 34 blocks per wavefront: 4.04 against 4.13 at batch 128)
        per_wave = -(-key_blocks // (n_splits * n_waves))
        # (and with 65 to 128 pairs behind 32,000 tokens: 5.77 against 5.85 at batch 64)
        lean = (per_wave <= 17 or pairs > 64) if hd == 64 else pairs * n_splits > 384
        return n_splits, n_waves, 1 if lean else 0

    def attention_decode_fused(self, prod, row_ss, hidden, eps, bias, positions, inv_freq, rotary_dim, slots, out,
                               k_cache, v_cache, block_table, q_start, kv_len, nq, nkv, hd, page_size, scale, window,
                               max_kv_len, combine=True, cos_sin=None):
        """Attention for a batch of single decoded tokens (token t belongs to request t) straight from the QKV
        product's float32 partial sums prod [S, T, W]: what qkv_rope_store and paged_attention do together, in
        one kernel.  Returns False if the case is not covered (nothing was done), else what paged_attention
        returns."""
        if prod.dim() != 3 or prod.dtype != _F32 or out.dtype != _BF16 or hd not in (64, 128) or page_size % 16:
            return False
        if rotary_dim != hd or nq // nkv > 16 or slots is None or inv_freq is None:
            return False
        in_splits, t, width = prod.shape
        b, table_width = block_table.shape
        if t != b or width != (nq + 2 * nkv) * hd:
            return False
        self._need(prod, "prod", _F32)
        self._need(out, "out", _BF16, (t, nq * hd))
        self._caches(k_cache, v_cache, _BF16, nkv, page_size, hd)
        self._need(block_table, "block_table", _I32)
        for name, v in (("q_start", q_start), ("kv_len", kv_len), ("positions", positions), ("slots", slots)):
            self._need(v, name, _I32, (b,))
        self._need(inv_freq, "inv_freq", _F32, (hd // 2,))
        if cos_sin is None:
            cos_sin = self.rope_table(positions, inv_freq)
        self._need(cos_sin, "cos_sin", _F32, (t, hd // 2, 2))
        if bias is not None:
            self._need(bias, "bias", _BF16, (width,))
        ss_splits = 0
        if row_ss is not None:
            ss_splits = int(row_ss.shape[0])
            self._need(row_ss, "row_ss", _F32, (ss_splits, t))
        if max_kv_len > table_width * page_size:
            raise ValueError(f"block table of width {table_width} cannot hold {max_kv_len} tokens at page size {page_size}")
        n_splits, n_waves, lean = self._decode_shape(b, nkv, hd, max_kv_len, combine)
        part_o = part_ml = None
        if n_splits > 1:
            part_o = torch.empty((n_splits, t, nq, hd), dtype=_F32, device=prod.device)
            part_ml = torch.empty((n_splits, t, nq, 2), dtype=_F32, device=prod.device)
        self._run("egpt_attention_decode_fused", prod.data_ptr(), int(in_splits), self._ptr(row_ss), ss_splits, int(hidden),
                  float(eps), self._ptr(bias), cos_sin.data_ptr(), slots.data_ptr(), out.data_ptr(),
                  self._ptr(part_o), self._ptr(part_ml), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(),
                  table_width, q_start.data_ptr(), kv_len.data_ptr(), b, nq, nkv, hd, page_size, float(scale),
                  int(window), n_splits, n_waves, 1 if combine else 0, lean, self._stream())
        return (part_o, part_ml) if (n_splits > 1 and not combine) else None

    def swiglu(self, gate_up, out, row_ss=None, hidden=0, eps=0.0):
        """out = up * silu(gate) for gate_up act [T, 2I] or float32 partial sums [S, T, 2I].  row_ss float32
        [S2, T]: the partial sums still lack each row's factor 1/sqrt(sum_s row_ss[s] / hidden + eps)."""
        t, inter = out.shape
        dt = self._act(out, "out")
        splits = self._product(gate_up, "gate_up", out.dtype, t, 2 * inter)
        self._need(out, "out")
        ss_splits = 0
        if row_ss is not None:
            if splits < 1:
                raise ValueError("a pending row factor needs float32 partial sums")
            ss_splits = int(row_ss.shape[0])
            self._need(row_ss, "row_ss", _F32, (ss_splits, t))
        self._run("egpt_swiglu", gate_up.data_ptr(), splits, self._ptr(row_ss), ss_splits, int(hidden), float(eps),
                  out.data_ptr(), t, inter, dt, self._stream())

    def argmax(self, logits, out):
        r, v = logits.shape
        self._need(logits, "logits", _F32)
        self._need(out, "out", _I32, (r,))
        scratch = torch.empty(r * 64, dtype=_F32, device=logits.device) if v >= 8192 else None
        self._run("egpt_argmax", logits.data_ptr(), out.data_ptr(), self._ptr(scratch), r, v, self._stream())

    def sample(self, logits, temperature, top_k, top_p, uniform, out):
        r, v = logits.shape
        self._need(logits, "logits", _F32)
        self._need(temperature, "temperature", _F32, (r,))
        self._need(top_k, "top_k", _I32, (r,))
        self._need(top_p, "top_p", _F32, (r,))
        self._need(uniform, "uniform", _F32, (r,))
        self._need(out, "out", _I32, (r,))
        if v >= 8192:
            # a wide vocabulary: the row-wide passes by many workgroups, the selection on the tokens that are left
            space = torch.empty(int(self.lib.egpt_sample_workspace(r, v)), dtype=torch.uint8, device=logits.device)
            self._run("egpt_sample_wide", logits.data_ptr(), temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(),
                      uniform.data_ptr(), out.data_ptr(), space.data_ptr(), r, v, self._stream())
            return
        weights = torch.empty((r, v), dtype=_F32, device=logits.device)
        self._run("egpt_sample", logits.data_ptr(), temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(),
                  uniform.data_ptr(), out.data_ptr(), weights.data_ptr(), r, v, self._stream())
