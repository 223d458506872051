"""Each HIP kernel alone against a plain float64 reference of the same operation, at sizes other than
the tiny models' (widths and vocabularies that are no power of two, head sizes in steps of 16, odd
numbers of heads and groups)."""
import math

import pytest
import torch

import plain_qwen2 as plain

pytestmark = pytest.mark.gpu
F64 = torch.float64
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype, scale=1.0):
    return (3e-6 if dtype == torch.float32 else 1.6e-2) * scale


@pytest.fixture(scope="module")
def k():
    from easy_gpt.cpp_amd import kernels

    kernels.use_backend(None)
    b = kernels.backend()
    assert b.name == "hip-gfx950"
    return b


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(k, dtype):
    table = rnd(301, 72, dtype=dtype)
    ids = torch.tensor([0, 300, 17, 17, 5], dtype=torch.int32, device=DEV)
    out = torch.empty(5, 72, dtype=torch.float32, device=DEV)
    k.embed(ids, table, out)
    assert torch.equal(out, table[ids.long()].float())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,eps,n_rows", [(72, 1e-6, 7), (896, 1e-5, 7), (3000, 1e-2, 7), (896, 1e-6, 70), (3000, 1e-5, 33),
                                               (100, 1e-6, 40), (896, 1e-6, 601), (1536, 1e-5, 512), (2000, 1e-6, 513),
                                               (2056, 1e-6, 600), (5000, 1e-6, 7), (4104, 1e-5, 33), (8192, 1e-6, 7), (5120, 1e-6, 8),
                                               (8200, 1e-6, 7), (12288, 1e-5, 7)])
def test_add_rmsnorm(k, dtype, hidden, eps, n_rows):
    h = rnd(n_rows, hidden, seed=1, scale=2.0)
    delta = rnd(n_rows, hidden, dtype=dtype, seed=2)
    w = (1 + rnd(hidden, seed=3, scale=0.1)).to(dtype)
    h0 = h.clone()
    out = torch.empty(n_rows, hidden, dtype=dtype, device=DEV)
    k.add_rmsnorm(h, delta, w, eps, out)
    summed = h0 + delta.float()                                   # the residual sum is made in float32
    assert torch.equal(h, summed)
    ref = plain.rms_norm(summed.double().cpu(), w.double().cpu(), eps)
    assert float((out.double().cpu() - ref).abs().max()) <= tol(dtype, float(ref.abs().max()))
    # without delta h is untouched
    h1 = h.clone()
    k.add_rmsnorm(h, None, w, eps, out)
    assert torch.equal(h, h1)
    # rows variant: gathers, adds, does not write back
    assert n_rows >= 7                                            # the rows picked below exist
    picked = [6, 0, 3] + (list(range(n_rows - 1, -1, -1)) if n_rows >= 33 else [])
    rows = torch.tensor(picked, dtype=torch.int32, device=DEV)
    out3 = torch.empty(len(picked), hidden, dtype=dtype, device=DEV)
    k.rows_add_rmsnorm(h, delta, rows, w, eps, out3)
    assert torch.equal(h, h1)
    ref3 = plain.rms_norm((h1 + delta.float())[rows.long()].double().cpu(), w.double().cpu(), eps)
    assert float((out3.double().cpu() - ref3).abs().max()) <= tol(dtype, float(ref3.abs().max()))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,kk", [(1, 75, 100), (37, 130, 96), (70, 1000, 200), (5, 64, 4864), (130, 33, 17)])
def test_linear(k, dtype, m, n, kk):
    x, w, b = rnd(m, kk, dtype=dtype, seed=1), rnd(n, kk, dtype=dtype, seed=2, scale=0.1), rnd(n, dtype=dtype, seed=3)
    ref = plain.linear(x.double().cpu(), w.double().cpu(), b.double().cpu())
    for out_dtype in {dtype, torch.float32}:
        out = torch.empty(m, n, dtype=out_dtype, device=DEV)
        k.linear(x, w, b, out)
        t = 3e-6 if out_dtype == torch.float32 else 1.6e-2
        assert float((out.double().cpu() - ref).abs().max()) <= t * float(ref.abs().max())
    out = torch.empty(m, n, dtype=torch.float32, device=DEV)
    k.linear(x, w, None, out)
    assert float((out.double().cpu() - (ref - b.double().cpu())).abs().max()) <= 3e-6 * float(ref.abs().max())


@pytest.mark.parametrize("m,n,kk", [(1, 75, 104), (8, 1152, 896), (16, 896, 4864), (17, 130, 96), (33, 1000, 200),
                                    (64, 9728, 896), (5, 777, 120), (48, 64, 4864), (8, 151936, 896), (40, 4100, 2056),
                                    (20, 5000, 1000), (17, 4096, 8)])
def test_skinny_product_and_partial_sums(k, m, n, kk):
    # the bfloat16 product for few rows: direct (float32 and bfloat16 output, with bias) and split over k
    dtype = torch.bfloat16
    x, w, b = rnd(m, kk, dtype=dtype, seed=1), rnd(n, kk, dtype=dtype, seed=2, scale=0.1), rnd(n, dtype=dtype, seed=3)
    ref = plain.linear(x.double().cpu(), w.double().cpu())
    scale = float(ref.abs().max())
    prod = k.product(x, w)
    if k._library_rows(m, n, kk):        # more than 16 rows of a large matrix without a split k range: the library
        assert prod.dtype == dtype and prod.shape == (m, n)
        assert float((prod.double().cpu() - ref).abs().max()) <= 1e-2 * scale
        prod = k.product(x, w, unrounded=True)
    assert prod.dtype == torch.float32 and prod.dim() == 3 and prod.shape[1:] == (m, n)
    assert float((prod.double().sum(0).cpu() - ref).abs().max()) <= 3e-6 * scale
    for s in sorted({1, 2, min(3, -(-kk // 128)), -(-kk // 128)}):
        steps = -(-kk // 128)
        if s > steps or (s - 1) * -(-steps // s) >= steps:
            continue
        for waves in (4, 8, 16):                 # wavefronts per workgroup
            out = torch.full((s, m, n), 7.0, dtype=torch.float32, device=DEV)
            k._run("egpt_gemm_skinny", x.data_ptr(), w.data_ptr(), None, out.data_ptr(), None, None, m, n, kk, s, waves,
                   k._stream())
            assert float((out.double().sum(0).cpu() - ref).abs().max()) <= 3e-6 * scale, (s, waves)
    out32 = torch.empty(m, n, dtype=torch.float32, device=DEV)
    k.linear(x, w, b, out32)
    assert float((out32.double().cpu() - ref - b.double().cpu()).abs().max()) <= 3e-6 * scale
    out16 = torch.empty(m, n, dtype=dtype, device=DEV)
    k.linear(x, w, b, out16)
    with_bias = ref + b.double().cpu()
    assert float((out16.double().cpu() - with_bias).abs().max()) <= 1e-2 * float(with_bias.abs().max())   # one bfloat16 rounding


@pytest.mark.parametrize("m,n,kk", [(1, 75, 100), (16, 1152, 896), (37, 130, 96), (64, 200, 4864), (130, 1000, 200),
                                    (300, 64, 68), (5, 777, 120)])
def test_float32_product_on_the_matrix_cores(k, m, n, kk):
    x, w, b = rnd(m, kk, seed=1), rnd(n, kk, seed=2, scale=0.1), rnd(n, seed=3)
    ref = plain.linear(x.double().cpu(), w.double().cpu())
    scale = float(ref.abs().max())

    def tol(splits):
        # a float32 sum of kk / splits terms one after the other: roundings of 6e-8 each that add up like a random walk
        # (the FMA kernel that this one replaced is at the same 3e-6 for 4,864 terms)
        return max(1e-6, 6e-8 * math.sqrt(kk / splits)) * scale

    prod = k.product(x, w)
    auto = k._f32_splits(n, kk)
    assert prod.dtype == torch.float32 and prod.shape == (auto, m, n)
    assert float((prod.double().sum(0).cpu() - ref).abs().max()) <= tol(auto)
    steps = -(-kk // 64)
    for s in sorted({1, 2, 3, steps}):
        if s > steps or (s - 1) * -(-steps // s) >= steps:
            continue
        out = torch.full((s, m, n), 7.0, device=DEV)
        k._run("egpt_gemm_f32", x.data_ptr(), w.data_ptr(), None, out.data_ptr(), m, n, kk, s, k._stream())
        assert float((out.double().sum(0).cpu() - ref).abs().max()) <= tol(s), s
    out = torch.empty(m, n, device=DEV)
    k.linear(x, w, b, out)
    assert float((out.double().cpu() - ref - b.double().cpu()).abs().max()) <= tol(1)
    # a row's values are the same bits alone, among the others, and at another place among them
    for r in sorted({0, m // 2, m - 1}):
        alone = k.product(x[r : r + 1].contiguous(), w)
        assert torch.equal(alone[:, 0], prod[:, r]), r
    if m > 1:
        turned = k.product(x.flip(0).contiguous(), w)
        assert torch.equal(turned.flip(1), prod)
    with pytest.raises(RuntimeError):
        k._run("egpt_gemm_f32", x.data_ptr(), w.data_ptr(), b.data_ptr(), out.data_ptr(), m, n, kk, 2, k._stream())   # bias with splits


def test_which_products_go_to_the_library():
    from easy_gpt.cpp_amd.kernels.hip import HipKernels

    lib = HipKernels._library_rows
    assert not lib(16, 151936, 896) and lib(65, 64, 64)                   # up to 16 rows never, beyond 64 always
    assert lib(64, 9728, 896) and lib(33, 151936, 896) and lib(48, 152064, 3584)
    assert not lib(17, 151936, 896) and not lib(32, 152064, 3584)         # an output matrix at up to 32 rows: the own kernel
    assert not lib(64, 896, 4864) and not lib(17, 3584, 18944)            # split-k shapes stay with the own kernels
    assert not lib(32, 9728, 896) and lib(32, 17920, 1536)                # small matrices with up to 32 rows, too
    assert not lib(64, 1152, 896) and lib(64, 4608, 3584) and not lib(64, 2048, 1536) and not lib(64, 2560, 2048)


def test_consumers_add_partial_sums_up(k):
    # residual add + norm, SwiGLU and the QKV epilogue take float32 partial sums [splits, rows, cols]
    dtype = torch.bfloat16
    t, hid = 5, 200
    parts = rnd(3, t, hid, seed=1)
    h = rnd(t, hid, seed=2)
    h0 = h.clone()
    w = (1 + rnd(hid, seed=3, scale=0.1)).to(dtype)
    out = torch.empty(t, hid, dtype=dtype, device=DEV)
    k.add_rmsnorm(h, parts, w, 1e-6, out)
    summed = h0 + (parts[0] + parts[1] + parts[2])
    assert torch.equal(h, summed)
    ref = plain.rms_norm(summed.double().cpu(), w.double().cpu(), 1e-6)
    assert float((out.double().cpu() - ref).abs().max()) <= 1.6e-2 * float(ref.abs().max())
    rows = torch.tensor([4, 0], dtype=torch.int32, device=DEV)
    out2 = torch.empty(2, hid, dtype=dtype, device=DEV)
    k.rows_add_rmsnorm(h0.clone(), parts, rows, w, 1e-6, out2)
    assert float((out2.double().cpu() - ref[[4, 0]]).abs().max()) <= 1.6e-2 * float(ref.abs().max())
    gu = rnd(2, t, 2 * 96, seed=4, scale=2.0)
    act = torch.empty(t, 96, dtype=dtype, device=DEV)
    k.swiglu(gu, act)
    g, u = (gu[0] + gu[1])[:, :96].double().cpu(), (gu[0] + gu[1])[:, 96:].double().cpu()
    refa = u * g / (1 + torch.exp(-g))
    assert float((act.double().cpu() - refa).abs().max()) <= 1.6e-2 * float(refa.abs().max())
    nq, nkv, hd, ps = 3, 1, 32, 4
    width = (nq + 2 * nkv) * hd
    qp = rnd(2, t, width, seed=5)
    bias = rnd(width, dtype=dtype, seed=6)
    positions = torch.arange(10, 10 + t, dtype=torch.int32, device=DEV)
    inv = torch.pow(torch.tensor(1e4), -2.0 * torch.arange(hd // 2, dtype=torch.float32) / hd).to(DEV)
    slots = torch.tensor([3, 9, 0, 14, 7], dtype=torch.int32, device=DEV)
    kc = torch.zeros(4, nkv, ps, hd, dtype=dtype, device=DEV)
    vc = torch.zeros(4, nkv, hd, ps, dtype=dtype, device=DEV)
    got = torch.empty(t, width, dtype=dtype, device=DEV)
    k.qkv_rope_store(qp, bias, positions, inv, hd, slots, kc, vc, nq, nkv, hd, ps, out=got)
    x = ((qp[0] + qp[1]).double() + bias.double()).cpu().view(t, nq + 2 * nkv, hd)
    refq = x.clone()
    refq[:, : nq + nkv] = plain.rope(x[:, : nq + nkv], positions.cpu(), 1e4)
    assert float((got.double().cpu().view(t, -1, hd) - refq).abs().max()) <= 1.6e-2 * float(refq.abs().max())
    assert torch.equal(kc[0, :, 3, :], got.view(t, -1, hd)[0, nq : nq + nkv])
    assert torch.equal(vc[3, :, :, 2], got.view(t, -1, hd)[3, nq + nkv :])


def to_fixed(t):
    """float32 -> the residual stream's 64-bit fixed point (units of 2^-32), as the kernels convert"""
    return torch.round(t.double() * 2.0 ** 32).to(torch.int64)


def from_fixed(t):
    return t.double() / 2.0 ** 32


@pytest.mark.parametrize("t,hid,inter,nq,hd", [(8, 896, 4864, 14, 64), (1, 200, 328, 5, 40), (16, 1536, 1000, 12, 128),
                                                (5, 120, 200, 3, 40)])
def test_residual_stream_in_fixed_point(k, t, hid, inter, nq, hd):
    # The stream of a step of few tokens is int64 in units of 2^-32.  Embedding and norms read and write it, the
    # products whose k range is split over workgroups add their parts into it with integer atomics: the sum is
    # the exact sum of the float32 parts (a float32 times 2^32 is an integer here), the same bits in any order.
    dtype = torch.bfloat16
    assert k.residual_dtype(t, dtype) == torch.int64 and k.residual_dtype(t, torch.float32) == torch.float32
    assert k.residual_dtype(17, dtype) == torch.float32
    # embedding
    table = rnd(50, hid, dtype=dtype, seed=1)
    ids = torch.arange(t, dtype=torch.int32, device=DEV) * 3
    h = torch.empty(t, hid, dtype=torch.int64, device=DEV)
    k.embed(ids, table, h)
    assert torch.equal(h, to_fixed(table[ids.long()].float()))
    # norm of the stream, with and without something to add (an ordinary tensor, or partial sums), all rows or some
    nw = (1 + rnd(hid, seed=2, scale=0.1)).to(dtype)
    parts = rnd(3, t, hid, seed=3)
    for delta in (None, parts[0].to(dtype), parts):
        hh = h.clone()
        out = torch.empty(t, hid, dtype=dtype, device=DEV)
        k.add_rmsnorm(hh, delta, nw, 1e-6, out)
        added = 0 if delta is None else (delta.double() if delta.dim() == 2 else delta.double().sum(0))
        want = from_fixed(h) + added
        assert float((from_fixed(hh) - want).abs().max()) <= 1e-6 * float(want.abs().max())
        ref = plain.rms_norm(want.cpu(), nw.double().cpu(), 1e-6)
        assert float((out.double().cpu() - ref).abs().max()) <= 1.6e-2 * float(ref.abs().max())
        rows = torch.tensor([t - 1, 0], dtype=torch.int32, device=DEV)
        out2 = torch.empty(2, hid, dtype=dtype, device=DEV)
        h_before = h.clone()
        k.rows_add_rmsnorm(h_before, delta, rows, nw, 1e-6, out2)
        assert torch.equal(h_before, h)                                       # rows only: the stream is not written
        assert float((out2.double().cpu() - ref[[t - 1, 0]]).abs().max()) <= 1.6e-2 * float(ref.abs().max())
    # the product with the norm folded in reads the stream as it is: the same as from the float32 stream
    w = rnd(200, hid, dtype=dtype, seed=4, scale=0.05)
    hf = from_fixed(h).float()
    a, b = k.product_normed(h, None, nw, w), k.product_normed(hf, None, nw, w)
    assert a[2] is h and torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert k.product_normed(h, parts, nw, w) is None                          # something to add: the norm's own kernel
    # products added into the stream: plain, with SwiGLU folded in, with the attention parts' combination folded in
    x = rnd(t, inter, dtype=dtype, seed=5)
    w_down = rnd(hid, inter, dtype=dtype, seed=6, scale=0.05)
    for run in range(2):                                                       # the same bits every time
        hh = h.clone()
        assert k.product(x, w_down, residual=hh) is hh
        want = from_fixed(h) + k.product(x, w_down).double().sum(0)
        assert torch.equal(hh, to_fixed(from_fixed(h)) + sum(to_fixed(p) for p in k.product(x, w_down)))
        assert float((from_fixed(hh) - want).abs().max()) <= 1e-9 * float(want.abs().max())
    gu = rnd(2, t, 2 * inter, seed=7)
    if inter % 8 == 0:
        parts_out = k.product_swiglu(gu, None, hid, 0.0, w_down)
        hh = h.clone()
        if parts_out is not None:
            assert k.product_swiglu(gu, None, hid, 0.0, w_down, residual=hh) is hh
            assert torch.equal(hh, h + sum(to_fixed(p) for p in parts_out))
    po = rnd(4, t, nq, hd, seed=8)
    pml = torch.stack([rnd(4, t, nq, seed=9), 1 + rnd(4, t, nq, seed=10).abs()], dim=-1).contiguous()
    w_o = rnd(hid, nq * hd, dtype=dtype, seed=11, scale=0.05)
    parts_out = k.product_attention(po, pml, w_o, max_splits=4)
    if parts_out is not None:
        hh = h.clone()
        assert k.product_attention(po, pml, w_o, max_splits=4, residual=hh) is hh
        assert torch.equal(hh, h + sum(to_fixed(p) for p in parts_out))
    # a stream of another shape, or a float32 one, is not added into: partial sums come back as before
    assert k.product(x, w_down, residual=hf).dim() == 3


def test_residual_stream_in_fixed_point_over_its_range(k):
    # magnitudes from 1e-6 to 1e6 side by side (models have channels of 1e3 to 1e5 beside ones of 1e-3): every value
    # keeps its own precision through the embedding, the norm's addition and the products' atomics; a value that the
    # stream cannot hold enters as the largest magnitude of its sign
    dtype, t, hid, inter = torch.bfloat16, 6, 256, 512
    g = torch.Generator().manual_seed(31)
    wide = lambda *shape: (10.0 ** (torch.rand(*shape, generator=g) * 12 - 6)) * (torch.randint(0, 2, shape, generator=g) * 2 - 1)
    table = wide(40, hid).to(dtype).to(DEV)
    ids = torch.arange(t, dtype=torch.int32, device=DEV) * 5
    h = torch.empty(t, hid, dtype=torch.int64, device=DEV)
    k.embed(ids, table, h)
    assert torch.equal(h, to_fixed(table[ids.long()].float()))                # bfloat16 values of these sizes are exact
    # the norm adds float32 values of any of these sizes to any other
    nw = (1 + rnd(hid, seed=2, scale=0.1)).to(dtype)
    delta = wide(2, t, hid).float().to(DEV)
    hh = h.clone()
    out = torch.empty(t, hid, dtype=dtype, device=DEV)
    k.add_rmsnorm(hh, delta, nw, 1e-6, out)
    want = from_fixed(h) + delta.double().sum(0)
    err = (from_fixed(hh) - want).abs()
    size = from_fixed(h).abs() + delta.double().abs().sum(0)                  # (the additions are float32 ones)
    assert bool((err <= 2e-7 * size + 2.0 ** -32).all())                      # per element, not against the row's largest
    ref = plain.rms_norm(want.cpu(), nw.double().cpu(), 1e-6)
    assert float((out.double().cpu() - ref).abs().max()) <= 1.6e-2 * float(ref.abs().max())
    # partial products of every size are added as the integers they are
    x = (torch.randn(t, inter, generator=g) * torch.tensor([1e-5, 1e-3, 1e-1, 1e1, 1e3, 1e4])[:, None]).to(dtype).to(DEV)
    w_down = rnd(hid, inter, dtype=dtype, seed=6, scale=0.05)
    parts = k.product(x, w_down)
    assert float(parts.abs().max()) > 1e2 and float(parts.abs().min()) < 1e-3
    hh = h.clone()
    assert k.product(x, w_down, residual=hh) is hh
    assert torch.equal(hh, h + sum(to_fixed(p) for p in parts))
    # what does not fit: 2^31 and beyond, infinities and NaN become the largest magnitude
    odd = torch.tensor([[3e9, -3e9, float("inf"), float("-inf"), float("nan"), 2.0 ** 31, 2.0 ** 31 - 128, 1.0]],
                       dtype=torch.float32, device=DEV).repeat(1, hid // 8)
    hz = torch.zeros(1, hid, dtype=torch.int64, device=DEV)
    k.add_rmsnorm(hz, odd.view(1, 1, hid), nw, 1e-6, torch.empty(1, hid, dtype=dtype, device=DEV))
    top, low = 2 ** 63 - 1, -(2 ** 63)
    assert hz[0, :8].tolist() == [top, low, top, low, low, top, (2 ** 31 - 128) * 2 ** 32, 2 ** 32]


@pytest.mark.parametrize("t,hid,n,d_splits", [(1, 896, 1152, 0), (8, 896, 9728, 4), (16, 200, 130, 3), (5, 1536, 2048, 13),
                                              (8, 3584, 4608, 19), (3, 1536, 17920, 12), (16, 256, 26000, 2)])
def test_product_with_norm_folded_in(k, t, hid, n, d_splits):
    # ((h + delta) * norm_weight) w^T with the rows' 1/rms applied afterwards equals rmsnorm(h + delta) w^T
    dtype = torch.bfloat16
    h = rnd(t, hid, seed=1, scale=2.0)
    delta = rnd(d_splits, t, hid, seed=2) if d_splits else None
    nw = (1 + rnd(hid, seed=3, scale=0.1)).to(dtype)
    w = rnd(n, hid, dtype=dtype, seed=4, scale=0.05)
    h0 = h.clone()
    summed = h0.clone()
    for s in range(d_splits):
        summed += delta[s]
    sd = summed.double().cpu()
    eps = 1e-6
    ref = plain.linear(plain.rms_norm(sd, nw.double().cpu(), eps), w.double().cpu())
    # every workgroup width; the k range in as many pieces as the wrapper likes (short ranges, staged at once),
    # in one piece and in two (long ranges, staged step by step)
    for waves, splits in ((None, None), (4, None), (8, None), (16, None), (4, 1), (16, 1), (8, 2)):
        if splits and splits > -(-hid // 128):
            continue
        fused = k.product_normed(h, delta, nw, w, waves=waves, splits=splits)
        if fused is None:                # many rows times many columns: left to a norm kernel of its own
            assert waves is None and (t * n > 400_000 or n * hid >= 64 << 20)
            continue
        prod, ss, h_new = fused
        assert torch.equal(h, h0)                                           # the input stream is left alone
        assert torch.equal(h_new, summed)
        assert torch.allclose(ss.double().sum(0).cpu(), (sd * sd).sum(-1), rtol=1e-5)
        inv = 1.0 / torch.sqrt(ss.double().sum(0).cpu() / hid + eps)
        got = prod.double().sum(0).cpu() * inv[:, None]
        assert float((got - ref).abs().max()) <= 1.2e-2 * float(ref.abs().max()), (waves, splits)
    # and the QKV epilogue applies that factor
    if n == 1152:
        nq, nkv, hd, ps = 14, 2, 64, 16
        positions = torch.zeros(t, dtype=torch.int32, device=DEV)
        out = torch.empty(t, n, dtype=dtype, device=DEV)
        kc = torch.zeros(1, nkv, ps, hd, dtype=dtype, device=DEV)
        vc = torch.zeros(1, nkv, hd, ps, dtype=dtype, device=DEV)
        inv_freq = torch.ones(hd // 2, device=DEV)
        k.qkv_rope_store(prod, None, positions, inv_freq, hd, None, kc, vc, nq, nkv, hd, ps, out=out, row_ss=ss, hidden=hid, eps=eps)
        assert float((out.double().cpu() - ref).abs().max()) <= 1.6e-2 * float(ref.abs().max())   # position 0: no rotation


@pytest.mark.parametrize("t,inter,n,g_splits", [(8, 4864, 896, 4), (3, 200, 120, 1), (16, 328, 192, 2), (7, 640, 100, 6),
                                                (5, 1000, 3080, 3)])
def test_product_with_swiglu_folded_in(k, t, inter, n, g_splits):
    gu = rnd(g_splits, t, 2 * inter, seed=1, scale=1.5)
    ss = torch.rand(3, t, generator=torch.Generator().manual_seed(2)).to(DEV) * 50 + 1
    w = rnd(n, inter, dtype=torch.bfloat16, seed=3, scale=0.05)
    hidden, eps = 77, 1e-5
    for row_ss in (None, ss):
        scale = 1.0 if row_ss is None else (1.0 / torch.sqrt(ss.double().sum(0).cpu() / hidden + eps))[:, None]
        z = gu.double().sum(0).cpu() * scale
        g, u = z[:, :inter], z[:, inter:]
        ref = plain.linear(u * g / (1 + torch.exp(-g)), w.double().cpu())
        for waves, max_splits in ((None, 20), (4, 20), (8, 20), (16, 20), (4, 1), (16, 2)):      # short and long k ranges
            prod = k.product_swiglu(gu, row_ss, hidden, eps, w, max_splits=max_splits, waves=waves)
            if prod is None:             # many columns: SwiGLU by itself, with the rows' factor, then the plain product
                assert waves is None and n >= 1536
                act = torch.empty(t, inter, dtype=torch.bfloat16, device=DEV)
                k.swiglu(gu, act, row_ss=row_ss, hidden=hidden, eps=eps)
                prod = k.product(act, w)
                act32 = torch.empty(t, inter, dtype=torch.float32, device=DEV)
                k.swiglu(gu, act32, row_ss=row_ss, hidden=hidden, eps=eps)
                assert float((act32.double().cpu() - u * g / (1 + torch.exp(-g))).abs().max()) <= 3e-6 * float((u * g).abs().max())
            assert prod is not None and prod.dim() == 3
            assert float((prod.double().sum(0).cpu() - ref).abs().max()) <= 1.2e-2 * float(ref.abs().max()), (waves, max_splits)


@pytest.mark.parametrize("t,inter,hid", [(64, 4864, 896), (17, 176, 64), (33, 250, 96), (48, 1000, 1544), (20, 23, 8),
                                          (64, 8960, 1536), (31, 40, 2056)])
def test_gate_up_product_with_swiglu(k, t, inter, hid):
    # one kernel for [gate | up] = x w^T and up * silu(gate); widths that are no multiple of a tile, of a chunk of 32 or
    # of the wavefronts' share of k; a k range of several rounds; one and two column groups per workgroup
    x = rnd(t, hid, dtype=torch.bfloat16, seed=1)
    w = rnd(2 * inter, hid, dtype=torch.bfloat16, seed=2, scale=1.5 / math.sqrt(hid))
    gu = plain.linear(x.double().cpu(), w.double().cpu())
    g, u = gu[:, :inter], gu[:, inter:]
    ref = u * (g / (1.0 + torch.exp(-g)))
    for groups in (1, 2, None):
        act = k.gate_up_swiglu(x, w, groups=groups)
        if act is None:                  # a large matrix: the wrapper leaves it to the product and the SwiGLU kernel
            assert groups is None and 2 * inter * hid >= 16 << 20
            continue
        assert act.dtype == torch.bfloat16 and tuple(act.shape) == (t, inter)
        assert float((act.double().cpu() - ref).abs().max()) <= 6e-3 * float(ref.abs().max()), groups
    # rows outside the kernel's range are refused by the wrapper, not computed wrongly
    assert k.gate_up_swiglu(x[:16].contiguous(), w) is None
    assert k.gate_up_swiglu(torch.cat([x, x, x, x, x])[:65].contiguous(), w) is None


@pytest.mark.parametrize("nq,nkv,hd,batch,ctx", [(14, 2, 64, 8, 700), (12, 2, 128, 3, 300), (14, 2, 64, 1, 2113), (3, 1, 64, 16, 90)])
def test_output_projection_combines_attention_parts(k, nq, nkv, hd, batch, ctx):
    # split attention left uncombined, then combined by the output projection: equals combine + plain product
    dtype, ps = torch.bfloat16, 16
    seqs = [(1, max(1, ctx - 37 * i % ctx)) for i in range(batch)]
    kc, vc, table, keys, vals = build_paged(seqs, nkv, hd, ps, dtype, seed=5)
    t = batch
    qkv = rnd(t, (nq + 2 * nkv) * hd, dtype=dtype, seed=6)
    q_len = torch.ones(t, dtype=torch.int32)
    q_start = torch.arange(t, dtype=torch.int32)
    kv_len = torch.tensor([kv for _, kv in seqs], dtype=torch.int32)
    args = (kc, vc, table, q_start.to(DEV), q_len.to(DEV), kv_len.to(DEV), nq, nkv, hd, ps, 1.0 / math.sqrt(hd), 0, 1,
            int(kv_len.max()))
    out = torch.empty(t, nq * hd, dtype=dtype, device=DEV)
    assert k.paged_attention(qkv, out, *args) is None
    parts = k.paged_attention(qkv, torch.empty_like(out), *args, combine=False)
    if parts is None:            # few requests with short contexts are not split
        assert int(kv_len.max()) < 512
        return
    again = torch.empty_like(out)
    k.combine_attention(parts[0], parts[1], again)
    assert float((again.float() - out.float()).abs().max()) <= 2e-2      # other splits, other rounding
    w = rnd(200, nq * hd, dtype=dtype, seed=7, scale=0.05)
    ref = plain.linear(again.double().cpu(), w.double().cpu())
    for waves, max_splits in ((None, None), (4, 4), (8, 4), (16, 4), (4, 1), (8, 2), (8, 14)):
        prod = k.product_attention(parts[0], parts[1], w, max_splits=max_splits, waves=waves)
        if prod is None:             # a long k range over too many heads
            assert max_splits is not None and max_splits < 4
            continue
        assert float((prod.double().sum(0).cpu() - ref).abs().max()) <= 1.2e-2 * float(ref.abs().max()), (waves, max_splits)


def test_consumers_take_a_float32_product_of_many_rows(k):
    # many-row products are written out in float32 and handed on as one "partial sum" [1, T, N]
    dtype = torch.bfloat16
    t, hid = 70, 896
    delta = rnd(1, t, hid, seed=1)
    h = rnd(t, hid, seed=2, scale=2.0)
    h0 = h.clone()
    w = (1 + rnd(hid, seed=3, scale=0.1)).to(dtype)
    out = torch.empty(t, hid, dtype=dtype, device=DEV)
    k.add_rmsnorm(h, delta, w, 1e-6, out)
    assert torch.equal(h, h0 + delta[0])
    ref = plain.rms_norm((h0 + delta[0]).double().cpu(), w.double().cpu(), 1e-6)
    assert float((out.double().cpu() - ref).abs().max()) <= 1.6e-2 * float(ref.abs().max())
    rows = torch.arange(t - 1, -1, -2, dtype=torch.int32, device=DEV)
    out2 = torch.empty(rows.shape[0], hid, dtype=dtype, device=DEV)
    k.rows_add_rmsnorm(h0.clone(), delta, rows, w, 1e-6, out2)
    assert float((out2.double().cpu() - ref[rows.long().cpu()]).abs().max()) <= 1.6e-2 * float(ref.abs().max())
    inter = 328
    gu = rnd(1, t, 2 * inter, seed=4, scale=2.0)
    act = torch.empty(t, inter, dtype=dtype, device=DEV)
    k.swiglu(gu, act)
    g, u = gu[0, :, :inter].double().cpu(), gu[0, :, inter:].double().cpu()
    refa = u * g / (1 + torch.exp(-g))
    assert float((act.double().cpu() - refa).abs().max()) <= 1.6e-2 * float(refa.abs().max())
    nq, nkv, hd, ps = 6, 2, 64, 16
    width = (nq + 2 * nkv) * hd
    qp = rnd(1, t, width, seed=5)
    bias = rnd(width, dtype=dtype, seed=6)
    positions = torch.arange(100, 100 + t, dtype=torch.int32, device=DEV)
    inv = plain.rope_inv_freq(hd, 1e6).to(DEV)
    slots = torch.randperm(6 * ps, generator=torch.Generator().manual_seed(7))[:t].to(torch.int32).to(DEV)
    kc = torch.zeros(6, nkv, ps, hd, dtype=dtype, device=DEV)
    vc = torch.zeros(6, nkv, hd, ps, dtype=dtype, device=DEV)
    got = torch.empty(t, width, dtype=dtype, device=DEV)
    k.qkv_rope_store(qp, bias, positions, inv, hd, slots, kc, vc, nq, nkv, hd, ps, out=got, cos_sin=k.rope_table(positions, inv))
    x = (qp[0].double() + bias.double()).cpu().view(t, nq + 2 * nkv, hd)
    refq = x.clone()
    refq[:, : nq + nkv] = plain.rope(x[:, : nq + nkv], positions.cpu(), 1e6)
    assert float((got.double().cpu().view(t, -1, hd) - refq).abs().max()) <= 1.6e-2 * float(refq.abs().max())
    for i in (0, 33, 69):
        pg, off = int(slots[i]) // ps, int(slots[i]) % ps
        assert torch.equal(kc[pg, :, off, :], got.view(t, -1, hd)[i, nq : nq + nkv])
        assert torch.equal(vc[pg, :, :, off], got.view(t, -1, hd)[i, nq + nkv :])


def test_rope_table_holds_what_the_kernels_compute(k):
    # the step's table of cosines and sines against float64, and: a kernel that takes the table leaves the same
    # bits as one that computes the angles itself
    hd, nq, nkv, ps, t = 64, 3, 1, 16, 9
    positions = torch.tensor([0, 1, 2, 17, 255, 4095, 32767, 100000, 5], dtype=torch.int32, device=DEV)
    inv = plain.rope_inv_freq(hd, 1e6).to(DEV)
    tab = k.rope_table(positions, inv)
    ang = (positions.cpu().float()[:, None] * inv.cpu()[None, :]).double()       # the float32 product, as the reference forms it
    assert tab.shape == (t, hd // 2, 2)
    assert float((tab[..., 0].double().cpu() - torch.cos(ang)).abs().max()) <= 2e-7
    assert float((tab[..., 1].double().cpu() - torch.sin(ang)).abs().max()) <= 2e-7
    width = (nq + 2 * nkv) * hd
    for dtype in DTYPES:
        qkv = rnd(t, width, dtype=dtype, seed=1)
        slots = torch.arange(t, dtype=torch.int32, device=DEV)
        outs = []
        for cs in (None, tab):
            kc = torch.zeros(1, nkv, ps, hd, dtype=dtype, device=DEV)
            vc = torch.zeros(1, nkv, hd, ps, dtype=dtype, device=DEV)
            out = torch.empty_like(qkv)
            k.qkv_rope_store(qkv, None, positions, inv, hd, slots, kc, vc, nq, nkv, hd, ps, out=out, cos_sin=cs)
            outs.append((out, kc, vc))
        for a, b in zip(*outs):
            assert torch.equal(a, b)


def test_linear_vector_of_the_reference(k):
    # /root/reference/test/matmul_3d_test.cpp:60-87
    x = torch.tensor([[1.0, 2, 3], [4, 5, 6]], device=DEV)
    w = torch.tensor([[1.0, 0, -1], [2, 3, 4]], device=DEV)
    b = torch.tensor([0.5, -1.0], device=DEV)
    out = torch.empty(2, 2, device=DEV)
    k.linear(x, w, b, out)
    assert torch.equal(out.cpu(), torch.tensor([[-1.5, 19.0], [-1.5, 46.0]]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inter", [211, 216, 4864])
def test_swiglu(k, dtype, inter):
    gu = rnd(9, 2 * inter, dtype=dtype, scale=3.0)
    out = torch.empty(9, inter, dtype=dtype, device=DEV)
    k.swiglu(gu, out)
    g, u = gu[:, :inter].double().cpu(), gu[:, inter:].double().cpu()
    ref = u * g / (1 + torch.exp(-g))
    assert float((out.double().cpu() - ref).abs().max()) <= tol(dtype, float(ref.abs().max()))
    z = torch.zeros(2, 2 * 16, dtype=dtype, device=DEV)
    z[:, 16:] = 5.0
    o = torch.ones(2, 16, dtype=dtype, device=DEV)
    k.swiglu(z, o)
    assert torch.equal(o, torch.zeros_like(o))                    # silu(0) = 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("t", [11, 77])
@pytest.mark.parametrize("table", [False, True])         # angles computed in the kernel, or taken from the step's table
@pytest.mark.parametrize("nq,nkv,hd,rd,theta", [(6, 3, 48, 48, 1e4), (5, 1, 80, 80, 1e6), (4, 4, 32, 16, 5e5), (14, 2, 64, 64, 1e6)])
def test_qkv_rope_store(k, dtype, nq, nkv, hd, rd, theta, t, table):
    ps, pages = 4, 9 if t == 11 else 30
    qkv = rnd(t, (nq + 2 * nkv) * hd, dtype=dtype, seed=1)
    bias = rnd((nq + 2 * nkv) * hd, dtype=dtype, seed=2)
    base_pos = [0, 1, 2, 3, 250, 251, 7, 8, 9, 4000, 31]
    positions = torch.tensor((base_pos * 8)[:t], dtype=torch.int32, device=DEV)
    inv = torch.pow(torch.tensor(theta, dtype=torch.float32), -2.0 * torch.arange(rd // 2, dtype=torch.float32) / rd).to(DEV)
    perm = torch.randperm(pages * ps, generator=torch.Generator().manual_seed(3))[:t]
    slots = perm.to(torch.int32).to(DEV)
    kc = torch.full((pages, nkv, ps, hd), 77.0, dtype=dtype, device=DEV)
    vc = torch.full((pages, nkv, hd, ps), 77.0, dtype=dtype, device=DEV)
    x = (qkv.double() + bias.double()).cpu().view(t, nq + 2 * nkv, hd)
    k.qkv_rope_store(qkv, bias, positions, inv, rd, slots, kc, vc, nq, nkv, hd, ps,
                     cos_sin=k.rope_table(positions, inv) if table else None)
    ang = (positions.cpu().float()[:, None] * inv.cpu()[None, :]).double()
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    ref = x.clone()
    x1, x2 = x[:, : nq + nkv, : rd // 2], x[:, : nq + nkv, rd // 2 : rd]
    ref[:, : nq + nkv, : rd // 2] = x1 * cos - x2 * sin
    ref[:, : nq + nkv, rd // 2 : rd] = x1 * sin + x2 * cos
    got = qkv.double().cpu().view(t, nq + 2 * nkv, hd)
    assert float((got - ref).abs().max()) <= tol(dtype, float(ref.abs().max()))
    written = torch.zeros(pages * ps, dtype=torch.bool)
    for i in range(t):
        p, o = int(perm[i]) // ps, int(perm[i]) % ps
        written[int(perm[i])] = True
        assert torch.equal(kc[p, :, o, :], qkv.view(t, -1, hd)[i, nq : nq + nkv])
        assert torch.equal(vc[p, :, :, o], qkv.view(t, -1, hd)[i, nq + nkv :])
    untouched = kc.permute(0, 2, 1, 3).reshape(pages * ps, -1)[~written]
    assert torch.all(untouched == 77.0)                          # nothing else was written


def paged_reference(q, keys, vals, nq, nkv, scale, window):
    """q [n, nq, hd] are the last n positions of a sequence whose keys/values [kv, nkv, hd] are given."""
    n, kv = q.shape[0], keys.shape[0]
    out = torch.empty_like(q)
    for i in range(n):
        p = kv - n + i
        lo = max(0, p - window + 1) if window else 0
        for h in range(nq):
            kh = h // (nq // nkv)
            s = (keys[lo : p + 1, kh] @ q[i, h]) * scale
            out[i, h] = torch.softmax(s, 0) @ vals[lo : p + 1, kh]
    return out


def build_paged(seqs, nkv, hd, ps, dtype, seed=0, extra_pages=3, ramp=0.0):
    """seqs: list of (q_len, kv_len).  Returns everything paged_attention needs, with pages handed out in a
    shuffled order and unused slots filled with huge values (reading one would wreck the result).  ramp: the keys'
    first feature is ramp * position instead of random."""
    g = torch.Generator().manual_seed(seed)
    n_pages = sum(-(-kv // ps) for _, kv in seqs) + extra_pages
    order = torch.randperm(n_pages, generator=g).tolist()
    kc = torch.full((n_pages, nkv, ps, hd), 1e4, dtype=dtype)
    vc = torch.full((n_pages, nkv, hd, ps), -1e4, dtype=dtype)
    width = max(-(-kv // ps) for _, kv in seqs)
    table = torch.full((len(seqs), width), -1, dtype=torch.int32)
    keys, vals = [], []
    for b, (_, kv) in enumerate(seqs):
        kk = torch.randn(kv, nkv, hd, generator=g).to(dtype)
        vv = torch.randn(kv, nkv, hd, generator=g).to(dtype)
        if ramp:
            kk[:, :, 0] = (ramp * torch.arange(kv, dtype=torch.float32))[:, None].to(dtype)
        keys.append(kk)
        vals.append(vv)
        n = -(-kv // ps)
        pages = torch.tensor([order.pop() for _ in range(n)], dtype=torch.int64)
        table[b, :n] = pages.to(torch.int32)
        kp = torch.full((n * ps, nkv, hd), 1e4, dtype=dtype)
        vp = torch.full((n * ps, nkv, hd), -1e4, dtype=dtype)
        kp[:kv], vp[:kv] = kk, vv
        kc[pages] = kp.view(n, ps, nkv, hd).permute(0, 2, 1, 3)
        vc[pages] = vp.view(n, ps, nkv, hd).permute(0, 2, 3, 1)
    return kc.to(DEV), vc.to(DEV), table.to(DEV), keys, vals


def run_paged(k, seqs, nq, nkv, hd, ps, dtype, window=0, seed=0, q_scale=1.0, tiled_shape=None, ramp=0.0,
              singles=(0, 0, 0), key_splits=1):
    kc, vc, table, keys, vals = build_paged(seqs, nkv, hd, ps, dtype, seed, ramp=ramp)
    t = sum(q for q, _ in seqs)
    g = torch.Generator().manual_seed(seed + 100)
    qkv = torch.randn(t, (nq + 2 * nkv) * hd, generator=g) * q_scale
    if ramp:
        qkv.view(t, nq + 2 * nkv, hd)[:, :nq, 0] = 1.0        # every query weighs the keys' ramp alike
    qkv = qkv.to(dtype).to(DEV)
    q_len = torch.tensor([q for q, _ in seqs], dtype=torch.int32)
    q_start = torch.cumsum(q_len, 0, dtype=torch.int32) - q_len
    kv_len = torch.tensor([kv for _, kv in seqs], dtype=torch.int32)
    out = torch.empty(t, nq * hd, dtype=dtype, device=DEV)
    scale = 1.0 / math.sqrt(hd)
    if tiled_shape is None:
        k.paged_attention(qkv, out, kc, vc, table, q_start.to(DEV), q_len.to(DEV), kv_len.to(DEV), nq, nkv, hd, ps,
                          scale, window, int(q_len.max()), int(kv_len.max()))
    else:
        # the LDS-tiled kernel with a given workgroup shape (the wrapper picks one by the amount of work)
        # singles = (key ranges, wavefronts, lean variant) of the decode kernel that takes the requests of one token
        qs, ql, kl = q_start.to(DEV), q_len.to(DEV), kv_len.to(DEV)
        # key_splits: workgroups that share the keys of a block of rows; both leave parts in the same memory
        part_rows = max(singles[0] * len(seqs), key_splits * t if key_splits > 1 else 0)
        part_o = torch.full((part_rows, nq, hd), float("nan"), device=DEV)
        part_ml = torch.full((part_rows, nq, 2), float("nan"), device=DEV)
        out.fill_(float("nan"))
        k._run("egpt_paged_attention_tiled", qkv.data_ptr(), out.data_ptr(), kc.data_ptr(), vc.data_ptr(),
               table.data_ptr(), table.shape[1], qs.data_ptr(), ql.data_ptr(), kl.data_ptr(), len(seqs), t, nq, nkv,
               hd, ps, scale, window, tiled_shape, key_splits, k._ptr(part_o), k._ptr(part_ml), *singles, k._stream())
        torch.cuda.synchronize()
    got = out.double().cpu().view(t, nq, hd)
    worst = 0.0
    for b, (n, kv) in enumerate(seqs):
        s = int(q_start[b])
        q = qkv[s : s + n].double().cpu().view(n, nq + 2 * nkv, hd)[:, :nq]
        ref = paged_reference(q, keys[b].double(), vals[b].double(), nq, nkv, scale, window)
        worst = max(worst, float((got[s : s + n] - ref).abs().max()))
    return worst


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,hd,ps", [(6, 3, 48, 4), (7, 1, 64, 16), (4, 4, 16, 5), (10, 5, 80, 16), (2, 1, 128, 64),
                                           (3, 3, 256, 16), (14, 2, 64, 16), (12, 2, 128, 16), (5, 5, 64, 32),
                                           (6, 2, 64, 4)])
def test_paged_attention_ragged_batch(k, dtype, nq, nkv, hd, ps):
    # prompt portions (with and without a prefix in the cache) beside single decoded tokens
    seqs = [(1, 1), (9, 9), (1, 130), (7, 71), (2, 64), (1, 65), (33, 33), (3, 200)]
    err = run_paged(k, seqs, nq, nkv, hd, ps, dtype)
    assert err <= (2e-6 if dtype == torch.float32 else 1.2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hd", [32, 64])
@pytest.mark.parametrize("window", [1, 7, 64, 65])
def test_paged_attention_window(k, dtype, window, hd):
    seqs = [(1, 100), (20, 90), (5, 5), (1, window), (1, window + 1), (3, 66), (40, 300)]
    err = run_paged(k, seqs, 6, 2, hd, 16, dtype, window=window)
    assert err <= (2e-6 if dtype == torch.float32 else 1.2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,hd,ps", [(4, 2, 16, 16), (6, 2, 32, 32), (6, 3, 48, 16), (14, 2, 64, 16), (10, 5, 80, 48),
                                           (8, 2, 96, 16), (7, 1, 112, 16), (12, 2, 128, 64), (4, 1, 144, 16),
                                           (5, 5, 160, 32), (3, 1, 192, 16), (2, 2, 224, 16), (20, 1, 256, 16)])
def test_attention_for_any_head_size_on_the_matrix_cores(k, dtype, nq, nkv, hd, ps):
    # every head size in steps of 16, both precisions (bfloat16 heads of 64 and 128 have kernels of their own, float32
    # ones do not): prompt portions with and without a prefix, lengths around the chunks of 32 and 64 keys and the
    # segments of 256, and a group of more than 16 heads
    seqs = [(1, 1), (9, 9), (1, 130), (7, 71), (2, 64), (1, 65), (33, 33), (3, 200), (70, 300), (40, 520), (5, 1029)]
    err = run_paged(k, seqs, nq, nkv, hd, ps, dtype)
    assert err <= (3e-6 if dtype == torch.float32 else 1.2e-2)
    # only decoded tokens: the kernel that gives every segment of 256 keys a wavefront, and the fold
    seqs = [(1, max(1, 1500 - 211 * i)) for i in range(8)] + [(1, 256), (1, 257), (1, 512), (1, 2113)]
    err = run_paged(k, seqs, nq, nkv, hd, ps, dtype, seed=2)
    assert err <= (3e-6 if dtype == torch.float32 else 1.2e-2)
    # peaked scores, where a skipped or misplaced key shows
    err = run_paged(k, [(1, 700), (4, 513), (1, 17), (60, 260)], nq, nkv, hd, ps, dtype, q_scale=5.0, seed=3)
    assert err <= (3e-5 if dtype == torch.float32 else 5e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hd,window", [(32, 7), (96, 64), (96, 300), (64, 257), (160, 1000)])
def test_attention_for_any_head_size_with_a_window(k, dtype, hd, window):
    seqs = [(1, 100), (20, 90), (5, 5), (1, window), (1, window + 1), (3, 66), (40, 300), (1, 900), (70, 1400)]
    assert run_paged(k, seqs, 6, 2, hd, 16, dtype, window=window) <= (3e-6 if dtype == torch.float32 else 1.2e-2)
    seqs = [(1, 100), (1, window), (1, window + 1), (1, 900), (1, 1400), (1, 2000)]
    assert run_paged(k, seqs, 6, 2, hd, 16, dtype, window=window) <= (3e-6 if dtype == torch.float32 else 1.2e-2)


@pytest.mark.parametrize("hd,ps,window", [(64, 16, 0), (48, 16, 0), (128, 32, 0), (256, 16, 0), (80, 16, 100), (64, 16, 300)])
def test_float32_attention_gives_the_same_bits_however_the_rows_are_cut(k, hd, ps, window):
    # a token's float32 result from the prompt kernel (as a row of a portion, beside other rows and requests) and
    # from the decode kernel (alone behind its context, in a batch of other lengths) are the same bits: both take
    # the keys in chunks and segments at fixed positions and fold them with the same operations
    nq, nkv, dtype = 6, 2, torch.float32
    n, kv = 70, 700
    seqs = [(3, 40), (n, kv), (1, 9)]
    kc, vc, table, keys, vals = build_paged(seqs, nkv, hd, ps, dtype, seed=21)
    t = sum(q for q, _ in seqs)
    qkv = rnd(t, (nq + 2 * nkv) * hd, seed=22, scale=2.0)
    ints = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    scale = 1.0 / math.sqrt(hd)
    whole = torch.empty(t, nq * hd, device=DEV)
    k.paged_attention(qkv, whole, kc, vc, table, ints([0, 3, 3 + n]), ints([3, n, 1]), ints([40, kv, 9]), nq, nkv, hd, ps,
                      scale, window, n, kv)
    # the same portion cut in two, the second part alone in its step
    cut = torch.empty(n - 33, nq * hd, device=DEV)
    k.paged_attention(qkv[3 + 33 : 3 + n].contiguous(), cut, kc, vc, table[1:2].contiguous(), ints([0]), ints([n - 33]),
                      ints([kv]), nq, nkv, hd, ps, scale, window, n - 33, kv)
    assert torch.equal(cut, whole[3 + 33 : 3 + n])
    # every token of the portion as a decoded token behind its own context, all of them in one batch
    lens = [kv - n + i + 1 for i in range(n)]
    single = torch.empty(n, nq * hd, device=DEV)
    k.paged_attention(qkv[3 : 3 + n].contiguous(), single, kc, vc, table[1:2].expand(n, -1).contiguous(),
                      ints(list(range(n))), ints([1] * n), ints(lens), nq, nkv, hd, ps, scale, window, 1, kv)
    assert torch.equal(single, whole[3 : 3 + n])


@pytest.mark.parametrize("hd,shape", [(64, 41), (64, 42), (64, 44), (64, 22), (64, 24), (128, 41), (128, 42), (128, 22),
                                      (64, 121), (64, 122), (64, 124), (64, 141), (64, 142), (128, 121), (128, 122), (128, 141)])
@pytest.mark.parametrize("window,ps", [(0, 16), (0, 64), (100, 32), (300, 16)])
def test_paged_attention_tiled_workgroup_shapes(k, hd, shape, window, ps):
    # every workgroup shape of the LDS-tiled kernel (row tiles x key splits): prompts over several row groups and
    # key tiles, a prefix in the cache, single tokens, lengths at and around the tile sizes
    seqs = [(300, 700), (1, 1), (64, 64), (65, 129), (2, 513), (1, 257), (127, 128), (17, 1000)]
    assert run_paged(k, seqs, 6, 2, hd, ps, torch.bfloat16, window=window, tiled_shape=shape) <= 1.2e-2
    assert run_paged(k, seqs, 7, 1, hd, ps, torch.bfloat16, window=window, tiled_shape=shape, q_scale=6.0, seed=3) <= 4e-2


@pytest.mark.parametrize("hd,shape", [(64, None), (64, 44), (128, None), (128, 41), (64, 142), (64, 124), (128, 122)])
@pytest.mark.parametrize("window", [0, 4099])
def test_paged_attention_long_prefixes(k, hd, shape, window):
    # prompt portions behind thousands of cached keys: many key tiles for each row tile, block tables hundreds of pages wide
    seqs = [(96, 9000), (1, 5000), (40, 12001), (3, 3)]
    assert run_paged(k, seqs, 6, 2, hd, 16, torch.bfloat16, window=window, tiled_shape=shape, seed=5) <= 1.2e-2


@pytest.mark.parametrize("hd,shape", [(64, 142), (64, 121), (128, 141), (64, 42), (128, 42)])
@pytest.mark.parametrize("ramp", [0.26, 0.9, -0.26, 4.0])
def test_prompt_attention_with_scores_that_grow_along_the_keys(k, hd, shape, ramp):
    # the kernel of 32-row blocks rescales what it has accumulated only when a row's maximum has grown by more than a
    # margin, and takes the exponentials against the old maximum until then.  Scores that rise by about 3 (in powers
    # of two) from one tile of 64 keys to the next keep it just below the margin for several tiles in a row; a rise
    # of 10 a tile goes over it in every tile, 45 a tile by far; falling scores never rescale after the first tile.
    seqs = [(300, 1500), (64, 64), (33, 700)]
    r = ramp * math.sqrt(hd / 64)
    assert run_paged(k, seqs, 6, 2, hd, 16, torch.bfloat16, tiled_shape=shape, seed=9, ramp=r) <= 1.2e-2
    assert run_paged(k, seqs, 6, 2, hd, 32, torch.bfloat16, window=200, tiled_shape=shape, seed=10, ramp=r) <= 1.2e-2
    # one head to a group, and sixteen
    assert run_paged(k, seqs, 3, 3, hd, 64, torch.bfloat16, tiled_shape=shape, seed=11, ramp=r) <= 1.2e-2
    assert run_paged(k, [(90, 400), (1, 77)], 16, 1, hd, 16, torch.bfloat16, tiled_shape=shape, seed=12, ramp=r) <= 1.2e-2


@pytest.mark.parametrize("hd,shape", [(64, 124), (64, 142), (64, 122), (64, 121), (128, 141), (128, 122)])
@pytest.mark.parametrize("key_splits", [2, 3, 7])
def test_portions_whose_blocks_of_rows_share_their_keys_among_workgroups(k, hd, shape, key_splits):
    # portions behind prefixes of different lengths (one with fewer tiles of keys than workgroups that share them), a
    # fresh prompt, a window; the keys' ramp makes every far key count, so a range that is left out or taken twice shows
    seqs = [(70, 1300), (33, 33), (5, 2100), (130, 130), (40, 700)]
    r = 8.0 / 2100
    assert run_paged(k, seqs, 6, 2, hd, 16, torch.bfloat16, tiled_shape=shape, key_splits=key_splits, seed=31, ramp=r) <= 1.2e-2
    assert run_paged(k, seqs, 7, 1, hd, 64, torch.bfloat16, window=500, tiled_shape=shape, key_splits=key_splits, seed=32) <= 1.2e-2
    assert run_paged(k, seqs, 4, 4, hd, 32, torch.bfloat16, tiled_shape=shape, key_splits=key_splits, seed=33, q_scale=5.0) <= 4e-2
    # with the requests of one token taken by the decode kernel behind it, parts in the same memory
    mixed = [(70, 1300), (1, 2500), (1, 77), (33, 33), (1, 1), (2, 900)]
    for singles in ((1, 8, 0), (5, 4, 1)):
        assert run_paged(k, mixed, 6, 2, hd, 16, torch.bfloat16, tiled_shape=shape, key_splits=key_splits, singles=singles,
                         seed=34, ramp=8.0 / 2500) <= 1.2e-2


def test_attention_parts_before_a_large_output_projection_are_combined_apart(k):
    # the product that combines the parts itself is for matrices on which that pays; beyond, the caller combines
    po = torch.zeros(2, 1, 40, 128, device=DEV)
    pml = torch.zeros(2, 1, 40, 2, device=DEV)
    assert k.product_attention(po, pml, torch.empty(5120, 5120, dtype=torch.bfloat16, device=DEV)) is None
    assert k.product_attention(po, pml, torch.zeros(1024, 5120, dtype=torch.bfloat16, device=DEV)) is not None


def test_paged_attention_tiled_refuses_other_page_sizes(k):
    z = torch.zeros(64, device=DEV)
    p = z.data_ptr()
    # not a power of two, too small, no such shape, pages larger than the tiles of the kernel of 32-row blocks
    for ps, shape in ((48, 42), (8, 42), (16, 43), (128, 142)):
        with pytest.raises(RuntimeError):
            k._run("egpt_paged_attention_tiled", p, p, p, p, p, 1, p, p, p, 1, 1, 2, 1, 64, ps, 0.1, 0, shape, 1, None,
                   None, 0, 0, 0, None)
    # shared keys: only in the kernel of 32-row blocks, and with room for the parts
    for shape, splits, parts in ((42, 2, p), (142, 2, None), (142, 0, p), (142, 65, p)):
        with pytest.raises(RuntimeError):
            k._run("egpt_paged_attention_tiled", p, p, p, p, p, 1, p, p, p, 1, 1, 2, 1, 64, 16, 0.1, 0, shape, splits, parts,
                   parts, 0, 0, 0, None)
    # single tokens to the decode kernel: more than 16 heads to a group, key ranges without room for their parts
    for nq, splits, parts in ((17, 1, None), (2, 2, None), (2, 65, p)):
        with pytest.raises(RuntimeError):
            k._run("egpt_paged_attention_tiled", p, p, p, p, p, 1, p, p, p, 1, 1, nq, 1, 64, 16, 0.1, 0, 42, 1, parts, parts,
                   splits, 4, 0, None)


@pytest.mark.parametrize("hd,shape", [(64, 24), (64, 44), (64, 142), (128, 42), (128, 141)])
@pytest.mark.parametrize("singles", [(1, 8, 0), (1, 1, 1), (3, 4, 1), (7, 8, 0)])
def test_a_mixed_step_hands_its_single_tokens_to_the_decode_kernel(k, hd, shape, singles):
    # portions beside requests of one token behind short and long contexts; the key ranges' parts are kept by
    # request, the results go to the tokens' rows; the keys' ramp makes every far key count
    seqs = [(70, 300), (1, 2500), (1, 77), (33, 33), (1, 1), (1, 4100), (2, 900), (1, 64)]
    r = 8.0 / 4100
    assert run_paged(k, seqs, 6, 2, hd, 16, torch.bfloat16, tiled_shape=shape, singles=singles, seed=21, ramp=r) <= 1.2e-2
    assert run_paged(k, seqs, 16, 1, hd, 32, torch.bfloat16, window=700, tiled_shape=shape, singles=singles, seed=22) <= 1.2e-2
    # nothing but single tokens and one portion at the end; no single tokens at all
    assert run_paged(k, [(1, 500)] * 5 + [(40, 1000)], 3, 3, hd, 64, torch.bfloat16, tiled_shape=shape, singles=singles, seed=23) <= 1.2e-2
    assert run_paged(k, [(5, 500), (40, 1000)], 4, 2, hd, 16, torch.bfloat16, tiled_shape=shape, singles=singles, seed=24) <= 1.2e-2


@pytest.mark.parametrize("nq,nkv,hd", [(14, 2, 64), (12, 2, 128), (3, 1, 64)])
@pytest.mark.parametrize("batch,ctx", [(1, 2113), (8, 700), (64, 130), (3, 33), (1, 20011), (4, 6007), (40, 1500)])
def test_paged_attention_decode_batches_split_the_key_range(k, nq, nkv, hd, batch, ctx):
    # only decoded tokens, different lengths: the matrix-core kernel splits the keys and combines the parts
    seqs = [(1, max(1, ctx - 37 * i % ctx)) for i in range(batch)]
    err = run_paged(k, seqs, nq, nkv, hd, 16, torch.bfloat16)
    assert err <= 1.2e-2
    assert run_paged(k, seqs, nq, nkv, hd, 16, torch.bfloat16, q_scale=6.0) <= 4e-2


@pytest.mark.parametrize("nq,nkv,hd,ps", [(14, 2, 64, 16), (12, 2, 128, 16), (3, 3, 64, 32), (16, 1, 64, 16)])
@pytest.mark.parametrize("batch,ctx,window", [(8, 700, 0), (1, 2113, 0), (64, 130, 0), (3, 33, 0), (5, 1, 0), (8, 300, 100),
                                              (1, 20011, 0), (4, 6007, 0), (40, 1500, 0), (2, 9000, 4099)])
@pytest.mark.parametrize("with_scale,with_bias", [(True, True), (False, False)])
def test_decode_attention_with_the_qkv_epilogue_folded_in(k, nq, nkv, hd, ps, batch, ctx, window, with_scale, with_bias):
    # one kernel for bias + rotation + store + attention must leave the same bits, in its output and in the
    # caches, as the two kernels it replaces (same operations in the same order), for every position of the new
    # token in its page and key block
    dtype = torch.bfloat16
    seqs = [(1, max(1, ctx - 37 * i % ctx)) for i in range(batch)]
    kc, vc, table, keys, vals = build_paged(seqs, nkv, hd, ps, dtype, seed=11)
    t, width = batch, (nq + 2 * nkv) * hd
    kv_len = torch.tensor([kv for _, kv in seqs], dtype=torch.int32)
    positions = (kv_len - 1).to(DEV)
    slots = torch.stack([table[b, (int(kv_len[b]) - 1) // ps].cpu() * ps + (int(kv_len[b]) - 1) % ps for b in range(t)]).to(torch.int32).to(DEV)
    prod = rnd(5, t, width, seed=12)
    row_ss = (torch.rand(3, t, generator=torch.Generator().manual_seed(13)) * 30 + 1).to(DEV) if with_scale else None
    bias = rnd(width, dtype=dtype, seed=14) if with_bias else None
    inv_freq = torch.as_tensor(plain.rope_inv_freq(hd, 1e4), dtype=torch.float32).to(DEV)
    q_start, q_len = torch.arange(t, dtype=torch.int32, device=DEV), torch.ones(t, dtype=torch.int32, device=DEV)
    scale = 1.0 / math.sqrt(hd)
    for combine in (True, False):
        kc1, vc1, kc2, vc2 = kc.clone(), vc.clone(), kc.clone(), vc.clone()
        qkv = torch.empty(t, width, dtype=dtype, device=DEV)
        k.qkv_rope_store(prod, bias, positions, inv_freq, hd, slots, kc1, vc1, nq, nkv, hd, ps, out=qkv,
                         row_ss=row_ss, hidden=96, eps=1e-5)
        out1 = torch.zeros(t, nq * hd, dtype=dtype, device=DEV)
        parts1 = k.paged_attention(qkv, out1, kc1, vc1, table, q_start, q_len, kv_len.to(DEV), nq, nkv, hd, ps, scale, window,
                                   1, int(kv_len.max()), combine=combine)
        out2 = torch.zeros(t, nq * hd, dtype=dtype, device=DEV)
        parts2 = k.attention_decode_fused(prod, row_ss, 96, 1e-5, bias, positions, inv_freq, hd, slots, out2, kc2, vc2, table,
                                          q_start, kv_len.to(DEV), nq, nkv, hd, ps, scale, window, int(kv_len.max()),
                                          combine=combine, cos_sin=k.rope_table(positions, inv_freq) if combine else None)
        assert parts2 is not False
        assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2)
        assert (parts1 is None) == (parts2 is None)
        if parts1 is None:
            assert torch.equal(out1, out2)
        else:
            assert torch.equal(parts1[0], parts2[0]) and torch.equal(parts1[1], parts2[1])


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_peaked_scores(k, dtype):
    # large queries make the softmax pick single keys, far ones included: a key skipped or read from the
    # wrong page then changes the output by O(1) instead of O(1/n)
    seqs = [(1, 700), (4, 513), (1, 17)]
    err = run_paged(k, seqs, 4, 2, 64, 16, dtype, q_scale=6.0)
    assert err <= (2e-5 if dtype == torch.float32 else 4e-2)


def test_paged_attention_one_far_key_stands_out(k):
    # one key among hundreds matches the query; the output must be that key's value, for every position of the key
    nq = nkv = 1
    hd, ps, kv = 32, 16, 500
    for far in (0, 15, 16, 255, 256, 498, 499):
        for dtype, hd in ((torch.float32, 32), (torch.bfloat16, 64)):
            _one_far_key(k, far, dtype, hd)


def _one_far_key(k, far, dtype, hd):
    nq = nkv = 1
    ps, kv = 16, 500
    if True:
        kk = torch.zeros(kv, 1, hd)
        vv = torch.randn(kv, 1, hd, generator=torch.Generator().manual_seed(far))
        kk[far, 0, 0] = 50.0
        pages = -(-kv // ps)
        kc = torch.zeros(pages, 1, ps, hd)
        vc = torch.zeros(pages, 1, hd, ps)
        table = torch.randperm(pages, generator=torch.Generator().manual_seed(1)).to(torch.int32)[None, :]
        for j in range(kv):
            kc[int(table[0, j // ps]), 0, j % ps] = kk[j, 0]
            vc[int(table[0, j // ps]), 0, :, j % ps] = vv[j, 0]
        qkv = torch.zeros(1, 3 * hd)
        qkv[0, 0] = 50.0
        out = torch.empty(1, hd, device=DEV, dtype=dtype)
        one = lambda v: torch.tensor([v], dtype=torch.int32, device=DEV)
        vv = vv.to(dtype)
        k.paged_attention(qkv.to(dtype).to(DEV), out, kc.to(dtype).to(DEV), vc.to(dtype).to(DEV), table.to(DEV), one(0),
                          one(1), one(kv), 1, 1, hd, ps, 1.0, 0, 1, kv)
        assert float((out.cpu()[0].float() - vv[far, 0].float()).abs().max()) < 1e-5, far


def test_paged_attention_refuses_bad_shapes(k):
    qkv = torch.zeros(2, 3 * 16, device=DEV)
    out = torch.zeros(2, 16, device=DEV)
    kc = torch.zeros(2, 1, 4, 16, device=DEV)
    vc = torch.zeros(2, 1, 16, 4, device=DEV)
    one = lambda v: torch.tensor([v], dtype=torch.int32, device=DEV)
    table = torch.zeros(1, 2, dtype=torch.int32, device=DEV)
    with pytest.raises(ValueError, match="block table"):
        k.paged_attention(qkv, out, kc, vc, table, one(0), one(2), one(9), 1, 1, 16, 4, 1.0, 0, 2, 9)
    with pytest.raises(ValueError, match="k_cache"):
        k.paged_attention(qkv, out, kc[:, :, :2].contiguous(), vc, table, one(0), one(2), one(8), 1, 1, 16, 4, 1.0, 0, 2, 8)
    with pytest.raises(TypeError):
        k.paged_attention(qkv.half(), out, kc, vc, table, one(0), one(2), one(8), 1, 1, 16, 4, 1.0, 0, 2, 8)
    big = torch.zeros(1, 3 * 512, device=DEV)
    with pytest.raises(ValueError, match="head size"):
        k.paged_attention(big, torch.zeros(1, 512, device=DEV), torch.zeros(2, 1, 4, 512, device=DEV),
                          torch.zeros(2, 1, 512, 4, device=DEV), table, one(0), one(1), one(1), 1, 1, 512, 4, 1.0, 0, 1, 1)


def test_argmax_lowest_index_wins(k):
    logits = rnd(6, 1000, seed=4)
    logits[2, 5] = logits[2, 900] = 99.0
    logits[3, 999] = 98.0
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    k.argmax(logits, out)
    exp = [plain.greedy(row) for row in logits.cpu()]
    assert out.tolist() == exp and exp[2] == 5 and exp[3] == 999
    wide = rnd(2, 151936, seed=5)
    out2 = torch.empty(2, dtype=torch.int32, device=DEV)
    k.argmax(wide, out2)
    assert out2.tolist() == wide.argmax(-1).tolist()


@pytest.mark.parametrize("vocab,scale", [(777, 2.5), (5000, 2.5), (9001, 2.5), (151936, 2.5), (40003, 0.02), (151936, 9.0),
                                         (8192, 0.0)])
def test_sample_follows_the_reference_s_distribution(k, vocab, scale):
    # narrow vocabularies go through one kernel, wide ones (from 8,192 tokens) through the staged one; logits nearly
    # flat (every token in one exponent of the weights: nothing can be cut before the selection), all equal, and peaked
    rows = 64
    logits = rnd(rows, vocab, seed=6, scale=scale)
    cases = [(0.8, 20, 0.95), (1.0, 0, 1.0), (0.5, 5, 0.5), (2.0, 0, 0.9), (1.3, 50, 1.0), (0.0, 0, 1.0), (0.7, 0, 0.3),
             (1.0, 3000, 0.99)]
    g = torch.Generator().manual_seed(9)
    temp = torch.tensor([cases[i % len(cases)][0] for i in range(rows)])
    topk = torch.tensor([cases[i % len(cases)][1] for i in range(rows)], dtype=torch.int32)
    topp = torch.tensor([cases[i % len(cases)][2] for i in range(rows)])
    if scale == 0.0:
        # all tokens tie: a cut by count or by mass has no boundary to fall on (the kernel keeps ties whole, the
        # reference's sort keeps the lowest indices); what is compared is the draw from the whole row
        topk.zero_()
        topp.fill_(1.0)
    # The kernel selects on float32 weights and keeps the tokens that tie with the k-th whole.  Where the k-th and the
    # next weight of a row are closer than float32 tells apart (it happens among thousands of nearly equal ones), the
    # float64 reference still separates them: such a row takes the next k whose boundary float32 resolves.
    for r in range(rows):
        kk = int(topk[r])
        if temp[r] > 0 and 0 < kk < vocab:
            srt = torch.sort(logits[r].cpu().double(), descending=True).values / float(temp[r])
            while kk < vocab and float(srt[kk - 1] - srt[kk]) < 1e-6:
                kk += 1
            topk[r] = kk
    u = torch.rand(rows, generator=g)
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    k.sample(logits, temp.to(DEV), topk.to(DEV), topp.to(DEV), u.to(DEV), out)
    out = out.tolist()
    for r in range(rows):
        row = logits[r].cpu()
        if temp[r] <= 0:
            assert out[r] == plain.greedy(row)
            continue
        dist = plain.sampling_distribution(row, float(temp[r]), int(topk[r]), float(topp[r]))
        assert dist[out[r]] > 0, f"row {r}: token {out[r]} is outside the kept set"
        cdf = torch.cumsum(dist, 0)
        lo = float(cdf[out[r]] - dist[out[r]])
        assert lo - 1e-4 <= float(u[r]) <= float(cdf[out[r]]) + 1e-4, f"row {r}"


def test_sample_frequencies(k):
    # many draws from one row: empirical frequencies follow softmax(logits / T) over the kept set
    vocab, n = 40, 4000
    row = rnd(1, vocab, seed=7, scale=1.5)
    logits = row.expand(n, vocab).contiguous()
    u = torch.rand(n, generator=torch.Generator().manual_seed(10)).to(DEV)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    full = lambda v, dt=torch.float32: torch.full((n,), v, dtype=dt, device=DEV)
    k.sample(logits, full(0.7), full(10, torch.int32), full(0.9), u, out)
    dist = plain.sampling_distribution(row[0].cpu(), 0.7, 10, 0.9)
    freq = torch.bincount(out.cpu().long(), minlength=vocab).double() / n
    assert float((freq - dist).abs().max()) < 0.03
    assert torch.all(freq[dist == 0] == 0)
