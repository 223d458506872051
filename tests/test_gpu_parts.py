"""Each part of a layer alone on the GPU against the plain implementation's function for it."""
from types import SimpleNamespace

import pytest
import torch

import plain_qwen2 as plain
from easy_gpt.cpp_amd.parts import CacheView, PartSpec, make_part

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return 5e-6 if dtype == torch.float32 else 2e-2


def whole(t):
    """A part may hand back float32 partial sums [splits, T, H] of its last product; their sum is the output."""
    return t.double().sum(0) if t.dim() == 3 else t.double()


def weights_for(part, dtype, seed=0, scale=0.05):
    g = torch.Generator().manual_seed(seed)
    w = {}
    for s in part.param_specs():
        t = torch.randn(s.shape, generator=g) * scale
        if s.role == "norm_scale":
            t = t + 1.0
        w[s.name] = t.to(dtype).float()          # values exactly representable in the engine's dtype
    part.load(lambda n: w[n], dtype, DEV)
    return {n: t.double() for n, t in w.items()}


@pytest.fixture(autouse=True)
def real_backend():
    from easy_gpt.cpp_amd import kernels

    kernels.use_backend(None)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    norm = make_part("norm", PartSpec("rmsnorm", dict(eps=3e-5), prefix="n."), hidden_size=200)
    w = weights_for(norm, dtype)
    h = torch.randn(6, 200, generator=torch.Generator().manual_seed(1)).to(DEV)
    delta = torch.randn(6, 200, generator=torch.Generator().manual_seed(2)).to(dtype).to(DEV)
    ref_h = (h + delta.float()).double().cpu()
    out = norm.forward(h, delta)
    ref = plain.rms_norm(ref_h, w["n.weight"], 3e-5)
    assert out.dtype == dtype and torch.equal(h.double().cpu(), ref_h)
    assert float((out.double().cpu() - ref).abs().max()) <= tol(dtype) * float(ref.abs().max())
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    out2 = norm.forward_rows(h, None, rows)
    assert float((out2.double().cpu() - ref[[4, 1]]).abs().max()) <= tol(dtype) * float(ref.abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_part(dtype):
    ff = make_part("feed_forward", PartSpec("swiglu", dict(intermediate_size=150), prefix="m."), hidden_size=72)
    w = weights_for(ff, dtype, scale=0.2)
    x = torch.randn(9, 72, generator=torch.Generator().manual_seed(3)).to(dtype)
    ref = plain.swiglu_mlp(x.double(), w, "m.")
    out = whole(ff.forward(x.to(DEV)))
    assert float((out.cpu() - ref).abs().max()) <= tol(dtype) * float(ref.abs().max())


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_output_head(dtype):
    emb = make_part("embedding", PartSpec("token_embedding", {}, prefix="e."), hidden_size=40, vocab_size=333)
    w = weights_for(emb, dtype, scale=1.0)
    ids = torch.tensor([0, 332, 7], dtype=torch.int32, device=DEV)
    # the embedding's output is the step's residual stream: float32, or for few tokens in bfloat16 the 64-bit fixed
    # point (units of 2^-32) that products add themselves into; for many tokens float32 in either precision
    from types import SimpleNamespace

    stream = emb.forward(SimpleNamespace(token_ids=ids))
    assert stream.dtype == (torch.int64 if dtype == torch.bfloat16 else torch.float32)
    values = stream.double().cpu() / (2.0 ** 32 if stream.dtype == torch.int64 else 1.0)
    assert torch.equal(values, w["e.weight"][[0, 332, 7]])
    many = torch.arange(40, dtype=torch.int32, device=DEV)
    assert emb.forward(SimpleNamespace(token_ids=many)).dtype == torch.float32
    assert torch.equal(emb.forward(SimpleNamespace(token_ids=many)).double().cpu(), w["e.weight"][:40])
    for tied in (True, False):
        head = make_part("output_head", PartSpec("linear_head", dict(tied=tied), prefix="o."), hidden_size=40, vocab_size=333)
        wh = weights_for(head, dtype, seed=5, scale=1.0)
        assert (len(head.param_specs()) == 0) == tied
        if tied:
            head.tie(emb.output_matrix())
        x = torch.randn(4, 40, generator=torch.Generator().manual_seed(6)).to(dtype)
        ref = plain.linear(x.double(), w["e.weight"] if tied else wh["o.weight"])
        out = head.forward(x.to(DEV))
        assert out.dtype == torch.float32
        assert float((out.double().cpu() - ref).abs().max()) <= (5e-6 if dtype == torch.float32 else 4e-3) * float(ref.abs().max())


def attention_setup(dtype, nq, nkv, hd, hidden, window, bias, theta, seed=0):
    att = make_part(
        "mixer",
        PartSpec("gq_attention", dict(n_heads=nq, n_kv_heads=nkv, head_dim=hd, qkv_bias=bias, out_bias=False, window=window,
                                      position=PartSpec("rope_half_split", dict(theta=theta))), prefix="a."),
        hidden_size=hidden,
    )
    w = weights_for(att, dtype, seed=seed, scale=0.15)
    return att, w


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,hd,hidden,window,bias,theta",
                         [(4, 2, 16, 64, None, True, 1e4), (3, 1, 32, 96, None, True, 1e6), (6, 3, 48, 120, 9, False, 5e4),
                          (5, 5, 80, 200, None, True, 1e6)])
def test_attention_part_whole_and_cut(dtype, nq, nkv, hd, hidden, window, bias, theta):
    att, w = attention_setup(dtype, nq, nkv, hd, hidden, window, bias, theta)
    s, ps = 45, 4
    x = torch.randn(s, hidden, generator=torch.Generator().manual_seed(7)).to(dtype)
    cfg = dict(num_attention_heads=nq, num_key_value_heads=nkv, head_dim=hd, hidden_size=hidden, rope_theta=theta)
    ref = plain.self_attention_block(x.double(), w, "a.", cfg, torch.arange(s), window)
    n_pages = 16
    kc = torch.zeros(n_pages, nkv, ps, hd, dtype=dtype, device=DEV)
    vc = torch.zeros(n_pages, nkv, hd, ps, dtype=dtype, device=DEV)
    table = torch.randperm(n_pages, generator=torch.Generator().manual_seed(8)).to(torch.int32)[None, :12].contiguous().to(DEV)
    outs, pos = [], 0
    for n in (20, 1, 2, 22):                      # a prompt portion, a decoded token, two more portions
        positions = torch.arange(pos, pos + n, dtype=torch.int32, device=DEV)
        slots = (table[0, (positions // ps).long()] * ps + positions % ps).to(torch.int32)
        one = lambda v: torch.tensor([v], dtype=torch.int32, device=DEV)
        ctx = SimpleNamespace(positions=positions, q_start=one(0), q_len=one(n), kv_len=one(pos + n), max_q_len=n,
                              max_kv_len=pos + n, shared={}, rows_independent=True)
        cache = CacheView({"k": kc, "v": vc}, ps, table, slots, window, True)
        outs.append(whole(att.forward(x[pos : pos + n].to(DEV), ctx, cache, None)))
        pos += n
    out = torch.cat(outs).cpu()
    assert float((out - ref).abs().max()) <= tol(dtype) * float(ref.abs().max())
    # a reader of the same cache that does not write (another layer's cache): same result for the last portion
    cache_ro = CacheView({"k": kc, "v": vc}, ps, table, slots, window, False)
    kc_before = kc.clone()
    again = whole(att.forward(x[pos - n : pos].to(DEV), ctx, cache_ro, None))
    assert torch.equal(kc, kc_before) and torch.equal(again, outs[-1])


@pytest.mark.parametrize("dtype", DTYPES)
def test_pre_norm_block(dtype):
    from easy_gpt.cpp_amd.parts import BLOCKS

    hidden, nq, nkv, hd, inter, eps = 96, 3, 1, 32, 130, 1e-5
    att, wa = attention_setup(dtype, nq, nkv, hd, hidden, None, True, 1e6, seed=1)
    ff = make_part("feed_forward", PartSpec("swiglu", dict(intermediate_size=inter), prefix="m."), hidden_size=hidden)
    n1 = make_part("norm", PartSpec("rmsnorm", dict(eps=eps), prefix="n1."), hidden_size=hidden)
    n2 = make_part("norm", PartSpec("rmsnorm", dict(eps=eps), prefix="n2."), hidden_size=hidden)
    w = dict(wa)
    w.update(weights_for(ff, dtype, 2, 0.2))
    w.update(weights_for(n1, dtype, 3))
    w.update(weights_for(n2, dtype, 4))
    block = BLOCKS["pre_norm"](att, ff, {"mixer": n1, "feed_forward": n2})
    s, ps = 19, 8
    x = torch.randn(s, hidden, generator=torch.Generator().manual_seed(9))
    # plain: a = x + Attn(N1 x); y = a + MLP(N2 a)   (/root/reference/src/models/block.cpp:23-29)
    cfg = dict(num_attention_heads=nq, num_key_value_heads=nkv, head_dim=hd, hidden_size=hidden, rope_theta=1e6)
    xd = x.double()
    a = xd + plain.self_attention_block(plain.rms_norm(xd, w["n1.weight"], eps), w, "a.", cfg, torch.arange(s))
    y = a + plain.swiglu_mlp(plain.rms_norm(a, w["n2.weight"], eps), w, "m.")
    kc = torch.zeros(3, nkv, ps, hd, dtype=dtype, device=DEV)
    vc = torch.zeros(3, nkv, hd, ps, dtype=dtype, device=DEV)
    table = torch.tensor([[2, 0, 1]], dtype=torch.int32, device=DEV)
    positions = torch.arange(s, dtype=torch.int32, device=DEV)
    slots = (table[0, (positions // ps).long()] * ps + positions % ps).to(torch.int32)
    one = lambda v: torch.tensor([v], dtype=torch.int32, device=DEV)
    ctx = SimpleNamespace(positions=positions, q_start=one(0), q_len=one(s), kv_len=one(s), max_q_len=s, max_kv_len=s, shared={},
                          rows_independent=True)
    h, delta = block.forward(x.to(DEV).clone(), None, ctx, CacheView({"k": kc, "v": vc}, ps, table, slots, None, True), None)
    got = h.double().cpu() + whole(delta).cpu()
    assert float((h.double().cpu() - a).abs().max()) <= tol(dtype) * float(a.abs().max())
    assert float((got - y).abs().max()) <= tol(dtype) * float(y.abs().max())
