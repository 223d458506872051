"""Generality of a layer's shape: arrangements, caches and states that the built-in model does not have, defined
here and run without a change to the framework's files.

  * a block arrangement with four norms (one before and one after each branch) and one with a mixer only and
    a single norm;
  * a mixer whose paged cache is not keys and values: one float32 tensor of latents per token, kept for a
    window (a page pool of its own beside attention's, pages given back behind the window);
  * a mixer with per-request state that is graph-safe (it reads the state's slots and freshness from device
    memory), so that its decode steps replay from captured graphs, padding rows included;
  * a weight whose random values come from a distribution registered here (a decay within (0, 1));
  * an embedding that adds a learned vector per position to the token's (it is handed the step context, so it finds
    the positions there) and shares its token matrix with a tied output head;
  * a norm that the backend has no kernel for (a layer norm with mean and bias), which reads and adds to the residual
    stream through the backend whichever way the stream is kept, also inside replayed graphs.
The toy parts compute with torch on the GPU; they are test equipment, not a model of anyone's."""
import os
from dataclasses import dataclass

import pytest
import torch

import helpers as H
import plain_qwen2 as plain
from easy_gpt.cpp_amd.config import Architecture, register_architecture, unregister_architecture
from easy_gpt.cpp_amd import kernels
from easy_gpt.cpp_amd.parts import (
    Block, CacheNeed, Embedding, LayerSpec, Mixer, ModelSpec, Norm, PagedTensor, ParamSpec, PartSpec, RunSpec, StateNeed, register_part,
)
from easy_gpt.cpp_amd.parts.base import BLOCKS, MIXERS, NORMS
from easy_gpt.cpp_amd.weights import random_init, register_role

pytestmark = pytest.mark.gpu


# --------------------------------------------------------------------------- toy arrangements
class SandwichBlock(Block):
    """a = h + Npost_m(Mixer(Npre_m(h))); y = a + Npost_f(FF(Npre_f(a))): a norm before and after each branch."""

    norm_slots = ("pre_mixer", "post_mixer", "pre_feed_forward", "post_feed_forward")

    def forward(self, h, delta, ctx, cache, state):
        zeros = lambda: torch.zeros(h.shape, dtype=torch.float32, device=h.device)
        x = self.norms["pre_mixer"].forward(h, delta)                        # h += delta
        a = self.mixer.forward(x, ctx, cache, state)                         # act, or partial sums: the norm adds either
        a = self.norms["post_mixer"].forward(zeros(), a)
        x = self.norms["pre_feed_forward"].forward(h, a)                     # h += a
        m = self.feed_forward.forward(x, ctx)
        return h, self.norms["post_feed_forward"].forward(zeros(), m)


class MixerOnlyBlock(Block):
    """y = h + Mixer(N(h)): no feed-forward."""

    norm_slots = ("mixer",)
    uses_feed_forward = False

    def forward(self, h, delta, ctx, cache, state):
        x = self.norms["mixer"].forward(h, delta)
        return h, self.mixer.forward(x, ctx, cache, state)


# --------------------------------------------------------------------------- a cache that is not keys and values
class LatentMeanMixer(Mixer):
    """z_t = x_t Win^T is kept per token (float32, one paged tensor); out_t = mean(z over the last W tokens) Wout^T."""

    def __init__(self, prefix, hidden_size, latent_size, window):
        self.prefix, self.hidden_size, self.latent_size, self.window = prefix, hidden_size, int(latent_size), int(window)

    def cache_need(self):
        return CacheNeed((PagedTensor("latent", (self.latent_size,), 0, dtype="float32"),), self.window)

    def param_specs(self):
        return [ParamSpec(self.prefix + "in.weight", (self.latent_size, self.hidden_size)),
                ParamSpec(self.prefix + "out.weight", (self.hidden_size, self.latent_size))]

    def load(self, get, dtype, device):
        self.w_in = self._to(get(self.prefix + "in.weight"), "compute", dtype, device)
        self.w_out = self._to(get(self.prefix + "out.weight"), "compute", dtype, device)

    def forward(self, x, ctx, cache, state):
        assert state is None and set(cache.tensors) == {"latent"} and cache.window == self.window
        store = cache.tensors["latent"]
        assert store.dtype == torch.float32 and tuple(store.shape[1:]) == (cache.page_size, self.latent_size)
        flat = store.view(-1, self.latent_size)
        z = x.float() @ self.w_in.float().T
        flat[cache.slots.long()] = z
        ps = cache.page_size
        means = torch.empty_like(z)
        for b, (start, n, kv) in enumerate(zip(ctx.q_start_host, ctx.q_len_host, ctx.kv_len_host)):
            table = cache.block_table[b]
            for i in range(n):
                p = kv - n + i
                pos = torch.arange(max(0, p - self.window + 1), p + 1, device=x.device)
                pages = table[(pos // ps).long()].long()
                assert int(pages.min()) >= 0                  # nothing within the window was given back
                means[start + i] = flat[pages * ps + pos % ps].mean(0)
        return (means @ self.w_out.float().T).to(x.dtype)


def latent_mean_plain(xn, w_in, w_out, window):
    z = xn @ w_in.T
    means = torch.stack([z[max(0, t - window + 1) : t + 1].mean(0) for t in range(z.shape[0])])
    return means @ w_out.T


# --------------------------------------------------------------------------- a state that replays from graphs
class ChannelDecayMixer(Mixer):
    """s_t = r * s_{t-1} + x_t W^T with a learned decay r per channel; out_t = s_t.  Decode steps read the state's
    slots and freshness from device memory only."""

    graph_safe = True

    def __init__(self, prefix, hidden_size):
        self.prefix, self.hidden_size = prefix, hidden_size

    def state_need(self):
        return StateNeed((self.hidden_size,), torch.float32)

    def param_specs(self):
        return [ParamSpec(self.prefix + "w.weight", (self.hidden_size, self.hidden_size)),
                ParamSpec(self.prefix + "rate", (self.hidden_size,), role="toy_decay_rate", dtype="float32")]

    def load(self, get, dtype, device):
        self.w = self._to(get(self.prefix + "w.weight"), "compute", dtype, device)
        self.rate = self._to(get(self.prefix + "rate"), "float32", dtype, device)

    def forward(self, x, ctx, cache, state):
        u = x.float() @ self.w.float().T
        if ctx.max_q_len == 1:                               # one token per request: no host value is read
            slots = state.slots.long()
            s = state.data[slots]
            s = torch.where(state.fresh_device[:, None], torch.zeros_like(s), s) * self.rate + u
            state.data[slots] = s
            return s.to(x.dtype)
        out = torch.empty_like(u)                            # a portion is walked in order (never captured)
        for b, (start, n) in enumerate(zip(ctx.q_start_host, ctx.q_len_host)):
            slot = state.slots_host[b]
            s = torch.zeros(self.hidden_size, device=x.device) if state.fresh[b] else state.data[slot].clone()
            for i in range(start, start + n):
                s = self.rate * s + u[i]
                out[i] = s
            state.data[slot] = s
        return out.to(x.dtype)


def channel_decay_plain(xn, w, rate):
    u = xn @ w.T
    s, outs = torch.zeros_like(u[0]), []
    for t in range(u.shape[0]):
        s = rate * s + u[t]
        outs.append(s)
    return torch.stack(outs)


# --------------------------------------------------------------------------- a norm of another kind
class MeanVarianceNorm(Norm):
    """y = (x - mean(x)) / sqrt(var(x) + eps) * w + b, computed in float32."""

    graph_safe = True

    def __init__(self, prefix, hidden_size, eps):
        self.prefix, self.hidden_size, self.eps = prefix, hidden_size, float(eps)

    def param_specs(self):
        return [ParamSpec(self.prefix + "weight", (self.hidden_size,), role="norm_scale"),
                ParamSpec(self.prefix + "bias", (self.hidden_size,), role="bias")]

    def load(self, get, dtype, device):
        self.w = self._to(get(self.prefix + "weight"), "compute", dtype, device)
        self.b = self._to(get(self.prefix + "bias"), "compute", dtype, device)

    def _norm(self, x):
        x = x - x.mean(-1, keepdim=True)
        y = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + self.eps) * self.w.float() + self.b.float()
        return y.to(self.w.dtype)

    def forward(self, h, delta):
        k = kernels.backend()
        if delta is not None:
            k.residual_add(h, delta)
        return self._norm(k.residual_values(h))

    def forward_rows(self, h, delta, rows):
        x = kernels.backend().residual_values(h)[rows.long()]
        if delta is not None:
            x = x + (delta.sum(0) if delta.dim() == 3 else delta.float())[rows.long()]
        return self._norm(x)


def mean_variance_norm_plain(x, w, b, eps):
    x = x - x.mean(-1, keepdim=True)
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w + b


# --------------------------------------------------------------------------- two toy architectures
@dataclass
class ShapesConfig:
    hidden_size: int
    vocab_size: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    intermediate_size: int
    latent_size: int
    latent_window: int
    eps_pre: float
    eps_post: float
    rope_theta: float
    max_position_embeddings: int

    @classmethod
    def from_dict(cls, d, where="config.json"):
        return cls(**{k: d[k] for k in cls.__dataclass_fields__})


def attention_spec(c, prefix):
    return PartSpec("gq_attention", dict(n_heads=c.n_heads, n_kv_heads=c.n_kv_heads, head_dim=c.head_dim, qkv_bias=True,
                                         out_bias=False, window=None,
                                         position=PartSpec("rope_half_split", dict(theta=c.rope_theta))), prefix)


def shapes_spec(c: ShapesConfig) -> ModelSpec:
    pre = lambda p: PartSpec("rmsnorm", dict(eps=c.eps_pre), prefix=p)
    post = lambda p: PartSpec("rmsnorm", dict(eps=c.eps_post), prefix=p)
    layers = (
        LayerSpec("toy_sandwich", attention_spec(c, "l0.attn."),
                  PartSpec("swiglu", dict(intermediate_size=c.intermediate_size), "l0.ff."),
                  {"pre_mixer": pre("l0.pre_m."), "post_mixer": post("l0.post_m."),
                   "pre_feed_forward": pre("l0.pre_f."), "post_feed_forward": post("l0.post_f.")}),
        LayerSpec("toy_mixer_only", PartSpec("toy_latent_mean", dict(latent_size=c.latent_size, window=c.latent_window), "l1.mix."),
                  None, {"mixer": pre("l1.n.")}),
    )
    return ModelSpec(
        hidden_size=c.hidden_size, vocab_size=c.vocab_size, max_position=c.max_position_embeddings,
        embedding=PartSpec("token_embedding", {}, "emb."), layers=layers,
        run_order=(RunSpec(0, cache=0), RunSpec(1, cache=1), RunSpec(0, cache=2)),      # the sandwich layer runs twice
        final_norm=pre("final."), output_head=PartSpec("linear_head", dict(tied=True), "head."),
    )


SHAPES_CONFIG = {"architectures": ["ToyShapesForCausalLM"], "hidden_size": 40, "vocab_size": 157, "n_heads": 4, "n_kv_heads": 2,
                 "head_dim": 16, "intermediate_size": 88, "latent_size": 12, "latent_window": 7, "eps_pre": 1e-5,
                 "eps_post": 3e-4, "rope_theta": 1e4, "max_position_embeddings": 128}


def shapes_plain(w, cfg, ids):
    x = w["emb.weight"][torch.tensor(ids)]
    s = len(ids)
    acfg = dict(num_attention_heads=cfg["n_heads"], num_key_value_heads=cfg["n_kv_heads"], head_dim=cfg["head_dim"],
                hidden_size=cfg["hidden_size"], rope_theta=cfg["rope_theta"])
    ffw = {k[len("l0.ff."):]: v for k, v in w.items() if k.startswith("l0.ff.")}

    def sandwich(x):
        a = plain.self_attention_block(plain.rms_norm(x, w["l0.pre_m.weight"], cfg["eps_pre"]), w, "l0.attn.", acfg, torch.arange(s))
        x = x + plain.rms_norm(a, w["l0.post_m.weight"], cfg["eps_post"])
        m = plain.swiglu_mlp(plain.rms_norm(x, w["l0.pre_f.weight"], cfg["eps_pre"]), ffw, "")
        return x + plain.rms_norm(m, w["l0.post_f.weight"], cfg["eps_post"])

    x = sandwich(x)
    x = x + latent_mean_plain(plain.rms_norm(x, w["l1.n.weight"], cfg["eps_pre"]), w["l1.mix.in.weight"], w["l1.mix.out.weight"],
                              cfg["latent_window"])
    x = sandwich(x)
    return plain.linear(plain.rms_norm(x, w["final.weight"], cfg["eps_pre"]), w["emb.weight"])


@dataclass
class GraphStateConfig:
    hidden_size: int
    vocab_size: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    intermediate_size: int
    eps_pre: float
    rope_theta: float
    max_position_embeddings: int

    @classmethod
    def from_dict(cls, d, where="config.json"):
        return cls(**{k: d[k] for k in cls.__dataclass_fields__})


def graph_state_spec(c: GraphStateConfig) -> ModelSpec:
    norm = lambda p: PartSpec("rmsnorm", dict(eps=c.eps_pre), prefix=p)
    other = lambda p: PartSpec("toy_mean_variance", dict(eps=c.eps_pre), prefix=p)
    ff = lambda p: PartSpec("swiglu", dict(intermediate_size=c.intermediate_size), p)
    layers = (LayerSpec("pre_norm", PartSpec("toy_channel_decay", {}, "l0.mix."), ff("l0.ff."),
                        {"mixer": norm("l0.n1."), "feed_forward": norm("l0.n2.")}),
              LayerSpec("pre_norm", attention_spec(c, "l1.attn."), ff("l1.ff."),
                        {"mixer": other("l1.n1."), "feed_forward": other("l1.n2.")}))
    return ModelSpec(
        hidden_size=c.hidden_size, vocab_size=c.vocab_size, max_position=c.max_position_embeddings,
        embedding=PartSpec("token_embedding", {}, "emb."), layers=layers,
        run_order=(RunSpec(0, state=0), RunSpec(1, cache=0)),
        final_norm=other("final."), output_head=PartSpec("linear_head", dict(tied=False), "head."),
    )


GRAPH_STATE_CONFIG = {"architectures": ["ToyGraphStateForCausalLM"], "hidden_size": 48, "vocab_size": 131, "n_heads": 3,
                      "n_kv_heads": 1, "head_dim": 16, "intermediate_size": 72, "eps_pre": 1e-5, "rope_theta": 1e4,
                      "max_position_embeddings": 96}


def graph_state_plain(w, cfg, ids):
    x = w["emb.weight"][torch.tensor(ids)]
    s = len(ids)
    acfg = dict(num_attention_heads=cfg["n_heads"], num_key_value_heads=cfg["n_kv_heads"], head_dim=cfg["head_dim"],
                hidden_size=cfg["hidden_size"], rope_theta=cfg["rope_theta"])
    eps = cfg["eps_pre"]
    ffn = lambda x, p: plain.swiglu_mlp(x, {k[len(p):]: v for k, v in w.items() if k.startswith(p)}, "")
    x = x + channel_decay_plain(plain.rms_norm(x, w["l0.n1.weight"], eps), w["l0.mix.w.weight"], w["l0.mix.rate"])
    x = x + ffn(plain.rms_norm(x, w["l0.n2.weight"], eps), "l0.ff.")
    other = lambda x, p: mean_variance_norm_plain(x, w[p + "weight"], w[p + "bias"], eps)
    x = x + plain.self_attention_block(other(x, "l1.n1."), w, "l1.attn.", acfg, torch.arange(s))
    x = x + ffn(other(x, "l1.n2."), "l1.ff.")
    return plain.linear(other(x, "final."), w["head.weight"])


@pytest.fixture()
def toys_registered():
    register_part("block", "toy_sandwich", SandwichBlock)
    register_part("block", "toy_mixer_only", MixerOnlyBlock)
    register_part("mixer", "toy_latent_mean", LatentMeanMixer)
    register_part("mixer", "toy_channel_decay", ChannelDecayMixer)
    register_part("norm", "toy_mean_variance", MeanVarianceNorm)
    register_role("toy_decay_rate", lambda shape, g, device: 0.5 + 0.45 * torch.rand(shape, generator=g, device=device))
    register_architecture(Architecture("ToyShapesForCausalLM", ShapesConfig, shapes_spec, ("toyshapes",)))
    register_architecture(Architecture("ToyGraphStateForCausalLM", GraphStateConfig, graph_state_spec, ("toygraphstate",)))
    yield
    unregister_architecture("ToyShapesForCausalLM")
    unregister_architecture("ToyGraphStateForCausalLM")
    BLOCKS.pop("toy_sandwich")
    BLOCKS.pop("toy_mixer_only")
    MIXERS.pop("toy_latent_mean")
    MIXERS.pop("toy_channel_decay")
    NORMS.pop("toy_mean_variance")
    random_init.ROLES.pop("toy_decay_rate")


def weights_as_engine_sees_them(folder, dtype, keep_float32=()):
    w = plain.read_safetensors(os.path.join(folder, "model.safetensors"))
    if dtype == "bfloat16":
        w = {k: (v if k in keep_float32 else v.float().to(torch.bfloat16).double()) for k, v in w.items()}
    return w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_four_norms_a_mixer_alone_and_a_cache_of_latents(toys_registered, tmp_path, dtype):
    from easy_gpt.cpp_amd import kernels
    from easy_gpt.cpp_amd.engine import Engine
    from easy_gpt.cpp_amd.weights import write_random_model

    kernels.use_backend(None)
    d = write_random_model(str(tmp_path / "toy"), SHAPES_CONFIG, seed=11)
    eng = Engine.from_dir(d, dtype=dtype, device="cuda:0", page_size=4, num_pages=40, max_requests=3)
    model = eng.model
    assert [type(b).__name__ for b in model.layers] == ["SandwichBlock", "MixerOnlyBlock"]
    assert len(model.layers[0].parts()) == 6 and len(model.layers[1].parts()) == 2
    # two page pools: keys and values of the two runs of the sandwich layer; the latents with their window
    groups = {g.cache_ids: g.need for g in model.cache_groups}
    assert set(groups) == {(0, 2), (1,)} and groups[(1,)].window == 7 and groups[(0, 2)].window is None
    g_lat = [i for i, g in enumerate(model.cache_groups) if g.cache_ids == (1,)][0]
    assert set(eng.kv.tensors[g_lat]) == {"latent"} and eng.kv.tensors[g_lat]["latent"].dtype == torch.float32
    assert set(eng.kv.tensors[1 - g_lat]) == {"k", "v"}
    w = weights_as_engine_sees_them(d, dtype)
    reqs = H.make_requests(SHAPES_CONFIG["vocab_size"], [37, 9, 70, 26], seed=6)
    ref = {rid: shapes_plain(w, SHAPES_CONFIG, ids) for rid, ids in reqs.items()}
    tol = 3e-5 if dtype == "float32" else 3e-2
    for trace in (H.trace_whole(reqs), H.trace_portions(reqs), H.trace_mixed(reqs, seed=4, max_live=3, decode_tail=8)):
        rows = H.replay(eng, trace)
        assert len(rows) == sum(len(v) for v in reqs.values())
        H.assert_rows_match(rows, ref, tol, f"toy shapes {dtype}")
    assert eng.cache.free_pages() == [40, 40]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_graph_safe_state_replays_from_graphs(toys_registered, tmp_path, dtype):
    from easy_gpt.cpp_amd import kernels
    from easy_gpt.cpp_amd.engine import Engine, StepEntry
    from easy_gpt.cpp_amd.weights import write_random_model

    kernels.use_backend(None)
    d = write_random_model(str(tmp_path / "toy"), GRAPH_STATE_CONFIG, seed=12)
    rate = plain.read_safetensors(os.path.join(d, "model.safetensors"))["l0.mix.rate"]
    assert rate.dtype == torch.float64 and 0.5 <= float(rate.min()) and float(rate.max()) < 0.95    # the registered role
    n_req = 20                                              # beyond 16, decode batches are padded to a multiple of 8
    eng = Engine.from_dir(d, dtype=dtype, device="cuda:0", page_size=4, max_tokens=n_req * 64, max_requests=n_req)
    assert eng.use_graphs and eng.model.graph_safe and list(eng.model.state_needs) == [0]
    assert eng.states.data[0].shape == (n_req + 1, 48) and eng.states.pad_slot == n_req
    w = weights_as_engine_sees_them(d, dtype, keep_float32=("l0.mix.rate",))
    lengths = [12 + (5 * i) % 17 for i in range(n_req)]
    lengths[3] = 1                                          # a request whose first token is already a decode-shaped step
    reqs = H.make_requests(GRAPH_STATE_CONFIG["vocab_size"], [n + 10 for n in lengths], seed=8)
    ref = {rid: graph_state_plain(w, GRAPH_STATE_CONFIG, ids) for rid, ids in reqs.items()}
    tol = 3e-5 if dtype == "float32" else 3e-2
    rows = {}
    rids = list(reqs)
    for rid, n in zip(rids, lengths):                       # the prompts: one step each (the one-token prompt from a graph)
        eng.add_request(rid)
        out = eng.step([StepEntry(rid, reqs[rid][:n], [n - 1])])
        rows[(rid, n - 1)] = out[0].float().cpu()
    for t in range(10):                                     # ten decode steps of all twenty, then of the first three
        live = rids if t < 6 else rids[:3]
        out = eng.step([StepEntry(rid, [reqs[rid][n + t]], [0]) for rid, n in zip(live, lengths)]).float().cpu()
        for i, (rid, n) in enumerate(zip(live, lengths)):
            rows[(rid, n + t)] = out[i].clone()
    H.assert_rows_match(rows, ref, tol, f"toy graph state {dtype}")
    plans = eng._decode_plans
    assert {key[0] for key in plans} >= {24, 3, 1} and all(p.graph is not None for key, p in plans.items() if key[0] in (24, 3))
    # the padding rows wrote the record that belongs to no request, and only that one beyond the requests' own
    assert float(eng.states.data[0][n_req].abs().max()) > 0


# --------------------------------------------------------------------------- an embedding that looks at positions
class PositionalEmbedding(Embedding):
    """x_t = E[id_t] + P[position_t]; the output head may tie itself to E."""

    graph_safe = True

    def __init__(self, prefix, hidden_size, vocab_size, max_position):
        self.prefix, self.hidden_size, self.vocab_size, self.max_position = prefix, hidden_size, vocab_size, max_position

    def param_specs(self):
        return [ParamSpec(self.prefix + "tokens.weight", (self.vocab_size, self.hidden_size), role="embedding"),
                ParamSpec(self.prefix + "positions.weight", (self.max_position, self.hidden_size), role="embedding")]

    def load(self, get, dtype, device):
        self.tokens = self._to(get(self.prefix + "tokens.weight"), "compute", dtype, device)
        self.positions = self._to(get(self.prefix + "positions.weight"), "compute", dtype, device)

    def output_matrix(self):
        return self.tokens

    def forward(self, ctx):
        k = kernels.backend()
        t = ctx.token_ids.shape[0]
        out = torch.empty((t, self.hidden_size), device=ctx.token_ids.device, dtype=k.residual_dtype(t, self.tokens.dtype))
        k.embed(ctx.token_ids, self.tokens, out)
        k.residual_add(out, self.positions.index_select(0, ctx.positions.long()))
        return out


@dataclass
class PosConfig:
    hidden_size: int
    vocab_size: int
    max_position_embeddings: int
    eps: float

    @classmethod
    def from_dict(cls, d, where="config.json"):
        return cls(**{k: d[k] for k in cls.__dataclass_fields__})


def pos_spec(c: PosConfig) -> ModelSpec:
    norm = lambda p: PartSpec("rmsnorm", dict(eps=c.eps), prefix=p)
    attn = PartSpec("gq_attention", dict(n_heads=2, n_kv_heads=1, head_dim=16, qkv_bias=True, out_bias=False, window=None,
                                         position=PartSpec("none", {})), "l0.attn.")
    layer = LayerSpec("pre_norm", attn, PartSpec("swiglu", dict(intermediate_size=72), prefix="l0.ff."),
                      {"mixer": norm("l0.n1."), "feed_forward": norm("l0.n2.")})
    return ModelSpec(hidden_size=c.hidden_size, vocab_size=c.vocab_size, max_position=c.max_position_embeddings,
                     embedding=PartSpec("toy_positional", dict(max_position=c.max_position_embeddings), "emb."),
                     layers=(layer,), run_order=(RunSpec(0, cache=0),), final_norm=norm("final."),
                     output_head=PartSpec("linear_head", dict(tied=True), "head."))


POS_CONFIG = {"architectures": ["ToyPositionalForCausalLM"], "hidden_size": 40, "vocab_size": 97,
              "max_position_embeddings": 80, "eps": 1e-5}


def pos_plain(w, cfg, ids):
    s = len(ids)
    x = w["emb.tokens.weight"][torch.tensor(ids)] + w["emb.positions.weight"][:s]
    xn = plain.rms_norm(x, w["l0.n1.weight"], cfg["eps"])
    p = "l0.attn."
    q = plain.linear(xn, w[p + "q_proj.weight"], w[p + "q_proj.bias"]).reshape(s, 2, 16)
    k = plain.linear(xn, w[p + "k_proj.weight"], w[p + "k_proj.bias"]).reshape(s, 1, 16)
    v = plain.linear(xn, w[p + "v_proj.weight"], w[p + "v_proj.bias"]).reshape(s, 1, 16)
    x = x + plain.linear(plain.attention(q, k, v, 2, 1).reshape(s, 32), w[p + "o_proj.weight"])
    x = x + plain.swiglu_mlp(plain.rms_norm(x, w["l0.n2.weight"], cfg["eps"]), w, "l0.ff.")
    return plain.linear(plain.rms_norm(x, w["final.weight"], cfg["eps"]), w["emb.tokens.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_an_embedding_that_reads_positions_and_ties_the_output_head(tmp_path, dtype):
    # without position encoding in the attention, the logits depend on positions through the embedding alone: tokens
    # decoded one by one (from graphs) and in portions must get the positions they stand at
    from easy_gpt.cpp_amd.engine import Engine
    from easy_gpt.cpp_amd.parts.base import EMBEDDINGS
    from easy_gpt.cpp_amd.weights import write_random_model

    kernels.use_backend(None)
    register_part("embedding", "toy_positional", PositionalEmbedding)
    register_architecture(Architecture("ToyPositionalForCausalLM", PosConfig, pos_spec, ("toypos",)))
    try:
        d = write_random_model(str(tmp_path / "pos"), POS_CONFIG, seed=6)
        eng = Engine.from_dir(d, dtype=dtype, device="cuda:0", page_size=16, max_tokens=256, max_requests=4)
        assert eng.model.output_head.weight is eng.model.embedding.tokens and eng.model.graph_safe
        w = plain.read_safetensors(os.path.join(d, "model.safetensors"))
        if dtype == "bfloat16":
            w = {k: v.float().to(torch.bfloat16).double() for k, v in w.items()}
        reqs = H.make_requests(POS_CONFIG["vocab_size"], [50, 9, 70], seed=7)
        ref = {rid: pos_plain(w, POS_CONFIG, ids) for rid, ids in reqs.items()}
        shifted = pos_plain(w, POS_CONFIG, [0] + reqs["r1"])[1:]                 # the same tokens one place further on
        assert float((shifted - ref["r1"]).abs().max()) > 1e-3 * float(ref["r1"].abs().max())
        tol = H.FP32_TOL if dtype == "float32" else H.BF16_TOL_RANDOM
        for trace in (H.trace_whole(reqs), H.trace_last_decoded(reqs, 32), H.trace_mixed(reqs, seed=5, max_live=3)):
            H.assert_rows_match(H.replay(eng, trace), ref, tol, f"positional embedding {dtype}")
        assert any(p.graph is not None for p in eng._decode_plans.values())
    finally:
        unregister_architecture("ToyPositionalForCausalLM")
        EMBEDDINGS.pop("toy_positional")
