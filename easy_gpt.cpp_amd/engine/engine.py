"""The engine: a loaded model, its cache, and the one step function.

`step` takes a batch of (request, its next tokens): portions of prompts beside
single decoded tokens, cut anywhere.  It runs only those tokens, as one batch,
against what earlier steps left in the cache, and returns float32 logits at the
wanted places.  The reference has two separate rectangular calls for this
(/root/reference/src/models/gpt_model.cpp:375-419: sample_prefill_continuous and
sample_decode_continuous, positions as offsets -pad_len / pos_len from
/root/reference/src/models/generation_invariants.cpp:25-51); here positions are
the true positions and nothing is padded.
"""
from __future__ import annotations

import sys
from dataclasses import dataclass, field
from typing import Sequence

import numpy as np
import torch

from ..cache.manager import _ints
from ..cache import CacheManager, PagedStorage, RequestCache, StateStorage
from ..config.registry import load_model_config
from ..parts.model import Model, build_model
from ..weights.loader import CheckedWeights
from .context import GroupTables, StepContext

DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32,
}


@dataclass
class StepEntry:
    """The next tokens of one request and the places among them whose logits are wanted."""

    request_id: object
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=tuple)


def load_model(model_dir: str, dtype="bfloat16", device="cuda:0", allow_unexpected_tensors: bool = False) -> Model:
    """Model folder -> model on the device: config.json picks the architecture, the weights
    are checked by name and shape and then taken by the parts.  A tensor that the model does not
    declare is an error, listed with the missing and misshapen ones; allow_unexpected_tensors=True only
    warns about it, as the reference does (/root/reference/src/models/model_param_validation.cpp:198-218)."""
    arch, cfg = load_model_config(model_dir)
    spec = arch.build_spec(cfg)
    model = build_model(spec)
    weights = CheckedWeights(model_dir, model.param_specs(), spec.ignorable_tensors, allow_unexpected_tensors)
    try:
        for name in weights.ignored:
            print(f"[weights] tensor '{name}' is not used by this model and was ignored", file=sys.stderr, flush=True)
        torch_dtype = DTYPES[dtype] if isinstance(dtype, str) else dtype
        model.load(weights.get, torch_dtype, torch.device(device))
    finally:
        weights.close()
    model.config = cfg
    return model


def load_random_model(config: dict, seed: int, dtype="bfloat16", device="cuda:0") -> Model:
    """A model with the random weights that `weights.write_random_model(folder, config, seed)` would write, drawn on
    the device and taken by the parts without a file in between (the values are the file's: a tensor's elements are
    a function of seed, tensor name and index).  `config` is a config.json mapping."""
    from ..config.registry import resolve_architecture
    from ..weights.random_init import RandomWeights

    arch = resolve_architecture(config)
    cfg = arch.config_class.from_dict(config, where="config")
    model = build_model(arch.build_spec(cfg))
    torch_dtype = DTYPES[dtype] if isinstance(dtype, str) else dtype
    stored = torch.bfloat16 if torch_dtype == torch.bfloat16 else torch.float32
    model.load(RandomWeights(model.param_specs(), seed, stored, device).get, torch_dtype, torch.device(device))
    model.config = cfg
    return model


class Engine:
    PAD_TO = 64          # steps that run from a padded graph are padded to a multiple of this many tokens

    def __init__(
        self,
        model: Model,
        *,
        page_size: int = 16,
        max_tokens: int | None = None,
        num_pages: int | None = None,
        max_requests: int = 64,
        use_graphs: bool = True,
        tune_products: bool = False,
    ):
        """max_tokens: the most tokens live requests hold at any time (each request's count
        rounded up to a page); the pools are made for that many.  num_pages sets the page
        count directly.  tune_products: the library's many-row products are chosen by measurement at a shape's
        first visit (`kernels.tune_library_products`: process-wide, about a second per new shape)."""
        if model.device is None:
            raise RuntimeError("the model has no weights yet (Model.load)")
        self.model = model
        self.device = model.device
        if tune_products and self.device.type == "cuda":
            from .. import kernels

            try:
                kernels.tune_library_products(True)
            except Exception as e:       # the products then stay the library's first choice, which is always right
                import warnings

                warnings.warn(f"the library's products cannot be chosen by measurement here: {e}")
        self.page_size = int(page_size)
        if num_pages is None:
            if max_tokens is None:
                raise ValueError("give max_tokens or num_pages")
            num_pages = -(-int(max_tokens) // self.page_size)
        groups = [g.need for g in model.cache_groups]
        self.cache = CacheManager(groups, self.page_size, int(num_pages), max_requests)
        # Beyond the pages that the manager hands out, a few that no request ever gets: where the padding tokens of
        # a step that runs from a padded graph (`_step_padded`) put their keys and values.
        self._pad_first_page = int(num_pages)
        self._pad_pages = -(-(self.PAD_TO - 1) // self.page_size)
        self.kv = PagedStorage(
            groups, [len(g.cache_ids) for g in model.cache_groups], [num_pages + self._pad_pages] * len(groups),
            self.page_size, model.dtype, self.device,
        )
        self.states = StateStorage(model.state_needs, max_requests, self.device)
        self.vocab_size = model.spec.vocab_size
        self.max_position = model.spec.max_position
        # steps that hold one token per request are replayed from captured device graphs
        self.use_graphs = bool(use_graphs) and self.device.type == "cuda" and model.graph_safe
        self._decode_plans: dict = {}
        self._row_plans: dict = {}
        self._padded_plans: dict = {}
        self.graph_tokens = 2048    # steps of at most this many tokens run from a graph for their padded size
        self.capture_after = 1      # a shape's graph is captured right after this visit (None: never, the same kernels one by one)
        self.graph_rows = 64        # steps of at most this many tokens in all run as rows of one token each,
        self.graph_row_reads = 1 << 18      # if the tokens of their portions read at most this many keys in all
        self._graph_pool = None
        self._has_windows = any(g.window is not None for g in groups)

    @classmethod
    def from_dir(cls, model_dir: str, dtype="bfloat16", device="cuda:0", allow_unexpected_tensors: bool = False,
                 **kw) -> "Engine":
        return cls(load_model(model_dir, dtype, device, allow_unexpected_tensors), **kw)

    # ------------------------------------------------------------------ requests
    def add_request(self, request_id) -> RequestCache:
        rc = self.cache.admit(request_id)
        self.states.reset(rc.slot)
        return rc

    def finish(self, request_id) -> None:
        self.cache.release(self.cache.requests[request_id])

    def has_request(self, request_id) -> bool:
        return request_id in self.cache.requests

    # ------------------------------------------------------------------ the step
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor | None:
        """Run one batch.  Returns float32 logits [wanted, vocab] in the order of the entries and
        of each entry's `want`, or None if nothing is wanted.  Raises OutOfPages (with the cache
        unchanged) if the tokens do not fit.  The returned tensor may be overwritten by the next
        call of `step`: use it (or copy it) before stepping again."""
        entries = [e for e in entries if len(e.tokens) > 0]
        if not entries:
            return None
        if self.use_graphs and all(len(e.tokens) == 1 and len(e.want) == 1 for e in entries):
            return self._step_decode(entries)
        if self.use_graphs and not self.model.state_needs and sum(len(e.tokens) for e in entries) <= self.graph_rows:
            # (as rows of one token, every token of a portion reads its request's keys for itself: not behind a
            # context so long that this outweighs what the graph saves)
            requests = self.cache.requests
            reads = sum(len(e.tokens) * (requests[e.request_id].num_tokens + len(e.tokens))
                        for e in entries if len(e.tokens) > 1 and e.request_id in requests)
            if reads <= self.graph_row_reads:
                return self._step_rows(entries)
        if self.use_graphs and not self.model.state_needs and sum(len(e.tokens) for e in entries) <= self.graph_tokens:
            return self._step_padded(entries)
        rcs = self._check(entries)
        counts = [len(e.tokens) for e in entries]
        with self.cache.reserved(rcs, counts):             # all of the step's pages or none; given back if it fails
            ctx = self._build_context(rcs, entries)
            logits = self.model.forward(ctx)
        return logits

    def _check(self, entries) -> list[RequestCache]:
        rcs, seen = [], set()
        for e in entries:
            if e.request_id in seen:
                raise ValueError(f"request {e.request_id!r} appears twice in one step")
            seen.add(e.request_id)
            if e.request_id not in self.cache.requests:
                raise KeyError(f"request {e.request_id!r} is not live (add_request first)")
            rc = self.cache.requests[e.request_id]
            n = len(e.tokens)
            ids = np.asarray(e.tokens, dtype=np.int64)          # one pass in C instead of a Python loop per token
            if ids.ndim != 1:
                raise ValueError(f"the tokens of request {e.request_id!r} must be a flat list of ids")
            lo, hi = int(ids.min()), int(ids.max())
            if lo < 0 or hi >= self.vocab_size:
                bad = lo if lo < 0 else hi
                raise IndexError(f"token id {bad} of request {e.request_id!r} is outside [0, {self.vocab_size})")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise IndexError(f"wanted place {w} of request {e.request_id!r} is outside its {n} tokens")
            if rc.num_tokens + n > self.max_position:
                raise ValueError(
                    f"request {e.request_id!r} would reach {rc.num_tokens + n} tokens, "
                    f"max_position_embeddings is {self.max_position}"
                )
            rcs.append(rc)
        return rcs

    def _build_context(self, rcs, entries) -> StepContext:
        ps = self.page_size
        n_groups = len(self.cache.groups)
        b = len(entries)
        q_len = [len(e.tokens) for e in entries]
        q_start = [0] * b
        for i in range(1, b):
            q_start[i] = q_start[i - 1] + q_len[i - 1]
        t = q_start[-1] + q_len[-1]
        kv_len = [rc.num_tokens + n for rc, n in zip(rcs, q_len)]
        widths = [max(max(rc.table_lens[g] for rc in rcs), 1) for g in range(n_groups)]
        want_rows: list[int] = []
        for s0, e in zip(q_start, entries):
            want_rows.extend(s0 + int(w) for w in e.want)
        # One packed int32 buffer for everything, filled in place (token ids and wanted rows here, the rest
        # by the cache manager's library) and uploaded with one copy:
        # token ids, positions [t each]; q_start, q_len, kv_len, state slots [b each]; wanted rows;
        # slots [t per group]; block tables [b x width per group]
        sizes = [t, t, b, b, b, b, len(want_rows)] + [t] * n_groups + [b * widths[g] for g in range(n_groups)]
        offsets = [0]
        for n in sizes:
            offsets.append(offsets[-1] + n)
        packed = torch.empty(offsets[-1], dtype=torch.int32, pin_memory=self.device.type == "cuda")
        host = packed.numpy()
        for s0, e in zip(q_start, entries):
            host[s0 : s0 + len(e.tokens)] = e.tokens
        host[offsets[6] : offsets[7]] = want_rows
        base = packed.data_ptr()
        ptr = lambda i: base + 4 * offsets[i]
        self.cache.fill_step(
            _ints([rc.handle for rc in rcs]), _ints(q_len), _ints(widths),
            (ptr(1), ptr(2), ptr(3), ptr(4), ptr(5), ptr(7) if n_groups else None, ptr(7 + n_groups) if n_groups else None),
        )
        dev = packed.to(self.device, non_blocking=True)
        views = [dev[offsets[i] : offsets[i + 1]] for i in range(len(sizes))]
        d_tok, d_pos, d_qs, d_ql, d_kv, d_slot, d_want = views[:7]
        groups = []
        for g in range(n_groups):
            groups.append(GroupTables(views[7 + n_groups + g].view(b, widths[g]), views[7 + g]))
        return StepContext(
            num_tokens=t, num_seqs=b, token_ids=d_tok, positions=d_pos, q_start=d_qs, q_len=d_ql, kv_len=d_kv,
            want_rows=d_want if want_rows else None, max_q_len=max(q_len), max_kv_len=max(kv_len),
            single_token_requests=1 in q_len,
            q_start_host=q_start, q_len_host=q_len, kv_len_host=kv_len,
            state_slots=d_slot, state_slots_host=[rc.slot for rc in rcs],
            groups=groups, page_size=ps, kv_storage=self.kv, state_storage=self.states,
            cache_location=self.model.cache_location, group_windows=[n.window for n in self.cache.groups],
        )

    # ------------------------------------------------------------------ the next decode step, tokens still on the device
    @property
    def supports_lookahead(self) -> bool:
        return self.use_graphs

    def step_decode_ahead(self, request_ids: Sequence, tokens: torch.Tensor) -> torch.Tensor:
        """A decode step of one token per request whose token ids the host has not seen yet: `tokens` int32 [B] on
        the device, row i the next token of request_ids[i] (what the sampler left behind the step before).  The
        step is queued behind whatever writes `tokens`, so a scheduler can launch it before it waits for that
        step's tokens, and the GPU goes from one step into the next.  Logits [B, vocab] as from `step`."""
        if not self.use_graphs:
            raise RuntimeError("steps are launched ahead only from captured graphs")
        if tokens.dtype != torch.int32 or tuple(tokens.shape) != (len(request_ids),) or tokens.device != self.device:
            raise ValueError("tokens must be int32 [number of requests] on the engine's device")
        return self._step_decode([StepEntry(rid, (0,), (0,)) for rid in request_ids], device_tokens=tokens)

    # ------------------------------------------------------------------ one token per request, from a graph
    def _step_decode(self, entries, device_tokens: torch.Tensor | None = None) -> torch.Tensor:
        """The step for batches of single tokens that all want their logits: the same model code, captured
        once per (batch size, block-table width) into a device graph and replayed with new metadata.  The
        launch of some two hundred kernels costs more host time than they run on the device; the graph
        removes that."""
        # the checks of `_check`, for one token each, in one pass
        requests = self.cache.requests
        rcs, tokens, seen = [], [], set()
        vocab, limit = self.vocab_size, self.max_position
        for e in entries:
            rc = requests.get(e.request_id)
            if rc is None:
                raise KeyError(f"request {e.request_id!r} is not live (add_request first)")
            tok = int(e.tokens[0])
            if not 0 <= tok < vocab:
                raise IndexError(f"token id {tok} of request {e.request_id!r} is outside [0, {vocab})")
            if e.want[0] != 0:
                raise IndexError(f"wanted place {e.want[0]} of request {e.request_id!r} is outside its 1 tokens")
            if rc.num_tokens >= limit:
                raise ValueError(
                    f"request {e.request_id!r} would reach {rc.num_tokens + 1} tokens, "
                    f"max_position_embeddings is {limit}"
                )
            rcs.append(rc)
            tokens.append(tok)
            seen.add(e.request_id)
        if len(seen) != len(entries):
            raise ValueError("a request appears twice in one step")
        ps = self.page_size
        # a token needs a new page only when it starts one (tables hold exactly the pages of the tokens so far)
        starters = [rc for rc in rcs if rc.num_tokens % ps == 0]
        if starters:
            self.cache.reserve_step(starters, [1] * len(starters))
        try:
            return self._decode_reserved(rcs, tokens, device_tokens)
        except BaseException:
            self.cache.unreserve_step(starters)            # a step that fails leaves the pools as it found them
            raise

    def _decode_reserved(self, rcs, tokens, device_tokens) -> torch.Tensor:
        b = len(rcs)
        # Beyond 16 requests the batch is padded to a multiple of 8 with rows of one token at position 0 on a page
        # that no request owns: requests finish one by one, and every batch size would otherwise be a graph of its
        # own, run kernel by kernel on its first visits (up to 16 the kernels' shapes follow the batch size).
        rows = b if b <= 16 else -(-b // 8) * 8
        widths = self._table_widths(rcs)
        # The kernels choose their shape (key splits of the attention) by the longest context, and a graph holds
        # one choice: contexts are bucketed in steps of 512 tokens beside the table widths.
        kv_bound = -(-(max(rc.num_tokens for rc in rcs) + 1) // 512) * 512
        key = (rows, tuple(widths), kv_bound)
        plan = self._plan(self._decode_plans, key, lambda: _DecodePlan(self, rows, widths, kv_bound))
        plan.fill(rcs, tokens)
        if device_tokens is not None:
            plan.ctx.token_ids[:b].copy_(device_tokens, non_blocking=True)      # (behind the upload of the metadata)
        logits = self._run(plan)
        self.cache.commit_step(rcs, [1] * b)
        return logits[:b]

    # ------------------------------------------------------------------ what the steps from graphs share
    MAX_PLANS = 128      # captured graphs kept per kind of step; the least recently used goes when one more is needed

    def _table_widths(self, rcs, at_least: int = 0) -> list[int]:
        """Block-table widths of a plan: for each group the next power of two (from 4) that holds the longest table."""
        widths = []
        for g in range(len(self.cache.groups)):
            need = max(max(rc.table_lens[g] for rc in rcs), at_least)
            w = 4
            while w < need:
                w *= 2
            widths.append(w)
        return widths

    def _run(self, plan) -> torch.Tensor:
        """The model on the plan's buffers: kernel by kernel on its first visits (the result, and the warm-up), the
        graph captured at visit `capture_after` and replayed from then on."""
        if plan.graph is not None:
            plan.graph.replay()
            return plan.logits
        logits = self.model.forward(plan.ctx)
        plan.runs += 1
        if self.capture_after is not None and plan.runs >= self.capture_after:
            graph = torch.cuda.CUDAGraph()
            plans = (self._decode_plans, self._row_plans, self._padded_plans)
            if self._graph_pool is None or not any(p.graph is not None for d in plans for p in d.values()):
                # the first graph, or the first after every earlier one was dropped (their pool went with the last)
                self._graph_pool = torch.cuda.graph_pool_handle()
            torch.cuda.synchronize()
            plan.logits = _capture(graph, self._graph_pool, lambda: self.model.forward(plan.ctx))
            plan.graph = graph
        return logits

    def _plan(self, plans: dict, key, make):
        plan = plans.pop(key, None)
        if plan is None:
            if len(plans) >= self.MAX_PLANS:
                plans.pop(next(iter(plans)))               # the one that was used longest ago
            plan = make()
        plans[key] = plan                                  # most recently used last
        return plan

    # ------------------------------------------------------------------ few tokens in all, from a graph
    def _step_rows(self, entries) -> torch.Tensor | None:
        """A step of few tokens that is not one token per request (a short portion of a prompt, alone or beside
        decoded tokens): every token becomes a row of its own, a "request" of one token whose context is its
        position + 1 and whose block table is its request's.  That shape depends on the number of tokens alone,
        so it is captured and replayed like a decode step, where the same step run kernel by kernel would spend
        twice its device time on the host.  Keys and values of all rows are stored before attention reads them
        (`rows_independent` is False).  Logits are computed for every row, the wanted ones are returned.  Not for
        models with per-request state, whose parts walk a portion token after token."""
        rcs = self._check(entries)
        counts = [len(e.tokens) for e in entries]
        t = sum(counts)
        with self.cache.reserved(rcs, counts):
            widths = self._table_widths(rcs)
            kv_bound = -(-max(rc.num_tokens + n for rc, n in zip(rcs, counts)) // 512) * 512
            key = (t, tuple(widths), kv_bound)
            plan = self._plan(self._row_plans, key, lambda: _DecodePlan(self, t, widths, kv_bound, rows_independent=False))
            plan.fill_rows(rcs, entries, counts)
            logits = self._run(plan)
        want, base = [], 0
        for e, n in zip(entries, counts):
            want.extend(base + int(w) for w in e.want)
            base += n
        if not want:
            return None
        if want == list(range(t)):
            return logits
        return logits.index_select(0, torch.tensor(want, dtype=torch.int64, device=self.device))


    # ------------------------------------------------------------------ any mix, from a graph for its padded size
    def _step_padded(self, entries) -> torch.Tensor | None:
        """Any step of up to `graph_tokens` tokens: the same model code as the general step, on static buffers of a
        padded size, captured once per (tokens rounded up to a multiple of 64, of 16 up to 256; requests rounded up to a power of two,
        block-table widths) and replayed.  The padding is one more "request" whose tokens have pages of their own
        that no real request ever gets; the requests after it have no tokens.  Every kernel takes the layout of the
        step (where each request's tokens start, how many, how long its context is) from device memory, so one graph
        serves every step of its size.  A step of a few hundred tokens run kernel by kernel takes 4 ms of host time
        whatever its size; from the graph it takes its device time."""
        rcs = self._check(entries)
        counts = [len(e.tokens) for e in entries]
        with self.cache.reserved(rcs, counts):
            return self._padded_reserved(rcs, entries, counts)

    def _padded_reserved(self, rcs, entries, counts) -> torch.Tensor | None:
        t = sum(counts)
        step = 16 if t <= 256 else self.PAD_TO          # small steps are padded less: their time grows with their rows
        t_pad = -(-t // step) * step
        b_pad = 2
        while b_pad < len(rcs) + 1:
            b_pad *= 2
        widths = self._table_widths(rcs, at_least=self._pad_pages)
        r_pad = b_pad                           # logits rows: usually one per request or fewer
        n_wanted = sum(len(e.want) for e in entries)
        while r_pad < n_wanted:
            r_pad *= 2
        # (steps with and without requests of one token have graphs of their own: the attention takes those requests
        # apart, in a kernel that the others need not launch; the padding's tokens go either way)
        singles = 1 in counts
        key = (t_pad, b_pad, r_pad, tuple(widths), singles)
        plan = self._plan(self._padded_plans, key, lambda: _PaddedPlan(self, t_pad, b_pad, r_pad, widths, singles))
        n_want = plan.fill(rcs, entries, counts)
        logits = self._run(plan)
        return logits[:n_want] if n_want else None


def _capture(graph, pool, run):
    """Capture `run` into `graph`.  The collector of reference cycles stays off meanwhile: what it would free (a
    dead engine's device memory, another graph) must not be freed while a stream is capturing."""
    import gc

    was_enabled = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph, pool=pool):
            return run()
    finally:
        if was_enabled:
            gc.enable()


class _PaddedPlan:
    """Static buffers, a pinned host mirror and the captured graph of one padded step size."""

    def __init__(self, engine: Engine, t_pad: int, b_pad: int, r_pad: int, widths: list[int], singles: bool = True):
        self.t_pad, self.b_pad, self.widths = t_pad, b_pad, list(widths)
        # (no reference back to the engine: engine and plan would keep each other alive until the collector of
        # reference cycles runs, which may be in the middle of another engine's graph capture, where memory of
        # the device must not be freed)
        self.cache, self.page_size = engine.cache, engine.page_size
        self.pad_first_page, self.pad_pages = engine._pad_first_page, engine._pad_pages
        self.pad_state_slot = engine.states.pad_slot
        dev = engine.device
        n_groups = len(widths)
        ps = engine.page_size
        # token ids, positions [t_pad each]; q_start, q_len, kv_len, state slots [b_pad each]; wanted rows [r_pad];
        # slots [t_pad per group]; block tables [b_pad x width per group]
        sizes = [t_pad, t_pad, b_pad, b_pad, b_pad, b_pad, r_pad] + [t_pad] * n_groups + [b_pad * w for w in widths]
        self.offsets = [0]
        for n in sizes:
            self.offsets.append(self.offsets[-1] + n)
        self.host = torch.zeros(self.offsets[-1], dtype=torch.int32).pin_memory()
        self.dev = torch.zeros(self.offsets[-1], dtype=torch.int32, device=dev)
        self.np = self.host.numpy()
        view = lambda i: self.dev[self.offsets[i] : self.offsets[i + 1]]
        groups = [GroupTables(view(7 + n_groups + g).view(b_pad, widths[g]), view(7 + g)) for g in range(n_groups)]
        self.ctx = StepContext(
            num_tokens=t_pad, num_seqs=b_pad, token_ids=view(0), positions=view(1), q_start=view(2), q_len=view(3),
            kv_len=view(4), want_rows=view(6), max_q_len=t_pad, max_kv_len=min(w * ps for w in widths) if widths else 0,
            q_start_host=[0] * b_pad, q_len_host=[0] * b_pad, kv_len_host=[0] * b_pad,
            state_slots=view(5), state_slots_host=[0] * b_pad, groups=groups, page_size=ps, kv_storage=engine.kv,
            state_storage=engine.states, cache_location=engine.model.cache_location,
            group_windows=[n.window for n in engine.cache.groups], single_token_requests=singles,
        )
        self.c_widths = _ints(self.widths)
        self.copied = None
        self.graph = None
        self.logits = None
        self.runs = 0

    def part(self, i: int) -> np.ndarray:
        return self.np[self.offsets[i] : self.offsets[i + 1]]

    def fill(self, rcs, entries, counts) -> int:
        """Writes the step's metadata; returns how many logits rows are wanted (the first rows of the result)."""
        if self.copied is not None:
            self.copied.synchronize()                       # the pinned mirror is free again
        t_pad, b_pad = self.t_pad, self.b_pad
        b, t = len(rcs), sum(counts)
        pad = t_pad - t
        n_groups = len(self.widths)
        ps = self.page_size
        tokens, positions = self.part(0), self.part(1)
        q_start, q_len, kv_len, state_slots, want_rows = (self.part(i) for i in range(2, 7))
        pos = 0
        want: list[int] = []
        for e, n in zip(entries, counts):
            tokens[pos : pos + n] = e.tokens
            want.extend(pos + int(w) for w in e.want)
            pos += n
        slots = np.empty(max(n_groups * t, 1), dtype=np.int32)
        tables = np.empty(max(sum(b * w for w in self.widths), 1), dtype=np.int32)
        self.cache.fill_step(
            _ints([rc.handle for rc in rcs]), _ints(counts), self.c_widths,
            (positions.ctypes.data, q_start.ctypes.data, q_len.ctypes.data, kv_len.ctypes.data, state_slots.ctypes.data,
             slots.ctypes.data if n_groups else None, tables.ctypes.data if n_groups else None),
        )
        # the padding: a request of `pad` tokens at positions 0.. on pages of its own, then requests without tokens
        tokens[t:] = 0
        positions[t:] = np.arange(pad, dtype=np.int32)
        q_start[b:] = t_pad
        q_len[b:] = 0
        kv_len[b:] = 0
        state_slots[b:] = self.pad_state_slot
        q_start[b], q_len[b], kv_len[b] = t, pad, pad
        want_rows[: len(want)] = want
        want_rows[len(want) :] = 0
        pad_slots = (self.pad_first_page + np.arange(pad, dtype=np.int32) // ps) * ps + np.arange(pad, dtype=np.int32) % ps
        off_in = 0
        for g, w in enumerate(self.widths):
            s_out = self.part(7 + g)
            s_out[:t] = slots[g * t : (g + 1) * t]
            s_out[t:] = pad_slots
            tab = self.part(7 + n_groups + g).reshape(b_pad, w)
            tab[:b] = tables[off_in : off_in + b * w].reshape(b, w)
            tab[b:] = -1
            tab[b, : self.pad_pages] = self.pad_first_page + np.arange(self.pad_pages, dtype=np.int32)
            off_in += b * w
        ctx = self.ctx
        ctx.q_start_host = q_start.tolist()
        ctx.q_len_host = q_len.tolist()
        ctx.kv_len_host = kv_len.tolist()
        ctx.state_slots_host = state_slots.tolist()
        self.dev.copy_(self.host, non_blocking=True)
        if self.copied is None:
            self.copied = torch.cuda.Event()
        self.copied.record()
        return len(want)



class _DecodePlan:
    """Static device buffers, a host mirror and the captured graph of one decode batch shape."""

    def __init__(self, engine: Engine, batch: int, widths: list[int], kv_bound: int, rows_independent: bool = True):
        self.batch, self.widths = batch, list(widths)
        dev = engine.device
        n_groups = len(widths)
        b = batch
        n_small = (7 + n_groups) * b
        self.host_small = torch.empty(n_small, dtype=torch.int32, pin_memory=True)
        self.dev_small = torch.empty(n_small, dtype=torch.int32, device=dev)
        n_tab = sum(b * w for w in widths)
        self.host_tab = torch.full((max(n_tab, 1),), -1, dtype=torch.int32).pin_memory()
        self.dev_tab = torch.full((max(n_tab, 1),), -1, dtype=torch.int32, device=dev)
        self.np_small = self.host_small.numpy()
        v = lambda i: self.dev_small[i * b : (i + 1) * b]
        groups, off = [], 0
        for g, w in enumerate(widths):
            groups.append(GroupTables(self.dev_tab[off : off + b * w].view(b, w), v(7 + g)))
            off += b * w
        ps = engine.page_size
        self.ctx = StepContext(
            num_tokens=b, num_seqs=b, token_ids=v(0), positions=v(1), q_start=v(2), q_len=v(3), kv_len=v(4),
            want_rows=v(6), max_q_len=1, max_kv_len=min([kv_bound] + [w * ps for w in widths]),
            q_start_host=list(range(b)), q_len_host=[1] * b, kv_len_host=[0] * b,
            state_slots=v(5), state_slots_host=[0] * b, groups=groups, page_size=ps, kv_storage=engine.kv,
            state_storage=engine.states, cache_location=engine.model.cache_location,
            group_windows=[n.window for n in engine.cache.groups], rows_independent=rows_independent,
        )
        self.row_state = np.full(2 * b, -1, dtype=np.int64)     # per row: (handle, table version) last written
        self.c_widths = _ints(self.widths)
        self.cache = engine.cache
        self.pad_page, self.page_size = engine._pad_first_page, ps
        self.pad_state_slot = engine.states.pad_slot
        self.copied = None           # event after the last host-to-device copy
        self.graph = None
        self.logits = None
        self.runs = 0

    def fill(self, rcs, tokens) -> None:
        if self.copied is not None:
            self.copied.synchronize()                       # the pinned mirror is free again
        rows, b = self.batch, len(rcs)
        self.np_small[0:b] = tokens
        handles = _ints([rc.handle for rc in rcs])
        tables_changed = self.cache.fill_decode(handles, self.c_widths, self.host_small.data_ptr(),
                                                self.host_tab.data_ptr(), self.row_state.ctypes.data, rows=rows)
        self.ctx.kv_len_host = [rc.num_tokens + 1 for rc in rcs] + [1] * (rows - b)
        self.ctx.state_slots_host = [rc.slot for rc in rcs] + [self.pad_state_slot] * (rows - b)
        if b < rows:
            # the padding: token 0 at position 0, alone in its context, all on the first slot of the padding's page
            # (the same key and value from every such row)
            n_groups = len(self.widths)
            small = self.np_small.reshape(7 + n_groups, rows)
            small[0, b:] = 0
            small[1, b:] = 0
            small[2, b:] = np.arange(b, rows, dtype=np.int32)
            small[3, b:] = 1
            small[4, b:] = 1
            small[5, b:] = self.pad_state_slot           # the state record that belongs to no request
            small[6, b:] = np.arange(b, rows, dtype=np.int32)
            small[7:, b:] = self.pad_page * self.page_size
            tab = self.host_tab.numpy()
            off = 0
            for w in self.widths:
                for i in range(b, rows):
                    if self.row_state[2 * i] != -2:          # the row held a request's table (or nothing yet)
                        tab[off + i * w : off + (i + 1) * w] = -1
                        tab[off + i * w] = self.pad_page
                        tables_changed = True
                off += rows * w
            self.row_state[2 * b : 2 * rows : 2] = -2
        self.dev_small.copy_(self.host_small, non_blocking=True)
        if tables_changed:
            self.dev_tab.copy_(self.host_tab, non_blocking=True)
        if self.copied is None:
            self.copied = torch.cuda.Event()
        self.copied.record()

    def fill_rows(self, rcs, entries, counts) -> None:
        """The metadata of a step whose tokens are laid out as rows of one token each: the cache manager's library
        writes the step as it is (positions and slots per token, a table per request), and the per-request parts
        are repeated for every token of the request."""
        if self.copied is not None:
            self.copied.synchronize()
        t, b = self.batch, len(rcs)
        n_groups = len(self.widths)
        small = self.np_small.reshape(7 + n_groups, t)
        pos = 0
        for e, n in zip(entries, counts):
            small[0, pos : pos + n] = e.tokens
            pos += n
        per_request = np.empty((4, b), dtype=np.int32)               # q_start, q_len, kv_len, state slots
        slots = np.empty(max(n_groups * t, 1), dtype=np.int32)
        tables = np.empty(max(sum(b * w for w in self.widths), 1), dtype=np.int32)
        self.cache.fill_step(
            _ints([rc.handle for rc in rcs]), _ints(counts), self.c_widths,
            (small[1].ctypes.data, per_request[0].ctypes.data, per_request[1].ctypes.data, per_request[2].ctypes.data,
             per_request[3].ctypes.data, slots.ctypes.data if n_groups else None, tables.ctypes.data if n_groups else None),
        )
        rows = np.arange(t, dtype=np.int32)
        reps = np.asarray(counts)
        small[2], small[3], small[4] = rows, 1, small[1] + 1
        small[5] = np.repeat(per_request[3], reps)
        small[6] = rows
        tab = self.host_tab.numpy()
        off_in = off_out = 0
        for g, w in enumerate(self.widths):
            small[7 + g] = slots[g * t : (g + 1) * t]
            tab[off_out : off_out + t * w] = np.repeat(tables[off_in : off_in + b * w].reshape(b, w), reps, axis=0).reshape(-1)
            off_in += b * w
            off_out += t * w
        self.ctx.kv_len_host = (small[4]).tolist()
        self.ctx.state_slots_host = small[5].tolist()
        self.dev_small.copy_(self.host_small, non_blocking=True)
        self.dev_tab.copy_(self.host_tab, non_blocking=True)
        if self.copied is None:
            self.copied = torch.cuda.Event()
        self.copied.record()

