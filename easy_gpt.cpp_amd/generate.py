"""The Python entry point: a model folder and prompts (token ids) in, generated token ids out.

    from easy_gpt.cpp_amd.generate import LLM
    llm = LLM("path/to/model", dtype="bfloat16")
    outputs = llm.generate([[1, 2, 3], [4, 5]], max_new_tokens=16, greedy=True)

It is the one-shot mode of the reference (GptEngine::run -> GptModel::forward,
/root/reference/src/gpt_engine.cpp:33-43, /root/reference/src/models/gpt_model.cpp:155-190) run
through the same scheduler as continuous batching, with all requests submitted up front.
"""
from __future__ import annotations

from typing import Sequence

from .engine.engine import Engine
from .engine.scheduler import Request, Scheduler, SchedulerConfig
from .sampling import SamplingParams


class RequestsFailed(RuntimeError):
    """Some requests failed (say, the cache cannot hold them even alone); the others ran to their end.
    `requests` holds every request of the call in the order of the prompts, each with its `status`
    ("finished" or "failed"), `finish_reason` and `output`."""

    def __init__(self, requests: list[Request]):
        self.requests = requests
        failed = [r for r in requests if r.status == "failed"]
        super().__init__("; ".join(f"request {r.request_id} failed: {r.finish_reason}" for r in failed))


class LLM:
    def __init__(
        self,
        model_dir: str,
        dtype: str = "bfloat16",
        device: str = "cuda:0",
        cache_tokens: int = 65536,
        page_size: int = 16,
        max_active: int = 16,
        max_admit_per_step: int = 4,
        max_tokens_per_step: int = 2048,
        prefill_chunk: int = 512,
        tune_products: bool = False,
        allow_unexpected_tensors: bool = False,
    ):
        self.engine = Engine.from_dir(model_dir, dtype=dtype, device=device, page_size=page_size,
                                      max_tokens=cache_tokens, max_requests=max_active, tune_products=tune_products,
                                      allow_unexpected_tensors=allow_unexpected_tensors)
        self.config = SchedulerConfig(max_active=max_active, max_admit_per_step=max_admit_per_step,
                                      max_tokens_per_step=max_tokens_per_step, prefill_chunk=prefill_chunk)
        self.eos_token_id = self.engine.model.spec.eos_token_id
        self.last_stats = None
        self.last_requests: list[Request] = []

    def generate_requests(
        self,
        prompts: Sequence[Sequence[int]],
        max_new_tokens: int = 100,
        temperature: float = 0.8,
        top_p: float = 0.95,
        top_k: int = 20,
        greedy: bool = False,
        seed: int = 42,
        ignore_eos: bool = False,
        max_steps: int | None = None,
        on_step=None,
    ) -> list[Request]:
        """One Request per prompt, in the order of the prompts, each with its `output`, `status` ("finished" or
        "failed") and `finish_reason`: a request that fails does not take the others with it.  `max_steps`, if
        given, is the reference's --max-steps: a cap on a request's total length, giving
        max(1, max_steps - len(prompt) + 1) new tokens
        (/root/reference/src/continuous_batch_server.cpp:313)."""
        params = SamplingParams(temperature=temperature, top_p=top_p, top_k=top_k, greedy=greedy, seed=seed)
        sched = Scheduler(self.engine, self.config, eos_token_id=self.eos_token_id)
        reqs = []
        for i, p in enumerate(prompts):
            n_new = max_new_tokens if max_steps is None else max(1, max_steps - len(p) + 1)
            reqs.append(sched.add(Request(i, list(int(t) for t in p), params, n_new, ignore_eos)))
        sched.run(on_step)
        self.last_stats = sched.stats
        self.last_requests = reqs
        return reqs

    def generate(self, prompts: Sequence[Sequence[int]], **options) -> list[list[int]]:
        """Generated token ids for each prompt, in the order of the prompts (options as `generate_requests`).
        Raises RequestsFailed, which holds all requests and their outputs, if any of them failed."""
        reqs = self.generate_requests(prompts, **options)
        if any(r.status == "failed" for r in reqs):
            raise RequestsFailed(reqs)
        return [r.output for r in reqs]


def generate(model_dir: str, prompts, dtype: str = "bfloat16", device: str = "cuda:0", **options) -> list[list[int]]:
    """One call: load `model_dir`, generate for `prompts` (lists of token ids)."""
    llm_keys = {"cache_tokens", "page_size", "max_active", "max_admit_per_step", "max_tokens_per_step",
                "prefill_chunk", "tune_products", "allow_unexpected_tensors"}
    llm_opts = {k: options.pop(k) for k in list(options) if k in llm_keys}
    return LLM(model_dir, dtype=dtype, device=device, **llm_opts).generate(prompts, **options)
