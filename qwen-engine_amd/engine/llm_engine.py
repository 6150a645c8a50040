"""The engine above the step function, with the reference's entry points:
``LLMEngine.submit`` and ``LLMEngine.serving`` (src/engine/llm_engine.py:75-80,101-152),
and ``generate`` for callers that want the results back instead of printed."""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Callable, List, Optional, Sequence, Union

from ..config.engine_config import EngineConfig
from ..sampling.sampler import Sampler, SamplingParams, uniform_for
from .runner import ModelRunner, StepEntry, load_model
from .scheduler import Request, Scheduler


@dataclass
class GenerationResult:
    request_id: int
    prompt_token_ids: List[int]
    token_ids: List[int]
    finish_reason: str
    text: Optional[str] = None
    error: Optional[str] = None


def load_tokenizer(folder: str):
    """The folder's tokenizer.json, or None.  Text goes in raw, without a chat template
    (src/engine/llm_engine.py:52-55)."""
    path = os.path.join(folder, "tokenizer.json")
    if not os.path.isfile(path):
        return None
    from tokenizers import Tokenizer
    return Tokenizer.from_file(path)


class LLMEngine:
    def __init__(self, model, tokenizer=None, engine_config: Optional[EngineConfig] = None):
        self.config = engine_config or EngineConfig()
        self.config.validate()
        self.model = model
        self.tokenizer = tokenizer
        cfg = self.config
        if cfg.num_blocks is None and cfg.gpu_memory_fraction is not None:
            import torch
            from ..parts.model import cache_plan
            plan = cache_plan(model.spec)
            itemsize = 2 if cfg.dtype == "bfloat16" else 4
            per_page = max(1, plan.bytes_per_token(itemsize) * cfg.block_size)   # (every group gets the same number of pages)
            pages = cfg.pages_per_group(torch.cuda.mem_get_info(model.rt.device)[0], per_page)
        else:
            pages = cfg.pages_per_group()
        self.runner = ModelRunner(model, page_size=cfg.block_size, num_pages=pages,
                                  max_requests=cfg.max_num_seqs, prefix_sharing=cfg.enable_prefix_sharing,
                                  keep_freed_prefixes=cfg.keep_freed_prefixes, scatter_pages=cfg.scatter_pages,
                                  debug_poison=cfg.debug_poison,
                                  record_mixed_steps=cfg.record_mixed_steps, graph_record_after=cfg.graph_record_after,
                                  graph_memory_bytes=cfg.graph_memory_bytes)
        max_len = min(cfg.max_model_len, model.spec.max_positions)
        self.scheduler = Scheduler(self.runner.cache, cfg.max_num_seqs, max_len, cfg.max_step_tokens,
                                   cfg.prefill_chunk, model.spec.eos_token_ids)
        self.sampler = Sampler()
        self._next_id = 0
        self._submitted: List[Request] = []

    @classmethod
    def from_folder(cls, folder: str, engine_config: Optional[EngineConfig] = None, device: str = "cuda:0"):
        cfg = engine_config or EngineConfig()
        model = load_model(folder, dtype=cfg.dtype, device=device)
        return cls(model, load_tokenizer(folder), cfg)

    # ---- text <-> tokens -----------------------------------------------------------------
    def encode(self, text: str) -> List[int]:
        if self.tokenizer is None:
            raise ValueError("a text prompt needs a tokenizer; the model folder has no tokenizer.json")
        return list(self.tokenizer.encode(text).ids)

    def decode(self, ids: Sequence[int]) -> Optional[str]:
        if self.tokenizer is None:
            return None
        return self.tokenizer.decode(list(ids), skip_special_tokens=True)

    # ---- the reference's interface ----------------------------------------------------------
    def submit(self, prompt_texts: Union[str, Sequence[int], Sequence[Union[str, Sequence[int]]]],
               max_new_tokens: int = 16, temperature: float = 0.0, seed: Optional[int] = None,
               ignore_eos: bool = False) -> List[int]:
        """Queue prompts: texts, or lists of token ids.  Returns the requests' ids."""
        if isinstance(prompt_texts, str) or (prompt_texts and isinstance(prompt_texts[0], int)):
            prompt_texts = [prompt_texts]
        ids = []
        for p in prompt_texts:
            text = p if isinstance(p, str) else None
            tokens = self.encode(p) if isinstance(p, str) else [int(t) for t in p]
            params = SamplingParams(max_new_tokens=max_new_tokens, temperature=temperature,
                                    seed=self.config.seed if seed is None else seed, ignore_eos=ignore_eos)
            req = Request(req_id=self._next_id, prompt=tokens, params=params, prompt_text=text)
            self._next_id += 1
            self._submitted.append(req)
            self.scheduler.add(req)
            ids.append(req.req_id)
        return ids

    def step(self) -> List[Request]:
        """One step of the engine; returns the requests that finished in it."""
        planned = self.scheduler.plan()
        if not planned:
            return []
        entries = [StepEntry(p.request.req_id, p.tokens, [len(p.tokens) - 1] if p.sample else [])
                   for p in planned]
        sampling = [p.request for p in planned if p.sample]
        temps = [r.params.temperature for r in sampling]
        if all(t <= 0 for t in temps):
            # every row is greedy: the step picks the tokens itself (inside its graph, where it is a
            # recorded one), and no logits are copied or read again
            tokens = self.runner.step(entries, greedy=True)
        else:
            logits = self.runner.step(entries)
            us = [uniform_for(r.params.seed, r.req_id, len(r.output)) if t > 0 else 0.0 for r, t in zip(sampling, temps)]
            tokens = self.sampler.sample(logits, temps, us)
        return self.scheduler.update(planned, tokens)

    def run(self) -> List[GenerationResult]:
        """Run until every submitted request is finished; results in submission order."""
        while self.scheduler.has_work():
            self.step()
        results = []
        for r in self._submitted:
            text = self.decode(r.prompt + r.output) if r.finish_reason != "error" else None
            results.append(GenerationResult(r.req_id, list(r.prompt), list(r.output),
                                            r.finish_reason or "error", text, r.error))
        self._submitted = []
        self.scheduler.finished = []
        return results

    def serving(self, print_func: Callable[[Optional[str], Optional[str]], None]) -> List[GenerationResult]:
        """Run everything that was submitted, then hand (prompt text, decoded prompt + output)
        of every request to ``print_func`` (src/engine/llm_engine.py:147-149)."""
        results = self.run()
        for r in results:
            ids = r.prompt_token_ids
            prompt_text = self.decode(ids) if self.tokenizer is not None else " ".join(map(str, ids))
            if r.error:
                shown = f"[failed: {r.error}]"
            elif r.text is not None:
                shown = r.text
            else:
                shown = " ".join(str(t) for t in ids + r.token_ids)
            print_func(prompt_text, shown)
        return results

    def stats(self) -> dict:
        d = dict(self.scheduler.stats)
        d.update(self.runner.cache.stats)
        d["free_pages"] = [p.num_free for p in self.runner.cache.pools]
        d["kept_pages"] = self.runner.cache.num_kept
        d["graph_steps"] = self.runner.graph_steps
        for kind, n in self.runner.graph_steps_of.items():
            d[f"graph_steps_{kind}"] = n
        d["graphs_recorded"] = self.runner.graphs_recorded
        d["graph_misses"] = self.runner.graph_misses      # steps of a recordable shape that ran as they came
        d["graph_bytes"] = self.runner.graph_bytes()
        return d


def generate(model_dir: str, prompts, sampling: Optional[SamplingParams] = None,
             engine_config: Optional[EngineConfig] = None, device: str = "cuda:0") -> List[GenerationResult]:
    """Load the model of ``model_dir`` and generate for every prompt (text or token ids)."""
    sampling = sampling or SamplingParams()
    engine = LLMEngine.from_folder(model_dir, engine_config, device=device)
    engine.submit(prompts, max_new_tokens=sampling.max_new_tokens, temperature=sampling.temperature,
                  seed=sampling.seed, ignore_eos=sampling.ignore_eos)
    return engine.run()
