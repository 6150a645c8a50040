"""Trace replay: feeds given token ids through the model step by step and writes
the logits at the wanted places.  It samples nothing, and has no forward pass,
cache or loader of its own: it drives ``ModelRunner``."""
from __future__ import annotations

import json
import os
import sys
from typing import IO

import numpy as np
import torch

from .runner import ModelRunner, StepEntry, load_model

MAX_LIVE = 4          # requests that are live at a time in a trace
TOKEN_ROUNDING = 64   # a request's token count is rounded up to this for --max-tokens


def replay(model_dir: str, dtype: str, out_dir: str, max_tokens: int, lines: IO[str],
           out: IO[str] = sys.stdout, page_size: int = 16, device: str = "cuda:0",
           debug_poison: bool = False) -> int:
    if TOKEN_ROUNDING % page_size:
        raise ValueError(f"page size {page_size} does not divide {TOKEN_ROUNDING}")
    os.makedirs(out_dir, exist_ok=True)
    model = load_model(model_dir, dtype=dtype, device=device)
    rounded = (max_tokens + TOKEN_ROUNDING - 1) // TOKEN_ROUNDING * TOKEN_ROUNDING
    num_pages = max(1, rounded // page_size)
    runner = ModelRunner(model, page_size=page_size, num_pages=num_pages, max_requests=MAX_LIVE, debug_poison=debug_poison)
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            if e["id"] not in runner.cache.requests:
                runner.add_request(e["id"])
            entries.append(StepEntry(e["id"], e["tokens"], e.get("want", [])))
        if entries:
            logits = runner.step(entries)
            if logits.shape[0]:
                arr = logits.detach().to("cpu", torch.float32).numpy().astype("<f4", copy=False)
                arr.tofile(os.path.join(out_dir, f"{step}.f32"))
        for req_id in rec.get("end", []):
            if req_id in runner.cache.requests:
                runner.free_request(req_id)
        print(f"done {step}", file=out, flush=True)
    return 0
