"""A plain, slow step function over a paged cache, written from the reference's slow accessors
(src/engine/kvcache.py:222-283: write_tokens, gather_sequence) and its plain attention over them
(src/layers/fused_ops/attn.py:715-788): CPU only, one token copy at a time, no code shared with
the engine.  A step takes (request, its next tokens) for any number of requests, portions of prompts
beside single tokens, writes the new keys and values into the requests' pages, gathers each
request's keys and values back through its page list, and attends with the explicit mask
q_abs_pos >= k_abs_pos.  What it proves on the CPU: that cutting and batching change nothing, and
what a page that is given back and used again has to look like.
"""
from __future__ import annotations

import math
from typing import Dict, Hashable, List, Sequence, Tuple

import torch

from . import qwen3_plain as P


class PagedCache:
    """k and v [layers, pages, page size, kv heads, head size]; a stack of free pages that hands out
    page 0 first and the page given back last next (kvcache.py:47-67,149-166)."""

    def __init__(self, layers: int, pages: int, page_size: int, kv_heads: int, head_dim: int, dtype=torch.float32):
        self.page_size = page_size
        self.k = torch.full((layers, pages, page_size, kv_heads, head_dim), float("nan"), dtype=dtype)
        self.v = torch.full_like(self.k, float("nan"))
        self.free = list(range(pages - 1, -1, -1))
        self.pages: Dict[Hashable, List[int]] = {}
        self.length: Dict[Hashable, int] = {}

    def grow(self, req: Hashable, new_len: int) -> None:
        held = self.pages.setdefault(req, [])
        self.length.setdefault(req, 0)
        while len(held) * self.page_size < new_len:
            if not self.free:
                raise RuntimeError("No free KV cache blocks available")       # kvcache.py:150-151
            held.append(self.free.pop())

    def release(self, req: Hashable) -> None:
        for page in self.pages.pop(req):
            self.k[:, page] = float("nan")             # (what is given back is poisoned: a later reader of it shows)
            self.v[:, page] = float("nan")
            self.free.append(page)
        del self.length[req]

    def write_tokens(self, layer: int, req: Hashable, start: int, k: torch.Tensor, v: torch.Tensor) -> None:
        held = self.pages[req]
        for i in range(k.shape[0]):                    # kvcache.py:245-252
            pos = start + i
            self.k[layer, held[pos // self.page_size], pos % self.page_size] = k[i]
            self.v[layer, held[pos // self.page_size], pos % self.page_size] = v[i]

    def gather_sequence(self, layer: int, req: Hashable, seq_len: int) -> Tuple[torch.Tensor, torch.Tensor]:
        held = self.pages[req]
        k = torch.stack([self.k[layer, held[p // self.page_size], p % self.page_size] for p in range(seq_len)])
        v = torch.stack([self.v[layer, held[p // self.page_size], p % self.page_size] for p in range(seq_len)])
        return k, v                                    # kvcache.py:274-281


def step(cfg: dict, w: Dict[str, torch.Tensor], cache: PagedCache, entries: Sequence[Tuple[Hashable, List[int]]],
         compute: torch.dtype = torch.float32) -> Dict[Hashable, torch.Tensor]:
    """Runs the entries' tokens as one flat batch from the cache; returns every entry's logits [its tokens, V]."""
    hq, hkv, d, eps = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["rms_norm_eps"]
    table = P.rope_table(P.rope_theta_of(cfg), d, cfg["max_position_embeddings"])
    spans, ids, pos = [], [], []
    for req, toks in entries:
        before = cache.length.get(req, 0)
        cache.grow(req, before + len(toks))
        spans.append((req, len(ids), len(toks), before))
        ids += list(toks)
        pos += list(range(before, before + len(toks)))
    positions = torch.tensor(pos)
    h = P.embedding(torch.tensor(ids), w["model.embed_tokens.weight"]).to(compute)
    T = len(ids)
    for layer in range(cfg["num_hidden_layers"]):
        pre = f"model.layers.{layer}"
        W = lambda name: w[f"{pre}.{name}"].to(compute)
        x = P.rms_norm(h, W("input_layernorm.weight"), eps)
        q = P.rms_norm(P.linear(x, W("self_attn.q_proj.weight")).view(T, hq, d), W("self_attn.q_norm.weight"), eps)
        k = P.rms_norm(P.linear(x, W("self_attn.k_proj.weight")).view(T, hkv, d), W("self_attn.k_norm.weight"), eps)
        v = P.linear(x, W("self_attn.v_proj.weight")).view(T, hkv, d)
        q, k = P.apply_rope(table, positions, q), P.apply_rope(table, positions, k)
        o = torch.empty_like(q)
        for req, first, n, before in spans:            # attn.py:729-786: write, gather, attend with the explicit mask
            cache.write_tokens(layer, req, before, k[first:first + n], v[first:first + n])
            k_all, v_all = cache.gather_sequence(layer, req, before + n)
            o[first:first + n] = P.attention(q[first:first + n], k_all.to(compute), v_all.to(compute), 1.0 / math.sqrt(d),
                                             torch.arange(before, before + n), torch.arange(before + n))
        h = h + P.linear(o.reshape(T, hq * d), W("self_attn.o_proj.weight"))
        h = h + P.mlp_block(P.rms_norm(h, W("post_attention_layernorm.weight"), eps), w, pre)
    x = P.rms_norm(h, w["model.norm.weight"].to(compute), eps)
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    logits = P.linear(x, head.to(compute))
    out = {}
    for req, first, n, before in spans:
        cache.length[req] = before + n
        out[req] = logits[first:first + n]
    return out
