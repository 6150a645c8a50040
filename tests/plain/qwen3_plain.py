"""A plain, slow implementation of the Qwen3 dense decoder, written from the
formulas of the reference's own files (cited per function as file:line of
kzw3933/Qwen-Engine).  Whole sequences, no cache, one function per part, CPU
only.  It shares no code with the engine: it reads config.json and
model.safetensors by itself.

``act_dtype`` imitates the engine's bfloat16 mode: tensors that the engine
stores in bfloat16 between kernels are rounded there; everything the engine
computes in 32-bit (norm statistics, rotation, softmax, accumulators, the
residual stream) stays in ``compute`` precision.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch


# ----------------------------------------------------------------------------
# helpers
# ----------------------------------------------------------------------------
def _round(x: torch.Tensor, act_dtype: Optional[torch.dtype]) -> torch.Tensor:
    if act_dtype is None:
        return x
    return x.to(act_dtype).to(x.dtype)


def read_folder(folder: str):
    """config.json as a dict and all tensors of model.safetensors, as stored."""
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name)
    return cfg, tensors


# ----------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------
def embedding(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """out[t, :] = table[ids[t], :]  (src/layers/ops/embedding.py:11-44,136-137)."""
    return table[ids.long()]


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x * rsqrt(mean(x^2) + eps) * w over the last dimension; a 3-D input is
    rows that share w (src/layers/ops/layernorm.py:50-89, commented form :200-207)."""
    mean_sq = (x * x).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(mean_sq + eps) * weight


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x W^T (+ b), W stored [out, in] (src/layers/ops/linear.py:101-132,181-185)."""
    y = x @ weight.t()
    if bias is not None:
        y = y + bias
    return y


def rope_table(theta: float, rotary_dim: int, max_positions: int) -> torch.Tensor:
    """Row p = [cos(p f_i) | sin(p f_i)], f_i = 1 / theta^(2i/D), all in 32-bit
    (src/models/qwen3/model.py:75-86)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    t = torch.arange(max_positions, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)
    return torch.cat([torch.cos(freqs), torch.sin(freqs)], dim=-1)


def apply_rope(table: torch.Tensor, positions: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """Half-split rotation of x [T, heads, D]: x1 = x[..., :D/2], x2 = x[..., D/2:],
    out = [cos x1 - sin x2 | sin x1 + cos x2]  (src/layers/ops/rope.py:250-274)."""
    half = table.shape[-1] // 2
    row = table[positions.long()].to(x.dtype)
    cos = row[:, None, :half]
    sin = row[:, None, half:]
    x1 = x[..., :half]
    x2 = x[..., half:]
    return torch.cat([cos * x1 - sin * x2, sin * x1 + cos * x2], dim=-1)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
              q_positions: Optional[torch.Tensor] = None,
              k_positions: Optional[torch.Tensor] = None,
              window: Optional[int] = None, causal: bool = True) -> torch.Tensor:
    """q [Tq, Hq, D], k and v [Tk, Hkv, D] -> [Tq, Hq, D].

    score = (q . k) * scale; a key at position j is seen by a query at position
    p iff j <= p (src/layers/fused_ops/attn.py:236-244,767-780); head h of q uses
    kv head h // (Hq / Hkv) (attn.py:181-182).  ``window`` (not in the reference)
    keeps only keys with p - j < window.
    """
    tq, hq, d = q.shape
    tk, hkv, _ = k.shape
    assert hq % hkv == 0
    group = hq // hkv
    if q_positions is None:
        q_positions = torch.arange(tk - tq, tk)
    if k_positions is None:
        k_positions = torch.arange(tk)
    out = torch.empty_like(q)
    allowed = torch.ones(tq, tk, dtype=torch.bool)
    if causal:
        allowed &= q_positions[:, None] >= k_positions[None, :]
    if window is not None:
        allowed &= (q_positions[:, None] - k_positions[None, :]) < window
    for h in range(hq):
        kv = h // group
        s = (q[:, h, :] @ k[:, kv, :].t()) * scale
        s = s.masked_fill(~allowed, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, h, :] = p @ v[:, kv, :]
    return out


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """silu(g) * u with silu(z) = z / (1 + exp(-z))  (src/layers/fused_ops/silumul.py:46-53,156-157).
    The product is formed before any rounding."""
    return gate / (1.0 + torch.exp(-gate)) * up


# ----------------------------------------------------------------------------
# blocks and the whole model
# ----------------------------------------------------------------------------
def attention_block(x, positions, w: Dict[str, torch.Tensor], prefix: str, cfg: dict, table,
                    act_dtype=None, window=None):
    """q/k/v projections, per-head q/k norm iff there is no bias, rotation, attention,
    output projection without bias (src/models/qwen3/model.py:200-213)."""
    hq = cfg["num_attention_heads"]
    hkv = cfg["num_key_value_heads"]
    d = cfg["head_dim"]
    eps = cfg["rms_norm_eps"]
    t = x.shape[0]
    dt = x.dtype
    bias = cfg.get("attention_bias", False)

    def W(name):
        return w[f"{prefix}.self_attn.{name}"].to(dt)

    q = _round(linear(x, W("q_proj.weight"), W("q_proj.bias") if bias else None), act_dtype).view(t, hq, d)
    k = _round(linear(x, W("k_proj.weight"), W("k_proj.bias") if bias else None), act_dtype).view(t, hkv, d)
    v = _round(linear(x, W("v_proj.weight"), W("v_proj.bias") if bias else None), act_dtype).view(t, hkv, d)
    if not bias:
        q = rms_norm(q, W("q_norm.weight"), eps)
        k = rms_norm(k, W("k_norm.weight"), eps)
    q = _round(apply_rope(table, positions, q), act_dtype)
    k = _round(apply_rope(table, positions, k), act_dtype)
    o = attention(q, k, v, 1.0 / math.sqrt(d), positions, positions, window=window)
    o = _round(o, act_dtype).reshape(t, hq * d)
    return _round(linear(o, W("o_proj.weight")), act_dtype)


def mlp_block(x, w, prefix: str, act_dtype=None):
    """down(silu(gate x) * up x)  (src/models/qwen3/model.py:232-237)."""
    dt = x.dtype
    g = _round(linear(x, w[f"{prefix}.mlp.gate_proj.weight"].to(dt)), act_dtype)
    u = _round(linear(x, w[f"{prefix}.mlp.up_proj.weight"].to(dt)), act_dtype)
    a = _round(silu_mul(g, u), act_dtype)
    return _round(linear(a, w[f"{prefix}.mlp.down_proj.weight"].to(dt)), act_dtype)


def decoder_layer(h, positions, w, prefix: str, cfg: dict, table, act_dtype=None, window=None):
    """r = x; x = norm(x); x = attn(x); x = r + x; r = x; x = norm(x); x = mlp(x); x = r + x
    (src/models/qwen3/model.py:278-298).  The residual stream h stays in compute precision."""
    dt = h.dtype
    eps = cfg["rms_norm_eps"]
    x = _round(rms_norm(h, w[f"{prefix}.input_layernorm.weight"].to(dt), eps), act_dtype)
    h = h + attention_block(x, positions, w, prefix, cfg, table, act_dtype, window)
    x = _round(rms_norm(h, w[f"{prefix}.post_attention_layernorm.weight"].to(dt), eps), act_dtype)
    h = h + mlp_block(x, w, prefix, act_dtype)
    return h


def rope_theta_of(cfg: dict) -> float:
    """rope_parameters.rope_theta first, else rope_theta (src/models/qwen3/config.py:23,35)."""
    rp = cfg.get("rope_parameters") or {}
    return float(rp.get("rope_theta", cfg.get("rope_theta")))


def forward_logits(cfg: dict, w: Dict[str, torch.Tensor], token_ids: List[int],
                   compute: torch.dtype = torch.float32,
                   act_dtype: Optional[torch.dtype] = None,
                   position_offset: int = 0, rows: Optional[List[int]] = None) -> torch.Tensor:
    """Logits [T, V] of one whole sequence: embedding, the layers in order, final
    norm, head (src/models/qwen3/model.py:349-359,420-422); the head is the
    embedding table when tie_word_embeddings (model.py:417-418).  With ``rows`` only those
    rows of the logits are formed (the layers still run on the whole sequence)."""
    ids = torch.tensor(token_ids, dtype=torch.long)
    t = ids.numel()
    positions = torch.arange(t) + position_offset
    table = rope_table(rope_theta_of(cfg), cfg["head_dim"], cfg["max_position_embeddings"])
    h = embedding(ids, w["model.embed_tokens.weight"]).to(compute)
    for i in range(cfg["num_hidden_layers"]):
        h = decoder_layer(h, positions, w, f"model.layers.{i}", cfg, table, act_dtype)
    if rows is not None:
        h = h[torch.tensor(list(rows), dtype=torch.long)]
    x = _round(rms_norm(h, w["model.norm.weight"].to(compute), cfg["rms_norm_eps"]), act_dtype)
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return linear(x, head.to(compute))


# ----------------------------------------------------------------------------
# sampling (the reference has greedy only: src/engine/executor.py:51-54)
# ----------------------------------------------------------------------------
def greedy(logits: torch.Tensor) -> List[int]:
    """argmax over the vocabulary, lowest index on ties (executor.py:54)."""
    return torch.argmax(logits, dim=-1).tolist()


def greedy_generate(cfg: dict, w, prompt: List[int], max_new_tokens: int,
                    compute=torch.float32, act_dtype=None) -> List[int]:
    """Whole-sequence recomputation for every new token; the first new token
    comes from the prompt's last logits and counts (src/engine/llm_engine.py:113-125)."""
    tokens = list(prompt)
    out = []
    for _ in range(max_new_tokens):
        logits = forward_logits(cfg, w, tokens, compute, act_dtype)
        nxt = int(torch.argmax(logits[-1]))
        out.append(nxt)
        tokens.append(nxt)
    return out


# ----------------------------------------------------------------------------
# temperature sampling (not in the reference, which is greedy only)
# ----------------------------------------------------------------------------
def uniform_number(seed: int, request: int, position: int) -> float:
    """The engine's rule for the one uniform number of a draw: the first 24 of the 64 bits (little
    endian) of blake2b-8 over the three numbers as little-endian int64, as a fraction of 2^24."""
    import hashlib
    import struct
    digest = hashlib.blake2b(struct.pack("<qqq", seed, request, position), digest_size=8).digest()
    return (int.from_bytes(digest, "little") >> 40) / float(1 << 24)


def sample_temperature(logits: torch.Tensor, temperature: float, u: float):
    """Inverse CDF of softmax(logits / temperature): the first token whose running sum of weights
    (in index order, 64-bit) exceeds u times the total.  Also returns how far u lies from the nearer
    edge of that token's interval, as a fraction of the total: a draw nearer to an edge than the
    logits are exact may fall on either side."""
    z = logits.double() / temperature
    w = torch.exp(z - z.max())
    cdf = torch.cumsum(w, dim=0) / w.sum()
    tok = int(torch.searchsorted(cdf, torch.tensor(u, dtype=torch.float64), right=True))
    tok = min(tok, logits.numel() - 1)
    lower = float(cdf[tok - 1]) if tok > 0 else 0.0
    return tok, min(u - lower, float(cdf[tok]) - u)
