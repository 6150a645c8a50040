"""Model folders whose weights are chosen so that the logits have a closed form, each pinning one
fact of the layer skeleton that random weights leave to the reading of the reference's text alone:
where the residual is taken, where each norm stands, which eps the per-head norms use and what the
scores are divided by.  Each case gives (config dict, tensors, token ids, expected logits), the
expectation being formed here from library routines and from parts that other tests pin; the CPU
tests hold the plain implementation against it, the GPU tests the engine, from the same folders."""
import json
import math
import os

import torch
import torch.nn.functional as F

from plain import qwen3_plain as P
from tiny import TINY_A, TINY_B, make_folder


def _base(tmp, which, std, **changes):
    """A tiny configuration's folder read back: (config dict with ``changes``, tensors in float32)."""
    folder = make_folder(tmp, which, dtype=torch.float32, std=std, norm_std=0.1)
    cfg, w = P.read_folder(folder)
    cfg = dict(cfg, **changes)
    return cfg, {k: v.clone() for k, v in w.items()}


def write_folder(folder, cfg, tensors):
    """config.json and model.safetensors as the engine's loader reads them."""
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def _ids(cfg, n, seed):
    return torch.randint(0, cfg["vocab_size"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def _head(cfg, w):
    return w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]


def _final(cfg, w, h):
    """Final norm, then the head (model.py:359,422), by library routines."""
    x = F.rms_norm(h, (h.shape[-1],), weight=w["model.norm.weight"], eps=cfg["rms_norm_eps"])
    return F.linear(x, _head(cfg, w))


def _layers(cfg):
    return [f"model.layers.{i}" for i in range(cfg["num_hidden_layers"])]


# ---- (a) every branch writes zeros: the stream passes the blocks untouched ----------------------
def stream_passes_untouched(tmp, which="A"):
    """o_proj = 0 and down_proj = 0 in every layer: x = residual + 0 twice a layer (model.py:291,296), so
    the logits are head(norm(E[ids])) (model.py:349,359,422).  A block that hands on the normed rows
    instead of the residual, or a model without its final norm, gives other logits."""
    cfg, w = _base(tmp, which, 0.3)
    for p in _layers(cfg):
        w[f"{p}.self_attn.o_proj.weight"].zero_()
        w[f"{p}.mlp.down_proj.weight"].zero_()
    ids = _ids(cfg, 11, 1)
    h = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    return cfg, w, ids, _final(cfg, w, h)


# ---- (b) the norms stand on the branches, not on the residual ------------------------------------
def first_norm_stands_on_the_branch(tmp, which="A"):
    """input_layernorm.weight = 0 (the attention's input is zero, so q = k = v = 0 and its output is
    o_proj(0) = 0) and down_proj = 0: the same logits as in (a).  A norm applied to the residual itself
    (x = norm(x) kept as the stream) would zero the stream."""
    cfg, w = _base(tmp, which, 0.3)
    for p in _layers(cfg):
        w[f"{p}.input_layernorm.weight"].zero_()
        w[f"{p}.mlp.down_proj.weight"].zero_()
    ids = _ids(cfg, 11, 2)
    h = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    return cfg, w, ids, _final(cfg, w, h)


def second_norm_stands_on_the_branch(tmp, which="B"):
    """post_attention_layernorm.weight = 0 while o_proj is not: the feed-forward sees zeros and gives
    down(silu(0) * 0) = 0, so the model is its attention blocks alone, each reading the norm of the
    stream and adding to the stream (model.py:280-296).  Formed here from the attention block, which its
    own tests pin, and library routines."""
    cfg, w = _base(tmp, which, 0.2)
    for p in _layers(cfg):
        w[f"{p}.post_attention_layernorm.weight"].zero_()
    ids = _ids(cfg, 9, 3)
    eps, d = cfg["rms_norm_eps"], cfg["head_dim"]
    table = P.rope_table(P.rope_theta_of(cfg), d, cfg["max_position_embeddings"])
    pos = torch.arange(len(ids))
    h = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    for p in _layers(cfg):
        x = F.rms_norm(h, (h.shape[-1],), weight=w[f"{p}.input_layernorm.weight"], eps=eps)
        h = h + P.attention_block(x, pos, w, p, cfg, table)
    return cfg, w, ids, _final(cfg, w, h)


# ---- (c) one eps for every norm, the per-head norms included --------------------------------------
def library_forward(cfg, w, ids, eps_layer, eps_heads, eps_final, scale):
    """The whole model by library routines (F.rms_norm, F.scaled_dot_product_attention with an explicit
    mask, F.silu, F.linear), with every eps and the score scale as arguments of their own, so that a test
    can say which of them the model's one ``rms_norm_eps`` and ``head_dim`` decide."""
    hq, hkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    T = len(ids)
    pos = torch.arange(T)
    table = P.rope_table(P.rope_theta_of(cfg), d, cfg["max_position_embeddings"])
    mask = pos[:, None] >= pos[None, :]
    h = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    for p in _layers(cfg):
        x = F.rms_norm(h, (h.shape[-1],), weight=w[f"{p}.input_layernorm.weight"], eps=eps_layer)
        q = F.linear(x, w[f"{p}.self_attn.q_proj.weight"]).view(T, hq, d)
        k = F.linear(x, w[f"{p}.self_attn.k_proj.weight"]).view(T, hkv, d)
        v = F.linear(x, w[f"{p}.self_attn.v_proj.weight"]).view(T, hkv, d)
        q = F.rms_norm(q, (d,), weight=w[f"{p}.self_attn.q_norm.weight"], eps=eps_heads)
        k = F.rms_norm(k, (d,), weight=w[f"{p}.self_attn.k_norm.weight"], eps=eps_heads)
        q, k = P.apply_rope(table, pos, q), P.apply_rope(table, pos, k)
        o = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                           attn_mask=mask[None, None], scale=scale, enable_gqa=True)[0].transpose(0, 1)
        h = h + F.linear(o.reshape(T, hq * d), w[f"{p}.self_attn.o_proj.weight"])
        x = F.rms_norm(h, (h.shape[-1],), weight=w[f"{p}.post_attention_layernorm.weight"], eps=eps_layer)
        a = F.silu(F.linear(x, w[f"{p}.mlp.gate_proj.weight"])) * F.linear(x, w[f"{p}.mlp.up_proj.weight"])
        h = h + F.linear(a, w[f"{p}.mlp.down_proj.weight"])
    x = F.rms_norm(h, (h.shape[-1],), weight=w["model.norm.weight"], eps=eps_final)
    return F.linear(x, _head(cfg, w))


def one_eps_for_every_norm(tmp, which="A"):
    """rms_norm_eps = 0.2, of the size of the rows' mean squares: the layer norms, the per-head norms
    (model.py:177-178) and the final norm (model.py:345) all take it.  Returns also the logits with 1e-6
    in the per-head norms alone, in the final norm alone and in the layer norms alone: all far from the
    expected."""
    eps = 0.2
    cfg, w = _base(tmp, which, 0.15, rms_norm_eps=eps)
    ids = _ids(cfg, 12, 4)
    s = 1.0 / math.sqrt(cfg["head_dim"])
    want = library_forward(cfg, w, ids, eps, eps, eps, s)
    others = {"per-head norms with another eps": library_forward(cfg, w, ids, eps, 1e-6, eps, s),
              "final norm with another eps": library_forward(cfg, w, ids, eps, eps, 1e-6, s),
              "layer norms with another eps": library_forward(cfg, w, ids, 1e-6, eps, eps, s)}
    return cfg, w, ids, want, others


# ---- (d) scores are divided by sqrt(head_dim), which is not hidden / heads ----------------------
def scale_is_one_over_root_head_dim(tmp):
    """Tiny B has heads of 32 while hidden / heads = 16 (config.py:46: scale = 1 / sqrt(head_dim)).  One
    layer, two tokens, down_proj = 0: token 0 sees itself alone and gets v0; token 1 gets
    v0 + (v1 - v0) sigmoid((q1.k1 - q1.k0) / sqrt(32)), the softmax over two keys in closed form.  Returns
    also the logits with sqrt(16), far from the expected."""
    cfg, w = _base(tmp, "B", 0.5, num_hidden_layers=1)
    w = {k: v for k, v in w.items() if not k.startswith("model.layers.") or k.startswith("model.layers.0.")}
    p = "model.layers.0"
    w[f"{p}.mlp.down_proj.weight"].zero_()
    ids = _ids(cfg, 2, 5)
    hq, hkv, d, eps = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["rms_norm_eps"]
    assert d == 32 and cfg["hidden_size"] // hq == 16
    table = P.rope_table(P.rope_theta_of(cfg), d, 8)
    pos = torch.arange(2)
    h = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"]).double()
    W = lambda name: w[f"{p}.{name}"].double()
    x = F.rms_norm(h, (h.shape[-1],), weight=W("input_layernorm.weight"), eps=eps)
    q = F.rms_norm((x @ W("self_attn.q_proj.weight").t()).view(2, hq, d), (d,), weight=W("self_attn.q_norm.weight"), eps=eps)
    k = F.rms_norm((x @ W("self_attn.k_proj.weight").t()).view(2, hkv, d), (d,), weight=W("self_attn.k_norm.weight"), eps=eps)
    v = (x @ W("self_attn.v_proj.weight").t()).view(2, hkv, d)
    q, k = P.apply_rope(table.double(), pos, q), P.apply_rope(table.double(), pos, k)

    def logits_with(divisor):
        o = torch.zeros(2, hq, d, dtype=torch.float64)
        for head in range(hq):
            kv = head // (hq // hkv)
            o[0, head] = v[0, kv]
            gate = torch.sigmoid((q[1, head] @ k[1, kv] - q[1, head] @ k[0, kv]) / divisor)
            o[1, head] = v[0, kv] + (v[1, kv] - v[0, kv]) * gate
        hh = h + o.reshape(2, hq * d) @ W("self_attn.o_proj.weight").t()
        xx = F.rms_norm(hh, (hh.shape[-1],), weight=w["model.norm.weight"].double(), eps=eps)
        return (xx @ _head(cfg, w).double().t()).float()

    return cfg, w, ids, logits_with(math.sqrt(32.0)), {"scores divided by sqrt(hidden / heads)": logits_with(math.sqrt(16.0))}


CASES = {
    "stream_passes_untouched": stream_passes_untouched,
    "first_norm_stands_on_the_branch": first_norm_stands_on_the_branch,
    "second_norm_stands_on_the_branch": second_norm_stands_on_the_branch,
    "one_eps_for_every_norm": one_eps_for_every_norm,
    "scale_is_one_over_root_head_dim": scale_is_one_over_root_head_dim,
}


def build(name, tmp):
    """(config, tensors, ids, expected logits, {what a mistake would give: its logits})."""
    out = CASES[name](tmp)
    return out if len(out) == 5 else (*out, {})


def relative_error(got, want):
    return float((got.double() - want.double()).abs().max()) / max(float(want.abs().max()), 1e-30)
