"""What pins the plain implementation beside the reference's text (CPU): the vectors
of the reference's own operator tests, special cases that reduce to a library routine,
and invariants; each chosen so that a plausible mistake fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

from plain import qwen3_plain as P
from tiny import TINY_A, TINY_B, make_folder


def rand(*shape, seed=0, dtype=torch.float32):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=dtype)


# ---- RMSNorm ----------------------------------------------------------------------------
def test_rms_norm_is_the_library_routine_at_the_reference_test_shape():
    x = torch.rand(32, 2048, generator=torch.Generator().manual_seed(1))     # layernorm.py:216-226,270
    w = rand(2048, seed=2)
    got = P.rms_norm(x, w, 1e-6)
    want = F.rms_norm(x, (2048,), weight=w, eps=1e-6)                      # layernorm.py:209-214
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)


def test_rms_norm_invariants():
    x = rand(5, 3, 48, seed=3)
    ones = torch.ones(48)
    y = P.rms_norm(x, ones, 1e-12)
    torch.testing.assert_close((y * y).mean(-1), torch.ones(5, 3), rtol=1e-5, atol=1e-6)   # rows have RMS 1
    torch.testing.assert_close(P.rms_norm(7.5 * x, ones, 1e-12), y, rtol=1e-5, atol=1e-6)  # scale invariant
    w = rand(48, seed=4)
    flat = P.rms_norm(x.reshape(15, 48), w, 1e-6).reshape(5, 3, 48)
    torch.testing.assert_close(P.rms_norm(x, w, 1e-6), flat)              # 3-D = rows sharing w
    # eps sits inside the root, next to the mean: a zero row stays zero and finite
    assert torch.equal(P.rms_norm(torch.zeros(2, 8), torch.ones(8), 1e-6), torch.zeros(2, 8))
    big_eps = P.rms_norm(torch.full((1, 4), 2.0), torch.ones(4), 5.0)
    torch.testing.assert_close(big_eps, torch.full((1, 4), 2.0 / 3.0))     # 2 / sqrt(4 + 5)


# ---- linear, embedding, silu.mul --------------------------------------------------------------
def test_linear_embedding_silu_reduce_to_library_routines():
    x, w = rand(256, 512, seed=5), rand(1024, 512, seed=6)                 # linear.py:188-201,255
    torch.testing.assert_close(P.linear(x, w), F.linear(x, w), rtol=1e-4, atol=1e-4)
    b = rand(1024, seed=7)
    torch.testing.assert_close(P.linear(x, w, b), F.linear(x, w, b), rtol=1e-4, atol=1e-4)
    ids = torch.randint(0, 1024, (32,), generator=torch.Generator().manual_seed(8))
    table = rand(1024, 2048, seed=9)                                       # embedding.py:140-151,196
    assert torch.equal(P.embedding(ids, table), F.embedding(ids, table))
    g, u = rand(256, 2048, seed=10), rand(256, 2048, seed=11)              # silumul.py:160-176,225
    torch.testing.assert_close(P.silu_mul(g, u), F.silu(g) * u, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(P.silu_mul(g, torch.ones_like(g)), F.silu(g), rtol=1e-5, atol=1e-6)
    assert torch.equal(P.silu_mul(torch.zeros(3), u[0, :3]), torch.zeros(3))


# ---- rotation -------------------------------------------------------------------------------
def test_rope_table_rows():
    t = P.rope_table(10000.0, 8, 16)
    assert t.shape == (16, 8)
    torch.testing.assert_close(t[0], torch.tensor([1., 1, 1, 1, 0, 0, 0, 0]))
    freqs = torch.tensor([1.0, 10000 ** -0.25, 10000 ** -0.5, 10000 ** -0.75])
    torch.testing.assert_close(t[5, :4], torch.cos(5 * freqs))
    torch.testing.assert_close(t[5, 4:], torch.sin(5 * freqs))


def test_rope_pairs_feature_i_with_i_plus_half_and_turns_counterclockwise():
    d = 8
    t = P.rope_table(10000.0, d, 4)
    x = torch.zeros(1, 1, d)
    x[0, 0, 0] = 1.0
    y = P.apply_rope(t, torch.tensor([1]), x)[0, 0]
    want = torch.zeros(d)
    want[0], want[d // 2] = math.cos(1.0), math.sin(1.0)   # interleaved pairing would put sin at index 1,
    torch.testing.assert_close(y, want)                     # a wrong sign would give -sin
    x = torch.zeros(1, 1, d)
    x[0, 0, d // 2 + 1] = 1.0
    y = P.apply_rope(t, torch.tensor([2]), x)[0, 0]
    f1 = 10000 ** -0.25
    want = torch.zeros(d)
    want[1], want[d // 2 + 1] = -math.sin(2 * f1), math.cos(2 * f1)
    torch.testing.assert_close(y, want)


def test_rope_invariants_at_the_reference_test_shape():
    d = 128
    t = P.rope_table(1e6, d, 2048)
    pos = torch.randint(0, 2048, (32,), generator=torch.Generator().manual_seed(12))   # rope.py:276-300,359-364
    q, k = rand(32, 32, d, seed=13), rand(32, 16, d, seed=14)
    rq, rk = P.apply_rope(t, pos, q), P.apply_rope(t, pos, k)
    assert torch.equal(P.apply_rope(t, torch.zeros(32, dtype=torch.long), q), q)       # position 0: identity
    pair = lambda z: z[..., :d // 2] ** 2 + z[..., d // 2:] ** 2
    torch.testing.assert_close(pair(rq), pair(q), rtol=1e-4, atol=1e-5)                # each pair keeps its length
    # <rope(q, m), rope(k, n)> depends on m - n only
    a, b = rand(1, 1, d, seed=15), rand(1, 1, d, seed=16)
    dot = lambda m, n: (P.apply_rope(t, torch.tensor([m]), a) * P.apply_rope(t, torch.tensor([n]), b)).sum()
    torch.testing.assert_close(dot(17, 5), dot(1012, 1000), rtol=1e-3, atol=1e-3)
    assert abs(dot(17, 5) - dot(17, 6)) > 1e-3


# ---- attention --------------------------------------------------------------------------------
def test_attention_without_mask_is_the_library_routine():
    q, k, v = rand(7, 4, 16, seed=20), rand(7, 4, 16, seed=21), rand(7, 4, 16, seed=22)
    got = P.attention(q, k, v, 0.3, causal=False)
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None],
                                          v.transpose(0, 1)[None], scale=0.3)[0].transpose(0, 1)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)


def test_causal_attention_with_cached_prefix_is_the_reference_twin():
    # 5 new tokens after 6 cached ones, explicit mask q_abs_pos >= k_abs_pos (attn.py:767-780)
    hq, hkv, d = 6, 2, 16
    q, k, v = rand(5, hq, d, seed=23), rand(11, hkv, d, seed=24), rand(11, hkv, d, seed=25)
    got = P.attention(q, k, v, 0.25)
    mask = (6 + torch.arange(5))[:, None] >= torch.arange(11)[None, :]
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None],
                                          v.transpose(0, 1)[None], attn_mask=mask[None, None],
                                          scale=0.25, enable_gqa=True)[0].transpose(0, 1)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)
    # grouped = each kv head repeated for the heads of its group, in blocks (h // group)
    rep = P.attention(q, k.repeat_interleave(3, dim=1), v.repeat_interleave(3, dim=1), 0.25)
    torch.testing.assert_close(got, rep)


def test_attention_edge_cases():
    q, k, v = rand(3, 2, 8, seed=26), rand(3, 1, 8, seed=27), rand(3, 1, 8, seed=28)
    out = P.attention(q, k, v, 1.0)
    torch.testing.assert_close(out[0], v[0].expand(2, 8))          # the first token sees one key: itself
    one_head = P.attention(q[:, :1], k, v, 1.0)
    torch.testing.assert_close(one_head, out[:, :1])
    # a window of 1 returns each token's own value; a window as long as the sequence changes nothing
    torch.testing.assert_close(P.attention(q, k, v, 1.0, window=1), v.expand(3, 2, 8))
    torch.testing.assert_close(P.attention(q, k, v, 1.0, window=3), out)
    w2 = P.attention(q, k, v, 1.0, window=2)
    torch.testing.assert_close(w2[:2], out[:2])
    assert not torch.allclose(w2[2], out[2])


# ---- whole model ----------------------------------------------------------------------------------
@pytest.mark.parametrize("which", ["A", "B"])
def test_logits_depend_on_distances_only(tmp_path, which):
    folder = make_folder(tmp_path, which, dtype=torch.float32, std=0.05)
    cfg, w = P.read_folder(folder)
    toks = torch.randint(0, cfg["vocab_size"], (20,), generator=torch.Generator().manual_seed(3)).tolist()
    base = P.forward_logits(cfg, w, toks)
    assert base.shape == (20, cfg["vocab_size"])
    shifted = P.forward_logits(cfg, w, toks, position_offset=37)
    torch.testing.assert_close(shifted, base, rtol=1e-3, atol=2e-4)
    # causal: a later token does not change earlier logits
    other = P.forward_logits(cfg, w, toks[:12] + [(toks[12] + 1) % cfg["vocab_size"]] + toks[13:])
    torch.testing.assert_close(other[:12], base[:12])
    assert not torch.allclose(other[12:], base[12:])
    f64 = P.forward_logits(cfg, w, toks, compute=torch.float64)
    torch.testing.assert_close(base.double(), f64, rtol=1e-4, atol=1e-5)


def test_tied_head_is_the_embedding_table(tmp_path):
    folder = make_folder(tmp_path, "A", dtype=torch.float32, std=0.05)
    cfg, w = P.read_folder(folder)
    assert "lm_head.weight" not in w
    toks = [1, 2, 3, 4]
    base = P.forward_logits(cfg, w, toks)
    untied = dict(cfg, tie_word_embeddings=False)
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"]
    torch.testing.assert_close(P.forward_logits(untied, w2, toks), base)


def test_norm_comes_before_rotation_and_only_without_bias(tmp_path):
    folder = make_folder(tmp_path, "B", dtype=torch.float32, std=0.05)
    cfg, w = P.read_folder(folder)
    x = rand(6, cfg["hidden_size"], seed=30)
    pos = torch.arange(6)
    table = P.rope_table(P.rope_theta_of(cfg), cfg["head_dim"], 64)
    w = dict(w)
    base = P.attention_block(x, pos, w, "model.layers.0", cfg, table)
    # scaling q_proj changes nothing when q is normalised per head afterwards (up to eps = 1e-5
    # beside a mean square near 0.2: a relative change of some 1e-5 in the scores)
    w["model.layers.0.self_attn.q_proj.weight"] = 3.0 * w["model.layers.0.self_attn.q_proj.weight"]
    torch.testing.assert_close(P.attention_block(x, pos, w, "model.layers.0", cfg, table), base, rtol=1e-3, atol=2e-5)
    # with bias there is no q/k norm (model.py:204-206): the same scaling now matters
    biased = dict(cfg, attention_bias=True)
    for n, width in (("q", 192), ("k", 32), ("v", 32)):
        w[f"model.layers.0.self_attn.{n}_proj.bias"] = torch.zeros(width)
    a = P.attention_block(x, pos, w, "model.layers.0", biased, table)
    w["model.layers.0.self_attn.q_proj.weight"] = w["model.layers.0.self_attn.q_proj.weight"] / 3.0
    b = P.attention_block(x, pos, w, "model.layers.0", biased, table)
    assert not torch.allclose(a, b, rtol=1e-3, atol=1e-5)


def test_the_per_head_norm_runs_before_the_rotation(tmp_path):
    """model.py:204-208: q and k are normed per head, then rotated.  With norm weights that are zero on
    the first half of the head, the normed head is [0 | x2], and its rotation [-sin x2 | cos x2]: the
    score of a query at i and a key at j is sum_d cos((i - j) f_d) x2q_d x2k_d, a function of the
    distance only.  Had the rotation come first, the weights would have cut the rotated head to
    [0 | sin x1 + cos x2] and the scores would be others.  The expected output is formed here from
    that closed form, without the functions that rotate."""
    folder = make_folder(tmp_path, "B", dtype=torch.float32, std=0.3)
    cfg, w = P.read_folder(folder)
    w = dict(w)
    hq, hkv, d, eps = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["rms_norm_eps"]
    half = d // 2
    mask = torch.cat([torch.zeros(half), torch.ones(half)])
    pre = "model.layers.0.self_attn"
    w[f"{pre}.q_norm.weight"] = mask * (1.0 + 0.1 * rand(d, seed=41))
    w[f"{pre}.k_norm.weight"] = mask * (1.0 + 0.1 * rand(d, seed=42))
    T = 9
    x = rand(T, cfg["hidden_size"], seed=40)
    pos = torch.arange(T) + 3                               # no token at position 0, where a rotation does nothing
    theta = P.rope_theta_of(cfg)
    table = P.rope_table(theta, d, 64)
    got = P.attention_block(x, pos, w, "model.layers.0", cfg, table)

    q = (x @ w[f"{pre}.q_proj.weight"].t()).view(T, hq, d).double()
    k = (x @ w[f"{pre}.k_proj.weight"].t()).view(T, hkv, d).double()
    v = (x @ w[f"{pre}.v_proj.weight"].t()).view(T, hkv, d).double()
    x2q = (q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * w[f"{pre}.q_norm.weight"].double())[..., half:]
    x2k = (k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * w[f"{pre}.k_norm.weight"].double())[..., half:]
    f = theta ** (-torch.arange(half, dtype=torch.float64) / half)
    dist = (pos[:, None] - pos[None, :]).double()
    cosd = torch.cos(dist[:, :, None] * f)                  # [i, j, d]
    out = torch.zeros(T, hq, d, dtype=torch.float64)
    for h in range(hq):
        kv = h // (hq // hkv)
        s = torch.einsum("id,jd,ijd->ij", x2q[:, h], x2k[:, kv], cosd) / (d ** 0.5)
        s = s.masked_fill(dist < 0, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, kv]
    want = out.reshape(T, hq * d) @ w[f"{pre}.o_proj.weight"].double().t()
    torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-5)
    # and the closed form is not blind to the order: with the rotation first the result is another
    qr = P.apply_rope(table, pos, (x @ w[f"{pre}.q_proj.weight"].t()).view(T, hq, d))
    kr = P.apply_rope(table, pos, (x @ w[f"{pre}.k_proj.weight"].t()).view(T, hkv, d))
    qn = P.rms_norm(qr, w[f"{pre}.q_norm.weight"], eps)
    kn = P.rms_norm(kr, w[f"{pre}.k_norm.weight"], eps)
    other = P.attention(qn, kn, v.float(), 1.0 / d ** 0.5, pos, pos).reshape(T, hq * d) @ w[f"{pre}.o_proj.weight"].t()
    assert float((other.double() - want).abs().max()) > 100 * float((got.double() - want).abs().max()) + 1e-3


def test_greedy_takes_the_lowest_index_on_ties():
    assert P.greedy(torch.tensor([[1.0, 3.0, 3.0, 2.0], [0.0, 0.0, 0.0, 0.0]])) == [1, 0]


def test_temperature_draw_is_the_inverse_cdf_of_the_softmax():
    logits = torch.tensor([0.3, -1.0, 2.0, 0.3, 1.1])
    p = torch.softmax(logits.double() / 0.7, dim=0)
    edges = torch.cumsum(p, 0)
    # a draw just inside each token's interval gives that token; the margin is the distance to its edge
    for tok in range(5):
        lo = float(edges[tok - 1]) if tok else 0.0
        got, margin = P.sample_temperature(logits, 0.7, lo + 0.25 * float(p[tok]))
        assert got == tok and abs(margin - 0.25 * float(p[tok])) < 1e-12
    assert P.sample_temperature(logits, 0.7, 0.0)[0] == 0 and P.sample_temperature(logits, 0.7, 0.999999)[0] == 4
    # over evenly spread draws the tokens come with the softmax's frequencies
    n = 20000
    counts = torch.zeros(5)
    for i in range(n):
        counts[P.sample_temperature(logits, 0.7, (i + 0.5) / n)[0]] += 1
    assert float((counts / n - p.float()).abs().max()) < 1e-3
    # a low temperature draws the largest logit whatever the number
    assert all(P.sample_temperature(logits, 0.01, u)[0] == 2 for u in (1e-9, 0.3, 0.9999))
    # the uniform number: 24 bits, fixed by its three arguments, different for neighbours
    u = P.uniform_number(5, 2, 9)
    assert 0.0 <= u < 1.0 and u * (1 << 24) == int(u * (1 << 24)) and u == P.uniform_number(5, 2, 9)
    assert len({P.uniform_number(5, 2, k) for k in range(50)}) == 50


# ---- the layer skeleton, by weights that give the logits a closed form -----------------------------
import skeleton


@pytest.mark.parametrize("name", sorted(skeleton.CASES))
def test_skeleton_by_closed_forms(tmp_path, name):
    """Where the residual is taken, where the norms stand, the final norm, the one eps and the scores'
    divisor (model.py:278-298,345-359,177-178; config.py:46), each by a model whose logits are known
    without running the plain implementation; and each expectation is far from what the mistake it
    guards against would give."""
    cfg, w, ids, want, mistakes = skeleton.build(name, tmp_path)
    got = P.forward_logits(cfg, w, ids)
    assert skeleton.relative_error(got, want) < 2e-5
    for what, other in mistakes.items():
        assert skeleton.relative_error(other, want) > 1e-2, what


def test_skeleton_cases_tell_the_mistakes_apart(tmp_path):
    """The closed forms are not blind: a block that keeps the normed rows as its stream, a model without
    its final norm and a norm on the residual all miss them by far."""
    cfg, w, ids, want, _ = skeleton.build("stream_passes_untouched", tmp_path)
    E = w["model.embed_tokens.weight"][torch.tensor(ids)]
    no_final_norm = E @ w["model.embed_tokens.weight"].t()
    assert skeleton.relative_error(no_final_norm, want) > 1e-2
    normed_stream = E
    for i in range(cfg["num_hidden_layers"]):                       # x = norm(x) kept as the stream
        normed_stream = P.rms_norm(normed_stream, w[f"model.layers.{i}.input_layernorm.weight"], cfg["rms_norm_eps"])
        normed_stream = P.rms_norm(normed_stream, w[f"model.layers.{i}.post_attention_layernorm.weight"], cfg["rms_norm_eps"])
    wrong = P.linear(P.rms_norm(normed_stream, w["model.norm.weight"], cfg["rms_norm_eps"]), w["model.embed_tokens.weight"])
    assert skeleton.relative_error(wrong, want) > 1e-2
    cfg, w, ids, want, _ = skeleton.build("first_norm_stands_on_the_branch", tmp_path)
    assert skeleton.relative_error(torch.zeros_like(want), want) > 0.5   # a zeroed stream gives zero logits
