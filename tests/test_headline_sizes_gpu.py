"""The engine at the sizes and context lengths that the measurements run at, against the plain
implementation, in float32 and in bfloat16.

(a) Two layers at the Qwen3-0.6B widths (src/models/qwen3/config.py:6-19: width 1024, 16 query heads
    on 8 key/value heads of 128, feed-forward 3072) with the whole tied vocabulary of 151 936: a prompt
    of 2048 tokens in one step and in portions of 512, then decoding with 1, 8 and 64 rows.
(b) A small model with heads of 128 and 4608 positions: one request decoded through the positions
    where the recorded decode graph changes (1024, 2048: the bucket of key splits,
    src/layers/fused_ops/attn.py:597-710 is the reference's split decode) and through 4095..4099 (33 splits
    of 128 keys), and 24 requests of different lengths decoding together beyond 1024 keys.

The q and k norm weights are scaled by 1.5, so that a query's weight lies on some dozens of keys
anywhere in the context instead of evenly on all of them (scores with a deviation of 2.25: the
largest of 2000 carries a tenth of the weight).  More would be better for showing a wrong page, but
the rounding of q and k to bfloat16 moves a score in proportion to its size: doubled weights bring
the differences between two correct bfloat16 computations to 1.7 % of the largest logit, at 1.5
they stay below 1.4 %.  What a single key far away does to the kernels is tested on the kernels
alone.  The cache pages are poisoned (NaN when handed out and when given back)."""
import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import qwen3_plain as P
from qwen_engine_amd.config import Qwen3Config
from qwen_engine_amd.engine import ModelRunner, StepEntry
from qwen_engine_amd.parts import DecoderModel, Runtime
from qwen_engine_amd.weights import random_tensors

pytestmark = pytest.mark.gpu

TOL = {"float32": 1e-4, "bfloat16": 2e-2}       # of the largest reference logit of the request
ACT = {"float32": None, "bfloat16": torch.bfloat16}
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}

CFG_06B = dict(architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=1024, intermediate_size=3072,
               num_hidden_layers=2, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
               max_position_embeddings=4096, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=True)
CFG_LONG = dict(architectures=["Qwen3ForCausalLM"], vocab_size=400, hidden_size=256, intermediate_size=320,
                num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=128,
                max_position_embeddings=4608, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False)


def make_weights(cfg_dict, seed, std):
    cfg = Qwen3Config.from_dict(cfg_dict)
    w = random_tensors(cfg, seed, dtype=torch.bfloat16, std=std, norm_std=0.05)
    for name in w:
        if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
            w[name] = (w[name].float() * 1.5).to(torch.bfloat16)
    return cfg, w, {k: v.float() for k, v in w.items()}


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def worst_error(got, ref_rows):
    """Largest error of the rows, as a fraction of the largest reference logit."""
    return float((got.float().cpu() - ref_rows).abs().max()) / float(ref_rows.abs().max())


# ---- (a) the 0.6B widths with the whole vocabulary -------------------------------------------------
LONG = (2048, 1500, 1100, 700, 300, 100, 50, 17)          # prompts of the eight requests that decode at 8 rows
WANT = [0, 1, 15, 16, 511, 512, 1023, 1024, 2047]         # places of the long prompt whose logits are compared


@pytest.fixture(scope="module")
def headline():
    cfg, w, plain_w = make_weights(CFG_06B, 11, 0.02)
    V = CFG_06B["vocab_size"]
    lengths = list(LONG) + [5 + (13 * i) % 110 for i in range(56)]
    # every request decodes after its prompt: the first alone (3 tokens), the first eight together (2), all 64 (2)
    extra = [7] + [4] * 7 + [2] * 56
    reqs = [tokens(n + e, V, 700 + i) for i, (n, e) in enumerate(zip(lengths, extra))]
    refs = {}
    for dt, act in ACT.items():
        refs[dt] = []
        for i, toks in enumerate(reqs):
            rows = (WANT if i == 0 else []) + list(range(lengths[i] - 1, len(toks)))
            refs[dt].append((rows, P.forward_logits(CFG_06B, plain_w, toks, act_dtype=act, rows=rows)))
    return cfg, w, lengths, reqs, refs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_small_model_widths_with_the_whole_vocabulary(headline, dtype):
    cfg, w, lengths, reqs, refs = headline
    model = DecoderModel(cfg.to_model_spec())
    model.load(w, Runtime(torch.device("cuda:0"), TORCH[dtype]))
    runner = ModelRunner(model, page_size=16, num_pages=900, max_requests=64, debug_poison=True)
    tol = TOL[dtype]

    def ref_of(i, positions):
        rows, logits = refs[dtype][i]
        return logits[[rows.index(p) for p in positions]]

    # the prompt of 2048 tokens in portions of 512
    runner.add_request("portions")
    got = []
    for a in range(0, 2048, 512):
        want = [p - a for p in WANT if a <= p < a + 512]
        got.append(runner.step([StepEntry("portions", reqs[0][a:a + 512], want)]))
    assert worst_error(torch.cat(got), ref_of(0, WANT)) <= tol, "a prompt of 2048 tokens in portions of 512"
    runner.free_request("portions")
    # ... and in one step; then three tokens decoded alone
    runner.add_request(0)
    got = runner.step([StepEntry(0, reqs[0][:2048], WANT)])
    assert worst_error(got, ref_of(0, WANT)) <= tol, "a prompt of 2048 tokens in one step"
    done = {0: 2048}
    for _ in range(3):
        p = done[0]
        got = runner.step([StepEntry(0, [reqs[0][p]], [0])])
        assert worst_error(got, ref_of(0, [p])) <= tol, f"decoding alone at position {p}"
        done[0] = p + 1
    # eight requests decode together, then all 64
    for n_live in (8, 64):
        for i in range(n_live):
            if i not in done:
                runner.add_request(i)
                runner.step([StepEntry(i, reqs[i][:lengths[i]], [])])
                done[i] = lengths[i]
        for _ in range(2):
            got = runner.step([StepEntry(i, [reqs[i][done[i]]], [0]) for i in range(n_live)])
            assert torch.isfinite(got).all()
            for i in range(n_live):
                err = worst_error(got[i:i + 1], ref_of(i, [done[i]]))
                assert err <= tol, f"{n_live} rows: request {i} at position {done[i]}: error {err}"
                done[i] += 1
    if dtype == "bfloat16":
        # every decode step went through a recorded graph, and so did the two portions of 512 tokens
        # that want at most one row of logits
        assert runner.graph_steps_of["decode"] == 3 + 2 + 2 and runner.graph_steps_of["portion"] == 2
        assert runner.graph_steps_of["mixed"] == 63           # the other requests' prompts, each filled up to a round length
    runner.cache.check_invariants()


# ---- (b) long contexts through the recorded decode graphs ------------------------------------------
@pytest.fixture(scope="module")
def long_model():
    cfg, w, plain_w = make_weights(CFG_LONG, 12, 0.06)
    return cfg, w, plain_w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_across_the_positions_where_the_graph_changes(long_model, dtype):
    """Decoded one by one: 1000..1100 (the bucket of key splits changes at 1024), 2040..2060 (at 2048),
    4090..4099 (33 splits from 4096 on); the tokens between are prompt portions."""
    cfg, w, plain_w = long_model
    toks = tokens(4100, CFG_LONG["vocab_size"], 31)
    decoded = list(range(1000, 1100)) + list(range(2040, 2060)) + list(range(4090, 4100))
    ref = P.forward_logits(CFG_LONG, plain_w, toks, act_dtype=ACT[dtype], rows=decoded)
    model = DecoderModel(cfg.to_model_spec())
    model.load(w, Runtime(torch.device("cuda:0"), TORCH[dtype]))
    runner = ModelRunner(model, page_size=16, num_pages=260, max_requests=1, debug_poison=True)
    runner.add_request("r")
    got, pos = [], 0
    for start, end in ((1000, 1100), (2040, 2060), (4090, 4100)):
        runner.step([StepEntry("r", toks[pos:start], [])])
        for p in range(start, end):
            got.append(runner.step([StepEntry("r", [toks[p]], [0])]))
        pos = end
    got = torch.cat(got).float().cpu()
    err = (got - ref).abs().amax(dim=1) / float(ref.abs().max())
    bad = torch.nonzero(err > TOL[dtype])
    assert bad.numel() == 0, f"first wrong position {decoded[int(bad[0])]}, error {float(err[bad[0]])}"
    if dtype == "bfloat16":
        assert runner.graph_steps_of["decode"] == len(decoded) and runner.graphs_recorded >= 4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_twenty_four_requests_decode_together_beyond_1024_keys(long_model, dtype):
    cfg, w, plain_w = long_model
    lengths = [1030 + 37 * i for i in range(24)]
    reqs = [tokens(n + 3, CFG_LONG["vocab_size"], 900 + i) for i, n in enumerate(lengths)]
    model = DecoderModel(cfg.to_model_spec())
    model.load(w, Runtime(torch.device("cuda:0"), TORCH[dtype]))
    runner = ModelRunner(model, page_size=16, num_pages=24 * 120, max_requests=24, debug_poison=True)
    for i, (toks, n) in enumerate(zip(reqs, lengths)):
        runner.add_request(i)
        runner.step([StepEntry(i, toks[:n], [])])
    outs = [runner.step([StepEntry(i, [reqs[i][lengths[i] + s]], [0]) for i in range(24)]).float().cpu()
            for s in range(3)]
    for i, (toks, n) in enumerate(zip(reqs, lengths)):
        ref = P.forward_logits(CFG_LONG, plain_w, toks, act_dtype=ACT[dtype], rows=[n, n + 1, n + 2])
        for s in range(3):
            err = float((outs[s][i] - ref[s]).abs().max()) / float(ref.abs().max())
            assert err <= TOL[dtype], f"request {i} (prompt {n}), step {s}: error {err}"


# ---- (c) portions of prompts deep in a context: the prefill kernel's key segments -------------------
@pytest.mark.parametrize("use_graphs", [True, False])
@pytest.mark.parametrize("heads", [(4, 2, 128), (8, 1, 64)])
def test_portions_deep_in_a_context(heads, use_graphs):
    """A prompt of some 4000 tokens in portions of 2 to 1500 tokens: from 1024 keys on, a portion of
    few tiles has its keys cut into segments whose partial results a second kernel merges, and a
    portion of a round length is replayed from a graph recorded for its bucket of keys.  The last
    row of every portion against the plain implementation (src/layers/fused_ops/attn.py:243-420 is the
    reference's attention over a paged cache, without such segments)."""
    hq, hkv, d = heads
    cfg_dict = dict(CFG_LONG, num_attention_heads=hq, num_key_value_heads=hkv, head_dim=d)
    cfg, w, plain_w = make_weights(cfg_dict, 13, 0.06)
    sizes = [1500, 512, 2, 256, 640, 17, 384, 128, 512, 77]
    L = sum(sizes)
    toks = tokens(L, cfg_dict["vocab_size"], 41)
    ends = [sum(sizes[:i + 1]) for i in range(len(sizes))]
    ref = P.forward_logits(cfg_dict, plain_w, toks, act_dtype=torch.bfloat16, rows=[e - 1 for e in ends])
    model = DecoderModel(cfg.to_model_spec())
    model.load(w, Runtime(torch.device("cuda:0"), torch.bfloat16))
    runner = ModelRunner(model, page_size=16, num_pages=L // 16 + 3, max_requests=1, use_graphs=use_graphs,
                         debug_poison=True)
    runner.add_request("r")
    got, a = [], 0
    for n in sizes:
        got.append(runner.step([StepEntry("r", toks[a:a + n], [n - 1])]))
        a += n
    got = torch.cat(got).float().cpu()
    assert torch.isfinite(got).all()
    err = (got - ref).abs().amax(dim=1) / float(ref.abs().max())
    bad = torch.nonzero(err > TOL["bfloat16"])
    assert bad.numel() == 0, f"first wrong portion ends at {ends[int(bad[0])]}, error {float(err[bad[0]])}"
    if use_graphs:
        # 512 (twice), 256, 640 and 384 tokens, all beyond the keys up to which nothing is cut; the other
        # portions are filled up to 1536 and (four of them) to 128 rows and replayed as well
        assert runner.graph_steps_of == {"decode": 0, "portion": 5, "mixed": 5} and runner.graphs_recorded == 4 + 2
    runner.cache.check_invariants()
