"""Steps of the shape that a server runs while requests keep arriving, against the plain
implementation: 20 and 64 requests that each decode one token, at contexts from a few dozen to
beyond 1024 and 2048 keys (the recorded step's buckets of 16 and 24 key splits of 128 keys; the split
decode is the reference's src/layers/fused_ops/attn.py:597-710), beside one request whose prompt arrives
in portions of 512, 300 and 77 tokens at positions 0, 1536 and 3000 (below and beyond the keys up to
which the prefill kernel leaves its walks uncut).  Heads of 128, as in the family's models; more than
16 single tokens, so that q and the new keys are prepared by the kernel of their own.  With recorded
graphs and without, in bfloat16 and in float32; every wanted row is compared; the cache pages are
poisoned.  The reference has no such steps (README.md:30-35 names them as missing): the contract is
that of its prefill attention (fused_ops/attn.py:184-195) applied to every entry of the batch.

And the head's product at the large models' widths against the whole vocabulary, in 64-bit on drawn
columns."""
import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import qwen3_plain as P
from qwen_engine_amd.config import Qwen3Config
from qwen_engine_amd.engine import ModelRunner, StepEntry
from qwen_engine_amd.kernels import ops
from qwen_engine_amd.parts import DecoderModel, Runtime
from qwen_engine_amd.weights import random_tensors

pytestmark = pytest.mark.gpu

TOL = {"float32": 1e-4, "bfloat16": 2e-2}       # of the largest reference logit of the request
ACT = {"float32": None, "bfloat16": torch.bfloat16}
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}

CFG = dict(architectures=["Qwen3ForCausalLM"], vocab_size=400, hidden_size=256, intermediate_size=320,
           num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=128,
           max_position_embeddings=4608, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False)
PORTIONS = ((0, 512), (1536, 300), (3000, 77))      # (first position, tokens) of the portions that run beside the single tokens
PROMPT = 3077


def tokens(n, seed):
    return torch.randint(0, CFG["vocab_size"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def lengths_of(n_dec):
    """Contexts of the requests that decode: 20 of them reach beyond 1024 keys but not 2048, 64 of them
    beyond 2048 as well; a few are short."""
    if n_dec == 20:
        return [7 + 97 * i for i in range(20)]                        # 7 .. 1850
    return [5 + (i * 37) % 2300 for i in range(60)] + [2049, 2200, 2290, 1024]


@pytest.fixture(scope="module")
def model_and_refs():
    cfg = Qwen3Config.from_dict(CFG)
    w = random_tensors(cfg, 21, dtype=torch.bfloat16, std=0.06, norm_std=0.05)
    for name in w:                      # (scores with a deviation above 2: the weight lies on some dozens of keys)
        if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
            w[name] = (w[name].float() * 1.5).to(torch.bfloat16)
    plain_w = {k: v.float() for k, v in w.items()}
    refs = {}

    def ref(dtype, n_dec):
        key = (dtype, n_dec)
        if key not in refs:
            lens = lengths_of(n_dec)
            reqs = [tokens(n + len(PORTIONS), 5000 + 100 * n_dec + i) for i, n in enumerate(lens)]
            prompt = tokens(PROMPT, 4999)
            rows = [[n + s for s in range(len(PORTIONS))] for n in lens]
            out = [P.forward_logits(CFG, plain_w, t, act_dtype=ACT[dtype], rows=r) for t, r in zip(reqs, rows)]
            prows = [a + n - 1 for a, n in PORTIONS]
            refs[key] = (lens, reqs, prompt, out, P.forward_logits(CFG, plain_w, prompt, act_dtype=ACT[dtype], rows=prows))
        return refs[key]

    return cfg, w, ref


@pytest.mark.parametrize("dtype,use_graphs", [("bfloat16", True), ("bfloat16", False), ("float32", True), ("float32", False)])
@pytest.mark.parametrize("n_dec", [20, 64])
def test_single_tokens_beside_a_portion_deep_in_a_context(model_and_refs, n_dec, dtype, use_graphs):
    cfg, w, ref = model_and_refs
    lens, reqs, prompt, want, want_portion = ref(dtype, n_dec)
    model = DecoderModel(cfg.to_model_spec())
    model.load(w, Runtime(torch.device("cuda:0"), TORCH[dtype]))
    pages = sum((n + len(PORTIONS)) // 16 + 1 for n in lens) + PROMPT // 16 + 2
    runner = ModelRunner(model, page_size=16, num_pages=pages, max_requests=n_dec + 1, use_graphs=use_graphs,
                         debug_poison=True)
    for i, (toks, n) in enumerate(zip(reqs, lens)):
        runner.add_request(i)
        runner.step([StepEntry(i, toks[:n], [])])
    runner.add_request("p")
    at = 0
    worst = 0.0
    for s, (first, n) in enumerate(PORTIONS):
        if at < first:                                    # the prompt's tokens between the portions, alone
            runner.step([StepEntry("p", prompt[at:first], [])])
        before = dict(runner.graph_steps_of)
        singles = [StepEntry(i, [reqs[i][lens[i] + s]], [0]) for i in range(n_dec)]
        portion = StepEntry("p", prompt[first:first + n], [n - 1])
        place = (0, n_dec // 2, n_dec)[s]                 # the portion first, in the middle, last among the entries
        entries = singles[:place] + [portion] + singles[place:]
        got = runner.step(entries).float().cpu()
        at = first + n
        assert got.shape[0] == n_dec + 1 and torch.isfinite(got).all()
        if use_graphs:
            assert runner.graph_steps_of["mixed"] == before["mixed"] + 1, "the step was not replayed from a recorded graph"
        row = 0
        for j, e in enumerate(entries):
            if e.req_id == "p":
                r = want_portion[s]
                err = float((got[row] - r).abs().max()) / float(want_portion.abs().max())
                assert err <= TOL[dtype], f"portion at {first} ({n} tokens): error {err}"
            else:
                r = want[e.req_id][s]
                err = float((got[row] - r).abs().max()) / float(want[e.req_id].abs().max())
                assert err <= TOL[dtype], f"request {e.req_id} (context {lens[e.req_id] + s}) beside the portion at {first}: error {err}"
            worst = max(worst, err)
            row += 1
    runner.cache.check_invariants()
    if use_graphs:
        # the key splits' bucket of the single tokens and whether the portion's keys are cut are part of a recorded step's key
        keys = [k for k in runner._graphs if k[0] == "mixed" and k[1] == ModelRunner.graph_rows(n_dec)]
        assert {k[3][0] for k in keys} == {(16 if n_dec == 20 else 24, False), (16 if n_dec == 20 else 24, True)}


@pytest.mark.parametrize("K", [4096, 5120])
def test_head_product_at_the_large_widths_against_the_whole_vocabulary(K):
    """logits = x . W^T with W [151 936, K] (src/models/qwen3/model.py:369-373,422), float32 out, for 1, 8, 16
    and 64 rows of a decode step at the 8B and 32B widths (up to 8 rows: one tile of outputs a block of the
    kernel for few rows, several rounds of chunks with the next in flight; 9 to 16: four tiles a block; 17 to
    64: the tiled kernel): compared in 64-bit on 3000 drawn columns and the last 100."""
    V = 151936
    g = torch.Generator().manual_seed(K)
    w = torch.empty(V, K, dtype=torch.bfloat16)
    for a in range(0, V, 16384):                   # (drawn in pieces: the 32-bit draws of the whole matrix are 3 GB)
        w[a:a + 16384] = (torch.randn(min(16384, V - a), K, generator=g) * 0.02).to(torch.bfloat16)
    w_dev = w.cuda()
    cols = torch.cat([torch.randint(0, V, (3000,), generator=g), torch.arange(V - 100, V)])
    w_cols = w[cols].double()
    for rows in (1, 8, 16, 64):
        x = torch.randn(rows, K, generator=g).to(torch.bfloat16)
        got = ops.gemm(x.cuda(), w_dev, out_dtype=torch.float32).cpu()
        assert got.shape == (rows, V) and torch.isfinite(got).all()
        want = x.double() @ w_cols.t()
        err = float((got[:, cols].double() - want).abs().max()) / float(want.abs().max())
        assert err < 2e-5, (rows, err)


@pytest.mark.parametrize("use_graphs", [True, False])
def test_greedy_steps_give_the_argmax_of_the_logits(model_and_refs, use_graphs):
    """step(..., greedy=True) returns the index of the largest logit of every wanted row (a recorded step
    picks it inside its graph): the same steps on a second runner that returns logits, for decode steps that
    are filled up to a recorded size, a portion of a round length, a portion beside single tokens in any
    order of the entries, and a step without wanted rows."""
    cfg, w, _ = model_and_refs
    model = DecoderModel(cfg.to_model_spec())
    model.load(w, Runtime(torch.device("cuda:0"), torch.bfloat16))
    runners = [ModelRunner(model, page_size=16, num_pages=200, max_requests=12, use_graphs=use_graphs, debug_poison=True)
               for _ in range(2)]
    prompts = [tokens(30 + 17 * i, 7000 + i) for i in range(11)]
    long = tokens(900, 7100)

    def both(entries):
        got = runners[0].step(entries, greedy=True)
        logits = runners[1].step(entries)
        assert isinstance(got, list) and got == logits.argmax(dim=1).tolist()
        return got

    for r in runners:
        for i in range(11):
            r.add_request(i)
        r.add_request("p")
    for i, p in enumerate(prompts):
        assert len(both([StepEntry(i, p, [len(p) - 1])])) == 1                      # a lone ragged portion
    last = [p[-1] for p in prompts]
    for step in range(3):                                                           # 11 rows: filled up to 16
        last = both([StepEntry(i, [last[i]], [0]) for i in range(11)])
    assert both([StepEntry("p", long[:256], [])]) == []                             # a portion of a round length, nothing wanted
    assert len(both([StepEntry("p", long[256:512], [255])])) == 1
    singles = [StepEntry(i, [last[i]], [0]) for i in range(11)]
    got = both(singles[:4] + [StepEntry("p", long[512:700], [187])] + singles[4:])  # the portion among the single tokens
    assert len(got) == 12
    got = both([StepEntry("p", long[700:830], [])] + [StepEntry(i, [got[i if i < 4 else i + 1]], [0]) for i in range(11)])
    assert len(got) == 11
    if use_graphs:
        assert runners[0].graph_steps_of == runners[1].graph_steps_of
        assert runners[0].graph_steps_of["decode"] == 3 and runners[0].graph_steps_of["portion"] == 2
        assert runners[0].graph_steps_of["mixed"] == 11 + 2
