"""Trace replay on the GPU against the plain implementation: the same requests whole,
with the last 32 tokens decoded one by one, in portions of changing size, and mixed
with other requests so that pages are used again; in float32 and in bfloat16."""
import os

import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import qwen3_plain as P
from tiny import TINY, make_folder
import traces

pytestmark = pytest.mark.gpu

# error allowed, as a fraction of the largest reference logit of the request
TOL = {"float32": 1e-4, "bfloat16": 2e-2}
ACT = {"float32": None, "bfloat16": torch.bfloat16}
LENGTHS = {"A": (70, 97, 133, 150, 41, 66), "B": (150, 65, 88, 129, 200, 77), "C": (100, 64, 131, 80, 45, 190),
           "D": (300, 130, 257, 90, 411, 64), "E": (350, 66, 257, 129, 480, 90)}


def make_requests(cfg, which):
    g = torch.Generator().manual_seed(100 + ord(which))
    return {f"r{i}": torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist()
            for i, n in enumerate(LENGTHS[which])}


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    """Per tiny configuration: the folder, the requests and the plain logits for both precisions."""
    tmp = tmp_path_factory.mktemp("models")
    out = {}
    for which in "ABCDE":
        folder = make_folder(tmp, which, dtype=torch.bfloat16, std=0.05)
        cfg, w = P.read_folder(folder)
        reqs = make_requests(cfg, which)
        ref = {dt: {rid: P.forward_logits(cfg, w, toks, act_dtype=ACT[dt]) for rid, toks in reqs.items()}
               for dt in TOL}
        out[which] = (folder, cfg, reqs, ref)
    return out


def check(trace, case, dtype, tmp_path, which, program=False):
    folder, cfg, reqs, ref = case
    out_dir = str(tmp_path / "out")
    page = TINY[which][2]
    (traces.run_program if program else traces.run_in_process)(trace, folder, dtype, out_dir, page)
    got = traces.collect(trace, out_dir, cfg["vocab_size"])
    bad, worst = traces.first_mismatch(got, ref[dtype], TOL[dtype])
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"
    return worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E"])
def test_whole_requests(cases, tmp_path, which, dtype):
    check(traces.whole(cases[which][2]), cases[which], dtype, tmp_path, which)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E"])
def test_last_32_tokens_one_by_one(cases, tmp_path, which, dtype):
    check(traces.tail_decoded(cases[which][2]), cases[which], dtype, tmp_path, which)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E"])
def test_portions_of_changing_size(cases, tmp_path, which, dtype):
    check(traces.portions(cases[which][2]), cases[which], dtype, tmp_path, which)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E"])
def test_mixed_with_pages_used_again(cases, tmp_path, which, dtype):
    trace = traces.mixed(cases[which][2], seed=7)
    assert max(len(s["entries"]) for s in trace.steps) >= 3
    total = sum(traces.round64(len(t)) for t in cases[which][2].values())
    assert trace.max_tokens < total            # the pool is smaller than all requests together
    check(trace, cases[which], dtype, tmp_path, which)


def test_float32_logits_do_not_depend_on_the_cut(cases, tmp_path):
    """Tighter than the comparison with the plain implementation: two cuttings of one request
    through the engine agree to rounding."""
    folder, cfg, reqs, _ = cases["B"]
    one = {"r0": reqs["r0"]}
    outs = []
    for k, trace in enumerate((traces.whole(one), traces.portions(one), traces.tail_decoded(one))):
        d = str(tmp_path / f"o{k}")
        traces.run_in_process(trace, folder, "float32", d, TINY["B"][2])
        outs.append(traces.collect(trace, d, cfg["vocab_size"])["r0"])
    for pos in range(len(reqs["r0"])):
        for other in outs[1:]:
            assert abs(other[pos] - outs[0][pos]).max() <= 2e-6 * abs(outs[0][pos]).max() + 1e-7


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_program_as_a_user_runs_it(cases, tmp_path, dtype):
    trace = traces.mixed(cases["A"][2], seed=3)
    check(trace, cases["A"], dtype, tmp_path, "A", program=True)


def test_a_step_without_wanted_logits_writes_no_file(cases, tmp_path):
    folder, cfg, reqs, ref = cases["A"]
    toks = reqs["r0"]
    t = traces.Trace()
    t.steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:10], "want": []}], "end": []},
               {"step": 1, "entries": [{"id": "x", "tokens": toks[10:20], "want": [9, 0]}], "end": ["x"]}]
    t.rows = [[], [("x", 19), ("x", 10)]]               # the order of `want` is kept
    t.max_tokens = 64
    out_dir = str(tmp_path / "o")
    traces.run_in_process(t, folder, "float32", out_dir, 4)
    assert not os.path.exists(os.path.join(out_dir, "0.f32"))
    got = traces.collect(t, out_dir, cfg["vocab_size"])["x"]
    for pos in (10, 19):
        assert abs(got[pos] - ref["float32"]["r0"][pos].numpy()).max() < 1e-4 * float(ref["float32"]["r0"].abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E"])
def test_random_traces(cases, tmp_path, which, dtype):
    """Six draws of the cutting: mixed traces with one to four live requests and 0 to 40 tokens
    decoded one by one at the end, or portions of drawn sizes; page sizes other than the usual."""
    import random
    folder, cfg, reqs, ref = cases[which]
    pages = {"A": [4, 1, 16], "B": [8, 2], "C": [16, 32], "D": [16, 32, 64], "E": [16, 32, 64]}[which]
    for seed in range(6):
        rng = random.Random(100 * ord(which) + seed)
        if rng.random() < 0.75:
            trace = traces.mixed(reqs, seed=seed, max_live=rng.randint(1, 4), tail=rng.choice([0, 1, 5, 12, 40]))
        else:
            trace = traces.portions(reqs, sizes=tuple(rng.choice([2, 3, 7, 16, 17, 33, 64, 65, 100, 129]) for _ in range(9)))
        page = rng.choice(pages)
        out_dir = str(tmp_path / f"out{seed}")
        traces.run_in_process(trace, folder, dtype, out_dir, page)
        got = traces.collect(trace, out_dir, cfg["vocab_size"])
        bad, _ = traces.first_mismatch(got, ref[dtype], TOL[dtype])
        assert bad is None, f"draw {seed}, page size {page}: first wrong logits at (request, position, relative error) {bad}"
