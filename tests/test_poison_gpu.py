"""Page poisoning and the tables' spare row.

With ``debug_poison`` every cache page is NaN when it is handed out and when it goes back.  A
table entry that names a wrong page in one cache group of one request then turns that request's
logits into NaN also in bfloat16, where a stale page among hundreds of keys would otherwise
move the logits by less than the rounding.  The other tests run their traces with the poison on;
this file shows that it bites.  It also runs more decoding requests than a recorded graph has
rows for, past the shortest window: the rows that fill the graph up must not follow a live
request's table (whose first entries are -1 by then)."""
import pytest
import torch

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
from plain import qwen3_plain as P
from test_window_layers_gpu import PAGE, V, WINDOWS, plain_forward, toy  # noqa: F401  (toy is a fixture)

pytestmark = pytest.mark.gpu


def _tokens(n, seed):
    return torch.randint(0, V, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("group", [0, 1, 2])
def test_a_wrong_table_entry_in_one_group_gives_nan(toy, dtype, group):
    """Three cache groups (windows of 40 and 17 keys, and all keys).  After a prompt of 100 tokens,
    one entry of one group's table on the device is pointed at a page that the request does not
    hold: the next token's logits are NaN; untouched, they are the plain implementation's."""
    model = load_model(toy, dtype=dtype)
    toks = _tokens(102, 5)
    _, w = P.read_folder(toy)
    ref = plain_forward(w, toks, None if dtype == "float32" else torch.bfloat16)
    tol = (1e-4 if dtype == "float32" else 2e-2) * float(ref.abs().max())
    for corrupt in (False, True):
        runner = ModelRunner(model, page_size=PAGE, num_pages=24, max_requests=2, debug_poison=True)
        runner.add_request("other")                      # another request came and went: its pages are poisoned
        runner.step([StepEntry("other", _tokens(50, 6), [])])
        runner.free_request("other")
        runner.add_request("a")
        runner.step([StepEntry("a", toks[:100], [])])
        rc = runner.cache.get("a")
        window = runner.cache.groups[group].window
        first_key = 0 if window is None else 100 - window + 1
        index = first_key // PAGE                        # a page that position 100 sees in this group
        assert rc.tables[group][index] >= 0
        if corrupt:
            free_page = runner.cache.pools[group].free[0]
            runner.tables[group][rc.state_slot, index] = free_page
        logits = runner.step([StepEntry("a", toks[100:101], [0])]).cpu()
        if corrupt:
            assert torch.isnan(logits).any(), f"group {group}: a read of a page that is not the request's went unseen"
        else:
            assert float((logits[0] - ref[100]).abs().max()) <= tol
        assert runner.pages_poisoned > 0


@pytest.mark.parametrize("use_graphs", [True, False])
def test_twenty_requests_decode_past_the_window(toy, use_graphs):
    """20 live requests (a graph of 24 rows, four of them fill rows) decode in bfloat16 after prompts
    longer than the windows, so that every live request's first table entries are -1."""
    model = load_model(toy, dtype="bfloat16")
    _, w = P.read_folder(toy)
    lengths = [60 + 7 * i for i in range(20)]
    reqs = [_tokens(n + 6, 100 + i) for i, n in enumerate(lengths)]
    runner = ModelRunner(model, page_size=PAGE, num_pages=20 * 14, max_requests=20, use_graphs=use_graphs,
                         debug_poison=True)
    for i, (toks, n) in enumerate(zip(reqs, lengths)):
        runner.add_request(i)
        runner.step([StepEntry(i, toks[:n], [])])
    for i in range(20):                                  # the windows have passed every request's first page
        assert runner.cache.get(i).tables[0][0] == -1 or runner.cache.groups[0].window is None
    outs = [runner.step([StepEntry(i, [reqs[i][lengths[i] + s]], [0]) for i in range(20)]).float().cpu()
            for s in range(6)]
    assert (runner.graph_steps_of["decode"] == 6) == use_graphs
    assert all(torch.isfinite(o).all() for o in outs)
    for i in (0, 7, 19):
        ref = plain_forward(w, reqs[i], torch.bfloat16)
        for s in range(6):
            err = float((outs[s][i] - ref[lengths[i] + s]).abs().max()) / float(ref.abs().max())
            assert err <= 2e-2, f"request {i}, step {s}: error {err}"
    runner.cache.check_invariants()


@pytest.mark.parametrize("use_graphs", [True, False])
def test_prompt_portions_through_recorded_graphs(toy, use_graphs):
    """Steps that are one prompt portion of a round length are recorded once per length and replayed:
    two requests, one after the other and then side by side in turns, each in portions of 256 and
    384 tokens, with windows that give pages back inside the portions; logits at the portions' ends
    against the plain implementation, and the recorded steps against steps run as they come."""
    model = load_model(toy, dtype="bfloat16")
    _, w = P.read_folder(toy)
    reqs = {"a": _tokens(640, 41), "b": _tokens(896, 42)}
    refs = {k: plain_forward(w, t, torch.bfloat16) for k, t in reqs.items()}
    runner = ModelRunner(model, page_size=PAGE, num_pages=100, max_requests=2, use_graphs=use_graphs, debug_poison=True)
    cuts = {"a": [(0, 256), (256, 640)], "b": [(0, 384), (384, 640), (640, 896)]}
    got = {}
    for order in (["a", "b"],):
        for rid in order:
            runner.add_request(rid)
        turns = [("a", 0), ("b", 0), ("b", 1), ("a", 1), ("b", 2)]
        for rid, i in turns:
            lo, hi = cuts[rid][i]
            want = [hi - lo - 1] if (rid, i) != ("b", 0) else []        # one portion wants no logits
            out = runner.step([StepEntry(rid, reqs[rid][lo:hi], want)])
            assert out.shape[0] == len(want)
            if want:
                got[rid, hi - 1] = out[0].float().cpu()
    assert (runner.graph_steps == 5) == use_graphs
    if use_graphs:
        assert runner.graphs_recorded == 3                  # 256 with logits, 384 with and without
    for (rid, pos), row in got.items():
        err = float((row - refs[rid][pos]).abs().max()) / float(refs[rid].abs().max())
        assert err <= 2e-2, f"request {rid}, position {pos}: error {err}"
    runner.cache.check_invariants()


def test_recorded_graphs_are_dropped_and_recorded_again(toy):
    """A runner that keeps two graphs: decode steps of 1, 2 and 3 requests in turns drop the graph used
    longest ago and record it again when its batch comes back; every step's logits stay right."""
    model = load_model(toy, dtype="bfloat16")
    _, w = P.read_folder(toy)
    reqs = {i: _tokens(60 + 7 * i, 70 + i) for i in range(3)}
    refs = {i: plain_forward(w, t, torch.bfloat16) for i, t in reqs.items()}
    runner = ModelRunner(model, page_size=PAGE, num_pages=40, max_requests=3, debug_poison=True)
    runner.MAX_GRAPHS = 2
    done = {}
    runner.use_graphs = False                      # (the prompts as they come: this test counts the decode steps' graphs)
    for i, t in reqs.items():
        runner.add_request(i)
        runner.step([StepEntry(i, t[:20], [])])
        done[i] = 20
    runner.use_graphs = True
    recorded_at = []
    for live in (1, 2, 3, 1, 2, 3, 3, 1):
        out = runner.step([StepEntry(i, [reqs[i][done[i]]], [0]) for i in range(live)]).float().cpu()
        for i in range(live):
            err = float((out[i] - refs[i][done[i]]).abs().max()) / float(refs[i].abs().max())
            assert err <= 2e-2, f"{live} requests, request {i} at position {done[i]}: error {err}"
            done[i] += 1
        assert len(runner._graphs) <= 2
        recorded_at.append(runner.graphs_recorded)
    # 1, 2, 3 record; 1 again (dropped when 3 came), 2 again, 3 again; 3 is there; 1 again
    assert recorded_at == [1, 2, 3, 4, 5, 6, 6, 7]
    runner.cache.check_invariants()


@pytest.mark.parametrize("use_graphs", [True, False])
def test_single_tokens_beside_one_portion_through_recorded_graphs(toy, use_graphs):
    """What a server runs while requests keep arriving: some requests decode, and beside them one new
    request brings its prompt in portions of any length.  Such steps are recorded with the portion
    filled up to a round length by rows that write nowhere, and replayed; the portion stands anywhere
    among the entries, wants its last row or nothing, and the windows give pages back meanwhile.
    Every wanted row against the plain implementation."""
    model = load_model(toy, dtype="bfloat16")
    _, w = P.read_folder(toy)
    reqs = {"a": _tokens(90, 81), "b": _tokens(75, 82), "c": _tokens(303, 83), "d": _tokens(260, 84)}
    refs = {k: plain_forward(w, t, torch.bfloat16) for k, t in reqs.items()}
    runner = ModelRunner(model, page_size=PAGE, num_pages=120, max_requests=4, use_graphs=use_graphs, debug_poison=True)
    done = {}

    def check(entries, out):
        row = 0
        for e in entries:
            for wpos in e.want:
                pos = done[e.req_id] + wpos
                got = out[row].float().cpu()
                assert torch.isfinite(got).all(), f"request {e.req_id} at {pos}"
                err = float((got - refs[e.req_id][pos]).abs().max()) / float(refs[e.req_id].abs().max())
                assert err <= 2e-2, f"request {e.req_id} at position {pos}: error {err}"
                row += 1
        assert row == out.shape[0]
        for e in entries:
            done[e.req_id] += len(e.tokens)

    def entry(rid, n, want_last=True):
        lo = done[rid]
        return StepEntry(rid, reqs[rid][lo:lo + n], [n - 1] if want_last else [])

    for rid in ("a", "b"):                             # two requests that will decode: their prompts alone
        runner.add_request(rid)
        done[rid] = 0
        e = [entry(rid, 40)]
        check(e, runner.step(e))
    runner.add_request("c")
    done["c"] = 0
    # the portion first, in the middle, last; with and without its last row; of 2 to 150 tokens
    plan = [(["c", "a", "b"], 150, False), (["a", "c", "b"], 2, True), (["a", "b", "c"], 100, True),
            (["a", "c"], 17, False), (["c", "b", "a"], 31, True)]
    for order, n, want_last in plan:
        e = [entry(r, n, want_last) if r == "c" else entry(r, 1) for r in order]
        check(e, runner.step(e))
    # a fourth request arrives while three decode: its whole prompt of 260 tokens beside them
    runner.add_request("d")
    done["d"] = 0
    e = [entry("a", 1), entry("b", 1), entry("c", 1), entry("d", 259, True)]
    check(e, runner.step(e))
    e = [entry(r, 1) for r in ("d", "c", "b", "a")]
    check(e, runner.step(e))
    if use_graphs:
        # the two prompts alone (filled up to 128 rows), the six mixed steps; the last step decodes
        assert runner.graph_steps_of == {"decode": 1, "portion": 0, "mixed": 2 + 6}
    else:
        assert runner.graph_steps == 0
    runner.cache.check_invariants()


def test_a_portion_is_not_filled_up_beyond_the_table_row(toy):
    """A pool of 7 pages: the group that keeps all keys has table rows of 7 entries (112 positions), and
    the rows that would fill a portion up to 128 would stand at positions beyond them.  Such a step
    runs as it comes; with 8 pages it is recorded."""
    model = load_model(toy, dtype="bfloat16")
    _, w = P.read_folder(toy)
    toks = _tokens(60, 91)
    ref = plain_forward(w, toks, torch.bfloat16)
    for pages, recorded in ((7, 0), (8, 2)):
        runner = ModelRunner(model, page_size=PAGE, num_pages=pages, max_requests=1, debug_poison=True)
        runner.add_request("r")
        a = runner.step([StepEntry("r", toks[:50], [49])])[0].float().cpu()
        b = runner.step([StepEntry("r", toks[50:59], [8])])[0].float().cpu()
        for got, pos in ((a, 49), (b, 58)):
            assert float((got - ref[pos]).abs().max()) <= 2e-2 * float(ref.abs().max())
        assert runner.graph_steps_of["mixed"] == recorded
