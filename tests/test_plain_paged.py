"""The plain step function over a paged cache (tests/plain/paged_plain.py) against the plain
whole-sequence forward, on the CPU: the same requests whole, with their last tokens one by one, in
portions of changing size, and mixed with other requests in a pool so small that pages are given
back (poisoned) and used again.  This is the reference's own story for its paged attention
(src/layers/fused_ops/attn.py:715-855 over src/engine/kvcache.py:222-283) carried to batches that
mix prompt portions and single tokens."""
import pytest
import torch

from plain import paged_plain as PP
from plain import qwen3_plain as P
from tiny import TINY, make_folder
import traces


def run(trace, cfg, w, page_size, pages):
    cache = PP.PagedCache(cfg["num_hidden_layers"], pages, page_size, cfg["num_key_value_heads"], cfg["head_dim"])
    got = {}
    for rec in trace.steps:
        out = PP.step(cfg, w, cache, [(e["id"], e["tokens"]) for e in rec["entries"]])
        for e in rec["entries"]:
            got.setdefault(e["id"], []).append(out[e["id"]])
        for rid in rec["end"]:
            cache.release(rid)
    assert sorted(cache.free) == list(range(pages))                 # every page came back
    return {rid: torch.cat(rows) for rid, rows in got.items()}


@pytest.mark.parametrize("which", ["A", "B"])
def test_every_cutting_of_the_plain_paged_step_gives_the_whole_sequence_logits(tmp_path, which):
    folder = make_folder(tmp_path, which, dtype=torch.float32, std=0.05)
    cfg, w = P.read_folder(folder)
    page = TINY[which][2]
    g = torch.Generator().manual_seed(50)
    reqs = {f"r{i}": torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for i, n in enumerate((37, 21, 50, 30, 44))}
    ref = {rid: P.forward_logits(cfg, w, toks) for rid, toks in reqs.items()}
    cuts = {"whole": traces.whole(reqs), "tail": traces.tail_decoded(reqs, tail=8), "portions": traces.portions(reqs),
            "mixed": traces.mixed(reqs, seed=4, max_live=3, tail=6)}
    for name, trace in cuts.items():
        pages = trace.max_tokens // page                             # so few that pages are used again
        got = run(trace, cfg, w, page, pages)
        for rid, rows in ref.items():
            assert got[rid].shape == rows.shape, (name, rid)
            assert torch.isfinite(got[rid]).all(), (name, rid)
            err = float((got[rid] - rows).abs().max()) / float(rows.abs().max())
            assert err < 2e-5, (name, rid, err)


def test_a_page_that_is_read_before_it_is_written_shows(tmp_path):
    """The pool's pages start as NaN and go back as NaN: gathering one token more than was written
    gives NaN, as a wrong table entry or an early read would."""
    folder = make_folder(tmp_path, "A", dtype=torch.float32, std=0.05)
    cfg, w = P.read_folder(folder)
    cache = PP.PagedCache(cfg["num_hidden_layers"], 4, 4, cfg["num_key_value_heads"], cfg["head_dim"])
    PP.step(cfg, w, cache, [("a", [1, 2, 3, 4, 5])])
    k, _ = cache.gather_sequence(0, "a", 5)
    assert torch.isfinite(k).all()
    k, _ = cache.gather_sequence(0, "a", 6)
    assert torch.isnan(k[5]).all()
    with pytest.raises(RuntimeError):
        PP.step(cfg, w, cache, [("b", list(range(9)))])              # two pages are left, three are needed
