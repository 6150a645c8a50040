"""Builds replay traces (the JSON steps that bin/trace_run reads) that cut the same
requests in different ways, runs them, and maps every logits row back to
(request, position) so that all cuttings can be compared with whole sequences."""
import io
import json
import os
import random
import subprocess
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def round64(n):
    return (n + 63) // 64 * 64


class Trace:
    def __init__(self):
        self.steps = []          # list of dicts as written to the program
        self.rows = []           # per step: list of (request, position) in output order
        self.held = {}           # request -> tokens held so far
        self.max_tokens = 0

    def step(self, entries, end=()):
        """entries: list of (request, tokens); every position's logits are wanted."""
        rec = {"step": len(self.steps), "entries": [], "end": list(end)}
        rows = []
        for rid, toks in entries:
            start = self.held.get(rid, 0)
            rec["entries"].append({"id": rid, "tokens": list(toks), "want": list(range(len(toks)))})
            rows.extend((rid, start + i) for i in range(len(toks)))
            self.held[rid] = start + len(toks)
        self.max_tokens = max(self.max_tokens, sum(round64(n) for n in self.held.values()))
        for rid in end:
            del self.held[rid]
        self.steps.append(rec)
        self.rows.append(rows)

    def text(self):
        return "".join(json.dumps(s) + "\n" for s in self.steps)


def whole(requests):
    t = Trace()
    for rid, toks in requests.items():
        t.step([(rid, toks)], end=[rid])
    return t


def tail_decoded(requests, tail=32):
    t = Trace()
    for rid, toks in requests.items():
        n = len(toks) - tail
        t.step([(rid, toks[:n])])
        for i in range(n, len(toks)):
            t.step([(rid, toks[i:i + 1])], end=[rid] if i == len(toks) - 1 else [])
    return t


def portions(requests, sizes=(2, 3, 17, 2, 31, 5, 64, 2, 9)):
    t = Trace()
    for rid, toks in requests.items():
        i, k = 0, 0
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            k += 1
            if len(toks) - i - n == 1:     # never leave a single token for a "portion"
                n += 1
            t.step([(rid, toks[i:i + n])], end=[rid] if i + n == len(toks) else [])
            i += n
    return t


def mixed(requests, seed=0, max_live=4, tail=12):
    """Up to max_live live requests; portions of some beside single decoded tokens of others;
    requests are sometimes left out of a step; finished ones end and new ones start, so pages
    come back and are used again."""
    rng = random.Random(seed)
    t = Trace()
    waiting = list(requests.items())
    live = {}                    # rid -> [tokens, done]
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0]
        entries, end = [], []
        for rid in list(live):
            toks, done = live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                                   # left out of this step
            left = len(toks) - done
            if left <= tail:
                n = 1                                      # decoding
            else:
                n = min(rng.choice([2, 3, 5, 8, 13, 21, 40]), left - tail)
                if n == 1:
                    n = 2 if left - tail >= 2 else 1
            entries.append((rid, toks[done:done + n]))
            live[rid][1] = done + n
            if done + n == len(toks):
                end.append(rid)
                del live[rid]
        if entries:
            rng.shuffle(entries)
            t.step(entries, end)
    return t


def run_in_process(trace, folder, dtype, out_dir, page_size, debug_poison=True):
    """(debug_poison: every page is NaN when it is handed out and when it goes back, so a read of a
    key that was never written, or of a page that is another request's by now, shows as NaN)"""
    from qwen_engine_amd.engine.replay import replay
    sink = io.StringIO()
    replay(folder, dtype, out_dir, trace.max_tokens, io.StringIO(trace.text()), sink, page_size=page_size,
           debug_poison=debug_poison)
    done = [ln for ln in sink.getvalue().splitlines() if ln.startswith("done ")]
    assert done == [f"done {i}" for i in range(len(trace.steps))]


def run_program(trace, folder, dtype, out_dir, page_size, env=None, debug_poison=True):
    """Runs bin/trace_run as a user would: steps go in one at a time, each after 'done <step>'."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(trace.max_tokens), "--block-size", str(page_size)]
    if debug_poison:
        cmd.append("--debug-poison")
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, env=env)
    try:
        for i, rec in enumerate(trace.steps):
            proc.stdin.write(json.dumps(rec) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {i}", f"expected 'done {i}', got {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()


def collect(trace, out_dir, vocab):
    """{request: {position: logits row}} from the <step>.f32 files."""
    got = {}
    for i, rows in enumerate(trace.rows):
        path = os.path.join(out_dir, f"{i}.f32")
        if not rows:
            assert not os.path.exists(path)
            continue
        arr = np.fromfile(path, dtype="<f4")
        assert arr.size == len(rows) * vocab, f"step {i}: {arr.size} floats for {len(rows)} rows"
        arr = arr.reshape(len(rows), vocab)
        for (rid, pos), row in zip(rows, arr):
            assert pos not in got.setdefault(rid, {})
            got[rid][pos] = row
    return got


def first_mismatch(got, ref, tol):
    """The first (request, position) whose logits differ from the reference by more than
    tol * max |reference|, with the error; None if all agree."""
    worst = 0.0
    for rid, rows in ref.items():
        scale = float(rows.abs().max())
        for pos in range(rows.shape[0]):
            err = float(np.abs(got[rid][pos] - rows[pos].numpy()).max())
            worst = max(worst, err / scale)
            if not err <= tol * scale:
                return (rid, pos, err / scale), worst
    return None, worst
