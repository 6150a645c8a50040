"""Generation through the entry points on the GPU: greedy tokens equal the plain
implementation's, whatever the engine's sizes; long decoding; the first tokens of a
sequence; temperature sampling does not depend on the batch."""
import json
import os
import subprocess
import sys

import pytest
import torch

import qwen_engine_amd
from qwen_engine_amd import EngineConfig, LLMEngine, SamplingParams, generate
from plain import qwen3_plain as P
from tiny import TINY, make_folder

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("gen")
    return {w: make_folder(tmp, w, dtype=torch.bfloat16, std=0.08) for w in "ABDE"}


def prompts_for(cfg, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in lengths]


def test_greedy_generation_equals_the_plain_implementation(folders):
    """The first tiny configuration's workload: prompts of 5, 9 and 13 tokens, 8 greedy tokens."""
    cfg, w = P.read_folder(folders["A"])
    prompts = prompts_for(cfg, (5, 9, 13), 1)
    want = [P.greedy_generate(cfg, w, p, 8) for p in prompts]
    res = generate(folders["A"], prompts, SamplingParams(max_new_tokens=8, ignore_eos=True),
                   EngineConfig(dtype="float32", block_size=4, max_num_seqs=4, max_model_len=64))
    assert [r.token_ids for r in res] == want
    assert all(r.finish_reason == "length" for r in res)
    assert [r.prompt_token_ids for r in res] == prompts


@pytest.mark.parametrize("sizes", [dict(max_num_seqs=1), dict(max_step_tokens=7, prefill_chunk=6),
                                   dict(num_blocks=9, block_size=8), dict(block_size=1, num_blocks=200),
                                   dict(enable_prefix_sharing=False), dict(scatter_pages=False),
                                   dict(scatter_pages=False, num_blocks=9)])
def test_outputs_do_not_depend_on_the_engine_sizes(folders, sizes):
    """Second tiny configuration: prompts of 1, 7, 16 and 30 tokens, two sharing 16 tokens; portions
    of 6 mixed with decoding; few pages (preemption); pages handed out in a scattered order (the
    default) and in the order 0, 1, 2, ...; greedy and temperature 0.7 with a fixed seed."""
    cfg, w = P.read_folder(folders["B"])
    p = prompts_for(cfg, (1, 7, 16, 30), 2)
    p[3] = p[2] + p[3][16:]                               # the last two share a prefix of 16 tokens
    want = [P.greedy_generate(cfg, w, q, 10) for q in p]
    base = dict(dtype="float32", block_size=8, max_num_seqs=4, max_model_len=48, prefill_chunk=6, debug_poison=True)
    base.update(sizes)
    eng = LLMEngine.from_folder(folders["B"], EngineConfig(**base))
    eng.submit(p, max_new_tokens=10, ignore_eos=True)
    res = eng.run()
    assert [r.token_ids for r in res] == want
    eng.runner.cache.check_invariants()
    cache = eng.runner.cache                                  # (pages kept for later requests count as free to take)
    assert all(cache.available(g) == pool.num_pages for g, pool in enumerate(cache.pools))
    # temperature: the same tokens as a run of each request alone with the same seed
    hits_before = eng.stats()["kept_page_hits"]
    eng.submit(p, max_new_tokens=10, temperature=0.7, seed=11, ignore_eos=True)
    together = [r.token_ids for r in eng.run()]
    # the second run found full pages of the first run's prompts, kept though those requests had ended
    if sizes.get("enable_prefix_sharing", True):
        assert eng.stats()["kept_page_hits"] > hits_before
    else:
        assert eng.stats()["kept_page_hits"] == 0 and cache.num_kept == 0
    ref_engine = LLMEngine.from_folder(folders["B"], EngineConfig(dtype="float32", block_size=8, max_num_seqs=1,
                                                                  max_model_len=48))
    alone = []
    for i, q in enumerate(p):
        ref_engine._next_id = eng._next_id - len(p) + i    # the draw is keyed by (seed, request id, position)
        ref_engine.submit([q], max_new_tokens=10, temperature=0.7, seed=11, ignore_eos=True)
        alone.append(ref_engine.run()[0].token_ids)
    assert together == alone
    assert together != want                                # and it is not greedy


@pytest.mark.parametrize("which", ["D", "E"])
@pytest.mark.parametrize("sizes", [dict(), dict(num_blocks=34, max_num_seqs=4), dict(max_step_tokens=48, prefill_chunk=32)])
def test_bfloat16_generation_on_the_mfma_kernels(folders, sizes, which):
    """The tiny configurations with head sizes 64 and 128 in bfloat16: decode steps run as recorded
    graphs on the MFMA kernels, prompts in portions, and with few pages requests are preempted.
    Every token the engine chose must be the plain implementation's choice for the engine's own
    sequence, or within rounding of it (bfloat16 results depend on the cut in the last bits)."""
    cfg, w = P.read_folder(folders[which])
    prompts = prompts_for(cfg, (150, 33, 70, 201, 16), 6)
    base = dict(dtype="bfloat16", block_size=16, max_num_seqs=3, max_model_len=320, debug_poison=True)
    base.update(sizes)
    eng = LLMEngine.from_folder(folders[which], EngineConfig(**base))
    eng.submit(prompts, max_new_tokens=40, ignore_eos=True)
    res = eng.run()
    assert eng.runner.graph_steps > 0
    if "num_blocks" in sizes:
        assert eng.stats()["preemptions"] > 0
    eng.runner.cache.check_invariants()
    cache = eng.runner.cache                                  # (pages kept for later requests count as free to take)
    assert all(cache.available(g) == pool.num_pages for g, pool in enumerate(cache.pools))
    for r, prompt in zip(res, prompts):
        assert r.finish_reason == "length" and len(r.token_ids) == 40
        logits = P.forward_logits(cfg, w, prompt + r.token_ids[:-1], act_dtype=torch.bfloat16)
        scale = float(logits.abs().max())
        for i, tok in enumerate(r.token_ids):
            row = logits[len(prompt) - 1 + i]
            assert float(row.max() - row[tok]) <= 2e-2 * scale, (i, tok, int(row.argmax()))


def test_shared_prefix_pages_are_taken_over(folders):
    cfg, w = P.read_folder(folders["B"])
    common = prompts_for(cfg, (32,), 3)[0]
    a, b = common + [5, 6, 7], common + [9]
    eng = LLMEngine.from_folder(folders["B"], EngineConfig(dtype="float32", block_size=8, max_num_seqs=2,
                                                           max_model_len=64))
    eng.submit([a], max_new_tokens=4, ignore_eos=True)
    eng.step()                                            # a's prompt is computed, a is still live
    eng.submit([b], max_new_tokens=4, ignore_eos=True)
    res = eng.run()
    assert eng.stats()["shared_prefix_tokens"] == 32
    assert res[0].token_ids == P.greedy_generate(cfg, w, a, 4)
    assert res[1].token_ids == P.greedy_generate(cfg, w, b, 4)
    # the kernels were told which request read keys of another's pages (its row of the device tables)
    assert sorted(eng.runner.shared_keys.tolist()) == [0, 0, 32]
    # a request without a shared prefix that takes the same row over is told so as well
    eng.submit([[1, 2, 3]] * 2, max_new_tokens=2, ignore_eos=True)
    eng.run()
    assert eng.runner.shared_keys.tolist() == [0, 0, 0]


def test_temperature_sampling_equals_the_plain_draw(folders):
    """Every token that the engine draws at temperature 0.8 is the plain implementation's draw from
    the plain logits of the engine's own sequence, with the same uniform number per (seed, request,
    output position); draws that lie within 1e-4 of an edge of their token's interval are not judged."""
    cfg, w = P.read_folder(folders["A"])
    prompts = prompts_for(cfg, (5, 9, 13, 2), 12)
    eng = LLMEngine.from_folder(folders["A"], EngineConfig(dtype="float32", block_size=4, max_num_seqs=3, max_model_len=64))
    first_id = eng._next_id
    eng.submit(prompts, max_new_tokens=12, temperature=0.8, seed=77, ignore_eos=True)
    res = eng.run()
    judged = 0
    for i, (r, prompt) in enumerate(zip(res, prompts)):
        logits = P.forward_logits(cfg, w, prompt + r.token_ids[:-1])
        for k, tok in enumerate(r.token_ids):
            u = P.uniform_number(77, first_id + i, k)
            want, margin = P.sample_temperature(logits[len(prompt) - 1 + k], 0.8, u)
            if margin > 1e-4:
                assert tok == want, (i, k, tok, want)
                judged += 1
    assert judged >= 40
    greedy = [P.greedy_generate(cfg, w, p, 12) for p in prompts]
    assert [r.token_ids for r in res] != greedy


def test_requests_submitted_together_share_their_beginning(folders):
    """Two prompts with 32 tokens in common and one that shares nothing, submitted in one call (the
    reference's prompts 2 and 3 begin alike, main.py:64-68): the second of the pair waits for the
    first one's pages instead of computing them again, and every output is the plain one."""
    cfg, w = P.read_folder(folders["B"])
    common = prompts_for(cfg, (32,), 3)[0]
    a, b, c = common + [5, 6, 7], prompts_for(cfg, (11,), 8)[0], common + [9]
    eng = LLMEngine.from_folder(folders["B"], EngineConfig(dtype="float32", block_size=8, max_num_seqs=3,
                                                           max_model_len=64, prefill_chunk=16, debug_poison=True))
    eng.submit([a, b, c], max_new_tokens=4, ignore_eos=True)
    res = eng.run()
    assert eng.stats()["shared_prefix_tokens"] == 32 and eng.stats()["held_back_for_prefix"] >= 1
    assert eng.stats()["prefill_tokens"] == len(a) + len(b) + len(c) - 32
    for r, prompt in zip(res, (a, b, c)):
        assert r.token_ids == P.greedy_generate(cfg, w, prompt, 4)


@pytest.mark.parametrize("dtype,which,page", [("float32", "A", 4), ("bfloat16", "A", 4), ("bfloat16", "E", 16), ("float32", "E", 16)])
def test_long_decoding(folders, dtype, which, page):
    """300 tokens decoded one by one after a short prompt: logits at every decoded position equal
    the plain implementation's on the whole sequence (pages fill and new ones are taken 75 times;
    with heads of 128 the recorded decode step passes the ends of two splits of 128 keys)."""
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    cfg, w = P.read_folder(folders[which])
    toks = prompts_for(cfg, (305,), 4)[0]
    act = None if dtype == "float32" else torch.bfloat16
    ref = P.forward_logits(cfg, w, toks, act_dtype=act)
    runner = ModelRunner(load_model(folders[which], dtype=dtype), page_size=page, num_pages=80, max_requests=1)
    runner.add_request("r")
    rows = [runner.step([StepEntry("r", toks[:5], [4])])]
    for i in range(5, 305):
        rows.append(runner.step([StepEntry("r", toks[i:i + 1], [0])]))
    got = torch.cat(rows).cpu()
    tol = 1e-4 if dtype == "float32" else 2e-2
    err = (got - ref[4:]).abs().max(dim=1).values / ref.abs().max()
    bad = torch.nonzero(err > tol)
    assert bad.numel() == 0, f"first wrong position {int(bad[0]) + 4}, error {float(err[bad[0]])}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(folders, dtype):
    """Positions 0, 1 and 2, each asked for alone and together, over a page size of 1 and of 8."""
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    cfg, w = P.read_folder(folders["B"])
    toks = prompts_for(cfg, (3,), 5)[0]
    act = None if dtype == "float32" else torch.bfloat16
    ref = P.forward_logits(cfg, w, toks, act_dtype=act)
    tol = (1e-4 if dtype == "float32" else 2e-2) * float(ref.abs().max())
    model = load_model(folders["B"], dtype=dtype)
    for page in (1, 8):
        runner = ModelRunner(model, page_size=page, num_pages=8, max_requests=2)
        runner.add_request("a")
        runner.add_request("b")
        one = [runner.step([StepEntry("a", toks[i:i + 1], [0])]).cpu()[0] for i in range(3)]
        together = runner.step([StepEntry("b", toks, [0, 1, 2])]).cpu()
        for i in range(3):
            assert (one[i] - ref[i]).abs().max() <= tol and (together[i] - ref[i]).abs().max() <= tol


def test_step_refuses_bad_entries(folders):
    from qwen_engine_amd.cache import OutOfPages
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    runner = ModelRunner(load_model(folders["A"], dtype="float32"), page_size=4, num_pages=2, max_requests=2)
    runner.add_request("a")
    with pytest.raises(ValueError):
        runner.step([StepEntry("a", [256], [0])])           # outside the vocabulary
    with pytest.raises(ValueError):
        runner.step([StepEntry("a", [1, 2], [2])])          # wants a place it does not bring
    with pytest.raises(ValueError):
        runner.step([StepEntry("a", [1], []), StepEntry("a", [2], [])])
    with pytest.raises(OutOfPages):
        runner.step([StepEntry("a", list(range(9)), [])])   # 3 pages, the pool has 2
    assert runner.cache.num_free_pages() == 2                # nothing was taken
    assert runner.step([StepEntry("a", list(range(8)), [7])]).shape == (1, 256)


def test_command_line(folders, tmp_path):
    """main.py with the reference's option names: random weights from a config file, prompts as ids."""
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(TINY["A"][0]))
    out = tmp_path / "model"
    cmd = [sys.executable, os.path.join(ROOT, "main.py"), "--random-weights", str(cfg_path), "--seed", "4",
           "--model-name-or-path", str(out), "--prompt-ids", "5,6,7,8", "--prompt-ids", "9,10",
           "--max-new-tokens", "5", "--max-num-seqs", "2", "--max-model-len", "32", "--block-size", "4",
           "--model-dtype", "float32", "--ignore-eos", "--stats"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr[-2000:]
    cfg, w = P.read_folder(str(out))
    want = [P.greedy_generate(cfg, w, p, 5) for p in ([5, 6, 7, 8], [9, 10])]
    lines = r.stdout.splitlines()
    assert "Prompt: 5 6 7 8" in lines and "Prompt: 9 10" in lines
    assert " ".join(map(str, [5, 6, 7, 8] + want[0])) in lines
    assert " ".join(map(str, [9, 10] + want[1])) in lines
    stats = json.loads(lines[-1])
    assert stats["decode_tokens"] == 8 and stats["prefill_tokens"] == 6


def test_text_prompts_through_the_command_line(folders, tmp_path):
    """Raw text goes through the folder's tokenizer.json without a template, and what is printed is
    the decoded prompt + output without special tokens (src/engine/llm_engine.py:52-55,67-73).  The
    tokenizer is a word-level one written here, with a vocabulary as large as the model's."""
    import shutil
    from tokenizers import Tokenizer
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import Whitespace
    folder = str(tmp_path / "model_with_tokenizer")
    shutil.copytree(folders["A"], folder)
    cfg, w = P.read_folder(folder)
    words = ["[UNK]", "[EOS]"] + [f"w{i}" for i in range(cfg["vocab_size"] - 2)]
    tok = Tokenizer(WordLevel({word: i for i, word in enumerate(words)}, unk_token="[UNK]"))
    tok.pre_tokenizer = Whitespace()
    tok.add_special_tokens(["[UNK]", "[EOS]"])
    tok.save(os.path.join(folder, "tokenizer.json"))
    texts = ["w5 w17 w3 w200", "w9 w9 w31 never_seen w4 w77 w12"]
    ids = [tok.encode(t).ids for t in texts]
    assert ids[0] == [7, 19, 5, 202] and ids[1][3] == 0                  # the unknown word
    cmd = [sys.executable, os.path.join(ROOT, "main.py"), "--model", folder, "--prompt", texts[0], "--prompt", texts[1],
           "--max-new-tokens", "6", "--max-num-seqs", "2", "--max-model-len", "32", "--block-size", "4",
           "--model-dtype", "float32", "--ignore-eos"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = r.stdout.splitlines()
    for t, p in zip(texts, ids):
        out = P.greedy_generate(cfg, w, p, 6)
        assert f"Prompt: {tok.decode(p, skip_special_tokens=True)}" in lines
        assert tok.decode(p + out, skip_special_tokens=True) in lines        # specials ([UNK], [EOS]) are left out
    # the Python entry point with text, and a request that stops at the end-of-sequence token
    res = generate(folder, [texts[0]], SamplingParams(max_new_tokens=6, ignore_eos=True),
                   EngineConfig(dtype="float32", block_size=4, max_model_len=32))
    assert res[0].prompt_token_ids == ids[0]
    assert res[0].text == tok.decode(ids[0] + res[0].token_ids, skip_special_tokens=True)


def test_decode_batches_between_recorded_sizes_are_filled_up(folders):
    """11 requests decode through the graph recorded for 16 rows, and after two of them have ended
    the 9 that remain replay the same graph: the logits are those of a runner without graphs."""
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    cfg, w = P.read_folder(folders["D"])
    model = load_model(folders["D"], dtype="bfloat16")
    prompts = prompts_for(cfg, tuple(range(5, 16)), 9)
    runners = [ModelRunner(model, page_size=16, num_pages=40, max_requests=11, use_graphs=flag) for flag in (True, False)]
    assert [ModelRunner.graph_rows(n) for n in (1, 8, 9, 11, 16, 57, 64, 65, 200)] == [1, 8, 16, 16, 16, 64, 64, 96, 224]
    outs = []
    for runner in runners:
        got = []
        recorded = runner.use_graphs
        runner.use_graphs = False                  # (the prompts through the same kernels in both runners: the
        for i, p in enumerate(prompts):            # comparison below is of the decode steps, to a thousandth)
            runner.add_request(i)
            runner.step([StepEntry(i, p, [])])
        runner.use_graphs = recorded
        live = list(range(11))
        for step in range(4):
            if step == 2:
                for i in (3, 7):
                    runner.free_request(i)
                    live.remove(i)
            got.append(runner.step([StepEntry(i, [(7 * i + step) % cfg["vocab_size"]], [0]) for i in live]))
        outs.append(got)
    assert runners[0].graph_steps_of["decode"] == 4 and runners[0].graphs_recorded == 1 and runners[1].graph_steps == 0
    for a, b in zip(*outs):
        assert a.shape == b.shape and a.shape[0] in (11, 9)
        assert float((a - b).abs().max()) <= 1e-3 * float(b.abs().max())
    # and they are the plain implementation's logits for the first request's sequence
    seq = prompts[0] + [(7 * 0 + s) % cfg["vocab_size"] for s in range(4)]
    ref = P.forward_logits(cfg, w, seq, act_dtype=torch.bfloat16)
    for s in range(4):
        assert float((outs[0][s][0].cpu() - ref[len(prompts[0]) + s]).abs().max()) <= 2e-2 * float(ref.abs().max())


@pytest.mark.parametrize("which", ["A", "B"])
def test_random_engine_sizes_and_prompt_sets(folders, which):
    """Twenty draws of prompts (some sharing a prefix, one a prefix of another, one twice) and of
    engine sizes (page size, pages from barely enough for one request to enough for all, live
    requests, token budget, portion size, prefix sharing on or off): greedy float32 tokens equal
    the plain implementation's, every request runs to its length, and every page comes back."""
    import random
    cfg, w = P.read_folder(folders[which])
    base = prompts_for(cfg, (1, 7, 16, 30, 45, 3), 21)
    plain = {}
    preempted = shared = 0
    for seed in range(20):
        rng = random.Random(31 * ord(which) + seed)
        prompts = list(base) + [base[3][:20] + base[2][:5], base[4][:32], list(base[4])]
        rng.shuffle(prompts)
        prompts = prompts[:rng.randint(2, len(prompts))]
        new = rng.choice([1, 2, 6, 12])
        page = rng.choice([1, 2, 4, 8, 16])
        longest = max(len(p) for p in prompts) + new
        per_request = -(-longest // page)
        sizes = dict(dtype="float32", block_size=page, max_num_seqs=rng.randint(1, 5), debug_poison=True,
                     num_blocks=rng.choice([per_request + 1, 2 * per_request, per_request * len(prompts) + 4]),
                     max_model_len=longest + rng.choice([0, 3, 50]), max_step_tokens=rng.choice([3, 8, 20, 64, 2048]),
                     prefill_chunk=rng.choice([2, 5, 16, 512]), enable_prefix_sharing=rng.random() < 0.7)
        want = []
        for p in prompts:
            if (tuple(p), new) not in plain:
                plain[tuple(p), new] = P.greedy_generate(cfg, w, p, new)
            want.append(plain[tuple(p), new])
        eng = LLMEngine.from_folder(folders[which], EngineConfig(**sizes))
        eng.submit(prompts, max_new_tokens=new, ignore_eos=True)
        res = eng.run()
        assert [r.token_ids for r in res] == want, (seed, sizes)
        assert all(r.finish_reason == "length" for r in res), (seed, sizes)
        cache = eng.runner.cache
        cache.check_invariants()
        assert all(cache.available(g) == pool.num_pages for g, pool in enumerate(cache.pools)), (seed, sizes)
        preempted += eng.stats()["preemptions"] > 0
        shared += eng.stats()["shared_prefix_tokens"] > 0
        if seed < 8:
            # temperature sampling with a seed: the same tokens as an engine with room for everything
            both = []
            for cfg_sizes in (sizes, dict(dtype="float32", block_size=8, max_num_seqs=len(prompts), max_model_len=longest + 8)):
                e2 = LLMEngine.from_folder(folders[which], EngineConfig(**cfg_sizes))
                e2.submit(prompts, max_new_tokens=new, temperature=0.9, seed=5, ignore_eos=True)
                both.append([r.token_ids for r in e2.run()])
                e2.runner.cache.check_invariants()
            assert both[0] == both[1], (seed, sizes)
    assert preempted >= 2 and shared >= 5          # the draws reach both


def test_pool_sized_from_the_free_memory(folders):
    """EngineConfig.gpu_memory_fraction: the pool gets what that fraction of the free device memory holds,
    and generation runs in it as in a pool of a given size."""
    folder = folders["A"]
    cfg, w = P.read_folder(folder)
    prompt = prompts_for(cfg, [9], 77)[0]
    want = P.greedy_generate(cfg, w, prompt, 5)
    ecfg = EngineConfig(dtype="float32", block_size=4, max_model_len=64, gpu_memory_fraction=0.001, graph_memory_bytes=0)
    engine = LLMEngine.from_folder(folder, ecfg)
    free = torch.cuda.mem_get_info()[0]
    pages = engine.runner.cache.pools[0].num_pages
    per_page = cfg["num_hidden_layers"] * 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * 4 * 4
    assert pages >= 16 and abs(pages * per_page - 0.001 * (free + pages * per_page)) < 0.0002 * free
    engine.submit([prompt], max_new_tokens=5, ignore_eos=True)
    assert engine.run()[0].token_ids == want
