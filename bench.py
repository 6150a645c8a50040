"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bf16] [--layers L]

The default run has the layer sizes of Qwen3-0.6B with
random weights, a batch of 8 requests and a context of 4096 tokens: every request is
first prefilled with random tokens through the engine's own step function, so that
the K timed decode steps end at that context.  A "step" is one decode step (one new
token per request, through the cache, sampled greedily on the device).  One JSON
line is printed:

  value      decoded tokens a second at batch 8
  prefill    one 2048-token prompt in one step: tokens a second, and flops / time / peak
  roofline   the decode step's bytes (every weight once + the live requests' cache) / time / 8 TB/s
  points     decoded tokens a second at batch 1 and at batch 64
  measured_copy_gbs   what a plain copy of 1 GiB reaches on this device (read + write), for scale
  measured_mfma_tflops   what register-resident bfloat16 MFMAs reach on this device, for scale

Other sizes and workloads (not what the default line reports):

  --model 8b|32b            the layer sizes of Qwen3-8B / Qwen3-32B; with
                            --layers L fewer layers than the model has (the line names both numbers)
  --workload serving        N requests (--requests, default 64) with prompt lengths uniform in [128, 2048]
                            and 256 new tokens each through the scheduler: continuous batching, prompt
                            portions of 512 tokens beside decoded tokens.  value = generated tokens a second
  --workload shared-prefix  N requests (default 32) that share a 1024-token prefix, each with 1024 tokens
                            of its own and 512 new tokens; the prefix's pages are shared
  --prefill-portion N       the prefill in portions of N tokens, one step each, instead of one step
  --workload arrivals       N requests (default 160) with prompts uniform in [128, 512] and 128 new tokens that
                            arrive one every --arrive-every steps (default 8: some 16 alive at a time), so that
                            most steps are single new tokens beside one prompt portion
  --eager-mixed-steps       all three: run such steps as they come instead of replaying a recorded graph
  --kernels                 no model step: each kernel of a layer alone, at 1, 8, 64, 512 and 2048 rows (the four
                            products, the head's, decode and prefill attention at --context), its time from a
                            recorded graph of repetitions over weights that do not fit the caches, and its rate
                            against the nominal and the measured peaks (the counterpart of the reference's
                            per-operator benchmarks, src/layers/ops/linear.py:204-249)
  --warmup-passes N         both: untimed passes over the workload with other tokens before the timed
                            one (default 2: the graphs are recorded there, a shape of steps when it is met
                            the second time, as in a server that has run for a while; 0 times the
                            recording too)
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

QWEN3_0_6B = dict(
    architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=1024, intermediate_size=3072,
    num_hidden_layers=28, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
    max_position_embeddings=40960, rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=True)


SIZES = {
    "0.6b": QWEN3_0_6B,
    "8b": dict(QWEN3_0_6B, hidden_size=4096, intermediate_size=12288, num_hidden_layers=36,
               num_attention_heads=32, num_key_value_heads=8, tie_word_embeddings=False),
    "32b": dict(QWEN3_0_6B, hidden_size=5120, intermediate_size=25600, num_hidden_layers=64,
                num_attention_heads=64, num_key_value_heads=8, tie_word_embeddings=False),
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--prefill-portion", type=int, default=0,
                    help="run the prefill in portions of this many tokens, one step each (0: one step)")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--skip-points", action="store_true", help="leave out the batch 1 and batch 64 runs")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--model", default="0.6b", choices=sorted(SIZES), help="whose layer sizes")
    ap.add_argument("--workload", default="decode", choices=["decode", "serving", "shared-prefix", "arrivals"])
    ap.add_argument("--arrive-every", type=int, default=8, help="arrivals: a request arrives every this many steps")
    ap.add_argument("--eager-mixed-steps", action="store_true",
                    help="run steps of single new tokens beside a prompt portion as they come, not from a recorded graph")
    ap.add_argument("--requests", type=int, default=None, help="requests of the serving workloads")
    ap.add_argument("--kernels", action="store_true", help="time each kernel of a layer alone over a range of rows")
    ap.add_argument("--warmup-passes", type=int, default=2,
                    help="serving workloads: untimed passes before the timed one (they record the decode graphs)")
    return ap.parse_args()


def serving_run(args, cfg, model, layers, full_layers) -> int:
    """The scheduler's workloads: every request through LLMEngine.submit / step until all have finished."""
    import torch
    from qwen_engine_amd import EngineConfig
    from qwen_engine_amd.engine.llm_engine import LLMEngine

    V = cfg.vocab_size
    arrive_every = 0
    if args.workload == "serving":
        n = args.requests or 64
        new_tokens, sharing = 256, False
        what = f"{n} requests, prompts uniform in [128, 2048], {new_tokens} new tokens each, portions of 512"
    elif args.workload == "arrivals":
        n = args.requests or 160
        new_tokens, sharing, arrive_every = 128, False, max(1, args.arrive_every)
        what = f"{n} requests, one every {arrive_every} steps, prompts uniform in [128, 512], {new_tokens} new tokens each"
    else:
        n = args.requests or 32
        new_tokens, sharing = 512, True
        what = f"{n} requests sharing a 1024-token prefix, 1024 tokens of their own, {new_tokens} new tokens each"

    def make_prompts(seed):
        g = torch.Generator().manual_seed(seed)
        if args.workload == "serving":
            lens = torch.randint(128, 2049, (n,), generator=g).tolist()
            return [torch.randint(0, V, (k,), generator=g).tolist() for k in lens]
        if args.workload == "arrivals":
            # (other lengths and other tokens in every pass: the timed pass meets shapes of steps that the
            # passes before it did not, as a server does; the line reports how many steps were replayed)
            lens = torch.randint(128, 513, (n,), generator=g).tolist()
            return [torch.randint(0, V, (k,), generator=g).tolist() for k in lens]
        prefix = torch.randint(0, V, (1024,), generator=g).tolist()
        return [prefix + torch.randint(0, V, (1024,), generator=g).tolist() for _ in range(n)]

    prompts = make_prompts(args.seed + 2)
    longest = (512 if arrive_every else 2048) + new_tokens
    P = args.block_size
    live = min(n, 64) if arrive_every else n
    pages = live * ((longest + P - 1) // P + 1)
    ecfg = EngineConfig(dtype="bfloat16" if args.dtype == "bf16" else "float32", block_size=P, num_blocks=pages,
                        max_num_seqs=live, max_model_len=longest, max_step_tokens=2048, prefill_chunk=512,
                        enable_prefix_sharing=sharing, seed=args.seed, record_mixed_steps=not args.eager_mixed_steps)
    engine = LLMEngine(model, None, ecfg)

    def run_all(ps, phase=0):
        """All at once, or one request every arrive_every steps (the first after ``phase`` steps); returns the steps."""
        steps, nxt, last = 0, 0, time.perf_counter()
        if not arrive_every:
            engine.submit(ps, max_new_tokens=new_tokens, ignore_eos=True)
            nxt = len(ps)
        while nxt < len(ps) or engine.scheduler.has_work():
            if nxt < len(ps) and (steps + phase) % arrive_every == 0:
                engine.submit([ps[nxt]], max_new_tokens=new_tokens, ignore_eos=True)
                nxt += 1
            engine.step()
            steps += 1
            if time.perf_counter() - last > 30:
                last = time.perf_counter()
                print(f"[bench] {steps} steps, {engine.stats()}", file=sys.stderr, flush=True)
        return steps

    # Untimed passes over the same workload with other tokens: a server records its graphs
    # once and runs for long, so the timed pass should find them recorded.
    for i in range(args.warmup_passes):
        run_all(make_prompts(args.seed + 100 + i), phase=i + 1)
        engine.run()
    before = engine.stats()
    torch.cuda.synchronize()
    t = time.perf_counter()
    steps = run_all(prompts)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t
    stats = engine.stats()
    results = engine.run()
    assert all(len(r.token_ids) == new_tokens for r in results), "a request did not run to its length"
    generated = n * new_tokens
    prompt_tokens = sum(len(p) for p in prompts)
    line = {
        "metric": f"generated tok/s, {args.workload} workload (Qwen3-{args.model.upper()} sizes)",
        "value": round(generated / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup_passes,
        "ms_per_step": round(dt / steps * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: random weights N(0, 0.02), uniform-random token ids",
        "config": {"model": f"Qwen3-{args.model.upper()} sizes (random weights)", "layers": layers,
                   "layers_of_model": full_layers, "hidden_size": cfg.hidden_size,
                   "num_attention_heads": cfg.num_attention_heads, "num_key_value_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate_size, "vocab_size": V,
                   "workload": what, "requests": n, "page_size": P, "prefix_sharing": sharing,
                   "parallelism": "single GPU"},
        "seconds": round(dt, 3), "prompt_tokens": prompt_tokens, "generated_tokens": generated,
        "all_tokens_per_s": round((prompt_tokens + generated) / dt, 1),
        "warmup_unit": "passes over the workload with other tokens",
        "scheduler": {k: v - before.get(k, 0) for k, v in stats.items() if isinstance(v, (int, float))},
    }
    # how many of the timed steps were replayed from a recorded graph (the others ran as they came: shapes
    # not met often enough yet, or of a kind that is not recorded)
    line["graph_hit_rate"] = round(line["scheduler"].get("graph_steps", 0) / max(1, steps), 4)
    line["scheduler"]["graph_bytes"] = stats.get("graph_bytes", 0)
    print(json.dumps(line), flush=True)
    return 0


def kernel_sweep(args, cfg) -> int:
    """Each kernel of a layer alone.  A kernel's time is that of a recorded graph of ``reps`` launches, each on
    another copy of its weights (or cache), the copies together larger than the 256 MB memory-side cache: as in
    a model step, where a layer's weights come from HBM.  Products are asked for as the parts ask for them."""
    import torch
    from qwen_engine_amd.kernels import ops

    dev = torch.device("cuda:0")
    bf = torch.bfloat16
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    Hq, Hkv, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    P, ctx_len = args.block_size, args.context
    copy_gbs = None
    probe = ops.mfma_probe() / 1e12
    g = torch.Generator(device="cpu").manual_seed(args.seed)

    def timed(launch, reps):
        """launch(i): the i-th launch.  Microseconds a launch, the best of three replays."""
        for i in range(min(reps, 3)):
            launch(i)
        torch.cuda.synchronize()
        stream = torch.cuda.Stream()
        stream.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            with ops.one_stream():
                for i in range(reps):
                    launch(i)
        best = None
        for _ in range(3):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()
            b.record()
            b.synchronize()
            t = a.elapsed_time(b) * 1e3 / reps
            best = t if best is None else min(best, t)
        return best

    def copies_of(nbytes):
        return max(2, min(48, -(-(640 << 20) // max(1, nbytes))))

    rows_all = (1, 8, 64, 512, 2048)
    out = []

    def record(name, rows, us, nbytes, flops, note=""):
        gbs, tf = nbytes / us / 1e3, flops / us / 1e6
        out.append({"kernel": name, "rows": rows, "us": round(us, 2), "gbs": round(gbs, 1), "tflops": round(tf, 1),
                    "frac_hbm": round(gbs / HBM_PEAK_GBS, 4), "frac_mfma": round(tf * 1e12 / PEAK_FLOPS["bf16"], 4),
                    "frac_mfma_measured": round(tf / probe, 4), **({"note": note} if note else {})})
        print(f"[bench] {name:28s} rows {rows:5d}  {us:9.2f} us  {gbs:8.1f} GB/s  {tf:8.1f} TFLOP/s  {note}",
              file=sys.stderr, flush=True)

    products = [("q|k|v product", (Hq + 2 * Hkv) * D, H, "store"), ("o product", H, Hq * D, "branch"),
                ("gate|up product + silu.mul", 2 * I, H, "silu"), ("down product", H, I, "branch"),
                ("head product (32-bit logits)", V, H, "head")]
    for name, N, K, kind in products:
        n = copies_of(N * K * 2)
        ws = [(torch.randn(N, K, generator=g) * 0.02).to(bf).to(dev) for _ in range(2)]
        ws = ws + [ws[i % 2].clone() for i in range(n - 2)]
        if kind == "silu":
            ws = [ops.interleave_gate_up(w[:N // 2], w[N // 2:]) for w in ws]
        for rows in rows_all:
            if kind == "head" and rows > 64:
                continue                                   # (logits are asked for at a step's wanted rows only)
            x = torch.randn(rows, K, generator=g).to(bf).to(dev)
            if kind == "silu":
                f = (lambda i: ops.gemm(x, ws[i % n], epilogue=ops.EPI_SILU_MUL_IL)) if ops.gemm_silu_supported(x, ws[0]) \
                    else (lambda i: ops.silu_mul(ops.gemm(x, ws[i % n]), interleaved=True))
            elif kind == "branch":
                splits = ops.gemm_branch_splits(x, ws[0])
                f = (lambda i: ops.gemm(x, ws[i % n], epilogue=ops.EPI_PARTIAL, splits=splits)) if splits \
                    else (lambda i: ops.gemm(x, ws[i % n]))
            elif kind == "head":
                f = lambda i: ops.gemm(x, ws[i % n], out_dtype=torch.float32)
            else:
                f = lambda i: ops.gemm(x, ws[i % n])
            us = timed(f, 2 * n)
            record(name, rows, us, N * K * 2 + rows * K * 2, 2.0 * rows * N * K,
                   f"{splits} partial products" if kind == "branch" and splits else "")
        del ws
        torch.cuda.empty_cache()

    # attention over the cache: decode (rows requests, one new token each, at the context), and one prompt portion
    scale = 1.0 / D ** 0.5
    pages_per_req = -(-ctx_len // P)
    for rows in (1, 8, 64):
        kv_bytes = rows * ctx_len * 2 * Hkv * D * 2
        n = max(2, min(8, -(-(640 << 20) // kv_bytes)))
        caches = [torch.randn(rows * pages_per_req, 2, Hkv, P, D, device=dev).to(bf) for _ in range(n)]
        table = torch.arange(rows * pages_per_req, dtype=torch.int32, device=dev).view(rows, pages_per_req)
        pos = torch.full((rows,), ctx_len - 1, dtype=torch.int32, device=dev)
        seq = torch.arange(rows, dtype=torch.int32, device=dev)
        q = torch.randn(rows, Hq, D, device=dev).to(bf)
        f = lambda i: ops.attention(q, caches[i % n], pos, seq, table, scale, dec_tokens=seq, max_dec_position=ctx_len - 1,
                                    other_tokens=None)
        us = timed(f, 4 * n)
        record("decode attention (split + merge)", rows, us, kv_bytes, 4.0 * rows * Hq * D * ctx_len, f"context {ctx_len}")
        del caches
        torch.cuda.empty_cache()
    from qwen_engine_amd.parts.attention import prefill_tiles
    for rows in (64, 512, 2048):
        for before in (0, max(0, ctx_len - rows)):
            if before == 0 and rows > ctx_len:
                continue
            keys = before + rows
            pages = -(-keys // P)
            cache = torch.randn(pages, 2, Hkv, P, D, device=dev).to(bf)
            table = torch.arange(pages, dtype=torch.int32, device=dev).view(1, pages)
            pos = torch.arange(before, keys, dtype=torch.int32, device=dev)
            seq = torch.zeros(rows, dtype=torch.int32, device=dev)
            q = torch.randn(rows, Hq, D, device=dev).to(bf)
            other = torch.arange(rows, dtype=torch.int32, device=dev)
            tiles = torch.tensor(prefill_tiles([(0, rows)], ops.prefill_tile_rows(Hq, Hkv)), dtype=torch.int32).view(-1, 2).to(dev)
            f = lambda i: ops.attention(q, cache, pos, seq, table, scale, dec_tokens=None, other_tokens=other,
                                        other_tiles=tiles, max_other_keys=keys)
            us = timed(f, 8)
            flops = 4.0 * Hq * D * (rows * before + rows * (rows + 1) / 2.0)
            record("prefill attention", rows, us, keys * 2 * Hkv * D * 2, flops, f"after {before} cached tokens")
            del cache
            if before == max(0, ctx_len - rows):
                break
    line = {"metric": f"per-kernel sweep (Qwen3-{args.model.upper()} sizes)", "unit": "us", "n_gpus": 1, "dtype": "bf16",
            "data": "synthetic: random operands", "config": {"model": f"Qwen3-{args.model.upper()} sizes", "hidden_size": H,
            "num_attention_heads": Hq, "num_key_value_heads": Hkv, "head_dim": D, "intermediate_size": I, "vocab_size": V,
            "context": ctx_len, "page_size": P},
            "peaks": {"hbm_gbs": HBM_PEAK_GBS, "mfma_tflops": PEAK_FLOPS["bf16"] / 1e12, "measured_mfma_tflops": round(probe, 1)},
            "kernels": out}
    print(json.dumps(line), flush=True)
    return 0


def main() -> int:
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only: --gpus {args.gpus} is not supported (the engine has no multi-GPU path)")
        return 2
    import torch
    import qwen_engine_amd  # noqa: F401
    from qwen_engine_amd.config import Qwen3Config
    from qwen_engine_amd.engine import ModelRunner, StepEntry
    from qwen_engine_amd.kernels import ops
    from qwen_engine_amd.parts import DecoderModel, Runtime
    from qwen_engine_amd.weights import random_tensors

    sizes = SIZES[args.model]
    full_layers = sizes["num_hidden_layers"]
    layers = args.layers or full_layers
    cfg = Qwen3Config.from_dict(dict(sizes, num_hidden_layers=layers))
    dtype = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    ops.load_library()

    if args.kernels:
        return kernel_sweep(args, cfg)

    t0 = time.time()
    model = DecoderModel(cfg.to_model_spec())
    model.load(random_tensors(cfg, args.seed, dtype=torch.bfloat16), Runtime(dev, dtype))
    print(f"[bench] random weights for {layers} layers in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)

    if args.workload != "decode":
        return serving_run(args, cfg, model, layers, full_layers)

    P = args.block_size
    itemsize = 2 if args.dtype == "bf16" else 4
    H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    Hq, Hkv, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    layer_params = (Hq + 2 * Hkv) * D * H + Hq * D * H + 3 * H * I
    # every weight a step uses once, as the model counts its own tensors; for this architecture that is
    # the layers' matrices and the head in the element type, and the norms' weights in 32-bit
    weight_bytes = model.weight_bytes_read_per_step()
    assert weight_bytes == (layers * layer_params + V * H) * itemsize + (layers * (2 * H + 2 * D) + H) * 4, weight_bytes
    kv_bytes_per_token = layers * 2 * Hkv * D * itemsize
    g = torch.Generator().manual_seed(args.seed + 1)

    def decode_run(batch, context, steps, warmup):
        """Prefill `batch` requests so that `warmup + steps` decode steps end at `context` tokens."""
        pages = batch * ((context + P - 1) // P + 1)
        runner = ModelRunner(model, page_size=P, num_pages=pages, max_requests=batch)
        start = context - (warmup + steps)
        ids = list(range(batch))
        for r in ids:
            runner.add_request(r)
        last = None
        chunk = 2048
        for r in ids:
            toks = torch.randint(0, V, (start,), generator=g).tolist()
            for a in range(0, start, chunk):
                part = toks[a:a + chunk]
                want = [len(part) - 1] if a + chunk >= start else []
                out = runner.step([StepEntry(r, part, want)])
            last = out
        tokens = torch.randint(0, V, (batch,), generator=g).tolist()

        def one_step(tokens):
            # greedy: the recorded step picks the tokens itself; the host needs them to go on (a sync per step)
            return runner.step([StepEntry(r, [tokens[i]], [0]) for i, r in enumerate(ids)], greedy=True)

        for _ in range(warmup):
            tokens = one_step(tokens)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            tokens = one_step(tokens)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        for r in ids:
            runner.free_request(r)
        del runner
        torch.cuda.empty_cache()
        mean_ctx = context - steps / 2.0
        step_bytes = weight_bytes + batch * mean_ctx * kv_bytes_per_token
        return dict(tok_s=batch * steps / dt, ms=dt / steps * 1e3, gbs=step_bytes / (dt / steps) / 1e9)

    def prefill_run(T, reps=3):
        runner = ModelRunner(model, page_size=P, num_pages=(T + P - 1) // P + 1, max_requests=1)
        toks = torch.randint(0, V, (T,), generator=g).tolist()
        portion = args.prefill_portion or T
        best = None
        for _ in range(reps + 1):
            runner.add_request("p")
            torch.cuda.synchronize()
            t = time.perf_counter()
            for a in range(0, T, portion):
                part = toks[a:a + portion]
                last = a + portion >= T
                first_token = runner.step([StepEntry("p", part, [len(part) - 1] if last else [])], greedy=last)
            assert len(first_token) == 1
            torch.cuda.synchronize()
            dt = time.perf_counter() - t
            runner.free_request("p")
            best = dt if best is None else min(best, dt)     # the first repetition warms up
        flops = 2.0 * T * layers * layer_params + 2.0 * V * H \
            + layers * 4.0 * Hq * D * T * (T + 1) / 2.0
        del runner
        torch.cuda.empty_cache()
        return dict(value=T / best, tokens=T, ms=best * 1e3, frac=flops / best / PEAK_FLOPS[args.dtype])

    def copy_gbs():
        """What a plain device-to-device copy of 1 GiB reaches (read + write), for scale beside the 8 TB/s."""
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t) / 10
        del src, dst
        torch.cuda.empty_cache()
        return 2 * (1 << 30) / dt / 1e9

    main_run = decode_run(args.batch, args.context, args.steps, args.warmup)
    print(f"[bench] decode batch {args.batch}: {main_run}", file=sys.stderr, flush=True)
    prefill = prefill_run(args.prefill_tokens)
    print(f"[bench] prefill: {prefill}", file=sys.stderr, flush=True)
    points = {}
    if not args.skip_points:
        for b in (1, 64):
            r = decode_run(b, args.context, max(8, args.steps // 2), max(2, args.warmup // 2))
            points[f"decode_b{b}"] = round(r["tok_s"], 1)
            print(f"[bench] decode batch {b}: {r}", file=sys.stderr, flush=True)

    line = {
        "metric": f"decode tok/s @ batch {args.batch} (Qwen3-{args.model.upper()} sizes, context {args.context})",
        "value": round(main_run["tok_s"], 1),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_run["ms"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic: random weights N(0, 0.02), uniform-random token ids",
        "config": {
            "model": f"Qwen3-{args.model.upper()} sizes (random weights)", "layers": layers, "layers_of_model": full_layers,
            "hidden_size": H, "num_attention_heads": Hq, "num_key_value_heads": Hkv, "head_dim": D,
            "intermediate_size": I, "vocab_size": V, "tie_word_embeddings": cfg.tie_word_embeddings,
            "global_batch": args.batch, "seq_len": args.context, "page_size": P,
            "prefill_tokens": args.prefill_tokens, "parallelism": "single GPU",
            **({"prefill_portion": args.prefill_portion} if args.prefill_portion else {}),
        },
        "prefill": {"value": round(prefill["value"], 1), "tokens": prefill["tokens"],
                    "ms": round(prefill["ms"], 3), "frac": round(prefill["frac"], 4),
                    "timing": "best of 3 repetitions (the decode figures are means over their steps)"},
        "roofline": {"bound": "hbm", "achieved": round(main_run["gbs"], 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(main_run["gbs"] / HBM_PEAK_GBS, 4)},
        "points": points,
        "measured_copy_gbs": round(copy_gbs(), 1),
        "measured_mfma_tflops": round(ops.mfma_probe() / 1e12, 1),
    }
    line["prefill"]["frac_of_measured"] = round(prefill["frac"] * PEAK_FLOPS[args.dtype] / (line["measured_mfma_tflops"] * 1e12), 4) \
        if args.dtype == "bf16" else None
    line["roofline"]["frac_of_measured_copy"] = round(main_run["gbs"] / line["measured_copy_gbs"], 4)
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
