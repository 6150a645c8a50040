"""Each part of a layer alone against the plain implementation, at sizes of their own."""
import math

import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
DTYPES = [torch.float32, torch.bfloat16]


def rand(*shape, seed=0, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def close(got, want, dtype):
    got, want = got.float().cpu(), want.float().cpu()
    tol = 2e-5 if dtype == torch.float32 else 1.5e-2
    err, s = float((got - want).abs().max()), float(want.abs().max())
    assert err <= tol * s, f"error {err} beside scale {s}"


def branch(y):
    """A mixer's or feed-forward's output: [T, H], or float32 partial products [S, T, H]."""
    return y.float().sum(0) if y.dim() == 3 else y.float()


def one_request_context(rt, positions, page, num_pages, want_rows=()):
    """A step context for one request whose tokens sit at the given positions, with the pages
    of its table shuffled; returns (ctx, table row)."""
    from qwen_engine_amd.engine.batch import SeqInfo, StepContext
    T = len(positions)
    n_pages = (max(positions) + page) // page
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(9))[:n_pages].to(torch.int32)
    slots = torch.tensor([int(perm[p // page]) * page + p % page for p in positions], dtype=torch.int32)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=rt.device)
    ctx = StepContext(rt=rt, page_size=page, num_tokens=T,
                      seqs=[SeqInfo("r", 0, T, positions[0], 0, True)],
                      token_ids=i32([0] * T), positions=i32(list(positions)), tok_seq=i32([0] * T),
                      block_tables=[perm[None].to(rt.device)], slots=[slots.to(rt.device)],
                      logit_rows=i32(list(want_rows)), state_slots=i32([0]), max_position=max(positions))
    return ctx


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    from qwen_engine_amd.config import RMSNormSpec
    from qwen_engine_amd.parts import Runtime, build_part
    rt = Runtime(DEV, dtype)
    part = build_part(RMSNormSpec(eps=3e-5), 112)
    w = (1 + rand(112, seed=1, scale=0.1)).to(torch.bfloat16)          # stored in 16 bits, held in 32
    part.load({"weight": w}, rt)
    assert part.weight.dtype == torch.float32
    h = rand(5, 112, seed=2)
    close(part.forward(h.to(DEV), rt), P.rms_norm(h, w.float(), 3e-5), dtype)


def test_rotary_table_is_the_reference_formula():
    from qwen_engine_amd.config import RopeSpec
    from qwen_engine_amd.parts import Runtime, build_part
    for theta, d, n in ((10000.0, 16, 100), (1e6, 128, 3000), (50000.0, 48, 77)):
        part = build_part(RopeSpec(theta=theta, rotary_dim=d, max_positions=n), 0)
        part.load({}, Runtime(DEV, torch.bfloat16))
        table = part.table()
        assert table.dtype == torch.float32 and tuple(table.shape) == (n, d)
        assert torch.equal(table.cpu(), P.rope_table(theta, d, n))      # same operations, same bits


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,I,T", [(80, 112, 6), (96, 160, 6), (128, 192, 70)])
def test_swiglu_part(dtype, H, I, T):
    """Widths with and without gate|up interleaving (multiples of 32 or not), few and many rows."""
    from qwen_engine_amd.config import SwiGLUSpec
    from qwen_engine_amd.parts import Runtime, build_part
    rt = Runtime(DEV, dtype)
    part = build_part(SwiGLUSpec(intermediate_size=I), H)
    w = {"gate_proj.weight": rand(I, H, seed=3, scale=0.2, dtype=torch.bfloat16),
         "up_proj.weight": rand(I, H, seed=4, scale=0.2, dtype=torch.bfloat16),
         "down_proj.weight": rand(H, I, seed=5, scale=0.2, dtype=torch.bfloat16)}
    part.load(w, rt)
    x = rand(T, H, seed=6, dtype=dtype)
    assert part.interleaved == (I % 32 == 0)
    got = branch(part.forward(x.to(DEV), None))
    act = None if dtype == torch.float32 else dtype
    want = P.mlp_block(x.float(), {f"p.mlp.{k}": v for k, v in w.items()}, "p", act_dtype=act)
    close(got, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("window", [None, 7])
def test_attention_part_in_two_portions(dtype, bias, window):
    """The mixer alone: 20 tokens as a portion of 13 and one of 7 over shuffled pages, against the
    plain block on the whole sequence; with q/k/v bias (and then no q/k norm) and with a window."""
    from qwen_engine_amd.config import AttentionSpec, RopeSpec
    from qwen_engine_amd.parts import CacheBinding, Runtime, build_part
    rt = Runtime(DEV, dtype)
    H, hq, hkv, d, page, T = 80, 6, 2, 48, 4, 20
    spec = AttentionSpec(num_heads=hq, num_kv_heads=hkv, head_dim=d, scale=1 / math.sqrt(d), qkv_bias=bias,
                         qk_norm_eps=None if bias else 1e-5, window=window,
                         position=RopeSpec(theta=10000.0, rotary_dim=d, max_positions=64))
    part = build_part(spec, H)
    names = {"q_proj.weight": (hq * d, H), "k_proj.weight": (hkv * d, H), "v_proj.weight": (hkv * d, H),
             "o_proj.weight": (H, hq * d)}
    w = {n: rand(*s, seed=10 + i, scale=0.2, dtype=torch.bfloat16) for i, (n, s) in enumerate(names.items())}
    if bias:
        for i, (n, width) in enumerate((("q", hq * d), ("k", hkv * d), ("v", hkv * d))):
            w[f"{n}_proj.bias"] = rand(width, seed=20 + i, scale=0.3, dtype=torch.bfloat16)
    else:
        w["q_norm.weight"] = (1 + rand(d, seed=30, scale=0.1)).to(torch.bfloat16)
        w["k_norm.weight"] = (1 + rand(d, seed=31, scale=0.1)).to(torch.bfloat16)
    assert set(part.expected_tensors(spec, H)) == set(w)
    part.load(w, rt)
    x = rand(T, H, seed=40, dtype=dtype)
    cache = torch.full((12, 2, hkv, page, d), float("nan"), dtype=dtype, device=DEV)
    binding = CacheBinding(kv=cache, group=0, write=True, state=None)
    outs = []
    for a, b in ((0, 13), (13, 20)):
        ctx = one_request_context(rt, list(range(a, b)), page, 12)
        # both portions must use the same pages: the table is a function of the seed only
        full = one_request_context(rt, list(range(0, T)), page, 12)
        ctx.block_tables = full.block_tables
        ctx.slots = [full.slots[0][a:b].contiguous()]
        outs.append(branch(part.forward(x[a:b].to(DEV), ctx, binding)))
    cfg = dict(num_attention_heads=hq, num_key_value_heads=hkv, head_dim=d, rms_norm_eps=1e-5, attention_bias=bias)
    act = None if dtype == torch.float32 else dtype
    want = P.attention_block(x.float(), torch.arange(T), {f"p.self_attn.{k}": v for k, v in w.items()}, "p",
                             cfg, P.rope_table(10000.0, d, 64), act_dtype=act, window=window)
    close(torch.cat(outs), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_part_defers_its_last_residual_sum(dtype):
    from qwen_engine_amd.config import Qwen3Config
    from qwen_engine_amd.parts import CacheBinding, Runtime, build_part
    from qwen_engine_amd.weights import random_tensors
    from tiny import TINY_C
    rt = Runtime(DEV, dtype)
    cfg = Qwen3Config.from_dict(TINY_C)
    spec = cfg.to_model_spec()
    block = build_part(spec.layers[1], cfg.hidden_size)
    w = random_tensors(cfg, 5, std=0.2, norm_std=0.1)
    pre = "model.layers.1."
    block.load({k[len(pre):]: v for k, v in w.items() if k.startswith(pre)}, rt)
    T, page = 9, 4
    h = rand(T, cfg.hidden_size, seed=50)
    pending = rand(T, cfg.hidden_size, seed=51, dtype=dtype)
    cache = torch.zeros(8, 2, cfg.num_key_value_heads, page, cfg.head_dim, dtype=dtype, device=DEV)
    ctx = one_request_context(rt, list(range(T)), page, 8)
    hd = h.to(DEV)
    out = block.forward(hd, pending.to(DEV), ctx, [CacheBinding(cache, 0, True, None)])
    act = None if dtype == torch.float32 else dtype
    table = P.rope_table(cfg.rope_theta, cfg.head_dim, cfg.max_position_embeddings)
    h_in = h + pending.float()
    h_ref = P.decoder_layer(h_in, torch.arange(T), w, "model.layers.1", TINY_C, table, act_dtype=act)
    close(hd.cpu() + branch(out).cpu(), h_ref, dtype)       # stream + pending branch = the layer's output
