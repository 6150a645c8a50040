"""Block kinds defined here, not in the framework: one with two mixers side by side
(x += a(norm(x)) + b(norm(x)), then the feed-forward), a being attention over all keys and b a
class derived from the framework's attention part, with a window, other head counts and a cache
group of its own; and one with no mixer at all (a feed-forward alone).  The framework asks a block
what its parts keep per request (``cache_needs``: two cache users, none) and hands the block one
binding per user; nothing in it assumes one mixer a block.  The toy is registered, built from a
model folder, and replayed in every cutting in both element types against a plain forward over
whole sequences; its decode steps run from recorded graphs."""
import math
from dataclasses import dataclass

import pytest
import torch

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.config import (AttentionSpec, LayerSpec, ModelSpec, RMSNormSpec, RopeSpec, ScheduleEntry,
                                    SwiGLUSpec, register_architecture, unregister_architecture)
from qwen_engine_amd.kernels import ops
from qwen_engine_amd.parts import TensorInfo, register_part, unregister_part
from qwen_engine_amd.parts.attention import PagedAttention
from qwen_engine_amd.parts.base import sub_tensors
from qwen_engine_amd.parts.registry import build_part, part_class
from qwen_engine_amd.weights import write_model_folder
from plain import qwen3_plain as P
import traces

pytestmark = pytest.mark.gpu

H, V, I, PAGE = 64, 113, 96, 4
A_HEADS, B_HEADS = (4, 2, 16), (6, 1, 32)        # (query heads, key/value heads, head size) of the two mixers
WINDOW = 11
EPS, THETA, MAXPOS = 1e-6, 10000.0, 384


class WindowedAttention(PagedAttention):
    """The framework's attention part under another class: what the step function prepares for it is filed
    under this class, and the part finds it there."""


@dataclass(frozen=True)
class TwoMixersSpec:
    prefix: str
    norm: object
    mixer_a: object
    mixer_b: object
    ffn_norm: object
    ffn: object
    kind: str = "toy_two_mixers"


class TwoMixersBlock:
    def __init__(self, spec, hidden):
        self.spec = spec
        self.norm = build_part(spec.norm, hidden)
        self.a = build_part(spec.mixer_a, hidden)
        self.b = build_part(spec.mixer_b, hidden)
        self.ffn_norm = build_part(spec.ffn_norm, hidden)
        self.ffn = build_part(spec.ffn, hidden)

    NAMES = ("norm", "att_a", "att_b", "ffn_norm", "mlp")

    def parts(self):
        return (self.norm, self.a, self.b, self.ffn_norm, self.ffn)

    @staticmethod
    def _specs(spec):
        return (spec.norm, spec.mixer_a, spec.mixer_b, spec.ffn_norm, spec.ffn)

    @staticmethod
    def expected_tensors(spec, hidden):
        out = {}
        for name, sub in zip(TwoMixersBlock.NAMES, TwoMixersBlock._specs(spec)):
            for rel, info in part_class(sub.kind).expected_tensors(sub, hidden).items():
                out[f"{name}.{rel}"] = info
        return out

    @staticmethod
    def cache_needs(spec, hidden):
        return [(part_class(m.kind).cache_need(m), None) for m in (spec.mixer_a, spec.mixer_b)]

    def load(self, tensors, rt):
        for name, part in zip(self.NAMES, self.parts()):
            part.load(sub_tensors(tensors, name + "."), rt)

    def forward(self, h, pending, ctx, bindings):
        assert len(bindings) == 2 and bindings[0].group != bindings[1].group
        stream = h if not isinstance(h, torch.Tensor) else None
        hh = stream.h if stream is not None else h
        x = self.norm.forward(hh, ctx.rt, delta=pending)
        ya = self.a.forward(x, ctx, bindings[0])
        yb = self.b.forward(x, ctx, bindings[1])
        ops.residual_add(hh, ya)                       # (a branch output may be partial products: added in order)
        x = self.ffn_norm.forward(hh, ctx.rt, delta=yb)
        return self.ffn.forward(x, ctx)


@dataclass(frozen=True)
class FeedForwardOnlySpec:
    prefix: str
    norm: object
    ffn: object
    kind: str = "toy_ffn_only"


class FeedForwardOnlyBlock:
    """x += ffn(norm(x)): no mixer, so no cache user (the class has no cache_needs at all)."""

    def __init__(self, spec, hidden):
        self.norm = build_part(spec.norm, hidden)
        self.ffn = build_part(spec.ffn, hidden)

    def parts(self):
        return (self.norm, self.ffn)

    @staticmethod
    def expected_tensors(spec, hidden):
        out = {}
        for name, sub in (("norm", spec.norm), ("mlp", spec.ffn)):
            for rel, info in part_class(sub.kind).expected_tensors(sub, hidden).items():
                out[f"{name}.{rel}"] = info
        return out

    def load(self, tensors, rt):
        self.norm.load(sub_tensors(tensors, "norm."), rt)
        self.ffn.load(sub_tensors(tensors, "mlp."), rt)

    def forward(self, h, pending, ctx, bindings):
        assert len(bindings) == 0
        hh = h.h if not isinstance(h, torch.Tensor) else h
        return self.ffn.forward(self.norm.forward(hh, ctx.rt, delta=pending), ctx)


class ToyBlocksConfig:
    architecture = "ToyBlocksForCausalLM"

    def __init__(self, d):
        self.d = d

    def to_dict(self):
        return dict(self.d)

    def to_model_spec(self):
        norm, ffn = RMSNormSpec(eps=EPS), SwiGLUSpec(intermediate_size=I)

        def att(heads, window, kind):
            hq, hkv, d = heads
            return AttentionSpec(num_heads=hq, num_kv_heads=hkv, head_dim=d, scale=1 / math.sqrt(d), qk_norm_eps=EPS,
                                 window=window, position=RopeSpec(theta=THETA, rotary_dim=d, max_positions=MAXPOS), kind=kind)

        layers = (TwoMixersSpec("model.layers.0", norm, att(A_HEADS, None, "paged_attention"),
                                att(B_HEADS, WINDOW, "toy_windowed_attention"), norm, ffn),
                  FeedForwardOnlySpec("model.layers.1", norm, ffn),
                  LayerSpec(prefix="model.layers.2", mixer_norm=norm, mixer=att(A_HEADS, None, "paged_attention"),
                            ffn_norm=norm, ffn=ffn))
        return ModelSpec(architecture=self.architecture, vocab_size=V, hidden_size=H, layers=layers,
                         schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2)), final_norm=norm,
                         embed_name="model.embed_tokens.weight", final_norm_name="model.norm.weight",
                         head_name="lm_head.weight", tie_head=False, max_positions=MAXPOS)


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    register_part("toy_two_mixers", TwoMixersBlock)
    register_part("toy_ffn_only", FeedForwardOnlyBlock)
    register_part("toy_windowed_attention", WindowedAttention)
    register_architecture(ToyBlocksConfig.architecture, ToyBlocksConfig)
    folder = str(tmp_path_factory.mktemp("toy_blocks") / "model")
    write_model_folder(folder, ToyBlocksConfig({"architectures": [ToyBlocksConfig.architecture]}), seed=17,
                       dtype=torch.bfloat16, std=0.15, norm_std=0.05)
    yield folder
    unregister_architecture(ToyBlocksConfig.architecture)
    for kind in ("toy_two_mixers", "toy_ffn_only", "toy_windowed_attention"):
        unregister_part(kind)


def plain_attention(x, pos, w, pre, heads, window, rnd):
    hq, hkv, d = heads
    t = x.shape[0]
    f = lambda name: w[f"{pre}.{name}"].float()
    table = P.rope_table(THETA, d, MAXPOS)
    q = P.rms_norm(rnd(P.linear(x, f("q_proj.weight"))).view(t, hq, d), f("q_norm.weight"), EPS)
    k = P.rms_norm(rnd(P.linear(x, f("k_proj.weight"))).view(t, hkv, d), f("k_norm.weight"), EPS)
    v = rnd(P.linear(x, f("v_proj.weight"))).view(t, hkv, d)
    q, k = rnd(P.apply_rope(table, pos, q)), rnd(P.apply_rope(table, pos, k))
    o = rnd(P.attention(q, k, v, 1 / math.sqrt(d), pos, pos, window=window)).reshape(t, hq * d)
    return rnd(P.linear(o, f("o_proj.weight")))


def plain_forward(w, toks, act=None):
    rnd = (lambda t: t) if act is None else (lambda t: t.to(act).float())
    f = lambda name: w[name].float()
    pos = torch.arange(len(toks))
    h = P.embedding(torch.tensor(toks), w["model.embed_tokens.weight"]).float()
    x = rnd(P.rms_norm(h, f("model.layers.0.norm.weight"), EPS))
    h = h + plain_attention(x, pos, w, "model.layers.0.att_a", A_HEADS, None, rnd) \
          + plain_attention(x, pos, w, "model.layers.0.att_b", B_HEADS, WINDOW, rnd)
    x = rnd(P.rms_norm(h, f("model.layers.0.ffn_norm.weight"), EPS))
    h = h + P.mlp_block(x, w, "model.layers.0", act)
    x = rnd(P.rms_norm(h, f("model.layers.1.norm.weight"), EPS))
    h = h + P.mlp_block(x, w, "model.layers.1", act)
    cfg = dict(num_attention_heads=A_HEADS[0], num_key_value_heads=A_HEADS[1], head_dim=A_HEADS[2], rms_norm_eps=EPS)
    h = P.decoder_layer(h, pos, w, "model.layers.2", cfg, P.rope_table(THETA, A_HEADS[2], MAXPOS), act_dtype=act)
    return P.linear(rnd(P.rms_norm(h, f("model.norm.weight"), EPS)), f("lm_head.weight"))


def test_the_plan_of_blocks_with_two_cache_users_and_with_none(toy):
    from qwen_engine_amd.config import config_from_folder
    from qwen_engine_amd.engine import ModelRunner, load_model
    from qwen_engine_amd.parts import cache_plan
    plan = cache_plan(config_from_folder(toy).to_model_spec())
    assert plan.entry_users == [[0, 1], [], [2]]
    assert [g.window for g in plan.groups] == [None, WINDOW] and plan.user_group == [0, 1, 0]
    model = load_model(toy, dtype="bfloat16")
    runner = ModelRunner(model, page_size=PAGE, num_pages=40, max_requests=2)
    assert [len(b) for b in runner.bindings] == [2, 0, 1] and runner.use_graphs
    assert WindowedAttention in runner._step_classes and PagedAttention in runner._step_classes
    # the step's weight bytes, counted through blocks of any kind: every tensor of the folder but the embedding table
    _, w = P.read_folder(toy)
    held = sum(t.numel() * (2 if t.dim() == 2 else 4) for name, t in w.items() if name != "model.embed_tokens.weight")
    assert model.weight_bytes_read_per_step() == held


@pytest.mark.parametrize("dtype,cut", [("float32", "whole"), ("float32", "tail"), ("float32", "portions"),
                                       ("float32", "mixed"), ("bfloat16", "tail"), ("bfloat16", "mixed")])
def test_toy_blocks_in_every_cutting(toy, tmp_path, dtype, cut):
    _, w = P.read_folder(toy)
    g = torch.Generator().manual_seed(35)
    reqs = {f"q{i}": torch.randint(0, V, (n,), generator=g).tolist() for i, n in enumerate((70, 45, 110, 64))}
    act = None if dtype == "float32" else torch.bfloat16
    ref = {rid: plain_forward(w, toks, act) for rid, toks in reqs.items()}
    trace = {"whole": traces.whole, "tail": traces.tail_decoded, "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, seed=9)}[cut](reqs)
    out_dir = str(tmp_path / "out")
    traces.run_in_process(trace, toy, dtype, out_dir, PAGE)
    got = traces.collect(trace, out_dir, V)
    bad, worst = traces.first_mismatch(got, ref, 1e-4 if dtype == "float32" else 2e-2)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"
