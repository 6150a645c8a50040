"""Two more parts defined here, not in the framework: a feed-forward with routing (four
experts, the best two per token, router logits and weights in 32-bit) and a position
encoding that is no rotation (the attention part then norms, hands q and k to the part, and
writes the cache from what it left).  One layer has both, with biases on q, k, v and without
the per-head norm; the other layer is the dense one with the rotary encoding.  The toy is
registered, built from a model folder and replayed in every cutting, in both element types,
against a plain forward over whole sequences."""
import math
from dataclasses import dataclass

import pytest
import torch

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.config import (AttentionSpec, LayerSpec, ModelSpec, RMSNormSpec, RopeSpec, ScheduleEntry,
                                    SwiGLUSpec, register_architecture, unregister_architecture)
from qwen_engine_amd.parts import TensorInfo, register_part, unregister_part
from qwen_engine_amd.weights import write_model_folder
from plain import qwen3_plain as P
import traces

pytestmark = pytest.mark.gpu

H, V, HQ, HKV, D, I, PAGE = 80, 131, 5, 1, 32, 96, 4
E, TOPK, IE = 4, 2, 48
EPS, THETA, MAXPOS = 1e-6, 50000.0, 400


# ---- a position encoding that scales: q_d *= 1 + a sin(p w_d), k_d *= 1 + a cos(p w_d) -------
@dataclass(frozen=True)
class WaveScaleSpec:
    amplitude: float
    kind: str = "toy_wave_scale"


def wave_factors(positions, amplitude):
    w = 1.0 / (torch.arange(D, dtype=torch.float32, device=positions.device) + 2.0)
    ang = positions.float()[:, None] * w[None, :]
    return 1.0 + amplitude * torch.sin(ang), 1.0 + amplitude * torch.cos(ang)


class WaveScale:
    fused = False            # the attention part calls apply() between its norm and its cache write

    def __init__(self, spec, hidden=0):
        self.amplitude = spec.amplitude

    @staticmethod
    def expected_tensors(spec, hidden):
        return {}

    def load(self, tensors, rt):
        pass

    def apply(self, packed, positions, num_q, num_k):
        fq, fk = wave_factors(positions, self.amplitude)
        q, k = packed[:, :num_q], packed[:, num_q:num_q + num_k]
        q.copy_((q.float() * fq[:, None, :]).to(packed.dtype))
        k.copy_((k.float() * fk[:, None, :]).to(packed.dtype))


# ---- a feed-forward with routing -------------------------------------------------------------
@dataclass(frozen=True)
class RoutedSpec:
    num_experts: int
    top_k: int
    intermediate_size: int
    kind: str = "toy_routed"


def routed(x, router, experts, top_k):
    """x [T, H] 32-bit; router [E, H]; experts: list of (gate, up, down).  Softmax over all experts
    in 32-bit, the best top_k (lowest index on ties), their weights renormalised to sum 1."""
    probs = torch.softmax(x @ router.t(), dim=-1)
    top_w, top_i = torch.topk(probs, top_k, dim=-1)
    top_w = top_w / top_w.sum(dim=-1, keepdim=True)
    y = torch.zeros_like(x)
    for e, (g, u, d) in enumerate(experts):
        for slot in range(top_k):
            rows = torch.nonzero(top_i[:, slot] == e)[:, 0]
            if rows.numel():
                xe = x[rows]
                a = torch.nn.functional.silu(xe @ g.t()) * (xe @ u.t())
                y[rows] += top_w[rows, slot, None] * (a @ d.t())
    return y


class RoutedFeedForward:
    graph_safe = False       # (nonzero() sizes its result by the data: not to be recorded into a graph)

    def __init__(self, spec, hidden):
        self.spec = spec

    @staticmethod
    def expected_tensors(spec, hidden):
        t = {"router.weight": TensorInfo((spec.num_experts, hidden))}
        for e in range(spec.num_experts):
            t[f"experts.{e}.gate_proj.weight"] = TensorInfo((spec.intermediate_size, hidden))
            t[f"experts.{e}.up_proj.weight"] = TensorInfo((spec.intermediate_size, hidden))
            t[f"experts.{e}.down_proj.weight"] = TensorInfo((hidden, spec.intermediate_size))
        return t

    def load(self, tensors, rt):
        f = lambda n: tensors[n].float().to(rt.device)
        self.router = f("router.weight")
        self.experts = [(f(f"experts.{e}.gate_proj.weight"), f(f"experts.{e}.up_proj.weight"),
                         f(f"experts.{e}.down_proj.weight")) for e in range(self.spec.num_experts)]

    def forward(self, x, ctx):
        return routed(x.float(), self.router, self.experts, self.spec.top_k).to(x.dtype)


# ---- the architecture ------------------------------------------------------------------------
class ToyRoutedConfig:
    architecture = "ToyRoutedForCausalLM"

    def __init__(self, d):
        self.d = d

    def to_dict(self):
        return dict(self.d)

    def to_model_spec(self):
        norm = RMSNormSpec(eps=EPS)
        plain_att = AttentionSpec(num_heads=HQ, num_kv_heads=HKV, head_dim=D, scale=0.3, qkv_bias=True,
                                  position=WaveScaleSpec(amplitude=0.4))
        rope_att = AttentionSpec(num_heads=HQ, num_kv_heads=HKV, head_dim=D, scale=1 / math.sqrt(D), qk_norm_eps=EPS,
                                 position=RopeSpec(theta=THETA, rotary_dim=D, max_positions=MAXPOS))
        layers = (LayerSpec(prefix="model.layers.0", mixer_norm=norm, mixer=plain_att, ffn_norm=norm,
                            ffn=RoutedSpec(num_experts=E, top_k=TOPK, intermediate_size=IE)),
                  LayerSpec(prefix="model.layers.1", mixer_norm=norm, mixer=rope_att, ffn_norm=norm,
                            ffn=SwiGLUSpec(intermediate_size=I)))
        return ModelSpec(architecture=self.architecture, vocab_size=V, hidden_size=H, layers=layers,
                         schedule=(ScheduleEntry(0), ScheduleEntry(1)), final_norm=norm,
                         embed_name="model.embed_tokens.weight", final_norm_name="model.norm.weight",
                         head_name="lm_head.weight", tie_head=False, max_positions=MAXPOS)


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    register_part("toy_wave_scale", WaveScale)
    register_part("toy_routed", RoutedFeedForward)
    register_architecture(ToyRoutedConfig.architecture, ToyRoutedConfig)
    folder = str(tmp_path_factory.mktemp("toy_routed") / "model")
    # (wide weights: the router's choices then differ from token to token, and biases count)
    write_model_folder(folder, ToyRoutedConfig({"architectures": [ToyRoutedConfig.architecture]}), seed=13,
                       dtype=torch.bfloat16, std=0.2, norm_std=0.05)
    # (random weights leave biases at zero: give them values, so that a bias that is lost shows)
    import os
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    g = torch.Generator().manual_seed(14)
    for name in tensors:
        if name.endswith(".bias"):
            tensors[name] = (0.5 * torch.randn(tensors[name].shape, generator=g)).to(tensors[name].dtype)
    save_file(tensors, path)
    yield folder
    unregister_architecture(ToyRoutedConfig.architecture)
    unregister_part("toy_routed")
    unregister_part("toy_wave_scale")


def plain_forward(w, toks, act=None):
    """Whole sequence, no cache.  act: the element type activations are rounded to between the
    parts (None: none), as the engine rounds them in that mode."""
    rnd = (lambda t: t) if act is None else (lambda t: t.to(act).float())
    f = lambda name: w[name].float()
    pos = torch.arange(len(toks))
    h = P.embedding(torch.tensor(toks), w["model.embed_tokens.weight"]).float()
    # layer 0: biases, no per-head norm, the scaling position encoding, routed feed-forward
    pre = "model.layers.0"
    x = rnd(P.rms_norm(h, f(f"{pre}.input_layernorm.weight"), EPS))
    t = len(toks)
    q = rnd(P.linear(x, f(f"{pre}.self_attn.q_proj.weight"), f(f"{pre}.self_attn.q_proj.bias"))).view(t, HQ, D)
    k = rnd(P.linear(x, f(f"{pre}.self_attn.k_proj.weight"), f(f"{pre}.self_attn.k_proj.bias"))).view(t, HKV, D)
    v = rnd(P.linear(x, f(f"{pre}.self_attn.v_proj.weight"), f(f"{pre}.self_attn.v_proj.bias"))).view(t, HKV, D)
    fq, fk = wave_factors(pos, 0.4)
    q, k = rnd(q * fq[:, None, :]), rnd(k * fk[:, None, :])
    o = rnd(P.attention(q, k, v, 0.3, pos, pos)).reshape(t, HQ * D)
    h = h + rnd(P.linear(o, f(f"{pre}.self_attn.o_proj.weight")))
    x = rnd(P.rms_norm(h, f(f"{pre}.post_attention_layernorm.weight"), EPS))
    experts = [(f(f"{pre}.mlp.experts.{e}.gate_proj.weight"), f(f"{pre}.mlp.experts.{e}.up_proj.weight"),
                f(f"{pre}.mlp.experts.{e}.down_proj.weight")) for e in range(E)]
    h = h + rnd(routed(x, f(f"{pre}.mlp.router.weight"), experts, TOPK))
    # layer 1: the dense layer of the framework
    cfg = dict(num_attention_heads=HQ, num_key_value_heads=HKV, head_dim=D, rms_norm_eps=EPS)
    h = P.decoder_layer(h, pos, w, "model.layers.1", cfg, P.rope_table(THETA, D, MAXPOS), act_dtype=act)
    x = rnd(P.rms_norm(h, f("model.norm.weight"), EPS))
    return P.linear(x, f("lm_head.weight"))


def test_the_toy_uses_both_new_parts(toy):
    from qwen_engine_amd.engine import load_model
    from qwen_engine_amd.parts import cache_plan
    from qwen_engine_amd.config import config_from_folder
    model = load_model(toy, dtype="float32")
    kinds = [(type(b.mixer.position).__name__, type(b.ffn).__name__) for b in model.blocks]
    assert kinds == [("WaveScale", "RoutedFeedForward"), ("RotaryHalf", "SwiGLU")]
    assert [b.graph_safe for b in model.blocks] == [False, True] and not model.graph_safe
    plan = cache_plan(config_from_folder(toy).to_model_spec())
    assert len(plan.groups) == 1 and plan.user_state == [None, None]
    # the router spreads the tokens over the experts (else the test would show little)
    _, w = P.read_folder(toy)
    x = torch.randn(200, H, generator=torch.Generator().manual_seed(1))
    top = torch.topk(torch.softmax(x @ w["model.layers.0.mlp.router.weight"].float().t(), -1), TOPK).indices
    assert all(int((top == e).sum()) >= 20 for e in range(E))


@pytest.mark.parametrize("dtype,cut", [("float32", "whole"), ("float32", "tail"), ("float32", "portions"),
                                       ("float32", "mixed"), ("bfloat16", "portions"), ("bfloat16", "mixed")])
def test_toy_parts_in_every_cutting(toy, tmp_path, dtype, cut):
    _, w = P.read_folder(toy)
    g = torch.Generator().manual_seed(33)
    reqs = {f"q{i}": torch.randint(0, V, (n,), generator=g).tolist() for i, n in enumerate((70, 45, 110, 64))}
    act = None if dtype == "float32" else torch.bfloat16
    ref = {rid: plain_forward(w, toks, act) for rid, toks in reqs.items()}
    trace = {"whole": traces.whole, "tail": traces.tail_decoded, "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, seed=8)}[cut](reqs)
    out_dir = str(tmp_path / "out")
    traces.run_in_process(trace, toy, dtype, out_dir, PAGE)
    got = traces.collect(trace, out_dir, V)
    bad, worst = traces.first_mismatch(got, ref, 1e-4 if dtype == "float32" else 2e-2)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"
