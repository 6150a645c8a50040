"""A toy architecture defined here, not in the framework: a mixer with per-request state
of fixed size, a layer with a windowed attention beside one over all keys (two cache
groups), a layer that runs twice, and a run that reads another run's cache.  It is
registered, built from a model folder and stepped through trace replay in every cutting,
without a change to the framework's files."""
import math
from dataclasses import dataclass
from typing import Optional

import pytest
import torch

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.cache import StateNeed
from qwen_engine_amd.config import (AttentionSpec, LayerSpec, ModelSpec, RMSNormSpec, RopeSpec, ScheduleEntry,
                                    SwiGLUSpec, register_architecture, unregister_architecture)
from qwen_engine_amd.parts import TensorInfo, register_part, unregister_part
from qwen_engine_amd.weights import write_model_folder
from plain import qwen3_plain as P
import traces

pytestmark = pytest.mark.gpu

H, V, HQ, HKV, D, I, WINDOW, PAGE = 48, 97, 4, 2, 16, 64, 24, 8
EPS, THETA, MAXPOS = 1e-5, 10000.0, 512


# ---- the toy mixer: a decaying sum over the request's tokens, kept in a state slot ----------
@dataclass(frozen=True)
class DecaySpec:
    decay: float
    kind: str = "toy_decay"


class DecayMixer:
    """s_t = decay * s_{t-1} + W x_t;  y_t = s_t.  The state s is carried from step to step."""

    def __init__(self, spec, hidden):
        self.decay, self.hidden = spec.decay, hidden

    @staticmethod
    def expected_tensors(spec, hidden):
        return {"proj.weight": TensorInfo((hidden, hidden))}

    @staticmethod
    def cache_need(spec):
        return None

    @staticmethod
    def state_need(spec, hidden):
        return StateNeed(shape=(hidden,), dtype="float32")

    def load(self, tensors, rt):
        self.w = tensors["proj.weight"].float().to(rt.device)

    def forward(self, x, ctx, binding):
        assert binding.kv is None and binding.state is not None
        y = torch.empty_like(x)
        u = x.float() @ self.w.t()
        for s in ctx.seqs:
            state = binding.state[s.state_slot]
            if s.new_request:
                assert float(state.abs().max()) == 0.0      # the runner cleared it
            for t in range(s.q_start, s.q_start + s.q_len):
                state.mul_(self.decay).add_(u[t])
                y[t] = state.to(x.dtype)
        return y


# ---- the toy architecture --------------------------------------------------------------------
class ToyConfig:
    architecture = "ToyMixedForCausalLM"

    def __init__(self, d):
        self.d = d

    def to_dict(self):
        return dict(self.d)

    def to_model_spec(self):
        rope = RopeSpec(theta=THETA, rotary_dim=D, max_positions=MAXPOS)
        att = lambda window: AttentionSpec(num_heads=HQ, num_kv_heads=HKV, head_dim=D, scale=1 / math.sqrt(D),
                                           qk_norm_eps=EPS, window=window, position=rope)
        norm, ffn = RMSNormSpec(eps=EPS), SwiGLUSpec(intermediate_size=I)
        mixers = [att(None), DecaySpec(decay=0.5), att(WINDOW)]
        layers = tuple(LayerSpec(prefix=f"model.layers.{i}", mixer_norm=norm, mixer=m, ffn_norm=norm, ffn=ffn)
                       for i, m in enumerate(mixers))
        schedule = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2), ScheduleEntry(0),
                    ScheduleEntry(0, cache_from=0), ScheduleEntry(1))
        return ModelSpec(architecture=self.architecture, vocab_size=V, hidden_size=H, layers=layers,
                         schedule=schedule, final_norm=norm, embed_name="model.embed_tokens.weight",
                         final_norm_name="model.norm.weight", head_name="lm_head.weight", tie_head=True,
                         max_positions=MAXPOS)


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    register_part("toy_decay", DecayMixer)
    register_architecture(ToyConfig.architecture, ToyConfig)
    folder = str(tmp_path_factory.mktemp("toy") / "model")
    write_model_folder(folder, ToyConfig({"architectures": [ToyConfig.architecture]}), seed=9,
                       dtype=torch.bfloat16, std=0.15, norm_std=0.05)
    yield folder
    unregister_architecture(ToyConfig.architecture)
    unregister_part("toy_decay")


# ---- its plain forward, whole sequences ------------------------------------------------------
def plain_attention(x, pos, w, pre, table, window, kv=None):
    t = x.shape[0]
    q = P.linear(x, w[f"{pre}.self_attn.q_proj.weight"].float()).view(t, HQ, D)
    q = P.apply_rope(table, pos, P.rms_norm(q, w[f"{pre}.self_attn.q_norm.weight"].float(), EPS))
    if kv is None:
        k = P.linear(x, w[f"{pre}.self_attn.k_proj.weight"].float()).view(t, HKV, D)
        k = P.apply_rope(table, pos, P.rms_norm(k, w[f"{pre}.self_attn.k_norm.weight"].float(), EPS))
        v = P.linear(x, w[f"{pre}.self_attn.v_proj.weight"].float()).view(t, HKV, D)
        kv = (k, v)
    o = P.attention(q, kv[0], kv[1], 1 / math.sqrt(D), pos, pos, window=window).reshape(t, HQ * D)
    return P.linear(o, w[f"{pre}.self_attn.o_proj.weight"].float()), kv


def plain_decay(x, w, pre):
    u = P.linear(x, w[f"{pre}.self_attn.proj.weight"].float())
    s, out = torch.zeros(H), []
    for t in range(x.shape[0]):
        s = 0.5 * s + u[t]
        out.append(s.clone())
    return torch.stack(out)


def plain_forward(w, toks):
    pos = torch.arange(len(toks))
    table = P.rope_table(THETA, D, MAXPOS)
    h = P.embedding(torch.tensor(toks), w["model.embed_tokens.weight"]).float()
    kept = {}
    for i, (layer, cache_from) in enumerate(((0, None), (1, None), (2, None), (0, None), (0, 0), (1, None))):
        pre = f"model.layers.{layer}"
        x = P.rms_norm(h, w[f"{pre}.input_layernorm.weight"].float(), EPS)
        if layer == 1:
            a = plain_decay(x, w, pre)
        else:
            a, kept[i] = plain_attention(x, pos, w, pre, table, WINDOW if layer == 2 else None,
                                         kv=kept[cache_from] if cache_from is not None else None)
        h = h + a
        x = P.rms_norm(h, w[f"{pre}.post_attention_layernorm.weight"].float(), EPS)
        h = h + P.mlp_block(x, w, pre)
    x = P.rms_norm(h, w["model.norm.weight"].float(), EPS)
    return P.linear(x, w["model.embed_tokens.weight"].float())


def test_cache_plan_of_the_toy(toy):
    from qwen_engine_amd.config import config_from_folder
    from qwen_engine_amd.parts import cache_plan
    plan = cache_plan(config_from_folder(toy).to_model_spec())
    assert [g.window for g in plan.groups] == [None, WINDOW]
    assert plan.user_group == [0, None, 1, 0, 0, None]
    assert plan.user_source == [0, None, 2, 3, 0, None]       # entry 4 reads entry 0's cache
    assert [s is not None for s in plan.user_state] == [False, True, False, False, False, True]


@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_toy_architecture_in_every_cutting(toy, tmp_path, cut):
    cfg, w = P.read_folder(toy)
    g = torch.Generator().manual_seed(21)
    reqs = {f"q{i}": torch.randint(0, V, (n,), generator=g).tolist() for i, n in enumerate((90, 64, 130, 75, 101))}
    ref = {rid: plain_forward(w, toks) for rid, toks in reqs.items()}
    trace = {"whole": traces.whole, "tail": traces.tail_decoded, "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, seed=5)}[cut](reqs)
    out_dir = str(tmp_path / "out")
    traces.run_in_process(trace, toy, "float32", out_dir, PAGE)
    got = traces.collect(trace, out_dir, V)
    bad, worst = traces.first_mismatch(got, ref, 1e-4)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"


def test_window_group_holds_few_pages(toy):
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    runner = ModelRunner(load_model(toy, dtype="float32"), page_size=PAGE, num_pages=[40, 6], max_requests=1)
    runner.add_request("r")
    toks = [(7 * i) % V for i in range(300)]
    for i in range(0, 300, 10):                              # 300 tokens through a window pool of 48
        runner.step([StepEntry("r", toks[i:i + 10], [])])
        runner.cache.check_invariants()
    held = sum(p >= 0 for p in runner.cache.block_table("r", 1))
    assert held <= (WINDOW + PAGE - 1) // PAGE + 1
    assert sum(p >= 0 for p in runner.cache.block_table("r", 0)) == 38
