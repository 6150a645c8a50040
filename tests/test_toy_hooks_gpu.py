"""What another architecture may need around and inside the layers, shown with toy parts that are
defined here and never become a model: a part that changes the stream right after the embedding (a
scale and an added table of positions), a part that changes the logits (a soft cap), a layer whose
parts have other checkpoint names, and a mixer with per-request state that says it can be recorded
into a graph and asks the step function, through step_extras / graph_key / graph_extras, for what it
wants prepared.  Registered, built from a model folder and replayed in every cutting without a
change to the framework's files."""
import math
from dataclasses import dataclass

import numpy as np
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

H, V, HQ, HKV, D, I, PAGE = 64, 113, 4, 2, 16, 96, 8
EPS, THETA, MAXPOS = 1e-6, 10000.0, 300
EMBED_SCALE, CAP, DECAY = 3.0, 2.5, 0.6


@dataclass(frozen=True)
class AddedPositionsSpec:
    scale: float
    max_positions: int
    prefix: str = "model.pos_embed"
    kind: str = "toy_added_positions"


class AddedPositions:
    """h = h * scale + table[position]: a stream prologue."""

    def __init__(self, spec, hidden):
        self.scale = spec.scale

    @staticmethod
    def expected_tensors(spec, hidden):
        return {"weight": TensorInfo((spec.max_positions, hidden))}

    def load(self, tensors, rt):
        self.table = tensors["weight"].float().to(rt.device)

    def forward(self, h, ctx):
        h.mul_(self.scale).add_(self.table.index_select(0, ctx.positions.long()))


@dataclass(frozen=True)
class SoftCapSpec:
    cap: float
    kind: str = "toy_soft_cap"


class SoftCap:
    """logits = cap * tanh(logits / cap): a logit epilogue."""

    def __init__(self, spec, hidden):
        self.cap = spec.cap

    @staticmethod
    def expected_tensors(spec, hidden):
        return {}

    def load(self, tensors, rt):
        pass

    def forward(self, logits, ctx):
        return torch.tanh(logits / self.cap) * self.cap


@dataclass(frozen=True)
class RunningSpec:
    decay: float
    kind: str = "toy_running"


class RunningMixer:
    """s_t = decay s_{t-1} + W x_t, y_t = s_t, the state s kept in the request's slot.  A step of
    single new tokens works on device tensors only (it can be recorded and replayed); a step with
    prompt portions walks the requests on the host."""
    graph_safe = True
    calls = {"step_extras": 0, "graph_extras": 0, "graph_key": 0}

    def __init__(self, spec, hidden):
        self.decay = spec.decay

    @staticmethod
    def expected_tensors(spec, hidden):
        return {"proj.weight": TensorInfo((hidden, hidden))}

    @staticmethod
    def cache_need(spec):
        return None

    @staticmethod
    def state_need(spec, hidden):
        return StateNeed(shape=(hidden,), dtype="float32")

    # ---- what the step function prepares for this part -------------------------------------
    @staticmethod
    def step_extras(seqs):
        RunningMixer.calls["step_extras"] += 1
        return {"single": all(s.q_len == 1 for s in seqs),
                "rows_of_requests": np.asarray([s.q_start for s in seqs], dtype=np.int32)}

    @staticmethod
    def graph_key(max_position):
        RunningMixer.calls["graph_key"] += 1
        return "any"                                     # nothing of its launches depends on the positions

    @staticmethod
    def graph_extras(rows, key, device):
        RunningMixer.calls["graph_extras"] += 1
        assert key == "any"
        return {"single": True, "rows_of_requests": torch.arange(rows, dtype=torch.int32, device=device)}

    def load(self, tensors, rt):
        self.w = tensors["proj.weight"].float().to(rt.device)

    def forward(self, x, ctx, binding):
        ex = ctx.extras[RunningMixer]
        u = x.float() @ self.w.t()
        if ex["single"]:
            assert ex["rows_of_requests"].shape[0] == x.shape[0]
            slots = ctx.state_slots.long()
            s = binding.state.index_select(0, slots) * self.decay + u.index_select(0, ex["rows_of_requests"].long())
            binding.state.index_copy_(0, slots, s)
            return s.to(x.dtype)
        y = torch.empty_like(x)
        for s in ctx.seqs:
            state = binding.state[s.state_slot]
            for t in range(s.q_start, s.q_start + s.q_len):
                state.mul_(self.decay).add_(u[t])
                y[t] = state.to(x.dtype)
        return y


class ToyHooksConfig:
    architecture = "ToyHooksForCausalLM"

    def __init__(self, d):
        self.d = d

    def to_dict(self):
        return dict(self.d)

    def to_model_spec(self):
        norm, ffn = RMSNormSpec(eps=EPS), SwiGLUSpec(intermediate_size=I)
        att = AttentionSpec(num_heads=HQ, num_kv_heads=HKV, head_dim=D, scale=1 / math.sqrt(D), qk_norm_eps=EPS,
                            position=RopeSpec(theta=THETA, rotary_dim=D, max_positions=MAXPOS))
        layers = (LayerSpec(prefix="h.0", mixer_norm=norm, mixer=att, ffn_norm=norm, ffn=ffn,
                            part_names=("ln_1", "attn", "ln_2", "ff")),
                  LayerSpec(prefix="h.1", mixer_norm=norm, mixer=RunningSpec(decay=DECAY), ffn_norm=norm, ffn=ffn,
                            part_names=("ln_1", "running", "ln_2", "ff")))
        return ModelSpec(architecture=self.architecture, vocab_size=V, hidden_size=H, layers=layers,
                         schedule=(ScheduleEntry(0), ScheduleEntry(1)), final_norm=norm, embed_name="wte.weight",
                         final_norm_name="ln_f.weight", head_name="head.weight", tie_head=True, max_positions=MAXPOS,
                         stream_prologue=AddedPositionsSpec(scale=EMBED_SCALE, max_positions=MAXPOS),
                         logit_epilogue=SoftCapSpec(cap=CAP))


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    register_part("toy_added_positions", AddedPositions)
    register_part("toy_soft_cap", SoftCap)
    register_part("toy_running", RunningMixer)
    register_architecture(ToyHooksConfig.architecture, ToyHooksConfig)
    folder = str(tmp_path_factory.mktemp("toy_hooks") / "model")
    write_model_folder(folder, ToyHooksConfig({"architectures": [ToyHooksConfig.architecture]}), seed=21,
                       dtype=torch.bfloat16, std=0.12, norm_std=0.05)
    yield folder
    unregister_architecture(ToyHooksConfig.architecture)
    for kind in ("toy_added_positions", "toy_soft_cap", "toy_running"):
        unregister_part(kind)


def plain_forward(w, toks, act=None):
    rnd = (lambda t: t) if act is None else (lambda t: t.to(act).float())
    f = lambda name: w[name].float()
    t = len(toks)
    pos = torch.arange(t)
    h = P.embedding(torch.tensor(toks), w["wte.weight"]).float() * EMBED_SCALE + f("model.pos_embed.weight")[:t]
    # layer 0: attention with the rotary encoding
    x = rnd(P.rms_norm(h, f("h.0.ln_1.weight"), EPS))
    q = rnd(P.linear(x, f("h.0.attn.q_proj.weight"))).view(t, HQ, D)
    k = rnd(P.linear(x, f("h.0.attn.k_proj.weight"))).view(t, HKV, D)
    v = rnd(P.linear(x, f("h.0.attn.v_proj.weight"))).view(t, HKV, D)
    table = P.rope_table(THETA, D, MAXPOS)
    q = rnd(P.apply_rope(table, pos, P.rms_norm(q, f("h.0.attn.q_norm.weight"), EPS)))
    k = rnd(P.apply_rope(table, pos, P.rms_norm(k, f("h.0.attn.k_norm.weight"), EPS)))
    o = rnd(P.attention(q, k, v, 1 / math.sqrt(D), pos, pos)).reshape(t, HQ * D)
    h = h + rnd(P.linear(o, f("h.0.attn.o_proj.weight")))
    for layer in (0, 1):
        if layer == 1:
            x = rnd(P.rms_norm(h, f("h.1.ln_1.weight"), EPS))
            u = x @ f("h.1.running.proj.weight").t()
            s, ys = torch.zeros(H), []
            for i in range(t):
                s = s * DECAY + u[i]
                ys.append(s)
            h = h + rnd(torch.stack(ys))
        x = rnd(P.rms_norm(h, f(f"h.{layer}.ln_2.weight"), EPS))
        g = rnd(P.linear(x, f(f"h.{layer}.ff.gate_proj.weight")))
        up = rnd(P.linear(x, f(f"h.{layer}.ff.up_proj.weight")))
        h = h + rnd(P.linear(rnd(P.silu_mul(g, up)), f(f"h.{layer}.ff.down_proj.weight")))
    x = rnd(P.rms_norm(h, f("ln_f.weight"), EPS))
    logits = P.linear(x, f("wte.weight"))
    return torch.tanh(logits / CAP) * CAP


def test_the_hooks_change_the_result(toy):
    """Without the prologue or without the cap the plain logits are others: a hook that is not called shows."""
    _, w = P.read_folder(toy)
    assert set(w) >= {"model.pos_embed.weight", "h.0.attn.q_proj.weight", "h.1.running.proj.weight", "h.0.ff.down_proj.weight"}
    toks = torch.randint(0, V, (40,), generator=torch.Generator().manual_seed(3)).tolist()
    ref = plain_forward(w, toks)
    assert float(ref.abs().max()) <= CAP and float(ref.abs().max()) > 0.8 * CAP      # the cap bites
    w2 = dict(w)
    w2["model.pos_embed.weight"] = torch.zeros_like(w["model.pos_embed.weight"])
    assert float((plain_forward(w2, toks) - ref).abs().max()) > 0.1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_toy_hooks_in_every_cutting(toy, tmp_path, dtype, cut):
    _, w = P.read_folder(toy)
    g = torch.Generator().manual_seed(34)
    reqs = {f"q{i}": torch.randint(0, V, (n,), generator=g).tolist() for i, n in enumerate((70, 45, 110, 64, 33))}
    act = None if dtype == "float32" else torch.bfloat16
    ref = {rid: plain_forward(w, toks, act) for rid, toks in reqs.items()}
    trace = {"whole": traces.whole, "tail": traces.tail_decoded, "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, seed=8)}[cut](reqs)
    out_dir = str(tmp_path / "out")
    traces.run_in_process(trace, toy, dtype, out_dir, PAGE)
    got = traces.collect(trace, out_dir, V)
    bad, worst = traces.first_mismatch(got, ref, 1e-4 if dtype == "float32" else 2e-2)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"


def test_a_mixer_with_state_is_recorded_when_it_says_it_can_be(toy):
    """Three requests decode through recorded graphs (five live rows would replay the graph of five):
    the state slots are read and written inside the graph, a request that starts with a single
    token has its state cleared, and the logits equal a runner's that records nothing."""
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    model = load_model(toy, dtype="bfloat16")
    _, w = P.read_folder(toy)
    g = torch.Generator().manual_seed(35)
    reqs = [torch.randint(0, V, (n,), generator=g).tolist() for n in (30, 12, 1)]
    before = dict(RunningMixer.calls)
    outs = []
    for use_graphs in (None, False):
        runner = ModelRunner(model, page_size=PAGE, num_pages=40, max_requests=3, use_graphs=use_graphs)
        assert runner.use_graphs == (use_graphs is None)
        for st in runner.state:                        # leftovers of an earlier owner of the slots
            if st is not None:
                st.fill_(7.0)
        for i, toks in enumerate(reqs):
            runner.add_request(i)
            if len(toks) > 1:
                runner.step([StepEntry(i, toks[:-1], [])])
        seqs = [list(t) for t in reqs]
        got = []
        for step in range(6):
            got.append(runner.step([StepEntry(i, [s[-1]], [0]) for i, s in enumerate(seqs)]).float().cpu())
            for i, s in enumerate(seqs):
                s.append((5 * i + 11 * step) % V)
        outs.append((got, seqs, runner.graph_steps))
    assert outs[0][2] == 6 and outs[1][2] == 0
    assert RunningMixer.calls["graph_extras"] > before["graph_extras"] and RunningMixer.calls["graph_key"] > before["graph_key"]
    for a, b in zip(outs[0][0], outs[1][0]):
        assert float((a - b).abs().max()) <= 1e-3 * float(b.abs().max())
    for i, s in enumerate(outs[0][1]):
        ref = plain_forward(w, s[:-1], torch.bfloat16)
        n = len(reqs[i])
        for step in range(6):
            err = float((outs[0][0][step][i] - ref[n - 1 + step]).abs().max()) / float(ref.abs().max())
            assert err <= 2e-2, f"request {i}, step {step}: error {err}"
