"""Windowed attention layers beside a layer over all keys, at a head size that the MFMA
attention kernels take: in bfloat16 the prefill and decode kernels then read block tables whose
entries behind the window have been given back (they are -1), and the two cache groups hand out
and take back pages at different rates.  Every cutting, both element types, against the plain
implementation with the same windows."""
import math

import pytest
import torch

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.config import (AttentionSpec, LayerSpec, ModelSpec, RMSNormSpec, RopeSpec, ScheduleEntry,
                                    SwiGLUSpec, register_architecture, unregister_architecture)
from qwen_engine_amd.weights import write_model_folder
from plain import qwen3_plain as P
import traces

pytestmark = pytest.mark.gpu

H, V, HQ, HKV, D, I, PAGE = 128, 300, 8, 2, 64, 192, 16
WINDOWS = (40, None, 17)            # per layer: two pages and a half; all keys; barely more than a page
EPS, THETA, MAXPOS = 1e-6, 10000.0, 3072


class ToyWindowConfig:
    architecture = "ToyWindowForCausalLM"

    def __init__(self, d):
        self.d = d

    def to_dict(self):
        return dict(self.d)

    def to_model_spec(self):
        norm = RMSNormSpec(eps=EPS)
        rope = RopeSpec(theta=THETA, rotary_dim=D, max_positions=MAXPOS)
        layers = tuple(
            LayerSpec(prefix=f"model.layers.{i}", mixer_norm=norm, ffn_norm=norm, ffn=SwiGLUSpec(intermediate_size=I),
                      mixer=AttentionSpec(num_heads=HQ, num_kv_heads=HKV, head_dim=D, scale=1 / math.sqrt(D),
                                          qk_norm_eps=EPS, window=win, position=rope))
            for i, win in enumerate(WINDOWS))
        return ModelSpec(architecture=self.architecture, vocab_size=V, hidden_size=H, layers=layers,
                         schedule=tuple(ScheduleEntry(i) for i in range(len(WINDOWS))), final_norm=norm,
                         embed_name="model.embed_tokens.weight", final_norm_name="model.norm.weight",
                         head_name="lm_head.weight", tie_head=False, max_positions=MAXPOS)


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    register_architecture(ToyWindowConfig.architecture, ToyWindowConfig)
    folder = str(tmp_path_factory.mktemp("toy_window") / "model")
    write_model_folder(folder, ToyWindowConfig({"architectures": [ToyWindowConfig.architecture]}), seed=17,
                       dtype=torch.bfloat16, std=0.08, norm_std=0.05)
    yield folder
    unregister_architecture(ToyWindowConfig.architecture)


def plain_forward(w, toks, act=None):
    pos = torch.arange(len(toks))
    cfg = dict(num_attention_heads=HQ, num_key_value_heads=HKV, head_dim=D, rms_norm_eps=EPS)
    table = P.rope_table(THETA, D, MAXPOS)
    h = P.embedding(torch.tensor(toks), w["model.embed_tokens.weight"]).float()
    for i, win in enumerate(WINDOWS):
        h = P.decoder_layer(h, pos, w, f"model.layers.{i}", cfg, table, act_dtype=act, window=win)
    x = P.rms_norm(h, w["model.norm.weight"].float(), EPS)
    if act is not None:
        x = x.to(act).float()
    return P.linear(x, w["lm_head.weight"].float())


def test_the_window_matters(toy):
    """Logits beyond the window differ from those without it, so a window that is not applied shows."""
    _, w = P.read_folder(toy)
    toks = torch.randint(0, V, (80,), generator=torch.Generator().manual_seed(2)).tolist()
    with_window = plain_forward(w, toks)
    cfg = dict(num_attention_heads=HQ, num_key_value_heads=HKV, head_dim=D, rms_norm_eps=EPS)
    pos, table = torch.arange(80), P.rope_table(THETA, D, MAXPOS)
    h = P.embedding(torch.tensor(toks), w["model.embed_tokens.weight"]).float()
    for i in range(len(WINDOWS)):
        h = P.decoder_layer(h, pos, w, f"model.layers.{i}", cfg, table)
    without = P.linear(P.rms_norm(h, w["model.norm.weight"].float(), EPS), w["lm_head.weight"].float())
    assert float((with_window[:17] - without[:17]).abs().max()) < 1e-5          # inside the shortest window: the same
    assert float((with_window[60:] - without[60:]).abs().max()) > 0.05 * float(without.abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_window_layers_in_every_cutting(toy, tmp_path, dtype, cut):
    from qwen_engine_amd.config import config_from_folder
    from qwen_engine_amd.parts import cache_plan
    plan = cache_plan(config_from_folder(toy).to_model_spec())
    assert sorted(str(g.window) for g in plan.groups) == ["17", "40", "None"]
    _, w = P.read_folder(toy)
    g = torch.Generator().manual_seed(41)
    reqs = {f"q{i}": torch.randint(0, V, (n,), generator=g).tolist() for i, n in enumerate((300, 70, 145, 257, 64, 33))}
    act = None if dtype == "float32" else torch.bfloat16
    ref = {rid: plain_forward(w, toks, act) for rid, toks in reqs.items()}
    trace = {"whole": traces.whole, "tail": traces.tail_decoded, "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, seed=9)}[cut](reqs)
    out_dir = str(tmp_path / "out")
    traces.run_in_process(trace, toy, dtype, out_dir, PAGE)
    got = traces.collect(trace, out_dir, V)
    bad, worst = traces.first_mismatch(got, ref, 1e-4 if dtype == "float32" else 2e-2)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"


@pytest.mark.parametrize("use_graphs", [True, False])
def test_windows_far_into_a_context(toy, use_graphs):
    """One request of 2600 tokens in portions of 1500, 512, 2, 256 and 330, then four decoded tokens:
    beyond 1024 keys the prefill kernel cuts the keys of a portion into segments (all of them matter
    in the layer over all keys; in the windowed layers a block's keys lie in one or two segments, and
    the pages behind the window have been given back), and round portions are replayed from recorded
    graphs.  The last row of every step against the plain implementation, pages poisoned."""
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    model = load_model(toy, dtype="bfloat16")
    _, w = P.read_folder(toy)
    sizes = [1500, 512, 2, 256, 330, 1, 1, 1, 1]
    L = sum(sizes)
    toks = torch.randint(0, V, (L,), generator=torch.Generator().manual_seed(43)).tolist()
    ref = plain_forward(w, toks, torch.bfloat16)
    runner = ModelRunner(model, page_size=PAGE, num_pages=L // PAGE + 8, max_requests=1, use_graphs=use_graphs,
                         debug_poison=True)
    runner.add_request("r")
    a = 0
    for n in sizes:
        got = runner.step([StepEntry("r", toks[a:a + n], [n - 1])])[0].float().cpu()
        a += n
        assert torch.isfinite(got).all(), f"the step that ends at {a}"
        err = float((got - ref[a - 1]).abs().max()) / float(ref.abs().max())
        assert err <= 2e-2, f"the step that ends at {a}: error {err}"
    if use_graphs:
        # the portions of 512 and 256 tokens; the decoded tokens; the other portions, filled up to round lengths
        assert runner.graph_steps_of == {"portion": 2, "decode": 4, "mixed": 3}
    # the windowed groups hold what their windows need, not the whole context
    held = sorted(sum(1 for p in t if p >= 0) for t in runner.cache.get("r").tables)
    assert held[-1] == math.ceil(L / PAGE) and held[0] <= 3 and held[1] <= 4
    runner.cache.check_invariants()
