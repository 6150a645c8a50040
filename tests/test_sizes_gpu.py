"""Configurations with awkward sizes through the engine, in float32 and in bfloat16, against the
plain implementation: head sizes 8 to 256 in steps that are no power of two, 1 to 16 query heads
per key/value head, widths and vocabularies that are no multiple of anything, with and without
the attention bias (which switches the q/k norm off), tied and untied heads, several page sizes.
Each request goes in two portions, then 30 tokens one by one; a second request goes whole.
Whichever kernel takes a size (MFMA or the general one), the logits have to be right."""
import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import qwen3_plain as P
from qwen_engine_amd.config import Qwen3Config
from qwen_engine_amd.engine import ModelRunner, StepEntry
from qwen_engine_amd.parts import DecoderModel, Runtime
from qwen_engine_amd.weights import random_tensors

pytestmark = pytest.mark.gpu

# hidden, intermediate, query heads, key/value heads, head size, vocabulary, page size, attention bias
CASES = [
    (72, 100, 5, 5, 16, 257, 16, False), (136, 200, 7, 1, 112, 301, 16, False), (64, 96, 2, 1, 256, 99, 32, False),
    (50, 70, 3, 3, 32, 131, 8, False), (128, 256, 16, 1, 64, 1000, 16, False), (96, 64, 12, 4, 80, 333, 16, True),
    (200, 328, 10, 2, 96, 500, 64, False), (64, 64, 1, 1, 64, 64, 16, True), (264, 520, 24, 8, 128, 777, 16, False),
    (40, 24, 5, 1, 8, 50, 4, False),
]
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}      # of the largest reference logit


@pytest.mark.parametrize("case", range(len(CASES)))
def test_awkward_sizes(case):
    H, I, hq, hkv, d, V, page, bias = CASES[case]
    cfg_dict = dict(architectures=["Qwen3ForCausalLM"], vocab_size=V, hidden_size=H, intermediate_size=I,
                    num_hidden_layers=2, num_attention_heads=hq, num_key_value_heads=hkv, head_dim=d,
                    max_position_embeddings=512, rms_norm_eps=1e-6, rope_theta=10000.0,
                    tie_word_embeddings=bool(case % 2), attention_bias=bias)
    cfg = Qwen3Config.from_dict(cfg_dict)
    w = random_tensors(cfg, 10 + case, dtype=torch.bfloat16, std=0.05)
    toks = torch.randint(0, V, (200,), generator=torch.Generator().manual_seed(case)).tolist()
    plain_w = {k: v.float() for k, v in w.items()}
    dev = torch.device("cuda:0")
    for dt, act in ((torch.float32, None), (torch.bfloat16, torch.bfloat16)):
        ref = P.forward_logits(cfg_dict, plain_w, toks, act_dtype=act)
        model = DecoderModel(cfg.to_model_spec())
        model.load(w, Runtime(dev, dt))
        runner = ModelRunner(model, page_size=page, num_pages=(220 // page + 2) * 2, max_requests=2)
        runner.add_request("a")
        runner.add_request("b")
        out = [runner.step([StepEntry("a", toks[:97], list(range(97)))]).float().cpu(),
               runner.step([StepEntry("a", toks[97:170], list(range(73)))]).float().cpu()]
        for i in range(170, 200):
            out.append(runner.step([StepEntry("a", [toks[i]], [0])]).float().cpu())
        got_a = torch.cat(out)
        got_b = runner.step([StepEntry("b", toks[:130], list(range(130)))]).float().cpu()
        scale = float(ref.abs().max())
        err_a = (got_a - ref).abs().amax(dim=1) / scale
        err_b = (got_b - ref[:130]).abs().amax(dim=1) / scale
        assert float(err_a.max()) <= TOL[dt], f"{dt}: first wrong position {int((err_a > TOL[dt]).nonzero()[0])}"
        assert float(err_b.max()) <= TOL[dt], f"{dt}: whole request, first wrong position {int((err_b > TOL[dt]).nonzero()[0])}"
        del runner, model
