"""One layer at the widths of the larger models of the family (8B: 32 query heads on 8
key/value heads, width 4096; 32B: 64 on 8, width 5120, feed-forward 25600) against the plain
implementation: a prompt portion of 150 tokens, then 30 tokens one by one, in float32 and in
bfloat16; and 40 requests decoding together (17 to 64 rows go through products cut along K).  The tiny configurations do not reach these shapes of the kernels: 8 query heads per
key/value head, widths that are no multiple of the tile sizes, long dot products.  The
vocabulary is cut to 1000 to keep the test short."""
import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import qwen3_plain as P
from qwen_engine_amd.config import Qwen3Config
from qwen_engine_amd.engine import ModelRunner, StepEntry
from qwen_engine_amd.parts import DecoderModel, Runtime
from qwen_engine_amd.weights import random_tensors

pytestmark = pytest.mark.gpu

WIDTHS = {
    "8B": dict(hidden_size=4096, intermediate_size=12288, num_attention_heads=32, num_key_value_heads=8, head_dim=128),
    "32B": dict(hidden_size=5120, intermediate_size=25600, num_attention_heads=64, num_key_value_heads=8, head_dim=128),
}
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}      # of the largest reference logit


@pytest.mark.parametrize("which", ["8B", "32B"])
def test_one_layer_at_the_widths_of_the_large_models(which):
    cfg_dict = dict(architectures=["Qwen3ForCausalLM"], vocab_size=1000, num_hidden_layers=1,
                    max_position_embeddings=2048, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False,
                    **WIDTHS[which])
    cfg = Qwen3Config.from_dict(cfg_dict)
    w = random_tensors(cfg, 5, dtype=torch.bfloat16)
    toks = torch.randint(0, 1000, (180,), generator=torch.Generator().manual_seed(3)).tolist()
    plain_w = {k: v.float() for k, v in w.items()}
    dev = torch.device("cuda:0")
    for dt, act in ((torch.float32, None), (torch.bfloat16, torch.bfloat16)):
        ref = P.forward_logits(cfg_dict, plain_w, toks, act_dtype=act)
        model = DecoderModel(cfg.to_model_spec())
        model.load(w, Runtime(dev, dt))
        runner = ModelRunner(model, page_size=16, num_pages=16, max_requests=1)
        runner.add_request("a")
        out = [runner.step([StepEntry("a", toks[:150], list(range(150)))]).float().cpu()]
        for i in range(150, 180):
            out.append(runner.step([StepEntry("a", [toks[i]], [0])]).float().cpu())
        got = torch.cat(out)
        scale = float(ref.abs().max())
        err = (got - ref).abs().amax(dim=1) / scale
        assert float(err.max()) <= TOL[dt], f"{which} {dt}: first wrong position {int((err > TOL[dt]).nonzero()[0])}"
        del runner, model
        torch.cuda.empty_cache()


def test_forty_requests_decode_together_at_the_8b_widths():
    """40 rows against matrices of 16 M elements and more: the q|k|v, o and down products are cut
    along K into partial products (the kernel that norms, rotates and writes the cache adds the
    q|k|v parts), gate|up goes through the tiled kernel.  Requests of different lengths, two
    decode steps, against the plain implementation."""
    cfg_dict = dict(architectures=["Qwen3ForCausalLM"], vocab_size=1000, num_hidden_layers=1,
                    max_position_embeddings=2048, rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False,
                    **WIDTHS["8B"])
    cfg = Qwen3Config.from_dict(cfg_dict)
    w = random_tensors(cfg, 6, dtype=torch.bfloat16)
    plain_w = {k: v.float() for k, v in w.items()}
    g = torch.Generator().manual_seed(4)
    reqs = [torch.randint(0, 1000, (3 + (7 * i) % 40,), generator=g).tolist() for i in range(40)]
    model = DecoderModel(cfg.to_model_spec())
    model.load(w, Runtime(torch.device("cuda:0"), torch.bfloat16))
    from qwen_engine_amd.kernels import ops
    x = torch.zeros(40, 4096, dtype=torch.bfloat16, device="cuda:0")
    assert ops.gemm_partial_preferred(x, model.blocks[0].mixer.w_qkv)          # the path this test is for
    runner = ModelRunner(model, page_size=16, num_pages=40 * 4, max_requests=40)
    for i, toks in enumerate(reqs):
        runner.add_request(i)
        runner.step([StepEntry(i, toks[:-2], [])])
    outs = [runner.step([StepEntry(i, [toks[len(toks) - 2 + s]], [0]) for i, toks in enumerate(reqs)]).float().cpu()
            for s in range(2)]
    for i, toks in enumerate(reqs):
        ref = P.forward_logits(cfg_dict, plain_w, toks, act_dtype=torch.bfloat16)
        for s in range(2):
            err = float((outs[s][i] - ref[len(toks) - 2 + s]).abs().max()) / float(ref.abs().max())
            assert err <= TOL[torch.bfloat16], f"request {i}, step {s}: error {err}"
