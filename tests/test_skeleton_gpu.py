"""The engine against the closed forms of tests/skeleton.py, in float32: the same model folders that
the CPU tests hold the plain implementation against (where the residual is taken, where the norms
stand, the final norm, the one eps of every norm, the scores' divisor)."""
import pytest
import torch

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
import skeleton

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("cut", ["whole", "token by token"])
@pytest.mark.parametrize("name", sorted(skeleton.CASES))
def test_engine_gives_the_closed_forms(tmp_path, name, cut):
    cfg, w, ids, want, mistakes = skeleton.build(name, tmp_path)
    folder = skeleton.write_folder(str(tmp_path / "folder"), cfg, w)
    model = load_model(folder, dtype="float32", device="cuda:0")
    runner = ModelRunner(model, page_size=4, num_pages=8, max_requests=1, debug_poison=True)
    runner.add_request("r")
    if cut == "whole":
        got = runner.step([StepEntry("r", ids, list(range(len(ids))))])
    else:
        got = torch.cat([runner.step([StepEntry("r", [t], [0])]) for t in ids])
    got = got.cpu()
    assert got.shape == want.shape
    assert skeleton.relative_error(got, want) < 1e-4
    for what, other in mistakes.items():
        assert skeleton.relative_error(got, other) > 1e-2, what
