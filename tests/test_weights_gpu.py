"""The random-weights mode in memory against the folder it writes: one seed, one model."""

from __future__ import annotations

import pytest
import torch

from tests.helpers import TINY_B, TINY_C

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
@pytest.mark.parametrize("config", [TINY_B, TINY_C], ids=["B", "C"])
def test_random_load_format_gives_the_model_of_the_written_folder(tmp_path, config, dtype):
    """``load_format="random"`` draws on the GPU, ``write_random_model`` on the host (or on the
    GPU when asked): the parameters are the same bits, stacked matrices included."""
    from kvcore_amd.engine.runner import build_model
    from kvcore_amd.weights.loader import write_random_model

    (tmp_path / "cfg").mkdir()
    import json
    (tmp_path / "cfg" / "config.json").write_text(json.dumps(config))
    in_memory = build_model(tmp_path / "cfg", dtype, "cuda:0", load_format="random", seed=31)
    for where in ("cpu", "cuda:0"):
        folder = write_random_model(tmp_path / f"written_{where[:3]}", config, seed=31, dtype=dtype, device=where)
        from_file = build_model(folder, dtype, "cuda:0")
        assert set(from_file.params) == set(in_memory.params)
        for name, bp in from_file.params.items():
            assert torch.equal(bp.tensor, in_memory.params[name].tensor), (where, name)
    other = build_model(tmp_path / "cfg", dtype, "cuda:0", load_format="random", seed=32)
    name = "model.layers.0.self_attn.qkv_proj.weight"
    assert not torch.equal(other.params[name].tensor, in_memory.params[name].tensor)
    w = in_memory.params[name].tensor.float()
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
