from __future__ import annotations

import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from kvcore_amd.engine.runner import build_model
from kvcore_amd.weights.loader import WeightError, checkpoint_layout, write_random_model
from kvcore_amd.weights.safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors
from tests.helpers import TINY_A, TINY_B, TINY_C, make_model_dir


def test_own_writer_and_reader_agree_with_the_library(tmp_path):
    tensors = {
        "a.weight": torch.randn(5, 7).to(torch.bfloat16),
        "b": torch.arange(12, dtype=torch.int32).reshape(3, 4),
        "c.gain": torch.randn(9),
        "empty": torch.zeros(0, 4),
    }
    write_safetensors(tmp_path / "mine.safetensors", tensors)
    theirs = load_file(str(tmp_path / "mine.safetensors"))
    assert set(theirs) == set(tensors)
    for k in tensors:
        assert theirs[k].dtype == tensors[k].dtype and torch.equal(theirs[k], tensors[k])
    save_file(tensors, str(tmp_path / "theirs.safetensors"))
    with SafetensorsFile(tmp_path / "theirs.safetensors") as f:
        assert set(f.entries) == set(tensors)
        for k in tensors:
            assert torch.equal(f.tensor(k).clone(), tensors[k])


def test_reader_refuses_a_broken_file(tmp_path):
    (tmp_path / "x.safetensors").write_bytes(b"\x10\x00\x00\x00\x00\x00\x00\x00{}")
    with pytest.raises(SafetensorsError):
        SafetensorsFile(tmp_path / "x.safetensors")


def test_random_weights_mode_is_a_function_of_seed_and_name(tmp_path):
    a = load_file(str(write_random_model(tmp_path / "a", TINY_A, seed=5) / "model.safetensors"))
    b = load_file(str(write_random_model(tmp_path / "b", TINY_A, seed=5) / "model.safetensors"))
    c = load_file(str(write_random_model(tmp_path / "c", TINY_A, seed=6) / "model.safetensors"))
    assert set(a) == set(checkpoint_layout_names(TINY_A))
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["lm_head.weight"], c["lm_head.weight"])
    assert a["model.layers.0.self_attn.q_proj.weight"].dtype == torch.bfloat16
    gain = a["model.norm.weight"]
    assert gain.dtype == torch.float32 and abs(float(gain.mean()) - 1.0) < 0.1  # 1 + N(0, 0.1)
    w = a["model.layers.1.mlp.down_proj.weight"].float()
    assert abs(float(w.std()) - 0.02) < 0.003  # N(0, 0.02)
    assert json.loads((tmp_path / "a" / "config.json").read_text())["vocab_size"] == 256
    assert "lm_head.weight" not in load_file(
        str(write_random_model(tmp_path / "t", TINY_B, seed=1) / "model.safetensors"))  # tied


def test_random_values_depend_on_seed_name_and_index_only():
    """Not on how the draw is cut into chunks, not on the tensor's shape or on what it is
    stacked with; the kernel's tables are the ones worked out here."""
    import math
    import re
    from pathlib import Path

    import numpy as np

    from kvcore_amd.weights import random_normal
    from kvcore_amd.weights.loader import random_tensor

    whole = random_normal.normal(11, 22, 100_000, 0.0, 0.02)
    for chunk in (1, 7, 4096, 1 << 20):
        n = 1000 if chunk < 100 else 100_000
        assert np.array_equal(random_normal.normal(11, 22, n, 0.0, 0.02, chunk=chunk), whole[:n])
    assert np.array_equal(random_normal.standard_normal(11, 22, 500, 100) * np.float32(0.02), whole[500:600])
    a = random_tensor(3, "model.layers.0.self_attn.k_proj.weight", (8, 16), "normal")
    b = random_tensor(3, "model.layers.0.self_attn.k_proj.weight", (4, 32), "normal")
    assert torch.equal(a.flatten(), b.flatten())
    assert not torch.equal(a, random_tensor(3, "model.layers.0.self_attn.v_proj.weight", (8, 16), "normal"))
    assert not torch.equal(a, random_tensor(4, "model.layers.0.self_attn.k_proj.weight", (8, 16), "normal"))
    gain = random_tensor(3, "model.norm.weight", (4096,), "gain")
    assert abs(float(gain.mean()) - 1.0) < 0.01 and abs(float(gain.std()) - 0.1) < 0.01
    assert (random_tensor(3, "x.bias", (5,), "zeros") == 0).all()
    # the distribution: mean, deviation, tails and a Kolmogorov-Smirnov distance
    z = np.sort(random_normal.standard_normal(5, 6, 0, 400_000).astype(np.float64))
    assert abs(z.mean()) < 5e-3 and abs(z.std() - 1.0) < 5e-3
    cdf = 0.5 * (1.0 + np.vectorize(math.erf)(z[::40] / math.sqrt(2.0)))
    assert np.abs(cdf - (np.arange(0, 400_000, 40) + 0.5) / 400_000).max() < 4e-3
    assert abs((np.abs(z) > 3).mean() - 0.0027) < 5e-4
    # the kernel's source holds the same two tables, bit for bit
    src = (Path(random_normal.__file__).resolve().parents[1] / "csrc" / "random_fill.hip").read_text()
    for name, table in (("kInvC", random_normal.INV_C), ("kLnC", random_normal.LN_C)):
        body = src[src.index(name + "[32]"):]
        body = body[:body.index("};")]
        assert [int(h, 16) for h in re.findall(r"0x([0-9A-F]{8})u", body)] == table.view(np.uint32).tolist()


def checkpoint_layout_names(config):
    from kvcore_amd.registry import resolve_architecture

    arch = resolve_architecture(config)
    return list(checkpoint_layout(arch.build_spec(arch.parse_config(config))))


def test_stacked_rows_are_q_k_v_and_gate_up(tmp_path):
    """tests/test_model_loading.py:217-241 fills q/k/v/gate/up with the constants 1..5."""
    folder = write_random_model(tmp_path / "m", TINY_A, seed=0, dtype=torch.float32)
    tensors = load_file(str(folder / "model.safetensors"))
    p = "model.layers.0"
    for value, name in enumerate(["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj",
                                  "mlp.gate_proj", "mlp.up_proj"], start=1):
        tensors[f"{p}.{name}.weight"].fill_(float(value))
    save_file(tensors, str(folder / "model.safetensors"))
    model = build_model(folder, torch.float32, "cpu")
    qkv = model.params[f"{p}.self_attn.qkv_proj.weight"].tensor
    assert torch.all(qkv[:64] == 1) and torch.all(qkv[64:96] == 2) and torch.all(qkv[96:128] == 3)
    gu = model.params[f"{p}.mlp.gate_up_proj.weight"].tensor
    assert torch.all(gu[:128] == 4) and torch.all(gu[128:] == 5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_round_trip_keeps_bits_and_dtypes(tmp_path, dtype):
    folder = make_model_dir(tmp_path / "c", TINY_C, seed=2)
    stored = load_file(str(folder / "model.safetensors"))
    model = build_model(folder, dtype, "cpu")
    for name, (bp, row, rows) in model.checkpoint_map().items():
        got = bp.tensor.narrow(0, row, rows)
        if bp.spec.kind == "vector":
            assert got.dtype == torch.float32  # a gain stored in 32-bit stays so
            assert torch.equal(got, stored[name].float())
        else:
            assert got.dtype == dtype
            assert torch.equal(got, stored[name].to(dtype))  # bfloat16 -> float32 is exact


def test_tied_head_shares_storage_and_ignores_a_stored_head(tmp_path):
    folder = make_model_dir(tmp_path / "b", TINY_B, seed=3)
    tensors = load_file(str(folder / "model.safetensors"))
    tensors["lm_head.weight"] = torch.zeros(384, 96, dtype=torch.bfloat16)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    save_file(tensors, str(folder / "model.safetensors"))
    model = build_model(folder, torch.float32, "cpu")
    assert model.head.params["weight"].data_ptr() == model.embed.params["weight"].data_ptr()
    assert float(model.head.params["weight"].abs().sum()) > 0


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = make_model_dir(tmp_path / "a", TINY_A, seed=4)
    tensors = load_file(str(folder / "model.safetensors"))
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64, dtype=torch.bfloat16)
    tensors["model.layers.0.extra.weight"] = torch.zeros(2)
    save_file(tensors, str(folder / "model.safetensors"))
    with pytest.raises(WeightError) as info:
        build_model(folder, torch.float32, "cpu")
    err = info.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.extra.weight"]
    assert err.mismatched == [("model.layers.0.self_attn.k_proj.weight", (32, 64), (16, 64))]
    text = str(err)
    for needle in ("missing tensors (2)", "model.norm.weight", "unexpected tensors (1)",
                   "model.layers.0.extra.weight", "wrong shapes (1)", "expected [32, 64] got [16, 64]"):
        assert needle in text
    # not strict: unexpected tensors pass, the rest still raises
    with pytest.raises(WeightError) as info:
        build_model(folder, torch.float32, "cpu", strict=False)
    assert info.value.unexpected == []


def test_sharded_folder_with_index_equals_single_file(tmp_path):
    """tests/test_model_loading.py:163-197."""
    single = make_model_dir(tmp_path / "one", TINY_A, seed=7)
    tensors = load_file(str(single / "model.safetensors"))
    names = sorted(tensors)
    sharded = tmp_path / "two"
    sharded.mkdir()
    (sharded / "config.json").write_text((single / "config.json").read_text())
    half = len(names) // 2
    weight_map = {}
    for i, part in enumerate([names[:half], names[half:]]):
        fname = f"model-{i + 1:05d}-of-00002.safetensors"
        save_file({n: tensors[n] for n in part}, str(sharded / fname))
        weight_map.update({n: fname for n in part})
    (sharded / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    save_file({"junk": torch.zeros(1)}, str(sharded / "not_in_index.safetensors"))
    a = build_model(single, torch.float32, "cpu")
    b = build_model(sharded, torch.float32, "cpu")
    for name in a.params:
        assert torch.equal(a.params[name].tensor, b.params[name].tensor)


def test_no_weight_files(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    with pytest.raises(RuntimeError, match="Cannot find any model weights"):
        build_model(tmp_path, torch.float32, "cpu")
