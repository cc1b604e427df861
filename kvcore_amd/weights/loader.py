"""Binds checkpoint tensors to a model's parameters by name, or fills them at random.

Reference: kvcore/model/model_utils.py:37-128 (bind by name; q/k/v and gate/up tensors
are copied into row ranges of stacked parameters) and kvcore/model/model_loader/
default_loader.py:179-196 (a strict check of what was loaded).  The reference reports
only missing names, drops unexpected ones silently (model_utils.py:65-76) and leaves
wrong shapes to torch's copy error; here all three are collected and raised as one
``WeightError`` that lists them.
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path

import torch

from kvcore_amd.models.decoder import BoundParam, DecoderModel

from .safetensors_io import SafetensorsFile, weight_files, write_safetensors


class WeightError(ValueError):
    """The checkpoint does not fit the model.  ``missing``, ``unexpected`` and
    ``mismatched`` hold the names; the message lists them all."""

    def __init__(self, missing: list[str], unexpected: list[str],
                 mismatched: list[tuple[str, tuple[int, ...], tuple[int, ...]]]) -> None:
        self.missing = missing
        self.unexpected = unexpected
        self.mismatched = mismatched
        lines = ["checkpoint does not match the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if mismatched:
            lines.append(f"  wrong shapes ({len(mismatched)}): " + ", ".join(
                f"{name} expected {list(exp)} got {list(got)}" for name, exp, got in mismatched))
        super().__init__("\n".join(lines))


def _expected_shape(bp: BoundParam, rows: int) -> tuple[int, ...]:
    return (rows, *bp.spec.shape[1:])


def load_weights(model: DecoderModel, model_dir: str | Path, *, strict: bool = True) -> None:
    """Copy every tensor of the folder's safetensors files into its parameter.

    Floating tensors are converted to the parameter's dtype on the way (the model dtype
    for matrices; float32 for vectors, so a gain stored in 32-bit keeps all its bits);
    integer tables become int32.
    """
    wanted = model.checkpoint_map()
    optional = model.optional_checkpoint_names()
    ignored_suffixes = model.spec.ignored_suffixes
    seen: set[str] = set()
    unexpected: list[str] = []
    mismatched: list[tuple[str, tuple[int, ...], tuple[int, ...]]] = []

    for path in weight_files(model_dir):
        if not path.is_file():
            raise RuntimeError(f"Weight file named by the index is missing: {path}")
        with SafetensorsFile(path) as f:
            for name, entry in f.entries.items():
                if name in wanted:
                    bp, row, rows = wanted[name]
                    expect = _expected_shape(bp, rows)
                    if entry.shape != expect:
                        mismatched.append((name, expect, entry.shape))
                        seen.add(name)
                        continue
                    src = f.tensor(name)
                    dst = bp.tensor.narrow(0, row, rows)
                    if src.dtype.is_floating_point != dst.dtype.is_floating_point:
                        mismatched.append((name, expect, entry.shape))
                        seen.add(name)
                        continue
                    dst.copy_(src)
                    seen.add(name)
                elif name in optional or any(name.endswith(s) for s in ignored_suffixes):
                    continue
                else:
                    unexpected.append(name)
    missing = sorted(set(wanted) - seen)
    if missing or mismatched or (strict and unexpected):
        raise WeightError(missing, sorted(unexpected) if strict else [], mismatched)
    if model.device.type == "cuda":
        torch.cuda.synchronize(model.device)


# ------------------------------------------------------------------- random weights
_INIT_RULES = {"normal": (0.0, 0.02), "gain": (1.0, 0.1)}  # (mean, standard deviation)


def _tensor_seed(seed: int, name: str) -> tuple[int, int]:
    """Two 32-bit words that key the generator for checkpoint tensor ``name``."""
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:4], "little"), int.from_bytes(digest[4:8], "little")


def random_tensor(seed: int, name: str, shape: tuple[int, ...], init: str,
                  device: torch.device | str = "cpu") -> torch.Tensor:
    """float32 values of checkpoint tensor ``name``: a function of (seed, name, element
    index) only, so they depend neither on the order in which tensors are made, nor on how
    they are stacked, nor on the device that draws them (the GPU kernel and its host twin,
    ``weights/random_normal.py``, give the same bits).  ``normal``: N(0, 0.02); ``gain``:
    1 + N(0, 0.1); ``zeros``."""
    out = torch.empty(shape, dtype=torch.float32, device=device)
    fill_random(out, seed, name, init)
    return out


def fill_random(out: torch.Tensor, seed: int, name: str, init: str) -> None:
    """Fill the contiguous tensor ``out`` (float32 or bfloat16; bfloat16 receives the float32
    values rounded to nearest even) with the values of checkpoint tensor ``name``."""
    if not out.is_contiguous():
        raise ValueError("fill_random needs a contiguous tensor")
    if init == "zeros":
        out.zero_()
        return
    mean, std = _INIT_RULES[init]
    lo, hi = _tensor_seed(seed, name)
    if out.is_cuda:
        from kvcore_amd.ops import library as ops

        ops.fill_normal(out, lo, hi, mean, std)
        return
    from . import random_normal

    values = torch.from_numpy(random_normal.normal(lo, hi, out.numel(), mean, std)).view(out.shape)
    out.copy_(values)


def init_random_weights(model: DecoderModel, seed: int) -> None:
    """Fill every parameter in place, checkpoint tensor by checkpoint tensor, on the model's
    device, from the same float32 draws that ``write_random_model`` makes for this seed.  A
    matrix kept in bfloat16 is the draw rounded once, as a folder of bfloat16 matrices holds
    it, so a bfloat16 model filled here equals one loaded from that folder bit for bit.  A
    float32 model keeps the draws unrounded: it equals a folder written with
    ``dtype=torch.float32``, and differs by that one rounding from a float32 model that loads
    a folder of bfloat16 matrices (the default of ``write_random_model``)."""
    for name, (bp, row, rows) in model.checkpoint_map().items():
        fill_random(bp.tensor.narrow(0, row, rows), seed, name, bp.spec.init)
    if model.device.type == "cuda":
        torch.cuda.synchronize(model.device)


def random_checkpoint_tensors(spec_params: dict[str, tuple[tuple[int, ...], str, str]], seed: int,
                              dtype: torch.dtype, device: torch.device | str = "cpu") -> dict[str, torch.Tensor]:
    """``{name: (shape, init, kind)}`` -> CPU tensors; matrices in ``dtype``, vectors in
    float32.  ``device`` is where the numbers are drawn (the values do not depend on it; a
    GPU draws a large model far sooner)."""
    out = {}
    for name, (shape, init, kind) in spec_params.items():
        t = torch.empty(shape, dtype=dtype if kind == "matrix" else torch.float32, device=device)
        fill_random(t, seed, name, init)
        out[name] = t.cpu()
    return out


def checkpoint_layout(model_spec) -> dict[str, tuple[tuple[int, ...], str, str]]:
    """The checkpoint tensors a model of this spec reads: name -> (shape, init rule,
    kind), derived from the parts' declarations without allocating the model."""
    from kvcore_amd.models.decoder import build_parts

    layout: dict[str, tuple[tuple[int, ...], str, str]] = {}
    for prefix, part in build_parts(model_spec).owned:
        for ps in part.param_specs():
            for src in ps.resolved_sources():
                layout[f"{prefix}.{src.name}"] = ((src.rows, *ps.shape[1:]), ps.init, ps.kind)
    return layout


def write_random_model(folder: str | Path, config: dict, seed: int,
                       dtype: torch.dtype = torch.bfloat16, device: torch.device | str = "cpu") -> Path:
    """The random-weights mode as a folder: ``config.json`` and ``model.safetensors``
    made from a configuration mapping and a seed.  Matrices are stored in ``dtype``,
    vectors (norm gains) in float32.  ``device``: where the numbers are drawn, which does
    not change them."""
    from kvcore_amd.registry import resolve_architecture

    arch = resolve_architecture(config)
    typed = arch.parse_config(config)
    spec = arch.build_spec(typed)
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    tensors = random_checkpoint_tensors(checkpoint_layout(spec), seed, dtype, device)
    write_safetensors(folder / "model.safetensors", tensors, metadata={"format": "pt", "seed": str(seed)})
    (folder / "config.json").write_text(json.dumps(dict(config), indent=2) + "\n")
    return folder
