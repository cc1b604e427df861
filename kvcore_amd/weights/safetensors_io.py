"""Reader and writer for the safetensors container.

The format: 8 bytes little-endian header length, a JSON header mapping each tensor
name to ``{"dtype", "shape", "data_offsets": [begin, end]}`` (offsets relative to the
end of the header), then the raw little-endian tensor bytes.  The reader memory-maps
the file, so a tensor's bytes are touched only when it is copied to its destination;
nothing in the file is executed.

The reference reads the same files through the safetensors package
(kvcore/model/model_loader/weight_utils.py:11-19).
"""

from __future__ import annotations

import json
import mmap
import struct
from dataclasses import dataclass
from pathlib import Path
from typing import Iterator

import numpy as np
import torch

# safetensors dtype tag -> (torch dtype, bytes per element)
_DTYPES: dict[str, tuple[torch.dtype, int]] = {
    "F64": (torch.float64, 8),
    "F32": (torch.float32, 4),
    "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2),
    "I64": (torch.int64, 8),
    "I32": (torch.int32, 4),
    "I16": (torch.int16, 2),
    "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_TAGS = {dt: tag for tag, (dt, _) in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: torch.dtype
    shape: tuple[int, ...]
    begin: int
    end: int


class SafetensorsFile:
    """One memory-mapped file.  ``entries`` lists what it holds; ``tensor(name)`` gives
    a CPU tensor that views the mapping (copy it before the file is closed)."""

    def __init__(self, path: str | Path) -> None:
        self.path = Path(path)
        self._file = open(self.path, "rb")
        try:
            head = self._file.read(8)
            if len(head) != 8:
                raise SafetensorsError(f"{self.path}: too short for a safetensors header")
            (header_len,) = struct.unpack("<Q", head)
            size = self.path.stat().st_size
            if header_len <= 0 or 8 + header_len > size:
                raise SafetensorsError(f"{self.path}: header length {header_len} exceeds the file")
            try:
                header = json.loads(self._file.read(header_len).decode("utf-8"))
            except (UnicodeDecodeError, json.JSONDecodeError) as exc:
                raise SafetensorsError(f"{self.path}: header is not valid JSON: {exc}") from exc
            if not isinstance(header, dict):
                raise SafetensorsError(f"{self.path}: header must be an object")
            self._data_start = 8 + header_len
            data_len = size - self._data_start
            self.metadata = header.pop("__metadata__", None)
            self.entries: dict[str, TensorEntry] = {}
            for name, info in header.items():
                tag = info.get("dtype")
                if tag not in _DTYPES:
                    raise SafetensorsError(f"{self.path}: tensor {name!r} has unsupported dtype {tag!r}")
                dtype, width = _DTYPES[tag]
                shape = tuple(int(s) for s in info["shape"])
                begin, end = (int(v) for v in info["data_offsets"])
                count = int(np.prod(shape, dtype=np.int64)) if shape else 1
                if begin < 0 or end > data_len or end - begin != count * width:
                    raise SafetensorsError(
                        f"{self.path}: tensor {name!r} has offsets [{begin}, {end}) that do not fit "
                        f"shape {shape} of {tag}"
                    )
                self.entries[name] = TensorEntry(name, dtype, shape, begin, end)
            self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ) if size else None
        except Exception:
            self._file.close()
            raise

    def tensor(self, name: str) -> torch.Tensor:
        e = self.entries[name]
        if e.end == e.begin:
            return torch.empty(e.shape, dtype=e.dtype)
        raw = np.frombuffer(self._map, dtype=np.uint8, count=e.end - e.begin,
                            offset=self._data_start + e.begin)
        import warnings

        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the mapping is read-only; we never write through it
            flat = torch.from_numpy(raw)
        return flat.view(e.dtype).view(e.shape)

    def close(self) -> None:
        if self._map is not None:
            try:
                self._map.close()
            except BufferError:
                pass  # tensors still view the mapping; the OS unmaps at exit
            self._map = None
        self._file.close()

    def __enter__(self) -> "SafetensorsFile":
        return self

    def __exit__(self, *exc) -> None:
        self.close()


def write_safetensors(path: str | Path, tensors: dict[str, torch.Tensor],
                      metadata: dict[str, str] | None = None) -> None:
    """Write ``tensors`` (CPU or GPU; made contiguous) in name order."""
    header: dict[str, object] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _TAGS:
            raise SafetensorsError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _TAGS[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")


def weight_files(model_dir: str | Path) -> list[Path]:
    """The folder's weight files: those named by ``model.safetensors.index.json``'s
    ``weight_map`` if there is one, else every ``*.safetensors``, sorted.
    Reference: kvcore/model/model_loader/default_loader.py:104-128 and
    weight_utils.py:38-73."""
    folder = Path(model_dir)
    index = folder / "model.safetensors.index.json"
    if index.is_file():
        data = json.loads(index.read_text())
        weight_map = data.get("weight_map")
        if not isinstance(weight_map, dict):
            raise SafetensorsError(f"Invalid weight index file: {index}")
        return [folder / name for name in sorted(set(weight_map.values()))]
    files = sorted(folder.glob("*.safetensors"))
    if not files:
        raise RuntimeError(f"Cannot find any model weights in {folder}")
    return files


def iter_tensors(model_dir: str | Path) -> Iterator[tuple[str, torch.Tensor, SafetensorsFile]]:
    for path in weight_files(model_dir):
        if not path.is_file():
            raise RuntimeError(f"Weight file named by the index is missing: {path}")
        f = SafetensorsFile(path)
        for name in f.entries:
            yield name, f.tensor(name), f
