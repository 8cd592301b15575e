"""Reader and writer of the safetensors container, without any third-party package.

File layout: 8 bytes little-endian header length N, N bytes of JSON mapping each tensor
name to {"dtype", "shape", "data_offsets": [begin, end]} (offsets relative to the end of
the header), then the raw little-endian tensor data.  Reading maps the file and hands out
views; nothing is copied until a tensor is moved to the device.

A model folder holds either `model.safetensors` or `model.safetensors.index.json` whose
`weight_map` names the shard of every tensor; the headers of all shards are merged into one
manifest (reference mini_llm/checkpoint.py:83-168).
"""

from __future__ import annotations

import json
import mmap
import struct
from dataclasses import dataclass
from pathlib import Path

import torch

from ..errors import CheckpointError

DTYPES = {
    "F32": (torch.float32, 4), "BF16": (torch.bfloat16, 2), "F16": (torch.float16, 2), "F64": (torch.float64, 8),
    "I64": (torch.int64, 8), "I32": (torch.int32, 4), "I16": (torch.int16, 2), "I8": (torch.int8, 1),
    "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {dtype: name for name, (dtype, _) in DTYPES.items()}


@dataclass(frozen=True)
class TensorInfo:
    name: str
    shape: tuple[int, ...]
    dtype: str
    file: Path
    begin: int  # absolute byte offsets in the file
    end: int

    @property
    def num_elements(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n


def read_header(path: Path) -> list[TensorInfo]:
    path = Path(path)
    if not path.is_file():
        raise CheckpointError(f"checkpoint file does not exist: {path}")
    size = path.stat().st_size
    with open(path, "rb") as handle:
        prefix = handle.read(8)
        if len(prefix) != 8:
            raise CheckpointError(f"not a safetensors file (too short): {path}")
        (header_len,) = struct.unpack("<Q", prefix)
        if header_len <= 0 or 8 + header_len > size:
            raise CheckpointError(f"not a safetensors file (bad header length {header_len}): {path}")
        try:
            header = json.loads(handle.read(header_len).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as exc:
            raise CheckpointError(f"not a safetensors file (header is not JSON): {path}") from exc
    if not isinstance(header, dict):
        raise CheckpointError(f"not a safetensors file (header is not an object): {path}")
    base = 8 + header_len
    infos = []
    for name, entry in header.items():
        if name == "__metadata__":
            continue
        try:
            dtype, shape = entry["dtype"], tuple(int(s) for s in entry["shape"])
            begin, end = (int(v) for v in entry["data_offsets"])
        except (KeyError, TypeError, ValueError) as exc:
            raise CheckpointError(f"malformed header entry for tensor {name!r} in {path}") from exc
        if dtype not in DTYPES:
            raise CheckpointError(f"unsupported safetensors dtype {dtype!r} for tensor {name!r} in {path}")
        info = TensorInfo(name, shape, dtype, path, base + begin, base + end)
        if begin < 0 or end < begin or base + end > size or end - begin != info.num_elements * DTYPES[dtype][1]:
            raise CheckpointError(f"tensor {name!r} in {path} has data offsets that do not match its shape")
        infos.append(info)
    return infos


class Checkpoint:
    """Merged manifest of a single-file or sharded checkpoint with lazy tensor access."""

    def __init__(self, infos: list[TensorInfo]):
        self.manifest = {info.name: info for info in sorted(infos, key=lambda i: i.name)}
        self._maps: dict[Path, mmap.mmap] = {}

    @classmethod
    def from_model_dir(cls, model_dir) -> "Checkpoint":
        model_dir = Path(model_dir)
        single = model_dir / "model.safetensors"
        if single.is_file():
            return cls(read_header(single))
        index = model_dir / "model.safetensors.index.json"
        if index.is_file():
            return cls._from_index(index)
        raise CheckpointError(
            f"model directory contains neither model.safetensors nor model.safetensors.index.json: {model_dir}")

    @classmethod
    def _from_index(cls, index: Path) -> "Checkpoint":
        try:
            weight_map = json.loads(index.read_text(encoding="utf-8"))["weight_map"]
        except (json.JSONDecodeError, KeyError, TypeError) as exc:
            raise CheckpointError(f"invalid checkpoint index: {index}") from exc
        if not isinstance(weight_map, dict) or not weight_map:
            raise CheckpointError(f"checkpoint index has no weight_map: {index}")
        infos, problems = [], []
        for shard in dict.fromkeys(weight_map.values()):
            shard_path = index.parent / shard
            if not shard_path.is_file():
                raise CheckpointError(f"checkpoint shard does not exist: {shard_path}")
            in_shard = {info.name: info for info in read_header(shard_path)}
            wanted = {name for name, s in weight_map.items() if s == shard}
            problems += [f"{name} is mapped to {shard} but is not stored there" for name in sorted(wanted - in_shard.keys())]
            problems += [f"{name} is stored in {shard} but the index does not map it there" for name in sorted(in_shard.keys() - wanted)]
            infos += [in_shard[name] for name in sorted(wanted & in_shard.keys())]
        if problems:
            raise CheckpointError("checkpoint index does not match its shards:\n  - " + "\n  - ".join(problems))
        return cls(infos)

    def tensor(self, name: str) -> torch.Tensor:
        """CPU tensor viewing the mapped file (read-only data: copy or move before writing)."""
        try:
            info = self.manifest[name]
        except KeyError:
            raise CheckpointError(f"tensor is not in the checkpoint: {name}") from None
        if info.file not in self._maps:
            with open(info.file, "rb") as handle:
                self._maps[info.file] = mmap.mmap(handle.fileno(), 0, access=mmap.ACCESS_COPY)
        dtype, _ = DTYPES[info.dtype]
        if info.num_elements == 0:
            return torch.empty(info.shape, dtype=dtype)
        view = memoryview(self._maps[info.file])[info.begin:info.end]
        return torch.frombuffer(view, dtype=dtype, count=info.num_elements).view(info.shape)

    def close(self) -> None:
        self._maps.clear()


def write_safetensors(path, tensors: dict[str, torch.Tensor], metadata: dict | None = None) -> None:
    """Write CPU tensors into one safetensors file, names sorted, data 8-byte aligned."""
    header, offset, blobs = {}, 0, []
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    for name in sorted(tensors):
        t = tensors[name].detach().cpu().contiguous()
        if t.dtype not in _NAMES:
            raise CheckpointError(f"cannot store tensor {name!r} of dtype {t.dtype}")
        raw = t.view(torch.uint8).numpy().tobytes() if t.numel() else b""
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    encoded = json.dumps(header, separators=(",", ":")).encode("utf-8")
    encoded += b" " * (-len(encoded) % 8)
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(encoded)))
        handle.write(encoded)
        for raw in blobs:
            handle.write(raw)
