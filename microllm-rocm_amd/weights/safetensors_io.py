"""Reading and writing safetensors files without executing anything from them.

Format facts as the reference checks them (src/io/safetensors.cpp:438-476,
492-526): an 8-byte little-endian header length, a JSON header whose members
give ``dtype``, ``shape`` and ``data_offsets`` [begin, end) into the payload;
``__metadata__`` is skipped; every byte range must equal numel x element size,
ranges must tile the payload without hole or overlap, and the last end must be
the payload's size. Tensors are memory-mapped and handed out as torch tensors
of the stored dtype.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, List, Mapping, Tuple

import numpy as np
import torch

MAX_HEADER_BYTES = 256 << 20  # src/io/safetensors.cpp:492-526

# safetensors dtype tag -> (torch dtype, numpy carrier dtype, bytes per element)
_DTYPES = {
    "F32": (torch.float32, np.dtype("<f4"), 4),
    "BF16": (torch.bfloat16, np.dtype("<u2"), 2),
    "F16": (torch.float16, np.dtype("<f2"), 2),
    "I32": (torch.int32, np.dtype("<i4"), 4),
    "I64": (torch.int64, np.dtype("<i8"), 8),
    "F64": (torch.float64, np.dtype("<f8"), 8),
}
_TAG_OF = {torch_dtype: tag for tag, (torch_dtype, _, _) in _DTYPES.items()}


class SafetensorsError(ValueError):
    """A file that is not a well-formed safetensors file."""


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    begin: int
    end: int

    @property
    def numel(self) -> int:
        count = 1
        for extent in self.shape:
            count *= extent
        return count


def _parse_header(raw: bytes, payload_size: int, path: str) -> Dict[str, TensorEntry]:
    try:
        header = json.loads(raw.decode("utf-8"))
    except (UnicodeDecodeError, json.JSONDecodeError) as error:
        raise SafetensorsError(f"{path}: header is not valid JSON: {error}") from None
    if not isinstance(header, dict):
        raise SafetensorsError(f"{path}: header must be a JSON object")
    entries: Dict[str, TensorEntry] = {}
    for name, member in header.items():
        if name == "__metadata__":
            continue
        if not isinstance(member, dict):
            raise SafetensorsError(f"{path}: entry {name!r} is not an object")
        dtype = member.get("dtype")
        shape = member.get("shape")
        offsets = member.get("data_offsets")
        if dtype not in _DTYPES:
            raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {dtype!r}")
        if (not isinstance(shape, list)
                or any(isinstance(e, bool) or not isinstance(e, int) or e < 0 for e in shape)):
            raise SafetensorsError(f"{path}: tensor {name!r} has a bad shape {shape!r}")
        if (not isinstance(offsets, list) or len(offsets) != 2
                or any(isinstance(e, bool) or not isinstance(e, int) for e in offsets)):
            raise SafetensorsError(f"{path}: tensor {name!r} has bad data_offsets {offsets!r}")
        entry = TensorEntry(name, dtype, tuple(shape), offsets[0], offsets[1])
        if entry.begin < 0 or entry.end < entry.begin or entry.end > payload_size:
            raise SafetensorsError(f"{path}: tensor {name!r} lies outside the payload")
        if entry.end - entry.begin != entry.numel * _DTYPES[dtype][2]:
            raise SafetensorsError(
                f"{path}: tensor {name!r} spans {entry.end - entry.begin} bytes but its shape "
                f"{list(entry.shape)} of {dtype} needs {entry.numel * _DTYPES[dtype][2]}")
        entries[name] = entry
    cursor = 0
    for entry in sorted(entries.values(), key=lambda item: (item.begin, item.end)):
        if entry.begin != cursor:
            kind = "overlap" if entry.begin < cursor else "hole"
            raise SafetensorsError(f"{path}: {kind} in the payload before tensor {entry.name!r}")
        cursor = entry.end
    if cursor != payload_size:
        raise SafetensorsError(f"{path}: payload has {payload_size - cursor} bytes no tensor owns")
    return entries


class SafetensorsFile:
    """One memory-mapped file; ``tensor(name)`` returns a view that shares the mapping."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too short to hold a header length")
        self._handle = open(path, "rb")
        (header_size,) = struct.unpack("<Q", self._handle.read(8))
        if header_size == 0 or header_size > MAX_HEADER_BYTES or 8 + header_size > size:
            self._handle.close()
            raise SafetensorsError(f"{path}: header length {header_size} is invalid")
        raw = self._handle.read(header_size)
        self._payload_start = 8 + header_size
        try:
            self.entries = _parse_header(raw, size - self._payload_start, path)
        except SafetensorsError:
            self._handle.close()
            raise
        self._map = mmap.mmap(self._handle.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def names(self) -> List[str]:
        return list(self.entries)

    def tensor(self, name: str) -> torch.Tensor:
        entry = self.entries[name]
        torch_dtype, carrier, _ = _DTYPES[entry.dtype]
        array = np.frombuffer(self._map, dtype=carrier, count=entry.numel,
                              offset=self._payload_start + entry.begin)
        # The mapping is read-only; torch only warns about that and nothing writes to it.
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            tensor = torch.from_numpy(array)
        if torch_dtype == torch.bfloat16:
            tensor = tensor.view(torch.bfloat16)
        return tensor.reshape(entry.shape)

    def close(self) -> None:
        # Views handed out keep the mapping alive through numpy's buffer reference.
        self._handle.close()


def save_file(tensors: Mapping[str, torch.Tensor], path: str, metadata: Mapping[str, str] | None = None) -> None:
    """Write ``tensors`` in the order given; payload ranges tile without holes."""
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    cursor = 0
    blobs: List[bytes] = []
    for name, tensor in tensors.items():
        tensor = tensor.detach().cpu().contiguous()
        if tensor.dtype not in _TAG_OF:
            raise SafetensorsError(f"cannot write tensor {name!r} of dtype {tensor.dtype}")
        tag = _TAG_OF[tensor.dtype]
        if tensor.dtype == torch.bfloat16:
            raw = tensor.view(torch.int16).numpy().tobytes()
        else:
            raw = tensor.numpy().tobytes()
        header[name] = {"dtype": tag, "shape": list(tensor.shape), "data_offsets": [cursor, cursor + len(raw)]}
        cursor += len(raw)
        blobs.append(raw)
    encoded = json.dumps(header, separators=(",", ":")).encode("utf-8")
    encoded += b" " * (-len(encoded) % 8)
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(encoded)))
        handle.write(encoded)
        for raw in blobs:
            handle.write(raw)


def open_model_files(folder: str) -> Tuple[Dict[str, SafetensorsFile], Dict[str, str]]:
    """Open ``model.safetensors``, or the shards an index names.

    Returns the open files by file name and a map from tensor name to file name.
    Shard paths must be relative and stay inside the folder, and no tensor may
    appear in two shards (src/io/safetensors.cpp:620-670).
    """
    single = os.path.join(folder, "model.safetensors")
    index = os.path.join(folder, "model.safetensors.index.json")
    files: Dict[str, SafetensorsFile] = {}
    owner: Dict[str, str] = {}
    if os.path.exists(single):
        files["model.safetensors"] = SafetensorsFile(single)
    elif os.path.exists(index):
        with open(index, "r", encoding="utf-8") as handle:
            weight_map = json.load(handle).get("weight_map")
        if not isinstance(weight_map, dict) or not weight_map:
            raise SafetensorsError(f"{index}: weight_map is missing or empty")
        for shard in sorted(set(weight_map.values())):
            if not isinstance(shard, str) or os.path.isabs(shard) or ".." in shard.replace("\\", "/").split("/"):
                raise SafetensorsError(f"{index}: shard path {shard!r} must be relative and inside the folder")
            files[shard] = SafetensorsFile(os.path.join(folder, shard))
    else:
        raise FileNotFoundError(f"{folder}: neither model.safetensors nor model.safetensors.index.json")
    for file_name, handle in files.items():
        for name in handle.names():
            if name in owner:
                raise SafetensorsError(f"tensor {name!r} is in both {owner[name]} and {file_name}")
            owner[name] = file_name
    return files, owner
