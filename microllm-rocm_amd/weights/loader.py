"""Binding of the tensors in a model folder to the tensors a model declares, by name.

Every declared tensor must be found and every tensor in the files must be
declared; shapes must agree. All failures are gathered into one error that lists
them, and nothing is handed out when there is any (the reference's strict load,
src/model/model.cpp:1786-1847). Element types: a tensor stored in 32-bit stays
32-bit; bfloat16 matrices stay bfloat16 in a bfloat16 engine and are widened in
a float32 engine; vectors (norm weights, biases) are always widened to float32,
which is exact; float16 is widened to float32; integer tables become int32.
"""
from __future__ import annotations

from typing import Dict, List, Mapping

import torch

from ..parts.base import INT_TABLE, MATRIX, TensorDecl, VECTOR
from .safetensors_io import open_model_files


class WeightsError(ValueError):
    """The files do not hold what the model declares; the text lists every difference."""

    def __init__(self, missing: List[str], unexpected: List[str], incompatible: List[str]):
        self.missing, self.unexpected, self.incompatible = missing, unexpected, incompatible
        lines = ["weights do not match the model:"]
        lines += [f"  missing: {name}" for name in missing]
        lines += [f"  unexpected: {name}" for name in unexpected]
        lines += [f"  incompatible: {text}" for text in incompatible]
        super().__init__("\n".join(lines))


def placed_dtype(stored: torch.dtype, decl: TensorDecl, engine_dtype: torch.dtype) -> torch.dtype:
    if decl.kind == INT_TABLE:
        return torch.int32
    if decl.kind == VECTOR:
        return torch.float32
    if stored == torch.bfloat16 and engine_dtype == torch.bfloat16:
        return torch.bfloat16
    return torch.float32


def check_names_and_shapes(decls: Mapping[str, TensorDecl], found: Mapping[str, tuple],
                           found_dtypes: Mapping[str, str] | None = None) -> None:
    missing = sorted(name for name in decls if name not in found)
    unexpected = sorted(name for name in found if name not in decls)
    incompatible = []
    for name, decl in decls.items():
        if name in found and tuple(found[name]) != tuple(decl.shape):
            incompatible.append(f"{name}: shape mismatch: source={list(found[name])} target={list(decl.shape)}")
        if name in found and found_dtypes is not None:
            is_int = found_dtypes[name] in ("I32", "I64")
            if is_int != (decl.kind == INT_TABLE):
                incompatible.append(f"{name}: dtype {found_dtypes[name]} does not fit a {decl.kind}")
    if missing or unexpected or incompatible:
        raise WeightsError(missing, unexpected, sorted(incompatible))


def place(tensor: torch.Tensor, decl: TensorDecl, engine_dtype: torch.dtype, device: torch.device) -> torch.Tensor:
    target = placed_dtype(tensor.dtype, decl, engine_dtype)
    if tensor.dtype == target:
        return tensor.to(device, copy=True).contiguous()
    if device.type == "cuda":
        return tensor.to(device).to(target).contiguous()  # widen on the GPU: the host copy stays small
    return tensor.to(target).contiguous()


def load_folder(folder: str, decls: Mapping[str, TensorDecl], engine_dtype: torch.dtype,
                device: torch.device) -> Dict[str, torch.Tensor]:
    files, owner = open_model_files(folder)
    try:
        shapes = {name: files[file_name].entries[name].shape for name, file_name in owner.items()}
        dtypes = {name: files[file_name].entries[name].dtype for name, file_name in owner.items()}
        check_names_and_shapes(decls, shapes, dtypes)
        out: Dict[str, torch.Tensor] = {}
        for name, decl in decls.items():
            out[name] = place(files[owner[name]].tensor(name), decl, engine_dtype, device)
        return out
    finally:
        for handle in files.values():
            handle.close()


def place_all(tensors: Mapping[str, torch.Tensor], decls: Mapping[str, TensorDecl], engine_dtype: torch.dtype,
              device: torch.device, consume: bool = False) -> Dict[str, torch.Tensor]:
    """The same checks and placement for tensors that are already in memory. With ``consume`` (``tensors`` must
    be a dict) every entry is taken out of ``tensors`` as it is placed, so that a copy replaces its source
    instead of standing beside it."""
    check_names_and_shapes(decls, {name: tuple(t.shape) for name, t in tensors.items()})
    placed: Dict[str, torch.Tensor] = {}
    for name, decl in decls.items():
        placed[name] = place(tensors.pop(name) if consume else tensors[name], decl, engine_dtype, device)
    return placed
