"""Random weights from a configuration and a seed, and the model folder they are written to.

Every tensor is drawn from its own generator, seeded by the seed and the tensor's
name, so a tensor's values do not depend on which other tensors exist or on the
order they are drawn in. Values are rounded to bfloat16 before they are written
(or to the dtype asked for), so float32 and bfloat16 engines read the same numbers.
"""
from __future__ import annotations

import hashlib
import os
from dataclasses import dataclass
from typing import Dict, Mapping, Optional, Sequence

import torch

from ..parts.base import INT_TABLE, TensorDecl
from .safetensors_io import save_file


@dataclass(frozen=True)
class InitRule:
    """Tensors whose name ends with ``suffix`` are drawn as ``mean + N(0, stds[std_key])``; first match wins."""
    suffix: str
    mean: float
    std_key: str


DEFAULT_STDS = {"std": 0.02, "norm_std": 0.0}


def _generator_for(seed: int, name: str, device: torch.device) -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    generator = torch.Generator(device=device)
    generator.manual_seed(int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF)
    return generator


def random_tensors(decls: Mapping[str, TensorDecl], rules: Sequence[InitRule], seed: int,
                   dtype: torch.dtype = torch.bfloat16, stds: Optional[Mapping[str, float]] = None,
                   device: torch.device | str = "cpu") -> Dict[str, torch.Tensor]:
    stds = {**DEFAULT_STDS, **(stds or {})}
    device = torch.device(device)
    out: Dict[str, torch.Tensor] = {}
    for name, decl in decls.items():
        if decl.kind == INT_TABLE:
            raise ValueError(f"no random rule for the integer table {name!r}")
        rule = next((rule for rule in rules if name.endswith(rule.suffix)), None)
        if rule is None:
            raise ValueError(f"no random rule matches tensor {name!r}")
        std = float(stds[rule.std_key])
        generator = _generator_for(seed, name, device)
        if std == 0.0:
            value = torch.full(decl.shape, rule.mean, dtype=torch.float32, device=device)
        else:
            value = torch.empty(decl.shape, dtype=torch.float32, device=device)
            value.normal_(rule.mean, std, generator=generator)
        out[name] = value.to(dtype)
    return out


def write_model_folder(folder: str, config, seed: int, dtype: torch.dtype = torch.bfloat16,
                       stds: Optional[Mapping[str, float]] = None) -> str:
    """Write ``config.json`` and ``model.safetensors`` with random weights; returns the folder."""
    from ..config.registry import architecture_named
    from ..parts import Model, Runtime

    architecture = architecture_named(config.architecture)
    if architecture.init_rules is None:
        raise ValueError(f"architecture {architecture.name} has no rules for random weights")
    spec = architecture.build_spec(config)
    model = Model(spec, Runtime(dtype=torch.float32, device=torch.device("cpu")))
    tensors = random_tensors(model.tensors(), architecture.init_rules(config), seed, dtype=dtype, stds=stds)
    os.makedirs(folder, exist_ok=True)
    config.save(folder)
    save_file(tensors, os.path.join(folder, "model.safetensors"), metadata={"format": "pt"})
    return folder


def main(argv=None) -> int:
    """``python -m microllm_rocm_amd.weights.random_init --config FILE --seed S --out DIR``: a model folder
    (config.json, model.safetensors) with random weights for the architecture the configuration names."""
    import argparse

    from ..config.registry import load_config

    parser = argparse.ArgumentParser(prog="microllm_make_model", description=main.__doc__)
    parser.add_argument("--config", required=True, help="a config.json (or a folder that holds one)")
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--out", required=True, help="folder to write")
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--std", type=float, default=0.02, help="standard deviation of matrices, tables and biases")
    parser.add_argument("--norm-std", type=float, default=0.0, help="norm weights are 1 + N(0, norm-std)")
    args = parser.parse_args(argv)
    _, config = load_config(args.config)
    dtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    write_model_folder(args.out, config, args.seed, dtype=dtype, stds={"std": args.std, "norm_std": args.norm_std})
    print(args.out)
    return 0


if __name__ == "__main__":
    import sys
    sys.exit(main())
