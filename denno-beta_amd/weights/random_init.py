"""Random weights: tensors drawn from a configuration's ParamSpecs and a seed, and a
writer of whole model folders (config.json + model.safetensors).

Each tensor's values depend on (seed, tensor name) only, so two models that share a
tensor name and shape share its values, and the order of drawing does not matter.
The reference has no such mode; its tests use synthetic models instead
(crates/denno-engine/src/testutil.rs:52-78).
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Sequence

import torch

from .safetensors_io import write_safetensors
from .spec import ParamSpec

_TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


def _generator(seed: int, name: str, device="cpu") -> torch.Generator:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device=device)
    g.manual_seed(int.from_bytes(h[:8], "little") & ((1 << 63) - 1))
    return g


def draw(spec: ParamSpec, seed: int, device="cpu") -> torch.Tensor:
    """The tensor in its stored shape, 32-bit (int64 for an integer table)."""
    g = _generator(seed, spec.name, device)
    kind = spec.init[0]
    if kind == "normal":
        _, mean, std = spec.init
        t = torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device)
        return t * std + mean
    if kind == "randint":
        _, lo, hi = spec.init
        return torch.randint(lo, hi, spec.shape, generator=g, device=device)
    raise ValueError(f"ParamSpec {spec.name}: unknown init {spec.init!r}")


def _piece(spec: ParamSpec, fname: str, shape) -> ParamSpec:
    """The spec of one file tensor of `spec`: itself, or one of its sources as a tensor of its own."""
    if spec.sources is None:
        return spec
    return ParamSpec(fname, tuple(shape), spec.role, spec.init, dtype_hint=spec.dtype_hint)


def draw_joined(spec: ParamSpec, seed: int, device="cpu") -> torch.Tensor:
    """The tensor in its stored shape: drawn whole, or each source drawn under its own name and joined."""
    if spec.sources is None:
        return draw(spec, seed, device)
    return torch.cat([draw(_piece(spec, fname, shape), seed, device) for fname, shape in spec.pieces()], dim=spec.concat_dim)


def stored_dtype(spec: ParamSpec, dtype: str) -> torch.dtype:
    if spec.role == "int_table":
        return torch.int32
    if spec.dtype_hint is not None:
        return _TORCH[spec.dtype_hint]
    return _TORCH[dtype]


def write_model_folder(folder: str, config: dict, seed: int, dtype: str = "float32",
                       name_prefix: str = "") -> str:
    """Writes `folder/config.json` and `folder/model.safetensors` for the architecture
    that `config` names.  `dtype` is the storage type of the floating tensors."""
    from ..config import resolve_architecture
    arch = resolve_architecture(config)
    cfg = arch.config_cls.from_dict(config)
    spec = arch.build(cfg)
    specs: Sequence[ParamSpec] = spec.param_specs()
    os.makedirs(folder, exist_ok=True)
    out = dict(config)
    out.setdefault("architectures", [arch.name])
    out["torch_dtype"] = dtype
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(out, f, indent=1)
    # (a tensor that a checkpoint stores in pieces is written in pieces, each drawn under its own name)
    pieces = {name_prefix + fname: _piece(s, fname, shape) for s in specs for fname, shape in s.pieces()}
    layout = [(n, stored_dtype(p, dtype), tuple(p.shape)) for n, p in pieces.items()]
    write_safetensors(
        os.path.join(folder, "model.safetensors"), layout,
        lambda n: draw(pieces[n], seed).to(stored_dtype(pieces[n], dtype)),
        metadata={"format": "pt", "seed": seed})
    return folder


def draw_all(specs: Sequence[ParamSpec], seed: int, *, engine_dtype: str, device,
             stored: str = "bfloat16") -> Dict[str, torch.Tensor]:
    """Random weights straight onto the device, as the loader would leave them after
    reading a folder written with storage type `stored`.  Values are drawn on the device,
    so they differ from a folder's (the generators differ), but the rule (seed, name) holds."""
    from .loader import held_dtype
    code = {"bfloat16": "BF16", "float32": "F32", "float16": "F16"}[stored]
    out = {}
    for s in specs:
        t = draw_joined(s, seed, device=device).to(stored_dtype(s, stored))
        dt = held_dtype(s, "I32" if s.role == "int_table" else code, engine_dtype, False)
        t = t.to(dt)
        out[s.name] = (t.t() if s.transpose else t).contiguous()
    return out
