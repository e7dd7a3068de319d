"""Weights from safetensors by tensor name, checked against the model's ParamSpecs.

Dtype rule.  float32 engine: every tensor is converted to 32-bit (exact for bfloat16 and
float16 files).  bfloat16 engine: a matrix or table stored in bfloat16 stays bfloat16; a
tensor stored in 32-bit (or float16) stays 32-bit unless `cast_matrices` asks to round
matrices and tables to bfloat16 once, at load; vectors (norm weights, biases) are always
held in 32-bit, which is exact for every storage type; integer tables become int32.

Errors.  The reference fails on the first missing tensor and checks no shapes
(crates/denno-engine/src/load.rs:129-133).  Here one CheckpointError lists all missing
tensors, all unexpected ones and all wrong shapes at once.
"""
from __future__ import annotations

import re
from typing import Dict, Iterable, List, Optional, Sequence

import torch

from .safetensors_io import open_checkpoint
from .spec import ParamSpec


class CheckpointError(ValueError):
    def __init__(self, where, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.wrong_dtype = list(wrong_shape), list(wrong_dtype)
        lines = [f"{where}: the checkpoint does not fit the model"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + ", ".join(
                f"{n}: file {list(got)}, model {list(want)}" for n, got, want in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  unsupported dtypes ({len(self.wrong_dtype)}): " + ", ".join(
                f"{n}: {dt}" for n, dt in self.wrong_dtype))
        super().__init__("\n".join(lines))


_FLOAT_STORED = ("F32", "BF16", "F16")
_INT_STORED = ("I32", "I64", "I16", "I8", "U8")


def held_dtype(spec: ParamSpec, stored: str, engine_dtype: str, cast_matrices: bool) -> torch.dtype:
    if spec.role == "int_table":
        return torch.int32
    if spec.role == "vector" or engine_dtype == "float32":
        return torch.float32
    if stored == "BF16" or cast_matrices:
        return torch.bfloat16
    return torch.float32


def load_checkpoint(model_dir: str, specs: Sequence[ParamSpec], *, engine_dtype: str, device,
                    cast_matrices: bool = False, prefixes: Sequence[str] = ("",),
                    ignore: Iterable[str] = (), tied: Optional[Dict[str, str]] = None,
                    notes: Optional[List[str]] = None) -> Dict[str, torch.Tensor]:
    """-> {spec.name: tensor on `device`}.

    prefixes: model-wide prefixes a file may put before every name ("transformer.").
    ignore:   regular expressions of file tensors that are buffers, not weights.
    tied:     {file name: spec name}: a file tensor that repeats another (a tied head);
              it must have that tensor's shape and is otherwise not read.
    A spec with `sources` is read from those file tensors, joined along its `concat_dim` (in the stored layout,
    before a transpose); missing pieces, unexpected tensors and wrong shapes are reported by the file's names.
    """
    where, files = open_checkpoint(model_dir)
    try:
        ignore_re = [re.compile(p) for p in ignore]
        tied = tied or {}
        # file name -> (spec, the piece's stored shape): a spec is one file tensor, or several joined at load
        by_name, spec_of = {}, {s.name: s for s in specs}
        for s in specs:
            for fname, shape in s.pieces():
                by_name[fname] = (s, shape)
        found, unexpected, wrong_shape, wrong_dtype = {}, [], [], []
        for fname in where:
            base = None
            for p in sorted(prefixes, key=len, reverse=True):
                if fname.startswith(p) and (fname[len(p):] in by_name or fname[len(p):] in tied):
                    base = fname[len(p):]
                    break
            if base is None:
                if not any(r.search(fname) for r in ignore_re):
                    unexpected.append(fname)
                continue
            stored, shape = where[fname].entries[fname]
            if base in tied:
                want = spec_of[tied[base]].shape
                if tuple(shape) != tuple(want):
                    wrong_shape.append((fname, shape, want))
                continue
            spec, want = by_name[base]
            if tuple(shape) != tuple(want):
                wrong_shape.append((fname, shape, want))
            ok = _INT_STORED if spec.role == "int_table" else _FLOAT_STORED
            if stored not in ok:
                wrong_dtype.append((fname, stored))
            if base in found:
                unexpected.append(fname + " (a second copy of " + found[base] + ")")
            else:
                found[base] = fname
        missing = [fname for s in specs for fname, _ in s.pieces() if fname not in found]
        if missing or unexpected or wrong_shape or wrong_dtype:
            raise CheckpointError(model_dir, missing, unexpected, wrong_shape, wrong_dtype)

        out, kept32 = {}, 0
        for spec in specs:
            names = [found[fname] for fname, _ in spec.pieces()]
            kinds = [where[n].entries[n][0] for n in names]
            # (pieces stored in different precisions: bfloat16 only if every piece is)
            stored = kinds[0] if all(k == kinds[0] for k in kinds) else "F32"
            dt = held_dtype(spec, stored, engine_dtype, cast_matrices)
            if (engine_dtype == "bfloat16" and spec.role in ("matrix", "table")
                    and dt == torch.float32):
                kept32 += 1
            if len(names) == 1:
                t = where[names[0]].tensor(names[0])
            else:
                host_dt = torch.int64 if spec.role == "int_table" else (torch.float32 if stored != "BF16" else torch.bfloat16)
                t = torch.cat([where[n].tensor(n).to(host_dt) for n in names], dim=spec.concat_dim)
            out[spec.name] = place(t, spec, dt, device)
        if kept32 and notes is not None:
            notes.append(f"{kept32} matrices are stored in 32-bit and stay so; their products run "
                         "in 32-bit (cast_matrices rounds them to bfloat16 at load)")
        return out
    finally:
        for f in files:
            f.close()


def place(t: torch.Tensor, spec: ParamSpec, dtype: torch.dtype, device) -> torch.Tensor:
    """Host tensor -> device, in the held dtype and layout."""
    t = t.to(device=device, dtype=dtype)      # copies: the source may be a read-only mapping
    if spec.transpose:
        t = t.t()
    return t.contiguous()
