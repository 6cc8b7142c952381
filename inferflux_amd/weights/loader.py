"""Weights by tensor name, with one error that says everything that is wrong with a file.

The model's parts declare the tensors they expect (name -> ParamSpec).  Loading compares that
with the file: tensors that are missing, tensors nobody asked for and tensors of the wrong
shape are collected and reported together.  The reference resolves the same Hugging Face
names (runtime/backends/cuda/native/weight_map.cpp:21-58) but stops at the first missing one
and only warns about sizes (safetensors_parser.cpp:279-299).

Storage rule.  In bfloat16 mode a 16-bit float tensor is kept as bfloat16, a tensor the file
stores in 32-bit (or wider) floats stays float32, and integer tables become int32.  In float32
mode every floating tensor is widened to float32 (exact for bfloat16 and float16 input).
The reference does not convert float32 files at all (it reinterprets them,
runtime/backends/cuda/native/transformer_forward.cu:1756-1761).
"""
from __future__ import annotations

import hashlib
import os
from typing import Dict, Iterable, List, Mapping, Optional, Tuple

import torch

from ..parts.plan import ParamSpec
from .. import log
from .safetensors_io import SafetensorsError, SafetensorsFile, open_model_files, write_safetensors, write_sharded


class WeightError(ValueError):
    """Raised once per load, listing every missing, unexpected and wrongly shaped tensor."""

    def __init__(self, folder: str, missing: List[str], unexpected: List[str],
                 wrong_shape: List[Tuple[str, Tuple[int, ...], Tuple[int, ...]]], other: List[str] = ()):
        self.missing, self.unexpected, self.wrong_shape, self.other = list(missing), list(unexpected), list(wrong_shape), list(other)
        lines = [f"{folder}: the weights do not fit the model"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, expected {list(want)}" for n, got, want in self.wrong_shape))
        for o in self.other:
            lines.append(f"  {o}")
        super().__init__("\n".join(lines))


def storage_dtype(file_dtype: torch.dtype, mode: torch.dtype, integer: bool) -> torch.dtype:
    if integer or not file_dtype.is_floating_point:
        return torch.int32
    if mode == torch.float32:
        return torch.float32
    if mode == torch.bfloat16:
        return torch.bfloat16 if file_dtype in (torch.bfloat16, torch.float16) else torch.float32
    raise ValueError(f"engine dtype must be float32 or bfloat16, got {mode}")


def check_against_specs(folder: str, files: List[SafetensorsFile], specs: Mapping[str, ParamSpec],
                        strict: bool = True, unused: Optional[List[str]] = None) -> Dict[str, SafetensorsFile]:
    """Where each tensor lives, or ``WeightError`` with everything that is wrong.  Tensors nobody asked for are an
    error when ``strict``; otherwise they are reported through ``unused`` (older exports carry buffers such as
    ``rotary_emb.inv_freq`` that no part reads) and everything else is still checked."""
    where: Dict[str, SafetensorsFile] = {}
    other: List[str] = []
    for f in files:
        for n in f.names():
            if n in where:
                other.append(f"tensor '{n}' appears in both {os.path.basename(where[n].path)} and {os.path.basename(f.path)}")
            else:
                where[n] = f
    missing = sorted(n for n, s in specs.items() if n not in where and not s.optional)
    unexpected = sorted(n for n in where if n not in specs)
    wrong = []
    for n, s in specs.items():
        if n in where:
            got = where[n].shape(n)
            if tuple(got) != tuple(s.shape):
                wrong.append((n, tuple(got), tuple(s.shape)))
            if s.integer == where[n].dtype(n).is_floating_point:
                other.append(f"tensor '{n}' is {where[n].dtype(n)}, expected {'an integer' if s.integer else 'a floating'} type")
    if missing or (unexpected and strict) or wrong or other:
        raise WeightError(folder, missing, unexpected, sorted(wrong), other)
    if unused is not None:
        unused[:] = unexpected
    return where


def load_weights(folder: str, specs: Mapping[str, ParamSpec], mode: torch.dtype, device, strict: bool = True,
                 report: Optional[Dict[str, List[str]]] = None) -> Dict[str, torch.Tensor]:
    """All tensors ``specs`` names that the folder holds, on ``device``, stored by the rule above.  With ``strict``
    False tensors that no part asked for are left alone, logged as a warning and listed in ``report["unused"]``."""
    try:
        files = open_model_files(folder)
    except SafetensorsError as e:
        raise WeightError(folder, [], [], [], [str(e)]) from None
    try:
        unused: List[str] = []
        where = check_against_specs(folder, files, specs, strict, unused)
        if unused:
            log.warn("weights", f"{folder}: {len(unused)} tensors are not used by the model: " + ", ".join(unused[:8])
                     + (" ..." if len(unused) > 8 else ""))
        if report is not None:
            report["unused"] = unused
        out: Dict[str, torch.Tensor] = {}
        for n, s in specs.items():
            if n not in where:
                continue
            src = where[n].tensor(n)
            t = src.to(device=device, dtype=storage_dtype(src.dtype, mode, s.integer)).contiguous()
            if t.data_ptr() == src.data_ptr():
                t = t.clone()  # never hand out memory of the mapping, which is closed below
            out[n] = t
        return out
    finally:
        for f in files:
            f.close()


def tensor_seed(seed: int, name: str) -> int:
    """The generator seed of one tensor: a function of the model seed and the tensor's name, so a
    tensor's values do not depend on which other tensors the model has or on their order."""
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & ((1 << 63) - 1)


def random_tensor(name: str, spec: ParamSpec, seed: int, dtype: torch.dtype, device="cpu") -> torch.Tensor:
    """Random values for one tensor by its spec's rule: N(0, std) rounded to ``dtype``, ones, or zeros."""
    if spec.integer:
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    kind = spec.init[0]
    if kind == "ones":
        return torch.ones(spec.shape, dtype=dtype, device=device)
    if kind == "zeros":
        return torch.zeros(spec.shape, dtype=dtype, device=device)
    if kind == "normal":
        g = torch.Generator(device=device)
        g.manual_seed(tensor_seed(seed, name))
        t = torch.empty(spec.shape, dtype=torch.float32, device=device)
        t.normal_(0.0, float(spec.init[1]), generator=g)
        return t.to(dtype)
    raise ValueError(f"tensor '{name}': unknown init rule {spec.init!r}")


def write_random_model(folder: str, config, seed: int, dtype: torch.dtype = torch.bfloat16,
                       float32_tensors: Iterable[str] = (), include_optional: bool = True, shards: int = 1) -> None:
    """Write ``config.json`` and ``model.safetensors`` with seeded random weights.

    Matrices, tables and biases are N(0, 0.02) and norm weights 1.0, as each part's specs say.
    Tensors named in ``float32_tensors`` (exact names or suffixes) are stored in float32
    instead of ``dtype``.  With ``shards`` > 1 the tensors go into that many files with an index, as large
    checkpoints are laid out; a tensor's values do not depend on the layout.
    """
    from ..engine.model import Model
    specs = Model.param_specs_for(config)
    f32 = tuple(float32_tensors)
    tensors = {}
    for name, spec in specs.items():
        if spec.optional and not include_optional:
            continue
        dt = torch.float32 if any(name == s or name.endswith(s) for s in f32) else dtype
        tensors[name] = random_tensor(name, spec, seed, dt)
    os.makedirs(folder, exist_ok=True)
    config.save(folder)
    meta = {"format": "pt", "seed": str(seed)}
    if shards > 1:
        write_sharded(folder, tensors, shards, meta)
    else:
        write_safetensors(os.path.join(folder, "model.safetensors"), tensors, metadata=meta)
