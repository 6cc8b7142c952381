"""Reading and writing the safetensors container.

Format, as the reference parses it (runtime/backends/cuda/native/safetensors_parser.cpp:144-259):
an 8-byte little-endian header length, a JSON header mapping tensor names to ``dtype``,
``shape`` and ``data_offsets`` (relative to the end of the header; keys starting with "__" are
metadata), then the raw little-endian data.  The reference only warns when a tensor's byte
count disagrees with its shape and type (safetensors_parser.cpp:279-299); here that, a tensor
reaching past the end of the file and a malformed header are errors that name the tensor.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, List, Mapping, Tuple

import torch


class SafetensorsError(ValueError):
    pass


_DTYPES = {
    "F64": (torch.float64, 8), "F32": (torch.float32, 4), "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}
MAX_HEADER = 100 * 1024 * 1024


class SafetensorsFile:
    """One memory-mapped .safetensors file; tensors are views of the mapping until copied."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too short to hold a header length")
        self._f = open(path, "rb")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        (hlen,) = struct.unpack("<Q", self._mm[:8])
        if hlen > MAX_HEADER or 8 + hlen > size:
            raise SafetensorsError(f"{path}: header length {hlen} exceeds the file ({size} bytes) or {MAX_HEADER}")
        try:
            header = json.loads(self._mm[8:8 + hlen].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON: {e}") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header must be a JSON object")
        self.data_start = 8 + hlen
        self.entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        for name, meta in header.items():
            if name.startswith("__"):
                continue
            try:
                dt, shape, (b, e) = meta["dtype"], tuple(int(s) for s in meta["shape"]), meta["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{path}: tensor '{name}' has a malformed header entry") from None
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor '{name}' has unsupported dtype {dt}")
            tdt, isz = _DTYPES[dt]
            numel = 1
            for s in shape:
                numel *= s
            if e - b != numel * isz or b < 0:
                raise SafetensorsError(
                    f"{path}: tensor '{name}' holds {e - b} bytes but shape {list(shape)} of {dt} needs {numel * isz}")
            if self.data_start + e > size:
                raise SafetensorsError(f"{path}: tensor '{name}' reaches past the end of the file (truncated?)")
            self.entries[name] = (tdt, shape, b, e)
        # No two tensors may share bytes: a header whose ranges overlap is not something a writer produces.
        last_end, last_name = 0, None
        for name, (_, _, b, e) in sorted(self.entries.items(), key=lambda kv: (kv[1][2], kv[1][3])):
            if e > b:
                if b < last_end:
                    raise SafetensorsError(f"{path}: tensors '{last_name}' and '{name}' overlap in the file")
                last_end, last_name = e, name

    def names(self) -> List[str]:
        return list(self.entries)

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.entries[name][1]

    def dtype(self, name: str) -> torch.dtype:
        return self.entries[name][0]

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that aliases the mapping (read-only memory: copy before writing to it)."""
        tdt, shape, b, e = self.entries[name]
        if e == b:
            return torch.empty(shape, dtype=tdt)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # torch warns that the mapping is not writable
            flat = torch.frombuffer(self._mm, dtype=tdt, count=(e - b) // _DTYPES[_NAMES[tdt]][1],
                                    offset=self.data_start + b)
        return flat.view(shape)

    def close(self) -> None:
        try:
            self._mm.close()
        except BufferError:
            pass  # tensors still alias the mapping; it is released with them
        self._f.close()


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor], metadata: Mapping[str, str] = None) -> None:
    """Write ``tensors`` (CPU, any listed dtype) in name order; the header is padded to 8 bytes."""
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor '{name}': dtype {t.dtype} cannot be stored")
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + n]}
        offset += n
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = f"{path}.tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().contiguous().cpu()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    os.replace(tmp, path)


def open_model_files(folder: str) -> List[SafetensorsFile]:
    """The safetensors files of a model folder: those an index names, else model.safetensors
    (the reference's rule: runtime/backends/cuda/inferflux_cuda_executor.cpp:366-402)."""
    index = os.path.join(folder, "model.safetensors.index.json")
    if os.path.isfile(index):
        try:
            with open(index) as f:
                wm = json.load(f)["weight_map"]
            shards = sorted(set(wm.values()))
        except (json.JSONDecodeError, KeyError, AttributeError, TypeError) as e:
            raise SafetensorsError(f"{index}: not a safetensors index ({e})") from None
        if not shards:
            raise SafetensorsError(f"{index}: the weight map names no files")
        root = os.path.realpath(folder)
        for s in shards:
            inside = isinstance(s, str) and s and not os.path.isabs(s) and \
                os.path.commonpath([root, os.path.realpath(os.path.join(root, s))]) == root
            if not inside:
                raise SafetensorsError(f"{index}: shard name {s!r} does not stay inside the model folder")
        missing = [s for s in shards if not os.path.isfile(os.path.join(folder, s))]
        if missing:
            raise SafetensorsError(f"{index} names shard files that do not exist: {missing}")
        return [SafetensorsFile(os.path.join(folder, s)) for s in shards]
    single = os.path.join(folder, "model.safetensors")
    if os.path.isfile(single):
        return [SafetensorsFile(single)]
    raise SafetensorsError(f"{folder}: no safetensors files found (model.safetensors or model.safetensors.index.json)")


def write_sharded(folder: str, tensors: Mapping[str, torch.Tensor], n_shards: int, metadata: Mapping[str, str] = None) -> List[str]:
    """Write ``tensors`` as ``n_shards`` files ``model-0000i-of-0000n.safetensors`` (names dealt out in sorted order, by
    bytes) plus ``model.safetensors.index.json``, the layout of large checkpoints; returns the shard names."""
    if n_shards < 1:
        raise SafetensorsError("a model needs at least one shard")
    names = sorted(tensors)
    total = sum(tensors[n].numel() * tensors[n].element_size() for n in names)
    shards: List[Dict[str, torch.Tensor]] = [{} for _ in range(n_shards)]
    seen = 0
    for n in names:
        shards[min(n_shards - 1, seen * n_shards // max(total, 1))][n] = tensors[n]
        seen += tensors[n].numel() * tensors[n].element_size()
    files, weight_map = [], {}
    for i, part in enumerate(shards):
        fn = f"model-{i + 1:05d}-of-{n_shards:05d}.safetensors"
        write_safetensors(os.path.join(folder, fn), part, metadata)
        files.append(fn)
        for n in part:
            weight_map[n] = fn
    tmp = os.path.join(folder, "model.safetensors.index.json.tmp")
    with open(tmp, "w") as f:
        json.dump({"metadata": {"total_size": total}, "weight_map": weight_map}, f, indent=1)
    os.replace(tmp, os.path.join(folder, "model.safetensors.index.json"))
    return files
