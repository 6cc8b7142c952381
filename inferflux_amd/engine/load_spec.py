"""What to load and how large to make the engine around it: one typed record that every entry point
(``Engine.load``, the command line, the replay tool, the benchmark) builds and hands to ``load_runner``.

The reference describes a model to load as a ``ModelLoadSpec`` {id, path, format, backend, default, device,
context_size, gpu_layers, max_parallel_sequences, embedding_batch_size, kv_cache_type} with a ``Validate`` that
returns the first complaint as a sentence (model/model_load_spec.h:17-37, model_load_spec.cpp:38-59).  Here
the fields are those this engine has a use for: the folder (or a config.json to make seeded random weights
for), the precision, the cache's shape (context_size x max_parallel_sequences tokens, or kv_pages; page_size)
and the step's limits.  ``format`` is safetensors only and ``backend`` is this engine, so neither is a field;
``kv_cache_type`` follows the precision (the reference rejects its own int8/fp8 as "not implemented yet",
runtime/backends/cuda/inferflux_cuda_executor.cpp:1595-1623).
"""
from __future__ import annotations

import dataclasses
import re
from typing import Any, Mapping, Optional

_DTYPES = {"bfloat16": "bfloat16", "bf16": "bfloat16", "float32": "float32", "fp32": "float32"}


class LoadSpecError(ValueError):
    pass


@dataclasses.dataclass
class ModelLoadSpec:
    path: Optional[str] = None              # folder with config.json and model.safetensors (or its shards)
    random_weights: Optional[str] = None    # instead of ``path``: a config.json whose model gets seeded random weights
    seed: int = 0                           # of the random weights
    dtype: str = "bfloat16"                 # "bfloat16" | "float32" ("bf16" / "fp32" are accepted)
    device: Optional[str] = None            # "rocm:N" or "cuda:N" (the same ordinal); None: the current device
    context_size: int = 4096                # tokens of context per sequence the cache is sized for
    max_parallel_sequences: int = 32        # live requests (state slots, rows of a decode step)
    kv_pages: Optional[int] = None          # pages per cache group; None: context_size * max_parallel_sequences tokens
    page_size: int = 16                     # tokens per page
    max_batch_tokens: int = 16384           # tokens in one step
    chunked_prefill_tokens: int = 512       # largest portion of a prompt in one step beside requests that are decoding
    prefill_tokens_alone: Optional[int] = None   # ... in a step in which nobody decodes (None: the larger of that and 2,048)
    decode_weight_copy: bool = True         # keep the tiled second copy of bfloat16 projections for decoding
    strict_weights: bool = True             # tensors in the file that no part reads are an error (else a warning)
    phase_timing: bool = False              # time every phase of every forward pass
    library_gemm_tuning: bool = False       # let the library time its kernels for every product shape of more than 64 rows it
                                            # meets (prompts: about a quarter faster once a shape is known, up to 0.3 s the first time)

    def validate(self) -> str:
        """The first thing wrong with the spec as a sentence, or "" (the reference's convention)."""
        if bool(self.path) == bool(self.random_weights):
            return "exactly one of path and random_weights must be given"
        if self.dtype not in _DTYPES:
            return "dtype must be bfloat16 or float32"
        if self.device is not None and not re.fullmatch(r"(cuda|rocm):\d+", self.device):
            return "device must be cuda:N or rocm:N"
        if self.context_size <= 0:
            return "context_size must be positive"
        if not 1 <= self.max_parallel_sequences <= 256:
            return "max_parallel_sequences must be between 1 and 256"
        if self.kv_pages is not None and self.kv_pages <= 0:
            return "kv_pages must be positive"
        if self.page_size <= 0:
            return "page_size must be positive"
        if self.max_batch_tokens <= 0:
            return "max_batch_tokens must be positive"
        if self.chunked_prefill_tokens <= 0:
            return "chunked_prefill_tokens must be positive"
        if self.prefill_tokens_alone is not None and self.prefill_tokens_alone <= 0:
            return "prefill_tokens_alone must be positive"
        if self.seed < 0:
            return "seed must be nonnegative"
        return ""

    def checked(self) -> "ModelLoadSpec":
        error = self.validate()
        if error:
            raise LoadSpecError(f"model load spec: {error}")
        return self

    @property
    def torch_dtype(self):
        import torch
        return {"bfloat16": torch.bfloat16, "float32": torch.float32}[_DTYPES[self.dtype]]

    @property
    def device_index(self) -> Optional[int]:
        return None if self.device is None else int(self.device.split(":")[1])

    @property
    def cache_tokens(self) -> int:
        return self.context_size * self.max_parallel_sequences

    @classmethod
    def from_mapping(cls, d: Mapping[str, Any]) -> "ModelLoadSpec":
        """From a mapping of field names (a parsed YAML / JSON entry, or parsed command-line options; dashes and
        underscores are the same).  Unknown keys are an error that names them."""
        known = {f.name for f in dataclasses.fields(cls)}
        given = {str(k).replace("-", "_"): v for k, v in d.items() if v is not None}
        unknown = sorted(set(given) - known)
        if unknown:
            raise LoadSpecError(f"model load spec: unknown keys {unknown}; known: {sorted(known)}")
        return cls(**given).checked()
