"""Loading a model folder into a runner: the one path every entry point takes."""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import load_config
from ..kernels import ops
from .load_spec import ModelLoadSpec
from .model import Model
from .runner import ModelRunner


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU visible: the engine has no CPU path (torch.cuda.is_available() is False)")
    return torch.device("cuda", torch.cuda.current_device())


def load_model(folder, dtype: torch.dtype = torch.bfloat16, device=None, decode_weight_copy: bool = True,
               strict_weights: bool = True) -> Model:
    """The model class is chosen by config.json; weights are read by tensor name.  With
    ``decode_weight_copy`` every bfloat16 projection also keeps the tiled copy that products with few
    rows stream from (twice the weights' memory for about a fifth off a decode step).  ``folder`` may be
    a ``ModelLoadSpec`` (then the other arguments are taken from it, and a spec that names ``random_weights``
    gets them made on the device, seeded, with no folder written)."""
    spec = folder if isinstance(folder, ModelLoadSpec) else ModelLoadSpec(
        path=folder, dtype={torch.bfloat16: "bfloat16", torch.float32: "float32"}[dtype],
        decode_weight_copy=decode_weight_copy, strict_weights=strict_weights)
    spec.checked()
    if isinstance(folder, ModelLoadSpec):
        dtype = spec.torch_dtype
        if spec.device_index is not None:
            device = torch.device("cuda", spec.device_index)
    device = device or require_gpu()
    if dtype == torch.float32:
        # The 32-bit path never uses a reduced-precision matrix mode; the engine's own float32
        # kernels do not consult these switches, they are set for any library call a part makes.
        torch.backends.cuda.matmul.allow_tf32 = False
    before = ops.decode_weight_copy
    ops.decode_weight_copy = bool(spec.decode_weight_copy)
    try:
        if spec.random_weights:
            import json
            from ..config.registry import config_from_dict
            with open(spec.random_weights) as f:
                config = config_from_dict(json.load(f))
            return Model(config).init_random(spec.seed, dtype, device)
        return Model(load_config(spec.path)).load_folder(spec.path, dtype, device, strict=spec.strict_weights)
    finally:
        ops.decode_weight_copy = before


def plan_kv_pages(model: Model, page_size: int, wanted_tokens: int, memory_fraction: float = 0.8) -> int:
    """Pages for ``wanted_tokens`` of cache, cut down to what ``memory_fraction`` of the free device
    memory holds.  bytes per token = 2 * sum over caching layers of kv heads * head size * element
    size, the reference's planner's arithmetic (runtime/backends/cuda/native/kv_cache_planner.h:22-37),
    which gives the cache 20 % of free memory (native_bootstrap_config.h:20); here the weights are
    already resident when this is called, so most of what is left can go to the cache."""
    per_token = 0
    esz = 2 if model.dtype == torch.bfloat16 else 4
    for e, mixer in zip(model.plan.schedule, model.schedule_mixers()):
        spec = mixer.cache_spec()
        if spec is not None and e.cache_from is None:
            per_token += spec.bytes_per_token(esz)
    want = max(1, -(-wanted_tokens // page_size))
    if per_token == 0:
        return want
    free, _ = torch.cuda.mem_get_info(model.device)
    fit = int(free * memory_fraction) // (per_token * page_size)
    if fit < 1:
        raise RuntimeError(f"no device memory left for the cache ({free} bytes free, a page needs {per_token * page_size})")
    return min(want, fit)


def load_runner(folder, dtype: torch.dtype = torch.bfloat16, num_pages: Optional[int] = 256, page_size: int = 16,
                max_requests: int = 64, device=None, cache_tokens: Optional[int] = None,
                phase_timing: bool = False, decode_weight_copy: bool = True) -> ModelRunner:
    """A model with its cache and step function.  ``folder`` is a ``ModelLoadSpec`` (every other argument is then
    taken from it) or a model folder with the arguments given here.  ``num_pages`` None: as many pages as
    ``cache_tokens`` need, within the free device memory."""
    if isinstance(folder, ModelLoadSpec):
        spec = folder.checked()
        if spec.library_gemm_tuning:
            from ..kernels import ops
            ops.enable_library_gemm_tuning()
        model = load_model(spec)
        num_pages = spec.kv_pages
        if num_pages is None:
            num_pages = plan_kv_pages(model, spec.page_size, spec.cache_tokens)
        return ModelRunner(model, num_pages=num_pages, page_size=spec.page_size, max_requests=spec.max_parallel_sequences,
                           phase_timing=spec.phase_timing)
    model = load_model(folder, dtype, device, decode_weight_copy)
    if num_pages is None:
        num_pages = plan_kv_pages(model, page_size, cache_tokens or 4096 * max_requests)
    return ModelRunner(model, num_pages=num_pages, page_size=page_size, max_requests=max_requests,
                       phase_timing=phase_timing)
