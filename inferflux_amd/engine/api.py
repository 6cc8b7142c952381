"""Loading a model folder into a runner: the one path every entry point takes."""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import load_config
from ..kernels import ops
from .model import Model
from .runner import ModelRunner


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU visible: the engine has no CPU path (torch.cuda.is_available() is False)")
    return torch.device("cuda", torch.cuda.current_device())


def load_model(folder: str, dtype: torch.dtype = torch.bfloat16, device=None, decode_weight_copy: bool = True) -> Model:
    """The model class is chosen by config.json; weights are read by tensor name.  With
    ``decode_weight_copy`` every bfloat16 projection also keeps the tiled copy that products with few
    rows stream from (twice the weights' memory for about a fifth off a decode step)."""
    device = device or require_gpu()
    if dtype == torch.float32:
        # The 32-bit path never uses a reduced-precision matrix mode; the engine's own float32
        # kernels do not consult these switches, they are set for any library call a part makes.
        torch.backends.cuda.matmul.allow_tf32 = False
    config = load_config(folder)
    before = ops.decode_weight_copy
    ops.decode_weight_copy = bool(decode_weight_copy)
    try:
        return Model(config).load_folder(folder, dtype, device)
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
            per_token += 2 * spec.n_kv_heads * spec.head_dim * esz
    want = max(1, -(-wanted_tokens // page_size))
    if per_token == 0:
        return want
    free, _ = torch.cuda.mem_get_info(model.device)
    fit = int(free * memory_fraction) // (per_token * page_size)
    if fit < 1:
        raise RuntimeError(f"no device memory left for the cache ({free} bytes free, a page needs {per_token * page_size})")
    return min(want, fit)


def load_runner(folder: str, dtype: torch.dtype = torch.bfloat16, num_pages: Optional[int] = 256, page_size: int = 16,
                max_requests: int = 64, device=None, cache_tokens: Optional[int] = None,
                phase_timing: bool = False, decode_weight_copy: bool = True) -> ModelRunner:
    """``num_pages`` None: as many pages as ``cache_tokens`` need, within the free device memory."""
    model = load_model(folder, dtype, device, decode_weight_copy)
    if num_pages is None:
        num_pages = plan_kv_pages(model, page_size, cache_tokens or 4096 * max_requests)
    return ModelRunner(model, num_pages=num_pages, page_size=page_size, max_requests=max_requests,
                       phase_timing=phase_timing)
