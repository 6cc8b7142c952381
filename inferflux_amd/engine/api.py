"""Loading a model folder into a runner: the one path every entry point takes."""
from __future__ import annotations

import torch

from ..config.registry import load_config
from .model import Model
from .runner import ModelRunner


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU visible: the engine has no CPU path (torch.cuda.is_available() is False)")
    return torch.device("cuda", torch.cuda.current_device())


def load_model(folder: str, dtype: torch.dtype = torch.bfloat16, device=None) -> Model:
    """The model class is chosen by config.json; weights are read by tensor name."""
    device = device or require_gpu()
    if dtype == torch.float32:
        # The 32-bit path never uses a reduced-precision matrix mode; the engine's own float32
        # kernels do not consult these switches, they are set for any library call a part makes.
        torch.backends.cuda.matmul.allow_tf32 = False
    config = load_config(folder)
    return Model(config).load_folder(folder, dtype, device)


def load_runner(folder: str, dtype: torch.dtype = torch.bfloat16, num_pages: int = 256, page_size: int = 16,
                max_requests: int = 64, device=None) -> ModelRunner:
    return ModelRunner(load_model(folder, dtype, device), num_pages=num_pages, page_size=page_size,
                       max_requests=max_requests)
