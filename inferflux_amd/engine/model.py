"""The generic model: parts built from a plan, weights bound by name, one forward over a step.

Nothing here is specific to an architecture.  The plan says which parts make each layer and
in which order layers run; the model builds them, collects the tensors they declare, hands
each part its tensors, and runs a step's rows through embedding, the scheduled layers, the
final norm on the wanted rows and the head.
"""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional

import torch

from .. import architectures  # noqa: F401  (registers the known architectures)
from .. import parts as _parts  # noqa: F401  (registers the built-in parts)
from ..config.registry import plan_for
from ..parts.base import build_part
from ..parts.block import normed_for
from ..parts.plan import ModelPlan, ParamSpec
from ..weights.loader import load_weights, random_tensor


def _walk(part):
    yield part
    for c in part.children():
        yield from _walk(c)


class Model:
    def __init__(self, config=None, plan: Optional[ModelPlan] = None):
        if plan is None:
            plan = plan_for(config)
        plan.validate()
        self.config, self.plan = config, plan
        H = plan.hidden_size
        self.embedding = build_part("embedding", plan.embedding, hidden_size=H)
        self.blocks = [build_part("block", l.block, layer=l, hidden_size=H) for l in plan.layers]
        self.final_norm = build_part("norm", plan.final_norm, hidden_size=H)
        self.head = build_part("head", plan.lm_head, hidden_size=H)
        self.dtype: Optional[torch.dtype] = None
        self.device = None

    # ---- structure ----------------------------------------------------------------
    def parts(self):
        yield from _walk(self.embedding)
        for b in self.blocks:
            yield from _walk(b)
        yield from _walk(self.final_norm)
        yield from _walk(self.head)

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in self.parts())

    def schedule_mixers(self) -> List:
        return [self.blocks[e.layer].mixer for e in self.plan.schedule]

    def param_specs(self) -> Dict[str, ParamSpec]:
        out: Dict[str, ParamSpec] = {}
        for p in self.parts():
            for n, s in p.param_specs().items():
                if n in out and out[n] != s:
                    raise ValueError(f"tensor '{n}' is declared twice with different specs")
                out[n] = s
        return out

    @staticmethod
    def param_specs_for(config) -> Dict[str, ParamSpec]:
        return Model(config).param_specs()

    # ---- weights ------------------------------------------------------------------
    def bind(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device) -> "Model":
        for p in self.parts():
            p.load(tensors)
        self.dtype, self.device = dtype, torch.device(device)
        return self

    def load_folder(self, folder: str, dtype: torch.dtype, device, strict: bool = True) -> "Model":
        return self.bind(load_weights(folder, self.param_specs(), dtype, device, strict=strict), dtype, device)

    def init_random(self, seed: int, dtype: torch.dtype, device, on_host: Optional[bool] = None) -> "Model":
        """Random weights without a folder.  Values follow each spec's rule, rounded to bfloat16 in both modes
        so the two modes see the same numbers.  ``on_host`` True draws them with the host's generator, tensor by
        tensor, which gives exactly the values ``write_random_model`` writes for the same seed; False draws them
        on the device (another stream of numbers, but no minutes of waiting for billions of weights).  None: on
        the host for models of up to 2**28 weights."""
        import math
        specs = self.param_specs()
        if on_host is None:
            on_host = sum(math.prod(s.shape) for s in specs.values()) <= (1 << 28)
        tensors = {}
        for n, s in specs.items():
            t = random_tensor(n, s, seed, torch.bfloat16, device="cpu" if on_host else device).to(device)
            tensors[n] = t if (dtype == torch.bfloat16 or s.integer) else t.float()
        return self.bind(tensors, dtype, device)

    # ---- forward ------------------------------------------------------------------
    def forward(self, ctx, storage) -> torch.Tensor:
        """float32 logits [len(ctx.logit_rows), vocab] for the step ``ctx`` describes."""
        t = ctx.timer
        if t is not None:
            t.begin()
            t.enter("embed")
        schedule = self.plan.schedule
        pending = None
        first_norm = self.blocks[schedule[0].layer].entry_norm() if schedule else None
        if first_norm is not None and getattr(self.embedding, "prepares_norm_rows", False):
            residual = self.embedding.forward(ctx, norm=first_norm)     # (an embedding that can do so prepares the first norm's rows)
            if isinstance(residual, tuple):
                residual, pending = residual
        else:
            residual = self.embedding.forward(ctx)
        if t is not None:
            t.mark("embed")
        for i, e in enumerate(schedule):
            block = self.blocks[e.layer]
            # a block that can hand on rows prepared for the next block's first norm is told that norm
            if i + 1 < len(schedule):
                following = self.blocks[schedule[i + 1].layer].entry_norm()
            else:       # the last block may prepare the final norm's rows where the head takes every row of the step
                following = self.final_norm if ctx.all_rows_wanted else None
            if following is not None and block.entry_norm() is not None:
                residual, pending = block.forward(residual, pending, ctx, storage.binding(i), following=following)
            else:
                residual, pending = block.forward(residual, pending, ctx, storage.binding(i))
        if ctx.n_logit_rows == 0:
            logits = torch.empty((0, self.plan.vocab_size), dtype=torch.float32, device=residual.device)
        else:
            if t is not None:
                t.enter("final_norm")
            if ctx.all_rows_wanted:
                h = normed_for(self.final_norm, self.head, residual, pending, ctx)
            else:
                h = self.final_norm.forward(residual, pending, ctx.act_dtype, rows=ctx.logit_rows)
            if t is not None:
                t.mark("final_norm")
                t.enter("lm_head")
            logits = self.head.forward(h)
            if t is not None:
                t.mark("lm_head")
        if t is not None:
            t.end(len(self.plan.schedule), ctx.n_tokens)
        return logits
