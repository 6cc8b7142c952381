"""The chip the kernels are written and tuned for, in one place: what launch shapes, work orders and thresholds
elsewhere in this package are derived from.  Kernels that deal work to the XCDs are given the count as an argument."""
from __future__ import annotations

ARCH = "gfx950"            # MI355X (CDNA4): what every kernel is compiled for
N_XCD = 8                  # accelerator dies, each with an L2 of its own; a launch deals its workgroups to them in turn
CUS_PER_XCD = 32           # compute units per die; a die deals its share of the workgroups to its units in turn
COMPUTE_UNITS = N_XCD * CUS_PER_XCD


def describe(device=None) -> str:
    """What the visible device says of itself beside what the kernels assume (for logs and bug reports)."""
    import torch
    p = torch.cuda.get_device_properties(device if device is not None else torch.cuda.current_device())
    arch = getattr(p, "gcnArchName", "?").split(":")[0]
    note = "" if (arch == ARCH and p.multi_processor_count == COMPUTE_UNITS) else \
        f" (the kernels assume {ARCH} with {COMPUTE_UNITS} compute units in {N_XCD} dies)"
    return f"{p.name}: {arch}, {p.multi_processor_count} compute units{note}"
