"""Host-side helpers of the optimizer step (counterpart of lit_gpt/optim/opt_utils.py).

On one GPU the reference's generator-based AsyncRuntime degenerates into a Python loop
over parameters; here parameters are grouped into shape classes and each class is one
batched launch, so no task runtime is needed.  What is kept is the grouping rule and the
DTensor unwrapping.
"""
from __future__ import annotations

from collections import defaultdict
from typing import Generator, List, Sequence, Union

import torch
from torch import Tensor

try:  # DTensor is optional at import time (CPU-only wheels ship it, but keep the guard cheap)
    from torch.distributed.tensor import DTensor
except Exception:  # pragma: no cover
    DTensor = ()  # type: ignore[assignment]


def to_local(tensor: Union[Tensor, Sequence[Tensor]]):
    """Local shard(s) of DTensor(s); identity for plain tensors (opt_utils.py:13-20 of the reference)."""
    if isinstance(tensor, Tensor):
        return tensor.to_local() if DTensor and isinstance(tensor, DTensor) else tensor
    return [t.to_local() if DTensor and isinstance(t, DTensor) else t for t in tensor]


def create_param_batches(params: List[Tensor], batch_size: int) -> Generator[List[Tensor], None, None]:
    """Batches of at most ``batch_size`` parameters that share shape, sharding and dtype, in first-seen
    order of the key (opt_utils.py:53-70 of the reference)."""
    if batch_size <= 0:
        raise ValueError(f"{batch_size=} cannot be <= 0")
    buckets = defaultdict(list)
    for p in params:
        placements = p.placements if DTensor and isinstance(p, DTensor) else None
        buckets[(p.shape, placements, p.dtype)].append(p)
    for same in buckets.values():
        for start in range(0, len(same), batch_size):
            yield same[start:start + batch_size]


def matrix_view_shape(shape: Sequence[int], flatten: bool):
    """(n_matrices, rows, cols) a parameter of ``shape`` is orthogonalised as: with ``flatten`` a 3-D+
    tensor is ONE matrix (d0, prod(rest)); otherwise leading dimensions are a batch of matrices
    (muon.py:830-836 of the reference)."""
    if len(shape) < 2:
        raise ValueError("Muon optimizer only supports matrix parameters.")
    if flatten and len(shape) >= 3:
        rest = 1
        for d in shape[1:]:
            rest *= d
        return 1, shape[0], rest
    lead = 1
    for d in shape[:-2]:
        lead *= d
    return lead, shape[-2], shape[-1]
