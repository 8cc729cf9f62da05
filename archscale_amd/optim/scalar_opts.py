"""AdamW / hyperball-AdamW / Lion for the non-matrix parameter groups of ``Muon`` on MI355X.

Counterpart of lit_gpt/optim/scalar_opts.py: the reference runs these groups (embeddings, norms, lm_head) as
compiled ``torch._foreach`` graphs; here each group is ONE multi-tensor HIP launch (three for the hyperball
variant: update moments + reduce norms, per-tensor coefficients, apply) through ``muon_scalar_update``.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import numpy as np
import torch
from torch import Tensor

from .. import _lib


class _ScalarPlan:
    """Device item table of one list of parameters (uploaded again only when a data pointer changes)."""

    def __init__(self, n: int, numels: List[int], device: torch.device, hyperball: bool):
        from .muon import _DeviceTable  # local import: muon imports this module
        chunk = _lib.CHUNK_ELEMS
        self.items = np.zeros(n, dtype=_lib.SCALAR_ITEM)
        prefix = np.zeros(n + 1, dtype=np.int32)
        for i, ne in enumerate(numels):
            prefix[i + 1] = prefix[i] + (ne + chunk - 1) // chunk
        self.chunks = int(prefix[-1])
        self.table = _DeviceTable(self.items.nbytes, device)
        self.prefix_dev = torch.from_numpy(prefix).to(device)
        n_scratch = _lib.lib().muon_muonh_scratch_floats(n, self.chunks) if hyperball else 0
        self.scratch = torch.empty(max(n_scratch, 1), dtype=torch.float32, device=device)
        self.sig: Optional[Tuple] = None

    def refresh(self, X, G, M, V) -> None:
        sig = tuple((x.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr() if v is not None else 0)
                    for x, g, m, v in zip(X, G, M, V))
        if sig == self.sig:
            return
        for row, x, g, m, v in zip(self.items, X, G, M, V):
            row["w"], row["g"], row["m"] = x.data_ptr(), g.data_ptr(), m.data_ptr()
            row["v"] = v.data_ptr() if v is not None else 0
            row["numel"] = x.numel()
            row["w_dtype"], row["g_dtype"] = _lib.dtype_code(x.dtype), _lib.dtype_code(g.dtype)
            row["m_dtype"] = _lib.dtype_code(m.dtype)
            row["v_dtype"] = _lib.dtype_code(v.dtype) if v is not None else 0
        self.table.upload(self.items)
        self.sig = sig


#: plans of calls made without an owner's cache (direct use of the functions below)
_plans: Dict[Tuple, _ScalarPlan] = {}


def _run(cache, key, algo: int, hyperball: bool, X: List[Tensor], G: List[Tensor], M: List[Tensor], V, lr: float, beta1: float,
         beta2: float, weight_decay: float, step: int, epsilon: float, cautious_wd: bool,
         hyper_dev: Optional[int] = None) -> None:
    if not X:
        return
    device = X[0].device
    V = V if V is not None else [None] * len(X)
    for t in (*X, *G, *M, *(v for v in V if v is not None)):
        _lib.require_cuda(t, "an optimizer tensor")
        if t.device != device:
            raise ValueError("all tensors of a parameter group must live on one device")
        if not t.is_contiguous():
            raise ValueError("parameters, gradients and optimizer state must be contiguous")
    struct = (key, algo, hyperball, tuple((tuple(x.shape), x.dtype, g.dtype, m.dtype) for x, g, m in zip(X, G, M)))
    cache = _plans if cache is None else cache
    plan = cache.get(struct)
    if plan is None:
        plan = _ScalarPlan(len(X), [x.numel() for x in X], device, hyperball)
        cache[struct] = plan
    with torch.cuda.device(device):
        plan.refresh(X, G, M, V)
        if hyper_dev is not None:   # hyper-parameters from a muon_hyper block in device memory (a captured step)
            st = _lib.lib().muon_scalar_update_dev(
                plan.table.dev.data_ptr(), plan.prefix_dev.data_ptr(), len(X), plan.chunks, algo, int(hyperball),
                hyper_dev, plan.scratch.data_ptr() if hyperball else 0, _lib.current_stream_ptr(device))
            _lib.check(st, "muon_scalar_update_dev")
            return
        st = _lib.lib().muon_scalar_update(
            plan.table.dev.data_ptr(), plan.prefix_dev.data_ptr(), len(X), plan.chunks, algo, int(hyperball),
            lr, beta1, beta2, lr * weight_decay, epsilon, max(int(step), 1), int(cautious_wd),
            plan.scratch.data_ptr() if hyperball else 0, _lib.current_stream_ptr(device))
    _lib.check(st, "muon_scalar_update")


def adamw_update_foreach(X, G, M, V, lr, beta1, beta2, weight_decay, step, epsilon, cautious_wd=False, *, key=None, cache=None,
                         hyper_dev=None):
    """AdamW with bias correction over a list of tensors (scalar_opts.py:118-198 of the reference)."""
    _run(cache, key or tuple(id(x) for x in X), _lib.ALGO_ADAMW, False, X, G, M, V, lr, beta1, beta2, weight_decay, step,
         epsilon, cautious_wd, hyper_dev)


def hyperball_adamw_update_foreach(X, G, M, V, lr, beta1, beta2, weight_decay, step, epsilon, cautious_wd=False, *,
                                   key=None, cache=None, hyper_dev=None):
    """Adam direction applied on the hypersphere, per tensor (scalar_opts.py:254-377, 396-437 of the reference)."""
    _run(cache, key or tuple(id(x) for x in X), _lib.ALGO_ADAMW, True, X, G, M, V, lr, beta1, beta2, weight_decay, step,
         epsilon, cautious_wd, hyper_dev)


def lion_update_foreach(X, G, M, lr, beta1, beta2, weight_decay, cautious_wd=False, *, key=None, cache=None, hyper_dev=None):
    """Lion over a list of tensors (scalar_opts.py:201-251 of the reference)."""
    _run(cache, key or tuple(id(x) for x in X), _lib.ALGO_LION, False, X, G, M, None, lr, beta1, beta2, weight_decay, 1, 0.0,
         cautious_wd, hyper_dev)


def release_plans() -> None:
    _plans.clear()
