"""Base class of the orthogonalized optimizers on MI355X
(counterpart of emerging_optimizers/orthogonalized_optimizers/orthogonalized_optimizer.py:62-270).

Per step and parameter the reference does: weight decay -> EMA momentum -> optional Nesterov blend ->
``orthogonalize`` -> ``p.add_(update, alpha=-lr)``, in a Python loop of eager ops.  Here the momentum of
all parameters is one multi-tensor HIP launch; when the subclass declares a batched Newton-Schulz recipe
(``_batched_recipe``) the orthogonalisation is one batched call per shape class and the weight update is
one more multi-tensor launch.  A user ``scaled_orthogonalize_fn`` or an overridden ``orthogonalize`` is
still honoured per parameter.
"""
from __future__ import annotations

import logging
from typing import Any, Callable, Dict, List, Optional, Tuple

import numpy as np
import torch
import torch.optim as optim
from torch.optim.optimizer import ParamsT

from .. import _lib
from ..optim import newton_schulz_hip as ns
from ..optim.muon import _DeviceTable
from ..optim.opt_utils import to_local
from .mixin import WeightDecayMixin, WeightDecayT, weight_decay_terms

_log = logging.getLogger(__name__)


class _Plan:
    """Device tables of one param group: momentum items for every parameter, update items for the batched path."""

    def __init__(self, params: List[torch.Tensor], grads: List[torch.Tensor], ratios: Optional[List[float]],
                 device: torch.device, fused: bool = False):
        self.params = params
        self.device = device
        self.fused = fused
        chunk = _lib.CHUNK_ELEMS
        n = len(params)
        self.classes: Dict[Tuple[int, ...], List[int]] = {}  # keyed by the full parameter shape
        for i, p in enumerate(params):
            self.classes.setdefault(tuple(p.shape), []).append(i)
        # U (fp32: the matrix sign normalises in fp32 before rounding) and O (bf16) per shape class; the fused
        # momentum + Newton-Schulz call never materialises U
        self.U: Dict[Tuple[int, ...], torch.Tensor] = {}
        self.O: Dict[Tuple[int, ...], torch.Tensor] = {}
        self.slot: List[Tuple[Tuple[int, ...], int]] = [((0, 0), 0)] * n
        for key, idx in self.classes.items():
            if not fused:
                self.U[key] = torch.empty((len(idx), *key), dtype=torch.float32, device=device)
            self.O[key] = torch.empty((len(idx), *key), dtype=torch.bfloat16, device=device)
            for k, i in enumerate(idx):
                self.slot[i] = (key, k)
        self.pre = np.zeros(n, dtype=_lib.PRE_ITEM)
        self.post = np.zeros(n, dtype=_lib.POST_ITEM)
        self.prefix = np.zeros(n + 1, dtype=np.int32)
        for i, p in enumerate(params):
            self.prefix[i + 1] = self.prefix[i] + (p.numel() + chunk - 1) // chunk
        self.chunks = int(self.prefix[-1])
        self.ratios = ratios
        self.pre_tab = _DeviceTable(self.pre.nbytes, device)
        self.post_tab = _DeviceTable(self.post.nbytes, device)
        self.prefix_dev = torch.from_numpy(self.prefix).to(device)
        self.sig: Optional[Tuple] = None
        self.fused_probs = None
        self.fused_keep: List = []

    @staticmethod
    def can_fuse(params: List[torch.Tensor], grads: List[torch.Tensor], bufs: List[torch.Tensor]) -> bool:
        """One (gradient, buffer, parameter) dtype triple per shape class, as the fused call takes them."""
        seen: Dict[Tuple[int, ...], Tuple] = {}
        for p, g, m in zip(params, grads, bufs):
            if seen.setdefault(tuple(p.shape), (g.dtype, m.dtype, p.dtype)) != (g.dtype, m.dtype, p.dtype):
                return False
        return True

    def refresh(self, grads: List[torch.Tensor], bufs: List[torch.Tensor]) -> None:
        sig = tuple((p.data_ptr(), g.data_ptr(), m.data_ptr()) for p, g, m in zip(self.params, grads, bufs))
        if sig == self.sig:
            return
        for i, (p, g, m) in enumerate(zip(self.params, grads, bufs)):
            key, k = self.slot[i]
            pre, post = self.pre[i], self.post[i]
            if not self.fused:
                pre["g"], pre["m"], pre["w"] = g.data_ptr(), m.data_ptr(), p.data_ptr()
                pre["u"] = self.U[key][k].data_ptr()
                pre["numel"] = p.numel()
                pre["g_dtype"], pre["m_dtype"] = _lib.dtype_code(g.dtype), _lib.dtype_code(m.dtype)
                pre["u_dtype"], pre["w_dtype"] = _lib.DTYPE_F32, _lib.dtype_code(p.dtype)
            post["w"], post["u"] = p.data_ptr(), self.O[key][k].data_ptr()
            post["numel"], post["w_dtype"] = p.numel(), _lib.dtype_code(p.dtype)
            post["lr_ratio"] = self.ratios[i] if self.ratios is not None else 1.0
        if not self.fused:
            self.pre_tab.upload(self.pre)
        self.post_tab.upload(self.post)
        self.sig = sig
        if self.fused:
            self._build_fused(grads, bufs)

    def _build_fused(self, grads: List[torch.Tensor], bufs: List[torch.Tensor]) -> None:
        """muon_mns_problem array: per shape class the (g, m, w) pointers of its matrices in the order of its O buffer."""
        import ctypes
        probs = (_lib.MnsProblem * len(self.classes))()
        keep = []
        for q, (key, idx) in zip(probs, self.classes.items()):
            cols = [[t[i].data_ptr() for i in idx] for t in (grads, bufs, self.params)]
            arrs = [(ctypes.c_void_p * len(idx))(*c) for c in cols]
            keep.append(arrs)
            q.g_ptrs, q.m_ptrs, q.w_ptrs = (ctypes.cast(a, ctypes.POINTER(ctypes.c_void_p)) for a in arrs)
            q.out, q.out_batch_stride, q.out_ld = self.O[key].data_ptr(), key[0] * key[1], key[1]
            i0 = idx[0]
            q.g_dtype, q.m_dtype = _lib.dtype_code(grads[i0].dtype), _lib.dtype_code(bufs[i0].dtype)
            q.w_dtype = _lib.dtype_code(self.params[i0].dtype)
            q.batch, q.rows, q.cols = len(idx), key[0], key[1]
        self.fused_probs, self.fused_keep = probs, keep


class OrthogonalizedOptimizer(WeightDecayMixin, optim.Optimizer):
    """Momentum SGD whose update is orthogonalised.

    Args: params, lr, momentum_beta, weight_decay, use_nesterov, weight_decay_method, fp32_matmul_prec,
    scaled_orthogonalize_fn, log_per_module_update_rms, log_per_module_grad_rms, **kwargs (stored in the
    param-group defaults) - as orthogonalized_optimizer.py:109-144 of the reference.  ``fp32_matmul_prec``
    is kept for signature compatibility; the HIP kernels always multiply bf16 with fp32 accumulation.
    """

    def __init__(
        self,
        params: ParamsT,
        lr: float,
        momentum_beta: float,
        weight_decay: float,
        *,
        use_nesterov: bool,
        weight_decay_method: WeightDecayT,
        fp32_matmul_prec: str,
        scaled_orthogonalize_fn: Callable | None = None,
        log_per_module_update_rms: bool = False,
        log_per_module_grad_rms: bool = False,
        **kwargs: Any,
    ):
        if scaled_orthogonalize_fn is None:
            _log.warning("scaled_orthogonalize_fn not provided. Using noop")
            scaled_orthogonalize_fn = torch.nn.Identity()
        self.fp32_matmul_prec = fp32_matmul_prec
        self.use_nesterov = use_nesterov
        self.weight_decay_method = weight_decay_method
        self.log_per_module_update_rms = log_per_module_update_rms
        self.per_module_update_rms: Dict[str, float] = {}
        self.log_per_module_grad_rms = log_per_module_grad_rms
        self.per_module_grad_rms: Dict[str, float] = {}
        super().__init__(params, dict(lr=lr, momentum_beta=momentum_beta, weight_decay=weight_decay, **kwargs))
        self.scaled_orthogonalize_fn = scaled_orthogonalize_fn
        #: batched path only: momentum and Newton-Schulz in one library call that never stores the blended
        #: momentum (its bf16 rounding goes straight into the operand of the iteration)
        self.fuse_momentum = True
        self._plans: Dict[int, Tuple[Tuple, _Plan]] = {}

    # A subclass whose update is "Newton-Schulz with a coefficient table, times a per-shape scale" returns
    # (coefficient rows, eps, eps_mode, precision, scale(rows, cols)) here to get the batched path.
    def _batched_recipe(self, group: dict):
        return None

    def _uses_default_orthogonalize(self) -> bool:
        return type(self).orthogonalize is OrthogonalizedOptimizer.orthogonalize

    @torch.no_grad()
    def step(self, closure: Callable[[], float] | None = None) -> float | None:
        loss = None if closure is None else closure()
        if self.log_per_module_update_rms:
            self.per_module_update_rms.clear()
        if self.log_per_module_grad_rms:
            self.per_module_grad_rms.clear()

        for gi, group in enumerate(self.param_groups):
            params, grads, bufs = [], [], []
            for p in group["params"]:
                if p.dim() == 1:
                    raise ValueError(f"{self.__class__.__name__} does not support 1D parameters")
                if p.grad is None:
                    continue
                state = self.state[p]
                if "momentum_buffer" not in state:
                    state["momentum_buffer"] = torch.zeros_like(p.grad)
                params.append(p)
                grads.append(p.grad)
                bufs.append(state["momentum_buffer"])
            if params:
                self._group_step(gi, group, params, to_local(params), to_local(grads), to_local(bufs))
        return loss

    def _group_step(self, gi, group, params, local, grads, bufs) -> None:
        device = local[0].device
        for t in (*local, *grads, *bufs):
            _lib.require_cuda(t, "an optimizer tensor")
            if not t.is_contiguous():
                raise ValueError("parameters, gradients and momentum buffers must be contiguous")
        lr, beta = float(group["lr"]), float(group["momentum_beta"])
        wd = group.get("wd_mult", 1.0) * group["weight_decay"]
        lr_wd, l2 = weight_decay_terms(self.weight_decay_method, lr, wd)
        recipe = self._batched_recipe(group)
        logging_on = self.log_per_module_update_rms or self.log_per_module_grad_rms
        batched = (recipe is not None and self._uses_default_orthogonalize() and not logging_on
                   and all(t.ndim == 2 for t in local))
        ratios = [recipe[4](t.shape[-2], t.shape[-1]) for t in local] if batched else None
        fused = batched and self.fuse_momentum and _Plan.can_fuse(local, grads, bufs)

        sig = (tuple((id(p), tuple(t.shape), t.dtype, g.dtype) for p, t, g in zip(params, local, grads)), batched,
               tuple(ratios) if ratios else None, fused)
        cached = self._plans.get(gi)
        if cached is None or cached[0] != sig:
            plan = _Plan(local, grads, ratios, device, fused)
            self._plans[gi] = (sig, plan)
        else:
            plan = cached[1]
            plan.params = local

        L = _lib.lib()
        with torch.cuda.device(device):
            plan.refresh(grads, bufs)
            stream = _lib.current_stream_ptr(device)
            # grad (+= wd*p for l2);  buf <- lerp(buf, grad, 1-beta);  U = lerp(grad, buf, beta) | buf
            um, ug = (beta, 1.0 - beta) if self.use_nesterov else (1.0, 0.0)
            if fused:
                coeffs, eps, eps_mode, prec, _ = recipe
                pm = ns._PREC[prec]
                em = _lib.EPS_CLAMP if eps_mode == "clamp" else _lib.EPS_ADD
                need = sum(L.muon_ns_workspace_bytes(q.batch, q.rows, q.cols, pm) for q in plan.fused_probs)
                ws = _lib.workspace(device, need)
                _lib.check(L.muon_momentum_ns_grouped(plan.fused_probs, len(plan.fused_probs), beta, 1.0 - beta, um, ug, l2,
                                                      _lib.abc_array(coeffs), len(coeffs), eps, em, pm,
                                                      _lib.ns_bsplit_tail(ns.BSPLIT_TAIL), ws.data_ptr(), ws.numel(),
                                                      stream), "muon_momentum_ns_grouped")
                _lib.check(L.muon_update_plain(plan.post_tab.dev.data_ptr(), plan.prefix_dev.data_ptr(), len(local),
                                               plan.chunks, lr, lr_wd, 0, stream), "muon_update_plain")
                return
            _lib.check(L.muon_momentum(plan.pre_tab.dev.data_ptr(), plan.prefix_dev.data_ptr(), len(local),
                                       plan.chunks, beta, 1.0 - beta, um, ug, l2, stream), "muon_momentum")
            if batched:
                coeffs, eps, eps_mode, prec, _ = recipe
                for key in plan.classes:
                    ns.newton_schulz(plan.U[key], coeffs, eps, eps_mode=eps_mode, prec=prec, cast_input_first=False,
                                     out=plan.O[key], bsplit_tail=ns.BSPLIT_TAIL)
                _lib.check(L.muon_update_plain(plan.post_tab.dev.data_ptr(), plan.prefix_dev.data_ptr(), len(local),
                                               plan.chunks, lr, lr_wd, 0, stream), "muon_update_plain")
                return
        # per-parameter path: user hook / overridden orthogonalize / RMS logging
        group_kwargs = {k: v for k, v in group.items() if k != "params"}
        for i, (p, t) in enumerate(zip(params, local)):
            key, k = plan.slot[i]
            u = plan.U[key][k].view(t.shape)
            if lr_wd != 0.0:
                t.mul_(1.0 - lr_wd)
            if self.log_per_module_grad_rms:
                name = getattr(p, "param_name", None)
                if name:
                    self.per_module_grad_rms[name] = torch.sqrt(torch.mean(u ** 2)).item()
            upd = self.orthogonalize(p, u, **group_kwargs)
            if self.log_per_module_update_rms:
                name = getattr(p, "param_name", None)
                if name:
                    self.per_module_update_rms[name] = torch.sqrt(torch.mean(upd.float() ** 2)).item()
            t.add_(upd, alpha=-lr)

    def get_update_rms_dict(self):
        return self.per_module_update_rms if self.log_per_module_update_rms else None

    def get_grad_rms_dict(self):
        return self.per_module_grad_rms if self.log_per_module_grad_rms else None

    def orthogonalize(self, p: torch.Tensor, grad: torch.Tensor, **kwargs: Any) -> torch.Tensor:
        """Default: apply ``scaled_orthogonalize_fn`` to the (Nesterov-blended) momentum. Subclasses may
        override to split fused parameters etc.; doing so selects the per-parameter path."""
        return self.scaled_orthogonalize_fn(grad)
