"""MuonBall on MI355X: Muon's msign update with the weights kept on a spectral sphere
(counterpart of emerging_optimizers/orthogonalized_optimizers/muon_ball.py:60-661).

Per step and matrix the reference runs, in a Python loop over parameters and over the pieces of fused parameters
(QKV groups / heads, gate|up, MoE experts): weight decay, EMA momentum, a 50-round power iteration with a host read of
sigma, an in-place retraction, msign of the momentum and the update.  Here a param group is

  1 multi-tensor launch   momentum (+ l2 decay) of every parameter,
  1 call                  spectral norms of every piece of every parameter (Gram matrices and their 2nd / 4th powers on the
                          matrix cores, then one launch per four rounds over all pieces; no host read),
  1 grouped call          msign of every piece (strided views into the momentum / update buffers, no copies),
  1 multi-tensor launch   W <- f * decay * W - lr * scale * Phi  with the retraction factor f taken from sigma on the
                          device.

When no parameter is split (every piece is a whole matrix) the momentum launch and the msign call are ONE library call
that never stores the blended momentum.  Pieces are described once per parameter set (``_Piece``) and cached.
"""
from __future__ import annotations

import ctypes
from typing import Any, Callable, Dict, List, Optional, Tuple

import numpy as np
import torch
from torch.optim.optimizer import ParamsT

from .. import _lib
from ..optim import newton_schulz_hip as ns
from ..optim.muon import _DeviceTable
from ..optim.opt_utils import to_local
from .mixin import WeightDecayT, weight_decay_terms
from .orthogonalized_optimizer import OrthogonalizedOptimizer, _Plan
from .spectral_ball_utils import (compute_target_radius, get_spectral_ball_scale_factor, msign, msign_schedule,
                                  spectral_norm)

__all__ = ["MuonBall"]


class _Piece:
    """One matrix that is orthogonalised and retracted on its own: a strided block of a parameter.

    ``off`` / ``rows`` / ``cols`` / ``ld`` give the block inside the row-major parameter (elements); ``shape`` is the
    logical [out, in] shape the radius and the scale factor are computed from (the transposed MoE slices differ from the
    stored orientation; sigma and msign commute with the transposition).  ``gather`` = (groups, split_sum, row_off,
    part) marks the one layout whose rows are not uniformly strided (QKV "component" mode)."""
    __slots__ = ("pi", "off", "rows", "cols", "ld", "shape", "label", "gather", "transposed")

    def __init__(self, pi, off, rows, cols, ld, shape, label, gather=None, transposed=False):
        self.pi, self.off, self.rows, self.cols, self.ld = pi, off, rows, cols, ld
        self.shape, self.label, self.gather = shape, label, gather
        self.transposed = transposed   # the matrix meant is the transpose of the stored block (MoE expert slices)


class _BallPlan:
    """Device tables and buffers of one param group beyond the momentum tables of the base class."""

    def __init__(self, opt: "MuonBall", base: _Plan, params: List[torch.Tensor], local: List[torch.Tensor],
                 device: torch.device):
        self.base = base
        self.pieces: List[_Piece] = []
        for i, (p, t) in enumerate(zip(params, local)):
            self.pieces.extend(opt._pieces_of(i, p, t))
        n = len(self.pieces)
        need_sigma = [pc.gather is None or opt.retract_mode == "dynamic" for pc in self.pieces]
        # spectral-norm problems: pieces of one geometry form one problem; their sigmas are contiguous
        order = sorted((i for i in range(n) if need_sigma[i]),
                       key=lambda i: (self.pieces[i].rows, self.pieces[i].cols, self._sn_ld(self.pieces[i]),
                                      self.pieces[i].transposed, local[self.pieces[i].pi].dtype == torch.float32))
        self.sigma = torch.zeros(max(n, 1), dtype=torch.float32, device=device)
        self.sigma_index = [-1] * n
        self.sn_classes: List[Tuple[Tuple, List[int]]] = []
        for rank, i in enumerate(order):
            pc = self.pieces[i]
            key = (pc.rows, pc.cols, self._sn_ld(pc), pc.transposed, local[pc.pi].dtype)
            if not self.sn_classes or self.sn_classes[-1][0] != key:
                self.sn_classes.append((key, []))
            self.sn_classes[-1][1].append(i)
            self.sigma_index[i] = rank
        # gathered pieces work on contiguous temporaries (fp32 momentum in, bf16 msign out, weights copy for sigma)
        self.tmp_u: Dict[int, torch.Tensor] = {}
        self.tmp_o: Dict[int, torch.Tensor] = {}
        self.tmp_w: Dict[int, torch.Tensor] = {}
        for i, pc in enumerate(self.pieces):
            if pc.gather is not None:
                self.tmp_u[i] = torch.empty((pc.rows, pc.cols), dtype=torch.float32, device=device)
                self.tmp_o[i] = torch.empty((pc.rows, pc.cols), dtype=torch.bfloat16, device=device)
                if need_sigma[i]:
                    self.tmp_w[i] = torch.empty((pc.rows, pc.cols), dtype=local[pc.pi].dtype, device=device)
        # msign problems: the same block of parameters at consecutive slots of a shape class's stacked buffers is one
        # batched problem
        self.ns_groups: List[Tuple[Tuple, List[int]]] = []
        last: Dict[Tuple, int] = {}
        for i, pc in enumerate(self.pieces):
            key, k = base.slot[pc.pi]
            if pc.gather is not None:
                self.ns_groups.append((("tmp", i), [i]))
                continue
            gkey = (key, pc.off, pc.rows, pc.cols, pc.ld)
            j = last.get(gkey)
            if j is not None and base.slot[self.pieces[self.ns_groups[j][1][-1]].pi][1] == k - 1:
                self.ns_groups[j][1].append(i)
            else:
                last[gkey] = len(self.ns_groups)
                self.ns_groups.append((gkey, [i]))
        self.ns_probs = (_lib.NsProblem * len(self.ns_groups))()
        self.sn_probs = (_lib.SnProblem * max(len(self.sn_classes), 1))()
        self.sn_ptrs = [(ctypes.c_void_p * len(idx))() for _, idx in self.sn_classes]
        # update items: one per piece; a gathered piece updates its `groups` row blocks separately and is not retracted
        self.items_of: List[List[int]] = []
        rows_total = 0
        for pc in self.pieces:
            cnt = 1 if pc.gather is None else pc.gather[0]
            self.items_of.append(list(range(rows_total, rows_total + cnt)))
            rows_total += cnt
        self.items = np.zeros(rows_total, dtype=_lib.BALL_ITEM)
        self.prefix = np.zeros(rows_total + 1, dtype=np.int32)
        self.item_tab = _DeviceTable(self.items.nbytes, device)
        self.log = torch.zeros(2 * max(rows_total, 1), dtype=torch.float32, device=device)
        self.sig: Optional[Tuple] = None
        self.prefix_dev: Optional[torch.Tensor] = None
        self.chunks = 0
        self.decay = 1.0

    @staticmethod
    def _sn_ld(pc: _Piece) -> int:
        return pc.cols if pc.gather is not None else pc.ld

    def refresh(self, opt: "MuonBall", local: List[torch.Tensor], device: torch.device) -> None:
        base = self.base
        sig = tuple(t.data_ptr() for t in local)
        if sig == self.sig:
            return
        chunk = _lib.CHUNK_ELEMS
        for ci, ((rows, cols, ld, transposed, dt), idx) in enumerate(self.sn_classes):
            q = self.sn_probs[ci]
            for b, i in enumerate(idx):
                pc = self.pieces[i]
                t = local[pc.pi]
                self.sn_ptrs[ci][b] = (self.tmp_w[i].data_ptr() if pc.gather is not None
                                       else t.data_ptr() + pc.off * t.element_size())
            q.w_ptrs = ctypes.cast(self.sn_ptrs[ci], ctypes.POINTER(ctypes.c_void_p))
            q.sigma_out = self.sigma.data_ptr() + 4 * self.sigma_index[idx[0]]
            q.dtype, q.ld, q.batch, q.rows, q.cols = _lib.dtype_code(dt), ld, len(idx), rows, cols
            q.flags = _lib.SN_TRANSPOSED if transposed else 0
        for q, (gkey, idx) in zip(self.ns_probs, self.ns_groups):
            if base.fused:
                break   # every piece is a whole matrix: the base plan's fused momentum + msign problems cover them
            pc = self.pieces[idx[0]]
            if gkey[0] == "tmp":
                i = idx[0]
                q.in_ptr, q.out_ptr = self.tmp_u[i].data_ptr(), self.tmp_o[i].data_ptr()
                q.in_batch_stride = q.out_batch_stride = pc.rows * pc.cols
                q.in_ld = q.out_ld = pc.cols
                q.batch = 1
            else:
                key, k0 = base.slot[pc.pi]
                U, Oo = base.U[key], base.O[key]
                numel = U[0].numel()
                q.in_ptr, q.out_ptr = U.data_ptr() + 4 * (k0 * numel + pc.off), Oo.data_ptr() + 2 * (k0 * numel + pc.off)
                q.in_batch_stride = q.out_batch_stride = numel
                q.in_ld = q.out_ld = pc.ld
                q.batch = len(idx)
            q.in_dtype, q.rows, q.cols = _lib.DTYPE_F32, pc.rows, pc.cols
        r = 0
        for i, pc in enumerate(self.pieces):
            t = local[pc.pi]
            key, k = base.slot[pc.pi]
            phi0 = base.O[key][k].data_ptr()
            radius = compute_target_radius(pc.shape, opt.radius_mode)
            ratio = get_spectral_ball_scale_factor(pc.shape[0], pc.shape[1], mode=opt.scale_mode)
            if pc.gather is None:
                blocks = [(pc.off, pc.rows, self.sigma.data_ptr() + 4 * self.sigma_index[i])]
            else:
                groups, ssum, row_off, part = pc.gather
                blocks = [((g * ssum + row_off) * pc.cols, part, 0) for g in range(groups)]
            for off, rows, sigma_ptr in blocks:
                it = self.items[r]
                it["w"], it["phi"], it["sigma"] = t.data_ptr() + off * t.element_size(), phi0 + 2 * off, sigma_ptr
                it["ld_w"] = it["ld_phi"] = pc.ld
                it["rows"], it["cols"] = rows, pc.cols
                it["radius"], it["lr_ratio"], it["w_dtype"] = radius, ratio, _lib.dtype_code(t.dtype)
                self.prefix[r + 1] = self.prefix[r] + (rows * pc.cols + chunk - 1) // chunk
                r += 1
        self.chunks = int(self.prefix[-1])
        self.item_tab.upload(self.items)
        self.prefix_dev = torch.from_numpy(self.prefix).to(device)
        self.sig = sig


class MuonBall(OrthogonalizedOptimizer):
    """Spectral Ball with lambda = 0: retraction of every weight matrix to spectral norm R, update by msign(momentum).

    Same constructor as the reference (muon_ball.py:196-279): params, lr, momentum_beta, weight_decay, use_nesterov,
    weight_decay_method, fp32_matmul_prec, power_iteration_steps, msign_steps, radius_mode ("spectral_mup" |
    "identity" | "initialize"), scale_mode, retract_mode ("hard" | "dynamic"), retract_alpha, split_qkv / is_qkv_fn /
    qkv_split_shapes / qkv_split_mode ("component" | "group" | "head"), split_fc1 / is_fc1_fn / fc1_split_shapes,
    split_moe_experts / is_grouped_moe_fn, pg_collection, tp_mode.  One GPU: a ``pg_collection`` whose tensor-parallel
    group has more than one rank raises ``NotImplementedError``.
    """

    def __init__(
        self,
        params: ParamsT,
        lr: float = 3e-4,
        momentum_beta: float = 0.9,
        weight_decay: float = 0.01,
        *,
        use_nesterov: bool = True,
        weight_decay_method: WeightDecayT = "decoupled",
        fp32_matmul_prec: str = "medium",
        power_iteration_steps: int = 10,
        msign_steps: int = 5,
        radius_mode: str = "spectral_mup",
        scale_mode: str = "align_adamw_rms",
        retract_mode: str = "hard",
        retract_alpha: float = 0.05,
        split_qkv: bool = False,
        is_qkv_fn: Optional[Callable[[torch.Tensor], bool]] = None,
        qkv_split_shapes: Optional[Tuple[int, int, int]] = None,
        qkv_split_mode: str = "component",
        split_fc1: bool = False,
        is_fc1_fn: Optional[Callable[[torch.Tensor], bool]] = None,
        fc1_split_shapes: Optional[Tuple[int, int]] = None,
        split_moe_experts: bool = False,
        is_grouped_moe_fn: Optional[Callable[[torch.Tensor], bool]] = None,
        pg_collection: Any | None = None,
        tp_mode: str = "duplicated",
    ) -> None:
        if power_iteration_steps < 1:
            raise ValueError(f"power_iteration_steps must be at least 1, got {power_iteration_steps}")
        if msign_steps < 1:
            raise ValueError(f"msign_steps must be at least 1, got {msign_steps}")
        if radius_mode not in ("spectral_mup", "identity", "initialize"):
            raise ValueError(f"Invalid radius_mode: {radius_mode}, must be one of: spectral_mup, identity, initialize")
        if retract_mode not in ("hard", "dynamic"):
            raise ValueError(f"Invalid retract_mode: {retract_mode}, must be one of: hard, dynamic")
        if qkv_split_mode not in ("component", "group", "head"):
            raise ValueError(f"Invalid qkv_split_mode: {qkv_split_mode}, must be one of: component, group, head")
        self.power_iteration_steps = power_iteration_steps
        self.msign_steps = msign_steps
        self.radius_mode = radius_mode
        self.scale_mode = scale_mode
        self.retract_mode = retract_mode
        self.retract_alpha = retract_alpha
        self.retract_bias_dict: Dict[str, float] = {}
        self.spectral_norm_dict: Dict[str, float] = {}
        self.split_qkv, self.is_qkv_fn = split_qkv, is_qkv_fn
        self.qkv_split_shapes, self.qkv_split_mode = qkv_split_shapes, qkv_split_mode
        self.split_fc1, self.is_fc1_fn, self.fc1_split_shapes = split_fc1, is_fc1_fn, fc1_split_shapes
        self.split_moe_experts, self.is_grouped_moe_fn = split_moe_experts, is_grouped_moe_fn
        self.pg_collection = pg_collection
        self.tp_mode = tp_mode
        for name in ("tp", "expt_tp"):
            grp = getattr(pg_collection, name, None) if pg_collection is not None else None
            if grp is not None and grp.size() > 1:
                raise NotImplementedError("MuonBall on MI355X runs on one GPU: tensor-parallel groups must have one rank")

        def scaled_orthogonalize_fn(grad: torch.Tensor) -> torch.Tensor:
            raise NotImplementedError(
                "MuonBall uses custom orthogonalize() method. scaled_orthogonalize_fn should not be called directly.")

        super().__init__(
            params, lr, momentum_beta, use_nesterov=use_nesterov, weight_decay=weight_decay,
            weight_decay_method=weight_decay_method, fp32_matmul_prec=fp32_matmul_prec,
            scaled_orthogonalize_fn=scaled_orthogonalize_fn, log_per_module_update_rms=False,
        )
        self._ball_plans: Dict[int, Tuple[Tuple, _BallPlan]] = {}

    def step(self, closure: Optional[Callable[[], float]] = None) -> Optional[float]:
        self.retract_bias_dict.clear()
        self.spectral_norm_dict.clear()
        return super().step(closure)

    # ---- pieces of one parameter (muon_ball.py:354-636) ---------------------------------------------------------
    def _pieces_of(self, pi: int, p: torch.Tensor, t: torch.Tensor) -> List[_Piece]:
        if t.ndim != 2:
            raise ValueError(f"MuonBall requires 2-D parameters, got shape {tuple(t.shape)}")
        out_dim, in_dim = t.shape
        name = getattr(p, "param_name", "") or ""
        if self.split_moe_experts and self.is_grouped_moe_fn is not None and self.is_grouped_moe_fn(p):
            experts = getattr(p, "num_local_experts", None)
            if experts is not None and experts > 1:
                if "weight1" in name:
                    # [hidden, experts * ffn * mult]: expert e owns a block of columns; it is treated as its transpose
                    mult = 2 if getattr(p, "is_gated", False) else 1
                    ffn = in_dim // (experts * mult)
                    pieces = []
                    for e in range(experts):
                        if self.split_fc1 and mult == 2:
                            for lo, lab in ((0, "gate"), (ffn, "up")):
                                pieces.append(_Piece(pi, e * ffn * mult + lo, out_dim, ffn, in_dim, (ffn, out_dim),
                                                     f"expert{e}.{lab}", transposed=True))
                        else:
                            pieces.append(_Piece(pi, e * ffn * mult, out_dim, ffn * mult, in_dim, (ffn * mult, out_dim),
                                                 f"expert{e}", transposed=True))
                    return pieces
                if "weight2" in name:
                    # [experts * ffn, hidden]: expert e owns a block of rows, again treated as its transpose
                    ffn = out_dim // experts
                    return [_Piece(pi, e * ffn * in_dim, ffn, in_dim, in_dim, (in_dim, ffn), f"expert{e}", transposed=True)
                            for e in range(experts)]
        if self.split_qkv and self.is_qkv_fn is not None and self.is_qkv_fn(p):
            assert self.qkv_split_shapes is not None, "qkv_split_shapes must be provided when split_qkv=True"
            shapes = list(self.qkv_split_shapes)
            ssum = sum(shapes)
            assert out_dim % ssum == 0, f"QKV split shapes {self.qkv_split_shapes} do not divide output dim {out_dim}"
            groups = out_dim // ssum
            offs = [0, shapes[0], shapes[0] + shapes[1]]
            names = ["q", "k", "v"]
            if self.qkv_split_mode == "component":
                return [_Piece(pi, 0, groups * shapes[i], in_dim, in_dim, (groups * shapes[i], in_dim), names[i],
                               gather=(groups, ssum, offs[i], shapes[i])) for i in range(3)]
            pieces = []
            kv = shapes[1]
            for g in range(groups):
                for i in range(3):
                    row0 = g * ssum + offs[i]
                    if self.qkv_split_mode == "head" and i == 0:
                        for h in range(shapes[0] // kv):
                            pieces.append(_Piece(pi, (row0 + h * kv) * in_dim, kv, in_dim, in_dim, (kv, in_dim), f"g{g}.Q.h{h}"))
                    else:
                        lab = f"g{g}.{names[i]}" if self.qkv_split_mode == "group" else f"g{g}.{names[i].upper()}"
                        pieces.append(_Piece(pi, row0 * in_dim, shapes[i], in_dim, in_dim, (shapes[i], in_dim), lab))
            return pieces
        if self.split_fc1 and self.is_fc1_fn is not None and self.is_fc1_fn(p):
            assert self.fc1_split_shapes is not None, "fc1_split_shapes must be provided when split_fc1=True"
            gate, up = self.fc1_split_shapes
            assert out_dim == gate + up, f"FC1 split shapes {self.fc1_split_shapes} do not match output dim {out_dim}"
            return [_Piece(pi, 0, gate, in_dim, in_dim, (gate, in_dim), "gate"),
                    _Piece(pi, gate * in_dim, up, in_dim, in_dim, (up, in_dim), "up")]
        return [_Piece(pi, 0, out_dim, in_dim, in_dim, (out_dim, in_dim), None)]

    # ---- one param group ------------------------------------------------------------------------------------------
    def _group_step(self, gi, group, params, local, grads, bufs) -> None:
        device = local[0].device
        for t in (*local, *grads, *bufs):
            _lib.require_cuda(t, "an optimizer tensor")
            if not t.is_contiguous():
                raise ValueError("parameters, gradients and momentum buffers must be contiguous")
        lr, beta = float(group["lr"]), float(group["momentum_beta"])
        wd = group.get("wd_mult", 1.0) * group["weight_decay"]
        lr_wd, l2 = weight_decay_terms(self.weight_decay_method, lr, wd)

        sig = (tuple((id(p), tuple(t.shape), t.dtype, g.dtype, getattr(p, "param_name", None),
                      getattr(p, "num_local_experts", None), getattr(p, "is_gated", None))
                     for p, t, g in zip(params, local, grads)), self.fuse_momentum, self.log_per_module_grad_rms)
        cached = self._ball_plans.get(gi)
        if cached is None or cached[0] != sig:
            # momentum fused into the msign call when every piece is a whole, contiguous matrix
            whole = all(pc.gather is None and pc.off == 0 and pc.ld == pc.cols and pc.rows * pc.cols == t.numel()
                        for i, (p, t) in enumerate(zip(params, local)) for pc in self._pieces_of(i, p, t))
            fused = (self.fuse_momentum and whole and not self.log_per_module_grad_rms
                     and _Plan.can_fuse(local, grads, bufs))
            base = _Plan(local, grads, None, device, fused)
            plan = _BallPlan(self, base, params, local, device)
            self._ball_plans[gi] = (sig, plan)
        else:
            plan = cached[1]
            plan.base.params = local
        base = plan.base

        L = _lib.lib()
        with torch.cuda.device(device):
            base.refresh(grads, bufs)
            plan.refresh(self, local, device)
            stream = _lib.current_stream_ptr(device)
            # grad (+= wd*p for l2);  buf <- lerp(buf, grad, 1-beta);  U = lerp(grad, buf, beta) | buf   (fp32)
            um, ug = (beta, 1.0 - beta) if self.use_nesterov else (1.0, 0.0)
            if not base.fused:
                _lib.check(L.muon_momentum(base.pre_tab.dev.data_ptr(), base.prefix_dev.data_ptr(), len(local),
                                           base.chunks, beta, 1.0 - beta, um, ug, l2, stream), "muon_momentum")
            if self.log_per_module_grad_rms:
                for p, i in zip(params, range(len(params))):
                    name = getattr(p, "param_name", None)
                    if name:
                        key, k = base.slot[i]
                        self.per_module_grad_rms[name] = torch.sqrt(torch.mean(base.U[key][k] ** 2)).item()
            # rows of a QKV component over all groups are gathered into contiguous temporaries
            for i, pc in enumerate(plan.pieces):
                if pc.gather is None:
                    continue
                groups, ssum, row_off, part = pc.gather
                key, k = base.slot[pc.pi]
                src = base.U[key][k].view(groups, ssum, pc.cols)[:, row_off:row_off + part]
                plan.tmp_u[i].view(groups, part, pc.cols).copy_(src)
                if i in plan.tmp_w:
                    plan.tmp_w[i].view(groups, part, pc.cols).copy_(
                        local[pc.pi].view(groups, ssum, pc.cols)[:, row_off:row_off + part])
            # spectral norms of the weights as they are now; the decay below scales them by the same factor
            if plan.sn_classes:
                n_sn = len(plan.sn_classes)
                ws = _lib.workspace(device, L.muon_spectral_norm_workspace_bytes(plan.sn_probs, n_sn), tag="sn")
                _lib.check(L.muon_spectral_norm(plan.sn_probs, n_sn, self.power_iteration_steps, ws.data_ptr(),
                                                ws.numel(), stream), "muon_spectral_norm")
            # Phi = msign(U) for every piece, written into the bf16 update buffers
            n_ns = len(plan.ns_groups)
            pm = ns._PREC[ns.ACCURATE_PREC]
            coeffs = msign_schedule(self.msign_steps)
            if base.fused:
                need = sum(L.muon_ns_workspace_bytes(q.batch, q.rows, q.cols, pm) for q in base.fused_probs)
                ws = _lib.workspace(device, need)
                _lib.check(L.muon_momentum_ns_grouped(base.fused_probs, len(base.fused_probs), beta, 1.0 - beta, um, ug, l2,
                                                      _lib.abc_array(coeffs), len(coeffs), 1e-7, _lib.EPS_CLAMP, pm,
                                                      _lib.ns_bsplit_tail(ns.BSPLIT_TAIL), ws.data_ptr(), ws.numel(),
                                                      stream), "muon_momentum_ns_grouped")
            else:
                ws = _lib.workspace(device, L.muon_ns_grouped_workspace_bytes(plan.ns_probs, n_ns, pm))
                _lib.check(L.muon_ns_grouped(plan.ns_probs, n_ns, _lib.abc_array(coeffs), len(coeffs), 1e-7,
                                             _lib.EPS_CLAMP, pm, _lib.ns_bsplit_tail(ns.BSPLIT_TAIL), ws.data_ptr(),
                                             ws.numel(), stream), "muon_ns_grouped")
            for i, pc in enumerate(plan.pieces):
                if pc.gather is None:
                    continue
                groups, ssum, row_off, part = pc.gather
                key, k = base.slot[pc.pi]
                base.O[key][k].view(groups, ssum, pc.cols)[:, row_off:row_off + part].copy_(
                    plan.tmp_o[i].view(groups, part, pc.cols))
            if self.log_per_module_update_rms:
                self._log_update_rms(plan, params)
            dynamic = self.retract_mode == "dynamic"
            plan.decay = 1.0 - lr_wd
            want_log = dynamic and any(getattr(p, "param_name", None) for p in params)
            _lib.check(L.muon_ball_apply(plan.item_tab.dev.data_ptr(), plan.prefix_dev.data_ptr(), len(plan.items),
                                         plan.chunks, lr, 1.0 - lr_wd,
                                         _lib.RETRACT_DYNAMIC if dynamic else _lib.RETRACT_HARD,
                                         self.retract_alpha * lr, plan.log.data_ptr() if want_log else 0, stream),
                       "muon_ball_apply")
            if want_log:
                self._collect_retract_log(plan, params)

    def _log_update_rms(self, plan: _BallPlan, params) -> None:
        base = plan.base
        for i, p in enumerate(params):
            name = getattr(p, "param_name", None)
            if not name:
                continue
            key, k = base.slot[i]
            sq = torch.zeros((), dtype=torch.float64, device=base.O[key].device)
            for pc in plan.pieces:
                if pc.pi != i:
                    continue
                ratio = get_spectral_ball_scale_factor(pc.shape[0], pc.shape[1], mode=self.scale_mode)
                if pc.gather is None:
                    blk = torch.as_strided(base.O[key][k], (pc.rows, pc.cols), (pc.ld, 1),
                                           base.O[key][k].storage_offset() + pc.off)
                else:
                    blk = plan.tmp_o[plan.pieces.index(pc)]
                sq += (blk.double() ** 2).sum() * ratio * ratio
            self.per_module_update_rms[name] = float(torch.sqrt(sq / p.numel()).item())

    def _collect_retract_log(self, plan: _BallPlan, params) -> None:
        """retract_bias_dict / spectral_norm_dict of the dynamic mode (muon_ball.py:343-346, 627-632): ONE device-to-host
        copy per step instead of one host read per piece."""
        log = plan.log.cpu().view(-1, 2)
        sigma = plan.sigma.cpu()
        for i, pc in enumerate(plan.pieces):
            name = getattr(params[pc.pi], "param_name", None)
            if not name:
                continue
            if pc.gather is None:
                s, bias = float(log[plan.items_of[i][0], 0]), float(log[plan.items_of[i][0], 1])
            else:
                # not retracted (the reference retracts a copy), but its sigma and bias are still reported
                s = float(sigma[plan.sigma_index[i]]) * plan.decay
                bias = -1.0 if s > compute_target_radius(pc.shape, self.radius_mode) else 1.0
            key = name if pc.label is None else f"{name}.{pc.label}"
            self.retract_bias_dict[key] = bias
            self.spectral_norm_dict[key] = s

    def _compute_component_update(self, W: torch.Tensor, M: torch.Tensor, tp_group: Any = None,
                                  partition_dim: Optional[int] = None, current_lr: Optional[float] = None,
                                  param_name: Optional[str] = None, component_label: Optional[str] = None) -> torch.Tensor:
        """One matrix (muon_ball.py:301-352): spectral norm by power iteration, retraction of ``W`` IN PLACE, then
        ``scale * msign(M)``. ``W`` and ``M`` may be views into a parameter and its momentum (transposed ones included).
        Hard retraction reads nothing back to the host; the dynamic mode reads sigma for its logging dictionaries, as the
        reference does."""
        if tp_group is not None and tp_group.size() > 1:
            raise NotImplementedError("MuonBall on MI355X runs on one GPU: tensor-parallel groups must have one rank")
        R = compute_target_radius(tuple(W.shape), self.radius_mode)
        sigma = spectral_norm(W, self.power_iteration_steps)            # 0-d fp32 device tensor
        # the factor stays in fp32 (the reference multiplies by a Python float in fp32 arithmetic): rounded to bf16 first,
        # R / sigma would be off by up to 0.4 % and 1 +- alpha * lr would round to exactly 1 for a small lr
        def scale_(factor: torch.Tensor) -> None:
            if W.dtype == torch.float32:
                W.mul_(factor)
            else:
                W.copy_(W.to(torch.float32) * factor)
        if self.retract_mode == "hard":
            scale_(R / (sigma.clamp_min(0.0) + 1e-8))
        else:
            bias_t = torch.where(sigma > R, -1.0, 1.0)
            step = self.retract_alpha * current_lr if current_lr is not None else self.retract_alpha
            scale_(1.0 + step * bias_t)
            if param_name and component_label:
                self.retract_bias_dict[f"{param_name}.{component_label}"] = float(bias_t.item())
                self.spectral_norm_dict[f"{param_name}.{component_label}"] = float(sigma.item())
        phi = msign(M if M.dtype == torch.float32 else M.to(torch.float32), self.msign_steps)
        return phi * get_spectral_ball_scale_factor(W.shape[0], W.shape[1], mode=self.scale_mode)

    @torch.no_grad()
    def orthogonalize(self, p: torch.Tensor, grad: torch.Tensor, **kwargs: Any) -> torch.Tensor:
        """The reference's public per-tensor entry (muon_ball.py:354-636): retracts ``p`` (every piece of a fused
        parameter on its own) in place and returns the update direction shaped like ``p``, to be applied as
        ``p.add_(update, alpha=-lr)``. ``grad`` is the momentum-processed gradient; ``lr`` comes in through ``kwargs``.
        ``step()`` does not go through here (it runs every piece of a param group in batched device calls); this is for
        callers and subclasses that use the reference's per-tensor contract. As in the reference, the QKV "component"
        layout works on gathered copies, so the parameter itself is not retracted in that mode."""
        lr = kwargs.get("lr", None)
        t = to_local([p])[0]
        g = to_local([grad])[0]
        _lib.require_cuda(t, "a MuonBall parameter")
        if not t.is_contiguous() or not g.is_contiguous() or g.shape != t.shape:
            raise ValueError("parameter and gradient must be contiguous and of one shape")
        name = getattr(p, "param_name", None)
        update = torch.empty(t.shape, dtype=torch.bfloat16, device=t.device)
        for pc in self._pieces_of(0, p, t):
            if pc.gather is not None:
                groups, ssum, row_off, part = pc.gather
                sl = (slice(None), slice(row_off, row_off + part))
                W = t.view(groups, ssum, pc.cols)[sl].reshape(-1, pc.cols)         # a copy, like the reference's reshape
                M = g.view(groups, ssum, pc.cols)[sl].reshape(-1, pc.cols)
                U = self._compute_component_update(W, M, None, None, lr, name, pc.label)
                update.view(groups, ssum, pc.cols)[sl] = U.view(groups, part, pc.cols)
                continue
            W = torch.as_strided(t, (pc.rows, pc.cols), (pc.ld, 1), t.storage_offset() + pc.off)
            M = torch.as_strided(g, (pc.rows, pc.cols), (pc.ld, 1), g.storage_offset() + pc.off)
            out = torch.as_strided(update, (pc.rows, pc.cols), (pc.ld, 1), pc.off)
            if pc.transposed:
                out.copy_(self._compute_component_update(W.t(), M.t(), None, None, lr, name, pc.label).t())
            else:
                out.copy_(self._compute_component_update(W, M, None, None, lr, name, pc.label))
        return update

    def get_retract_bias_dict(self):
        if self.retract_mode == "hard" or not self.retract_bias_dict:
            return None
        return self.retract_bias_dict

    def get_spectral_norm_dict(self):
        if not self.spectral_norm_dict:
            return None
        return self.spectral_norm_dict
