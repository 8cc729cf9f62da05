"""Muon / MuonH optimizer for MI355X: drop-in for ``lit_gpt.optim.muon.Muon`` on one GPU.

Same constructor, param-group keys, state keys and ``step()`` contract as the reference
(lit_gpt/optim/muon.py:27-197), but the per-parameter task loop is replaced by

  1. ONE multi-tensor momentum launch over every matrix parameter of a group,
  2. one batched Newton-Schulz call per shape class (all same-shape layers / experts together),
  3. ONE multi-tensor weight update (plain Muon, or MuonH in two passes),

all hand-written gfx950 kernels reached through the C ABI in ``include/archscale_muon.h``.
There is no CPU or PyTorch fallback for the Muon groups: tensors must live on the GPU.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, List, Optional, Sequence, Tuple, Union

import numpy as np
import torch
from torch import Tensor
from torch.optim.optimizer import Optimizer, ParamsT

from .. import _lib
from . import newton_schulz_hip as ns
from . import scalar_opts
from .opt_utils import matrix_view_shape, to_local

try:
    from torch.distributed.device_mesh import DeviceMesh
except Exception:  # pragma: no cover
    DeviceMesh = None  # type: ignore[assignment]
try:
    from torch.distributed import ProcessGroup
except Exception:  # pragma: no cover
    ProcessGroup = None  # type: ignore[assignment]


def adjust_lr_rms_norm(lr, param_shape, flatten):
    """lr for a constant element-wise RMS of the update (lit_gpt/optim/muon.py:841-851)."""
    fan_out, fan_in = _fans(param_shape, flatten)
    return lr * 0.2 * math.sqrt(max(fan_out, fan_in))


def adjust_lr_spectral_norm(lr, param_shape, flatten, clip_norm: bool = False):
    """lr from spectral norm 1 to RMS operator norm 1 (lit_gpt/optim/muon.py:854-866)."""
    fan_out, fan_in = _fans(param_shape, flatten)
    if clip_norm:
        return lr * max(1.0, fan_out / fan_in) ** 0.5
    return lr * math.sqrt(fan_out / fan_in)


def _fans(param_shape, flatten):
    if flatten:
        return param_shape[0], math.prod(param_shape[1:])
    return param_shape[-2], param_shape[-1]


def _lr_ratio(shape, mode: Optional[str], flatten: bool) -> float:
    if mode is None:
        return 1.0
    if mode == "spectral_norm":
        return adjust_lr_spectral_norm(1.0, shape, flatten)
    if mode == "clip_norm":
        return adjust_lr_spectral_norm(1.0, shape, flatten, clip_norm=True)
    if mode == "rms_norm":
        return adjust_lr_rms_norm(1.0, shape, flatten)
    raise ValueError(f"Unknown adjust_lr value: {mode}")


class _DeviceTable:
    """A small host table mirrored on the device; uploads go through two alternating pinned buffers so a
    refill never overwrites bytes an earlier asynchronous copy may still be reading."""

    def __init__(self, nbytes: int, device: torch.device):
        self.dev = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
        self._pinned = [torch.empty(max(nbytes, 1), dtype=torch.uint8, pin_memory=True) for _ in range(2)]
        self._events: List[Optional[torch.cuda.Event]] = [None, None]
        self._turn = 0

    def upload(self, host: np.ndarray) -> None:
        i = self._turn
        self._turn ^= 1
        if self._events[i] is not None:
            self._events[i].synchronize()
        raw = host.view(np.uint8).reshape(-1)
        self._pinned[i][: raw.size].copy_(torch.from_numpy(raw))
        self.dev[: raw.size].copy_(self._pinned[i][: raw.size], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._events[i] = ev


class _PhaseTimer:
    """Context manager that brackets a phase with two events on the current stream when timing is on."""

    def __init__(self, sink: Optional[list], name: str):
        self.sink, self.name = sink, name

    def __enter__(self):
        if self.sink is not None:
            self.start = torch.cuda.Event(enable_timing=True)
            self.start.record()
        return self

    def __exit__(self, *exc):
        if self.sink is not None:
            stop = torch.cuda.Event(enable_timing=True)
            stop.record()
            self.sink.append((self.name, self.start, stop))
        return False


class _ShapeClass:
    """All matrices of one (rows, cols) in a group: one U buffer, one batched Newton-Schulz call."""

    def __init__(self, rows: int, cols: int):
        self.rows, self.cols = rows, cols
        self.n_mats = 0
        self.U: Optional[Tensor] = None


class _GroupPlan:
    """Launch plan of one muon param group: which tensors, where their U lives, the device tables."""

    def __init__(self, params: List[Tensor], flatten: bool, use_muonh: bool, per_matrix: bool,
                 adjust_lr: Optional[str], device: torch.device):
        self.params = params
        self.device = device
        self.flatten = flatten
        self.classes: Dict[Tuple[int, int], _ShapeClass] = {}
        self.views: List[Tuple[_ShapeClass, int, int]] = []  # per param: (class, first matrix, n matrices)
        for p in params:
            n, r, c = matrix_view_shape(p.shape, flatten)
            cls = self.classes.setdefault((r, c), _ShapeClass(r, c))
            self.views.append((cls, cls.n_mats, n))
            cls.n_mats += n
        for cls in self.classes.values():
            cls.U = torch.empty((cls.n_mats, cls.rows, cls.cols), dtype=torch.bfloat16, device=device)

        chunk = _lib.CHUNK_ELEMS
        n = len(params)
        self.pre = np.zeros(n, dtype=_lib.PRE_ITEM)
        self.pre_prefix = np.zeros(n + 1, dtype=np.int32)
        for i, p in enumerate(params):
            self.pre_prefix[i + 1] = self.pre_prefix[i] + (p.numel() + chunk - 1) // chunk
        # update items: whole tensors (the reference takes ONE MuonH norm per tensor, also for a 3-D
        # stack: lit_gpt/optim/muon.py:754-758), or one item per matrix when asked
        post_rows = []
        for i, p in enumerate(params):
            cls, first, nm = self.views[i]
            ratio = _lr_ratio(p.shape, adjust_lr, flatten)
            if use_muonh and per_matrix and nm > 1:
                per = cls.rows * cls.cols
                post_rows += [(i, k * per, per, ratio) for k in range(nm)]
            else:
                post_rows.append((i, 0, p.numel(), ratio))
        self.post_rows = post_rows
        self.post = np.zeros(len(post_rows), dtype=_lib.POST_ITEM)
        self.post_prefix = np.zeros(len(post_rows) + 1, dtype=np.int32)
        for k, (_, _, numel, _) in enumerate(post_rows):
            self.post_prefix[k + 1] = self.post_prefix[k] + (numel + chunk - 1) // chunk
        self.pre_chunks = int(self.pre_prefix[-1])
        self.post_chunks = int(self.post_prefix[-1])

        self.pre_tab = _DeviceTable(self.pre.nbytes, device)
        self.post_tab = _DeviceTable(self.post.nbytes, device)
        self.pre_prefix_dev = torch.from_numpy(self.pre_prefix).to(device)
        self.post_prefix_dev = torch.from_numpy(self.post_prefix).to(device)
        n_scratch = _lib.lib().muon_muonh_scratch_floats(len(post_rows), self.post_chunks) if use_muonh else 0
        self.scratch = torch.empty(max(n_scratch, 1), dtype=torch.float32, device=device)
        self.ptr_sig: Optional[Tuple] = None
        # fused momentum + Newton-Schulz call: one problem per (shape class, dtypes), matrices listed by pointer
        self.fused_probs = None
        self.fused_keep: List = []

    def refresh_pointers(self, grads: List[Tensor], moms: List[Tensor]) -> None:
        sig = tuple((p.data_ptr(), g.data_ptr(), m.data_ptr()) for p, g, m in zip(self.params, grads, moms))
        if sig == self.ptr_sig:
            return
        for i, (p, g, m) in enumerate(zip(self.params, grads, moms)):
            cls, first, _ = self.views[i]
            row = self.pre[i]
            row["g"], row["m"], row["w"] = g.data_ptr(), m.data_ptr(), p.data_ptr()
            row["u"] = cls.U.data_ptr() + first * cls.rows * cls.cols * 2
            row["numel"] = p.numel()
            row["g_dtype"], row["m_dtype"] = _lib.dtype_code(g.dtype), _lib.dtype_code(m.dtype)
            row["u_dtype"], row["w_dtype"] = _lib.DTYPE_BF16, _lib.dtype_code(p.dtype)
        for k, (i, off, numel, ratio) in enumerate(self.post_rows):
            p = self.params[i]
            row = self.post[k]
            row["w"] = p.data_ptr() + off * p.element_size()
            row["u"] = int(self.pre[i]["u"]) + off * 2
            row["numel"], row["lr_ratio"], row["w_dtype"] = numel, ratio, _lib.dtype_code(p.dtype)
        self.pre_tab.upload(self.pre)
        self.post_tab.upload(self.post)
        self.ptr_sig = sig
        self._build_fused(grads, moms)

    def _build_fused(self, grads: List[Tensor], moms: List[Tensor]) -> None:
        """muon_mns_problem array: per shape class the (g, m, w) pointers of its matrices in the order of its U buffer.
        A class whose tensors do not share one dtype triple is left to the unfused path (fused_probs = None)."""
        import ctypes
        per_class: Dict[Tuple[int, int], List[Tuple[int, int, int, Tuple]]] = {k: [] for k in self.classes}
        for i, (p, g, m) in enumerate(zip(self.params, grads, moms)):
            cls, first, nm = self.views[i]
            per = cls.rows * cls.cols
            for k in range(nm):
                per_class[(cls.rows, cls.cols)].append((g.data_ptr() + k * per * g.element_size(),
                                                        m.data_ptr() + k * per * m.element_size(),
                                                        p.data_ptr() + k * per * p.element_size(),
                                                        (g.dtype, m.dtype, p.dtype)))
        probs = (_lib.MnsProblem * len(self.classes))()
        keep = []
        for q, (key, cls) in zip(probs, self.classes.items()):
            rows = per_class[key]
            if len({r[3] for r in rows}) != 1:
                self.fused_probs = None
                return
            arrs = [(ctypes.c_void_p * len(rows))(*[r[j] for r in rows]) for j in range(3)]
            keep.append(arrs)
            q.g_ptrs, q.m_ptrs, q.w_ptrs = (ctypes.cast(a, ctypes.POINTER(ctypes.c_void_p)) for a in arrs)
            q.out, q.out_batch_stride, q.out_ld = cls.U.data_ptr(), cls.rows * cls.cols, cls.cols
            gd, md, wd = rows[0][3]
            q.g_dtype, q.m_dtype, q.w_dtype = _lib.dtype_code(gd), _lib.dtype_code(md), _lib.dtype_code(wd)
            q.batch, q.rows, q.cols = len(rows), cls.rows, cls.cols
        self.fused_probs, self.fused_keep = probs, keep


class Muon(Optimizer):
    """Distributed-Muon API of the reference, single-GPU, on hand-written MI355X kernels.

    Args (as lit_gpt/optim/muon.py:58-74): params, distributed_mesh, lr, mu, betas, weight_decay,
    cautious_wd, epsilon, nesterov, adjust_lr, flatten, use_triton, newton_schulz_func, use_muonh.
    ``use_triton`` is accepted and ignored: the built-in Newton-Schulz is always the HIP path.
    ``newton_schulz_func(X, epsilon=...)`` replaces it per tensor, as in the reference.

    Extra keyword-only knobs of this implementation:
      ns_coefficients   (a, b, c) rows, one per iteration (default: the reference's 5-row schedule)
      ns_precision      "bf16" or "f16" (the iteration's matrices in IEEE half inside the workspace, scaled by powers of
                        two: 8x the mantissa at the same rate; what the constant and polar-express tables need).
                        "bsplit" (B = bA + cA^2 kept as a bf16 hi+lo pair, a second walk over K in BX) is still
                        accepted as a diagnostic mode: "f16" is both faster and more accurate
      ns_gram_tail      None (default): with "bf16" the last two iterations are stored in IEEE half and, for matrices whose
                        long side is at least twice the short one, finished on the Gram side (one BX and one XX^T
                        product less); False: five plain iterations; True: the tail also with "f16"
      muonh_per_matrix  renormalise each matrix of a 3-D parameter on its own instead of the whole tensor
      fuse_momentum     momentum and Newton-Schulz in one library call that never stores the bf16 update in the
                        parameter's orientation (default; falls back to separate calls with a hook or a tight limit)
      ns_workspace_limit  upper bound in bytes for one batched Newton-Schulz workspace (larger classes
                          are processed in slices)
      device_hyperparams  the weight-update kernels of every group read lr, lr*weight_decay, eps (and, for the AdamW /
                          Lion groups, the betas' complements and bias corrections) from a small block in device
                          memory instead of kernel arguments, so a ``step()`` captured in a HIP graph follows the
                          schedule that the training loop writes into ``group["lr"]`` (pretrain.py:829-877): call
                          ``sync_hyperparameters(advance_step=True)`` before each replay.  The momentum factor, the
                          Newton-Schulz epsilon and the coefficient table stay kernel arguments.
    """

    def __init__(
        self,
        params: ParamsT,
        distributed_mesh=None,
        lr: float = 0.01,
        mu: float = 0.95,
        betas: Tuple[float, float] = (0.9, 0.95),
        weight_decay: float = 0.01,
        cautious_wd: bool = False,
        epsilon: float = 1e-8,
        nesterov: bool = False,
        adjust_lr: Optional[str] = "spectral_norm",
        flatten: bool = False,
        use_triton: bool = False,
        newton_schulz_func: Optional[Callable] = None,
        use_muonh: bool = False,
        *,
        ns_coefficients: Optional[Sequence[Tuple[float, float, float]]] = None,
        ns_precision: str = "bf16",
        ns_gram_tail: Optional[bool] = None,
        muonh_per_matrix: bool = False,
        ns_workspace_limit: int = 48 << 30,
        fuse_momentum: bool = True,
        device_hyperparams: bool = False,
    ):
        if lr < 0.0:
            raise ValueError(f"Invalid learning rate: {lr}")
        if mu < 0.0:
            raise ValueError(f"Invalid momentum factor (mu): {mu}")
        if len(betas) != 2 or betas[0] < 0.0 or betas[1] < 0.0:
            raise ValueError(f"Invalid betas: {betas}")
        if adjust_lr not in ("spectral_norm", "rms_norm", "clip_norm", None):
            raise ValueError(
                f"Invalid adjust_lr value: {adjust_lr}. Must be 'spectral_norm', 'rms_norm', 'clip_norm', or None."
            )
        if ns_precision not in ("bf16", "bsplit", "f16"):
            raise ValueError(f"Invalid ns_precision: {ns_precision}")

        defaults = dict(
            lr=lr, mu=mu, beta1=betas[0], beta2=betas[1], weight_decay=weight_decay, cautious_wd=cautious_wd,
            algorithm="muon", step=0, epsilon=epsilon, nesterov=nesterov, flatten=flatten, adjust_lr=adjust_lr,
        )
        super().__init__(params, defaults)

        self.use_muonh = use_muonh
        self._hyperball_excluded: set = set()

        # one GPU: a mesh or group of size 1 is accepted, anything larger is outside this build
        if distributed_mesh is None:
            world = 1
        elif DeviceMesh is not None and isinstance(distributed_mesh, DeviceMesh):
            if distributed_mesh.ndim != 1:
                raise ValueError(
                    f"Only 1D DeviceMesh is supported, but got {distributed_mesh.ndim}D. "
                    "For HSDP, provide the 1D sharded sub-mesh.")
            world = distributed_mesh.size()
        elif ProcessGroup is not None and isinstance(distributed_mesh, ProcessGroup):
            world = torch.distributed.get_world_size(distributed_mesh)
        else:
            raise TypeError(
                f"Invalid distributed_mesh type: {type(distributed_mesh)}. Expected DeviceMesh or ProcessGroup.")
        if world != 1:
            raise NotImplementedError(
                "this build runs the Muon step on one GPU; sharded parameters (world size > 1) are not supported")
        self._device_rank, self._world_size, self._process_group = 0, 1, None
        self._distributed_mesh = distributed_mesh

        if newton_schulz_func is not None and not callable(newton_schulz_func):
            raise TypeError(f"newton_schulz_func must be a callable function, got {type(newton_schulz_func)}")
        self._newton_schulz_func = newton_schulz_func
        self._ns_coefficients = tuple(tuple(map(float, r)) for r in (ns_coefficients or ns.QUINTIC_SCHEDULE))
        self._ns_precision = ns_precision
        self._ns_gram_tail = ns_gram_tail
        self._ns_tail_flags = 0 if ns_gram_tail is None else (_lib.NS_GRAM_TAIL if ns_gram_tail else _lib.NS_NO_GRAM_TAIL)
        self._muonh_per_matrix = muonh_per_matrix
        self._ns_workspace_limit = int(ns_workspace_limit)
        self._fuse_momentum = bool(fuse_momentum)
        self._device_hyper = bool(device_hyperparams)
        self._hyper_tables: Dict[int, _DeviceTable] = {}
        self._plans: Dict[int, Tuple[Tuple, _GroupPlan]] = {}
        self._scalar_plans: dict = {}
        #: when set to a list, every phase of a muon group step appends (name, start_event, stop_event)
        self.phase_events: Optional[list] = None

    def _timed(self, name: str):
        return _PhaseTimer(self.phase_events, name)

    def exclude_from_hyperball(self, *params):
        """Keep these parameters (e.g. embeddings) out of hyperball normalisation in "adamw" groups
        (lit_gpt/optim/muon.py:144-157)."""
        for p in params:
            self._hyperball_excluded.add(p)

    # ------------------------------------------------------------------ hyper-parameters in device memory
    def _group_device(self, group: dict) -> Optional[torch.device]:
        for p in group["params"]:
            return to_local([p])[0].device
        return None

    def _hyper_table(self, gi: int, group: dict) -> Optional[_DeviceTable]:
        tab = self._hyper_tables.get(gi)
        if tab is None:
            device = self._group_device(group)
            if device is None or device.type != "cuda":
                return None
            tab = _DeviceTable(_lib.HYPER.itemsize, device)
            self._hyper_tables[gi] = tab
        return tab

    def _upload_group_hyper(self, gi: int, group: dict) -> None:
        tab = self._hyper_table(gi, group)
        if tab is None:
            return
        lr, wd = float(group["lr"]), float(group["weight_decay"])
        rec = _lib.hyper_record(lr, lr * wd, float(group["epsilon"]), float(group["beta1"]), float(group["beta2"]),
                                int(group["step"]), bool(group["cautious_wd"]))
        with torch.cuda.device(tab.dev.device):
            tab.upload(rec)

    def sync_hyperparameters(self, advance_step: bool = False) -> None:
        """With ``device_hyperparams``: copy the current hyper-parameters of every param group to the device block that
        the kernels read (one small asynchronous copy per group on the current stream). ``step()`` does this itself
        when it runs eagerly; a step that was captured in a HIP graph cannot, so call this before each replay, with
        ``advance_step=True`` to count the replay as a step (``group["step"]``, the AdamW bias corrections)."""
        if not self._device_hyper:
            raise RuntimeError("sync_hyperparameters() needs Muon(..., device_hyperparams=True)")
        for gi, group in enumerate(self.param_groups):
            if advance_step:
                group["step"] += 1
            self._upload_group_hyper(gi, group)

    # ------------------------------------------------------------------ step
    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()

        # a step that is being captured in a graph runs nothing now: its replays are counted, and their hyper-parameters
        # uploaded, by sync_hyperparameters()
        capturing = self._device_hyper and torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()
        muon_groups, lion_groups, adamw_groups = [], [], []
        for gi, group in enumerate(self.param_groups):
            if not capturing:
                group["step"] += 1
            algo = group["algorithm"]
            if algo == "muon":
                muon_groups.append((gi, group))
            elif algo == "lion":
                lion_groups.append((gi, group))
            elif algo == "adamw":
                adamw_groups.append((gi, group))
            else:
                raise ValueError(f"Unknown algorithm: {algo}")
            if self._device_hyper and not capturing:
                self._upload_group_hyper(gi, group)

        for gi, group in muon_groups:
            self._muon_group_step(gi, group)
        for gi, group in lion_groups:
            self._lion_group_step(gi, group)
        for gi, group in adamw_groups:
            self._adamw_group_step(gi, group)
        return loss

    def _hyper_ptr(self, gi: int, group: dict) -> Optional[int]:
        if not self._device_hyper:
            return None
        tab = self._hyper_table(gi, group)
        return None if tab is None else tab.dev.data_ptr()

    def _get_or_initialize_state(self, param: Tensor, algo: str) -> dict:
        state = self.state[param]
        if not state:
            state["momentum"] = torch.zeros_like(param)
            if algo == "adamw":
                state["variance"] = torch.zeros_like(param)
        return state

    # ------------------------------------------------------------------ muon
    def _muon_group_step(self, gi: int, group: dict) -> None:
        assert all(p.ndim >= 2 for p in group["params"]), "Muon optimizer only supports matrix parameters."
        params = [p for p in group["params"] if p.grad is not None]
        if not params:
            return
        moms = to_local([self._get_or_initialize_state(p, "muon")["momentum"] for p in params])
        local = to_local(params)
        grads = to_local([p.grad for p in params])
        device = local[0].device
        for t in local:
            _lib.require_cuda(t, "a Muon parameter")
            if t.device != device:
                raise ValueError("all parameters of a muon group must live on one device")
            if not t.is_contiguous():
                raise ValueError("Muon parameters must be contiguous")
        grads = [g if g.is_contiguous() else g.contiguous() for g in grads]
        for m in moms:
            if not m.is_contiguous():
                raise ValueError("Muon momentum buffers must be contiguous")

        flatten, adjust = group["flatten"], group["adjust_lr"]
        _lr_ratio((2, 2), adjust, flatten)  # raises on an unknown mode, like the reference
        struct_sig = (tuple((id(p), tuple(t.shape), t.dtype, g.dtype) for p, t, g in zip(params, local, grads)),
                      flatten, adjust, self.use_muonh, self._muonh_per_matrix, device)
        cached = self._plans.get(gi)
        if cached is None or cached[0] != struct_sig:
            plan = _GroupPlan(local, flatten, self.use_muonh, self._muonh_per_matrix, adjust, device)
            self._plans[gi] = (struct_sig, plan)
        else:
            plan = cached[1]
            plan.params = local

        L = _lib.lib()
        lr, mu, wd, eps = float(group["lr"]), float(group["mu"]), float(group["weight_decay"]), float(group["epsilon"])
        nesterov, cautious = bool(group["nesterov"]), bool(group["cautious_wd"])
        with torch.cuda.device(device):
            plan.refresh_pointers(grads, moms)
            stream = _lib.current_stream_ptr(device)
            c_um, c_ug = (mu, 1.0) if nesterov else (1.0, 0.0)
            if not self._momentum_and_ns_fused(plan, mu, c_um, c_ug, eps, stream):
                # M <- mu*M + G ; U <- mu*M + G (nesterov) | M, in bf16       (muon.py:653-681)
                with self._timed("momentum"):
                    _lib.check(L.muon_momentum(plan.pre_tab.dev.data_ptr(), plan.pre_prefix_dev.data_ptr(), len(local),
                                               plan.pre_chunks, mu, 1.0, c_um, c_ug, 0.0, stream), "muon_momentum")
                # U <- NS(U), one batched call per shape class                    (muon.py:821-838)
                if self._newton_schulz_func is None:
                    with self._timed("newton_schulz"):
                        self._orthogonalize_classes(list(plan.classes.values()), eps)
                else:
                    self._orthogonalize_with_hook(plan, eps)
            # weight update                                                   (muon.py:598-650)
            hyper = self._hyper_ptr(gi, group)
            with self._timed("update_muonh" if self.use_muonh else "update_plain"):
                if hyper is not None and self.use_muonh:
                    _lib.check(L.muon_update_muonh_dev(plan.post_tab.dev.data_ptr(), plan.post_prefix_dev.data_ptr(),
                                                       len(plan.post_rows), plan.post_chunks, hyper,
                                                       plan.scratch.data_ptr(), stream), "muon_update_muonh_dev")
                elif hyper is not None:
                    _lib.check(L.muon_update_plain_dev(plan.post_tab.dev.data_ptr(), plan.post_prefix_dev.data_ptr(),
                                                       len(plan.post_rows), plan.post_chunks, hyper, stream),
                               "muon_update_plain_dev")
                elif self.use_muonh:
                    _lib.check(L.muon_update_muonh(plan.post_tab.dev.data_ptr(), plan.post_prefix_dev.data_ptr(),
                                                   len(plan.post_rows), plan.post_chunks, lr, lr * wd, eps,
                                                   int(cautious), plan.scratch.data_ptr(), stream),
                               "muon_update_muonh")
                else:
                    _lib.check(L.muon_update_plain(plan.post_tab.dev.data_ptr(), plan.post_prefix_dev.data_ptr(),
                                                   len(plan.post_rows), plan.post_chunks, lr, lr * wd, int(cautious),
                                                   stream), "muon_update_plain")

    def _momentum_and_ns_fused(self, plan: _GroupPlan, mu: float, c_um: float, c_ug: float, eps: float, stream) -> bool:
        """Momentum and Newton-Schulz of the whole group in ONE library call in which the bf16 update goes straight
        into the operand of the iteration (no separate store, norm pass and layout pass over it). Used with the
        built-in Newton-Schulz when the workspace of all classes together fits the limit; returns False otherwise."""
        if self._newton_schulz_func is not None or not self._fuse_momentum or plan.fused_probs is None:
            return False
        L = _lib.lib()
        pm = ns._PREC[self._ns_precision]
        n = len(plan.fused_probs)
        need = sum(L.muon_ns_workspace_bytes(q.batch, q.rows, q.cols, pm) for q in plan.fused_probs)
        if need > self._ns_workspace_limit:
            return False
        ws = _lib.workspace(plan.device, need)
        coeffs = self._ns_coefficients
        with self._timed("momentum+newton_schulz"):
            _lib.check(L.muon_momentum_ns_grouped(plan.fused_probs, n, mu, 1.0, c_um, c_ug, 0.0, _lib.abc_array(coeffs),
                                                  len(coeffs), eps, _lib.EPS_ADD, pm,
                                                  _lib.ns_bsplit_tail(ns.BSPLIT_TAIL) | self._ns_tail_flags,
                                                  ws.data_ptr(), ws.numel(), stream), "muon_momentum_ns_grouped")
        return True

    def _orthogonalize_classes(self, classes: List[_ShapeClass], eps: float) -> None:
        """U <- NS(U) for every shape class in ONE grouped call (each product of the iteration is one launch over
        all classes); classes are sliced / the call is split only when the workspace would exceed the limit."""
        L = _lib.lib()
        pm = ns._PREC[self._ns_precision]
        parts: List[Tensor] = []
        used = 0

        def run():
            nonlocal parts, used
            if parts:
                ns.newton_schulz_grouped(parts, self._ns_coefficients, eps, prec=self._ns_precision, outs=parts,
                                         bsplit_tail=ns.BSPLIT_TAIL, gram_tail=self._ns_gram_tail)
            parts, used = [], 0

        for cls in classes:
            per = max(1, L.muon_ns_workspace_bytes(1, cls.rows, cls.cols, pm))
            lo = 0
            while lo < cls.n_mats:
                room = (self._ns_workspace_limit - used) // per
                if room < 1 and parts:
                    run()
                    continue
                take = max(1, min(cls.n_mats - lo, room))
                parts.append(cls.U[lo:lo + take])
                used += take * per
                lo += take
        run()

    def _orthogonalize_with_hook(self, plan: _GroupPlan, eps: float) -> None:
        # user hook, one tensor at a time with the reference's flatten policy (muon.py:821-838);
        # the reference hands it epsilon as a 0-d tensor
        eps_t = torch.tensor(eps)
        for p, (cls, first, nm) in zip(plan.params, plan.views):
            u = cls.U[first:first + nm].view(p.shape)
            x = u
            if plan.flatten and u.ndim >= 3:
                x = u.flatten(start_dim=1)
            elif u.ndim >= 4:
                x = u.flatten(end_dim=-3)
            u.copy_(self._newton_schulz_func(x, epsilon=eps_t).reshape(p.shape))

    # ------------------------------------------------------------------ lion / adamw
    def _lion_group_step(self, gi: int, group: dict) -> None:
        params = [p for p in group["params"] if p.grad is not None]
        if not params:
            return
        moms = [self._get_or_initialize_state(p, "lion")["momentum"] for p in params]
        grads = [g if g.is_contiguous() else g.contiguous() for g in to_local([p.grad for p in params])]
        scalar_opts.lion_update_foreach(
            to_local(params), grads, to_local(moms), float(group["lr"]),
            float(group["beta1"]), float(group["beta2"]), float(group["weight_decay"]), bool(group["cautious_wd"]),
            key=("lion", tuple(id(p) for p in params)), cache=self._scalar_plans, hyper_dev=self._hyper_ptr(gi, group))

    def _adamw_group_step(self, gi: int, group: dict) -> None:
        params = [p for p in group["params"] if p.grad is not None]
        if not params:
            return
        # hyperball applies to 2-D parameters that were not excluded (muon.py:399-413)
        if self.use_muonh:
            ball = [p for p in params if p.ndim == 2 and p not in self._hyperball_excluded]
            flat = [p for p in params if p.ndim != 2 or p in self._hyperball_excluded]
        else:
            ball, flat = [], params
        args = (float(group["lr"]), float(group["beta1"]), float(group["beta2"]), float(group["weight_decay"]),
                int(group["step"]), float(group["epsilon"]), bool(group["cautious_wd"]))
        for plist, fn in ((ball, scalar_opts.hyperball_adamw_update_foreach), (flat, scalar_opts.adamw_update_foreach)):
            if plist:
                states = [self._get_or_initialize_state(p, "adamw") for p in plist]
                grads = [g if g.is_contiguous() else g.contiguous() for g in to_local([p.grad for p in plist])]
                fn(to_local(plist), grads, to_local([s["momentum"] for s in states]),
                   to_local([s["variance"] for s in states]), *args,
                   key=("adamw", tuple(id(p) for p in plist)), cache=self._scalar_plans,
                   hyper_dev=self._hyper_ptr(gi, group))


def zeropower_via_newtonschulz5(G: Tensor, epsilon: Union[float, Tensor] = 1e-7) -> Tensor:
    """Same name and signature as lit_gpt/optim/muon.py:869-897; runs the HIP path."""
    return ns.zeropower_via_newtonschulz5(G, epsilon)
