"""ctypes binding of the gfx950 shared library (include/archscale_muon.h).

There is no fallback: if the library is missing or a call fails, this raises.
"""
from __future__ import annotations

import ctypes
import math
import os
import threading
from typing import Dict, Optional, Sequence, Tuple

import numpy as np
import torch

from .build import LIB_PATH

# enums of include/archscale_muon.h
DTYPE_BF16, DTYPE_F32 = 0, 1
EPS_ADD, EPS_CLAMP = 0, 1
PREC_BF16, PREC_BF16_BSPLIT, PREC_F16 = 0, 1, 2
ALGO_ADAMW, ALGO_LION = 0, 1
RETRACT_HARD, RETRACT_DYNAMIC = 0, 1
SN_TRANSPOSED = 1
NS_CAST_INPUT_FIRST = 1
NS_NO_NORMALIZE = 2
NS_NO_DIAG_FOLD = 4
NS_NO_GRAM_TAIL = 8
NS_GRAM_TAIL = 16
CHUNK_ELEMS = 8192
NS_STATIC_SCRATCH_BYTES = 64 << 20
STREAM_COPY, STREAM_READ, STREAM_MIX = 0, 1, 2
E_STATIC_LIMIT = -4
PROF_KEY_MOMENTUM_LAYOUT = 90000
ABI_VERSION = 3

#: numpy layouts of muon_pre_item / muon_post_item (natural C alignment)
PRE_ITEM = np.dtype(
    [("g", "<u8"), ("m", "<u8"), ("u", "<u8"), ("w", "<u8"), ("numel", "<i8"),
     ("g_dtype", "<i4"), ("m_dtype", "<i4"), ("u_dtype", "<i4"), ("w_dtype", "<i4")], align=True)
POST_ITEM = np.dtype(
    [("w", "<u8"), ("u", "<u8"), ("numel", "<i8"), ("lr_ratio", "<f4"), ("w_dtype", "<i4")], align=True)
SCALAR_ITEM = np.dtype(
    [("w", "<u8"), ("g", "<u8"), ("m", "<u8"), ("v", "<u8"), ("numel", "<i8"),
     ("w_dtype", "<i4"), ("g_dtype", "<i4"), ("m_dtype", "<i4"), ("v_dtype", "<i4")], align=True)
BALL_ITEM = np.dtype(
    [("w", "<u8"), ("phi", "<u8"), ("sigma", "<u8"), ("ld_w", "<i8"), ("ld_phi", "<i8"), ("rows", "<i4"), ("cols", "<i4"),
     ("radius", "<f4"), ("lr_ratio", "<f4"), ("w_dtype", "<i4"), ("reserved", "<i4")], align=True)
#: muon_hyper: the hyper-parameter block the *_dev entry points read from device memory
HYPER = np.dtype([("lr", "<f4"), ("lr_wd", "<f4"), ("eps", "<f4"), ("w1", "<f4"), ("w2", "<f4"), ("bias1", "<f4"),
                  ("bias2_sqrt", "<f4"), ("cautious", "<i4")], align=True)
assert HYPER.itemsize == 32
assert PRE_ITEM.itemsize == 56 and POST_ITEM.itemsize == 32 and SCALAR_ITEM.itemsize == 56 and BALL_ITEM.itemsize == 64


class NsProblem(ctypes.Structure):
    """muon_ns_problem of include/archscale_muon.h."""
    _fields_ = [("in_ptr", ctypes.c_void_p), ("out_ptr", ctypes.c_void_p),
                ("in_batch_stride", ctypes.c_int64), ("out_batch_stride", ctypes.c_int64),
                ("in_dtype", ctypes.c_int32), ("in_ld", ctypes.c_int32), ("out_ld", ctypes.c_int32),
                ("batch", ctypes.c_int32), ("rows", ctypes.c_int32), ("cols", ctypes.c_int32)]


class SnProblem(ctypes.Structure):
    """muon_sn_problem of include/archscale_muon.h."""
    _fields_ = [("w_ptrs", ctypes.POINTER(ctypes.c_void_p)), ("sigma_out", ctypes.c_void_p),
                ("dtype", ctypes.c_int32), ("ld", ctypes.c_int32), ("batch", ctypes.c_int32),
                ("rows", ctypes.c_int32), ("cols", ctypes.c_int32), ("flags", ctypes.c_int32)]


class MnsProblem(ctypes.Structure):
    """muon_mns_problem of include/archscale_muon.h."""
    _fields_ = [("g_ptrs", ctypes.POINTER(ctypes.c_void_p)), ("m_ptrs", ctypes.POINTER(ctypes.c_void_p)),
                ("w_ptrs", ctypes.POINTER(ctypes.c_void_p)), ("out", ctypes.c_void_p),
                ("out_batch_stride", ctypes.c_int64), ("out_ld", ctypes.c_int32),
                ("g_dtype", ctypes.c_int32), ("m_dtype", ctypes.c_int32), ("w_dtype", ctypes.c_int32),
                ("batch", ctypes.c_int32), ("rows", ctypes.c_int32), ("cols", ctypes.c_int32),
                ("reserved", ctypes.c_int32)]


class MuonLibraryError(RuntimeError):
    """The HIP library is missing, has the wrong ABI, or a call into it failed."""


_lock = threading.Lock()
_lib: Optional[ctypes.CDLL] = None

_SIGNATURES = {
    "muon_abi_version": (ctypes.c_int, []),
    "muon_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "muon_ns_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int] * 4),
    "muon_ns_batched": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
        ctypes.c_void_p, ctypes.c_int64, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.POINTER(ctypes.c_float), ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "muon_ns_batched_static": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
        ctypes.c_void_p, ctypes.c_int64, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.POINTER(ctypes.c_float), ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_void_p]),
    "muon_ns_grouped_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(NsProblem), ctypes.c_int, ctypes.c_int]),
    "muon_ns_grouped": (ctypes.c_int, [
        ctypes.POINTER(NsProblem), ctypes.c_int,
        ctypes.POINTER(ctypes.c_float), ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "muon_momentum_ns_grouped": (ctypes.c_int, [
        ctypes.POINTER(MnsProblem), ctypes.c_int,
        ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_float,
        ctypes.POINTER(ctypes.c_float), ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "muon_ns_flops": (None, [ctypes.c_int] * 5 + [ctypes.POINTER(ctypes.c_double)] * 3),
    "muon_ns_ksplit_info": (None, [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_int)]),
    "muon_profile_begin": (ctypes.c_int, []),
    "muon_profile_collect": (ctypes.c_int, [
        ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_double),
        ctypes.POINTER(ctypes.c_double), ctypes.c_int]),
    "muon_scalar_update": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_int,
        ctypes.c_void_p, ctypes.c_void_p]),
    "muon_calibration_copy": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "muon_calibration_stream": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                               ctypes.c_size_t, ctypes.c_void_p]),
    "muon_syrk_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int] * 3),
    "muon_syrk": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_int64, ctypes.c_int,
        ctypes.c_void_p, ctypes.c_int64, ctypes.c_int,
        ctypes.c_void_p, ctypes.c_int64, ctypes.c_int,
        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float,
        ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "muon_momentum": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
        ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_void_p]),
    "muon_update_plain": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
        ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_void_p]),
    "muon_muonh_scratch_floats": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int]),
    "muon_update_muonh": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
        ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]),
    "muon_update_plain_dev": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]),
    "muon_update_muonh_dev": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]),
    "muon_scalar_update_dev": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
        ctypes.c_void_p, ctypes.c_void_p]),
    "muon_spectral_norm_workspace_bytes": (ctypes.c_size_t, [ctypes.POINTER(SnProblem), ctypes.c_int]),
    "muon_spectral_norm": (ctypes.c_int, [
        ctypes.POINTER(SnProblem), ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "muon_power_iteration": (ctypes.c_int, [
        ctypes.POINTER(ctypes.c_void_p), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "muon_ball_apply": (ctypes.c_int, [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_int,
        ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def lib() -> ctypes.CDLL:
    """Load the shared library once; raise if it is not built or has another ABI."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise MuonLibraryError(
                f"{LIB_PATH} is not built; run `python -m archscale_amd.build` (needs hipcc). "
                "There is no PyTorch or CPU fallback for the Muon kernels.")
        try:
            handle = ctypes.CDLL(LIB_PATH)
        except OSError as e:  # pragma: no cover - depends on the machine
            raise MuonLibraryError(f"cannot load {LIB_PATH}: {e}") from e
        for name, (res, args) in _SIGNATURES.items():
            try:
                fn = getattr(handle, name)
            except AttributeError as e:
                raise MuonLibraryError(f"{LIB_PATH} does not export {name}; rebuild it") from e
            fn.restype = res
            fn.argtypes = args
        got = handle.muon_abi_version()
        if got != ABI_VERSION:
            raise MuonLibraryError(f"{LIB_PATH} has ABI {got}, this package needs {ABI_VERSION}; rebuild it")
        _lib = handle
    return _lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = lib().muon_status_string(status).decode()
        if status < 0:
            raise ValueError(f"{what}: {msg}")
        raise MuonLibraryError(f"{what}: HIP error {status}: {msg}")


def hyper_record(lr: float, lr_wd: float, eps: float = 0.0, beta1: float = 0.0, beta2: float = 0.0, step: int = 1,
                 cautious: bool = False) -> np.ndarray:
    """One muon_hyper record with the derived fields computed exactly as the by-value entry points compute them
    (w1, w2 in float arithmetic on the float-rounded betas; the bias corrections in double, then rounded)."""
    rec = np.zeros(1, dtype=HYPER)
    b1, b2 = np.float32(beta1), np.float32(beta2)
    rec["lr"], rec["lr_wd"], rec["eps"] = lr, lr_wd, eps
    rec["w1"], rec["w2"] = np.float32(1.0) - b1, np.float32(1.0) - b2
    step = max(int(step), 1)
    rec["bias1"] = 1.0 - float(b1) ** step
    rec["bias2_sqrt"] = math.sqrt(1.0 - float(b2) ** step)
    rec["cautious"] = int(bool(cautious))
    return rec


def ns_bsplit_tail(t: int) -> int:
    """MUON_NS_BSPLIT_TAIL(t) of the header."""
    if not 0 <= t <= 255:
        raise ValueError(f"bsplit_tail must be in 0..255, got {t}")
    return t << 8


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.bfloat16:
        return DTYPE_BF16
    if dt == torch.float32:
        return DTYPE_F32
    raise TypeError(f"the Muon kernels take bfloat16 or float32 tensors, got {dt}")


def current_stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_cuda(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise MuonLibraryError(
            f"{what} is on {t.device}: the Muon kernels run on an AMD GPU only (no CPU fallback)")


# ---------------------------------------------------------------------------
# workspace: one growing byte buffer per (device, stream, tag); torch owns the memory.  The stream is part of the key
# because torch's allocator orders the reuse of a freed block only against the stream it was allocated on.
# ---------------------------------------------------------------------------
_workspaces: Dict[Tuple[int, int, str], torch.Tensor] = {}


def workspace(device: torch.device, nbytes: int, tag: str = "ns") -> torch.Tensor:
    """Scratch bytes for library calls issued on the current stream of ``device``."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    key = (index, torch.cuda.current_stream(device).cuda_stream, tag)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            del _workspaces[key]
            del buf
        buf = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


def release_workspaces() -> None:
    """Drop the cached workspaces (they are re-created on demand)."""
    _workspaces.clear()


_abc_cache: Dict[Tuple, ctypes.Array] = {}


def abc_array(coeffs: Sequence[Tuple[float, float, float]]):
    key = tuple((float(a), float(b), float(c)) for a, b, c in coeffs)
    arr = _abc_cache.get(key)
    if arr is None:
        flat = [v for row in key for v in row]
        arr = (ctypes.c_float * len(flat))(*flat)
        _abc_cache[key] = arr
    return arr


def ns_flops(batch: int, rows: int, cols: int, iters: int, prec_mode: int) -> Tuple[float, float, float]:
    """(dense, symmetric, issued) FLOP counts of one muon_ns_batched call."""
    d, s, i = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
    lib().muon_ns_flops(batch, rows, cols, iters, prec_mode, ctypes.byref(d), ctypes.byref(s), ctypes.byref(i))
    return d.value, s.value, i.value


def ns_ksplit_info(rows: int, cols: int):
    """((whole tiles, cut tiles, parts) for the reduction over the long side, the same for the short side) of one
    rows x cols matrix: how the library cuts its symmetric products along K (parts == 1: not at all)."""
    info = (ctypes.c_int * 6)()
    lib().muon_ns_ksplit_info(rows, cols, info)
    return tuple(info[:3]), tuple(info[3:])


def profile_begin() -> None:
    check(lib().muon_profile_begin(), "muon_profile_begin")


def profile_collect(capacity: int = 4096):
    """Per-launch records of the Newton-Schulz GEMMs since profile_begin():
    list of dicts {kind="gemm", ms, tile, mode, split, final, folded, flops_algorithmic, flops_issued} (``folded`` marks
    the X' = (B + aI) X launches that read no addend) and {kind="momentum_layout", ms, bytes} for the fused momentum
    launches (``bytes`` = algorithmic HBM bytes of the launch)."""
    ms = (ctypes.c_float * capacity)()
    key = (ctypes.c_int32 * capacity)()
    fa = (ctypes.c_double * capacity)()
    fi = (ctypes.c_double * capacity)()
    n = lib().muon_profile_collect(ms, key, fa, fi, capacity)
    if n < 0:
        raise MuonLibraryError(f"muon_profile_collect failed with {n}")
    out = []
    for i in range(min(n, capacity)):
        k = key[i]
        if k == PROF_KEY_MOMENTUM_LAYOUT:   # the fused momentum launch: the work fields carry bytes
            out.append(dict(kind="momentum_layout", ms=ms[i], bytes=fa[i]))
            continue
        out.append(dict(kind="gemm", ms=ms[i], tile=k // 100, mode=(k // 10) % 10, split=bool((k % 10) & 2),
                        final=bool((k % 10) & 1), folded=bool((k % 10) & 4), flops_algorithmic=fa[i], flops_issued=fi[i]))
    return out
