"""muon_ns_batched_static (the entry point that allocates nothing) against muon_ns_batched, through the C ABI.

Both entry points run the same kernels; only the workspace differs (the library's built-in device array instead of a
caller buffer), so the results must be bit-identical.  Two calls in a row, the second on a smaller input, show that
nothing left in the shared array by one call reaches the next.
"""
import ctypes

import pytest
import torch

from oracle import muon_oracle as O

pytestmark = pytest.mark.gpu


def _randn(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


def _call(L, _lib, entry, x, coeffs, prec, eps=1e-7, ws=None):
    batch = x.shape[0] if x.ndim == 3 else 1
    rows, cols = x.shape[-2], x.shape[-1]
    out = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device)
    args = [x.data_ptr(), _lib.dtype_code(x.dtype), rows * cols, cols, out.data_ptr(), rows * cols, cols,
            batch, rows, cols, _lib.abc_array(coeffs), len(coeffs), eps, _lib.EPS_ADD, prec, _lib.NS_CAST_INPUT_FIRST]
    if entry == "static":
        st = L.muon_ns_batched_static(*args, _lib.current_stream_ptr(x.device))
    else:
        st = L.muon_ns_batched(*args, ws.data_ptr(), ws.numel(), _lib.current_stream_ptr(x.device))
    return st, out


@pytest.mark.parametrize("prec_name", ["bf16", "bsplit", "f16"])
def test_static_scratch_matches_caller_workspace(gpu_device, prec_name):
    from archscale_amd import _lib
    L = _lib.lib()
    prec = {"bf16": _lib.PREC_BF16, "bsplit": _lib.PREC_BF16_BSPLIT, "f16": _lib.PREC_F16}[prec_name]
    coeffs = O.coefficient_schedule("quintic" if prec_name == "bf16" else "simple", 5)
    # first a batch of ragged wide matrices, then a smaller tall one (the transposed layout, fewer tiles)
    for shape, seed in [((3, 320, 1100), 5), ((200, 136), 6)]:
        print("case", prec_name, shape, flush=True)
        x = _randn(shape, seed).to(gpu_device)
        batch = shape[0] if len(shape) == 3 else 1
        need = L.muon_ns_workspace_bytes(batch, shape[-2], shape[-1], prec)
        assert 0 < need <= _lib.NS_STATIC_SCRATCH_BYTES
        ws = torch.empty(need, dtype=torch.uint8, device=gpu_device)
        st, want = _call(L, _lib, "workspace", x, coeffs, prec, ws=ws)
        assert st == 0
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info(gpu_device)[0]
        st, got = _call(L, _lib, "static", x, coeffs, prec)
        assert st == 0, L.muon_status_string(st)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        ref = O.newton_schulz(x.cpu(), coeffs, 1e-7, storage="fp32")
        err = ((got.double().cpu() - ref.double()).norm() / ref.double().norm()).item()
        assert err <= 1e-2, err
        if seed == 6:   # the array's address is known by now: a call must leave the free device memory as it is
            assert torch.cuda.mem_get_info(gpu_device)[0] == free_before


def test_static_scratch_rejects_what_does_not_fit(gpu_device):
    from archscale_amd import _lib
    L = _lib.lib()
    coeffs = O.coefficient_schedule("quintic", 5)
    shape = (8, 2048, 2048)   # 8 matrices of 8 MiB: far beyond the 64 MiB array
    assert L.muon_ns_workspace_bytes(8, 2048, 2048, _lib.PREC_BF16) > _lib.NS_STATIC_SCRATCH_BYTES
    x = torch.zeros(shape, dtype=torch.bfloat16, device=gpu_device)
    st, out = _call(L, _lib, "static", x, coeffs, _lib.PREC_BF16)
    assert st == _lib.E_STATIC_LIMIT
    assert b"MUON_NS_STATIC_SCRATCH_BYTES" in L.muon_status_string(st)
    # bad extents are argument errors, as in muon_ns_batched
    abc = _lib.abc_array(coeffs)
    assert L.muon_ns_batched_static(x.data_ptr(), 0, 0, 0, out.data_ptr(), 0, 0, 0, 16, 16, abc, 5, 1e-7, 0, 0, 0, None) == -1


def test_static_scratch_calls_on_two_streams_take_turns(gpu_device):
    """Two streams that share the array without any host synchronisation between their calls: a call on another stream
    than the last one waits on the device for the end of that one, so neither sees the other's iterates."""
    from archscale_amd import _lib
    L = _lib.lib()
    coeffs = O.coefficient_schedule("quintic", 5)
    xs = [_randn((4, 256, 640), 11).to(gpu_device), _randn((2, 384, 512), 12).to(gpu_device)]
    want = []
    for x in xs:
        need = L.muon_ns_workspace_bytes(x.shape[0], x.shape[1], x.shape[2], _lib.PREC_BF16)
        ws = torch.empty(need, dtype=torch.uint8, device=gpu_device)
        st, w = _call(L, _lib, "workspace", x, coeffs, _lib.PREC_BF16, ws=ws)
        assert st == 0
        want.append(w)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = [None, None]
    for rep in range(3):
        for i in (0, 1, 1, 0):
            with torch.cuda.stream(streams[i]):
                st, got[i] = _call(L, _lib, "static", xs[i], coeffs, _lib.PREC_BF16)
                assert st == 0, L.muon_status_string(st)
        torch.cuda.synchronize()
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), rep


def test_static_scratch_call_replays_in_a_graph(gpu_device):
    """What the entry point is for: a call captured in a HIP graph (after one eager call, which looks the array up)
    allocates nothing and replays; every replay, with eager work and synchronisations in between, equals the eager
    result bit for bit (the input buffer is refilled before each replay)."""
    from archscale_amd import _lib
    L = _lib.lib()
    coeffs = O.coefficient_schedule("quintic", 5)
    shape = (3, 320, 1100)
    x = _randn(shape, 21).to(gpu_device)
    st, _ = _call(L, _lib, "static", x, coeffs, _lib.PREC_BF16)      # eager warm-up: address lookup happens here
    assert st == 0
    torch.cuda.synchronize()
    out = torch.empty(shape, dtype=torch.bfloat16, device=gpu_device)
    args = lambda stream: [x.data_ptr(), _lib.dtype_code(x.dtype), shape[1] * shape[2], shape[2], out.data_ptr(),
                           shape[1] * shape[2], shape[2], shape[0], shape[1], shape[2], _lib.abc_array(coeffs), len(coeffs),
                           1e-7, _lib.EPS_ADD, _lib.PREC_BF16, _lib.NS_CAST_INPUT_FIRST, stream]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        st = L.muon_ns_batched_static(*args(_lib.current_stream_ptr(gpu_device)))
    assert st == 0, L.muon_status_string(st)
    need = L.muon_ns_workspace_bytes(shape[0], shape[1], shape[2], _lib.PREC_BF16)
    ws = torch.empty(need, dtype=torch.uint8, device=gpu_device)
    for k in range(4):
        x.copy_(_randn(shape, 30 + k).to(gpu_device))
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        st, want = _call(L, _lib, "workspace", x, coeffs, _lib.PREC_BF16, ws=ws)     # eager work between the replays
        assert st == 0
        torch.cuda.synchronize()
        assert torch.equal(out, want), k
    del graph
