#!/usr/bin/env python3
"""Benchmark of the Muon / MuonH hot path on one MI355X.

A "step" is one full MuonH optimizer step (momentum -> Newton-Schulz-5 -> hypersphere update) over every 2-D
weight of the depth-16 GQA transformer parameter set: 112 bf16 matrices, 721.4 M elements, seeded synthetic
weights N(0, 0.02^2) and gradients N(0, 1e-3^2), resident in HBM before the timed region.

Prints ONE JSON line: headline = matrix-core FLOPs that the step EXECUTES (the library's own count per GEMM launch:
whole tiles, upper triangles only, the products of the Gram-side tail as they are) over the wall time of the whole step
(GEMMs and HBM-bound kernels), so value / 2500 is the share of the bf16 peak that the whole step sustains; beside it the
dense-equivalent figure (what a GEMM library or the CPU path would execute: 5*(4 m^2 n + 2 m^3) per matrix), ms per
step, the same step with five plain iterations (no half-storage / Gram-side tail), the roofline of the dominant kernel
measured with HIP events per launch, and the CPU baseline (the oracle's eager-bf16 restatement of the reference's CPU
path) timed on a bounded sample in the same run.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
HBM_PEAK_GBS = 8000.0

LAYER_SHAPES = [  # one layer of the depth-16 config: Wq, Wk, Wv, Wo, W1, W3, W2
    (2048, 2048), (512, 2048), (512, 2048), (2048, 2048), (5632, 2048), (5632, 2048), (2048, 5632)]
N_LAYERS = 16


def dense_flops(shape, iters=5):
    m, n = min(shape), max(shape)
    return iters * (4.0 * m * m * n + 2.0 * m ** 3)


def sym_flops(shape, iters=5):
    m, n = min(shape), max(shape)
    return iters * (3.0 * m * m * n + 1.0 * m ** 3)


def make_tensors(device, seed, layers=N_LAYERS):
    g = torch.Generator(device=device).manual_seed(seed)
    params, grads = [], []
    for _ in range(layers):
        for s in LAYER_SHAPES:
            w = (torch.randn(*s, generator=g, device=device) * 0.02).to(torch.bfloat16)
            params.append(torch.nn.Parameter(w))
            grads.append((torch.randn(*s, generator=g, device=device) * 1e-3).to(torch.bfloat16))
    return params, grads


def cpu_baseline(coeffs_name, seed, budget_s=15.0):
    """The oracle (a port of the reference's eager CPU path: bf16 storage, every op rounds) on whole layers of
    the same workload, all host cores, until about ``budget_s`` seconds are spent (at most the full step)."""
    from oracle import muon_oracle as O
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(seed)
    coeffs = O.coefficient_schedule(coeffs_name, 5)
    kw = dict(lr=0.02, mu=0.95, wd=0.0, eps=1e-8, nesterov=True, adjust="spectral_norm", flatten=False,
              cautious=False, use_muonh=True, coeffs=coeffs, ns_storage="bf16_eager")
    warm = (torch.randn(512, 2048, generator=g) * 0.02).to(torch.bfloat16)
    O.lit_gpt_muon_step(warm, warm * 0.05, torch.zeros_like(warm), **kw)  # untimed warm-up
    spent, layers = 0.0, 0
    while layers < N_LAYERS and spent < budget_s:
        Ws = [(torch.randn(*s, generator=g) * 0.02).to(torch.bfloat16) for s in LAYER_SHAPES]
        Gs = [(torch.randn(*s, generator=g) * 1e-3).to(torch.bfloat16) for s in LAYER_SHAPES]
        Ms = [torch.zeros_like(w) for w in Ws]
        t0 = time.perf_counter()
        for w, gr, m in zip(Ws, Gs, Ms):
            O.lit_gpt_muon_step(w, gr, m, **kw)
        spent += time.perf_counter() - t0
        layers += 1
    flops = layers * sum(dense_flops(s) for s in LAYER_SHAPES)
    full_ms = spent / layers * N_LAYERS * 1e3
    return {
        "value": round(flops / spent / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": f"{layers} of {N_LAYERS} layers ({7 * layers} matrices, {flops / 1e12:.2f} TFLOP dense), one timed "
                  f"pass of the eager-bf16 oracle (the reference's CPU semantics), {spent:.1f} s of CPU work",
        "ms_per_step": round(full_ms, 1), "extrapolated": layers < N_LAYERS,
    }


def _gemm_summary(recs):
    """(ms, issued FLOPs, algorithmic FLOPs) summed over the GEMM launches of one instrumented call."""
    gem = [r for r in recs if r["kind"] == "gemm"]
    return (sum(r["ms"] for r in gem), sum(r["flops_issued"] for r in gem), sum(r["flops_algorithmic"] for r in gem))


def _time_calls(fn, reps, warm=2):
    """Average milliseconds of `fn` over `reps` back-to-back calls on the current stream."""
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def _instrumented(fn):
    from archscale_amd import _lib
    _lib.profile_begin()
    fn()
    torch.cuda.synchronize()
    return _lib.profile_collect()


def other_configs(dev, which):
    """The remaining benchmark configurations (1, 3, 4, 5) on the same code paths as the GPU tests: seeded synthetic
    inputs generated on the device, each timed by HIP events over several back-to-back calls, plus one instrumented call
    for the share of the bf16 matrix-core peak that the GEMM launches reach (issued FLOPs over their summed durations)."""
    from archscale_amd import _lib
    from archscale_amd.optim.muon import Muon
    import archscale_amd.optim.newton_schulz_hip as H
    out = {}

    def gen(shape, seed, scale):
        g = torch.Generator(device=dev).manual_seed(seed)
        return (torch.randn(*shape, generator=g, device=dev) * scale).to(torch.bfloat16)

    def pack(ms, shapes_counts, recs, **extra):
        dense = sum(c * dense_flops(s) for s, c in shapes_counts)
        gms, fi, fa = _gemm_summary(recs)
        d = {"ms": round(ms, 4), "executed_tflops": round(fi / ms / 1e9, 1), "dense_equivalent_tflops": round(dense / ms / 1e9, 1),
             "gemm_ms": round(gms, 4),
             "gemm_pct_mfma_peak_issued": round(fi / gms / 1e9 / MFMA_BF16_PEAK_TFLOPS * 100, 2) if gms else None,
             "gemm_pct_mfma_peak_algorithmic": round(fa / gms / 1e9 / MFMA_BF16_PEAK_TFLOPS * 100, 2) if gms else None}
        d.update(extra)
        return d

    def muonh_step_config(shapes, seed, reps):
        params = [torch.nn.Parameter(gen(s, seed + 2 * i, 0.02)) for i, s in enumerate(shapes)]
        for i, p in enumerate(params):
            p.grad = gen(tuple(p.shape), seed + 2 * i + 1, 1e-3)
        opt = Muon(params, lr=0.02, mu=0.95, weight_decay=0.0, epsilon=1e-8, nesterov=True, use_muonh=True,
                   muonh_per_matrix=True)
        ms = _time_calls(opt.step, reps)
        recs = _instrumented(opt.step)
        return ms, recs, sum(p.numel() for p in params)

    if 1 in which:   # one 512x2048 gradient, N(0,1), constant coefficient row x5, eps 1e-7 (legacy_optim.py:187-213)
        G = gen((512, 2048), 1235, 1.0)
        fn = lambda: H.zeropower_via_newtonschulz5_legacy(G, steps=5)
        ms = _time_calls(fn, 200, warm=5)
        out["config1"] = pack(ms, [((512, 2048), 1)], _instrumented(fn),
                              workload="NS5 of one 512x2048 matrix, constant coefficients, half-precision workspace")
    if 3 in which:   # 64 experts: stacked W1/W3 512x2048 and W2 2048x256, full MuonH step with per-expert norms
        ms, recs, n = muonh_step_config([(64, 512, 2048), (64, 2048, 256)], 1237, 100)
        out["config3"] = pack(ms, [((512, 2048), 64), ((2048, 256), 64)], recs, elements=n,
                              workload="full MuonH step, (64,512,2048) + (64,2048,256) expert stacks")
        _lib.release_workspaces()
    if 4 in which:   # NS5 of one large heavy-tailed matrix (Student-t df=3, std 1e-3, 1 % of the rows zeroed)
        for name, shape, seed in (("config4_8192x8192", (8192, 8192), 1239), ("config4_4096x14336", (4096, 14336), 1238)):
            g = torch.Generator(device=dev).manual_seed(seed)
            z = torch.randn(*shape, generator=g, device=dev)
            chi = torch.randn(3, *shape, generator=g, device=dev).square().sum(0)
            t = z / (chi / 3).sqrt() / (3.0 ** 0.5) * 1e-3
            t[torch.randperm(shape[0], generator=g, device=dev)[: shape[0] // 100]] = 0
            G = t.to(torch.bfloat16)
            del z, chi, t
            fn = lambda: H.zeropower_via_newtonschulz5(G, 1e-7)
            ms = _time_calls(fn, 10)
            out[name] = pack(ms, [(shape, 1)], _instrumented(fn), workload=f"NS5 of one {shape[0]}x{shape[1]} matrix, "
                             "production coefficients")
            del G
            _lib.release_workspaces()
            torch.cuda.empty_cache()
    if 5 in which and torch.cuda.mem_get_info(dev)[0] > (150 << 30):
        layer = [(3072, 3072), (768, 3072), (768, 3072), (3072, 3072), (1536, 3072), (1536, 3072), (3072, 1536),
                 (64, 768, 3072), (64, 3072, 384)]
        torch.cuda.reset_peak_memory_stats(dev)
        ms, recs, n = muonh_step_config(layer * 24, 1240, 5)
        counts = [((3072, 3072), 48), ((768, 3072), 48 + 24 * 64), ((1536, 3072), 72), ((3072, 384), 24 * 64)]
        out["config5"] = pack(ms, counts, recs, elements=n,
                              peak_hbm_allocated_gib=round(torch.cuda.max_memory_allocated(dev) / 2 ** 30, 1),
                              workload="full MuonH step, depth-24 MoE set (6.34 G elements, 64 routed experts per layer)")
        _lib.release_workspaces()
        torch.cuda.empty_cache()
    return out


TRAFFIC_PROFILE = "profiles/bench_config2_ns_gemm_and_epilogues.md"
GEMM_SOURCE = "archscale_amd/csrc/ns_gemm.hip"


def source_fingerprint(rel_path):
    """First 16 hex digits of the SHA-256 of a source file (what a counter summary records about the kernels it measured)."""
    import hashlib
    try:
        return hashlib.sha256(open(os.path.join(ROOT, rel_path), "rb").read()).hexdigest()[:16]
    except OSError:
        return None


def measured_traffic(kernel_name):
    """(HBM bytes per launch of `kernel_name`, fingerprint of the GEMM source the summary was measured with) from the
    committed counter summary (two `rocprofv3 --pmc` runs, FETCH_SIZE and WRITE_SIZE, each scaled by the reading of a
    plain copy of known size).  The byte count is None when the summary is missing or was measured with another version
    of the GEMM kernels than the one in the tree (a stale figure is not reported)."""
    path = os.path.join(ROOT, TRAFFIC_PROFILE)
    traffic, measured_with = None, None
    try:
        for line in open(path):
            line = line.strip()
            if line.startswith("traffic_bytes_per_launch") and kernel_name in line:
                traffic = float(line.split("=")[1])
            if line.startswith("measured_with_source_sha256_16") and GEMM_SOURCE in line:
                measured_with = line.split("=")[1].strip()
    except OSError:
        pass
    if measured_with is None or measured_with != source_fingerprint(GEMM_SOURCE):
        traffic = None
    return traffic, measured_with


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--coeffs", choices=["quintic", "simple"], default="quintic",
                    help="quintic = the reference's production 5-row schedule; simple = constant row with the B split")
    ap.add_argument("--layers", type=int, default=N_LAYERS, help="(debug) fewer layers; the result is then not the metric")
    ap.add_argument("--precision", choices=["bf16", "f16"], default="bf16",
                    help="storage of the iteration's matrices inside the Newton-Schulz workspace (inputs and outputs stay bf16)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--separate-momentum", action="store_true",
                    help="(comparison) momentum kernel and Newton-Schulz as separate library calls instead of the fused one")
    ap.add_argument("--no-plain-row", action="store_true",
                    help="skip the extra timing of the same step with five plain iterations (no half / Gram-side tail)")
    ap.add_argument("--seed", type=int, default=1236)
    ap.add_argument("--min-timed-seconds", type=float, default=2.0,
                    help="the block of --steps steps is repeated until the timed region is at least this long")
    ap.add_argument("--dump-launches", action="store_true", help="(debug) every timed launch of the instrumented step on stderr")
    ap.add_argument("--other-configs", default="1,3,4,5",
                    help="comma-separated benchmark configurations reported beside the headline (empty: none)")
    ap.add_argument("--only-config", type=int, default=0, choices=[0, 1, 3, 4, 5],
                    help="(profiling) run just this one of the other configurations and print its record instead of the headline line")
    ap.add_argument("--calibration-copy-mib", type=int, default=1024,
                    help="size of the plain device copy run once after the steps (yardstick for HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (every box here has one); --gpus must be 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")

    from archscale_amd import _lib
    from archscale_amd.optim.muon import Muon
    import archscale_amd.optim.newton_schulz_hip as H

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.only_config:
        print(json.dumps({"only_config": args.only_config, **other_configs(dev, [args.only_config])}))
        return
    params, grads = make_tensors(dev, args.seed, args.layers)
    for p, g in zip(params, grads):
        p.grad = g
    simple = args.coeffs == "simple"
    opt = Muon(params, lr=0.02, mu=0.95, weight_decay=0.0, epsilon=1e-8, nesterov=True, adjust_lr="spectral_norm",
               use_muonh=True, ns_coefficients=[H.SIMPLE_ROW] * 5 if simple else None,
               ns_precision=("f16" if args.precision == "f16" else "bsplit" if simple else "bf16"),
               fuse_momentum=not args.separate_momentum)

    for _ in range(args.warmup):  # also warms the momentum so that M != G
        opt.step()
    torch.cuda.synchronize()
    # the timed region: blocks of exactly --steps steps, repeated (whole blocks only) until at least
    # --min-timed-seconds have passed; ms_per_step is the mean over every timed step
    repeats, wall = 0, 0.0
    t0 = time.perf_counter()
    while True:
        for _ in range(args.steps):
            opt.step()
        torch.cuda.synchronize()
        repeats += 1
        wall = time.perf_counter() - t0
        if wall >= args.min_timed_seconds or repeats >= 1000:
            break
    ms_per_step = wall / (args.steps * repeats) * 1e3

    # one more, instrumented step: HIP events around every phase and every Newton-Schulz GEMM launch
    opt.phase_events = []
    _lib.profile_begin()
    opt.step()
    torch.cuda.synchronize()
    recs = _lib.profile_collect()
    if args.dump_launches:
        for r in recs:
            print(json.dumps({k: (round(v, 4) if isinstance(v, float) and k == "ms" else v) for k, v in r.items()}), file=sys.stderr)
    phases = {}
    for name, a, b in opt.phase_events:
        phases[name] = phases.get(name, 0.0) + a.elapsed_time(b)
    opt.phase_events = None

    # the same step with five plain iterations (no half-storage tail, no Gram-side finish): the figure that stays
    # comparable when the tail changes the amount of work
    plain_row = None
    if not args.no_plain_row and not simple and args.precision == "bf16":
        opt2 = Muon(params, lr=0.02, mu=0.95, weight_decay=0.0, epsilon=1e-8, nesterov=True, adjust_lr="spectral_norm",
                    use_muonh=True, ns_gram_tail=False, fuse_momentum=not args.separate_momentum)
        ms2 = _time_calls(opt2.step, args.steps, warm=2)
        gms2, fi2, fa2 = _gemm_summary(_instrumented(opt2.step))
        plain_row = {"ms_per_step": round(ms2, 3), "ns_gemm_ms": round(gms2, 3),
                     "issued_tflop_per_step": round(fi2 / 1e12, 3),
                     "executed_tflops": round(fi2 / ms2 / 1e9, 1),
                     "ns_gemm_pct_mfma_peak_issued": round(fi2 / gms2 / 1e9 / MFMA_BF16_PEAK_TFLOPS * 100, 2),
                     "what": "five plain bf16 iterations (ns_gram_tail=False): 15 GEMM launches, bf16 storage throughout"}
        del opt2

    # one plain copy of known size: `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE` readings are scaled by what the same
    # counter reports for this dispatch (calibration_copy_kernel)
    cal_bytes = args.calibration_copy_mib << 20
    if cal_bytes:
        src = torch.empty(cal_bytes, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        _lib.check(_lib.lib().muon_calibration_copy(src.data_ptr(), dst.data_ptr(), cal_bytes,
                                                    _lib.current_stream_ptr(dev)), "muon_calibration_copy")
        torch.cuda.synchronize()
        del src, dst

    # what the memory delivers to plain streaming kernels of known size on this GPU, right now: read-only, copy, and
    # the two-read / two-write mix of the fused momentum kernel (the HBM-bound kernels are reported beside these)
    yard = {}
    if cal_bytes:
        bufs = [torch.empty(cal_bytes, dtype=torch.uint8, device=dev).fill_(k + 1) for k in range(3)]
        for name, mode, moved in (("read", _lib.STREAM_READ, 1), ("copy", _lib.STREAM_COPY, 2), ("mix_2r2w", _lib.STREAM_MIX, 4)):
            fn = lambda: _lib.check(_lib.lib().muon_calibration_stream(mode, bufs[0].data_ptr(), bufs[1].data_ptr(),
                                                                       bufs[2].data_ptr(), cal_bytes,
                                                                       _lib.current_stream_ptr(dev)), "muon_calibration_stream")
            gbs = moved * cal_bytes / _time_calls(fn, 10) / 1e6
            yard[name] = {"GB/s": round(gbs), "frac": round(gbs / HBM_PEAK_GBS, 3)}
        del bufs

    shapes = [tuple(p.shape) for p in params]
    n_elem = sum(p.numel() for p in params)
    f_dense = sum(dense_flops(s) for s in shapes)
    f_sym = sum(sym_flops(s) for s in shapes)

    # dominant kernel: the X' = aX + BX product in its main (non-final) instantiation
    by_kernel = {}
    mom = [r for r in recs if r["kind"] == "momentum_layout"]
    recs = [r for r in recs if r["kind"] == "gemm"]
    for r in recs:
        k = (r["tile"], r["mode"], r["split"], r["final"], r["folded"])
        d = by_kernel.setdefault(k, dict(n=0, ms=0.0, fa=0.0, fi=0.0))
        d["n"] += 1; d["ms"] += r["ms"]; d["fa"] += r["flops_algorithmic"]; d["fi"] += r["flops_issued"]
    names = {0: "symprod", 1: "syrk2", 2: "bx", 3: "syrkt"}   # symprod: the m x m products of the Gram-side tail
    kernels = []
    for (tile, mode, split, final, folded), d in sorted(by_kernel.items(), key=lambda kv: -kv[1]["ms"]):
        kernels.append({
            "kernel": f"ns_gemm<{tile},{names[mode]}{',split' if split else ''}{',final' if final else ''}>",
            "addend": (not folded) if mode == 2 else None,
            "launches_per_step": d["n"], "avg_ms": round(d["ms"] / d["n"], 4),
            "algorithmic_tflops": round(d["fa"] / d["ms"] / 1e9, 1), "issued_tflops": round(d["fi"] / d["ms"] / 1e9, 1),
            "ms_per_step": round(d["ms"], 3)})
    # dominant kernel: the product (kernel mode) with the largest share of the step, in the instantiation that takes
    # most of that share
    ms_of_mode = {}
    for k, d in by_kernel.items():
        ms_of_mode[k[1]] = ms_of_mode.get(k[1], 0.0) + d["ms"]
    dom_mode = max(ms_of_mode, key=ms_of_mode.get)
    dom_key = max((k for k in by_kernel if k[1] == dom_mode), key=lambda k: by_kernel[k]["ms"])
    # the roofline line is per launch: of the dominant kernel's launches take those that cover every matrix (with the
    # Gram-side tail one launch of the last-but-one iteration covers only the classes that do not take it)
    dom_recs = [r for r in recs if (r["tile"], r["mode"], r["split"], r["final"], r["folded"]) == dom_key]
    full = max(r["flops_algorithmic"] for r in dom_recs)
    dom_recs = [r for r in dom_recs if r["flops_algorithmic"] >= 0.999 * full]
    dom = dict(n=len(dom_recs), ms=sum(r["ms"] for r in dom_recs), fa=sum(r["flops_algorithmic"] for r in dom_recs),
               fi=sum(r["flops_issued"] for r in dom_recs))
    achieved = dom["fa"] / dom["ms"] / 1e9
    roofline = {
        "bound": "mfma", "achieved": round(achieved, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
        "kernel": f"ns_gemm_kernel<{dom_key[0]},{names[dom_key[1]]}{',split' if dom_key[2] else ''}"
                  f"{',final' if dom_key[3] else ''}>",
        "algorithmic_bytes_per_launch": None,
        "launches": dom["n"], "avg_launch_ms": round(dom["ms"] / dom["n"], 4),
        "flops_per_launch": dom["fa"] / dom["n"],
        "issued_frac": round(dom["fi"] / dom["ms"] / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
    }
    if args.layers == N_LAYERS:
        roofline["traffic"], measured_with = measured_traffic(roofline["kernel"])
        # not measured in this run: counters need rocprofv3 passes of their own
        roofline["traffic_source"] = (f"{TRAFFIC_PROFILE} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, "
                                      "scaled by the calibration copy; committed summary, not measured in this run; "
                                      f"null when it was measured with another version of {GEMM_SOURCE})")
        roofline["traffic_measured_with_source"] = measured_with
        roofline["source_in_tree"] = source_fingerprint(GEMM_SOURCE)
    if dom_key[1] == 2:  # B (m^2), X^T read (once more as the addend unless a*I is folded into B), X'^T written: bf16
        reads_x = 1 if dom_key[4] else 2
        per = [(min(s) ** 2 + (reads_x + 1) * min(s) * max(s)) * 2.0 for s in shapes]
        roofline["algorithmic_bytes_per_launch"] = sum(per)   # one grouped launch covers every matrix
    gemm_ms = sum(d["ms"] for d in by_kernel.values())
    f_issued = sum(d["fi"] for d in by_kernel.values())
    hbm = {}
    bytes_per_elem = {"momentum": 8.0, "update_muonh": 10.0, "update_plain": 6.0}
    for name, ms in phases.items():
        if name in bytes_per_elem:
            gbs = n_elem * bytes_per_elem[name] / ms / 1e6
            hbm[name] = {"ms": round(ms, 3), "GB/s": round(gbs, 0), "frac": round(gbs / HBM_PEAK_GBS, 3),
                         "bytes_per_elem": bytes_per_elem[name]}
    if mom:   # fused momentum + layout launches (one per shape class), timed per launch inside the library call
        mms, mbytes = sum(r["ms"] for r in mom), sum(r["bytes"] for r in mom)
        hbm["momentum_layout"] = {"ms": round(mms, 3), "GB/s": round(mbytes / mms / 1e6, 0),
                                  "frac": round(mbytes / mms / 1e6 / HBM_PEAK_GBS, 3), "bytes_per_elem": 8.0,
                                  "launches": len(mom),
                                  "GB/s_per_launch": [round(r["bytes"] / r["ms"] / 1e6) for r in mom]}
    # per-product share of the bf16 matrix-core peak (issued / algorithmic FLOPs over the summed launch durations)
    kernel_fracs = {}
    for label, modes in (("syrkt", (3,)), ("syrk2", (1,)), ("symprod", (0,)), ("bx", (2,))):
        sel = [r for r in recs if r["mode"] in modes]
        if sel:
            t = sum(r["ms"] for r in sel)
            kernel_fracs[label] = {
                "issued_frac": round(sum(r["flops_issued"] for r in sel) / t / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
                "algorithmic_frac": round(sum(r["flops_algorithmic"] for r in sel) / t / 1e9 / MFMA_BF16_PEAK_TFLOPS, 4),
                "ms_per_step": round(t, 3)}
    ns_ms = sum(ms for n, ms in phases.items() if n.startswith("newton_schulz"))  # norms, layout and the 15 grouped GEMMs

    out = {
        "metric": "Muon NS5 TFLOP/s (% bf16 MFMA peak) + MuonH step ms, d16 param set, 1 GPU",
        "value": round(f_issued / ms_per_step / 1e9, 1),
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "timed_repeats": repeats, "timed_region_s": round(wall, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if args.precision == "f16" else "bf16", "data": "synthetic",
        "config": {"workload": f"config 2: full MuonH step, depth-{args.layers} GQA transformer, "
                               f"{len(params)} bf16 matrices, {n_elem / 1e6:.1f} M elements, "
                               f"mu 0.95 nesterov, NS5 {args.coeffs} coefficients, lr 0.02, seed {args.seed}",
                   "coefficients": args.coeffs,
                   "ns_precision": ("f16" if args.precision == "f16" else "bsplit" if simple else
                                    "bf16; last two iterations in IEEE half, finished on the Gram side for n >= 2m")},
        "value_definition": "matrix-core FLOPs the step EXECUTES (the library's count per GEMM launch: whole tiles, upper "
                            "triangles only, three quarters of a diagonal tile, the Gram-side tail's products as they "
                            "are) / wall time of the WHOLE step; value / 2500 is the share of the bf16 peak over the step",
        "pct_mfma_peak_whole_step": round(f_issued / ms_per_step / 1e9 / MFMA_BF16_PEAK_TFLOPS * 100, 2),
        "issued_tflop_per_step": round(f_issued / 1e12, 3),
        "symmetric_tflop_per_step": round(f_sym / 1e12, 3),
        "dense_tflop_per_step": round(f_dense / 1e12, 3),
        "dense_equivalent_tflops": round(f_dense / ms_per_step / 1e9, 1),
        "dense_equivalent_definition": "5*(4m^2n+2m^3) per matrix (what a GEMM library or the CPU path executes for five "
                                       "plain iterations) / wall time of the whole step: a speed-up yardstick against "
                                       "such a path, NOT a share of the peak (about 0.66 of these FLOPs are executed)",
        "plain_iterations": plain_row,
        "ns_gemm_pct_mfma_peak_issued": round(f_issued / gemm_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS * 100, 2),
        "ns_gemm_pct_mfma_peak_symmetric": round(f_sym / gemm_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS * 100, 2),
        "ns_gemm_ms": round(gemm_ms, 3), "ns_phase_ms": round(ns_ms, 3),
        "roofline": roofline,
        "kernel_fracs": kernel_fracs,
        "kernels": kernels,
        "hbm_kernels": hbm,
        "hbm_yardsticks": yard,
        "phases_ms": {k: round(v, 3) for k, v in phases.items()},
        "calibration_copy_bytes": cal_bytes,
    }
    which = [int(x) for x in args.other_configs.split(",") if x.strip()]
    if which and args.layers == N_LAYERS:
        # the headline's tensors are released first (config 5 needs 80 GiB of its own)
        del opt, params, grads, p, g
        _lib.release_workspaces()
        torch.cuda.empty_cache()
        try:
            out["other_configs"] = other_configs(dev, which)
        except Exception as e:   # the headline above stands on its own
            out["other_configs"] = {"error": f"{type(e).__name__}: {e}"}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.coeffs, args.seed)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
