"""The benchmark configurations at FULL size on the GPU, checked through size-independent properties and against
the CPU oracle on sampled matrices (the oracle finishes those in seconds).

config 2: full MuonH step over the depth-16 dense parameter set (112 matrices, 721 M elements)
config 4: large-matrix NS5 on heavy-tailed gradients with zeroed rows (8192x8192, 4096x14336)
config 5: full MuonH step for the depth-24 MoE parameter set (6.3 G elements; 3-D expert stacks)
"""
import math

import pytest
import torch

from oracle import muon_oracle as O

pytestmark = pytest.mark.gpu

NS_TOL = 1e-2
W_TOL = 2e-2


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).norm() / b.norm()).item()


def _oracle_muonh(w, g, m, **kw):
    x, mm = w.clone(), m.clone()
    O.lit_gpt_muon_step(x, g, mm, lr=0.02, mu=0.95, wd=0.0, eps=1e-8, nesterov=True, adjust="spectral_norm",
                        flatten=False, cautious=False, use_muonh=True, **kw)
    return x, mm


def test_config2_full_step(gpu_device):
    from archscale_amd.optim.muon import Muon
    layer = [(2048, 2048), (512, 2048), (512, 2048), (2048, 2048), (5632, 2048), (5632, 2048), (2048, 5632)]
    g = torch.Generator(device=gpu_device).manual_seed(1236)
    params, grads = [], []
    for _ in range(16):
        for s in layer:
            params.append(torch.nn.Parameter((torch.randn(*s, generator=g, device=gpu_device) * 0.02).to(torch.bfloat16)))
            grads.append((torch.randn(*s, generator=g, device=gpu_device) * 1e-3).to(torch.bfloat16))
    for p, gr in zip(params, grads):
        p.grad = gr
    opt = Muon(params, lr=0.02, mu=0.95, weight_decay=0.0, epsilon=1e-8, nesterov=True, use_muonh=True)
    # every kind of matrix of a layer (Wq, Wk, Wv, Wo, W1, W3, W2), early, middle and late layers
    sample = [0, 1, 6, 4, 2 * 7 + 5, 7 * 7 + 3, 8 * 7 + 3, 59, 12 * 7 + 2, 15 * 7 + 0, 15 * 7 + 5, 111]
    w0 = {i: params[i].detach().cpu().clone() for i in sample}
    norms0 = torch.stack([p.detach().float().norm() for p in params])
    # two steps, so that the second one runs with momentum != gradient
    opt.step()
    w1 = {i: params[i].detach().cpu().clone() for i in sample}
    m1 = {i: opt.state[params[i]]["momentum"].detach().cpu().clone() for i in sample}
    norms1 = torch.stack([p.detach().float().norm() for p in params])
    opt.step()
    torch.cuda.synchronize()
    norms2 = torch.stack([p.detach().float().norm() for p in params])
    # hypersphere: every matrix keeps its Frobenius norm (bf16 weights: rounding noise only)
    assert ((norms1 / norms0 - 1).abs().max().item() < 2e-3) and ((norms2 / norms0 - 1).abs().max().item() < 3e-3)
    for i in sample:
        x1, mm1 = _oracle_muonh(w0[i], grads[i].cpu(), torch.zeros_like(w0[i]), ns_storage="fp32")
        assert _rel(w1[i], x1) <= W_TOL
        assert _rel(w1[i], x1) < 0.3 * _rel(w0[i], x1)        # the step is really there (a no-op sits at ~lr)
        assert _rel(m1[i], mm1) < 1e-6
        # second step from the GPU's own state after step 1
        x2, _ = _oracle_muonh(w1[i], grads[i].cpu(), m1[i], ns_storage="fp32")
        assert _rel(params[i].detach(), x2) <= W_TOL
        assert _rel(params[i].detach(), x2) < 0.3 * _rel(w1[i], x2)
    assert opt.param_groups[0]["step"] == 2


def _heavy_tailed(shape, seed):
    """Student-t(df=3) scaled to std 1e-3, 1 % of the rows zeroed (exercises the norm epsilon and fp32 accumulation)."""
    g = torch.Generator().manual_seed(seed)
    z = torch.randn(*shape, generator=g)
    chi = torch.randn(3, *shape, generator=g).square().sum(0)
    t = z / (chi / 3).sqrt() / math.sqrt(3.0) * 1e-3
    rows = torch.randperm(shape[0], generator=g)[: max(1, shape[0] // 100)]
    t[rows] = 0
    return t.to(torch.bfloat16), rows


@pytest.mark.parametrize("shape,seed", [((4096, 14336), 1238), ((8192, 8192), 1239)])
@pytest.mark.parametrize("table", ["quintic", "simple"])
def test_config4_large_heavy_tailed(gpu_device, shape, seed, table):
    import archscale_amd.optim.newton_schulz_hip as H
    G, zero_rows = _heavy_tailed(shape, seed)
    coeffs = O.coefficient_schedule(table, 5)
    got = H.newton_schulz(G.to(gpu_device), coeffs, 1e-7, prec="bsplit" if table == "simple" else "bf16")
    torch.cuda.synchronize()
    got = got.cpu()
    assert torch.all(got[zero_rows] == 0)
    assert torch.isfinite(got.float()).all()
    # full fp32 oracle on the host (seconds for 4096x14336, under a minute for 8192^2)
    want = O.newton_schulz(G, coeffs, 1e-7, storage="fp32")
    assert _rel(got, want) <= NS_TOL
    # squared row norms are the diagonal of O O^T = U p(S)^2 U^T: bounded by the square of the band's upper end,
    # and their sum is the number of singular values pushed to ~1 (the rank, here the non-zero rows)
    sq = got.float().square().sum(dim=1)
    assert sq.max().item() <= 1.25 ** 2
    rank = shape[0] - len(zero_rows)
    assert 0.6 * rank <= sq.sum().item() <= 1.25 ** 2 * rank


def test_config5_moe_full_step(gpu_device):
    """24 layers x {Wq, Wo 3072^2; Wk, Wv 768x3072; shared W1, W3 1536x3072, W2 3072x1536; routed experts
    (64, 768, 3072) and (64, 3072, 384)}: 6.34 G elements in bf16. Reports step time and HBM footprint."""
    from archscale_amd.optim.muon import Muon
    free, total = torch.cuda.mem_get_info()
    if free < 150 << 30:
        pytest.skip("needs ~110 GiB of free HBM")
    layer = [(3072, 3072), (768, 3072), (768, 3072), (3072, 3072), (1536, 3072), (1536, 3072), (3072, 1536),
             (64, 768, 3072), (64, 3072, 384)]
    g = torch.Generator(device=gpu_device).manual_seed(1240)
    params, grads = [], []
    for _ in range(24):
        for s in layer:
            params.append(torch.nn.Parameter((torch.randn(*s, generator=g, device=gpu_device) * 0.02).to(torch.bfloat16)))
            grads.append((torch.randn(*s, generator=g, device=gpu_device) * 1e-3).to(torch.bfloat16))
    n_elem = sum(p.numel() for p in params)
    assert n_elem == 24 * (2 * 3072 ** 2 + 2 * 768 * 3072 + 3 * 1536 * 3072 + 64 * 768 * 3072 + 64 * 3072 * 384)
    for p, gr in zip(params, grads):
        p.grad = gr
    opt = Muon(params, lr=0.02, mu=0.95, weight_decay=0.0, epsilon=1e-8, nesterov=True, use_muonh=True,
               muonh_per_matrix=True)
    sample = [(0, None), (6, None), (7, 5), (8, 63), (9 * 23 + 7, 0), (9 * 23 + 8, 31)]
    w0 = {}
    for i, e in sample:
        w0[(i, e)] = (params[i] if e is None else params[i][e]).detach().cpu().clone()
    n0 = params[7].detach().float().flatten(1).norm(dim=1)
    torch.cuda.synchronize()
    opt.step()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    opt.step()
    ev1.record()
    torch.cuda.synchronize()
    ms = ev0.elapsed_time(ev1)
    peak = torch.cuda.max_memory_allocated() / 2 ** 30
    print(f"config 5: {n_elem / 1e9:.2f} G elements, second step {ms:.1f} ms, peak HBM allocated {peak:.1f} GiB", flush=True)
    n2 = params[7].detach().float().flatten(1).norm(dim=1)
    assert (n2 / n0 - 1).abs().max().item() < 3e-3          # every expert keeps its own norm
    for i, e in sample:
        gr = (grads[i] if e is None else grads[i][e]).cpu()
        x1, m1 = _oracle_muonh(w0[(i, e)], gr, torch.zeros_like(gr), ns_storage="fp32")
        x2, _ = _oracle_muonh(x1, gr, m1, ns_storage="fp32")
        got = (params[i] if e is None else params[i][e]).detach()
        # two steps of 2e-2 each: the oracle chain and the GPU chain stay within the single-step bar of each other
        assert _rel(got, x2) <= W_TOL
        assert _rel(got, x2) < 0.3 * _rel(w0[(i, e)], x2)


@pytest.mark.parametrize("config,shapes", [
    ("config 2", [(512, 2048), (2048, 2048), (2048, 5632), (5632, 2048)]),
    ("config 5", [(768, 3072), (3072, 1536), (3, 768, 3072), (3, 3072, 384)]),
])
def test_singular_values_land_in_the_band(gpu_device, config, shapes):
    """One matrix of every shape class of the depth-16 and depth-24 parameter sets through ONE grouped Newton-Schulz call
    (the launch pattern of the optimizer step, classes of different tile counts and K in the same launches): each result
    within 1e-2 of the fp32 oracle, and its singular values inside the band that the scalar map of the production
    table assigns to the input's normalised spectrum (lit_gpt/optim/muon.py:875-897)."""
    import archscale_amd.optim.newton_schulz_hip as H
    g = torch.Generator().manual_seed(1243)
    ins = [(torch.randn(*s, generator=g) * 1e-3).to(torch.bfloat16) for s in shapes]
    outs = H.newton_schulz_grouped([x.to(gpu_device) for x in ins], O.QUINTIC, 1e-7)
    torch.cuda.synchronize()
    for x, o in zip(ins, outs):
        mats_in = x if x.ndim == 3 else x[None]
        mats_out = (o if o.ndim == 3 else o[None]).cpu()
        for gi, go in zip(mats_in, mats_out):
            want = O.newton_schulz(gi, O.QUINTIC, 1e-7, storage="fp32")
            err = _rel(go, want)
            s_in = torch.linalg.svdvals(gi.double()) / gi.double().norm()
            band = O.ns_singular_value_map(s_in, O.QUINTIC)
            s_out = torch.linalg.svdvals(go.double())
            print(config, tuple(gi.shape), "err", err, "sv", s_out.min().item(), s_out.max().item(), "band",
                  band.min().item(), band.max().item(), flush=True)
            assert err <= NS_TOL
            assert s_out.min().item() >= band.min().item() - 0.02 and s_out.max().item() <= band.max().item() + 0.02


def test_config2_muon_ball_full_step(gpu_device):
    """MuonBall over the depth-16 dense parameter set (112 matrices): 50 power-iteration rounds, hard retraction,
    msign with the polar-express table. Sampled matrices against the CPU oracle, every matrix against the sphere."""
    from archscale_amd.emerging import MuonBall
    from oracle import muon_ball_oracle as B
    layer = [(2048, 2048), (512, 2048), (512, 2048), (2048, 2048), (5632, 2048), (5632, 2048), (2048, 5632)]
    g = torch.Generator(device=gpu_device).manual_seed(1241)
    params, grads = [], []
    for _ in range(16):
        for s in layer:
            params.append(torch.nn.Parameter((torch.randn(*s, generator=g, device=gpu_device) * 0.02).to(torch.bfloat16)))
            grads.append((torch.randn(*s, generator=g, device=gpu_device) * 1e-3).to(torch.bfloat16))
    for p, gr in zip(params, grads):
        p.grad = gr
    lr = 0.02
    opt = MuonBall(params, lr=lr, momentum_beta=0.95, weight_decay=0.0, use_nesterov=True, power_iteration_steps=50,
                   msign_steps=5)
    sample = [1, 6, 4, 59]
    w0 = {i: params[i].detach().cpu().clone() for i in sample}
    opt.step()
    torch.cuda.synchronize()
    for i in sample:
        x, m = w0[i].clone(), torch.zeros_like(w0[i])
        B.muon_ball_step(x, grads[i].cpu().clone(), m, lr=lr, beta=0.95, wd=0.0, nesterov=True, wd_method="decoupled",
                         radius_mode="spectral_mup", scale_mode="align_adamw_rms", power_iteration_steps=50, msign_steps=5,
                         retract_mode="hard", retract_alpha=0.05, ns_storage="fp32", sigma_fn=B.power_iteration_fp64)
        assert _rel(params[i].detach(), x) <= W_TOL
        assert _rel(opt.state[params[i]]["momentum_buffer"], m) < 1e-2          # bf16 state
    # every matrix: spectral norm R up to the size of the update, lr * scale * |msign| <= lr * 0.2 sqrt(max dim) * 1.2
    for p in params[:14]:
        rows, cols = p.shape
        R = math.sqrt(rows / cols)
        top = torch.linalg.matrix_norm(p.detach().float(), ord=2).item()
        assert abs(top - R) <= lr * 0.2 * math.sqrt(max(rows, cols)) * 1.2 + 0.02 * R
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(3):
        opt.step()
    ev1.record()
    torch.cuda.synchronize()
    print(f"config 2 MuonBall: {ev0.elapsed_time(ev1) / 3:.1f} ms/step (50 power-iteration rounds, msign 5 steps)", flush=True)


def test_config2_emerging_muon_full_step(gpu_device):
    """emerging_optimizers-style Muon (EMA momentum, polar-express msign, decoupled weight decay) over the depth-16
    dense parameter set in fp32 (msign takes fp32 only, spectral_ball_utils.py:25-74); sampled matrices against the CPU
    oracle, then the step time."""
    from archscale_amd.emerging import Muon as EMuon
    from oracle import muon_oracle as O
    layer = [(2048, 2048), (512, 2048), (512, 2048), (2048, 2048), (5632, 2048), (5632, 2048), (2048, 5632)]
    g = torch.Generator(device=gpu_device).manual_seed(1242)
    params, grads = [], []
    for _ in range(16):
        for s in layer:
            params.append(torch.nn.Parameter(torch.randn(*s, generator=g, device=gpu_device) * 0.02))
            grads.append(torch.randn(*s, generator=g, device=gpu_device) * 1e-3)
    for p, gr in zip(params, grads):
        p.grad = gr
    lr, beta, wd = 0.02, 0.95, 0.01
    opt = EMuon(params, lr=lr, momentum_beta=beta, weight_decay=wd, use_nesterov=True, num_ns_steps=5,
                scale_mode="spectral_mup")
    sample = [0, 1, 4, 6, 111]
    w0 = {i: params[i].detach().cpu().clone() for i in sample}
    opt.step()
    torch.cuda.synchronize()
    for i in sample:
        x, m = w0[i].clone(), torch.zeros_like(w0[i])
        O.emerging_muon_step(x, grads[i].cpu().clone(), m, lr=lr, beta=beta, wd=wd, nesterov=True, wd_method="decoupled",
                             steps=5, scale_mode="spectral_mup", extra_scale=1.0, ns_storage="fp32")
        assert _rel(params[i].detach(), x) <= W_TOL
        d_got, d_want = params[i].detach().float().cpu() - w0[i].float(), x.float() - w0[i].float()
        assert _rel(d_got, d_want) <= 2e-2         # fp32 weights: the delta carries the Newton-Schulz error only
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(3):
        opt.step()
    ev1.record()
    torch.cuda.synchronize()
    print(f"config 2 emerging Muon: {ev0.elapsed_time(ev1) / 3:.1f} ms/step (msign 5 steps, half-precision workspace)", flush=True)


def test_scalar_groups_throughput(gpu_device):
    """AdamW, hyperball-AdamW and Lion over the non-matrix tensors of the depth-16 model (token embedding and
    lm_head 50304 x 2048, 33 norm vectors), bf16 state: one multi-tensor launch each; prints the HBM rate against the
    bytes each algorithm has to move and checks it against a loose floor."""
    from archscale_amd.optim import scalar_opts as H
    dev = gpu_device
    g = torch.Generator(device=dev).manual_seed(5)
    shapes = [(50304, 2048), (50304, 2048)] + [(2048,)] * 33
    mk = lambda scale: [(torch.randn(*s, generator=g, device=dev) * scale).to(torch.bfloat16) for s in shapes]
    X, G, M = mk(0.02), mk(1e-3), mk(1e-3)
    V = [(torch.rand(*s, generator=g, device=dev) * 1e-6).to(torch.bfloat16) for s in shapes]
    n = sum(x.numel() for x in X)
    # bytes per element with bf16 everywhere: AdamW reads w,g,m,v and writes w,m,v; Lion reads w,g,m and writes w,m;
    # hyperball: pass 1 reads w,g,m,v and writes m,v, pass 2 reads w,m,v and writes w (2-D tensors only)
    cases = [
        ("adamw", 14, lambda step: H.adamw_update_foreach(X, G, M, V, 1e-3, 0.9, 0.95, 0.1, step, 1e-8, False)),
        ("lion", 10, lambda step: H.lion_update_foreach(X, G, M, 1e-4, 0.9, 0.99, 0.1, False)),
        ("hyperball", 20, lambda step: H.hyperball_adamw_update_foreach(X[:2], G[:2], M[:2], V[:2], 1e-3, 0.9, 0.95, 0.1,
                                                                       step, 1e-8, False)),
    ]
    for name, bpe, fn in cases:
        elems = n if name != "hyperball" else X[0].numel() * 2
        fn(1)
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for s in range(5):
            fn(2 + s)
        ev1.record()
        torch.cuda.synchronize()
        ms = ev0.elapsed_time(ev1) / 5
        rate = elems * bpe / (ms * 1e-3) / 1e12
        print(f"scalar groups {name}: {elems / 1e6:.0f} M elements, {ms:.3f} ms/step, {rate:.2f} TB/s of {bpe} B/elem", flush=True)
        assert all(torch.isfinite(x.float()).all() for x in X[:1])
        assert rate > 2.0
