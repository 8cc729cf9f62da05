"""Parity of the Muon / MuonH optimizer step (HIP, through the C ABI) against the CPU oracle.

Bars (from the path's contract): updated weights within 2e-2 relative error of the reference step.
Because a MuonH step at lr 0.02 moves the weights by exactly 2e-2, W parity alone cannot see a
missing update, so every test also checks the weight DELTA (with fp32 weights, where it is meaningful).
"""
import copy
import math

import pytest
import torch

from oracle import muon_oracle as O

pytestmark = pytest.mark.gpu

W_TOL = 2e-2      # relative Frobenius error on updated weights (contract)
DW_TOL = 3e-2     # on the weight delta with fp32 weights: NS error (<= 1e-2) plus bf16 rounding of U


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def _make(shapes, dtype, seed, device, gdtype=None):
    g = torch.Generator().manual_seed(seed)
    ps = []
    for s in shapes:
        w = (torch.randn(*s, generator=g) * 0.02).to(dtype)
        p = torch.nn.Parameter(w.to(device))
        ps.append(p)
    return ps


def _grads(shapes, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(*s, generator=g) * 1e-3).to(dtype) for s in shapes]


SHAPES = [(128, 256), (256, 128), (128, 256), (64, 64), (3, 64, 192), (2, 192, 64)]


def _oracle_run(shapes, w0, grads_per_step, *, wdtype, hp, use_muonh, ns_storage, per_matrix=False):
    X = [w.clone().to(wdtype) for w in w0]
    M = [torch.zeros_like(x) for x in X]
    for grads in grads_per_step:
        for x, g, m in zip(X, grads, M):
            if use_muonh and per_matrix and x.ndim == 3:
                # per-matrix renormalisation = the reference applied to each expert as its own parameter
                U = O.muon_pre_orthogonalize(g, m, hp["mu"], hp["nesterov"])
                Oo = O.newton_schulz(U, O.QUINTIC, hp["eps"], storage=ns_storage).to(torch.bfloat16)
                for e in range(x.shape[0]):
                    O.muonh_post_orthogonalize(x[e], Oo[e], hp["lr"], hp["wd"], hp["eps"], hp["cautious"])
            else:
                O.lit_gpt_muon_step(x, g, m, lr=hp["lr"], mu=hp["mu"], wd=hp["wd"], eps=hp["eps"],
                                    nesterov=hp["nesterov"], adjust=hp["adjust"], flatten=False,
                                    cautious=hp["cautious"], use_muonh=use_muonh, ns_storage=ns_storage)
    return X, M


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("use_muonh", [False, True])
@pytest.mark.parametrize("wd,cautious", [(0.0, False), (0.1, True)])
def test_step_matches_oracle(gpu_device, wdtype, use_muonh, wd, cautious):
    from archscale_amd.optim.muon import Muon
    hp = dict(lr=0.02, mu=0.95, wd=wd, eps=1e-8, nesterov=True, adjust="spectral_norm", cautious=cautious)
    params = _make(SHAPES, wdtype, 1, gpu_device)
    w0 = [p.detach().cpu().clone() for p in params]
    opt = Muon(params, lr=hp["lr"], mu=hp["mu"], weight_decay=wd, cautious_wd=cautious, epsilon=hp["eps"],
               nesterov=True, adjust_lr="spectral_norm", use_muonh=use_muonh)
    steps = [_grads(SHAPES, wdtype, 100 + k) for k in range(3)]
    for grads in steps:
        for p, g in zip(params, grads):
            p.grad = g.to(gpu_device)
        opt.step()
    torch.cuda.synchronize()
    # reference semantics, bf16 eager NS (what the reference's CPU path computes)
    Xr, Mr = _oracle_run(SHAPES, w0, steps, wdtype=wdtype, hp=hp, use_muonh=use_muonh, ns_storage="bf16_eager")
    # the same step with the tolerance oracle for NS (fp32 on the same bf16 inputs)
    Xf, _ = _oracle_run(SHAPES, w0, steps, wdtype=wdtype, hp=hp, use_muonh=use_muonh, ns_storage="fp32")
    for p, xr, xf, w, mr in zip(params, Xr, Xf, w0, Mr):
        assert _rel(p.detach(), xr) <= W_TOL
        assert _rel(p.detach(), xf) <= W_TOL
        m = opt.state[p]["momentum"]
        assert m.dtype == p.dtype and _rel(m, mr) <= (1e-6 if wdtype == torch.float32 else 1e-2)
        if wdtype == torch.float32:
            dw, dwf = p.detach().cpu() - w, xf - w
            assert _rel(dw, dwf) <= DW_TOL
            if use_muonh:
                # norm preservation (after the decay, which is the only thing allowed to change the norm)
                assert p.detach().norm().item() == pytest.approx(xf.norm().item(), rel=1e-4)
    for g in opt.param_groups:
        assert g["step"] == 3


def test_muonh_per_matrix_and_whole_tensor(gpu_device):
    """A 3-D expert stack: the default renormalises the whole tensor (what the reference does for one
    3-D Parameter), ``muonh_per_matrix`` renormalises each expert."""
    from archscale_amd.optim.muon import Muon
    shapes = [(8, 64, 128), (8, 128, 32)]
    hp = dict(lr=0.05, mu=0.95, wd=0.0, eps=1e-8, nesterov=True, adjust="spectral_norm", cautious=False)
    grads = [_grads(shapes, torch.float32, 7)]
    for per_matrix in (False, True):
        params = _make(shapes, torch.float32, 2, gpu_device)
        # give the experts different scales so that the two conventions differ visibly
        with torch.no_grad():
            for p in params:
                p.mul_(torch.linspace(0.5, 2.0, 8, device=gpu_device).view(8, 1, 1))
        w0 = [p.detach().cpu().clone() for p in params]
        opt = Muon(params, lr=hp["lr"], mu=hp["mu"], weight_decay=0.0, nesterov=True, use_muonh=True,
                   muonh_per_matrix=per_matrix)
        for p, g in zip(params, grads[0]):
            p.grad = g.to(gpu_device)
        opt.step()
        Xf, _ = _oracle_run(shapes, w0, grads, wdtype=torch.float32, hp=hp, use_muonh=True, ns_storage="fp32",
                            per_matrix=per_matrix)
        for p, xf, w in zip(params, Xf, w0):
            assert _rel(p.detach().cpu() - w, xf - w) <= DW_TOL
            if per_matrix:
                for e in range(8):
                    assert p[e].norm().item() == pytest.approx(w[e].norm().item(), rel=1e-4)
            else:
                assert p.norm().item() == pytest.approx(w.norm().item(), rel=1e-4)
                assert max(abs(p[e].norm().item() / w[e].norm().item() - 1) for e in range(8)) > 1e-4


def test_batched_equals_one_by_one(gpu_device):
    """Shape-class batching must not change any tensor's result: one optimizer over all parameters
    equals one optimizer per parameter, bit for bit."""
    from archscale_amd.optim.muon import Muon
    grads = _grads(SHAPES, torch.bfloat16, 9)
    pa = _make(SHAPES, torch.bfloat16, 3, gpu_device)
    pb = _make(SHAPES, torch.bfloat16, 3, gpu_device)
    kw = dict(lr=0.02, nesterov=True, use_muonh=True, weight_decay=0.0)
    oa = Muon(pa, **kw)
    obs = [Muon([p], **kw) for p in pb]
    for _ in range(2):
        for p, q, g in zip(pa, pb, grads):
            p.grad = g.to(gpu_device)
            q.grad = g.to(gpu_device)
        oa.step()
        for o in obs:
            o.step()
    for p, q in zip(pa, pb):
        assert torch.equal(p, q)


def test_hook_state_dict_and_groups(gpu_device):
    from archscale_amd.optim.muon import Muon
    import archscale_amd.optim.newton_schulz_hip as H
    shapes = [(64, 128), (128, 64)]
    torch.manual_seed(4)      # the device-side draws below: the same values whichever tests ran before this one
    params = _make(shapes, torch.float32, 4, gpu_device)
    vec = torch.nn.Parameter(torch.randn(128, device=gpu_device))
    emb = torch.nn.Parameter(torch.randn(50, 64, device=gpu_device))
    head = torch.nn.Parameter(torch.randn(50, 64, device=gpu_device))
    calls = []

    def hook(X, epsilon):
        calls.append((tuple(X.shape), float(epsilon)))
        return H.newton_schulz_hip(X, epsilon)

    lion_vec = torch.nn.Parameter(torch.randn(32, device=gpu_device))
    groups = [dict(params=params), dict(params=[vec, emb, head], algorithm="adamw", lr=1e-3),
              dict(params=[lion_vec], algorithm="lion", lr=1e-3)]
    opt = Muon(groups, lr=0.02, nesterov=True, use_muonh=True, weight_decay=0.0, newton_schulz_func=hook)
    opt.exclude_from_hyperball(emb)
    ref = Muon(copy.deepcopy(groups), lr=0.02, nesterov=True, use_muonh=True, weight_decay=0.0, fuse_momentum=False)
    for p, q in zip(opt.param_groups[0]["params"], ref.param_groups[0]["params"]):
        g = torch.randn_like(p) * 1e-3
        p.grad, q.grad = g, g.clone()
    for p, q in zip(opt.param_groups[1]["params"], ref.param_groups[1]["params"]):
        g = torch.randn_like(p) * 1e-2
        p.grad, q.grad = g, g.clone()
    emb_norm, head_norm = emb.norm().item(), head.norm().item()
    opt.step()
    ref.step()
    assert sorted(calls) == sorted([((64, 128), 1e-8), ((128, 64), 1e-8)]) or len(calls) == 2
    for p, q in zip(opt.param_groups[0]["params"], ref.param_groups[0]["params"]):
        assert torch.equal(p, q)  # the hook runs the same kernels as the built-in path
    # hyperball AdamW keeps the norm of 2-D non-excluded tensors only
    assert head.norm().item() == pytest.approx(head_norm, rel=1e-5)
    assert abs(emb.norm().item() / emb_norm - 1) > 1e-6
    # state dict round trip
    sd = opt.state_dict()
    assert all("momentum" in s for s in sd["state"].values())
    assert sd["param_groups"][0]["step"] == 1 and sd["param_groups"][1]["algorithm"] == "adamw"
    opt2 = Muon(groups, lr=0.02, nesterov=True, use_muonh=True, weight_decay=0.0)
    opt2.load_state_dict(sd)
    assert opt2.param_groups[0]["step"] == 1
    for p in params:
        assert torch.equal(opt2.state[p]["momentum"], opt.state[p]["momentum"])
    # closure and unknown algorithm
    assert opt.step(lambda: torch.tensor(3.0)).item() == 3.0
    opt.param_groups[2]["algorithm"] = "sgd"
    with pytest.raises(ValueError):
        opt.step()


def test_first_step_and_missing_grads(gpu_device):
    from archscale_amd.optim.muon import Muon
    import archscale_amd.optim.newton_schulz_hip as H
    params = _make([(64, 128), (64, 128)], torch.float32, 5, gpu_device)
    w0 = [p.detach().clone() for p in params]
    opt = Muon(params, lr=0.1, mu=0.9, nesterov=True, weight_decay=0.0, adjust_lr=None)
    g = (torch.randn(64, 128, device=gpu_device) * 1e-3)
    params[0].grad = g
    opt.step()                       # params[1] has no grad: untouched, no state
    assert torch.equal(params[1], w0[1]) and len(opt.state[params[1]]) == 0
    # from zero momentum U = (1+mu) G, so the update is lr * NS(bf16((1+mu) G))
    ns_out = H.newton_schulz_hip(((1.9 * g)).to(torch.bfloat16), 1e-8).float()
    assert _rel(params[0].detach() - w0[0], -0.1 * ns_out) < 1e-2
    assert torch.allclose(opt.state[params[0]]["momentum"], g)


def test_emerging_muon_matches_oracle(gpu_device):
    from archscale_amd.emerging import Muon as EMuon
    shapes = [(64, 128), (128, 64), (64, 128)]
    for method, nesterov in (("decoupled", True), ("independent", False), ("l2", True)):
        params = _make(shapes, torch.float32, 6, gpu_device)
        w0 = [p.detach().cpu().clone() for p in params]
        opt = EMuon(params, lr=0.01, momentum_beta=0.9, weight_decay=0.1, use_nesterov=nesterov,
                    weight_decay_method=method, scale_mode="spectral_mup", extra_scale_factor=1.5)
        steps = [_grads(shapes, torch.float32, 40 + k) for k in range(2)]
        X = [w.clone() for w in w0]
        B = [torch.zeros_like(w) for w in w0]
        for grads in steps:
            for p, g in zip(params, grads):
                p.grad = g.clone().to(gpu_device)
            opt.step()
            for x, g, b in zip(X, grads, B):
                O.emerging_muon_step(x, g.clone(), b, lr=0.01, beta=0.9, wd=0.1, nesterov=nesterov,
                                     wd_method=method, steps=5, scale_mode="spectral_mup", extra_scale=1.5,
                                     ns_storage="fp32")
        for p, x, w, b in zip(params, X, w0, B):
            assert _rel(p.detach(), x) <= W_TOL
            assert _rel(p.detach().cpu() - w, x - w) <= DW_TOL
            # with l2 the gradient includes wd*p, so the buffer inherits the (tolerated) difference in p
            assert _rel(opt.state[p]["momentum_buffer"], b) <= (2e-3 if method == "l2" else 1e-5)
    with pytest.raises(ValueError):
        o = EMuon([torch.nn.Parameter(torch.randn(8, device=gpu_device))])
        o.param_groups[0]["params"][0].grad = torch.randn(8, device=gpu_device)
        o.step()


def test_emerging_hook_path(gpu_device):
    from archscale_amd.emerging import OrthogonalizedOptimizer, msign
    p = torch.nn.Parameter((torch.randn(64, 96) * 0.02).to(gpu_device))
    p.param_name = "blk.w"
    w0 = p.detach().clone()
    opt = OrthogonalizedOptimizer([p], 0.1, 0.9, 0.0, use_nesterov=False, weight_decay_method="decoupled",
                                  fp32_matmul_prec="medium", scaled_orthogonalize_fn=lambda g: msign(g, 5),
                                  log_per_module_update_rms=True, log_per_module_grad_rms=True)
    g = torch.randn(64, 96, device=gpu_device) * 1e-3
    p.grad = g
    opt.step()
    want = msign(0.1 * g, 5).float()
    assert _rel(p.detach() - w0, -0.1 * want) < 1e-2
    assert opt.get_update_rms_dict()["blk.w"] == pytest.approx(math.sqrt(1 / 96), rel=0.2)
    assert opt.get_grad_rms_dict()["blk.w"] == pytest.approx((0.1 * g).pow(2).mean().sqrt().item(), rel=1e-3)


def _sv_in_band(out, G, coeffs, tol=0.02):
    """Singular values of an orthogonalised matrix against the band that the scalar map of the coefficient table
    assigns to the normalised singular values of its input (lit_gpt/optim/muon.py:875-897 in exact arithmetic)."""
    s_in = torch.linalg.svdvals(G.double().cpu()) / G.double().cpu().norm()
    band = O.ns_singular_value_map(s_in, coeffs)
    s_out = torch.linalg.svdvals(out.double().cpu())
    return s_out.min().item() >= band.min().item() - tol and s_out.max().item() <= band.max().item() + tol


def test_config3_expert_batches(gpu_device):
    """64 experts, W1/W3 stacked 512x2048 and W2 2048x256 (tall => transposed), one batched launch per kernel, per-expert
    MuonH renormalisation (lit_gpt/optim/muon.py:309-322, 754-758 applied per expert).
    (i) the 64-batch 3-D Newton-Schulz call of either stack against the fp32 oracle on nine experts each, with the
        singular values in the band of the table;
    (ii) the full MuonH step with bf16 weights (the benchmark's configuration): weights within 2e-2 of the
        reference-semantics oracle (bf16 eager) and of the fp32-NS oracle, norms kept per expert;
    (iii) the same step with fp32 weights, where the weight DELTA is meaningful: within 3e-2 of the fp32-NS oracle."""
    from archscale_amd.optim.muon import Muon
    import archscale_amd.optim.newton_schulz_hip as H
    shapes = [(64, 512, 2048), (64, 2048, 256)]
    g = torch.Generator().manual_seed(1237)
    W = [(torch.randn(*s, generator=g) * 0.02).to(torch.bfloat16) for s in shapes]
    G = [(torch.randn(*s, generator=g) * 1e-3).to(torch.bfloat16) for s in shapes]
    experts = (0, 1, 9, 17, 26, 31, 40, 55, 63)
    # (i) at the first step the update that enters Newton-Schulz is the gradient times (1 + mu) (Nesterov, zero
    # momentum): the batched call on the gradients is the product's own NS input up to that factor
    for gr in G:
        got = H.newton_schulz(gr.to(gpu_device), O.QUINTIC, 1e-7)
        torch.cuda.synchronize()
        assert got.shape == gr.shape
        for e in experts:
            want = O.newton_schulz(gr[e], O.QUINTIC, 1e-7, storage="fp32")
            assert _rel(got[e], want) <= 1e-2, (tuple(gr.shape), e)
        for e in experts[:3]:
            assert _sv_in_band(got[e], gr[e], O.QUINTIC)
    for wdtype in (torch.bfloat16, torch.float32):
        params = [torch.nn.Parameter(w.to(wdtype).to(gpu_device)) for w in W]
        opt = Muon(params, lr=0.02, mu=0.95, nesterov=True, weight_decay=0.0, use_muonh=True, muonh_per_matrix=True)
        for p, gr in zip(params, G):
            p.grad = gr.to(wdtype).to(gpu_device)
        opt.step()
        torch.cuda.synchronize()
        for p, w, gr in zip(params, W, G):
            n_new = p.detach().float().flatten(1).norm(dim=1).cpu()
            n_old = w.float().flatten(1).norm(dim=1)
            assert ((n_new / n_old - 1).abs().max().item() < (2e-3 if wdtype == torch.bfloat16 else 1e-4))
            for e in experts:
                w0 = w[e].to(wdtype)
                xf = w0.clone()
                O.lit_gpt_muon_step(xf, gr[e].to(wdtype), torch.zeros_like(xf), lr=0.02, mu=0.95, wd=0.0, eps=1e-8,
                                    nesterov=True, adjust="spectral_norm", flatten=False, cautious=False,
                                    use_muonh=True, ns_storage="fp32")
                assert _rel(p[e].detach(), xf) <= W_TOL
                if wdtype == torch.float32:
                    assert _rel(p[e].detach().cpu() - w0, xf - w0) <= DW_TOL, (tuple(w.shape), e)
                elif e in experts[:3]:
                    xr = w0.clone()
                    O.lit_gpt_muon_step(xr, gr[e], torch.zeros_like(xr), lr=0.02, mu=0.95, wd=0.0, eps=1e-8,
                                        nesterov=True, adjust="spectral_norm", flatten=False, cautious=False,
                                        use_muonh=True, ns_storage="bf16_eager")
                    assert _rel(p[e].detach(), xr) <= W_TOL
                    # the update is really there: distance to the OLD weights is ~lr, to the new ones much less
                    assert _rel(p[e].detach(), xr) < 0.3 * _rel(w[e], xr)
        del opt, params


def test_step_replays_under_a_hip_graph(gpu_device):
    """In steady state step() is a fixed sequence of kernel launches on the current stream (no allocation, no host read,
    no table upload), so it can be captured once and replayed. Every replay is checked bit for bit against an eager twin,
    with eager work and synchronisations between the replays."""
    from archscale_amd.optim.muon import Muon
    shapes = [(128, 256), (256, 128), (128, 256), (2, 192, 64)]
    g = torch.Generator().manual_seed(77)
    W0 = [(torch.randn(*s, generator=g) * 0.02).to(torch.bfloat16) for s in shapes]
    pa = [torch.nn.Parameter(w.clone().to(gpu_device)) for w in W0]
    pb = [torch.nn.Parameter(w.clone().to(gpu_device)) for w in W0]
    static_g = [torch.zeros_like(p) for p in pa]
    for p, sg in zip(pa, static_g):
        p.grad = sg
    kw = dict(lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True, use_muonh=True)
    oa, ob = Muon(pa, **kw), Muon(pb, **kw)

    def new_grads(k):
        gg = torch.Generator().manual_seed(1000 + k)
        return [(torch.randn(*s, generator=gg) * 1e-3).to(torch.bfloat16).to(gpu_device) for s in shapes]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for k in range(2):                                   # warm-up: plans, tables and workspaces get built here
            for sg, gr in zip(static_g, new_grads(k)):
                sg.copy_(gr)
            oa.step()
    torch.cuda.current_stream().wait_stream(side)
    for k in range(2):
        for p, gr in zip(pb, new_grads(k)):
            p.grad = gr
        ob.step()
    graph = torch.cuda.CUDAGraph()
    for sg, gr in zip(static_g, new_grads(2)):
        sg.copy_(gr)
    with torch.cuda.graph(graph):
        oa.step()
    # capture does not execute: weights of the twin after two steps must equal the captured optimizer's
    for a, b in zip(pa, pb):
        assert torch.equal(a, b)
    for k in range(2, 6):
        for sg, gr in zip(static_g, new_grads(k)):
            sg.copy_(gr)
        graph.replay()
        for p, gr in zip(pb, new_grads(k)):
            p.grad = gr
        ob.step()
        junk = torch.randn(256, 256, device=gpu_device) @ torch.randn(256, 256, device=gpu_device)   # eager work in between
        torch.cuda.synchronize()
        assert torch.isfinite(junk).all()
        for a, b in zip(pa, pb):
            assert torch.equal(a, b), k
        for a, b in zip(pa, pb):
            assert torch.equal(oa.state[a]["momentum"], ob.state[b]["momentum"])


@pytest.mark.parametrize("wdtype,gdtype", [(torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32)])
@pytest.mark.parametrize("nesterov", [True, False])
def test_fused_momentum_equals_separate_calls(gpu_device, wdtype, gdtype, nesterov):
    """The call that feeds the momentum update straight into the Newton-Schulz operand against momentum kernel + batched
    Newton-Schulz: momentum buffers bit-identical; weights equal up to the one bf16 rounding of the normalised input that
    the fused path leaves out (it scales in the first iteration's epilogues instead)."""
    from archscale_amd.optim.muon import Muon
    shapes = [(128, 256), (256, 128), (128, 256), (64, 64), (3, 64, 192), (2, 192, 64), (300, 100), (100, 300), (37, 53)]
    g = torch.Generator().manual_seed(5)
    W0 = [(torch.randn(*s, generator=g) * 0.02).to(wdtype) for s in shapes]
    pa = [torch.nn.Parameter(w.clone().to(gpu_device)) for w in W0]
    pb = [torch.nn.Parameter(w.clone().to(gpu_device)) for w in W0]
    kw = dict(lr=0.02, mu=0.95, weight_decay=0.01, nesterov=nesterov, use_muonh=True)
    oa, ob = Muon(pa, fuse_momentum=True, **kw), Muon(pb, fuse_momentum=False, **kw)
    for step in range(3):
        grads = [(torch.randn(*s, generator=g) * 1e-3).to(gdtype).to(gpu_device) for s in shapes]
        for a, b, gr in zip(pa, pb, grads):
            a.grad, b.grad = gr.clone(), gr.clone()
        oa.step(); ob.step()
    assert oa._plans[0][1].fused_probs is not None
    for a, b, w0 in zip(pa, pb, W0):
        assert torch.equal(oa.state[a]["momentum"], ob.state[b]["momentum"])
        assert _rel(a.detach(), b.detach()) < 2e-3
        if wdtype == torch.float32:
            assert _rel(a.detach().cpu() - w0, b.detach().cpu() - w0) < 1e-2


def test_fused_momentum_falls_back(gpu_device):
    from archscale_amd.optim.muon import Muon
    p = torch.nn.Parameter((torch.randn(64, 96) * 0.02).to(gpu_device))
    p.grad = torch.randn_like(p) * 1e-3
    opt = Muon([p], lr=0.02, ns_workspace_limit=1)      # nothing fits: separate calls, sliced
    opt.phase_events = []
    opt.step()
    torch.cuda.synchronize()
    assert [n for n, _, _ in opt.phase_events][:2] == ["momentum", "newton_schulz"]
    opt2 = Muon([p], lr=0.02)
    opt2.phase_events = []
    opt2.step()
    torch.cuda.synchronize()
    assert [n for n, _, _ in opt2.phase_events][0] == "momentum+newton_schulz"


@pytest.mark.parametrize("nesterov", [True, False])
def test_emerging_fused_momentum_matches_separate_calls(gpu_device, nesterov):
    """The batched emerging path with momentum fused into the Newton-Schulz call against the same optimizer with the
    separate momentum kernel: identical buffers, weights equal up to where the update is rounded to bf16 (before or
    after its normalisation)."""
    from archscale_amd.emerging import Muon as EMuon
    shapes = [(256, 512), (512, 256), (256, 512), (96, 200)]
    outs = []
    for fuse in (True, False):
        params = _make(shapes, torch.float32, 9, gpu_device)
        w0 = [p.detach().clone() for p in params]
        opt = EMuon(params, lr=0.02, momentum_beta=0.9, weight_decay=0.1, use_nesterov=nesterov,
                    weight_decay_method="l2", scale_mode="shape_scaling")
        opt.fuse_momentum = fuse
        for k in range(2):
            for p, g in zip(params, _grads(shapes, torch.float32, 70 + k)):
                p.grad = g.clone().to(gpu_device)
            opt.step()
        torch.cuda.synchronize()
        outs.append(([p.detach().clone() for p in params], [opt.state[p]["momentum_buffer"].clone() for p in params], w0))
    (wf, mf, w0), (ws, ms, _) = outs
    for a, b, m1, m2, w in zip(wf, ws, mf, ms, w0):
        assert _rel(m1, m2) <= 2e-3       # second step: the buffers see the slightly different weights through l2
        assert _rel(a - w, b - w) <= 1e-2
        assert _rel(a, b) <= 3e-3


@pytest.mark.parametrize("table", ["quintic", "simple", "one_row"])
def test_fused_momentum_with_half_precision_workspace(gpu_device, table):
    """``ns_precision="f16"`` on the fused path: the first iteration runs in bfloat16 on the unnormalised update (deferred
    scale) and hands the iterate over as scaled half.  From zero momentum with Nesterov the update is (1 + mu) G, and with
    fp32 weights, no weight decay and no lr adjustment the orthogonalised update is (W0 - W1) / lr: it must stay within
    the half-precision bar of an fp32 run, well below what bfloat16 storage gives, and agree with the unfused path."""
    from archscale_amd.optim.muon import Muon
    shapes = [(512, 768), (768, 512), (2, 256, 640), (96, 200), (320, 129)]   # 256- and 128-tile classes, ragged, 3-D
    coeffs = {"quintic": O.QUINTIC, "simple": list(O.SIMPLE) * 5, "one_row": list(O.SIMPLE)}[table]
    grads = _grads(shapes, torch.float32, 41)
    mu, lr = 0.9, 0.5
    want = [O.newton_schulz(((1.0 + mu) * g).to(torch.bfloat16), coeffs, 1e-8, storage="fp32").float() for g in grads]
    got = {}
    for prec, fuse in (("f16", True), ("f16", False), ("bf16", True)):
        params = _make(shapes, torch.float32, 12, gpu_device)
        w0 = [p.detach().clone() for p in params]
        opt = Muon(params, lr=lr, mu=mu, weight_decay=0.0, epsilon=1e-8, nesterov=True, adjust_lr=None,
                   ns_coefficients=coeffs, ns_precision=prec, fuse_momentum=fuse)
        for p, g in zip(params, grads):
            p.grad = g.to(gpu_device)
        opt.step()
        torch.cuda.synchronize()
        got[(prec, fuse)] = [((w - p.detach()) / lr).cpu() for w, p in zip(w0, params)]
    for i, w in enumerate(want):
        e16, e16u, ebf = (_rel(got[k][i], w) for k in (("f16", True), ("f16", False), ("bf16", True)))
        print(table, shapes[i], "f16 fused %.2e  f16 unfused %.2e  bf16 fused %.2e" % (e16, e16u, ebf), flush=True)
        assert e16 <= 4e-3 and e16u <= 4e-3
        if table != "one_row":
            assert e16 <= 0.6 * ebf
        assert _rel(got[("f16", True)][i], got[("f16", False)][i]) <= 3e-3


def test_random_parameter_sets(gpu_device):
    """Seeded sweep: parameter sets with ragged 2-D and 3-D shapes, both weight dtypes, plain and MuonH updates, with and
    without Nesterov, weight decay and the fused momentum path; two steps each against the reference-semantics oracle
    (fp32 Newton-Schulz on the same bf16 inputs)."""
    import random
    from archscale_amd.optim.muon import Muon
    rng = random.Random(77)
    dims = [64, 96, 100, 129, 200, 256, 320, 513]
    for case in range(6):
        shapes = []
        for _ in range(rng.choice([3, 5])):
            r, c = rng.choice(dims), rng.choice(dims)
            shapes.append((rng.choice([2, 3]), r, c) if rng.random() < 0.3 else (r, c))
        wdtype = rng.choice([torch.float32, torch.bfloat16])
        use_muonh, nesterov = case % 2 == 0, case % 3 != 0
        wd, cautious = [(0.1, False), (0.0, False), (0.1, True)][case % 3]
        fuse = case % 4 != 3
        adjust = rng.choice(["spectral_norm", "rms_norm", "clip_norm", None])
        print("case", case, shapes, wdtype, "muonh", use_muonh, "nesterov", nesterov, "wd", wd, cautious, "fuse", fuse, adjust,
              flush=True)
        hp = dict(lr=0.02, mu=0.9, wd=wd, eps=1e-8, nesterov=nesterov, adjust=adjust, cautious=cautious)
        params = _make(shapes, wdtype, 300 + case, gpu_device)
        w0 = [p.detach().cpu().clone() for p in params]
        opt = Muon(params, lr=hp["lr"], mu=hp["mu"], weight_decay=wd, cautious_wd=cautious, epsilon=hp["eps"],
                   nesterov=nesterov, adjust_lr=adjust, use_muonh=use_muonh, fuse_momentum=fuse)
        steps = [_grads(shapes, wdtype, 400 + 10 * case + k) for k in range(2)]
        for grads in steps:
            for p, g in zip(params, grads):
                p.grad = g.to(gpu_device)
            opt.step()
        torch.cuda.synchronize()
        Xf, Mf = _oracle_run(shapes, w0, steps, wdtype=wdtype, hp=hp, use_muonh=use_muonh, ns_storage="fp32")
        for p, xf, mf in zip(params, Xf, Mf):
            assert torch.isfinite(p.detach().float()).all()
            assert _rel(p.detach(), xf) <= W_TOL, (case, tuple(p.shape))
            assert _rel(opt.state[p]["momentum"], mf) <= (1e-6 if wdtype == torch.float32 else 1e-2)


def test_captured_step_follows_the_schedule(gpu_device):
    """With device_hyperparams the weight-update kernels read lr, lr*wd, eps and the AdamW bias corrections from device
    memory: a step captured ONCE follows a learning-rate schedule and the step count over its replays. Every replay is
    checked bit for bit against an eager twin that gets the same values as kernel arguments (pretrain.py:829-877 rewrites
    group["lr"] before every step)."""
    from archscale_amd.optim.muon import Muon
    shapes = [(128, 256), (256, 128), (2, 192, 64)]
    g = torch.Generator().manual_seed(78)
    W0 = [(torch.randn(*s, generator=g) * 0.02).to(torch.bfloat16) for s in shapes]
    E0 = (torch.randn(300, 64, generator=g) * 0.02).to(torch.bfloat16)      # an AdamW matrix (hyperball), and a vector
    V0 = torch.ones(64, dtype=torch.bfloat16)

    def build(**kw):
        mats = [torch.nn.Parameter(w.clone().to(gpu_device)) for w in W0]
        emb, vec = torch.nn.Parameter(E0.clone().to(gpu_device)), torch.nn.Parameter(V0.clone().to(gpu_device))
        groups = [dict(params=mats), dict(params=[emb, vec], algorithm="adamw", weight_decay=0.05)]
        opt = Muon(groups, lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True, use_muonh=True, cautious_wd=True, **kw)
        return mats + [emb, vec], opt

    pa, oa = build(device_hyperparams=True)
    pb, ob = build()
    all_shapes = shapes + [(300, 64), (64,)]
    static_g = [torch.zeros_like(p) for p in pa]
    for p, sg in zip(pa, static_g):
        p.grad = sg

    def new_grads(k):
        gg = torch.Generator().manual_seed(2000 + k)
        return [(torch.randn(*s, generator=gg) * 1e-3).to(torch.bfloat16).to(gpu_device) for s in all_shapes]

    def schedule(k):
        return 0.02 * (0.5 + 0.1 * k), 0.01 * (1 + k % 3)

    def set_hyper(opt, k):
        lr, wd = schedule(k)
        for group in opt.param_groups:
            group["lr"] = lr * (0.1 if group["algorithm"] == "adamw" else 1.0)
            if group["algorithm"] == "muon":
                group["weight_decay"] = wd

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for k in range(2):                                   # eager warm-up with the device block in use
            for sg, gr in zip(static_g, new_grads(k)):
                sg.copy_(gr)
            set_hyper(oa, k)
            oa.step()
    torch.cuda.current_stream().wait_stream(side)
    for k in range(2):
        for p, gr in zip(pb, new_grads(k)):
            p.grad = gr
        set_hyper(ob, k)
        ob.step()
    torch.cuda.synchronize()
    for a, b in zip(pa, pb):
        assert torch.equal(a, b)                             # device block and kernel arguments: the same arithmetic
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        oa.step()
    assert [grp["step"] for grp in oa.param_groups] == [2, 2]      # the capture itself is not a step
    for k in range(2, 7):
        for sg, gr in zip(static_g, new_grads(k)):
            sg.copy_(gr)
        set_hyper(oa, k)
        oa.sync_hyperparameters(advance_step=True)
        graph.replay()
        for p, gr in zip(pb, new_grads(k)):
            p.grad = gr
        set_hyper(ob, k)
        ob.step()
        junk = torch.randn(128, 128, device=gpu_device) @ torch.randn(128, 128, device=gpu_device)   # eager work in between
        torch.cuda.synchronize()
        assert torch.isfinite(junk).all()
        for a, b in zip(pa, pb):
            assert torch.equal(a, b), k
        assert [grp["step"] for grp in oa.param_groups] == [grp["step"] for grp in ob.param_groups]
    # and the schedule really reached the kernels: a replay without the refresh repeats the last learning rate
    before = [p.detach().clone() for p in pa]
    for sg, gr in zip(static_g, new_grads(7)):
        sg.copy_(gr)
    graph.replay()
    for p, gr in zip(pb, new_grads(7)):
        p.grad = gr
    set_hyper(ob, 7)
    ob.step()
    torch.cuda.synchronize()
    assert not all(torch.equal(a, b) for a, b in zip(pa, pb))
    assert not all(torch.equal(a, b) for a, b in zip(pa, before))
    with pytest.raises(RuntimeError):
        ob.sync_hyperparameters()
