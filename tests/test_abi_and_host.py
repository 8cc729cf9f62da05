"""CPU-only checks: the shared library loads and exports every symbol the header declares, the ctypes
layouts match the header's structs, and the host-side logic (grouping, flatten policy, lr ratios,
constructor validation) behaves like the reference's."""
import ctypes
import math
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "archscale_muon.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(muon_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from archscale_amd import _lib
    from archscale_amd.build import LIB_PATH
    assert os.path.exists(LIB_PATH), "build the library first: python -m archscale_amd.build"
    handle = _lib.lib()
    declared = _declared_functions()
    assert len(declared) >= 12
    for name in declared:
        assert hasattr(handle, name), f"{name} is declared in the header but not exported"
    assert sorted(_lib.EXPORTED_SYMBOLS) == declared
    assert handle.muon_abi_version() == _lib.ABI_VERSION == 3
    assert b"success" in handle.muon_status_string(0)
    assert b"workspace" in handle.muon_status_string(-2)


def test_struct_layouts_and_constants_match_header():
    from archscale_amd import _lib
    text = open(HEADER).read()
    assert int(re.search(r"#define MUON_CHUNK_ELEMS (\d+)", text).group(1)) == _lib.CHUNK_ELEMS
    assert int(re.search(r"#define MUON_ABI_VERSION (\d+)", text).group(1)) == _lib.ABI_VERSION

    class Pre(ctypes.Structure):
        _fields_ = [("g", ctypes.c_void_p), ("m", ctypes.c_void_p), ("u", ctypes.c_void_p), ("w", ctypes.c_void_p),
                    ("numel", ctypes.c_int64), ("g_dtype", ctypes.c_int32), ("m_dtype", ctypes.c_int32),
                    ("u_dtype", ctypes.c_int32), ("w_dtype", ctypes.c_int32)]

    class Post(ctypes.Structure):
        _fields_ = [("w", ctypes.c_void_p), ("u", ctypes.c_void_p), ("numel", ctypes.c_int64),
                    ("lr_ratio", ctypes.c_float), ("w_dtype", ctypes.c_int32)]

    class Hyper(ctypes.Structure):
        _fields_ = [(n, ctypes.c_float) for n in ("lr", "lr_wd", "eps", "w1", "w2", "bias1", "bias2_sqrt")] + [
            ("cautious", ctypes.c_int32)]

    m = re.search(r"typedef struct muon_hyper \{(.*?)\} muon_hyper;", text, re.S)
    fields = re.findall(r"\b(\w+)\s*[,;]", re.sub(r"/\*.*?\*/", "", m.group(1), flags=re.S))
    assert fields == [n for n, _ in Hyper._fields_]          # the header declares the fields in the binding's order
    for cs, nd in ((Pre, _lib.PRE_ITEM), (Post, _lib.POST_ITEM), (Hyper, _lib.HYPER)):
        assert ctypes.sizeof(cs) == nd.itemsize
        for name, _ in cs._fields_:
            assert getattr(cs, name).offset == nd.fields[name][1]


def test_k_split_rule_is_a_function_of_the_shape():
    """Which symmetric products are cut along K: none of the shapes that come in large batches (every class of the
    depth-16 and depth-24 parameter sets, expert stacks), the leftover tiles of large single matrices with K >= 8192.
    The workspace query includes the partial results."""
    from archscale_amd import _lib
    L = _lib.lib()
    none = ((None, 0, 1), (None, 0, 1))
    for shape in [(2048, 2048), (512, 2048), (5632, 2048), (2048, 5632), (3072, 3072), (768, 3072), (1536, 3072),
                  (3072, 384), (256, 2048), (256, 8192), (1024, 8192), (4096, 4096), (100, 36)]:
        lk, sk = _lib.ns_ksplit_info(*shape)
        assert lk[1:] == none[0][1:] and sk[1:] == none[1][1:], shape
    # 4096 x 14336: 16 * 17 / 2 = 136 tiles, all left over; only the reduction over the long side is long enough
    assert _lib.ns_ksplit_info(4096, 14336) == ((0, 136, 4), (136, 0, 1))
    assert _lib.ns_ksplit_info(14336, 4096) == _lib.ns_ksplit_info(4096, 14336)
    # 8192 x 8192: 528 tiles = two whole rounds of 256 and 16 left over, both reductions have K = 8192
    assert _lib.ns_ksplit_info(8192, 8192) == ((512, 16, 4), (512, 16, 4))
    # 1536 x 8192: 21 tiles, K = 8192 over the long side only
    assert _lib.ns_ksplit_info(1536, 8192) == ((0, 21, 4), (21, 0, 1))
    # the partial results (64 KiB per quadrant and part) are part of the workspace
    base = 2 * 4096 * 14336 * 2 + 2 * 4096 * 4096 * 2
    need = L.muon_ns_workspace_bytes(1, 4096, 14336, 0)
    assert need >= base + 136 * 4 * 4 * 65536 and need < base + 136 * 4 * 4 * 65536 + (8 << 20)
    assert L.muon_ns_workspace_bytes(3, 4096, 14336, 0) >= 3 * (base + 136 * 4 * 4 * 65536)


def test_workspace_and_flops_queries_need_no_gpu():
    from archscale_amd import _lib
    L = _lib.lib()
    assert L.muon_ns_workspace_bytes(0, 8, 8, 0) == 0
    small = L.muon_ns_workspace_bytes(1, 512, 2048, 0)
    split = L.muon_ns_workspace_bytes(1, 512, 2048, 1)
    assert split - small >= 512 * 512 * 2 and small >= 2 * 512 * 2048 * 2 + 2 * 512 * 512 * 2
    assert L.muon_ns_workspace_bytes(1, 2048, 512, 0) == small            # orientation does not matter
    d, s, i = _lib.ns_flops(1, 512, 2048, 5, 0)
    assert d == pytest.approx(5 * (4 * 512 ** 2 * 2048 + 2 * 512 ** 3))
    assert s == pytest.approx(5 * (3 * 512 ** 2 * 2048 + 512 ** 3))
    assert s < i < d                                                        # full diagonal tiles cost a little
    d2, s2, i2 = _lib.ns_flops(1, 512, 2048, 5, 1)
    assert i2 > i and d2 == d
    assert L.muon_muonh_scratch_floats(3, 10) >= 3 * 10 + 2 * 3
    # the hyper-parameter record: derived fields as the by-value entry points compute them
    rec = _lib.hyper_record(0.02, 0.02 * 0.1, 1e-8, 0.9, 0.95, 3, True)[0]
    assert rec["w1"] == np.float32(1.0) - np.float32(0.9) and rec["cautious"] == 1
    assert rec["bias1"] == np.float32(1.0 - float(np.float32(0.9)) ** 3)
    assert rec["bias2_sqrt"] == np.float32((1.0 - float(np.float32(0.95)) ** 3) ** 0.5)


def test_argument_errors_without_touching_the_gpu():
    from archscale_amd import _lib
    L = _lib.lib()
    abc = _lib.abc_array([(1.0, 0.0, 0.0)])
    assert L.muon_ns_batched(None, 0, 0, 8, None, 0, 8, 1, 8, 8, abc, 1, 1e-7, 0, 0, 0, None, 0, None) == -1
    assert L.muon_momentum(None, None, 3, 3, 0.9, 1.0, 0.9, 1.0, 0.0, None) == -1
    assert L.muon_momentum(None, None, 0, 0, 0.9, 1.0, 0.9, 1.0, 0.0, None) == 0   # nothing to do
    assert L.muon_update_muonh(None, None, 2, 2, 0.1, 0.0, 1e-8, 0, None, None) == -1
    with pytest.raises(ValueError):
        _lib.check(-1, "x")
    with pytest.raises(_lib.MuonLibraryError):
        _lib.check(1, "x")
    with pytest.raises(TypeError):
        _lib.dtype_code(torch.float16)


def test_no_cpu_fallback():
    import archscale_amd.optim.newton_schulz_hip as H
    from archscale_amd._lib import MuonLibraryError
    from archscale_amd.optim.muon import Muon
    with pytest.raises(MuonLibraryError):
        H.zeropower_via_newtonschulz5(torch.randn(8, 16))
    p = torch.nn.Parameter(torch.randn(8, 16))
    p.grad = torch.randn(8, 16)
    opt = Muon([p])
    with pytest.raises(MuonLibraryError):
        opt.step()
    assert opt.param_groups[0]["step"] == 1   # counted before the work, as in the reference


def test_constructor_validation_and_defaults():
    from archscale_amd.optim.muon import Muon
    p = torch.nn.Parameter(torch.randn(4, 4))
    for bad in (dict(lr=-1.0), dict(mu=-0.1), dict(betas=(0.9,)), dict(betas=(-0.1, 0.9)), dict(adjust_lr="nope")):
        with pytest.raises(ValueError):
            Muon([p], **bad)
    with pytest.raises(TypeError):
        Muon([p], distributed_mesh="mesh")
    with pytest.raises(TypeError):
        Muon([p], newton_schulz_func=3)
    opt = Muon([p], betas=(0.8, 0.9), use_triton=True)
    g = opt.param_groups[0]
    assert (g["lr"], g["mu"], g["beta1"], g["beta2"], g["weight_decay"], g["epsilon"]) == (0.01, 0.95, 0.8, 0.9, 0.01, 1e-8)
    assert g["algorithm"] == "muon" and g["step"] == 0 and g["nesterov"] is False and g["flatten"] is False
    assert g["adjust_lr"] == "spectral_norm" and g["cautious_wd"] is False
    assert opt.use_muonh is False and opt._world_size == 1
    opt.exclude_from_hyperball(p)
    assert p in opt._hyperball_excluded
    # 1-D parameter in a muon group is refused
    v = torch.nn.Parameter(torch.randn(4))
    v.grad = torch.randn(4)
    with pytest.raises(AssertionError):
        Muon([v]).step()


def test_loads_a_state_dict_in_the_reference_layout():
    """A checkpoint written by the reference's optimizer (torch.optim.Optimizer.state_dict() of lit_gpt/optim/muon.py:86-101,
    199-209: param-group keys lr, mu, beta1, beta2, weight_decay, cautious_wd, algorithm, step, epsilon, nesterov, flatten,
    adjust_lr plus the trainer's lr_mult; per-parameter state "momentum", and "variance" in the adamw groups) loads into
    the drop-in, which then goes on counting steps from the loaded value and hands the same dictionary back."""
    from archscale_amd.optim.muon import Muon
    w = torch.nn.Parameter(torch.randn(8, 16))
    e = torch.nn.Parameter(torch.randn(32, 8))
    b = torch.nn.Parameter(torch.randn(8))
    common = dict(mu=0.95, beta1=0.9, beta2=0.95, cautious_wd=False, epsilon=1e-8, nesterov=True, flatten=False,
                  adjust_lr="spectral_norm")
    ref_sd = {
        "state": {
            0: {"momentum": torch.full((8, 16), 0.25)},
            1: {"momentum": torch.full((32, 8), -0.5), "variance": torch.full((32, 8), 2.0)},
            2: {"momentum": torch.full((8,), 0.125), "variance": torch.full((8,), 3.0)},
        },
        "param_groups": [
            dict(common, lr=0.02, weight_decay=0.0, algorithm="muon", step=1234, lr_mult=1.0, params=[0]),
            dict(common, lr=0.004, weight_decay=0.1, algorithm="adamw", step=1234, lr_mult=0.2, params=[1, 2]),
        ],
    }
    opt = Muon([dict(params=[w]), dict(params=[e, b], algorithm="adamw", lr=0.1)], lr=0.5, use_muonh=True)
    opt.load_state_dict(ref_sd)
    g0, g1 = opt.param_groups
    assert g0["step"] == 1234 and g0["lr"] == 0.02 and g0["algorithm"] == "muon" and g0["lr_mult"] == 1.0
    assert g1["step"] == 1234 and g1["lr"] == 0.004 and g1["algorithm"] == "adamw" and g1["weight_decay"] == 0.1
    assert torch.equal(opt.state[w]["momentum"], torch.full((8, 16), 0.25))
    assert torch.equal(opt.state[e]["variance"], torch.full((32, 8), 2.0))
    assert torch.equal(opt.state[b]["momentum"], torch.full((8,), 0.125))
    back = opt.state_dict()
    assert [sorted(g.keys()) for g in back["param_groups"]] == [sorted(g.keys()) for g in ref_sd["param_groups"]]
    assert sorted(back["state"][1].keys()) == ["momentum", "variance"] and sorted(back["state"][0].keys()) == ["momentum"]
    # the step counter continues from the loaded value (counted before the work, which needs the GPU)
    from archscale_amd._lib import MuonLibraryError
    w.grad = torch.randn(8, 16)
    with pytest.raises(MuonLibraryError):
        opt.step()
    assert opt.param_groups[0]["step"] == 1235 and opt.param_groups[1]["step"] == 1235


def test_lr_ratios_flatten_policy_and_batches():
    from archscale_amd.optim import muon as M
    from archscale_amd.optim.opt_utils import create_param_batches, matrix_view_shape
    assert M.adjust_lr_spectral_norm(0.02, (5632, 2048), False) == pytest.approx(0.02 * math.sqrt(2.75))
    assert M.adjust_lr_spectral_norm(0.02, (2048, 5632), False, clip_norm=True) == pytest.approx(0.02)
    assert M.adjust_lr_rms_norm(0.02, (64, 512, 2048), False) == pytest.approx(0.02 * 0.2 * math.sqrt(2048))
    assert M.adjust_lr_spectral_norm(1.0, (64, 8, 4), True) == pytest.approx(math.sqrt(2.0))
    assert M._lr_ratio((8, 2), None, False) == 1.0
    with pytest.raises(ValueError):
        M._lr_ratio((8, 2), "bad", False)
    assert matrix_view_shape((6, 4), False) == (1, 6, 4)
    assert matrix_view_shape((3, 6, 4), False) == (3, 6, 4)
    assert matrix_view_shape((2, 3, 6, 4), False) == (6, 6, 4)
    assert matrix_view_shape((2, 3, 6, 4), True) == (1, 2, 72)
    with pytest.raises(ValueError):
        matrix_view_shape((5,), False)
    ps = [torch.zeros(2, 3), torch.zeros(3, 2), torch.zeros(2, 3), torch.zeros(2, 3, dtype=torch.bfloat16),
          torch.zeros(2, 3)]
    got = [[id(t) for t in b] for b in create_param_batches(ps, 2)]
    assert got == [[id(ps[0]), id(ps[2])], [id(ps[4])], [id(ps[1])], [id(ps[3])]]


def test_emerging_host_logic():
    from archscale_amd.emerging import get_muon_scale_factor
    from archscale_amd.emerging.mixin import weight_decay_terms
    from archscale_amd.emerging.spectral_ball_utils import msign_schedule, MSIGN_COEFFICIENTS
    from archscale_amd.emerging import Muon as EMuon, newton_schulz, msign
    assert get_muon_scale_factor(8, 2, "shape_scaling") == 2.0
    assert get_muon_scale_factor(100, 400, "align_adamw_rms") == pytest.approx(4.0)
    assert get_muon_scale_factor(8, 2, "spectral_mup") == 2.0
    with pytest.raises(ValueError):
        get_muon_scale_factor(1, 1)          # the reference's default "spectral" is not a valid mode either
    assert weight_decay_terms("decoupled", 0.1, 0.5) == (0.05, 0.0)
    assert weight_decay_terms("independent", 0.1, 0.5) == (0.5, 0.0)
    assert weight_decay_terms("l2", 0.1, 0.5) == (0.0, 0.5)
    assert weight_decay_terms("l2", 0.1, 0.0) == (0.0, 0.0)
    with pytest.raises(ValueError):
        weight_decay_terms("bad", 0.1, 0.5)
    assert msign_schedule(10)[9] == MSIGN_COEFFICIENTS[7] and len(msign_schedule(5)) == 5
    with pytest.raises(ValueError):
        EMuon([torch.nn.Parameter(torch.zeros(2, 2))], num_ns_steps=0)
    with pytest.raises(ValueError):
        msign(torch.zeros(4, 4, dtype=torch.bfloat16), 5)
    with pytest.raises(ValueError):
        newton_schulz(torch.zeros(4, 4), steps=3, coefficient_type="quintic")   # 3 is no multiple of 5
    with pytest.raises(ValueError):
        newton_schulz(torch.zeros(4, 4), steps=5, coefficient_type="nope")
    o = EMuon([torch.nn.Parameter(torch.zeros(2, 2))])
    g = o.param_groups[0]
    assert (g["lr"], g["momentum_beta"], g["weight_decay"]) == (3e-4, 0.95, 0.01)
    assert np.isclose(o._extra_scale_factor, 1.0)


def test_transpose_read_results_are_not_touched_before_the_explicit_wait(tmp_path):
    """The K-major GEMM variant issues its LDS transpose reads as inline assembly (the compiler would otherwise wait for
    every outstanding global->LDS copy before each of them), so the compiler does not know that their results arrive
    late: the kernel waits explicitly (s_waitcnt lgkmcnt(0)) before the first use. This checks the generated code: no
    instruction between such a read and the next full LGKM wait may mention the registers the read writes."""
    import re
    import subprocess
    from archscale_amd.build import CSRC, HIPCC_FLAGS, find_hipcc
    out = tmp_path / "ns_gemm.s"
    subprocess.run([find_hipcc(), *HIPCC_FLAGS, "--cuda-device-only", "-S", os.path.join(CSRC, "ns_gemm.hip"), "-o", str(out)],
                   check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    text = out.read_text().splitlines()
    reg = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")

    def regs(s):
        found = set()
        for a, b, c in reg.findall(s):
            found |= set(range(int(a), int(b) + 1)) if a else {int(c)}
        return found

    # template arguments of an instantiation from its mangled name: <BM, BN, WM, WN, MODE, SPLIT, FINAL, ADDEND, F16, SK>
    targs = re.compile(r"ns_gemm_kernelILi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELb([01])ELb([01])ELb([01])ELi(\d+)ELb([01])EE")
    # pass 1: cut every K-major instantiation into basic blocks (label -> instructions, each tagged "inline asm or not")
    seen, reads_of, kernels = set(), {}, {}
    all_kernels = 0
    inside, in_asm, cur, blocks, label = False, False, None, None, None
    for line in text:
        if "#ASMSTART" in line or "#ASMEND" in line:
            in_asm = "#ASMSTART" in line
            continue
        code = line.split(";")[0].strip()
        if code.endswith(":") and "ns_gemm_kernel" in code:
            m = targs.search(code)
            assert m, f"cannot read the template arguments of {code}: the name mangling changed, adapt this test"
            all_kernels += 1
            bm, mode, f16, sk = int(m.group(1)), int(m.group(5)), int(m.group(9)), int(m.group(10))
            inside = mode == 3                   # MODE_SYRKT instantiations
            cur = (bm, f16, sk)
            if inside:
                assert cur not in seen, f"{code} seen twice"
                seen.add(cur)
                reads_of[cur] = 0
                label = "<entry>"
                blocks = kernels[cur] = [[label, []]]
            continue
        if not inside or not code:
            continue
        if code.startswith(".Lfunc_end"):   # (blocks may follow the first s_endpgm: the function ends here)
            inside = False
            continue
        if code.endswith(":") and code.startswith(".LBB"):
            label = code[:-1]
            blocks.append([label, []])
            continue
        if code.startswith("."):
            continue
        blocks[-1][1].append((code, in_asm))
        if code.startswith(("s_cbranch", "s_branch", "s_endpgm")):
            blocks.append([f"<after {len(blocks)}>", []])   # a branch or the end of the program ends its block

    # pass 2, per kernel: the set of registers with a transpose read in flight at the entry of each block is the union
    # over its predecessors (fall-through, conditional and unconditional branches, loop back-edges included), iterated
    # to a fixed point; then no instruction may mention a register that is pending where it stands
    def walk(instrs, pending, check, key):
        pending = set(pending)
        for code, asm in instrs:
            if code.startswith("ds_read_b64_tr_b16") and asm:   # the compiler tracks the ones it emits itself
                dst, addr = code[len("ds_read_b64_tr_b16"):].split(",")[:2]
                if check:
                    assert not (regs(addr) & pending), code
                    assert not (regs(dst) & pending), code
                    reads_of[key] += 1
                pending |= regs(dst)
            elif code.startswith("s_waitcnt") and "lgkmcnt(0)" in code:
                pending = set()
            elif check:
                assert not (regs(code) & pending), f"uses a transpose-read result before the wait: {code}"
        return pending

    for key, blocks in kernels.items():
        index = {lab: i for i, (lab, _) in enumerate(blocks)}
        succ = []
        for i, (lab, instrs) in enumerate(blocks):
            out = set()
            last = instrs[-1][0] if instrs else ""
            assert not any(c.startswith(("s_cbranch", "s_branch", "s_setpc", "s_swappc")) for c, _ in instrs[:-1]), lab
            assert not last.startswith(("s_setpc", "s_swappc")), f"indirect jump in {key}"
            if last.startswith(("s_cbranch", "s_branch")):
                target = last.split()[-1]
                assert target in index, f"branch to an unknown label: {last}"
                out.add(index[target])
            if not (last.startswith("s_branch") or last.startswith("s_endpgm")) and i + 1 < len(blocks):
                out.add(i + 1)
            succ.append(out)
        pend_in = [set() for _ in blocks]
        changed = True
        while changed:
            changed = False
            for i, (lab, instrs) in enumerate(blocks):
                out = walk(instrs, pend_in[i], False, key)
                for j in succ[i]:
                    if not out <= pend_in[j]:
                        pend_in[j] |= out
                        changed = True
        for i, (lab, instrs) in enumerate(blocks):
            out = walk(instrs, pend_in[i], True, key)
            if instrs and instrs[-1][0].startswith("s_endpgm"):
                assert not out, f"{key}: transpose reads in flight at the end of the program"
    # every K-major instantiation was visited by name: two tile configurations x {bfloat16, half} workspace, and the
    # small configuration once more with the K-split
    assert seen == {(256, 0, 0), (256, 1, 0), (128, 0, 0), (128, 1, 0), (128, 0, 1), (128, 1, 1)}, seen
    assert all_kernels > len(seen)
    # per k-tile: 4 k-steps x (FM + FN) fragments x 2 reads; the loop body appears at least once
    assert all(reads_of[(256, f, 0)] >= 4 * 6 * 2 for f in (0, 1)), reads_of
    assert all(reads_of[(128, f, k)] >= 4 * 4 * 2 for f in (0, 1) for k in (0, 1)), reads_of
