"""The two ways the chunked entry points build the states at the start of every tile — per-tile contributions
by all tiles in parallel followed by a scan, or one pass per (sequence, head) with the running state in
registers — must agree: same algorithm, same bf16 operands, fp32 sums taken in a different order.  Each form is
also checked against the oracle (Palimpsa) or the float64 closed form (scalar-gated path) on its own, so that
neither is only ever compared with the other.
"""
import pytest
import torch

from tests import helpers as hp

pytestmark = pytest.mark.gpu


@pytest.fixture
def state_pass_mode():
    from palimpsa_amd import _lib
    yield _lib.set_state_pass_mode
    _lib.set_state_pass_mode(0)


def _pal_inputs(B, T, H, dk, dv, seed, dev):
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen)
    inp = dict(
        q=torch.nn.functional.normalize(r(B, T, H, dk), dim=-1), k=torch.nn.functional.normalize(r(B, T, H, dk), dim=-1),
        v=r(B, T, H, dv), b=torch.rand(B, T, H, dv, generator=gen) + 0.1,
        gt=torch.nn.functional.softplus(r(B, T, H)) * 0.2, g=torch.linspace(0.3, 3.0, H), Ip=torch.linspace(0.5, 2.0, H))
    return hp.to_device(hp.rounded(inp, torch.bfloat16), dev)


def _run_palimpsa(inp, mu0, I0, cu, grads):
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa
    names = ("q", "k", "v", "b", "gt", "g", "Ip")
    leaves = {n: inp[n].detach().clone().requires_grad_(grads) for n in names}
    st = [s.detach().clone().requires_grad_(grads) for s in (mu0, I0)] if mu0 is not None else [None, None]
    o, fmu, fI = chunk_palimpsa(*[leaves[n] for n in names], initial_mu_state=st[0], initial_I_state=st[1],
                                output_final_state=True, cu_seqlens=cu)
    out = [o, fmu, fI]
    if grads:
        gen = torch.Generator().manual_seed(5)
        do = torch.randn(o.shape, generator=gen).to(o)
        (o.float() * do.float()).sum().backward()
        out += [leaves[n].grad for n in names] + ([s.grad for s in st] if mu0 is not None else [])
    return out


@pytest.mark.parametrize("case", ["batched", "varlen_ragged", "wide_heads", "init_state_grads", "key_slices"])
def test_palimpsa_forms_agree(gpu_device, state_pass_mode, case):
    dev = gpu_device
    cu = mu0 = I0 = None
    grads = False
    if case == "batched":
        inp = _pal_inputs(3, 300, 4, 64, 64, 1, dev)
    elif case == "varlen_ragged":       # full and partial tiles, a one-token document
        inp = _pal_inputs(1, 64 + 1 + 130 + 257, 2, 32, 48, 2, dev)
        cu = torch.tensor([0, 64, 65, 195, 452], dtype=torch.int32, device=dev)
    elif case == "wide_heads":            # few (sequence, head) pairs: the one-pass form also slices the key columns
        inp = _pal_inputs(2, 129, 2, 256, 144, 3, dev)
    elif case == "key_slices":            # the same with an initial state, at the shape class of a long single prefill
        inp = _pal_inputs(1, 300, 12, 128, 128, 6, dev)
        gen = torch.Generator().manual_seed(10)
        mu0 = (torch.randn(1, 12, 128, 128, generator=gen) * 0.3).to(dev)
        I0 = (torch.rand(1, 12, 128, 128, generator=gen) + inp["Ip"].cpu()[None, :, None, None]).to(dev)
    else:
        inp = _pal_inputs(2, 200, 3, 48, 96, 4, dev)
        gen = torch.Generator().manual_seed(9)
        mu0 = (torch.randn(2, 3, 96, 48, generator=gen) * 0.3).to(dev)
        I0 = (torch.rand(2, 3, 96, 48, generator=gen) + inp["Ip"].cpu()[None, :, None, None]).to(dev)
        grads = True
    state_pass_mode(1)
    a = _run_palimpsa(inp, mu0, I0, cu, grads)
    state_pass_mode(2)
    b = _run_palimpsa(inp, mu0, I0, cu, grads)
    assert hp.max_abs(a[0].float(), b[0].float()) <= 1e-2            # outputs: bf16, a last-bit flip at most
    assert hp.max_rel(a[1], b[1]) <= 1e-4 and hp.max_rel(a[2], b[2]) <= 1e-4   # fp32 final states: order of sums only
    for x, y in zip(a[3:], b[3:]):
        assert hp.max_rel(x.float(), y.float()) <= 2e-2
    # the one-pass form against the oracle
    o_ref, _, fmu_ref, fI_ref = hp.oracle_forward({k: v.cpu() for k, v in inp.items()}, mu0=None if mu0 is None else mu0.cpu(),
                                                  I0=None if I0 is None else I0.cpu(), cu=None if cu is None else cu.cpu().tolist())
    assert hp.max_abs(b[0].float(), o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(b[1], fmu_ref) <= 2e-2 and hp.max_rel(b[2], fI_ref) <= 2e-2


def _gla_inputs(B, T, H, dk, dv, seed):
    gen = torch.Generator().manual_seed(seed)
    q = torch.nn.functional.normalize(torch.randn(B, T, H, dk, generator=gen), dim=-1).bfloat16()
    k = torch.nn.functional.normalize(torch.randn(B, T, H, dk, generator=gen), dim=-1).bfloat16()
    v = torch.randn(B, T, H, dv, generator=gen).bfloat16()
    g = -torch.nn.functional.softplus(torch.randn(B, T, H, generator=gen)) * torch.linspace(0.05, 2.0, H)
    S0 = torch.randn(B, H, dk, dv, generator=gen) * 0.2
    do = torch.randn(B, T, H, dv, generator=gen).bfloat16()
    return q, k, v, g, S0, do


def _run_gla(x, dev, cu=None):
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    q, k, v, g, S0, do = x
    leaves = [t.to(dev).clone().requires_grad_(True) for t in (q, k, v, g, S0)]
    o, S = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3], initial_state=leaves[4],
                            output_final_state=True, cu_seqlens=cu)
    (o.float() * do.to(dev).float()).sum().backward()
    return [o, S] + [t.grad for t in leaves]


@pytest.mark.parametrize("shape", [(2, 200, 3, 64, 64), (1, 777, 2, 96, 192), (2, 65, 2, 256, 32), (3, 64, 1, 16, 16)])
def test_simple_gla_forms_agree_forward_and_backward(gpu_device, state_pass_mode, shape):
    x = _gla_inputs(*shape, seed=21)
    state_pass_mode(1)
    a = _run_gla(x, gpu_device)
    state_pass_mode(2)
    b = _run_gla(x, gpu_device)
    assert hp.max_abs(a[0].float(), b[0].float()) <= 1e-2
    assert hp.max_rel(a[1], b[1]) <= 1e-4                     # fp32 final state
    names = ("dq", "dk", "dv", "dg", "dS0")
    for n, p, r in zip(names, a[2:], b[2:]):
        assert hp.max_rel(p.float(), r.float()) <= 2e-2, n


def test_simple_gla_one_pass_form_against_closed_form(gpu_device, state_pass_mode):
    from tests.test_gpu_simple_gla import _closed_form
    B, T, H, dk, dv = 2, 260, 3, 64, 32
    q, k, v, g, S0, do = _gla_inputs(B, T, H, dk, dv, seed=22)
    state_pass_mode(2)
    got = _run_gla((q, k, v, g, S0, do), gpu_device)
    leaves = [t.double().clone().requires_grad_(True) for t in (q, k, v, g, S0)]
    o_ref, S_ref = _closed_form(*leaves[:4], dk ** -0.5, leaves[4])
    (o_ref * do.double()).sum().backward()
    assert hp.max_abs(got[0].float(), o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(got[1], S_ref) <= 1e-2
    for n, p, r in zip(("dq", "dk", "dv", "dg", "dS0"), got[2:], leaves):
        assert hp.max_rel(p.float(), r.grad) <= hp.BF16_GRAD_NORM_TOL, n


def test_varlen_simple_gla_forms_agree(gpu_device, state_pass_mode):
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    dev = gpu_device
    lens = [1, 64, 0, 100, 300]
    T = sum(lens)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=dev)
    q, k, v, g, _, do = _gla_inputs(1, T, 2, 48, 96, seed=23)
    outs = []
    for mode in (1, 2):
        state_pass_mode(mode)
        leaves = [t.to(dev).clone().requires_grad_(True) for t in (q, k, v, g)]
        o, S = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3], output_final_state=True, cu_seqlens=cu)
        (o.float() * do.to(dev).float()).sum().backward()
        outs.append([o, S] + [t.grad for t in leaves])
    a, b = outs
    assert a[1].shape[0] == len(lens)
    assert hp.max_abs(a[0].float(), b[0].float()) <= 1e-2
    assert hp.max_rel(a[1], b[1]) <= 1e-4
    for p, r in zip(a[2:], b[2:]):
        assert hp.max_rel(p.float(), r.float()) <= 2e-2
