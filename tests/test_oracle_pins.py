"""Pins for the CPU oracle (oracle/palimpsa_oracle.py).

The reference repository holds no golden vectors for the operator (it has no
tests directory; palimpsa/check_palimpsa.py prints tables and stores nothing),
so the oracle is pinned by what the mathematics fixes: closed forms, special
cases that reduce to a textbook routine, float64 brute force, invariants and
gradcheck.  Each check is chosen so that a plausible slip (dropped (1-f)*Ip
term, inclusive/exclusive output, transposed state, wrong scale power) fails it.
"""
import numpy as np
import pytest
import torch

from oracle import palimpsa_oracle as po

torch.manual_seed(0)
F64 = torch.float64


def rnd(*shape, gen):
    return torch.randn(*shape, generator=gen, dtype=F64)


def small_inputs(B=2, T=7, H=3, dk=4, dv=5, seed=1, normalize=False):
    gen = torch.Generator().manual_seed(seed)
    q = rnd(B, T, H, dk, gen=gen)
    k = rnd(B, T, H, dk, gen=gen)
    v = rnd(B, T, H, dv, gen=gen)
    b = torch.sigmoid(rnd(B, T, H, dv, gen=gen))
    gt = torch.sigmoid(rnd(B, T, H, gen=gen))
    g = rnd(H, gen=gen).abs() * 3 + 0.5
    Ip = rnd(H, gen=gen).abs() + 0.1
    if normalize:
        q = torch.nn.functional.normalize(q, dim=-1)
        k = torch.nn.functional.normalize(k, dim=-1)
    return q, k, v, b, gt, g, Ip


def run(*a, **kw):
    kw.setdefault("compute_dtype", F64)
    return po.palimpsa_recurrence(*a, **kw)


# ---------------------------------------------------------------- closed forms
def test_single_token_closed_form():
    q, k, v, b, gt, g, Ip = small_inputs(T=1)
    scale = 0.37
    o, ov, mu, I = run(q, k, v, b, gt, g, Ip, scale=scale, output_uncertainty=True)
    # from (mu0, I0) = (0, Ip):  I = b k^2 + (1-f) Ip + f Ip = b k^2 + Ip ; M = v k^T
    I_ref = b[:, 0].unsqueeze(-1) * (k[:, 0] ** 2).unsqueeze(-2) + Ip.view(1, -1, 1, 1)
    mu_ref = v[:, 0].unsqueeze(-1) * k[:, 0].unsqueeze(-2) / I_ref
    o_ref = scale * torch.einsum("bhdn,bhn->bhd", mu_ref, q[:, 0])
    ov_ref = scale * torch.einsum("bhdn,bhn->bhd", 1 / I_ref, q[:, 0] ** 2)
    assert torch.allclose(I[:, :], I_ref, rtol=1e-13, atol=0)
    assert torch.allclose(mu, mu_ref, rtol=1e-13, atol=1e-15)
    assert torch.allclose(o[:, 0], o_ref, rtol=1e-12, atol=1e-14)
    assert torch.allclose(ov[:, 0], ov_ref, rtol=1e-12, atol=1e-14)


def test_var_scale_power_conventions():
    q, k, v, b, gt, g, Ip = small_inputs()
    s = 0.5
    _, ov1, _, _ = run(q, k, v, b, gt, g, Ip, scale=s, output_uncertainty=True, var_scale_power=1)
    _, ov2, _, _ = run(q, k, v, b, gt, g, Ip, scale=s, output_uncertainty=True, var_scale_power=2)
    assert torch.allclose(ov2, ov1 * s, rtol=1e-13)


def test_b_zero_is_gated_linear_attention():
    """b == 0 => I == Ip => o = scale/Ip * ((Q K^T) * L) V with L[t,s]=prod_{r=s+1..t} f_r."""
    q, k, v, b, gt, g, Ip = small_inputs(T=9)
    b = torch.zeros_like(b)
    scale = 0.8
    o, _, mu, I = run(q, k, v, b, gt, g, Ip, scale=scale)
    B, T, H, _ = q.shape
    logf = -(gt * g.view(1, 1, H))                      # [B,T,H]
    c = torch.cumsum(logf, dim=1)
    L = torch.exp(c.unsqueeze(2) - c.unsqueeze(1))      # [B,t,s,H]
    mask = torch.tril(torch.ones(T, T, dtype=F64)).view(1, T, T, 1)
    A = torch.einsum("bthn,bshn->btsh", q, k) * L * mask
    o_ref = scale * torch.einsum("btsh,bshd->bthd", A, v) / Ip.view(1, 1, H, 1)
    assert torch.allclose(o, o_ref, rtol=1e-11, atol=1e-13)
    assert torch.allclose(I, Ip.view(1, H, 1, 1).expand_as(I), rtol=1e-13)


def test_gt_zero_is_cumsum():
    q, k, v, b, gt, g, Ip = small_inputs(T=6)
    gt = torch.zeros_like(gt)
    o, _, mu, I = run(q, k, v, b, gt, g, Ip, scale=1.0)
    M_T = torch.einsum("bthd,bthn->bhdn", v, k)
    J_T = torch.einsum("bthd,bthn->bhdn", b, k * k)
    assert torch.allclose(I, J_T + Ip.view(1, -1, 1, 1), rtol=1e-12)
    assert torch.allclose(mu * I, M_T, rtol=1e-11, atol=1e-13)


def test_infinite_decay_is_memoryless():
    q, k, v, b, gt, g, Ip = small_inputs(T=5)
    g = torch.full_like(g, 1e4)
    gt = gt + 1.0
    scale = 1.3
    o, _, _, _ = run(q, k, v, b, gt, g, Ip, scale=scale)
    for t in range(q.shape[1]):
        sl = slice(t, t + 1)
        o1, _, _, _ = run(q[:, sl], k[:, sl], v[:, sl], b[:, sl], gt[:, sl], g, Ip, scale=scale)
        assert torch.allclose(o[:, sl], o1, rtol=1e-12, atol=1e-14)


def test_scalar_recurrence_by_hand():
    """dk = dv = 1, two tokens, every number written out."""
    q = torch.tensor([[[[2.0]], [[-1.0]]]], dtype=F64)       # [1,2,1,1]
    k = torch.tensor([[[[0.5]], [[3.0]]]], dtype=F64)
    v = torch.tensor([[[[4.0]], [[1.0]]]], dtype=F64)
    b = torch.tensor([[[[0.25]], [[0.5]]]], dtype=F64)
    gt = torch.tensor([[[0.3], [0.7]]], dtype=F64)
    g = torch.tensor([2.0], dtype=F64)
    Ip = torch.tensor([1.5], dtype=F64)
    o, ov, mu, I = run(q, k, v, b, gt, g, Ip, scale=1.0, output_uncertainty=True)
    f2 = np.exp(-0.7 * 2.0)
    M1 = 4.0 * 0.5
    I1 = 0.25 * 0.25 + 1.5
    M2 = f2 * M1 + 1.0 * 3.0
    I2 = 0.5 * 9.0 + (1 - f2) * 1.5 + f2 * I1
    assert o[0, 0, 0, 0].item() == pytest.approx(2.0 * M1 / I1, rel=1e-14)
    assert o[0, 1, 0, 0].item() == pytest.approx(-1.0 * M2 / I2, rel=1e-14)
    assert ov[0, 1, 0, 0].item() == pytest.approx(1.0 / I2, rel=1e-14)
    assert I[0, 0, 0, 0].item() == pytest.approx(I2, rel=1e-14)
    assert mu[0, 0, 0, 0].item() == pytest.approx(M2 / I2, rel=1e-14)


# ---------------------------------------------------------------- brute force
@pytest.mark.parametrize("with_state", [False, True])
def test_against_direct_summation(with_state):
    q, k, v, b, gt, g, Ip = small_inputs(B=1, T=6, H=2, dk=3, dv=4, seed=5)
    gen = torch.Generator().manual_seed(9)
    mu0 = I0 = None
    if with_state:
        mu0 = rnd(1, 2, 4, 3, gen=gen)
        I0 = Ip.view(1, 2, 1, 1) + rnd(1, 2, 4, 3, gen=gen).abs() + 0.2
    scale = 0.61
    o, ov, mu, I = run(q, k, v, b, gt, g, Ip, mu0, I0, scale=scale, output_uncertainty=True)
    for h in range(2):
        o_r, ov_r, mu_r, I_r = po.direct_sum_outputs(
            q[0, :, h], k[0, :, h], v[0, :, h], b[0, :, h], gt[0, :, h], g[h], Ip[h], scale,
            None if mu0 is None else mu0[0, h], None if I0 is None else I0[0, h])
        assert np.allclose(o[0, :, h].numpy(), o_r, rtol=1e-11, atol=1e-13)
        assert np.allclose(ov[0, :, h].numpy(), ov_r, rtol=1e-11, atol=1e-13)
        assert np.allclose(mu[0, h].numpy(), mu_r, rtol=1e-11, atol=1e-13)
        assert np.allclose(I[0, h].numpy(), I_r, rtol=1e-12)


# ---------------------------------------------------------------- invariants
def test_split_resume_equivalence():
    q, k, v, b, gt, g, Ip = small_inputs(T=11)
    o, ov, mu, I = run(q, k, v, b, gt, g, Ip, output_uncertainty=True)
    T1 = 4
    o1, ov1, mu1, I1 = run(q[:, :T1], k[:, :T1], v[:, :T1], b[:, :T1], gt[:, :T1], g, Ip,
                           output_uncertainty=True)
    o2, ov2, mu2, I2 = run(q[:, T1:], k[:, T1:], v[:, T1:], b[:, T1:], gt[:, T1:], g, Ip,
                           mu1, I1, output_uncertainty=True)
    assert torch.allclose(torch.cat([o1, o2], 1), o, rtol=1e-12, atol=1e-14)
    assert torch.allclose(torch.cat([ov1, ov2], 1), ov, rtol=1e-12, atol=1e-14)
    assert torch.allclose(mu2, mu, rtol=1e-12, atol=1e-14)
    assert torch.allclose(I2, I, rtol=1e-12)


def test_varlen_equals_per_document_runs():
    q, k, v, b, gt, g, Ip = small_inputs(B=1, T=13)
    cu = [0, 3, 4, 10, 13]
    gen = torch.Generator().manual_seed(3)
    mu0 = rnd(4, 3, 5, 4, gen=gen)
    I0 = Ip.view(1, 3, 1, 1) + rnd(4, 3, 5, 4, gen=gen).abs()
    o, _, mu, I = run(q, k, v, b, gt, g, Ip, mu0, I0, cu_seqlens=cu)
    for n in range(4):
        s, e = cu[n], cu[n + 1]
        on, _, mun, In = run(q[:, s:e], k[:, s:e], v[:, s:e], b[:, s:e], gt[:, s:e], g, Ip,
                             mu0[n:n + 1], I0[n:n + 1])
        assert torch.equal(o[:, s:e], on)
        assert torch.equal(mu[n:n + 1], mun)
        assert torch.equal(I[n:n + 1], In)


def test_linearity_in_v_and_precision_bound():
    q, k, v, b, gt, g, Ip = small_inputs()
    gen = torch.Generator().manual_seed(4)
    v2 = rnd(*v.shape, gen=gen)
    o1, _, _, I1 = run(q, k, v, b, gt, g, Ip)
    o2, _, _, _ = run(q, k, v2, b, gt, g, Ip)
    o12, _, _, _ = run(q, k, 2.0 * v - 3.0 * v2, b, gt, g, Ip)
    assert torch.allclose(o12, 2.0 * o1 - 3.0 * o2, rtol=1e-11, atol=1e-12)
    # b >= 0 and I0 = Ip  =>  I_t >= Ip
    assert (I1 >= Ip.view(1, -1, 1, 1) * (1 - 1e-14)).all()


def test_head_and_batch_permutation_equivariance():
    q, k, v, b, gt, g, Ip = small_inputs()
    perm = torch.tensor([2, 0, 1])
    o, _, mu, I = run(q, k, v, b, gt, g, Ip)
    op, _, mup, Ipp = run(q[:, :, perm], k[:, :, perm], v[:, :, perm], b[:, :, perm], gt[:, :, perm],
                          g[perm], Ip[perm])
    assert torch.equal(op, o[:, :, perm])
    assert torch.equal(mup, mu[:, perm])


# ---------------------------------------------------------------- gradients
def test_gradcheck_float64():
    q, k, v, b, gt, g, Ip = small_inputs(B=1, T=4, H=2, dk=2, dv=3)
    gen = torch.Generator().manual_seed(8)
    mu0 = rnd(1, 2, 3, 2, gen=gen)
    I0 = Ip.view(1, 2, 1, 1) + rnd(1, 2, 3, 2, gen=gen).abs() + 0.3
    leaves = [x.clone().requires_grad_(True) for x in (q, k, v, b, gt, g, Ip, mu0, I0)]

    def fn(*xs):
        o, ov, mu, I = run(*xs, scale=0.7, output_uncertainty=True)
        return o, ov, mu, I

    assert torch.autograd.gradcheck(fn, leaves, eps=1e-6, atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("with_state,with_var", [(False, False), (True, False), (False, True), (True, True)])
def test_hand_derived_backward_matches_autograd(with_state, with_var):
    """The formulas the HIP backward kernels implement (incl. the reverse-cumsum form of dgt)."""
    B, T, H, dk, dv = 1, 9, 2, 3, 4
    q, k, v, b, gt, g, Ip = small_inputs(B=B, T=T, H=H, dk=dk, dv=dv, seed=11)
    gen = torch.Generator().manual_seed(12)
    mu0 = I0 = None
    if with_state:
        mu0 = rnd(B, H, dv, dk, gen=gen)
        I0 = Ip.view(1, H, 1, 1) + rnd(B, H, dv, dk, gen=gen).abs() + 0.3
    do = rnd(B, T, H, dv, gen=gen)
    dovar = rnd(B, T, H, dv, gen=gen) if with_var else None
    scale = 0.45
    names = ["q", "k", "v", "b", "gt", "g", "Ip"] + (["mu0", "I0"] if with_state else [])
    leaves = [x.clone().requires_grad_(True) for x in (q, k, v, b, gt, g, Ip)]
    if with_state:
        leaves += [mu0.clone().requires_grad_(True), I0.clone().requires_grad_(True)]
    o, ov, _, _ = run(*leaves, scale=scale, output_uncertainty=with_var)
    loss = (o * do).sum()
    if with_var:
        loss = loss + (ov * dovar).sum()
    grads = dict(zip(names, torch.autograd.grad(loss, leaves)))
    dg_tot = np.zeros(H)
    dIp_tot = np.zeros(H)
    for h in range(H):
        r = po.backward_formulas(
            q[0, :, h], k[0, :, h], v[0, :, h], b[0, :, h], gt[0, :, h], g[h], Ip[h], scale,
            do[0, :, h], None if dovar is None else dovar[0, :, h],
            None if mu0 is None else mu0[0, h], None if I0 is None else I0[0, h])
        for nm, key in (("q", "dq"), ("k", "dk"), ("v", "dv"), ("b", "db"), ("gt", "dgt")):
            ref = grads[nm][0, :, h].numpy()
            assert np.allclose(r[key], ref, rtol=1e-9, atol=1e-11), (nm, np.abs(r[key] - ref).max())
        dg_tot[h] = r["dg"]
        dIp_tot[h] = r["dIp"]
        if with_state:
            assert np.allclose(r["dmu0"], grads["mu0"][0, h].numpy(), rtol=1e-9, atol=1e-11)
            assert np.allclose(r["dI0"], grads["I0"][0, h].numpy(), rtol=1e-9, atol=1e-11)
    assert np.allclose(dg_tot, grads["g"].numpy(), rtol=1e-9, atol=1e-11)
    assert np.allclose(dIp_tot, grads["Ip"].numpy(), rtol=1e-9, atol=1e-11)


# ---------------------------------------------------------------- integer helpers
def test_chunk_table_helpers():
    cu = [0, 5, 5 + 64, 5 + 64 + 130]
    assert po.chunk_offsets(cu, 64) == [0, 1, 2, 5]
    rows = po.build_chunk_table(cu, 64)
    assert rows == [(0, 0, 5), (1, 5, 64), (2, 69, 64), (2, 133, 64), (2, 197, 2)]
    assert po.chunk_offsets([0, 16], 16) == [0, 1]
    assert sum(r[2] for r in rows) == cu[-1]


def test_varlen_length_generator():
    cu = po.make_varlen_lengths(32768, seed=0)
    lens = np.diff(cu)
    assert cu[0] == 0 and cu[-1] == 32768
    assert lens.min() >= 16 and lens.max() <= 4096 + 16
    assert cu == po.make_varlen_lengths(32768, seed=0)
