"""Pins of oracle/layer_glue_oracle.py that need no GPU: library routines and invariants the formulas reduce to."""
import torch
import torch.nn.functional as F

from oracle import layer_glue_oracle as lo


def _inputs(lead, Hqk, H, dk, dv, seed, dtype=torch.float64):
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64).to(dtype)
    return dict(q_raw=r(*lead, Hqk, dk), k_raw=r(*lead, Hqk, dk), x=r(*lead, H, dv), dt_raw=r(*lead, H),
                dt_bias=r(H), bs_raw=r(*lead, H), b_raw=r(*lead, H, dv), b_scale=r(H))


def test_prologue_unit_norm_repeat_and_ranges():
    a = _inputs((2, 5), 2, 6, 16, 24, 0)
    q, k, v, b, gt = lo.prologue(**a)
    assert q.shape == (2, 5, 6, 16) and v.shape == (2, 5, 6, 24) and gt.shape == (2, 5, 6)
    assert torch.allclose(q.norm(dim=-1), torch.ones(2, 5, 6, dtype=torch.float64), atol=1e-12)
    # einops' '... h d -> ... (h g) d' puts the g copies of a head next to each other
    for h in range(6):
        assert torch.equal(q[..., h, :], q[..., (h // 3) * 3, :])
        src = a["k_raw"][..., h // 3, :]
        assert torch.allclose(k[..., h, :], src / src.norm(dim=-1, keepdim=True), atol=1e-12)
    assert (gt > 0).all()
    bs = torch.sigmoid(a["bs_raw"])
    assert torch.allclose(v, a["x"] * bs[..., None], atol=1e-12)
    # b lies in (0, softplus(b_scale)) as the layer intends
    assert (b > 0).all() and (b < F.softplus(a["b_scale"]).view(-1, 1)).all()
    assert torch.allclose(b / bs[..., None] / F.softplus(a["b_scale"]).view(-1, 1), torch.sigmoid(a["b_raw"]), atol=1e-12)
    # the reference rounds bs to the model dtype before it is used
    _, _, v16, _, _ = lo.prologue(**a, model_dtype=torch.bfloat16)
    assert torch.equal(v16, a["x"] * bs.to(torch.bfloat16).double()[..., None])
    # without b
    a2 = dict(a, b_raw=None, b_scale=None)
    assert lo.prologue(**a2)[3] is None


def test_prologue_zero_row_is_clamped_not_nan():
    a = _inputs((3,), 1, 1, 8, 8, 1)
    a["q_raw"][1] = 0
    q = lo.prologue(**a)[0]
    assert torch.isfinite(q).all() and (q[1] == 0).all()


def test_epilogue_reduces_to_library_routines():
    gen = torch.Generator().manual_seed(2)
    o = torch.randn(4, 7, 3, 32, generator=gen, dtype=torch.float64)
    x = torch.randn(4, 7, 3, 32, generator=gen, dtype=torch.float64)
    g = torch.randn(4, 7, 3, 32, generator=gen, dtype=torch.float64)
    D = torch.randn(3, generator=gen, dtype=torch.float64)
    w = torch.randn(32, generator=gen, dtype=torch.float64)
    eps = 1e-5
    assert torch.allclose(lo.epilogue(o, None, None, None, w, eps), F.rms_norm(o, (32,), w, eps), atol=1e-12)
    r = o + x * D.view(3, 1)
    assert torch.allclose(lo.epilogue(o, x, D, None, w, eps), F.rms_norm(r, (32,), w, eps), atol=1e-12)
    assert torch.allclose(lo.epilogue(o, x, D, g, w, eps), F.rms_norm(r, (32,), w, eps) * F.silu(g), atol=1e-12)
    # scale invariance of the norm (eps -> 0)
    assert torch.allclose(lo.epilogue(3.0 * o, None, None, None, w, 0.0), lo.epilogue(o, None, None, None, w, 0.0), atol=1e-12)


def test_gradcheck_of_both_functions():
    a = _inputs((2,), 1, 2, 8, 8, 3)
    names = list(a)
    leaves = [a[n].clone().requires_grad_(True) for n in names]

    def f(*xs):
        q, k, v, b, gt = lo.prologue(**dict(zip(names, xs)))
        return q, k, v, b, gt

    assert torch.autograd.gradcheck(f, leaves, atol=1e-8)
    gen = torch.Generator().manual_seed(4)
    ts = [torch.randn(2, 2, 8, generator=gen, dtype=torch.float64).requires_grad_(True) for _ in range(3)]
    D = torch.randn(2, generator=gen, dtype=torch.float64).requires_grad_(True)
    w = torch.randn(8, generator=gen, dtype=torch.float64).requires_grad_(True)
    assert torch.autograd.gradcheck(lambda o, x, g, D, w: lo.epilogue(o, x, D, g, w, 1e-5), ts + [D, w], atol=1e-8)


def test_mamba_prologue_clamp_and_products():
    a = _inputs((2, 9), 1, 4, 8, 16, 5)
    v, b, dt = lo.mamba_prologue(a["x"], a["dt_raw"], a["dt_bias"], a["b_raw"], a["b_scale"], dt_limit=(0.3, 1.2))
    sp = F.softplus(a["dt_raw"] + a["dt_bias"])
    assert dt.min() >= 0.3 and dt.max() <= 1.2
    inside = (sp > 0.3) & (sp < 1.2)
    assert inside.any() and (~inside).any()
    assert torch.equal(dt[inside], sp[inside])
    assert torch.allclose(v, a["x"] * dt[..., None], atol=1e-12)
    assert torch.allclose(b / dt[..., None] / F.softplus(a["b_scale"]).view(-1, 1), torch.sigmoid(a["b_raw"]), atol=1e-12)
    # the layer's default limits leave softplus as it is
    assert torch.equal(lo.mamba_prologue(a["x"], a["dt_raw"], a["dt_bias"])[2], sp)
    assert lo.mamba_prologue(a["x"], a["dt_raw"], a["dt_bias"])[1] is None


def test_mamba_epilogue_reduces_to_library_routines():
    gen = torch.Generator().manual_seed(6)
    o = torch.randn(3, 5, 4, 24, generator=gen, dtype=torch.float64)
    x = torch.randn(3, 5, 4, 24, generator=gen, dtype=torch.float64)
    g = torch.randn(3, 5, 96, generator=gen, dtype=torch.float64)
    D = torch.randn(4, generator=gen, dtype=torch.float64)
    w = torch.randn(96, generator=gen, dtype=torch.float64)
    eps = 1e-5
    r = (o + x * D.view(4, 1)).flatten(-2)
    assert torch.allclose(lo.mamba_epilogue(o, None, None, None, w, eps).flatten(-2), F.rms_norm(o.flatten(-2), (96,), w, eps), atol=1e-12)
    assert torch.allclose(lo.mamba_epilogue(o, x, D, g, w, eps).flatten(-2), F.rms_norm(r * F.silu(g), (96,), w, eps), atol=1e-12)
    # the mean square runs over all heads of a token: scaling one head changes the others' outputs
    o2 = o.clone()
    o2[..., 0, :] *= 3.0
    assert not torch.allclose(lo.mamba_epilogue(o2, None, None, None, w, eps)[..., 1, :], lo.mamba_epilogue(o, None, None, None, w, eps)[..., 1, :])


def test_mamba_glue_gradcheck():
    a = _inputs((3,), 1, 2, 8, 8, 7)
    leaves = [a[n].clone().requires_grad_(True) for n in ("x", "dt_raw", "dt_bias", "b_raw", "b_scale")]
    assert torch.autograd.gradcheck(lambda *t: lo.mamba_prologue(*t, dt_limit=(0.0, 50.0)), leaves, atol=1e-8)
    gen = torch.Generator().manual_seed(8)
    mk = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64).requires_grad_(True)
    o, x, g, D, w = mk(3, 2, 8), mk(3, 2, 8), mk(3, 2, 8), mk(2), mk(16)
    assert torch.autograd.gradcheck(lambda *t: lo.mamba_epilogue(*t, 1e-5), (o, x, D, g, w), atol=1e-8)
