"""The reference's own correctness script, run on the chunked HIP path, and the second caller's call shape.

palimpsa/check_palimpsa.py of the reference compares ``chunk_palimpsa`` with ``palimpsa_ref`` on deliberately
awkward inputs (:43-59): B,L,H,D,N = 4,511,4,65,31 (dv = 65, dk = 31, L not a multiple of any tile), seed 42,
q, k ~ N(0,1) *not* normalised, b = sigmoid(N), gt = sigmoid(N), g = |N|*10 + 1, Ip = |N| + 0.1, scale = 1,
both outputs requested, loss ((o - target)^2 / (o_var + 1e-6)).sum() so that both dO and dO_var flow
(:89-123); then the same packed into one row with seqlens [128, 64, rest] against a per-document loop
(:129-187); then with an initial state I0 = Ip + relu(N) + 1 (:193-246).  The script prints and asserts
nothing; its own pass criterion (:34-37) is allclose(atol=1e-2, rtol=1e-2).  Here the same topology (fewer
batch rows, to keep the float64 oracle short) is asserted, fwd + every gradient, with the plain max-norm:

* bf16 rows: outputs max|d| <= 2e-2 * max(1, max|ref|) (rows are not normalised here, so |o| reaches ~10 and one
  bf16 ulp of the output is already 2e-2 absolute; for |o| <= 1 this is the 2e-2 absolute bar), gradients
  max|d| / max|ref| <= 5e-2;
* fp32 rows: the bars of helpers.CHUNK_FP32_* (see there).

The loss is evaluated through the kernel's own outputs (as the script does), so the comparison includes the
effect of output rounding on dO.

MetaMamba2.forward (palimpsa/layers/meta_mamba2.py:281-299, :333) calls the same operator with scale = 1.0,
q = C and k = B straight from the convolution (not normalised), v = x*dt, b = b*dt with dt a small positive
step, heads repeated from n_groups, dk = state_size in {48, 96}, dv = head_dim in {96, 192}.
"""
import pytest
import torch

from oracle import palimpsa_oracle as po
from tests import helpers as hp

pytestmark = pytest.mark.gpu

NAMES = ["q", "k", "v", "b", "gt", "g", "Ip"]


def _check_script_inputs(B=2, L=511, H=4, D=65, N=31, seed=42):
    gen = torch.Generator().manual_seed(seed)
    v = torch.randn(B, L, H, D, generator=gen)
    q = torch.randn(B, L, H, N, generator=gen)
    k = torch.randn(B, L, H, N, generator=gen)
    b = torch.sigmoid(torch.randn(B, L, H, D, generator=gen))
    gt = torch.sigmoid(torch.randn(B, L, H, generator=gen))
    g = torch.randn(H, generator=gen).abs() * 10 + 1
    Ip = torch.randn(H, generator=gen).abs() + 0.1
    target = torch.randn(B, L, H, D, generator=gen)
    return dict(q=q, k=k, v=v, b=b, gt=gt, g=g, Ip=Ip), target


def _loss(o, o_var, target):
    return ((o - target) ** 2 / (o_var + 1e-6)).sum()


def _oracle(inp, target, cu=None, mu0=None, I0=None):
    """float64 oracle on the rows as the kernel sees them: outputs and gradients of the script's loss."""
    leaves = [inp[n].detach().double().clone().requires_grad_(True) for n in NAMES]
    st = []
    if mu0 is not None:
        st = [mu0.detach().double().clone().requires_grad_(True), I0.detach().double().clone().requires_grad_(True)]
    o, ov, fmu, fI = po.palimpsa_recurrence(*leaves, *(st if st else [None, None]), scale=1.0, cu_seqlens=cu,
                                            output_uncertainty=True, var_scale_power=1, compute_dtype=torch.float64)
    gr = torch.autograd.grad(_loss(o, ov, target.double()), leaves + st)
    out = dict(zip(NAMES + (["mu0", "I0"] if st else []), gr))
    out.update(o=o.detach(), o_var=ov.detach(), fmu=fmu.detach(), fI=fI.detach())
    return out


def _kernel(inp, target, dev, dtype, cu=None, mu0=None, I0=None):
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa
    leaves = {n: inp[n].to(dev).clone().requires_grad_(True) for n in NAMES}
    kw = {}
    if mu0 is not None:
        leaves["mu0"] = mu0.to(dev).clone().requires_grad_(True)
        leaves["I0"] = I0.to(dev).clone().requires_grad_(True)
        kw.update(initial_mu_state=leaves["mu0"], initial_I_state=leaves["I0"])
    if cu is not None:
        kw["cu_seqlens"] = torch.tensor(cu, device=dev)
    (o, ov), fmu, fI = chunk_palimpsa(*[leaves[n] for n in NAMES], scale=1, chunk_size=16, output_final_state=True,
                                      output_uncertainty=True, **kw)
    assert o.dtype == dtype and ov.dtype == dtype
    _loss(o.float(), ov.float(), target.to(dev)).backward()
    out = {n: x.grad for n, x in leaves.items()}
    out.update(o=o.detach(), o_var=ov.detach(), fmu=fmu, fI=fI)
    return out


def _assert_close(got, ref, names, dtype):
    bad = {}
    for n in ("o", "o_var"):
        den = max(1.0, ref[n].abs().max().item())
        e = hp.max_abs(got[n].float(), ref[n]) / den
        tol = hp.BF16_OUT_ABS_TOL if dtype == torch.bfloat16 else hp.CHUNK_FP32_OUT_TOL
        print(f"{n:5s}: max|d|/max(1,max|ref|) = {e:.3e}   (max|ref| = {ref[n].abs().max().item():.3g})")
        if not e <= tol:
            bad[n] = e
    for n in ("fmu", "fI"):
        e = hp.max_rel(got[n], ref[n])
        tol = 5e-3 if dtype == torch.bfloat16 else hp.CHUNK_FP32_OUT_TOL
        print(f"{n:5s}: max|d|/max|ref| = {e:.3e}")
        if not e <= tol:
            bad[n] = e
    for n in names:
        e = hp.max_rel(got[n], ref[n])
        e_mean = hp.mean_norm(got[n], ref[n])
        tol = hp.BF16_GRAD_NORM_TOL if dtype == torch.bfloat16 else hp.CHUNK_FP32_GRAD_TOL
        print(f"d{n:4s}: max|d|/max|ref| = {e:.3e}   max|d|/mean|ref| = {e_mean:.3e}")
        if not e <= tol:
            bad["d" + n] = e
    assert not bad, bad


def _rows(inp, dtype):
    return hp.rounded(inp, dtype) if dtype == torch.bfloat16 else inp


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_check_script_dense(gpu_device, dtype):
    """TEST 1 of the script (check_palimpsa.py:89-123)."""
    inp, target = _check_script_inputs()
    inp = _rows(inp, dtype)
    ref = _oracle(inp, target)
    got = _kernel(inp, target, gpu_device, dtype)
    _assert_close(got, ref, NAMES, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_check_script_packed(gpu_device, dtype):
    """TEST 2 (check_palimpsa.py:129-187): the batch packed into one row, seqlens [128, 64, rest]; dg and dIp are
    summed over the documents."""
    inp, target = _check_script_inputs()
    B, L = inp["q"].shape[:2]
    packed = {n: (inp[n].reshape(1, B * L, *inp[n].shape[2:]) if n in ("q", "k", "v", "b", "gt") else inp[n])
              for n in NAMES}
    packed = _rows(packed, dtype)
    target = target.reshape(1, B * L, *target.shape[2:])
    cu = [0, 128, 192, B * L]
    ref = _oracle(packed, target, cu=cu)
    got = _kernel(packed, target, gpu_device, dtype, cu=cu)
    _assert_close(got, ref, NAMES, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_check_script_initial_state(gpu_device, dtype):
    """TEST 3 (check_palimpsa.py:193-246): mu0 ~ N(0,1), I0 = Ip + relu(N) + 1; the gradients of the initial state
    (None in the reference, :617-620) are compared as well."""
    inp, target = _check_script_inputs()
    inp = _rows(inp, dtype)
    B, _, H, D = inp["v"].shape
    N = inp["k"].shape[-1]
    gen = torch.Generator().manual_seed(43)
    mu0 = torch.randn(B, H, D, N, generator=gen)
    I0 = inp["Ip"].view(1, H, 1, 1) + torch.relu(torch.randn(B, H, D, N, generator=gen)) + 1.0
    ref = _oracle(inp, target, mu0=mu0, I0=I0)
    got = _kernel(inp, target, gpu_device, dtype, mu0=mu0, I0=I0)
    _assert_close(got, ref, NAMES + ["mu0", "I0"], dtype)


# --------------------------------------------------------------------------- MetaMamba2 call shape
def _mamba_inputs(B, T, H, n_groups, dk, dv, seed):
    """Operator inputs as MetaMamba2.forward builds them (meta_mamba2.py:281-299): B, C from a SiLU-activated
    convolution (O(1), not normalised), repeated over the heads of a group; dt = softplus(.) clamped to a small
    positive step; v = x*dt, b = sigmoid(.)*dt; g = A in (1, 16)."""
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen)
    silu = torch.nn.functional.silu
    Bm = silu(r(B, T, n_groups, dk) * 1.5)
    Cm = silu(r(B, T, n_groups, dk) * 1.5)
    rep = H // n_groups
    k = Bm.repeat_interleave(rep, dim=2)
    q = Cm.repeat_interleave(rep, dim=2)
    dt = torch.clamp(torch.nn.functional.softplus(r(B, T, H) - 3.0), 1e-3, 0.1)
    x = silu(r(B, T, H, dv))
    v = x * dt.unsqueeze(-1)
    b = torch.sigmoid(r(B, T, H, dv)) * dt.unsqueeze(-1)
    g = torch.rand(H, generator=gen) * 15 + 1
    Ip = torch.ones(H)
    return dict(q=q, k=k, v=v, b=b, gt=dt, g=g, Ip=Ip)


@pytest.mark.parametrize("dk,dv", [(48, 96), (96, 192)])
def test_meta_mamba2_call_shape_forward_backward(gpu_device, dk, dv):
    """scale = 1.0, q = C, k = B not normalised, v = x*dt and b = b*dt of order 1e-2, grouped heads: chunked
    forward + backward of every input against the float64 oracle; squared-error loss (dO correlated with the
    state, as in training), plain max-norm bars."""
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa
    B, T, H, G = 2, 300, 4, 2
    inp = hp.rounded(_mamba_inputs(B, T, H, G, dk, dv, seed=dk + dv), torch.bfloat16)
    gen = torch.Generator().manual_seed(9)
    target = 0.05 * torch.randn(B, T, H, dv, generator=gen)
    leaves64 = [inp[n].double().clone().requires_grad_(True) for n in NAMES]
    o_ref, _, fmu_ref, fI_ref = po.palimpsa_recurrence(*leaves64, scale=1.0, compute_dtype=torch.float64)
    ref = dict(zip(NAMES, torch.autograd.grad(0.5 * ((o_ref - target.double()) ** 2).sum(), leaves64)))
    dev = gpu_device
    leaves = {n: inp[n].to(dev).clone().requires_grad_(True) for n in NAMES}
    o, fmu, fI = chunk_palimpsa(*[leaves[n] for n in NAMES], scale=1.0, chunk_size=16, output_final_state=True)
    (0.5 * ((o.float() - target.to(dev)) ** 2).sum()).backward()
    e_o = hp.max_abs(o.float(), o_ref.detach()) / max(1.0, o_ref.abs().max().item())
    print(f"o: max|d| = {hp.max_abs(o.float(), o_ref.detach()):.3e}, max|ref| = {o_ref.abs().max().item():.3g}")
    assert e_o <= hp.BF16_OUT_ABS_TOL
    # relative as well: the outputs are small here (v carries dt), an absolute bar alone would be empty
    assert hp.max_rel(o.float(), o_ref.detach()) <= 2e-2
    assert hp.max_rel(fmu, fmu_ref.detach()) <= 5e-3 and hp.max_rel(fI, fI_ref.detach()) <= 5e-3
    bad = {}
    for n in NAMES:
        e = hp.max_rel(leaves[n].grad, ref[n])
        print(f"d{n:4s}: max|d|/max|ref| = {e:.3e}   max|d|/mean|ref| = {hp.mean_norm(leaves[n].grad, ref[n]):.3e}")
        if not e <= hp.BF16_GRAD_NORM_TOL:
            bad[n] = e
    assert not bad, bad


@pytest.mark.parametrize("path", ["chunk_bf16", "chunk_fp32", "recurrent_fp32"])
def test_shared_qk_heads_are_indexed_not_repeated(gpu_device, path):
    """q = C and k = B of MetaMamba2 belong to n_groups < H groups and the layer repeats them over the heads of a
    group before the call (meta_mamba2.py:281-282; Palimpsa.forward does the same with num_heads < num_v_heads,
    palimpsa.py:266-267).  Both entry points also take the un-repeated [B,T,Hq,dk] tensors and index the shared rows:
    outputs, states and every gradient must equal the oracle on the repeated inputs, with dq, dk summed over the
    heads of each group."""
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa, fused_recurrent_palimpsa
    B, T, H, G, dk, dv = 2, 200, 6, 2, 48, 96
    rep = H // G
    full = _mamba_inputs(B, T, H, G, dk, dv, seed=31)
    dtype = torch.bfloat16 if path == "chunk_bf16" else torch.float32
    if dtype == torch.bfloat16:
        full = hp.rounded(full, dtype)
    gen = torch.Generator().manual_seed(32)
    target = 0.05 * torch.randn(B, T, H, dv, generator=gen)
    mu0 = torch.randn(B, H, dv, dk, generator=gen) * 0.05
    I0 = 1.0 + torch.rand(B, H, dv, dk, generator=gen)
    leaves64 = [full[n].double().clone().requires_grad_(True) for n in NAMES]
    st64 = [mu0.double().clone().requires_grad_(True), I0.double().clone().requires_grad_(True)]
    o_ref, _, fmu_ref, fI_ref = po.palimpsa_recurrence(*leaves64, *st64, scale=1.0, compute_dtype=torch.float64)
    gr = torch.autograd.grad(0.5 * ((o_ref - target.double()) ** 2).sum(), leaves64 + st64)
    ref = dict(zip(NAMES + ["mu0", "I0"], gr))
    for n in ("q", "k"):     # the gradient of a shared row is the sum over the heads that read it
        ref[n] = ref[n].reshape(B, T, G, rep, dk).sum(3)
    dev = gpu_device
    leaves = {n: full[n].to(dev).clone() for n in NAMES}
    for n in ("q", "k"):
        leaves[n] = leaves[n][:, :, ::rep].contiguous()              # one row per group
        assert leaves[n].shape == (B, T, G, dk)
    leaves = {n: x.requires_grad_(True) for n, x in leaves.items()}
    leaves["mu0"] = mu0.to(dev).requires_grad_(True)
    leaves["I0"] = I0.to(dev).requires_grad_(True)
    fn = fused_recurrent_palimpsa if path == "recurrent_fp32" else chunk_palimpsa
    o, fmu, fI = fn(*[leaves[n] for n in NAMES], scale=1.0, initial_mu_state=leaves["mu0"],
                    initial_I_state=leaves["I0"], output_final_state=True)
    (0.5 * ((o.float() - target.to(dev)) ** 2).sum()).backward()
    bf = dtype == torch.bfloat16
    assert hp.max_rel(o.float(), o_ref.detach()) <= (2e-2 if bf else hp.FP32_REL_TOL)
    assert hp.max_rel(fmu, fmu_ref.detach()) <= (5e-3 if bf else hp.FP32_REL_TOL)
    assert hp.max_rel(fI, fI_ref.detach()) <= (5e-3 if bf else hp.FP32_REL_TOL)
    bad = {}
    for n in NAMES + ["mu0", "I0"]:
        assert leaves[n].grad.shape == leaves[n].shape
        e = hp.max_rel(leaves[n].grad, ref[n])
        print(f"d{n:4s}: max|d|/max|ref| = {e:.3e}")
        if not e <= (hp.BF16_GRAD_NORM_TOL if bf else hp.CHUNK_FP32_GRAD_TOL):
            bad[n] = e
    assert not bad, bad


# --------------------------------------------------------------------------- prefill -> decode hand-off
def test_chunk_prefill_then_recurrent_decode_steps(gpu_device):
    """The layer's generate flow (layers/palimpsa.py:302-331): a chunked prefill returns (final_mu, final_I), which
    the cache hands to fused_recurrent_palimpsa for the following single-token steps.  Checked against one oracle
    run over the concatenation."""
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa, fused_recurrent_palimpsa
    B, T0, steps, H, dk, dv = 2, 150, 16, 3, 48, 96
    inp = hp.rounded(po.make_inputs(B, T0 + steps, H, dk, dv, seed=17), torch.bfloat16)
    inp["g"] = torch.tensor([0.5, 2.0, 9.0])
    o_ref, _, mu_ref, I_ref = hp.oracle_forward(inp, dtype=torch.float64)
    d = hp.to_device(inp, gpu_device)
    rows = ("q", "k", "v", "b", "gt")
    head = [d[n][:, :T0] for n in rows]
    o0, mu, I = chunk_palimpsa(*head, d["g"], d["Ip"], chunk_size=16, output_final_state=True)
    outs = [o0]
    for t in range(T0, T0 + steps):
        tok = [d[n][:, t:t + 1] for n in rows]
        o1, mu, I = fused_recurrent_palimpsa(*tok, d["g"], d["Ip"], initial_mu_state=mu, initial_I_state=I,
                                             output_final_state=True)
        outs.append(o1)
    o = torch.cat(outs, dim=1)
    assert hp.max_abs(o.float(), o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_abs(o[:, T0:].float(), o_ref[:, T0:]) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu, mu_ref) <= 5e-3 and hp.max_rel(I, I_ref) <= 5e-3
