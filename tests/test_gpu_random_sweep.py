"""Seeded random sweep over shapes and call options: the chunked kernels against the token-serial kernels.

Both run on the GPU through the C ABI; the token-serial kernels are fp32 end to end and are themselves checked
against the oracle (test_gpu_recurrent.py), so this sweep reaches head dims, packings and option combinations that
the fixed cases do not list, at sizes where the float64 oracle would take minutes.  Every case is derived from its
seed alone, so a failure names its case."""
import random

import pytest
import torch

from oracle import palimpsa_oracle as po
from tests import helpers as hp

pytestmark = pytest.mark.gpu

HEAD_DIMS = [16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256]


def _case(seed):
    rng = random.Random(seed)
    dk, dv = rng.choice(HEAD_DIMS), rng.choice(HEAD_DIMS)
    H = rng.choice([1, 2, 3, 4, 6])
    hq = rng.choice([d for d in (1, 2, 3, 4, 6) if H % d == 0])
    packed = rng.random() < 0.5
    if packed:
        n = rng.randint(1, 5)
        lens = [rng.choice([0, 1, 2, 17, 63, 64, 65, 100, 129, 200]) for _ in range(n)]
        if sum(lens) == 0:
            lens[-1] = 33
        cu = [0]
        for ln in lens:
            cu.append(cu[-1] + ln)
        B, T = 1, cu[-1]
    else:
        cu = None
        B, T = rng.randint(1, 3), rng.choice([1, 40, 64, 130, 257])
    return dict(dk=dk, dv=dv, H=H, hq=hq, cu=cu, B=B, T=T, var=rng.random() < 0.4, init=rng.random() < 0.5,
                g_value=rng.choice([0.3, 1.0, 4.0, 12.0]), scale=rng.choice([None, 1.0]),
                normalize=rng.random() < 0.7)


def _inputs(c, seed, dev):
    inp = po.make_inputs(c["B"], c["T"], c["H"], c["dk"], c["dv"], seed=seed, g_value=c["g_value"],
                         normalize_qk=c["normalize"])
    if c["hq"] != c["H"]:
        inp["q"] = inp["q"][:, :, :c["hq"]].contiguous()
        inp["k"] = inp["k"][:, :, :c["hq"]].contiguous()
    if not c["normalize"]:
        inp["q"] = inp["q"] * 0.5
        inp["k"] = inp["k"] * 0.5
    inp = hp.rounded(inp, torch.bfloat16)
    n = (len(c["cu"]) - 1) if c["cu"] else c["B"]
    gen = torch.Generator().manual_seed(seed + 1)
    mu0 = I0 = None
    if c["init"]:
        mu0 = (torch.randn(n, c["H"], c["dv"], c["dk"], generator=gen) * 0.1).to(dev)
        I0 = (1.0 + torch.rand(n, c["H"], c["dv"], c["dk"], generator=gen)).to(dev)
    cu = torch.tensor(c["cu"], device=dev) if c["cu"] else None
    return hp.to_device(inp, dev), mu0, I0, cu


@pytest.mark.parametrize("seed", range(100, 164))
def test_chunked_forward_matches_token_serial(gpu_device, seed):
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa, fused_recurrent_palimpsa
    c = _case(seed)
    d, mu0, I0, cu = _inputs(c, seed, gpu_device)
    kw = dict(scale=c["scale"], initial_mu_state=mu0, initial_I_state=I0, output_final_state=True,
              output_uncertainty=c["var"], cu_seqlens=cu)
    with torch.no_grad():
        out_c, mu_c, I_c = chunk_palimpsa(d["q"], d["k"], d["v"], d["b"], d["gt"], d["g"], d["Ip"], chunk_size=64, **kw)
        rows = {n: d[n].float() for n in ("q", "k", "v", "b")}          # fp32 rows: the fp32 token-serial kernel
        out_r, mu_r, I_r = fused_recurrent_palimpsa(rows["q"], rows["k"], rows["v"], rows["b"], d["gt"], d["g"],
                                                    d["Ip"], **kw)
    o_c, o_r = (out_c[0], out_r[0]) if c["var"] else (out_c, out_r)
    # the output bar is an absolute one for O(1) outputs; un-normalised q, k with scale = 1 give larger ones
    assert hp.max_abs(o_c, o_r) <= hp.BF16_OUT_ABS_TOL * max(1.0, o_r.abs().max().item()), c
    if c["var"]:
        assert hp.max_rel(out_c[1], out_r[1]) <= 2e-2, c
    assert hp.max_rel(mu_c, mu_r) <= 5e-3 and hp.max_rel(I_c, I_r) <= 5e-3, c


@pytest.mark.parametrize("seed", range(200, 232))
def test_chunked_backward_matches_token_serial(gpu_device, seed):
    from palimpsa_amd import _lib as L
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa, fused_recurrent_palimpsa
    c = _case(seed)
    if not L.load().pal_chunk_bwd_supported(-(-c["dk"] // 16) * 16, -(-c["dv"] // 16) * 16, L.PAL_DTYPE_BF16, 0) == 0:
        c["dk"], c["dv"] = 96, 64
    d, mu0, I0, cu = _inputs(c, seed, gpu_device)
    gen = torch.Generator().manual_seed(seed + 2)
    do = torch.randn(c["B"], c["T"], c["H"], c["dv"], generator=gen).to(gpu_device)
    dov = torch.randn(c["B"], c["T"], c["H"], c["dv"], generator=gen).to(gpu_device) * 0.1
    names = ("q", "k", "v", "b", "gt", "g", "Ip")

    def grads(fn, rows_dtype):
        leaves = [d[n].to(rows_dtype if n in ("q", "k", "v", "b") else torch.float32).clone().requires_grad_(True)
                  for n in names]
        st = [x.clone().requires_grad_(True) for x in (mu0, I0)] if c["init"] else [None, None]
        out = fn(*leaves, scale=c["scale"], initial_mu_state=st[0], initial_I_state=st[1],
                 output_uncertainty=c["var"], cu_seqlens=cu)
        loss = ((out[0].float() * do).sum() + (out[1].float() * dov).sum()) if c["var"] else (out.float() * do).sum()
        gr = torch.autograd.grad(loss, leaves + ([s for s in st] if c["init"] else []))
        return dict(zip(names + (("mu0", "I0") if c["init"] else ()), gr))

    g_c = grads(lambda *a, **k: chunk_palimpsa(*a, chunk_size=64, **k), torch.bfloat16)
    g_r = grads(fused_recurrent_palimpsa, torch.float32)
    for n in g_r:
        if n == "g":
            continue                     # an ill-conditioned sum under a random dO: see test_gpu_chunk_bwd.py
        assert hp.max_rel(g_c[n].float(), g_r[n].float()) <= hp.BF16_GRAD_NORM_TOL, (n, c)


@pytest.mark.parametrize("seed", range(300, 320))
def test_chunked_forward_fp32_rows_match_token_serial_at_the_fp32_bar(gpu_device, seed):
    """fp32 rows: the split-operand variants of the chunked kernels against the fp32 token-serial kernel on the same
    rows, outputs, uncertainty and final states within 1e-4 (max-norm)."""
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa, fused_recurrent_palimpsa
    c = _case(seed)
    d, mu0, I0, cu = _inputs(c, seed, gpu_device)
    rows = {n: d[n].float() for n in ("q", "k", "v", "b")}
    kw = dict(scale=c["scale"], initial_mu_state=mu0, initial_I_state=I0, output_final_state=True,
              output_uncertainty=c["var"], cu_seqlens=cu)
    with torch.no_grad():
        out_c, mu_c, I_c = chunk_palimpsa(rows["q"], rows["k"], rows["v"], rows["b"], d["gt"], d["g"], d["Ip"],
                                          chunk_size=64, **kw)
        out_r, mu_r, I_r = fused_recurrent_palimpsa(rows["q"], rows["k"], rows["v"], rows["b"], d["gt"], d["g"],
                                                    d["Ip"], **kw)
    o_c, o_r = (out_c[0], out_r[0]) if c["var"] else (out_c, out_r)
    assert hp.max_abs(o_c, o_r) <= hp.CHUNK_FP32_OUT_TOL * max(1.0, o_r.abs().max().item()), c
    if c["var"]:
        assert hp.max_rel(out_c[1], out_r[1]) <= hp.CHUNK_FP32_OUT_TOL, c
    assert hp.max_rel(mu_c, mu_r) <= hp.CHUNK_FP32_OUT_TOL and hp.max_rel(I_c, I_r) <= hp.CHUNK_FP32_OUT_TOL, c
