"""GPU parity of the token-serial (fused-recurrent / decode) HIP path against the CPU oracle.

Every call goes through palimpsa_amd.ops.palimpsa -> ctypes -> the C ABI of
libpalimpsa_hip.so.  Tolerances: fp32 max|x-ref|/max|ref| <= 1e-4; bf16 rows
max|x-ref| <= 2e-2 on outputs (oracle fed the same bf16-rounded rows).
"""
import pytest
import torch

from oracle import palimpsa_oracle as po
from tests import helpers as hp

pytestmark = pytest.mark.gpu


def _ops():
    from palimpsa_amd.ops.palimpsa import fused_recurrent_palimpsa
    return fused_recurrent_palimpsa


def test_c0_fp32_forward_and_final_state(gpu_device):
    """Benchmark configuration 0: B=2, T=256, H=4, dk=dv=32, fp32, seed 0, zero mean state, I0 = Ip."""
    fr = _ops()
    inp = po.make_inputs(2, 256, 4, 32, 32, seed=0)
    o_ref, _, mu_ref, I_ref = hp.oracle_forward(inp)
    d = hp.to_device(inp, gpu_device)
    o, mu, I = fr(d["q"], d["k"], d["v"], d["b"], d["gt"], d["g"], d["Ip"], output_final_state=True)
    assert o.dtype == torch.float32 and o.shape == (2, 256, 4, 32)
    assert mu.shape == (2, 4, 32, 32) and I.dtype == torch.float32
    assert hp.max_rel(o, o_ref) <= hp.FP32_REL_TOL
    assert hp.max_rel(mu, mu_ref) <= hp.FP32_REL_TOL
    assert hp.max_rel(I, I_ref) <= hp.FP32_REL_TOL


@pytest.mark.parametrize("dk,dv", [(16, 16), (48, 96), (64, 64), (96, 96), (128, 128), (192, 48), (256, 32)])
def test_fp32_all_compiled_head_dims_with_state_and_var(gpu_device, dk, dv):
    fr = _ops()
    B, T, H = 2, 37, 3
    inp = po.make_inputs(B, T, H, dk, dv, seed=dk + dv, g_value=2.0)
    inp["g"] = torch.linspace(1.0, 16.0, H)
    inp["Ip"] = torch.tensor([0.5, 1.0, 2.5])
    gen = torch.Generator().manual_seed(5)
    mu0 = torch.randn(B, H, dv, dk, generator=gen) * 0.1
    I0 = inp["Ip"].view(1, H, 1, 1) + torch.nn.functional.softplus(torch.randn(B, H, dv, dk, generator=gen))
    o_ref, ov_ref, mu_ref, I_ref = hp.oracle_forward(inp, scale=0.7, mu0=mu0, I0=I0, want_var=True)
    d = hp.to_device(inp, gpu_device)
    (o, ov), mu, I = fr(d["q"], d["k"], d["v"], d["b"], d["gt"], d["g"], d["Ip"], scale=0.7,
                        initial_mu_state=mu0.to(gpu_device), initial_I_state=I0.to(gpu_device),
                        output_final_state=True, output_uncertainty=True)
    assert hp.max_rel(o, o_ref) <= hp.FP32_REL_TOL
    assert hp.max_rel(ov, ov_ref) <= hp.FP32_REL_TOL
    assert hp.max_rel(mu, mu_ref) <= hp.FP32_REL_TOL
    assert hp.max_rel(I, I_ref) <= hp.FP32_REL_TOL


def test_reference_check_script_shape_odd_dims(gpu_device):
    """Topology of the reference's own check (check_palimpsa.py:43-59): dv=65, dk=31, L=511,
    unnormalised q,k, g = |N|*10+1, Ip = |N|+0.1, scale=1; fewer batch rows to keep the CPU side short."""
    fr = _ops()
    gen = torch.Generator().manual_seed(42)
    B, T, H, D, N = 2, 511, 4, 65, 31
    v = torch.randn(B, T, H, D, generator=gen)
    q = torch.randn(B, T, H, N, generator=gen)
    k = torch.randn(B, T, H, N, generator=gen)
    b = torch.sigmoid(torch.randn(B, T, H, D, generator=gen))
    gt = torch.sigmoid(torch.randn(B, T, H, generator=gen))
    g = torch.randn(H, generator=gen).abs() * 10 + 1
    Ip = torch.randn(H, generator=gen).abs() + 0.1
    inp = dict(q=q, k=k, v=v, b=b, gt=gt, g=g, Ip=Ip)
    o_ref, ov_ref, mu_ref, I_ref = hp.oracle_forward(inp, scale=1.0, want_var=True)
    d = hp.to_device(inp, gpu_device)
    (o, ov), mu, I = fr(d["q"], d["k"], d["v"], d["b"], d["gt"], d["g"], d["Ip"], scale=1,
                        output_final_state=True, output_uncertainty=True)
    assert o.shape == (B, T, H, D) and mu.shape == (B, H, D, N)
    assert hp.max_rel(o, o_ref) <= hp.FP32_REL_TOL
    assert hp.max_rel(ov, ov_ref) <= hp.FP32_REL_TOL
    assert hp.max_rel(mu, mu_ref) <= hp.FP32_REL_TOL
    assert hp.max_rel(I, I_ref) <= hp.FP32_REL_TOL


def test_varlen_with_states(gpu_device):
    fr = _ops()
    H, dk, dv = 2, 32, 48
    cu = [0, 1, 18, 19, 83, 200]
    T = cu[-1]
    N = len(cu) - 1
    inp = po.make_inputs(1, T, H, dk, dv, seed=3)
    gen = torch.Generator().manual_seed(6)
    mu0 = torch.randn(N, H, dv, dk, generator=gen) * 0.1
    I0 = 1.0 + torch.rand(N, H, dv, dk, generator=gen)
    o_ref, _, mu_ref, I_ref = hp.oracle_forward(inp, mu0=mu0, I0=I0, cu=cu)
    d = hp.to_device(inp, gpu_device)
    cu_t = torch.tensor(cu, dtype=torch.int64, device=gpu_device)
    o, mu, I = fr(d["q"], d["k"], d["v"], d["b"], d["gt"], d["g"], d["Ip"],
                  initial_mu_state=mu0.to(gpu_device), initial_I_state=I0.to(gpu_device),
                  output_final_state=True, cu_seqlens=cu_t)
    assert hp.max_rel(o, o_ref) <= hp.FP32_REL_TOL
    assert hp.max_rel(mu, mu_ref) <= hp.FP32_REL_TOL
    assert hp.max_rel(I, I_ref) <= hp.FP32_REL_TOL


def test_bf16_rows_decode_steps(gpu_device):
    """Config-3 style decode on a small batch: bf16 rows, fp32 states fed back for 16 steps."""
    fr = _ops()
    B, H, d, steps = 3, 2, 128, 16
    inp = hp.rounded(po.make_inputs(B, steps, H, d, d, seed=0), torch.bfloat16)
    gen = torch.Generator().manual_seed(1)
    mu0 = torch.randn(B, H, d, d, generator=gen) * 0.1
    I0 = torch.nn.functional.softplus(torch.randn(B, H, d, d, generator=gen))
    o_ref, _, mu_ref, I_ref = hp.oracle_forward(inp, mu0=mu0, I0=I0)
    dd = hp.to_device(inp, gpu_device)
    mu, I = mu0.to(gpu_device), I0.to(gpu_device)
    outs = []
    for t in range(steps):
        sl = slice(t, t + 1)
        o, mu, I = fr(dd["q"][:, sl], dd["k"][:, sl], dd["v"][:, sl], dd["b"][:, sl], dd["gt"][:, sl],
                      dd["g"], dd["Ip"], initial_mu_state=mu, initial_I_state=I, output_final_state=True)
        assert o.dtype == torch.bfloat16
        outs.append(o)
    o = torch.cat(outs, dim=1)
    assert hp.max_abs(o, o_ref) <= hp.BF16_OUT_ABS_TOL
    # states are fp32 end to end: same bar as the fp32 kernels
    assert hp.max_rel(mu, mu_ref) <= hp.FP32_REL_TOL
    assert hp.max_rel(I, I_ref) <= hp.FP32_REL_TOL


def test_split_resume_property_full_width(gpu_device):
    """Size-independent property at a decode-sized head (H=16, d=128): [0,T) == [0,T1) + [T1,T)."""
    fr = _ops()
    B, T, H, d = 4, 96, 16, 128
    inp = hp.to_device(hp.rounded(po.make_inputs(B, T, H, d, d, seed=9), torch.bfloat16), gpu_device)
    a = (inp["g"], inp["Ip"])
    o, mu, I = fr(inp["q"], inp["k"], inp["v"], inp["b"], inp["gt"], *a, output_final_state=True)
    T1 = 41
    s1, s2 = slice(0, T1), slice(T1, T)
    o1, mu1, I1 = fr(inp["q"][:, s1], inp["k"][:, s1], inp["v"][:, s1], inp["b"][:, s1], inp["gt"][:, s1], *a,
                     output_final_state=True)
    o2, mu2, I2 = fr(inp["q"][:, s2], inp["k"][:, s2], inp["v"][:, s2], inp["b"][:, s2], inp["gt"][:, s2], *a,
                     initial_mu_state=mu1, initial_I_state=I1, output_final_state=True)
    assert hp.max_abs(torch.cat([o1, o2], 1).float(), o.float()) <= 1e-2
    assert hp.max_rel(mu2, mu) <= 1e-5
    assert hp.max_rel(I2, I) <= 1e-5


def test_error_paths_match_reference(gpu_device):
    fr = _ops()
    inp = hp.to_device(po.make_inputs(2, 8, 2, 16, 16, seed=0), gpu_device)
    cu = torch.tensor([0, 8], device=gpu_device)
    with pytest.raises(ValueError):
        fr(inp["q"], inp["k"], inp["v"], inp["b"], inp["gt"], inp["g"], inp["Ip"], cu_seqlens=cu)


# ------------------------------------------------------------------ backward (fp32 end to end)
def _rec_grads(inp, dev, do, dovar=None, mu0=None, I0=None, cu=None, scale=None):
    fr = _ops()
    names = ["q", "k", "v", "b", "gt", "g", "Ip"]
    leaves = {n: inp[n].to(dev).clone().requires_grad_(True) for n in names}
    kw = {}
    if mu0 is not None:
        leaves["mu0"] = mu0.to(dev).clone().requires_grad_(True)
        leaves["I0"] = I0.to(dev).clone().requires_grad_(True)
        kw.update(initial_mu_state=leaves["mu0"], initial_I_state=leaves["I0"])
    if cu is not None:
        kw["cu_seqlens"] = torch.tensor(cu, device=dev)
    out = fr(*[leaves[n] for n in names], scale=scale, output_uncertainty=dovar is not None, **kw)
    if dovar is not None:
        loss = (out[0].float() * do.to(dev)).sum() + (out[1].float() * dovar.to(dev)).sum()
    else:
        loss = (out.float() * do.to(dev)).sum()
    loss.backward()
    return {n: x.grad for n, x in leaves.items()}


# fp32 gradients against float64 autograd of the oracle: same bar as the fp32 forward
GRAD_TOL = 1e-4


@pytest.mark.parametrize("dk,dv,T", [(16, 16, 1), (32, 32, 37), (64, 64, 70), (128, 128, 20), (192, 48, 33), (256, 32, 19),
                                     (31, 65, 45)])
def test_fp32_backward_matches_oracle(gpu_device, dk, dv, T):
    B, H = 2, 2
    inp = po.make_inputs(B, T, H, dk, dv, seed=dk + dv + T)
    inp["g"] = torch.tensor([1.0, 6.0])
    inp["Ip"] = torch.tensor([0.6, 1.7])
    gen = torch.Generator().manual_seed(3)
    mu0 = torch.randn(B, H, dv, dk, generator=gen) * 0.1
    I0 = inp["Ip"].view(1, H, 1, 1) + torch.rand(B, H, dv, dk, generator=gen)
    do = torch.randn(B, T, H, dv, generator=gen)
    dovar = torch.randn(B, T, H, dv, generator=gen) * 0.3
    ref = hp.oracle_grads(inp, do, dovar, scale=0.6, mu0=mu0, I0=I0)
    got = _rec_grads(inp, gpu_device, do, dovar, mu0=mu0, I0=I0, scale=0.6)
    for n in ["q", "k", "v", "b", "gt", "g", "Ip", "mu0", "I0"]:
        assert hp.max_rel(got[n], ref[n]) <= GRAD_TOL, (n, hp.max_rel(got[n], ref[n]))


def test_fp32_backward_varlen_and_no_state(gpu_device):
    H, d = 3, 32
    cu = [0, 1, 18, 19, 83, 130]
    T = cu[-1]
    inp = po.make_inputs(1, T, H, d, d, seed=13)
    do = torch.randn(1, T, H, d, generator=torch.Generator().manual_seed(14))
    ref = hp.oracle_grads(inp, do, cu=cu)
    got = _rec_grads(inp, gpu_device, do, cu=cu)
    for n in ["q", "k", "v", "b", "gt", "g", "Ip"]:
        assert hp.max_rel(got[n], ref[n]) <= GRAD_TOL, (n, hp.max_rel(got[n], ref[n]))


def test_bf16_rows_backward(gpu_device):
    B, T, H, d = 2, 50, 2, 64
    inp = hp.rounded(po.make_inputs(B, T, H, d, d, seed=17), torch.bfloat16)
    do = torch.randn(B, T, H, d, generator=torch.Generator().manual_seed(18))
    ref = hp.oracle_grads(inp, do)
    got = _rec_grads(inp, gpu_device, do)
    assert got["q"].dtype == torch.bfloat16
    # arithmetic is fp32, but o is a bf16 tensor, so autograd hands the kernel dO rounded to bf16
    # (2^-9 relative) and the row gradients are stored in bf16: every gradient carries that rounding
    for n in ["q", "k", "v", "b", "gt"]:
        assert hp.max_rel(got[n], ref[n]) <= 5e-3, n
    # per-head reductions over all tokens of those rounded terms: the bf16 gradient bar
    for n in ["g", "Ip"]:
        assert hp.max_rel(got[n], ref[n]) <= hp.BF16_GRAD_NORM_TOL, n


@pytest.mark.parametrize("rows", ["fp32", "bf16"])
def test_long_sequences_take_the_chunked_backward(gpu_device, rows):
    """Sequences of 64 tokens or more on average: the backward of the token-serial entry point runs the chunked
    backward kernels on tile-start states from a states-only forward pass.  Dense and packed, initial state and
    uncertainty gradients included: against float64 autograd through the oracle at the bar of the row dtype, and
    against the token-serial backward kernel (the route switched off) on the same inputs."""
    from palimpsa_amd import _lib as L
    H, dk, dv = 2, 64, 32
    cu = [0, 200, 201, 520, 700]
    T, N = cu[-1], len(cu) - 1
    inp = po.make_inputs(1, T, H, dk, dv, seed=71)
    if rows == "bf16":
        inp = hp.rounded(inp, torch.bfloat16)
    inp["g"] = torch.tensor([0.7, 5.0])
    gen = torch.Generator().manual_seed(72)
    mu0 = torch.randn(N, H, dv, dk, generator=gen) * 0.1
    I0 = 1.0 + torch.rand(N, H, dv, dk, generator=gen)
    do = torch.randn(1, T, H, dv, generator=gen)
    dovar = torch.randn(1, T, H, dv, generator=gen) * 0.3
    ref = hp.oracle_grads(inp, do, dovar, mu0=mu0, I0=I0, cu=cu)
    assert L.recurrent_bwd_chunk_min() is not None and T >= L.recurrent_bwd_chunk_min() * N
    L.profile_enable(True)
    got = _rec_grads(inp, gpu_device, do, dovar, mu0=mu0, I0=I0, cu=cu)
    torch.cuda.synchronize()
    ran = L.profile_read()
    L.profile_enable(False)
    assert "chunk_bwd_local_kernel" in ran and "recurrent_bwd_kernel" not in ran, sorted(ran)
    keep = L.recurrent_bwd_chunk_min()
    try:
        L.set_recurrent_bwd_chunk_min(None)
        serial = _rec_grads(inp, gpu_device, do, dovar, mu0=mu0, I0=I0, cu=cu)
    finally:
        L.set_recurrent_bwd_chunk_min(keep)
    names = ["q", "k", "v", "b", "gt", "g", "Ip", "mu0", "I0"]
    if rows == "fp32":
        for n in names:
            assert hp.max_rel(got[n], ref[n]) <= GRAD_TOL, (n, hp.max_rel(got[n], ref[n]))
            assert hp.max_rel(got[n], serial[n]) <= 2 * GRAD_TOL, (n, hp.max_rel(got[n], serial[n]))
    else:
        mass = ((inp["gt"].double() * ref["gt"].double()).abs().sum(dim=(0, 1)) / inp["g"].double()).max().item()
        for n in names:
            if n == "g":    # random dO: |dg| is far below the l1 mass of its terms (tests/test_gpu_chunk_bwd.py)
                err = (got[n].double().cpu() - ref[n].double()).abs().max().item() / mass
            else:
                err = hp.max_rel(got[n], ref[n])
            assert err <= hp.BF16_GRAD_NORM_TOL, (n, err)
    # a dense batch of short sequences stays with the token-serial kernel
    short = po.make_inputs(2, 50, H, dk, dv, seed=73)
    L.profile_enable(True)
    _rec_grads(short, gpu_device, torch.randn(2, 50, H, dv, generator=gen))
    torch.cuda.synchronize()
    ran = L.profile_read()
    L.profile_enable(False)
    assert "recurrent_bwd_kernel" in ran and "chunk_bwd_local_kernel" not in ran, sorted(ran)


def test_bound_decode_step_matches_entry_point_and_replays_in_a_graph(gpu_device):
    """DecodeStep binds tensors once and updates the state in place: same kernel as
    fused_recurrent_palimpsa with T = 1, so results agree exactly; recorded into a HIP graph (the step
    allocates nothing and records no memset) every replay agrees with the eager result too."""
    from palimpsa_amd.ops.palimpsa import DecodeStep, fused_recurrent_palimpsa
    B, H, dk, dv, steps = 5, 3, 64, 32, 6
    dev = gpu_device
    inp = hp.rounded(po.make_inputs(B, steps, H, dk, dv, seed=61), torch.bfloat16)
    d = hp.to_device(inp, dev)
    gen = torch.Generator().manual_seed(62)
    mu0 = (torch.randn(B, H, dv, dk, generator=gen) * 0.1).to(dev)
    I0 = (1.0 + torch.rand(B, H, dv, dk, generator=gen)).to(dev)
    # eager entry point, state fed back
    mu, I = mu0.clone(), I0.clone()
    outs = []
    for t in range(steps):
        r = {n: d[n][:, t:t + 1].contiguous() for n in ("q", "k", "v", "b", "gt")}
        (o, ov), mu, I = fused_recurrent_palimpsa(r["q"], r["k"], r["v"], r["b"], r["gt"], d["g"], d["Ip"],
                                                  initial_mu_state=mu, initial_I_state=I, output_final_state=True,
                                                  output_uncertainty=True)
        outs.append((o, ov))
    # bound step, rows copied into fixed buffers
    dec = DecodeStep(B, H, dk, dv, dev, torch.bfloat16, output_uncertainty=True)
    buf = {n: torch.empty_like(d[n][:, :1].contiguous()) for n in ("q", "k", "v", "b", "gt")}
    mu_b, I_b = mu0.clone(), I0.clone()
    dec.bind(buf["q"], buf["k"], buf["v"], buf["b"], buf["gt"], d["g"], d["Ip"], mu_b, I_b)
    for t in range(steps):
        for n in buf:
            buf[n].copy_(d[n][:, t:t + 1])
        o = dec.step()
        assert torch.equal(o, outs[t][0]) and torch.equal(dec.o_var, outs[t][1])
    assert torch.equal(mu_b, mu) and torch.equal(I_b, I)
    # the same steps from a captured graph, replayed with eager work in between
    mu_b.copy_(mu0); I_b.copy_(I0)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        buf_warm = {n: buf[n].clone() for n in buf}
        dec.step()                       # warm-up on the capture stream
        mu_b.copy_(mu0); I_b.copy_(I0)
        with torch.cuda.graph(graph, stream=side):
            dec.step()
    torch.cuda.current_stream().wait_stream(side)
    for t in range(steps):
        for n in buf:
            buf[n].copy_(d[n][:, t:t + 1])
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(dec.o, outs[t][0]), t
    assert torch.equal(mu_b, mu) and torch.equal(I_b, I)
    with pytest.raises(ValueError):
        dec.bind(buf["q"].float(), buf["k"], buf["v"], buf["b"], buf["gt"], d["g"], d["Ip"], mu_b, I_b)
    with pytest.raises(ValueError):
        DecodeStep(B, H, 40, dv, dev)


@pytest.mark.parametrize("k", [3, 5, 7, 8, 13])
def test_bound_decode_step_with_several_tokens_per_step(gpu_device, k):
    """A bound step over blocks of k tokens equals the same tokens one at a time (state in place); k <= 4 takes the
    decode form of the kernel, longer blocks the form that keeps the rows of several tokens in flight (its group and
    tail loops at every remainder)."""
    from palimpsa_amd.ops.palimpsa import DecodeStep
    B, H, dk, dv, blocks = 4, 2, 32, 48, 3
    dev = gpu_device
    inp = hp.rounded(po.make_inputs(B, blocks * k, H, dk, dv, seed=71), torch.bfloat16)
    d = hp.to_device(inp, dev)
    gen = torch.Generator().manual_seed(72)
    mu0 = (torch.randn(B, H, dv, dk, generator=gen) * 0.1).to(dev)
    I0 = (1.0 + torch.rand(B, H, dv, dk, generator=gen)).to(dev)

    def run(tokens):
        dec = DecodeStep(B, H, dk, dv, dev, torch.bfloat16, tokens=tokens)
        buf = {n: torch.empty_like(d[n][:, :tokens].contiguous()) for n in ("q", "k", "v", "b", "gt")}
        mu, I = mu0.clone(), I0.clone()
        dec.bind(buf["q"], buf["k"], buf["v"], buf["b"], buf["gt"], d["g"], d["Ip"], mu, I)
        outs = []
        for t in range(0, blocks * k, tokens):
            for n in buf:
                buf[n].copy_(d[n][:, t:t + tokens])
            outs.append(dec.step().clone())
        return torch.cat(outs, dim=1), mu, I

    o1, mu1, I1 = run(1)
    o3, mu3, I3 = run(k)
    assert o3.shape == (B, blocks * k, H, dv)
    # inside a block the state stays in registers as (M, J); between single steps it crosses as (mu, I)
    assert hp.max_abs(o3.float(), o1.float()) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu3, mu1) <= 1e-5 and hp.max_rel(I3, I1) <= 1e-5
    o_ref, _, mu_ref, I_ref = hp.oracle_forward(inp, mu0=mu0.cpu(), I0=I0.cpu())
    assert hp.max_abs(o3.float(), o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu3, mu_ref) <= hp.FP32_REL_TOL and hp.max_rel(I3, I_ref) <= hp.FP32_REL_TOL
    with pytest.raises(ValueError):
        DecodeStep(B, H, dk, dv, dev, tokens=0)


def test_decode_with_the_mean_state_kept_in_bf16(gpu_device):
    """DecodeStep(mu_dtype=bfloat16): mu is rounded to bf16 once per step, I stays fp32.  Over 64 steps with a slow
    (f ~ 0.98), a medium and a fast head the outputs stay within the bf16 output bar of the float64 oracle, and the
    state within 2 % (max-norm) of the oracle's; the first step equals the fp32-state step exactly (same inputs
    after mu_to_cache)."""
    from palimpsa_amd.ops.palimpsa import DecodeStep, mu_from_cache, mu_to_cache
    B, H, dk, dv, steps = 3, 3, 64, 32, 64
    dev = gpu_device
    inp = hp.rounded(po.make_inputs(B, steps, H, dk, dv, seed=71), torch.bfloat16)
    inp["g"] = torch.tensor([0.04, 1.0, 8.0])
    gen = torch.Generator().manual_seed(72)
    mu0 = (torch.randn(B, H, dv, dk, generator=gen) * 0.1).to(torch.bfloat16).float()   # exactly representable
    I0 = 1.0 + torch.rand(B, H, dv, dk, generator=gen)
    o_ref, _, mu_ref, I_ref = hp.oracle_forward(inp, mu0=mu0, I0=I0, dtype=torch.float64)
    d = hp.to_device(inp, dev)
    outs = {}
    for name, mu_dtype in (("fp32", torch.float32), ("bf16", torch.bfloat16)):
        dec = DecodeStep(B, H, dk, dv, dev, torch.bfloat16, mu_dtype=mu_dtype)
        buf = {n: torch.empty_like(d[n][:, :1].contiguous()) for n in ("q", "k", "v", "b", "gt")}
        mu = mu0.to(dev) if mu_dtype == torch.float32 else mu_to_cache(mu0.to(dev))
        I = I0.to(dev).clone()
        dec.bind(buf["q"], buf["k"], buf["v"], buf["b"], buf["gt"], d["g"], d["Ip"], mu, I)
        o_all = []
        for t in range(steps):
            for n in buf:
                buf[n].copy_(d[n][:, t:t + 1])
            o_all.append(dec.step().clone())
        outs[name] = (torch.cat(o_all, dim=1), mu if mu_dtype == torch.float32 else mu_from_cache(mu), I)
        with pytest.raises(ValueError):
            dec.bind(buf["q"], buf["k"], buf["v"], buf["b"], buf["gt"], d["g"], d["Ip"],
                     mu.float() if mu_dtype == torch.bfloat16 else mu.bfloat16(), I)
    assert torch.equal(outs["bf16"][0][:, 0], outs["fp32"][0][:, 0])
    for name in outs:
        assert hp.max_abs(outs[name][0], o_ref) <= hp.BF16_OUT_ABS_TOL, name
    assert hp.max_rel(outs["fp32"][1], mu_ref) <= 1e-4 and hp.max_rel(outs["fp32"][2], I_ref) <= 1e-4
    assert hp.max_rel(outs["bf16"][1], mu_ref) <= 2e-2
    assert hp.max_rel(outs["bf16"][2], I_ref) <= 1e-4          # I never sees the rounding of mu
