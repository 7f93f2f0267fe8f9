"""pal_chunk_fwd_static: the chunked forward on the library's own static scratch (for callers that cannot
allocate device memory).  Called through the C ABI (ctypes) and compared with pal_chunk_fwd on the same inputs:
the same kernels run on the same data, so outputs and final states must agree bit for bit; the existing entry
point itself is held to the oracle at the bf16 bar.  Two calls in a row share the scratch, the second on a
smaller input, so that left-overs of the first call would show.
"""
import ctypes as C

import pytest
import torch

from oracle import palimpsa_oracle as po
from tests import helpers as hp

pytestmark = pytest.mark.gpu


def _call(entry, inp, dev, cu=None, want_var=False, mu0=None, I0=None, with_states=True):
    """One forward through the raw C ABI; returns (rc, o, o_var, final_mu, final_I)."""
    from palimpsa_amd import _lib as L
    from palimpsa_amd.ops.palimpsa import _common as cm
    lib = L.load()
    d = hp.to_device(inp, dev)
    cu_t = None if cu is None else torch.tensor(cu, device=dev, dtype=torch.int32)
    p = cm.prepare_inputs(d["q"], d["k"], d["v"], d["b"], d["gt"], d["g"], d["Ip"],
                          None if mu0 is None else mu0.to(dev), None if I0 is None else I0.to(dev), cu_t, recurrent=False)
    B, T, H, _ = p.q.shape
    flags = L.PAL_FLAG_STORE_FINAL
    table = offsets = None
    if cu is not None:
        meta, total_chunks = cm.chunk_meta(cu_t, T, dev)
        offsets, table = meta[: p.n_seqs + 1], meta[p.n_seqs + 1:]
        flags |= L.PAL_FLAG_VARLEN
    else:
        total_chunks = (T + L.PAL_CHUNK - 1) // L.PAL_CHUNK * B
    if mu0 is not None:
        flags |= L.PAL_FLAG_HAS_INIT
    if want_var:
        flags |= L.PAL_FLAG_HAS_VAR
    o = torch.full((B, T, H, p.dv_p), float("nan"), dtype=p.compute_dtype, device=dev)
    ov = torch.full_like(o, float("nan")) if want_var else None
    fmu = torch.full((p.n_seqs, H, p.dv_p, p.dk_p), float("nan"), dtype=torch.float32, device=dev)
    fI = torch.full_like(fmu, float("nan"))
    cmu = cI = None
    if with_states:
        cmu = torch.empty(total_chunks, H, p.dv_p, p.dk_p, dtype=torch.float32, device=dev)
        cI = torch.empty_like(cmu)
    dims = cm.make_dims(p, p.dk ** -0.5, flags, total_chunks, var_dtype=p.compute_dtype)
    tens = cm.make_fwd_tensors(p, o, ov, fmu, fI, table, offsets, cmu, cI)
    with torch.cuda.device(dev):
        rc = getattr(lib, entry)(dims, tens, cm.current_stream_ptr(dev))
    torch.cuda.synchronize(dev)
    return rc, o, ov, fmu, fI


def test_static_scratch_forward_matches_the_allocating_entry_point(gpu_device):
    dev = gpu_device
    gen = torch.Generator().manual_seed(3)
    # first call: packed documents, both outputs, an initial state; second call: smaller, dense, other head dims
    cu = [0, 70, 71, 400, 530]
    big = hp.rounded(po.make_inputs(1, cu[-1], 3, 64, 96, seed=11), torch.bfloat16)
    big["g"] = torch.tensor([0.5, 2.0, 8.0])
    mu0 = torch.randn(len(cu) - 1, 3, 96, 64, generator=gen) * 0.1
    I0 = 1.0 + torch.rand(len(cu) - 1, 3, 96, 64, generator=gen)
    small = hp.rounded(po.make_inputs(2, 100, 2, 32, 48, seed=12), torch.bfloat16)
    cases = [dict(inp=big, cu=cu, want_var=True, mu0=mu0, I0=I0), dict(inp=small)]
    for kw in cases:
        rc_s, o_s, ov_s, fmu_s, fI_s = _call("pal_chunk_fwd_static", dev=dev, with_states=False, **kw)
        rc_a, o_a, ov_a, fmu_a, fI_a = _call("pal_chunk_fwd", dev=dev, **kw)
        assert rc_s == 0 and rc_a == 0, (rc_s, rc_a)
        assert torch.equal(o_s, o_a) and torch.equal(fmu_s, fmu_a) and torch.equal(fI_s, fI_a)
        if kw.get("want_var"):
            assert torch.equal(ov_s, ov_a)
        o_ref, ov_ref, mu_ref, I_ref = hp.oracle_forward(kw["inp"], mu0=kw.get("mu0"), I0=kw.get("I0"), cu=kw.get("cu"),
                                                        want_var=bool(kw.get("want_var")), dtype=torch.float64)
        assert hp.max_abs(o_s.float(), o_ref) <= hp.BF16_OUT_ABS_TOL
        assert hp.max_rel(fmu_s, mu_ref) <= 5e-3 and hp.max_rel(fI_s, I_ref) <= 5e-3
        if kw.get("want_var"):
            assert hp.max_abs(ov_s.float(), ov_ref) <= hp.BF16_OUT_ABS_TOL


def test_static_scratch_refuses_what_does_not_fit(gpu_device):
    from palimpsa_amd import _lib as L
    dev = gpu_device
    # H = 16, 128 x 128: 2 Mi state entries per 8 tiles -> 40 tiles need 10 Mi entries, the scratch holds 8 Mi
    inp = hp.rounded(po.make_inputs(1, 40 * 64, 16, 128, 128, seed=1), torch.bfloat16)
    rc, o, _, _, _ = _call("pal_chunk_fwd_static", inp, dev, with_states=False)
    assert rc == L.PAL_E_SCRATCH
    assert torch.isnan(o.float()).all()          # nothing ran
    with pytest.raises(ValueError, match="static scratch"):
        L.check(rc, "pal_chunk_fwd_static")
    # caller-provided state buffers are refused: the states of this entry point live in the library
    small = hp.rounded(po.make_inputs(1, 64, 1, 16, 16, seed=1), torch.bfloat16)
    rc, _, _, _, _ = _call("pal_chunk_fwd_static", small, dev, with_states=True)
    assert rc == L.PAL_E_STATE
    # the largest call that fits: 32 tiles at H = 16, 128 x 128
    inp = hp.rounded(po.make_inputs(1, 32 * 64, 16, 128, 128, seed=2), torch.bfloat16)
    rc_s, o_s, _, fmu_s, _ = _call("pal_chunk_fwd_static", inp, dev, with_states=False)
    rc_a, o_a, _, fmu_a, _ = _call("pal_chunk_fwd", inp, dev)
    assert rc_s == 0 and rc_a == 0
    assert torch.equal(o_s, o_a) and torch.equal(fmu_s, fmu_a)


def test_static_scratch_forward_allocates_nothing_and_replays_from_a_graph(gpu_device):
    """The use the entry point exists for: after one call outside capture (which looks up the scratch address and
    raises the kernels' LDS limits), the call is recorded into a HIP graph and replayed on changed inputs; every replay
    is compared with pal_chunk_fwd on the same inputs, with eager work and synchronisations between the replays.
    The free device memory reported by the driver does not move across eager calls of the entry point (the graph and
    the eager torch work of this test have allocations of their own, so the figure is read around the calls alone)."""
    from palimpsa_amd import _lib as L
    from palimpsa_amd.ops.palimpsa import _common as cm
    dev = gpu_device
    lib = L.load()
    B, T, H, dk, dv = 2, 200, 3, 64, 64
    inputs = [hp.to_device(hp.rounded(po.make_inputs(B, T, H, dk, dv, seed=s), torch.bfloat16), dev) for s in (21, 22, 23)]
    static_in = {n: x.clone() for n, x in inputs[0].items()}
    p = cm.prepare_inputs(*[static_in[n] for n in ("q", "k", "v", "b", "gt", "g", "Ip")], None, None, None, recurrent=False)
    for n in ("q", "k", "v", "b", "gt"):    # prepare_inputs hands contiguous inputs through: the graph reads these buffers
        assert getattr(p, n).data_ptr() == static_in[n].data_ptr()
    total_chunks = (T + L.PAL_CHUNK - 1) // L.PAL_CHUNK * B
    o = torch.empty(B, T, H, dv, dtype=torch.bfloat16, device=dev)
    fmu = torch.empty(B, H, dv, dk, dtype=torch.float32, device=dev)
    fI = torch.empty_like(fmu)
    dims = cm.make_dims(p, dk ** -0.5, L.PAL_FLAG_STORE_FINAL, total_chunks, var_dtype=torch.bfloat16)
    tens = cm.make_fwd_tensors(p, o, None, fmu, fI, None, None, None, None)

    def reference(inp):
        rc, o_a, _, fmu_a, fI_a = _call("pal_chunk_fwd", {n: x.cpu() for n, x in inp.items()}, dev)
        assert rc == 0
        return o_a, fmu_a, fI_a

    refs = [reference(inp) for inp in inputs]
    with torch.cuda.device(dev):
        assert lib.pal_chunk_fwd_static(dims, tens, cm.current_stream_ptr(dev)) == 0     # outside capture
        torch.cuda.synchronize(dev)
        free_before = torch.cuda.mem_get_info(dev)[0]
        for _ in range(3):
            assert lib.pal_chunk_fwd_static(dims, tens, cm.current_stream_ptr(dev)) == 0
        torch.cuda.synchronize(dev)
        assert torch.cuda.mem_get_info(dev)[0] == free_before
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            assert lib.pal_chunk_fwd_static(dims, tens, cm.current_stream_ptr(dev)) == 0
        for i in (1, 2, 0, 1):
            for n in ("q", "k", "v", "b", "gt"):
                static_in[n].copy_(inputs[i][n])
            o.fill_(float("nan"))
            fmu.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize(dev)
            o_a, fmu_a, fI_a = refs[i]
            assert torch.equal(o, o_a) and torch.equal(fmu, fmu_a) and torch.equal(fI, fI_a), i
            # eager work between the replays
            _ = (o.float() @ torch.ones(dv, 4, device=dev)).sum().item()
