"""hw_fused_attention_static (the entry point that allocates nothing: split-K partials in a device array that is part
of the library image) against hw_fused_attention on the same inputs, through the C ABI.  Same kernels, same split
plan, so the results must be bit-identical.  Two calls in a row, the second with a smaller input, because every call
on a GPU shares that GPU's array and finds the previous call's contents in it."""
import pytest
import torch

from helpers import TOL, assert_close, oracle_fused

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


def _both(case):
    """(out, lse, rq) of the workspace entry point and of the static-scratch entry point."""
    from inference_lib_amd import _lib
    cd = case.to(_dev())
    W, Hq, S, E = cd.q.shape
    res = []
    for static in (False, True):
        out = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
        lse = torch.full((W, Hq, S), float("nan"), dtype=torch.float32, device=_dev())
        rq = torch.full((case.F, W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
        pr = _lib.Problem(q=cd.q, locations=cd.locations, keys=cd.keys, values=cd.values, scale=cd.scale, out=out,
                          cosines=cd.cos, sines=cd.sin, rq=rq, lse=lse)
        if static:
            pr.run_static()
        else:
            pr.run()
        torch.cuda.synchronize()
        res.append((out, lse, rq))
    return res


def test_static_scratch_matches_workspace_entry(oracle):
    from inference_lib_amd import cases
    big = cases.baseline_case(3)                      # headline shape: 256 workgroups, 2.7 MB of partials
    small = cases.small_case(dtype="bf16", W=2, S=1, Hq=8, Hkv=2, E=128, lens=(100, 37, 65), seed=11)
    part = cases.small_case(dtype="f16", W=3, S=2, Hq=6, Hkv=2, E=64, lens=(70, 33, 1, 64), seed=5)   # prompt + 3 segments
    for c in (big, small, part, big):                 # larger, smaller, other dtype / head dim, larger again
        print(f"case {c.name} lens={c.lens}", flush=True)
        (o0, l0, r0), (o1, l1, r1) = _both(c)
        assert torch.equal(o0, o1), "out differs between the two entry points"
        assert torch.equal(l0, l1), "lse differs between the two entry points"
        assert torch.equal(r0.view(torch.int16), r1.view(torch.int16)), "rotated queries differ"
        o_ref, l_ref, _ = oracle_fused(oracle, c)
        assert_close("out", o1, o_ref, TOL[c.dtype])
        assert_close("lse", l1, l_ref, TOL[c.dtype])


def test_static_scratch_partial_rotary_uses_the_array_for_the_rotated_queries(oracle):
    """Rotary width != head dim: the standalone rotation writes the rotated queries into the scratch as well."""
    from inference_lib_amd import _lib, cases
    c = cases.small_case(dtype="bf16", W=2, S=1, Hq=8, Hkv=2, E=128, lens=(90, 40, 17), seed=3, rot_dim=64)
    cd = c.to(_dev())
    W, Hq, S, E = cd.q.shape
    outs = []
    for static in (False, True):
        out = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
        pr = _lib.Problem(q=cd.q, locations=cd.locations, keys=cd.keys, values=cd.values, scale=cd.scale, out=out,
                          cosines=cd.cos, sines=cd.sin)
        pr.run_static() if static else pr.run()
        torch.cuda.synchronize()
        outs.append(out)
    assert torch.equal(outs[0], outs[1])
    o_ref, _, _ = oracle_fused(oracle, c)
    assert_close("out", outs[1], o_ref, TOL[c.dtype])


def test_static_scratch_takes_the_kernel_with_fewer_partials(oracle):
    """128 rows per kv head: the 128-row workgroups would need 17 MB of partials, more than the array holds.  Left the
    choice (row_blocks = 0), the entry point plans the 32-row kernel instead (4.3 MB) and gives bit for bit what the
    workspace entry point gives with row_blocks = 2."""
    from inference_lib_amd import _lib, cases
    c = cases.baseline_case(5)
    cd = c.to(_dev())
    W, Hq, S, E = cd.q.shape
    res = []
    for static in (False, True):
        out = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
        lse = torch.full((W, Hq, S), float("nan"), dtype=torch.float32, device=_dev())
        pr = _lib.Problem(q=cd.q, locations=cd.locations, keys=cd.keys, values=cd.values, scale=cd.scale, out=out,
                          cosines=cd.cos, sines=cd.sin, lse=lse, row_blocks=0 if static else 2)
        if static:
            assert pr.workspace_bytes() > _lib.HW_STATIC_SCRATCH_BYTES      # what the automatic plan would need
            pr.run_static()
        else:
            pr.run()
        torch.cuda.synchronize()
        res.append((out, lse))
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1])
    o_ref, l_ref, _ = oracle_fused(oracle, c)
    assert_close("out", res[1][0], o_ref, TOL[c.dtype])
    assert_close("lse", res[1][1], l_ref, TOL[c.dtype])
    # asked for by name, the 128-row workgroups are refused: the caller's choice is not overridden
    pr = _lib.Problem(q=cd.q, locations=cd.locations, keys=cd.keys, values=cd.values, scale=cd.scale, out=res[1][0],
                      cosines=cd.cos, sines=cd.sin, row_blocks=8)
    with pytest.raises(_lib.HogwildError) as ei:
        pr.run_static()
    assert ei.value.status == -9


def test_static_scratch_refuses_what_does_not_fit():
    """A problem whose partials exceed the array is refused on the host, before anything is queued."""
    from inference_lib_amd import _lib
    dev = _dev()
    W, Hq, Hkv, S, E = 64, 64, 8, 4, 128               # 2048 rows per kv head
    L = 4096
    q = torch.zeros((W, Hq, S, E), dtype=torch.bfloat16, device=dev)
    k = torch.zeros((Hkv, L, E), dtype=torch.bfloat16, device=dev)
    loc = torch.full((1, W, S), L - 1, dtype=torch.int32, device=dev)
    cs = torch.zeros((1, W, S, E), dtype=torch.float32, device=dev)
    out = torch.empty_like(q)
    pr = _lib.Problem(q=q, locations=loc, keys=[k], values=[k], scale=0.1, out=out, cosines=cs, sines=cs)
    assert pr.workspace_bytes() > _lib.HW_STATIC_SCRATCH_BYTES
    with pytest.raises(_lib.HogwildError) as ei:
        pr.run_static()
    assert ei.value.status == -9
    assert "HW_STATIC_SCRATCH_BYTES" in str(ei.value)


def test_static_scratch_entry_allocates_nothing_and_can_be_captured(oracle):
    """What the entry point exists for: on a warmed library it takes no device memory (the driver's free-byte count does
    not move over a series of calls), and it can run under stream capture (an allocation there would fail the capture):
    every replay of the captured call gives the eager call's bits."""
    from inference_lib_amd import _lib, cases
    c = cases.small_case(dtype="bf16", W=4, S=1, Hq=20, Hkv=4, E=128, lens=(700, 300, 257, 64, 129), seed=7)
    cd = c.to(_dev())
    W, Hq, S, E = cd.q.shape
    out = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
    lse = torch.full((W, Hq, S), float("nan"), dtype=torch.float32, device=_dev())
    pr = _lib.Problem(q=cd.q, locations=cd.locations, keys=cd.keys, values=cd.values, scale=cd.scale, out=out,
                      cosines=cd.cos, sines=cd.sin, lse=lse)
    pr.run_static()                                      # first call on this device: takes the array's address
    torch.cuda.synchronize()
    eager_o, eager_l = out.clone(), lse.clone()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(20):
        pr.run_static()
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, f"device memory moved by {free0 - free1} bytes over 20 calls"
    assert torch.equal(out, eager_o) and torch.equal(lse, eager_l)

    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            pr.run_static()
        for rep in range(3):
            out.fill_(float("nan"))
            lse.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager_o) and torch.equal(lse, eager_l), f"replay {rep} differs from the eager call"
    o_ref, l_ref, _ = oracle_fused(oracle, c)
    assert_close("out", out, o_ref, TOL[c.dtype])
    assert_close("lse", lse, l_ref, TOL[c.dtype])
