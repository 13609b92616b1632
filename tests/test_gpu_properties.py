"""Properties of the HIP path that hold at any size, checked on the GPU through the C ABI: independence of the
split plan, of fragment order and of fragment splitting, determinism, empty rows / empty fragments, the fragment
limit, streams and HIP-graph replay, and the two stages run separately."""
import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, np64, oracle_fused, run_fused

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def _problem(cd, out, *, rq=None, lse=None, **kw):
    from inference_lib_amd import _lib
    return _lib.Problem(q=cd.q, locations=cd.locations, keys=cd.keys, values=cd.values, scale=cd.scale, out=out,
                        cosines=cd.cos, sines=cd.sin, rq=rq, lse=lse, **kw)


def test_split_plan_does_not_change_the_result(oracle):
    """Any number of workgroups per head and either row-block setting gives the same answer up to fp32
    accumulation order, at the full size of the headline workload."""
    from inference_lib_amd import cases
    c = cases.baseline_case(3)
    cd = c.to(_dev())
    o_ref, l_ref, _ = oracle_fused(oracle, c)
    W, Hq, S, E = cd.q.shape
    base = None
    for splits, rb in [(0, 0), (1, 0), (3, 0), (17, 0), (64, 0), (256, 0), (0, 1), (5, 1)]:
        print(f"splits={splits} row_blocks={rb}", flush=True)
        out = torch.empty((W, Hq, S, E), dtype=cd.q.dtype, device=_dev())
        lse = torch.empty((W, Hq, S), dtype=torch.float32, device=_dev())
        _problem(cd, out, lse=lse, splits=splits, row_blocks=rb).run()
        torch.cuda.synchronize()
        assert_close("out", out, o_ref, TOL[c.dtype])
        assert_close("lse", lse, l_ref, TOL[c.dtype])
        if base is None:
            base = (out.clone(), lse.clone())
        else:
            assert (out.float() - base[0].float()).abs().max().item() <= 2 ** -7      # one bf16 ulp at |x| < 1 is 2^-8
            assert (lse - base[1]).abs().max().item() <= 1e-4


def test_runs_are_bit_identical():
    from inference_lib_amd import cases
    cd = cases.baseline_case(2).to(_dev())
    a = run_fused(cd)
    b = run_fused(cd)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


def test_fragment_order_and_fragment_split_invariance(oracle):
    from inference_lib_amd import cases
    c = cases.small_case(dtype="f32", W=2, S=2, Hq=4, Hkv=2, E=64, lens=(150, 70, 90), seed=13)
    cd = c.to(_dev())
    out, lse, _ = run_fused(cd)
    # reorder the fragments
    perm = [2, 0, 1]
    c2 = cases.small_case(dtype="f32", W=2, S=2, Hq=4, Hkv=2, E=64, lens=(150, 70, 90), seed=13)
    c2.keys = [c.keys[i] for i in perm]
    c2.values = [c.values[i] for i in perm]
    c2.lens = [c.lens[i] for i in perm]
    c2.locations = c.locations[perm].contiguous()
    c2.cos = c.cos[perm].contiguous()
    c2.sin = c.sin[perm].contiguous()
    out2, lse2, _ = run_fused(c2.to(_dev()))
    assert (out - out2).abs().max().item() < 1e-5 and (lse - lse2).abs().max().item() < 1e-5
    # cut fragment 0 at token 37 with pre-rotated queries (only the mask bound moves: loc2 = loc - 37)
    from inference_lib_amd import _lib
    rq = torch.empty((c.F, 2, 4, 2, 64), dtype=torch.float32, device=_dev())
    _lib.rope(cd.q, cd.cos, cd.sin, rq)
    L1 = 37
    keys = [cd.keys[0][:, :L1].contiguous(), cd.keys[0][:, L1:].contiguous()] + cd.keys[1:]
    vals = [cd.values[0][:, :L1].contiguous(), cd.values[0][:, L1:].contiguous()] + cd.values[1:]
    loc = torch.cat([cd.locations[:1], cd.locations[:1] - L1, cd.locations[1:]]).contiguous()
    rq2 = torch.cat([rq[:1], rq[:1], rq[1:]]).contiguous()
    out3 = torch.empty_like(out)
    lse3 = torch.empty_like(lse)
    _lib.Problem(q=rq2, locations=loc, keys=keys, values=vals, scale=c.scale, out=out3, lse=lse3, prerotated=True).run()
    torch.cuda.synchronize()
    assert (out - out3).abs().max().item() < 1e-5 and (lse - lse3).abs().max().item() < 1e-5


def test_rows_that_see_nothing_and_empty_fragments(oracle):
    """A worker whose locations are all -1 gets zeros and lse = -inf (the kernel's convention,
    kernel_v21.cuh:238-245,627-629); zero-length fragments are legal and their rotated queries are still written."""
    from inference_lib_amd import cases
    c = cases.small_case(dtype="bf16", W=3, S=1, Hq=6, Hkv=2, E=128, lens=(70, 0, 33, 40), seed=17)
    c.locations[:, 2, :] = -1                      # worker 2 sees nothing at all
    cd = c.to(_dev())
    out, lse, rq = run_fused(cd)
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    assert_close("out", out, o_ref, TOL["bf16"])
    assert_close("lse", lse, l_ref, TOL["bf16"])
    assert torch.all(out[2] == 0) and torch.all(torch.isneginf(lse[2]))
    assert_close("rq incl. the empty fragment", rq, rq_ref, 3.2e-2)


def _many_fragments(dtype, F, W, S, Hq, Hkv, E, seed, rot_dim=None):
    """F short fragments (some empty, some longer than a tile), every worker seeing all of them in its own order."""
    from inference_lib_amd import cases
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(0, 71, (F,), generator=g).tolist()
    lens[F // 3] = 150
    lens[-1] = 33
    orders = [list(torch.randperm(F, generator=g).tolist()) for _ in range(W)]
    return cases.build_case(f"many{F}_{dtype}", dtype, W, S, Hq, Hkv, E, 1e4, lens, orders, g, rot_dim=rot_dim)


def test_fragment_limit(oracle):
    """64 fragments fill one launch; the call takes up to 512 (the reference's limit, src/binding.cu:79-82)."""
    from inference_lib_amd import _lib, cases
    lens = [40] + [3 + (i % 5) for i in range(63)]
    W = 63
    c = cases.build_case("f32max", "bf16", W, 1, 2 * W // W * 2, 2, 64, 1e4, lens, [[0, 1 + w] for w in range(W)],
                         torch.Generator().manual_seed(3))
    assert c.F == 64
    out, lse, _ = run_fused(c.to(_dev()))
    o_ref, l_ref, _ = oracle_fused(oracle, c)
    assert_close("out", out, o_ref, TOL["bf16"])
    assert_close("lse", lse, l_ref, TOL["bf16"])
    with pytest.raises(_lib.HogwildError) as ei:
        c513 = _many_fragments("bf16", 513, 1, 1, 2, 1, 64, 9).to(_dev())
        _lib.Problem(q=c513.q, locations=c513.locations, keys=c513.keys, values=c513.values, scale=c513.scale,
                     out=torch.empty_like(c513.q), cosines=c513.cos, sines=c513.sin)
    assert ei.value.status == -5


@pytest.mark.parametrize("dtype,F,W,S,Hq,Hkv,E", [
    ("bf16", 130, 4, 1, 8, 2, 128),      # three launches of 44 / 43 / 43 fragments, 16 rows per kv head
    ("f32", 65, 3, 2, 6, 2, 64),         # two launches, fp32
    ("f16", 129, 8, 2, 32, 2, 128),      # 256 rows per kv head: every launch runs the 128-row kernel
    ("bf16", 512, 2, 1, 4, 2, 64),       # the limit: eight launches
])
def test_more_fragments_than_one_launch_takes(oracle, dtype, F, W, S, Hq, Hkv, E):
    """More than 64 fragments: groups of at most 64 per attention launch, their split-K partials side by side in the
    workspace, one merge over all of them.  Checked against the oracle, rotated queries included, and against the same
    call with the fragments' order reversed (other groups, other partials, same mathematics)."""
    from inference_lib_amd import _lib
    c = _many_fragments(dtype, F, W, S, Hq, Hkv, E, seed=F)
    print(f"case {c.name} F={F} W={W} S={S} Hq={Hq} Hkv={Hkv} E={E}", flush=True)
    out, lse, rq = run_fused(c.to(_dev()))
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    assert_close("rq", rq, rq_ref, 1e-5 if dtype == "f32" else 3.2e-2)
    assert_close("out", out, o_ref, TOL[dtype])
    assert_close("lse", lse, l_ref, TOL[dtype])
    cd = c.to(_dev())
    rev = lambda t: torch.flip(t, dims=[0]).contiguous()
    out2 = torch.full_like(out, float("nan"))
    lse2 = torch.full_like(lse, float("nan"))
    pr = _lib.Problem(q=cd.q, locations=rev(cd.locations), keys=cd.keys[::-1], values=cd.values[::-1], scale=c.scale, out=out2,
                      cosines=rev(cd.cos), sines=rev(cd.sin), lse=lse2)
    pr.run()
    torch.cuda.synchronize()
    assert_close("out (reversed)", out2, o_ref, TOL[dtype])
    assert_close("lse (reversed)", lse2, l_ref, TOL[dtype])
    # the two stages separately give the same bits as the one call
    out3 = torch.full_like(out, float("nan"))
    lse3 = torch.full_like(lse, float("nan"))
    p3 = _lib.Problem(q=cd.q, locations=cd.locations, keys=cd.keys, values=cd.values, scale=c.scale, out=out3, cosines=cd.cos,
                      sines=cd.sin, lse=lse3)
    p3.run(stages=1)
    p3.run(stages=2)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.uint8), out3.view(torch.uint8)) and torch.equal(lse.view(torch.uint8), lse3.view(torch.uint8))


def test_more_fragments_pre_rotated_and_partial_rotary(oracle):
    """The other two ways into the attention kernel with more than 64 fragments: hw_sdpa (queries rotated per fragment by
    the caller) and a rotary width below the head dimension (rotated by the standalone kernel into the workspace)."""
    from inference_lib_amd import _lib
    c = _many_fragments("bf16", 100, 3, 1, 6, 2, 128, seed=77)
    cd = c.to(_dev())
    W, Hq, S, E = cd.q.shape
    rq = torch.full((c.F, W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
    _lib.rope(cd.q, cd.cos, cd.sin, rq)
    out = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
    lse = torch.full((W, Hq, S), float("nan"), dtype=torch.float32, device=_dev())
    _lib.Problem(q=rq, locations=cd.locations, keys=cd.keys, values=cd.values, scale=c.scale, out=out, lse=lse, prerotated=True).run()
    torch.cuda.synchronize()
    o2, l2 = oracle.sdpa_fragments(np64(rq), c.locations.numpy(), [np64(k) for k in c.keys], [np64(v) for v in c.values], c.scale)
    assert_close("sdpa out", out, o2, TOL["bf16"])
    assert_close("sdpa lse", lse, l2, TOL["bf16"])
    c = _many_fragments("f16", 70, 2, 2, 4, 2, 64, seed=78, rot_dim=32)
    out, lse, rq = run_fused(c.to(_dev()))
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    assert_close("rq", rq, rq_ref, 3.2e-2)
    assert_close("out", out, o_ref, TOL["f16"])
    assert_close("lse", lse, l_ref, TOL["f16"])
    out2, lse2, _ = run_fused(c.to(_dev()), with_rq=False)     # rotated queries go to the workspace instead
    assert torch.equal(out, out2) and torch.equal(lse, lse2)


def test_long_fragment_many_tiles_per_workgroup(oracle):
    """One kv head and a 150k-token fragment: every workgroup walks hundreds of tiles; S=3 gives a causal tail."""
    from inference_lib_amd import cases
    g = torch.Generator().manual_seed(5)
    c = cases.build_case("long", "f16", 1, 3, 4, 1, 128, 1e6, [150_001, 77], [[0, 1]], g)
    out, lse, _ = run_fused(c.to(_dev()))
    o_ref, l_ref, _ = oracle_fused(oracle, c)
    assert_close("out", out, o_ref, TOL["f16"])
    assert_close("lse", lse, l_ref, TOL["f16"])


def test_fragment_at_the_32_bit_offset_limit():
    """The longest fragment the byte-offset arithmetic allows (just under 2^31 bytes per kv head, 8.39 M tokens of
    bf16 at head dim 128).  Closed form instead of the oracle: all keys are zero except one, which is a large multiple
    of the query, so the softmax is that token alone and the output must be exactly its value row -- at the last
    token (highest offsets), in the middle, and at the first.  One token more is refused."""
    from inference_lib_amd import _lib
    dev = _dev()
    L, E = 8_388_000, 128
    g = torch.Generator().manual_seed(17)
    q = torch.randn((1, 1, 1, E), generator=g).to(torch.bfloat16).to(dev)
    K = torch.zeros((1, L, E), dtype=torch.bfloat16, device=dev)
    V = torch.empty((1, L, E), dtype=torch.bfloat16, device=dev).normal_(generator=torch.Generator(device=dev).manual_seed(1))
    loc = torch.tensor([[[L - 1]]], dtype=torch.int32, device=dev)
    cos = torch.ones((1, 1, 1, E), dtype=torch.float32, device=dev)
    sin = torch.zeros((1, 1, 1, E), dtype=torch.float32, device=dev)
    out = torch.empty((1, 1, 1, E), dtype=torch.bfloat16, device=dev)
    lse = torch.empty((1, 1, 1), dtype=torch.float32, device=dev)
    scale = E ** -0.5
    for idx in (L - 1, 5_000_001, 0):
        print(f"peak at token {idx} of {L}", flush=True)
        K.zero_()
        K[0, idx] = (4.0 * q[0, 0, 0].float()).to(torch.bfloat16)
        _lib.Problem(q=q, locations=loc, keys=[K], values=[V], scale=scale, out=out, cosines=cos, sines=sin, lse=lse).run()
        torch.cuda.synchronize()
        score = float((q[0, 0, 0].float() * K[0, idx].float()).sum()) * scale
        assert score > 30
        assert torch.equal(out[0, 0, 0], V[0, idx])
        assert abs(float(lse) - score) <= 1e-3          # the other 8.4 M tokens weigh e^(16 - score)
    del K, V
    too_long = 0x7fff0000 // (E * 2)                     # first length whose byte size reaches the limit
    K = torch.zeros((1, too_long, E), dtype=torch.bfloat16, device=dev)
    with pytest.raises(_lib.HogwildError) as ei:
        _lib.Problem(q=q, locations=loc, keys=[K], values=[K], scale=scale, out=out, cosines=cos, sines=sin, lse=lse).run()
    assert ei.value.status == -3


def test_two_stages_equal_the_fused_call():
    from inference_lib_amd import cases
    cd = cases.baseline_case(2).to(_dev())
    W, Hq, S, E = cd.q.shape
    out1 = torch.empty((W, Hq, S, E), dtype=cd.q.dtype, device=_dev())
    out2 = torch.full_like(out1, float("nan"))
    lse1 = torch.empty((W, Hq, S), dtype=torch.float32, device=_dev())
    lse2 = torch.full_like(lse1, float("nan"))
    _problem(cd, out1, lse=lse1).run()
    pr = _problem(cd, out2, lse=lse2)
    pr.run(stages=1)
    torch.cuda.synchronize()
    assert torch.isnan(out2.float()).all()          # the attention stage alone does not touch the output
    pr.run(stages=2)
    torch.cuda.synchronize()
    assert torch.equal(out1, out2) and torch.equal(lse1, lse2)


@pytest.mark.parametrize("dtype,W,S,Hq,Hkv,E,lens", [
    ("bf16", 2, 1, 8, 2, 128, (128, 0, 0)),            # 4 tiles: one workgroup per head by itself
    ("f16", 2, 1, 8, 2, 64, (500, 0, 0)),              # 16 tiles in one fragment: the planner prefers one workgroup
    ("bf16", 3, 2, 12, 4, 128, (100, 0, 33, 57)),      # three short fragments, an empty one, 18 rows
    ("f32", 2, 1, 8, 2, 64, (64, 20, 5)),              # fp32, 4 tiles
    ("f16", 4, 3, 8, 2, 128, (64, 30, 0, 0, 31)),      # 48 rows per kv head: two row groups, each writing its rows
])
def test_one_workgroup_per_head_writes_the_result_itself(oracle, dtype, W, S, Hq, Hkv, E, lens):
    """A plan with one workgroup per kv head normalises in the attention kernel and launches no merge; the result is
    that of the two stages (attention kernel into the workspace, merge kernel) bit for bit, and the oracle's within the
    usual tolerance."""
    from inference_lib_amd import _lib, cases
    c = cases.small_case(dtype=dtype, W=W, S=S, Hq=Hq, Hkv=Hkv, E=E, lens=lens, seed=41)
    pl = _lib.plan(list(lens), W=W, S=S, Hq=Hq, Hkv=Hkv, Ev=E, num_cus=256,
                   dtype={"f32": _lib.HW_F32, "f16": _lib.HW_F16, "bf16": _lib.HW_BF16}[dtype])
    assert pl.wgs_per_head == 1
    cd = c.to(_dev())
    out1 = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
    out2 = torch.full_like(out1, float("nan"))
    lse1 = torch.full((W, Hq, S), float("nan"), dtype=torch.float32, device=_dev())
    lse2 = torch.full_like(lse1, float("nan"))
    p1 = _problem(cd, out1, lse=lse1)
    ws = torch.full((p1.workspace_bytes(),), 0xAB, dtype=torch.uint8, device=_dev())
    p1.set_workspace(ws)
    p1.run()
    torch.cuda.synchronize()
    assert bool((ws == 0xAB).all())                      # the single launch leaves the workspace alone
    p2 = _problem(cd, out2, lse=lse2)
    p2.run(stages=1)
    torch.cuda.synchronize()
    assert torch.isnan(out2.float()).all()
    p2.run(stages=2)
    torch.cuda.synchronize()
    assert torch.equal(out1.view(torch.uint8), out2.view(torch.uint8)) and torch.equal(lse1.view(torch.uint8), lse2.view(torch.uint8))
    want_o, want_l, _ = oracle_fused(oracle, c)
    assert_close("out", out1, want_o, TOL[dtype])
    assert_close("lse", lse1, want_l, TOL[dtype])


def test_side_stream_and_concurrent_streams(oracle):
    from inference_lib_amd import cases
    ca = cases.small_case(dtype="bf16", W=2, S=1, Hq=8, Hkv=2, E=128, lens=(900, 300, 411), seed=31)
    cb = cases.small_case(dtype="f16", W=2, S=2, Hq=4, Hkv=2, E=64, lens=(500, 123, 77), seed=32)
    da, db = ca.to(_dev()), cb.to(_dev())
    oa = torch.empty((2, 8, 1, 128), dtype=torch.bfloat16, device=_dev())
    ob = torch.empty((2, 4, 2, 64), dtype=torch.float16, device=_dev())
    pa, pb = _problem(da, oa), _problem(db, ob)
    pa.set_workspace()
    pb.set_workspace()
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    for _ in range(5):
        with torch.cuda.stream(sa):
            pa.run()
        with torch.cuda.stream(sb):
            pb.run()
    torch.cuda.synchronize()
    assert_close("stream a", oa, oracle_fused(oracle, ca)[0], TOL["bf16"])
    assert_close("stream b", ob, oracle_fused(oracle, cb)[0], TOL["f16"])


def test_graph_replay_matches_eager():
    """Captured once, replayed several times with eager launches and synchronisations in between; the inputs
    change between replays and every replay must equal the eager result on the same inputs."""
    from inference_lib_amd import cases
    cd = cases.baseline_case(2).to(_dev())
    W, Hq, S, E = cd.q.shape
    out_g = torch.empty((W, Hq, S, E), dtype=cd.q.dtype, device=_dev())
    out_e = torch.empty_like(out_g)
    pg, pe = _problem(cd, out_g), _problem(cd, out_e)
    pg.set_workspace()
    pe.set_workspace()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        pg.run()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            pg.run()
    for it in range(4):
        cd.q.mul_(1.0 + 0.25 * it)                  # same buffers, new contents
        cd.keys[1].add_(0.125)
        torch.cuda.synchronize()
        out_g.fill_(float("nan"))
        graph.replay()
        pe.run()
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_e), f"replay {it} differs from the eager launch"


# ------------------------------------------------------------------------------------------------ many rows per kv head
@pytest.mark.parametrize("dtype,E,W,S,Hq,Hkv,lens", [
    ("f16", 128, 4, 4, 16, 2, (300, 64, 33, 70, 129)),        # 128 rows per kv head: one full row group
    ("bf16", 128, 3, 3, 14, 2, (257, 31, 0, 64)),             # 63 rows forced into the wide kernel, an empty fragment
    ("bf16", 64, 5, 4, 16, 2, (200, 40, 41, 42, 43, 44)),     # 160 rows: two row groups, the second partly filled
    ("f16", 64, 9, 2, 6, 2, (90, 10, 20, 30, 40, 50, 60, 70, 80, 33)),   # GQA 3: more (worker, token) pairs than staged table rows
    ("bf16", 128, 2, 40, 8, 2, (500, 100, 120)),              # 40 query tokens per worker (prefill-like), 320 rows
])
def test_wide_kernel_against_oracle(oracle, dtype, E, W, S, Hq, Hkv, lens):
    """The 128-row workgroups (row_blocks = 8; chosen automatically beyond 96 rows per kv head) against the oracle, and
    bit-identical to nothing: the narrow kernel sums in another order, so both are compared with the oracle."""
    from inference_lib_amd import _lib, cases
    c = cases.small_case(dtype=dtype, W=W, S=S, Hq=Hq, Hkv=Hkv, E=E, lens=lens, seed=len(lens) + W)
    cd = c.to(_dev())
    rows = W * S * (Hq // Hkv)
    print(f"wide case {c.name}: {rows} rows per kv head, lens {lens}", flush=True)
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    for rb in (8, 2):
        out = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
        lse = torch.full((W, Hq, S), float("nan"), dtype=torch.float32, device=_dev())
        rq = torch.full((c.F, W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
        pr = _lib.Problem(q=cd.q, locations=cd.locations, keys=cd.keys, values=cd.values, scale=cd.scale, out=out, cosines=cd.cos,
                          sines=cd.sin, rq=rq, lse=lse, row_blocks=rb)
        pr.run()
        torch.cuda.synchronize()
        assert_close(f"out rb={rb}", out, o_ref, TOL[dtype])
        assert_close(f"lse rb={rb}", lse, l_ref, TOL[dtype])
        assert_close(f"rq rb={rb}", rq, rq_ref, 3.2e-2)
    # pre-rotated queries through the same kernel
    out = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
    pr = _lib.Problem(q=rq, locations=cd.locations, keys=cd.keys, values=cd.values, scale=cd.scale, out=out, prerotated=True, row_blocks=8)
    pr.run()
    torch.cuda.synchronize()
    o2, _ = oracle.sdpa_fragments(np64(rq), c.locations.numpy(), [np64(k) for k in c.keys], [np64(v) for v in c.values], c.scale)
    assert_close("sdpa out", out, o2, TOL[dtype])


def test_wide_kernel_split_invariance_and_refusals():
    from inference_lib_amd import _lib, cases
    c = cases.small_case(dtype="bf16", W=4, S=4, Hq=16, Hkv=2, E=128, lens=(700, 64, 33, 70, 129), seed=4)
    cd = c.to(_dev())
    W, Hq, S, E = cd.q.shape
    outs = []
    for splits in (0, 1, 3, 7):
        out = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
        pr = _lib.Problem(q=cd.q, locations=cd.locations, keys=cd.keys, values=cd.values, scale=cd.scale, out=out, cosines=cd.cos,
                          sines=cd.sin, row_blocks=8, splits=splits)
        pr.run()
        torch.cuda.synchronize()
        outs.append(out.float())
    for o in outs[1:]:
        assert (o - outs[0]).abs().max().item() <= 2.0 ** -7 * outs[0].abs().max().item() + 1e-3
    # fp32 has no such kernel: the request is ignored (the narrow kernel runs), never a wrong launch
    c32 = cases.small_case(dtype="f32", W=4, S=4, Hq=16, Hkv=2, E=64, lens=(100, 20, 21, 22, 23), seed=2).to(_dev())
    out32 = torch.full(c32.q.shape, float("nan"), dtype=torch.float32, device=_dev())
    _lib.Problem(q=c32.q, locations=c32.locations, keys=c32.keys, values=c32.values, scale=c32.scale, out=out32, cosines=c32.cos,
                 sines=c32.sin, row_blocks=8).run()
    torch.cuda.synchronize()
    assert torch.isfinite(out32).all()


@pytest.mark.parametrize("row_blocks", [8, 2])
@pytest.mark.parametrize("dtype,E", [("bf16", 128), ("f16", 64)])
def test_waves_leave_the_unmasked_tiles_at_different_places(oracle, row_blocks, dtype, E):
    """The tile loop is two loops (tiles every row of a wave sees completely, then the rest).  Here the rows of one
    workgroup see different amounts of every fragment, so its waves change loops at different tiles: bounds exactly on a
    tile boundary, one token beyond it, nothing at all, one token, everything, per worker and per fragment."""
    from inference_lib_amd import cases
    W, S, Hq, Hkv = 8, 4, 8, 2                     # 128 rows per kv head; a wave of the 128-row kernel owns two workers
    lens = (200, 96, 33, 64, 40, 17, 128, 31, 70)  # prompt + one segment per worker
    c = cases.small_case(dtype=dtype, W=W, S=S, Hq=Hq, Hkv=Hkv, E=E, lens=lens, seed=21)
    loc = c.locations.clone()                      # [F, W, S]: a row sees positions <= its location
    for f, L in enumerate(lens):
        marks = [0, 1, 31, 32, 33, 64, L - 1, L]   # visible tokens of the fragment: tile boundaries and their neighbours
        for w in range(W):
            seen = min(marks[(3 * f + w) % 8], L)
            for s in range(S):
                loc[f, w, s] = min(seen + (s % 2), L) - 1      # the tokens of a worker differ by one
    c.locations = loc
    c.cos, c.sin = cases.rope_tables(loc, E, 1e4)
    print(f"{dtype} E={E} row_blocks={row_blocks} lens={lens}", flush=True)
    want_o, want_l, want_rq = oracle_fused(oracle, c)
    out, lse, rq = run_fused(c.to(_dev()), row_blocks=row_blocks)
    assert_close("out", out, want_o, TOL[dtype])
    assert_close("lse", lse, want_l, TOL[dtype])
    assert_close("rq", rq, want_rq, 3.2e-2)
