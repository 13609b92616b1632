"""GPU parity for head dimension 256 (E = Ev = 256: one 16-row block per workgroup; the fragment operators in all
three dtypes, the paged operators in the 16-bit types) against the oracle, through the C ABI.
Tolerances: bf16 / fp16 2e-2 with the signal-relative bound of helpers.Tol, fp32 1e-4."""
import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, oracle_fused, run_fused
from test_gpu_paged import build_paged, check as check_paged

pytestmark = pytest.mark.gpu


def _dev():
    return torch.device("cuda:0")


@pytest.mark.parametrize("dtype", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("W,S,Hq,Hkv,lens", [
    (2, 1, 8, 2, (100, 37, 65)),          # 8 rows per kv head, one workgroup per head: the result is written directly
    (2, 1, 8, 2, (1500, 700, 650)),       # split over many workgroups: merge launch
    (4, 2, 8, 2, (900, 40, 33, 64, 1)),   # 32 rows per kv head: two row groups of 16
    (3, 1, 10, 2, (300, 31, 32, 33)),     # 15 rows: GQA ratio 5
])
def test_fused_head_dim_256(oracle, dtype, W, S, Hq, Hkv, lens):
    from inference_lib_amd import cases
    c = cases.small_case(dtype=dtype, W=W, S=S, Hq=Hq, Hkv=Hkv, E=256, lens=lens, seed=17 + W)
    print(f"case {c.name} E=256 lens={lens}", flush=True)
    out, lse, rq = run_fused(c.to(_dev()))
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    tol = TOL[dtype]
    assert_close("out", out, o_ref, tol)
    assert_close("lse", lse, l_ref, tol)
    assert_close("rq", rq, rq_ref, 1e-5 if dtype == "f32" else 3.2e-2)


@pytest.mark.parametrize("splits", [1, 2, 7])
def test_split_invariance_head_dim_256(oracle, splits):
    """A forced split and a request for two row blocks (which this head dimension does not have: the planner keeps one)."""
    from inference_lib_amd import cases
    c = cases.small_case(dtype="bf16", W=2, S=3, Hq=8, Hkv=2, E=256, lens=(700, 90, 45), seed=3)
    out, lse, _ = run_fused(c.to(_dev()), splits=splits, row_blocks=2)
    o_ref, l_ref, _ = oracle_fused(oracle, c)
    assert_close("out", out, o_ref, TOL["bf16"])
    assert_close("lse", lse, l_ref, TOL["bf16"])


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_rope_and_sdpa_entries_head_dim_256(oracle, dtype):
    """hw_rope and hw_sdpa (pre-rotated queries) at head dimension 256."""
    from inference_lib_amd import _lib, cases
    c = cases.small_case(dtype=dtype, W=3, S=2, Hq=6, Hkv=2, E=256, lens=(70, 33, 1, 64), seed=5)
    cd = c.to(_dev())
    W, Hq, S, E = cd.q.shape
    rq = torch.full((c.F, W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
    _lib.rope(cd.q, cd.cos, cd.sin, rq)
    torch.cuda.synchronize()
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    assert_close("rq", rq, rq_ref, 1e-5 if dtype == "f32" else 3.2e-2)
    out = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=_dev())
    lse = torch.full((W, Hq, S), float("nan"), dtype=torch.float32, device=_dev())
    _lib.Problem(q=rq, locations=cd.locations, keys=cd.keys, values=cd.values, scale=c.scale, out=out, lse=lse, prerotated=True).run()
    torch.cuda.synchronize()
    assert_close("out", out, o_ref, TOL[dtype])
    assert_close("lse", lse, l_ref, TOL[dtype])


def test_partial_rotary_head_dim_256(oracle):
    """Rotary width 128 of a 256-wide head: rotated by the standalone kernel, then the pre-rotated attention kernel."""
    from inference_lib_amd import cases
    c = cases.small_case(dtype="f16", W=2, S=2, Hq=4, Hkv=2, E=256, lens=(90, 40, 47), seed=21, rot_dim=128)
    out, lse, rq = run_fused(c.to(_dev()))
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    assert_close("out", out, o_ref, TOL["f16"])
    assert_close("lse", lse, l_ref, TOL["f16"])
    assert_close("rq", rq, rq_ref, 3.2e-2)


def test_device_lengths_head_dim_256(oracle):
    """Fragment lengths in device memory; the buffers are longer than the fragments and hold NaN beyond them."""
    from inference_lib_amd import _lib, cases
    c = cases.small_case(dtype="bf16", W=2, S=1, Hq=8, Hkv=2, E=256, lens=(800, 37, 65), seed=9)
    dev = _dev()
    cd = c.to(dev)
    keys, values = [], []
    for k, v, extra in zip(cd.keys, cd.values, (33, 0, 70)):
        keys.append(torch.cat([k, torch.full((k.size(0), extra, k.size(2)), float("nan"), dtype=k.dtype, device=dev)], dim=1).contiguous())
        values.append(torch.cat([v, torch.full((v.size(0), extra, v.size(2)), float("nan"), dtype=v.dtype, device=dev)], dim=1).contiguous())
    len_dev = torch.tensor(c.lens, dtype=torch.int32, device=dev)
    W, Hq, S, E = cd.q.shape
    out = torch.full((W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=dev)
    lse = torch.full((W, Hq, S), float("nan"), dtype=torch.float32, device=dev)
    rq = torch.full((c.F, W, Hq, S, E), float("nan"), dtype=cd.q.dtype, device=dev)
    _lib.Problem(q=cd.q, locations=cd.locations, keys=keys, values=values, scale=c.scale, out=out, cosines=cd.cos, sines=cd.sin,
                 rq=rq, lse=lse, len_dev=len_dev).run()
    torch.cuda.synchronize()
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    assert_close("out", out, o_ref, TOL["bf16"])
    assert_close("lse", lse, l_ref, TOL["bf16"])
    assert_close("rq", rq, rq_ref, 3.2e-2)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("bs,S,F", [(16, 1, 1), (8, 3, 2), (128, 4, 1)])
def test_paged_head_dim_256(dtype, bs, S, F):
    mb = max(1, 300 // bs)
    c = build_paged(dtype, F, 3, 10, 2, 256, bs, mb, seq_lens=[200, 37, 1 + S + 3 * F], S=S, seed=bs + S)
    check_paged(c)


def test_paged_many_rows_head_dim_256():
    """More than 16 rows per sequence (where the other head dimensions use 128-row workgroups): row groups of 16."""
    c = build_paged("bf16", 1, 2, 8, 2, 256, 16, 50, seq_lens=[700, 129], S=6, seed=11)
    check_paged(c)
    check_paged(c, splits=3, row_blocks=8)       # (a request for the 128-row kernel is not honoured at this head dimension)


def test_varlen_head_dim_256():
    c = build_paged("f16", 2, 5, 10, 2, 256, 16, 30, seq_lens=[400, 50, 9, 130, 64], q_lens=[3, 0, 9, 40, 1], seed=21)
    check_paged(c)


def test_what_head_dim_256_does_not_have():
    """The fp32 paged kernel and the VALU-logits variant are refused with HW_ERR_UNSUPPORTED, never run as something else."""
    from inference_lib_amd import _lib, cases
    c = build_paged("f32", 1, 2, 4, 2, 256, 16, 8, seq_lens=[100, 37], S=1, seed=1)
    dev = _dev()
    d = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in c.items()}
    out = torch.zeros((2, 4, 1, 256), dtype=torch.float32, device=dev)
    pr = _lib.PagedProblem(q=d["q"], locations=d["loc"], fragment_lengths=d["fl"], key_cache=d["kc"], value_cache=d["vc"],
                           block_table=d["bt"], scale=c["scale"], out=out)
    with pytest.raises(_lib.HogwildError) as ei:
        pr.run()
    assert ei.value.status == -4     # HW_ERR_UNSUPPORTED
    cs = cases.small_case(dtype="bf16", W=2, S=1, Hq=8, Hkv=2, E=256, lens=(100, 37, 5), seed=2).to(dev)
    o = torch.zeros((2, 8, 1, 256), dtype=torch.bfloat16, device=dev)
    with pytest.raises(_lib.HogwildError) as ei:
        _lib.Problem(q=cs.q, locations=cs.locations, keys=cs.keys, values=cs.values, scale=cs.scale, out=o, cosines=cs.cos,
                     sines=cs.sin, variant=_lib.HW_VARIANT_VALU_QK).run()
    assert ei.value.status == -4     # HW_ERR_UNSUPPORTED


EDGE = [0, 1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 255, 256, 257, 1000, 1023, 1025]


@pytest.mark.parametrize("seed", range(18))
def test_fused_random_shapes_head_dim_256(oracle, seed):
    """Random shapes as in test_gpu_random.py, at head dimension 256: fragment lengths around the tile size, empty fragments,
    random worker orders, 1..9 workers, several query tokens, GQA 1..7 and 16, explicit split factors, all three dtypes."""
    from inference_lib_amd import cases
    rng = np.random.default_rng(25600 + seed)
    dtype = ["bf16", "f16", "f32"][seed % 3]
    W = int(rng.integers(1, 10))
    S = int(rng.choice([1, 1, 1, 2, 3]))
    Hkv = int(rng.choice([1, 2, 4, 8]))
    GQ = 16 if seed % 9 == 8 else int(rng.integers(1, 8))
    F = int(rng.integers(1, 13))
    lens = [int(rng.choice(EDGE)) if rng.random() < 0.7 else int(rng.integers(0, 3000)) for _ in range(F)]
    if sum(lens) == 0:
        lens[0] = 40
    orders = [[int(x) for x in rng.permutation(F)] for _ in range(W)]
    c = cases.build_case(f"rand256_{seed}", dtype, W, S, Hkv * GQ, Hkv, 256, 1e4, lens, orders, torch.Generator().manual_seed(seed))
    splits = int(rng.choice([0, 0, 1, 3, 7, 40]))
    print(f"seed {seed}: {dtype} W={W} S={S} Hq={Hkv * GQ} Hkv={Hkv} lens={lens} splits={splits}", flush=True)
    want_o, want_l, want_rq = oracle_fused(oracle, c)
    out, lse, rq = run_fused(c.to(_dev()), splits=splits)
    assert_close("out", out, want_o, TOL[dtype])
    assert_close("lse", lse, want_l, TOL[dtype])
    assert_close("rq", rq, want_rq, 1e-5 if dtype == "f32" else 3.2e-2)


@pytest.mark.parametrize("seed", range(12))
def test_paged_random_shapes_head_dim_256(seed):
    rng = np.random.default_rng(25700 + seed)
    dtype = ["bf16", "f16"][seed % 2]
    W = int(rng.integers(1, 7))
    Hkv = int(rng.choice([1, 2, 4, 8]))
    GQ = int(rng.integers(1, 8))
    bs = int(rng.choice([1, 4, 8, 16, 16, 32, 48, 64, 256]))
    F = int(rng.integers(1, 4))
    varlen = bool(rng.random() < 0.4)
    S = int(rng.choice([1, 1, 2, 5]))
    longest = int(rng.choice([40, 130, 700, 2100]))
    seq = [int(rng.integers(S + 3 * F + 1, longest + S + 3 * F + 2)) for _ in range(W)]
    mb = (max(seq) + bs - 1) // bs + int(rng.integers(0, 3))
    kw = dict(seed=seed, loc_mode="random" if rng.random() < 0.5 else "causal")
    if varlen:
        ql = [int(min(s - 3 * F, x)) for s, x in zip(seq, rng.integers(0, 7, size=W))]
        if sum(ql) == 0:
            ql[0] = 1
        c = build_paged(dtype, F, W, Hkv * GQ, Hkv, 256, bs, mb, seq_lens=seq, q_lens=ql, **kw)
    else:
        c = build_paged(dtype, F, W, Hkv * GQ, Hkv, 256, bs, mb, seq_lens=seq, S=S, **kw)
    check_paged(c, splits=int(rng.choice([0, 0, 1, 5])))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_repeated_runs_are_bit_identical_head_dim_256(dtype):
    """The same call repeated with the caches overwritten in between gives the same bits every time.  (A 256-wide fp32
    tile is 64 vector-memory operations in flight; the operand reads once ran ahead of the tile's transfers and the result
    depended on how fast memory answered.)"""
    from inference_lib_amd import cases
    c = cases.small_case(dtype=dtype, W=4, S=2, Hq=8, Hkv=2, E=256, lens=(900, 40, 33, 64, 1), seed=21)
    cd = c.to(_dev())
    flush = torch.empty(384 * 1024 * 1024, dtype=torch.uint8, device=_dev())
    ref = None
    for rep in range(25):
        flush.fill_(rep)
        out, lse, rq = run_fused(cd)
        cur = [t.clone().view(torch.uint8) for t in (out, lse, rq)]
        if ref is None:
            ref = cur
        else:
            assert all(torch.equal(a, b) for a, b in zip(ref, cur)), f"run {rep} differs from the first"
