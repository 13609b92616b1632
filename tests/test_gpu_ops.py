"""The torch operator surface (namespace libhogatt) and the python wrappers that mirror
python/hogwild/attention.py:19-35,70-74 of the reference, on the GPU, against the oracle."""
import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, np64, oracle_fused

pytestmark = pytest.mark.gpu


def _dev():
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


def test_torch_ops_are_the_hip_path():
    from inference_lib_amd import attention
    assert attention.HAVE_TORCH_OPS, "hogatt.abi3.so not built"
    for name in ("hogwild_fused", "hogwild_sdpa", "hogwild_rope", "hogwild_fused_lse", "hogwild_sdpa_lse"):
        assert hasattr(torch.ops.libhogatt, name)


@pytest.mark.parametrize("dtype", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("E", [128, 256])
def test_wrappers_match_oracle(oracle, dtype, E):
    from inference_lib_amd import attention, cases
    c = cases.small_case(dtype=dtype, W=2, S=1, Hq=8, Hkv=2, E=E, lens=(300, 70, 129, 5, 9), seed=3, with_cur=True)
    cd = c.to(_dev())
    print(f"case {c.name}", flush=True)
    W, Hq, S, E = cd.q.shape
    frag = torch.tensor(c.lens, dtype=torch.int32, device=_dev())
    # fragments handed over the way the caller does: [1, Hkv, L, D] (python/hogwild/attention.py:199-203)
    keys = [k.unsqueeze(0) for k in cd.keys]
    vals = [v.unsqueeze(0) for v in cd.values]
    rq = torch.empty((c.F, W, Hq, S, E), dtype=cd.q.dtype, device=_dev())
    out = torch.empty((W, Hq, S, E), dtype=cd.q.dtype, device=_dev())
    lse = torch.empty((W, Hq, S), dtype=torch.float32, device=_dev())
    ret = attention.hogwild_fused(cd.q, cd.locations, keys, vals, c.scale, frag, cd.cos, cd.sin, rotated_queries=rq, out=out)
    assert ret is out
    out_l = torch.empty_like(out)
    attention.hogwild_fused(cd.q, cd.locations, keys, vals, c.scale, frag, cd.cos, cd.sin, rotated_queries=rq, out=out_l, lse=lse)
    torch.cuda.synchronize()
    o_ref, l_ref, rq_ref = oracle_fused(oracle, c)
    assert_close("out", out, o_ref, TOL[dtype])
    assert torch.equal(out, out_l)
    assert_close("lse", lse, l_ref, TOL[dtype])
    assert_close("rq", rq, rq_ref, 1e-5 if dtype == "f32" else 3.2e-2)

    # the two halves separately, with the defaults of the reference wrappers (allocated outputs, derived lengths)
    rq2 = attention.hogwild_rope(cd.q, cd.cos, cd.sin)
    assert torch.equal(rq2, rq)
    out2 = attention.hogwild_sdpa(rq2, cd.locations, keys, vals, c.scale)
    torch.cuda.synchronize()
    assert out2.shape == out.shape and out2.dtype == out.dtype
    assert_close("sdpa out", out2, o_ref, TOL[dtype])


def test_fused_accepts_noncontiguous_fragments(oracle):
    """hogwild_fused copies non-contiguous fragments (src/binding.cu:330-337); hogwild_sdpa via the raw op rejects them."""
    from inference_lib_amd import attention, cases
    c = cases.small_case(dtype="bf16", W=2, S=1, Hq=4, Hkv=2, E=128, lens=(64, 40, 33), seed=8)
    cd = c.to(_dev())
    W, Hq, S, E = cd.q.shape
    keys = [torch.cat([k, k], dim=1)[:, ::2, :] for k in cd.keys]     # strided views with the same content per row pair
    vals = [torch.cat([v, v], dim=1)[:, ::2, :] for v in cd.values]
    for i in range(c.F):
        L = c.lens[i]
        keys[i] = torch.stack([cd.keys[i], cd.keys[i]], dim=2).reshape(cd.keys[i].shape[0], 2 * L, E)[:, ::2, :]
        vals[i] = torch.stack([cd.values[i], cd.values[i]], dim=2).reshape(cd.values[i].shape[0], 2 * L, E)[:, ::2, :]
        assert not keys[i].is_contiguous() and torch.equal(keys[i], cd.keys[i])
    frag = torch.tensor(c.lens, dtype=torch.int32, device=_dev())
    rq = torch.empty((c.F, W, Hq, S, E), dtype=cd.q.dtype, device=_dev())
    out = torch.empty((W, Hq, S, E), dtype=cd.q.dtype, device=_dev())
    attention.hogwild_fused(cd.q, cd.locations, keys, vals, c.scale, frag, cd.cos, cd.sin, rotated_queries=rq, out=out)
    torch.cuda.synchronize()
    o_ref, _, _ = oracle_fused(oracle, c)
    assert_close("out", out, o_ref, TOL["bf16"])
    with pytest.raises(RuntimeError):
        torch.ops.libhogatt.hogwild_sdpa(out, c.scale, cd.locations, rq, frag, keys, vals)


def test_errors_are_loud():
    """Unsupported shapes and dtypes raise (the reference prints and returns, kernel_v21.cuh:992-995, or silently
    does nothing, binding.cu:260-266)."""
    from inference_lib_amd import _lib, cases
    dev = _dev()
    c = cases.small_case(dtype="bf16", W=1, S=1, Hq=2, Hkv=1, E=128, lens=(40, 8), seed=1).to(dev)
    out = torch.empty((1, 2, 1, 128), dtype=torch.bfloat16, device=dev)
    # head dim 96 is not instantiated
    q96 = torch.zeros((1, 2, 1, 96), dtype=torch.bfloat16, device=dev)
    k96 = [torch.zeros((1, 40, 96), dtype=torch.bfloat16, device=dev)]
    loc = torch.zeros((1, 1, 1), dtype=torch.int32, device=dev)
    cs = torch.zeros((1, 1, 1, 96), dtype=torch.float32, device=dev)
    o96 = torch.empty((1, 2, 1, 96), dtype=torch.bfloat16, device=dev)
    pr = _lib.Problem(q=q96, locations=loc, keys=k96, values=k96, scale=0.1, out=o96, cosines=cs, sines=cs)
    with pytest.raises(_lib.HogwildError) as ei:
        pr.run()
    assert ei.value.status == -4
    # float64 is no dtype of the library
    with pytest.raises(_lib.HogwildError):
        _lib.Problem(q=c.q.double(), locations=c.locations, keys=[k.double() for k in c.keys], values=[v.double() for v in c.values],
                     scale=0.1, out=out.double(), cosines=c.cos, sines=c.sin)
    # workspace too small
    pr = _lib.Problem(q=c.q, locations=c.locations, keys=c.keys, values=c.values, scale=0.1, out=out, cosines=c.cos, sines=c.sin)
    pr.set_workspace(torch.empty(16, dtype=torch.uint8, device=dev))
    with pytest.raises(_lib.HogwildError) as ei:
        pr.run()
    assert ei.value.status == -6
    # a torch op with an int64 locations tensor
    with pytest.raises(RuntimeError):
        torch.ops.libhogatt.hogwild_sdpa(out, 0.1, c.locations.long(), torch.zeros((2, 1, 2, 1, 128), dtype=torch.bfloat16, device=dev),
                                         torch.tensor(c.lens, dtype=torch.int32, device=dev), c.keys, c.values)


def test_reference_import_path_and_call_sequence(oracle):
    """An unchanged caller: `from hogwild.attention import hogwild_fused` (python/hogwild/attention.py:12-23) and the call
    sequence of AttentionModule.forward (:325-336) -- buffers shaped as the cache object shapes them (:206-218), fragments
    as [1, Hkv, L, D] views of segment caches, the fused operator through its wrapper and through torch.ops.libhogatt
    directly, then the transpose/reshape of :338-339."""
    import hogwild.attention as ref_api
    from hogwild.attention import hogwild_fused, hogwild_rope, hogwild_sdpa
    from inference_lib_amd import cases
    assert not hasattr(ref_api, "hogwild_sdpa_pt"), "the pure-torch path is test infrastructure, not part of the package"
    c = cases.small_case(dtype="bf16", W=3, S=1, Hq=12, Hkv=4, E=128, lens=(257, 40, 64, 9, 3, 1, 2), seed=21, with_cur=True)
    cd = c.to(_dev())
    W, Hq, S, E = cd.q.shape
    segs = [ref_api.SegmentCache(1, c.Hkv, E, L + 4, dtype=cd.q.dtype, device=_dev()) for L in c.lens]
    for sg, k, v in zip(segs, cd.keys, cd.values):
        sg.update(k.unsqueeze(0), v.unsqueeze(0), 0)
    query_states = cd.q
    frags = torch.tensor(c.lens, dtype=torch.int32, device=_dev())
    keys = [sg.key_cache[0] for sg in segs]          # views [1, Hkv, L, D] into the segment buffers
    values = [sg.value_cache[0] for sg in segs]
    assert keys[0].dim() == 4 and keys[0].size(0) == 1
    rq = torch.empty((cd.cos.size(0), W, Hq, S, E), dtype=query_states.dtype, device=_dev())                       # :206-211
    att_buffer = torch.empty((rq.size(1), rq.size(2), rq.size(3), values[0].size(3)), dtype=rq.dtype, device=_dev())   # :213-218
    attn_output = hogwild_fused(query_states, cd.locations, keys, values, c.scale, frags, cd.cos, cd.sin, rotated_queries=rq,
                                out=att_buffer)
    out_op = torch.empty_like(attn_output)
    rq_op = torch.empty_like(rq)
    torch.ops.libhogatt.hogwild_fused(out_op, rq_op, c.scale, cd.locations, query_states.contiguous(), frags, keys, values, cd.cos, cd.sin)
    torch.cuda.synchronize()
    o_ref, _, rq_ref = oracle_fused(oracle, c)
    assert_close("out", attn_output, o_ref, TOL["bf16"])
    assert torch.equal(attn_output, out_op) and torch.equal(rq.view(torch.int16), rq_op.view(torch.int16))
    assert_close("rq", rq, rq_ref, 3.2e-2)
    flat = attn_output.transpose(1, 2).reshape(W, S, -1).contiguous()
    assert flat.shape == (W, S, Hq * E)
    # the two halves through the same import path
    out2 = hogwild_sdpa(hogwild_rope(query_states, cd.cos, cd.sin), cd.locations, keys, values, c.scale)
    torch.cuda.synchronize()
    assert_close("sdpa out", out2, o_ref, TOL["bf16"])
