"""GPU parity of the caller-side steps (hw_build_inputs, hw_rope_append, the HogwildCache / merge_caches mirror)
against oracle/cache_oracle.py, and of the attention operators reading segments that grow in place.
Key rotation in eager mode and every append are bit-exact; rotary tables: float32 within 5e-7, rounded tables equal up
to rare one-ulp flips; attention outputs bf16/fp16 2e-2, fp32 1e-4."""
import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, np64

pytestmark = pytest.mark.gpu

TDT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
DEV = "cuda:0"


def inv_freq(D, base=10000.0):
    return (base ** (-np.arange(0, D, 2, dtype=np.float64) / D)).astype(np.float32)


# ---------------------------------------------------------------------------------------------- input builder
@pytest.mark.parametrize("table", [None, "bf16", "f16"])
def test_build_inputs_matches_oracle(table):
    from inference_lib_amd import _lib
    from oracle import cache_oracle as co
    lens = [4096, 200, 33, 1, 950_000]
    orders = [[0, 1, 2, 3, 4], [4, 0, 2, 1, 3], [3, 2, 1, 0, 4]]
    S, D = 3, 128
    pe = co.pos_end_from_orders(orders, lens)
    f = inv_freq(D)
    want_loc, want_cos, want_sin = co.build_inputs(pe, S, f, attention_scaling=0.9, table_dtype=table or "f32")
    loc, cos, sin = _lib.build_inputs(pe.tolist(), S, torch.from_numpy(f).to(DEV), attention_scaling=0.9,
                                      table_dtype=None if table is None else TDT[table])
    torch.cuda.synchronize()
    assert loc.dtype == torch.int32 and cos.dtype == torch.float32 and tuple(cos.shape) == (5, 3, S, D)
    assert np.array_equal(loc.cpu().numpy(), want_loc)
    for got, want in ((cos, want_cos), (sin, want_sin)):
        g = got.cpu().numpy()
        if table is None:
            assert np.abs(g - want).max() <= 5e-7
        else:
            ulp = 2.0 ** -8 if table == "bf16" else 2.0 ** -11
            assert np.abs(g - want).max() <= ulp and np.mean(g == want) > 0.995
    # both halves of the rotary width carry the same angles
    assert torch.equal(cos[..., : D // 2], cos[..., D // 2:]) and torch.equal(sin[..., : D // 2], sin[..., D // 2:])


def test_build_inputs_many_fragments_and_no_rotation():
    from inference_lib_amd import _lib
    from oracle import cache_oracle as co
    F, W, S = 30, 40, 2                                   # more (fragment, worker) pairs than one launch takes
    pe = np.arange(F * W).reshape(F, W) * 3 + S
    f = inv_freq(64)
    want_loc, want_cos, _ = co.build_inputs(pe, S, f)
    loc, cos, sin = _lib.build_inputs(pe.tolist(), S, torch.from_numpy(f).to(DEV))
    torch.cuda.synchronize()
    assert np.array_equal(loc.cpu().numpy(), want_loc) and np.abs(cos.cpu().numpy() - want_cos).max() <= 5e-7
    loc0, cos0, _ = _lib.build_inputs(pe.tolist(), S, None, device=DEV)
    assert np.array_equal(loc0.cpu().numpy(), want_loc) and cos0.shape[-1] == 0


# ---------------------------------------------------------------------------------------------- rotate + append
def tables(pos, R, cs):
    ang = pos.float()[..., None] * torch.from_numpy(inv_freq(R))
    emb = torch.cat([ang, ang], -1)
    return emb.cos().to(TDT[cs]), emb.sin().to(TDT[cs])


@pytest.mark.parametrize("dtype,cs", [("bf16", "bf16"), ("f16", "f16"), ("f32", "f32"), ("bf16", "f32"), ("f16", "f32")])
@pytest.mark.parametrize("E,Ev,R", [(128, 128, 128), (64, 64, 32), (20, 12, 10), (128, 64, 0)])
def test_rope_append_eager_is_bit_exact(dtype, cs, E, Ev, R):
    from inference_lib_amd import _lib
    from oracle import cache_oracle as co
    g = torch.Generator().manual_seed(E + R)
    W, Hkv, S = 3, 2, 5
    tdt = TDT[dtype]
    # the layout a projection produces: [W, S, Hkv, D] viewed as [W, Hkv, S, D]
    ks = torch.randn((W, S, Hkv, E), generator=g).to(tdt).transpose(1, 2)
    vs = torch.randn((W, S, Hkv, Ev), generator=g).to(tdt).transpose(1, 2)
    pos = torch.tensor([[10, 11, 12, 13, 14], [0, 1, 2, 3, 4], [70000, 70001, 70002, 70003, 70004]])
    cos, sin = tables(pos, R, cs) if R > 0 else (None, None)
    caps, lens, n_new = [16, 9, 40], [3, 0, 35], [5, 2, 4]
    kd = [torch.randn((Hkv, c, E), generator=g).to(tdt) for c in caps]
    vd = [torch.randn((Hkv, c, Ev), generator=g).to(tdt) for c in caps]
    want_k, want_v = [np64(t) for t in kd], [np64(t) for t in vd]
    for w in range(W):
        rk = co.rope_keys(np64(ks[w]), np64(cos[w])[None], np64(sin[w])[None], storage=dtype, cs_storage=cs, mode="eager") if R > 0 else np64(ks[w])
        co.append_left_masked(want_k[w], lens[w], rk, n_new[w])
        co.append_left_masked(want_v[w], lens[w], np64(vs[w]), n_new[w])
    dk, dv = [t.to(DEV) for t in kd], [t.to(DEV) for t in vd]
    print(f"rope_append {dtype}/{cs} E={E} Ev={Ev} R={R}", flush=True)
    _lib.rope_append(ks.to(DEV), vs.to(DEV), dk, dv, lens, cosines=None if cos is None else cos.to(DEV),
                     sines=None if sin is None else sin.to(DEV), n_new=n_new)
    torch.cuda.synchronize()
    for w in range(W):
        assert np.array_equal(np64(dk[w]), want_k[w]), f"keys of worker {w}"
        assert np.array_equal(np64(dv[w]), want_v[w]), f"values of worker {w}"


def test_rope_append_fused_mode_is_within_one_rounding():
    from inference_lib_amd import _lib
    from oracle import cache_oracle as co
    g = torch.Generator().manual_seed(5)
    ks = torch.randn((2, 4, 7, 128), generator=g).to(torch.bfloat16)
    vs = torch.randn((2, 4, 7, 128), generator=g).to(torch.bfloat16)
    pos = torch.arange(7)[None] + torch.tensor([[100], [3000]])
    cos, sin = tables(pos, 128, "f32")
    kd = [torch.zeros((4, 7, 128), dtype=torch.bfloat16, device=DEV) for _ in range(2)]
    vd = [torch.zeros((4, 7, 128), dtype=torch.bfloat16, device=DEV) for _ in range(2)]
    _lib.rope_append(ks.to(DEV), vs.to(DEV), kd, vd, [0, 0], cosines=cos.to(DEV), sines=sin.to(DEV), mode=_lib.HW_ROPE_FUSED)
    torch.cuda.synchronize()
    for w in range(2):
        want = co.rope_keys(np64(ks[w]), np64(cos[w])[None], np64(sin[w])[None], storage="bf16", mode="exact")
        assert np.abs(np64(kd[w]) - want).max() <= 2.0 ** -6          # one bf16 ulp at |x| < 4
        assert np.mean(np64(kd[w]) == want) > 0.99
        assert torch.equal(vd[w].cpu(), vs[w])


def test_rope_append_rejects_a_full_segment_and_many_workers_work():
    from inference_lib_amd import _lib
    ks = torch.zeros((1, 1, 4, 64), dtype=torch.float16, device=DEV)
    kd = [torch.zeros((1, 5, 64), dtype=torch.float16, device=DEV)]
    with pytest.raises(_lib.HogwildError) as e:
        _lib.rope_append(ks, ks, kd, kd, [2])
    assert e.value.status == -3
    W = 70                                               # more workers than one launch takes
    ks = torch.randn((W, 2, 1, 64), device=DEV).half()
    kd = [torch.zeros((2, 3, 64), dtype=torch.float16, device=DEV) for _ in range(W)]
    vd = [torch.zeros((2, 3, 64), dtype=torch.float16, device=DEV) for _ in range(W)]
    _lib.rope_append(ks, ks, kd, vd, [w % 3 for w in range(W)])
    torch.cuda.synchronize()
    for w in range(W):
        assert torch.equal(kd[w][:, w % 3], ks[w, :, 0]) and torch.equal(vd[w][:, w % 3], ks[w, :, 0])
        assert float(kd[w].abs().sum()) == float(ks[w].abs().sum())


# ---------------------------------------------------------------------------------------------- segments in place
def test_attention_reads_segments_that_grow_in_place():
    """Fragments handed over as views into [Hkv, capacity, D] buffers give the same bits as packed copies."""
    from inference_lib_amd import attention, cases
    c = cases.small_case(dtype="bf16", W=2, S=1, Hq=8, Hkv=2, E=128, lens=(300, 70, 129), seed=3)
    cd = c.to(torch.device(DEV))
    W, Hq, S, E = cd.q.shape
    big_k = [torch.full((2, L + 37 * (i + 1), E), float("nan"), dtype=torch.bfloat16, device=DEV) for i, L in enumerate(c.lens)]
    big_v = [torch.full((2, L + 37 * (i + 1), E), float("nan"), dtype=torch.bfloat16, device=DEV) for i, L in enumerate(c.lens)]
    for i, L in enumerate(c.lens):
        big_k[i][:, :L] = cd.keys[i]
        big_v[i][:, :L] = cd.values[i]
    views_k = [b[:, :L].unsqueeze(0) for b, L in zip(big_k, c.lens)]
    views_v = [b[:, :L].unsqueeze(0) for b, L in zip(big_v, c.lens)]
    assert not views_k[0].is_contiguous()
    frag = torch.tensor(c.lens, dtype=torch.int32, device=DEV)
    outs = []
    for ks, vs in ((cd.keys, cd.values), (views_k, views_v)):
        rq = torch.empty((c.F, W, Hq, S, E), dtype=torch.bfloat16, device=DEV)
        out = torch.empty((W, Hq, S, E), dtype=torch.bfloat16, device=DEV)
        attention.hogwild_fused(cd.q, cd.locations, list(ks), list(vs), c.scale, frag, cd.cos, cd.sin, rotated_queries=rq, out=out)
        outs.append(out)
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1]) and torch.isfinite(outs[1].float()).all()


# ---------------------------------------------------------------------------------------------- the cache mirror
class NumpyMirror:
    """Plain numpy bookkeeping of the same decode loop, on top of the oracle functions."""

    def __init__(self, n_seg, layers, Hkv, D, cap):
        self.k = [[np.zeros((Hkv, cap, D)) for _ in range(layers)] for _ in range(n_seg)]
        self.v = [[np.zeros((Hkv, cap, D)) for _ in range(layers)] for _ in range(n_seg)]
        self.len = [[0] * layers for _ in range(n_seg)]


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_hogwild_cache_decode_loop_matches_oracle(dtype):
    """Three workers, a shared prompt, one private segment each, different orders; a prefill of the prompt, then decode
    steps with two layers: new keys rotated and appended (update_fused), inputs built at layer 0, attention through the
    fused operator.  Everything is compared with the oracles fed from a numpy mirror of the same state."""
    from inference_lib_amd import attention, cache
    from oracle import cache_oracle as co
    from oracle import hogwild_oracle as fo
    tdt = TDT[dtype]
    g = torch.Generator().manual_seed(17)
    layers, W, Hq, Hkv, D, cap = 2, 3, 8, 2, 64, 64
    f = inv_freq(D)
    segs = [cache.SegmentCache(layers, Hkv, D, cap, dtype=tdt, device=DEV) for _ in range(1 + W)]      # 0 = prompt
    mir = NumpyMirror(1 + W, layers, Hkv, D, cap)
    # prompt prefill through the segment's own update (keys arrive rotated)
    P = 21
    for layer in range(layers):
        pk = torch.randn((1, Hkv, P, D), generator=g).to(tdt)
        pv = torch.randn((1, Hkv, P, D), generator=g).to(tdt)
        segs[0].update(pk.to(DEV), pv.to(DEV), layer)
        mir.len[0][layer] = co.append_left_masked(mir.k[0][layer], 0, np64(pk[0]), P)
        co.append_left_masked(mir.v[0][layer], 0, np64(pv[0]), P)
    # worker w sees: prompt, the other workers' segments, its own last
    orders = [[0] + [1 + o for o in range(W) if o != w] + [1 + w] for w in range(W)]
    hc = cache.HogwildCache([[segs[i] for i in o] for o in orders], inv_freq=torch.from_numpy(f).to(DEV))
    seg_order = orders[0]                                    # fragments are listed in worker 0's order
    scale = D ** -0.5
    for step in range(3):
        S = 2 if step == 0 else 1
        mask = None
        n_new = [S] * W
        if step == 0:                                        # left-masked first step: worker 1 brings one real token
            mask = torch.tensor([[1, 1], [0, 1], [1, 1]], dtype=torch.int64, device=DEV)
            n_new = [2, 1, 2]
        kw = hc.get_input_kwargs(torch.zeros((W, S), dtype=torch.int64, device=DEV), mask)
        pos_ids = kw["position_ids"].cpu()
        want_pos = np.array([[mir.len[1 + w][0] + n_new[w] - S + s for s in range(S)] for w in range(W)])
        assert np.array_equal(pos_ids.numpy(), want_pos)
        cos_k, sin_k = tables(pos_ids, D, dtype)             # the model hands the tables out in its own dtype
        for layer in range(layers):
            q = torch.randn((W, Hq, S, D), generator=g).to(tdt)
            k_new = torch.randn((W, S, Hkv, D), generator=g).to(tdt).transpose(1, 2)
            v_new = torch.randn((W, S, Hkv, D), generator=g).to(tdt).transpose(1, 2)
            cs = hc.update_fused(k_new.to(DEV), v_new.to(DEV), cos_k.to(DEV), sin_k.to(DEV), layer, mask=mask)
            # ---- mirror: rotate + append
            for w in range(W):
                rk = co.rope_keys(np64(k_new[w]), np64(cos_k[w])[None], np64(sin_k[w])[None], storage=dtype, cs_storage=dtype, mode="eager")
                i = 1 + w
                co.append_left_masked(mir.k[i][layer], mir.len[i][layer], rk, n_new[w])
                mir.len[i][layer] = co.append_left_masked(mir.v[i][layer], mir.len[i][layer], np64(v_new[w]), n_new[w])
            lens = [mir.len[i][layer] for i in seg_order]
            # ---- what update returned
            assert cs.frags.tolist() == [mir.len[i][0] for i in seg_order]
            for fidx, i in enumerate(seg_order):
                assert tuple(cs.keys[fidx].shape) == (1, Hkv, lens[fidx], D)
                assert np.array_equal(np64(cs.keys[fidx][0]), mir.k[i][layer][:, : lens[fidx]]), (step, layer, i)
                assert np.array_equal(np64(cs.values[fidx][0]), mir.v[i][layer][:, : lens[fidx]])
            pe = co.pos_end_from_orders([[seg_order.index(i) for i in o] for o in orders], [mir.len[i][0] for i in seg_order])
            want_loc, want_cos, want_sin = co.build_inputs(pe, S, f, table_dtype=dtype)
            assert np.array_equal(cs.loc.cpu().numpy(), want_loc)
            assert np.abs(cs.cos.cpu().numpy() - want_cos).max() <= (5e-7 if dtype == "f32" else 2.0 ** -8)
            # ---- attention through the fused operator, exactly as the model's attention layer calls it
            rq = hc.get_queries_buffer(q.to(DEV), layer)
            out = attention.hogwild_fused(q.to(DEV), cs.loc, cs.keys, cs.values, scale, cs.frags, cs.cos, cs.sin,
                                          rotated_queries=rq, out=hc.get_att_buffer(rq, layer))
            torch.cuda.synchronize()
            want_out, _, _ = fo.fused_reference(np64(q), want_loc, [mir.k[i][layer][:, :L] for i, L in zip(seg_order, lens)],
                                                [mir.v[i][layer][:, :L] for i, L in zip(seg_order, lens)], scale,
                                                np64(cs.cos), np64(cs.sin), storage=dtype)
            assert_close(f"out step {step} layer {layer}", out, want_out, TOL[dtype])
    assert hc.get_seq_length() == segs[orders[0][-1]].get_seq_length()


@pytest.mark.parametrize("dtype", ["bf16", "f16", "f32"])
def test_merge_caches_rerotates_and_appends(dtype):
    from inference_lib_amd import cache
    from oracle import cache_oracle as co
    tdt = TDT[dtype]
    g = torch.Generator().manual_seed(23)
    layers, Hkv, D = 2, 2, 128
    f = inv_freq(D)
    target = cache.SegmentCache(layers, Hkv, D, 200, dtype=tdt, device=DEV)
    source = cache.SegmentCache(layers, Hkv, D, 50, dtype=tdt, device=DEV)
    tk, tv, sk, sv = [], [], [], []
    for layer in range(layers):
        for seg, n, ks_, vs_ in ((target, 77, tk, tv), (source, 31, sk, sv)):
            k = torch.randn((1, Hkv, n, D), generator=g).to(tdt)
            v = torch.randn((1, Hkv, n, D), generator=g).to(tdt)
            seg.update(k.to(DEV), v.to(DEV), layer)
            ks_.append(np64(k[0]))
            vs_.append(np64(v[0]))
    cache.merge_caches(target, source, inv_freq=torch.from_numpy(f).to(DEV))
    torch.cuda.synchronize()
    assert target.get_seq_length() == 108 and source.get_seq_length() == 31
    for layer in range(layers):
        want = co.merge_rerotate(sk[layer], 77, f, storage=dtype, mode="eager")
        got_k, got_v = np64(target.key_cache[layer][0]), np64(target.value_cache[layer][0])
        assert np.array_equal(got_k[:, :77], tk[layer]) and np.array_equal(got_v[:, :77], tv[layer])
        assert np.array_equal(got_v[:, 77:], sv[layer])
        if dtype == "f32":
            assert np.abs(got_k[:, 77:] - want).max() <= 2e-6          # device cos/sin vs the oracle's: float32 ulps
        else:
            ulp = 2.0 ** -6 if dtype == "bf16" else 2.0 ** -9
            assert np.abs(got_k[:, 77:] - want).max() <= ulp and np.mean(got_k[:, 77:] == want) > 0.99


def test_merge_caches_grows_a_target_that_is_too_small():
    """The source holds more rows than the target has room for: the target moves into larger buffers (as every other
    append does), keeps its rows, and receives the re-rotated source behind them."""
    from inference_lib_amd import cache
    from oracle import cache_oracle as co
    tdt = torch.bfloat16
    g = torch.Generator().manual_seed(29)
    layers, Hkv, D = 2, 2, 128
    f = inv_freq(D)
    target = cache.SegmentCache(layers, Hkv, D, 40, dtype=tdt, device=DEV)      # 33 of 40 rows used: room for 7
    source = cache.SegmentCache(layers, Hkv, D, 64, dtype=tdt, device=DEV)      # 50 rows to merge
    tk, tv, sk, sv = [], [], [], []
    for layer in range(layers):
        for seg, n, ks_, vs_ in ((target, 33, tk, tv), (source, 50, sk, sv)):
            k = torch.randn((1, Hkv, n, D), generator=g).to(tdt)
            v = torch.randn((1, Hkv, n, D), generator=g).to(tdt)
            seg.update(k.to(DEV), v.to(DEV), layer)
            ks_.append(np64(k[0]))
            vs_.append(np64(v[0]))
    assert target.k[0].size(1) == 40
    cache.merge_caches(target, source, inv_freq=torch.from_numpy(f).to(DEV))
    torch.cuda.synchronize()
    assert target.get_seq_length() == 83 and target.k[0].size(1) >= 83 and target.k[1].size(1) >= 83
    for layer in range(layers):
        want = co.merge_rerotate(sk[layer], 33, f, storage="bf16", mode="eager")
        got_k, got_v = np64(target.key_cache[layer][0]), np64(target.value_cache[layer][0])
        assert got_k.shape[1] == 83
        assert np.array_equal(got_k[:, :33], tk[layer]) and np.array_equal(got_v[:, :33], tv[layer])
        assert np.array_equal(got_v[:, 33:], sv[layer])
        assert np.abs(got_k[:, 33:] - want).max() <= 2.0 ** -6 and np.mean(got_k[:, 33:] == want) > 0.99


def test_segment_grows_when_full():
    """A segment that runs out of room moves into buffers of twice the size; contents and later appends are unaffected."""
    from inference_lib_amd.cache import SegmentCache
    dev = torch.device("cuda:0")
    seg = SegmentCache(2, 2, 64, 3, dtype=torch.float16, device=dev)
    g = torch.Generator().manual_seed(0)
    parts_k = [torch.randn((1, 2, n, 64), generator=g).half().to(dev) for n in (2, 2, 5, 1)]
    parts_v = [torch.randn((1, 2, n, 64), generator=g).half().to(dev) for n in (2, 2, 5, 1)]
    for pk, pv in zip(parts_k, parts_v):
        print("append", pk.size(2), "to a segment of", seg.get_seq_length(1), "capacity", seg.k[1].size(1), flush=True)
        seg.update(pk, pv, 1)
    torch.cuda.synchronize()
    assert seg.get_seq_length(1) == 10 and seg.get_seq_length(0) == 0 and seg.k[1].size(1) >= 10 and seg.k[0].size(1) == 3
    assert torch.equal(seg.key_cache[1], torch.cat(parts_k, dim=2)) and torch.equal(seg.value_cache[1], torch.cat(parts_v, dim=2))


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_decode_steps_replayed_from_one_graph_with_device_lengths(dtype):
    """The same three-worker, two-layer decode loop twice: cache A with host-side lengths, stepped eagerly (the path the
    test above checks against the oracles), and cache B with the lengths in device memory, whose step is captured in a
    HIP graph once and replayed while its segments grow.  Every step must give the same attention output (the split is
    planned for different lengths, so to tolerance, not bit for bit), and at the end the segments must hold the same
    rows bit for bit."""
    from inference_lib_amd import attention, cache
    tdt = TDT[dtype]
    g = torch.Generator().manual_seed(29)
    layers, W, Hq, Hkv, D, S = 2, 3, 8, 2, 128, 1
    f = torch.from_numpy(inv_freq(D)).to(DEV)
    scale = D ** -0.5
    P = [40, 7, 0, 19]                                                     # prompt and what the workers have written so far

    def make():
        segs = [cache.SegmentCache(layers, Hkv, D, 8, dtype=tdt, device=DEV) for _ in range(1 + W)]
        gg = torch.Generator().manual_seed(3)
        for i, n in enumerate(P):
            for layer in range(layers):
                if n:
                    segs[i].update(torch.randn((1, Hkv, n, D), generator=gg).to(tdt).to(DEV), torch.randn((1, Hkv, n, D), generator=gg).to(tdt).to(DEV), layer)
        orders = [[0] + [1 + o for o in range(W) if o != w] + [1 + w] for w in range(W)]
        return segs, cache.HogwildCache([[segs[i] for i in o] for o in orders], inv_freq=f)

    segs_a, hc_a = make()
    segs_b, hc_b = make()
    hc_b.use_device_lengths(headroom=16, new_tokens=S)
    qbuf = torch.zeros((layers, W, Hq, S, D), dtype=tdt, device=DEV)
    kbuf = torch.zeros((layers, W, S, Hkv, D), dtype=tdt, device=DEV)
    vbuf = torch.zeros((layers, W, S, Hkv, D), dtype=tdt, device=DEV)
    out_a = torch.zeros((layers, W, Hq, S, D), dtype=tdt, device=DEV)
    out_b = torch.zeros((layers, W, Hq, S, D), dtype=tdt, device=DEV)
    ids = torch.zeros((W, S), dtype=torch.int64, device=DEV)

    def step(hc, outs):
        pos = hc.get_input_kwargs(ids)["position_ids"]
        ang = pos.to(torch.float32)[..., None] * f
        emb = torch.cat([ang, ang], dim=-1)
        cos_k, sin_k = emb.cos().to(tdt), emb.sin().to(tdt)
        for layer in range(layers):
            cs = hc.update_fused(kbuf[layer].transpose(1, 2), vbuf[layer].transpose(1, 2), cos_k, sin_k, layer)
            rq = hc.get_queries_buffer(qbuf[layer], layer)
            o = attention.hogwild_fused(qbuf[layer], cs.loc, cs.keys, cs.values, scale, cs.frags, cs.cos, cs.sin, rotated_queries=rq,
                                        out=hc.get_att_buffer(rq, layer), device_lengths=hc.device_lengths)
            outs[layer].copy_(o)

    def new_inputs():
        qbuf.copy_(torch.randn(qbuf.shape, generator=g).to(tdt))
        kbuf.copy_(torch.randn(kbuf.shape, generator=g).to(tdt))
        vbuf.copy_(torch.randn(vbuf.shape, generator=g).to(tdt))

    tol = TOL[dtype]
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        new_inputs()
        step(hc_a, out_a)                       # step 0 eagerly on both (warms the capture stream up as well)
        step(hc_b, out_b)
        torch.cuda.synchronize()
        assert (out_a.float() - out_b.float()).abs().max().item() <= tol
        with torch.cuda.graph(graph, stream=stream):
            step(hc_b, out_b)
        for it in range(1, 7):
            new_inputs()
            step(hc_a, out_a)
            torch.cuda.synchronize()
            print(f"replay {it}: device lengths {hc_b._dev['len_dev'].tolist()}", flush=True)
            graph.replay()
            torch.cuda.synchronize()
            err = (out_a.float() - out_b.float()).abs().max().item()
            assert torch.isfinite(out_b.float()).all() and err <= tol, (it, err)
            (out_b.float().sum() + 1).item()    # eager work between the replays
    assert hc_b.device_steps_left() == 16 - 7
    assert hc_b.get_seq_length() == hc_a.get_seq_length()        # read from the device in this mode
    hc_b.use_host_lengths()
    for sa, sb in zip(segs_a, segs_b):
        assert sa.lengths == sb.lengths == [sa.lengths[0]] * layers
        for layer in range(layers):
            assert torch.equal(sa.key_cache[layer], sb.key_cache[layer]) and torch.equal(sa.value_cache[layer], sb.value_cache[layer])
    assert [s.get_seq_length() for s in segs_b] == [P[0]] + [p + 7 for p in P[1:]]


def test_workers_that_share_a_write_segment_append_in_worker_order():
    """Two workers writing to one segment: worker 0's tokens first, then worker 1's (the reference updates the caches
    in a loop over the workers, python/hogwild/attention.py:148-158)."""
    from inference_lib_amd import cache
    Hkv, D = 2, 64
    shared = cache.SegmentCache(1, Hkv, D, 4, dtype=torch.float16, device=DEV)
    other = cache.SegmentCache(1, Hkv, D, 4, dtype=torch.float16, device=DEV)
    hc = cache.HogwildCache([[other, shared], [other, shared], [shared, other]], inv_freq=torch.from_numpy(inv_freq(D)).to(DEV),
                            write_to=[shared, shared, other])
    g = torch.Generator().manual_seed(2)
    k = torch.randn((3, Hkv, 2, D), generator=g).half().to(DEV)
    v = torch.randn((3, Hkv, 2, D), generator=g).half().to(DEV)
    mask = torch.tensor([[1, 1], [0, 1], [1, 1]], device=DEV)
    hc.update(k, v, 0, {"mask": mask})
    torch.cuda.synchronize()
    assert shared.get_seq_length() == 3 and other.get_seq_length() == 2
    assert torch.equal(shared.key_cache[0][0], torch.cat([k[0], k[1, :, 1:]], dim=1))
    assert torch.equal(shared.value_cache[0][0], torch.cat([v[0], v[1, :, 1:]], dim=1))
    assert torch.equal(other.key_cache[0][0], k[2])
    with pytest.raises(ValueError):
        hc.use_device_lengths(8)


def test_replaying_beyond_the_planned_lengths_is_reported():
    from inference_lib_amd import _lib, cache
    Hkv, D = 2, 64
    seg = cache.SegmentCache(1, Hkv, D, 64, dtype=torch.float16, device=DEV)
    hc = cache.HogwildCache([[seg]], inv_freq=torch.from_numpy(inv_freq(D)).to(DEV))
    hc.use_device_lengths(headroom=2)
    assert hc.device_steps_left() == 2
    for _ in range(3):
        _lib.advance_lengths(hc._dev["len_dev"], hc._dev["add"])
    assert hc.device_steps_left() < 0
    with pytest.raises(RuntimeError):
        hc.sync_lengths()
