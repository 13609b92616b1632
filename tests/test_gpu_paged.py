"""GPU parity of the paged operators (hw_paged_sdpa, hw_varlen_paged_sdpa, hw_copy_to_blocks) against
oracle/paged_oracle.py, through the C ABI.  Tolerances: bf16/fp16 2e-2, fp32 1e-4 (max abs, out and lse);
copy_to_blocks is bit-exact."""
import numpy as np
import pytest
import torch

from helpers import TOL, assert_close, np64

pytestmark = pytest.mark.gpu

TDT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def build_paged(dtype, F, W, Hq, Hkv, D, bs, max_blocks, seq_lens, S=None, q_lens=None, seed=0, poison=True,
                frag_lens=None, loc_mode="causal"):
    """Synthetic paged problem on the CPU.  seq_lens[w] = tokens in sequence w.  Either S (fixed-length operator) or
    q_lens[w] (variable-length operator).  Blocks a sequence does not need are left NaN and their table entries hold
    garbage, so any read outside the visible part of a sequence shows up in the result."""
    g = torch.Generator().manual_seed(seed)
    tdt = TDT[dtype]
    NB = W * max_blocks + 5
    kc = torch.full((NB, Hkv, bs, D), float("nan") if poison else 0.0, dtype=torch.float32)
    vc = torch.full((NB, Hkv, bs, D), float("nan") if poison else 0.0, dtype=torch.float32)
    perm = torch.randperm(NB, generator=g)[: W * max_blocks].reshape(W, max_blocks).to(torch.int32)
    bt = perm.clone()
    for w in range(W):
        need = (seq_lens[w] + bs - 1) // bs
        for b in range(need):
            n_tok = min(bs, seq_lens[w] - b * bs)
            kc[perm[w, b], :, :n_tok] = torch.randn((Hkv, n_tok, D), generator=g)
            vc[perm[w, b], :, :n_tok] = torch.randn((Hkv, n_tok, D), generator=g)
        bt[w, need:] = torch.tensor([-7, 2 ** 30, NB, -1] * max_blocks, dtype=torch.int32)[: max_blocks - need]
    varlen = q_lens is not None
    if varlen:
        cu = torch.zeros(W + 1, dtype=torch.int32)
        cu[1:] = torch.cumsum(torch.tensor(q_lens), 0)
        T = int(cu[-1])
        q = torch.randn((F, T, Hq, D), generator=g)
        loc = torch.zeros((F, T), dtype=torch.int32)
        fl = torch.zeros((F, W), dtype=torch.int32)
        for w in range(W):
            a, b = int(cu[w]), int(cu[w + 1])
            for f in range(F):
                fl[f, w] = seq_lens[w] if frag_lens is None else min(frag_lens[f], seq_lens[w])
                if loc_mode == "causal":   # the last q_lens[w] positions of the sequence, shifted per fragment
                    loc[f, a:b] = torch.arange(seq_lens[w] - (b - a), seq_lens[w], dtype=torch.int32) - 3 * f
                else:
                    loc[f, a:b] = torch.randint(-2, seq_lens[w] + 3, (b - a,), generator=g, dtype=torch.int32)
    else:
        cu = None
        q = torch.randn((F, W, Hq, S, D), generator=g)
        loc = torch.zeros((F, W, S), dtype=torch.int32)
        # a fragment length applies to all workers: it may not exceed the shortest sequence (longer would be unwritten cache)
        fl = torch.tensor([min(seq_lens) if frag_lens is None else min(frag_lens[f], min(seq_lens)) for f in range(F)], dtype=torch.int32)
        if frag_lens is None and F == 1:
            fl[0] = max(seq_lens)          # visibility is then bounded by the locations alone
        for w in range(W):
            for f in range(F):
                if loc_mode == "causal":
                    loc[f, w] = torch.arange(seq_lens[w] - S, seq_lens[w], dtype=torch.int32) - 3 * f
                else:
                    loc[f, w] = torch.randint(-2, seq_lens[w], (S,), generator=g, dtype=torch.int32)
    q = q.to(tdt)
    kc = kc.to(tdt)
    vc = vc.to(tdt)
    return dict(q=q, loc=loc, fl=fl, kc=kc, vc=vc, bt=bt, cu=cu, scale=1.0 / D ** 0.5, dtype=dtype, F=F, W=W, Hq=Hq,
                Hkv=Hkv, D=D, S=S)


def oracle_paged(c):
    from oracle import paged_oracle as po
    kc = np.nan_to_num(np64(c["kc"]), nan=1e30)      # poisoned rows are never visible; keep the oracle's einsum finite
    vc = np.nan_to_num(np64(c["vc"]), nan=1e30)
    bt = np.clip(c["bt"].numpy(), 0, kc.shape[0] - 1)
    if c["cu"] is None:
        return po.paged_sdpa(np64(c["q"]), c["loc"].numpy(), c["fl"].numpy(), kc, vc, bt, c["scale"])
    return po.varlen_paged_sdpa(np64(c["q"]), c["loc"].numpy(), c["fl"].numpy(), kc, vc, bt, c["cu"].numpy(), c["scale"])


def run_paged(c, splits=0, row_blocks=0, with_lse=True):
    from inference_lib_amd import _lib
    dev = torch.device("cuda:0")
    d = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in c.items()}
    if c["cu"] is None:
        out = torch.full((c["W"], c["Hq"], c["S"], c["D"]), float("nan"), dtype=d["q"].dtype, device=dev)
    else:
        out = torch.full((d["q"].size(1), c["Hq"], c["D"]), float("nan"), dtype=d["q"].dtype, device=dev)
    lse = torch.full(out.shape[:-1], float("nan"), dtype=torch.float32, device=dev) if with_lse else None
    pr = _lib.PagedProblem(q=d["q"], locations=d["loc"], fragment_lengths=d["fl"], key_cache=d["kc"], value_cache=d["vc"],
                           block_table=d["bt"], scale=c["scale"], out=out, cu_seqlens_q=d["cu"], lse=lse, splits=splits,
                           row_blocks=row_blocks)
    print(f"paged run: dtype={c['dtype']} F={c['F']} W={c['W']} Hq={c['Hq']} Hkv={c['Hkv']} D={c['D']} S={c['S']} "
          f"bs={c['kc'].size(2)} mb={c['bt'].size(1)} varlen={c['cu'] is not None} splits={splits} rb={row_blocks}", flush=True)
    pr.run()
    torch.cuda.synchronize()
    return out, lse


def check(c, **kw):
    want_o, want_l = oracle_paged(c)
    out, lse = run_paged(c, **kw)
    tol = TOL[c["dtype"]]
    assert_close("out", out, want_o, tol)
    assert_close("lse", lse, want_l, tol)
    return out, lse


@pytest.mark.parametrize("dtype", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("bs,S,F", [(16, 1, 1), (32, 1, 1), (8, 3, 2), (1, 2, 1), (24, 1, 2), (128, 4, 1)])
def test_paged_small(dtype, D, bs, S, F):
    mb = max(1, 300 // bs)
    c = build_paged(dtype, F, 3, 10, 2, D, bs, mb, seq_lens=[200, 37, 1 + S + 3 * F], S=S, seed=bs + S)
    check(c)


def test_paged_random_locations_and_fragment_lengths():
    c = build_paged("bf16", 3, 4, 8, 2, 128, 16, 40, seq_lens=[600, 64, 333, 17], S=2, seed=5, frag_lens=[9, 17, 16], loc_mode="random")
    check(c)


@pytest.mark.parametrize("splits", [1, 3, 16])
@pytest.mark.parametrize("row_blocks", [1, 2])
def test_paged_split_and_row_block_invariance(splits, row_blocks):
    c = build_paged("bf16", 1, 2, 8, 2, 128, 16, 80, seq_lens=[1000, 129], S=6, seed=11)
    check(c, splits=splits, row_blocks=row_blocks)


def test_paged_qwq_shape_decode():
    """The headline model shape as a paged decode step: 4 workers with their own 3-4k-token sequences."""
    c = build_paged("bf16", 1, 4, 40, 8, 128, 16, 256, seq_lens=[4096, 3001, 3500, 2048], S=1, seed=3)
    out, lse = check(c)
    out2, lse2 = run_paged(c)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)     # deterministic


def test_paged_gqa16_and_wide_rows():
    c = build_paged("f16", 1, 2, 32, 2, 128, 32, 20, seq_lens=[500, 77], S=5, seed=9)     # 80 rows per worker
    check(c)


@pytest.mark.parametrize("dtype,D,bs,S,F,splits", [
    ("bf16", 128, 16, 7, 1, 0),      # 112 rows per sequence: chosen automatically
    ("f16", 128, 24, 9, 2, 3),       # blocks of 24 positions: a tile touches three blocks; two fragments
    ("bf16", 64, 128, 3, 1, 1),      # forced with few rows (48), one split
    ("f16", 64, 17, 20, 1, 7),       # 320 rows: three row groups, the last partly filled; odd block size
])
def test_paged_wide_rows(dtype, D, bs, S, F, splits):
    """The 128-row workgroups of the paged operators (row_blocks = 8) against the oracle."""
    c = build_paged(dtype, F, 3, 32, 2, D, bs, (700 + bs - 1) // bs + 1, seq_lens=[700, 131, 64], S=S, seed=31 + bs)
    check(c, splits=splits, row_blocks=8)
    c = build_paged(dtype, F, 2, 32, 2, D, bs, (300 + bs - 1) // bs + 1, seq_lens=[300, 290], S=S, seed=5, loc_mode="random")
    check(c, splits=splits, row_blocks=8)


def test_varlen_wide_rows():
    """Packed variable-length queries with many tokens per sequence: 5 .. 1000 rows per kv head and sequence, empty and
    one-token sequences in between, sequences shorter than a tile."""
    c = build_paged("bf16", 1, 6, 10, 2, 128, 16, 60, seq_lens=[900, 50, 9, 430, 64, 777], q_lens=[200, 0, 9, 64, 1, 33], seed=77)
    check(c)                              # the split decided on the device
    check(c, row_blocks=8, splits=5)
    check(c, row_blocks=2)                # and the narrow kernel agrees with the same oracle
    c = build_paged("f16", 2, 3, 8, 2, 64, 32, 20, seq_lens=[600, 31, 222], q_lens=[100, 31, 64], seed=3, loc_mode="random")
    check(c, row_blocks=8)


def test_varlen_split_decided_on_the_device():
    """Packed queries in 128-row workgroups (16-bit types, more than 16 rows per sequence on average, at most 256 sequences
    and possible row groups): every workgroup works out from cu_seqlens_q and the fragment lengths which row group of
    which sequence it serves and which share of that sequence's tiles.  Sequences of very different KV lengths and query
    counts, empty ones, groups of exactly 64 / 65 / 128 / 129 rows (one or two 16-row blocks per wave, one or two
    groups), more sequences than a wave has lanes, against the oracle."""
    from inference_lib_amd import _lib
    c = build_paged("bf16", 2, 6, 10, 2, 128, 16, 200, seq_lens=[3000, 40, 700, 64, 1500, 9], q_lens=[64, 1, 0, 30, 7, 9], seed=41)
    pl = _lib.paged_plan(W=6, Hq=10, Hkv=2, Ev=128, block_size=16, max_blocks=200, num_cus=_lib.lib.hw_device_cus(), total_q=111)
    assert pl.device_planned == 1 and pl.row_blocks == 8
    check(c)
    c = build_paged("f16", 1, 4, 2, 2, 64, 32, 40, seq_lens=[1000, 1200, 300, 1280], q_lens=[64, 65, 128, 129], seed=42, loc_mode="random")
    check(c)
    rng = np.random.default_rng(12)
    W = 200
    seq = [int(x) for x in rng.integers(9, 400, size=W)]
    ql = [int(min(s, x)) for s, x in zip(seq, rng.integers(2, 10, size=W))]
    ql[17] = 0
    c = build_paged("bf16", 1, W, 8, 2, 64, 16, 25, seq_lens=seq, q_lens=ql, seed=43)
    pl = _lib.paged_plan(W=W, Hq=8, Hkv=2, Ev=64, block_size=16, max_blocks=25, num_cus=_lib.lib.hw_device_cus(), total_q=sum(ql))
    assert pl.device_planned == 1
    check(c)
    # one long prompt among one-token sequences: the long one gets most of the workgroups
    seq = [6000] + [int(x) for x in rng.integers(20, 300, size=30)]
    c = build_paged("bf16", 1, 31, 10, 2, 128, 16, 380, seq_lens=seq, q_lens=[120] + [1] * 30, seed=44)
    check(c)


def test_varlen_mixed_1_8_32_64_query_tokens():
    """The shape of the packed-query benchmark at a size the oracle finishes: four sequences with 1 / 8 / 32 / 64 query
    tokens at the QwQ-32B head shape (5 / 40 / 160 / 320 rows per kv head: row groups of 5, 40, 128 + 32 and 128 + 128 + 64
    rows), planned on the device, against the oracle; and the launches with a fixed split agree with the same oracle."""
    c = build_paged("bf16", 1, 4, 40, 8, 128, 16, 100, seq_lens=[1500, 1100, 1300, 1600], q_lens=[1, 8, 32, 64], seed=61)
    check(c)
    check(c, row_blocks=8, splits=3)
    check(c, row_blocks=2)


def test_paged_decode_full_size_of_the_benchmark():
    """The paged decode benchmark workload at its full size (four sequences of 12 528 tokens, one query token each)."""
    c = build_paged("bf16", 1, 4, 40, 8, 128, 16, 784, seq_lens=[12528] * 4, S=1, seed=63)
    check(c)


def test_varlen_full_size_of_the_benchmark():
    """The packed-query benchmark workload at its full size (four sequences of 12 528 tokens with 1 / 8 / 32 / 64 query
    tokens, QwQ-32B head shape, blocks of 16): the launch planned on the device against the oracle, and the 32-row kernel
    (another kernel, another split, another order of summation) against the same oracle."""
    c = build_paged("bf16", 1, 4, 40, 8, 128, 16, 784, seq_lens=[12528] * 4, q_lens=[1, 8, 32, 64], seed=62)
    check(c)
    check(c, row_blocks=2)


def test_varlen_tokens_behind_the_last_sequence_give_zeros():
    """total_q may exceed cu_seqlens_q[-1]: the tokens behind the last sequence belong to none.  The device-planned launch
    gives them zeros (lse -inf); the other launches leave them unspecified, like the reference, but must get the tokens of
    the sequences right all the same."""
    c = build_paged("bf16", 1, 3, 10, 2, 128, 16, 40, seq_lens=[500, 300, 77], q_lens=[40, 9, 33], seed=51)
    want_o, want_l = oracle_paged(c)
    pad = 7
    c2 = dict(c)
    c2["q"] = torch.cat([c["q"], torch.randn((1, pad, 10, 128)).to(c["q"].dtype)], dim=1)
    c2["loc"] = torch.cat([c["loc"], torch.full((1, pad), 5, dtype=torch.int32)], dim=1)
    for kw in (dict(), dict(row_blocks=2), dict(row_blocks=8, splits=3)):
        out, lse = run_paged(c2, **kw)
        assert_close("out", out[:-pad], want_o, TOL["bf16"])
        assert_close("lse", lse[:-pad], want_l, TOL["bf16"])
        if not kw:
            assert (out[-pad:] == 0).all() and torch.isneginf(lse[-pad:]).all()


def test_paged_wide_small_blocks_and_fallbacks():
    """Any block size works in the 128-row workgroups (the table is looked up per position); fp32 and block tables that do
    not fit into LDS (more than 8192 entries per sequence) have no such kernel: the request is ignored, never a wrong launch."""
    c = build_paged("bf16", 1, 2, 32, 2, 128, 8, 40, seq_lens=[300, 200], S=6, seed=2)
    check(c, row_blocks=8)
    c = build_paged("f16", 2, 2, 16, 2, 64, 1, 150, seq_lens=[150, 77], S=9, seed=4)
    check(c, row_blocks=8)
    c = build_paged("f32", 1, 2, 32, 2, 64, 16, 20, seq_lens=[300, 200], S=6, seed=2)
    check(c, row_blocks=8)
    c = build_paged("bf16", 1, 1, 32, 2, 64, 1, 8200, seq_lens=[8195], S=6, seed=6, poison=False)
    check(c, row_blocks=8)


def test_paged_nothing_visible():
    c = build_paged("bf16", 1, 2, 4, 2, 64, 16, 4, seq_lens=[20, 20], S=1, seed=1)
    c["loc"][:, 0] = -1
    out, lse = check(c)
    assert (out[0] == 0).all() and torch.isneginf(lse[0]).all()


@pytest.mark.parametrize("dtype,D", [("bf16", 128), ("f32", 64), ("f16", 64)])
def test_varlen_ragged(dtype, D):
    c = build_paged(dtype, 2, 5, 10, 2, D, 16, 30, seq_lens=[400, 50, 9, 130, 64], q_lens=[3, 0, 9, 40, 1], seed=21)
    check(c)


def test_varlen_many_sequences():
    W = 150     # more than one 64-wide chunk of the sequence lookup
    rng = np.random.default_rng(4)
    seq = [int(x) for x in rng.integers(5, 90, size=W)]
    ql = [int(min(s, x)) for s, x in zip(seq, rng.integers(0, 4, size=W))]
    c = build_paged("bf16", 1, W, 4, 2, 64, 16, 6, seq_lens=seq, q_lens=ql, seed=8, loc_mode="random")
    check(c)


def test_varlen_equals_fixed_when_lengths_are_equal():
    c = build_paged("bf16", 1, 3, 8, 2, 128, 16, 20, seq_lens=[300, 200, 100], S=4, seed=2)
    out, lse = run_paged(c)
    v = dict(c)
    v["q"] = c["q"].permute(0, 1, 3, 2, 4).reshape(1, 12, 8, 128).contiguous()
    v["loc"] = c["loc"].reshape(1, 12).contiguous()
    v["fl"] = c["fl"][:, None].repeat(1, 3).contiguous()
    v["cu"] = torch.arange(4, dtype=torch.int32) * 4
    vo, vl = run_paged(v)
    assert torch.equal(vo, out.permute(0, 2, 1, 3).reshape(12, 8, 128))
    assert torch.equal(vl, lse.permute(0, 2, 1).reshape(12, 8))


# --------------------------------------------------------------------------------------------------- copy_to_blocks
@pytest.mark.parametrize("dtype", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("E,Ev,S_new,bs", [(128, 128, 1, 16), (64, 64, 37, 16), (128, 64, 5, 1), (6, 10, 3, 4), (128, 128, 9, 24)])
def test_copy_to_blocks_bit_exact(dtype, E, Ev, S_new, bs):
    from inference_lib_amd import _lib
    from oracle import paged_oracle as po
    g = torch.Generator().manual_seed(S_new + bs)
    tdt = TDT[dtype]
    B, Hkv, mb = 3, 2, (60 + S_new) // bs + 2
    NB = B * mb + 2
    kc = torch.randn((NB, Hkv, bs, E), generator=g).to(tdt)
    vc = torch.randn((NB, Hkv, bs, Ev), generator=g).to(tdt)
    bt = torch.randperm(NB, generator=g)[: B * mb].reshape(B, mb).to(torch.int32)
    seq = torch.tensor([0, 17, 60], dtype=torch.int32)
    # the usual layout of fresh projections: [B, S_new, Hkv, D], viewed as [B, Hkv, S_new, D]
    ks = torch.randn((B, S_new, Hkv, E), generator=g).to(tdt).transpose(1, 2)
    vs = torch.randn((B, S_new, Hkv, Ev), generator=g).to(tdt).transpose(1, 2)
    want_k, want_v = np64(kc), np64(vc)
    po.copy_to_blocks(np64(ks), np64(vs), want_k, want_v, bt.numpy(), seq.numpy())
    dev = torch.device("cuda:0")
    dk, dv = kc.to(dev), vc.to(dev)
    print(f"copy_to_blocks: {dtype} E={E} Ev={Ev} S_new={S_new} bs={bs}", flush=True)
    _lib.copy_to_blocks(ks.to(dev), vs.to(dev), dk, dv, bt.to(dev), seq.to(dev))
    torch.cuda.synchronize()
    assert np.array_equal(np64(dk), want_k) and np.array_equal(np64(dv), want_v)


def test_copy_to_blocks_skips_positions_outside_the_table():
    from inference_lib_amd import _lib
    dev = torch.device("cuda:0")
    kc = torch.zeros((4, 1, 4, 8), dtype=torch.float16, device=dev)
    vc = torch.zeros((4, 1, 4, 8), dtype=torch.float16, device=dev)
    bt = torch.tensor([[2, 9]], dtype=torch.int32, device=dev)        # second entry lies outside the cache
    seq = torch.tensor([2], dtype=torch.int32, device=dev)
    ks = torch.ones((1, 1, 9, 8), dtype=torch.float16, device=dev)    # positions 2..10: 2,3 land; 4..7 bad block; 8.. off the table
    _lib.copy_to_blocks(ks, ks, kc, vc, bt, seq)
    torch.cuda.synchronize()
    assert float(kc.sum()) == 2 * 8 and float(kc[2, 0, 2:].sum()) == 16 and float(vc.sum()) == 16


def test_append_then_attend_round_trip():
    """Decode loop in miniature: append one token per sequence with copy_to_blocks, then attend over the grown cache."""
    from inference_lib_amd import _lib
    from oracle import paged_oracle as po
    dev = torch.device("cuda:0")
    c = build_paged("bf16", 1, 3, 8, 2, 128, 16, 10, seq_lens=[100, 31, 64], S=1, seed=13, poison=False)
    g = torch.Generator().manual_seed(99)
    ks = torch.randn((3, 2, 1, 128), generator=g).to(torch.bfloat16)
    vs = torch.randn((3, 2, 1, 128), generator=g).to(torch.bfloat16)
    seq = torch.tensor([100, 31, 64], dtype=torch.int32)
    bt = c["bt"].clone()
    # give every sequence a valid block for its position seq_len (the builder left garbage beyond the used blocks)
    used = set(int(x) for w in range(3) for x in bt[w, : (seq[w] + 15) // 16])
    free = [b for b in range(c["kc"].size(0)) if b not in used]
    for w in range(3):
        if int(seq[w]) % 16 == 0:
            bt[w, int(seq[w]) // 16] = free.pop()
    c["bt"] = bt
    want_k, want_v = np64(c["kc"]), np64(c["vc"])
    po.copy_to_blocks(np64(ks), np64(vs), want_k, want_v, bt.numpy(), seq.numpy())
    c["loc"] = seq.reshape(1, 3, 1).clone()
    c["fl"] = torch.tensor([200], dtype=torch.int32)
    want_o, want_l = po.paged_sdpa(np64(c["q"]), c["loc"].numpy(), c["fl"].numpy(), want_k, want_v, bt.numpy(), c["scale"])
    d = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in c.items()}
    _lib.copy_to_blocks(ks.to(dev), vs.to(dev), d["kc"], d["vc"], d["bt"], seq.to(dev))
    out = torch.empty((3, 8, 1, 128), dtype=torch.bfloat16, device=dev)
    lse = torch.empty((3, 8, 1), dtype=torch.float32, device=dev)
    _lib.PagedProblem(q=d["q"], locations=d["loc"], fragment_lengths=d["fl"], key_cache=d["kc"], value_cache=d["vc"],
                      block_table=d["bt"], scale=c["scale"], out=out, lse=lse).run()
    torch.cuda.synchronize()
    assert_close("out", out, want_o, 2e-2)
    assert_close("lse", lse, want_l, 2e-2)


# --------------------------------------------------------------------------------------------------- torch operators
def test_paged_torch_ops_match_c_abi_and_raise_loudly():
    from inference_lib_amd import attention
    assert attention.HAVE_TORCH_OPS, "hogatt.abi3.so not built"
    for name in ("hogwild_paged_sdpa", "copy_to_blocks", "hogwild_varlen_paged_sdpa"):
        assert hasattr(torch.ops.libhogatt, name)
    dev = torch.device("cuda:0")
    c = build_paged("bf16", 2, 3, 10, 2, 128, 16, 12, seq_lens=[150, 40, 99], S=2, seed=31)
    want_o, _ = oracle_paged(c)
    d = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in c.items()}
    out = attention.hogwild_paged_sdpa(d["q"], d["loc"], d["fl"], d["kc"], d["vc"], d["bt"], c["scale"])
    torch.cuda.synchronize()
    assert_close("paged op", out, want_o, 2e-2)
    ref, _ = run_paged(c)
    assert torch.equal(out, ref)

    v = build_paged("f16", 1, 4, 8, 2, 64, 16, 12, seq_lens=[150, 40, 99, 12], q_lens=[5, 0, 2, 12], seed=32)
    want_o, _ = oracle_paged(v)
    dv = {k: (t.to(dev) if torch.is_tensor(t) else t) for k, t in v.items()}
    out = attention.hogwild_varlen_paged_sdpa(dv["q"], dv["loc"], dv["fl"], dv["kc"], dv["vc"], dv["bt"], dv["cu"], None, v["scale"])
    torch.cuda.synchronize()
    assert_close("varlen op", out, want_o, 2e-2)

    # copy_to_blocks through the operator, with the transposed view a projection produces
    kc, vc = d["kc"].clone(), d["vc"].clone()
    ks = torch.randn((3, 4, 2, 128), device=dev).to(torch.bfloat16).transpose(1, 2)
    seq = torch.tensor([150, 40, 99], dtype=torch.int32, device=dev)
    bt = d["bt"].clone()
    bt[:, 9] = torch.tensor([0, 1, 2], dtype=torch.int32, device=dev)
    attention.copy_to_blocks(ks, ks, kc, vc, bt, seq)
    kc2, vc2 = d["kc"].clone(), d["vc"].clone()
    from inference_lib_amd import _lib
    _lib.copy_to_blocks(ks, ks, kc2, vc2, bt, seq)
    torch.cuda.synchronize()
    assert torch.equal(kc.view(torch.int16), kc2.view(torch.int16)) and torch.equal(vc.view(torch.int16), vc2.view(torch.int16))

    # unsupported head dimension and mismatched dtypes are errors, never silent no-ops
    bad_kc = torch.zeros((4, 2, 16, 96), dtype=torch.bfloat16, device=dev)
    bad_q = torch.zeros((1, 1, 4, 1, 96), dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="no kernel instantiated"):
        attention.hogwild_paged_sdpa(bad_q, torch.zeros((1, 1, 1), dtype=torch.int32, device=dev),
                                     torch.ones(1, dtype=torch.int32, device=dev), bad_kc, bad_kc,
                                     torch.zeros((1, 2), dtype=torch.int32, device=dev), 1.0)
    with pytest.raises(RuntimeError, match="dtype"):
        torch.ops.libhogatt.hogwild_paged_sdpa(out.new_zeros((3, 10, 2, 128)), 1.0, d["loc"], d["q"].float(), d["fl"], d["kc"], d["vc"], d["bt"])


def test_paged_cache_larger_than_4_gib():
    """Caches of 5 GiB each: cache rows beyond the first 4 GiB are reached only if the row address is formed in 64 bits,
    in the attention kernel and in copy_to_blocks alike.  Closed form instead of the oracle: all keys of the sequence
    are zero except the newest, appended through copy_to_blocks into the block with the highest id and a large multiple
    of the query, so the output must be exactly that token's value row."""
    from inference_lib_amd import _lib
    dev = torch.device("cuda:0")
    Hkv, bs, D = 2, 16, 128
    NB = (5 << 30) // (Hkv * bs * D * 2)              # blocks in a 5 GiB bf16 cache
    kc = torch.zeros((NB, Hkv, bs, D), dtype=torch.bfloat16, device=dev)
    vc = torch.zeros((NB, Hkv, bs, D), dtype=torch.bfloat16, device=dev)
    L = 100                                            # tokens before the append: blocks 0..6 of the table
    bt = torch.tensor([[NB - 2, 5, NB // 2, NB - 7, 11, NB - 3, NB - 1, NB - 4]], dtype=torch.int32, device=dev)
    g = torch.Generator().manual_seed(23)
    for b in bt[0, :7].tolist():                       # random values in the blocks the sequence already occupies
        vc[b] = torch.randn((Hkv, bs, D), generator=g).to(torch.bfloat16).to(dev)
    q = torch.randn((1, 1, 4, 1, D), generator=g).to(torch.bfloat16).to(dev)            # [F, W, Hq, S, D], GQA 2
    k_new = torch.stack([4.0 * q[0, 0, 0, 0].float(), 4.0 * q[0, 0, 2, 0].float()])[None, :, None, :].to(torch.bfloat16)   # [1, Hkv, 1, D]
    v_new = torch.randn((1, Hkv, 1, D), generator=g).to(torch.bfloat16).to(dev)
    seq = torch.tensor([L], dtype=torch.int32, device=dev)
    print(f"copy_to_blocks into block {NB - 1} of {NB}", flush=True)
    _lib.copy_to_blocks(k_new, v_new, kc, vc, bt, seq)                                   # position 100 = row 4 of table entry 6 = block NB-1
    torch.cuda.synchronize()
    assert torch.equal(kc[NB - 1, :, 4], k_new[0, :, 0]) and torch.equal(vc[NB - 1, :, 4], v_new[0, :, 0])
    assert int((kc != 0).any(dim=-1).sum()) == Hkv                                       # nothing else was written
    out = torch.full((1, 4, 1, D), float("nan"), dtype=torch.bfloat16, device=dev)
    lse = torch.empty((1, 4, 1), dtype=torch.float32, device=dev)
    loc = torch.tensor([[[L]]], dtype=torch.int32, device=dev)
    fl = torch.tensor([L + 1], dtype=torch.int32, device=dev)
    print("paged attention over blocks on both sides of the 4 GiB line", flush=True)
    _lib.PagedProblem(q=q, locations=loc, fragment_lengths=fl, key_cache=kc, value_cache=vc, block_table=bt, scale=D ** -0.5,
                      out=out, lse=lse).run()
    torch.cuda.synchronize()
    for h in (0, 2):                                   # the heads whose query the new key is a multiple of
        assert torch.equal(out[0, h, 0], v_new[0, h // 2, 0])
    # and a second token, in the middle of the sequence (table entry 3 = block NB-7, beyond 4 GiB as well)
    kc[NB - 1, :, 4] = 0
    kc[NB - 7, 1, 9] = k_new[0, 1, 0]                  # position 3 * 16 + 9 = 57, kv head 1
    _lib.PagedProblem(q=q, locations=loc, fragment_lengths=fl, key_cache=kc, value_cache=vc, block_table=bt, scale=D ** -0.5,
                      out=out, lse=lse).run()
    torch.cuda.synchronize()
    assert torch.equal(out[0, 2, 0], vc[NB - 7, 1, 9])


def test_paged_decode_steps_replayed_from_one_graph():
    """A whole paged decode step (append the new token with copy_to_blocks, advance the sequence lengths, attend) is
    captured once and replayed while the sequences grow: lengths, locations and block tables live in device memory, the
    library allocates nothing and records no memset.  Every replay is checked against the oracle on the state it saw,
    with eager work and synchronisations between the replays."""
    from inference_lib_amd import _lib
    from oracle import paged_oracle as po
    dev = torch.device("cuda:0")
    W, Hq, Hkv, D, bs, mb = 3, 8, 2, 128, 16, 12
    seq0 = [37, 150, 16]
    c = build_paged("bf16", 1, W, Hq, Hkv, D, bs, mb, seq_lens=seq0, S=1, seed=41, poison=False)
    kc, vc, bt = c["kc"].to(dev), c["vc"].to(dev), c["bt"].to(dev)
    for w in range(W):      # every table entry a sequence can grow into must be a real block
        bt[w] = torch.arange(w * mb, (w + 1) * mb, dtype=torch.int32, device=dev)
    for w in range(W):
        for p in range(seq0[w]):
            kc[bt[w, p // bs], :, p % bs] = torch.randn((Hkv, D), generator=torch.Generator().manual_seed(1000 * w + p)).to(torch.bfloat16).to(dev)
            vc[bt[w, p // bs], :, p % bs] = torch.randn((Hkv, D), generator=torch.Generator().manual_seed(5000 + 1000 * w + p)).to(torch.bfloat16).to(dev)
    seq = torch.tensor(seq0, dtype=torch.int32, device=dev)
    loc = torch.zeros((1, W, 1), dtype=torch.int32, device=dev)
    fl = torch.tensor([bs * mb], dtype=torch.int32, device=dev)        # visibility is bounded by the locations alone
    q = torch.zeros((1, W, Hq, 1, D), dtype=torch.bfloat16, device=dev)
    k_new = torch.zeros((W, Hkv, 1, D), dtype=torch.bfloat16, device=dev)
    v_new = torch.zeros((W, Hkv, 1, D), dtype=torch.bfloat16, device=dev)
    out = torch.empty((W, Hq, 1, D), dtype=torch.bfloat16, device=dev)
    lse = torch.empty((W, Hq, 1), dtype=torch.float32, device=dev)
    pr = _lib.PagedProblem(q=q, locations=loc, fragment_lengths=fl, key_cache=kc, value_cache=vc, block_table=bt, scale=c["scale"],
                           out=out, lse=lse)
    pr.set_workspace()

    def step():
        _lib.copy_to_blocks(k_new, v_new, kc, vc, bt, seq)      # position seq[w] of every sequence
        loc.copy_(seq.view(1, W, 1))                             # the new token sits at the old length ...
        seq.add_(1)                                              # ... and the sequence is one longer
        pr.run()

    stream = torch.cuda.Stream()
    g = torch.Generator().manual_seed(7)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        step()                                                   # warm-up (also a real step)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            step()
        seq.copy_(torch.tensor(seq0, dtype=torch.int32))         # capture does not execute; start over from the initial state
        for it in range(6):
            q.copy_(torch.randn(q.shape, generator=g).to(torch.bfloat16))
            k_new.copy_(torch.randn(k_new.shape, generator=g).to(torch.bfloat16))
            v_new.copy_(torch.randn(v_new.shape, generator=g).to(torch.bfloat16))
            torch.cuda.synchronize()
            print(f"replay {it}: sequence lengths {seq.tolist()}", flush=True)
            graph.replay()
            torch.cuda.synchronize()
            assert seq.tolist() == [s + it + 1 for s in seq0]
            want_o, want_l = po.paged_sdpa(np64(q), loc.cpu().numpy(), fl.cpu().numpy(), np64(kc), np64(vc), bt.cpu().numpy(), c["scale"])
            assert_close("out", out, want_o, TOL["bf16"])
            assert_close("lse", lse, want_l, TOL["bf16"])
            for w in range(W):                                   # the appended rows are where the next step expects them
                p = seq0[w] + it
                assert torch.equal(kc[bt[w, p // bs], :, p % bs], k_new[w, :, 0])
            (out.float().sum() + 1).item()                       # eager work between the replays
