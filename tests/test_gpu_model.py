"""End-to-end: a small randomly initialised Qwen2 decoder from the model library with its attention layers swapped for
AttentionModule, driven through HogwildCache and the fused operator, against the same model's own eager forward pass.

What the equalities rest on:
  * one worker, structure [prompt, own segment]: the worker's view is an ordinary causal sequence, so every logit must
    equal the plain model's at the same position (any number of layers);
  * two workers that read each other's segments: worker w's view is the sequence [prompt, the other's tokens, its own
    tokens].  With ONE decoder layer the keys and values of a token do not depend on its context, so the logits of
    worker w's newest token equal the plain model's last-position logits on that sequence; the keys were rotated for
    their positions inside their own segment and only the per-fragment query rotation makes the relative distances
    come out right.
Tolerances on the logits: fp32 5e-5 (observed 1e-6), bf16 3e-2 (observed 8e-3: two different bf16 pipelines)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

transformers = pytest.importorskip("transformers")

DEV = "cuda:0"


def tiny_model(layers, dtype, seed=0, hidden=256, heads=4, kv=2, vocab=101):
    from transformers import Qwen2Config, Qwen2ForCausalLM
    cfg = Qwen2Config(vocab_size=vocab, hidden_size=hidden, intermediate_size=2 * hidden, num_hidden_layers=layers,
                      num_attention_heads=heads, num_key_value_heads=kv, max_position_embeddings=1024, attn_implementation="eager")
    torch.manual_seed(seed)
    model = Qwen2ForCausalLM(cfg).eval().to(dtype).to(DEV)
    return cfg, model


def swapped_copy(model):
    import copy
    from inference_lib_amd.model import model_surgery
    m = copy.deepcopy(model)
    model_surgery(m)
    return m


def segment(cfg, capacity, dtype):
    from inference_lib_amd.cache import SegmentCache
    return SegmentCache(cfg.num_hidden_layers, cfg.num_key_value_heads, cfg.hidden_size // cfg.num_attention_heads, capacity,
                        dtype=dtype, device=DEV)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 5e-5), (torch.bfloat16, 3e-2)])
def test_single_worker_decode_matches_the_plain_causal_model(dtype, tol):
    from inference_lib_amd.cache import HogwildCache
    from inference_lib_amd.model import decode_step
    cfg, plain = tiny_model(2, dtype, seed=1)
    hog = swapped_copy(plain)
    T, N = 37, 9
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, cfg.vocab_size, (1, T + N), generator=g).to(DEV)
    with torch.no_grad():
        want = plain(ids).logits.float()
    prompt, seg = segment(cfg, 16, dtype), segment(cfg, 2, dtype)        # both too small: they grow on the way
    print(f"prefill of {T} tokens through the fused operator, {dtype}", flush=True)
    got = decode_step(hog, HogwildCache([[prompt]], hog), ids[:, :T]).float()
    assert prompt.get_seq_length() == T
    err = (got - want[:, :T]).abs().max().item()
    print(f"  prefill max err {err:.3e}", flush=True)
    assert err <= tol
    cache = HogwildCache([[prompt, seg]], hog)
    for i in range(0, N, 3):         # three tokens per step
        print(f"decode tokens {T + i}..{T + i + 2}", flush=True)
        got = decode_step(hog, cache, ids[:, T + i: T + i + 3]).float()
        err = (got - want[:, T + i: T + i + 3]).abs().max().item()
        print(f"  max err {err:.3e}", flush=True)
        assert err <= tol
    assert seg.get_seq_length() == N and prompt.get_seq_length() == T
    assert prompt.k[0].size(1) >= T and seg.k[1].size(1) >= N


def test_two_workers_reading_each_others_segments_one_layer():
    from inference_lib_amd.cache import HogwildCache
    from inference_lib_amd.model import decode_step
    dtype, tol = torch.float32, 5e-5
    cfg, plain = tiny_model(1, dtype, seed=2, hidden=512, heads=4, kv=1)      # head_dim 128, GQA 4
    hog = swapped_copy(plain)
    T, N = 21, 6
    g = torch.Generator().manual_seed(9)
    p_ids = torch.randint(0, cfg.vocab_size, (1, T), generator=g).to(DEV)
    w_ids = torch.randint(0, cfg.vocab_size, (2, N), generator=g).to(DEV)     # what the two workers write, step by step
    prompt, sa, sb = segment(cfg, 32, dtype), segment(cfg, 16, dtype), segment(cfg, 16, dtype)
    decode_step(hog, HogwildCache([[prompt]], hog), p_ids)
    cache = HogwildCache([[prompt, sb, sa], [prompt, sa, sb]], hog)          # worker 0 writes to sa, worker 1 to sb
    for t in range(N):
        print(f"step {t}", flush=True)
        got = decode_step(hog, cache, w_ids[:, t: t + 1]).float()             # [2, 1, vocab]
        views = [torch.cat([p_ids[0], w_ids[1, : t + 1], w_ids[0, : t + 1]]), torch.cat([p_ids[0], w_ids[0, : t + 1], w_ids[1, : t + 1]])]
        for w in range(2):
            with torch.no_grad():
                want = plain(views[w][None]).logits[0, -1].float()
            err = (got[w, 0] - want).abs().max().item()
            print(f"  worker {w}: max err {err:.3e}", flush=True)
            assert err <= tol
    assert sa.get_seq_length() == N and sb.get_seq_length() == N


def test_left_masked_workers():
    """Workers that bring different numbers of new tokens in one step (left padding, attention.py:148-155): the worker
    with fewer tokens must end up exactly where it would have with separate calls."""
    from inference_lib_amd.cache import HogwildCache
    from inference_lib_amd.model import decode_step
    dtype, tol = torch.float32, 5e-5
    cfg, plain = tiny_model(1, dtype, seed=3)
    hog = swapped_copy(plain)
    T = 12
    g = torch.Generator().manual_seed(11)
    p_ids = torch.randint(0, cfg.vocab_size, (1, T), generator=g).to(DEV)
    a_ids = torch.randint(0, cfg.vocab_size, (3,), generator=g).to(DEV)
    b_ids = torch.randint(0, cfg.vocab_size, (1,), generator=g).to(DEV)
    prompt, sa, sb = segment(cfg, 32, dtype), segment(cfg, 16, dtype), segment(cfg, 16, dtype)
    decode_step(hog, HogwildCache([[prompt]], hog), p_ids)
    cache = HogwildCache([[prompt, sb, sa], [prompt, sa, sb]], hog)
    ids = torch.stack([a_ids, torch.cat([torch.zeros(2, dtype=a_ids.dtype, device=DEV), b_ids])])     # worker 1: two pads, one token
    mask = torch.tensor([[1, 1, 1], [0, 0, 1]], device=DEV)
    print("masked step", flush=True)
    got = decode_step(hog, cache, ids, mask).float()
    assert sa.get_seq_length() == 3 and sb.get_seq_length() == 1
    with torch.no_grad():
        want_a = plain(torch.cat([p_ids[0], b_ids, a_ids])[None]).logits[0, -1].float()
        want_b = plain(torch.cat([p_ids[0], a_ids, b_ids])[None]).logits[0, -1].float()
    assert (got[0, -1] - want_a).abs().max().item() <= tol
    assert (got[1, -1] - want_b).abs().max().item() <= tol
    # the same kind of step (three tokens for worker 0, one for worker 1) with the lengths in device memory
    a2 = torch.randint(0, cfg.vocab_size, (3,), generator=g).to(DEV)
    b2 = torch.randint(0, cfg.vocab_size, (1,), generator=g).to(DEV)
    cache.use_device_lengths(headroom=8, new_tokens=3, n_new=[3, 1])
    ids2 = torch.stack([a2, torch.cat([torch.zeros(2, dtype=a2.dtype, device=DEV), b2])])
    print("masked step, device-resident lengths", flush=True)
    got2 = decode_step(hog, cache, ids2, mask).float()
    cache.use_host_lengths()
    assert sa.get_seq_length() == 6 and sb.get_seq_length() == 2
    with torch.no_grad():
        want_a2 = plain(torch.cat([p_ids[0], b_ids, b2, a_ids, a2])[None]).logits[0, -1].float()
        want_b2 = plain(torch.cat([p_ids[0], a_ids, a2, b_ids, b2])[None]).logits[0, -1].float()
    assert (got2[0, -1] - want_a2).abs().max().item() <= tol
    assert (got2[1, -1] - want_b2).abs().max().item() <= tol


def test_decode_steps_replayed_from_one_graph():
    """The whole decode step of the swapped model (embedding, rotary embedding, both decoder layers with key rotation +
    append + fused attention, head) captured in a HIP graph once, with the segment lengths in device memory, and replayed
    while the worker's segment grows; every replay must give the plain model's logits at that position."""
    from inference_lib_amd.cache import HogwildCache
    from inference_lib_amd.model import decode_step
    dtype, tol = torch.float32, 5e-5
    cfg, plain = tiny_model(2, dtype, seed=4)
    hog = swapped_copy(plain)
    T, N = 21, 9
    g = torch.Generator().manual_seed(13)
    ids = torch.randint(0, cfg.vocab_size, (1, T + N), generator=g).to(DEV)
    with torch.no_grad():
        want = plain(ids).logits.float()
    prompt, seg = segment(cfg, 32, dtype), segment(cfg, 4, dtype)
    decode_step(hog, HogwildCache([[prompt]], hog), ids[:, :T])
    cache = HogwildCache([[prompt, seg]], hog)
    cache.use_device_lengths(headroom=16, new_tokens=1)
    tok = torch.zeros((1, 1), dtype=ids.dtype, device=DEV)
    logits = torch.zeros((1, 1, cfg.vocab_size), dtype=dtype, device=DEV)

    def step():
        logits.copy_(decode_step(hog, cache, tok))

    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        tok.copy_(ids[:, T: T + 1])
        step()                                   # first token eagerly
        torch.cuda.synchronize()
        assert (logits.float() - want[:, T: T + 1]).abs().max().item() <= tol
        with torch.cuda.graph(graph, stream=stream):
            step()
        for i in range(1, N):
            tok.copy_(ids[:, T + i: T + i + 1])
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            err = (logits.float() - want[:, T + i: T + i + 1]).abs().max().item()
            print(f"replay {i}: max err {err:.3e}", flush=True)
            assert err <= tol
    cache.use_host_lengths()
    assert seg.get_seq_length() == N and prompt.get_seq_length() == T
