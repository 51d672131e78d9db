"""BASELINE config 4 at its real size: the random-init Llama-3-8B-shaped decoder that bench.py times
(32 layers, hidden 4096, 32 q / 8 kv heads of 128, ffn 14336, vocab 128256, SBVR S=4 G=128 on the
linears), its 128-token uniform-random prompt and 128 greedy tokens, built by bench.decode_workload().

The step it stands for is models/sbvr_llama.py:368-408 (decoder layer) inside :836-924 (model
forward) of the reference.  Checked here:
  (i)   teacher-forced: the whole sequence of 256 inputs (the prompt, then the tokens the decoder
        itself chose) goes through an fp64 restatement, one layer at a time over the oracle's decode
        of that layer's encodings (only one layer's dense weights exist at a time); at sampled
        positions, one of them among the generated ones, the residual stream after every layer, the
        final hidden state and the greedy choice are compared;
  (ii)  eager steps and HIP-graph replays generate the same 256 tokens, twice each;
  (iii) the first generated tokens are the ones recorded below, which bench.py prints as
        decode.first_tokens.
"""
import math
import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

PROMPT, NEW = 128, 128
SAMPLED = (0, 1, 64, 127, 128, 200, 255)       # positions whose hidden states are compared after every layer
# decode.first_tokens of bench.py: the first four tokens generate() returns for this workload.  They follow from
# the seeds alone; a change in the order of a kernel's fp32 additions may move a near-tie and with it these.
FIRST_TOKENS = (21700, 85045, 83730, 21615)


def _decode_layer(oracle, pool, lin):
    """Dense fp64 weight (out, in) of one encoded linear, decoded by the oracle in column blocks on the pool."""
    bvr, idx, cache = lin.bvr.cpu().numpy(), lin.idx.cpu().numpy(), lin.cache.cpu().numpy()
    n = bvr.shape[1]
    step = 512
    jobs = [(c, min(n, c + step)) for c in range(0, n, step)]

    def one(job):
        a, b = job
        return oracle.C.decode(np.ascontiguousarray(bvr[:, a:b, :]), np.ascontiguousarray(idx[:, a:b]), cache, lin.bvr_len)

    return np.concatenate(list(pool.map(one, jobs)), axis=0)


def _reference(dec, oracle, tokens):
    """fp64 decoder over all positions at once, layer by layer (torch on the device does the fp64 products; the
    weights come from the oracle).  Returns the residual stream after every layer at the SAMPLED positions,
    (layers + 1, len(SAMPLED), hidden) with index 0 the embedding, and the logits at those positions."""
    s, dev = dec.shape, dec.device
    T = len(tokens)
    q_out, kv_out, half = s.heads * s.head_dim, s.kv_heads * s.head_dim, s.head_dim // 2
    X = dec.embed[torch.as_tensor(tokens, device=dev)].double()
    cos, sin = dec.cos[:T].double(), dec.sin[:T].double()
    sampled = torch.as_tensor(SAMPLED, device=dev)

    def norm(x):
        return x / torch.sqrt((x * x).mean(dim=1, keepdim=True) + s.rms_eps)

    def rope(t):                                   # (T, heads, head_dim)
        a, b = t[..., :half], t[..., half:]
        c, d = cos[:, None, :], sin[:, None, :]
        return torch.cat((a * c - b * d, b * c + a * d), dim=-1)

    causal = torch.ones((T, T), dtype=torch.bool, device=dev).tril()
    hidden = [X[sampled].cpu().numpy()]
    with ThreadPoolExecutor(max_workers=min(16, os.cpu_count() or 1)) as pool:
        for layer in dec.layers:
            W = {k: torch.from_numpy(_decode_layer(oracle, pool, layer[k]).astype(np.float32)).to(dev).double()
                 for k in ("qkv", "o", "gate_up", "down")}
            qkv = norm(X) @ W["qkv"].t()
            q = rope(qkv[:, :q_out].reshape(T, s.heads, s.head_dim))
            k = rope(qkv[:, q_out:q_out + kv_out].reshape(T, s.kv_heads, s.head_dim))
            v = qkv[:, q_out + kv_out:].reshape(T, s.kv_heads, s.head_dim)
            group = s.heads // s.kv_heads
            k, v = k.repeat_interleave(group, dim=1), v.repeat_interleave(group, dim=1)
            sc = torch.einsum("thd,uhd->htu", q, k) / math.sqrt(s.head_dim)
            sc = sc.masked_fill(~causal[None], float("-inf"))
            ctx = torch.einsum("htu,uhd->thd", torch.softmax(sc, dim=-1), v).reshape(T, q_out)
            X = X + ctx @ W["o"].t()
            gu = norm(X) @ W["gate_up"].t()
            g, u = gu[:, :s.ffn], gu[:, s.ffn:]
            X = X + (g / (1.0 + torch.exp(-g)) * u) @ W["down"].t()
            hidden.append(X[sampled].cpu().numpy())
            del W
    logits = (norm(X[sampled]) @ dec.lm_head.double().t()).cpu().numpy()
    return np.stack(hidden), logits


def test_config4_full_model(oracle):
    import bench
    dec, prompt = bench.decode_workload(PROMPT, NEW)
    assert dec.shape.layers == 32 and dec.max_seq == PROMPT + NEW

    # (ii) graph replays and eager steps: the same tokens, twice each
    dec.capture()
    graph_a, _ = dec.generate(prompt, NEW)
    graph_b, _ = dec.generate(prompt, NEW)
    graph = dec.graph
    dec.graph = None
    eager_a, _ = dec.generate(prompt, NEW)
    eager_b, _ = dec.generate(prompt, NEW)
    assert torch.equal(graph_a, graph_b), "two graph-replayed generations differ"
    assert torch.equal(eager_a, eager_b), "two eager generations differ"
    assert torch.equal(graph_a, eager_a), "graph replay and eager steps generate different tokens"
    generated = [int(t) for t in graph_a]                     # NEW + 1 tokens: the choices at positions 127 .. 255
    assert len(generated) == NEW + 1

    # (iii) what bench.py prints as decode.first_tokens
    print("config 4 first tokens:", generated[:4], flush=True)
    if FIRST_TOKENS is not None:
        assert generated[:4] == list(FIRST_TOKENS), f"first tokens {generated[:4]}, recorded {list(FIRST_TOKENS)}"

    # (i) teacher-forced: the inputs of the 256 steps, eager, with the residual stream probed
    tokens = [int(t) for t in prompt] + generated[:NEW]
    assert len(tokens) == PROMPT + NEW
    seen = {}
    position = [0]

    def probe(layer, residual):
        if position[0] in SAMPLED:
            seen[(position[0], layer)] = residual.float().cpu().numpy()[0]

    dec.reset()
    dec.probe = probe
    with torch.cuda.stream(dec.stream):
        for p, t in enumerate(tokens):
            position[0] = p
            dec.tok.fill_(t)
            dec.step()
        torch.cuda.synchronize()
    dec.probe = None
    picked = dec.generated[:len(tokens)].cpu().numpy()
    # the teacher-forced run reproduces the free-running one
    assert [int(t) for t in picked[PROMPT - 1:PROMPT + NEW]] == generated, "teacher-forced and free-running choices differ"

    hidden, logits = _reference(dec, oracle, tokens)
    layers = dec.shape.layers
    err_max = np.zeros((len(SAMPLED), layers + 1))
    err_rms = np.zeros((len(SAMPLED), layers + 1))
    for i, p in enumerate(SAMPLED):
        for layer in range(layers + 1):
            ref, got = hidden[layer, i], seen[(p, layer)]
            err_max[i, layer] = np.abs(got - ref).max() / np.abs(ref).max()
            err_rms[i, layer] = np.sqrt(np.mean((got - ref) ** 2) / np.mean(ref ** 2))
    for layer in range(layers + 1):
        print(f"config 4: after layer {layer:2d}: residual stream off by at most {err_max[:, layer].max():.2e} of its largest "
              f"element, {err_rms[:, layer].max():.2e} in RMS", flush=True)
    # The decoder keeps the residual stream in fp16 (as the reference's model does) and the fp64 restatement does not:
    # every layer adds two roundings of the stream and two fp16 deltas, and attention and the SiLU pass earlier
    # differences on, so the distance grows with depth.  A wrong layer would show as a jump; the bound is a
    # line through the noise with a margin of about three: 4e-3 at the embedding's successor, 4e-2 after 32 layers.
    for i, p in enumerate(SAMPLED):
        for layer in range(layers + 1):
            bound = 4e-3 + 1.2e-3 * layer
            assert err_max[i, layer] < bound, (f"position {p}, after layer {layer}: residual stream differs by "
                                              f"{err_max[i, layer]:.3e} of its largest element (bound {bound:.1e})")
            assert err_rms[i, layer] < bound, f"position {p}, after layer {layer}: RMS difference {err_rms[i, layer]:.3e}"
        # the greedy choice at this position is one of the reference's near-maximal logits
        ref = logits[i]
        assert ref[picked[p]] >= ref.max() - 4e-2 * np.abs(ref).max(), f"position {p}: token {picked[p]} is not near the reference's maximum"
    dec.graph = graph
    del dec, graph
    torch.cuda.empty_cache()
