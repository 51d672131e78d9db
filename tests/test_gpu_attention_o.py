"""sbvr_hip_dec_attention_o_f16: attention of one decoded token and its SBVR-encoded output projection in one
launch (reference models/sbvr_llama.py:307-354, `attn_output = self.o_proj(attn_output)` at :352), through the C ABI.

Checked per case:
  * the context row it hands out (ctx) against an fp64 restatement of rotary embedding + softmax attention over
    the cache, and against the two-launch path's context (sbvr_hip_dec_attention_f16): both within the same bound;
  * the projection against the oracle's linear of that very context row (the decode kernels' bound: 2 fp16 ulps),
    so the two halves are pinned separately;
  * the caches: the rotated key and the value appended at the position, in the kernel's blocked element order,
    equal to what the two-launch path appends, everything else untouched;
  * cache rows past the position hold NaN: nothing of them may reach the result.
"""
import math

import numpy as np
import pytest
import torch

from parity import tight

pytestmark = pytest.mark.gpu

HEADS, KV_HEADS, HEAD_DIM = 32, 8, 128


def _encoding(N, K, S, G, L, seed):
    from sbvr import synth
    return synth.random_encoding(N, K, S, G, L, seed=seed)


def _reference_ctx(qkv, cos, sin, kc, vc, p, heads, kv_heads):
    """fp64: rotate q and the new k with row p, attention over cache rows 0..p-1 and the new row."""
    hd, half = HEAD_DIM, HEAD_DIM // 2
    c, s = cos[p].double().numpy(), sin[p].double().numpy()

    def rope(t):
        a, b = t[..., :half], t[..., half:]
        return np.concatenate((a * c - b * s, b * c + a * s), axis=-1)

    x = qkv.double().numpy().reshape(-1)
    # (the kernel keeps the rotated vectors in fp16, as the reference's fp16 model does)
    q = rope(x[:heads * hd].reshape(heads, hd)).astype(np.float16).astype(np.float64)
    k_new = rope(x[heads * hd:(heads + kv_heads) * hd].reshape(kv_heads, hd)).astype(np.float16).astype(np.float64)
    v_new = x[(heads + kv_heads) * hd:].reshape(kv_heads, hd)
    K = kc.double().numpy()[:, :p + 1].copy()
    V = vc.double().numpy()[:, :p + 1].copy()
    K[:, p], V[:, p] = k_new, v_new
    want = np.zeros((heads, hd))
    group = heads // kv_heads
    for h in range(heads):
        sc = K[h // group] @ q[h] / math.sqrt(hd)
        pr = np.exp(sc - sc.max())
        want[h] = (pr / pr.sum()) @ V[h // group]
    return want.reshape(-1), k_new, v_new


def _run_case(oracle, max_seq, p, ready_rotation, heads=HEADS, kv_heads=KV_HEADS, N=4096, S=4, G=128, L=256, bias=False,
              seed=0, twice=False):
    from sbvr import hip
    dev = torch.device("cuda:0")
    hd = HEAD_DIM
    K = heads * hd
    print(f"attention + o: max_seq={max_seq} p={p} rot={ready_rotation} heads={heads}/{kv_heads} N={N} S={S} G={G} L={L} "
          f"bias={bias}", flush=True)
    assert hip.dec_attention_o_supported(heads, kv_heads, hd, max_seq, N, S, G)
    bvr, idx, cache = _encoding(N, K, S, G, L, seed + 11)
    gen = torch.Generator().manual_seed(seed * 1000 + p + max_seq)
    qkv = torch.randn((1, (heads + 2 * kv_heads) * hd), generator=gen).to(torch.float16)
    ang = torch.rand((max_seq, hd // 2), generator=gen, dtype=torch.float64) * 6.28
    cos, sin = torch.cos(ang).float(), torch.sin(ang).float()
    kc = torch.randn((kv_heads, max_seq, hd), generator=gen).to(torch.float16)
    vc = torch.randn((kv_heads, max_seq, hd), generator=gen).to(torch.float16)
    kc[:, p:], vc[:, p:] = float("nan"), float("nan")          # nothing at or past the position may be used
    b = (torch.randn(N, generator=gen) * 0.1).to(torch.float16) if bias else None
    pos = torch.tensor([p], device=dev)
    rot = torch.cat((cos[p], sin[p])).to(dev) if ready_rotation else None
    d = dict(qkv=qkv.to(dev), cos=cos.to(dev), sin=sin.to(dev), bvr=bvr.to(dev), idx=idx.to(dev), cache=cache.to(dev),
             bias=b.to(dev) if bias else None)

    # the two-launch path on the natural cache layout
    kc1, vc1 = kc.to(dev), vc.to(dev)
    ctx1 = torch.empty((1, K), dtype=torch.float16, device=dev)
    hip.dec_attention(d["qkv"], d["cos"], d["sin"], pos, kc1, vc1, ctx1, heads, kv_heads, hd, rot)

    # the one launch, on the blocked layout
    kc2 = hip.attention_o_cache_layout(kc.to(dev))
    vc2 = hip.attention_o_cache_layout(vc.to(dev), values=True)
    ctx2 = torch.zeros((1, K), dtype=torch.float16, device=dev)
    out = torch.full((1, N), 7.0, dtype=torch.float16, device=dev)
    outs = []
    for _ in range(2 if twice else 1):
        out.fill_(7.0)
        hip.dec_attention_o(d["qkv"], d["cos"], d["sin"], pos, kc2, vc2, heads, kv_heads, hd, d["bvr"], d["idx"],
                            d["cache"], d["bias"], G, out=out, rot_now=rot, ctx=ctx2)
        torch.cuda.synchronize()
        outs.append(out.cpu().clone())
    if twice:       # the split-K accumulators were left zero, and the appended row is not read back
        assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16)), "a second launch gives another result"

    want, k_new, v_new = _reference_ctx(qkv, cos, sin, kc, vc, p, heads, kv_heads)
    got_ctx = ctx2.float().cpu().numpy().astype(np.float64).reshape(-1)
    old_ctx = ctx1.float().cpu().numpy().astype(np.float64).reshape(-1)
    assert np.isfinite(got_ctx).all() and np.isfinite(outs[0].float().numpy()).all()
    bound = 3e-3 * np.abs(want).max()
    assert np.abs(got_ctx - want).max() <= bound, f"context off by {np.abs(got_ctx - want).max():.3e} (bound {bound:.1e})"
    assert np.abs(got_ctx - old_ctx).max() <= bound, "the one-launch and two-launch contexts differ"

    # the projection of the context row it reports
    _, yd = oracle.C.linear_f16(ctx2.cpu().numpy(), bvr.numpy(), idx.numpy(), cache.numpy(), G)
    y = outs[0].float().numpy().astype(np.float64)
    if bias:        # added after the rounding (sbvr_kernel.cu:555-559)
        yref = (yd.astype(np.float16).astype(np.float32) + b.float().numpy()[None, :]).astype(np.float16)
        assert np.abs(y - yref.astype(np.float64)).max() <= 2.0 ** -9 * max(1.0, np.abs(yref).max()), "with bias"
    else:
        tight(y, yd, "projection of the reported context")

    # caches: the same row appended as by the two-launch path, everything else untouched
    k_nat = hip.attention_o_cache_layout(kc2, inverse=True).cpu()
    v_nat = hip.attention_o_cache_layout(vc2, inverse=True, values=True).cpu()
    assert torch.equal(k_nat[:, p].view(torch.int16), kc1[:, p].cpu().view(torch.int16))
    assert torch.equal(v_nat[:, p].view(torch.int16), vc1[:, p].cpu().view(torch.int16))
    assert np.abs(k_nat[:, p].double().numpy() - k_new).max() <= 2e-3 * np.abs(k_new).max()
    keep = torch.ones(max_seq, dtype=torch.bool)
    keep[p] = False
    assert torch.equal(k_nat[:, keep].view(torch.int16), kc[:, keep].view(torch.int16))
    assert torch.equal(v_nat[:, keep].view(torch.int16), vc[:, keep].view(torch.int16))


@pytest.mark.parametrize("max_seq,p", [(256, 0), (256, 1), (256, 15), (256, 16), (256, 31), (256, 32), (256, 33), (256, 127),
                                       (256, 200), (256, 255), (512, 255), (512, 256), (512, 300), (512, 511), (64, 40),
                                       (32, 31), (1024, 777), (4096, 4095)])
def test_positions(oracle, max_seq, p):
    _run_case(oracle, max_seq, p, ready_rotation=True, twice=p in (0, 200, 300))


@pytest.mark.parametrize("p", [0, 100, 300])
def test_rotation_from_the_tables(oracle, p):
    _run_case(oracle, 512, p, ready_rotation=False)


@pytest.mark.parametrize("kw", [dict(S=2), dict(S=3), dict(S=6), dict(S=8), dict(G=256), dict(G=512), dict(L=300), dict(L=16),
                                dict(bias=True), dict(N=128), dict(N=1152), dict(heads=4, kv_heads=1, N=256),
                                dict(heads=8, kv_heads=2, N=512, G=256), dict(heads=64, kv_heads=16, N=8192)])
def test_formats_and_shapes(oracle, kw):
    _run_case(oracle, 256, 77, ready_rotation=True, seed=3, **kw)


@pytest.mark.parametrize("stored,used", [(-3, 0), (64 + 5, 63)])
def test_position_outside_the_cache_is_clamped(stored, used):
    """*pos below 0 or beyond the cache is taken as the nearest valid position, as by the two-launch kernel."""
    from sbvr import hip
    dev = torch.device("cuda:0")
    heads, kv_heads, hd, max_seq, N, S, G, L = 32, 8, HEAD_DIM, 64, 4096, 4, 128, 256
    bvr, idx, cache = (t.to(dev) for t in _encoding(N, heads * hd, S, G, L, 21))
    gen = torch.Generator().manual_seed(stored + 100)
    qkv = torch.randn((1, (heads + 2 * kv_heads) * hd), generator=gen).to(torch.float16).to(dev)
    ang = torch.rand((max_seq, hd // 2), generator=gen, dtype=torch.float64) * 6.28
    cos, sin = torch.cos(ang).float().to(dev), torch.sin(ang).float().to(dev)
    kc = torch.randn((kv_heads, max_seq, hd), generator=gen).to(torch.float16).to(dev)
    vc = torch.randn((kv_heads, max_seq, hd), generator=gen).to(torch.float16).to(dev)
    results = []
    for p in (stored, used):
        k2, v2 = hip.attention_o_cache_layout(kc), hip.attention_o_cache_layout(vc, values=True)
        ctx = torch.zeros((1, heads * hd), dtype=torch.float16, device=dev)
        out = torch.empty((1, N), dtype=torch.float16, device=dev)
        hip.dec_attention_o(qkv, cos, sin, torch.tensor([p], device=dev), k2, v2, heads, kv_heads, hd, bvr, idx, cache, None, G,
                            out=out, ctx=ctx)
        torch.cuda.synchronize()
        results.append((out.clone(), ctx.clone(), k2, v2))
    for a, b in zip(results[0], results[1]):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_refusals():
    """Shapes the launch does not take are refused, and so is a call without its accumulators."""
    import ctypes
    from sbvr import hip
    ok = hip.dec_attention_o_supported
    assert ok(32, 8, 128, 256, 4096, 4, 128)
    assert not ok(32, 8, 64, 256, 4096, 4, 128)          # head size
    assert not ok(32, 4, 128, 256, 4096, 4, 128)         # eight query heads per key/value head
    assert not ok(32, 8, 128, 250, 4096, 4, 128)         # cache length not a multiple of 32
    assert not ok(32, 8, 128, 8192, 4096, 4, 128)        # cache too long for LDS
    assert not ok(32, 8, 128, 256, 4000, 4, 128)         # N not a multiple of 128
    assert not ok(32, 8, 128, 256, 4096, 5, 128)         # plane count
    assert not ok(32, 8, 128, 256, 4096, 4, 64)          # group size
    lib = hip._load()
    dev = torch.device("cuda:0")
    hip._sbvr_hip_init(dev)
    heads, kv, hd, max_seq, N, S, G, L = 32, 8, 128, 64, 4096, 4, 128, 256
    bvr, idx, cache = [t.to(dev) for t in _encoding(N, heads * hd, S, G, L, 1)]
    qkv = torch.zeros((heads + 2 * kv) * hd, dtype=torch.float16, device=dev)
    cos = torch.ones((max_seq, hd // 2), device=dev)
    sin = torch.zeros((max_seq, hd // 2), device=dev)
    pos = torch.zeros(1, dtype=torch.int64, device=dev)
    kc = torch.zeros((kv, max_seq, hd), dtype=torch.float16, device=dev)
    vc = torch.zeros_like(kc)
    out = torch.full((N,), 3.0, dtype=torch.float16, device=dev)

    def call(head_dim=hd, ws=None, ws_bytes=0):
        return lib.sbvr_hip_dec_attention_o_f16(qkv.data_ptr(), cos.data_ptr(), sin.data_ptr(), None, pos.data_ptr(),
                                                kc.data_ptr(), vc.data_ptr(), None, heads, kv, head_dim, max_seq,
                                                bvr.data_ptr(), idx.data_ptr(), 1, cache.data_ptr(), None, out.data_ptr(),
                                                N, S, G, L, ws, ws_bytes, None)

    assert call(head_dim=64) == -2
    assert call() == -4 and b"workspace" in lib.sbvr_hip_last_error()
    small = torch.zeros(N * 8 - 8, dtype=torch.uint8, device=dev)
    assert call(ws=small.data_ptr(), ws_bytes=small.numel()) == -4
    torch.cuda.synchronize()
    assert bool((out == 3.0).all()), "a refused call wrote to its output"
    assert lib.sbvr_hip_dec_attention_o_workspace(kv, N) == N * 8 and lib.sbvr_hip_dec_attention_o_workspace(1, N) == 0


def test_decoder_steps_agree_with_the_two_launch_path():
    """The Llama-shaped decoder with attention and o in one launch against the same decoder with two: the
    residual streams stay within fp16 rounding of each other over a few steps (two layers at the real widths)."""
    from sbvr.decoder import LlamaShape, SbvrLlamaDecoder
    shape = LlamaShape(layers=2)
    logits = {}
    for mode in (True, False):
        dec = SbvrLlamaDecoder(shape, "cuda:0", max_seq=32, seed=11, attention_o=mode)
        assert dec.attention_o == mode
        for layer in dec.layers:
            for k in ("qkv", "o", "gate_up", "down"):
                layer[k].cache.mul_(1.5)
        dec.reset()
        rows = []
        with torch.cuda.stream(dec.stream):
            for t in (5, 77777, 128255, 4096, 9):
                dec.tok.fill_(t)
                rows.append(dec.step().float().cpu().numpy()[0].astype(np.float64))
                torch.cuda.synchronize()
        logits[mode] = np.stack(rows)
        del dec
        torch.cuda.empty_cache()
    diff = np.abs(logits[True] - logits[False]).max() / np.abs(logits[False]).max()
    assert diff < 5e-3, f"logits of the two paths differ by {diff:.2e} of the largest"
