#!/usr/bin/env python3
"""Benchmark of the SBVR compressed-domain GEMV on one MI355X.

Workload (BASELINE.json configs[1], the shape the metric is quoted on): the
Llama-3-8B gate projection 4096 -> 14336 at batch 1, 4 bit planes, group 128,
uint32-packed planes, fp16 coefficient table of 256 lines (uint8 indices),
fp16 N(0,1) activations, synthetic seeded encodings.  A step is one GEMV over
one weight copy; consecutive steps walk through COPIES distinct weight copies
(about 480 MB) so that every step streams its planes from HBM and not from the
256 MB Infinity Cache.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

prints one JSON line: whole-job throughput in GB/s of algorithmic bytes, the
roofline of the kernel (HIP events on the launch stream), the second half of
the metric ("decode": tokens/s of a random-init Llama-3-8B-shaped decoder whose
linears are SBVR-encoded, 128-token prompt + 128 greedy tokens) and the CPU
baseline (the x86 port of the reference's timed CPU kernel on the host's own
cores: the gate GEMV, and the linears of one token for the decode figure).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "sbvr-cpu-arm_amd"))
sys.path.insert(0, ROOT)

N_OUT, K_IN, NUM_SUMS, GROUP, LINES, BATCH = 14336, 4096, 4, 128, 256, 1
COPIES = 16
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the gate GEMV as the hardware counters saw them: rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE, each scaled by what the same counter reads for a 256 MiB copy.  A profiler run's figure,
# not measured by this script: the line names the file it comes from.
TRAFFIC_FROM_PROFILE_BYTES = 30.07e6
TRAFFIC_PROFILE = "profiles/sbvr_gemv_mfma_gate_4096x14336.txt"
MIN_TIMED_LAUNCHES = 200
_WEIGHTS = None        # the rotating weight copies on the device (built once per process)


def algorithmic_bytes(n, k, s, g, lines, m):
    """Bytes one GEMV has to move: planes + indices + table + activations + outputs."""
    idx_bytes = 1 if lines <= 256 else 2
    return n * k * s // 8 + (k // g) * n * idx_bytes + 2 * lines * s + 2 * m * k + 2 * m * n


def gpu_leg(steps, warmup, floor=False):
    """Times `steps` launches of the gate GEMV (or, with `floor`, of the launch that only makes its
    memory requests), recorded into one HIP graph.  Returns the wall-clock ms per step of ONE replay
    (the figure `value` is made from: exactly `steps` launches between two synchronisations) and the
    HIP-event time per launch over enough further replays to cover at least MIN_TIMED_LAUNCHES
    launches (median and minimum over the replays)."""
    import torch
    import sbvr
    from sbvr import synth, hip, _sbvr_hip_ops as ops

    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU (torch.cuda.is_available() is False)")
    dev = torch.device("cuda:0")
    sbvr._sbvr_hip_init(dev)
    global _WEIGHTS
    if _WEIGHTS is None:
        _WEIGHTS = []
        for c in range(COPIES):
            bvr, idx, cache = synth.random_encoding(N_OUT, K_IN, NUM_SUMS, GROUP, LINES, seed=c)
            _WEIGHTS.append((bvr.to(dev), idx.to(dev), cache.to(dev)))
    weights = _WEIGHTS
    x = torch.randn((BATCH, K_IN), generator=torch.Generator().manual_seed(1234)).to(torch.float16).to(dev)
    out = torch.empty((BATCH, N_OUT), dtype=torch.float16, device=dev)

    def step(i):
        bvr, idx, cache = weights[i % COPIES]
        if floor:
            hip._sbvr_linear_f16_stream_floor(bvr, idx, cache, GROUP, out=out)
        else:
            # the PyTorch extension over the C ABI (csrc/sbvr_ops_hip.cpp)
            ops._sbvr_linear_f16(x, bvr, idx, cache, None, GROUP, 0, out)

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()

    # The K timed steps are recorded once into a HIP graph and replayed, so that
    # the launch path is the driver's and not the Python interpreter's.
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    launcher = "hipGraph"
    try:
        with torch.cuda.stream(stream):
            step(0)                      # workspace for this stream exists before capture
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=stream):
                for i in range(steps):
                    step(warmup + i)
            graph.replay()               # first replay uploads the graph
            torch.cuda.synchronize()
    except Exception as exc:             # capture is an optimisation, not a requirement
        print(f"bench.py: graph capture failed ({exc}); timing eager launches", file=sys.stderr)
        graph = None
        launcher = "eager"

    def run_steps():
        if graph is not None:
            graph.replay()
        else:
            for i in range(steps):
                step(warmup + i)

    with torch.cuda.stream(stream):
        # the timed region of the contract: exactly `steps` steps between two synchronisations
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run_steps()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        wall_ms = (t1 - t0) * 1e3 / steps
        # the kernel's own time: HIP events on the launch stream around each of several replays
        replays = max(3, -(-MIN_TIMED_LAUNCHES // steps))
        per_launch = []
        for _ in range(replays):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            run_steps()
            e1.record(stream)
            torch.cuda.synchronize()
            per_launch.append(e0.elapsed_time(e1) / steps)
    per_launch.sort()
    timing = {"median_ms": per_launch[len(per_launch) // 2], "min_ms": per_launch[0],
              "launches_timed": replays * steps, "replays": replays}
    return wall_ms, timing, launcher, torch.cuda.get_device_name(0)


def decode_workload(prompt_tokens=128, new_tokens=128):
    """The decoder and the prompt of the "8B decode tokens/s" figure (BASELINE.json configs[3]): 32 layers at the
    Llama-3-8B widths, random init, seeded synthetic encodings, a 128-token uniform-random prompt.  Also what
    tests/test_gpu_config4.py checks against the oracle."""
    import torch
    from sbvr.decoder import LlamaShape, SbvrLlamaDecoder

    shape = LlamaShape()
    dec = SbvrLlamaDecoder(shape, "cuda:0", num_sums=NUM_SUMS, bvr_len=GROUP, lines=LINES,
                           max_seq=prompt_tokens + new_tokens)
    prompt = torch.randint(0, shape.vocab, (prompt_tokens,), generator=torch.Generator().manual_seed(0))
    return dec, prompt


def decode_leg(prompt_tokens=128, new_tokens=128):
    """Random-init Llama-3-8B-shaped decoder with SBVR linears (sbvr/decoder.py):
    a 128-token uniform-random prompt, then 128 greedy tokens at batch 1, one
    HIP-graph replay per prompt token and per 16 new tokens (the same launches
    either way; the GPU idles some 8 us between two replays); the figure covers
    the new tokens only."""
    import torch

    dec, prompt = decode_workload(prompt_tokens, new_tokens)
    shape = dec.shape
    dec.capture()
    best = None
    for _ in range(2):
        tokens, seconds = dec.generate(prompt, new_tokens)
        best = seconds if best is None else min(best, seconds)
    per_token = dec.bytes_per_token()
    out = {
        "tokens_per_s": round(new_tokens / best, 1),
        "ms_per_token": round(best / new_tokens * 1e3, 4),
        "prompt_tokens": prompt_tokens,
        "new_tokens": new_tokens,
        "bytes_per_token": per_token,
        "achieved_GBps": round(per_token * new_tokens / best / 1e9, 1),
        "frac_of_hbm_peak": round(per_token * new_tokens / best / 1e9 / HBM_PEAK_GBS, 4),
        "model": f"Llama-3-8B shape ({shape.layers} layers, d={shape.hidden}, {shape.heads}q/{shape.kv_heads}kv heads, "
                 f"ffn {shape.ffn}, vocab {shape.vocab}), random init, SBVR S={NUM_SUMS} G={GROUP} on q|k|v, o, gate|up, "
                 "down; fp16 embedding and head",
        "first_tokens": [int(t) for t in tokens[:4]],
        "breakdown_us_per_token": decode_breakdown(dec),
    }
    del dec
    torch.cuda.empty_cache()
    return out


def decode_breakdown(dec):
    """Where a token's time goes: the three kinds of launches of a step, each recorded into a HIP graph of
    its own (all 32 layers' worth) and replayed on the decoder's buffers after the timed generation.
    Launches of one kind run back to back here, so the parts add up to a little less than a whole step."""
    import torch
    from sbvr import hip
    s = dec.shape

    def linears():
        a, b, ctx, delta = dec.x, dec.x_alt, dec.ctx, dec.zero
        for layer in dec.layers:
            layer["qkv"].after_add_rmsnorm(a, delta, layer["norm1"], s.rms_eps, b)
            if not dec.attention_o:
                delta = layer["o"](ctx)
            gate_up = layer["gate_up"].after_add_rmsnorm(b, delta, layer["norm2"], s.rms_eps, a)
            delta = layer["down"].after_swiglu(gate_up)

    def attention():
        for layer in dec.layers:
            if dec.attention_o:
                o = layer["o"]
                hip.dec_attention_o(layer["qkv"].out, dec.cos, dec.sin, dec.pos, layer["k"], layer["v"], s.heads,
                                    s.kv_heads, s.head_dim, o.bvr, o.idx, o.cache, None, o.bvr_len, out=o.out,
                                    rot_now=dec.rot_now)
            else:
                hip.dec_attention(layer["qkv"].out, dec.cos, dec.sin, dec.pos, layer["k"], layer["v"], dec.ctx,
                                  s.heads, s.kv_heads, s.head_dim, dec.rot_now)

    def head():
        hip.dec_head_argmax(dec.x, dec.zero, dec.final_norm, s.rms_eps, dec.lm_head, dec.logits, dec.tok,
                            dec.generated, dec.pos, dec.head_ws, dec.cos, dec.sin, dec.rot_now)

    if dec.attention_o:
        parts = {"linears (3 per layer, prologues folded in)": linears,
                 "attention + o projection (1 launch per layer)": attention}
    else:
        parts = {"linears (4 per layer, prologues folded in)": linears, "attention (1 per layer)": attention}
    if hip.dec_head_argmax_supported(s.hidden):
        parts["final norm + fp16 head + argmax"] = head
    out = {}
    dec.reset()
    dec.pos.fill_(dec.max_seq // 2)          # attention over half the cache, as in the middle of the timed run
    for name, fn in parts.items():
        out[name] = round(_graph_time(lambda i: fn(), 1, stream=dec.stream) * 1e6, 1)
        dec.pos.fill_(dec.max_seq // 2)
    dec.reset()
    return out


def attention_o_leg(eager=0):
    """The decoder layer's attention and o projection at the Llama-3-8B shape (32 / 8 heads of 128, hidden 4096,
    cache of 256 positions, SBVR S=4 G=128 projection), as one launch (sbvr_hip_dec_attention_o_f16) and as two
    (sbvr_hip_dec_attention_f16, then the linear), 32 layers' worth of distinct weights and caches replayed from
    one HIP graph, at three positions.  eager > 0: only that many eager launches of the one-launch form per
    position (no graph, no timing): what a counter pass of a profiler wants."""
    import torch
    from sbvr import hip, synth
    dev = torch.device("cuda:0")
    hip._sbvr_hip_init(dev)
    heads, kv_heads, hd, max_seq, hidden, layers = 32, 8, 128, 256, 4096, 32
    gen = torch.Generator(device=dev).manual_seed(0)
    ws = []
    for l in range(layers):
        b, i, c = (t.to(dev) for t in synth.random_encoding(hidden, heads * hd, NUM_SUMS, GROUP, LINES, seed=l))
        kc = torch.randn((kv_heads, max_seq, hd), generator=gen, device=dev).to(torch.float16)
        vc = torch.randn((kv_heads, max_seq, hd), generator=gen, device=dev).to(torch.float16)
        ws.append((b, i, c, kc, vc, kc.clone(), vc.clone()))
    qkv = torch.randn((1, (heads + 2 * kv_heads) * hd), generator=gen, device=dev).to(torch.float16)
    ang = torch.rand((max_seq, hd // 2), generator=gen, device=dev) * 6.28
    cos, sin = torch.cos(ang), torch.sin(ang)
    ctx = torch.empty((1, heads * hd), dtype=torch.float16, device=dev)
    out = torch.empty((1, hidden), dtype=torch.float16, device=dev)
    rows = []
    for p in (128, 200, 255):
        pos = torch.tensor([p], device=dev)
        rot = torch.cat((cos[p], sin[p])).contiguous()

        def one(_):
            for (b, i, c, kc, vc, kb, vb) in ws:
                hip.dec_attention_o(qkv, cos, sin, pos, kb, vb, heads, kv_heads, hd, b, i, c, None, GROUP, out=out,
                                    rot_now=rot)

        def two(_):
            for (b, i, c, kc, vc, kb, vb) in ws:
                hip.dec_attention(qkv, cos, sin, pos, kc, vc, ctx, heads, kv_heads, hd, rot)
                hip._sbvr_linear_f16(ctx, b, i, c, None, GROUP, out=out)

        if eager:
            for _ in range(max(1, eager // layers)):
                one(0)
            torch.cuda.synchronize()
            rows.append({"position": p, "eager_launches": max(1, eager // layers) * layers})
            continue
        rows.append({"position": p,
                     "one_launch_us": round(_graph_time(one, 1) * 1e6 / layers, 2),
                     "two_launches_us": round(_graph_time(two, 1) * 1e6 / layers, 2)})
    return rows


def _graph_time(fn, iters, stream=None):
    """Seconds per call of fn(i), i = 0..iters-1, recorded into one HIP graph and replayed (best of 3)."""
    import torch
    stream = stream or torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        fn(0)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(iters):
                fn(i)
        graph.replay()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            graph.replay()
            e1.record(stream)
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) * 1e-3 / iters
            best = t if best is None else min(best, t)
    return best


def read_floor_leg(quick=False):
    """What the memory system hands to a launch that only reads, whatever grid the decode kernel uses
    (sbvr_hip_read_floor): the 28 672 KiB of plane words of the gate shape, one request of 1 KiB per wave
    instruction, over workgroups per CU in {1, 2, 4} x waves in {4, 8, 16} x requests in flight per wave, as one
    contiguous band (pattern 0), a contiguous piece per wave (1) and in the decode kernel's own 896-byte windows
    of 229 376-byte rows (2); plus one stream of 1 GiB.  The buffers rotate through the same 16 weight copies as
    the timed GEMV (beyond the 256 MB memory-side cache).  quick: the few shapes the default line reports."""
    import torch
    from sbvr import hip
    dev = torch.device("cuda:0")
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    plane_bytes = N_OUT * K_IN * NUM_SUMS // 8
    bufs = [torch.randint(-2 ** 31, 2 ** 31, (plane_bytes // 4,), dtype=torch.int32, device=dev) for _ in range(COPIES)]
    rows = []

    def one(wgs_per_cu, waves, ahead, pattern):
        wgs = cus * wgs_per_cu
        units = plane_bytes // 1024
        per_wave = units // (wgs * waves)
        if pattern == 2:
            # the gate launch's own geometry: one window of 56 columns x 16 bytes per workgroup
            wgs, win, row = 256, 56 * NUM_SUMS * 4, N_OUT * NUM_SUMS * 4
            per_wave = (K_IN // 128 // waves) * 4            # 4 tiles of 256 bytes (the last one half used) per sub-group
            if K_IN // 128 % waves or per_wave % ahead:
                return
            nbytes = per_wave * wgs * waves * 1024
            t = _graph_time(lambda i: hip.read_floor(bufs[i % COPIES], nbytes, wgs, waves, ahead, 2, row, win), 64)
            moved = plane_bytes                                # (bytes of the buffer actually touched)
        else:
            if per_wave == 0 or per_wave % ahead:
                return
            nbytes = per_wave * wgs * waves * 1024
            t = _graph_time(lambda i: hip.read_floor(bufs[i % COPIES], nbytes, wgs, waves, ahead, pattern), 64)
            moved = nbytes
        rows.append({"pattern": pattern, "workgroups_per_cu": wgs_per_cu if pattern != 2 else 1, "waves": waves, "in_flight": ahead,
                     "KiB_per_wave": per_wave, "bytes": moved, "us": round(t * 1e6, 3),
                     "GBps": round(moved / t / 1e9, 1), "frac_of_hbm_peak": round(moved / t / 1e9 / HBM_PEAK_GBS, 4)})

    if quick:
        grid = [(1, 16, 7, 0), (2, 8, 7, 0), (1, 8, 14, 0), (4, 4, 7, 0), (1, 16, 4, 2), (1, 16, 8, 2)]
    else:
        grid = [(w, v, a, p) for p in (0, 1) for w in (1, 2, 4) for v in (4, 8, 16) for a in (1, 2, 4, 7, 14)]
        grid += [(1, v, a, 2) for v in (8, 16) for a in (1, 2, 4, 8, 16)]
    for w, v, a, p in grid:
        one(w, v, a, p)
    del bufs
    torch.cuda.empty_cache()
    best = max(rows, key=lambda r: r["GBps"]) if rows else None
    out = {"rows": rows, "best": best}
    if not quick:
        big = torch.randint(-2 ** 31, 2 ** 31, ((1 << 30) // 4,), dtype=torch.int32, device=dev)
        big2 = torch.randint(-2 ** 31, 2 ** 31, ((1 << 30) // 4,), dtype=torch.int32, device=dev)
        pair = (big, big2)
        streams = []
        for wgs_per_cu, waves, ahead in ((4, 16, 4), (8, 8, 8), (4, 16, 16), (16, 4, 16)):
            wgs = cus * wgs_per_cu
            t = _graph_time(lambda i: hip.read_floor(pair[i % 2], 1 << 30, wgs, waves, ahead, 0), 8)
            streams.append({"workgroups_per_cu": wgs_per_cu, "waves": waves, "in_flight": ahead, "us": round(t * 1e6, 1),
                            "GBps": round((1 << 30) / t / 1e9, 1), "frac_of_hbm_peak": round((1 << 30) / t / 1e9 / HBM_PEAK_GBS, 4)})
        out["one_GiB_stream"] = streams
    return out


def sweep_leg(only=None):
    """The other decode configurations of the reference's benchmark plan: every linear of a
    Llama-3-8B layer at batch 1, and gate / down at batch 1..16 with 2, 3 and 4 planes.
    Weights rotate through enough copies to exceed the 256 MB Infinity Cache.
    only = (N, K, M): that one linear alone (4 planes, groups of 128, 256 lines), e.g. under a profiler."""
    import torch
    from sbvr import synth, hip
    dev = torch.device("cuda:0")
    rows = []

    def one(n, k, s, m, tag, g=GROUP, lines=LINES):
        per = n * k * s // 8
        copies = max(2, min(16, int(600e6 // per)))
        ws = [tuple(t.to(dev) for t in synth.random_encoding(n, k, s, g, lines, seed=c)) for c in range(copies)]
        x = torch.randn((m, k), generator=torch.Generator().manual_seed(5)).to(torch.float16).to(dev)
        out = torch.empty((m, n), dtype=torch.float16, device=dev)
        t = _graph_time(lambda i: hip._sbvr_linear_f16(x, *ws[i % copies], None, g, out=out), 100)
        nbytes = algorithmic_bytes(n, k, s, g, lines, m)
        rows.append({"linear": tag, "N": n, "K": k, "S": s, "M": m, "G": g, "lines": lines,
                     "idx": "uint8" if lines <= 256 else "uint16", "us": round(t * 1e6, 2),
                     "GBps": round(nbytes / t / 1e9, 1), "frac_of_hbm_peak": round(nbytes / t / 1e9 / HBM_PEAK_GBS, 4)})
        del ws
        torch.cuda.empty_cache()

    if only is not None:
        one(only[0], only[1], 4, only[2], "%dx%d" % (only[0], only[1]))
        return rows
    for tag, n, k in (("q/o", 4096, 4096), ("k/v", 1024, 4096), ("q|k|v", 6144, 4096), ("gate/up", 14336, 4096),
                      ("gate|up", 28672, 4096), ("down", 4096, 14336)):
        one(n, k, 4, 1, tag)
    # tables of more than 256 lines, hence uint16 line indices (the reference switches the index width at
    # L = 256, sbvr_kernel.cu:931-932): config 1 and the gate shape with 300 lines, and the fused matrices of the
    # decoder with the tables they really carry (three and two tables of 256 lines one behind the other)
    for tag, n, k, lines in (("q/o", 4096, 4096, 300), ("gate/up", 14336, 4096, 300), ("q|k|v", 6144, 4096, 768),
                             ("gate|up", 28672, 4096, 512)):
        one(n, k, 4, 1, tag, lines=lines)
    # the reference's own group length of 256 elements (sbvr/core.py:222) at the four layer shapes
    for tag, n, k in (("q/o", 4096, 4096), ("k/v", 1024, 4096), ("gate/up", 14336, 4096), ("down", 4096, 14336)):
        one(n, k, 4, 1, tag, g=256)
    for tag, n, k in (("gate", 14336, 4096), ("down", 4096, 14336)):
        for s in (2, 3, 4):
            for m in (1, 2, 4, 8, 16):
                if not (s == 4 and m == 1):
                    one(n, k, s, m, tag)
    # beyond the reference's plan: 17 and 32 rows, the range of the 32-row kernel
    for tag, n, k in (("q/o", 4096, 4096), ("gate", 14336, 4096), ("down", 4096, 14336)):
        for m in (17, 32):
            one(n, k, 4, m, tag)
    return rows


def other_ops_leg():
    """The reference's own operator forms at the Llama-3-8B layer shapes, batch 1: both operands
    encoded (_sbvr_mm_T, the form its CPU kernels time) and fp16 activations against a
    trans=True weight (_sbvr_row_deq_mm_T).  Same bytes as the linear of the same shape."""
    import torch
    from sbvr import synth, hip
    dev = torch.device("cuda:0")
    rows = []
    none = torch.zeros(0, dtype=torch.float16, device=dev)
    for tag, n, k in (("q/o", 4096, 4096), ("gate/up", 14336, 4096), ("down", 4096, 14336)):
        per = n * k * NUM_SUMS // 8
        copies = max(2, min(16, int(600e6 // per)))
        nbytes = algorithmic_bytes(n, k, NUM_SUMS, GROUP, LINES, 1)
        ws = [tuple(t.to(dev) for t in synth.random_encoding(n, k, NUM_SUMS, GROUP, LINES, seed=c)) for c in range(copies)]
        left = tuple(t.to(dev) for t in synth.random_encoding(1, k, NUM_SUMS, GROUP, 16, seed=99))
        t = _graph_time(lambda i: hip._sbvr_mm_T(*left, *ws[i % copies], none, bvr_len=GROUP), 100)
        rows.append({"op": "_sbvr_mm_T", "linear": tag, "N": n, "K": k, "S": NUM_SUMS, "M": 1, "us": round(t * 1e6, 2),
                     "GBps": round(nbytes / t / 1e9, 1), "frac_of_hbm_peak": round(nbytes / t / 1e9 / HBM_PEAK_GBS, 4)})
        del ws
        torch.cuda.empty_cache()
        # trans=True: the encoded tensor is W^T (k rows of n columns, groups along n)
        wt = [tuple(t.to(dev) for t in synth.random_encoding(k, n, NUM_SUMS, GROUP, LINES, seed=c)) for c in range(copies)]
        x = torch.randn((1, k), generator=torch.Generator().manual_seed(5)).to(torch.float16).to(dev)
        t = _graph_time(lambda i: hip._sbvr_row_deq_mm_T(x, *wt[i % copies], none, 0, bvr_len=GROUP), 100)
        rows.append({"op": "_sbvr_row_deq_mm_T", "linear": tag, "N": n, "K": k, "S": NUM_SUMS, "M": 1,
                     "us": round(t * 1e6, 2), "GBps": round(nbytes / t / 1e9, 1),
                     "frac_of_hbm_peak": round(nbytes / t / 1e9 / HBM_PEAK_GBS, 4)})
        del wt
        torch.cuda.empty_cache()
    return rows


def prefill_leg():
    """Prefill GEMM at the 70B-width linears, S=4, G=128: dense-equivalent TFLOP/s against
    the fp16 MFMA peak."""
    import torch
    from sbvr import synth, hip
    dev = torch.device("cuda:0")
    rows = []
    for n, k in ((28672, 8192), (8192, 28672)):
        w = tuple(t.to(dev) for t in synth.random_encoding(n, k, NUM_SUMS, GROUP, LINES, seed=1))
        dense = (torch.randn((n, k), generator=torch.Generator().manual_seed(5)) * 0.02).to(torch.float16).to(dev)
        for m in (256, 512, 1024, 2048):
            x = torch.randn((m, k), generator=torch.Generator().manual_seed(6)).to(torch.float16).to(dev)
            out = torch.empty((m, n), dtype=torch.float16, device=dev)
            t = _graph_time(lambda i: hip._sbvr_linear_f16(x, *w, None, GROUP, out=out), 5)
            flops = 2.0 * m * n * k
            # for scale: the library's GEMM on ready-made dense fp16 weights of the same shape (nothing to decode)
            for _ in range(2):
                torch.matmul(x, dense.t(), out=out)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(5):
                torch.matmul(x, dense.t(), out=out)
            e1.record()
            torch.cuda.synchronize()
            t_dense = e0.elapsed_time(e1) * 1e-3 / 5
            rows.append({"N": n, "K": k, "M": m, "us": round(t * 1e6, 1), "TFLOPs": round(flops / t / 1e12, 1),
                         "frac_of_fp16_mfma_peak": round(flops / t / 1e12 / 2500.0, 4),
                         "dense_fp16_library_gemm_us": round(t_dense * 1e6, 1)})
        del w, dense
        torch.cuda.empty_cache()
    return rows


def cpu_decode_estimate(threads, per_shape_budget_s=1.5):
    """Time of the linears of one token on the host: the reference CPU kernel (x86 port)
    on each of the seven layer shapes, times 32 layers.  Excludes head, norms and attention."""
    import numpy as np
    from oracle import sbvr_oracle as O

    rng = np.random.default_rng(11)
    shapes = {"q/o": (4096, 4096, 2), "k/v": (1024, 4096, 2), "gate/up": (14336, 4096, 2), "down": (4096, 14336, 1)}
    total = 0.0
    detail = {}
    for name, (n, k, count) in shapes.items():
        l_bvr = O.np_planes_to_default(rng.integers(0, 256, size=(4, k // 8), dtype=np.uint8), 1)
        l_idx = rng.integers(0, 16, size=(k // GROUP, 1)).astype(np.uint8)
        l_cache = (rng.standard_normal((16, 4)) * 0.3).astype(np.float16)
        r_bvr = O.np_planes_to_v1(rng.integers(0, 256, size=(NUM_SUMS, n * k // 8), dtype=np.uint8), n)
        r_idx = rng.integers(0, LINES, size=(k // GROUP, n)).astype(np.uint8)
        r_cache = (rng.standard_normal((LINES, NUM_SUMS)) * 0.02).astype(np.float16)
        args = (l_bvr, l_idx, l_cache, r_bvr, r_idx, r_cache, GROUP)
        probe = O.PORT.time_mm_T_v1(*args, warmup=2, iters=3)
        iters = max(5, int(per_shape_budget_s / max(probe, 1e-6)))
        t = O.PORT.time_mm_T_v1(*args, warmup=3, iters=iters)
        detail[name] = round(t * 1e6, 1)
        total += count * t
    per_token = 32 * total
    return {"tokens_per_s_linears_only": round(1.0 / per_token, 2), "ms_per_token_linears_only": round(per_token * 1e3, 2),
            "us_per_gemv": detail, "cores": threads}


def cpu_leg(budget_s=12.0, decode=True):
    """The reference's CPU algorithm (both operands encoded, popcount of AND,
    fp16 coefficient products) ported to x86, timed on this host for about
    `budget_s` seconds at the same shape."""
    import numpy as np
    from oracle import sbvr_oracle as O

    rng = np.random.default_rng(7)
    threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    threads = O.PORT.init_pool(threads)

    def planes(rows, s):
        return rng.integers(0, 256, size=(s, rows * K_IN // 8), dtype=np.uint8)

    s_l = 4
    l_bvr = O.np_planes_to_default(planes(1, s_l), 1)
    l_idx = rng.integers(0, 16, size=(K_IN // GROUP, 1)).astype(np.uint8)
    l_cache = (rng.standard_normal((16, s_l)) * 0.3).astype(np.float16)
    r_bvr = O.np_planes_to_v1(planes(N_OUT, NUM_SUMS), N_OUT)
    r_idx = rng.integers(0, LINES, size=(K_IN // GROUP, N_OUT)).astype(np.uint8)
    r_cache = (rng.standard_normal((LINES, NUM_SUMS)) * 0.02).astype(np.float16)
    args = (l_bvr, l_idx, l_cache, r_bvr, r_idx, r_cache, GROUP)
    probe = O.PORT.time_mm_T_v1(*args, warmup=2, iters=3)
    iters = max(10, int(budget_s / max(probe, 1e-6)))
    per_call = O.PORT.time_mm_T_v1(*args, warmup=10, iters=iters)
    decode_cpu = cpu_decode_estimate(threads) if decode else None
    O.PORT.finalize_pool()
    # the same kernel on one thread (a shorter sample), and the fp16 GEMV of torch's CPU backend, which the
    # reference's own benchmark times beside its kernel (test_sbvr.py:663-668)
    O.PORT.init_pool(1)
    probe1 = O.PORT.time_mm_T_v1(*args, warmup=1, iters=2)
    one_thread = O.PORT.time_mm_T_v1(*args, warmup=2, iters=max(3, int(3.0 / max(probe1, 1e-6))))
    O.PORT.finalize_pool()
    import torch
    torch.set_num_threads(threads)
    w16 = (torch.randn((N_OUT, K_IN), generator=torch.Generator().manual_seed(3)) * 0.02).to(torch.float16)
    x16 = torch.randn((1, K_IN), generator=torch.Generator().manual_seed(4)).to(torch.float16)
    for _ in range(3):
        torch.matmul(x16, w16.t())
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < 2.0:
        torch.matmul(x16, w16.t())
        reps += 1
    torch_gemv = (time.perf_counter() - t0) / reps
    nbytes = algorithmic_bytes(N_OUT, K_IN, NUM_SUMS, GROUP, LINES, BATCH)
    return {
        "value": round(nbytes / per_call / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "us_per_gemv": round(per_call * 1e6, 1),
        "isa": O.PORT.isa(),
        "one_thread_us": round(one_thread * 1e6, 1),
        "torch_fp16_gemv_us": round(torch_gemv * 1e6, 1),
        "torch_fp16_gemv_threads": threads,
        "sample": f"{iters} timed calls (10 warm-ups) of the full 4096->14336 GEMV, both operands SBVR-encoded "
                  f"(S_l=4, S_r=4, group 128), reference CPU algorithm ported to x86, N split over {threads} pinned threads",
        "decode": decode_cpu,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-decode", action="store_true", help="skip the 8B decode tokens/s leg")
    ap.add_argument("--decode-only", action="store_true", help="run only the 8B decode leg and print its figures")
    ap.add_argument("--sweep", action="store_true",
                    help="run only the layer-shape / batch / plane-count sweep of the decode kernel and print it")
    ap.add_argument("--shape", default=None, metavar="NxK[xM]",
                    help="run only the linear of this shape (4 planes, groups of 128, batch M, default 1) and print it")
    ap.add_argument("--prefill", action="store_true", help="run only the prefill GEMM sizes and print them")
    ap.add_argument("--other-ops", action="store_true",
                    help="run only _sbvr_mm_T and _sbvr_row_deq_mm_T at the layer shapes and print them")
    ap.add_argument("--attention-o", action="store_true",
                    help="run only the decoder's attention + o projection, as one launch and as two, and print both")
    ap.add_argument("--eager", type=int, default=0, metavar="N",
                    help="with --attention-o: N eager launches of the one-launch form per position instead of timed "
                         "graph replays (for counter passes of a profiler)")
    ap.add_argument("--stream-floor", action="store_true",
                    help="run only the launch that makes the gate GEMV's memory requests and nothing else "
                         "(sbvr_hip_linear_f16_stream_floor) and print its time beside the kernel's")
    ap.add_argument("--read-floor", action="store_true",
                    help="run only the launches that read 28 MiB and do nothing else, over grids, depths and access "
                         "patterns (sbvr_hip_read_floor), and print them")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy, the known-size kernel that "
                         "hardware byte counters are scaled by when profiling")
    a = ap.parse_args()
    if a.gpus != 1:
        raise SystemExit("bench.py measures one GPU: the path is single-GPU in this build (run with --gpus 1)")

    if a.decode_only:
        print(json.dumps({"metric": "8B decode tokens/s", "decode": decode_leg()}))
        return
    if a.shape:
        dims = [int(v) for v in a.shape.lower().split("x")]
        only = (dims[0], dims[1], dims[2] if len(dims) > 2 else 1)
        print(json.dumps({"metric": "SBVR decode linear, us and GB/s of algorithmic bytes", "sweep": sweep_leg(only)}))
        return
    if a.sweep:
        print(json.dumps({"metric": "SBVR decode linears, us and GB/s of algorithmic bytes", "sweep": sweep_leg()}))
        return
    if a.prefill:
        print(json.dumps({"metric": "SBVR prefill GEMM, dense-equivalent TFLOP/s", "prefill": prefill_leg()}))
        return
    if a.read_floor:
        print(json.dumps({"metric": "read-only launches of the gate shape's plane words, us and GB/s", "read_floor": read_floor_leg()}))
        return
    if a.attention_o:
        print(json.dumps({"metric": "decoder attention + SBVR o projection at the 8B shape, us per layer",
                          "attention_o": attention_o_leg(a.eager)}))
        return
    if a.other_ops:
        print(json.dumps({"metric": "SBVR operator forms of the reference, us and GB/s of algorithmic bytes",
                          "other_ops": other_ops_leg()}))
        return
    if a.calibrate_copy:
        import torch
        src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
    nbytes = algorithmic_bytes(N_OUT, K_IN, NUM_SUMS, GROUP, LINES, BATCH)
    _, floor_t, _, _ = gpu_leg(a.steps, a.warmup, floor=True)
    floor = {
        "what": "the same launch with only its plane-word and index requests (no activations, no arithmetic, no output)",
        "us_per_launch": round(floor_t["median_ms"] * 1e3, 3),
        "us_per_launch_min": round(floor_t["min_ms"] * 1e3, 3),
        "frac_of_hbm_peak": round(nbytes / (floor_t["median_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
    }
    wall_ms, timing, launcher, device = gpu_leg(a.steps, a.warmup)
    global _WEIGHTS
    _WEIGHTS = None                      # (the legs below want the memory)
    reads = read_floor_leg(quick=True)
    read_floor = dict(reads["best"], what="the fastest of a few launches that only read the gate shape's 28 MiB of plane words "
                                          "(sbvr_hip_read_floor; python bench.py --read-floor runs the whole grid of shapes)")
    read_floor["us_for_the_workload_bytes"] = round(nbytes / (read_floor["GBps"] * 1e9) * 1e6, 3)
    if a.stream_floor:
        print(json.dumps({"metric": "SBVR gate GEMV 4096->14336: kernel and its memory-request floor, us per launch",
                          "kernel_us": round(timing["median_ms"] * 1e3, 3), "kernel_us_min": round(timing["min_ms"] * 1e3, 3),
                          "stream_floor": floor,
                          "kernel_over_floor": round(timing["median_ms"] / floor_t["median_ms"], 3)}))
        return
    value = nbytes / (wall_ms * 1e-3) / 1e9
    achieved = nbytes / (timing["median_ms"] * 1e-3) / 1e9
    line = {
        "metric": "SBVR GEMV achieved HBM GB/s (%peak) at 4096x14336; 8B decode tokens/s",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(wall_ms, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 (fp8 x fp4 MFMA plane sums, f32 accumulate)",
        "data": "synthetic",
        "config": {
            "workload": "Llama-3-8B gate linear 4096->14336, batch 1, SBVR 4 bit planes, group 128, "
                        "256 coefficient lines (uint8 idx), fp16 activations",
            "weight_copies_rotated": COPIES,
            "bytes_per_step": nbytes,
            "launcher": launcher,
            "binding": "sbvr._sbvr_hip_ops (PyTorch extension over the C ABI)",
            "device": device,
        },
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "clocks": "value and ms_per_step: host wall clock around one replay of `steps` launches between two "
                  "synchronisations; roofline: HIP events on the launch stream, median over the replays",
        "roofline": {
            "bound": "hbm",
            "kernel": "sbvr_gemv_mfma_kernel",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "us_per_launch": round(timing["median_ms"] * 1e3, 3),
            "us_per_launch_min": round(timing["min_ms"] * 1e3, 3),
            "frac_at_min": round(nbytes / (timing["min_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "launches_timed": timing["launches_timed"],
            "traffic": TRAFFIC_FROM_PROFILE_BYTES,
            "traffic_source": TRAFFIC_PROFILE + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run of this "
                              "command, scaled by a 256 MiB copy; not measured in this run)",
            "stream_floor": floor,
            "read_floor": read_floor,
            "kernel_over_read_floor": round(timing["median_ms"] * 1e3 / read_floor["us_for_the_workload_bytes"], 3),
        },
    }
    if not a.no_decode:
        line["decode"] = decode_leg()
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_leg(decode=not a.no_decode)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
