"""A Llama-3-8B-shaped decoder whose seven linears per layer are SBVR-encoded.

Stands in for models/sbvr_llama.py of the reference (a copy of the Hugging Face
Llama whose SBVRLinear, :66-106, is a stub) as the workload of the "8B decode
tokens/s" figure: random-init weights of the real shapes, batch 1, greedy
decoding with a key/value cache.  The linears run through the HIP operator on
synthetic encodings (the encoder would need days for 8B parameters); q|k|v and
gate|up are each one encoded matrix, which is what encoding the concatenated
weight gives.  Embedding and output head stay fp16, as in the reference's
model.  Everything else (norms, rotary embedding, attention over the cache) is
a handful of small kernels in this package's library or plain torch ops.

One decode step is recorded into a HIP graph once and replayed per token (and
sixteen steps into a second graph, replayed per sixteen new tokens); the token
id and the position live on the device, so a replay needs no host work.
"""
import time
from dataclasses import dataclass

import torch

from . import hip


@dataclass
class LlamaShape:
    hidden: int = 4096
    layers: int = 32
    heads: int = 32
    kv_heads: int = 8
    head_dim: int = 128
    ffn: int = 14336
    vocab: int = 128256
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5


def _device_encoding(rows, cols, num_sums, bvr_len, num_lines, seed, device):
    """Random default-layout encoding drawn on the device (see synth.random_encoding)."""
    from .synth import make_lines
    gen = torch.Generator(device=device).manual_seed(seed)
    bvr = torch.randint(-2 ** 31, 2 ** 31, (cols // 32, rows, num_sums), dtype=torch.int32,
                        generator=gen, device=device).view(torch.uint32)
    idx = torch.randint(0, num_lines, (cols // bvr_len, rows), dtype=torch.int32, generator=gen, device=device)
    idx = idx.to(torch.uint8 if num_lines <= 256 else torch.uint16)
    cache = make_lines(num_lines, num_sums, 0.02, seed).to(device)
    return bvr, idx, cache


class _Linear:
    """Encoded (out, in) weight plus a preallocated output row."""

    def __init__(self, out_features, in_features, num_sums, bvr_len, lines, seed, device):
        self.bvr, self.idx, self.cache = _device_encoding(out_features, in_features, num_sums, bvr_len, lines,
                                                          seed, device)
        self.bvr_len = bvr_len
        self.out = torch.empty((1, out_features), dtype=torch.float16, device=device)
        self.bytes = self.bvr.numel() * 4 + self.idx.numel() * self.idx.element_size() + self.cache.numel() * 2

    def __call__(self, x):
        return hip._sbvr_linear_f16(x, self.bvr, self.idx, self.cache, None, self.bvr_len, out=self.out)

    def after_swiglu(self, gate_up):
        """The linear of silu(gate) * up, for gate_up = gate | up."""
        return hip._sbvr_linear_f16_swiglu(gate_up, self.bvr, self.idx, self.cache, None, self.bvr_len, out=self.out)

    def after_add_rmsnorm(self, x, delta, weight, eps, x_out):
        """x_out <- x + delta, then the linear of RMSNorm(x_out) * weight."""
        return hip._sbvr_linear_f16_add_rmsnorm(x, delta, weight, eps, x_out, self.bvr, self.idx, self.cache, None,
                                                self.bvr_len, out=self.out)


class SbvrLlamaDecoder:
    def __init__(self, shape=None, device="cuda:0", num_sums=4, bvr_len=128, lines=256, max_seq=256, seed=0,
                 fused=True, attention_o=None):
        self.shape = s = shape or LlamaShape()
        # fused: the residual add + norm and the SiLU * up run inside the linear that follows them
        # (5 launches per layer instead of 8)
        self.fused = fused
        # attention_o: attention and the o projection in one launch (4 launches per layer) where the shape has
        # that kernel; None = wherever it has.  The caches are then kept in that kernel's blocked element order.
        supported = fused and hip.dec_attention_o_supported(s.heads, s.kv_heads, s.head_dim, max_seq, s.hidden,
                                                            num_sums, bvr_len)
        if attention_o and not supported:
            raise ValueError("attention_o: this shape has no fused attention + projection kernel")
        self.attention_o = supported if attention_o is None else bool(attention_o)
        self.device = dev = torch.device(device)
        self.max_seq = max_seq
        hip._sbvr_hip_init(dev)
        g = torch.Generator(device=dev).manual_seed(seed)
        self.embed = (torch.randn((s.vocab, s.hidden), generator=g, device=dev) * 0.02).to(torch.float16)
        self.lm_head = (torch.randn((s.vocab, s.hidden), generator=g, device=dev) * 0.02).to(torch.float16)
        self.final_norm = torch.ones(s.hidden, dtype=torch.float16, device=dev)
        q_out, kv_out = s.heads * s.head_dim, s.kv_heads * s.head_dim
        self.layers = []
        for l in range(s.layers):
            base = (seed + l) * 7
            layer = {
                "norm1": torch.ones(s.hidden, dtype=torch.float16, device=dev),
                "norm2": torch.ones(s.hidden, dtype=torch.float16, device=dev),
                # one table per original linear: the fused matrices carry 3 and 2 tables
                "qkv": _Linear(q_out + 2 * kv_out, s.hidden, num_sums, bvr_len, 3 * lines, base, dev),
                "o": _Linear(s.hidden, q_out, num_sums, bvr_len, lines, base + 3, dev),
                "gate_up": _Linear(2 * s.ffn, s.hidden, num_sums, bvr_len, 2 * lines, base + 4, dev),
                "down": _Linear(s.hidden, s.ffn, num_sums, bvr_len, lines, base + 6, dev),
                "k": torch.zeros((s.kv_heads, max_seq, s.head_dim), dtype=torch.float16, device=dev),
                "v": torch.zeros((s.kv_heads, max_seq, s.head_dim), dtype=torch.float16, device=dev),
            }
            self.layers.append(layer)
        inv = 1.0 / (s.rope_theta ** (torch.arange(0, s.head_dim, 2, dtype=torch.float64) / s.head_dim))
        ang = torch.arange(max_seq, dtype=torch.float64)[:, None] * inv[None, :]
        self.cos = torch.cos(ang).to(torch.float32).to(dev)       # (max_seq, head_dim/2)
        self.sin = torch.sin(ang).to(torch.float32).to(dev)
        self.rot_now = torch.empty(s.head_dim, dtype=torch.float32, device=dev)   # cos | sin of the current position
        self.x = torch.empty((1, s.hidden), dtype=torch.float16, device=dev)      # residual stream
        self.x_alt = torch.empty((1, s.hidden), dtype=torch.float16, device=dev)  # its other buffer (fused steps)
        self.zero = torch.zeros((1, s.hidden), dtype=torch.float16, device=dev)   # the first layer's "delta"
        self.h = torch.empty((1, s.hidden), dtype=torch.float16, device=dev)      # normed input of a linear
        self.ctx = torch.empty((1, q_out), dtype=torch.float16, device=dev)
        self.act = torch.empty((1, s.ffn), dtype=torch.float16, device=dev)
        self.tok = torch.zeros(1, dtype=torch.int64, device=dev)
        self.pos = torch.zeros(1, dtype=torch.int64, device=dev)
        self.generated = torch.zeros(max_seq, dtype=torch.int64, device=dev)
        self.logits = torch.empty((1, s.vocab), dtype=torch.float16, device=dev)
        self.head_ws = torch.zeros(2, dtype=torch.int64, device=dev)              # cross-workgroup argmax of the head kernel
        self.graph = None
        self.graph_many, self.steps_per_replay = None, 1
        self.stream = torch.cuda.Stream(device=dev)
        # probe(layer, residual): called by an eager fused step with the residual stream as it enters each layer
        # (layer 0: the embedding row) and, as layer == layers, as it enters the final norm; for tests
        self.probe = None

    # -- sizes ---------------------------------------------------------------
    def encoded_bytes(self):
        return sum(l[k].bytes for l in self.layers for k in ("qkv", "o", "gate_up", "down"))

    def bytes_per_token(self):
        """Bytes a decode step has to read: encoded linears, fp16 head, one embedding row."""
        return self.encoded_bytes() + self.lm_head.numel() * 2 + self.shape.hidden * 2

    # -- one token -------------------------------------------------------------
    def step(self, gather=True):
        """One decode step.  gather=False (fused steps with the one-launch end of the step): the input row is
        not looked up, it is what the previous step's last launch left for the token it chose."""
        return self._step_fused(gather) if self.fused else self._step_unfused()

    def _step_unfused(self):
        """8 launches per layer (norm, q|k|v, attention, o, norm, gate|up,
        SiLU*up, down), the residual adds folded into the norms."""
        s = self.shape
        x, h, ctx, act = self.x, self.h, self.ctx, self.act
        torch.index_select(self.embed, 0, self.tok, out=x)            # (1, hidden)
        delta = None
        for layer in self.layers:
            hip.dec_add_rmsnorm(x, delta, layer["norm1"], h, s.rms_eps)
            qkv = layer["qkv"](h)
            hip.dec_attention(qkv, self.cos, self.sin, self.pos, layer["k"], layer["v"], ctx,
                              s.heads, s.kv_heads, s.head_dim, self.rot_now)
            delta = layer["o"](ctx)
            hip.dec_add_rmsnorm(x, delta, layer["norm2"], h, s.rms_eps)
            hip.dec_silu_mul(layer["gate_up"](h), act)
            delta = layer["down"](act)
        hip.dec_add_rmsnorm(x, delta, self.final_norm, h, s.rms_eps)
        logits = torch.matmul(h, self.lm_head.t())                      # (1, vocab)
        hip.dec_argmax_advance(logits, self.tok, self.generated, self.pos, self.cos, self.sin, self.rot_now)
        return logits

    def _step_fused(self, gather=True):
        """One launch for the end of the step (final norm, head, argmax) where the
        hidden size has a kernel, and 5 launches per layer: q|k|v (with the residual add and norm in front),
        attention, o, gate|up (same), down (with SiLU*up in front); 4 with attention and o in one launch
        (self.attention_o).  The residual
        stream alternates between two buffers: a linear reads one and writes the
        sum to the other, since its workgroups do not run in step."""
        s = self.shape
        a, b, ctx = self.x, self.x_alt, self.ctx
        if gather or not hip.dec_head_argmax_supported(s.hidden):
            torch.index_select(self.embed, 0, self.tok, out=a)        # (1, hidden)
        delta = self.zero
        for number, layer in enumerate(self.layers):
            qkv = layer["qkv"].after_add_rmsnorm(a, delta, layer["norm1"], s.rms_eps, b)
            if self.probe is not None:
                self.probe(number, b)
            if self.attention_o:
                o = layer["o"]
                delta = hip.dec_attention_o(qkv, self.cos, self.sin, self.pos, layer["k"], layer["v"], s.heads,
                                            s.kv_heads, s.head_dim, o.bvr, o.idx, o.cache, None, o.bvr_len,
                                            out=o.out, rot_now=self.rot_now)
            else:
                hip.dec_attention(qkv, self.cos, self.sin, self.pos, layer["k"], layer["v"], ctx,
                                  s.heads, s.kv_heads, s.head_dim, self.rot_now)
                delta = layer["o"](ctx)
            gate_up = layer["gate_up"].after_add_rmsnorm(b, delta, layer["norm2"], s.rms_eps, a)
            delta = layer["down"].after_swiglu(gate_up)
        if self.probe is not None:
            self.probe(len(self.layers), (a.float() + delta.float()).to(torch.float16))
        if hip.dec_head_argmax_supported(s.hidden):
            # final norm, head, argmax and position advance in one launch, which also leaves the chosen token's
            # embedding row where the next step starts
            hip.dec_head_argmax(a, delta, self.final_norm, s.rms_eps, self.lm_head, self.logits, self.tok,
                                self.generated, self.pos, self.head_ws, self.cos, self.sin, self.rot_now,
                                embed=self.embed, x_next=a)
            return self.logits
        hip.dec_add_rmsnorm(a, delta, self.final_norm, self.h, s.rms_eps)
        logits = torch.matmul(self.h, self.lm_head.t())                 # (1, vocab)
        hip.dec_argmax_advance(logits, self.tok, self.generated, self.pos, self.cos, self.sin, self.rot_now)
        return logits

    # -- driving ---------------------------------------------------------------
    def capture(self, steps_per_replay=16):
        """Records one step into a HIP graph (after one eager step on the same
        stream, which also creates the operator's workspace for that stream), and
        `steps_per_replay` steps into a second one: token and position live on the
        device, so consecutive steps are the same launches, and between two replays
        the GPU idles for some 8 us that a replay of several steps pays once."""
        with torch.cuda.stream(self.stream):
            self.step()
            torch.cuda.synchronize()
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph, stream=self.stream):
                self.step()
            torch.cuda.synchronize()
            self.graph_many, self.steps_per_replay = None, int(steps_per_replay)
            if self.steps_per_replay > 1:
                self.graph_many = torch.cuda.CUDAGraph()
                with torch.cuda.graph(self.graph_many, stream=self.stream):
                    for _ in range(self.steps_per_replay):
                        self.step(gather=False)     # (each step's input is the choice of the step before)
                torch.cuda.synchronize()
        self.reset()

    def reset(self):
        self.pos.zero_()
        self.tok.zero_()
        self.generated.zero_()
        self.rot_now.copy_(torch.cat((self.cos[0], self.sin[0])))
        for layer in self.layers:
            layer["k"].zero_()
            layer["v"].zero_()
        torch.cuda.synchronize()

    def _advance(self):
        if self.graph is not None:
            self.graph.replay()
        else:
            self.step()

    def generate(self, prompt, new_tokens):
        """Feeds `prompt` (1-D int64 tensor) token by token, then decodes
        `new_tokens` greedily.  Returns (tokens, seconds spent on the new tokens)."""
        if len(prompt) + new_tokens > self.max_seq:
            raise ValueError("prompt + new tokens exceed the cache length")
        self.reset()
        prompt = prompt.to(self.device)
        with torch.cuda.stream(self.stream):
            for t in range(len(prompt)):
                self.tok.copy_(prompt[t:t + 1])
                self._advance()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            left = new_tokens
            many = self.graph_many if self.graph is not None else None
            while many is not None and left >= self.steps_per_replay:
                many.replay()
                left -= self.steps_per_replay
            for _ in range(left):
                self._advance()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
        first = len(prompt) - 1
        return self.generated[first:first + new_tokens + 1].cpu(), dt
