"""A Llama-shaped decoder in plain torch around QuantizedLinear, for the end-to-end configuration of bench.py.

Nothing here is part of the quantized-linear library: it is the smallest model that exercises the reference's
use (README.md:46-59: build a model, Bitween(...).quantize(rtn=True, ignore_layers=[...]), generate) with the
attention / norm / rotary / cache glue written as a few torch ops per layer, so that one decode step can be
captured in a HIP graph and replayed without the Python interpreter in the way:

  * RMSNorm (torch.nn.functional.rms_norm), rotary embedding over q and k together in four elementwise
    kernels, attention of the one new row over a preallocated KV cache as two batched products and a softmax
    (an additive bias hides the unwritten tail; the prompt goes through scaled_dot_product_attention), SwiGLU;
    embeddings and lm_head stay float16 (ignore_layers=['lm_head', 'embed_tokens'], README.md:58);
  * the position, the current token and the generated tokens live in device tensors that the step itself
    advances, so replaying the captured step N times generates N tokens with no host round trip.

With use_hip_glue() the decode step runs the same arithmetic through five small HIP kernels of this benchmark
(bench_decoder_glue.hip: residual add + RMSNorm, rotary + cache write, split attention + combine, SwiGLU) instead
of about seventeen torch kernels per layer; the prompt always goes through the torch ops.

Random weights N(0, 0.02) from a seed (no checkpoint can be fetched); the numbers say how fast the path runs,
not what it generates.
"""
import ctypes
import os
import subprocess
import time

import torch
import torch.nn as nn
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
GLUE_SRC = os.path.join(HERE, "bench_decoder_glue.hip")
GLUE_LIB = os.path.join(HERE, "bench_decoder_glue.so")


def build_glue():
    """hipcc the glue kernels for gfx950 into bench_decoder_glue.so next to this file (works without a GPU)."""
    cmd = [os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-o", GLUE_LIB, GLUE_SRC]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stderr)
    return GLUE_LIB


class HipGlue:
    """ctypes front of bench_decoder_glue.so for one Decoder: every call launches on torch's current stream."""

    def __init__(self, model, splits=12):
        if not os.path.exists(GLUE_LIB):
            raise RuntimeError(f"{GLUE_LIB} is not built: run bench_decoder.build_glue() (or __graft_entry__.build()) first")
        lib = ctypes.CDLL(GLUE_LIB)
        vp, i32, f32 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_float
        lib.glue_add_rmsnorm.argtypes = [vp, vp, vp, vp, vp, i32, f32, vp]
        lib.glue_rope_kv.argtypes = [vp] * 9 + [i32, i32, i32, vp]
        lib.glue_attention.argtypes = [vp] * 6 + [i32, i32, i32, i32, f32, vp]
        lib.glue_silu_mul.argtypes = [vp, vp, vp, i32, vp]
        lib.glue_rope_attention.argtypes = [vp] * 10 + [i32, i32, i32, i32, f32, vp]
        for f in (lib.glue_add_rmsnorm, lib.glue_rope_kv, lib.glue_attention, lib.glue_rope_attention, lib.glue_silu_mul):
            f.restype = i32
        self.lib, self.m, self.splits = lib, model, splits
        dev = model.lm_head.weight.device
        self.index = dev.index if dev.index is not None else torch.cuda.current_device()
        self.part = torch.empty(model.heads * splits * (model.head_dim + 2), dtype=torch.float32, device=dev)

    def _stream(self):
        return torch._C._cuda_getCurrentRawStream(self.index)

    @staticmethod
    def _ok(st, what):
        if st:
            raise RuntimeError(f"{what} refused its arguments or failed to launch (status {st})")

    def add_rmsnorm(self, x, delta, gamma):
        m = self.m
        x_out, h = torch.empty_like(x), torch.empty_like(x)
        self._ok(self.lib.glue_add_rmsnorm(x.data_ptr(), None if delta is None else delta.data_ptr(), gamma.data_ptr(), x_out.data_ptr(),
                                           h.data_ptr(), m.hidden, m.eps, self._stream()), "glue_add_rmsnorm")
        return x_out, h

    def rope_kv(self, q, k, v, layer):
        m = self.m
        q_out = torch.empty(1, m.hidden, dtype=torch.float16, device=q.device)
        self._ok(self.lib.glue_rope_kv(q.data_ptr(), k.data_ptr(), v.data_ptr(), m.cos.data_ptr(), m.sin.data_ptr(), m.pos.data_ptr(),
                                       q_out.data_ptr(), m.kv[layer, 0].data_ptr(), m.kv[layer, 1].data_ptr(), m.heads, m.head_dim,
                                       m.max_len, self._stream()), "glue_rope_kv")
        return q_out

    def attention(self, q, layer):
        m = self.m
        o = torch.empty(1, m.hidden, dtype=torch.float16, device=q.device)
        self._ok(self.lib.glue_attention(q.data_ptr(), m.kv[layer, 0].data_ptr(), m.kv[layer, 1].data_ptr(), m.pos.data_ptr(),
                                         self.part.data_ptr(), o.data_ptr(), m.heads, m.head_dim, m.max_len, self.splits,
                                         m.head_dim ** -0.5, self._stream()), "glue_attention")
        return o

    def rope_attention(self, q, k, v, layer):
        """rope_kv and attention in one call (two launches)."""
        m = self.m
        o = torch.empty(1, m.hidden, dtype=torch.float16, device=q.device)
        self._ok(self.lib.glue_rope_attention(q.data_ptr(), k.data_ptr(), v.data_ptr(), m.cos.data_ptr(), m.sin.data_ptr(), m.pos.data_ptr(),
                                              m.kv[layer, 0].data_ptr(), m.kv[layer, 1].data_ptr(), self.part.data_ptr(), o.data_ptr(),
                                              m.heads, m.head_dim, m.max_len, self.splits, m.head_dim ** -0.5, self._stream()),
                 "glue_rope_attention")
        return o

    def silu_mul(self, gate, up):
        out = torch.empty_like(gate)
        self._ok(self.lib.glue_silu_mul(gate.data_ptr(), up.data_ptr(), out.data_ptr(), gate.numel(), self._stream()), "glue_silu_mul")
        return out


class Attention(nn.Module):
    def __init__(self, hidden, heads):
        super().__init__()
        self.heads, self.head_dim = heads, hidden // heads
        self.q_proj = nn.Linear(hidden, hidden, bias=False)
        self.k_proj = nn.Linear(hidden, hidden, bias=False)
        self.v_proj = nn.Linear(hidden, hidden, bias=False)
        self.o_proj = nn.Linear(hidden, hidden, bias=False)


class MLP(nn.Module):
    def __init__(self, hidden, inter):
        super().__init__()
        self.gate_proj = nn.Linear(hidden, inter, bias=False)
        self.up_proj = nn.Linear(hidden, inter, bias=False)
        self.down_proj = nn.Linear(inter, hidden, bias=False)


class Layer(nn.Module):
    def __init__(self, hidden, heads, inter):
        super().__init__()
        self.self_attn = Attention(hidden, heads)
        self.mlp = MLP(hidden, inter)
        self.input_layernorm = nn.Parameter(torch.ones(hidden))
        self.post_attention_layernorm = nn.Parameter(torch.ones(hidden))


class Decoder(nn.Module):
    """model.layers.{i}.self_attn.{q,k,v,o}_proj / mlp.{gate,up,down}_proj, embed_tokens, norm, lm_head: the module
    names of a Llama checkpoint, so that per-layer precision maps written for one apply to the other."""

    def __init__(self, layers=32, hidden=4096, heads=32, inter=11008, vocab=32000, max_len=768, eps=1e-5):
        super().__init__()
        self.hidden, self.heads, self.head_dim, self.max_len, self.eps = hidden, heads, hidden // heads, max_len, eps
        self.embed_tokens = nn.Embedding(vocab, hidden)
        self.layers = nn.ModuleList([Layer(hidden, heads, inter) for _ in range(layers)])
        self.norm = nn.Parameter(torch.ones(hidden))
        self.lm_head = nn.Linear(hidden, vocab, bias=False)
        self.glue = None

    def use_hip_glue(self, splits=12):
        """Run step() through the HIP glue kernels (head dimension 128, float16 parameters; call after alloc_state)."""
        self.glue = HipGlue(self, splits)

    @torch.no_grad()
    def init_weights(self, seed):
        gen = torch.Generator(device=self.lm_head.weight.device).manual_seed(seed)
        for p in self.parameters():
            if p.dim() > 1:
                p.normal_(0, 0.02, generator=gen)

    def alloc_state(self):
        """KV cache [layer][k|v][1, heads, max_len, head_dim], rotary table, and the device-side counters."""
        dev = self.lm_head.weight.device
        self.kv = torch.zeros(len(self.layers), 2, 1, self.heads, self.max_len, self.head_dim, dtype=torch.float16, device=dev)
        half = self.head_dim // 2
        inv = 1.0 / (10000.0 ** (torch.arange(0, half, device=dev, dtype=torch.float32) / half))
        ang = torch.arange(self.max_len, device=dev, dtype=torch.float32)[:, None] * inv[None, :]
        self.cos, self.sin = ang.cos().to(torch.float16), ang.sin().to(torch.float16)   # [max_len, head_dim / 2]
        self.pos = torch.zeros(1, dtype=torch.int64, device=dev)          # position of the token being fed
        self.tok = torch.zeros(1, 1, dtype=torch.int64, device=dev)       # the token being fed
        self.out = torch.zeros(self.max_len, dtype=torch.int64, device=dev)   # out[p] = token chosen after position p
        self.key_index = torch.arange(self.max_len, device=dev)

    def _rope(self, qk):
        """qk [T, 2 * heads, head_dim] float16 -> the same with pairs (x_i, x_{i + d/2}) rotated by the angle of the
        row's position, in four elementwise kernels (cos / sin come as [T, 1, head_dim / 2] float16)."""
        d = self.head_dim // 2
        x1, x2 = qk[..., :d], qk[..., d:]
        out = torch.empty_like(qk)
        o1, o2 = out[..., :d], out[..., d:]
        torch.mul(x1, self._cos, out=o1)
        o1.addcmul_(x2, self._sin, value=-1)
        torch.mul(x2, self._cos, out=o2)
        o2.addcmul_(x1, self._sin)
        return out

    def _layer(self, i, layer, x, pos_index, bias, causal):
        t = x.shape[0]
        att = layer.self_attn
        h = F.rms_norm(x, (self.hidden,), layer.input_layernorm, self.eps)
        q, k, v = att.q_proj(h), att.k_proj(h), att.v_proj(h)
        if (q.untyped_storage().data_ptr() == k.untyped_storage().data_ptr() and q.data_ptr() + 2 * q.shape[-1] == k.data_ptr()
                and q.stride(0) == k.stride(0)):
            qk = torch.as_strided(q, (t, 2 * self.hidden), (q.stride(0), 1))     # q and k came out of one fused launch
        else:
            qk = torch.cat([q, k], dim=-1)
        qk = self._rope(qk.view(t, 2 * self.heads, self.head_dim))
        q, k = qk[:, : self.heads], qk[:, self.heads:]
        v = v.view(t, self.heads, self.head_dim)
        kc, vc = self.kv[i, 0], self.kv[i, 1]
        kc.index_copy_(2, pos_index, k.transpose(0, 1)[None])
        vc.index_copy_(2, pos_index, v.transpose(0, 1)[None])
        if causal:                                                       # prefill from an empty cache
            o = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                               is_causal=True)[0].transpose(0, 1)
        else:
            # one query row against the whole cache (bias hides the unwritten tail): two small batched products and
            # a softmax - the fused attention kernel takes 45 us for this, these three together about 15
            scores = torch.baddbmm(bias, q.transpose(0, 1), kc[0].transpose(1, 2), alpha=self.head_dim ** -0.5)
            o = torch.bmm(torch.softmax(scores, dim=-1, dtype=torch.float32).to(torch.float16), vc[0]).transpose(0, 1)
        x = x + att.o_proj(o.reshape(t, self.hidden))
        h = F.rms_norm(x, (self.hidden,), layer.post_attention_layernorm, self.eps)
        return x + layer.mlp.down_proj(F.silu(layer.mlp.gate_proj(h)) * layer.mlp.up_proj(h))

    @torch.no_grad()
    def prefill(self, ids):
        """ids [T] from an empty cache; leaves pos = T and tok = the greedy next token."""
        t = ids.shape[0]
        x = self.embed_tokens(ids)
        pos_index = torch.arange(t, device=ids.device)
        self._cos, self._sin = self.cos[:t, None, :], self.sin[:t, None, :]
        for i, layer in enumerate(self.layers):
            x = self._layer(i, layer, x, pos_index, None, True)
        logits = self.lm_head(F.rms_norm(x[-1:], (self.hidden,), self.norm, self.eps))
        self.tok.copy_(logits.argmax(-1, keepdim=True))
        self.pos.fill_(t)
        self.out.index_copy_(0, self.pos - 1, self.tok[0])
        return logits

    def _step_hip(self):
        """step() with the glue of a layer in five launches: the residual add of a block is folded into the RMSNorm
        that follows it, the rotary embedding and the cache write into the attention."""
        g = self.glue
        x = self.embed_tokens(self.tok[0])
        delta = None
        for i, layer in enumerate(self.layers):
            att, mlp = layer.self_attn, layer.mlp
            x, h = g.add_rmsnorm(x, delta, layer.input_layernorm)
            delta = att.o_proj(g.rope_attention(att.q_proj(h), att.k_proj(h), att.v_proj(h), i))
            x, h = g.add_rmsnorm(x, delta, layer.post_attention_layernorm)
            delta = mlp.down_proj(g.silu_mul(mlp.gate_proj(h), mlp.up_proj(h)))
        _, h = g.add_rmsnorm(x, delta, self.norm)
        return self.lm_head(h)

    @torch.no_grad()
    def step(self):
        """Feed tok at position pos, choose the next token greedily, advance: every tensor it touches is static, so
        the call can be captured once and replayed."""
        if self.glue is not None:
            logits = self._step_hip()
            self.tok.copy_(logits.argmax(-1, keepdim=True))
            self.out.index_copy_(0, self.pos, self.tok[0])
            self.pos.add_(1)
            return logits
        x = self.embed_tokens(self.tok[0])
        self._cos, self._sin = self.cos.index_select(0, self.pos)[:, None, :], self.sin.index_select(0, self.pos)[:, None, :]
        # additive attention bias [heads, 1, max_len]: 0 up to the current position, -inf behind it
        bias = torch.where(self.key_index <= self.pos, 0.0, float("-inf")).to(torch.float16).expand(self.heads, 1, self.max_len)
        for i, layer in enumerate(self.layers):
            x = self._layer(i, layer, x, self.pos, bias, False)
        logits = self.lm_head(F.rms_norm(x, (self.hidden,), self.norm, self.eps))
        self.tok.copy_(logits.argmax(-1, keepdim=True))
        self.out.index_copy_(0, self.pos, self.tok[0])
        self.pos.add_(1)
        return logits


def mixed_recipe(layers):
    """The per-layer widths a Gradual run would hand over (BASELINE configs[4]): attention 8-bit g128, MLP 4-bit
    g128, down_proj of the two first and two last layers 2-bit g32."""
    recipe = {}
    for i in range(layers):
        recipe["layers.%d.self_attn" % i] = (8, 128)
        recipe["layers.%d.mlp" % i] = (4, 128)
    for i in sorted({0, 1, layers - 2, layers - 1}):
        recipe["layers.%d.mlp.down_proj" % i] = (2, 32)
    return recipe


def capture_step(model):
    """One decode step as a HIP graph (warmed on a side stream first, as torch asks)."""
    state = (model.pos.clone(), model.tok.clone(), model.out.clone(), model.kv.clone())
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        model.step()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        model.step()
    # capture ran nothing, the warm-up ran one step: put the state back where it was
    model.pos.copy_(state[0]); model.tok.copy_(state[1]); model.out.copy_(state[2]); model.kv.copy_(state[3])
    torch.cuda.synchronize()
    return graph


def generate(model, ids, new_tokens, graph=None):
    """Greedy decode of `new_tokens` after the prompt `ids`; returns (prefill ms, decode seconds, tokens [new_tokens])."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    model.prefill(ids)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for _ in range(new_tokens - 1):
        if graph is None:
            model.step()
        else:
            graph.replay()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    t = ids.shape[0]
    return (t1 - t0) * 1e3, t2 - t1, model.out[t - 1: t - 1 + new_tokens].clone()
