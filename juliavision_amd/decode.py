"""Decode-step plumbing: device-resident KV cache and a replayable decoder-layer step.

The reference keeps the cache functional -- the exported step returns a new cache
and ``decodestep!`` copies it back (WhisperRunner/src/decode.jl:186-203) -- and
pays ~63 us of host dispatch per op (plans/whisper-decoder.md:161-166).  Here the
cache is written in place at a position that lives in device memory, so the work
a step enqueues does not depend on the position and one captured graph serves
every token (the reference's ``Lava.capture/replay``, plans/whisper-decoder.md:244-259).

Shapes follow torch order as in the reference's ``KVCache`` (decode.jl:52-58):
``self_k``/``self_v`` ``(layers, B, H, max_target, E)``, ``cross_k``/``cross_v``
``(layers, B, H, src_len, E)``.
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Callable, List, Optional

import torch

from . import _lib as L
from .kernels import Ctx, DeclineError, Workspace, _strides_elbh, layernorm_, ln_matmul_, matmul_, matmul_heads_, relayout_weight, sdpa, sdpa_append


# Fold the cache write into the self-attention launch where the one-launch kernel covers the shape.
FUSE_APPEND = True


class KVCache:
    """The decoder's state between steps (KVCache, decode.jl:52-58), fixed capacity.

    ``length`` is an int32 ``(B,)`` device tensor: how many self-attention slots
    are live per batch row (the reference's host-side ``position``)."""

    def __init__(self, layers: int, batch: int, heads: int, headdim: int, *, max_target: int = 448, src_len: int = 1500,
                 device="cuda"):
        z = lambda n: torch.zeros((layers, batch, heads, n, headdim), dtype=torch.float16, device=device)
        self.self_k, self.self_v = z(max_target), z(max_target)
        self.cross_k, self.cross_v = z(src_len), z(src_len)
        self.length = torch.zeros((batch,), dtype=torch.int32, device=device)
        self.max_target = max_target
        self.layers, self.batch, self.heads, self.headdim = layers, batch, heads, headdim

    def reset(self):
        self.length.zero_()

    def advance(self, ctx: Ctx, delta: int = 1):
        """length += delta on the device (``c.position += 1``, decode.jl:201).  The counter stops at ``max_target + 1``:
        a step that finds the cache full stores nothing, attends over the stored keys and leaves that mark, which
        ``overflowed()`` reads back (the reference's greedy loop bounds its token count on the host, decode.jl:206-230; a
        replayed graph has no host in the loop, so the device keeps the evidence instead)."""
        rc = L.init().mi_kv_advance(self.length.data_ptr(), self.batch, int(delta), self.max_target + 1, ctx.stream)
        if rc != L.OK:
            raise DeclineError("mi_kv_advance", rc)

    def overflowed(self) -> bool:
        """True if some row was stepped past ``max_target`` since the last ``reset()`` (synchronises with the device)."""
        return bool((self.length > self.max_target).any().item())

    def fill_cross(self, ctx: Ctx, layer: int, enc: torch.Tensor, wk, bk, wv, bv):
        """Project the encoder output into ``layer``'s cross-attention K/V, once per window (fillcross!, decode.jl:173-177:
        the ``whispercross`` graph's two matmuls per layer).  ``enc``: ``(B, src_len, d)`` fp16; ``wk``, ``wv``: ``(d, H*E)``
        weights in either memory layout; ``bk``, ``bv``: ``(H*E,)`` or None.  The GEMMs write the cache's head-major rows
        themselves: no intermediate, no permute, no copy."""
        if enc.dim() != 3 or enc.shape[0] != self.batch or enc.shape[1] != self.cross_k.shape[3]:
            raise DeclineError("fill_cross: enc must be (B, src_len, d)", L.DECLINE_OPERANDS)
        for store, w, bias in ((self.cross_k, wk, bk), (self.cross_v, wv, bv)):
            for b in range(self.batch):
                matmul_heads_(ctx, store[layer, b], w, enc[b], bias)

    def append(self, ctx: Ctx, layer: int, k_new: torch.Tensor, v_new: torch.Tensor):
        """Write the new token's K/V rows ``(B,H,1,E)`` into slot ``length-1`` of ``layer``."""
        ck, cv = self.self_k[layer], self.self_v[layer]
        if k_new.shape != (self.batch, self.heads, 1, self.headdim) or v_new.shape != k_new.shape:
            raise DeclineError("kv append: new rows must be (B,H,1,E)", L.DECLINE_OPERANDS)
        if k_new.dtype != torch.float16 or v_new.dtype != torch.float16 or k_new.stride() != v_new.stride():
            raise DeclineError("kv append: fp16 rows with equal strides", L.DECLINE_OPERANDS)
        rc = L.init().mi_kv_append_f16(ck.data_ptr(), cv.data_ptr(), _strides_elbh(ck), self.max_target,
                                       k_new.data_ptr(), v_new.data_ptr(), _strides_elbh(k_new), self.length.data_ptr(),
                                       self.headdim, self.heads, self.batch, ctx.stream)
        if rc != L.OK:
            raise DeclineError("mi_kv_append_f16", rc)


@dataclass
class DecoderLayerWeights:
    """One pre-LN decoder layer.  Linear weights are ``(K, F)`` tensors in either
    memory layout (``[K][F]`` as the reference's hoisted form, or a transposed
    view of ``[F][K]``); biases ``(F,)``."""
    ln1_g: torch.Tensor
    ln1_b: torch.Tensor
    wqkv: torch.Tensor
    bqkv: torch.Tensor
    wo: torch.Tensor
    bo: torch.Tensor
    ln2_g: torch.Tensor
    ln2_b: torch.Tensor
    wq_c: torch.Tensor
    bq_c: torch.Tensor
    wo_c: torch.Tensor
    bo_c: torch.Tensor
    ln3_g: torch.Tensor
    ln3_b: torch.Tensor
    w1: torch.Tensor
    b1: torch.Tensor
    w2: torch.Tensor
    b2: torch.Tensor

    LINEARS = ("wqkv", "wo", "wq_c", "wo_c", "w1", "w2")

    def k_contiguous(self, ctx: Ctx) -> "DecoderLayerWeights":
        """The same layer with every linear weight held as ``[F][K]`` memory (a transposed ``(K, F)`` view): what the
        decode-sized kernels stream fastest -- one launch per linear instead of K-slices plus a sum.  Done once at load
        with the layout kernel; weights that already lie that way are kept as they are."""
        out = {}
        for name in self.LINEARS:
            w = getattr(self, name)
            if w.stride(0) == 1:                           # already [F][K]
                out[name] = w
                continue
            out[name] = relayout_weight(ctx, w)
        return replace(self, **out)


class DecodeBuffers:
    """Activation slots of one layer step, allocated once (the planner's slab, plan.jl:29)."""

    def __init__(self, batch: int, d_model: int, ffn: int, device="cuda"):
        e = lambda n: torch.empty((batch, n), dtype=torch.float16, device=device)
        self.h, self.qkv, self.att, self.x1 = e(d_model), e(3 * d_model), e(d_model), e(d_model)
        self.qc, self.catt, self.x2, self.f = e(d_model), e(d_model), e(d_model), e(ffn)


def decoder_layer_step(ctx: Ctx, W: DecoderLayerWeights, cache: KVCache, layer: int, x: torch.Tensor, out: torch.Tensor,
                       buf: DecodeBuffers, eps: float = 1e-5):
    """One token through one decoder layer: self-attention over the cache (the new
    row appended in place first), cross-attention over the window's encoder K/V,
    GELU MLP; the three layer norms ride in the prologues of the GEMVs that read
    them (batch <= 4; separate launches above), the residuals in the epilogues.  ``cache.advance`` must have
    run once for this step.  ``x``, ``out``: ``(B, d_model)`` fp16."""
    B, d = x.shape
    H, E = cache.heads, cache.headdim
    heads = lambda t: t.view(B, H, 1, E)
    def normed_linear(dst, w, src, g, b_, bias, epi="none"):
        # every workgroup of the folded form recomputes the row statistics: worth it for a few rows
        # (one launch less per norm), not for eight
        ctx.ws.reset()
        if B <= 4:
            ln_matmul_(ctx, dst, w, src, g, b_, eps, bias, epi=epi)
        else:
            layernorm_(ctx, buf.h, None, None, src, g, b_, d, eps)
            matmul_(ctx, dst, w, buf.h, bias, epi=epi)

    normed_linear(buf.qkv, W.wqkv, x, W.ln1_g, W.ln1_b, W.bqkv)
    q, k_new, v_new = (buf.qkv[:, i * d:(i + 1) * d].unflatten(1, (H, 1, E)) for i in range(3))
    if FUSE_APPEND and E <= 64 and E % 8 == 0:
        # one launch: the new row is key length - 1 and goes into its cache slot on the way
        sdpa_append(ctx, q, cache.self_k[layer], cache.self_v[layer], k_new, v_new, cache.length, out=heads(buf.att))
    else:
        cache.append(ctx, layer, k_new, v_new)
        ctx.ws.reset()
        sdpa(ctx, q, cache.self_k[layer], cache.self_v[layer], out=heads(buf.att), kv_len=cache.length)
    ctx.ws.reset()
    matmul_(ctx, buf.x1, W.wo, buf.att, W.bo, residual=x)
    normed_linear(buf.qc, W.wq_c, buf.x1, W.ln2_g, W.ln2_b, W.bq_c)
    ctx.ws.reset()
    sdpa(ctx, heads(buf.qc), cache.cross_k[layer], cache.cross_v[layer], out=heads(buf.catt))
    ctx.ws.reset()
    matmul_(ctx, buf.x2, W.wo_c, buf.catt, W.bo_c, residual=buf.x1)
    normed_linear(buf.f, W.w1, buf.x2, W.ln3_g, W.ln3_b, W.b1, epi="gelu")
    ctx.ws.reset()
    matmul_(ctx, out, W.w2, buf.f, W.b2, residual=buf.x2)
    return out


class StepGraph:
    """Capture ``fn()`` (kernel launches through the C ABI on the current stream, no
    allocation) once and replay it: hipGraph launch instead of per-op dispatch.
    ``fn`` is run eagerly first so that the workspace has reached its final size."""

    def __init__(self, fn: Callable[[], None], warmup: int = 2, restore: Optional[Callable[[], None]] = None):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):
                fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        if restore is not None:
            restore()
        Workspace.pin_all()                                # the capture holds addresses inside the workspaces from here on
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            fn()
        if restore is not None:
            restore()

    def replay(self):
        self.graph.replay()
