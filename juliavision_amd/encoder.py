"""Encoder-side compositions of the kernel entry points: a pre-LN transformer block and a
ViT-style encoder (patch embedding as convolution-as-GEMM, class token, position
embedding, blocks, final norm).

The reference runs these as exported op graphs (WhisperRunner/src/WhisperRunner.jl's
``encode``; DepthAnythingRunner's ViT-S/14 backbone); here they are the same op sequence
issued directly, seven launches per block: layer norm, one GEMM for the three projections,
fused attention reading q/k/v in place and writing token-major, the output projection with
the residual in its epilogue, layer norm, the GELU GEMM, and the second MLP GEMM with the
residual in its epilogue -- six from the second block on, because that last GEMM also writes
the next block's first norm (``matmul_ln_``).  ``encoder_layer_folded`` is the same block in five launches: the norms
are folded into the linears that read them (``lnfold_prepare`` at load), whose GEMMs run on the raw residual stream with
the row statistics the previous GEMM left behind.  Nothing allocates after construction, so a whole encoder can be
captured and replayed (``decode.StepGraph``).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import torch

from .kernels import (Ctx, LnFoldedLinear, add_, convolution_tokens_, convsize, layernorm_, ln_matmul_, ln_matmul_folds, ln_matmul_pays,
                      lnfold_matmul_, lnfold_prepare, matmul_, matmul_ln_, matmul_rowstats_, rowstats_, rowstats_new, sdpa)


@dataclass
class EncoderLayerWeights:
    """One pre-LN block.  Linear weights are ``(K, F)`` tensors in either memory layout; ``wqkv`` is the
    three projections side by side, ``(d, 3d)``."""
    ln1_g: torch.Tensor
    ln1_b: torch.Tensor
    wqkv: torch.Tensor
    bqkv: torch.Tensor
    wo: torch.Tensor
    bo: torch.Tensor
    ln2_g: torch.Tensor
    ln2_b: torch.Tensor
    w1: torch.Tensor
    b1: torch.Tensor
    w2: torch.Tensor
    b2: torch.Tensor


class EncoderBuffers:
    """Activation slots of one block, allocated once and reused by every layer."""

    def __init__(self, tokens: int, d_model: int, ffn: int, device="cuda"):
        e = lambda n: torch.empty((tokens, n), dtype=torch.float16, device=device)
        self.h, self.qkv, self.att, self.x1, self.f = e(d_model), e(3 * d_model), e(d_model), e(d_model), e(ffn)


def encoder_layer(ctx: Ctx, W: EncoderLayerWeights, x: torch.Tensor, out: torch.Tensor, buf: EncoderBuffers, heads: int,
                  eps: float = 1e-5, act: str = "gelu", *, normed_in: bool = False, next_norm=None):
    """``out = x1 + W2 act(W1 LN2(x1))`` with ``x1 = x + Wo attention(LN1(x))``; ``x``, ``out``: ``(T, d)`` fp16
    (``out`` may be ``x``, which is last read as the output projection's residual).

    ``next_norm = (gamma, beta, dst)``: the norm that reads ``out`` next (the following layer's first norm, or the
    encoder's final one) is written to ``dst`` by this layer's last GEMM (``matmul_ln_``).  ``normed_in``: the
    previous layer did that for this one, ``buf.h`` already holds ``LN1(x)``."""
    T, d = x.shape
    E = d // heads
    # where the norm is cheaper as the prologue of the GEMM that reads it (today: at most 8 token rows), it is one
    fold1 = not normed_in and ln_matmul_folds(T, d, 3 * d) and ln_matmul_pays(T, d, 3 * d)
    fold2 = ln_matmul_folds(T, d, W.w1.shape[1]) and ln_matmul_pays(T, d, W.w1.shape[1])
    if not normed_in and not fold1:
        layernorm_(ctx, buf.h, None, None, x, W.ln1_g, W.ln1_b, d, eps)
    ctx.ws.reset()
    if fold1:
        ln_matmul_(ctx, buf.qkv, W.wqkv, x, W.ln1_g, W.ln1_b, eps, W.bqkv)
    else:
        matmul_(ctx, buf.qkv, W.wqkv, buf.h, W.bqkv)
    # q, k, v are column bands of the projection, heads are 64-wide column bands of those: (B,H,L,E) views, no copy
    q, k, v = (buf.qkv[:, i * d:(i + 1) * d].unflatten(1, (heads, E)).permute(1, 0, 2).unsqueeze(0) for i in range(3))
    ctx.ws.reset()
    sdpa(ctx, q, k, v, out=buf.att.unflatten(1, (heads, E)).permute(1, 0, 2).unsqueeze(0))
    ctx.ws.reset()
    matmul_(ctx, buf.x1, W.wo, buf.att, W.bo, residual=x)
    ctx.ws.reset()
    if fold2:
        ln_matmul_(ctx, buf.f, W.w1, buf.x1, W.ln2_g, W.ln2_b, eps, W.b1, epi=act)
    else:
        layernorm_(ctx, buf.h, None, None, buf.x1, W.ln2_g, W.ln2_b, d, eps)
        matmul_(ctx, buf.f, W.w1, buf.h, W.b1, epi=act)
    ctx.ws.reset()
    if next_norm is None:
        matmul_(ctx, out, W.w2, buf.f, W.b2, residual=buf.x1)
    else:
        matmul_ln_(ctx, out, next_norm[2], W.w2, buf.f, next_norm[0], next_norm[1], eps, W.b2, residual=buf.x1)
    return out


@dataclass
class EncoderLayerFolded:
    """A pre-LN block whose two norms have no pass of their own (``lnfold_prepare``): ``qkv`` is the three projections
    behind the first norm (three planes of one launch), ``fc1`` the first MLP linear behind the second; the output
    projection and the second MLP linear are as they were."""
    qkv: LnFoldedLinear
    fc1: LnFoldedLinear
    wo: torch.Tensor
    bo: torch.Tensor
    w2: torch.Tensor
    b2: torch.Tensor


def fold_layer_norms(ctx: Ctx, W: EncoderLayerWeights) -> EncoderLayerFolded:
    """Once per layer, at load: gamma into the rows of the weights that read the norms, beta into their biases."""
    return EncoderLayerFolded(lnfold_prepare(ctx, W.wqkv, W.ln1_g, W.ln1_b, W.bqkv, planes=3),
                              lnfold_prepare(ctx, W.w1, W.ln2_g, W.ln2_b, W.b1), W.wo, W.bo, W.w2, W.b2)


class FoldedStats:
    """Row statistics of the residual stream at its two points per block (``rowstats_new``), allocated once."""

    def __init__(self, tokens: int, d_model: int, device="cuda"):
        self.x, self.x1 = rowstats_new(tokens, d_model, device), rowstats_new(tokens, d_model, device)


def encoder_layer_folded(ctx: Ctx, W: EncoderLayerFolded, x: torch.Tensor, out: torch.Tensor, buf: EncoderBuffers, st: FoldedStats,
                         heads: int, eps: float = 1e-5, act: str = "gelu", *, stats_out: bool = True):
    """``encoder_layer`` in five launches: neither norm is computed as a pass over the rows.  ``st.x`` must hold the row
    statistics of ``x`` on entry (left by the previous layer's last GEMM, or by ``rowstats_`` for the first layer); on
    return it holds those of ``out`` (unless ``stats_out`` is False: the last layer of a stack).  The linears that read a
    norm run on the raw rows (``lnfold_matmul_``); the two GEMMs that write the residual stream leave its statistics
    behind (``matmul_rowstats_``).  Same op sequence as the reference's exported block (layer_norm, addmm x 3, attention,
    addmm, add, layer_norm, addmm + gelu, addmm, add); held to the parity gate against it, not to the bits of
    ``encoder_layer``."""
    T, d = x.shape
    E = d // heads
    ctx.ws.reset()
    lnfold_matmul_(ctx, buf.qkv, W.qkv, x, st.x, eps)
    q, k, v = (buf.qkv[:, i * d:(i + 1) * d].unflatten(1, (heads, E)).permute(1, 0, 2).unsqueeze(0) for i in range(3))
    ctx.ws.reset()
    sdpa(ctx, q, k, v, out=buf.att.unflatten(1, (heads, E)).permute(1, 0, 2).unsqueeze(0))
    ctx.ws.reset()
    matmul_rowstats_(ctx, buf.x1, st.x1, W.wo, buf.att, W.bo, residual=x)
    ctx.ws.reset()
    lnfold_matmul_(ctx, buf.f, W.fc1, buf.x1, st.x1, eps, epi=act)
    ctx.ws.reset()
    if stats_out:
        matmul_rowstats_(ctx, out, st.x, W.w2, buf.f, W.b2, residual=buf.x1)
    else:
        matmul_(ctx, out, W.w2, buf.f, W.b2, residual=buf.x1)
    return out


@dataclass
class ViTWeights:
    """Patch embedding ``patch_w (d, 3, P, P)``, ``patch_b (d,)``; ``cls (1, d)``; ``pos (1 + patches, d)``;
    the blocks; the final norm."""
    patch_w: torch.Tensor
    patch_b: torch.Tensor
    cls: torch.Tensor
    pos: torch.Tensor
    layers: List[EncoderLayerWeights]
    norm_g: Optional[torch.Tensor] = None
    norm_b: Optional[torch.Tensor] = None


class ViTEncoder:
    """ViT-style encoder over one image: ``tokens = [cls; patches] + pos`` and the blocks in sequence."""

    def __init__(self, W: ViTWeights, image_hw, heads: int, ffn: int, eps: float = 1e-6, device="cuda", *, fold_norms: Optional[Ctx] = None):
        """``fold_norms``: a context to prepare the folded form of every block with (``fold_layer_norms``); the encoder
        then runs five launches a block and computes no block norm as a pass of its own (the final norm stays one)."""
        self.W, self.heads, self.eps = W, heads, eps
        self.folded = None if fold_norms is None else [fold_layer_norms(fold_norms, lw) for lw in W.layers]
        d, cin, P, _ = W.patch_w.shape
        self.P = P
        self.gh, self.gw = convsize(image_hw[0], P, P, 0, 1), convsize(image_hw[1], P, P, 0, 1)
        self.T = 1 + self.gh * self.gw
        if tuple(W.pos.shape) != (self.T, d) or tuple(W.cls.shape) != (1, d):
            raise ValueError(f"pos must be ({self.T}, {d}) and cls (1, {d})")
        f16 = torch.float16
        self.tokens = [torch.empty((self.T, d), dtype=f16, device=device) for _ in range(2)]
        self.out = torch.empty((self.T, d), dtype=f16, device=device)
        self.buf = EncoderBuffers(self.T, d, ffn, device)
        self.stats = None if self.folded is None else FoldedStats(self.T, d, device)

    def embed(self, ctx: Ctx, image: torch.Tensor):
        """``image``: (1, 3, H, W) fp16.  Fills and returns ``tokens[0]``."""
        W, tok = self.W, self.tokens[0]
        ctx.ws.reset()
        # the convolution's GEMM writes token rows 1.. itself, position embedding joined in its store
        convolution_tokens_(ctx, tok[1:].unsqueeze(0), image, W.patch_w, W.patch_b, (self.P, self.P), (0, 0), (1, 1), residual=W.pos[1:])
        add_(ctx, tok[:1], W.cls, W.pos[:1])
        return tok

    def __call__(self, ctx: Ctx, image: torch.Tensor):
        W = self.W
        src = self.embed(ctx, image)
        n = len(W.layers)
        if self.folded is not None:
            rowstats_(ctx, self.stats.x, src)
            for i, fw in enumerate(self.folded):
                dst = self.tokens[(i + 1) % 2]
                encoder_layer_folded(ctx, fw, src, dst, self.buf, self.stats, self.heads, self.eps, stats_out=i + 1 < n)
                src = dst
            if W.norm_g is None:
                return src
            layernorm_(ctx, self.out, None, None, src, W.norm_g, W.norm_b, src.shape[1], self.eps)
            return self.out
        for i, lw in enumerate(W.layers):
            dst = self.tokens[(i + 1) % 2]
            # the norm that reads this layer's output rides in its last GEMM: the next layer's first norm into the
            # shared slot buf.h, the encoder's final norm into self.out
            folds = ln_matmul_folds(self.T, lw.wqkv.shape[0], lw.wqkv.shape[1]) and ln_matmul_pays(self.T, lw.wqkv.shape[0], lw.wqkv.shape[1])
            if i + 1 < n:
                nxt = None if folds else (W.layers[i + 1].ln1_g, W.layers[i + 1].ln1_b, self.buf.h)
            else:
                nxt = None if W.norm_g is None else (W.norm_g, W.norm_b, self.out)
            encoder_layer(ctx, lw, src, dst, self.buf, self.heads, self.eps, normed_in=i > 0 and not folds, next_norm=nxt)
            src = dst
        return src if W.norm_g is None else self.out
