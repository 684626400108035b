"""Host-side mirror of the reference's kernel entry points, over the C ABI.

The reference's op handlers (DNNKernels/src/ops.jl:575-647,1114-1222,1347-1399) call
``matmul!``, ``batchedmatmul!``, ``sdpa``, ``convolution!`` and ``layernorm!`` with a
per-run ``Ctx``; a new implementation plugs in as a *plan type* plus one method
per entry point (DNNKernels/src/kernels/extern/matmul.jl:97-100,
attention.jl:767-776, kernelplans.jl:1-35).  This module is that seam in
Python: the same entry points (``!`` spelled ``_``), the same argument meaning,
``Decline(reason)`` from every planner instead of an exception, and one
``_run`` method per plan -- each of which is a single call into
``libmi355dnn.so``.  A Julia shim binds the identical symbols with ``ccall``.

Array convention: a Julia column-major array ``(a, b, c, d)`` is the torch
tensor of shape ``(d, c, b, a)`` with the same bytes (safetensors.jl:7-12).
So ``matmul_``'s ``A`` (Julia ``(M, K)``, the hoisted weight) is a torch
``(K, M)`` tensor, ``B`` (Julia ``(K, N)``, the activations) is torch
``(N, K)``, ``out`` is torch ``(N, M)``; attention operands (Julia ``(E, L, H, B)``)
are torch ``(B, H, L, E)`` views with arbitrary strides; convolution operands
are torch NCHW / OIHW.

PyTorch is used only to own device memory and the stream.
"""
from __future__ import annotations

import weakref

import ctypes as C
import math
from dataclasses import dataclass
from typing import NamedTuple, Optional

import torch

from . import _lib as L


# ----------------------------------------------------------------------------- Decline / caps / ctx

@dataclass(frozen=True)
class Decline:
    """Why a path was not taken (kernelplans.jl:21-35).  Truthiness is False."""
    reason: str

    def __bool__(self):
        return False


class DeclineError(RuntimeError):
    """A launch the library refused after a plan had been made."""

    def __init__(self, what: str, status: int):
        super().__init__(f"{what}: mi355dnn status {status} ({L.STATUS_NAMES.get(status, '?')})")
        self.status = status
        self.reason = L.STATUS_NAMES.get(status, "?")


class DeviceCaps(NamedTuple):
    """The device facts planners read -- the named fields of Lava.DeviceCaps
    (context.jl:68, test_flash.jl:373).  A value, so a test can plan for
    hardware it does not have."""
    coopmat: bool
    tile: int
    subgroup: int
    sharedbudget: int
    workgrouplimit: int
    cores: int


MI355X = DeviceCaps(True, 16, 64, 160 * 1024, 1024, 256)


def _caps_array(dev: DeviceCaps):
    """The six values of mi_device_caps, for the planners that answer for a described device."""
    return (C.c_int64 * 6)(int(dev.coopmat), dev.tile, dev.subgroup, dev.sharedbudget, dev.workgrouplimit, dev.cores)


def caps() -> DeviceCaps:
    """Query the current device (context.jl:55)."""
    lib = L.init()
    out = (C.c_int64 * 6)()
    rc = lib.mi_device_caps(out)
    if rc != L.OK:
        raise DeclineError("mi_device_caps", rc)
    return DeviceCaps(bool(out[0]), int(out[1]), int(out[2]), int(out[3]), int(out[4]), int(out[5]))


class Workspace:
    """Per-op bump scratch (workspace.jl:19-106): ``reset()`` before every op,
    ``scratch(nbytes)`` hands out 256-byte aligned device memory valid until the
    next reset.  Grows by reallocation between ops, never inside one.

    A captured graph (``StepGraph``, ``Executor.replayable``) holds the addresses it was captured with -- split-K
    planes, split-KV partials, convolution scratch -- for as long as it may be replayed, and says so with ``pin()``.
    From then on a buffer that is outgrown is retired into ``_retired`` instead of given back, where it stays until
    the workspace itself goes, so a replay after later growth still writes memory that nothing else owns.  Before any
    graph has pinned the workspace an outgrown buffer is simply dropped: the kernels already enqueued on it run on the
    stream the allocator frees it on, so it is not reused under them.  (Buffers double, so even retired ones add up to
    less than the current one.)  Growing *during* a capture cannot work (the allocation would be captured too) and
    raises: run the step eagerly once first, as both graph wrappers do, so that the workspace has reached its size."""

    ALIGN = 256
    _live = weakref.WeakSet()                             # every workspace alive: a capture pins them all (pin_all)

    @classmethod
    def pin_all(cls):
        """Called by whoever captures a device graph of kernel launches: a capture does not know which workspaces the
        launches inside it drew from, so all of them keep what they have handed out."""
        for ws in list(cls._live):
            ws.pin()

    def __init__(self, device="cuda", nbytes: int = 0):
        self.device = torch.device(device)
        self.buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=self.device)
        self.off = 0
        self._retired = []
        self._pinned = False
        Workspace._live.add(self)

    def reset(self):
        self.off = 0

    def pin(self):
        """A graph has captured addresses inside this workspace: nothing it handed out may be given back any more."""
        self._pinned = True

    def scratch(self, nbytes: int) -> int:
        if nbytes <= 0:
            return 0
        base = self.buf.data_ptr()
        start = (-(base + self.off)) % self.ALIGN + self.off
        if start + nbytes > self.buf.numel():
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError(f"Workspace would have to grow to {nbytes} bytes inside a graph capture: run the step eagerly once before capturing it")
            if self._pinned:
                self._retired.append(self.buf)          # graphs already captured keep using it
            self.buf = torch.empty(max(2 * self.buf.numel(), nbytes + self.ALIGN), dtype=torch.uint8, device=self.device)
            self.off = 0
            base = self.buf.data_ptr()
            start = (-base) % self.ALIGN
        self.off = start + nbytes
        return base + start


class Ctx:
    """Per-run context (context.jl:240-331): device caps, workspace, policy flags.
    ``clampattn`` is accepted for signature parity; the fused kernel here masks
    ragged tails itself, so the flag changes nothing."""

    def __init__(self, device="cuda", *, ws: Optional[Workspace] = None, dev: Optional[DeviceCaps] = None, clampattn: bool = False):
        L.init()
        self.device = torch.device(device)
        self.dev = dev if dev is not None else caps()
        self.ws = ws if ws is not None else Workspace(self.device)
        self.clampattn = clampattn

    @property
    def stream(self) -> int:
        return torch.cuda.current_stream(self.device).cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _is_f16_cuda(*ts) -> bool:
    return all(isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float16 for t in ts)


def _vec_problem(name: str, t, n: int, dtype=torch.float16, *, require_cuda: bool = True) -> Optional[str]:
    """Why a small per-feature / per-row operand (bias, gamma, beta, mean, rstd) cannot be handed to a kernel as a raw
    pointer, or None if it can: the kernels read exactly ``n`` contiguous elements of ``dtype`` from it, so a shorter,
    strided or differently typed tensor would be an out-of-bounds or misinterpreted device read."""
    if t is None:
        return None
    if not isinstance(t, torch.Tensor):
        return f"{name} is not a tensor"
    if require_cuda and not t.is_cuda:
        return f"{name} is not on the GPU"
    if t.dtype != dtype:
        return f"{name} is {t.dtype}, the kernel reads {dtype}"
    if t.numel() != n:
        return f"{name} has {t.numel()} elements, the kernel reads {n}"
    if not t.is_contiguous():
        return f"{name} is not contiguous"
    return None


def _check_vecs(what: str, status: int, *specs):
    """specs: (name, tensor, n[, dtype]); raises DeclineError naming the first operand a kernel could not read."""
    for spec in specs:
        why = _vec_problem(*spec)
        if why is not None:
            raise DeclineError(f"{what}: {why}", status)


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float16:
        return L.F16
    if t.dtype == torch.float32:
        return L.F32
    raise TypeError(f"unsupported output dtype {t.dtype}")


# ----------------------------------------------------------------------------- GEMM

@dataclass(frozen=True)
class MMMfmaPlan:
    """Tiled MFMA kernel (the counterpart of MMCoopMatPlan, kernelplans.jl:370-374)."""
    w_layout: int


@dataclass(frozen=True)
class MMSkinnyPlan:
    """Split-K bandwidth kernel for T <= 8 (the counterpart of MMGemvPlan, kernelplans.jl:382-385)."""
    w_layout: int


@dataclass(frozen=True)
class MMScalarPlan:
    """One thread per output (the reference's Decline path, matmul.jl:140-148)."""
    w_layout: int


def _mat2(t: torch.Tensor):
    """(layout, ld) of a 2-D operand: 0 = last axis contiguous, 1 = first axis contiguous."""
    if t.dim() != 2:
        return None
    if t.stride(1) == 1 or t.shape[1] == 1:
        return 0, (t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1))
    if t.stride(0) == 1:
        return 1, (t.stride(1) if t.shape[1] > 1 else max(t.shape[0], 1))
    return None


def mmplan(dev: DeviceCaps, out, A, B, bias=None):
    """Which GEMM path this call takes (mmplan, matmul.jl:87-95).  ``A``: torch (K, F)
    weight, ``B``: torch (T, K) activations, ``out``: torch (T, F)."""
    if not _is_f16_cuda(A, B) or not isinstance(out, torch.Tensor) or out.dtype not in (torch.float16, torch.float32):
        return Decline("operands")
    la, lb, lo = _mat2(A), _mat2(B), _mat2(out)
    if la is None or lb is None or lo is None or lb[0] != 0 or lo[0] != 0:
        return Decline("operands")
    K, F = A.shape
    T = B.shape[0]
    if B.shape[1] != K or tuple(out.shape) != (T, F):
        return Decline("extent")
    if bias is not None and not (bias.dim() == 1 and bias.numel() in (F, T) and _vec_problem("bias", bias, bias.numel()) is None):
        return Decline("bias")                          # e.g. an fp32 bias of a mixed-precision export: not read as fp16
    if not dev.coopmat:
        return Decline("nocoopmat")
    w_layout = L.W_KF if la[0] == 0 else L.W_FK
    lib = L.load()
    path = lib.mi_gemm_f16_plan_caps(_caps_array(dev), out.data_ptr(), B.data_ptr(), A.data_ptr(), T, K, F, lo[1], lb[1], la[1],
                                     w_layout, _dtype_code(out), 1, 0, 0, 0, None)
    return {1: MMMfmaPlan, 2: MMSkinnyPlan, 3: MMScalarPlan}.get(path, lambda _: Decline("extent"))(w_layout)


def matmul_(ctx: Ctx, out, A, B, bias=None, *, epi="none", residual=None, bias_mode=None):
    """``out[T,F] = epi(round(B[T,K] . A[K,F] + bias)) (+ residual)`` -- matmul!, matmul.jl:78-79.

    ``epi`` is ``"none" | "gelu" | "gelu_tanh" | "relu"`` (actfn, ops.jl:1684-1685)."""
    plan = mmplan(ctx.dev, out, A, B, bias)
    if isinstance(plan, Decline):
        raise DeclineError(f"matmul_ declined ({plan.reason})", L.DECLINE_OPERANDS)
    return _matmul_run(ctx, plan, out, A, B, bias, epi, residual, bias_mode)


def _matmul_run(ctx, plan, out, A, B, bias, epi, residual, bias_mode):
    lib = L.init()
    K, F = A.shape
    T = B.shape[0]
    la, lb, lo = _mat2(A), _mat2(B), _mat2(out)
    if bias is None:
        bm = L.BIAS_NONE
    elif bias_mode is not None:
        bm = {"col": L.BIAS_COL, "row": L.BIAS_ROW}[bias_mode]
    else:
        bm = L.BIAS_COL if bias.numel() == F else L.BIAS_ROW
    if bias is not None and bias.numel() != (F if bm == L.BIAS_COL else T):
        raise DeclineError("matmul_: bias length does not match its mode (col: F values, row: T values)", L.DECLINE_BIAS)
    if residual is not None and (residual.shape != out.shape or residual.stride() != out.stride() or residual.dtype != torch.float16):
        raise DeclineError("matmul_: residual must match out's shape, strides and be fp16", L.DECLINE_OPERANDS)
    need = lib.mi_gemm_f16_workspace(T, K, F, plan.w_layout, 1)
    ws = ctx.ws.scratch(need)
    rc = lib.mi_gemm_f16(out.data_ptr(), B.data_ptr(), A.data_ptr(), _ptr(bias), _ptr(residual),
                         T, K, F, lo[1], lb[1], la[1], plan.w_layout, bm, L.EPI[epi], _dtype_code(out),
                         ws, need, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_gemm_f16", rc)
    return out


def matmul_ln_(ctx: Ctx, out, normed, A, B, gamma, beta, eps, bias=None, *, epi="none", residual=None, clamp=None):
    """``out[T,F] = epi(B[T,K] . A[K,F] + bias) (+ residual)`` as ``matmul_`` writes it, and ``normed[T,F]`` = layer norm
    of ``out`` over ``F`` (``layernorm_``, layernorm.jl:125): a linear op whose result is both the residual stream and
    the input of the next norm.  One launch less than the two calls when the GEMM splits K; the same bits either way.
    ``clamp``: ``out`` is limited to ``[-clamp, clamp]`` after the residual add (a ``clamp`` op folded in, ops.jl:300-310);
    with it ``normed`` may be None (no norm)."""
    plan = mmplan(ctx.dev, out, A, B, bias)
    if isinstance(plan, Decline):
        raise DeclineError(f"matmul_ln_ declined ({plan.reason})", L.DECLINE_OPERANDS)
    lib = L.init()
    K, F = A.shape
    T = B.shape[0]
    la, lb = _mat2(A), _mat2(B)
    if normed is None and clamp is None:
        raise DeclineError("matmul_ln_: nothing to add to matmul_ (no norm, no clamp)", L.DECLINE_OPERANDS)
    if out.dtype != torch.float16 or not out.is_contiguous() or (normed is not None and (
            not _is_f16_cuda(normed) or not normed.is_contiguous() or normed.shape != out.shape)):
        raise DeclineError("matmul_ln_: out and normed must be dense fp16 (T,F)", L.DECLINE_OPERANDS)
    if residual is not None and (residual.shape != out.shape or residual.stride() != out.stride() or residual.dtype != torch.float16):
        raise DeclineError("matmul_ln_: residual must match out's shape, strides and be fp16", L.DECLINE_OPERANDS)
    _check_vecs("matmul_ln_", L.DECLINE_OPERANDS, ("gamma", gamma, F), ("beta", beta, F))
    bm = L.BIAS_NONE if bias is None else (L.BIAS_COL if bias.numel() == F else L.BIAS_ROW)
    need = lib.mi_gemm_f16_workspace(T, K, F, plan.w_layout, 1)
    ws = ctx.ws.scratch(need)
    if clamp is not None:
        rc = lib.mi_gemm_clamp_ln_f16(out.data_ptr(), _ptr(normed), B.data_ptr(), A.data_ptr(), _ptr(bias), _ptr(residual),
                                      _ptr(gamma), _ptr(beta), float(eps), float(clamp), T, K, F, lb[1], la[1], plan.w_layout, bm,
                                      L.EPI[epi], ws, need, ctx.stream)
    else:
        rc = lib.mi_gemm_ln_f16(out.data_ptr(), normed.data_ptr(), B.data_ptr(), A.data_ptr(), _ptr(bias), _ptr(residual),
                                _ptr(gamma), _ptr(beta), float(eps), T, K, F, lb[1], la[1], plan.w_layout, bm, L.EPI[epi],
                                ws, need, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_gemm_clamp_ln_f16" if clamp is not None else "mi_gemm_ln_f16", rc)
    return out


# ----------------------------------------------------------------------------- a layer norm with no pass of its own

@dataclass
class LnFoldedLinear:
    """A linear layer with the norm in front of it folded away (``mi_lnfold_prepare_f16``): ``wp`` = fp16(gamma W) as a
    ``(K, F)`` tensor in W's memory layout, ``colsum`` / ``biasp`` fp32 ``(F,)``; ``planes`` > 1: ``F`` is that many
    equal column bands run as planes of one launch (q, k, v)."""
    wp: torch.Tensor
    colsum: torch.Tensor
    biasp: torch.Tensor
    planes: int = 1


def rowstats_segments(C: int) -> int:
    return (C + 31) // 32


def lnfold_applies(T: int, K: int, F: int) -> bool:
    """Whether ``lnfold_matmul_`` takes a ``(T, K) -> (T, F)`` linear (no GPU needed): the tiled kernels' pipelined form
    (64-deep tiles, at least two of them) with 16-byte result rows, and enough rows that the tiled kernels are the ones
    that would run it anyway."""
    return T >= 64 and K >= 128 and K % 64 == 0 and F % 8 == 0


def rowstats_rides(T: int, K: int, F: int) -> bool:
    """Whether ``matmul_rowstats_`` takes a ``(T, K) -> (T, F)`` linear: the same conditions, seen from the GEMM that writes
    the rows whose statistics are wanted."""
    return lnfold_applies(T, K, F)


def rowstats_new(rows: int, C: int, device="cuda") -> torch.Tensor:
    """Storage for the row statistics of ``rows`` rows of ``C`` elements: (sum, squares about its mean) per 32-column
    segment, segment-major ``(segments, rows, 2)``."""
    return torch.empty((rowstats_segments(C), rows, 2), dtype=torch.float32, device=device)


def lnfold_prepare(ctx: Ctx, W, gamma, beta, bias=None, planes: int = 1) -> LnFoldedLinear:
    """Once per weight, at load: ``LN(x) . W + b = r (x . W') - r mu colsum(W') + b'`` with ``W' = gamma W`` and
    ``b' = b + beta . W``.  ``W``: ``(K, F)`` fp16 in either memory layout; ``gamma`` / ``beta`` ``(K,)`` or None."""
    lay = _mat2(W)
    if W.dim() != 2 or not _is_f16_cuda(W) or lay is None:
        raise DeclineError("lnfold_prepare: a 2-D fp16 device weight with one contiguous axis", L.DECLINE_OPERANDS)
    K, F = W.shape
    if F % planes:
        raise DeclineError("lnfold_prepare: planes must divide F", L.DECLINE_EXTENT)
    _check_vecs("lnfold_prepare", L.DECLINE_OPERANDS, ("gamma", gamma, K), ("beta", beta, K), ("bias", bias, F))
    wp = torch.empty_like(W)                       # preserves W's strides (dense in its own layout)
    if wp.stride() != W.stride():
        raise DeclineError("lnfold_prepare: the weight must be dense in its layout", L.DECLINE_OPERANDS)
    colsum = torch.empty((F,), dtype=torch.float32, device=W.device)
    biasp = torch.empty((F,), dtype=torch.float32, device=W.device)
    rc = L.init().mi_lnfold_prepare_f16(wp.data_ptr(), colsum.data_ptr(), biasp.data_ptr(), W.data_ptr(), _ptr(gamma), _ptr(beta), _ptr(bias),
                                        K, F, lay[1], L.W_KF if lay[0] == 0 else L.W_FK, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_lnfold_prepare_f16", rc)
    return LnFoldedLinear(wp, colsum, biasp, planes)


def rowstats_(ctx: Ctx, stats, x):
    """``stats`` (``rowstats_new``) of the rows of ``x`` ``(rows, C)`` fp16, rows contiguous: for rows no GEMM here wrote."""
    if x.dim() != 2 or not _is_f16_cuda(x) or x.stride(1) != 1 or stats.dtype != torch.float32 or \
            tuple(stats.shape) != (rowstats_segments(x.shape[1]), x.shape[0], 2) or not stats.is_contiguous():
        raise DeclineError("rowstats_: operands", L.DECLINE_OPERANDS)
    rc = L.init().mi_rowstats_f16(stats.data_ptr(), x.data_ptr(), x.stride(0), x.shape[1], x.shape[0], ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_rowstats_f16", rc)
    return stats


def matmul_rowstats_(ctx: Ctx, out, stats, A, B, bias=None, *, epi="none", residual=None, clamp=None):
    """``matmul_`` into dense fp16 rows that also leaves ``stats`` (``rowstats_new(T, F)``) of the finished rows -- after
    residual and clamp -- for a folded norm that reads them next (``lnfold_matmul_``)."""
    plan = mmplan(ctx.dev, out, A, B, bias)
    if not isinstance(plan, MMMfmaPlan):
        raise DeclineError(f"matmul_rowstats_: the tiled kernels only (plan {plan})", L.DECLINE_EXTENT)
    lib = L.init()
    K, F = A.shape
    T = B.shape[0]
    la, lb = _mat2(A), _mat2(B)
    if out.dtype != torch.float16 or not out.is_contiguous() or tuple(stats.shape) != (rowstats_segments(F), T, 2) or \
            stats.dtype != torch.float32 or not stats.is_contiguous():
        raise DeclineError("matmul_rowstats_: out dense fp16 (T,F), stats from rowstats_new(T, F)", L.DECLINE_OPERANDS)
    if residual is not None and (residual.shape != out.shape or residual.stride() != out.stride() or residual.dtype != torch.float16):
        raise DeclineError("matmul_rowstats_: residual must match out's shape, strides and be fp16", L.DECLINE_OPERANDS)
    bm = L.BIAS_NONE if bias is None else (L.BIAS_COL if bias.numel() == F else L.BIAS_ROW)
    need = lib.mi_gemm_f16_workspace(T, K, F, plan.w_layout, 1)
    ws = ctx.ws.scratch(need)
    rc = lib.mi_gemm_rowstats_f16(out.data_ptr(), stats.data_ptr(), B.data_ptr(), A.data_ptr(), _ptr(bias), _ptr(residual),
                                  0.0 if clamp is None else float(clamp), T, K, F, lb[1], la[1], plan.w_layout, bm, L.EPI[epi], ws, need, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_gemm_rowstats_f16", rc)
    return out


def lnfold_matmul_(ctx: Ctx, out, fw: LnFoldedLinear, B, stats, eps, *, epi="none", residual=None, stats_out=None, clamp=None):
    """``out = epi(layernorm(B) . W + b) (+ residual)`` with no pass over ``B``: ``B`` ``(T, K)`` holds the RAW rows,
    ``stats`` their row statistics (left by the GEMM that wrote them, or ``rowstats_``), ``fw`` the prepared weight.
    ``fw.planes`` > 1: ``out`` is ``(T, F)`` whose ``planes`` column bands are written by the planes of one launch.
    ``stats_out``: also leave the statistics of ``out``'s rows (single plane, dense ``out``).  Held to the parity gate
    against ``layernorm_`` -> ``matmul_``, not to their bits."""
    lib = L.init()
    K, F = fw.wp.shape
    T = B.shape[0]
    la, lb, lo = _mat2(fw.wp), _mat2(B), _mat2(out)
    if not _is_f16_cuda(B) or lb is None or lb[0] != 0 or B.shape[1] != K or lo is None or lo[0] != 0 or tuple(out.shape) != (T, F) or \
            out.dtype not in (torch.float16, torch.float32):
        raise DeclineError("lnfold_matmul_: operands", L.DECLINE_OPERANDS)
    if tuple(stats.shape) != (rowstats_segments(K), T, 2) or stats.dtype != torch.float32 or not stats.is_contiguous():
        raise DeclineError("lnfold_matmul_: stats must come from rowstats_new(T, K)", L.DECLINE_OPERANDS)
    if residual is not None and (residual.shape != out.shape or residual.stride() != out.stride() or residual.dtype != torch.float16):
        raise DeclineError("lnfold_matmul_: residual must match out's shape, strides and be fp16", L.DECLINE_OPERANDS)
    P = fw.planes
    Fp = F // P
    w_layout = L.W_KF if la[0] == 0 else L.W_FK
    sW = Fp if w_layout == L.W_KF else Fp * la[1]            # the next band of columns: F-contiguous, or Fp rows of K further
    need = lib.mi_gemm_f16_workspace(T, K, Fp, w_layout, P)
    ws = ctx.ws.scratch(need)
    rc = lib.mi_lnfold_gemm_f16(out.data_ptr(), _ptr(stats_out), B.data_ptr(), stats.data_ptr(), float(eps),
                                fw.wp.data_ptr(), fw.colsum.data_ptr(), fw.biasp.data_ptr(), _ptr(residual), 0.0 if clamp is None else float(clamp),
                                T, K, Fp, lo[1], lb[1], la[1], w_layout, L.EPI[epi], _dtype_code(out),
                                P, Fp, sW, Fp, ws, need, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_lnfold_gemm_f16", rc)
    return out


LN_GEMM_KMAX = 512


def ln_matmul_folds(T: int, K: int, F: int, w_layout: int = L.W_KF) -> bool:
    """Whether ``ln_matmul_`` takes these extents (no GPU needed): decode-sized ``T``, or a tiled launch whose
    workgroups can hold their normalised 64 x K panel in LDS and whose plain GEMM would not split K."""
    if 1 <= T <= 8:
        return True
    return 128 <= K <= LN_GEMM_KMAX and K % 64 == 0 and L.load().mi_gemm_f16_workspace(T, K, F, w_layout, 1) == 0


def ln_matmul_pays(T: int, K: int, F: int) -> bool:
    """Whether folding the norm is also the faster choice.  Decode-sized rows: yes (one launch less, the statistics are
    a few KB).  Tiled launches: measured, no -- every workgroup of a row of tiles repeats the norm of its 64 rows, about
    120 vector instructions per row on a single wave, 6.5 us before its first MFMA (1370 x 384 -> 1152: 11.2 us folded
    against 2.6 + 5.7 us for the two launches, and the same 6.5 us at every other extent tried), which is more than the
    norm's own launch costs.  The rewrites and the encoder compositions ask this; ``ln_matmul_`` itself takes any
    call ``ln_matmul_folds`` admits."""
    return 1 <= T <= 8


def ln_matmul_(ctx: Ctx, out, A, B, gamma, beta, eps, bias=None, *, epi="none", residual=None):
    """``out[T,F] = epi(layernorm(B[T,K]) . A[K,F] + bias) (+ residual)`` in one launch: ``layernorm_``
    (layernorm.jl:125) folded into ``matmul_``'s activation staging, bit-identical to the two calls in sequence.
    ``T <= 8``: one pass over the weights (the decode-sized kernels).  Larger ``T``: the tiled kernel with the norm as
    its prologue, for ``128 <= K <= 512`` (``ln_matmul_folds``); anything else declines (run the two ops)."""
    plan = mmplan(ctx.dev, out, A, B, bias)
    if not isinstance(plan, (MMSkinnyPlan, MMMfmaPlan)):
        raise DeclineError(f"ln_matmul_: no kernel folds the norm for this call (plan {plan})", L.DECLINE_EXTENT)
    lib = L.init()
    K, F = A.shape
    T = B.shape[0]
    la, lb, lo = _mat2(A), _mat2(B), _mat2(out)
    if isinstance(plan, MMMfmaPlan) and not ln_matmul_folds(T, K, F, plan.w_layout):
        raise DeclineError(f"ln_matmul_: T={T} K={K} F={F} does not fold (tiled launches need 128 <= K <= {LN_GEMM_KMAX})", L.DECLINE_EXTENT)
    if residual is not None and (residual.shape != out.shape or residual.stride() != out.stride() or residual.dtype != torch.float16):
        raise DeclineError("ln_matmul_: residual must match out's shape, strides and be fp16", L.DECLINE_OPERANDS)
    _check_vecs("ln_matmul_", L.DECLINE_OPERANDS, ("gamma", gamma, K), ("beta", beta, K))
    if bias is not None and bias.numel() != F:
        raise DeclineError("ln_matmul_: bias must have one value per output feature", L.DECLINE_BIAS)
    need = lib.mi_gemm_f16_workspace(T, K, F, plan.w_layout, 1) if T <= 8 else 0
    ws = ctx.ws.scratch(need)
    rc = lib.mi_ln_gemm_f16(out.data_ptr(), B.data_ptr(), _ptr(gamma), _ptr(beta), float(eps), A.data_ptr(), _ptr(bias), _ptr(residual),
                            T, K, F, lo[1], lb[1], la[1], plan.w_layout, L.BIAS_NONE if bias is None else L.BIAS_COL, L.EPI[epi],
                            _dtype_code(out), ws, need, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_ln_gemm_f16", rc)
    return out


def batchedmatmul_(ctx: Ctx, out, A, B, bias=None):
    """``out[b] = B[b] . A[b] (+ bias[b])`` over the leading torch axis -- batchedmatmul!, matmul.jl:383.
    ``A``: torch (Bt, K, F), ``B``: torch (Bt, T, K), ``out``: (Bt, T, F); a leading
    extent of 1 on ``A`` or ``B`` shares that operand.  ``bias``: (Bt, F), one row per plane (several linear ops over
    the same activations issued as one launch)."""
    lib = L.init()
    if not _is_f16_cuda(A, B) or A.dim() != 3 or B.dim() != 3 or out.dim() != 3:
        raise DeclineError("batchedmatmul_: operands", L.DECLINE_OPERANDS)
    nb = out.shape[0]
    K, F = A.shape[1:]
    T = B.shape[1]
    la = _mat2(A[0])                  # the planes of A may be [K][F] or, as a transposed view (k^T of attention), [F][K]
    if la is None or B.stride(2) != 1 or out.stride(2) != 1:
        raise DeclineError("batchedmatmul_: planes must be row-major (A's may be transposed views)", L.DECLINE_OPERANDS)
    sA = 0 if A.shape[0] == 1 else A.stride(0)
    sB = 0 if B.shape[0] == 1 else B.stride(0)
    if bias is not None and (not _is_f16_cuda(bias) or tuple(bias.shape) != (nb, F) or bias.stride(1) != 1):
        raise DeclineError("batchedmatmul_: bias must be (Bt, F) fp16 rows", L.DECLINE_BIAS)
    rc = lib.mi_gemm_f16_batched(out.data_ptr(), B.data_ptr(), A.data_ptr(), _ptr(bias), None, T, K, F,
                                 out.stride(1), B.stride(1), la[1], L.W_KF if la[0] == 0 else L.W_FK,
                                 L.BIAS_NONE if bias is None else L.BIAS_COL, L.EPI["none"],
                                 _dtype_code(out), nb, out.stride(0), sB, sA, 0 if bias is None else bias.stride(0), None, 0, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_gemm_f16_batched", rc)
    return out


def matmul_heads_(ctx: Ctx, out, A, B, bias=None):
    """A projection written head-major: ``out[h] = B[T,K] . A[:, h*E:(h+1)*E] + bias[h*E:(h+1)*E]`` for ``out`` torch
    ``(H, T, E)`` with contiguous rows -- the ``(E, L, H)`` operand attention reads, with no permute between the linear
    op and the cache (the reference's graphs do ``view`` + ``permute`` + ``copyto!``, decode.jl:173-177).  ``A``: torch
    ``(K, H*E)`` weight in either memory layout.  One batched launch, a head per batch plane."""
    lib = L.init()
    la, lb = _mat2(A), _mat2(B)
    if not _is_f16_cuda(A, B, out) or out.dim() != 3 or la is None or lb is None or lb[0] != 0:
        raise DeclineError("matmul_heads_: operands", L.DECLINE_OPERANDS)
    H, T, E = out.shape
    K, F = A.shape
    if F != H * E or tuple(B.shape) != (T, K) or out.stride(2) != 1 or (bias is not None and bias.numel() != F):
        raise DeclineError("matmul_heads_: out must be (H,T,E) with F = H*E", L.DECLINE_OPERANDS)
    w_layout = L.W_KF if la[0] == 0 else L.W_FK
    sW = E if w_layout == L.W_KF else E * la[1]
    rc = lib.mi_gemm_f16_batched(out.data_ptr(), B.data_ptr(), A.data_ptr(), _ptr(bias), None, T, K, E,
                                 out.stride(1), lb[1], la[1], w_layout, L.BIAS_NONE if bias is None else L.BIAS_COL,
                                 L.EPI["none"], L.F16, H, out.stride(0), 0, sW, E, None, 0, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_gemm_f16_batched", rc)
    return out


# ----------------------------------------------------------------------------- attention

@dataclass(frozen=True)
class FlashPlan:
    """Fused MFMA kernel (the counterpart of FlashCMPlan, kernelplans.jl:54-324)."""
    nsplit: int = 1


@dataclass(frozen=True)
class RowsSDPAPlan:
    """One workgroup per query row and key split: decode-sized Lq, additive masks,
    strided or odd-sized heads (takes the place of the three-pass path, attention.jl:790-834)."""
    nsplit: int = 1


def _strides_elbh(t: torch.Tensor):
    return L.strides4(t.stride(3), t.stride(2), t.stride(1), t.stride(0))


def _bias_strides(bias, Lk, Lq, H, B):
    full = (B, H, Lq, Lk)
    st = []
    for ax in (3, 2, 1, 0):
        if bias.shape[ax] not in (1, full[ax]):
            return None
        st.append(0 if bias.shape[ax] == 1 else bias.stride(ax))
    return L.strides4(*st)


def sdpaplan(ctx: Ctx, q, k, v, bias=None, scale=None, kv_len=None):
    """Which attention implementation a call gets (sdpaplan, attention.jl:735-759)."""
    if not _is_f16_cuda(q, k, v) or q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        return Decline("operands")
    Bq, H, Lq, E = q.shape
    Lk = k.shape[2]
    if tuple(k.shape) != (Bq, H, Lk, E) or tuple(v.shape) != (Bq, H, Lk, E):
        return Decline("extent")
    if bias is not None:
        if bias.dim() != 4 or bias.dtype not in (torch.float16, torch.float32) or _bias_strides(bias, Lk, Lq, H, Bq) is None:
            return Decline("bias")
    if not ctx.dev.coopmat:
        return Decline("nocoopmat")
    scale = (1.0 / math.sqrt(E)) if scale is None else float(scale)
    ns = C.c_int(1)
    devcaps = _caps_array(ctx.dev)
    path = L.load().mi_sdpa_f16_plan_caps(devcaps, q.data_ptr(), _strides_elbh(q), k.data_ptr(), _strides_elbh(k), v.data_ptr(), _strides_elbh(v),
                                          0, int(kv_len is not None), E, Lq, Lk, H, Bq, scale, C.byref(ns))
    if bias is not None:
        # The fused kernel carries a mask whose keys are contiguous and whose fp16 rows start on 4-byte boundaries (any
        # other axis may broadcast); everything else is the rows kernel's.  The C planner sees only "a mask" and plans a
        # dense fp16 one, so the mask's own layout is judged here, as mi_sdpa_f16 judges it at the call.
        bst = list(_bias_strides(bias, Lk, Lq, H, Bq))
        by_key = bias.dtype == torch.float16 and (bst[1] == 0 or Lq == 1) and Lk <= 4096    # the same for every query: no layout conditions
        fused = path == 1 and (by_key or ((bst[0] == 1 or Lk == 1) and bias.data_ptr() % 4 == 0 and
                                          (bias.dtype == torch.float32 or all(x % 2 == 0 for x in bst[1:]))))
        if fused:
            return FlashPlan(1)
        ns1 = C.c_int(1)
        L.load().mi_sdpa_f16_plan_caps(devcaps, q.data_ptr(), _strides_elbh(q), k.data_ptr(), _strides_elbh(k), v.data_ptr(), _strides_elbh(v),
                                       1, int(kv_len is not None), E, Lq, Lk, H, Bq, scale, C.byref(ns1))
        return RowsSDPAPlan(ns1.value if Lq < 64 else 1) if path in (1, 2) else Decline("extent")
    if path == 1:
        return FlashPlan(ns.value)
    if path == 2:
        return RowsSDPAPlan(ns.value)
    return Decline("extent")


def sdpa(ctx: Ctx, q, k, v, bias=None, scale=None, *, out=None, kv_len=None):
    """``softmax(scale q.k + bias) v`` -- sdpa, attention.jl:712.  ``out`` (torch (B,H,Lq,E),
    fp16 or fp32; dense, or a strided view such as a token-major buffer permuted) is the planner's slot; allocated as fp32 when absent
    (sdpaout, attention.jl:762-765).  ``kv_len``: optional int32 (B,) tensor of valid keys."""
    plan = sdpaplan(ctx, q, k, v, bias, scale, kv_len)
    if isinstance(plan, Decline):
        raise DeclineError(f"sdpa declined ({plan.reason})", L.DECLINE_OPERANDS)
    lib = L.init()
    Bq, H, Lq, E = q.shape
    Lk = k.shape[2]
    scale = (1.0 / math.sqrt(E)) if scale is None else float(scale)
    if out is None:
        out = torch.empty((Bq, H, Lq, E), dtype=torch.float32, device=q.device)
    if tuple(out.shape) != (Bq, H, Lq, E):
        raise DeclineError("sdpa: out must have shape (B,H,Lq,E)", L.DECLINE_OPERANDS)
    bst = _bias_strides(bias, Lk, Lq, H, Bq) if bias is not None else None
    if kv_len is not None and (kv_len.dtype != torch.int32 or not kv_len.is_cuda or kv_len.numel() != Bq):
        raise DeclineError("sdpa: kv_len must be a cuda int32 (B,) tensor", L.DECLINE_OPERANDS)
    need = lib.mi_sdpa_f16_workspace(E, Lq, Lk, H, Bq, int(bias is not None))
    ws = ctx.ws.scratch(need)
    rc = lib.mi_sdpa_f16(out.data_ptr(), _dtype_code(out), (None if out.is_contiguous() else _strides_elbh(out)), q.data_ptr(), _strides_elbh(q), k.data_ptr(), _strides_elbh(k),
                         v.data_ptr(), _strides_elbh(v), _ptr(bias), (L.F32 if bias is not None and bias.dtype == torch.float32 else L.F16),
                         bst, _ptr(kv_len), E, Lq, Lk, H, Bq, scale, ws, need, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_sdpa_f16", rc)
    return out


def sdpa_append(ctx: Ctx, q, cache_k, cache_v, k_new, v_new, kv_len, scale=None, *, out):
    """Self-attention of one new token over its cache with the cache write folded in: ``k_new``/``v_new`` (B,H,1,E)
    become key ``kv_len[b] - 1`` and are stored into that slot of ``cache_k``/``cache_v`` (B,H,Lmax,E); ``out``
    (B,H,1,E) = attention of ``q`` (B,H,1,E) over the first ``kv_len[b]`` keys.  One launch in place of the exported
    step's ``index_put`` + ``cat`` + attention (WhisperRunner/src/decode.jl:186-203).  Raises ``DeclineError`` with
    ``L.DECLINE_UNSUPPORTED`` for shapes the single-launch kernel does not cover (head dim > 64, rows not 16-byte addressable):
    the caller then appends and attends in two calls."""
    if not _is_f16_cuda(q, cache_k, cache_v, k_new, v_new) or q.dim() != 4 or cache_k.dim() != 4:
        raise DeclineError("sdpa_append: operands", L.DECLINE_OPERANDS)
    Bq, H, Lq, E = q.shape
    Lk = cache_k.shape[2]
    if Lq != 1 or tuple(cache_k.shape) != (Bq, H, Lk, E) or tuple(cache_v.shape) != (Bq, H, Lk, E) or \
            tuple(k_new.shape) != (Bq, H, 1, E) or tuple(v_new.shape) != (Bq, H, 1, E) or k_new.stride() != v_new.stride() or \
            tuple(out.shape) != (Bq, H, 1, E):
        raise DeclineError("sdpa_append: shapes", L.DECLINE_OPERANDS)
    if kv_len.dtype != torch.int32 or not kv_len.is_cuda or kv_len.numel() != Bq:
        raise DeclineError("sdpa_append: kv_len must be a cuda int32 (B,) tensor", L.DECLINE_OPERANDS)
    scale = (1.0 / math.sqrt(E)) if scale is None else float(scale)
    rc = L.init().mi_sdpa_append_f16(out.data_ptr(), _dtype_code(out), (None if out.is_contiguous() else _strides_elbh(out)),
                                     q.data_ptr(), _strides_elbh(q), cache_k.data_ptr(), _strides_elbh(cache_k),
                                     cache_v.data_ptr(), _strides_elbh(cache_v), k_new.data_ptr(), v_new.data_ptr(), _strides_elbh(k_new),
                                     kv_len.data_ptr(), E, Lk, H, Bq, scale, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_sdpa_append_f16", rc)
    return out


# ----------------------------------------------------------------------------- convolution

@dataclass(frozen=True)
class ConvGemmPlan:
    """1x1 or im2col + MFMA GEMM (the counterpart of ConvCoopMatPlan, kernelplans.jl:405-410)."""
    path: str
    workspace: int


def convsize(n, k, s, p, d) -> int:
    """ATen's output extent (convsize, conv.jl:309)."""
    return (n + 2 * p - d * (k - 1) - 1) // s + 1


def conv_plan(dev: DeviceCaps, out, x, w, stride=(1, 1), padding=(0, 0), dilation=(1, 1), groups=1):
    """conv_coopmat_plan, conv_coopmat.jl:83-155.  stride/padding/dilation are (x, y) pairs."""
    if not _is_f16_cuda(x, w) or x.dim() != 4 or w.dim() != 4 or not x.is_contiguous() or not w.is_contiguous():
        return Decline("operands")
    if not dev.coopmat:
        return Decline("nocoopmat")
    N, Cin, Hi, Wi = x.shape
    Cout, cing, KH, KW = w.shape
    if cing * groups != Cin:
        return Decline("extent")
    lib = L.load()
    args = (Wi, Hi, Cin, N, KW, KH, Cout, stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1])
    path = lib.mi_conv2d_f16_plan(*args, groups)
    if path == 0:
        return Decline("extent")
    return ConvGemmPlan(L.CONV_PATHS[path], int(lib.mi_conv2d_f16_workspace(*args)))


def convolution_(ctx: Ctx, out, x, w, bias, stride, padding, dilation, groups, *, act="none"):
    """convolution!(ctx, out, x, w, bias, stride, padding, dilation, groups; act) -- conv.jl:100-145.
    ``x`` torch (N,Cin,H,W), ``w`` torch (Cout,Cin/groups,KH,KW), ``out`` torch (N,Cout,OH,OW), all
    contiguous fp16; ``stride``/``padding``/``dilation`` are ``(x, y)`` pairs, the reverse of ATen's
    ``(h, w)``; ``act`` is ``"none"`` or ``"relu"``."""
    plan = conv_plan(ctx.dev, out, x, w, stride, padding, dilation, groups)
    if isinstance(plan, Decline):
        raise DeclineError(f"convolution_ declined ({plan.reason})", L.DECLINE_OPERANDS)
    lib = L.init()
    N, Cin, Hi, Wi = x.shape
    Cout, _, KH, KW = w.shape
    OW = convsize(Wi, KW, stride[0], padding[0], dilation[0])
    OH = convsize(Hi, KH, stride[1], padding[1], dilation[1])
    if tuple(out.shape) != (N, Cout, OH, OW) or not out.is_contiguous() or out.dtype != torch.float16:
        raise DeclineError("convolution_: out must be dense fp16 (N,Cout,OH,OW)", L.DECLINE_OPERANDS)
    ws = ctx.ws.scratch(plan.workspace)
    rc = lib.mi_conv2d_f16(out.data_ptr(), x.data_ptr(), w.data_ptr(), _ptr(bias), Wi, Hi, Cin, N, KW, KH, Cout,
                           stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1], groups,
                           L.EPI[act], ws, plan.workspace, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_conv2d_f16", rc)
    return out


def convolution_tokens_(ctx: Ctx, out, x, w, bias, stride, padding, dilation, *, residual=None, act="none"):
    """The convolution with its output as tokens: ``x`` (N,Cin,H,W), ``w`` (Cout,Cin,KH,KW) contiguous fp16, ``out``
    (N, OH*OW, Cout) with the last axis contiguous (a view into a token matrix will do) = ``convolution_``'s result
    after ``flatten(2).transpose(1, 2)``, plus ``residual`` -- (OH*OW, Cout) for every image or (N, OH*OW, Cout), with
    ``out``'s row pitch -- added with one more rounding (a position embedding).  ``mi_conv2d_tokens_f16``."""
    if not _is_f16_cuda(x, w, out) or x.dim() != 4 or w.dim() != 4 or out.dim() != 3 or not (x.is_contiguous() and w.is_contiguous()):
        raise DeclineError("convolution_tokens_: operands", L.DECLINE_OPERANDS)
    lib = L.init()
    N, Cin, Hi, Wi = x.shape
    Cout, cin_w, KH, KW = w.shape
    OW = convsize(Wi, KW, stride[0], padding[0], dilation[0])
    OH = convsize(Hi, KH, stride[1], padding[1], dilation[1])
    if cin_w != Cin or tuple(out.shape) != (N, OH * OW, Cout) or out.stride(2) != 1:
        raise DeclineError("convolution_tokens_: out must be (N, OH*OW, Cout) with contiguous rows and w (Cout,Cin,KH,KW)", L.DECLINE_OPERANDS)
    _check_vecs("convolution_tokens_", L.DECLINE_OPERANDS, ("bias", bias, Cout))
    rs = 0
    if residual is not None:
        if not _is_f16_cuda(residual) or residual.dim() not in (2, 3) or tuple(residual.shape[-2:]) != (OH * OW, Cout) or \
                residual.stride(-1) != 1 or residual.stride(-2) != out.stride(1) or (residual.dim() == 3 and residual.shape[0] != N):
            raise DeclineError("convolution_tokens_: residual must be ([N,] OH*OW, Cout) fp16 with out's row pitch", L.DECLINE_OPERANDS)
        rs = residual.stride(0) if residual.dim() == 3 and N > 1 else 0
    args = (Wi, Hi, Cin, N, KW, KH, Cout, stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1])
    need = lib.mi_conv2d_tokens_f16_workspace(*args)
    ws = ctx.ws.scratch(need)
    rc = lib.mi_conv2d_tokens_f16(out.data_ptr(), out.stride(1), out.stride(0) if N > 1 else 0, x.data_ptr(), w.data_ptr(), _ptr(bias),
                                  _ptr(residual), rs, *args, L.EPI[act], ws, need, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_conv2d_tokens_f16", rc)
    return out


def convolution_nhwc_(ctx: Ctx, out, x, w, bias, stride, padding, dilation, *, act="none"):
    """The convolution over channels-last tensors: ``x`` (N,H,W,Cin), ``w`` (Cout,KH,KW,Cin), ``out`` (N,OH,OW,Cout), all
    contiguous fp16; pairs are ``(x, y)``.  An implicit GEMM with no staging pass (``mi_conv2d_nhwc_f16``); needs
    ``Cin % 64 == 0``, otherwise ``DeclineError`` with ``L.DECLINE_UNSUPPORTED`` (use ``convolution_`` on NCHW views)."""
    if not _is_f16_cuda(x, w, out) or x.dim() != 4 or w.dim() != 4 or not (x.is_contiguous() and w.is_contiguous() and out.is_contiguous()):
        raise DeclineError("convolution_nhwc_: operands", L.DECLINE_OPERANDS)
    lib = L.init()
    N, Hi, Wi, Cin = x.shape
    Cout, KH, KW, cin_w = w.shape
    OW = convsize(Wi, KW, stride[0], padding[0], dilation[0])
    OH = convsize(Hi, KH, stride[1], padding[1], dilation[1])
    if cin_w != Cin or tuple(out.shape) != (N, OH, OW, Cout):
        raise DeclineError("convolution_nhwc_: out must be (N,OH,OW,Cout) and w (Cout,KH,KW,Cin)", L.DECLINE_OPERANDS)
    args = (Wi, Hi, Cin, N, KW, KH, Cout, stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1])
    need = lib.mi_conv2d_nhwc_f16_workspace(*args)
    ws = ctx.ws.scratch(need)
    rc = lib.mi_conv2d_nhwc_f16(out.data_ptr(), x.data_ptr(), w.data_ptr(), _ptr(bias), *args, L.EPI[act], ws, need, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_conv2d_nhwc_f16", rc)
    return out


def convtransposesize(n, k, s, p, d, op):
    """convtransposesize, conv.jl:201."""
    return (n - 1) * s - 2 * p + d * (k - 1) + op + 1


def convtranspose_plan(dev: DeviceCaps, out, x, w, stride=(1, 1), padding=(0, 0), dilation=(1, 1), outpad=(0, 0), groups=1):
    """Which route a transposed convolution takes: ``gemm_shuffle`` (shufflecase, conv.jl:204-209) or
    ``gather``.  Pairs are (x, y)."""
    if not _is_f16_cuda(x, w) or x.dim() != 4 or w.dim() != 4 or not x.is_contiguous() or not w.is_contiguous():
        return Decline("operands")
    if not dev.coopmat:
        return Decline("nocoopmat")
    N, Cin, Hi, Wi = x.shape
    cin_w, coutg, KH, KW = w.shape
    if cin_w != Cin:
        return Decline("extent")
    lib = L.load()
    args = (Wi, Hi, Cin, N, KW, KH, coutg * groups, stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1],
            outpad[0], outpad[1], groups)
    path = lib.mi_convtranspose2d_f16_plan(*args)
    if path == 0:
        return Decline("extent")
    return ConvGemmPlan(L.CONVT_PATHS[path], int(lib.mi_convtranspose2d_f16_workspace(*args)))


def convolutiontranspose_(ctx: Ctx, out, x, w, bias, stride, padding, dilation, outpad, groups):
    """convolutiontranspose!(ctx, out, x, w, bias, stride, padding, dilation, outpad, groups) -- conv.jl:226-294.
    ``x`` torch (N,Cin,H,W), ``w`` torch (Cin,Cout/groups,KH,KW), ``out`` torch (N,Cout,OH,OW), all contiguous
    fp16; the pairs are ``(x, y)``, the reverse of ATen's ``(h, w)``."""
    plan = convtranspose_plan(ctx.dev, out, x, w, stride, padding, dilation, outpad, groups)
    if isinstance(plan, Decline):
        raise DeclineError(f"convolutiontranspose_ declined ({plan.reason})", L.DECLINE_OPERANDS)
    lib = L.init()
    N, Cin, Hi, Wi = x.shape
    _, coutg, KH, KW = w.shape
    Cout = coutg * groups
    OW = convtransposesize(Wi, KW, stride[0], padding[0], dilation[0], outpad[0])
    OH = convtransposesize(Hi, KH, stride[1], padding[1], dilation[1], outpad[1])
    if tuple(out.shape) != (N, Cout, OH, OW) or not out.is_contiguous() or out.dtype != torch.float16:
        raise DeclineError("convolutiontranspose_: out must be dense fp16 (N,Cout,OH,OW)", L.DECLINE_OPERANDS)
    ws = ctx.ws.scratch(plan.workspace)
    rc = lib.mi_convtranspose2d_f16(out.data_ptr(), x.data_ptr(), w.data_ptr(), _ptr(bias), Wi, Hi, Cin, N, KW, KH, Cout,
                                    stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1],
                                    outpad[0], outpad[1], groups, ws, plan.workspace, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_convtranspose2d_f16", rc)
    return out


# ----------------------------------------------------------------------------- layout

def transposeLE_(ctx: Ctx, out, a):
    """transposeLE(ctx, a) -- attention.jl:374-396.  ``a`` torch (B,H,L,E) fp16 with any strides (the reference's
    (E,L,H,B)); ``out`` torch (B,H,E,L) fp16 whose last axis is contiguous.  2-D tensors are taken as H = B = 1:
    ``out (C,R) = a (R,C)`` transposed."""
    if a.dim() == 2 and out.dim() == 2:
        a, out = a[None, None], out[None, None]
    if not _is_f16_cuda(a, out) or a.dim() != 4 or out.dim() != 4:
        raise DeclineError("transposeLE_: operands", L.DECLINE_OPERANDS)
    B, H, Ln, E = a.shape
    if tuple(out.shape) != (B, H, E, Ln) or (Ln > 1 and out.stride(3) != 1):
        raise DeclineError("transposeLE_: out must be (B,H,E,L) with L contiguous", L.DECLINE_OPERANDS)
    ost = L.strides4(1, out.stride(2) if E > 1 else Ln, out.stride(1), out.stride(0))
    rc = L.init().mi_transpose_le_f16(out.data_ptr(), ost, a.data_ptr(), _strides_elbh(a), E, Ln, H, B, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_transpose_le_f16", rc)
    return out


def relayout_weight(ctx: Ctx, w):
    """A ``(K, F)`` weight held as ``[K][F]`` memory (the reference's hoisted layout, hoistcasts.jl:47-112) returned as
    the same ``(K, F)`` tensor over ``[F][K]`` memory -- a transposed view of a new buffer -- through
    ``mi_relayout_weight_f16``; a weight that already lies that way is returned as it is.  Once, at load."""
    if w.dim() != 2 or not _is_f16_cuda(w):
        raise DeclineError("relayout_weight: a 2-D fp16 device tensor", L.DECLINE_OPERANDS)
    if w.stride(0) == 1 and w.shape[0] > 1:
        return w
    if w.stride(1) != 1:
        raise DeclineError("relayout_weight: rows must be contiguous", L.DECLINE_OPERANDS)
    K, F = w.shape
    fk = torch.empty((F, K), dtype=w.dtype, device=w.device)
    rc = L.init().mi_relayout_weight_f16(fk.data_ptr(), K, w.data_ptr(), w.stride(0), K, F, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_relayout_weight_f16", rc)
    return fk.t()


# ----------------------------------------------------------------------------- layer norm, add

def layernorm_(ctx: Ctx, out, mean, rstd, a, gamma, beta, C_: int, eps: float):
    """layernorm!(ctx, out, mean, rstd, a, gamma, beta, C, eps) -- layernorm.jl:125.
    ``a`` contiguous fp16 with the normalised axis last; ``mean``/``rstd`` fp32 (groups,) or None."""
    lib = L.init()
    if not _is_f16_cuda(a, out) or not a.is_contiguous() or not out.is_contiguous():
        raise DeclineError("layernorm_: operands", L.DECLINE_OPERANDS)
    if C_ < 1 or a.numel() % C_ or out.shape != a.shape:
        raise DeclineError("layernorm_: the normalised extent must divide the operand, out must have a's shape", L.DECLINE_EXTENT)
    groups = a.numel() // C_
    _check_vecs("layernorm_", L.DECLINE_OPERANDS, ("gamma", gamma, C_), ("beta", beta, C_),
                ("mean", mean, groups, torch.float32), ("rstd", rstd, groups, torch.float32))
    rc = lib.mi_layernorm_f16(out.data_ptr(), _ptr(mean), _ptr(rstd), a.data_ptr(), _ptr(gamma), _ptr(beta),
                              C_, groups, float(eps), ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_layernorm_f16", rc)
    return out


def softmax_(ctx: Ctx, out, a, scale: float = 1.0):
    """Softmax over the last axis of a contiguous fp16 or fp32 tensor, ``exp(scale * a - max) / sum`` in fp32
    (softmax_kernel!, ops.jl:474-573; attn_softmax_rows!, attention.jl:528-615)."""
    lib = L.init()
    if not (a.is_cuda and out.is_cuda and a.dtype == out.dtype and a.dtype in (torch.float16, torch.float32)) or a.shape != out.shape \
            or not (a.is_contiguous() and out.is_contiguous()) or a.dim() < 1:
        raise DeclineError("softmax_: operands", L.DECLINE_OPERANDS)
    n = a.shape[-1]
    rc = lib.mi_softmax_f16(out.data_ptr(), a.data_ptr(), _dtype_code(a), n, a.numel() // max(n, 1), float(scale), ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_softmax_f16", rc)
    return out


def scale_(ctx: Ctx, out, a, c: float):
    """out = fp16(a * c), contiguous fp16 tensors (mul.Tensor / div.Tensor with a constant)."""
    lib = L.init()
    if not _is_f16_cuda(a, out) or a.shape != out.shape or not (a.is_contiguous() and out.is_contiguous()):
        raise DeclineError("scale_: operands", L.DECLINE_OPERANDS)
    rc = lib.mi_scale_f16(out.data_ptr(), a.data_ptr(), float(c), a.numel(), ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_scale_f16", rc)
    return out


def act_(ctx: Ctx, out, a, act: str):
    """out = fp16(act(a)), ``act`` as in ``matmul_``'s ``epi``; contiguous fp16 tensors (may be the same tensor)."""
    lib = L.init()
    if not _is_f16_cuda(a, out) or a.shape != out.shape or not (a.is_contiguous() and out.is_contiguous()):
        raise DeclineError("act_: operands", L.DECLINE_OPERANDS)
    rc = lib.mi_act_f16(out.data_ptr(), a.data_ptr(), L.EPI[act], a.numel(), ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_act_f16", rc)
    return out


def clamp_(ctx: Ctx, out, a, lo: float, hi: float):
    """out = min(max(a, lo), hi); contiguous fp16 tensors (clamp, ops.jl:300-310)."""
    lib = L.init()
    if not _is_f16_cuda(a, out) or a.shape != out.shape or not (a.is_contiguous() and out.is_contiguous()):
        raise DeclineError("clamp_: operands", L.DECLINE_OPERANDS)
    rc = lib.mi_clamp_f16(out.data_ptr(), a.data_ptr(), float(lo), float(hi), a.numel(), ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_clamp_f16", rc)
    return out


def add_(ctx: Ctx, out, a, b):
    """out = fp16(a + b), the residual add.Tensor (ops.jl:186-197)."""
    lib = L.init()
    if not _is_f16_cuda(a, b, out) or not (a.is_contiguous() and b.is_contiguous() and out.is_contiguous()):
        raise DeclineError("add_: operands", L.DECLINE_OPERANDS)
    drop1 = lambda t: [d for d in t.shape if d != 1]       # (1, T, D) + (T, D) are the same elements
    if not (drop1(a) == drop1(b) == drop1(out)):
        raise DeclineError(f"add_: shapes differ ({tuple(a.shape)}, {tuple(b.shape)}, {tuple(out.shape)}); nothing is broadcast",
                           L.DECLINE_EXTENT)
    rc = lib.mi_add_f16(out.data_ptr(), a.data_ptr(), b.data_ptr(), a.numel(), ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_add_f16", rc)
    return out


# ----------------------------------------------------------------------------- the decoder step's gathers

def embedding_(ctx: Ctx, out, table, ids, table2=None, ids2=None):
    """``out[i] = table[ids[i]]`` (+ ``table2[ids2[i]]``, ``ids2`` one id for every row or one per row): aten::embedding
    (ops.jl:1754-1783) and the first-axis gather of aten::index.Tensor; with both tables the decoder step's token +
    position embedding.  ``ids``: int64, any shape; ``out``: fp16 ``ids.shape + (D,)`` (leading singleton axes free)."""
    lib = L.init()
    if not _is_f16_cuda(out, table) or table.dim() != 2 or not table.is_contiguous() or not out.is_contiguous():
        raise DeclineError("embedding_: fp16 cuda operands, a contiguous (V, D) table", L.DECLINE_OPERANDS)
    V, D = table.shape
    n = ids.numel()
    if ids.dtype != torch.int64 or not ids.is_cuda or not ids.is_contiguous() or n < 1 or out.numel() != n * D or out.shape[-1] != D:
        raise DeclineError(f"embedding_: ids must be contiguous cuda int64 and out hold ids.numel() rows of {D}", L.DECLINE_OPERANDS)
    n2 = V2 = 0
    if table2 is not None:
        if not _is_f16_cuda(table2) or table2.dim() != 2 or not table2.is_contiguous() or table2.shape[1] != D:
            raise DeclineError("embedding_: the second table must be a contiguous fp16 (V2, D) matrix", L.DECLINE_OPERANDS)
        if ids2 is None or ids2.dtype != torch.int64 or not ids2.is_cuda or not ids2.is_contiguous() or ids2.numel() not in (1, n):
            raise DeclineError("embedding_: ids2 must be cuda int64 with one id, or one per row", L.DECLINE_OPERANDS)
        n2, V2 = ids2.numel(), table2.shape[0]
    rc = lib.mi_embedding_f16(out.data_ptr(), table.data_ptr(), ids.data_ptr(), n, D, V, _ptr(table2), _ptr(ids2), n2, V2, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_embedding_f16", rc)
    return out


def kv_len_from_position_(ctx: Ctx, kv_len, position, cap: int):
    """``kv_len[b] = clamp(position + 1, 0, cap)``: the exported step's ``cache_position`` (int64, one for all rows or one
    per row) as the count of valid keys the attention kernels take (decode.jl:186-203)."""
    if kv_len.dtype != torch.int32 or not kv_len.is_cuda or not kv_len.is_contiguous() or \
            position.dtype != torch.int64 or not position.is_cuda or not position.is_contiguous() or position.numel() not in (1, kv_len.numel()):
        raise DeclineError("kv_len_from_position_: int32 (B,) lengths and int64 positions (1 or B of them) on the GPU", L.DECLINE_OPERANDS)
    rc = L.init().mi_kv_len_from_position(kv_len.data_ptr(), position.data_ptr(), position.numel(), kv_len.numel(), int(cap), ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_kv_len_from_position", rc)
    return kv_len


def kv_append_(ctx: Ctx, cache_k, cache_v, k_new, v_new, kv_len):
    """Write the new token's rows ``(B,H,1,E)`` into slot ``kv_len[b] - 1`` of ``cache_k`` / ``cache_v`` ``(B,H,Lmax,E)``,
    in place: the exported step's ``index_put`` on the cache (ops.jl:1003-1025) without the copy of the whole tensor."""
    if not _is_f16_cuda(cache_k, cache_v, k_new, v_new) or cache_k.dim() != 4 or k_new.dim() != 4:
        raise DeclineError("kv_append_: operands", L.DECLINE_OPERANDS)
    B, H, Lmax, E = cache_k.shape
    if tuple(cache_v.shape) != (B, H, Lmax, E) or cache_v.stride() != cache_k.stride() or tuple(k_new.shape) != (B, H, 1, E) or \
            tuple(v_new.shape) != (B, H, 1, E) or k_new.stride() != v_new.stride():
        raise DeclineError("kv_append_: caches (B,H,Lmax,E) with equal strides, new rows (B,H,1,E) with equal strides", L.DECLINE_OPERANDS)
    if kv_len.dtype != torch.int32 or not kv_len.is_cuda or kv_len.numel() != B:
        raise DeclineError("kv_append_: kv_len must be a cuda int32 (B,) tensor", L.DECLINE_OPERANDS)
    rc = L.init().mi_kv_append_f16(cache_k.data_ptr(), cache_v.data_ptr(), _strides_elbh(cache_k), Lmax, k_new.data_ptr(), v_new.data_ptr(),
                                   _strides_elbh(k_new), kv_len.data_ptr(), E, H, B, ctx.stream)
    if rc != L.OK:
        raise DeclineError("mi_kv_append_f16", rc)
