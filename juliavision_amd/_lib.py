"""ctypes binding of ``libmi355dnn.so`` -- the same C ABI a Julia ``ccall`` shim binds.

There is no fallback: if the shared object is missing or a symbol does not
resolve, importing the binding raises.  Device memory and streams come from
PyTorch-ROCm; only raw pointers cross this boundary.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi355dnn.so")

# enum mi_status
OK, DECLINE_OPERANDS, DECLINE_EXTENT, DECLINE_WORKSPACE, DECLINE_BIAS, DECLINE_UNSUPPORTED, ERROR_LAUNCH, ERROR_DEVICE, DECLINE_SCRATCH_LIMIT = range(9)
STATUS_NAMES = {0: "ok", 1: "operands", 2: "extent", 3: "workspace", 4: "bias", 5: "unsupported", 6: "launch", 7: "device", 8: "scratch_limit"}
NOALLOC_SCRATCH_BYTES = 32 * 1024 * 1024
EPI = {"none": 0, "identity": 0, "gelu": 1, "gelu_erf": 1, "gelu_tanh": 2, "relu": 3}
F16, F32 = 0, 1
W_KF, W_FK = 0, 1
BIAS_NONE, BIAS_COL, BIAS_ROW = 0, 1, 2
GEMM_PATHS = {0: "decline", 1: "mfma", 2: "skinny", 3: "scalar"}
SDPA_PATHS = {0: "decline", 1: "flash", 2: "rows"}
CONV_PATHS = {0: "decline", 1: "gemm_1x1", 2: "im2col_gemm", 3: "direct", 4: "implicit_gemm"}
CONVT_PATHS = {0: "decline", 1: "gemm_shuffle", 2: "gather"}

_i64, _int, _vp, _sz, _f32 = C.c_int64, C.c_int, C.c_void_p, C.c_size_t, C.c_float
_i64p = C.POINTER(C.c_int64)

# name -> (restype, argtypes); every symbol include/mi355dnn.h declares.
SIGNATURES = {
    "mi_version": (_int, []),
    "mi_init": (_int, []),
    "mi_device_caps": (_int, [_i64p]),
    "mi_set_clock_probe": (_int, [_vp]),
    "mi_set_phase_probe": (_int, [_vp, _i64]),
    "mi_probe_mfma": (_int, [_vp, _vp, _i64, _i64, _int, _vp]),
    "mi_probe_copy": (_int, [_vp, _vp, _sz, _vp]),
    "mi_probe_grid_barrier": (_int, [_vp, _i64, _i64, _int, _vp]),
    "mi_device_status": (_int, [_int]),
    "mi_set_in_launch_exchange": (_int, [_int]),
    "mi_test_exchange_faults": (_int, [_int, C.c_uint, C.c_uint]),
    "mi_gemm_f16": (_int, [_vp] * 5 + [_i64] * 6 + [_int] * 4 + [_vp, _sz, _vp]),
    "mi_gemm_f16_batched": (_int, [_vp] * 5 + [_i64] * 6 + [_int] * 4 + [_i64] * 5 + [_vp, _sz, _vp]),
    "mi_gemv_f16": (_int, [_vp] * 5 + [_i64] * 6 + [_int] * 4 + [_vp, _sz, _vp]),
    "mi_ln_gemv_f16": (_int, [_vp, _vp, _vp, _vp, _f32, _vp, _vp, _vp] + [_i64] * 6 + [_int] * 4 + [_vp, _sz, _vp]),
    "mi_ln_gemm_f16": (_int, [_vp, _vp, _vp, _vp, _f32, _vp, _vp, _vp] + [_i64] * 6 + [_int] * 4 + [_vp, _sz, _vp]),
    "mi_gemm_ln_f16": (_int, [_vp] * 8 + [_f32] + [_i64] * 5 + [_int] * 3 + [_vp, _sz, _vp]),
    "mi_gemm_clamp_ln_f16": (_int, [_vp] * 8 + [_f32, _f32] + [_i64] * 5 + [_int] * 3 + [_vp, _sz, _vp]),
    "mi_gemm_f16_workspace": (_sz, [_i64, _i64, _i64, _int, _i64]),
    "mi_lnfold_prepare_f16": (_int, [_vp] * 7 + [_i64, _i64, _i64, _int, _vp]),
    "mi_rowstats_f16": (_int, [_vp, _vp, _i64, _i64, _i64, _vp]),
    "mi_gemm_rowstats_f16": (_int, [_vp] * 6 + [_f32] + [_i64] * 5 + [_int] * 3 + [_vp, _sz, _vp]),
    "mi_lnfold_gemm_f16": (_int, [_vp, _vp, _vp, _vp, _f32, _vp, _vp, _vp, _vp, _f32] + [_i64] * 6 + [_int] * 3 + [_i64] * 4 + [_vp, _sz, _vp]),
    "mi_gemm_f16_noalloc": (_int, [_vp] * 5 + [_i64] * 6 + [_int] * 4 + [_vp]),
    "mi_gemm_f16_plan": (_int, [_vp] * 3 + [_i64] * 6 + [_int] * 2 + [_i64] * 4),
    "mi_gemm_f16_plan_caps": (_int, [_i64p] + [_vp] * 3 + [_i64] * 6 + [_int] * 2 + [_i64] * 4 + [C.POINTER(C.c_int)]),
    "mi_sdpa_f16_plan_caps": (_int, [_i64p, _vp, _i64p, _vp, _i64p, _vp, _i64p, _int, _int] + [_i64] * 5 + [_f32, C.POINTER(C.c_int)]),
    "mi_sdpa_f16": (_int, [_vp, _int, _i64p, _vp, _i64p, _vp, _i64p, _vp, _i64p, _vp, _int, _i64p, _vp] + [_i64] * 5 + [_f32, _vp, _sz, _vp]),
    "mi_sdpa_f16_workspace": (_sz, [_i64] * 5 + [_int]),
    "mi_sdpa_f16_plan": (_int, [_vp, _i64p, _vp, _i64p, _vp, _i64p, _int, _int] + [_i64] * 5 + [_f32, C.POINTER(C.c_int)]),
    "mi_conv2d_f16": (_int, [_vp] * 4 + [_i64] * 14 + [_int, _vp, _sz, _vp]),
    "mi_conv2d_f16_workspace": (_sz, [_i64] * 13),
    "mi_conv2d_f16_plan": (_int, [_i64] * 14),
    "mi_conv2d_nhwc_f16": (_int, [_vp] * 4 + [_i64] * 13 + [_int, _vp, _sz, _vp]),
    "mi_conv2d_nhwc_f16_workspace": (_sz, [_i64] * 13),
    "mi_conv2d_tokens_f16": (_int, [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _i64] + [_i64] * 13 + [_int, _vp, _sz, _vp]),
    "mi_conv2d_tokens_f16_workspace": (_sz, [_i64] * 13),
    "mi_convsize": (_i64, [_i64] * 5),
    "mi_convtranspose2d_f16": (_int, [_vp] * 4 + [_i64] * 16 + [_vp, _sz, _vp]),
    "mi_convtranspose2d_f16_workspace": (_sz, [_i64] * 16),
    "mi_convtranspose2d_f16_plan": (_int, [_i64] * 16),
    "mi_convtransposesize": (_i64, [_i64] * 6),
    "mi_transpose_le_f16": (_int, [_vp, _i64p, _vp, _i64p, _i64, _i64, _i64, _i64, _vp]),
    "mi_relayout_weight_f16": (_int, [_vp, _i64, _vp, _i64, _i64, _i64, _vp]),
    "mi_layernorm_f16": (_int, [_vp] * 6 + [_i64, _i64, _f32, _vp]),
    "mi_softmax_f16": (_int, [_vp, _vp, _int, _i64, _i64, _f32, _vp]),
    "mi_scale_f16": (_int, [_vp, _vp, _f32, _i64, _vp]),
    "mi_act_f16": (_int, [_vp, _vp, _int, _i64, _vp]),
    "mi_clamp_f16": (_int, [_vp, _vp, _f32, _f32, _i64, _vp]),
    "mi_add_f16": (_int, [_vp, _vp, _vp, _i64, _vp]),
    "mi_kv_append_f16": (_int, [_vp, _vp, _i64p, _i64, _vp, _vp, _i64p, _vp, _i64, _i64, _i64, _vp]),
    "mi_sdpa_append_f16": (_int, [_vp, _int, _i64p, _vp, _i64p, _vp, _i64p, _vp, _i64p, _vp, _vp, _i64p, _vp, _i64, _i64, _i64, _i64, _f32, _vp]),
    "mi_kv_advance": (_int, [_vp, _i64, C.c_int32, C.c_int32, _vp]),
    "mi_kv_len_from_position": (_int, [_vp, _vp, _i64, _i64, C.c_int32, _vp]),
    "mi_embedding_f16": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _i64, _vp]),
}

_lib = None


def load() -> C.CDLL:
    """dlopen the library and bind every declared symbol (no GPU needed for this)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m juliavision_amd.build` "
            "(hipcc --offload-arch=gfx950). There is no CPU or PyTorch fallback.")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)      # AttributeError if the symbol is absent
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


_initialised = False


def init() -> C.CDLL:
    """load() + mi_init() on the current HIP device; raises if it is not a gfx950."""
    global _initialised
    lib = load()
    if not _initialised:
        import torch
        if not torch.cuda.is_available():
            raise RuntimeError("mi355dnn needs a gfx950 GPU: torch.cuda.is_available() is False")
        torch.cuda.init()
        torch.zeros(1, device="cuda")     # make sure a HIP context exists on this thread
        rc = lib.mi_init()
        if rc != OK:
            raise RuntimeError(f"mi_init failed with status {rc} ({STATUS_NAMES.get(rc)}): not a gfx950 device?")
        _initialised = True
    return lib


def strides4(*s) -> "C.Array":
    return (C.c_int64 * 4)(*[int(x) for x in s])
