"""The C-ABI library loads and exports every symbol ``include/mi355dnn.h`` declares, and its
planners (which launch nothing) answer without a GPU: every refusal is a named decline that can
be asserted by constructing the call, the reference's own way of testing plans
(DNNKernels/test/test_flash.jl:358-365, test_coopmat_attention.jl:92-134)."""
import ctypes as C
import os
import re

import pytest

from juliavision_amd import _lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "mi355dnn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    names = _declared()
    assert len(names) >= 17
    lib = L.load()
    for n in names:
        assert hasattr(lib, n), n
        assert n in L.SIGNATURES, f"{n} has no ctypes signature"
    assert set(L.SIGNATURES) == set(names)
    assert lib.mi_version() == 1


def test_compute_calls_refuse_without_a_device():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    lib = L.load()
    assert lib.mi_layernorm_f16(0x1000, None, None, 0x2000, None, None, 8, 1, 1e-5, None) == L.ERROR_DEVICE
    assert lib.mi_add_f16(0x1000, 0x1000, 0x1000, 8, None) == L.ERROR_DEVICE
    with pytest.raises(RuntimeError):
        L.init()


def _gemm_plan(T, K, F, *, ldY=None, ldX=None, ldW=None, layout=L.W_KF, y=0x10000, x=0x20000, w=0x30000, dt=L.F16, nb=1):
    ldY = F if ldY is None else ldY
    ldX = K if ldX is None else ldX
    ldW = (F if layout == L.W_KF else K) if ldW is None else ldW
    return L.GEMM_PATHS[L.load().mi_gemm_f16_plan(y, x, w, T, K, F, ldY, ldX, ldW, layout, dt, nb, T * ldY, T * ldX, 0)]


def test_gemm_planner():
    assert _gemm_plan(1500, 1280, 5120) == "mfma"
    assert _gemm_plan(1500, 1280, 5120, layout=L.W_FK) == "mfma"
    assert _gemm_plan(1370, 384, 1152) == "mfma"
    for T in (1, 4, 8):
        assert _gemm_plan(T, 1280, 1280) == "skinny"
        assert _gemm_plan(T, 1280, 5120, layout=L.W_FK) == "skinny"
    assert _gemm_plan(9, 1280, 1280) == "mfma"
    assert _gemm_plan(8, 1280, 1280, nb=2) == "mfma"
    # extents or pointers the 16-byte loads cannot address fall to the scalar kernel, as a ragged
    # extent falls off the reference's fast kernel (tools/census_gemm_declines.jl:8-14)
    assert _gemm_plan(1288, 1284, 1288) == "scalar"
    assert _gemm_plan(64, 64, 60) == "scalar"                    # [K][F] rows of 60 halves
    assert _gemm_plan(64, 64, 60, layout=L.W_FK) == "mfma"       # [F][K] rows are K-contiguous
    assert _gemm_plan(64, 64, 64, x=0x20002) == "scalar"
    assert _gemm_plan(64, 64, 64, ldX=60) == "decline"
    assert _gemm_plan(0, 64, 64) == "decline"
    assert _gemm_plan(64, 64, 64, dt=7) == "decline"


def test_planning_for_a_device_one_does_not_have():
    """The reference's planners take a DeviceCaps value, so its tests ask about hardware they do not have
    (test_flash.jl:328 `DeviceCaps(dev; cores=1)`, :363 `coopmat=false`, :373-377 a wave64 device).  The C planners
    answer the same questions through the *_plan_caps entry points; the description does not outlive the call."""
    lib = L.load()
    caps = lambda mfma, cus: (C.c_int64 * 6)(mfma, 16, 64, 160 * 1024, 1024, cus)
    ks, ns = C.c_int(0), C.c_int(0)

    def gemm(c, T, K, F):
        r = lib.mi_gemm_f16_plan_caps(c, 0x10000, 0x20000, 0x30000, T, K, F, F, K, F, L.W_KF, L.F16, 1, 0, 0, 0, C.byref(ks))
        return L.GEMM_PATHS[r], ks.value

    def sdpa(c, E, Lq, Lk, H, B):
        d = lambda n: L.strides4(1, E, E * n, E * n * H)
        r = lib.mi_sdpa_f16_plan_caps(c, 0x10000, d(Lq), 0x20000, d(Lk), 0x30000, d(Lk), 0, 0, E, Lq, Lk, H, B, 0.125, C.byref(ns))
        return L.SDPA_PATHS[r], ns.value

    # config 2's second MLP linear: 120 tiles of 128 x 128 leave half of 256 compute units idle, so K is cut in two;
    # on 64 units the tiles alone fill the device twice over and nothing is cut; without a matrix unit there is no
    # tiled path at all (mm_coopmat_plan's `dev.coopmat` gate, matmul.jl:172-179), the decode-sized kernel remains
    assert gemm(None, 1500, 5120, 1280) == gemm(caps(1, 256), 1500, 5120, 1280) == ("mfma", 2)
    assert gemm(caps(1, 64), 1500, 5120, 1280) == ("mfma", 1)
    assert gemm(caps(1, 64), 300, 5120, 1280)[1] < gemm(caps(1, 1024), 300, 5120, 1280)[1]
    assert gemm(caps(0, 256), 1500, 5120, 1280) == ("scalar", 1)
    assert gemm(caps(0, 256), 4, 1280, 1280)[0] == "skinny"
    # 23 queries over 4096 keys, the reference's flash-decoding case: the key splits follow the compute units
    # (two workgroups per unit, splitcount, flash.jl:1288-1303); a one-unit device does not split, a device without a
    # matrix unit gets the always-available path (Decline(:nocoopmat) -> three-pass, attention.jl:735-759)
    assert sdpa(caps(1, 256), 16, 23, 4096, 8, 1) == ("flash", 16)
    assert sdpa(caps(1, 48), 16, 23, 4096, 8, 1) == ("flash", 11)
    assert sdpa(caps(1, 1), 16, 23, 4096, 8, 1) == ("rows", 1)
    assert sdpa(caps(0, 256), 64, 4096, 4096, 16, 1)[0] == "rows"
    assert sdpa(caps(1, 1), 64, 1, 1500, 20, 1) == ("rows", 1) and sdpa(caps(1, 256), 64, 1, 1500, 20, 1) == ("rows", 4)
    # nothing leaks into the planners of the running device
    assert _sdpa_plan(64, 4096, 4096, 16, 1) == ("flash", 1) and _gemm_plan(1500, 5120, 1280) == "mfma"


def test_gemm_workspace():
    lib = L.load()
    assert lib.mi_gemm_f16_workspace(1500, 1280, 5120, L.W_KF, 1) == 0
    n = lib.mi_gemm_f16_workspace(4, 1280, 1280, L.W_KF, 1)
    assert n > 0 and n % 256 == 0 and n % (4 * 1280 * 4) == 0
    assert lib.mi_gemm_f16_workspace(4, 1280, 1280, L.W_FK, 1) == 0      # that kernel finishes its outputs itself


def _sdpa_plan(E, Lq, Lk, H, B, *, bias=0, scale=0.125, qs=None, ptr=0x10000):
    dense = lambda L_: L.strides4(1, E, E * L_, E * L_ * H)
    ns = C.c_int(0)
    path = L.load().mi_sdpa_f16_plan(ptr, qs or dense(Lq), 0x20000, dense(Lk), 0x30000, dense(Lk), bias, 0, E, Lq, Lk, H, B, scale, C.byref(ns))
    return L.SDPA_PATHS[path], ns.value


def test_sdpa_planner():
    assert _sdpa_plan(64, 4096, 4096, 16, 1) == ("flash", 1)
    assert _sdpa_plan(64, 1500, 1500, 20, 1)[0] == "flash"
    assert _sdpa_plan(72, 256, 256, 8, 16)[0] == "flash"
    # an additive mask (planned as a dense fp16 (Lk, Lq, H, B) array) stays in the fused kernel where its rows start on
    # 4-byte boundaries -- the reference's fused plan declines every mask, Decline(:bias), flash.jl:1327 -- keys unsplit
    assert _sdpa_plan(64, 1500, 1500, 20, 1, bias=1) == ("flash", 1)
    assert _sdpa_plan(64, 128, 8192, 1, 1, bias=1) == ("flash", 1) and _sdpa_plan(64, 128, 8192, 1, 1)[1] > 1
    # head size 64 on few tiles: four waves a 32-query tile, each with a quarter of the keys, unless the keys are so many
    # that splits over workgroups win (above); a wider head keeps the splits
    assert _sdpa_plan(64, 128, 2048, 1, 1) == ("flash", 1) and _sdpa_plan(64, 1370, 1370, 6, 1) == ("flash", 1)
    assert _sdpa_plan(72, 128, 2048, 1, 1)[1] > 1
    assert _sdpa_plan(64, 1500, 1371, 20, 1, bias=1)[0] == "rows"          # odd row length: fp16 rows at 2-byte offsets
    assert _sdpa_plan(64, 1, 448, 20, 1)[0] == "rows"
    assert _sdpa_plan(20, 128, 128, 2, 1)[0] == "rows"                     # E not a multiple of 8
    assert _sdpa_plan(64, 128, 128, 2, 1, qs=L.strides4(2, 128, 128 * 128, 0))[0] == "rows"   # head dim not contiguous
    assert _sdpa_plan(64, 128, 128, 2, 1, ptr=0x10002)[0] == "rows"
    assert _sdpa_plan(64, 128, 128, 2, 1, scale=-1.0)[0] == "rows"
    assert _sdpa_plan(512, 128, 128, 2, 1)[0] == "decline"
    # a single query row runs in one launch whose key range is cut over workgroups that merge inside it: at most one
    # workgroup per CU, a round of six 64-key passes each (24 passes over 20 rows -> 4 ways; 160 rows fill the chip whole);
    # anything the one-launch kernel does not take (here a mask) gets the rows kernel's splits, two workgroups per CU,
    # never more than one per 64 keys (flash.jl:1288-1303)
    p1, n1 = _sdpa_plan(64, 1, 1500, 20, 1)
    p8, n8 = _sdpa_plan(64, 1, 1500, 20, 8)
    assert p1 == p8 == "rows" and n1 == 4 and n8 == 1
    assert _sdpa_plan(64, 1, 448, 20, 1) == ("rows", 1)                      # a short key range: one workgroup per head
    assert _sdpa_plan(64, 1, 700, 20, 1)[1] == 2                             # 11 passes: two rounds
    assert _sdpa_plan(64, 1, 1500, 20, 1, bias=1)[1] == 24                   # masked: the rows kernel, split 24 ways
    assert _sdpa_plan(64, 23, 17, 4, 1)[1] == 1
    # 8 to 63 queries over a long key range on few (head, batch) tiles: the fused kernel with its keys cut over
    # workgroups (the reference's flash-decoding case), not one workgroup per query row
    assert _sdpa_plan(16, 23, 4096, 8, 1) == ("flash", 16) and _sdpa_plan(16, 23, 4096, 8, 1, bias=1)[0] == "rows"
    assert _sdpa_plan(64, 23, 300, 8, 1)[0] == "rows" and _sdpa_plan(64, 23, 4096, 200, 1)[0] == "rows"


def test_conv_planner_and_extents():
    lib = L.load()
    plan = lambda *a: L.CONV_PATHS[lib.mi_conv2d_f16_plan(*a)]
    assert plan(518, 518, 3, 1, 14, 14, 384, 14, 14, 0, 0, 1, 1, 1) == "im2col_gemm"
    assert plan(64, 64, 256, 1, 3, 3, 256, 1, 1, 1, 1, 1, 1, 1) == "implicit_gemm"   # stride 1, OW % 8 == 0, Cin % 64 == 0
    assert plan(64, 64, 32, 1, 3, 3, 256, 1, 1, 1, 1, 1, 1, 1) == "im2col_gemm"      # 32 channels do not fill a 64-deep tile
    assert plan(60, 64, 256, 1, 3, 3, 256, 1, 1, 1, 1, 1, 1, 1) == "im2col_gemm"     # OW = 60
    assert plan(256, 256, 144, 1, 1, 1, 256, 1, 1, 0, 0, 1, 1, 1) == "gemm_1x1"     # onebyone, conv.jl:63-66
    assert plan(256, 256, 144, 1, 1, 1, 256, 2, 2, 0, 0, 1, 1, 1) == "im2col_gemm"
    assert plan(64, 64, 256, 1, 3, 3, 256, 1, 1, 1, 1, 1, 1, 4) == "direct"
    assert plan(64, 64, 255, 1, 3, 3, 256, 1, 1, 1, 1, 1, 1, 4) == "decline"
    assert plan(2, 2, 3, 1, 5, 5, 8, 1, 1, 0, 0, 1, 1, 1) == "decline"              # empty output
    assert lib.mi_convsize(518, 14, 14, 0, 1) == 37 and lib.mi_convsize(256, 7, 4, 3, 1) == 64
    # implicit GEMM scratch: the zero-padded input [Cin][H+2][W+2 -> 72] fp16 twice (the second copy shifted by one
    # element, for taps that start at an odd column), the weights re-laid tap-major; K = 2304 is shallow enough for
    # one pass of 64 x 64 tiles, K = 9216 is split into fp32 planes of the 256 x 4096 output
    ws = lib.mi_conv2d_f16_workspace(64, 64, 256, 1, 3, 3, 256, 1, 1, 1, 1, 1, 1)
    assert ws == 2 * 256 * 66 * 72 * 2 + 256 * 2304 * 2
    ws = lib.mi_conv2d_f16_workspace(64, 64, 1024, 1, 3, 3, 256, 1, 1, 1, 1, 1, 1)
    planes = ws - (2 * 1024 * 66 * 72 * 2 + 256 * 9216 * 2)
    assert planes >= 2 * 256 * 4096 * 4 and planes % (256 * 4096 * 4) == 0
    # im2col scratch: col[CRS->64][PQ->8] fp16 + the weights padded likewise (588 taps: 640; under 256 taps the depth
    # is rounded up to 8 only)
    ws3 = lib.mi_conv2d_f16_workspace(518, 518, 3, 1, 14, 14, 384, 14, 14, 0, 0, 1, 1)
    assert ws3 == -(-(640 * 1376 * 2) // 256) * 256 + 384 * 640 * 2
    ws4 = lib.mi_conv2d_f16_workspace(64, 64, 5, 1, 3, 3, 32, 1, 1, 1, 1, 1, 1)                # 45 taps -> 48
    assert ws4 >= 48 * 4096 * 2 + 32 * 48 * 2 and ws4 < 56 * 4096 * 2 + 32 * 56 * 2 + (1 << 20)
    assert lib.mi_conv2d_f16_workspace(256, 256, 144, 1, 1, 1, 256, 1, 1, 0, 0, 1, 1) == 0


def test_convtranspose_planner_takes_only_the_non_overlapping_case():
    """The case list of test_convtranspose_gemm.jl:64-75."""
    lib = L.load()
    plan = lambda *a: L.CONVT_PATHS[lib.mi_convtranspose2d_f16_plan(*a)]
    #            W  H  Cin N KW KH Cout sx sy px py dx dy ox oy g
    assert plan(8, 8, 8, 1, 2, 2, 8, 2, 2, 0, 0, 1, 1, 0, 0, 1) == "gemm_shuffle"
    assert plan(8, 8, 8, 1, 3, 3, 8, 2, 2, 0, 0, 1, 1, 0, 0, 1) == "gather"        # overlapping fields
    assert plan(8, 8, 8, 1, 2, 2, 8, 2, 2, 1, 1, 1, 1, 0, 0, 1) == "gather"        # padding
    assert plan(8, 8, 8, 1, 2, 2, 8, 2, 2, 0, 0, 2, 2, 0, 0, 1) == "gather"        # dilation
    assert plan(8, 8, 8, 1, 2, 2, 8, 2, 2, 0, 0, 1, 1, 1, 1, 1) == "gather"        # output padding
    assert plan(8, 8, 8, 1, 2, 2, 8, 2, 2, 0, 0, 1, 1, 0, 0, 2) == "gather"        # groups
    assert plan(8, 8, 8, 1, 2, 2, 8, 2, 2, 0, 0, 1, 1, 2, 0, 1) == "decline"       # output padding >= stride
    assert plan(8, 8, 9, 1, 2, 2, 8, 2, 2, 0, 0, 1, 1, 0, 0, 2) == "decline"
    assert lib.mi_convtransposesize(64, 2, 2, 0, 1, 0) == 128 and lib.mi_convtransposesize(8, 3, 2, 0, 1, 0) == 17
    # scratch of SAM 2's first upsampler (256 -> 64 channels on 64x64, test_convtranspose_gemm.jl:36): the transposed
    # weights [Cout*4][Cin], the expanded bias, the unshuffled GEMM result [Cout*4][H*W]; the GEMM itself needs none
    ws = lib.mi_convtranspose2d_f16_workspace(64, 64, 256, 1, 2, 2, 64, 2, 2, 0, 0, 1, 1, 0, 0, 1)
    assert ws == 256 * 256 * 2 + 256 * 2 + 256 * 4096 * 2 + lib.mi_gemm_f16_workspace(256, 256, 4096, L.W_KF, 1)
    assert lib.mi_convtranspose2d_f16_workspace(8, 8, 8, 1, 3, 3, 8, 2, 2, 0, 0, 1, 1, 0, 0, 1) == 0


def test_host_planners_decline_by_name_on_cpu_tensors():
    import torch
    import juliavision_amd as jv
    a = torch.zeros((8, 8), dtype=torch.float16)
    assert jv.mmplan(jv.MI355X, a, a, a) == jv.Decline("operands")
    assert not jv.mmplan(jv.MI355X, a, a, a)
    x = torch.zeros((1, 8, 8, 8), dtype=torch.float16)
    assert jv.conv_plan(jv.MI355X, x, x, x) == jv.Decline("operands")
    assert jv.convsize(518, 14, 14, 0, 1) == 37


def test_small_operands_are_validated_before_their_pointer_is_taken():
    """bias / gamma / beta / mean / rstd reach the kernels as raw pointers read at a fixed length and type: the host
    wrappers refuse a wrong dtype, length or stride by name instead of launching an out-of-bounds read."""
    import torch
    from juliavision_amd import kernels as K
    f16 = torch.float16
    ok = torch.zeros(16, dtype=f16)
    assert K._vec_problem("bias", ok, 16, require_cuda=False) is None
    assert K._vec_problem("bias", None, 16) is None
    assert "GPU" in K._vec_problem("bias", ok, 16)
    assert "float32" in K._vec_problem("bias", torch.zeros(16), 16, require_cuda=False)          # fp32 bias of a mixed-precision export
    assert "16 elements" in K._vec_problem("gamma", ok, 24, require_cuda=False)                  # shorter than the row
    assert "contiguous" in K._vec_problem("beta", torch.zeros(32, dtype=f16)[::2], 16, require_cuda=False)
    assert K._vec_problem("mean", torch.zeros(4), 4, torch.float32, require_cuda=False) is None
    assert "float16" in K._vec_problem("mean", torch.zeros(4, dtype=f16), 4, torch.float32, require_cuda=False)
    with pytest.raises(K.DeclineError, match="layernorm_: gamma is not on the GPU"):
        K._check_vecs("layernorm_", L.DECLINE_OPERANDS, ("beta", None, 24), ("gamma", ok, 24))
    # the planner turns an unreadable bias into a decline (on the CPU every operand declines first, so only the order
    # of the checks is visible here: operands, then extents, then the bias)
    dev = K.MI355X
    assert K.mmplan(dev, torch.zeros(4, 8, dtype=f16), torch.zeros(8, 8, dtype=f16), torch.zeros(4, 8, dtype=f16)).reason == "operands"
