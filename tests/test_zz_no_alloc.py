"""mi_gemm_f16_noalloc: the GEMM entry point that allocates nothing (its split-K / decode planes live in a static
device array of the library) against mi_gemm_f16 with a caller workspace, through the raw C ABI.  Both run the same
plan and kernels, so the outputs must agree bit for bit; mi_gemm_f16 itself is held to the oracle by
test_gemm_gpu.py, and the first case is checked against the oracle here as well.  Two calls in a row share the
static array, the second with a smaller input; a call whose planes exceed the array is refused by name."""
import numpy as np
import pytest

import oracle
from util import assert_parity, poison, to_dev, to_host

pytestmark = pytest.mark.gpu


def _both(lib, L, T, K, F, layout, epi, seed, residual):
    import torch
    X = oracle.randn_f16((T, K), seed, 0, 1.0 / np.sqrt(K))
    Wkf = oracle.randn_f16((K, F), seed + 1, 0, 1.0)
    b = oracle.randn_f16((F,), seed + 2, 0, 0.02)
    R = oracle.randn_f16((T, F), seed + 3, 0, 1.0) if residual else None
    dX, db = to_dev(X), to_dev(b)
    dW = to_dev(Wkf) if layout == L.W_KF else to_dev(np.ascontiguousarray(Wkf.T))
    dR = None if R is None else to_dev(R)
    ldW = F if layout == L.W_KF else K
    need = lib.mi_gemm_f16_workspace(T, K, F, layout, 1)
    assert 0 < need <= L.NOALLOC_SCRATCH_BYTES, "the case must use scratch, within the static array"
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    want = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
    got = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
    rp = None if dR is None else dR.data_ptr()
    rc = lib.mi_gemm_f16(want.data_ptr(), dX.data_ptr(), dW.data_ptr(), db.data_ptr(), rp, T, K, F, F, K, ldW,
                         layout, L.BIAS_COL, L.EPI[epi], L.F16, ws.data_ptr(), need, st)
    assert rc == L.OK
    rc = lib.mi_gemm_f16_noalloc(got.data_ptr(), dX.data_ptr(), dW.data_ptr(), db.data_ptr(), rp, T, K, F, F, K, ldW,
                                 layout, L.BIAS_COL, L.EPI[epi], L.F16, st)
    assert rc == L.OK
    torch.cuda.synchronize()
    g, w = to_host(got), to_host(want)
    assert np.all(np.isfinite(g)), "unwritten output"
    assert np.array_equal(g.view(np.uint16), w.view(np.uint16)), f"noalloc differs from mi_gemm_f16 at T{T} K{K} F{F}"
    return g, (X, Wkf, b, R)


def test_noalloc_matches_workspace_entry_on_two_calls_in_a_row():
    import torch
    from juliavision_amd import _lib as L
    lib = L.init()
    # split-K over fp32 planes (tiled kernels): the larger call first, then a smaller one on the same static array
    g, (X, W, b, R) = _both(lib, L, 1500, 5120, 1280, L.W_KF, "none", 11, True)
    assert_parity(g, oracle.gemm_f16(X, W, b, w_layout="kf", bias_mode="col", epi="none", residual=R), what="noalloc fc2")
    _both(lib, L, 200, 4096, 256, L.W_FK, "gelu", 21, False)
    # decode-sized rows: the [K][F] kernel's planes
    _both(lib, L, 8, 1280, 5120, L.W_KF, "gelu", 31, True)
    _both(lib, L, 1, 1280, 1280, L.W_KF, "none", 41, False)
    # a call that needs no scratch goes straight through
    T, K, F = 300, 256, 384
    assert lib.mi_gemm_f16_workspace(T, K, F, L.W_KF, 1) == 0
    X = oracle.randn_f16((T, K), 51, 0, 1.0 / np.sqrt(K))
    W = oracle.randn_f16((K, F), 52)
    out = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
    dX, dW = to_dev(X), to_dev(W)
    rc = lib.mi_gemm_f16_noalloc(out.data_ptr(), dX.data_ptr(), dW.data_ptr(), None, None, T, K, F, F, K, F,
                                 L.W_KF, L.BIAS_NONE, L.EPI["none"], L.F16, torch.cuda.current_stream().cuda_stream)
    assert rc == L.OK
    torch.cuda.synchronize()
    assert_parity(to_host(out), oracle.gemm_f16(X, W, None), what="noalloc without scratch")


def test_noalloc_refuses_beyond_its_static_array():
    import torch
    from juliavision_amd import _lib as L
    lib = L.init()
    big = None
    for T, K, F in [(1100, 65536, 1024), (2048, 32768, 1280), (1500, 40960, 1536), (8, 8192, 200000)]:
        if lib.mi_gemm_f16_workspace(T, K, F, L.W_KF, 1) > L.NOALLOC_SCRATCH_BYTES:
            big = (T, K, F)
            break
    assert big is not None, "no candidate shape plans more scratch than the static array"
    T, K, F = big
    y = poison(torch.empty((8, 8), dtype=torch.float16, device="cuda"))
    # refused before anything is read: the operand pointers only have to be non-null
    rc = lib.mi_gemm_f16_noalloc(y.data_ptr(), y.data_ptr(), y.data_ptr(), None, None, T, K, F, F, K, F,
                                 L.W_KF, L.BIAS_NONE, L.EPI["none"], L.F16, torch.cuda.current_stream().cuda_stream)
    assert rc == L.DECLINE_SCRATCH_LIMIT
    torch.cuda.synchronize()
    assert bool(torch.isnan(y).all()), "a refused call wrote something"


def test_noalloc_under_graph_capture():
    """The callers this entry point exists for: the call is captured into a device graph (in the capture mode that turns
    any allocation, free or synchronisation made by the thread into an error), replayed over changed inputs with eager
    work in between, and every replay must give the bits of mi_gemm_f16 with a caller workspace; free device memory
    does not shrink across the replays."""
    import torch
    from juliavision_amd import _lib as L
    lib = L.init()
    T, K, F = 200, 4096, 256
    need = lib.mi_gemm_f16_workspace(T, K, F, L.W_FK, 1)
    assert 0 < need <= L.NOALLOC_SCRATCH_BYTES
    Wkf = oracle.randn_f16((K, F), 62, 0, 1.0)
    dW, db = to_dev(np.ascontiguousarray(Wkf.T)), to_dev(oracle.randn_f16((F,), 63, 0, 0.02))
    dX = to_dev(oracle.randn_f16((T, K), 61, 0, 1.0 / np.sqrt(K)))
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    got = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))
    want = poison(torch.empty((T, F), dtype=torch.float16, device="cuda"))

    def noalloc(stream):
        return lib.mi_gemm_f16_noalloc(got.data_ptr(), dX.data_ptr(), dW.data_ptr(), db.data_ptr(), None, T, K, F, F, K, K,
                                       L.W_FK, L.BIAS_COL, L.EPI["gelu"], L.F16, stream)
    assert noalloc(torch.cuda.current_stream().cuda_stream) == L.OK      # a first call outside the capture, as a host would warm up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, capture_error_mode="global"):
        assert noalloc(torch.cuda.current_stream().cuda_stream) == L.OK
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for seed in (71, 72, 73):
        dX.copy_(to_dev(oracle.randn_f16((T, K), seed, 0, 1.0 / np.sqrt(K))))
        poison(got)
        graph.replay()
        rc = lib.mi_gemm_f16(want.data_ptr(), dX.data_ptr(), dW.data_ptr(), db.data_ptr(), None, T, K, F, F, K, K,
                             L.W_FK, L.BIAS_COL, L.EPI["gelu"], L.F16, ws.data_ptr(), need, torch.cuda.current_stream().cuda_stream)
        assert rc == L.OK
        torch.cuda.synchronize()
        g, w = to_host(got), to_host(want)
        assert np.all(np.isfinite(g)), "unwritten output"
        assert np.array_equal(g.view(np.uint16), w.view(np.uint16)), f"replay with seed {seed} differs from mi_gemm_f16"
    assert torch.cuda.mem_get_info()[0] >= free_before, "device memory shrank across replays of a call that allocates nothing"
