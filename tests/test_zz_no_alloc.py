"""rt_matmul_enqueue_static: the K-split product with the library's own static scratch buffer.

The entry point allocates nothing; its results must be those of rt_matmul_enqueue_ws with a
caller-provided workspace, bit for bit (the same kernels run), on calls that follow each other on
one GPU and share the one buffer: a large product first, then a smaller one whose shares cover
only the front of the buffer the first call filled.
"""
import ctypes

import numpy as np
import pytest
import torch

from ratchet_amd import _ffi

pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()).cuda()


def _run(device, oracle, weights, N, M, K, act, seed):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    x = rng.standard_normal((1, M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    if weights == "f16":
        wbuf, wdt, odt = w.astype(np.float16), _ffi.RT_F16, oracle.F16
    else:
        wbuf, wdt, odt = oracle.make_q8_0h(w), _ffi.RT_Q8_0H, oracle.Q8_0H
    desc = _ffi.make_desc(wdt, (N, K), _ffi.RT_F16, (1, M, K), False, True, True, _ffi.RT_F16, (N,))
    need = ctypes.c_uint64()
    L = _ffi.lib()
    assert L.rt_matmul_workspace_bytes(device.ctx, ctypes.byref(desc), ctypes.byref(need)) == _ffi.RT_OK
    assert need.value > 0, "the test shapes are meant to take the split path"
    dw, dx, db = _dev(wbuf), _dev(x), _dev(bias)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # the existing entry point, with a workspace the caller allocated
    ws = torch.empty(need.value, dtype=torch.uint8, device="cuda")
    out_ws = torch.full((M * N * 2,), 0xEE, dtype=torch.uint8, device="cuda")
    st = L.rt_matmul_enqueue_ws(device.ctx, ctypes.byref(desc), dw.data_ptr(), dx.data_ptr(), db.data_ptr(),
                                ctypes.c_void_p(out_ws.data_ptr()), act, ctypes.c_void_p(ws.data_ptr()), need.value, stream)
    assert st == _ffi.RT_OK, L.rt_last_error(device.ctx)
    # the new one: no workspace argument
    out_st = torch.full((M * N * 2,), 0xEE, dtype=torch.uint8, device="cuda")
    st = L.rt_matmul_enqueue_static(device.ctx, ctypes.byref(desc), dw.data_ptr(), dx.data_ptr(), db.data_ptr(),
                                    ctypes.c_void_p(out_st.data_ptr()), act, stream)
    assert st == _ffi.RT_OK, L.rt_last_error(device.ctx)
    torch.cuda.synchronize()
    a = out_ws.cpu().numpy().view(np.float16).reshape(1, M, N)
    b = out_st.cpu().numpy().view(np.float16).reshape(1, M, N)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16)), (weights, N, M, K)
    want = oracle.matmul_ref(wbuf, odt, (N, K), x, oracle.F16, x.shape, bias, False, True, True, act=act)
    assert oracle.max_rel_err(b, want) <= 2e-2, (weights, N, M, K)


@pytest.mark.parametrize("weights", ["q8_0h", "f16"])
def test_static_scratch_matches_workspace_on_consecutive_calls(device, oracle, weights):
    # the Phi-2 prefill down-projection (the whole 20 MiB of scratch), then a smaller product
    _run(device, oracle, weights, 2560, 512, 10240, _ffi.RT_ACT_NONE, 1)
    _run(device, oracle, weights, 320, 96, 2048, _ffi.RT_ACT_GELU, 2)


def test_static_scratch_unsplit_product_and_errors(device, oracle):
    """A product that is not split runs as rt_matmul_enqueue_fused; descriptor errors are statuses."""
    rng = np.random.default_rng(3)
    N, M, K = 4000, 1024, 2048      # thousands of tiles: never split
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    x = rng.standard_normal((1, M, K)).astype(np.float16)
    desc = _ffi.make_desc(_ffi.RT_F16, (N, K), _ffi.RT_F16, (1, M, K), False, True, True)
    L = _ffi.lib()
    dw, dx = _dev(w), _dev(x)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for fn in ("fused", "static"):
        out = torch.full((M * N * 2,), 0xEE, dtype=torch.uint8, device="cuda")
        if fn == "fused":
            st = L.rt_matmul_enqueue_fused(device.ctx, ctypes.byref(desc), dw.data_ptr(), dx.data_ptr(), None,
                                           ctypes.c_void_p(out.data_ptr()), _ffi.RT_ACT_NONE, stream)
        else:
            st = L.rt_matmul_enqueue_static(device.ctx, ctypes.byref(desc), dw.data_ptr(), dx.data_ptr(), None,
                                            ctypes.c_void_p(out.data_ptr()), _ffi.RT_ACT_NONE, stream)
        assert st == _ffi.RT_OK
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy())
    assert np.array_equal(outs[0], outs[1])
    bad = _ffi.make_desc(_ffi.RT_F16, (N, K), _ffi.RT_F16, (1, M, K + 8), False, True, True)
    assert L.rt_matmul_enqueue_static(device.ctx, ctypes.byref(bad), dw.data_ptr(), dx.data_ptr(), None,
                                      ctypes.c_void_p(dx.data_ptr()), _ffi.RT_ACT_NONE, stream) == _ffi.RT_ERR_INVALID_SHAPE
    assert L.rt_matmul_enqueue_static(None, ctypes.byref(desc), None, None, None, None, 0, None) == _ffi.RT_ERR_INVALID_ARG


def test_static_scratch_allocates_nothing_and_passes_checked_mode(device, oracle, monkeypatch):
    """What the entry point exists for: device memory in use is the same before and after its calls; the buffer
    holds what the Phi-2 prefill down-projection's split asks for; and in checked mode (RATCHET_CHECKED) the library
    does not look its own static buffer up as if it were a caller's allocation."""
    L = _ffi.lib()
    N, M, K = 2560, 512, 10240
    desc = _ffi.make_desc(_ffi.RT_Q8_0H, (N, K), _ffi.RT_F16, (1, M, K), False, True, True, _ffi.RT_F16, (N,))
    need = ctypes.c_uint64()
    assert L.rt_matmul_workspace_bytes(device.ctx, ctypes.byref(desc), ctypes.byref(need)) == _ffi.RT_OK
    static_bytes = 20 << 20   # RT_STATIC_SCRATCH_BYTES of include/ratchet_hip.h
    assert 0 < need.value <= static_bytes
    rng = np.random.default_rng(4)
    wbuf = oracle.make_q8_0h((rng.standard_normal((N, K)) * 0.05).astype(np.float32))
    x = rng.standard_normal((1, M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    dw, dx, db = _dev(wbuf), _dev(x), _dev(bias)
    out = torch.empty(M * N * 2, dtype=torch.uint8, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def call(ctx):
        return L.rt_matmul_enqueue_static(ctx, ctypes.byref(desc), dw.data_ptr(), dx.data_ptr(), db.data_ptr(),
                                          ctypes.c_void_p(out.data_ptr()), _ffi.RT_ACT_NONE, stream)
    assert call(device.ctx) == _ffi.RT_OK   # warm-up: code objects loaded, kernel attributes set
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        assert call(device.ctx) == _ffi.RT_OK
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    first = out.cpu().numpy().copy()
    # checked mode: a context created with RATCHET_CHECKED set runs the same call
    monkeypatch.setenv("RATCHET_CHECKED", "1")
    ctx = ctypes.c_void_p()
    assert L.rt_ctx_create(device.ordinal, ctypes.byref(ctx)) == _ffi.RT_OK
    try:
        out.fill_(0xEE)
        assert call(ctx) == _ffi.RT_OK, L.rt_last_error(ctx)
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), first)
    finally:
        L.rt_ctx_destroy(ctx)
