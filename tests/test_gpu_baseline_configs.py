"""The five BASELINE configurations at full size: HIP path vs the CPU oracle on the
same seeded inputs, plus size-independent properties (linearity, one-hot selection,
stack independence)."""
import numpy as np
import pytest

from ratchet_amd import DType, Device, Tensor

pytestmark = pytest.mark.gpu


def gpu_matmul(device, lhs, rhs, bias, tl, tr, to):
    c = lhs.to(device).gemm(rhs.to(device), None if bias is None else bias.to(device), tl, tr, to).resolve()
    return c.to(Device.CPU).storage


def test_c1_f32_whisper_mlp(device, oracle):
    rng = np.random.default_rng(0)   # seed 0, N(0,1) * 0.05
    a = (rng.standard_normal((1500, 384)) * 0.05).astype(np.float32)
    b = (rng.standard_normal((384, 1536)) * 0.05).astype(np.float32)
    bias = (rng.standard_normal(1536) * 0.05).astype(np.float32)
    got = gpu_matmul(device, Tensor.from_data(a), Tensor.from_data(b), Tensor.from_data(bias), False, False, False)
    want = oracle.matmul_ref(a, oracle.F32, a.shape, b, oracle.F32, b.shape, bias)
    assert oracle.max_rel_err(got, want) <= 1e-3
    assert oracle.all_close(want, got, 1e-4, 1e-4)[0]


@pytest.fixture(scope="module")
def phi2_up(oracle):
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((10240, 2560)) * 0.02).astype(np.float32)
    buf = oracle.make_q8_0h(w)
    bias = rng.standard_normal(10240).astype(np.float16)
    return buf, bias


@pytest.mark.parametrize("M", [1, 4, 8])
def test_c2_q8_gemv_phi2_decode(device, oracle, phi2_up, M):
    buf, bias = phi2_up
    rng = np.random.default_rng(M)
    x = rng.standard_normal((1, M, 2560)).astype(np.float16)
    W = Tensor.from_quantized(buf, DType.Q8_0H, (10240, 2560))
    got = gpu_matmul(device, W, Tensor.from_data(x), Tensor.from_data(bias), False, True, True)
    want = oracle.matmul_ref(buf, oracle.Q8_0H, (10240, 2560), x, oracle.F16, x.shape, bias, False, True, True)
    assert got.shape == (1, M, 10240) and oracle.max_rel_err(got, want) <= 2e-2


def test_c2_properties_full_size(device, oracle, phi2_up):
    buf, _ = phi2_up
    W = Tensor.from_quantized(buf, DType.Q8_0H, (10240, 2560)).to(device)
    rng = np.random.default_rng(9)
    # one-hot rows select dequantized weights exactly (ties the GEMV to the bit-exact dequantizer)
    cols = rng.integers(0, 2560, size=8)
    x = np.zeros((8, 2560), np.float16)
    x[np.arange(8), cols] = 1
    got = gpu_matmul(device, W, Tensor.from_data(x), None, False, True, True)
    dq = oracle.q8_0_dequantize(buf, 10240 * 2560, True).reshape(10240, 2560)
    assert np.array_equal(got, dq[:, cols].T.astype(np.float16))
    # rows of a batch are independent: M = 8 (matrix-core kernel) equals M = 1 calls (row-streaming kernel) and M = 4
    # calls (the 4x4x4 kernel) as closely as f32 accumulation in a different order allows.  Every product q * x is exact
    # in f32 and every kernel applies the block scales in f32, so two kernels' f32 sums differ by a few f32 roundings
    # of the magnitude that was summed, S = sum_k |w x|; the results are those sums rounded to f16 once: they differ by
    # at most one f16 unit in the last place plus that f32 noise (which only shows where a result is much smaller than S)
    x = rng.standard_normal((8, 2560)).astype(np.float16)
    full = gpu_matmul(device, W, Tensor.from_data(x), None, False, True, True)
    S = np.abs(dq) @ np.abs(x.astype(np.float32)).T                                      # [10240, 8]
    for rows in ([0], [3], [7], [2, 3, 4, 5]):
        part = gpu_matmul(device, W, Tensor.from_data(x[rows]), None, False, True, True)
        a, b = part.astype(np.float32), full[rows].astype(np.float32)
        ulp = np.spacing(np.maximum(np.abs(part), np.abs(full[rows])).astype(np.float16)).astype(np.float32)
        assert np.all(np.abs(a - b) <= ulp + 2e-6 * S[:, rows].T), (rows, float(np.max(np.abs(a - b) / ulp)))
    # linearity in x (exact scaling by a power of two)
    two = gpu_matmul(device, W, Tensor.from_data((x * np.float16(2)).astype(np.float16)), None, False, True, True)
    f32 = full.astype(np.float32)
    assert np.all(np.abs(two.astype(np.float32) - 2 * f32) <= 2.0 ** -23 + 1e-3 * np.abs(f32))


def test_c3_attention_matmuls(device, oracle):
    rng = np.random.default_rng(1)   # seed 1
    q = rng.standard_normal((1, 32, 512, 80)).astype(np.float16)
    k = rng.standard_normal((1, 32, 512, 80)).astype(np.float16)
    v = rng.standard_normal((1, 32, 512, 80)).astype(np.float16)
    p = (rng.random((1, 32, 512, 512)) / 512).astype(np.float16)
    s = gpu_matmul(device, Tensor.from_data(q), Tensor.from_data(k), None, False, True, False)
    want = oracle.matmul_ref(q, oracle.F16, q.shape, k, oracle.F16, k.shape, None, False, True, False)
    assert s.shape == (1, 32, 512, 512) and oracle.max_rel_err(s, want) <= 2e-2
    o = gpu_matmul(device, Tensor.from_data(p), Tensor.from_data(v), None, False, False, False)
    want = oracle.matmul_ref(p, oracle.F16, p.shape, v, oracle.F16, v.shape)
    assert o.shape == (1, 32, 512, 80) and oracle.max_rel_err(o, want) <= 2e-2


def test_c4_q8_gemm_phi2_prefill(device, oracle, phi2_up):
    buf, bias = phi2_up
    rng = np.random.default_rng(4)
    x = rng.standard_normal((1, 512, 2560)).astype(np.float16)
    got = gpu_matmul(device, Tensor.from_quantized(buf, DType.Q8_0H, (10240, 2560)), Tensor.from_data(x),
                     Tensor.from_data(bias), False, True, True)
    want = oracle.matmul_ref(buf, oracle.Q8_0H, (10240, 2560), x, oracle.F16, x.shape, bias, False, True, True)
    assert got.shape == (1, 512, 10240) and oracle.max_rel_err(got, want) <= 2e-2
    # down projection [512 x 10240] . W_down[2560 x 10240]^T
    wd = oracle.make_q8_0h((rng.standard_normal((2560, 10240)) * 0.02).astype(np.float32))
    bd = rng.standard_normal(2560).astype(np.float16)
    h = rng.standard_normal((1, 512, 10240)).astype(np.float16)
    got = gpu_matmul(device, Tensor.from_quantized(wd, DType.Q8_0H, (2560, 10240)), Tensor.from_data(h),
                     Tensor.from_data(bd), False, True, True)
    want = oracle.matmul_ref(wd, oracle.Q8_0H, (2560, 10240), h, oracle.F16, h.shape, bd, False, True, True)
    assert got.shape == (1, 512, 2560) and oracle.max_rel_err(got, want) <= 2e-2


def test_c4_f16_weights_phi2_prefill(device, oracle):
    """The metric's f16 GEMM: [512 x 2560] . [10240 x 2560]^T + b with f16 weights, full size, then the
    down-projection [512 x 10240] . [2560 x 10240]^T; each output against the oracle's f32 GEMM."""
    rng = np.random.default_rng(4)
    w = (rng.standard_normal((10240, 2560)) * 0.02).astype(np.float16)
    bias = rng.standard_normal(10240).astype(np.float16)
    x = rng.standard_normal((1, 512, 2560)).astype(np.float16)
    got = gpu_matmul(device, Tensor.from_data(w), Tensor.from_data(x), Tensor.from_data(bias), False, True, True)
    want = oracle.matmul_ref(w, oracle.F16, w.shape, x, oracle.F16, x.shape, bias, False, True, True)
    assert got.shape == (1, 512, 10240) and oracle.max_rel_err(got, want) <= 2e-2
    # the same product spelled from the activation side: x.matmul(W, false, true) + no bias
    got = gpu_matmul(device, Tensor.from_data(x), Tensor.from_data(w), None, False, True, False)
    want = oracle.matmul_ref(x, oracle.F16, x.shape, w, oracle.F16, w.shape, None, False, True, False)
    assert got.shape == (1, 512, 10240) and oracle.max_rel_err(got, want) <= 2e-2
    wd = (rng.standard_normal((2560, 10240)) * 0.02).astype(np.float16)
    bd = rng.standard_normal(2560).astype(np.float16)
    h = rng.standard_normal((1, 512, 10240)).astype(np.float16)
    got = gpu_matmul(device, Tensor.from_data(wd), Tensor.from_data(h), Tensor.from_data(bd), False, True, True)
    want = oracle.matmul_ref(wd, oracle.F16, wd.shape, h, oracle.F16, h.shape, bd, False, True, True)
    assert got.shape == (1, 512, 2560) and oracle.max_rel_err(got, want) <= 2e-2


@pytest.mark.parametrize("M", [1, 16, 256])
def test_c5_q4k_phi3(device, oracle, M):
    rng = np.random.default_rng(5)
    blocks = oracle.q4k_quantize((rng.standard_normal((8192, 3072)) * 0.02).astype(np.float32))
    assert blocks.size == 14155776
    x = rng.standard_normal((1, M, 3072)).astype(np.float16)
    got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (8192, 3072)), Tensor.from_data(x), None,
                     False, True, True)
    want = oracle.matmul_ref(blocks, oracle.Q4_K, (8192, 3072), x, oracle.F16, x.shape, None, False, True, True)
    assert got.shape == (1, M, 8192) and oracle.max_rel_err(got, want) <= 2e-2


# ---------------------------------------------------------------------------
# Maximum sizes: element offsets beyond 2^31 (64-bit addressing in every kernel the shapes reach)
# ---------------------------------------------------------------------------
def _q8_rows_dequant(oracle, buf, N, K, rows):
    """f32 values of chosen rows of a Q8_0H [N, K] segment buffer, through the oracle's dequantizer row by row."""
    soff = oracle.q8_0_scale_offset(N * K)
    out = np.empty((len(rows), K), dtype=np.float32)
    for i, r in enumerate(rows):
        one = np.zeros(oracle.q8_0_nbytes(K, True), dtype=np.uint8)
        one[:K] = buf[r * K:(r + 1) * K]
        so = oracle.q8_0_scale_offset(K)
        one[so:so + K // 16] = buf[soff + r * (K // 16): soff + (r + 1) * (K // 16)]
        out[i] = oracle.q8_0_dequantize(one, K, True)
    return out


@pytest.mark.parametrize("M", [1, 192], ids=["streaming", "tiled"])
def test_q8_weight_beyond_2_31_elements(device, oracle, M):
    """W [135168 x 16384] Q8_0H = 2.21e9 codes (2.3 GB): the last rows lie beyond byte offset 2^31.  With one-hot
    activations every output is one dequantized weight, so rows from the start, the middle and the end are
    compared bit for bit with the oracle's dequantizer; a wrong 32-bit offset would select another weight."""
    N, K = 135168, 16384
    assert N * K > 2**31
    rng = np.random.default_rng(77)
    nbytes = oracle.q8_0_nbytes(N * K, True)
    buf = np.empty(nbytes, dtype=np.uint8)
    soff = oracle.q8_0_scale_offset(N * K)
    buf[:soff] = rng.integers(0, 256, size=soff, dtype=np.uint8)
    # f16 scales 2^-8 .. 2^-5, exact: exponent bits 7..10, no mantissa
    buf[soff:] = 0
    sc = (rng.integers(7, 11, size=N * K // 32, dtype=np.uint16) << 10).astype(np.uint16)
    buf[soff:soff + sc.size * 2] = sc.view(np.uint8)
    cols = rng.integers(0, K, size=M)
    x = np.zeros((1, M, K), dtype=np.float16)
    x[0, np.arange(M), cols] = 1
    w = Tensor.from_quantized(buf, DType.Q8_0H, (N, K)).to(device)
    got = w.gemm(Tensor.from_data(x).to(device), None, False, True, True).resolve().to(Device.CPU).storage  # [1, M, N]
    rows = np.concatenate([np.arange(0, 48), np.arange(N // 2 - 8, N // 2 + 8), np.arange(N - 200, N)])
    dq = _q8_rows_dequant(oracle, buf, N, K, rows)                     # [rows, K]
    want = dq[:, cols].T.astype(np.float16)                            # [M, rows]
    assert np.array_equal(got[0][:, rows], want)
    # and no output anywhere is out of the weights' range (a stray read would very likely show here)
    assert np.isfinite(got).all() and np.abs(got.astype(np.float32)).max() <= 128 * 2.0**-5


def test_f16_weight_beyond_2_31_elements(device, oracle):
    """The same for the f16 large-tile kernel: W [135168 x 16384] f16 (4.4 GB), 192 one-hot activation rows; every
    output is one weight, bit for bit.  The weight repeats a random block of 2039 rows: 2039 does not divide the
    65536 rows that 2^31 bytes span, so an offset that wrapped would pick a row with other values."""
    N, K, M, period = 135168, 16384, 192, 2039
    rng = np.random.default_rng(78)
    block = rng.standard_normal((period, K)).astype(np.float16)
    w = np.empty((N, K), dtype=np.float16)
    for r0 in range(0, N, period):
        n = min(period, N - r0)
        w[r0:r0 + n] = block[:n]
    cols = rng.integers(0, K, size=M)
    x = np.zeros((1, M, K), dtype=np.float16)
    x[0, np.arange(M), cols] = 1
    got = Tensor.from_data(w).to(device).gemm(Tensor.from_data(x).to(device), None, False, True, True).resolve()
    got = got.to(Device.CPU).storage                                    # [1, M, N]
    assert np.array_equal(got[0], w[:, cols].T)


def test_plan_enqueue_equals_plain_enqueue_on_the_five_configs(device, oracle):
    """rt_matmul_plan_create + rt_matmul_plan_enqueue against rt_matmul_enqueue_ws on the BASELINE shapes (C1, C2 at
    1 / 4 / 8 vectors, both C3 products, C4 up and down with a workspace, C5 at 1 / 16 / 256 rows): the same kernels
    run, so the outputs agree bit for bit, on the first enqueue of a plan (which asks every kernel family in turn)
    and on the second (which goes straight to the one that took it)."""
    import ctypes

    import torch

    from ratchet_amd import _ffi
    L = _ffi.lib()
    rng = np.random.default_rng(50)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()).cuda()
    f16 = lambda *s: rng.standard_normal(s).astype(np.float16)
    q8 = lambda n, k: oracle.make_q8_0h((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    q4 = lambda n, k: oracle.q4k_quantize((rng.standard_normal(n * k) * 0.02).astype(np.float32))
    F32, F16, Q8, Q4 = _ffi.RT_F32, _ffi.RT_F16, _ffi.RT_Q8_0H, _ffi.RT_Q4_K
    cases = [  # (lhs, dtype, shape, rhs, dtype, shape, bias, trans flags, output bytes)
        ((rng.standard_normal((1500, 384)) * 0.05).astype(np.float32), F32, (1500, 384),
         (rng.standard_normal((384, 1536)) * 0.05).astype(np.float32), F32, (384, 1536),
         (rng.standard_normal(1536) * 0.05).astype(np.float32), (False, False, False), 1500 * 1536 * 4)]
    w_up = q8(10240, 2560)
    for m in (1, 4, 8, 512):
        cases.append((w_up, Q8, (10240, 2560), f16(1, m, 2560), F16, (1, m, 2560), f16(10240), (False, True, True), m * 10240 * 2))
    cases.append((q8(2560, 10240), Q8, (2560, 10240), f16(1, 512, 10240), F16, (1, 512, 10240), f16(2560), (False, True, True), 512 * 2560 * 2))
    cases.append((f16(1, 32, 512, 80), F16, (1, 32, 512, 80), f16(1, 32, 512, 80), F16, (1, 32, 512, 80), None, (False, True, False), 32 * 512 * 512 * 2))
    cases.append(((rng.random((1, 32, 512, 512)) / 512).astype(np.float16), F16, (1, 32, 512, 512), f16(1, 32, 512, 80), F16,
                  (1, 32, 512, 80), None, (False, False, False), 32 * 512 * 80 * 2))
    w_q4 = q4(8192, 3072)
    for m in (1, 16, 256):
        cases.append((w_q4, Q4, (8192, 3072), f16(1, m, 3072), F16, (1, m, 3072), None, (False, True, True), m * 8192 * 2))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for i, (lhs, ldt, lshape, rhs, rdt, rshape, bias, flags, out_bytes) in enumerate(cases):
        desc = (_ffi.make_desc(ldt, lshape, rdt, rshape, *flags) if bias is None else
                _ffi.make_desc(ldt, lshape, rdt, rshape, *flags, F16 if bias.dtype == np.float16 else F32, bias.shape))
        dl, dr, db = dev(lhs), dev(rhs), None if bias is None else dev(bias)
        bp = None if db is None else ctypes.c_void_p(db.data_ptr())
        need = ctypes.c_uint64()
        assert L.rt_matmul_workspace_bytes(device.ctx, ctypes.byref(desc), ctypes.byref(need)) == _ffi.RT_OK
        ws = torch.empty(need.value, dtype=torch.uint8, device="cuda") if need.value else None
        wp = None if ws is None else ctypes.c_void_p(ws.data_ptr())
        outs = [torch.full((out_bytes,), 0xEE, dtype=torch.uint8, device="cuda") for _ in range(3)]
        st = L.rt_matmul_enqueue_ws(device.ctx, ctypes.byref(desc), dl.data_ptr(), dr.data_ptr(), bp,
                                    ctypes.c_void_p(outs[0].data_ptr()), 0, wp, need.value, stream)
        assert st == _ffi.RT_OK, (i, L.rt_last_error(device.ctx))
        plan = ctypes.c_void_p()
        assert L.rt_matmul_plan_create(device.ctx, ctypes.byref(desc), 0, ctypes.byref(plan)) == _ffi.RT_OK, i
        try:
            for o in outs[1:]:
                st = L.rt_matmul_plan_enqueue(plan, dl.data_ptr(), dr.data_ptr(), bp, ctypes.c_void_p(o.data_ptr()), wp, need.value, stream)
                assert st == _ffi.RT_OK, (i, L.rt_last_error(device.ctx))
            torch.cuda.synchronize()
        finally:
            L.rt_matmul_plan_destroy(plan)
        a = outs[0].cpu().numpy()
        assert not np.all(a == 0xEE)
        assert np.array_equal(a, outs[1].cpu().numpy()) and np.array_equal(a, outs[2].cpu().numpy()), i
    # descriptor errors surface when the plan is created; a null plan is a status
    bad = _ffi.make_desc(F16, (64, 32), F16, (1, 8, 40), False, True, True)
    plan = ctypes.c_void_p()
    assert L.rt_matmul_plan_create(device.ctx, ctypes.byref(bad), 0, ctypes.byref(plan)) == _ffi.RT_ERR_INVALID_SHAPE and not plan.value
    assert L.rt_matmul_plan_create(device.ctx, ctypes.byref(bad), 99, ctypes.byref(plan)) == _ffi.RT_ERR_INVALID_ARG
    assert L.rt_matmul_plan_enqueue(None, None, None, None, None, None, 0, None) == _ffi.RT_ERR_INVALID_ARG
