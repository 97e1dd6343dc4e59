"""The operators around a Linear in the reference's models: Gelu / Silu (crates/ratchet-core/src/ops/unary.rs),
Cast (ops/cast.rs), and the same activations fused into the product's epilogue.

The oracle is pinned against library routines it does not share code with (torch's
gelu(approximate="tanh") and silu in float64, numpy's and torch's f32 -> f16 conversion) and
against closed forms; the device kernels are compared with the oracle, and with torch at the
reference's own tolerances (ops/unary.rs:397-400: Gelu all_close(5e-2, 5e-2), Silu 1e-4;
ops/cast.rs:255-257: 1e-4)."""
import ctypes

import numpy as np
import pytest
import torch

import ratchet_amd.tensor as rt_tensor
from ratchet_amd import DType, Device, InvariantError, Tensor, _ffi


def torch_act64(x, act):
    t = torch.from_numpy(np.asarray(x, dtype=np.float64))
    r = torch.nn.functional.gelu(t, approximate="tanh") if act == 1 else torch.nn.functional.silu(t)
    return r.numpy()


# ---------------------------------------------------------------------------
# CPU: the oracle
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("act", [1, 2], ids=["gelu", "silu"])
def test_oracle_activation_against_torch(oracle, act):
    rng = np.random.default_rng(10 + act)
    x = np.concatenate([(rng.standard_normal(20000) * 3).astype(np.float32),
                        np.linspace(-30, 30, 4001, dtype=np.float32),
                        np.array([0.0, -0.0, 1e-20, -1e-20, 9.999, 10.0, 10.001, -9.999, -10.0, 80.0, -80.0, 88.0, -88.0,
                                  -104.0, 1e4, -1e4], np.float32)])
    got = oracle.unary(x, act)
    assert got.dtype == np.float32 and got.shape == x.shape
    # f32 evaluation of a formula with cancellation near the negative tail: a few 1e-7 absolute
    np.testing.assert_allclose(got, torch_act64(x, act), rtol=3e-6, atol=6e-7)
    # f16 storage: widened, computed in f32, rounded once
    xh = x[np.abs(x) < 6e4].astype(np.float16)
    np.testing.assert_array_equal(oracle.unary(xh, act), oracle.unary(xh.astype(np.float32), act).astype(np.float16))


def test_oracle_activation_closed_forms(oracle):
    G, S = oracle.ACT_GELU, oracle.ACT_SILU
    z = np.array([0.0], np.float32)
    assert oracle.unary(z, G)[0] == 0 and oracle.unary(z, S)[0] == 0
    # silu(x) - silu(-x) = x (sigmoid(x) + sigmoid(-x) = 1); gelu(x) - gelu(-x) = x for the tanh form (odd tanh)
    x = np.linspace(0.01, 20, 997, dtype=np.float32)
    for act in (G, S):
        d = oracle.unary(x, act).astype(np.float64) - oracle.unary(-x, act).astype(np.float64)
        np.testing.assert_allclose(d, x, rtol=3e-7, atol=1e-7)
    # saturation: safe_tanh is exactly +-1 once |x| >= 10 (unary.rs:112-118), so gelu(x) = x, gelu(-x) = -0
    big = np.array([10.0, 12.5, 1e3, 3e38], np.float32)
    assert np.array_equal(oracle.unary(big, G), big)
    assert np.all(oracle.unary(-big, G) == 0)
    # sigmoid's two branches (unary.rs:121-130) never overflow: silu(-1e4) = -0, silu(1e4) = 1e4, no NaN
    assert np.array_equal(oracle.unary(np.array([1e4, 3e38], np.float32), S), np.array([1e4, 3e38], np.float32))
    assert np.all(oracle.unary(np.array([-1e4, -3e38], np.float32), S) == 0)
    # silu(1) = 1 / (1 + e^-1); the minimum of silu sits at x = -1.2784645 with value -0.27846454
    assert abs(float(oracle.unary(np.array([1.0], np.float32), S)[0]) - 1 / (1 + np.exp(-1.0))) < 1e-7
    assert abs(float(oracle.unary(np.array([-1.2784645], np.float32), S)[0]) + 0.27846454) < 1e-7
    # NaN passes through
    assert np.isnan(oracle.unary(np.array([np.nan], np.float32), G)[0])
    assert np.isnan(oracle.unary(np.array([np.nan], np.float32), S)[0])


def test_oracle_cast_against_numpy_and_torch(oracle):
    rng = np.random.default_rng(12)
    x = np.concatenate([(rng.standard_normal(50000) * 10).astype(np.float32),
                        (rng.standard_normal(5000) * 1e-6).astype(np.float32),      # f16 subnormals and underflow
                        np.array([65504.0, 65519.99, 65520.0, 1e9, -1e9, np.inf, -np.inf, 0.0, -0.0,
                                  2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -24, 2049.0, 2051.0], np.float32)])
    got = oracle.cast(x, np.float16)
    assert got.dtype == np.float16
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(got.view(np.uint16), x.astype(np.float16).view(np.uint16))
    np.testing.assert_array_equal(got.view(np.uint16), torch.from_numpy(x).half().numpy().view(np.uint16))
    assert np.isnan(oracle.cast(np.array([np.nan], np.float32), np.float16)[0])
    # widening is exact for every one of the 65536 encodings (NaNs compared as NaNs)
    allh = np.arange(65536, dtype=np.uint16).view(np.float16)
    wide = oracle.cast(allh, np.float32)
    ref = allh.astype(np.float32)
    assert np.array_equal(wide[~np.isnan(ref)], ref[~np.isnan(ref)]) and np.isnan(wide[np.isnan(ref)]).all()
    # narrowing what was widened gives the value back
    fin = allh[np.isfinite(allh)]
    np.testing.assert_array_equal(oracle.cast(oracle.cast(fin, np.float32), np.float16).view(np.uint16), fin.view(np.uint16))


def test_oracle_fused_is_activation_of_the_f32_product(oracle):
    rng = np.random.default_rng(13)
    a = rng.standard_normal((2, 9, 40)).astype(np.float32)
    b = rng.standard_normal((2, 40, 7)).astype(np.float32)
    bias = rng.standard_normal(7).astype(np.float32)
    plain = oracle.matmul_ref(a, 0, a.shape, b, 0, b.shape, bias)
    for act in (1, 2):
        fused = oracle.matmul_ref(a, 0, a.shape, b, 0, b.shape, bias, act=act)
        np.testing.assert_array_equal(fused, oracle.unary(plain, act))            # f32 output: no rounding between
        np.testing.assert_allclose(fused, torch_act64(plain, act), rtol=3e-6, atol=6e-7)
    # f16 output: one rounding of act(f32 sum), not act(rounded sum)
    ah, bh = a.astype(np.float16), b.astype(np.float16)
    f32sum = oracle.matmul_ref(ah.astype(np.float32), 0, a.shape, bh.astype(np.float32), 0, b.shape)
    fused = oracle.matmul_ref(ah, 1, a.shape, bh, 1, b.shape, act=1)
    np.testing.assert_array_equal(fused, oracle.unary(f32sum, 1).astype(np.float16))


def test_guards_without_a_device():
    t = Tensor.from_data(np.zeros((2, 3), np.float32))
    with pytest.raises(InvariantError):
        t.cast(DType.Q8_0H)
    assert t.cast(DType.F32) is t                       # same dtype: no node
    assert t.half().dt == DType.F16 and t.half().shape == (2, 3)
    assert t.half().full().dt == DType.F32
    assert t.gelu().shape == (2, 3) and t.silu().dt == DType.F32
    L = _ffi.lib()
    # argument checks come before any device work; a null context is refused
    assert L.rt_unary_enqueue(None, 1, 0, None, None, 0, None) == _ffi.RT_ERR_INVALID_ARG
    assert L.rt_cast_enqueue(None, 0, 1, None, None, 0, None) == _ffi.RT_ERR_INVALID_ARG


# ---------------------------------------------------------------------------
# GPU
# ---------------------------------------------------------------------------
gpu = pytest.mark.gpu
SIZES = [1, 3, 7, 8, 9, 255, 256, 257, 4099, 65536 + 5, 1 << 20, (1 << 22) + 3]


def assert_act_close(got, want, dt, what=""):
    if dt == DType.F32:   # the device's tanhf / expf differ from libm's in the last places
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6, err_msg=str(what))
    else:                 # one f16 rounding on each side of f32 values that may differ in the last place
        np.testing.assert_allclose(got.astype(np.float32), want.astype(np.float32), rtol=1e-3, atol=1e-6, err_msg=str(what))


@gpu
@pytest.mark.parametrize("dt", [DType.F32, DType.F16], ids=["f32", "f16"])
@pytest.mark.parametrize("name,act", [("gelu", 1), ("silu", 2)])
def test_unary_against_oracle_and_torch(device, oracle, dt, name, act):
    rng = np.random.default_rng(20 + act)
    for n in SIZES:
        x = (rng.standard_normal(n) * 4).astype(dt.numpy())
        k = min(7, n)
        x[:k] = [-12.0, 11.0, 0.0, -0.0, 30.0, -30.0, 9.99][:k]
        t = Tensor.from_data(x).to(device)
        got = getattr(t, name)().resolve().to(Device.CPU).storage
        assert got.shape == x.shape and got.dtype == x.dtype
        assert_act_close(got, oracle.unary(x, act), dt, (name, n))
        # the reference's own check against torch (ops/unary.rs:397-403)
        atol, rtol = (5e-2, 5e-2) if act == 1 else (1e-4, 1e-4)
        if dt == DType.F32:
            ground = Tensor.from_data(torch_act64(x, act).astype(np.float32))
            ground.all_close(Tensor.from_data(got), atol, rtol)
        assert np.array_equal(t.to(Device.CPU).storage, x)     # the source keeps its values
    # a tensor of rank 4, as the models hold them
    x = rng.standard_normal((2, 3, 17, 33)).astype(dt.numpy())
    got = getattr(Tensor.from_data(x).to(device), name)().resolve().to(Device.CPU).storage
    assert_act_close(got, oracle.unary(x, act), dt, "rank 4")


@gpu
def test_unary_in_place_and_extremes(device, oracle):
    L = _ffi.lib()
    x = np.array([np.nan, np.inf, -np.inf, 1e4, -1e4, 10.0, -10.0, 88.0, -88.0, -104.0, 0.0, -0.0, 3e38, -3e38, 1.0, -1.0,
                  0.5], np.float32)
    for act in (1, 2):
        d = torch.from_numpy(x).to(f"cuda:{device.ordinal}")
        st = L.rt_unary_enqueue(device.ctx, act, _ffi.RT_F32, ctypes.c_void_p(d.data_ptr()), ctypes.c_void_p(d.data_ptr()),
                                x.size, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert st == _ffi.RT_OK
        got = d.cpu().numpy()
        want = oracle.unary(x, act)
        assert np.array_equal(np.isnan(got), np.isnan(want)), act
        m = ~np.isnan(want)
        np.testing.assert_allclose(got[m], want[m], rtol=1e-5, atol=1e-6)
    # errors: unknown activation, quantized dtype, misaligned buffer
    d = torch.zeros(64, device=f"cuda:{device.ordinal}")
    p, s = ctypes.c_void_p(d.data_ptr()), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert L.rt_unary_enqueue(device.ctx, 0, _ffi.RT_F32, p, p, 64, s) == _ffi.RT_ERR_INVALID_ARG
    assert L.rt_unary_enqueue(device.ctx, 7, _ffi.RT_F32, p, p, 64, s) == _ffi.RT_ERR_INVALID_ARG
    assert L.rt_unary_enqueue(device.ctx, 1, _ffi.RT_Q8_0H, p, p, 64, s) == _ffi.RT_ERR_DTYPE_MISMATCH
    assert L.rt_unary_enqueue(device.ctx, 1, _ffi.RT_F32, ctypes.c_void_p(d.data_ptr() + 4), p, 8, s) == _ffi.RT_ERR_INVALID_ARG
    assert L.rt_unary_enqueue(device.ctx, 1, _ffi.RT_F32, None, None, 0, s) == _ffi.RT_OK
    assert L.rt_cast_enqueue(device.ctx, _ffi.RT_F32, _ffi.RT_F32, p, p, 8, s) == _ffi.RT_ERR_DTYPE_MISMATCH
    assert L.rt_cast_enqueue(device.ctx, _ffi.RT_F32, _ffi.RT_F16, p, p, 8, s) == _ffi.RT_ERR_INVALID_ARG   # in place


@gpu
def test_cast_is_bit_exact(device, oracle):
    rng = np.random.default_rng(30)
    for n in SIZES:
        x = (rng.standard_normal(n) * 100).astype(np.float32)
        x[::5] *= 1e-7                                  # the f16 subnormal range and below
        x[::11] *= 1e4                                  # beyond the f16 range: infinities
        h = Tensor.from_data(x).to(device).half().resolve().to(Device.CPU).storage
        assert h.dtype == np.float16
        np.testing.assert_array_equal(h.view(np.uint16), oracle.cast(x, np.float16).view(np.uint16), err_msg=str(n))
    # every f16 encoding widens exactly, and narrows back to itself
    allh = np.arange(65536, dtype=np.uint16).view(np.float16)
    w = Tensor.from_data(allh).to(device).full().resolve()
    wide = w.to(Device.CPU).storage
    want = oracle.cast(allh, np.float32)
    nan = np.isnan(want)
    assert np.array_equal(wide[~nan].view(np.uint32), want[~nan].view(np.uint32)) and np.isnan(wide[nan]).all()
    back = w.half().resolve().to(Device.CPU).storage
    assert np.array_equal(back[~nan].view(np.uint16), allh[~nan].view(np.uint16)) and np.isnan(back[nan]).all()
    # the reference's test (ops/cast.rs:231-262) on a rank-3 tensor
    a = rng.standard_normal((3, 77, 129)).astype(np.float32)
    ground = Tensor.from_data(torch.from_numpy(a).half().numpy())
    ground.all_close(Tensor.from_data(a).to(device).cast(DType.F16).resolve().to(Device.CPU), 1e-4, 1e-4)


def fused_case(device, oracle, lhs_t, lhs_raw, lhs_dt, lhs_shape, x, bias, tl, tr, to, act, what):
    """Every kernel family's epilogue: fused on the device against the oracle's fused statement."""
    adt = DType.F32 if x.dtype == np.float32 else DType.F16
    name = "gelu" if act == 1 else "silu"
    node = lhs_t.to(device).gemm(Tensor.from_data(x).to(device), None if bias is None else Tensor.from_data(bias).to(device),
                                 tl, tr, to)
    got = getattr(node, name)().resolve().to(Device.CPU).storage
    want = oracle.matmul_ref(lhs_raw, int(lhs_dt), lhs_shape, x, int(adt), x.shape, bias, tl, tr, to, act=act)
    assert got.shape == want.shape, what
    err = oracle.max_rel_err(got, want)
    assert err <= (1e-3 if adt == DType.F32 else 2e-2), (what, err)
    assert node.storage is None          # the product itself was never written: it ran fused
    return got


@gpu
@pytest.mark.parametrize("act", [1, 2], ids=["gelu", "silu"])
def test_fused_activation_every_kernel_family(device, oracle, act):
    rng = np.random.default_rng(40 + act)
    # Q8_0 Linear: streaming kernel widths 1..8, the VALU kernel's shapes, the tiled kernels
    for dt in (DType.Q8_0H, DType.Q8_0F):
        adt = dt.activation_dt().numpy()
        for (M, N, K) in [(1, 256, 512), (4, 130, 96), (8, 512, 4096), (3, 33, 2560), (64, 256, 256), (200, 320, 512),
                          (129, 257, 64)]:
            w = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
            buf = oracle.make_q8_0h(w) if dt == DType.Q8_0H else oracle.q8_0_quantize_f32(w)
            x = rng.standard_normal((1, M, K)).astype(adt)
            bias = rng.standard_normal(N).astype(adt)
            fused_case(device, oracle, Tensor.from_quantized(buf, dt, (N, K)), buf, dt, (N, K), x, bias, False, True, True,
                       act, (dt.name, M, N, K))
    # Q4_K Linear: streaming (M <= 16) and through the tiled kernel
    for (M, N, K) in [(1, 64, 512), (16, 128, 1024), (40, 96, 256)]:
        w = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
        buf = oracle.q4k_quantize(w)
        x = rng.standard_normal((1, M, K)).astype(np.float16)
        bias = rng.standard_normal(N).astype(np.float16)
        fused_case(device, oracle, Tensor.from_quantized(buf, DType.Q4_K, (N, K)), buf, DType.Q4_K, (N, K), x, bias,
                   False, True, True, act, ("q4k", M, N, K))
    # float products: large-tile NT kernels (plain, short K), narrow untransposed rhs, the generic kernel, GEMV
    for dt in (DType.F16, DType.F32):
        npdt = dt.numpy()
        for (B, M, K, N, tl, tr, to, has_bias) in [(1, 300, 512, 260, False, True, False, True),
                                                   (2, 256, 80, 256, False, True, False, False),
                                                   (2, 192, 256, 80, False, False, False, True),
                                                   (1, 100, 70, 50, True, False, False, True),
                                                   (1, 130, 64, 90, False, False, True, False),
                                                   (1, 1, 512, 384, False, False, False, True),
                                                   (3, 17, 33, 1, False, False, False, False)]:
            a = (rng.standard_normal((B, K, M) if tl else (B, M, K)) * 0.3).astype(npdt)
            b = (rng.standard_normal((B, N, K) if tr else (B, K, N)) * 0.3).astype(npdt)
            bias = None if (not has_bias or to) else rng.standard_normal(N).astype(npdt)
            fused_case(device, oracle, Tensor.from_data(a), a, dt, a.shape, b, bias, tl, tr, to, act,
                       (dt.name, B, M, K, N, tl, tr, to))


@gpu
def test_fused_equals_two_operators_for_f32(device, oracle):
    """With f32 outputs nothing is rounded between the product and the activation, so the fused
    kernel and the two-operator sequence agree bit for bit; the mirror's switch selects which runs."""
    rng = np.random.default_rng(50)
    a = rng.standard_normal((2, 65, 96)).astype(np.float32)
    b = rng.standard_normal((2, 96, 70)).astype(np.float32)
    bias = rng.standard_normal(70).astype(np.float32)
    A, B_, Bi = (Tensor.from_data(v).to(device) for v in (a, b, bias))
    for name in ("gelu", "silu"):
        fused = getattr(A.gemm(B_, Bi, False, False, False), name)().resolve().to(Device.CPU).storage
        rt_tensor.FUSE_ACTIVATIONS = False
        try:
            node = A.gemm(B_, Bi, False, False, False)
            two = getattr(node, name)().resolve().to(Device.CPU).storage
            assert node.storage is not None          # the product was written, then the operator ran on it
        finally:
            rt_tensor.FUSE_ACTIVATIONS = True
        assert np.array_equal(fused, two), name
    # a product with a second consumer is computed once and the activation reads it: both consumers see the same values
    a16, b16 = a.astype(np.float16), b.astype(np.float16)
    A16, B16 = Tensor.from_data(a16).to(device), Tensor.from_data(b16).to(device)
    node = A16.matmul(B16, False, False)
    act, again = node.gelu(), node.silu()
    got = act.resolve().to(Device.CPU).storage
    assert node.resolved()                            # not fused: the rounded product exists
    prod16 = node.to(Device.CPU).storage
    assert np.array_equal(got, oracle.unary(prod16, oracle.ACT_GELU).astype(np.float16)) or np.allclose(
        got.astype(np.float32), oracle.unary(prod16, oracle.ACT_GELU).astype(np.float32), rtol=2e-3, atol=1e-6)
    assert np.allclose(again.resolve().to(Device.CPU).storage.astype(np.float32),
                       oracle.unary(prod16, oracle.ACT_SILU).astype(np.float32), rtol=2e-3, atol=1e-6)
    # an activation on a resolved product runs as its own operator
    prod = A.gemm(B_, Bi, False, False, False).resolve()
    np.testing.assert_array_equal(prod.gelu().resolve().to(Device.CPU).storage,
                                  A.gemm(B_, Bi, False, False, False).gelu().resolve().to(Device.CPU).storage)


@gpu
def test_phi2_mlp_block(device, oracle):
    """phi2/mlp.rs:13-15: fc2(gelu(fc1(x))) with Q8_0H weights, at a reduced width, for a decode
    step (one token) and a prefill (48 tokens)."""
    rng = np.random.default_rng(60)
    D, H = 320, 1280
    w1 = (rng.standard_normal((H, D)) * 0.05).astype(np.float32)
    w2 = (rng.standard_normal((D, H)) * 0.05).astype(np.float32)
    q1, q2 = oracle.make_q8_0h(w1), oracle.make_q8_0h(w2)
    b1, b2 = (rng.standard_normal(H) * 0.1).astype(np.float16), (rng.standard_normal(D) * 0.1).astype(np.float16)
    W1, W2 = Tensor.from_quantized(q1, DType.Q8_0H, (H, D)).to(device), Tensor.from_quantized(q2, DType.Q8_0H, (D, H)).to(device)
    B1, B2 = Tensor.from_data(b1).to(device), Tensor.from_data(b2).to(device)
    for T in (1, 48):
        x = rng.standard_normal((1, T, D)).astype(np.float16)
        h = W1.gemm(Tensor.from_data(x).to(device), B1, False, True, True).gelu()
        y = W2.gemm(h, B2, False, True, True).resolve().to(Device.CPU).storage
        h_ref = oracle.matmul_ref(q1, int(DType.Q8_0H), (H, D), x, 1, x.shape, b1, False, True, True, act=1)
        y_ref = oracle.matmul_ref(q2, int(DType.Q8_0H), (D, H), h_ref, 1, h_ref.shape, b2, False, True, True)
        assert y.shape == (1, T, D)
        assert oracle.max_rel_err(y, y_ref) <= 2e-2, T
