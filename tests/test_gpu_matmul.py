"""Parity of the HIP Matmul path with the CPU oracle, through the C ABI.

Mirrors the reference's own matmul tests (crates/ratchet-core/src/ops/matmul.rs:649-927)
with the same shapes and tolerances, then the BASELINE configs at full size.
Tolerances: the reference's all_close(atol, rtol) where it states one; against
the oracle max-rel-err <= 1e-3 for f32 and <= 2e-2 for f16 I/O with f32
accumulation (max_i |y_i - r_i| / max(|r_i|, 1e-3 * max_j |r_j|)).
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from ratchet_amd import DType, Device, InvariantError, OperationError, Quantization, Quantizer, Tensor, _ffi

pytestmark = pytest.mark.gpu
G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = {DType.F32: 1e-3, DType.F16: 2e-2}

TRANS_KINDS = {  # ops/matmul.rs:720-741
    "None": (False, False, False), "LHS": (True, False, False), "LHSAndOut": (True, False, True),
    "RHS": (False, True, False), "RHSAndOut": (False, True, True), "Out": (False, False, True),
}


def ground_truth(a, b, bias, tl, tr, to):
    """The reference's torch ground truth (ops/matmul.rs:663-718), f32 on the CPU."""
    ta, tb = torch.from_numpy(a.astype(np.float32)), torch.from_numpy(b.astype(np.float32))
    ta = ta.transpose(-1, -2) if tl else ta
    tb = tb.transpose(-1, -2) if tr else tb
    r = torch.matmul(ta, tb)
    if bias is not None:
        r = r + torch.from_numpy(bias.astype(np.float32))
    r = r.transpose(-1, -2) if to else r
    return np.ascontiguousarray(r.numpy())


def gpu_matmul(device, lhs: Tensor, rhs: Tensor, bias, tl, tr, to) -> np.ndarray:
    c = lhs.to(device).gemm(rhs.to(device), None if bias is None else bias.to(device), tl, tr, to).resolve()
    return c.to(Device.CPU).storage


def check(oracle, got, want, dt, what=""):
    assert got.shape == want.shape, (what, got.shape, want.shape)
    err = oracle.max_rel_err(got, want)
    assert err <= TOL[dt], (what, err)


# ---------------------------------------------------------------------------
# test_sgemm (ops/matmul.rs:757-829): 64 cases of the proptest space
# ---------------------------------------------------------------------------
def sgemm_cases(n, seed):
    rng = np.random.default_rng(seed)
    kinds = list(TRANS_KINDS)
    out = []
    for i in range(n):
        B, M, K, N = int(rng.integers(1, 4)), *(int(v) for v in rng.integers(1, 257, 3))
        out.append((B, M, K, N, bool(rng.integers(0, 2)), kinds[i % len(kinds)]))
    # extremes of the space
    out += [(1, 1, 1, 1, True, "None"), (3, 256, 256, 256, True, "None"), (2, 1, 256, 1, False, "RHS"),
            (1, 256, 1, 256, False, "LHSAndOut"), (2, 255, 33, 129, True, "LHS")]
    return out


@pytest.mark.parametrize("dt", [DType.F32, DType.F16], ids=["f32", "f16"])
def test_sgemm(device, oracle, dt):
    npdt = dt.numpy()
    for case in sgemm_cases(64, seed=100):
        B, M, K, N, has_bias, kind = case
        tl, tr, to = TRANS_KINDS[kind]
        if to:
            has_bias = False  # ops/matmul.rs:786-789
        rng = np.random.default_rng(abs(hash(case)) % 2**32)
        a = rng.standard_normal((B, K, M) if tl else (B, M, K)).astype(npdt)
        b = rng.standard_normal((B, N, K) if tr else (B, K, N)).astype(npdt)
        bias = rng.standard_normal(N).astype(npdt) if has_bias else None
        got = gpu_matmul(device, Tensor.from_data(a), Tensor.from_data(b),
                         None if bias is None else Tensor.from_data(bias), tl, tr, to)
        want = oracle.matmul_ref(a, int(dt), a.shape, b, int(dt), b.shape, bias, tl, tr, to)
        check(oracle, got, want, dt, case)
        if dt == DType.F32:  # the reference's own bar against torch
            ok, mae = oracle.all_close(ground_truth(a, b, bias, tl, tr, to), got, 1e-4, 1e-4)
            assert ok, (case, mae)


def test_sgemm_golden(device, oracle):
    f = np.load(os.path.join(G, "sgemm.npz"))
    for name, (tl, tr, to) in TRANS_KINDS.items():
        a, b = f[f"{name}_a"], f[f"{name}_b"]
        bias = f[f"{name}_bias"] if f"{name}_bias" in f.files else None
        got = gpu_matmul(device, Tensor.from_data(a), Tensor.from_data(b),
                         None if bias is None else Tensor.from_data(bias), tl, tr, to)
        ok, mae = oracle.all_close(f[f"{name}_out"], got, 1e-4, 1e-4)
        assert ok, (name, mae)


def test_many_tiles_all_layouts(device, oracle):
    """Problems large enough for the 128 x 128 tiling (hundreds of workgroups), every
    transposition kind, extents off the tile and vector sizes."""
    for dt in (DType.F32, DType.F16):
        npdt = dt.numpy()
        for ci, (B, M, K, N) in enumerate([(6, 1200, 40, 1300), (5, 1301, 24, 1203)]):
            for kind, (tl, tr, to) in TRANS_KINDS.items():
                rng = np.random.default_rng(900 + ci)
                a = rng.standard_normal((B, K, M) if tl else (B, M, K)).astype(npdt)
                b = rng.standard_normal((B, N, K) if tr else (B, K, N)).astype(npdt)
                bias = None if to else rng.standard_normal(N).astype(npdt)
                got = gpu_matmul(device, Tensor.from_data(a), Tensor.from_data(b),
                                 None if bias is None else Tensor.from_data(bias), tl, tr, to)
                want = oracle.matmul_ref(a, int(dt), a.shape, b, int(dt), b.shape, bias, tl, tr, to)
                check(oracle, got, want, dt, (dt, B, M, K, N, kind))


def test_qgemm(device, oracle):
    """ops/matmul.rs:831-852, full size, through Quantizer::sint8_quantize on the device."""
    rng = np.random.default_rng(101)
    a = rng.standard_normal((6, 1500, 64)).astype(np.float32)
    b = rng.standard_normal((6, 64, 1500)).astype(np.float32)
    aq = Quantizer(Quantization.SInt8, device).sint8_quantize(Tensor.from_data(a))
    assert np.array_equal(aq.storage, oracle.q8_0_quantize_f32(a))
    got = gpu_matmul(device, aq, Tensor.from_data(b), None, False, False, False)
    ok, mae = oracle.all_close(ground_truth(a, b, None, False, False, False), got, 1e1, 1e-1)
    assert ok, mae
    want = oracle.matmul_ref(aq.storage, oracle.Q8_0F, a.shape, b, oracle.F32, b.shape)
    check(oracle, got, want, DType.F32, "qgemm")


def test_debug_gemm(device, oracle):
    """ops/matmul.rs:854-890."""
    rng = np.random.default_rng(102)
    a = rng.standard_normal((2, 222, 252)).astype(np.float32)
    b = rng.standard_normal((1, 222, 238)).astype(np.float32)
    bias = rng.standard_normal(238).astype(np.float32)
    got = gpu_matmul(device, Tensor.from_data(a), Tensor.from_data(b), Tensor.from_data(bias), True, False, False)
    ok, mae = oracle.all_close(ground_truth(a, b, bias, True, False, False), got, 1e-3, 1e-3)
    assert ok and got.shape == (2, 252, 238), mae


def test_debug_gemv(device, oracle):
    """ops/matmul.rs:892-926."""
    rng = np.random.default_rng(103)
    a = rng.standard_normal((1, 51865, 384)).astype(np.float32)
    b = rng.standard_normal((1, 1, 384)).astype(np.float32)
    got = gpu_matmul(device, Tensor.from_data(a), Tensor.from_data(b), None, False, True, True)
    ok, mae = oracle.all_close(ground_truth(a, b, None, False, True, True), got, 1e-3, 1e-3)
    assert ok and got.shape == (1, 1, 51865), mae


# ---------------------------------------------------------------------------
# Quantized Linear: W.gemm(x, bias, false, true, true)  (nn::Linear, linear.rs:17-24)
# ---------------------------------------------------------------------------
def q8_weight(oracle, rng, N, K, dt):
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    buf = oracle.make_q8_0h(w) if dt == DType.Q8_0H else oracle.q8_0_quantize_f32(w)
    return buf


@pytest.mark.parametrize("dt", [DType.Q8_0H, DType.Q8_0F], ids=["q8_0h", "q8_0f"])
def test_q8_linear_shapes(device, oracle, dt):
    adt = dt.activation_dt()
    shapes = [(1, 64, 32), (1, 10, 96), (2, 257, 64), (3, 33, 2560), (4, 128, 160), (5, 1000, 352), (7, 77, 1024),
              (8, 512, 4096), (9, 64, 64), (16, 130, 96), (100, 200, 320), (129, 257, 64), (512, 384, 256)]
    for i, (M, N, K) in enumerate(shapes):
        rng = np.random.default_rng(200 + i)
        buf = q8_weight(oracle, rng, N, K, dt)
        x = rng.standard_normal((1, M, K)).astype(adt.numpy())
        bias = rng.standard_normal(N).astype(adt.numpy()) if i % 2 == 0 else None
        got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (N, K)), Tensor.from_data(x),
                         None if bias is None else Tensor.from_data(bias), False, True, True)
        want = oracle.matmul_ref(buf, int(dt), (N, K), x, int(adt), x.shape, bias, False, True, True)
        check(oracle, got, want, adt, (M, N, K))


def test_q8_streaming_regular_and_ragged_variants(device, oracle):
    """The streaming Q8_0H kernel has a variant for the regular case (whole 16-row groups, exactly
    1, 2, 4, 8 or 16 vectors, every wavefront's units present) next to the general one: both, for
    every vector-count ceiling and for one, two and four 256-wide units of K per wavefront."""
    dt, adt = DType.Q8_0H, np.float16
    cases = [(M, 64, K) for M in (1, 2, 4, 8, 16) for K in (2560, 5120, 12288)]          # regular
    cases += [(3, 64, 2560), (5, 48, 5120), (16, 40, 12288), (1, 17, 1024), (12, 64, 768), (1, 64, 256)]  # general
    for i, (M, N, K) in enumerate(cases):
        rng = np.random.default_rng(250 + i)
        buf = q8_weight(oracle, rng, N, K, dt)
        x = rng.standard_normal((1, M, K)).astype(adt)
        bias = rng.standard_normal(N).astype(adt) if i % 3 else None
        got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (N, K)), Tensor.from_data(x),
                         None if bias is None else Tensor.from_data(bias), False, True, True)
        want = oracle.matmul_ref(buf, int(dt), (N, K), x, int(DType.F16), x.shape, bias, False, True, True)
        check(oracle, got, want, DType.F16, (M, N, K))
    # one-hot activations through the regular variant: the dequantized weight, bit for bit
    N, K = 32, 5120
    rng = np.random.default_rng(299)
    buf = q8_weight(oracle, rng, N, K, dt)
    dq = oracle.q8_0_dequantize(buf, N * K, True).reshape(N, K)
    cols = rng.integers(0, K, size=4)
    x = np.zeros((4, K), dtype=adt)
    x[np.arange(4), cols] = 1
    got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (N, K)), Tensor.from_data(x), None, False, True, True)
    assert np.array_equal(got, dq[:, cols].T.astype(adt))


def test_q8_streaming_regular_variant_below_its_vector_ceiling(device, oracle):
    """5, 6, 7 (ceiling 8) and 3 (ceiling 4, K too long for the 4x4x4 kernel) vectors against whole 16-row groups run
    the regular variant, which loads the weights in address order and turns them to operand order through LDS: the
    bias along the rows and along the vectors (read at indices below the vector count only), GELU fused, and
    one-hot activations bit for bit with -128 planted."""
    dt = DType.Q8_0H
    for i, (M, N, K) in enumerate([(5, 10240, 2560), (6, 4096, 2560), (7, 640, 5120), (3, 2048, 8192), (8, 10240, 2560)]):
        rng = np.random.default_rng(2700 + i)
        buf = q8_weight(oracle, rng, N, K, dt)
        x = rng.standard_normal((1, M, K)).astype(np.float16)
        for to in (True, False):
            bias = rng.standard_normal(N if to else M).astype(np.float16)
            got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (N, K)), Tensor.from_data(x), Tensor.from_data(bias),
                             False, True, to)
            want = oracle.matmul_ref(buf, oracle.Q8_0H, (N, K), x, oracle.F16, x.shape, bias, False, True, to)
            check(oracle, got, want, DType.F16, (M, N, K, to))
    N, K = 4096, 2560
    rng = np.random.default_rng(2750)
    buf = q8_weight(oracle, rng, N, K, dt)
    x = rng.standard_normal((1, 6, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    y = Tensor.from_quantized(buf, dt, (N, K)).to(device).gemm(Tensor.from_data(x).to(device), Tensor.from_data(bias).to(device),
                                                                False, True, True).gelu().resolve()
    want = oracle.matmul_ref(buf, oracle.Q8_0H, (N, K), x, oracle.F16, x.shape, bias, False, True, True, act=oracle.ACT_GELU)
    assert np.all(np.abs(y.to(Device.CPU).storage.astype(np.float64) - want) <= 2e-3 + 2e-2 * np.abs(want))
    buf[: N * K][5::97] = 0x80
    dq = oracle.q8_0_dequantize(buf, N * K, True).reshape(N, K)
    for M in (5, 7, 8):
        cols = np.concatenate([[5 + 97 * 3], rng.integers(0, K, size=M)])[:M]
        x = np.zeros((M, K), dtype=np.float16)
        x[np.arange(M), cols] = 1
        got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (N, K)), Tensor.from_data(x), None, False, True, True)
        assert np.array_equal(got, dq[:, cols].T.astype(np.float16)), M


def test_q8_streaming_rows_dealt_one_workgroup_per_compute_unit(device, oracle):
    """With 9..16 vectors the activations' LDS lets one or two workgroups of the Q8_0H streaming kernel live on a
    compute unit; when the 16-row workgroups would then run in rounds, every compute unit gets one workgroup with
    its share of the rows instead (24, 40 or 48 of them: row groups whose last one is half empty or ragged)."""
    dt = DType.Q8_0H
    for i, (M, N, K) in enumerate([(16, 4104, 2560), (9, 10240, 2560), (13, 10248, 2560)]):
        rng = np.random.default_rng(290 + i)
        buf = q8_weight(oracle, rng, N, K, dt)
        x = rng.standard_normal((1, M, K)).astype(np.float16)
        for to in (True, False):
            bias = rng.standard_normal(N if to else M).astype(np.float16)
            got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (N, K)), Tensor.from_data(x), Tensor.from_data(bias),
                             False, True, to)
            want = oracle.matmul_ref(buf, oracle.Q8_0H, (N, K), x, oracle.F16, x.shape, bias, False, True, to)
            check(oracle, got, want, DType.F16, (M, N, K, to))
    # one-hot activations: every row of the weight, bit for bit, through the half-empty row group
    N, K = 4104, 2560
    buf = q8_weight(oracle, np.random.default_rng(295), N, K, dt)
    dq = oracle.q8_0_dequantize(buf, N * K, True).reshape(N, K)
    cols = np.arange(16) * 157 + 3
    x = np.zeros((16, K), dtype=np.float16)
    x[np.arange(16), cols] = 1
    got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (N, K)), Tensor.from_data(x), None, False, True, True)
    assert np.array_equal(got, dq[:, cols].T.astype(np.float16))


def test_q8_row_streaming_one_and_two_vectors(device, oracle):
    """Q8_0H weights against one or two vectors with K a multiple of 512 up to 10240 take the row-streaming
    kernel: every step count of the half-wave-per-row layout (K = 512 .. 3584), of the wavefront-per-row layout
    (K = 4096 .. 10240 in steps of 1024) and of its form with a short last step (K = 4608 .. 9728), row counts off
    the rows of a workgroup, stacks of weights and of activations with broadcast either way, the bias along the
    rows (trans_out) and along the vectors, and a fused activation; then one-hot activations, bit for bit, with
    -128 planted."""
    dt = DType.Q8_0H
    cases = [(1, 1, 64, 512 * k) for k in range(1, 21)] + [(1, 2, 21, 512 * k) for k in (7, 8, 9, 16, 19)]
    cases += [(1, 2, 61, 2560), (1, 2, 3, 1024), (1, 1, 1, 512), (1, 2, 27, 8192), (1, 1, 10240, 2560), (1, 2, 13, 10240),
              (3, 1, 19, 1536), (2, 2, 9, 7168)]
    for i, (S, M, N, K) in enumerate(cases):
        rng = np.random.default_rng(260 + i)
        for ws, xs_ in ((S, S), (1, S), (S, 1)) if S > 1 else ((1, 1),):
            w = (rng.standard_normal((ws, N, K)) * 0.05).astype(np.float32)
            buf = oracle.make_q8_0h(w)
            x = rng.standard_normal((xs_, M, K)).astype(np.float16)
            for to in (True, False):
                bias = rng.standard_normal(N if to else M).astype(np.float16) if (i + to) % 3 else None
                got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (ws, N, K)), Tensor.from_data(x),
                                 None if bias is None else Tensor.from_data(bias), False, True, to)
                want = oracle.matmul_ref(buf, oracle.Q8_0H, (ws, N, K), x, oracle.F16, x.shape, bias, False, True, to)
                check(oracle, got, want, DType.F16, (S, ws, xs_, M, N, K, to))
    # GELU / SiLU behind the Linear, fused
    rng = np.random.default_rng(280)
    N, K = 100, 3072
    buf = oracle.make_q8_0h((rng.standard_normal((N, K)) * 0.05).astype(np.float32))
    x = rng.standard_normal((1, 2, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    for name, act in (("gelu", oracle.ACT_GELU), ("silu", oracle.ACT_SILU)):
        y = getattr(Tensor.from_quantized(buf, dt, (N, K)).to(device).gemm(
            Tensor.from_data(x).to(device), Tensor.from_data(bias).to(device), False, True, True), name)().resolve()
        want = oracle.matmul_ref(buf, oracle.Q8_0H, (N, K), x, oracle.F16, x.shape, bias, False, True, True, act=act)
        assert np.all(np.abs(y.to(Device.CPU).storage.astype(np.float64) - want) <= 2e-3 + 2e-2 * np.abs(want))
    # one-hot: the dequantized weight, bit for bit, in both forms
    for N, K in ((37, 2560), (21, 10240), (9, 4608)):
        buf = q8_weight(oracle, rng, N, K, dt)
        buf[: N * K][5::97] = 0x80
        dq = oracle.q8_0_dequantize(buf, N * K, True).reshape(N, K)
        for M in (1, 2):
            cols = np.concatenate([[5 + 97 * 3], rng.integers(0, K, size=M)])[:M]
            x = np.zeros((M, K), dtype=np.float16)
            x[np.arange(M), cols] = 1
            got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (N, K)), Tensor.from_data(x), None, False, True, True)
            assert np.array_equal(got, dq[:, cols].T.astype(np.float16)), (N, K, M)


def test_q8_row_streaming_three_and_four_vectors(device, oracle):
    """Q8_0H weights against three or four vectors, K a multiple of 256 up to 4096 and at least 16 rows per compute
    unit take the row-streaming kernel on the 4x4x4 matrix instruction: every step count (K = 256 .. 4096), row
    counts off the 16 rows of a workgroup and off the four of a wavefront, stacks of weights and of activations with
    broadcast either way, the bias along the rows (trans_out) and along the vectors, a fused activation; then
    one-hot activations, bit for bit, with -128 planted."""
    dt = DType.Q8_0H
    cases = [(1, 3 + (k & 1), 4096 + 3 * k, 256 * k) for k in range(1, 17)]
    cases += [(1, 4, 10240, 2560), (1, 3, 4097, 2560), (2, 4, 2069, 768), (3, 3, 1400, 1280)]
    for i, (S, M, N, K) in enumerate(cases):
        rng = np.random.default_rng(2600 + i)
        for ws, xs_ in ((S, S), (1, S), (S, 1)) if S > 1 else ((1, 1),):
            w = (rng.standard_normal((ws, N, K)) * 0.05).astype(np.float32)
            buf = oracle.make_q8_0h(w)
            x = rng.standard_normal((xs_, M, K)).astype(np.float16)
            for to in (True, False):
                bias = rng.standard_normal(N if to else M).astype(np.float16) if (i + to) % 3 else None
                got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (ws, N, K)), Tensor.from_data(x),
                                 None if bias is None else Tensor.from_data(bias), False, True, to)
                want = oracle.matmul_ref(buf, oracle.Q8_0H, (ws, N, K), x, oracle.F16, x.shape, bias, False, True, to)
                check(oracle, got, want, DType.F16, (S, ws, xs_, M, N, K, to))
    # GELU / SiLU behind the Linear, fused
    rng = np.random.default_rng(2680)
    N, K = 4200, 1024
    buf = oracle.make_q8_0h((rng.standard_normal((N, K)) * 0.05).astype(np.float32))
    x = rng.standard_normal((1, 4, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    for name, act in (("gelu", oracle.ACT_GELU), ("silu", oracle.ACT_SILU)):
        y = getattr(Tensor.from_quantized(buf, dt, (N, K)).to(device).gemm(
            Tensor.from_data(x).to(device), Tensor.from_data(bias).to(device), False, True, True), name)().resolve()
        want = oracle.matmul_ref(buf, oracle.Q8_0H, (N, K), x, oracle.F16, x.shape, bias, False, True, True, act=act)
        assert np.all(np.abs(y.to(Device.CPU).storage.astype(np.float64) - want) <= 2e-3 + 2e-2 * np.abs(want))
    # one-hot: the dequantized weight, bit for bit
    for N, K in ((4099, 2560), (4200, 256), (4096, 4096)):
        buf = q8_weight(oracle, rng, N, K, dt)
        buf[: N * K][5::97] = 0x80
        dq = oracle.q8_0_dequantize(buf, N * K, True).reshape(N, K)
        for M in (3, 4):
            cols = np.concatenate([[5 + 97 * 2], rng.integers(0, K, size=M)])[:M]
            x = np.zeros((M, K), dtype=np.float16)
            x[np.arange(M), cols] = 1
            got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (N, K)), Tensor.from_data(x), None, False, True, True)
            assert np.array_equal(got, dq[:, cols].T.astype(np.float16)), (N, K, M)


@pytest.mark.parametrize("dt", [DType.Q8_0H, DType.Q8_0F], ids=["q8_0h", "q8_0f"])
def test_q8_one_hot_is_bit_exact_dequant(device, oracle, dt):
    """A one-hot activation selects one dequantized weight per row: the GEMV / GEMM
    result must equal the oracle's dequantized value rounded to the activation dtype,
    bit for bit, for every column index and for -128."""
    adt = dt.activation_dt()
    f16 = dt == DType.Q8_0H
    rng = np.random.default_rng(300)
    N, K = 96, 128
    buf = q8_weight(oracle, rng, N, K, dt)
    buf[: N * K][5::97] = 0x80  # plant int8 -128 values
    dq = oracle.q8_0_dequantize(buf, N * K, f16).reshape(N, K)
    for M in (1, 4, 8, 32):      # GEMV widths and the tiled GEMM
        cols = rng.integers(0, K, size=M)
        x = np.zeros((M, K), dtype=adt.numpy())
        x[np.arange(M), cols] = 1
        got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (N, K)), Tensor.from_data(x), None, False, True, True)
        want = dq[:, cols].T.astype(adt.numpy())
        if M <= 8 or not f16:
            assert np.array_equal(got, want), M
        else:
            # the f16 tile path rounds the dequantized weight to f16 once: same value
            assert np.array_equal(got, want), M


def test_q8_mirrored_spelling(device, oracle):
    """x.matmul(W, false, true) == W.gemm(x, None, false, true, true)."""
    rng = np.random.default_rng(301)
    N, K = 320, 256
    buf = q8_weight(oracle, rng, N, K, DType.Q8_0H)
    W = Tensor.from_quantized(buf, DType.Q8_0H, (N, K))
    for M in (1, 6, 40):
        x = rng.standard_normal((M, K)).astype(np.float16)
        a = gpu_matmul(device, W, Tensor.from_data(x), None, False, True, True)
        b = gpu_matmul(device, Tensor.from_data(x), W, None, False, True, False)
        assert a.shape == b.shape == (M, N) and np.array_equal(a, b)
        bias = rng.standard_normal(N).astype(np.float16)
        a = gpu_matmul(device, W, Tensor.from_data(x), Tensor.from_data(bias), False, True, True)
        b = gpu_matmul(device, Tensor.from_data(x), W, Tensor.from_data(bias), False, True, False)
        assert np.array_equal(a, b)


def test_q8_stacked_and_untransposed_rhs(device, oracle):
    rng = np.random.default_rng(302)
    # quantized lhs stack broadcast against per-stack activations, rhs read untransposed (test_qgemm's form)
    a = rng.standard_normal((3, 70, 64)).astype(np.float32)
    b = rng.standard_normal((3, 64, 5)).astype(np.float32)
    aq = oracle.q8_0_quantize_f32(a)
    got = gpu_matmul(device, Tensor.from_quantized(aq, DType.Q8_0F, a.shape), Tensor.from_data(b), None, False, False, False)
    check(oracle, got, oracle.matmul_ref(aq, oracle.Q8_0F, a.shape, b, oracle.F32, b.shape), DType.F32)
    a1 = a[:1]
    aq1 = oracle.q8_0_quantize_f32(a1)
    x = rng.standard_normal((3, 4, 64)).astype(np.float32)
    got = gpu_matmul(device, Tensor.from_quantized(aq1, DType.Q8_0F, a1.shape), Tensor.from_data(x), None, False, True, True)
    check(oracle, got, oracle.matmul_ref(aq1, oracle.Q8_0F, a1.shape, x, oracle.F32, x.shape, None, False, True, True),
          DType.F32)


def test_q4k_linear(device, oracle):
    f = np.load(os.path.join(G, "q4_k.npz"))
    shape = tuple(int(v) for v in f["shape"])
    got = gpu_matmul(device, Tensor.from_quantized(f["blocks"], DType.Q4_K, shape), Tensor.from_data(f["x"]), None,
                     False, True, True)
    assert oracle.max_rel_err(got, f["linear_out_f64"]) <= 2e-2
    for i, (M, N, K) in enumerate([(1, 64, 256), (2, 100, 512), (8, 257, 768), (16, 96, 1024), (33, 130, 256),
                                   (256, 128, 512)]):
        rng = np.random.default_rng(400 + i)
        blocks = oracle.q4k_quantize((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
        x = rng.standard_normal((1, M, K)).astype(np.float16)
        got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (N, K)), Tensor.from_data(x), None,
                         False, True, True)
        want = oracle.matmul_ref(blocks, oracle.Q4_K, (N, K), x, oracle.F16, x.shape, None, False, True, True)
        check(oracle, got, want, DType.F16, (M, N, K))


def test_q4k_streaming_shapes(device, oracle):
    """Q4_K weights with 1..16 activation vectors (the streaming kernels), with and without
    bias, row counts off the 16-row grouping, K up to and past the 4096 one wavefront column
    per super-block covers, a lone vector given as rank 2, and both bias orientations."""
    shapes = [(1, 16, 3072), (1, 50, 4096), (3, 33, 1280), (5, 257, 256), (8, 130, 3072), (9, 64, 768),
              (12, 100, 2048), (16, 513, 3072), (16, 48, 4096), (2, 40, 4352), (11, 24, 8192)]
    # the kernel's regular-case variant: whole 16-row groups, 1 / 2 / 4 / 8 / 16 vectors, K >= 1024
    shapes += [(M, 64, K) for M in (1, 2, 4, 8, 16) for K in (1024, 3072)]
    for i, (M, N, K) in enumerate(shapes):
        rng = np.random.default_rng(420 + i)
        blocks = oracle.q4k_quantize((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
        x = rng.standard_normal((1, M, K)).astype(np.float16)
        bias = rng.standard_normal(N).astype(np.float16) if i % 2 == 0 else None
        got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (N, K)), Tensor.from_data(x),
                         None if bias is None else Tensor.from_data(bias), False, True, True)
        want = oracle.matmul_ref(blocks, oracle.Q4_K, (N, K), x, oracle.F16, x.shape, bias, False, True, True)
        check(oracle, got, want, DType.F16, (M, N, K))
    # W @ x^T without transposing the output: (N, K) x (K, M) -> (N, M); bias then runs along M
    rng = np.random.default_rng(440)
    N, K, M = 70, 1024, 6
    blocks = oracle.q4k_quantize((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
    x = rng.standard_normal((M, K)).astype(np.float16)
    bias = rng.standard_normal(M).astype(np.float16)
    got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (N, K)), Tensor.from_data(x),
                     Tensor.from_data(bias), False, True, False)
    want = oracle.matmul_ref(blocks, oracle.Q4_K, (N, K), x, oracle.F16, x.shape, bias, False, True, False)
    check(oracle, got, want, DType.F16, "no trans_out")


def test_q4k_streaming_rows_dealt_one_workgroup_per_compute_unit(device, oracle):
    """With 9..16 vectors and K from 2560 one workgroup of the Q4_K streaming kernel fits a compute unit; more than
    256 of the 16-row workgroups would run in rounds, so every compute unit gets one workgroup of up to 32 rows:
    whole double groups (8192 rows), a half-empty second group (4104 rows: 24 per workgroup), and a row count
    whose share is above 32 (back to 16-row workgroups); then one-hot activations, bit for bit."""
    for i, (M, N, K) in enumerate([(16, 8192, 3072), (13, 4104, 2560), (16, 8200, 2560)]):
        rng = np.random.default_rng(490 + i)
        blocks = oracle.q4k_quantize((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
        x = rng.standard_normal((1, M, K)).astype(np.float16)
        for to in (True, False):
            bias = rng.standard_normal(N if to else M).astype(np.float16)
            got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (N, K)), Tensor.from_data(x),
                             Tensor.from_data(bias), False, True, to)
            want = oracle.matmul_ref(blocks, oracle.Q4_K, (N, K), x, oracle.F16, x.shape, bias, False, True, to)
            check(oracle, got, want, DType.F16, (M, N, K, to))
    N, K = 4104, 2560
    blocks = oracle.q4k_quantize((np.random.default_rng(495).standard_normal((N, K)) * 0.02).astype(np.float32))
    dq = oracle.q4k_dequantize(blocks).reshape(N, K)
    cols = np.arange(16) * 157 + 3
    x = np.zeros((16, K), dtype=np.float16)
    x[np.arange(16), cols] = 1
    got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (N, K)), Tensor.from_data(x), None, False, True, True)
    assert np.array_equal(got, dq[:, cols].T.astype(np.float16))


def test_q4k_row_streaming_long_rows(device, oracle):
    """Q4_K weights with K above 4096 against one vector take the row-streaming kernel (a wavefront per row, the
    row read as a run of 16-byte vectors, block headers handed to the lanes of their blocks through LDS): K from
    4352 to 10752 (three to six steps of 64 vectors, the last one short or whole), row counts off the 16 / 8 / 4
    rows of a workgroup, both bias orientations and none, stacks of weights and of activations with broadcast
    either way, a fused activation; then one-hot activations, which must return the dequantized column bit for bit."""
    cases = [(1, 50, 4352), (1, 9, 5120), (1, 1, 6144), (1, 37, 8192), (1, 130, 10752), (1, 3072, 8192), (3, 7, 4608),
             (2, 21, 7168)]
    for i, (S, N, K) in enumerate(cases):
        rng = np.random.default_rng(470 + i)
        for ws, xs_ in ((S, S), (1, S), (S, 1)) if S > 1 else ((1, 1),):
            blocks = oracle.q4k_quantize((rng.standard_normal((ws, N, K)) * 0.02).astype(np.float32))
            x = rng.standard_normal((xs_, 1, K)).astype(np.float16)
            for to in (True, False):
                bias = rng.standard_normal(N if to else 1).astype(np.float16) if (i + to) % 3 else None
                got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (ws, N, K)), Tensor.from_data(x),
                                 None if bias is None else Tensor.from_data(bias), False, True, to)
                want = oracle.matmul_ref(blocks, oracle.Q4_K, (ws, N, K), x, oracle.F16, x.shape, bias, False, True, to)
                check(oracle, got, want, DType.F16, (S, ws, xs_, N, K, to))
    rng = np.random.default_rng(480)
    N, K = 100, 4864
    blocks = oracle.q4k_quantize((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
    x = rng.standard_normal((1, 1, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    for name, act in (("gelu", oracle.ACT_GELU), ("silu", oracle.ACT_SILU)):
        y = getattr(Tensor.from_quantized(blocks, DType.Q4_K, (N, K)).to(device).gemm(
            Tensor.from_data(x).to(device), Tensor.from_data(bias).to(device), False, True, True), name)().resolve()
        want = oracle.matmul_ref(blocks, oracle.Q4_K, (N, K), x, oracle.F16, x.shape, bias, False, True, True, act=act)
        assert np.all(np.abs(y.to(Device.CPU).storage.astype(np.float64) - want) <= 2e-3 + 2e-2 * np.abs(want))
    for N, K in ((23, 8192), (5, 4352)):
        blocks = oracle.q4k_quantize((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
        dq = oracle.q4k_dequantize(blocks).reshape(N, K)
        for col in (0, K - 1, 255, 256, 4096 + 31, int(rng.integers(0, K)), int(rng.integers(0, K))):
            x = np.zeros((1, K), dtype=np.float16)
            x[0, col] = 1
            got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (N, K)), Tensor.from_data(x), None,
                             False, True, True)
            assert np.array_equal(got.reshape(-1), dq[:, col].astype(np.float16)), (N, K, col)


def test_q4k_streaming_long_rows_few_vectors(device, oracle):
    """Q4_K weights with K above 4096 (up to 8192) against 2..8 vectors: the matrix-core streaming kernel with two
    super-blocks per wavefront (an odd number of super-blocks leaves the last wavefront's second one empty); row counts
    off the 16 rows of a workgroup, stacks, both bias orientations; one-hot activations return the dequantized
    columns bit for bit."""
    cases = [(1, 50, 4352, 2), (1, 9, 5120, 3), (1, 16, 6144, 8), (1, 37, 8192, 5), (1, 3072, 8192, 2), (2, 21, 7168, 4),
             (1, 130, 7936, 7)]
    for i, (S, N, K, M) in enumerate(cases):
        rng = np.random.default_rng(490 + i)
        for ws, xs_ in ((S, S), (1, S), (S, 1)) if S > 1 else ((1, 1),):
            blocks = oracle.q4k_quantize((rng.standard_normal((ws, N, K)) * 0.02).astype(np.float32))
            x = rng.standard_normal((xs_, M, K)).astype(np.float16)
            for to in (True, False):
                bias = rng.standard_normal(N if to else M).astype(np.float16) if (i + to) % 3 else None
                got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (ws, N, K)), Tensor.from_data(x),
                                 None if bias is None else Tensor.from_data(bias), False, True, to)
                want = oracle.matmul_ref(blocks, oracle.Q4_K, (ws, N, K), x, oracle.F16, x.shape, bias, False, True, to)
                check(oracle, got, want, DType.F16, (S, ws, xs_, N, K, M, to))
    rng = np.random.default_rng(499)
    N, K, M = 23, 8192, 6
    blocks = oracle.q4k_quantize((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
    dq = oracle.q4k_dequantize(blocks).reshape(N, K)
    cols = np.array([0, K - 1, 4095, 4096, 255, int(rng.integers(0, K))])
    x = np.zeros((1, M, K), dtype=np.float16)
    x[0, np.arange(M), cols] = 1
    got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (N, K)), Tensor.from_data(x), None, False, True, True)
    assert np.array_equal(got[0], dq[:, cols].T.astype(np.float16))


def test_q4k_one_hot_is_bit_exact_dequant(device, oracle):
    rng = np.random.default_rng(401)
    N, K = 40, 512
    blocks = oracle.q4k_quantize((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
    dq = oracle.q4k_dequantize(blocks).reshape(N, K)
    for M in (1, 8, 13, 16, 32):
        cols = rng.integers(0, K, size=M)
        x = np.zeros((M, K), dtype=np.float16)
        x[np.arange(M), cols] = 1
        got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (N, K)), Tensor.from_data(x), None,
                         False, True, True)
        assert np.array_equal(got, dq[:, cols].T.astype(np.float16)), M


# ---------------------------------------------------------------------------
# Stack broadcast, float GEMV, empty tensors, errors
# ---------------------------------------------------------------------------
def test_stack_broadcast(device, oracle):
    rng = np.random.default_rng(500)
    for a_shape, b_shape in [((3, 40, 24), (24, 17)), ((40, 24), (2, 3, 24, 17)), ((1, 1, 40, 24), (2, 5, 24, 17)),
                             ((2, 2, 9, 8), (2, 2, 8, 300)), ((6, 70, 33), (1, 33, 129))]:
        a = rng.standard_normal(a_shape).astype(np.float32)
        b = rng.standard_normal(b_shape).astype(np.float32)
        got = gpu_matmul(device, Tensor.from_data(a), Tensor.from_data(b), None, False, False, False)
        want = np.matmul(a.astype(np.float64), b.astype(np.float64))
        check(oracle, got, want, DType.F32, (a_shape, b_shape))
        check(oracle, got, oracle.matmul_ref(a, oracle.F32, a_shape, b, oracle.F32, b_shape), DType.F32)
    # stacks that are neither equal nor 1 on one side trip GEMMSpec::new's assert (ops/matmul.rs:90-94)
    a = Tensor.from_data(np.zeros((1, 5, 4, 8), np.float32)).to(device)
    b = Tensor.from_data(np.zeros((2, 5, 8, 3), np.float32)).to(device)
    with pytest.raises(InvariantError):
        a.matmul(b, False, False)


@pytest.mark.parametrize("dt", [DType.F32, DType.F16], ids=["f32", "f16"])
def test_float_gemv_paths(device, oracle, dt):
    rng = np.random.default_rng(501)
    npdt = dt.numpy()
    for N, K, M in [(1000, 384, 1), (333, 100, 3), (64, 7, 8), (129, 1, 2), (5000, 2048, 4)]:
        w = rng.standard_normal((N, K)).astype(npdt)
        x = rng.standard_normal((M, K)).astype(npdt)
        bias = rng.standard_normal(N).astype(npdt)
        got = gpu_matmul(device, Tensor.from_data(w), Tensor.from_data(x), Tensor.from_data(bias), False, True, True)
        want = oracle.matmul_ref(w, int(dt), w.shape, x, int(dt), x.shape, bias, False, True, True)
        check(oracle, got, want, dt, (N, K, M))
        # the same product spelled x . W^T (few lhs rows, many rhs columns)
        got2 = gpu_matmul(device, Tensor.from_data(x), Tensor.from_data(w), Tensor.from_data(bias), False, True, False)
        assert np.array_equal(got, got2)


@pytest.mark.parametrize("dt", [DType.F32, DType.F16], ids=["f32", "f16"])
def test_float_row_streaming_few_vectors(device, oracle, dt):
    """f16 / f32 weights against two activation vectors (rows of up to 10 KiB), and f16 against three or four
    (rows of up to 5 KiB), take the row-streaming kernel too: step counts, short last steps, stacks with
    broadcast, a bias along the weight rows or along the vectors, both output orientations, a fused activation.
    Other counts and longer rows fall to the one-load-at-a-time kernel and must agree as well."""
    npdt = dt.numpy()
    E = 16 // np.dtype(npdt).itemsize
    cases = [(1, 70, 64 * E * k, 2) for k in (1, 2, 5, 7, 10)] + [(1, 33, E, 2), (1, 1030, 65 * E, 2), (2, 19, 96 * E, 2),
             (1, 10240, 2560, 2), (1, 41, 64 * E * 3 + 3 * E, 3), (1, 77, 64 * E * 5, 4), (1, 10240, 2560, 4), (2, 9, 300 * E, 4),
             (1, 50, 64 * E * 6, 4), (1, 50, 64 * E * 2, 5), (1, 37, 641 * E, 2)]
    for i, (S, N, K, M) in enumerate(cases):
        rng = np.random.default_rng(560 + i)
        for ws, xs_ in ((S, S), (1, S), (S, 1)) if S > 1 else ((1, 1),):
            w = rng.standard_normal((ws, N, K)).astype(npdt)
            x = rng.standard_normal((xs_, M, K)).astype(npdt)
            for to in (True, False):
                bias = rng.standard_normal(N if to else M).astype(npdt) if (i + to) % 3 else None
                got = gpu_matmul(device, Tensor.from_data(w), Tensor.from_data(x),
                                 None if bias is None else Tensor.from_data(bias), False, True, to)
                want = oracle.matmul_ref(w, int(dt), w.shape, x, int(dt), x.shape, bias, False, True, to)
                check(oracle, got, want, dt, (S, ws, xs_, N, K, M, to))
    rng = np.random.default_rng(580)
    N, K, M = 100, 1536, 3
    w, x, bias = (rng.standard_normal(sh).astype(npdt) for sh in ((N, K), (1, M, K), (N,)))
    y = Tensor.from_data(w).to(device).gemm(Tensor.from_data(x).to(device), Tensor.from_data(bias).to(device), False, True, True).gelu().resolve()
    want = oracle.matmul_ref(w, int(dt), w.shape, x, int(dt), x.shape, bias, False, True, True, act=oracle.ACT_GELU)
    assert np.all(np.abs(y.to(Device.CPU).storage.astype(np.float64) - want) <= 2e-3 + 2e-2 * np.abs(want))
    # one-hot activations return weight columns bit for bit
    cols = rng.integers(0, K, size=M)
    x1 = np.zeros((1, M, K), dtype=npdt)
    x1[0, np.arange(M), cols] = 1
    got = gpu_matmul(device, Tensor.from_data(w), Tensor.from_data(x1), None, False, True, True)
    assert np.array_equal(got[0], w[:, cols].T)


@pytest.mark.parametrize("dt", [DType.F32, DType.F16], ids=["f32", "f16"])
def test_float_row_streaming_one_vector(device, oracle, dt):
    """f16 / f32 weights against one vector take the row-streaming kernels while a row is whole 16-byte vectors
    and at most 64 KiB: every step count (1..10 KiB of row), rows whose last step is short or a single
    vector, longer rows (the form that loops over 8 KiB passes), row counts off the 4 (2) rows of a workgroup, stacks of weights and of activations with
    broadcast either way, both bias orientations and none, a fused activation; then one-hot
    activations, which must return the weight column bit for bit."""
    npdt = dt.numpy()
    E = 16 // np.dtype(npdt).itemsize  # elements per 16-byte vector
    cases = [(1, 70, 64 * E * k) for k in range(1, 11)]                       # whole steps
    cases += [(1, 33, E), (1, 5, 63 * E), (1, 1030, 65 * E), (1, 41, 64 * E * 7 + 3 * E), (1, 1, 640 * E - E),
              (1, 10240, 2560), (3, 19, 96 * E), (2, 9, 300 * E)]
    # rows longer than 10 KiB (the looping form): one vector past it, an odd and an even number of 8 KiB passes, 64 KiB
    cases += [(1, 37, 641 * E), (1, 300, 1024 * E), (1, 6, 1537 * E), (1, 5, 4096 * E), (2, 7, 700 * E), (1, 2560, 10240)]
    for i, (S, N, K) in enumerate(cases):
        rng = np.random.default_rng(520 + i)
        for ws, xs_ in ((S, S), (1, S), (S, 1)) if S > 1 else ((1, 1),):
            w = rng.standard_normal((ws, N, K)).astype(npdt)
            x = rng.standard_normal((xs_, 1, K)).astype(npdt)
            for to in (True, False):
                bias = rng.standard_normal(N if to else 1).astype(npdt) if (i + to) % 3 else None
                got = gpu_matmul(device, Tensor.from_data(w), Tensor.from_data(x),
                                 None if bias is None else Tensor.from_data(bias), False, True, to)
                if dt == DType.F32 and K >= 8192:
                    # the oracle sums K products one after the other in f32: at this K its own rounding reaches the
                    # tolerance on outputs near zero, so the exact (f64) product is the reference here
                    want = np.einsum("snk,sk->sn", np.broadcast_to(w, (S, N, K)).astype(np.float64),
                                     np.broadcast_to(x[:, 0], (S, K)).astype(np.float64))
                    want = want + (0 if bias is None else bias.astype(np.float64))
                    want = want[:, None, :] if to else want[:, :, None]
                else:
                    want = oracle.matmul_ref(w, int(dt), w.shape, x, int(dt), x.shape, bias, False, True, to)
                check(oracle, got, want, dt, (S, ws, xs_, N, K, to))
    rng = np.random.default_rng(540)
    N, K = 100, 1536
    w, x, bias = (rng.standard_normal(sh).astype(npdt) for sh in ((N, K), (1, 1, K), (N,)))
    for name, act in (("gelu", oracle.ACT_GELU), ("silu", oracle.ACT_SILU)):
        y = getattr(Tensor.from_data(w).to(device).gemm(
            Tensor.from_data(x).to(device), Tensor.from_data(bias).to(device), False, True, True), name)().resolve()
        want = oracle.matmul_ref(w, int(dt), w.shape, x, int(dt), x.shape, bias, False, True, True, act=act)
        assert np.all(np.abs(y.to(Device.CPU).storage.astype(np.float64) - want) <= 2e-3 + 2e-2 * np.abs(want))
    for N, K in ((37, 2560), (6, 639 * E)):
        w = rng.standard_normal((N, K)).astype(npdt)
        for col in (0, K - 1, int(rng.integers(0, K))):
            x = np.zeros((1, K), dtype=npdt)
            x[0, col] = 1
            got = gpu_matmul(device, Tensor.from_data(w), Tensor.from_data(x), None, False, True, True)
            assert np.array_equal(got.reshape(-1), w[:, col]), (N, K, col)


def test_empty_and_k_zero(device):
    a = Tensor.from_data(np.zeros((0, 8), np.float32))
    b = Tensor.from_data(np.zeros((8, 3), np.float32))
    assert gpu_matmul(device, a, b, None, False, False, False).shape == (0, 3)
    a = Tensor.from_data(np.zeros((4, 0), np.float32))
    b = Tensor.from_data(np.zeros((0, 130), np.float32))
    bias = np.arange(130, dtype=np.float32)
    got = gpu_matmul(device, a, b, Tensor.from_data(bias), False, False, False)
    assert np.array_equal(got, np.tile(bias, (4, 1)))


def test_enqueue_errors(device):
    L = _ffi.lib()
    d = _ffi.make_desc(_ffi.RT_F32, (4, 8), _ffi.RT_F32, (8, 3))
    assert L.rt_matmul_enqueue(device.ctx, ctypes.byref(d), None, None, None, None, None) == _ffi.RT_ERR_INVALID_ARG
    assert b"null" in L.rt_last_error(device.ctx)
    d = _ffi.make_desc(_ffi.RT_F32, (4, 8), _ffi.RT_F32, (9, 3))
    assert L.rt_matmul_enqueue(device.ctx, ctypes.byref(d), None, None, None, None, None) == _ffi.RT_ERR_INVALID_SHAPE
    # more stacks than any kernel's grid takes: a limit of the library (UNSUPPORTED), not a runtime failure
    d = _ffi.make_desc(_ffi.RT_F32, (70000, 2, 3), _ffi.RT_F32, (70000, 3, 2))
    buf = torch.zeros(70000 * 6 * 4, dtype=torch.uint8, device="cuda")
    st = L.rt_matmul_enqueue(device.ctx, ctypes.byref(d), buf.data_ptr(), buf.data_ptr(), None, ctypes.c_void_p(buf.data_ptr()), None)
    assert st == _ffi.RT_ERR_UNSUPPORTED and L.rt_last_hip_error(device.ctx) == 0 or st == _ffi.RT_OK
    a = Tensor.from_data(np.zeros(8, np.float32)).to(device)
    b = Tensor.from_data(np.zeros((8, 3), np.float32)).to(device)
    with pytest.raises(OperationError):   # GEMMSpec::new: inputs must be at least 2D
        a.matmul(b, False, False).resolve()


def test_buffer_api_round_trip(device):
    L = _ffi.lib()
    src = np.arange(1000, dtype=np.float32)
    dst = np.zeros_like(src)
    p = ctypes.c_void_p()
    assert L.rt_buf_alloc(device.ctx, src.nbytes, ctypes.byref(p)) == _ffi.RT_OK
    assert L.rt_buf_upload(device.ctx, p, src.ctypes.data, src.nbytes, None) == _ffi.RT_OK
    assert L.rt_buf_download(device.ctx, dst.ctypes.data, p, src.nbytes, None) == _ffi.RT_OK
    assert L.rt_sync(device.ctx, None) == _ffi.RT_OK
    assert np.array_equal(src, dst)
    assert L.rt_buf_free(device.ctx, p) == _ffi.RT_OK


# ---------------------------------------------------------------------------
# Large-tile K-contiguous GEMM (f16 and Q8_0H): ragged edges, K tails, stacks,
# both output orientations and both bias axes
# ---------------------------------------------------------------------------
NT_SHAPES = [  # (stack, A rows, B rows, K)
    (1, 160, 64, 64), (1, 161, 65, 64), (1, 319, 127, 128), (1, 320, 128, 192), (1, 333, 200, 72),
    (1, 512, 512, 80), (3, 200, 96, 40), (2, 170, 70, 8), (1, 1000, 64, 256), (1, 160, 1000, 320),
]


@pytest.mark.parametrize("trans_out", [False, True], ids=["out", "out_t"])
def test_f16_nt_gemm_edges(device, oracle, trans_out):
    for i, (S, M, N, K) in enumerate(NT_SHAPES):
        rng = np.random.default_rng(600 + i)
        a = rng.standard_normal((S, M, K)).astype(np.float16)
        b = rng.standard_normal((S, N, K)).astype(np.float16)
        # bias runs along A's rows under trans_out, along B's rows otherwise
        bias = rng.standard_normal(M if trans_out else N).astype(np.float16) if i % 2 == 0 else None
        got = gpu_matmul(device, Tensor.from_data(a), Tensor.from_data(b),
                         None if bias is None else Tensor.from_data(bias), False, True, trans_out)
        want = oracle.matmul_ref(a, oracle.F16, a.shape, b, oracle.F16, b.shape, bias, False, True, trans_out)
        check(oracle, got, want, DType.F16, (S, M, N, K, trans_out))


def test_f16_weights_few_activation_rows(device, oracle):
    """5..64 activation rows against f16 weights of 160 rows or more: the tiled kernel's 64 x 64 tiles with a
    nine-stage ring (K of fewer tiles than stages included) and a partly empty column of activation rows
    (fewer than 5 rows, and 5..8 against weights of few rows, stay on the streaming or generic kernels; K up to
    256 on the short-K kernels)."""
    for i, (M, N, K) in enumerate([(512, 8, 320), (700, 9, 128), (1000, 33, 512), (161, 63, 64), (2560, 17, 2560),
                                   (4100, 64, 576), (650, 40, 1024), (10240, 64, 2560),
                                   # 5..8 vectors against a tall weight leave the streaming kernel for the same tiles
                                   (8200, 5, 320), (8192, 7, 576), (10240, 6, 2560)]):
        rng = np.random.default_rng(660 + i)
        w = (rng.standard_normal((M, K)) * 0.05).astype(np.float16)
        x = rng.standard_normal((1, N, K)).astype(np.float16)
        for to in (True, False):
            bias = rng.standard_normal(M if to else N).astype(np.float16) if (i + to) % 2 == 0 else None
            got = gpu_matmul(device, Tensor.from_data(w), Tensor.from_data(x),
                             None if bias is None else Tensor.from_data(bias), False, True, to)
            want = oracle.matmul_ref(w, oracle.F16, w.shape, x, oracle.F16, x.shape, bias, False, True, to)
            check(oracle, got, want, DType.F16, (M, N, K, to))


def test_weight_streaming_short_prompts(device, oracle):
    """f16 weights against 5..128 and Q8_0H weights against 17..48 activation rows, K a multiple of 256 and enough
    weight rows for three quarters of the compute units, take the weight-streaming GEMM: every tile count of
    activation rows (and counts off the 16 of a tile), one to three tiles of weight rows per workgroup, row counts
    off the 8 of a share (the scalar output path) and off the 16 of a tile, K from one step per wavefront (256) to
    more steps than the weight loader's register ring holds (and step counts off its four), the bias along the
    weight rows (trans_out) and along the activation rows, a fused activation; then Q8_0H one-hot activations, bit
    for bit, with -128 planted."""
    cases = [(10240, n, 2560) for n in (5, 16, 17, 31, 33, 48, 49, 64, 65, 80, 96, 97, 112, 113, 128, 129)]
    cases += [(6152, 24, 256), (6152, 40, 512), (2001, 9, 1280), (2008, 64, 768), (12288, 20, 4096), (4100, 7, 1024),
              (6152, 90, 1536), (8200, 70, 3328), (2008, 128, 256), (4096, 100, 768), (12288, 120, 1280), (2001, 77, 512),
              (2560, 33, 10240)]  # the last has too few rows for this kernel: the tiled one, same answer
    for i, (M, N, K) in enumerate(cases):
        rng = np.random.default_rng(3100 + i)
        w = (rng.standard_normal((M, K)) * 0.05).astype(np.float16)
        x = rng.standard_normal((1, N, K)).astype(np.float16)
        for to in (True, False):
            bias = rng.standard_normal(M if to else N).astype(np.float16) if (i + to) % 3 else None
            got = gpu_matmul(device, Tensor.from_data(w), Tensor.from_data(x),
                             None if bias is None else Tensor.from_data(bias), False, True, to)
            want = oracle.matmul_ref(w, oracle.F16, w.shape, x, oracle.F16, x.shape, bias, False, True, to)
            check(oracle, got, want, DType.F16, ("f16", M, N, K, to))
    dt = DType.Q8_0H
    for i, (M, N, K) in enumerate([(10240, 17, 2560), (10240, 32, 2560), (6152, 24, 256), (2001, 19, 1280),
                                   (12288, 20, 4096), (8200, 31, 512), (10240, 33, 2560), (10240, 48, 2560),
                                   (10240, 49, 2560), (6152, 40, 1536)]):
        rng = np.random.default_rng(3200 + i)
        buf = oracle.make_q8_0h((rng.standard_normal((M, K)) * 0.05).astype(np.float32))
        x = rng.standard_normal((1, N, K)).astype(np.float16)
        for to in (True, False):
            bias = rng.standard_normal(M if to else N).astype(np.float16) if (i + to) % 3 else None
            got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (M, K)), Tensor.from_data(x),
                             None if bias is None else Tensor.from_data(bias), False, True, to)
            want = oracle.matmul_ref(buf, oracle.Q8_0H, (M, K), x, oracle.F16, x.shape, bias, False, True, to)
            check(oracle, got, want, DType.F16, ("q8_0h", M, N, K, to))
    # GELU / SiLU behind the Linear, fused
    rng = np.random.default_rng(3280)
    M, K, N = 6152, 1024, 24
    w = (rng.standard_normal((M, K)) * 0.05).astype(np.float16)
    buf = oracle.make_q8_0h(w.astype(np.float32))
    x = rng.standard_normal((1, N, K)).astype(np.float16)
    bias = rng.standard_normal(M).astype(np.float16)
    for name, act in (("gelu", oracle.ACT_GELU), ("silu", oracle.ACT_SILU)):
        for wt, odt, src in ((Tensor.from_data(w), oracle.F16, w), (Tensor.from_quantized(buf, dt, (M, K)), oracle.Q8_0H, buf)):
            y = getattr(wt.to(device).gemm(Tensor.from_data(x).to(device), Tensor.from_data(bias).to(device),
                                           False, True, True), name)().resolve()
            want = oracle.matmul_ref(src, odt, (M, K), x, oracle.F16, x.shape, bias, False, True, True, act=act)
            assert np.all(np.abs(y.to(Device.CPU).storage.astype(np.float64) - want) <= 2e-3 + 2e-2 * np.abs(want)), (name, odt)
    # one-hot: the dequantized weight, bit for bit
    for M, K in ((10240, 2560), (6152, 256), (2001, 1280)):
        buf = q8_weight(oracle, rng, M, K, dt)
        buf[: M * K][5::97] = 0x80
        dq = oracle.q8_0_dequantize(buf, M * K, True).reshape(M, K)
        for N in (17, 32, 48):
            cols = np.concatenate([[5 + 97 * 2], rng.integers(0, K, size=N)])[:N]
            x = np.zeros((N, K), dtype=np.float16)
            x[np.arange(N), cols] = 1
            got = gpu_matmul(device, Tensor.from_quantized(buf, dt, (M, K)), Tensor.from_data(x), None, False, True, True)
            assert np.array_equal(got, dq[:, cols].T.astype(np.float16)), (M, K, N)


def test_f16_nt_gemm_stack_broadcast(device, oracle):
    rng = np.random.default_rng(650)
    a = rng.standard_normal((1, 200, 128)).astype(np.float16)      # one weight, four activation stacks
    b = rng.standard_normal((4, 70, 128)).astype(np.float16)
    got = gpu_matmul(device, Tensor.from_data(a), Tensor.from_data(b), None, False, True, True)
    want = oracle.matmul_ref(a, oracle.F16, a.shape, b, oracle.F16, b.shape, None, False, True, True)
    check(oracle, got, want, DType.F16, "stack broadcast")


def test_q8_nt_gemm_edges(device, oracle):
    for i, (S, M, N, K) in enumerate([(1, 160, 64, 64), (1, 161, 65, 96), (1, 333, 200, 160), (2, 170, 70, 32),
                                      (1, 1000, 129, 2560), (1, 2560, 77, 1024), (2, 200, 100, 256), (3, 161, 64, 512),
                                      # 17..64 activation rows against many weight rows: 64 x 64 tiles instead of streaming launches
                                      (1, 8300, 33, 512), (1, 8200, 24, 256), (1, 10240, 17, 2560)]):
        rng = np.random.default_rng(700 + i)
        w = (rng.standard_normal((S, M, K)) * 0.02).astype(np.float32)
        buf = oracle.make_q8_0h(w)
        x = rng.standard_normal((S, N, K)).astype(np.float16)
        bias = rng.standard_normal(M).astype(np.float16) if i % 2 == 0 else None
        got = gpu_matmul(device, Tensor.from_quantized(buf, DType.Q8_0H, (S, M, K)), Tensor.from_data(x),
                         None if bias is None else Tensor.from_data(bias), False, True, True)
        want = oracle.matmul_ref(buf, oracle.Q8_0H, (S, M, K), x, oracle.F16, x.shape, bias, False, True, True)
        check(oracle, got, want, DType.F16, (S, M, N, K))
        # untransposed output: [S, M, N]
        got = gpu_matmul(device, Tensor.from_quantized(buf, DType.Q8_0H, (S, M, K)), Tensor.from_data(x), None,
                         False, True, False)
        want = oracle.matmul_ref(buf, oracle.Q8_0H, (S, M, K), x, oracle.F16, x.shape, None, False, True, False)
        check(oracle, got, want, DType.F16, (S, M, N, K, "untransposed"))


def test_q8_tiled_one_hot_is_bit_exact_dequant(device, oracle):
    """The tiled Q8_0H kernels (K % 256 == 0 and not) with one-hot activations: each output is one
    dequantized weight, which must match the oracle's dequantizer bit for bit, -128 included."""
    rng = np.random.default_rng(720)
    for N, K, M in [(320, 256, 64), (200, 512, 100), (170, 96, 70), (2100, 256, 1300), (9000, 256, 200), (9000, 256, 20)]:  # 160-row, 96-row and 64 x 64 tiles last
        buf = q8_weight(oracle, rng, N, K, DType.Q8_0H)
        buf[: N * K][3::89] = 0x80
        dq = oracle.q8_0_dequantize(buf, N * K, True).reshape(N, K)
        cols = rng.integers(0, K, size=M)
        x = np.zeros((1, M, K), dtype=np.float16)
        x[0, np.arange(M), cols] = 1
        got = gpu_matmul(device, Tensor.from_quantized(buf, DType.Q8_0H, (N, K)), Tensor.from_data(x), None,
                         False, True, True)
        assert np.array_equal(got[0], dq[:, cols].T.astype(np.float16)), (N, K, M)


def test_f16_untransposed_narrow_rhs(device, oracle):
    """`lhs.matmul(rhs)` with an N-contiguous rhs of at most 128 columns (the attention P.V form):
    row counts off the 32-row grouping, K off the 64 tile, every N tile count, stacks, broadcast, bias."""
    shapes = [(2, 64, 64, 80), (1, 100, 72, 8), (3, 257, 200, 128), (1, 512, 512, 80), (1, 65, 8, 16),
              (2, 96, 136, 48), (1, 1000, 320, 104),
              # more K tiles than are in flight at once (whole and ragged), and stack counts that take the
              # XCD-aware workgroup order with whole and ragged row blocks
              (1, 128, 1024, 80), (2, 70, 1160, 40), (8, 100, 72, 24), (16, 128, 576, 64)]
    for i, (S, M, K, N) in enumerate(shapes):
        rng = np.random.default_rng(800 + i)
        a = rng.standard_normal((S, M, K)).astype(np.float16)
        b = rng.standard_normal((S, K, N)).astype(np.float16)
        bias = rng.standard_normal(N).astype(np.float16) if i % 2 == 0 else None
        got = gpu_matmul(device, Tensor.from_data(a), Tensor.from_data(b),
                         None if bias is None else Tensor.from_data(bias), False, False, False)
        want = oracle.matmul_ref(a, oracle.F16, a.shape, b, oracle.F16, b.shape, bias, False, False, False)
        check(oracle, got, want, DType.F16, (S, M, K, N))
    rng = np.random.default_rng(820)
    a = rng.standard_normal((4, 70, 96)).astype(np.float16)
    b = rng.standard_normal((1, 96, 64)).astype(np.float16)   # one rhs for four lhs stacks
    got = gpu_matmul(device, Tensor.from_data(a), Tensor.from_data(b), None, False, False, False)
    check(oracle, got, oracle.matmul_ref(a, oracle.F16, a.shape, b, oracle.F16, b.shape), DType.F16, "broadcast")
    # one-hot rows select rows of the rhs exactly
    x = np.zeros((1, 64, 96), dtype=np.float16)
    cols = rng.integers(0, 96, size=64)
    x[0, np.arange(64), cols] = 1
    got = gpu_matmul(device, Tensor.from_data(x), Tensor.from_data(b), None, False, False, False)
    assert np.array_equal(got[0], b[0][cols])


# ---------------------------------------------------------------------------
# Few output tiles, long K: the large-tile kernels cut K among workgroups when given a workspace
# ---------------------------------------------------------------------------
def _workspace_bytes(device, lhs_dt, lhs_shape, rhs_shape, flags, bias_shape):
    desc = _ffi.make_desc(int(lhs_dt), lhs_shape, _ffi.RT_F16, rhs_shape, *flags,
                          None if bias_shape is None else _ffi.RT_F16, bias_shape)
    need = ctypes.c_uint64(123)
    assert _ffi.lib().rt_matmul_workspace_bytes(device.ctx, ctypes.byref(desc), ctypes.byref(need)) == _ffi.RT_OK
    return need.value


@pytest.mark.parametrize("weights", ["f16", "q8_0h"])
def test_long_k_few_tiles_split_among_workgroups(device, oracle, weights, monkeypatch):
    """[S, N, K] weights against [S, M, K] activations (a prefill down-projection and ragged relatives):
    the split launch, the single pass and the oracle agree; the workspace query says which shapes split."""
    import ratchet_amd.tensor as T
    #        S  N(weight rows) M(activation rows) K     split expected
    shapes = [(1, 320, 128, 2048, True), (1, 161, 77, 4096, True), (2, 200, 100, 2560, True),
              (1, 2560, 512, 10240, True), (1, 1000, 129, 2304, False), (1, 320, 128, 512, False),
              (1, 4000, 1024, 2048, False)]
    for i, (S, N, M, K, expect) in enumerate(shapes):
        rng = np.random.default_rng(900 + i)
        w = (rng.standard_normal((S, N, K)) * 0.05).astype(np.float32)
        x = rng.standard_normal((S, M, K)).astype(np.float16)
        bias = rng.standard_normal(N).astype(np.float16) if i % 2 == 0 else None
        if weights == "f16":
            wt, wbuf, odt, ddt = Tensor.from_data(w.astype(np.float16)), w.astype(np.float16), oracle.F16, DType.F16
        else:
            wbuf = oracle.make_q8_0h(w)
            wt, odt, ddt = Tensor.from_quantized(wbuf, DType.Q8_0H, (S, N, K)), oracle.Q8_0H, DType.Q8_0H
        for flags in ((False, True, True), (False, True, False)):
            b = bias if flags[2] else None   # bias runs along the weight rows, the output's last axis under trans_out
            need = _workspace_bytes(device, ddt, (S, N, K), (S, M, K), flags, None if b is None else b.shape)
            if flags[2] or weights == "q8_0h":   # (f16 operands change roles for a row-major output; no fixed expectation)
                assert (need > 0) == expect, (S, N, M, K, flags, need)
            if need:
                assert need % (S * N * M * 4) == 0 and 2 <= need // (S * N * M * 4) <= 8
            want = oracle.matmul_ref(wbuf, odt, (S, N, K), x, oracle.F16, x.shape, b, *flags)
            monkeypatch.setattr(T, "SPLIT_K", True)
            got = gpu_matmul(device, wt, Tensor.from_data(x), None if b is None else Tensor.from_data(b), *flags)
            check(oracle, got, want, DType.F16, (weights, S, N, M, K, flags, "split"))
            monkeypatch.setattr(T, "SPLIT_K", False)
            one = gpu_matmul(device, wt, Tensor.from_data(x), None if b is None else Tensor.from_data(b), *flags)
            check(oracle, one, want, DType.F16, (weights, S, N, M, K, flags, "one pass"))
            if not need:
                assert np.array_equal(got, one)
            else:   # same products, f32 sums associated differently: the two roundings differ by an ulp at most
                assert np.abs(got.astype(np.float64) - one.astype(np.float64)).max() <= 2e-3 * np.abs(want).max()


def test_split_k_with_fused_activation_and_short_workspace(device, oracle):
    rng = np.random.default_rng(950)
    N, M, K = 320, 96, 2048
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    x = rng.standard_normal((1, M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    desc = _ffi.make_desc(_ffi.RT_F16, (N, K), _ffi.RT_F16, (1, M, K), False, True, True, _ffi.RT_F16, (N,))
    need = _workspace_bytes(device, DType.F16, (N, K), (1, M, K), (False, True, True), (N,))
    assert need > 0
    dw, dx, db = (torch.from_numpy(a.view(np.uint8).reshape(-1).copy()).cuda() for a in (w, x, bias))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for nbytes in (need, need - 16, 0):   # the full workspace; one too short and none: a single pass
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
        out = torch.zeros(M * N * 2, dtype=torch.uint8, device="cuda")
        st = _ffi.lib().rt_matmul_enqueue_ws(device.ctx, ctypes.byref(desc), dw.data_ptr(), dx.data_ptr(), db.data_ptr(),
                                             ctypes.c_void_p(out.data_ptr()), _ffi.RT_ACT_GELU,
                                             ctypes.c_void_p(ws.data_ptr()) if nbytes else None, nbytes, stream)
        assert st == _ffi.RT_OK
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy().view(np.float16).reshape(1, M, N))
    want = oracle.matmul_ref(w, oracle.F16, (N, K), x, oracle.F16, x.shape, bias, False, True, True, act=oracle.ACT_GELU)
    for o in outs:
        assert np.all(np.abs(o.astype(np.float64) - want) <= 2e-3 + 2e-2 * np.abs(want))
    assert np.array_equal(outs[1], outs[2])


# ---------------------------------------------------------------------------
# f32 operands with a contiguous axis each and K a multiple of 32: the f32 matrix-core kernel
# ---------------------------------------------------------------------------
def test_f32_contiguous_operands(device, oracle):
    """`lhs.matmul(rhs)` (rhs N-contiguous) and the Linear form (rhs K-contiguous), with and without trans_out:
    tile edges in both dimensions, K from one tile to many (both tile heights), stacks, broadcast, both bias axes."""
    #        S  M    N    K
    shapes = [(1, 48, 48, 32), (1, 97, 100, 64), (1, 1500, 1536, 384), (2, 130, 52, 96), (1, 50, 333, 1024),
              (3, 200, 96, 800), (1, 96, 4000, 32),
              # K that is not a whole number of 32-wide tiles (any multiple of 4): the head dimension of 80 of the
              # phi2 / whisper score product q.matmul(k.permute([0, 1, 3, 2]), false, false), shorter than a tile, ragged
              (32, 512, 512, 80), (2, 100, 64, 4), (1, 60, 120, 20), (2, 129, 200, 100), (1, 96, 96, 36), (1, 300, 52, 1000),
              # Whisper's two attention products (whisper/mha.rs:105-124) at a third of its 1500 positions: output rows that do
              # not start on a cache line, and 64 output columns
              (2, 500, 500, 64), (2, 500, 64, 500)]
    for i, (S, M, N, K) in enumerate(shapes):
        rng = np.random.default_rng(1000 + i)
        a = (rng.standard_normal((S, M, K)) * 0.1).astype(np.float32)
        for tr, to in ((False, False), (True, True), (True, False), (False, True)):
            if not tr and N % 4:
                continue   # an N-contiguous rhs needs whole vectors along N (other shapes take the generic kernel)
            b = (rng.standard_normal((S, N, K) if tr else (S, K, N)) * 0.1).astype(np.float32)
            bias = (rng.standard_normal(M if to else N) * 0.1).astype(np.float32) if (i + tr + to) % 2 == 0 else None
            got = gpu_matmul(device, Tensor.from_data(a), Tensor.from_data(b), None if bias is None else Tensor.from_data(bias),
                             False, tr, to)
            want = oracle.matmul_ref(a, oracle.F32, a.shape, b, oracle.F32, b.shape, bias, False, tr, to)
            check(oracle, got, want, DType.F32, (S, M, N, K, tr, to))
    # one rhs for three lhs stacks, and GELU fused
    rng = np.random.default_rng(1010)
    a = (rng.standard_normal((3, 70, 64)) * 0.1).astype(np.float32)
    b = (rng.standard_normal((1, 64, 60)) * 0.1).astype(np.float32)
    got = gpu_matmul(device, Tensor.from_data(a), Tensor.from_data(b), None, False, False, False)
    check(oracle, got, oracle.matmul_ref(a, oracle.F32, a.shape, b, oracle.F32, b.shape, None, False, False, False), DType.F32, "broadcast")
    x = Tensor.from_data(a[:1]).to(device).gemm(Tensor.from_data(b).to(device), None, False, False, False).gelu().resolve()
    want = oracle.matmul_ref(a[:1], oracle.F32, (1, 70, 64), b, oracle.F32, b.shape, None, False, False, False, act=oracle.ACT_GELU)
    assert np.all(np.abs(x.to(Device.CPU).storage.astype(np.float64) - want) <= 1e-5 + 1e-3 * np.abs(want))


# ---------------------------------------------------------------------------
# Q4_K weights against 33 or more activation rows: the tiled kernel that decodes the weights in registers
# ---------------------------------------------------------------------------
def test_q4k_prefill_tiles(device, oracle):
    """Tile edges in both dimensions (64 or 128 weight rows x 64 activation rows per workgroup: the last two
    shapes have more than 256 workgroups of 64 weight rows and take the 128-row form), one super-block of K to
    many, per-stack activations against one weight, both bias axes, both output orientations (contiguous along
    the weight rows: 16-byte stores through LDS, whole tiles only; the other: scalar stores)."""
    #        S  N(weight rows) M(activation rows) K
    shapes = [(1, 64, 64, 256), (1, 65, 129, 512), (1, 200, 100, 1024), (2, 130, 257, 768), (1, 1000, 70, 256),
              (3, 96, 64, 2048), (1, 64, 700, 512), (1, 128, 49, 512), (2, 70, 63, 256), (1, 64, 96, 1280),
              (1, 136, 33, 512), (1, 2100, 520, 512), (2, 2056, 530, 256)]
    for i, (S, N, M, K) in enumerate(shapes):
        rng = np.random.default_rng(1200 + i)
        blocks = oracle.q4k_quantize((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
        x = rng.standard_normal((S, M, K)).astype(np.float16)
        for to in (True, False):
            bias = rng.standard_normal(N if to else M).astype(np.float16) if (i + to) % 2 == 0 else None
            got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (N, K)), Tensor.from_data(x),
                             None if bias is None else Tensor.from_data(bias), False, True, to)
            want = oracle.matmul_ref(blocks, oracle.Q4_K, (N, K), x, oracle.F16, x.shape, bias, False, True, to)
            check(oracle, got, want, DType.F16, (S, N, M, K, to))
    # GELU behind the Linear, fused into the kernel's epilogue
    rng = np.random.default_rng(1210)
    N, M, K = 192, 80, 512
    blocks = oracle.q4k_quantize((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
    x = rng.standard_normal((1, M, K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    y = Tensor.from_quantized(blocks, DType.Q4_K, (N, K)).to(device).gemm(
        Tensor.from_data(x).to(device), Tensor.from_data(bias).to(device), False, True, True).gelu().resolve()
    want = oracle.matmul_ref(blocks, oracle.Q4_K, (N, K), x, oracle.F16, x.shape, bias, False, True, True, act=oracle.ACT_GELU)
    assert np.all(np.abs(y.to(Device.CPU).storage.astype(np.float64) - want) <= 2e-3 + 2e-2 * np.abs(want))


def test_q4k_prefill_one_hot_is_the_dequantized_weight(device, oracle):
    """A one-hot activation row selects one dequantized weight per weight row: the tiled kernel must return
    d * sc * q - dmin * mn rounded to f32 and then to f16, bit for bit, for every super-block position.
    d * sc, (d * sc) * q and dmin * mn are exact in f32 (11 + 6 + 4 bits), so the order in which the kernel
    forms d * (sc * q) cannot matter: only the subtraction rounds, in the oracle and in the kernel alike."""
    rng = np.random.default_rng(1220)
    N, K, M = 150, 1024, 300
    blocks = oracle.q4k_quantize((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
    dq = oracle.q4k_dequantize(blocks).reshape(N, K)
    cols = np.concatenate([np.arange(0, K, 37), rng.integers(0, K, size=M)])[:M]
    x = np.zeros((1, M, K), dtype=np.float16)
    x[0, np.arange(M), cols] = 1
    got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (N, K)), Tensor.from_data(x), None, False, True, True)
    want = dq[:, cols].T.astype(np.float16)
    bad = np.argwhere(got[0].view(np.uint16) != want.view(np.uint16))
    assert bad.size == 0, (len(bad), bad[:8].tolist())
    # the same through the form with 128 weight rows per workgroup (more than 256 workgroups of 64 rows)
    N, K, M = 4200, 512, 300
    blocks = oracle.q4k_quantize((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
    dq = oracle.q4k_dequantize(blocks).reshape(N, K)
    cols = np.concatenate([np.arange(0, K, 19), rng.integers(0, K, size=M)])[:M]
    x = np.zeros((1, M, K), dtype=np.float16)
    x[0, np.arange(M), cols] = 1
    got = gpu_matmul(device, Tensor.from_quantized(blocks, DType.Q4_K, (N, K)), Tensor.from_data(x), None, False, True, True)
    want = dq[:, cols].T.astype(np.float16)
    bad = np.argwhere(got[0].view(np.uint16) != want.view(np.uint16))
    assert bad.size == 0, (len(bad), bad[:8].tolist())


@pytest.mark.parametrize("M", [1, 16, 64, 256], ids=["streaming-1", "streaming-16", "tiled-64", "tiled-256"])
def test_q4k_known_answer_block_through_every_kernel(device, oracle, q4k_kat, M):
    """The hand-typed known-answer super-block (tests/conftest.py) as a weight: 64 weight rows x 4 super-blocks,
    every block a copy of it with its f16 d scaled by an exact power of two per (row, block) so that a
    misplaced block shows.  One-hot activations return single dequantized weights: compared bit for bit
    with the hand-worked values, not with the oracle."""
    blk, w, _ = q4k_kat
    N, NB = 64, 4
    K = 256 * NB
    blocks = np.tile(blk, (N, NB, 1))
    expo = (np.arange(N)[:, None] + 3 * np.arange(NB)[None, :]) % 5          # d, dmin *= 2^-expo
    for f in (0, 2):                                                          # the two f16 headers: exponent field -= expo
        h = blocks[:, :, f:f + 2].copy().view(np.uint16)[:, :, 0] - (expo.astype(np.uint16) << 10)
        blocks[:, :, f:f + 2] = h[:, :, None].view(np.uint8)
    dense = (w[None, None, :] * (2.0 ** -expo)[:, :, None]).reshape(N, K).astype(np.float32)
    rng = np.random.default_rng(1230 + M)
    cols = np.concatenate([np.arange(0, K, 257), rng.integers(0, K, size=M)])[:M]
    x = np.zeros((1, M, K), dtype=np.float16)
    x[0, np.arange(M), cols] = 1
    got = gpu_matmul(device, Tensor.from_quantized(blocks.reshape(-1), DType.Q4_K, (N, K)), Tensor.from_data(x), None,
                     False, True, True)
    want = dense[:, cols].T.astype(np.float16)
    assert np.array_equal(got[0].view(np.uint16), want.view(np.uint16))


# ---------------------------------------------------------------------------
# 17..32 activation vectors against Q8_0H or Q4_K weights: one streaming launch per 16 of them (33..64: the tiled kernels)
# ---------------------------------------------------------------------------
def test_quantized_weights_a_few_more_vectors_than_one_streaming_launch(device, oracle):
    rng = np.random.default_rng(1100)
    cases = [("q8", 1, 512, 2560, m) for m in (17, 32, 48, 64)] + [("q8", 2, 96, 512, 33)] + \
            [("q4k", 1, 256, 3072, m) for m in (17, 32, 40, 48)] + [("q4k", 2, 64, 1024, 31)]
    for kind, S, N, K, M in cases:
        w = (rng.standard_normal((S, N, K)) * 0.05).astype(np.float32)
        if kind == "q8":
            buf, odt, ddt = oracle.make_q8_0h(w), oracle.Q8_0H, DType.Q8_0H
        else:
            buf, odt, ddt = oracle.q4k_quantize(w), oracle.Q4_K, DType.Q4_K
        x = rng.standard_normal((S, M, K)).astype(np.float16)
        wt = Tensor.from_quantized(buf, ddt, (S, N, K))
        for to in (True, False):
            # the bias runs along the output's last axis: the weight rows under trans_out, the vectors otherwise
            bias = rng.standard_normal(N if to else M).astype(np.float16)
            got = gpu_matmul(device, wt, Tensor.from_data(x), Tensor.from_data(bias), False, True, to)
            want = oracle.matmul_ref(buf, odt, (S, N, K), x, oracle.F16, x.shape, bias, False, True, to)
            check(oracle, got, want, DType.F16, (kind, S, N, K, M, to))


@pytest.mark.parametrize("rows_w,rows_x", [(1280, 768), (1280, 1408), (2560, 640), (2100, 1300), (9000, 200), (4100, 100)],
                         ids=["8x6", "8x11", "16x5", "160-row-tiles-14x11-edges", "96-row-tiles", "64-row-tiles-edges"])
@pytest.mark.parametrize("quant", [False, True], ids=["f16", "q8_0h"])
def test_large_tile_panel_order(device, oracle, rows_w, rows_x, quant):
    """Large-tile NT GEMMs with whole weight row blocks per XCD and more than four activation column blocks walk
    their tiles in panels of four column blocks (a narrower last panel included): every output tile must be
    written exactly once.  The output of each tile depends on its position (distinct rows of both
    operands), so a tile computed twice or never shows against the oracle.  A grid of 160-row tiles that would
    leave half the compute units idle is cut into 64-row tiles, or 96-row ones where those no longer run all at
    once: the ids name the form a shape takes on 256 compute units (the first three: 64-row tiles)."""
    rng = np.random.default_rng(rows_w + rows_x)
    K = 256
    w = (rng.standard_normal((rows_w, K)) * 0.05).astype(np.float32)
    x = rng.standard_normal((1, rows_x, K)).astype(np.float16)
    bias = rng.standard_normal(rows_w).astype(np.float16)
    if quant:
        buf = oracle.make_q8_0h(w)
        lhs = Tensor.from_quantized(buf, DType.Q8_0H, (rows_w, K))
        want = oracle.matmul_ref(buf, oracle.Q8_0H, (rows_w, K), x, oracle.F16, x.shape, bias, False, True, True)
    else:
        wh = w.astype(np.float16)
        lhs = Tensor.from_data(wh)
        want = oracle.matmul_ref(wh, oracle.F16, wh.shape, x, oracle.F16, x.shape, bias, False, True, True)
    got = gpu_matmul(device, lhs, Tensor.from_data(x), Tensor.from_data(bias), False, True, True)
    assert got.shape == (1, rows_x, rows_w)
    assert oracle.max_rel_err(got, want) <= 2e-2


def test_checked_mode_refuses_short_buffers(device, oracle, monkeypatch):
    """RATCHET_CHECKED (read by rt_ctx_create): an operand or output allocation smaller than the descriptor
    implies is refused with a status before anything is launched; exact allocations pass and compute."""
    import ctypes

    from ratchet_amd import _ffi
    L = _ffi.lib()
    monkeypatch.setenv("RATCHET_CHECKED", "1")
    ctx = ctypes.c_void_p()
    assert L.rt_ctx_create(device.ordinal, ctypes.byref(ctx)) == _ffi.RT_OK
    try:
        N, M, K = 256, 64, 512
        rng = np.random.default_rng(77)
        w = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
        buf = oracle.make_q8_0h(w)
        x = rng.standard_normal((1, M, K)).astype(np.float16)
        desc = _ffi.make_desc(_ffi.RT_Q8_0H, (N, K), _ffi.RT_F16, (1, M, K), False, True, True)

        def alloc(nbytes, data=None):
            p = ctypes.c_void_p()
            assert L.rt_buf_alloc(ctx, nbytes, ctypes.byref(p)) == _ffi.RT_OK
            if data is not None:
                host = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
                assert L.rt_buf_upload(ctx, p, host.ctypes.data_as(ctypes.c_void_p), host.size, None) == _ffi.RT_OK
                assert L.rt_sync(ctx, None) == _ffi.RT_OK
            return p

        dw, dx = alloc(buf.nbytes, buf), alloc(x.nbytes, x)
        out_ok, out_short = alloc(M * N * 2), alloc(M * N * 2 - 256)
        w_short = alloc(buf.nbytes - 4096)
        bufs = [dw, dx, out_ok, out_short, w_short]
        stream = ctypes.c_void_p(0)
        st = L.rt_matmul_enqueue(ctx, ctypes.byref(desc), dw, dx, None, out_short, stream)
        assert st == _ffi.RT_ERR_INVALID_ARG and b"out holds" in L.rt_last_error(ctx)
        st = L.rt_matmul_enqueue(ctx, ctypes.byref(desc), w_short, dx, None, out_ok, stream)
        assert st == _ffi.RT_ERR_INVALID_ARG and b"lhs holds" in L.rt_last_error(ctx)
        # a pointer into the middle of an allocation counts from there
        st = L.rt_matmul_enqueue(ctx, ctypes.byref(desc), dw, dx, None, ctypes.c_void_p(out_ok.value + 512), stream)
        assert st == _ffi.RT_ERR_INVALID_ARG
        st = L.rt_matmul_enqueue(ctx, ctypes.byref(desc), dw, dx, None, out_ok, stream)
        assert st == _ffi.RT_OK, L.rt_last_error(ctx)
        assert L.rt_sync(ctx, stream) == _ffi.RT_OK
        got = np.empty((1, M, N), dtype=np.float16)
        assert L.rt_buf_download(ctx, got.ctypes.data_as(ctypes.c_void_p), out_ok, got.nbytes, None) == _ffi.RT_OK
        assert L.rt_sync(ctx, None) == _ffi.RT_OK
        want = oracle.matmul_ref(buf, oracle.Q8_0H, (N, K), x, oracle.F16, x.shape, None, False, True, True)
        assert oracle.max_rel_err(got, want) <= 2e-2
        for b in bufs:
            L.rt_buf_free(ctx, b)
    finally:
        L.rt_ctx_destroy(ctx)
