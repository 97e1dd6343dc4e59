"""A seeded sweep over the shapes at which the Matmul dispatch changes kernels, through the C ABI, against the CPU oracle.

The dispatch (ratchet-core picks between its GEMV and GEMM shaders by `rhs.is_vector()`, ops/matmul.rs:215-245; here a
cascade of launchers that each decline what they do not take) switches kernel at vector counts 1/2, 2/3, 4/5, 8/9, 16/17,
32/33, 64/65, 128/129, at weight row counts that give a compute unit a workgroup or not, and at K multiples of 32, 64,
256 and 512.  Every Linear-form product `W.gemm(x, bias, false, true, to)` here sits on or next to one of those edges.
Tolerances: max-rel-err <= 2e-2 for f16 I/O and <= 1e-3 for f32 (max_i |y_i - r_i| / max(|r_i|, 1e-3 max_j |r_j|)).
"""
import numpy as np
import pytest

from ratchet_amd import DType, Device, Tensor

pytestmark = pytest.mark.gpu

VECTORS = [1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 24, 31, 32, 33, 40, 48, 49, 63, 64, 65, 100, 128, 129]
ROWS = [16, 40, 161, 640, 1000, 2001, 2048, 4100, 6152, 8192, 10240]
KS = [32, 64, 96, 256, 320, 512, 768, 1024, 1280, 2560, 4096]


def cases(seed, n, k_multiple, max_work):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        M, N, K = int(rng.choice(ROWS)), int(rng.choice(VECTORS)), int(rng.choice(KS))
        if K % k_multiple or M * N * K > max_work:
            continue
        out.append((M, N, K, bool(rng.integers(0, 2)), int(rng.integers(0, 3))))
    return out


def run(device, oracle, w_tensor, w_src, w_odt, M, N, K, to, bias_kind, adt, tol, rng, mirrored=False):
    """`W.gemm(x, bias, false, true, to)`, or mirrored (the reference's own spelling of a Linear over activations,
    `x.gemm(W, bias, false, true, to)`, crates/ratchet-nn/src/linear.rs:17-24 with the operands the other way round)."""
    x = rng.standard_normal((1, N, K)).astype(adt)
    xdt = oracle.F16 if adt == np.float16 else oracle.F32
    last = (N if to else M) if mirrored else (M if to else N)   # the bias runs along the output's last dimension
    bias = None if bias_kind == 0 else rng.standard_normal(last).astype(adt)
    bt = None if bias is None else Tensor.from_data(bias).to(device)
    if mirrored:
        got = Tensor.from_data(x).to(device).gemm(w_tensor.to(device), bt, False, True, to).resolve().to(Device.CPU).storage
        # x . W^T is (W . x^T)^T: the oracle takes the quantized operand on the left, so it is asked for the other transposition
        want = oracle.matmul_ref(w_src, w_odt, (M, K), x, xdt, x.shape, bias, False, True, not to)
    else:
        got = w_tensor.to(device).gemm(Tensor.from_data(x).to(device), bt, False, True, to).resolve().to(Device.CPU).storage
        want = oracle.matmul_ref(w_src, w_odt, (M, K), x, xdt, x.shape, bias, False, True, to)
    assert got.shape == want.shape, (M, N, K, to, mirrored)
    err = oracle.max_rel_err(got, want)
    assert err <= tol, (M, N, K, to, bias_kind, mirrored, err)


def test_f16_weights(device, oracle):
    for i, (M, N, K, to, bk) in enumerate(cases(4100, 150, 32, 3_000_000_000)):
        rng = np.random.default_rng(4200 + i)
        w = (rng.standard_normal((M, K)) * 0.05).astype(np.float16)
        run(device, oracle, Tensor.from_data(w), w, oracle.F16, M, N, K, to, bk, np.float16, 2e-2, rng, mirrored=i % 3 == 2)


def test_q8_0h_weights(device, oracle):
    for i, (M, N, K, to, bk) in enumerate(cases(4300, 150, 32, 3_000_000_000)):
        rng = np.random.default_rng(4400 + i)
        buf = oracle.make_q8_0h((rng.standard_normal((M, K)) * 0.05).astype(np.float32))
        run(device, oracle, Tensor.from_quantized(buf, DType.Q8_0H, (M, K)), buf, oracle.Q8_0H, M, N, K, to, bk, np.float16, 2e-2, rng, mirrored=i % 3 == 2)


def test_q4_k_weights(device, oracle):
    for i, (M, N, K, to, bk) in enumerate(cases(4500, 100, 256, 3_000_000_000)):
        rng = np.random.default_rng(4600 + i)
        blocks = oracle.q4k_quantize((rng.standard_normal((M, K)) * 0.05).astype(np.float32))
        run(device, oracle, Tensor.from_quantized(blocks, DType.Q4_K, (M, K)), blocks, oracle.Q4_K, M, N, K, to, bk, np.float16, 2e-2, rng)


def test_f32_and_q8_0f_weights(device, oracle):
    for i, (M, N, K, to, bk) in enumerate(cases(4700, 100, 32, 1_500_000_000)):
        rng = np.random.default_rng(4800 + i)
        w = (rng.standard_normal((M, K)) * 0.05).astype(np.float32)
        if i % 2:
            run(device, oracle, Tensor.from_data(w), w, oracle.F32, M, N, K, to, bk, np.float32, 1e-3, rng)
        else:
            buf = oracle.q8_0_quantize_f32(w)
            run(device, oracle, Tensor.from_quantized(buf, DType.Q8_0F, (M, K)), buf, oracle.Q8_0F, M, N, K, to, bk, np.float32, 1e-3, rng)
