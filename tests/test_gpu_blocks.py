"""Block-format kernels on the GPU, through the C ABI: bit-exact against the oracle
and the golden fixtures."""
import os

import numpy as np
import pytest

from ratchet_amd import DType, Device, Quantization, Quantizer, Tensor, dequantize, transcode_gguf_q8_0

pytestmark = pytest.mark.gpu
G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def raw(t: Tensor) -> np.ndarray:
    return t.to(Device.CPU).storage


def test_quantize_bit_exact(device, oracle):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((64, 64)).astype(np.float32)        # the reference's test_sint8_qdq shape
    x[3, 32:64] = 0.0
    x[5, :32] = np.arange(-16, 16) + 0.5                          # ties
    x[6, :32] = 1e-30                                             # tiny scale
    x[7, :32] = 3e38                                              # huge scale
    q = Quantizer(Quantization.SInt8, device).sint8_quantize(Tensor.from_data(x))
    assert q.dt == DType.Q8_0F and q.shape == (64, 64)
    assert np.array_equal(raw(q), oracle.q8_0_quantize_f32(x))
    f = np.load(os.path.join(G, "q8_0_quantize.npz"))
    q = Quantizer(Quantization.SInt8, device).sint8_quantize(Tensor.from_data(f["x"]))
    buf = raw(q)
    n = f["x"].size
    assert np.array_equal(buf[:n].view(np.int8).reshape(f["q"].shape), f["q"])
    assert np.array_equal(buf[oracle.q8_0_scale_offset(n):][: 4 * (n // 32)].view(np.float32), f["d"])


@pytest.mark.parametrize("numel", [32, 288, 4096, 1000 * 32, 2560 * 512])
def test_quantize_sizes(device, oracle, numel):
    rng = np.random.default_rng(numel)
    x = (rng.standard_normal(numel) * 0.02).astype(np.float32)
    q = Quantizer(Quantization.SInt8, device).sint8_quantize(Tensor.from_data(x))
    assert np.array_equal(raw(q), oracle.q8_0_quantize_f32(x))


@pytest.mark.parametrize("dt", [DType.Q8_0F, DType.Q8_0H])
def test_dequantize_q8_bit_exact(device, oracle, dt):
    f16 = dt == DType.Q8_0H
    rng = np.random.default_rng(1)
    nb = 1024
    buf = np.zeros(oracle.q8_0_nbytes(nb * 32, f16), np.uint8)
    buf[: nb * 32] = np.tile(np.arange(256, dtype=np.uint8), nb * 32 // 256)    # every byte incl. -128
    sc = rng.standard_normal(nb).astype(np.float16 if f16 else np.float32)
    sc[:4] = [0.0, 6.1e-5, -2.0, 1000.0]
    off = oracle.q8_0_scale_offset(nb * 32)
    buf[off: off + sc.nbytes] = sc.view(np.uint8)
    got = dequantize(Tensor.from_quantized(buf, dt, (nb, 32), device)).to_ndarray()
    want = oracle.q8_0_dequantize(buf, nb * 32, f16).reshape(nb, 32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_quantizer_round_trip_api(device, oracle):
    """Quantizer::sint8_quantize then sint8_dequantize (quant.rs:26-124)."""
    rng = np.random.default_rng(2)
    x = rng.standard_normal((64, 64)).astype(np.float32)
    qz = Quantizer(Quantization.SInt8, device)
    dq = qz.sint8_dequantize(qz.sint8_quantize(Tensor.from_data(x)))
    want = oracle.q8_0_dequantize(oracle.q8_0_quantize_f32(x), x.size, False).reshape(x.shape)
    assert dq.dt == DType.F32 and np.array_equal(dq.to_ndarray(), want)


def test_dequantize_q4k_bit_exact(device, oracle):
    f = np.load(os.path.join(G, "q4_k.npz"))
    t = Tensor.from_quantized(f["blocks"], DType.Q4_K, tuple(int(v) for v in f["shape"]), device)
    assert np.array_equal(dequantize(t).to_ndarray().reshape(-1), f["dequant"])
    rng = np.random.default_rng(3)
    # random bytes are valid Q4_K blocks as long as d, dmin are finite
    nb = 2000
    blocks = rng.integers(0, 256, size=(nb, 144), dtype=np.int64).astype(np.uint8)
    blocks[:, 0:4] = (rng.standard_normal((nb, 2)) * 0.01).astype(np.float16).view(np.uint8).reshape(nb, 4)
    got = dequantize(Tensor.from_quantized(blocks, DType.Q4_K, (nb, 256), device)).to_ndarray().reshape(-1)
    want = oracle.q4k_dequantize(blocks.reshape(-1))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequantize_q4k_known_answer_block(device, q4k_kat):
    """The hand-typed super-block and its hand-worked values (tests/conftest.py): no packer, no oracle."""
    blk, want, _ = q4k_kat
    blocks = np.tile(blk, 3)
    got = dequantize(Tensor.from_quantized(blocks, DType.Q4_K, (3, 256), device)).to_ndarray()
    assert np.array_equal(got.view(np.uint32), np.tile(want, (3, 1)).view(np.uint32))


@pytest.mark.parametrize("dt", [DType.Q8_0F, DType.Q8_0H])
def test_transcode_bit_exact(device, oracle, dt):
    f16 = dt == DType.Q8_0H
    f = np.load(os.path.join(G, "q8_0.npz"))
    shape = tuple(int(v) for v in f["shape"])
    t = transcode_gguf_q8_0(f["gguf_blocks"], shape, dt, device)
    assert np.array_equal(raw(t), f["segments_h" if f16 else "segments_f"])
    rng = np.random.default_rng(4)
    w = (rng.standard_normal((333, 96)) * 0.02).astype(np.float32)     # 999 blocks: ragged tail for the padding
    blocks = oracle.gguf_q8_0_quantize(w)
    t = transcode_gguf_q8_0(blocks, w.shape, dt, device)
    assert np.array_equal(raw(t), oracle.transcode_gguf_q8_0(blocks, f16))
