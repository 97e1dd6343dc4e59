"""Pins the oracle's block-format functions (CPU only).

Each check is chosen so that a plausible mistake in oracle/oracle.c fails it;
none of them re-types the oracle's own formula.  Reference citations are
relative to the reference checkout.
"""
import numpy as np
import pytest


# ---- f16 conversion: against numpy's IEEE binary16 -------------------------
def test_f16_to_f32_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.lib().orc_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_rounding(oracle):
    rng = np.random.default_rng(0)
    # random bit patterns across the whole exponent range, plus every tie between two halves
    xs = rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    h = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    ties = ((h[:-1] + h[1:]) / 2).astype(np.float32)  # exactly representable midpoints
    special = np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e10, -1e10, 5.96e-8, 2.98e-8, 2.9803e-8,
                        np.inf, -np.inf], dtype=np.float32)
    xs = np.concatenate([xs[np.isfinite(xs)], ties, -ties, special])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    f = oracle.lib().orc_f32_to_f16
    got = np.array([f(float(x)) for x in xs], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert (f(float("nan")) & 0x7C00) == 0x7C00 and (f(float("nan")) & 0x3FF) != 0


# ---- segment layout: dtype/blocks.rs:61-74, gpu/align.rs:25-39 ---------------
@pytest.mark.parametrize("numel,f16,scale_off,total", [
    (32, True, 256, 512),            # 32 B of qs pad to 256; 1 scale (2 B) pads to 256
    (32, False, 256, 512),
    (256, True, 256, 512),           # qs exactly one alignment unit: no padding
    (288, True, 512, 768),           # 288 -> 512; 9 scales = 18 B -> 256
    (4096, False, 4096, 4096 + 512),  # 128 f32 scales = 512 B
    (10240 * 2560, True, 26214400, 27852800),   # Phi-2 MLP weight: 26,214,400 + 1,638,400
    (10240 * 2560, False, 26214400, 26214400 + 3276800),
])
def test_q8_0_layout_known_answers(oracle, numel, f16, scale_off, total):
    assert oracle.q8_0_scale_offset(numel) == scale_off
    assert oracle.q8_0_nbytes(numel, f16) == total


# ---- Q8_0 quantizer: quant.rs:26-79 ---------------------------------------------
def test_q8_0_quantize_known_block(oracle):
    # max|x| = 127 -> d = 1 exactly, so q = round_half_away(x)
    x = np.zeros(32, dtype=np.float32)
    x[:10] = [127, -127, 0.5, -0.5, 1.5, -1.5, 2.4999, -2.5, 126.5, -0.49]
    buf = oracle.q8_0_quantize_f32(x)
    q = buf[:32].view(np.int8)
    assert list(q[:10]) == [127, -127, 1, -1, 2, -2, 2, -3, 127, 0]
    assert buf.size == 512 and not buf[32:256].any()
    d = buf[256:260].view(np.float32)[0]
    assert d == np.float32(1.0)
    assert not buf[260:].any()


def test_q8_0_quantize_packing_is_little_endian_per_u32(oracle):
    # the reference packs 4 values per u32 with element 0 in the low byte (quant.rs:63-67)
    x = np.arange(-16, 16, dtype=np.float32) * (127.0 / 16.0) / (127.0 / 16.0)
    x[0] = -127.0  # force d = 1
    buf = oracle.q8_0_quantize_f32(x)
    words = buf[:32].view("<u4")
    for w in range(8):
        for b in range(4):
            byte = (int(words[w]) >> (8 * b)) & 0xFF
            assert np.int8(np.uint8(byte)) == np.int8(round(float(x[4 * w + b])))


def test_q8_0_quantize_zero_block_and_invariants(oracle):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((64, 64)).astype(np.float32)  # the reference's test_sint8_qdq shape
    x[3, 32:64] = 0.0                                      # an all-zero group
    buf = oracle.q8_0_quantize_f32(x)
    n = x.size
    q = buf[:n].view(np.int8).reshape(-1, 32).astype(np.int32)
    d = buf[oracle.q8_0_scale_offset(n):][: (n // 32) * 4].view(np.float32)
    xg = x.reshape(-1, 32)
    zero = 3 * 2 + 1
    assert d[zero] == 0 and not q[zero].any()
    amax = np.abs(xg).max(axis=1)
    assert np.array_equal(d, (amax / np.float32(127.0)).astype(np.float32))
    nz = d > 0
    # the group's largest magnitude maps to +-127, nothing exceeds it
    assert (np.abs(q[nz]).max(axis=1) == 127).all() and np.abs(q).max() <= 127
    # round-to-nearest: reconstruction error at most half a step (plus f32 slack)
    err = np.abs(q * d[:, None].astype(np.float64) - xg)
    assert (err[nz] <= 0.5 * d[nz, None] * (1 + 1e-5)).all()
    # dequantize inverts exactly what was stored
    dq = oracle.q8_0_dequantize(buf, n, False).reshape(-1, 32)
    assert np.array_equal(dq, (q.astype(np.float32) * d[:, None]))


# ---- Q8_0 dequantize: quant.rs:81-124 (closed form, exact in f32) --------------
@pytest.mark.parametrize("f16", [True, False])
def test_q8_0_dequantize_exhaustive_bytes(oracle, f16):
    rng = np.random.default_rng(2)
    nb = 64
    qs = np.tile(np.arange(256, dtype=np.uint8), nb * 32 // 256)  # every byte value, incl. 0x80 = -128
    if f16:
        scales = rng.standard_normal(nb).astype(np.float16)
        scales[:4] = [0.0, 6.1e-5, 65504.0, -2.0]  # zero, near-subnormal, max, negative
        sbytes = scales.view(np.uint8)
    else:
        scales = rng.standard_normal(nb).astype(np.float32)
        scales[:3] = [0.0, 1e-30, -3.5]
        sbytes = scales.view(np.uint8)
    buf = np.zeros(oracle.q8_0_nbytes(nb * 32, f16), dtype=np.uint8)
    buf[: nb * 32] = qs
    off = oracle.q8_0_scale_offset(nb * 32)
    buf[off: off + sbytes.size] = sbytes
    got = oracle.q8_0_dequantize(buf, nb * 32, f16)
    # int8 x (f16|f32 scale): computed in float64 then rounded to f32 once.  For f16
    # scales the product has <= 18 significant bits, so it is exact in f32.
    want = (qs.view(np.int8).astype(np.float64).reshape(nb, 32) * scales.astype(np.float64)[:, None])
    assert np.array_equal(got.reshape(nb, 32), want.astype(np.float32))
    # -128 follows the CPU rule (sign-extended byte), not the WGSL snorm clamp to -127
    i = int(np.where(qs == 0x80)[0][0])
    assert got[i] == np.float32(-128.0) * np.float32(scales[i // 32])


# ---- GGUF Q8_0 blocks and transcode: k_quants.rs:57-63, gguf/dtype.rs:40-110 ----
def _hand_blocks(nb, rng):
    d = rng.standard_normal(nb).astype(np.float16)
    qs = rng.integers(-128, 128, size=(nb, 32), dtype=np.int64).astype(np.int8)
    blocks = np.zeros((nb, 34), dtype=np.uint8)
    blocks[:, :2] = d.view(np.uint8).reshape(nb, 2)
    blocks[:, 2:] = qs.view(np.uint8)
    return d, qs, blocks.reshape(-1)


@pytest.mark.parametrize("f16", [True, False])
def test_transcode_known_layout(oracle, f16):
    rng = np.random.default_rng(3)
    nb = 9  # 288 weights: qs pads 288 -> 512
    d, qs, blocks = _hand_blocks(nb, rng)
    out = oracle.transcode_gguf_q8_0(blocks, f16)
    assert out.size == (512 + 256)
    assert np.array_equal(out[:288].view(np.int8).reshape(nb, 32), qs)
    assert not out[288:512].any()
    if f16:
        assert np.array_equal(out[512:512 + 18].view(np.float16), d)       # bit-identical f16
        assert not out[512 + 18:].any()
    else:
        assert np.array_equal(out[512:512 + 36].view(np.float32), d.astype(np.float32))  # widened exactly
        assert not out[512 + 36:].any()
    # values survive the trip: dequantize(transcode(blocks)) == q * d
    got = oracle.q8_0_dequantize(out, nb * 32, f16).reshape(nb, 32)
    assert np.array_equal(got, qs.astype(np.float32) * d.astype(np.float32)[:, None])


def test_gguf_quantizer_properties(oracle):
    rng = np.random.default_rng(4)
    w = (rng.standard_normal(32 * 50) * 0.02).astype(np.float32)
    w[64:96] = 0
    blocks = oracle.gguf_q8_0_quantize(w).reshape(-1, 34)
    d = blocks[:, :2].copy().view(np.float16).reshape(-1).astype(np.float32)
    q = blocks[:, 2:].view(np.int8).astype(np.float32)
    assert d[2] == 0 and not q[2].any()
    amax = np.abs(w.reshape(-1, 32)).max(axis=1)
    assert np.array_equal(d, (amax / np.float32(127)).astype(np.float16).astype(np.float32))
    # reconstruction within half a step of the unrounded scale + the f16 rounding of d
    err = np.abs(q * d[:, None] - w.reshape(-1, 32))
    assert (err <= (0.5 + 127 * 2.0 ** -11) * (amax / 127)[:, None] * (1 + 1e-5) + 1e-12).all()


# ---- Q4_K (parity unpinned by the reference; pinned by construction here) -----
def _q4k_block(d, dmin, sc, mn, q):
    """Packs one super-block from explicit fields, following the layout of
    k_quants.rs:94-103 and the 6-bit packing ggml documents for get_scale_min_k4."""
    blk = np.zeros(144, dtype=np.uint8)
    blk[0:2] = np.array([d], dtype=np.float16).view(np.uint8)
    blk[2:4] = np.array([dmin], dtype=np.float16).view(np.uint8)
    s = np.zeros(12, dtype=np.uint8)
    for j in range(4):
        s[j] = (sc[j] & 63) | ((sc[j + 4] >> 4) << 6)
        s[j + 4] = (mn[j] & 63) | ((mn[j + 4] >> 4) << 6)
        s[j + 8] = (sc[j + 4] & 0xF) | ((mn[j + 4] & 0xF) << 4)
    blk[4:16] = s
    q = np.asarray(q, dtype=np.uint8).reshape(4, 2, 32)  # chunk, (low, high) sub-block, element
    blk[16:] = (q[:, 0, :] | (q[:, 1, :] << 4)).reshape(-1)
    return blk


def test_q4k_scale_min_unpacking(oracle):
    rng = np.random.default_rng(5)
    for _ in range(50):
        sc = rng.integers(0, 64, 8)
        mn = rng.integers(0, 64, 8)
        blk = _q4k_block(1.0, 1.0, sc, mn, np.zeros(256))
        for j in range(8):
            assert oracle.q4k_scale_min(j, blk[4:16]) == (sc[j], mn[j])


def test_q4k_dequantize_hand_built(oracle):
    rng = np.random.default_rng(6)
    # identity scales: w == nibble, which pins the nibble order (low = first 32 of a 64-chunk)
    q = rng.integers(0, 16, 256)
    got = oracle.q4k_dequantize(_q4k_block(1.0, 0.0, [1] * 8, [0] * 8, q))
    assert np.array_equal(got, q.astype(np.float32))
    # general block against the formula evaluated in float64
    sc, mn = rng.integers(0, 64, 8), rng.integers(0, 64, 8)
    d, dmin = np.float16(0.0123), np.float16(0.0456)
    got = oracle.q4k_dequantize(_q4k_block(d, dmin, sc, mn, q)).astype(np.float64)
    want = (np.float64(d) * np.repeat(sc, 32) * q - np.float64(dmin) * np.repeat(mn, 32))
    # d*sc, dmin*mn and d*sc*q are exact in f32; only the subtraction rounds
    assert np.array_equal(got.astype(np.float32), want.astype(np.float32))


def test_q4k_known_answer_block(oracle, q4k_kat):
    """The hand-typed 144 bytes and hand-worked values of tests/conftest.py: independent of _q4k_block above,
    including the j >= 4 scales and mins whose two high bits live in scales[0..7]."""
    blk, want, scmn = q4k_kat
    for j in range(8):
        assert oracle.q4k_scale_min(j, blk[4:16]) == scmn[j]
    assert np.array_equal(oracle.q4k_dequantize(blk).view(np.uint32), want.view(np.uint32))
    # and the packer used by the other tests agrees with the hand-typed bytes
    assert np.array_equal(_q4k_block(q4k_kat.d, q4k_kat.dmin, [s for s, _ in scmn], [m for _, m in scmn], q4k_kat.nibbles), blk)


def test_q4k_quantizer_round_trip(oracle):
    rng = np.random.default_rng(7)
    w = (rng.standard_normal(256 * 40) * 0.02).astype(np.float32)
    blocks = oracle.q4k_quantize(w)
    assert blocks.size == 40 * 144
    dq = oracle.q4k_dequantize(blocks)
    # affine 4-bit fit per 32: error bounded by about one step of the sub-block range
    wg, dg = w.reshape(-1, 32), dq.reshape(-1, 32)
    step = (np.maximum(wg.max(axis=1), 0) - np.minimum(wg.min(axis=1), 0)) / 15
    assert (np.abs(wg - dg) <= 1.6 * step[:, None] + 1e-4).all()
    assert np.corrcoef(w, dq)[0, 1] > 0.99
