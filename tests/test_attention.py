"""Fused attention against the reference's operator sequence (crates/ratchet-models/src/phi2/attn.rs:138-152,
phi3/attn.rs:142-158, whisper/mha.rs:105-124): matmul(q, k^T) * scale (+ mask) -> softmax -> cast -> matmul(p, v).

The oracle restates that sequence, roundings included, and is pinned against torch's
scaled_dot_product_attention in float64 (a library routine that shares no code with it) and against
closed forms.  The device kernel keeps the scores in f32 from the first product to the division by the
row sum, so it is compared with the oracle (either placement of the reference's score rounding) and with
torch at the f16 tolerance: |y - r| <= 2e-3 + 2e-2 |r| for outputs of order one."""
import ctypes

import numpy as np
import pytest
import torch

from ratchet_amd import DType, Device, InvariantError, OperationError, Tensor, _ffi

ATOL, RTOL = 2e-3, 2e-2


def sdpa64(q, k, v, mask=None, scale=None, causal=False):
    tq, tk, tv = (torch.from_numpy(a.astype(np.float64)) for a in (q, k, v))
    m = None if mask is None else torch.from_numpy(mask.astype(np.float64))
    if causal:
        Lq, Lk = q.shape[-2], k.shape[-2]
        cm = torch.full((Lq, Lk), -np.inf, dtype=torch.float64).triu(1 + Lk - Lq)
        m = cm if m is None else m + cm
    return torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=m, scale=scale).numpy()


def assert_close(got, want, what=""):
    got, want = got.astype(np.float64), want.astype(np.float64)
    bad = ~((np.abs(got - want) <= ATOL + RTOL * np.abs(want)) | (np.isnan(got) & np.isnan(want)))
    assert not bad.any(), (what, int(bad.sum()), float(np.nanmax(np.abs(got - want))))


def rand_qkv(rng, B, H, Lq, Lk, D, spread=1.0):
    q = (rng.standard_normal((B, H, Lq, D)) * spread).astype(np.float16)
    k = (rng.standard_normal((B, H, Lk, D)) * spread).astype(np.float16)
    v = rng.standard_normal((B, H, Lk, D)).astype(np.float16)
    return q, k, v


# ---------------------------------------------------------------------------
# CPU: the oracle
# ---------------------------------------------------------------------------
def test_oracle_against_torch_sdpa(oracle):
    rng = np.random.default_rng(0)
    for i, (B, H, Lq, Lk, D) in enumerate([(1, 1, 1, 1, 8), (2, 3, 17, 23, 40), (1, 4, 64, 64, 80), (1, 2, 5, 130, 64),
                                           (1, 2, 33, 33, 96)]):
        q, k, v = rand_qkv(rng, B, H, Lq, Lk, D)
        for rs in (False, True):
            assert_close(oracle.attention(q, k, v, round_scores=rs), sdpa64(q, k, v), ("plain", i, rs))
            assert_close(oracle.attention(q, k, v, causal=True, round_scores=rs), sdpa64(q, k, v, causal=True), ("causal", i, rs))
        mask = (rng.standard_normal((Lq, Lk)) * 2).astype(np.float32)
        mask[rng.random((Lq, Lk)) < 0.2] = -np.inf
        mask[:, 0] = 0                                        # every row keeps a visible key
        assert_close(oracle.attention(q, k, v, mask=mask, scale=0.3), sdpa64(q, k, v, mask=mask, scale=0.3), ("mask", i))
    # the causal flag is the callers' -inf upper-triangular mask
    q, k, v = rand_qkv(rng, 1, 2, 9, 14, 16)
    tri = np.triu(np.full((9, 14), -np.inf, np.float32), 1 + 14 - 9)
    assert np.array_equal(oracle.attention(q, k, v, causal=True), oracle.attention(q, k, v, mask=tri))


def test_oracle_closed_forms(oracle):
    rng = np.random.default_rng(1)
    q, k, v = rand_qkv(rng, 1, 2, 6, 12, 16)
    # one key only: the output is that value row, whatever the scores
    assert np.array_equal(oracle.attention(q, k[:, :, :1], v[:, :, :1]), np.broadcast_to(v[:, :, :1], q.shape))
    # identical keys: uniform weights 1/12 (f16-rounded), the mean of the values
    ksame = np.broadcast_to(k[:, :, :1], k.shape).copy()
    want = (np.float32(np.float16(1 / 12)) * v.astype(np.float32)).sum(axis=2, keepdims=True)
    np.testing.assert_allclose(oracle.attention(q, ksame, v).astype(np.float32), np.broadcast_to(want, q.shape), rtol=2e-3, atol=1e-3)
    # a key aligned with the query and far longer than the rest takes all the weight
    kbig = k.copy()
    kbig[:, :, 5] = 0
    qs = np.zeros_like(q)
    qs[..., 0] = 8
    kbig[:, :, 5, 0] = 60
    assert np.array_equal(oracle.attention(qs, kbig, v, scale=1.0), np.broadcast_to(v[:, :, 5:6], q.shape))
    # a row whose every key is masked is NaN (softmax of -inf everywhere), the others are untouched
    mask = np.zeros((6, 12), np.float32)
    mask[2] = -np.inf
    o = oracle.attention(q, k, v, mask=mask)
    assert np.isnan(o[:, :, 2]).all() and not np.isnan(np.delete(o, 2, axis=2)).any()
    # causal with q_len == kv_len: the first query sees only the first key
    o = oracle.attention(q, k[:, :, :6], v[:, :, :6], causal=True)
    assert np.array_equal(o[:, :, 0], v[:, :, 0])


def test_guards_without_a_device():
    L = _ffi.lib()
    d = _ffi.AttentionDesc()
    d.dtype, d.batch, d.heads, d.q_len, d.kv_len, d.head_dim = _ffi.RT_F16, 1, 2, 8, 8, 80
    for s in (d.q_strides, d.k_strides, d.v_strides, d.o_strides):
        s[:] = [2 * 8 * 80, 8 * 80, 80]
    d.scale = 0.1
    assert L.rt_attention_validate(ctypes.byref(d)) == _ffi.RT_OK
    d.dtype = _ffi.RT_F32
    assert L.rt_attention_validate(ctypes.byref(d)) == _ffi.RT_ERR_DTYPE_MISMATCH
    d.dtype, d.head_dim = _ffi.RT_F16, 84
    assert L.rt_attention_validate(ctypes.byref(d)) == _ffi.RT_ERR_INVALID_SHAPE      # head_dim % 8
    d.head_dim = 136
    assert L.rt_attention_validate(ctypes.byref(d)) == _ffi.RT_ERR_INVALID_SHAPE      # head_dim <= 128
    d.head_dim = 80
    d.k_strides[2] = 84
    assert L.rt_attention_validate(ctypes.byref(d)) == _ffi.RT_ERR_UNSUPPORTED        # rows off 16-byte alignment
    d.k_strides[2] = 80
    d.causal = 2
    assert L.rt_attention_validate(ctypes.byref(d)) == _ffi.RT_ERR_INVALID_ARG
    assert L.rt_attention_validate(None) == _ffi.RT_ERR_INVALID_ARG
    q = Tensor.from_data(np.zeros((1, 2, 4, 16), np.float16))
    with pytest.raises(OperationError):
        q.attention(Tensor.from_data(np.zeros((1, 3, 4, 16), np.float16)), Tensor.from_data(np.zeros((1, 3, 4, 16), np.float16)))
    with pytest.raises(OperationError):
        q.attention(q, q, kv_len=5)
    # one [q_len, kv_len] mask serves every batch and head; a mask per batch or head is refused, not misapplied
    m = np.zeros((4, 4), np.float32)
    q.attention(q, q, Tensor.from_data(m))
    q.attention(q, q, Tensor.from_data(m.reshape(1, 1, 4, 4)))
    for shape in ((2, 4, 4), (1, 2, 4, 4)):
        with pytest.raises(OperationError, match="per batch or head"):
            q.attention(q, q, Tensor.from_data(np.zeros(shape, np.float32)))
    with pytest.raises(InvariantError):
        Tensor.from_data(np.zeros((1, 2, 4, 16), np.float32)).attention(q, q)


# ---------------------------------------------------------------------------
# GPU
# ---------------------------------------------------------------------------
gpu = pytest.mark.gpu


def run(device, q, k, v, mask=None, **kw):
    T = lambda a: Tensor.from_data(a).to(device)
    return T(q).attention(T(k), T(v), None if mask is None else T(mask), **kw).resolve().to(Device.CPU).storage


@gpu
def test_shapes_and_head_dims(device, oracle):
    rng = np.random.default_rng(10)
    cases = [(1, 32, 512, 512, 80), (2, 3, 64, 64, 64), (1, 4, 100, 100, 96), (1, 2, 257, 130, 128), (3, 2, 1, 77, 80),
             (1, 1, 16, 1, 8), (1, 5, 63, 65, 40), (2, 2, 200, 513, 72), (1, 2, 5, 1500, 64), (1, 1, 1, 1, 8)]
    for i, (B, H, Lq, Lk, D) in enumerate(cases):
        q, k, v = rand_qkv(rng, B, H, Lq, Lk, D)
        got = run(device, q, k, v)
        assert got.shape == q.shape and got.dtype == np.float16
        assert_close(got, oracle.attention(q, k, v), ("phi2 order", cases[i]))
        assert_close(got, oracle.attention(q, k, v, round_scores=True), ("phi3 order", cases[i]))
        assert_close(got, sdpa64(q, k, v), ("torch", cases[i]))


@gpu
def test_causal_and_masks(device, oracle):
    rng = np.random.default_rng(11)
    for i, (B, H, Lq, Lk, D) in enumerate([(1, 4, 128, 128, 80), (1, 2, 70, 70, 64), (2, 2, 33, 200, 96), (1, 3, 1, 300, 80),
                                           (1, 2, 256, 256, 128)]):
        q, k, v = rand_qkv(rng, B, H, Lq, Lk, D)
        got = run(device, q, k, v, causal=True)
        assert_close(got, oracle.attention(q, k, v, causal=True), ("causal", i))
        assert_close(got, sdpa64(q, k, v, causal=True), ("causal torch", i))
        # the same mask as a tensor, F32 and F16 (what the callers pass, phi3/attn.rs:148-151)
        tri = np.triu(np.full((Lq, Lk), -np.inf, np.float32), 1 + Lk - Lq)
        # (not bit for bit: blocks clear of the diagonal fold the scale into the exponent's argument)
        m32, m16 = run(device, q, k, v, mask=tri), run(device, q, k, v, mask=tri.astype(np.float16))
        assert np.array_equal(m32, m16)
        np.testing.assert_allclose(m32.astype(np.float32), got.astype(np.float32), rtol=4e-3, atol=1e-3)
        # an arbitrary additive mask and a scale of its own
        mask = (rng.standard_normal((Lq, Lk)) * 2).astype(np.float32)
        mask[rng.random((Lq, Lk)) < 0.3] = -np.inf
        mask[:, 0] = 0
        assert_close(run(device, q, k, v, mask=mask, scale=0.25), oracle.attention(q, k, v, mask=mask, scale=0.25), ("mask", i))
    # rows with no visible key are NaN, like the unfused sequence; the rest is untouched
    q, k, v = rand_qkv(rng, 1, 2, 40, 90, 64)
    mask = np.zeros((40, 90), np.float32)
    mask[7] = -np.inf
    got, want = run(device, q, k, v, mask=mask), oracle.attention(q, k, v, mask=mask)
    assert np.isnan(got[:, :, 7]).all() and np.array_equal(np.isnan(got), np.isnan(want))
    assert_close(got, want, "masked row")
    # kv_len < q_len with the causal rule: the first q_len - kv_len queries see nothing
    q, k, v = rand_qkv(rng, 1, 1, 12, 8, 32)
    got, want = run(device, q, k, v, causal=True), oracle.attention(q, k, v, causal=True)
    assert np.isnan(got[:, :, :4]).all() and np.array_equal(np.isnan(got), np.isnan(want))
    assert_close(got, want, "short kv")


@gpu
def test_long_key_streams_one_pass(device, oracle):
    """From 1280 keys a launch in one pass (128 workgroups or more, so the keys are not shared out) runs sixteen
    wavefronts over blocks of 128 keys for head_dim up to 96: key counts on and off a block, every masking mode, a late
    dominant key, and head_dim 128, which stays with eight wavefronts."""
    rng = np.random.default_rng(14)
    for i, (B, H, Lq, Lk, D) in enumerate([(1, 64, 128, 1280, 80), (1, 64, 70, 1301, 64), (2, 32, 128, 1535, 96), (1, 128, 64, 1408, 40),
                                           (1, 64, 128, 1300, 128)]):
        q, k, v = rand_qkv(rng, B, H, Lq, Lk, D)
        assert_close(run(device, q, k, v), oracle.attention(q, k, v), ("plain", i))
        got = run(device, q, k, v, causal=True)
        assert_close(got, oracle.attention(q, k, v, causal=True), ("causal", i))
        tri = np.triu(np.full((Lq, Lk), -np.inf, np.float32), 1 + Lk - Lq)
        np.testing.assert_allclose(run(device, q, k, v, mask=tri).astype(np.float32), got.astype(np.float32), rtol=4e-3, atol=1e-3)
        mask = (rng.standard_normal((Lq, Lk)) * 2).astype(np.float32)
        mask[rng.random((Lq, Lk)) < 0.3] = -np.inf
        mask[:, 0] = 0
        assert_close(run(device, q, k, v, mask=mask, scale=0.25), oracle.attention(q, k, v, mask=mask, scale=0.25), ("mask", i))
    q, k, v = rand_qkv(rng, 1, 128, 64, 1400, 64)
    q[..., 0], k[..., 0] = 30, 0
    k[:, :, 1390, 0] = 30                      # key 1390 scores 900 above the rest: it arrives in the last block, fourth part
    got = run(device, q, k, v, scale=1.0)
    assert np.array_equal(got, np.broadcast_to(v[:, :, 1390:1391], q.shape))


@gpu
def test_softmax_extremes(device, oracle):
    """Scores far apart (one key takes everything) and large scores that would overflow exp without
    the running maximum; a change of the maximum late in the key stream rescales what was summed."""
    rng = np.random.default_rng(12)
    q, k, v = rand_qkv(rng, 1, 2, 64, 256, 64)
    q[..., 0], k[..., 0] = 30, 0
    k[:, :, 200, 0] = 30                       # key 200 scores 900 above the rest: it arrives in the fourth block
    got = run(device, q, k, v, scale=1.0)
    assert np.array_equal(got, np.broadcast_to(v[:, :, 200:201], q.shape))
    assert_close(got, oracle.attention(q, k, v, scale=1.0), "dominant key")
    q, k, v = rand_qkv(rng, 1, 2, 48, 300, 80, spread=6.0)   # scores of +-300 at scale 1
    assert_close(run(device, q, k, v, scale=1.0), oracle.attention(q, k, v, scale=1.0), "large scores")
    # identical keys: the mean of the values
    q, k, v = rand_qkv(rng, 1, 1, 32, 128, 64)
    k[:] = k[:, :, :1]
    np.testing.assert_allclose(run(device, q, k, v).astype(np.float32),
                               np.broadcast_to(v.astype(np.float32).mean(axis=2, keepdims=True), q.shape), rtol=2e-3, atol=2e-3)


@gpu
def test_key_value_cache_in_place_and_merged_heads(device, oracle):
    """k and v may be the first kv_len rows of a longer cache (the reference's Cache operator would copy
    them into a fresh tensor, ops/cache.rs:71-96); merge_heads writes [batch, q_len, heads * head_dim],
    the callers' permute(0, 2, 1, 3) + view (phi3/attn.rs:157-158)."""
    rng = np.random.default_rng(13)
    B, H, cap, D = 2, 4, 160, 80
    kc = rng.standard_normal((B, H, cap, D)).astype(np.float16)
    vc = rng.standard_normal((B, H, cap, D)).astype(np.float16)
    K, V = Tensor.from_data(kc).to(device), Tensor.from_data(vc).to(device)
    for Lq, kv_len in [(1, 1), (1, 77), (5, 130), (33, 160)]:
        q = rng.standard_normal((B, H, Lq, D)).astype(np.float16)
        want = oracle.attention(q, kc[:, :, :kv_len], vc[:, :, :kv_len], causal=True)
        Q = Tensor.from_data(q).to(device)
        got = Q.attention(K, V, causal=True, kv_len=kv_len).resolve().to(Device.CPU).storage
        assert_close(got, want, ("cache", Lq, kv_len))
        merged = Q.attention(K, V, causal=True, kv_len=kv_len, merge_heads=True).resolve().to(Device.CPU).storage
        assert merged.shape == (B, Lq, H * D)
        assert np.array_equal(merged, got.transpose(0, 2, 1, 3).reshape(B, Lq, H * D))
    # rows of the cache past kv_len are never read into the result: poison them
    kc[:, :, 100:], vc[:, :, 100:] = np.nan, np.nan
    K, V = Tensor.from_data(kc).to(device), Tensor.from_data(vc).to(device)
    q = rng.standard_normal((B, H, 3, D)).astype(np.float16)
    got = Tensor.from_data(q).to(device).attention(K, V, kv_len=100).resolve().to(Device.CPU).storage
    assert not np.isnan(got).any()
    assert_close(got, oracle.attention(q, kc[:, :, :100], vc[:, :, :100]), "poisoned tail")


@gpu
def test_few_queries_many_keys_share_the_keys_among_workgroups(device, oracle):
    """A decode-shaped launch (few query blocks, a long cache) splits the keys of a head over several
    workgroups when given a workspace, and merges the partial results in a second kernel: the same
    answer as the single pass (up to the order of the f32 sums) and as the oracle."""
    rng = np.random.default_rng(15)
    L = _ffi.lib()
    for (B, H, Lq, Lk, D, causal) in [(1, 32, 1, 2048, 80, True), (1, 8, 1, 300, 64, True), (2, 4, 5, 777, 96, True),
                                      (1, 2, 64, 1024, 128, False), (1, 1, 70, 513, 80, True), (1, 3, 16, 256, 72, False),
                                      (1, 2, 33, 257, 40, True)]:
        q, k, v = rand_qkv(rng, B, H, Lq, Lk, D)
        T = lambda a: Tensor.from_data(a).to(device)
        node = T(q).attention(T(k), T(v), causal=causal)
        need = ctypes.c_uint64()
        assert L.rt_attention_workspace_bytes(ctypes.byref(node.op.desc), ctypes.byref(need)) == _ffi.RT_OK
        assert need.value > 0, (B, H, Lq, Lk)                      # these shapes do split
        split = node.resolve().to(Device.CPU).storage
        single_node = T(q).attention(T(k), T(v), causal=causal)
        single_node.op.use_workspace = False
        single = single_node.resolve().to(Device.CPU).storage
        np.testing.assert_allclose(split.astype(np.float32), single.astype(np.float32), rtol=4e-3, atol=1e-3, err_msg=str((B, H, Lq, Lk, D)))
        assert_close(split, oracle.attention(q, k, v, causal=causal), ("split", B, H, Lq, Lk, D))
    # a prefill-shaped launch fills the device by itself: no workspace asked for
    q, k, v = rand_qkv(rng, 1, 32, 512, 512, 80)
    node = Tensor.from_data(q).to(device).attention(Tensor.from_data(k).to(device), Tensor.from_data(v).to(device))
    need = ctypes.c_uint64(1)
    assert L.rt_attention_workspace_bytes(ctypes.byref(node.op.desc), ctypes.byref(need)) == _ffi.RT_OK and need.value == 0
    # rows with no visible key stay NaN through the merge; a dominant key in the last split takes everything
    q, k, v = rand_qkv(rng, 1, 2, 12, 520, 64)
    mask = np.zeros((12, 520), np.float32)
    mask[3] = -np.inf
    got = run(device, q, k, v, mask=mask)
    want = oracle.attention(q, k, v, mask=mask)
    assert np.isnan(got[:, :, 3]).all() and np.array_equal(np.isnan(got), np.isnan(want))
    assert_close(got, want, "masked row through the merge")
    q[..., 0], k[..., 0] = 30, 0
    k[:, :, 515, 0] = 30
    assert np.array_equal(run(device, q, k, v, scale=1.0), np.broadcast_to(v[:, :, 515:516], q.shape))


@gpu
def test_equals_the_three_operator_sequence(device, oracle):
    """The fused kernel against this library's own matmul -> softmax -> matmul (each checked on its own
    elsewhere), composed as phi2/attn.rs:138-152 does."""
    rng = np.random.default_rng(14)
    B, H, L, D = 1, 8, 192, 80
    q, k, v = rand_qkv(rng, B, H, L, L, D)
    scale = np.float16(1 / np.sqrt(D))
    Q, K, V = (Tensor.from_data(a).to(device) for a in ((q.astype(np.float32) * np.float32(scale)).astype(np.float16), k, v))
    scores = Q.matmul(K, False, True).full().softmax(3).half()
    three = scores.matmul(V, False, False).resolve().to(Device.CPU).storage
    fused = Q.attention(K, V, scale=1.0).resolve().to(Device.CPU).storage
    assert_close(fused, three, "fused vs three operators")


@gpu
def test_one_query_against_a_long_cache_streams_the_keys(device, oracle):
    """A decode step (one query row, at least 256 cached keys, no mask tensor, a workspace) takes the streaming
    kernel: every head dimension it serves (idle lanes past head_dim / 8), key counts off the 128-key workgroups
    and off the 16-key loads, the cache read in place with rows past kv_len poisoned, heads merged on the way
    out, a dominant key in the last workgroup's share, and the causal flag, which hides nothing from one query."""
    rng = np.random.default_rng(21)
    L = _ffi.lib()
    for (B, H, kv_len, cap, D) in [(1, 32, 1024, 2048, 80), (2, 3, 257, 300, 8), (1, 2, 1000, 1000, 128), (1, 5, 384, 400, 64),
                                   (1, 1, 256, 256, 96), (3, 2, 2049, 2100, 40), (1, 2, 511, 600, 72)]:
        q = rng.standard_normal((B, H, 1, D)).astype(np.float16)
        kc = rng.standard_normal((B, H, cap, D)).astype(np.float16)
        vc = rng.standard_normal((B, H, cap, D)).astype(np.float16)
        want = oracle.attention(q, kc[:, :, :kv_len], vc[:, :, :kv_len])
        kc[:, :, kv_len:], vc[:, :, kv_len:] = np.nan, np.nan   # never read
        Q, K, V = (Tensor.from_data(a).to(device) for a in (q, kc, vc))
        node = Q.attention(K, V, causal=True, kv_len=kv_len)
        need = ctypes.c_uint64()
        assert L.rt_attention_workspace_bytes(ctypes.byref(node.op.desc), ctypes.byref(need)) == _ffi.RT_OK and need.value > 0
        got = node.resolve().to(Device.CPU).storage
        assert not np.isnan(got).any(), (B, H, kv_len, D)
        assert_close(got, want, ("decode", B, H, kv_len, D))
        single = Q.attention(K, V, kv_len=kv_len)
        single.op.use_workspace = False                        # the tiled kernel, one pass
        np.testing.assert_allclose(got.astype(np.float32), single.resolve().to(Device.CPU).storage.astype(np.float32),
                                   rtol=4e-3, atol=1e-3, err_msg=str((B, H, kv_len, D)))
        merged = Q.attention(K, V, kv_len=kv_len, merge_heads=True).resolve().to(Device.CPU).storage
        assert np.array_equal(merged, got.transpose(0, 2, 1, 3).reshape(B, 1, H * D))
    # a dominant key in the last share takes everything; keys that score -inf (q . k overflows to -inf) weigh nothing
    q, k, v = rand_qkv(rng, 1, 2, 1, 700, 64)
    q[..., 0], k[..., 0] = 30, 0
    k[:, :, 699, 0] = 30
    assert np.array_equal(run(device, q, k, v, scale=1.0), v[:, :, 699:700])
