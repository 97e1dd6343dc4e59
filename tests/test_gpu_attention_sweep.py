"""A seeded sweep of the fused attention over the places where its kernel changes what it does, against the CPU oracle.

The reference runs attention as matmul(q, k^T) * scale (+ mask) -> softmax -> cast -> matmul(p, v)
(crates/ratchet-models/src/phi2/attn.rs:138-152, phi3/attn.rs:142-158, whisper/mha.rs:105-124); the oracle restates
that sequence.  The device side switches on: head_dim (kernels built for 64 / 80 / 96 / 128, one per padded size for the
rest), key blocks of 64 or 128 (one-pass launches from 1280 keys), blocks that cross the end of the keys or the causal
diagonal against those that do not, grids that divide by eight (renumbered so that a head's query blocks share an XCD)
against those that do not, launches that share the keys of a query block among workgroups (with the workspace) against
one pass (without), one query against a long cache (a kernel of its own), and caches read in place through a row
count smaller than their capacity.  Tolerance as in test_attention.py: |y - r| <= 2e-3 + 2e-2 |r|.
"""
import numpy as np
import pytest

from ratchet_amd import Device, Tensor

pytestmark = pytest.mark.gpu

ATOL, RTOL = 2e-3, 2e-2
HEAD_DIMS = [8, 40, 64, 64, 72, 80, 80, 88, 96, 96, 104, 128, 128]
Q_LENS = [1, 2, 15, 16, 17, 63, 64, 65, 100, 128, 129, 200, 256, 300]
KV_LENS = [1, 31, 32, 33, 63, 64, 65, 127, 128, 129, 191, 192, 200, 255, 256, 257, 320, 511, 512, 640, 700, 1279, 1280, 1281, 1344, 1500]
STACKS = [(1, 1), (1, 2), (1, 3), (2, 2), (1, 5), (1, 8), (2, 4), (1, 16), (3, 3), (1, 32), (2, 16), (1, 64)]


def assert_close(got, want, what):
    got, want = got.astype(np.float64), want.astype(np.float64)
    bad = ~((np.abs(got - want) <= ATOL + RTOL * np.abs(want)) | (np.isnan(got) & np.isnan(want)))
    assert not bad.any(), (what, int(bad.sum()), float(np.nanmax(np.abs(got - want))))


def cases(seed, n, max_work):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        (B, H), Lq, Lk, D = STACKS[rng.integers(len(STACKS))], int(rng.choice(Q_LENS)), int(rng.choice(KV_LENS)), int(rng.choice(HEAD_DIMS))
        if B * H * Lq * Lk * D > max_work:
            continue
        out.append((B, H, Lq, Lk, D, int(rng.integers(0, 3)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2))))
    return out


def test_attention_sweep(device, oracle):
    rng = np.random.default_rng(77)
    for case in cases(2024, 400, 1e9):
        B, H, Lq, Lk, D, mode, in_cache, workspace = case
        q = rng.standard_normal((B, H, Lq, D)).astype(np.float16)
        cap = Lk + int(rng.integers(1, 40)) if in_cache else Lk      # rows of the cache past kv_len are poisoned, never read
        kc = rng.standard_normal((B, H, cap, D)).astype(np.float16)
        vc = rng.standard_normal((B, H, cap, D)).astype(np.float16)
        k, v = kc[:, :, :Lk].copy(), vc[:, :, :Lk].copy()
        kc[:, :, Lk:], vc[:, :, Lk:] = np.nan, np.nan
        mask, kw = None, {}
        if mode == 1:
            kw["causal"] = True
        elif mode == 2:
            mask = (rng.standard_normal((Lq, Lk)) * 2).astype(np.float32)
            mask[rng.random((Lq, Lk)) < 0.3] = -np.inf
            mask[:, 0] = 0                                           # every row sees a key
            kw["scale"] = 0.25
        want = oracle.attention(q, k, v, mask=mask, **kw)
        T = lambda a: Tensor.from_data(a).to(device)
        node = T(q).attention(T(kc), T(vc), None if mask is None else T(mask), kv_len=Lk if in_cache else None, **kw)
        node.op.use_workspace = workspace
        got = node.resolve().to(Device.CPU).storage
        assert got.shape == q.shape and got.dtype == np.float16, case
        assert_close(got, want, case)
