import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O
    O.lib()
    return O


@pytest.fixture(scope="session")
def device():
    """Device::request_device(DeviceRequest::GPU); GPU tests fail loudly without it.  Every GPU test runs in
    checked mode: outputs are NaN-filled before the operator that writes them is enqueued."""
    import ratchet_amd.tensor as mirror
    from ratchet_amd import Device, DeviceRequest
    mirror.POISON_OUTPUTS = True
    return Device.request_device(DeviceRequest.GPU)


# ---------------------------------------------------------------------------
# Q4_K known-answer super-block.
#
# The 144 bytes are typed by hand from the layout text of ggml's block_q4_K
# (k_quants.rs:94-103 holds the same struct): f16 d, f16 dmin, 12 bytes of 6-bit
# scales / mins, 128 bytes of nibbles.  No packer of this repository produced them, and
# the expected values below were worked out by hand from ggml's published
# get_scale_min_k4 / dequantize_row_q4_K, so a mistake shared by this build's packer and
# unpacker would show here.  The reference itself holds no vector for this format (its
# Q4_K fixture is a missing blob), so the format stays unpinned BY THE REFERENCE.
#
#   d    = 0.375 = 0x3600 -> bytes 00 36        dmin = 0.625 = 0x3900 -> bytes 00 39
#   sub-block        j : 0   1   2   3   4   5   6   7
#   6-bit scale  sc[j] : 1   2   3   4  17  34  51  60
#   6-bit min    mn[j] : 5   6   7   8  21  38  55  63
#   scales[0..3]  = sc[j]   | (sc[j+4] >> 4) << 6 : 01|40=41  02|80=82  03|C0=C3  04|C0=C4
#   scales[4..7]  = mn[j]   | (mn[j+4] >> 4) << 6 : 05|40=45  06|80=86  07|C0=C7  08|C0=C8
#   scales[8..11] = sc[j+4] & 15 | (mn[j+4] & 15) << 4 : 1|50=51  2|60=62  3|70=73  C|F0=FC
#   qs: chunk c (bytes 32c .. 32c+31), byte l: low nibble (l + c) % 16 -> sub-block 2c, element l
#                                             high nibble (15 - l - c) % 16 -> sub-block 2c+1, element l
# ---------------------------------------------------------------------------
Q4K_KAT_HEX = (
    "0036" "0039"
    "4182C3C4" "4586C7C8" "516273FC"
    # chunk 0
    "F0E1D2C3B4A5968778695A4B3C2D1E0F" "F0E1D2C3B4A5968778695A4B3C2D1E0F"
    # chunk 1
    "E1D2C3B4A5968778695A4B3C2D1E0FF0" "E1D2C3B4A5968778695A4B3C2D1E0FF0"
    # chunk 2
    "D2C3B4A5968778695A4B3C2D1E0FF0E1" "D2C3B4A5968778695A4B3C2D1E0FF0E1"
    # chunk 3
    "C3B4A5968778695A4B3C2D1E0FF0E1D2" "C3B4A5968778695A4B3C2D1E0FF0E1D2"
)
# per sub-block: (d * sc, dmin * mn, first 16 nibbles; elements 16..31 repeat them)
Q4K_KAT_SUBBLOCKS = [
    (0.375, 3.125, [0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15]),
    (0.75, 3.75, [15, 14, 13, 12, 11, 10, 9, 8, 7, 6, 5, 4, 3, 2, 1, 0]),
    (1.125, 4.375, [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 0]),
    (1.5, 5.0, [14, 13, 12, 11, 10, 9, 8, 7, 6, 5, 4, 3, 2, 1, 0, 15]),
    (6.375, 13.125, [2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 0, 1]),
    (12.75, 23.75, [13, 12, 11, 10, 9, 8, 7, 6, 5, 4, 3, 2, 1, 0, 15, 14]),
    (19.125, 34.375, [3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 0, 1, 2]),
    (22.5, 39.375, [12, 11, 10, 9, 8, 7, 6, 5, 4, 3, 2, 1, 0, 15, 14, 13]),
]
# a few values written out in full: w[0] = 0.375*0 - 3.125, w[47] = 0.75*0 - 3.75,
# w[128] = 6.375*2 - 13.125, w[191] = 12.75*14 - 23.75, w[224] = 22.5*12 - 39.375, w[255] = 22.5*13 - 39.375
Q4K_KAT_SPOT = {0: -3.125, 47: -3.75, 128: -0.375, 191: 154.75, 224: 230.625, 255: 253.125}


@pytest.fixture(scope="session")
def q4k_kat():
    """(144 block bytes as uint8, the 256 dequantized values as float32, the 8 (sc, mn) pairs)."""
    import numpy as np
    blk = np.frombuffer(bytes.fromhex(Q4K_KAT_HEX), dtype=np.uint8).copy()
    assert blk.size == 144
    want = np.empty(256, dtype=np.float64)
    for j, (dsc, dm, nib) in enumerate(Q4K_KAT_SUBBLOCKS):
        want[32 * j: 32 * j + 32] = dsc * np.array(nib + nib, dtype=np.float64) - dm
    for i, v in Q4K_KAT_SPOT.items():
        assert want[i] == v
    scmn = [(1, 5), (2, 6), (3, 7), (4, 8), (17, 21), (34, 38), (51, 55), (60, 63)]
    return blk, want.astype(np.float32), scmn
