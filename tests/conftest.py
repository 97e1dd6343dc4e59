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


# A second block with the same header bytes' layout (d = 0.5 = 0x3800, dmin = 0.25 = 0x3400, the same twelve scale
# bytes) whose 32 byte positions per chunk all carry different (low, high) nibble pairs, and whose elements 16..31
# do not repeat elements 0..15: exchanging the two halves of a sub-block, or two bytes of a chunk, changes the
# expected values.  Byte l of chunk c: low nibble (5 l + 3 c + 7 (l // 16)) % 16, high nibble
# (11 l + c + 3 (l // 16) + 1) % 16; the lists below are those nibbles written out.
Q4K_KAT2_HEX = (
    "0038" "0034"
    "4182C3C4" "4586C7C8" "516273FC"
    # chunk 0
    "10C57A2FD4893EE3984DF2A75C01B66B" "47FCA1560BB0651ACF7429DE8338ED92"
    # chunk 1
    "23D88D32E79C41F6AB5005BA6F14C97E" "5A0FB4691EC3782DD2873CE1964BF0A5"
    # chunk 2
    "36EB9045FAAF5409BE6318CD7227DC81" "6D12C77C21D68B30E59A4FF4A95E03B8"
    # chunk 3
    "49FEA3580DB2671CC1762BD0853AEF94" "7025DA8F34E99E43F8AD5207BC6116CB"
)
# per sub-block: (d * sc, dmin * mn, the 32 nibbles)
Q4K_KAT2_SUBBLOCKS = [
    (0.5, 1.25, [0, 5, 10, 15, 4, 9, 14, 3, 8, 13, 2, 7, 12, 1, 6, 11, 7, 12, 1, 6, 11, 0, 5, 10, 15, 4, 9, 14, 3, 8, 13, 2]),
    (1.0, 1.5, [1, 12, 7, 2, 13, 8, 3, 14, 9, 4, 15, 10, 5, 0, 11, 6, 4, 15, 10, 5, 0, 11, 6, 1, 12, 7, 2, 13, 8, 3, 14, 9]),
    (1.5, 1.75, [3, 8, 13, 2, 7, 12, 1, 6, 11, 0, 5, 10, 15, 4, 9, 14, 10, 15, 4, 9, 14, 3, 8, 13, 2, 7, 12, 1, 6, 11, 0, 5]),
    (2.0, 2.0, [2, 13, 8, 3, 14, 9, 4, 15, 10, 5, 0, 11, 6, 1, 12, 7, 5, 0, 11, 6, 1, 12, 7, 2, 13, 8, 3, 14, 9, 4, 15, 10]),
    (8.5, 5.25, [6, 11, 0, 5, 10, 15, 4, 9, 14, 3, 8, 13, 2, 7, 12, 1, 13, 2, 7, 12, 1, 6, 11, 0, 5, 10, 15, 4, 9, 14, 3, 8]),
    (17.0, 9.5, [3, 14, 9, 4, 15, 10, 5, 0, 11, 6, 1, 12, 7, 2, 13, 8, 6, 1, 12, 7, 2, 13, 8, 3, 14, 9, 4, 15, 10, 5, 0, 11]),
    (25.5, 13.75, [9, 14, 3, 8, 13, 2, 7, 12, 1, 6, 11, 0, 5, 10, 15, 4, 0, 5, 10, 15, 4, 9, 14, 3, 8, 13, 2, 7, 12, 1, 6, 11]),
    (30.0, 15.75, [4, 15, 10, 5, 0, 11, 6, 1, 12, 7, 2, 13, 8, 3, 14, 9, 7, 2, 13, 8, 3, 14, 9, 4, 15, 10, 5, 0, 11, 6, 1, 12]),
]
# a few values written out in full: w[1] = 0.5*5 - 1.25, w[16] = 0.5*7 - 1.25, w[48] = 1.0*4 - 1.5,
# w[143] = 8.5*1 - 5.25, w[144] = 8.5*13 - 5.25, w[255] = 30*12 - 15.75
Q4K_KAT2_SPOT = {1: 1.25, 16: 2.25, 48: 2.5, 143: 3.25, 144: 105.25, 255: 344.25}


class _Q4kKat(tuple):
    """(block bytes, dequantized values, (sc, mn) pairs) with the header values and the 256 nibbles as attributes."""
    def __new__(cls, blk, want, scmn, d, dmin, nibbles):
        self = super().__new__(cls, (blk, want, scmn))
        self.d, self.dmin, self.nibbles = d, dmin, nibbles
        return self


@pytest.fixture(scope="session", params=["rotated-nibble-runs", "32-distinct-positions"])
def q4k_kat(request):
    """(144 block bytes as uint8, the 256 dequantized values as float32, the 8 (sc, mn) pairs), for each of the two
    hand-typed blocks."""
    import numpy as np
    scmn = [(1, 5), (2, 6), (3, 7), (4, 8), (17, 21), (34, 38), (51, 55), (60, 63)]
    if request.param == "32-distinct-positions":
        blk = np.frombuffer(bytes.fromhex(Q4K_KAT2_HEX), dtype=np.uint8).copy()
        assert blk.size == 144
        want = np.empty(256, dtype=np.float64)
        for j, (dsc, dm, nib) in enumerate(Q4K_KAT2_SUBBLOCKS):
            assert len(nib) == 32 and nib[:16] != nib[16:]
            want[32 * j: 32 * j + 32] = dsc * np.array(nib, dtype=np.float64) - dm
        for i, v in Q4K_KAT2_SPOT.items():
            assert want[i] == v
        return _Q4kKat(blk, want.astype(np.float32), scmn, 0.5, 0.25, np.concatenate([np.array(n) for _, _, n in Q4K_KAT2_SUBBLOCKS]))
    blk = np.frombuffer(bytes.fromhex(Q4K_KAT_HEX), dtype=np.uint8).copy()
    assert blk.size == 144
    want = np.empty(256, dtype=np.float64)
    for j, (dsc, dm, nib) in enumerate(Q4K_KAT_SUBBLOCKS):
        want[32 * j: 32 * j + 32] = dsc * np.array(nib + nib, dtype=np.float64) - dm
    for i, v in Q4K_KAT_SPOT.items():
        assert want[i] == v
    return _Q4kKat(blk, want.astype(np.float32), scmn, 0.375, 0.625, np.concatenate([np.array(n + n) for _, _, n in Q4K_KAT_SUBBLOCKS]))
