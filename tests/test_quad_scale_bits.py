"""Bit arithmetic of the quad-shared scale loads (candy_amd/csrc/units.h UnitQ6KQuad, formats_more.h UnitQ3KQuad),
restated with Python integers and checked against the plain per-byte definitions for every half, unit and group.

The kernels let the four lanes of a quad load one 32-bit word each of a block's scale bytes and pick a unit's four
scales with byte permutes (v_perm_b32) and shifts; a wrong selector or shift would still produce plausible numbers,
so the picking is pinned here without a GPU."""
import numpy as np


def perm(hi, lo, sel):
    """v_perm_b32: result byte i = byte sel[i] of the eight bytes {lo[0..3], hi[0..3]} (selectors 0..7 only)."""
    src = [(lo >> (8 * i)) & 0xFF for i in range(4)] + [(hi >> (8 * i)) & 0xFF for i in range(4)]
    return sum(src[(sel >> (8 * i)) & 0xFF] << (8 * i) for i in range(4))


def word(b, i):
    return int.from_bytes(bytes(b[i:i + 4]), "little")


def test_q6k_scales_from_two_words():
    # quantized.cu:2367-2389: unit (ip, j) uses scales[8 ip + (j >> 1) + {0, 2, 4, 6}]
    rng = np.random.default_rng(6)
    for _ in range(50):
        scales = rng.integers(0, 256, 16).tolist()
        for ip in range(2):
            lo, hi = word(scales, 8 * ip), word(scales, 8 * ip + 4)  # what lanes 0 and 1 of the quad load
            for j in range(4):
                got = perm(hi, lo, 0x07050301) if (j & 2) else perm(hi, lo, 0x06040200)
                want = sum(scales[8 * ip + (j >> 1) + 2 * k] << (8 * k) for k in range(4))
                assert got == want, (ip, j)


def q3k_scale6(sc, i):
    # 6-bit scale of 16-value group i: low nibble in bytes 0..7, high bit pair in bytes 8..11
    return ((sc[i & 7] >> (4 * (i >> 3))) & 0xF) | (((sc[8 + (i & 3)] >> (2 * (i >> 2))) & 3) << 4)


def test_q3k_scales_from_three_words():
    # unit (n, j) uses the groups 8 n + 2 k + (j >> 1), k = 0 .. 3
    rng = np.random.default_rng(3)
    for _ in range(50):
        sc = rng.integers(0, 256, 12).tolist()
        w0, w1, w2 = word(sc, 0), word(sc, 4), word(sc, 8)  # lanes 0, 1 and 2 of the quad
        for n in range(2):
            for j in range(4):
                odd = (j & 2) != 0
                lo4 = (perm(w1, w0, 0x07050301 if odd else 0x06040200) >> (4 * n)) & 0x0F0F0F0F
                t = perm(w2, w2, 0x03010301 if odd else 0x02000200)
                hi4 = ((t >> (4 * n)) & 0x00000303) | ((t >> (4 * n + 2)) & 0x03030000)
                got = lo4 | (hi4 << 4)
                want = sum(q3k_scale6(sc, 8 * n + 2 * k + (j >> 1)) << (8 * k) for k in range(4))
                assert got == want, (n, j)


def test_q5k_and_q4k_words_of_a_quad():
    # Q5_K: lane j of a quad loads words 3 j .. 3 j + 2 of the block's first 48 bytes; the dot takes header word i from
    # lane i // 3, slot i % 3 (i = 0 .. 3) and fifth-bit word i from lane (4 + i) // 3, slot (4 + i) % 3 (i = 0 .. 7).
    held = {(lane, slot): 3 * lane + slot for lane in range(4) for slot in range(3)}
    hdr_from = [(0, 0), (0, 1), (0, 2), (1, 0)]
    h_from = [(1, 1), (1, 2), (2, 0), (2, 1), (2, 2), (3, 0), (3, 1), (3, 2)]
    assert [held[x] for x in hdr_from] == [0, 1, 2, 3]
    assert [held[x] for x in h_from] == list(range(4, 12))
    # Q4_K: lane j loads header word j; quad_perm [i, i, i, i] has the control byte i * 0x55
    for i in range(4):
        ctrl = i * 0x55
        assert [(ctrl >> (2 * lane)) & 3 for lane in range(4)] == [i] * 4
