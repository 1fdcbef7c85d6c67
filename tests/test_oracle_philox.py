"""Pins the oracle's Philox4x32-10 and its stream convention.

Known answers: the Random123 distribution's kat_vectors for philox4x32 with
10 rounds (counter, key -> output)."""
import numpy as np

from oracle import binding as orc

KAT = [
    ((0, 0, 0, 0), (0, 0),
     (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    ((0xffffffff,) * 4, (0xffffffff,) * 2,
     (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
     (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
]


def test_philox_known_answers():
    for ctr, key, want in KAT:
        got = orc.philox4x32_10(ctr, key)
        assert tuple(int(v) for v in got) == want


def test_stream_layout():
    # key = seed + call_id * golden (mod 2^64); counter = (draw lo, draw hi, pos lo, pos hi)
    seed, call_id, pos, draw = 7777, 3, (5 << 32) | 9, (2 << 32) | 11
    k = (seed + call_id * 0x9E3779B97F4A7C15) & (2**64 - 1)
    want = orc.philox4x32_10((11, 2, 9, 5), (k & 0xffffffff, k >> 32))
    got = orc.stream_words(seed, call_id, pos, draw)
    assert np.array_equal(got, want)


def test_stream_words_are_uniform_bits():
    # 64 draws x 128 bits: every bit position is set about half of the time
    bits = np.zeros(128)
    n = 4096
    for d in range(n):
        w = orc.stream_words(1, 0, 0, d)
        bits += np.unpackbits(w.view(np.uint8))
    assert np.all(np.abs(bits / n - 0.5) < 0.05)
