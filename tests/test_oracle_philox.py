"""Pins the oracle's Philox4x32-10 and its stream convention.

Known answers: the Random123 distribution's kat_vectors for philox4x32 with
10 rounds (counter, key -> output)."""
import numpy as np

from oracle import binding as orc

from tests.conftest import golden

KAT = [(tuple(int(w, 16) for w in v["ctr"]), tuple(int(w, 16) for w in v["key"]),
        tuple(int(w, 16) for w in v["out"]))
       for v in golden()["philox4x32_10_kat"]["vectors"]]


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
