"""Pins the oracle's Philox4x32-10 to the Random123 known-answer vectors."""
import numpy as np

KAT = [
    ([0, 0, 0, 0], [0, 0], [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]),
    ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
    ([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0],
     [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]),
]


def test_philox_known_answers(orc):
    for ctr, key, want in KAT:
        got = orc.philox(ctr, key)
        assert [int(x) for x in got] == want


def test_philox_counter_sensitivity(orc):
    # every counter word and key word changes the output (a dropped word would not)
    base = orc.philox([1, 2, 3, 4], [5, 6])
    for i in range(4):
        c = [1, 2, 3, 4]
        c[i] += 1
        assert not np.array_equal(orc.philox(c, [5, 6]), base)
    for i in range(2):
        k = [5, 6]
        k[i] += 1
        assert not np.array_equal(orc.philox([1, 2, 3, 4], k), base)
