"""Pins oracle/philox.py: the Philox4x32-10 restatement against the
known-answer vectors of the Random123 distribution (`kat_vectors`, entries
`philox4x32 10`), and the two position-based masks against direct calls."""
import numpy as np

from oracle import philox


def test_philox4x32_10_known_answers():
    kat = [
        ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
        ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
        ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
         (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
    ]
    for counter, key, want in kat:
        got = philox.philox4x32_10(counter, key).reshape(-1)
        assert [int(x) for x in got] == list(want)


def test_vectorised_call_equals_one_counter_at_a_time():
    rng = np.random.default_rng(5)
    c = rng.integers(0, 2 ** 32, size=(7, 4), dtype=np.uint64)
    key = (0x12345678, 0x9ABCDEF0)
    all_at_once = philox.philox4x32_10((c[:, 0], c[:, 1], c[:, 2], c[:, 3]), key)
    for i in range(7):
        one = philox.philox4x32_10(tuple(int(x) for x in c[i]), key).reshape(-1)
        assert (all_at_once[i] == one).all()


def test_dropkey_mask_is_the_documented_function_of_position():
    seed, offset, p = 0x1234567887654321, (5 << 32) | 12, 0.3
    rows = np.array([0, 3, 70000, 2 ** 32 - 1], dtype=np.uint64)
    m = philox.dropkey_mask(rows, 11, p, seed, offset)
    assert m.shape == (4, 11)
    for a, i in enumerate(rows):
        for j in range(11):
            w = philox.philox4x32_10((j // 4, int(i), 12, 5), (0x87654321, 0x12345678)).reshape(-1)[j % 4]
            u = np.float32(int(w) >> 8) * np.float32(2.0 ** -24)
            assert bool(m[a, j]) == bool(u < np.float32(p))


def test_masks_have_the_right_rate_and_are_offset_dependent():
    m = philox.dropkey_mask(np.arange(512), 512, 0.25, seed=7, offset=0)
    n = m.size
    assert abs(m.mean() - 0.25) < 5 * (0.25 * 0.75 / n) ** 0.5
    m2 = philox.dropkey_mask(np.arange(512), 512, 0.25, seed=7, offset=4)
    assert 0.3 < (m != m2).mean() < 0.45          # independent masks differ at rate 2 p (1 - p) = 0.375
    k = philox.dropout_keep(100003, 0.1, seed=9, offset=8)
    assert k.shape == (100003,) and abs((~k).mean() - 0.1) < 5 * (0.09 / 100003) ** 0.5
    assert philox.dropout_keep(10, 0.0, 1, 0).all() and not philox.dropout_keep(10, 1.0, 1, 0).any()
