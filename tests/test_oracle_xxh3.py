"""The numpy restatement of XXH3-128 against the ``xxhash`` package the reference calls (slime/utils/disk_delta.py:40-44)."""

import numpy as np
import pytest

from oracle import xxh3_ref as X

xxhash = pytest.importorskip("xxhash")


def _data(n, seed):
    return np.random.default_rng(seed).integers(0, 256, n, dtype=np.uint8)


@pytest.mark.parametrize("n", [241, 255, 256, 257, 304, 305, 1023, 1024, 1025, 1087, 1088, 1089, 2047, 2048, 2049, 3000,
                               4096, 16384, 16385, 65536 + 63, 65536 + 64, 65536 + 65, 1 << 20, (1 << 20) + 2])
def test_against_the_library_at_every_boundary(n):
    d = _data(n, n)
    assert X.hexdigest(d) == xxhash.xxh3_128(d.tobytes()).hexdigest()
    low, high = X.xxh3_128(d)
    assert (high << 64) | low == xxhash.xxh3_128(d.tobytes()).intdigest()


def test_special_contents_and_streaming_equivalence():
    for d in (np.zeros(5000, np.uint8), np.full(5000, 255, np.uint8), np.arange(70000, dtype=np.uint32).view(np.uint8)):
        assert X.hexdigest(d) == xxhash.xxh3_128(d.tobytes()).hexdigest()
    # the reference feeds the hasher with one update(); pieces give the same digest
    d = _data(10000, 3)
    h = xxhash.xxh3_128()
    for i in range(0, d.size, 777):
        h.update(d[i:i + 777].tobytes())
    assert h.hexdigest() == X.hexdigest(d)


def test_block_sums_are_order_free_and_the_chain_is_not():
    d = _data(8 * 1024 + 1, 5)
    s = X.block_sums(d, 8)
    # summing the stripes of a block in any order gives the same block sum (what lets a GPU reduce them across lanes)
    words = np.frombuffer(d[:1024].tobytes(), dtype="<u8").reshape(16, 8)
    keys = np.stack([X.secret64(8 * k) for k in range(16)])
    with np.errstate(over="ignore"):
        shuffled = X.stripe_terms(words, keys)[np.random.default_rng(0).permutation(16)].sum(axis=0, dtype=np.uint64)
    assert np.array_equal(shuffled, s[0])
    assert not np.array_equal(X.chain(s), X.chain(s[::-1]))


def test_short_forms_every_length():
    for n in range(0, 241):
        for seed in (n, n + 1000):
            d = _data(n, seed)
            assert X.hexdigest(d) == xxhash.xxh3_128(d.tobytes()).hexdigest(), n
    for n in (1, 3, 8, 16, 17, 128, 129, 240):
        for fill in (0, 255):
            d = np.full(n, fill, np.uint8)
            assert X.hexdigest(d) == xxhash.xxh3_128(d.tobytes()).hexdigest(), (n, fill)
