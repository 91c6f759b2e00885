"""Pins the delta part of the oracle: the numpy restatement against closed forms, an independent bytewise
adler32, and the apply round trip."""

import zlib

import numpy as np
import pytest

from oracle import delta_ref as D


def _pair(n, density, seed):
    rng = np.random.default_rng(seed)
    old = rng.integers(0, 256, n, dtype=np.uint8)
    new = old.copy()
    idx = rng.random(n) < density
    new[idx] = rng.integers(0, 256, int(idx.sum()), dtype=np.uint8)     # some draws equal the old byte: unchanged
    return new, old


def test_adler32_known_answers_and_bytewise_witness():
    assert D.adler32_ref(np.zeros(0, np.uint8)) == "00000001"
    assert D.adler32_ref(np.frombuffer(b"Wikipedia", np.uint8)) == "11e60398"       # the textbook example
    for n in (1, 15, 16, 17, 5552, 5553, 70000):
        x = np.random.default_rng(n).integers(0, 256, n, dtype=np.uint8)
        assert D.adler32_ref(x) == D.adler32_bytewise(x) == f"{zlib.adler32(x.tobytes()):08x}"
    assert D.adler32_ref(np.full(100000, 255, np.uint8)) == D.adler32_bytewise(np.full(100000, 255, np.uint8))


def test_xor_delta_is_an_involution_and_counts_changed_bytes():
    new, old = _pair(10000, 0.1, 1)
    diff, changed = D.xor_delta_ref(new, old)
    assert np.array_equal(diff ^ old, new) and np.array_equal(diff ^ new, old)
    assert changed == int((new != old).sum()) and 0 < changed < 1500
    assert D.xor_delta_ref(old, old)[1] == 0


def test_overwrite_encoding_layout_and_round_trip():
    new, old = _pair(5000, 0.05, 2)
    enc, changed = D.overwrite_delta_ref(new, old)
    assert enc.dtype == np.uint8 and enc.size == 4 + 5 * changed
    assert int.from_bytes(enc[:4].tobytes(), "little") == changed
    pos = np.frombuffer(enc[4:4 + 4 * changed].tobytes(), "<u4")
    assert np.all(np.diff(pos.astype(np.int64)) > 0) and np.array_equal(pos, np.flatnonzero(new != old))
    assert np.array_equal(enc[4 + 4 * changed:], new[pos])
    assert np.array_equal(D.overwrite_apply_ref(old, enc), new)
    assert np.array_equal(D.overwrite_apply_ref(D.overwrite_apply_ref(old, enc), enc), new)     # idempotent
    enc0, c0 = D.overwrite_delta_ref(old, old)
    assert c0 == 0 and enc0.tolist() == [0, 0, 0, 0]


def test_host_digests():
    # blake3 is the one digest left to the host (slime/utils/disk_delta.py:46-49): through the `blake3` package when it
    # is installed (ImportError otherwise, as in the reference); unknown names raise KeyError, as the reference's do
    import torch

    from slime_amd.delta_host import host_checksum

    w = torch.arange(1000, dtype=torch.float32).to(torch.bfloat16).view(20, 50)
    raw = w.view(torch.uint8).numpy().tobytes()
    try:
        import blake3
    except ImportError:
        with pytest.raises(ImportError):
            host_checksum("blake3", w)
    else:
        assert host_checksum("blake3", w) == blake3.blake3(raw).hexdigest()
    for name in ("md5", "xxh3-128", "adler32"):
        with pytest.raises(KeyError):
            host_checksum(name, w)
