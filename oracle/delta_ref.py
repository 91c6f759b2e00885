"""numpy restatement of the reference's per-tensor delta step.  TEST INFRASTRUCTURE ONLY.

Follows slime/backends/megatron_utils/update_weight/update_weight_from_disk_delta.py:230-241
(diff_and_compress without the zstd call) and slime/utils/disk_delta.py:21-58.  adler32 is zlib's, which is
what the reference calls; a bytewise definition sits beside it as an independent witness."""

from __future__ import annotations

import zlib

import numpy as np


def xor_delta_ref(new: np.ndarray, old: np.ndarray):
    """-> (diff, changed): `diff = new ^ old; changed = int(np.count_nonzero(diff))`  (:232-234)."""
    diff = new ^ old
    return diff, int(np.count_nonzero(diff))


def overwrite_encode_ref(new: np.ndarray, changed_mask: np.ndarray) -> np.ndarray:
    """disk_delta.py:21-25: changed-position count (u4), positions (u4 each), then new values."""
    pos = np.flatnonzero(changed_mask).astype("<u4")
    return np.concatenate([np.array([pos.size], "<u4").view(np.uint8), pos.view(np.uint8), new[changed_mask]])


def overwrite_delta_ref(new: np.ndarray, old: np.ndarray):
    """-> (encoded, changed)  (:235-238)."""
    mask = new != old
    return overwrite_encode_ref(new, mask), int(np.count_nonzero(mask))


def overwrite_apply_ref(base: np.ndarray, encoded: np.ndarray) -> np.ndarray:
    """Inverse used by the round-trip tests: write the new values at their positions."""
    count = int(encoded[:4].view("<u4")[0])
    pos = encoded[4:4 + 4 * count].view("<u4")
    out = base.copy()
    out[pos] = encoded[4 + 4 * count:4 + 5 * count]
    return out


def adler32_ref(buf: np.ndarray) -> str:
    """checksum("adler32", buf), disk_delta.py:28-37,55-58."""
    return f"{zlib.adler32(buf.tobytes(), 1):08x}"


def adler32_bytewise(buf: np.ndarray) -> str:
    a, b = 1, 0
    for d in buf.tolist():
        a = (a + d) % 65521
        b = (b + a) % 65521
    return f"{(b << 16) | a:08x}"
