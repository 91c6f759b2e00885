"""Byte-level delta of weights against a snapshot kept in HBM (delta weight sync), on MI355X.

The reference diffs every gathered HF tensor against a CPU snapshot with numpy in a thread pool
(``UpdateWeightFromDiskDelta._encode_delta``, slime/backends/megatron_utils/update_weight/
update_weight_from_disk_delta.py:198-274; helpers in slime/utils/disk_delta.py:21-58).  Here the snapshot
lives in device memory - 288 GB of HBM hold a full model next to the live weights - and one kernel pass per
tensor yields the xor diff, the changed-byte count, the adler32 of the new bytes and the updated snapshot;
only the diff of a tensor that did change has to cross PCIe for compression.

``xor_diff`` / ``overwrite_encode`` / ``checksum`` are the per-tensor operations, ``DeltaEncoder`` the
snapshot-keeping loop body (``diff_and_compress`` + ``collect`` without the zstd step, which stays on the
host).  ``adler32`` comes out of the diff pass itself; ``xxh3-128`` - the reference's default - is computed on the GPU
too (its per-block sums at memory speed, the sequential scramble chain by eight lanes per tensor: ``xxh3_128`` /
``xxh3_128_many``), so a changed tensor's bytes never cross PCIe for their digest.  ``blake3`` is a host digest, as in
the reference.
"""

from __future__ import annotations

import torch

from . import _lib

CHUNK = 16384        # WQ_DELTA_CHUNK: bytes of a tensor one workgroup handles


def _as_bytes(t: torch.Tensor, what: str) -> torch.Tensor:
    _lib.require_gpu(t, what)
    flat = t.detach().contiguous().view(torch.uint8).reshape(-1)
    if flat.data_ptr() % 16:
        flat = flat.clone()
    return flat


def _as_bytes_in_place(t: torch.Tensor, what: str) -> torch.Tensor:
    """For plans, which read the tensor again on every run: a byte view of the tensor itself, never a copy."""
    _lib.require_gpu(t, what)
    if not t.is_contiguous() or t.data_ptr() % 16:
        raise ValueError(f"{what}: tensors of a plan must be contiguous at 16-byte aligned addresses (a copy would be "
                         f"hashed / diffed instead of the live weight); got strides {t.stride()}, address % 16 = {t.data_ptr() % 16}")
    return t.detach().view(torch.uint8).reshape(-1)


def _workspace(n: int, device) -> torch.Tensor:
    return torch.empty(_lib.load().wq_delta_workspace_bytes(n) // 8, dtype=torch.int64, device=device)


def _xor_pass(new: torch.Tensor, old: torch.Tensor, diff, update_old: bool, workspace, result) -> None:
    with torch.cuda.device(new.device):
        rc = _lib.load().wq_delta_xor(new.data_ptr(), old.data_ptr(), diff.data_ptr() if diff is not None else None,
                                      new.numel(), int(update_old), workspace.data_ptr(), result.data_ptr(),
                                      _lib.stream_ptr(new.device))
    _lib.check(rc, "delta xor pass")


def xor_diff(new: torch.Tensor, old: torch.Tensor, update_snapshot: bool = False):
    """-> (diff uint8 [nbytes] = new ^ old, result int64 [2] on the device = [changed bytes, adler32(new)]).

    ``old`` must be a contiguous uint8 tensor of the same byte size; with ``update_snapshot`` it is overwritten
    with the new bytes in the same pass.  Nothing synchronises: read ``result`` when the values are needed."""
    nw = _as_bytes(new, "xor_diff")
    _check_old(nw, old)
    diff = torch.empty_like(nw)
    result = torch.empty(2, dtype=torch.int64, device=nw.device)
    _xor_pass(nw, old, diff, update_snapshot, _workspace(nw.numel(), nw.device), result)
    return diff, result


def _align(n: int, a: int = 256) -> int:
    return (n + a - 1) // a * a


def _bucket_tables(flat, olds, want_diff: bool, xxh3: bool, device):
    """Buffers and the per-tensor descriptor rows (wq_delta_desc: new, old, diff, n, workspace, result, xxh3_sums,
    xxh3_digest) of a bucket: one flat diff buffer, one flat workspace (delta rows, then the digest's block sums)."""
    lib = _lib.load()
    d_off, w_off, x_off, d_total, w_total = [], [], [], 0, 0
    for nw, old in zip(flat, olds):
        _check_old(nw, old)
        d_off.append(d_total)
        w_off.append(w_total)
        d_total += _align(nw.numel())
        w_total += _align(lib.wq_delta_workspace_bytes(nw.numel()))
    for nw in flat:
        x_off.append(w_total)
        if xxh3:
            w_total += _align(lib.wq_xxh3_workspace_bytes(nw.numel()))
    flat_diff = torch.empty(max(d_total, 1), dtype=torch.uint8, device=device) if want_diff else None
    flat_ws = torch.empty(w_total // 8, dtype=torch.int64, device=device)
    results = torch.empty((len(flat), 2), dtype=torch.int64, device=device)
    digests = torch.empty((len(flat), 2), dtype=torch.int64, device=device) if xxh3 else None     # [low64, high64]
    rows = []
    for i, (nw, old) in enumerate(zip(flat, olds)):
        rows.append([nw.data_ptr(), old.data_ptr(), flat_diff.data_ptr() + d_off[i] if want_diff else 0, nw.numel(),
                     flat_ws.data_ptr() + w_off[i], results.data_ptr() + 16 * i,
                     flat_ws.data_ptr() + x_off[i] if xxh3 else 0, digests.data_ptr() + 16 * i if xxh3 else 0])
    diffs = [flat_diff[o:o + nw.numel()] for o, nw in zip(d_off, flat)] if want_diff else None
    return rows, flat_diff, flat_ws, results, digests, diffs


def xor_diff_many(news, olds, update_snapshot: bool = False, want_diff: bool = True, xxh3: bool = False):
    """``xor_diff`` over a bucket of tensors with two kernel launches in total (three with ``xxh3``).

    -> (diffs: list of uint8 views into one flat buffer, or None without ``want_diff``;
        results: int64 [len(news), 2] on the device = [changed bytes, adler32(new)] per tensor)
       and, with ``xxh3``, a third value: int64 [len(news), 2] on the device = [low64, high64] of xxh3-128 of the new
       bytes of every tensor that changed ([0, 0] for the others), computed by the same pass over the tensors."""
    if len(news) != len(olds):
        raise ValueError("xor_diff_many: need one snapshot per tensor")
    if not news:
        empty = torch.empty((0, 2), dtype=torch.int64)
        return (([] if want_diff else None), empty) + ((empty,) if xxh3 else ())
    p = _grouped_pass([_as_bytes(t, "xor_diff_many") for t in news], olds, update_snapshot, want_diff, xxh3)
    return (p["diffs"], p["results"]) + ((p["digests"],) if xxh3 else ())


def _grouped_pass(flat, olds, update_snapshot: bool, want_diff: bool, xxh3: bool) -> dict:
    """One wq_delta_xor_grouped over byte views ``flat``; keeps the workspace (its per-chunk counts are what the
    overwrite encoding consumes) next to the results."""
    device = flat[0].device
    rows, flat_diff, flat_ws, results, digests, diffs = _bucket_tables(flat, olds, want_diff, xxh3, device)
    starts, chunks = [0], 0
    for nw in flat:
        chunks += -(-nw.numel() // CHUNK)
        starts.append(chunks)
    descs = torch.tensor(rows, dtype=torch.int64).to(device)
    start_t = torch.tensor(starts, dtype=torch.int64).to(device)
    with torch.cuda.device(device):
        rc = _lib.load().wq_delta_xor_grouped(descs.data_ptr(), start_t.data_ptr(), len(flat), chunks, int(want_diff),
                                              int(update_snapshot), int(xxh3), _lib.stream_ptr(device))
    _lib.check(rc, "xor_diff_many")
    return {"rows": rows, "workspace": flat_ws, "results": results, "digests": digests, "diffs": diffs, "tables": (descs, start_t)}


class XorDiffPlan:
    """``xor_diff_many`` for a FIXED bucket - the same weight tensors against the same snapshots every weight sync - with
    the per-chunk work table built once: every 16 KiB chunk has its own pre-resolved descriptor (64 bytes per 64 KiB of
    traffic), so the kernel does one scalar load instead of searching the per-tensor prefix sums, and ``run()`` does no
    host-side table work.  ``diffs`` (uint8 views into one flat buffer), ``results`` (int64 [n, 2] = [changed bytes,
    adler32(new)]) and, with ``xxh3``, ``digests`` (int64 [n, 2] = [low64, high64] of xxh3-128 of the new bytes, [0, 0]
    for a tensor that did not change) are owned by the plan and overwritten by every run."""

    def __init__(self, news, olds, want_diff: bool = True, xxh3: bool = False):
        if not news or len(news) != len(olds):
            raise ValueError("XorDiffPlan: need one snapshot per tensor and at least one tensor")
        self.news = [_as_bytes_in_place(t, "XorDiffPlan") for t in news]
        self.olds = list(olds)
        self.want_diff, self.xxh3 = bool(want_diff), bool(xxh3)
        device = self.news[0].device
        rows, self._flat_diff, self._flat_ws, self.results, self.digests, self.diffs = _bucket_tables(
            self.news, self.olds, self.want_diff, self.xxh3, device)
        desc = torch.tensor(rows, dtype=torch.int64)
        counts = (desc[:, 3] + CHUNK - 1) // CHUNK
        owner = torch.repeat_interleave(torch.arange(len(rows)), counts)
        chunk = torch.arange(int(counts.sum()), dtype=torch.int64) - (torch.cumsum(counts, 0) - counts)[owner]
        picked = desc[owner]
        # wq_delta_chunk_item: new, old, diff, n, workspace, chunk, xxh3_sums, reserved
        items = torch.cat([picked[:, :5], chunk.unsqueeze(1), picked[:, 6:7], torch.zeros_like(chunk).unsqueeze(1)], dim=1)
        self._descs, self._items, self.n_items = desc.to(device), items.contiguous().to(device), items.shape[0]
        self.device = device
        self.nbytes = sum(nw.numel() for nw in self.news)

    def run(self, update_snapshot: bool = False):
        with torch.cuda.device(self.device):
            rc = _lib.load().wq_delta_xor_items(self._items.data_ptr(), self.n_items, self._descs.data_ptr(), len(self.news),
                                                int(self.want_diff), int(update_snapshot), int(self.xxh3),
                                                _lib.stream_ptr(self.device))
        _lib.check(rc, "XorDiffPlan.run")
        return self.diffs, self.results

    def hexdigests(self) -> list:
        """xxh3-128 hex digests after a run (synchronises); None for a tensor that did not change."""
        if not self.xxh3:
            raise ValueError("XorDiffPlan was built without xxh3")
        changed = self.results[:, 0].tolist()
        return [_hex128(low, high) if c else None for (low, high), c in zip(self.digests.tolist(), changed)]


def _check_old(nw: torch.Tensor, old: torch.Tensor) -> None:
    if old.dtype != torch.uint8 or old.dim() != 1 or not old.is_contiguous() or old.numel() != nw.numel():
        raise ValueError(f"snapshot must be a contiguous uint8 vector of {nw.numel()} bytes, got "
                         f"{tuple(old.shape)} {old.dtype}")
    if old.device != nw.device or old.data_ptr() % 16:
        raise ValueError("snapshot must live on the tensor's device at a 16-byte aligned address")


def overwrite_encode(new: torch.Tensor, old: torch.Tensor, update_snapshot: bool = False) -> torch.Tensor:
    """The 'overwrite' delta of slime/utils/disk_delta.py:21-25 for ``changed_mask = new != old``:
    uint8 vector [count u32 LE][positions u32 LE x count][new values x count].  Synchronises once (the output
    size depends on the count).  With ``update_snapshot`` the pass that writes the encoding also sets ``old`` to the
    new bytes."""
    nw = _as_bytes(new, "overwrite_encode")
    _check_old(nw, old)
    if nw.numel() > 0xFFFFFFFF:
        raise ValueError("overwrite_encode: positions are uint32; tensor too large")
    ws = _workspace(nw.numel(), nw.device)
    result = torch.empty(2, dtype=torch.int64, device=nw.device)
    _xor_pass(nw, old, None, False, ws, result)
    count = int(result[0].item())
    out = torch.empty(4 + 5 * count, dtype=torch.uint8, device=nw.device)
    with torch.cuda.device(nw.device):
        rc = _lib.load().wq_delta_overwrite_encode(nw.data_ptr(), old.data_ptr(), nw.numel(), ws.data_ptr(), count,
                                                   out.data_ptr(), int(update_snapshot), _lib.stream_ptr(nw.device))
    _lib.check(rc, "overwrite_encode")
    return out


def _hex128(low: int, high: int) -> str:
    return f"{high & 0xFFFFFFFFFFFFFFFF:016x}{low & 0xFFFFFFFFFFFFFFFF:016x}"


class Xxh3Plan:
    """xxh3-128 of a fixed list of tensors: the descriptor table, the workspace (64 bytes per KiB) and the digest buffer
    are set up once; ``run()`` is two launches and no host work, ``hexdigests()`` synchronises and formats.  The tensors
    are hashed where they are, so they must stay contiguous at 16-byte aligned addresses (what ``run()`` hashes is their
    content at that moment)."""

    def __init__(self, tensors, in_place: bool = True):
        self.tensors = [(_as_bytes_in_place if in_place else _as_bytes)(t, "Xxh3Plan") for t in tensors]
        self.n = len(self.tensors)
        if not self.n:
            return
        self.device = self.tensors[0].device
        lib = _lib.load()
        ws_off, total_ws, items, n_items = [], 0, [0], 0
        for f in self.tensors:
            n = f.numel()
            ws_off.append(total_ws)
            total_ws += (lib.wq_xxh3_workspace_bytes(n) + 255) // 256 * 256
            n_items += -(-((n - 1) // 1024) // 16) if n > 0 else 0
            items.append(n_items)
        self._ws = torch.empty(total_ws // 8, dtype=torch.int64, device=self.device)
        self.digests = torch.empty((self.n, 2), dtype=torch.int64, device=self.device)       # [low64, high64] per tensor
        rows = [[f.data_ptr(), f.numel(), self._ws.data_ptr() + o, self.digests.data_ptr() + 16 * k]
                for k, (f, o) in enumerate(zip(self.tensors, ws_off))]
        self._descs = torch.tensor(rows, dtype=torch.int64).to(self.device)
        self._starts = torch.tensor(items, dtype=torch.int64).to(self.device)
        self._n_items = n_items

    def run(self) -> torch.Tensor:
        if self.n:
            with torch.cuda.device(self.device):
                rc = _lib.load().wq_xxh3_128_grouped(self._descs.data_ptr(), self._starts.data_ptr(), self.n, self._n_items,
                                                     _lib.stream_ptr(self.device))
            _lib.check(rc, "xxh3_128")
            return self.digests
        return torch.empty((0, 2), dtype=torch.int64)

    def hexdigests(self) -> list:
        return [_hex128(low, high) for low, high in self.digests.tolist()] if self.n else []


def xxh3_128_many(tensors) -> list:
    """``xxhash.xxh3_128(bytes of t).hexdigest()`` for every tensor, computed on the GPU with two launches and one
    synchronisation.  -> list of 32-digit hex strings."""
    plan = Xxh3Plan(tensors, in_place=False)       # one-shot: unaligned or strided inputs may be hashed from a copy
    plan.run()
    return plan.hexdigests()


def xxh3_128(buf: torch.Tensor) -> str:
    """``checksum("xxh3-128", buf)`` of slime/utils/disk_delta.py:55-58 with the tensor left in device memory."""
    return xxh3_128_many([buf])[0]


def checksum(algorithm: str, buf: torch.Tensor) -> str:
    """``checksum(algorithm, tensor)`` of slime/utils/disk_delta.py:55-58 on the GPU: "adler32" -> 8 hex digits,
    "xxh3-128" -> 32.  "blake3" is hashed on the host (it needs the ``blake3`` package, as in the reference); unknown
    names raise KeyError as the reference does."""
    if algorithm == "xxh3-128":
        return xxh3_128(buf)
    if algorithm != "adler32":
        from .delta_host import host_checksum

        return host_checksum(algorithm, buf)
    nw = _as_bytes(buf, "checksum")
    result = torch.empty(2, dtype=torch.int64, device=nw.device)
    _xor_pass(nw, nw, None, False, _workspace(nw.numel(), nw.device), result)
    return f"{int(result[1].item()):08x}"


class DeltaEncoder:
    """Snapshot in HBM + the per-tensor body of ``_encode_delta``.

    ``capture(name, tensor)`` seeds the snapshot (``_capture_baseline``, update_weight_from_disk_delta.py:96-128).
    ``encode(name, tensor)`` returns ``(diff_or_None, checksum_or_None, changed)`` like ``diff_and_compress`` minus
    compression: ``diff`` is the xor bytes or the overwrite encoding (device uint8 tensor), ``None`` when nothing
    changed; the snapshot is updated either way (``collect``: ``snapshot[name] = new``).  ``changed_bytes`` /
    ``total_bytes`` accumulate as in the reference."""

    def __init__(self, delta_encoding: str = "xor", checksum_algorithm: str = "xxh3-128"):
        if delta_encoding not in ("xor", "overwrite"):
            raise ValueError(f"unknown delta encoding {delta_encoding!r}")
        self.delta_encoding = delta_encoding
        self.checksum_algorithm = checksum_algorithm
        self.snapshot: dict[str, torch.Tensor] = {}
        self.changed_bytes = self.total_bytes = 0

    def capture(self, name: str, tensor: torch.Tensor) -> None:
        self.snapshot[name] = _as_bytes(tensor, "DeltaEncoder.capture").clone()

    def encode_bucket(self, named_tensors):
        """``encode`` for a list of (name, tensor) with one synchronisation: one pass over the whole bucket for the xor
        diff (or, for the overwrite encoding, the counts), adler32, the xxh3-128 digest and the snapshot update, then -
        overwrite only - one scatter launch per tensor that changed.
        -> list of (name, diff_or_None, checksum_or_None, changed) in input order."""
        named_tensors = list(named_tensors)
        if not named_tensors:
            return []
        xor = self.delta_encoding == "xor"
        fused = self.checksum_algorithm == "xxh3-128"       # the digest rides on the pass: no second read
        flat = [_as_bytes(t, "DeltaEncoder.encode_bucket") for _, t in named_tensors]
        olds = [self.snapshot[n] for n, _ in named_tensors]
        if not xor and any(f.numel() > 0xFFFFFFFF for f in flat):
            raise ValueError("overwrite encoding: positions are uint32; tensor too large")
        p = _grouped_pass(flat, olds, update_snapshot=xor, want_diff=xor, xxh3=fused)
        results = p["results"].tolist()                      # the one synchronisation
        digests = p["digests"].tolist() if fused else None
        lib, out = _lib.load(), []
        for i, ((name, t), nw, old, (changed, adler)) in enumerate(zip(named_tensors, flat, olds, results)):
            self.total_bytes += nw.numel()
            if not changed:
                out.append((name, None, None, 0))
                continue
            self.changed_bytes += changed
            if xor:
                diff = p["diffs"][i]
            else:                                            # scatter + snapshot update, from the counts the pass left
                diff = torch.empty(4 + 5 * changed, dtype=torch.uint8, device=nw.device)
                with torch.cuda.device(nw.device):
                    rc = lib.wq_delta_overwrite_encode(nw.data_ptr(), old.data_ptr(), nw.numel(), p["rows"][i][4], changed,
                                                       diff.data_ptr(), 1, _lib.stream_ptr(nw.device))
                _lib.check(rc, "DeltaEncoder.encode_bucket")
            if self.checksum_algorithm == "adler32":
                digest = f"{adler:08x}"
            elif fused:
                digest = _hex128(*digests[i])
            else:
                digest = checksum(self.checksum_algorithm, t)
            out.append((name, diff, digest, changed))
        return out

    def encode(self, name: str, tensor: torch.Tensor):
        nw = _as_bytes(tensor, "DeltaEncoder.encode")
        old = self.snapshot[name]
        _check_old(nw, old)
        n = nw.numel()
        self.total_bytes += n
        lib = _lib.load()
        ws = _workspace(n, nw.device)
        both = torch.empty(4, dtype=torch.int64, device=nw.device)      # [changed bytes, adler32], then the digest
        fused = self.checksum_algorithm == "xxh3-128"                   # the digest rides on the pass that counts / diffs
        xor = self.delta_encoding == "xor"
        diff = torch.empty_like(nw) if xor else None
        with torch.cuda.device(nw.device):
            if fused:
                xws = torch.empty(lib.wq_xxh3_workspace_bytes(n) // 8, dtype=torch.int64, device=nw.device)
                rc = lib.wq_delta_xor_xxh3(nw.data_ptr(), old.data_ptr(), diff.data_ptr() if xor else None, n, int(xor),
                                           ws.data_ptr(), both.data_ptr(), xws.data_ptr(), both.data_ptr() + 16,
                                           _lib.stream_ptr(nw.device))
            else:
                rc = lib.wq_delta_xor(nw.data_ptr(), old.data_ptr(), diff.data_ptr() if xor else None, n, int(xor),
                                      ws.data_ptr(), both.data_ptr(), _lib.stream_ptr(nw.device))
        _lib.check(rc, "DeltaEncoder.encode")
        changed, adler, low, high = (int(v) for v in both.tolist())
        digest = _hex128(low, high) if fused else None
        if not xor and changed:                      # the second pass writes the encoding and brings the snapshot up to date
            diff = torch.empty(4 + 5 * changed, dtype=torch.uint8, device=nw.device)
            with torch.cuda.device(nw.device):
                rc = lib.wq_delta_overwrite_encode(nw.data_ptr(), old.data_ptr(), n, ws.data_ptr(), changed, diff.data_ptr(), 1,
                                                   _lib.stream_ptr(nw.device))
            _lib.check(rc, "DeltaEncoder.encode")
        if not changed:
            return None, None, 0
        self.changed_bytes += changed
        if digest is None:
            digest = f"{adler:08x}" if self.checksum_algorithm == "adler32" else checksum(self.checksum_algorithm, nw)
        return diff, digest, changed
