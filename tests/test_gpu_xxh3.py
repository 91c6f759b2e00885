"""XXH3-128 on the GPU against the ``xxhash`` package the reference calls, and against the numpy restatement."""

import numpy as np
import pytest
import torch

from oracle import xxh3_ref as X
from slime_amd import _lib, delta

pytestmark = pytest.mark.gpu
xxhash = pytest.importorskip("xxhash")


def _lib_hex(t):
    return xxhash.xxh3_128(t.contiguous().view(torch.uint8).numpy().tobytes()).hexdigest()


def _bytes(n, seed):
    return torch.from_numpy(np.random.default_rng(seed).integers(0, 256, n, dtype=np.uint8))


def test_short_forms_every_length(cuda):
    xs = [_bytes(n, 300 + n) for n in range(0, 241)] + [torch.full((n,), 255, dtype=torch.uint8) for n in (1, 3, 8, 16, 17, 128, 129, 240)]
    got = delta.xxh3_128_many([x.to(cuda) for x in xs])
    for x, g in zip(xs, got):
        assert g == _lib_hex(x) and g == X.hexdigest(x.numpy()), x.numel()


@pytest.mark.parametrize("n", [241, 256, 305, 1023, 1024, 1025, 1088, 1089, 2047, 2048, 2049, 16383, 16384, 16385, 16384 * 3 + 1,
                               65536 + 64, (1 << 20) - 2, 1 << 20, (1 << 20) + 2, 5 * (1 << 20) + 777])
def test_every_boundary_against_the_library(cuda, n):
    x = _bytes(n, n)
    got = delta.xxh3_128(x.to(cuda))
    assert got == _lib_hex(x) and got == X.hexdigest(x.numpy())


def test_many_tensors_two_launches(cuda):
    sizes = [0, 5, 240, 241, 1024, 1025, 100000, 49152, 1, (1 << 20) + 3, 16384 * 40, 2 * 2560 * 9728]
    xs = [_bytes(n, 50 + i) for i, n in enumerate(sizes)]
    got = delta.xxh3_128_many([x.to(cuda) for x in xs])
    assert got == [_lib_hex(x) for x in xs]
    plan = delta.Xxh3Plan([x.to(cuda) for x in xs])
    for _ in range(2):                       # a plan is reusable: it hashes what the tensors hold when run() is called
        plan.run()
        assert plan.hexdigests() == got
    plan.tensors[6][:100] ^= 0xFF
    plan.run()
    again = plan.hexdigests()
    assert again[6] != got[6] and again[:6] == got[:6] and again[7:] == got[7:]
    assert delta.Xxh3Plan([]).hexdigests() == [] and delta.xxh3_128_many([]) == []
    # bf16 weights and views: the digest is over the bytes of the contiguous tensor, as tensor.contiguous().view(uint8) gives
    g = torch.Generator().manual_seed(1)
    w = (torch.randn(300, 520, generator=g) * 0.02).to(torch.bfloat16)
    for view in (lambda t: t, lambda t: t[:, 8:], lambda t: t.t(), lambda t: t[1:]):
        assert delta.checksum("xxh3-128", view(w.to(cuda))) == _lib_hex(view(w).contiguous())


def test_special_contents_and_unaligned_base(cuda):
    for x in (torch.zeros(70000, dtype=torch.uint8), torch.full((70000,), 255, dtype=torch.uint8),
              torch.arange(70000, dtype=torch.int32).view(torch.uint8)):
        assert delta.xxh3_128(x.to(cuda)) == _lib_hex(x)
    # through the C ABI at byte offsets 1..15 from an aligned base (the Python layer would copy to an aligned buffer)
    lib = _lib.load()
    x = _bytes(40000, 9)
    xg = x.to(cuda)
    for off in (1, 2, 7, 8, 15):
        n = 40000 - off - 3
        ws = torch.empty(lib.wq_xxh3_workspace_bytes(n) // 8, dtype=torch.int64, device=cuda)
        out = torch.zeros(2, dtype=torch.int64, device=cuda)
        assert lib.wq_xxh3_128(xg.data_ptr() + off, n, ws.data_ptr(), out.data_ptr(), _lib.stream_ptr(cuda)) == 0
        low, high = out.tolist()
        assert delta._hex128(low, high) == _lib_hex(x[off:off + n]), off
    out = torch.zeros(2, dtype=torch.int64, device=cuda)
    ws = torch.empty(64, dtype=torch.int64, device=cuda)
    assert lib.wq_xxh3_128(xg.data_ptr() + 3, 240, ws.data_ptr(), out.data_ptr(), _lib.stream_ptr(cuda)) == 0    # short form
    assert delta._hex128(*out.tolist()) == _lib_hex(x[3:243])
    assert lib.wq_xxh3_128(None, 0, ws.data_ptr(), out.data_ptr(), _lib.stream_ptr(cuda)) == 0
    assert delta._hex128(*out.tolist()) == xxhash.xxh3_128(b"").hexdigest()
    assert lib.wq_xxh3_128(xg.data_ptr(), -1, ws.data_ptr(), out.data_ptr(), _lib.stream_ptr(cuda)) == -2
    assert lib.wq_xxh3_128(None, 1000, ws.data_ptr(), out.data_ptr(), _lib.stream_ptr(cuda)) == -1


def test_large_tensor(cuda):
    # 1.5 GiB: 1.5 M blocks in one chain; compared with the library on the host
    g = torch.Generator(device=cuda).manual_seed(3)
    x = torch.randint(0, 256, (3 << 29,), dtype=torch.uint8, device=cuda, generator=g)
    assert delta.xxh3_128(x) == _lib_hex(x.cpu())


def test_delta_encoder_uses_the_gpu_digest_by_default(cuda, monkeypatch):
    from slime_amd import delta_host

    def no_host(*a, **k):
        raise AssertionError("an xxh3-128 digest must not be computed on the host")

    monkeypatch.setattr(delta_host, "host_checksum", no_host)
    g = torch.Generator().manual_seed(9)
    state = {f"l{i}.weight": torch.randn(64 + i, 96, generator=g).to(torch.bfloat16) for i in range(6)}
    enc = delta.DeltaEncoder()
    assert enc.checksum_algorithm == "xxh3-128"            # --update-weight-delta-checksum default
    for n, t in state.items():
        enc.capture(n, t.to(cuda))
    state["l2.weight"] = state["l2.weight"] * 2
    state["l5.weight"] = state["l5.weight"] + 1
    out = enc.encode_bucket([(n, t.to(cuda)) for n, t in state.items()])
    for name, diff, digest, changed in out:
        if name in ("l2.weight", "l5.weight"):
            assert changed and digest == _lib_hex(state[name])
        else:
            assert diff is None and digest is None and changed == 0
    state["l0.weight"] = state["l0.weight"] - 1
    _, digest, changed = enc.encode("l0.weight", state["l0.weight"].to(cuda))
    assert changed and digest == _lib_hex(state["l0.weight"])


# ---- the digest computed by the delta pass itself ----------------------------------------------------------------

FUSED_SIZES = [0, 1, 15, 16, 17, 240, 241, 1023, 1024, 1025, 1088, 2049, 16383, 16384, 16385, 16384 + 1024, 16384 + 1025,
               65521, 100000, (1 << 20) + 3, 16384 * 300, 16384 * 300 + 1, 2 * 2560 * 9728]


def _fused_pairs():
    rng = np.random.default_rng(77)
    pairs = []
    for i, n in enumerate(FUSED_SIZES):
        new = rng.integers(0, 256, n, dtype=np.uint8)
        old = new.copy()
        if i % 5 != 3 and n:                      # every fifth tensor is left unchanged
            flip = rng.random(n) < 0.05
            flip[rng.integers(0, n)] = True
            old[flip] ^= rng.integers(1, 256, int(flip.sum()), dtype=np.uint8)
        pairs.append((new, old))
    return pairs


@pytest.mark.parametrize("form", ["searched", "per_chunk", "single"])
@pytest.mark.parametrize("update", [False, True])
def test_digest_from_the_delta_pass(cuda, form, update):
    from oracle import delta_ref as D

    pairs = _fused_pairs()
    news = [torch.from_numpy(p[0]).to(cuda) for p in pairs]
    olds = [torch.from_numpy(p[1]).to(cuda) for p in pairs]
    if form == "searched":
        diffs, results, digests = delta.xor_diff_many(news, olds, update_snapshot=update, xxh3=True)
        hexes = [delta._hex128(lo, hi) if c else None for (lo, hi), (c, _) in zip(digests.tolist(), results.tolist())]
    elif form == "per_chunk":
        keep = [(a, b) for a, b in zip(news, olds) if a.numel()]          # a plan wants real addresses
        plan = delta.XorDiffPlan([a for a, _ in keep], [b for _, b in keep], xxh3=True)
        diffs, results = plan.run(update_snapshot=update)
        hexes = plan.hexdigests()
        pairs = [p for p in pairs if p[0].size]
        olds = [b for _, b in keep]
    else:
        lib = _lib.load()
        diffs, rows, hexes = [], [], []
        for a, b in zip(news, olds):
            n = a.numel()
            diff = torch.empty_like(a)
            ws = torch.empty(lib.wq_delta_workspace_bytes(n) // 8, dtype=torch.int64, device=cuda)
            xws = torch.empty(lib.wq_xxh3_workspace_bytes(n) // 8, dtype=torch.int64, device=cuda)
            out = torch.empty(4, dtype=torch.int64, device=cuda)
            _lib.check(lib.wq_delta_xor_xxh3(a.data_ptr() if n else None, b.data_ptr() if n else None, diff.data_ptr() if n else None,
                                             n, int(update), ws.data_ptr(), out.data_ptr(), xws.data_ptr(), out.data_ptr() + 16,
                                             _lib.stream_ptr(cuda)), "wq_delta_xor_xxh3")
            c, adler, lo, hi = out.tolist()
            diffs.append(diff)
            rows.append([c, adler])
            hexes.append(delta._hex128(lo, hi) if c else None)
            if not c:
                assert (lo, hi) == (0, 0)
        results = torch.tensor(rows)
    for (new, old), diff, res, og, hx in zip(pairs, diffs, results.tolist(), olds, hexes):
        want, changed = D.xor_delta_ref(new, old)
        assert np.array_equal(diff.cpu().numpy(), want), new.size
        assert res == [changed, int(D.adler32_ref(new), 16)], new.size
        assert np.array_equal(og.cpu().numpy(), new if update else old), new.size
        assert hx == (xxhash.xxh3_128(new.tobytes()).hexdigest() if changed else None), new.size


def test_plan_with_digest_is_reusable_and_matches_the_two_pass_form(cuda):
    g = torch.Generator(device=cuda).manual_seed(5)
    news = [torch.randint(0, 256, (n,), dtype=torch.uint8, device=cuda, generator=g) for n in (300000, 16384 * 64, 5000, 2 * 1024 * 2560)]
    olds = [t.clone() for t in news]
    plan = delta.XorDiffPlan(news, olds, xxh3=True)
    plan.run(update_snapshot=True)
    assert plan.hexdigests() == [None] * 4 and plan.results[:, 0].tolist() == [0] * 4
    news[1][12345] ^= 1
    news[3][-1] ^= 0x80
    plan.run(update_snapshot=True)
    want = delta.xxh3_128_many(news)
    assert plan.hexdigests() == [None, want[1], None, want[3]] and plan.results[:, 0].tolist() == [0, 1, 0, 1]
    assert all(torch.equal(a, b) for a, b in zip(news, olds))
    plan.run(update_snapshot=True)                     # snapshot caught up: nothing changed, no digests
    assert plan.hexdigests() == [None] * 4
