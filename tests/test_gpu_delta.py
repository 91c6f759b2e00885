"""HIP delta kernels (through the C ABI) against the numpy restatement of the reference: bit-exact bytes,
counts and digests."""

import numpy as np
import pytest
import torch

from oracle import delta_ref as D
from slime_amd import delta

pytestmark = pytest.mark.gpu


def _pair(n, density, seed):
    rng = np.random.default_rng(seed)
    old = rng.integers(0, 256, n, dtype=np.uint8)
    new = old.copy()
    idx = rng.random(n) < density
    new[idx] = rng.integers(0, 256, int(idx.sum()), dtype=np.uint8)
    return new, old


SIZES = [0, 1, 15, 16, 17, 255, 4096, 16384, 16385, 65521, 100000, (1 << 20) + 3, 16384 * 300, 16384 * 2049 + 7]


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("density", [0.0, 0.03, 1.0])
def test_xor_diff_count_and_adler32(cuda, n, density):
    new, old = _pair(n, density, n + 1)
    ng, og = torch.from_numpy(new).to(cuda), torch.from_numpy(old).to(cuda)
    diff, result = delta.xor_diff(ng, og)
    want, changed = D.xor_delta_ref(new, old)
    assert np.array_equal(diff.cpu().numpy(), want)
    assert result.tolist() == [changed, int(D.adler32_ref(new), 16)]
    assert np.array_equal(og.cpu().numpy(), old)                   # snapshot untouched unless asked
    diff2, _ = delta.xor_diff(ng, og, update_snapshot=True)
    assert np.array_equal(diff2.cpu().numpy(), want) and np.array_equal(og.cpu().numpy(), new)
    assert delta.checksum("adler32", ng) == D.adler32_ref(new)


def test_adler32_extreme_bytes(cuda):
    for fill in (0, 255):
        x = np.full(16384 * 700 + 5, fill, np.uint8)
        assert delta.checksum("adler32", torch.from_numpy(x).to(cuda)) == D.adler32_ref(x)
    with pytest.raises(KeyError):
        delta.checksum("sha1", torch.zeros(4, dtype=torch.uint8, device=cuda))


@pytest.mark.parametrize("n", SIZES)
@pytest.mark.parametrize("density", [0.0, 0.002, 0.3, 1.0])
def test_overwrite_encode(cuda, n, density):
    new, old = _pair(n, density, 7 * n + 3)
    old_dev = torch.from_numpy(old).to(cuda)
    enc = delta.overwrite_encode(torch.from_numpy(new).to(cuda), old_dev).cpu().numpy()
    want, _ = D.overwrite_delta_ref(new, old)
    assert np.array_equal(enc, want)
    assert np.array_equal(D.overwrite_apply_ref(old, enc), new)
    assert np.array_equal(old_dev.cpu().numpy(), old)                       # left alone unless asked
    enc2 = delta.overwrite_encode(torch.from_numpy(new).to(cuda), old_dev, update_snapshot=True).cpu().numpy()
    assert np.array_equal(enc2, want) and np.array_equal(old_dev.cpu().numpy(), new)


def test_weights_of_any_dtype_and_views(cuda):
    w_old = torch.randn(300, 200, generator=torch.Generator().manual_seed(0)).to(torch.bfloat16)
    w_new = w_old.clone()
    w_new[::7] += 0.01
    snap = w_old.view(torch.uint8).reshape(-1).to(cuda)
    diff, result = delta.xor_diff(w_new.to(cuda).t().contiguous().t(), snap)        # strided input is made contiguous
    want, changed = D.xor_delta_ref(w_new.view(torch.uint8).reshape(-1).numpy(), w_old.view(torch.uint8).reshape(-1).numpy())
    assert np.array_equal(diff.cpu().numpy(), want) and int(result[0]) == changed


@pytest.mark.parametrize("digest_name", ["adler32", "xxh3-128"])
@pytest.mark.parametrize("encoding", ["xor", "overwrite"])
def test_delta_encoder_follows_the_reference_loop(cuda, encoding, digest_name):
    if digest_name == "adler32":
        digest_ref = D.adler32_ref
    else:
        xxhash = pytest.importorskip("xxhash")
        digest_ref = lambda b: xxhash.xxh3_128(b.tobytes()).hexdigest()   # noqa: E731
    names = ["a.weight", "b.weight", "c.bias"]
    shapes = [(512, 384), (129, 77), (1000,)]
    g = torch.Generator().manual_seed(5)
    state = {n: torch.randn(*s, generator=g).to(torch.bfloat16) for n, s in zip(names, shapes)}
    enc = delta.DeltaEncoder(encoding, digest_name)
    snapshot = {}
    for n, t in state.items():
        enc.capture(n, t.to(cuda))
        snapshot[n] = t.view(torch.uint8).reshape(-1).numpy().copy()
    for step in range(3):
        state["a.weight"] = (state["a.weight"].float() * (1 + 1e-3 * (step + 1))).to(torch.bfloat16)
        if step == 1:
            state["c.bias"] = state["c.bias"] + 1
        changed_total = 0
        for n, t in state.items():
            new = t.view(torch.uint8).reshape(-1).numpy()
            diff, digest, changed = enc.encode(n, t.to(cuda))
            if encoding == "xor":
                want, want_changed = D.xor_delta_ref(new, snapshot[n])
            else:
                want, want_changed = D.overwrite_delta_ref(new, snapshot[n])
            assert changed == want_changed
            if want_changed:
                assert np.array_equal(diff.cpu().numpy(), want) and digest == digest_ref(new)
            else:
                assert diff is None and digest is None
            snapshot[n] = new.copy()
            changed_total += want_changed
            assert np.array_equal(enc.snapshot[n].cpu().numpy(), new)
    assert enc.total_bytes == 3 * sum(v.size for v in snapshot.values()) and enc.changed_bytes > 0


def test_encoder_with_the_xxh3_digest(cuda):
    import xxhash

    x = torch.arange(100000, dtype=torch.int32).view(torch.uint8)
    enc = delta.DeltaEncoder("xor", "xxh3-128")
    enc.capture("w", torch.zeros_like(x).to(cuda))
    _, digest, changed = enc.encode("w", x.to(cuda))
    assert changed > 0 and digest == xxhash.xxh3_128(x.numpy().tobytes()).hexdigest()


def test_argument_errors(cuda):
    x = torch.zeros(64, dtype=torch.uint8, device=cuda)
    with pytest.raises(ValueError):
        delta.xor_diff(x, x[:32])
    with pytest.raises(ValueError):
        delta.xor_diff(x, torch.zeros(64, dtype=torch.int8, device=cuda))
    with pytest.raises(RuntimeError):
        delta.xor_diff(x.cpu(), x.cpu())
    with pytest.raises(ValueError):
        delta.DeltaEncoder("patch")


def test_bucket_launch_equals_single_calls(cuda):
    sizes = [0, 5, 16384, 16385, 100000, 49152, 1, (1 << 20) + 3, 16384 * 40]
    pairs = [_pair(n, 0.0 if i == 4 else 0.05, 100 + i) for i, n in enumerate(sizes)]
    news = [torch.from_numpy(p[0]).to(cuda) for p in pairs]
    for update in (False, True):
        olds = [torch.from_numpy(p[1]).to(cuda) for p in pairs]
        diffs, results = delta.xor_diff_many(news, olds, update_snapshot=update)
        for (new, old), diff, res, og in zip(pairs, diffs, results.tolist(), olds):
            want, changed = D.xor_delta_ref(new, old)
            assert np.array_equal(diff.cpu().numpy(), want)
            assert res == [changed, int(D.adler32_ref(new), 16)]
            assert np.array_equal(og.cpu().numpy(), new if update else old)
    none, results2 = delta.xor_diff_many(news, [torch.from_numpy(p[1]).to(cuda) for p in pairs], want_diff=False)
    assert none is None and torch.equal(results2, results)


@pytest.mark.parametrize("digest_name", ["adler32", "xxh3-128"])
@pytest.mark.parametrize("encoding", ["xor", "overwrite"])
def test_delta_encoder_bucket(cuda, encoding, digest_name):
    if digest_name == "adler32":
        digest_ref = D.adler32_ref
    else:
        xxhash = pytest.importorskip("xxhash")
        digest_ref = lambda b: xxhash.xxh3_128(b.tobytes()).hexdigest()   # noqa: E731
    g = torch.Generator().manual_seed(9)
    state = {f"l{i}.weight": torch.randn(64 + i, 96 + 300 * i, generator=g).to(torch.bfloat16) for i in range(6)}
    enc = delta.DeltaEncoder(encoding, digest_name)
    for n, t in state.items():
        enc.capture(n, t.to(cuda))
    old = {n: t.view(torch.uint8).reshape(-1).numpy().copy() for n, t in state.items()}
    assert enc.encode_bucket([]) == []
    for step in range(2):
        state["l2.weight"] = state["l2.weight"] * 2
        state["l5.weight"] = state["l5.weight"] + 1
        if step:
            state["l0.weight"] = -state["l0.weight"]
        out = enc.encode_bucket([(n, t.to(cuda)) for n, t in state.items()])
        assert [o[0] for o in out] == list(state)
        for name, diff, digest, changed in out:
            new = state[name].view(torch.uint8).reshape(-1).numpy()
            want, want_changed = (D.xor_delta_ref if encoding == "xor" else D.overwrite_delta_ref)(new, old[name])
            assert changed == want_changed
            if changed:
                assert np.array_equal(diff.cpu().numpy(), want) and digest == digest_ref(new)
            else:
                assert diff is None and digest is None and name not in ("l2.weight", "l5.weight")
            assert np.array_equal(enc.snapshot[name].cpu().numpy(), new)
            old[name] = new.copy()
    assert enc.total_bytes == 2 * sum(v.size for v in old.values()) and enc.changed_bytes > 0


def test_unknown_digest_names(cuda):
    x = torch.zeros(64, dtype=torch.uint8, device=cuda)
    with pytest.raises(KeyError):
        delta.checksum("md5", x)
    assert delta.checksum("xxh3-128", x[:0]) == "99aa06d3014798d86001c324468d497f"      # XXH3_128bits of the empty input


def test_plans_refuse_inputs_they_would_have_to_copy(cuda):
    """A plan reads its tensors again on every run; an unaligned or strided tensor would be frozen into a copy at
    construction time, so it is refused (the one-shot functions copy and are fine)."""
    base = torch.zeros(4096 + 16, dtype=torch.uint8, device=cuda)
    odd = base[1:4097]                                   # 1 byte off a 16-byte boundary
    strided = torch.zeros(64, 128, dtype=torch.bfloat16, device=cuda)[:, ::2]
    for bad in (odd, strided):
        with pytest.raises(ValueError, match="contiguous at 16-byte aligned"):
            delta.Xxh3Plan([bad])
        with pytest.raises(ValueError, match="contiguous at 16-byte aligned"):
            delta.XorDiffPlan([bad], [torch.zeros(bad.numel() * bad.element_size(), dtype=torch.uint8, device=cuda)])
        assert len(delta.xxh3_128(bad)) == 32            # one-shot form: hashed from a copy
    good = base[:4096]
    plan = delta.Xxh3Plan([good])
    plan.run()
    before = plan.hexdigests()
    good[7] = 9                                          # the live tensor changes ...
    plan.run()
    assert plan.hexdigests() != before                   # ... and the plan sees it
