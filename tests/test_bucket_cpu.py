"""Host-side logic of the bucket converter that needs no GPU: the identity of a bucket's layout, the metadata records
and the reference's back-to-back packing."""

import pickle

import pytest
import torch

from slime_amd import bucket as B


def _params(shift=0):
    big = torch.zeros(4 * 64 * 32 + 8 + shift, dtype=torch.bfloat16)
    fc1 = big[shift:shift + 4 * 64 * 32].view(4, 64, 32)
    out = [("m.norm", [("h.norm.weight", torch.ones(32, dtype=torch.bfloat16))])]
    for e in range(2):
        gate, up = fc1[e].chunk(2, dim=0)
        out.append((f"m.fc1.{e}", [(f"h.{e}.gate.weight", gate), (f"h.{e}.up.weight", up)]))
    out.append(("m.t", [("h.t.weight", fc1[3].t())]))                      # a non-contiguous member
    return out


def test_layout_identity_ignores_addresses_and_sees_everything_else():
    key = B.BucketConverter._key
    a, b = _params(), _params(shift=8)
    assert a[1][1][0][1].data_ptr() != b[1][1][0][1].data_ptr()
    assert key(a) == key(b) and hash(key(a)) == hash(key(b))               # same bucket somewhere else
    renamed = [(mn, [(n + "x", t) for n, t in cv]) for mn, cv in a]
    regrouped = [a[0], (a[1][0], a[1][1] + a[2][1]), ("m.fc1.1", []), a[3]]
    reshaped = [(mn, [(n, t.reshape(-1, 16) if t.is_contiguous() and t.dim() == 2 else t) for n, t in cv]) for mn, cv in a]
    retyped = [(mn, [(n, t.view(torch.float16)) for n, t in cv]) for mn, cv in a]
    restrided = a[:3] + [("m.t", [("h.t.weight", a[3][1][0][1].t().contiguous().t()[::1, ::1].transpose(0, 1).contiguous())])]
    other_stride = a[:3] + [("m.t", [("h.t.weight", torch.zeros(64, 64, dtype=torch.bfloat16)[:, ::2].t())])]
    for other in (renamed, regrouped, reshaped, retyped, restrided, other_stride):
        assert key(other) != key(a)


def test_metadata_records_and_back_to_back_packing():
    named = [("a", torch.arange(6, dtype=torch.float32).view(2, 3)), ("b", torch.arange(5, dtype=torch.uint8)),
             ("c", torch.ones(3, 2, dtype=torch.bfloat16).t())]
    flat = B.flatten_named_tensors(named)
    meta = flat.get_metadata()
    assert [(m.name, m.start_idx, m.end_idx, m.numel) for m in meta] == [("a", 0, 24, 24), ("b", 24, 29, 5), ("c", 29, 41, 12)]
    assert meta[2].shape == torch.Size([2, 3]) and meta[2].dtype == torch.bfloat16
    assert flat.get_flattened_tensor().dtype == torch.uint8 and flat.get_flattened_tensor().numel() == 41
    back = dict((n, flat.get_flattened_tensor()[m.start_idx:m.end_idx].clone().view(m.dtype).reshape(m.shape))
                for n, m in zip("abc", meta))
    for n, t in named:
        assert torch.equal(back[n], t.contiguous())
    m = pickle.loads(pickle.dumps(meta[0]))                                 # crosses process boundaries with the bucket
    assert m == meta[0] and m.shape == torch.Size([2, 3])
    with pytest.raises(AttributeError):
        meta[0].name = "z"                                                  # records are immutable (shared with the cached layout)


def test_converter_refuses_a_bucket_without_gpu_tensors():
    cfg = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic", "weight_block_size": [128, 128]}
    with pytest.raises(RuntimeError, match="no CPU path"):
        B.BucketConverter(None, cfg).convert(_params())
