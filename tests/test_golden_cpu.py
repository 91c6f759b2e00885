"""The scalar C oracle against the committed golden vectors (made by tests/golden/make_golden.py)."""

import os

import torch
from safetensors.torch import load_file

from oracle import c_oracle as C
from tests import wq_inputs as I

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _cases(f):
    return sorted({k.split("/")[0] for k in f})


def test_fp8_golden():
    f = load_file(os.path.join(GOLDEN, "fp8_golden.safetensors"))
    assert len(_cases(f)) >= 5
    for case in _cases(f):
        w = f[f"{case}/w"]
        for mode, tag in ((0, "block"), (1, "cast"), (2, "block_dev")):
            q, s = C.fp8_block_quant(w, (128, 128), mode)
            assert torch.equal(q, f[f"{case}/q_{tag}"].view(torch.uint8)), (case, tag)
            assert I.same_bits(s, f[f"{case}/s_{tag}"]), (case, tag)
        d = C.fp8_block_dequant(f[f"{case}/q_block"].view(torch.uint8), f[f"{case}/s_block"], 128, 0)
        assert I.same_bits(d, f[f"{case}/deq"]), case


def test_kat_golden():
    f = load_file(os.path.join(GOLDEN, "kat_golden.safetensors"))
    got = C.fp8_block_dequant(f["kat_hf_to_megatron/codes"].view(torch.uint8), f["kat_hf_to_megatron/scale"], 128, 1)
    assert I.same_bits(got, f["kat_hf_to_megatron/expect"])


def test_int4_golden():
    f = load_file(os.path.join(GOLDEN, "int4_golden.safetensors"))
    for case in _cases(f):
        w = f[f"{case}/w"]
        gs = int(case.split("_")[0][1:])
        q, s, _ = C.int4_fake_quant(w, (1, gs), True)
        assert I.same_bits(q, f[f"{case}/q"]) and I.same_bits(s, f[f"{case}/scale"]), case
        p, s2, _ = C.int4_pack_layer(w, gs, True)
        assert torch.equal(p, f[f"{case}/packed"]) and I.same_bits(s2, f[f"{case}/pack_scale"]), case
        assert I.same_bits(C.int4_dequant(p, s2, tuple(w.shape), gs), f[f"{case}/deq"]), case
        assert I.same_bits(C.int4_fake_ste(w, gs, 0), f[f"{case}/ste"]), case
        assert I.same_bits(C.int4_fake_ste(w, gs, 1), f[f"{case}/ste_dev"]), case
        qa, sa, za = C.int4_fake_quant(w, (1, gs), False)
        assert I.same_bits(qa, f[f"{case}/q_asym"]) and I.same_bits(sa, f[f"{case}/scale_asym"])
        assert I.same_bits(za, f[f"{case}/zero_asym"]), case
        if f"{case}/packed_asym" in f:
            pa, _, pz = C.int4_pack_layer(w, gs, False)
            assert torch.equal(pa, f[f"{case}/packed_asym"]) and torch.equal(pz, f[f"{case}/packed_zp"]), case
