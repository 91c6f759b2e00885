"""Writes the golden vectors under tests/golden/.

Inputs are seeded; expected outputs come from the op-for-op torch restatement of the reference
(oracle/torch_ref.py) run on the CPU - the same torch primitives, in the same order and dtypes, as
tools/convert_hf_to_fp8.py:41-75, fp8_kernel.py:24-58 (read as IEEE arithmetic), tools/fp8_cast_bf16.py:25-28,
tools/convert_hf_to_int4_direct.py:32-153, tools/convert_k2_thinking_int4_to_bf16.py:55-84 and
docker/patch/latest/megatron.patch:212-246.  The `*_dev` entries hold the same functions with `tensor / scalar`
evaluated as torch's GPU kernels do (a multiplication by the rounded reciprocal).  The reference's own Python was NOT imported or run to make
them: its functions on this path are pinned by the checks in tests/test_oracle_*.py, and its INT4 kernel
cannot run without a CUDA device.  Also stored: the data of the reference's known-answer test
tests/test_hf_to_megatron.py:345-358.

Run from the repository root:  python tests/golden/make_golden.py
"""

import os
import sys

import torch
from safetensors.torch import save_file

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import torch_ref as T  # noqa: E402
from tests import wq_inputs as I  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def fp8_cases():
    torch.manual_seed(0)
    cases = {
        "randn256_seed0": torch.randn(256, 256, dtype=torch.float32).to(torch.bfloat16),   # reference test input
        "ragged300x200": I.weights(300, 200, seed=1),
        "zero_and_one": torch.zeros(256, 256, dtype=torch.bfloat16),
        "special": torch.cat([I.subnormal_block(seed=1), I.near_max_block(seed=2),
                              -torch.zeros(128, 128, dtype=torch.bfloat16)], dim=1),
        "outliers384": I.zero_blocks(I.weights(384, 384, seed=3, outlier_p=0.01), 0.2, seed=3),
    }
    cases["zero_and_one"][0, 0] = 1.0
    return cases


def main():
    out = {}
    for name, w in fp8_cases().items():
        q, s = T.block_fp8_ref(w, (128, 128))
        qc, sc = T.blockwise_cast_ref(w, (128, 128))
        out[f"{name}/w"] = w.contiguous()
        out[f"{name}/q_block"], out[f"{name}/s_block"] = q.contiguous(), s.contiguous()
        qd, sd = T.block_fp8_ref(w, (128, 128), device_arith=True)      # as torch evaluates `/ 448` on GPU tensors
        out[f"{name}/q_block_dev"], out[f"{name}/s_block_dev"] = qd.contiguous(), sd.contiguous()
        out[f"{name}/q_cast"], out[f"{name}/s_cast"] = qc.contiguous(), sc.contiguous()
        out[f"{name}/deq"] = T.weight_dequant_ref(q, s, 128).contiguous()
    kat_w = torch.linspace(-2, 2, 128 * 128).view(128, 128).to(torch.float8_e4m3fn)
    out["kat_hf_to_megatron/codes"] = kat_w
    out["kat_hf_to_megatron/scale"] = torch.tensor([[2.0]])
    out["kat_hf_to_megatron/expect"] = kat_w.to(torch.bfloat16) * 2
    kat = {k: v for k, v in out.items() if k.startswith("kat_")}
    fp8 = {k: v for k, v in out.items() if not k.startswith("kat_")}
    save_file(fp8, os.path.join(HERE, "fp8_golden.safetensors"))
    save_file(kat, os.path.join(HERE, "kat_golden.safetensors"))

    i4 = {}
    for name, (shape, gs) in {"g128_24x512": ((24, 512), 128), "g32_16x96": ((16, 96), 32),
                              "g128_outliers": ((16, 1024), 128)}.items():
        w = I.weights(*shape, seed=gs + shape[0], outlier_p=0.01)
        w[0, :gs] = 0
        q, sc, zp = T.fake_int4_quant_ref(w, (1, gs), True)
        p, s2, _ = T.pack_layer_ref(w, gs, True)
        i4[f"{name}/w"] = w
        i4[f"{name}/q"], i4[f"{name}/scale"] = q, sc.contiguous()
        i4[f"{name}/packed"], i4[f"{name}/pack_scale"] = p.contiguous(), s2.contiguous()
        i4[f"{name}/deq"] = T.int4_dequant_ref(p, s2, shape, gs)
        i4[f"{name}/ste"] = T.fake_int4_ste_ref(w, gs)
        i4[f"{name}/ste_dev"] = T.fake_int4_ste_ref(w, gs, device_arith=True)
        qa, sa, za = T.fake_int4_quant_ref(w, (1, gs), False)
        i4[f"{name}/q_asym"], i4[f"{name}/scale_asym"], i4[f"{name}/zero_asym"] = qa, sa.contiguous(), za.contiguous()
        if shape[0] % 8 == 0:
            pa, s3, pz = T.pack_layer_ref(w, gs, False)
            i4[f"{name}/packed_asym"], i4[f"{name}/packed_zp"] = pa.contiguous(), pz.contiguous()
    save_file(i4, os.path.join(HERE, "int4_golden.safetensors"))
    for f in ("fp8_golden.safetensors", "kat_golden.safetensors", "int4_golden.safetensors"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
