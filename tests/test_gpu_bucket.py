"""One-launch bucket conversion against the per-parameter loop it replaces: same names in the same order, same
shapes and dtypes, same bytes - and against the CPU oracle for the quantised members."""

import pytest
import torch

import slime_amd
from oracle import c_oracle as C
from slime_amd import bucket as B
from tests import wq_inputs as I

pytestmark = pytest.mark.gpu

FP8_CFG = {"quant_method": "fp8", "fmt": "e4m3", "activation_scheme": "dynamic", "weight_block_size": [128, 128]}
INT4_CFG = {"quant_method": "compressed-tensors",
            "config_groups": {"group_0": {"weights": {"group_size": 128, "symmetric": True, "num_bits": 4}}},
            "ignore": ["re:.*lm_head.*", "re:.*norm.*", "re:.*embed.*", "re:.*self_attn.*", "re:.*shared_experts.*",
                       "re:.*mlp\\.(gate|up|gate_up|down)_proj.*", "re:.*mlp\\.gate\\.*"]}      # the converter's default rules
L = "module.module.decoder.layers.{}."


def _moe_layer(layer, cuda, seed, experts=3, hidden=256, ffn=384):
    """A small MoE layer after name conversion: q/k/v from one fused parameter, gate/up as chunk views of one fc1
    weight per expert, norms (1-D), a router (fp32) - the shapes of what _convert_to_hf_core yields."""
    hf = f"model.layers.{layer}."
    g = lambda *sh, s=0: I.weights(*sh, seed=seed + s).to(cuda)
    params = [
        (L.format(layer) + "self_attention.linear_qkv.layer_norm_weight", [(hf + "input_layernorm.weight", g(1, hidden, s=1)[0])]),
        (L.format(layer) + "self_attention.linear_qkv.weight",
         [(hf + "self_attn.q_proj.weight", g(512, hidden, s=2)), (hf + "self_attn.k_proj.weight", g(128, hidden, s=3)),
          (hf + "self_attn.v_proj.weight", g(128, hidden, s=4))]),
        (L.format(layer) + "self_attention.linear_proj.weight", [(hf + "self_attn.o_proj.weight", g(hidden, 512, s=5))]),
        (L.format(layer) + "mlp.router.weight", [(hf + "mlp.gate.weight", g(experts, hidden, s=6).float())]),
    ]
    for e in range(experts):
        fc1 = g(2 * ffn, hidden, s=10 + 2 * e)
        gate, up = fc1.chunk(2, dim=0)
        params.append((L.format(layer) + f"mlp.experts.linear_fc1.weight{e}",
                       [(hf + f"mlp.experts.{e}.gate_proj.weight", gate), (hf + f"mlp.experts.{e}.up_proj.weight", up)]))
        params.append((L.format(layer) + f"mlp.experts.linear_fc2.weight{e}",
                       [(hf + f"mlp.experts.{e}.down_proj.weight", g(hidden, ffn, s=11 + 2 * e))]))
    return params


def _same_as_loop(bucket, want):
    got = bucket.reconstruct_tensors()
    assert [n for n, _ in got] == [n for n, _ in want]
    for (n, a), (_, b), m in zip(got, want, bucket.metadata):
        assert a.shape == b.shape and a.dtype == b.dtype and m.numel == b.numel() * b.element_size(), n
        assert I.same_bits(a.cpu(), b.cpu()), n
    ends = [m.end_idx for m in bucket.metadata]
    assert all(m.start_idx >= e for m, e in zip(bucket.metadata[1:], ends))         # in order, no overlap
    assert bucket.get_flattened_tensor().dtype == torch.uint8 and bucket.get_flattened_tensor().numel() == ends[-1]


def test_fp8_bucket_equals_per_param_loop_and_oracle(cuda):
    params = _moe_layer(0, cuda, 100) + _moe_layer(1, cuda, 200) + [
        ("module.module.embedding.word_embeddings.weight", [("model.embed_tokens.weight", I.weights(1000, 256, seed=7).to(cuda))]),
        ("module.module.decoder.final_layernorm.weight", [("model.norm.weight", I.weights(1, 256, seed=8)[0].to(cuda))])]
    conv = B.BucketConverter(None, FP8_CFG)
    out = conv.convert(params)
    want = B.per_param_loop(None, params, FP8_CFG)
    _same_as_loop(out, want)
    assert out.launches == 2 and conv.plan_builds == 1      # these small matrices leave their successors 32 bytes off a line (below)
    # every size here is a multiple of its successor's element size: the buffer is the plain concatenation
    assert torch.equal(out.get_flattened_tensor(), B.flatten_named_tensors(want).get_flattened_tensor())
    # quantised members against the CPU oracle (weight-sync arithmetic = mode 1)
    named = dict(out.reconstruct_tensors())
    for mn, cv in params:
        for n, t in cv:
            if n.endswith("proj.weight"):
                qo, so = C.fp8_block_quant(t.cpu().contiguous(), (128, 128), 1)
                assert torch.equal(named[n].cpu().view(torch.uint8), qo), n
                assert torch.equal(named[n.replace(".weight", ".weight_scale_inv")].cpu().view(torch.int32), so.view(torch.int32)), n
    # same tensors again: cached table, fresh buffer; inputs changed in place: outputs follow
    params[1][1][0][1].mul_(3)
    out2 = conv.convert(params)
    assert conv.plan_builds == 1 and out2.get_flattened_tensor().data_ptr() != out.get_flattened_tensor().data_ptr()
    assert conv.resolves == 1
    _same_as_loop(out2, B.per_param_loop(None, params, FP8_CFG))
    # same shapes at other addresses: the layout is kept, only the addresses are resolved again (on the GPU)
    moved = [(mn, [(n, t.clone()) for n, t in cv]) for mn, cv in params]
    _same_as_loop(conv.convert(moved), B.per_param_loop(None, moved, FP8_CFG))
    assert conv.plan_builds == 1 and conv.resolves == 2
    # into a caller-owned buffer
    buf = torch.empty(out.get_flattened_tensor().numel() + 64, dtype=torch.uint8, device=cuda)
    out3 = conv.convert(moved, out=buf)
    assert out3.get_flattened_tensor().data_ptr() == buf.data_ptr()
    _same_as_loop(out3, B.per_param_loop(None, moved, FP8_CFG))
    assert conv.plan_builds == 1 and conv.resolves == 2


@pytest.mark.parametrize("cfg", ["fp8", "int4", "int4_asym"])
def test_bucket_inputs_reallocated_every_sync(cuda, cfg):
    """What a sharded model presents: the same names and shapes every sync, each time in freshly allocated tensors
    (gathered partitions, concatenated experts).  The layout is built once; every sync after that uploads the new
    addresses and resolves the work-item table on the GPU - bytes equal to the per-parameter loop and to the oracle."""
    config = {"fp8": FP8_CFG, "int4": INT4_CFG,
              "int4_asym": {**INT4_CFG, "config_groups": {"group_0": {"weights": {"group_size": 128, "symmetric": False}}}}}[cfg]
    conv = B.BucketConverter(None, config)
    keep = []                                     # earlier syncs' tensors stay allocated: the new ones cannot reuse their addresses
    for sync in range(4):
        params = _moe_layer(0, cuda, 900 + sync) + _moe_layer(1, cuda, 950 + sync)
        keep.append(params)
        out = conv.convert(params, bucket_id="layers 0-1")
        _same_as_loop(out, B.per_param_loop(None, params, config))
        assert conv.plan_builds == 1 and conv.resolves == sync + 1
        named = dict(out.reconstruct_tensors())
        n, t = params[4][1][0]                   # an expert's gate projection: a chunk view of its fc1 weight
        assert n.endswith("experts.0.gate_proj.weight")
        if cfg == "fp8":
            qo, so = C.fp8_block_quant(t.cpu().contiguous(), (128, 128), 1)
            assert torch.equal(named[n].cpu().view(torch.uint8), qo)
            assert torch.equal(named[n.replace(".weight", ".weight_scale_inv")].cpu().view(torch.int32), so.view(torch.int32))
        else:
            po, so, zo = C.int4_pack_layer(t.cpu().contiguous(), 128, cfg == "int4")
            assert torch.equal(named[n.replace(".weight", ".weight_packed")].cpu(), po)
            assert I.same_bits(named[n.replace(".weight", ".weight_scale")].cpu(), so)
    # the first sync's tensors again (another move), without the id: found by the layout's identity
    again = conv.convert(keep[0])
    _same_as_loop(again, B.per_param_loop(None, keep[0], config))
    assert conv.plan_builds == 2 and conv.convert(keep[0]).launches == again.launches and conv.plan_builds == 2


def test_int4_bucket_input_that_lost_its_alignment(cuda):
    """The cached routing of an INT4 bucket sends 16-byte aligned weights to the one-launch kernel.  The same bucket
    with a weight at an address that is not (a view into a larger allocation) must not reuse it."""
    w = I.weights(64, 512, seed=11).to(cuda)
    name = [(L.format(0) + "mlp.experts.linear_fc2.weight0", "model.layers.0.mlp.experts.0.down_proj.weight")]
    params = [(name[0][0], [(name[0][1], w)])]
    conv = B.BucketConverter(None, INT4_CFG)
    _same_as_loop(conv.convert(params, bucket_id=0), B.per_param_loop(None, params, INT4_CFG))
    big = torch.zeros(64 * 512 + 4, dtype=torch.bfloat16, device=cuda)
    shifted = big[4:].view(64, 512)
    shifted.copy_(w)
    assert shifted.data_ptr() % 16 == 8
    params2 = [(name[0][0], [(name[0][1], shifted)])]
    out = conv.convert(params2, bucket_id=0)
    _same_as_loop(out, B.per_param_loop(None, params, INT4_CFG))
    assert conv.plan_builds == 2


def test_bucket_with_an_odd_sized_member_is_the_plain_concatenation(cuda):
    """FlattenedTensorBucket packs back to back without padding.  When that puts a wider tensor at an offset that is not
    a multiple of its element size, the converter must still produce exactly that buffer (no gap bytes, cumulative
    offsets): it runs the per-parameter loop and concatenates."""
    params = [("module.module.x.flags", [("flags", torch.arange(7, device=cuda, dtype=torch.uint8))]),
              (L.format(0) + "self_attention.linear_proj.weight", [("model.layers.0.self_attn.o_proj.weight", I.weights(256, 128, seed=1).to(cuda))]),
              ("module.module.x.norm", [("model.norm.weight", I.weights(1, 64, seed=2)[0].to(cuda))])]
    conv = B.BucketConverter(None, FP8_CFG)
    want = B.per_param_loop(None, params, FP8_CFG)
    for _ in range(2):
        out = conv.convert(params)
        flat = B.flatten_named_tensors(want)
        assert torch.equal(out.get_flattened_tensor(), flat.get_flattened_tensor())
        assert [(m.name, m.start_idx, m.end_idx) for m in out.metadata] == [(m.name, m.start_idx, m.end_idx) for m in flat.metadata]
        assert out.metadata[1].start_idx == 7 and out.metadata[2].start_idx == 7 + 256 * 128      # the scale sits at an odd offset
    assert conv.plan_builds == 1


def test_bucket_accepts_generators(cuda):
    params = _moe_layer(0, cuda, 990, experts=1)
    want = B.per_param_loop(None, params, FP8_CFG)
    conv = B.BucketConverter(None, FP8_CFG)
    for _ in range(2):
        lazy = ((mn, ((n, t) for n, t in cv)) for mn, cv in params)
        _same_as_loop(conv.convert(lazy, bucket_id="lazy"), want)


def test_fp8_bucket_odd_members(cuda):
    # ragged shapes, a strided quantised member (generic tiles), a non-contiguous pass-through, members whose byte
    # sizes put the next one at 4-byte and 2-byte aligned offsets (every tensor still at a multiple of its element
    # size), an empty tensor, an fp32 weight and a *_scale entry that the expert rule drops
    w = I.weights(300, 200, seed=1).to(cuda)
    wide = I.weights(264, 520, seed=2).to(cuda)
    params = [
        ("module.module.decoder.layers.0.mlp.router.expert_bias", [("model.layers.0.mlp.gate.e_score_correction_bias", torch.arange(3, device=cuda, dtype=torch.float32))]),
        (L.format(0) + "self_attention.linear_proj.weight", [("model.layers.0.self_attn.o_proj.weight", w)]),
        ("module.module.x.odd", [("odd.bf16", I.weights(1, 3, seed=3)[0].to(cuda))]),
        (L.format(0) + "mlp.linear_fc2.weight", [("model.layers.0.mlp.down_proj.weight", wide[:263, 8:516][:, ::2])]),
        ("module.module.x.strided", [("strided.pass", wide.t())]),
        ("module.module.x.empty", [("empty", torch.empty(0, 4, device=cuda, dtype=torch.bfloat16))]),
        (L.format(0) + "mlp.linear_fc1.weight", [("model.layers.0.mlp.gate_proj.weight", I.weights(7, 7168, seed=4).to(cuda)),
                                                 ("model.layers.0.mlp.up_proj.weight", I.weights(129, 128, seed=5).to(cuda).float())]),
        (L.format(0) + "mlp.experts.linear_fc1.weight0", [("model.layers.0.mlp.experts.0.gate_proj.weight", I.weights(128, 128, seed=6).to(cuda)),
                                                         ("model.layers.0.mlp.experts.0.gate_proj.weight_scale", torch.ones(1, device=cuda))]),
    ]
    conv = B.BucketConverter(None, FP8_CFG)
    want = B.per_param_loop(None, params, FP8_CFG)
    assert "model.layers.0.mlp.experts.0.gate_proj.weight_scale" not in [n for n, _ in want]
    for _ in range(2):
        _same_as_loop(conv.convert(params), want)
    assert conv.plan_builds == 1
    o, so = C.fp8_block_quant(wide[:263, 8:516][:, ::2].cpu(), (128, 128), 1)
    out = conv.convert(params)
    assert out.launches > 1 and not conv._layouts[next(iter(conv._layouts))].fallback       # the one-launch path plus the late members
    starts = {m.name: m.start_idx for m in out.metadata}
    assert starts["model.layers.0.mlp.down_proj.weight"] % 4 == 2 and starts["model.layers.0.self_attn.o_proj.weight"] % 16 == 12
    named = dict(out.reconstruct_tensors())
    assert torch.equal(named["model.layers.0.mlp.down_proj.weight"].cpu().view(torch.uint8), o)


def test_bucket_other_configurations(cuda):
    params = _moe_layer(0, cuda, 300, experts=2)
    for cfg in (None, {"quant_method": "awq"}, {**FP8_CFG, "weight_block_size": None}, {**FP8_CFG, "weight_block_size": [64, 32]}):
        conv = B.BucketConverter(None, cfg)
        _same_as_loop(conv.convert(params), B.per_param_loop(None, params, cfg))
    assert B.BucketConverter(None, FP8_CFG).convert([]).get_flattened_tensor().numel() == 0
    assert B.quantize_bucket(None, [("m", [])], FP8_CFG).get_metadata() == []
    with pytest.raises(ValueError):
        B.BucketConverter(None, FP8_CFG).convert(params, out=torch.empty(16, dtype=torch.uint8, device=cuda))


def test_int4_bucket_equals_per_param_loop_and_oracle(cuda):
    params = _moe_layer(0, cuda, 400) + _moe_layer(3, cuda, 500) + [
        ("module.module.output_layer.weight", [("lm_head.weight", I.weights(640, 256, seed=9).to(cuda))])]
    conv = B.BucketConverter(None, INT4_CFG)
    out = conv.convert(params)
    want = B.per_param_loop(None, params, INT4_CFG)
    _same_as_loop(out, want)
    assert out.launches == 1
    assert torch.equal(out.get_flattened_tensor(), B.flatten_named_tensors(want).get_flattened_tensor())
    named = dict(out.reconstruct_tensors())
    n_q = 0
    for mn, cv in params:
        for n, t in cv:
            if ".experts." in n:
                po, so, _ = C.int4_pack_layer(t.cpu().contiguous(), 128, True)
                assert torch.equal(named[n.replace(".weight", ".weight_packed")].cpu(), po), n
                assert I.same_bits(named[n.replace(".weight", ".weight_scale")].cpu(), so), n
                assert named[n.replace(".weight", ".weight_shape")].tolist() == list(t.shape)
                n_q += 1
            elif "self_attn" in n or n == "lm_head.weight":
                assert I.same_bits(named[n].cpu(), t.cpu())              # ignored by the rules: passes through
    assert n_q == 18
    _same_as_loop(conv.convert(params), want)
    assert conv.plan_builds == 1


def test_int4_bucket_asymmetric_and_other_groups(cuda):
    params = _moe_layer(0, cuda, 600, experts=2)
    asym = {**INT4_CFG, "config_groups": {"group_0": {"weights": {"group_size": 128, "symmetric": False}}}}
    g32 = {**INT4_CFG, "config_groups": {"group_0": {"weights": {"group_size": 32, "symmetric": True}}}}
    g256 = {**INT4_CFG, "config_groups": {"group_0": {"weights": {"group_size": 256, "symmetric": True}}}, "ignore": []}
    everything = {**INT4_CFG, "ignore": []}       # nothing ignored: the fp32 router goes through the per-tensor path
    for cfg in (asym, g32, everything):
        conv = B.BucketConverter(None, cfg)
        for _ in range(2):
            out = conv.convert(params)
            _same_as_loop(out, B.per_param_loop(None, params, cfg))
        assert conv.plan_builds == 1
        if cfg is asym:
            assert out.launches == 2        # the pack kernel (with the pass-through copies) + the zero-point packer
            assert [m.name.rsplit(".", 1)[1] for m in out.metadata if ".experts.0.gate_proj" in m.name] == [
                "weight_zero_point", "weight_packed", "weight_scale", "weight_shape"]
    # rows that are not a multiple of 8 under an asymmetric configuration go through the per-tensor path, with whatever
    # the reference's zeros.reshape(-1, M // 8, 8) makes of them: a [3, 1] tensor for 12 x 256, an error for 12 x 128
    odd = [(L.format(0) + "mlp.experts.linear_fc2.weight0", [("model.layers.0.mlp.experts.0.down_proj.weight", I.weights(12, 256, seed=3).to(cuda))])]
    _same_as_loop(B.BucketConverter(None, asym).convert(odd), B.per_param_loop(None, odd, asym))
    bad = [(L.format(0) + "mlp.experts.linear_fc2.weight0", [("model.layers.0.mlp.experts.0.down_proj.weight", I.weights(12, 128, seed=3).to(cuda))])]
    with pytest.raises(RuntimeError, match="invalid for input of size"):
        B.per_param_loop(None, bad, asym)
    with pytest.raises(RuntimeError, match="invalid for input of size"):
        B.BucketConverter(None, asym).convert(bad)
    one = [(L.format(0) + "mlp.experts.linear_fc2.weight0", [("model.layers.0.mlp.experts.0.down_proj.weight", I.weights(64, 512, seed=3).to(cuda))])]
    _same_as_loop(B.BucketConverter(None, g256).convert(one), B.per_param_loop(None, one, g256))


def test_quantize_params_fp8_groups_one_parameter_into_one_launch(cuda):
    # the per-parameter entry point puts q/k/v (or gate/up) of one parameter into one launch whose descriptors travel
    # in the kernel arguments: no table, nothing cached, and the same bytes wherever the tensors live
    from slime_amd import processors

    params = _moe_layer(0, cuda, 700, experts=1)
    for mn, cv in (params[1], params[4]):                     # q/k/v (3 tensors), gate/up (2 chunk views)
        first = processors.quantize_params_fp8(None, mn, cv, FP8_CFG)
        moved = [(n, t.clone()) for n, t in cv]
        again = processors.quantize_params_fp8(None, mn, moved, FP8_CFG)
        assert [n for n, _ in first] == [n for n, _ in again] and len(first) == 2 * len(cv)
        for (n0, a), (_, sa), (n1, b), (_, sb), (_, t) in zip(first[::2], first[1::2], again[::2], again[1::2], cv):
            qo, so = C.fp8_block_quant(t.cpu().contiguous(), (128, 128), 1)
            assert n0 == n1 and torch.equal(a.cpu().view(torch.uint8), qo) and torch.equal(b.cpu().view(torch.uint8), qo)
            assert torch.equal(sa.cpu().view(torch.int32), so.view(torch.int32)) and I.same_bits(sa, sb)
            assert a.data_ptr() != b.data_ptr()          # fresh outputs on every call, like the reference
    # more tensors than one launch's kernel arguments hold: split over launches, same results
    many = [(f"model.layers.0.self_attn.p{i}.weight", I.weights(130 + i, 264, seed=i).to(cuda)) for i in range(6)]
    outs = processors.quantize_params_fp8(None, L.format(0) + "self_attention.linear_qkv.weight", many, FP8_CFG)
    for (n, t), (nq, q), (ns, s) in zip(many, outs[::2], outs[1::2]):
        qo, so = C.fp8_block_quant(t.cpu(), (128, 128), 1)
        assert nq == n and ns == n.replace(".weight", ".weight_scale_inv")
        assert torch.equal(q.cpu().view(torch.uint8), qo) and torch.equal(s.cpu().view(torch.int32), so.view(torch.int32))


def test_fp8_bucket_tensors_off_the_lines_take_the_plain_store_launch(cuda):
    """Back-to-back packing decides where every tensor starts.  While code rows start on 64-byte boundaries the bucket is ONE
    launch; a matrix whose scales are not a multiple of 64 bytes long (280 tiles here, the shape class of DeepSeek-V3's
    [576, 7168] kv_a_proj_with_mqa) moves everything after it off the lines, and those tensors go through the launch with
    plain stores - same bytes, two launches."""
    name = lambda i: (L.format(0) + f"mlp.experts.linear_fc2.weight{i}", f"model.layers.0.mlp.experts.{i}.down_proj.weight")
    friendly = [(name(i)[0], [(name(i)[1], I.weights(256, 2048, seed=40 + i).to(cuda))]) for i in range(3)]
    conv = B.BucketConverter(None, FP8_CFG)
    out = conv.convert(friendly)
    assert out.launches == 1 and all(m.start_idx % 64 == 0 for m in out.metadata)
    _same_as_loop(out, B.per_param_loop(None, friendly, FP8_CFG))
    shifting = friendly[:1] + [(name(7)[0], [(name(7)[1], I.weights(576, 1024, seed=47).to(cuda))])] + friendly[1:]
    out = conv.convert(shifting)
    starts = [m.start_idx % 64 for m in out.metadata]
    assert out.launches == 2 and starts[:4] == [0, 0, 0, 0] and starts[4] == 32          # 5 x 8 tiles: 160 bytes of scales
    want = B.per_param_loop(None, shifting, FP8_CFG)
    _same_as_loop(out, want)
    named = dict(out.reconstruct_tensors())
    for mn, cv in shifting:
        for n, t in cv:
            qo, so = C.fp8_block_quant(t.cpu(), (128, 128), 1)
            assert torch.equal(named[n].cpu().view(torch.uint8), qo), n
            assert torch.equal(named[n.replace(".weight", ".weight_scale_inv")].cpu().view(torch.int32), so.view(torch.int32)), n
    # 8 bytes of a pass-through tensor ahead: every tile of the matrix is off the lines, the copy item stays in the first launch
    ahead = [("module.module.x.pair", [("pair.f32", torch.ones(2, device=cuda))])] + friendly[:1]
    out = conv.convert(ahead)
    assert out.launches == 2 and out.metadata[1].start_idx == 8
    _same_as_loop(out, B.per_param_loop(None, ahead, FP8_CFG))


@pytest.mark.parametrize("width", [4, 5, 8])
def test_resolve_items_through_the_c_abi(cuda, width):
    """wq_bucket_resolve_items: items = template with bases[owner] added to word 0, nothing else touched."""
    from slime_amd import _lib
    from slime_amd._tables import ResolvedTable

    g = I.gen(width)
    n, n_bases = 10_007, 37
    template = torch.randint(-2 ** 40, 2 ** 40, (n, width), generator=g, dtype=torch.int64)
    owner = torch.randint(0, n_bases, (n,), generator=g, dtype=torch.int64)
    bases = torch.randint(0, 2 ** 47, (n_bases,), generator=g, dtype=torch.int64)
    want = template.clone()
    want[:, 0] += bases[owner]
    table = ResolvedTable(template, owner, n_bases, cuda)
    table.resolve(bases.numpy(), tag="a")
    assert torch.equal(table.items.cpu(), want) and torch.equal(table.template.cpu(), template) and table.resolved_for == "a"
    other = bases + 4096                                        # the same inputs somewhere else: five resolves cycle the staging
    for _ in range(5):
        table.resolve(other.numpy(), tag="b")
    want[:, 0] += 4096
    assert torch.equal(table.items.cpu(), want) and table.resolves == 6
    lib = _lib.load()
    assert lib.wq_bucket_resolve_items(table.template.data_ptr(), table.owner.data_ptr(), table.bases.data_ptr(), n, width,
                                       table.template.data_ptr(), None) == -4          # in place: refused
    assert lib.wq_bucket_resolve_items(table.template.data_ptr(), table.owner.data_ptr(), table.bases.data_ptr(), n, 17,
                                       table.items.data_ptr(), None) == -2


def _random_bucket(seed, cuda, int4):
    """A bucket of random composition: expert / dense / attention weights of ragged and aligned shapes (row-chunk views of a
    fused parameter, now and then a strided or transposed view, a float16 or float32 weight, an empty one), 1-D members of
    odd lengths between them (they move their successors off the 16-byte and 128-byte grids) and fp32 router weights."""
    g = torch.Generator().manual_seed(seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    pick = lambda xs: xs[r(0, len(xs) - 1)]
    # mostly shapes that keep the bucket on the one-launch kernels (INT4: rows a multiple of 8 for the zero points; FP8: a
    # multiple of 4 codes so that the fp32 scales behind them can be addressed), now and then one that does not
    cols = [128, 256, 384, 512, 1024] if int4 else [128, 200, 256, 384, 520, 1000, 2052, 132, 4100] + [7, 2049] * (r(0, 5) == 0)
    rows = [8, 128, 136, 256, 304, 512, 1000] + ([1, 7, 129, 513] if not int4 or r(0, 7) == 0 else [])
    params = []
    for k in range(r(3, 14)):
        layer, kind = r(0, 3), r(0, 9)
        hf, mc = f"model.layers.{layer}.", L.format(layer)
        w = lambda: I.weights(pick(rows), pick(cols), seed=seed * 100 + k).to(cuda)
        if kind <= 3:                                             # an expert's fused fc1 -> gate, up; or its fc2
            e = r(0, 7)
            if r(0, 1):
                fc1 = I.weights(2 * pick(rows), pick(cols), seed=seed * 100 + k).to(cuda)
                gate, up = fc1.chunk(2, dim=0)
                params.append((mc + f"mlp.experts.linear_fc1.weight{e}", [(hf + f"mlp.experts.{e}.gate_proj.weight", gate),
                                                                         (hf + f"mlp.experts.{e}.up_proj.weight", up)]))
            else:
                params.append((mc + f"mlp.experts.linear_fc2.weight{e}", [(hf + f"mlp.experts.{e}.down_proj.weight", w())]))
        elif kind == 4:
            params.append((mc + "self_attention.linear_proj.weight", [(hf + "self_attn.o_proj.weight", w())]))
        elif kind == 5:                                           # a dense MLP weight in another dtype, or a view with strides
            t = w()
            how = r(0, 4)
            if how == 0 and not int4: t = t.float()
            elif how == 1 and not int4: t = t.half()
            elif how == 2 and not int4 and t.shape[1] >= 16: t = t[:, 4:t.shape[1] - 4]
            elif how == 3 and not int4: t = t.t()
            params.append((mc + "mlp.linear_fc2.weight", [(hf + "mlp.down_proj.weight", t)]))
        elif kind == 6:
            params.append((mc + "mlp.router.weight", [(hf + "mlp.gate.weight", I.weights(r(1, 9), pick(cols), seed=k).to(cuda).float())]))
        elif kind == 7:                                           # a 1-D member of odd length: bf16, fp32 or fp16
            v = I.weights(1, r(1, 301) * pick([1, 2, 8]), seed=k)[0].to(cuda)
            params.append((mc + "self_attention.linear_qkv.layer_norm_weight", [(hf + "input_layernorm.weight", pick([v, v.float(), v.half()]))]))
        elif kind == 8:
            params.append((f"module.module.x.empty{k}", [(f"empty{k}", torch.empty(0, pick(cols), device=cuda, dtype=torch.bfloat16))]))
        else:
            params.append((f"module.module.x.pass{k}", [(f"model.pass{k}.weight", w().t() if r(0, 1) and not int4 else w())]))
    return params


def _same_bytes_as_loop(bucket, want):
    """Buffer and metadata equal the plain concatenation of the loop's tensors; members read back where torch can view them
    (an offset that is no multiple of a member's element size cannot be viewed, in the reference's bucket class either)."""
    ref = B.flatten_named_tensors(want)
    assert bucket.get_metadata() == ref.get_metadata()
    assert torch.equal(bucket.get_flattened_tensor(), ref.get_flattened_tensor())
    if all(m.start_idx % torch.empty(0, dtype=m.dtype).element_size() == 0 for m in ref.get_metadata()):
        _same_as_loop(bucket, want)


RANDOM_CFGS = {"fp8": FP8_CFG, "fp8_64x32": {**FP8_CFG, "weight_block_size": [64, 32]}, "int4": INT4_CFG,
               "int4_asym": {**INT4_CFG, "config_groups": {"group_0": {"weights": {"group_size": 128, "symmetric": False}}}},
               "int4_g32": {**INT4_CFG, "config_groups": {"group_0": {"weights": {"group_size": 32, "symmetric": True}}}}}


@pytest.mark.parametrize("seed", range(10))
@pytest.mark.parametrize("cfg", list(RANDOM_CFGS))
def test_random_buckets_equal_the_per_param_loop(cuda, cfg, seed):
    """Buckets of random composition: first sync, second sync on the cached layout, third sync with every input at a new
    address, fourth into the caller's buffer - each identical to the per-parameter loop, also where that loop refuses
    (a weight whose columns are no multiple of the INT4 group)."""
    qcfg = RANDOM_CFGS[cfg]
    params = _random_bucket(seed, cuda, cfg.startswith("int4"))
    conv = B.BucketConverter(None, qcfg)
    try:
        want = B.per_param_loop(None, params, qcfg)
    except Exception as e:
        with pytest.raises(type(e)):
            conv.convert(params, bucket_id=seed)
        return
    _same_bytes_as_loop(conv.convert(params, bucket_id=seed), want)
    _same_bytes_as_loop(conv.convert(params, bucket_id=seed), want)
    pad = [torch.empty(r, device=cuda) for r in (3, 17, 33)]                # moves the clones off the originals' alignment pattern
    moved = [(mn, [(n, t.clone(memory_format=torch.preserve_format) if t.is_contiguous() else t) for n, t in cv]) for mn, cv in params]
    _same_bytes_as_loop(conv.convert(moved, bucket_id=seed), want)
    del pad
    if want:
        total = conv.convert(params, bucket_id=seed).get_flattened_tensor().numel()
        buf = torch.empty(total + 128, dtype=torch.uint8, device=cuda)
        buf = buf[(-buf.data_ptr()) % 128:][:total]
        out = conv.convert(params, out=buf, bucket_id=seed)
        assert out.get_flattened_tensor().data_ptr() == buf.data_ptr()
        _same_bytes_as_loop(out, want)
