"""The reference's own destination-map vectors, run through BOTH the CPU oracle and the
product planner (C++, via the C ABI; its boxes interpreted with numpy on the host).

Each test restates one test of modelexpress_client/python/tests/test_mdl_tp.py or
test_mdl_fp8.py (cited), with the checkpoint written by the third-party safetensors
writer so the product's parser is exercised on files it did not write itself.
"""

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

from helpers import apply_plan_numpy
from modelexpress_amd._lib import MxpError, ERR_COVERAGE, ERR_UNSUPPORTED
from modelexpress_amd.engine import Checkpoint, ParamSpec, PlacementPlan

F8 = torch.float8_e4m3fn
ST = {torch.float32: "F32", F8: "F8_E4M3", torch.int64: "I64", torch.bfloat16: "BF16"}


def _bytes(t: torch.Tensor) -> bytes:
    return t.contiguous().reshape(-1).view(torch.uint8).numpy().tobytes()


def _run_both(oracle, tmp_path, weights, params, *, tp_size=1, tp_rank=0, stacked=None, experts=None,
              expert_local=None, strict=True, **plan_kw):
    """weights: [(name, torch tensor)], params: {name: (dtype, shape)} -> {name: bytes} from both sides."""
    path = tmp_path / f"ck_{tp_rank}"
    path.mkdir(exist_ok=True)
    save_file({n: t.contiguous() for n, t in weights}, str(path / "model.safetensors"))
    # oracle
    OT = oracle.OTensor
    oparams = {n: OT.zeros(shape, dt) for n, (dt, shape) in params.items()}
    ow = dict(oracle.load_checkpoint(str(path)))
    m = oracle.MdlOracle(oparams, tp_size, tp_rank, stacked, [e[:4] for e in experts] if experts else None,
                         expert_local)
    m.load_weights([(n, ow[n]) for n, _ in weights], strict_params=strict)
    want = {n: p.tobytes() for n, p in oparams.items()}
    # product planner
    ck = Checkpoint(str(path))
    specs = [ParamSpec(n, dt, tuple(shape)) for n, (dt, shape) in params.items()]
    plan = PlacementPlan(ck, specs, tp_size=tp_size, tp_rank=tp_rank, stacked_params_mapping=stacked,
                         expert_mapping=experts, allow_uncovered=not strict, **plan_kw)
    got = {n: v.tobytes() for n, v in apply_plan_numpy(ck, plan).items()}
    assert got == want
    return want, plan


def test_tp_local_tensor_axis_zero_and_one(oracle, tmp_path):
    # test_mdl_tp.py:28-39: arange(24) as (6,4) rank 1 -> rows 3..5; as (4,6) -> cols 3..5
    a = torch.arange(24).reshape(6, 4)
    b = torch.arange(24).reshape(4, 6)
    want, plan = _run_both(oracle, tmp_path, [("a.weight", a), ("b.weight", b)],
                           {"a.weight": ("I64", (3, 4)), "b.weight": ("I64", (4, 3))}, tp_size=2, tp_rank=1)
    assert want["a.weight"] == _bytes(a[3:6])
    assert want["b.weight"] == _bytes(b[:, 3:6])
    by = {w.tensor: w for w in plan.writes()}
    assert by["a.weight"].paired_runs == 1 and by["b.weight"].paired_runs == 4  # slice_plan.py:259-294


def test_tp_shape_compatibility_requires_one_sharded_dimension(oracle, mxp, tmp_path):
    # test_mdl_tp.py:42-47
    m = oracle.MdlOracle({}, tp_size=2, tp_rank=1)
    assert m.tp_shape_compatible((6, 4), (3, 4)) and m.tp_shape_compatible((4, 6), (4, 3))
    assert not m.tp_shape_compatible((6, 8), (3, 4)) and not m.tp_shape_compatible((5, 4), (3, 4))
    for shape in [(6, 8), (5, 4)]:
        save_file({"w.weight": torch.zeros(shape)}, str(tmp_path / "model.safetensors"))
        with pytest.raises(MxpError) as e:
            PlacementPlan(Checkpoint(str(tmp_path)), [ParamSpec("w.weight", "F32", (3, 4))], tp_size=2, tp_rank=1)
        assert e.value.code == ERR_COVERAGE


@pytest.mark.parametrize("rank", [0, 1])
def test_premerged_gate_up_is_sharded_per_member(oracle, tmp_path, rank):
    # test_mdl_tp.py:50-81
    source = torch.arange(16).reshape(8, 2)
    want, plan = _run_both(oracle, tmp_path, [("mlp.gate_up_proj.weight", source)],
                           {"mlp.gate_up_proj.weight": ("I64", (4, 2))}, tp_size=2, tp_rank=rank)
    gate = source[rank * 2:(rank + 1) * 2]
    up = source[4 + rank * 2:4 + (rank + 1) * 2]
    assert want["mlp.gate_up_proj.weight"] == _bytes(torch.cat((gate, up)))
    assert {w.kind for w in plan.writes()} == {"premerged"}


def test_fp8_direct_weight_and_scale_alias(oracle, tmp_path):
    # test_mdl_fp8.py:31-48
    weight = torch.tensor([[1, 2], [3, 4]], dtype=torch.float32).to(F8)
    scale = torch.tensor([[0.25], [0.5]])
    want, plan = _run_both(oracle, tmp_path, [("proj.weight", weight), ("proj.weight_scale_inv", scale)],
                           {"proj.weight": ("F8_E4M3", (2, 2)), "proj.weight_scale": ("F32", (2, 1))})
    assert want["proj.weight"] == _bytes(weight) and want["proj.weight_scale"] == _bytes(scale)
    assert {w.kind for w in plan.writes()} == {"direct"}


def test_fp8_fused_qkv_gate_up_and_activation_scales(oracle, tmp_path):
    # test_mdl_fp8.py:50-108
    weights, exp_qkv, exp_qkv_s, exp_gu, exp_gu_s = [], [], [], [], []
    for index, (name, rows) in enumerate((("q_proj", 2), ("k_proj", 1), ("v_proj", 1))):
        value = torch.full((rows, 2), index + 1.0).to(F8)
        scale = torch.full((rows, 1), index + 0.25)
        weights += [(f"attn.{name}.weight", value), (f"attn.{name}.weight_scale_inv", scale),
                    (f"attn.{name}.input_scale", torch.tensor([index + 0.5]))]
        exp_qkv.append(value)
        exp_qkv_s.append(scale)
    for index, name in enumerate(("gate_proj", "up_proj")):
        value = torch.full((2, 2), index + 5.0).to(F8)
        scale = torch.full((2, 1), index + 1.25)
        weights += [(f"mlp.{name}.weight", value), (f"mlp.{name}.weight_scale_inv", scale),
                    (f"mlp.{name}.activation_scale", torch.tensor([index + 2.5]))]
        exp_gu.append(value)
        exp_gu_s.append(scale)
    params = {
        "attn.qkv_proj.weight": ("F8_E4M3", (4, 2)), "attn.qkv_proj.weight_scale": ("F32", (4, 1)),
        "attn.qkv_proj.input_scale": ("F32", (3,)), "mlp.gate_up_proj.weight": ("F8_E4M3", (4, 2)),
        "mlp.gate_up_proj.weight_scale": ("F32", (4, 1)), "mlp.gate_up_proj.input_scale": ("F32", (2,)),
    }
    want, plan = _run_both(oracle, tmp_path, weights, params)
    assert want["attn.qkv_proj.weight"] == _bytes(torch.cat(exp_qkv))
    assert want["attn.qkv_proj.weight_scale"] == _bytes(torch.cat(exp_qkv_s))
    assert want["attn.qkv_proj.input_scale"] == _bytes(torch.tensor([0.5, 1.5, 2.5]))
    assert want["mlp.gate_up_proj.weight"] == _bytes(torch.cat(exp_gu))
    assert want["mlp.gate_up_proj.weight_scale"] == _bytes(torch.cat(exp_gu_s))
    assert want["mlp.gate_up_proj.input_scale"] == _bytes(torch.tensor([2.5, 3.5]))
    assert len(plan.writes()) == len(weights) and {w.kind for w in plan.writes()} == {"fused"}


def _expert_mapping(local=0):
    prefix = "model.layers.0.mlp."
    return [(prefix + "experts.w13_", prefix + "experts.0.gate_proj.", 0, "w1", local),
            (prefix + "experts.w2_", prefix + "experts.0.down_proj.", 0, "w2", local),
            (prefix + "experts.w13_", prefix + "experts.0.up_proj.", 0, "w3", local)]


def test_fp8_expert_weight_scale_and_input_scale_layouts(oracle, tmp_path):
    # test_mdl_fp8.py:111-169
    gate = torch.full((2, 2), 3.0).to(F8)
    up = torch.full((2, 2), 7.0).to(F8)
    down = torch.full((2, 2), 9.0).to(F8)
    p = "model.layers.0.mlp.experts."
    weights = [
        (p + "0.gate_proj.weight", gate), (p + "0.gate_proj.weight_scale_inv", torch.full((2, 1), 0.3)),
        (p + "0.gate_proj.input_scale", torch.tensor([1.0])),
        (p + "0.up_proj.weight", up), (p + "0.up_proj.weight_scale_inv", torch.full((2, 1), 0.7)),
        (p + "0.up_proj.input_scale", torch.tensor([2.0])),
        (p + "0.down_proj.weight", down), (p + "0.down_proj.weight_scale_inv", torch.full((2, 1), 0.9)),
        (p + "0.down_proj.input_scale", torch.tensor([3.0])),
    ]
    params = {p + "w13_weight": ("F8_E4M3", (1, 4, 2)), p + "w2_weight": ("F8_E4M3", (1, 2, 2)),
              p + "w13_weight_scale": ("F32", (1, 4, 1)), p + "w2_weight_scale": ("F32", (1, 2, 1)),
              p + "w13_input_scale": ("F32", (1, 2)), p + "w2_input_scale": ("F32", (1, 1))}
    want, plan = _run_both(oracle, tmp_path, weights, params, experts=_expert_mapping())
    assert want[p + "w13_weight"] == _bytes(torch.cat((gate, up)))
    assert want[p + "w2_weight"] == _bytes(down)
    assert want[p + "w13_weight_scale"] == _bytes(torch.tensor([0.3, 0.3, 0.7, 0.7]))
    assert want[p + "w13_input_scale"] == _bytes(torch.tensor([1.0, 2.0]))
    assert want[p + "w2_input_scale"] == _bytes(torch.tensor([3.0]))
    assert len(plan.writes()) == len(weights) and {w.kind for w in plan.writes()} == {"expert"}


def test_fp8_tp2_direct_weight_and_block_scale(oracle, tmp_path):
    # test_mdl_fp8.py:202-228: global (4,2) -> local (2,2), block scale (2,1) -> (1,1)
    gw = torch.tensor([[1, 2], [3, 4], [5, 6], [7, 8]], dtype=torch.float32).to(F8)
    gs = torch.tensor([[0.25], [0.5]])
    for rank in (0, 1):
        want, _ = _run_both(oracle, tmp_path, [("proj.weight", gw), ("proj.weight_scale_inv", gs)],
                            {"proj.weight": ("F8_E4M3", (2, 2)), "proj.weight_scale": ("F32", (1, 1))},
                            tp_size=2, tp_rank=rank)
        assert want["proj.weight"] == _bytes(gw[rank * 2:rank * 2 + 2])
        assert want["proj.weight_scale"] == _bytes(gs[rank:rank + 1])


def test_fp8_tp2_expert_gate_up_weight_and_scale_shards(oracle, tmp_path):
    # test_mdl_fp8.py:279-356 (the TP2 collision: a global member has the local w13 shape)
    gate = torch.tensor([[1, 2], [3, 4], [5, 6], [7, 8]], dtype=torch.float32).to(F8)
    up = torch.tensor([[11, 12], [13, 14], [15, 16], [17, 18]], dtype=torch.float32).to(F8)
    down = torch.tensor([[21, 22, 23, 24], [25, 26, 27, 28]], dtype=torch.float32).to(F8)
    gate_s, up_s, down_s = torch.tensor([[0.1], [0.2]]), torch.tensor([[0.3], [0.4]]), torch.tensor([[0.5, 0.6]])
    p = "model.layers.0.mlp.experts."
    weights = [(p + "0.gate_proj.weight", gate), (p + "0.gate_proj.weight_scale_inv", gate_s),
               (p + "0.up_proj.weight", up), (p + "0.up_proj.weight_scale_inv", up_s),
               (p + "0.down_proj.weight", down), (p + "0.down_proj.weight_scale_inv", down_s)]
    params = {p + "w13_weight": ("F8_E4M3", (1, 4, 2)), p + "w2_weight": ("F8_E4M3", (1, 2, 2)),
              p + "w13_weight_scale": ("F32", (1, 2, 1)), p + "w2_weight_scale": ("F32", (1, 1, 1))}
    for rank in (0, 1):
        want, _ = _run_both(oracle, tmp_path, weights, params, tp_size=2, tp_rank=rank, experts=_expert_mapping())
        rows = slice(rank * 2, rank * 2 + 2)
        assert want[p + "w13_weight"] == _bytes(torch.cat((gate[rows], up[rows])))
        assert want[p + "w13_weight_scale"] == _bytes(torch.cat((gate_s[rank:rank + 1], up_s[rank:rank + 1])))
        assert want[p + "w2_weight"] == _bytes(down[:, rows])
        assert want[p + "w2_weight_scale"] == _bytes(down_s[:, rank:rank + 1])


def test_coverage_fails_closed(oracle, mxp, tmp_path):
    # test_mdl_fp8.py:359-367: a local fp8 scale parameter nothing writes -> refuse everything
    save_file({"proj.weight": torch.ones((2, 2)).to(F8)}, str(tmp_path / "model.safetensors"))
    specs = [ParamSpec("proj.weight", "F8_E4M3", (2, 2)), ParamSpec("proj.weight_scale", "F32", (2, 1))]
    for kw in ({}, {"allow_uncovered": True}):  # fp8 / scale parameters stay mandatory either way
        with pytest.raises(MxpError, match="uncovered local parameters") as e:
            PlacementPlan(Checkpoint(str(tmp_path)), specs, **kw)
        assert e.value.code == ERR_COVERAGE
    OT = oracle.OTensor
    oparams = {"proj.weight": OT.zeros((2, 2), "F8_E4M3"), "proj.weight_scale": OT.zeros((2, 1), "F32")}
    with pytest.raises(oracle.CoverageError, match="uncovered"):
        oracle.MdlOracle(oparams).load_weights(oracle.load_checkpoint(str(tmp_path)), strict_params=False)
    assert not any(oparams["proj.weight"].data.reshape(-1))


def test_unmapped_tensor_fails_before_any_write(oracle, mxp, tmp_path):
    # test_mdl_fp8.py:370-394
    save_file({"proj.weight": torch.full((2, 2), 5.0).to(F8), "proj.weight_scale_inv": torch.ones((2, 1)),
               "unknown.weight": torch.ones((1,)).to(F8)}, str(tmp_path / "model.safetensors"))
    specs = [ParamSpec("proj.weight", "F8_E4M3", (2, 2)), ParamSpec("proj.weight_scale", "F32", (2, 1))]
    with pytest.raises(MxpError, match="unmapped checkpoint tensors") as e:
        PlacementPlan(Checkpoint(str(tmp_path)), specs)
    assert e.value.code == ERR_COVERAGE
    plan = PlacementPlan(Checkpoint(str(tmp_path)), specs, allow_unmapped=True)
    assert len(plan.writes()) == 2


def test_expert_id_translation_failure_does_not_use_global_id(oracle, mxp, tmp_path):
    # test_mdl_fp8.py:397-434: local id unknown -> unmapped, never the global id
    p = "model.layers.0.mlp.experts."
    save_file({p + "0.down_proj.weight": torch.ones((2, 2)).to(F8),
               p + "0.down_proj.weight_scale_inv": torch.ones((2, 1))}, str(tmp_path / "model.safetensors"))
    specs = [ParamSpec(p + "w2_weight", "F8_E4M3", (1, 2, 2)), ParamSpec(p + "w2_weight_scale", "F32", (1, 2, 1))]
    mapping = [("model.layers.0.mlp.experts.w2_", "model.layers.0.mlp.experts.0.down_proj.", 0, "w2", -2)]
    with pytest.raises(MxpError, match="unmapped checkpoint tensors"):
        PlacementPlan(Checkpoint(str(tmp_path)), specs, expert_mapping=mapping)
    OT = oracle.OTensor
    oparams = {s.name: OT.zeros(s.shape, s.dtype) for s in specs}
    with pytest.raises(oracle.CoverageError, match="unmapped"):
        oracle.MdlOracle(oparams, expert_mapping=[m[:4] for m in mapping],
                         expert_local=lambda _f, _g: None).load_weights(oracle.load_checkpoint(str(tmp_path)))


def test_swizzled_or_mismatched_expert_layout_is_unmapped(mxp, tmp_path):
    # installer.py:833-843: a 4-D expert parameter cannot be addressed as [e, rows, cols]
    p = "model.layers.0.mlp.experts."
    save_file({p + "0.down_proj.weight": torch.ones((2, 2))}, str(tmp_path / "model.safetensors"))
    mapping = [("model.layers.0.mlp.experts.w2_", "model.layers.0.mlp.experts.0.down_proj.", 0, "w2", 0)]
    with pytest.raises(MxpError, match="unmapped checkpoint tensors"):
        PlacementPlan(Checkpoint(str(tmp_path)), [ParamSpec(p + "w2_weight", "F32", (1, 2, 1, 2))], expert_mapping=mapping)


def test_unaligned_fp8_block_slice_is_rejected(mxp, tmp_path):
    # The 128x128 rule the reference leaves implicit: a [256,256] fp8 weight with [2,2]
    # scale tiles cannot be split 4 ways on rows (64-row slices cut through a block).
    w = torch.zeros((256, 256)).to(F8)
    s = torch.ones((2, 2))
    save_file({"proj.weight": w, "proj.weight_scale_inv": s}, str(tmp_path / "model.safetensors"))
    specs = [ParamSpec("proj.weight", "F8_E4M3", (64, 256)), ParamSpec("proj.weight_scale_inv", "F32", (2, 2))]
    with pytest.raises(MxpError, match="128x128") as e:
        PlacementPlan(Checkpoint(str(tmp_path)), specs, tp_size=4, tp_rank=1, allow_unmapped=True, allow_uncovered=True)
    assert e.value.code == ERR_UNSUPPORTED
    # a 2-way split is block aligned and the scale follows by the same shape rule
    specs = [ParamSpec("proj.weight", "F8_E4M3", (128, 256)), ParamSpec("proj.weight_scale_inv", "F32", (1, 2))]
    plan = PlacementPlan(Checkpoint(str(tmp_path)), specs, tp_size=2, tp_rank=1)
    by = {w_.tensor: w_ for w_ in plan.writes()}
    assert by["proj.weight"].src_offset == 128 * 256 and by["proj.weight_scale_inv"].src_offset == 2 * 4


def test_dtype_mismatch_needs_the_cast_flag(mxp, tmp_path):
    save_file({"w.weight": torch.ones((4, 4))}, str(tmp_path / "model.safetensors"))
    with pytest.raises(MxpError, match="no conversion") as e:
        PlacementPlan(Checkpoint(str(tmp_path)), [ParamSpec("w.weight", "BF16", (4, 4))])
    assert e.value.code == ERR_UNSUPPORTED
    plan = PlacementPlan(Checkpoint(str(tmp_path)), [ParamSpec("w.weight", "BF16", (4, 4))], allow_cast=True)
    assert plan.writes()[0].cast == 1 and plan.writes()[0].row_bytes == 32


def test_widening_and_half_conversions_are_planned(mxp, oracle, tmp_path):
    # receiver.py:962-969 converts the served bf16 staging into an fp32 receive buffer
    w = torch.arange(32, dtype=torch.float32).reshape(4, 8)
    save_file({"a.weight": w.to(torch.bfloat16), "b.weight": w.to(torch.float16), "c.weight": w},
              str(tmp_path / "model.safetensors"))
    ck = Checkpoint(str(tmp_path))
    specs = [ParamSpec("a.weight", "F32", (4, 4)), ParamSpec("b.weight", "F32", (4, 4)), ParamSpec("c.weight", "F16", (4, 4))]
    with pytest.raises(MxpError, match="no conversion"):
        PlacementPlan(ck, specs, tp_size=2, tp_rank=1)
    plan = PlacementPlan(ck, specs, tp_size=2, tp_rank=1, allow_cast=True)
    by = {x.tensor: x for x in plan.writes()}
    # column slice [:, 4:8]: 4 rows; destination rows are 16 B (fp32) from 8 B of bf16 / fp16, 8 B (fp16) from 16 B of fp32
    a, b, c = by["a.weight"], by["b.weight"], by["c.weight"]
    assert (a.cast, a.rows, a.row_bytes, a.src_offset, a.src_pitch, a.dst_pitch) == (2, 4, 16, 8, 16, 16)
    assert (b.cast, b.rows, b.row_bytes, b.src_offset, b.src_pitch, b.dst_pitch) == (3, 4, 16, 8, 16, 16)
    assert (c.cast, c.rows, c.row_bytes, c.src_offset, c.src_pitch, c.dst_pitch) == (4, 4, 8, 16, 32, 8)
    # fp8-e4m3 into bf16 (receiver.py:258-261): one byte in, two out
    save_file({"d.weight": w.to(torch.float8_e4m3fn)}, str(tmp_path / "model.safetensors"))
    plan8 = PlacementPlan(Checkpoint(str(tmp_path)), [ParamSpec("d.weight", "BF16", (4, 4))], tp_size=2, tp_rank=1, allow_cast=True)
    d = plan8.writes()[0]
    assert (d.cast, d.rows, d.row_bytes, d.src_offset, d.src_pitch, d.dst_pitch) == (5, 4, 8, 4, 8, 8)
    assert apply_plan_numpy(Checkpoint(str(tmp_path)), plan8)["d.weight"].tobytes() == \
        w[:, 4:].to(torch.float8_e4m3fn).to(torch.bfloat16).contiguous().view(torch.uint8).numpy().tobytes()
    with pytest.raises(MxpError, match="no conversion"):  # pairs outside the table stay refused
        PlacementPlan(ck, [ParamSpec("a.weight", "F8_E4M3", (4, 8))], allow_cast=True, allow_uncovered=True, allow_unmapped=True)
    # the two 16-bit formats convert into each other through fp32 (copy_ semantics)
    p16 = PlacementPlan(ck, [ParamSpec("a.weight", "F16", (4, 8)), ParamSpec("b.weight", "BF16", (4, 8))], allow_cast=True,
                        allow_unmapped=True)
    assert {x.tensor: (x.cast, x.row_bytes, x.src_pitch) for x in p16.writes()} == {"a.weight": (7, 64, 64), "b.weight": (6, 64, 64)}


def _in_checkpoint_order(tmp_path, weights, tag):
    """`weights` in the order the product iterates the file the third-party writer produces (the
    oracle, like the reference's serial copy loop, installs in the order it is handed the tensors)."""
    path = tmp_path / f"order_{tag}"
    path.mkdir(exist_ok=True)
    save_file({n: t.contiguous() for n, t in weights}, str(path / "model.safetensors"))
    order = [t.name for t in Checkpoint(str(path)).tensors()]
    by = dict(weights)
    return [(n, by[n]) for n in order]


@pytest.mark.parametrize("tp", [1, 2])
def test_later_write_wins_where_two_tensors_meet_in_one_parameter(oracle, tmp_path, tp):
    """engines/vllm/refit/installer.py:419-424 installs tensor after tensor, so the later tensor's bytes stay
    where two of them map to the same bytes.  A checkpoint that holds gate_proj and up_proj AND a premerged
    gate_up_proj: each half of the parameter keeps what the iteration met last; the product settles that
    when it plans, so every destination byte still has one writer."""
    merged = torch.arange(32, dtype=torch.int64).reshape(16, 2)
    up = torch.arange(16, dtype=torch.int64).reshape(8, 2) + 1000
    gate = torch.arange(16, dtype=torch.int64).reshape(8, 2) + 2000
    local, half = 16 // tp, 8 // tp
    weights = _in_checkpoint_order(tmp_path, [("mlp.gate_up_proj.weight", merged), ("mlp.up_proj.weight", up),
                                              ("mlp.gate_proj.weight", gate)], f"m{tp}")
    for rank in range(tp):
        want, plan = _run_both(oracle, tmp_path, weights, {"mlp.gate_up_proj.weight": ("I64", (local, 2))},
                               tp_size=tp, tp_rank=rank)
        g_rows = u_rows = None
        for name, _t in weights:  # replay of the serial loop, half by half
            if name == "mlp.gate_up_proj.weight":
                g_rows, u_rows = merged[rank * half:(rank + 1) * half], merged[8 + rank * half:8 + (rank + 1) * half]
            elif name == "mlp.up_proj.weight":
                u_rows = up[rank * half:(rank + 1) * half]
            else:
                g_rows = gate[rank * half:(rank + 1) * half]
        assert want["mlp.gate_up_proj.weight"] == _bytes(torch.cat((g_rows, u_rows))), (tp, rank, [n for n, _ in weights])
        info = {q["name"]: q for q in plan.param_info()}["mlp.gate_up_proj.weight"]
        assert info["bytes_written"] == local * 2 * 8  # the size of the union, not the sum of the writes
        spans = sorted((w.dst_offset, w.dst_offset + (w.rows - 1) * w.dst_pitch + w.row_bytes) for w in plan.writes())
        assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))  # what is left is disjoint
        assert weights[-1][0] != "mlp.gate_up_proj.weight" and len(spans) < 2 + 2 * tp  # some write lost bytes


def test_two_experts_mapped_to_one_slot_leave_the_later_one(oracle, tmp_path):
    p = "model.layers.0.mlp."
    e0 = torch.full((2, 2), 3.0).to(F8)
    e1 = torch.full((2, 2), 5.0).to(F8)
    weights = _in_checkpoint_order(tmp_path, [(p + "experts.0.down_proj.weight", e0), (p + "experts.1.down_proj.weight", e1)], "ex")
    mapping = [(p + "experts.w2_", p + "experts.0.down_proj.", 0, "w2", 0), (p + "experts.w2_", p + "experts.1.down_proj.", 1, "w2", 0)]
    want, plan = _run_both(oracle, tmp_path, weights, {p + "experts.w2_weight": ("F8_E4M3", (1, 2, 2))}, experts=mapping,
                           expert_local=lambda _name, _gid: 0)
    assert want[p + "experts.w2_weight"] == _bytes(dict(weights)[weights[-1][0]])
    assert len(plan.writes()) == 1 and plan.writes()[0].tensor == weights[-1][0]


def test_expert_outside_the_rank_is_skipped_or_unmapped_on_request(tmp_path):
    """installer.py:708-710: an expert whose local id is negative has no destination; the reference's loaderless
    mode then refuses the load (installer.py:219-251), its normal mode hands the tensor to the stock loader.  The
    product skips it by default (each rank reads the whole checkpoint) and offers the refusal as a plan flag."""
    p = "model.layers.0.mlp."
    e0 = torch.full((2, 2), 3.0).to(F8)
    e1 = torch.full((2, 2), 5.0).to(F8)
    save_file({p + "experts.0.down_proj.weight": e0, p + "experts.1.down_proj.weight": e1}, str(tmp_path / "model.safetensors"))
    ck = Checkpoint(str(tmp_path))
    mapping = [(p + "experts.w2_", p + "experts.0.down_proj.", 0, "w2", 0), (p + "experts.w2_", p + "experts.1.down_proj.", 1, "w2", -1)]
    specs = [ParamSpec(p + "experts.w2_weight", "F8_E4M3", (1, 2, 2))]
    plan = PlacementPlan(ck, specs, expert_mapping=mapping)
    assert [w.tensor for w in plan.writes()] == [p + "experts.0.down_proj.weight"]
    assert apply_plan_numpy(ck, plan)[p + "experts.w2_weight"].tobytes() == _bytes(e0)
    with pytest.raises(MxpError, match="experts.1.down_proj.weight") as e:
        PlacementPlan(ck, specs, expert_mapping=mapping, nonlocal_experts_unmapped=True)
    assert e.value.code == ERR_COVERAGE
