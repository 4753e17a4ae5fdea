"""Trainer-native layouts: Megatron's by-KV-group interleaved QKV and fused [gate; up]
enter the planner as virtual tensors made of row bands.  Vectors and geometries are those
of the reference's tests/test_reshard_megatron_gqa.py:65-76,154-258 (fused = arange, the
expected q/k/v is the concatenation of each group's rows)."""

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

from helpers import apply_plan_numpy
from modelexpress_amd import megatron
from modelexpress_amd._lib import ERR_COVERAGE, MxpError
from modelexpress_amd.engine import Checkpoint, ParamSpec, PlacementPlan, VirtualTensor

HF = ("attn.q_proj.weight", "attn.k_proj.weight", "attn.v_proj.weight")


def _fused(q_heads, kv_heads, head_dim, hidden):
    rows = (q_heads + 2 * kv_heads) * head_dim
    return torch.arange(rows * hidden, dtype=torch.float32).reshape(rows, hidden)


def _expected_hf(fused, q_heads, kv_heads, head_dim):
    # tests/test_reshard_megatron_gqa.py:65-76
    q_rows = (q_heads // kv_heads) * head_dim
    group_rows = q_rows + 2 * head_dim
    q, k, v = [], [], []
    for g in range(kv_heads):
        lo = g * group_rows
        q.append(fused[lo:lo + q_rows])
        k.append(fused[lo + q_rows:lo + q_rows + head_dim])
        v.append(fused[lo + q_rows + head_dim:lo + group_rows])
    return tuple(torch.cat(p) for p in (q, k, v))


def _b(t):
    return t.contiguous().reshape(-1).view(torch.uint8).numpy().tobytes()


GEOMETRIES = [(32, 4, 2, 4), (32, 4, 1, 4), (64, 2, 8, 8), (24, 6, 4, 2)]  # (q_heads, kv_heads, trainer tp, head_dim)


@pytest.mark.parametrize("q_heads,kv_heads,src_tp,head_dim", GEOMETRIES)
def test_oracle_qkv_split_and_bands(oracle, q_heads, kv_heads, src_tp, head_dim):
    hidden = 3
    fused = _fused(q_heads, kv_heads, head_dim, hidden)
    want = _expected_hf(fused, q_heads, kv_heads, head_dim)
    got = oracle.megatron_qkv_split(oracle.OTensor.from_array(fused.numpy(), "F32"), q_heads, kv_heads, head_dim)
    assert [g.tobytes() for g in got] == [_b(w) for w in want]
    # the product's band list tiles the fused rows exactly once, in order
    bands = list(megatron.qkv_bands(head_dim, q_heads, kv_heads))
    pos = 0
    for _proj, start, rows, _dst in bands:
        assert start == pos
        pos += rows
    assert pos == fused.shape[0]
    for proj, total in zip((0, 1, 2), (q_heads * head_dim, kv_heads * head_dim, kv_heads * head_dim)):
        dst = sorted((d, r) for p, _s, r, d in bands if p == proj)
        assert dst[0][0] == 0 and all(a[0] + a[1] == b[0] for a, b in zip(dst, dst[1:])) and dst[-1][0] + dst[-1][1] == total


@pytest.mark.parametrize("q_heads,kv_heads,src_tp,head_dim", GEOMETRIES)
@pytest.mark.parametrize("dst_tp", [1, 2])
def test_planner_places_interleaved_qkv(oracle, mxp, tmp_path, q_heads, kv_heads, src_tp, head_dim, dst_tp):
    """Source: the fused tensor saved as `src_tp` row shards (one per trainer rank).
    Destination: a serving rank's fused qkv_proj under `dst_tp`-way tensor parallelism."""
    hidden = 3
    fused = _fused(q_heads, kv_heads, head_dim, hidden)
    local_rows = fused.shape[0] // src_tp
    tensors = {f"attn.linear_qkv.rank{r}": fused[r * local_rows:(r + 1) * local_rows].clone() for r in range(src_tp)}
    tensors["attn.norm.weight"] = torch.ones(hidden)
    save_file(tensors, str(tmp_path / "model.safetensors"))
    sources = [(f"attn.linear_qkv.rank{r}", r * local_rows, (r + 1) * local_rows) for r in range(src_tp)]
    virtuals = megatron.qkv_virtuals(sources, HF, hidden, head_dim=head_dim, q_heads=q_heads, kv_heads=kv_heads)
    q, k, v = _expected_hf(fused, q_heads, kv_heads, head_dim)
    ck = Checkpoint(str(tmp_path))
    for rank in range(dst_tp):
        qs, ks = q.shape[0] // dst_tp, k.shape[0] // dst_tp
        params = [ParamSpec("attn.qkv_proj.weight", "F32", (qs + 2 * ks, hidden)), ParamSpec("attn.norm.weight", "F32", (hidden,))]
        plan = PlacementPlan(ck, params, tp_size=dst_tp, tp_rank=rank, virtual_tensors=virtuals)
        got = apply_plan_numpy(ck, plan)
        want = torch.cat((q[rank * qs:(rank + 1) * qs], k[rank * ks:(rank + 1) * ks], v[rank * ks:(rank + 1) * ks]))
        assert got["attn.qkv_proj.weight"].tobytes() == _b(want)
        # the oracle route: assemble the virtual tensors from the same shards, then the MDL rules
        ow = dict(oracle.load_checkpoint(str(tmp_path)))
        weights = [(vt.name, oracle.assemble_virtual(vt.shape, "F32", [(ow[s], so, do, sh) for s, so, do, sh in vt.shards]))
                   for vt in virtuals] + [("attn.norm.weight", ow["attn.norm.weight"])]
        oparams = {p.name: oracle.OTensor.zeros(p.shape, p.dtype) for p in params}
        oracle.MdlOracle(oparams, dst_tp, rank).load_weights(weights)
        assert oparams["attn.qkv_proj.weight"].tobytes() == _b(want)
        assert all(w.kind == "fused" for w in plan.writes() if w.tensor.startswith("attn.linear_qkv"))


def test_gated_virtuals_and_coverage_gate(oracle, mxp, tmp_path):
    # aliases.py:116-168: two trainer ranks each hold [gate_local; up_local]
    gate = torch.arange(8 * 3, dtype=torch.float32).reshape(8, 3)
    up = gate + 100
    tensors = {f"mlp.linear_fc1.rank{r}": torch.cat((gate[4 * r:4 * r + 4], up[4 * r:4 * r + 4])) for r in range(2)}
    save_file(tensors, str(tmp_path / "model.safetensors"))
    ck = Checkpoint(str(tmp_path))
    virtuals = megatron.gated_virtuals([("mlp.linear_fc1.rank0", 0, 2), ("mlp.linear_fc1.rank1", 1, 2)],
                                       ("mlp.gate_proj.weight", "mlp.up_proj.weight"), (3,), global_rows=16)
    for rank in range(4):
        plan = PlacementPlan(ck, [ParamSpec("mlp.gate_up_proj.weight", "F32", (4, 3))], tp_size=4, tp_rank=rank,
                             virtual_tensors=virtuals)
        want = torch.cat((gate[2 * rank:2 * rank + 2], up[2 * rank:2 * rank + 2]))
        assert apply_plan_numpy(ck, plan)["mlp.gate_up_proj.weight"].tobytes() == _b(want)
    with pytest.raises(ValueError, match="gate_then_up"):
        megatron.gated_virtuals([], ("a", "b"), (3,), global_rows=16, order="up_then_gate")
    # a missing publisher: the needed box is not covered -> nothing is planned
    partial = [VirtualTensor(v.name, v.shape, v.shards[:1]) for v in virtuals]
    with pytest.raises(MxpError, match="shards cover") as e:
        PlacementPlan(ck, [ParamSpec("mlp.gate_up_proj.weight", "F32", (16, 3))], virtual_tensors=partial, allow_unmapped=True)
    assert e.value.code == ERR_COVERAGE
    # ranks that need only the covered half still plan
    PlacementPlan(ck, [ParamSpec("mlp.gate_up_proj.weight", "F32", (4, 3))], tp_size=4, tp_rank=0, virtual_tensors=partial,
                  allow_unmapped=True)
    with pytest.raises(oracle.CoverageError):
        ow = dict(oracle.load_checkpoint(str(tmp_path)))
        oracle.assemble_virtual(partial[0].shape, "F32", [(ow[s], so, do, sh) for s, so, do, sh in partial[0].shards])
    with pytest.raises(MxpError, match="not in the checkpoint"):
        PlacementPlan(ck, [], virtual_tensors=[VirtualTensor("x", (2, 3), (("nope", (0, 0), (0, 0), (2, 3)),))],
                      allow_unmapped=True, allow_uncovered=True)


def test_reference_alias_vectors():
    """The reference's own alias cases (tests/test_reshard_megatron.py:345-470), as virtual-tensor shards
    ``(source, offset in the source, offset in the HF tensor, shape)``."""
    from modelexpress_amd.megatron import gated_virtuals, qkv_virtuals

    # :345-368 a [gate; up] shard of TP rank 1 of 2, local (8, 4) of global (16, 4): gate and up are (8, 4)
    # globally, this rank's halves are (4, 4) at rows 4.., read from local rows 0 and 4
    gate, up = gated_virtuals([("linear_fc1.weight", 1, 2)], ("gate_proj.weight", "up_proj.weight"), (4,), global_rows=16)
    assert gate.shape == up.shape == (8, 4)
    assert gate.shards == (("linear_fc1.weight", (0, 0), (4, 0), (4, 4)),)
    assert up.shards == (("linear_fc1.weight", (4, 0), (4, 0), (4, 4)),)
    # :372-417 the storage order must be stated and must be gate-then-up
    with pytest.raises(ValueError, match="gate_then_up"):
        gated_virtuals([("linear_fc1.weight", 1, 2)], ("gate_proj.weight", "up_proj.weight"), (4,), global_rows=16, order="up_then_gate")
    # :443-475 fused QKV rows 12..24 of 24 (TP rank 1 of 2; 4 local query heads, 1 local KV head, head_dim 2):
    # q is (16, 4) globally and this rank's 8 rows land at row 8 from local row 0; k and v are (4, 4) and
    # this rank's 2 rows land at row 2, from local rows 8 and 10
    q, k, v = qkv_virtuals([("linear_qkv.weight", 12, 24)], ("q_proj.weight", "k_proj.weight", "v_proj.weight"), 4,
                           head_dim=2, q_heads=8, kv_heads=2)
    assert (q.shape, k.shape, v.shape) == ((16, 4), (4, 4), (4, 4))
    assert q.shards == (("linear_qkv.weight", (0, 0), (8, 0), (8, 4)),)
    assert k.shards == (("linear_qkv.weight", (8, 0), (2, 0), (2, 4)),)
    assert v.shards == (("linear_qkv.weight", (10, 0), (2, 0), (2, 4)),)
    # :503-527 a shard range beyond the global extent is rejected
    with pytest.raises(ValueError, match="row interval"):
        qkv_virtuals([("linear_qkv.weight", 12, 26)], ("q", "k", "v"), 4, head_dim=2, q_heads=8, kv_heads=2)
