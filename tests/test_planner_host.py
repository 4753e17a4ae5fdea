"""The product planner (C++, through the C ABI) against the CPU oracle, on the host:
its pitched-box writes are interpreted with numpy and compared byte for byte with the
oracle's parameter buffers.  No device work happens here."""

import numpy as np
import pytest

from helpers import apply_plan_numpy, cast_setup, make_plan, oracle_place, tiny_layouts
from modelexpress_amd import synth


@pytest.mark.parametrize("name", list(tiny_layouts()))
def test_plan_matches_oracle_for_every_rank(name, mxp, oracle, tmp_path):
    layout, tp, ep, shards, ck_kw = tiny_layouts()[name]
    ck_kw, param_dtype, cast, _ratio = cast_setup(ck_kw)
    synth.write_checkpoint(layout.checkpoint(**ck_kw), str(tmp_path), n_shards=shards, seed=3)
    for tp_rank in range(tp):
        for ep_rank in range(ep):
            if ep > 1 and ep_rank != tp_rank % ep:
                continue
            rv = layout.rank_view(tp_size=tp, tp_rank=tp_rank, ep_size=ep, ep_rank=ep_rank, param_dtype=param_dtype)
            want = oracle_place(oracle, str(tmp_path), rv, tp_size=tp, tp_rank=tp_rank, allow_cast=cast)
            ck, plan = make_plan(str(tmp_path), rv, tp_size=tp, tp_rank=tp_rank, allow_cast=cast)
            got = apply_plan_numpy(ck, plan)
            for p in plan.params:
                assert got[p.name].tobytes() == want[p.name].tobytes(), (name, tp_rank, p.name)
            info = plan.param_info()
            assert all(i["bytes_written"] == i["nbytes"] for i in info)


def test_deepseek_v3_full_scale_plan(mxp, tmp_path):
    """The whole DeepSeek-V3-shaped checkpoint (90,427 tensors, 673 GB as sparse header-only
    shards) planned for one TP=8 / EP=8 rank: ~85 GB per rank, the share the reference
    reports for this model (docs/ARCHITECTURE.md:1128-1136: 681 GB = 8 x 85 GB)."""
    from modelexpress_amd import models
    from modelexpress_amd.engine import Checkpoint, PlacementPlan

    layout = models.DeepSeekV3()
    tensors = layout.checkpoint()
    synth.write_headers_only(tensors, str(tmp_path), n_shards=163)
    ck = Checkpoint(str(tmp_path))
    assert len(ck) == len(tensors) == 90427
    rv = layout.rank_view(tp_size=8, tp_rank=5, ep_size=8, ep_rank=5)
    plan = PlacementPlan(ck, rv.params, tp_size=8, tp_rank=5, stacked_params_mapping=rv.stacked_params_mapping,
                         expert_mapping=rv.expert_mapping)
    placed = plan.totals()["placed_bytes"]
    assert placed == sum(p.nbytes for p in rv.params)
    assert 84e9 < placed < 86e9
    info = plan.param_info()
    assert all(i["bytes_written"] == i["nbytes"] for i in info)
    # 58 MoE layers x 32 local experts x (gate, up, down) x (weight, scale) expert writes
    assert sum(1 for w in plan.writes() if w.kind == "expert") == 58 * 32 * 3 * 2
