"""End-to-end placement on the GPU (ingest from files and from HBM-staged shards)
against the CPU oracle, on small instances of the five benchmark families."""

import numpy as np
import pytest
import torch

from helpers import make_plan, oracle_place, tiny_layouts
from modelexpress_amd import synth

pytestmark = pytest.mark.gpu


def _stage_files(ck):
    return [torch.from_numpy(np.fromfile(f["path"], dtype=np.uint8)).cuda() for f in ck.files()]


@pytest.mark.parametrize("name", list(tiny_layouts()))
def test_families_match_oracle(name, gpu_engine, gpu_engine_band, oracle, tmp_path):
    layout, tp, ep, shards, ck_kw = tiny_layouts()[name]
    cast = ck_kw.get("dtype") == "F32"
    synth.write_checkpoint(layout.checkpoint(**ck_kw), str(tmp_path), n_shards=shards, seed=7)
    for tp_rank in sorted({0, tp - 1}):
        ep_rank = tp_rank % ep
        rv = layout.rank_view(tp_size=tp, tp_rank=tp_rank, ep_size=ep, ep_rank=ep_rank,
                              param_dtype="BF16" if cast else None)
        want = oracle_place(oracle, str(tmp_path), rv, tp_size=tp, tp_rank=tp_rank, allow_cast=cast)
        ck, plan = make_plan(str(tmp_path), rv, tp_size=tp, tp_rank=tp_rank, allow_cast=cast)
        for mode in ("ingest", "ingest_band", "resident"):
            eng = gpu_engine_band if mode == "ingest_band" else gpu_engine
            dst = eng.allocate(plan, fill=0xAB)
            if mode == "resident":
                eng.execute_resident(plan, _stage_files(ck), dst)
            else:
                stats = eng.execute(plan, dst)
                assert stats["placed_bytes"] == sum(p.nbytes for p in plan.params)
                if mode == "ingest":  # packed on the host: nothing but placed bytes (times the cast factor) is read
                    assert stats["file_bytes"] == sum(p.nbytes for p in plan.params) * (2 if cast else 1)
            sums = eng.checksums(plan)
            for p, d, s in zip(plan.params, dst, sums):
                assert d.cpu().numpy().tobytes() == want[p.name].tobytes(), (name, mode, tp_rank, p.name)
                assert s == oracle.safe_checksum(want[p.name]), (name, mode, tp_rank, p.name)


@pytest.mark.parametrize("name", ["llama_tp4", "llama_f32_refit", "deepseek_ep"])
def test_direct_io_ranges_match_oracle(name, oracle, tmp_path, mxp):
    """O_DIRECT mode: every range is widened to 4 KiB blocks (also past the end of the last
    tensor) and boxes start inside the slot; results must not change.  Where the file system
    refuses O_DIRECT the engine falls back to buffered reads of the same widened ranges."""
    from modelexpress_amd.engine import PlacementEngine

    layout, tp, ep, shards, ck_kw = tiny_layouts()[name]
    cast = ck_kw.get("dtype") == "F32"
    synth.write_checkpoint(layout.checkpoint(**ck_kw), str(tmp_path), n_shards=shards, seed=9)
    tp_rank = tp - 1
    rv = layout.rank_view(tp_size=tp, tp_rank=tp_rank, ep_size=ep, ep_rank=tp_rank % ep,
                          param_dtype="BF16" if cast else None)
    want = oracle_place(oracle, str(tmp_path), rv, tp_size=tp, tp_rank=tp_rank, allow_cast=cast)
    ck, plan = make_plan(str(tmp_path), rv, tp_size=tp, tp_rank=tp_rank, allow_cast=cast)
    eng = PlacementEngine(0, ring_slots=3, slot_bytes=1 << 17, reader_threads=2, streams=2, use_o_direct=True)
    dst = eng.allocate(plan, fill=0x11)
    eng.execute(plan, dst)
    for p, d, s in zip(plan.params, dst, eng.checksums(plan)):
        assert d.cpu().numpy().tobytes() == want[p.name].tobytes(), p.name
        assert s == oracle.safe_checksum(want[p.name]), p.name
    with pytest.raises(mxp.MxpError, match="direct I/O"):
        PlacementEngine(0, use_o_direct=True, pack_strided_on_host=True)
    eng.close()
