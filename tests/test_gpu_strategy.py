"""The strategy chain, the iterator-shaped path and the refit flow on a real GPU."""

import os
from types import SimpleNamespace

import numpy as np
import pytest
import torch
from torch import nn

from helpers import oracle_place
from modelexpress_amd import models, synth
from modelexpress_amd.adapter import EngineAdapter, StrategyFailed
from modelexpress_amd.load_strategy import (HipPlacementStrategy, LoadContext, LoadResult, LoadStrategyChain,
                                            iter_checkpoint_tensors, layout_from_module)
from modelexpress_amd.refit import HipRefitAdapter, RefitInputs

pytestmark = pytest.mark.gpu

LAYOUT = models.Llama(layers=2, hidden=64, ffn=96, q_heads=8, kv_heads=4, head_dim=8, vocab=256)
TP, RANK = 4, 1


class RankModule(nn.Module):
    """A module whose parameters are exactly one rank's table (what an engine allocates)."""

    stacked_params_mapping = [("qkv_proj", "q_proj"), ("qkv_proj", "k_proj"), ("qkv_proj", "v_proj"),
                              ("gate_up_proj", "gate_proj"), ("gate_up_proj", "up_proj")]

    def __init__(self, rv, device="cuda"):
        super().__init__()
        self._names = []
        for p in rv.params:
            key = p.name.replace(".", "__")
            self.register_parameter(key, nn.Parameter(torch.zeros(p.shape, dtype=torch.bfloat16, device=device),
                                                      requires_grad=False))
            self._names.append((key, p.name))

    def named_parameters(self, *a, **k):
        for key, name in self._names:
            yield name, getattr(self, key)


class RankAdapter(EngineAdapter):
    def __init__(self, rv):
        self.rv = rv
        self.reinit_calls = 0
        self.native_calls = 0

    def get_device_id(self):
        return 0

    def placement_layout(self, result):
        return layout_from_module(result.model, tp_size=TP, tp_rank=RANK)

    def reinit_for_retry(self, result):
        self.reinit_calls += 1
        fresh = RankModule(self.rv)
        return LoadResult(value=fresh, model=fresh)

    def load_via_native(self, result):
        self.native_calls += 1
        return result


def _ctx(adapter, path):
    return LoadContext(model_config=SimpleNamespace(model=path), adapter=adapter)


def test_chain_places_into_param_data(oracle, tmp_path, monkeypatch, mxp):
    synth.write_checkpoint(LAYOUT.checkpoint(), str(tmp_path), n_shards=2, seed=21)
    rv = LAYOUT.rank_view(tp_size=TP, tp_rank=RANK)
    want = oracle_place(oracle, str(tmp_path), rv, tp_size=TP, tp_rank=RANK)
    monkeypatch.setenv("MX_MODEL_URI", str(tmp_path))
    model = RankModule(rv)
    ptrs = {n: p.data_ptr() for n, p in model.named_parameters()}
    ad = RankAdapter(rv)
    ctx = _ctx(ad, str(tmp_path))
    out = LoadStrategyChain.run(model, ctx)
    assert out is model and ad.reinit_calls == 0 and ad.native_calls == 0
    for name, p in model.named_parameters():
        assert p.data_ptr() == ptrs[name]  # written in place, never replaced
        assert p.data.view(torch.uint8).cpu().numpy().tobytes() == want[name].tobytes(), name
    assert set(ctx.tensors) == set(want)


def test_manifest_of_a_placed_rank_matches_a_source_manifest(oracle, tmp_path, monkeypatch, mxp):
    """Source side: names, sizes, dtypes, checksums and digests computed by the oracle.  Target
    side: the manifest the strategy leaves in the result plus device digests of the live
    parameters.  One flipped byte on the target must fail the comparison."""
    from modelexpress_amd.engine import PlacementEngine
    from modelexpress_amd.manifest import ManifestMismatchError, TensorRecord, build_manifest, compare_manifests

    synth.write_checkpoint(LAYOUT.checkpoint(), str(tmp_path), n_shards=2, seed=23)
    rv = LAYOUT.rank_view(tp_size=TP, tp_rank=RANK)
    want = oracle_place(oracle, str(tmp_path), rv, tp_size=TP, tp_rank=RANK)
    source = [TensorRecord(p.name, p.nbytes, p.dtype, oracle.safe_checksum(want[p.name]), oracle.tensor_digest(want[p.name]))
              for p in rv.params]
    monkeypatch.setenv("MX_MODEL_URI", str(tmp_path))
    model = RankModule(rv)
    ad = RankAdapter(rv)
    result = HipPlacementStrategy().load(LoadResult(value=model, model=model), _ctx(ad, str(tmp_path)))
    assert compare_manifests(source, result.metadata["manifest"], require_exact_match=True) == len(rv.params)
    eng = PlacementEngine(0)
    live = dict(model.named_parameters())
    local = build_manifest(eng, rv.params, [live[p.name].data for p in rv.params])
    assert compare_manifests(source, local, require_exact_match=True) == len(rv.params)
    victim = rv.params[1]
    live[victim.name].data.view(torch.uint8).view(-1)[3] ^= 1
    with pytest.raises(ManifestMismatchError, match=f"'{victim.name}' checksum mismatch"):
        compare_manifests(source, build_manifest(eng, rv.params, [live[p.name].data for p in rv.params]))
    eng.close()


def test_truncated_shard_fails_the_strategy_and_the_chain_recovers(tmp_path, monkeypatch, mxp):
    """A shard that shrinks between planning and ingest: the read error surfaces as
    StrategyFailed (mutated once any chunk reached the GPU), the chain rolls back,
    re-initialises the model if bytes moved, and the next strategy loads."""
    import modelexpress_amd.engine as E

    info = synth.write_checkpoint(LAYOUT.checkpoint(), str(tmp_path), n_shards=2, seed=22)
    rv = LAYOUT.rank_view(tp_size=TP, tp_rank=RANK)
    monkeypatch.setenv("MX_MODEL_URI", str(tmp_path))
    monkeypatch.setenv("MXP_SLOT_MIB", "1")
    real_execute = E.PlacementEngine.execute

    def execute_after_truncation(eng, plan, dst, **kw):
        size = os.path.getsize(info["files"][-1])
        with open(info["files"][-1], "r+b") as f:
            f.truncate(size // 2)
        return real_execute(eng, plan, dst, **kw)

    monkeypatch.setattr(E.PlacementEngine, "execute", execute_after_truncation)
    model = RankModule(rv)
    ad = RankAdapter(rv)
    with pytest.raises(StrategyFailed) as e:
        HipPlacementStrategy().load(LoadResult(value=model, model=model), _ctx(ad, str(tmp_path)))
    assert "MXP_ERR_IO" in str(e.value)

    synth.write_checkpoint(LAYOUT.checkpoint(), str(tmp_path), n_shards=2, seed=22)
    model2 = RankModule(rv)
    out = LoadStrategyChain.run(model2, _ctx(ad, str(tmp_path)))
    assert ad.native_calls == 1  # hip_placement failed, model_streamer is not offered by this adapter
    assert (out is not model2) == (ad.reinit_calls == 1)


def test_bad_checkpoint_is_a_clean_miss(tmp_path, monkeypatch, mxp):
    (tmp_path / "model.safetensors").write_bytes(b"\x05\x00\x00\x00\x00\x00\x00\x00{nope")
    rv = LAYOUT.rank_view(tp_size=TP, tp_rank=RANK)
    monkeypatch.setenv("MX_MODEL_URI", str(tmp_path))
    model = RankModule(rv)
    with pytest.raises(StrategyFailed) as e:
        HipPlacementStrategy().load(LoadResult(value=model, model=model), _ctx(RankAdapter(rv), str(tmp_path)))
    assert e.value.mutated is False
    assert all(int(p.data.view(torch.uint8).sum()) == 0 for _n, p in model.named_parameters())


def test_iter_checkpoint_tensors_matches_oracle(oracle, tmp_path, mxp):
    synth.write_checkpoint(LAYOUT.checkpoint(), str(tmp_path), n_shards=3, seed=23)
    want = dict(oracle.load_checkpoint(str(tmp_path)))
    seen = []
    for name, t in iter_checkpoint_tensors(str(tmp_path)):
        assert t.is_cuda and t.dtype == torch.bfloat16 and tuple(t.shape) == want[name].shape
        assert t.contiguous().view(torch.uint8).cpu().numpy().tobytes() == want[name].tobytes(), name
        seen.append(name)
    assert seen == [n for n, _ in oracle.load_checkpoint(str(tmp_path))]


def test_copy_batch_and_overlap_rule(gpu_engine, oracle_c, mxp):
    rng = np.random.default_rng(30)
    sizes = [0, 16, 100, 4096, 65536 + 48, 1 << 20]
    srcs = [torch.from_numpy(rng.integers(0, 256, max(n, 1), dtype=np.uint8)).cuda()[:n] for n in sizes]
    dsts = [torch.zeros(max(n, 16), dtype=torch.uint8, device="cuda") for n in sizes]
    sums = gpu_engine.copy_batch(srcs, dsts, sizes)
    for s, d, n, c in zip(srcs, dsts, sizes, sums):
        assert torch.equal(d[:n], s)
        assert c == oracle_c.checksum32(s.cpu().numpy())
    big = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    with pytest.raises(mxp.MxpError, match="overlap"):  # receiver.py:289-321: only disjoint copies are batched
        gpu_engine.copy_batch([srcs[3], srcs[3]], [big, big[16:]], [4096 - 16, 4096 - 16])


def test_refit_stage_verify_apply(oracle, tmp_path, mxp):
    # config 3 in miniature: resident bf16 rank slice, new fp32 checkpoint with edge cases
    base, new = tmp_path / "v0", tmp_path / "v1"
    synth.write_checkpoint(LAYOUT.checkpoint(), str(base), n_shards=2, seed=24)
    synth.write_checkpoint(LAYOUT.checkpoint(dtype="F32", edge_cases=models.NORMAL_EDGE_DENSE), str(new), n_shards=3, seed=25)
    rv = LAYOUT.rank_view(tp_size=TP, tp_rank=RANK)
    model = RankModule(rv)
    layout = layout_from_module(model, tp_size=TP, tp_rank=RANK)
    os.environ["MX_MODEL_URI"] = str(base)
    try:
        LoadStrategyChain.run(model, _ctx(RankAdapter(rv), str(base)))
    finally:
        del os.environ["MX_MODEL_URI"]
    v0 = {n: p.data.view(torch.uint8).cpu().numpy().tobytes() for n, p in model.named_parameters()}
    want = oracle_place(oracle, str(new), rv, tp_size=TP, tp_rank=RANK, allow_cast=True)
    digests = {n: oracle.tensor_digest(t) for n, t in want.items()}

    ad = HipRefitAdapter(layout)
    # a wrong published digest: nothing is installed
    bad = dict(digests)
    first = next(iter(bad))
    bad[first] = "0" * 32
    plan = ad.create_transfer_plan(RefitInputs("v1", str(new), "sig", bad, require_digests=True))
    with pytest.raises(RuntimeError, match="digest mismatch"):  # nixl_staged_transfer.py:529-549
        ad.stage_weight(plan)
    assert {n: p.data.view(torch.uint8).cpu().numpy().tobytes() for n, p in model.named_parameters()} == v0
    # a missing digest when they are required
    plan = ad.create_transfer_plan(RefitInputs("v1", str(new), "sig", {}, require_digests=True))
    with pytest.raises(RuntimeError, match="no published digest"):
        ad.stage_weight(plan)
    # digests per publisher shard (nixl_staged_transfer.py:529-549; tests/test_refit_nixl_staged_transfer.py:192-203):
    # every 2-D parameter as two row halves, each with the digest of its own region
    def shard_table(tamper=None, drop=None):
        table = {}
        for n, t in want.items():
            if len(t.shape) != 2 or t.shape[0] % 2:
                continue
            half = t.shape[0] // 2
            rows = []
            for k in range(2):
                region = oracle.shard_region(t, t.shape, (k * half, 0), (half, t.shape[1]))
                d = oracle.tensor_digest(region)
                if (n, k) == tamper:
                    d = "f" * 32
                if (n, k) == drop:
                    d = None
                rows.append(((k * half, 0), (half, t.shape[1]), d))
            table[n] = rows
        return table

    victim = next(iter(shard_table()))
    plan = ad.create_transfer_plan(RefitInputs("v1", str(new), "sig", digests, True, shard_table(tamper=(victim, 1))))
    with pytest.raises(RuntimeError, match=r"staged weight digest mismatch for source .* at offset \(\d+, 0\)"):
        ad.stage_weight(plan)
    plan = ad.create_transfer_plan(RefitInputs("v1", str(new), "sig", digests, True, shard_table(drop=(victim, 0))))
    with pytest.raises(RuntimeError, match="did not publish a verification digest"):
        ad.stage_weight(plan)
    assert {n: p.data.view(torch.uint8).cpu().numpy().tobytes() for n, p in model.named_parameters()} == v0
    # the good path
    inputs = RefitInputs("v1", str(new), "sig", digests, require_digests=True, expected_shard_digests=shard_table())
    plan = ad.create_transfer_plan(inputs)
    assert ad.validate_transfer_plan(plan, inputs)
    assert not ad.validate_transfer_plan(plan, RefitInputs("v2", str(new), "other-layout", digests))
    staged = ad.stage_weight(plan)
    assert {n: p.data.view(torch.uint8).cpu().numpy().tobytes() for n, p in model.named_parameters()} == v0
    sums = ad.apply_weight(staged)
    for n, p in model.named_parameters():
        assert p.data.view(torch.uint8).cpu().numpy().tobytes() == want[n].tobytes(), n
        assert sums[n] == oracle.safe_checksum(want[n])
    assert ad.coverage["schema"] == "refit-coverage-v1" and ad.coverage["coverage_pct"] == 100.0
    assert ad.coverage["engine_bytes"] == ad.coverage["dest_bytes"] == sum(p.nbytes for p in rv.params)
    assert ad.coverage["planned_wire_bytes"] >= 2 * ad.coverage["dest_bytes"]  # fp32 over PCIe for bf16 parameters
    rec = ad.timing.as_dict()
    assert rec["backend"] == "hip_placement" and rec["version"] == "v1" and rec["bytes"] == sum(p.nbytes for p in rv.params)
    assert {"transfer_planning", "wire_transfer", "receive_sync", "installation"} <= set(rec["stages"])
    assert rec["cast_nan_bits"] == "0x7fc0"  # the image the casts of this cycle wrote (torch's device image)
    assert ad.timing.emit().startswith("MX_REFIT_TIMING {")
    ad.release_staged_weight(staged)
    ad.close()


def test_loader_class_has_the_reference_loader_interface(oracle, tmp_path, mxp):
    # modelexpress/gds_loader.py:52-160: load() -> dict, load_iter() per file with prefetch, shutdown()
    from modelexpress_amd.accelerators import HipAcceleratorBackend
    from modelexpress_amd.loader import MxHipLoader

    synth.write_checkpoint(LAYOUT.checkpoint(), str(tmp_path), n_shards=3, seed=24)
    want = oracle.load_checkpoint(str(tmp_path))
    loader = MxHipLoader(HipAcceleratorBackend())
    for _ in range(2):  # the engine is kept between calls
        got = loader.load(str(tmp_path))
        assert list(got) == [n for n, _ in want]
        for n, t in want:
            assert got[n].is_cuda and tuple(got[n].shape) == t.shape
            assert got[n].contiguous().view(torch.uint8).cpu().numpy().tobytes() == t.tobytes(), n
    first = next(iter(loader.load_iter(str(tmp_path), use_tqdm=False)))  # an abandoned iterator shuts its pool down
    assert first[0] == want[0][0]
    loader.shutdown()
    loader.shutdown()
    with pytest.raises(FileNotFoundError):
        loader.load(str(tmp_path / "missing"))
