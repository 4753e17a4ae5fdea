"""Chain and strategy semantics on the host, restating the assertions of the reference's
tests/test_model_streamer_strategy.py (cited per test) against this package's classes."""

from types import SimpleNamespace

import pytest
import torch

from modelexpress_amd import envs
from modelexpress_amd.adapter import EngineAdapter, StrategyFailed, UnsupportedCapability, gated_capability
from modelexpress_amd.accelerators import HipAcceleratorBackend, accelerator_backend_for
from modelexpress_amd.load_strategy import (DefaultStrategy, HipPlacementStrategy, HipStreamerStrategy, LoadContext,
                                            LoadResult, LoadStrategy, LoadStrategyChain, _resolve_model_uri)


class _Backend(HipAcceleratorBackend):
    def supports_hip_placement(self) -> bool:
        return True


def _ctx(adapter=None, **cfg):
    return LoadContext(model_config=SimpleNamespace(**cfg), adapter=adapter, accelerator_backend=_Backend())


class _IterAdapter(EngineAdapter):
    def __init__(self, fail_apply=False, fail_build=False):
        self.fail_apply, self.fail_build = fail_apply, fail_build
        self.applied, self.reinit_calls, self.after_calls = [], 0, 0

    def apply_weight_iter(self, result, weights_iter):
        for name, t in weights_iter:
            self.applied.append(name)
            if self.fail_apply:
                raise RuntimeError("boom mid-stream")
        return result

    def build_model_streamer_weight_iter(self, model_uri, model=None):
        if self.fail_build:
            raise FileNotFoundError(model_uri)
        yield "a", torch.zeros(1)
        yield "b", torch.zeros(1)

    def after_weight_iter_load(self, result):
        self.after_calls += 1
        return result

    def reinit_for_retry(self, result):
        self.reinit_calls += 1
        return LoadResult(value="fresh-model", model=None)

    def load_via_native(self, result):
        result.metadata["native"] = True
        return result


def test_gated_capability_identity_rule():
    # adapter.py:37-51, base.py:53-60: eligible only when the concrete class overrides
    assert HipStreamerStrategy().is_available(_ctx(EngineAdapter())) is False
    assert getattr(EngineAdapter.apply_weight_iter, "__gated_capability__", False)
    with pytest.raises(UnsupportedCapability):
        EngineAdapter().placement_layout(None)
    assert HipStreamerStrategy().is_available(_ctx(None)) is False


def test_streamer_requires_uri(monkeypatch):
    # test_model_streamer_strategy.py:145-226
    monkeypatch.delenv("MX_MODEL_URI", raising=False)
    assert HipStreamerStrategy().is_available(_ctx(_IterAdapter())) is False
    monkeypatch.setenv("MX_MODEL_URI", "/models/x")
    assert HipStreamerStrategy().is_available(_ctx(_IterAdapter())) is True
    assert envs.MX_MODEL_URI == "/models/x"  # live read


def test_uri_resolution_order(monkeypatch):
    # model_streamer_strategy.py:27-35: env -> model_weights -> model -> model_path
    monkeypatch.setenv("MX_MODEL_URI", "/env")
    assert _resolve_model_uri(_ctx(model_weights="/w", model="/m", model_path="/p")) == "/env"
    monkeypatch.delenv("MX_MODEL_URI")
    assert _resolve_model_uri(_ctx(model_weights="/w", model="/m", model_path="/p")) == "/w"
    assert _resolve_model_uri(_ctx(model_weights=None, model="/m", model_path="/p")) == "/m"
    assert _resolve_model_uri(_ctx(model_path="/p")) == "/p"
    assert _resolve_model_uri(_ctx()) == ""


def test_streamer_mutated_flags(monkeypatch):
    # test_model_streamer_strategy.py:228-283
    monkeypatch.setenv("MX_MODEL_URI", "/models/x")
    ok = _IterAdapter()
    out = HipStreamerStrategy().load(LoadResult(value="m"), _ctx(ok))
    assert ok.applied == ["a", "b"] and ok.after_calls == 1 and out.value == "m"
    with pytest.raises(StrategyFailed) as e:
        HipStreamerStrategy().load(LoadResult(value="m"), _ctx(_IterAdapter(fail_apply=True)))
    assert e.value.mutated is True
    # the iterator is lazy: a build failure surfaces inside apply and counts as mutated,
    # exactly as in the reference where _stream_weights is a generator
    with pytest.raises(StrategyFailed) as e:
        HipStreamerStrategy().load(LoadResult(value="m"), _ctx(_IterAdapter(fail_build=True)))
    assert e.value.mutated is True
    monkeypatch.delenv("MX_MODEL_URI")
    with pytest.raises(StrategyFailed) as e:
        HipStreamerStrategy().load(LoadResult(value="m"), _ctx(_IterAdapter()))
    assert e.value.mutated is False


class _Scripted(LoadStrategy):
    def __init__(self, name, behaviour, available=True):
        self.name, self.behaviour, self.available = name, behaviour, available
        self.rolled_back = 0

    def is_available(self, ctx):
        return self.available

    def load(self, result, ctx):
        if self.behaviour == "ok":
            return result
        if self.behaviour == "miss":
            raise StrategyFailed("clean miss", mutated=False)
        if self.behaviour == "dirty":
            raise StrategyFailed("dirty", mutated=True)
        raise ValueError("unexpected")

    def rollback(self, ctx):
        self.rolled_back += 1


def test_chain_order_skip_rollback_and_reinit():
    # test_model_streamer_strategy.py:405-502, load_strategy/__init__.py:79-117
    ad = _IterAdapter()
    s = [_Scripted("unavailable", "ok", available=False), _Scripted("miss", "miss"), _Scripted("boom", "raise"),
         _Scripted("dirty", "dirty"), _Scripted("winner", "ok"), _Scripted("never", "ok")]
    out = LoadStrategyChain.run("model", _ctx(ad), s)
    assert out == "fresh-model"  # re-initialised after the dirty failure, then loaded by "winner"
    assert [x.rolled_back for x in s] == [0, 1, 1, 1, 0, 0]
    assert ad.reinit_calls == 1


def test_chain_exhaustion_and_reinit_errors():
    with pytest.raises(RuntimeError, match="No loading strategy succeeded"):
        LoadStrategyChain.run("model", _ctx(_IterAdapter()), [_Scripted("miss", "miss")])
    with pytest.raises(RuntimeError, match="no adapter can reinitialize"):
        LoadStrategyChain.run("model", _ctx(None), [_Scripted("dirty", "dirty")])
    with pytest.raises(RuntimeError, match="does not support retry"):
        LoadStrategyChain.run("model", _ctx(EngineAdapter()), [_Scripted("dirty", "dirty")])


def test_default_chain_falls_through_to_native(monkeypatch):
    monkeypatch.delenv("MX_MODEL_URI", raising=False)
    ad = _IterAdapter()
    assert [s.name for s in LoadStrategyChain.default_strategies()] == ["hip_placement", "model_streamer", "default"]
    assert LoadStrategyChain.run("model", _ctx(ad)) == "model"
    assert DefaultStrategy().is_available(_ctx(EngineAdapter())) is False


class _PlaceAdapter(_IterAdapter):
    def placement_layout(self, result):
        raise RuntimeError("layout unavailable")


def test_hip_placement_availability_and_clean_miss(monkeypatch, tmp_path):
    monkeypatch.delenv("MX_MODEL_URI", raising=False)
    st = HipPlacementStrategy()
    assert st.is_available(_ctx(_IterAdapter())) is False  # capability not overridden
    assert st.is_available(_ctx(_PlaceAdapter())) is False  # no URI
    monkeypatch.setenv("MX_MODEL_URI", "s3://bucket/model")
    assert st.is_available(_ctx(_PlaceAdapter())) is False  # object stores are not this strategy's
    monkeypatch.setenv("MX_MODEL_URI", str(tmp_path))
    assert st.is_available(_ctx(_PlaceAdapter())) is True
    ctx = _ctx(_PlaceAdapter())
    ctx.accelerator_backend = HipAcceleratorBackend()
    if not torch.cuda.is_available():
        assert st.is_available(ctx) is False  # no device
    with pytest.raises(StrategyFailed) as e:  # planning failures never count as mutated
        st.load(LoadResult(value="m"), _ctx(_PlaceAdapter()))
    assert e.value.mutated is False


def test_accelerator_backend_selection():
    # accelerators/__init__.py:41-61, base.py:16-72
    b = accelerator_backend_for("cuda:0")
    assert b.name == "rocm" and b.torch_device_type == "cuda" and b.nixl_mem_type == "VRAM"
    assert not (b.supports_gds() or b.supports_vmm() or b.supports_pool_reg() or b.supports_rdma_p2p())
    assert b.torch_device(1) == torch.device("cuda", 1)
    with pytest.raises(ValueError, match="Unsupported accelerator backend"):
        accelerator_backend_for("xpu:0")


def test_refit_timing_vocabulary():
    # modelexpress/refit/timing.py:23-35: ten fixed stages, one JSON record with a fixed prefix
    import json

    from modelexpress_amd.timing import MX_REFIT_TIMING_PREFIX, REFIT_TIMING_STAGES, RefitTimingRecorder

    assert REFIT_TIMING_STAGES == ("control_discovery", "source_preparation", "setup_registration", "transfer_planning",
                                   "wire_transfer", "receive_sync", "transformation", "installation", "post_install",
                                   "rollout_readiness")
    ticks = iter([0.0, 1.0, 3.0, 3.0, 3.5, 10.0, 10.0])
    rec = RefitTimingRecorder(backend="test", version=7, cold=True, clock=lambda: next(ticks))
    with rec.span("wire_transfer"):
        pass
    with pytest.raises(RuntimeError):
        with rec.span("installation"):
            raise RuntimeError("boom")
    with pytest.raises(ValueError):
        rec.add_duration("not_a_stage", 1.0)
    line = rec.emit()
    assert line.startswith(MX_REFIT_TIMING_PREFIX + " ")
    payload = json.loads(line[len(MX_REFIT_TIMING_PREFIX) + 1:])
    assert payload["cold_warm"] == "cold" and payload["stages"]["wire_transfer"] == {"duration_s": 2.0, "count": 1, "statuses": ["ok"]}
    assert payload["stages"]["installation"]["statuses"] == ["error"]


def test_manifest_comparison_rules(caplog):
    # modelexpress/nixl_transfer.py:835-897: size and dtype must agree per shared name; a name diff
    # fails closed only when an exact match is required; nothing matched is an error in that mode
    from modelexpress_amd.manifest import ManifestMismatchError, TensorRecord, compare_manifests, dumps, loads

    a = [TensorRecord("w", 64, "BF16", "0000abcd", "00" * 16), TensorRecord("b", 8, "F32", "00000001")]
    assert compare_manifests(a, loads(dumps(a)), require_exact_match=True) == 2
    with pytest.raises(ManifestMismatchError, match="size mismatch: source=64 bytes, local=32 bytes"):
        compare_manifests(a, [TensorRecord("w", 32, "BF16")])
    with pytest.raises(ManifestMismatchError, match="dtype mismatch: source='BF16', local='F16'"):
        compare_manifests(a, [TensorRecord("w", 64, "F16")])
    with pytest.raises(ManifestMismatchError, match="checksum mismatch"):
        compare_manifests(a, [TensorRecord("w", 64, "BF16", "0000abce")])
    with pytest.raises(ManifestMismatchError, match="digest mismatch"):
        compare_manifests(a, [TensorRecord("w", 64, "BF16", "0000abcd", "11" * 16)])
    assert compare_manifests(a, [TensorRecord("w", 64, "BF16", "0000abce")], check_content=False) == 1
    assert compare_manifests(a, [TensorRecord("w", 64, "BF16")]) == 1  # a side without content fields is not compared
    with caplog.at_level("WARNING", logger="modelexpress_amd.manifest"):
        assert compare_manifests(a, [TensorRecord("w", 64, "BF16"), TensorRecord("extra", 4, "F32")]) == 1
    assert "1 local-only, 1 source-only" in caplog.text
    with pytest.raises(ManifestMismatchError, match="1 local-only .first: .'extra'.., 1 source-only"):
        compare_manifests(a, [TensorRecord("w", 64, "BF16"), TensorRecord("extra", 4, "F32")], require_exact_match=True)
    with pytest.raises(ManifestMismatchError, match="No matching tensors"):
        compare_manifests([], [], require_exact_match=True)
    assert compare_manifests([], []) == 0


# ---------------------------------------------------------------- refit coverage record
def _coverage(caplog, **kw):
    import json
    import logging

    from modelexpress_amd.refit import log_coverage

    caplog.clear()
    with caplog.at_level(logging.INFO, logger="modelexpress_amd.refit"):
        rec = log_coverage(**kw)
    lines = [r for r in caplog.records if "MX_REFIT_COVERAGE" in r.getMessage()]
    assert len(lines) == 1 and json.loads(lines[0].getMessage().split("MX_REFIT_COVERAGE ", 1)[1]) == rec
    return rec, lines[0].levelname


def test_coverage_record_reference_cases(caplog, monkeypatch):
    """tests/test_reshard_refit_coverage.py:116-193: coverage is a byte ratio over the engine's complete
    parameter set, dtype widths count, the missing names are sampled, severity follows the content."""
    import torch

    monkeypatch.delenv("MX_RESHARD_REQUIRE_FULL_COVERAGE", raising=False)
    monkeypatch.delenv("MX_RESHARD_COVERAGE_FLOOR", raising=False)
    names = [f"layers.{i}.weight" for i in range(4)]
    rec, level = _coverage(caplog, param_layout={n: ((4, 8), torch.bfloat16) for n in names}, all_params=names)
    assert (rec["coverage_pct"], rec["params_installed"], rec["engine_params"], rec["params_never_written"]) == (100.0, 4, 4, 0)
    assert rec["dest_bytes"] == rec["engine_bytes"] and rec["params_never_written_sample"] == [] and level == "INFO"
    # :127-143 48 engine layers, the first 24 installed: 50 %, and the sample names the missing ones
    engine = [f"layers.{i}.weight" for i in range(48)]
    rec, level = _coverage(caplog, param_layout={n: ((4, 8), "BF16") for n in engine}, all_params=engine[:24])
    assert (rec["coverage_pct"], rec["params_installed"], rec["engine_params"], rec["params_never_written"]) == (50.0, 24, 48, 24)
    assert rec["params_never_written_sample"][0].startswith("layers.2") and len(rec["params_never_written_sample"]) == 10
    assert level == "WARNING"
    # :146-162 bytes, not parameter count
    rec, _ = _coverage(caplog, param_layout={"big": ((1024, 1024), torch.bfloat16), "small": ((1, 1), torch.bfloat16)},
                       all_params=["small"])
    assert rec["params_installed"] == 1 and rec["engine_params"] == 2 and rec["coverage_pct"] < 0.001 and rec["dest_bytes"] == 2
    # :165-179 dtype widths
    for dtype, width in ((torch.float8_e4m3fn, 1), (torch.bfloat16, 2), (torch.float32, 4), ("F8_E4M3", 1), ("F32", 4)):
        rec, _ = _coverage(caplog, param_layout={"w": ((4, 8), dtype)}, all_params=["w"])
        assert rec["engine_bytes"] == rec["dest_bytes"] == 32 * width, dtype
    # :182-193 unsupported sources are counted, sampled and clipped
    rec, level = _coverage(caplog, param_layout={n: ((4, 8), "BF16") for n in "ab"}, all_params=["a", "b"],
                           unsupported=[f"cannot reshard {i} " + "x" * 200 for i in range(15)])
    assert rec["unsupported"] == 15 and len(rec["unsupported_sample"]) == 10 and all(len(x) <= 120 for x in rec["unsupported_sample"])
    assert level == "WARNING"
    # :337-342 an engine with no parameters does not divide by zero
    rec, _ = _coverage(caplog, param_layout={}, all_params=[])
    assert rec["coverage_pct"] == 0.0


def test_coverage_gate(caplog, monkeypatch):
    """:278-366 the gate is off by default, raises below the floor naming what is missing, passes at the
    floor, rejects a floor outside [0, 1], and reads its settings live."""
    from modelexpress_amd.mla import IncompleteRefit

    engine = [f"layers.{i}.weight" for i in range(48)]
    layout = {n: ((4, 8), "BF16") for n in engine}
    monkeypatch.delenv("MX_RESHARD_REQUIRE_FULL_COVERAGE", raising=False)
    monkeypatch.delenv("MX_RESHARD_COVERAGE_FLOOR", raising=False)
    _coverage(caplog, param_layout=layout, all_params=engine[:24])  # off: a partial refit goes through
    monkeypatch.setenv("MX_RESHARD_REQUIRE_FULL_COVERAGE", "1")
    with pytest.raises(IncompleteRefit, match=r"covers 50\.00% .* 24 of 48 params .*layers\.24\.weight"):
        _coverage(caplog, param_layout=layout, all_params=engine[:24])
    assert any("MX_REFIT_COVERAGE" in r.getMessage() for r in caplog.records)  # recorded before it is rejected
    monkeypatch.setenv("MX_RESHARD_COVERAGE_FLOOR", "0.5")
    _coverage(caplog, param_layout=layout, all_params=engine[:24])  # at the floor: passes
    for floor in ("-0.1", "1.5"):
        monkeypatch.setenv("MX_RESHARD_COVERAGE_FLOOR", floor)
        with pytest.raises(ValueError, match="MX_RESHARD_COVERAGE_FLOOR"):
            _coverage(caplog, param_layout=layout, all_params=engine[:24])
