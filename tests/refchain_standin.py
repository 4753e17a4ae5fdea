"""A stand-in for the reference package at the strategy boundary, and scenarios that drive
``HipPlacementStrategy`` through it the way a ModelExpress maintainer would register it.

The reference package cannot be imported in this build's containers (its generated protobuf
stubs reject the installed runtime and its engine integrations import vLLM), so the contract is
restated here, minimal and in this file's own words, from the reference's sources:

* ``modelexpress.adapter``: ``UnsupportedCapability``, ``StrategyFailed(message, *, mutated)``,
  ``gated_capability`` and an ``EngineAdapter`` with the gated methods the load path uses and NO
  ``placement_layout`` (modelexpress/adapter.py:19-196);
* ``modelexpress.load_strategy.context``: ``LoadResult`` / ``LoadContext`` with the fields the
  strategies read (load_strategy/context.py:39-87);
* ``modelexpress.load_strategy.base``: ``LoadStrategy`` with the identity rule written as the
  reference writes it - ``getattr(cls, m.__name__) is not m``, which raises AttributeError for a
  capability the adapter class lacks (load_strategy/base.py:37-76) - plus ``_as_load_result`` and a
  ``register_tensors`` that records its calls;
* ``run_chain``: the loop of ``LoadStrategyChain.run`` (load_strategy/__init__.py:79-136): the
  eligible list is built outside any try, ``except StrategyFailed`` names THIS module's class,
  a mutated failure calls ``adapter.reinit_for_retry``, any other exception only rolls back.

``install()`` must run before ``modelexpress_amd`` is imported, which is why the scenarios run in
a process of their own: ``python tests/refchain_standin.py <scenario> <workdir>`` prints one JSON
object.  tests/test_reference_binding.py asserts on it.
"""

from __future__ import annotations

import functools
import json
import os
import sys
import types
from abc import ABC, abstractmethod
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, ClassVar

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(ROOT / "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

REGISTERED: list = []  # (result, ctx) pairs register_tensors was called with


def install() -> types.SimpleNamespace:
    """Create the stand-in modules in ``sys.modules`` and return their public names."""
    pkg = types.ModuleType("modelexpress")
    pkg.__path__ = []  # a package, so that submodule imports resolve through sys.modules
    adapter = types.ModuleType("modelexpress.adapter")
    ls_pkg = types.ModuleType("modelexpress.load_strategy")
    ls_pkg.__path__ = []
    base = types.ModuleType("modelexpress.load_strategy.base")
    context = types.ModuleType("modelexpress.load_strategy.context")

    class UnsupportedCapability(NotImplementedError):
        pass

    class StrategyFailed(RuntimeError):
        def __init__(self, message: str, *, mutated: bool = False):
            super().__init__(message)
            self.mutated = mutated

    def gated_capability(method):
        @functools.wraps(method)
        def default(self, *args, **kwargs):
            raise UnsupportedCapability(method.__name__)

        default.__gated_capability__ = True
        return default

    class EngineAdapter:
        @gated_capability
        def get_device_id(self): ...

        @gated_capability
        def apply_weight_iter(self, result, weights_iter): ...

        @gated_capability
        def build_model_streamer_weight_iter(self, model_uri, model=None): ...

        @gated_capability
        def load_via_native(self, result): ...

        @gated_capability
        def reinit_for_retry(self, result): ...

        def after_weight_iter_load(self, result):
            return result

        def after_native_load(self, result):
            return result

    @dataclass
    class LoadResult:
        value: Any
        model: Any = None
        publishable: bool = True
        metadata: dict = field(default_factory=dict)

    @dataclass
    class LoadContext:
        model_config: Any
        load_config: Any
        target_device: Any
        global_rank: int
        worker_rank: int
        device_id: int
        identity: Any
        mx_client: Any
        worker_id: str
        adapter: Any = None
        accelerator_backend: Any = None
        tensors: dict = field(default_factory=dict)

    class LoadStrategy(ABC):
        name: str
        requires: ClassVar[tuple] = ()

        def is_available(self, ctx) -> bool:
            if not self.requires:
                return True
            if ctx.adapter is None:
                return False
            cls = type(ctx.adapter)
            return all(getattr(cls, m.__name__) is not m for m in self.requires)

        @abstractmethod
        def load(self, result, ctx): ...

        def rollback(self, ctx) -> None:
            return None

    def _as_load_result(result_or_model):
        if isinstance(result_or_model, LoadResult):
            return result_or_model
        return LoadResult(value=result_or_model, model=result_or_model)

    def register_tensors(result, ctx, **_kw):
        REGISTERED.append((result, ctx))

    for name in ("UnsupportedCapability", "StrategyFailed", "gated_capability", "EngineAdapter"):
        setattr(adapter, name, locals()[name])
    context.LoadResult, context.LoadContext = LoadResult, LoadContext
    for name in ("LoadStrategy", "LoadResult", "LoadContext", "_as_load_result", "register_tensors"):
        setattr(base, name, locals()[name])
    pkg.adapter, pkg.load_strategy = adapter, ls_pkg
    ls_pkg.base, ls_pkg.context = base, context
    sys.modules.update({"modelexpress": pkg, "modelexpress.adapter": adapter, "modelexpress.load_strategy": ls_pkg,
                        "modelexpress.load_strategy.base": base, "modelexpress.load_strategy.context": context})
    return types.SimpleNamespace(UnsupportedCapability=UnsupportedCapability, StrategyFailed=StrategyFailed,
                                 gated_capability=gated_capability, EngineAdapter=EngineAdapter, LoadResult=LoadResult,
                                 LoadContext=LoadContext, LoadStrategy=LoadStrategy)


def run_chain(ref, model, ctx, all_strategies, log: list):
    """``LoadStrategyChain.run`` of the reference with the strategy list passed in."""
    eligible = [s for s in all_strategies if s.is_available(ctx)]
    log.append(("eligible", [s.name for s in eligible]))
    result = ref.LoadResult(value=model, model=model)
    for strategy in eligible:
        try:
            result = strategy.load(result, ctx)
            log.append(("loaded", strategy.name))
            return result.value
        except ref.StrategyFailed as e:
            log.append(("strategy_failed", strategy.name, bool(e.mutated)))
            strategy.rollback(ctx)
            if e.mutated:
                if ctx.adapter is None:
                    raise RuntimeError("mutated the model but no adapter can reinitialize it")
                try:
                    result = ctx.adapter.reinit_for_retry(result)
                except ref.UnsupportedCapability as exc:
                    raise RuntimeError("adapter does not support retry reinitialization") from exc
            continue
        except Exception as e:  # noqa: BLE001 - the generic branch: rollback only, no reinit
            log.append(("unexpected", strategy.name, type(e).__name__))
            strategy.rollback(ctx)
    raise RuntimeError("No loading strategy succeeded")


def _scenarios(ref, workdir: str, scenario: str) -> dict:
    # Only now: the package binds to whatever `modelexpress` it finds when it is first imported.
    from types import SimpleNamespace

    import torch

    import modelexpress_amd.adapter as A
    import modelexpress_amd.load_strategy as LS
    from modelexpress_amd import models, synth

    out: dict = {"scenario": scenario}
    out["bound"] = bool(A.BOUND_TO_REFERENCE)
    out["same_strategy_failed"] = A.StrategyFailed is ref.StrategyFailed
    out["same_engine_adapter"] = A.EngineAdapter is ref.EngineAdapter
    out["same_load_strategy_base"] = LS.LoadStrategy is ref.LoadStrategy
    out["strategy_is_reference_subclass"] = issubclass(LS.HipPlacementStrategy, ref.LoadStrategy)
    out["requires_is_base_default"] = LS.HipPlacementStrategy.requires == (ref.EngineAdapter.placement_layout,)

    if scenario == "mutated":
        # several staging slots' worth per rank and one reader thread: the chunks go out in file order, so
        # the intact first shard has reached the GPU when the truncated last one fails
        layout = models.Llama(layers=4, hidden=256, ffn=1024, q_heads=8, kv_heads=4, head_dim=32, vocab=8192)
        os.environ["MXP_READER_THREADS"] = "1"
    else:
        layout = models.Llama(layers=2, hidden=64, ffn=96, q_heads=8, kv_heads=4, head_dim=8, vocab=256)
    tp, rank = 4, 1
    rv = layout.rank_view(tp_size=tp, tp_rank=rank)
    device = "cuda" if torch.cuda.is_available() else "cpu"

    class RankModule(torch.nn.Module):
        stacked_params_mapping = [("qkv_proj", "q_proj"), ("qkv_proj", "k_proj"), ("qkv_proj", "v_proj"),
                                  ("gate_up_proj", "gate_proj"), ("gate_up_proj", "up_proj")]

        def __init__(self):
            super().__init__()
            self._names = []
            for p in rv.params:
                key = p.name.replace(".", "__")
                self.register_parameter(key, torch.nn.Parameter(
                    torch.zeros(p.shape, dtype=torch.bfloat16, device=device), requires_grad=False))
                self._names.append((key, p.name))

        def named_parameters(self, *a, **k):
            for key, name in self._names:
                yield name, getattr(self, key)

    class BareAdapter(ref.EngineAdapter):
        """Overrides nothing this package added: merely ineligible."""

        def __init__(self):
            self.reinit_calls = self.native_calls = 0
            self.native_model = None

        def get_device_id(self):
            return 0

        def reinit_for_retry(self, result):
            self.reinit_calls += 1
            fresh = RankModule()
            return ref.LoadResult(value=fresh, model=fresh)

        def load_via_native(self, result):
            self.native_calls += 1
            self.native_model = result.model
            return result

    class PlacingAdapter(BareAdapter):
        def placement_layout(self, result):
            return LS.layout_from_module(result.model, tp_size=tp, tp_rank=rank)

    class DuckAdapter:
        """Not derived from the adapter base class at all."""

        def get_device_id(self):
            return 0

    class _Backend:  # what the reference's context would carry on a ROCm box: no supports_hip_placement
        pass

    def ctx_for(adapter, path):
        return ref.LoadContext(model_config=SimpleNamespace(model=path), load_config=None, target_device=device,
                               global_rank=0, worker_rank=0, device_id=0, identity=SimpleNamespace(model_name="toy"),
                               mx_client=None, worker_id="w0", adapter=adapter, accelerator_backend=_Backend())

    os.environ["MX_MODEL_URI"] = workdir
    os.environ["MXP_SLOT_MIB"] = "1"
    strategies = lambda: [LS.HipPlacementStrategy(), LS.DefaultStrategy()]  # noqa: E731

    if scenario == "ineligible":
        # the registration of a maintainer whose adapter has not adopted the capability yet
        ok = {}
        for label, ad in (("bare", BareAdapter()), ("duck", DuckAdapter())):
            try:
                ok[label] = LS.HipPlacementStrategy().is_available(ctx_for(ad, workdir))
            except AttributeError as e:
                ok[label] = f"AttributeError: {e}"
        out["is_available"] = ok
        out["placing_overrides"] = type(PlacingAdapter()).placement_layout is not ref.EngineAdapter.placement_layout
        log: list = []
        ad = BareAdapter()
        model = RankModule()
        got = run_chain(ref, model, ctx_for(ad, workdir), strategies(), log)
        out["chain_log"], out["native_calls"], out["same_model"] = log, ad.native_calls, got is model
        return out

    if scenario == "clean_miss":
        # nothing at the URI: planning fails before any byte moves
        missing = os.path.join(workdir, "no_such_checkpoint")
        os.environ["MX_MODEL_URI"] = missing
        ad = PlacingAdapter()
        log = []
        ctx = ctx_for(ad, missing)
        # eligibility needs a device; the failure semantics do not
        chain = [s for s in strategies()]
        chain[0].is_available = lambda _ctx: True
        model = RankModule()
        got = run_chain(ref, model, ctx, chain, log)
        out["chain_log"], out["reinit_calls"], out["native_calls"] = log, ad.reinit_calls, ad.native_calls
        out["same_model"] = got is model
        return out

    # ---- the two device scenarios ----
    from helpers import oracle_place
    from oracle import oracle as O

    info = synth.write_checkpoint(layout.checkpoint(), workdir, n_shards=2, seed=31)
    want = oracle_place(O, workdir, rv, tp_size=tp, tp_rank=rank)

    if scenario == "success":
        ad = PlacingAdapter()
        log = []
        model = RankModule()
        ctx = ctx_for(ad, workdir)
        out["eligible_with_plain_backend"] = LS.HipPlacementStrategy().is_available(ctx)
        got = run_chain(ref, model, ctx, strategies(), log)
        out["chain_log"], out["same_model"] = log, got is model
        out["bit_exact"] = all(p.data.view(torch.uint8).cpu().numpy().tobytes() == want[n].tobytes()
                               for n, p in model.named_parameters())
        out["register_tensors_calls"] = len(REGISTERED)
        out["ctx_tensors"] = sorted(ctx.tensors) == sorted(want)
        out["reinit_calls"], out["native_calls"] = ad.reinit_calls, ad.native_calls
        return out

    if scenario == "mutated":
        import modelexpress_amd.engine as E

        real_execute = E.PlacementEngine.execute

        def execute_after_truncation(eng, plan, dst, **kw):
            size = os.path.getsize(info["files"][-1])
            with open(info["files"][-1], "r+b") as f:
                f.truncate(size // 2)
            return real_execute(eng, plan, dst, **kw)

        E.PlacementEngine.execute = execute_after_truncation
        ad = PlacingAdapter()
        log = []
        model = RankModule()
        got = run_chain(ref, model, ctx_for(ad, workdir), strategies(), log)
        out["chain_log"], out["reinit_calls"], out["native_calls"] = log, ad.reinit_calls, ad.native_calls
        out["fresh_model_returned"] = got is not model
        out["native_loaded_over_fresh_model"] = ad.native_model is got
        dirty = any(bool(p.data.view(torch.uint8).any()) for _n, p in model.named_parameters())
        out["old_model_was_written"] = dirty
        out["fresh_model_clean"] = not any(bool(p.data.view(torch.uint8).any()) for _n, p in got.named_parameters())
        return out
    raise SystemExit(f"unknown scenario {scenario!r}")


def main(argv: list) -> int:
    scenario, workdir = argv[1], argv[2]
    ref = install()
    print(json.dumps(_scenarios(ref, workdir, scenario)), flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main(sys.argv))
