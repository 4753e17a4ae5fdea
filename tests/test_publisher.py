"""Trainer-side staging (modelexpress_amd/publisher.py) against the reference adapter's rules
(tests/test_refit_fsdp_adapter.py:69-162, test_refit_fsdp_publisher.py:21-47) and, on the device, against
``arena.copy_(src)`` evaluated by torch on the CPU."""

import pytest
import torch

from modelexpress_amd.publisher import COPY_TO_DEVICE, IN_PLACE, WIRE_DTYPE, WireStager


def test_layout_rules_of_the_reference_adapter():
    st = WireStager(None)
    w = torch.ones(2, 4, dtype=torch.bfloat16)
    out = st.stage({"w": w, "step": torch.tensor(3)}, IN_PLACE)  # a non-float entry is skipped, not published
    assert out["tensor_count"] == 1 and out["total_bytes"] == 2 * 4 * 2 and st.skipped == ["step"]
    assert out["served"]["w"].data_ptr() == w.data_ptr()          # IN_PLACE performs no copy
    st.stage({"w": w}, IN_PLACE)                                    # same storage again: fine
    with pytest.raises(NotImplementedError, match="source storage moved"):
        st.stage({"w": torch.ones(2, 4, dtype=torch.bfloat16)}, IN_PLACE)
    with pytest.raises(ValueError, match="tensor set changed"):
        st.stage({"w": w, "b": torch.ones(4, dtype=torch.bfloat16)}, IN_PLACE)
    with pytest.raises(ValueError, match="shard geometry changed"):
        st.stage({"w": torch.ones(4, 4, dtype=torch.bfloat16)}, IN_PLACE)
    with pytest.raises(ValueError, match="initialized for"):
        st.stage({"w": w}, COPY_TO_DEVICE)
    with pytest.raises(NotImplementedError, match="use COPY_TO_DEVICE to cast"):
        WireStager(None).stage({"w": torch.ones(2, 4)}, IN_PLACE)
    with pytest.raises(NotImplementedError, match="contiguous"):
        WireStager(None).stage({"w": torch.ones(4, 4, dtype=torch.bfloat16).t()}, IN_PLACE)
    with pytest.raises(NotImplementedError, match="copy_to_host"):
        WireStager(None).stage({"w": w}, "copy_to_host")
    with pytest.raises(TypeError, match="state_dict"):
        WireStager(None).stage([w], IN_PLACE)
    with pytest.raises(ValueError, match="no local shards"):
        WireStager(None).stage({"step": torch.tensor(1)}, IN_PLACE)


@pytest.mark.gpu
def test_copy_to_device_snapshot_matches_copy_(gpu_engine, oracle):
    """fp32 masters, an fp16 tensor, a bf16 tensor (copied as is), a scalar and a strided source, staged in one
    launch per step; the arenas keep their addresses across steps and the digests are those of the served bytes."""
    g = torch.Generator().manual_seed(21)
    state = {"embed": torch.randn(1000, 256, generator=g).cuda(), "w16": torch.randn(64, 96, generator=g).half().cuda(),
             "wire": torch.randn(32, 48, generator=g).bfloat16().cuda(), "scale": torch.tensor(0.37).cuda(),
             "strided": torch.randn(128, 64, generator=g).cuda().t(), "steps": torch.tensor(7).cuda()}
    st = WireStager(gpu_engine, publish_digests=True)
    addrs = None
    for step in range(3):
        out = st.stage(state)
        torch.cuda.synchronize()
        assert set(out["served"]) == {"embed", "w16", "wire", "scale", "strided"} and st.skipped == ["steps"]
        assert out["total_bytes"] == sum(state[n].numel() * 2 for n in out["served"])
        for n, arena in out["served"].items():
            want = torch.empty(state[n].shape, dtype=WIRE_DTYPE)
            want.copy_(state[n].cpu())
            assert arena.dtype == WIRE_DTYPE and torch.equal(arena.cpu().view(torch.int16), want.view(torch.int16)), (step, n)
            assert out["digests"][n] == oracle.tensor_digest_bytes(want.contiguous().reshape(-1).view(torch.uint8).numpy().tobytes())
        now = {n: a.data_ptr() for n, a in out["served"].items()}
        assert addrs is None or now == addrs  # the served buffers are registered once
        addrs = now
        for t in state.values():
            if t.is_floating_point():
                t.mul_(1.5)  # the next step's weights, same storage: the lowered plan is replayed
    moved = dict(state, embed=state["embed"].clone())
    out = st.stage(moved)  # a re-materialised source is still published (the plan is lowered again)
    torch.cuda.synchronize()
    assert torch.equal(out["served"]["embed"], moved["embed"].to(WIRE_DTYPE)) and out["served"]["embed"].data_ptr() == addrs["embed"]
    st.close()


@pytest.mark.gpu
def test_digest_publication_follows_the_environment_live(gpu_engine, monkeypatch):
    # tests/test_reshard_refit_verify.py:175-194: off by default, read at every stage, not frozen at import
    st = WireStager(gpu_engine)
    state = {"w": torch.arange(64, dtype=torch.float32).cuda()}
    monkeypatch.delenv("MX_RESHARD_PUBLISH_DIGEST", raising=False)
    assert st.stage(state)["digests"] is None
    monkeypatch.setenv("MX_RESHARD_PUBLISH_DIGEST", "1")
    out = st.stage(state)
    assert out["digests"] == {"w": gpu_engine.digest([out["served"]["w"]])[0]}
    monkeypatch.setenv("MX_RESHARD_PUBLISH_DIGEST", "0")
    assert st.stage(state)["digests"] is None
    st.close()


@pytest.mark.gpu
def test_colocated_refit_trainer_snapshot_to_engine_parameters(gpu_engine):
    """Both ends on one GPU: the trainer's fp32 state dict is snapshotted into bf16 arenas (one launch), the
    engine's loaders are described once as recorded copies, and each step re-slices the arenas into the live
    parameters (one launch) - the bytes are those of the loaders fed the bf16 tensors on the CPU."""
    from decoder_layer import MiniDecoderLayer
    from modelexpress_amd.reshard import ReslicePlan

    tp_size, tp_rank = 2, 1
    kw = dict(hidden=256, heads=8, kv_heads=4, head_dim=32, inter=768, vocab=1000)
    shapes = {"q": (256, 256), "k": (128, 256), "v": (128, 256), "gate": (768, 256), "up": (768, 256), "o_proj": (256, 256),
              "down": (256, 768), "embed": (1000, 256), "c_fc": (256, 768), "norm": (256,)}
    g = torch.Generator().manual_seed(33)
    trainer = {n: torch.randn(s, generator=g).cuda() for n, s in shapes.items()}
    live = MiniDecoderLayer(tp_size, tp_rank, **kw).cuda()
    copies = live.recorded_copies(premerged=False, dtype=WIRE_DTYPE)
    params = dict(live.named_parameters())
    stager = WireStager(gpu_engine)
    plan = None
    for step in range(3):
        served = stager.stage(trainer)["served"]
        if plan is None:
            plan = ReslicePlan(copies, served, params)
            plan.run(gpu_engine, served, params)
        else:
            plan.replay()
        torch.cuda.synchronize()
        truth = MiniDecoderLayer(tp_size, tp_rank, **kw)
        truth.load_weights([(n, t.cpu().to(WIRE_DTYPE)) for n, t in trainer.items()])
        for name, p in truth.named_parameters():
            assert torch.equal(params[name].cpu().view(torch.int16), p.view(torch.int16)), (step, name)
        for t in trainer.values():
            t.add_(torch.randn(t.shape, generator=g).cuda() * 0.01)  # an optimizer step
    plan.close()
    stager.close()
