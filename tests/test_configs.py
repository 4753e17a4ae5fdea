"""The five benchmark configurations have the sizes the reference-derived tables state, and
the environment registry reads live."""

from modelexpress_amd import envs, models


def _bytes(tensors):
    return sum(t.nbytes for t in tensors)


def test_gpt2_small():
    layout, tp, ep, shards, dt, kind = models.baseline_config(1)
    t = layout.checkpoint()
    assert len(t) == 148 and _bytes(t) == 248_879_616 and (tp, ep, shards, dt) == (1, 1, 1, "F16")
    assert sum(p.nbytes for p in layout.rank_view().params) == 248_879_616
    kinds = {x.name: x.kind for x in t}
    assert kinds["h.0.ln_1.weight"] == models.ONES and kinds["h.0.attn.c_attn.bias"] == models.ZEROS


def test_llama3_8b_tp8():
    layout, tp, ep, shards, dt, kind = models.baseline_config(2)
    t = layout.checkpoint()
    assert len(t) == 291 and _bytes(t) == 16_060_522_496 and (tp, shards) == (8, 4)
    rv = layout.rank_view(tp_size=8, tp_rank=3)
    assert len(rv.params) == 195 and sum(p.nbytes for p in rv.params) == 2_008_031_232
    shapes = {p.name: p.shape for p in rv.params}
    assert shapes["model.layers.0.self_attn.qkv_proj.weight"] == (768, 4096)
    assert shapes["model.layers.0.self_attn.o_proj.weight"] == (4096, 512)
    assert shapes["model.layers.0.mlp.gate_up_proj.weight"] == (3584, 4096)
    assert shapes["model.layers.0.mlp.down_proj.weight"] == (4096, 1792)
    assert shapes["model.embed_tokens.weight"] == (16032, 4096)
    # the fp32 refit checkpoint of the same shapes
    layout3, *_rest, dt3, kind3 = models.baseline_config(3)
    assert _bytes(layout3.checkpoint(dtype=dt3, edge_cases=kind3)) == 32_121_044_992 and kind3 == models.NORMAL_EDGE


def test_mixtral_8x7b():
    layout, tp, ep, shards, dt, kind = models.baseline_config(4)
    t = layout.checkpoint()
    assert _bytes(t) == 93_405_585_408 and shards == 19 and tp == 1
    rv = layout.rank_view()
    shapes = {p.name: p.shape for p in rv.params}
    assert shapes["model.layers.0.block_sparse_moe.experts.w13_weight"] == (8, 28672, 4096)
    assert shapes["model.layers.0.block_sparse_moe.experts.w2_weight"] == (8, 4096, 14336)
    assert sum(p.nbytes for p in rv.params) == 93_405_585_408
    assert ("experts.w13_", "experts.7.w3.", 7, "w3", 7) in rv.expert_mapping


def test_deepseek_v3_shapes():
    layout, tp, ep, shards, dt, kind = models.baseline_config(5)
    rv = layout.rank_view(tp_size=8, tp_rank=1, ep_size=8, ep_rank=1)
    shapes = {p.name: (p.dtype, p.shape) for p in rv.params}
    l = "model.layers.3."
    assert shapes[l + "mlp.experts.w13_weight"] == ("F8_E4M3", (32, 4096, 7168))
    assert shapes[l + "mlp.experts.w13_weight_scale_inv"] == ("F32", (32, 32, 56))
    assert shapes[l + "mlp.experts.w2_weight"] == ("F8_E4M3", (32, 7168, 2048))
    assert shapes[l + "mlp.experts.w2_weight_scale_inv"] == ("F32", (32, 56, 16))
    assert shapes[l + "self_attn.q_b_proj.weight"] == ("F8_E4M3", (3072, 1536))
    assert shapes[l + "self_attn.q_b_proj.weight_scale_inv"] == ("F32", (24, 12))
    assert shapes[l + "self_attn.kv_b_proj.weight_scale_inv"] == ("F32", (32, 4))
    assert shapes[l + "self_attn.o_proj.weight"] == ("F8_E4M3", (7168, 2048))
    assert shapes[l + "self_attn.o_proj.weight_scale_inv"] == ("F32", (56, 16))
    local = [r for r in rv.expert_mapping if r[4] >= 0]
    assert len(local) == 32 * 3 and {r[2] for r in local} == set(range(32, 64))
    ck = {t.name: t for t in layout.checkpoint()}
    e = ck[l + "mlp.experts.0.gate_proj.weight_scale_inv"]
    assert e.shape == (16, 56) and e.dtype == "F32" and ck[l + "mlp.experts.0.down_proj.weight_scale_inv"].shape == (56, 16)


def test_env_registry_reads_live(monkeypatch):
    monkeypatch.delenv("MXP_SLOT_MIB", raising=False)
    assert envs.MXP_SLOT_MIB == 0 and envs.MXP_O_DIRECT is False and envs.MXP_VERIFY_CHECKSUMS is True
    monkeypatch.setenv("MXP_SLOT_MIB", "32")
    monkeypatch.setenv("MXP_O_DIRECT", "yes")
    monkeypatch.setenv("MXP_NAN_BITS", "0xFFFF")
    assert envs.MXP_SLOT_MIB == 32 and envs.MXP_O_DIRECT is True and envs.MXP_NAN_BITS == 0xFFFF
    assert "MX_MODEL_URI" in dir(envs) and envs.is_set("MXP_SLOT_MIB")
    try:
        envs.NOT_A_VARIABLE
    except AttributeError:
        pass
    else:
        raise AssertionError("unknown variables must raise")


def test_product_never_imports_the_oracle_or_scratch_files():
    """The oracle is test infrastructure: nothing under modelexpress_amd/ or include/ may import,
    load or name it, and no committed file may reach into the scratch directory."""
    import re
    from pathlib import Path

    root = Path(__file__).resolve().parent.parent
    for path in list((root / "modelexpress_amd").rglob("*.py")) + list((root / "modelexpress_amd" / "csrc").iterdir()) + \
            list((root / "include").iterdir()):
        if path.is_file() and path.suffix in (".py", ".cpp", ".hpp", ".h", ".hip"):
            text = path.read_text()
            assert not re.search(r"\boracle\b", text), f"{path} mentions the oracle"
            assert "_work/" not in text, f"{path} names the scratch directory"
    for path in [root / "bench.py", root / "__graft_entry__.py"] + list((root / "tests").rglob("*.py")) + list((root / "oracle").glob("*.py")):
        assert "_work/" not in path.read_text() or path.name == "test_configs.py", f"{path} names the scratch directory"
