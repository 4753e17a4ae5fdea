"""Full-size checks of the benchmark configurations (2: Llama-3-8B, one TP=8 rank slice, 16 GB staged
in HBM; 3: the same rank refitted from a 32 GB fp32 checkpoint with the real 1e-6 edge-case density;
4: one Mixtral-8x7B layer's expert stack at its real shapes; 5: the dense and MoE layers of a
DeepSeek-V3 rank share at their real shapes, fp8 weights with their 128x128 scale tiles) through
properties that do not need the oracle to process the whole checkpoint:

* the checkpoint is generated on the device by the seeded generator, which produces the
  same bytes as the host generator, so any single tensor can be regenerated on the host
  and pushed through the CPU oracle's slice rule;
* the checksum accumulated inside the placement kernel must equal the stand-alone
  checksum of the finished buffer (a second, independent device pass) for all 195
  buffers, and the oracle's checksum for the regenerated ones;
* placing twice gives identical bytes (no dependence on what the buffers held).
"""

import ctypes as C

import numpy as np
import pytest
import torch

from modelexpress_amd import _lib as L
from modelexpress_amd import models, synth
from modelexpress_amd.engine import Checkpoint, PlacementEngine, PlacementPlan

pytestmark = pytest.mark.gpu

SEED = 77
TP, RANK = 8, 5


def _host_tensor(spec, seed) -> np.ndarray:
    n = spec.nbytes // L.DTYPE_SIZE[spec.dtype]
    buf = np.empty(spec.nbytes, dtype=np.uint8)
    L.check(L.lib().mxp_synth_host(C.c_void_p(buf.ctypes.data), n, L.DTYPE_CODE[spec.dtype], spec.kind,
                                   synth.tensor_seed(seed, spec.name), 8))
    return buf.reshape(tuple(spec.shape) + (L.DTYPE_SIZE[spec.dtype],))


def test_llama3_8b_rank_slice_full_size(oracle, oracle_c, tmp_path, mxp):
    layout = models.Llama()
    tensors = layout.checkpoint()
    by_name = {t.name: t for t in tensors}
    synth.write_headers_only(tensors, str(tmp_path), n_shards=4)
    ck = Checkpoint(str(tmp_path))
    assert len(ck) == 291 and sum(t.nbytes for t in ck.tensors()) == 16_060_522_496
    rv = layout.rank_view(tp_size=TP, tp_rank=RANK)
    plan = PlacementPlan(ck, rv.params, tp_size=TP, tp_rank=RANK, stacked_params_mapping=rv.stacked_params_mapping)
    assert len(plan.params) == 195 and plan.totals()["placed_bytes"] == 2_008_031_232
    eng = PlacementEngine(0)
    staged = synth.stage_on_device(ck, tensors, seed=SEED)
    dst = eng.allocate(plan, fill=0x5A)
    eng.execute_resident(plan, staged, dst)
    fused = eng.checksums(plan)
    alone = eng.checksum32(dst)
    assert fused == alone  # 195 buffers, two independent device passes

    # regenerate single tensors on the host and apply the oracle's slice rule
    OT = oracle.OTensor
    m = oracle.MdlOracle({}, tp_size=TP, tp_rank=RANK)
    idx = {p.name: i for i, p in enumerate(plan.params)}
    layer = "model.layers.17."
    q, k, v = (OT(_host_tensor(by_name[layer + f"self_attn.{x}_proj.weight"], SEED), "BF16") for x in "qkv")
    qkv_shape = plan.params[idx[layer + "self_attn.qkv_proj.weight"]].shape
    parts = [m.tp_local_tensor(t, (t.shape[0] // TP, t.shape[1])) for t in (q, k, v)]
    want_qkv = np.concatenate([np.ascontiguousarray(p.data) for p in parts])
    assert want_qkv.shape[:2] == tuple(qkv_shape)
    checks = {layer + "self_attn.qkv_proj.weight": want_qkv}
    o = OT(_host_tensor(by_name[layer + "self_attn.o_proj.weight"], SEED), "BF16")
    checks[layer + "self_attn.o_proj.weight"] = np.ascontiguousarray(m.tp_local_tensor(o, (4096, 512)).data)
    d = OT(_host_tensor(by_name[layer + "mlp.down_proj.weight"], SEED), "BF16")
    checks[layer + "mlp.down_proj.weight"] = np.ascontiguousarray(m.tp_local_tensor(d, (4096, 1792)).data)
    n = OT(_host_tensor(by_name["model.norm.weight"], SEED), "BF16")
    checks["model.norm.weight"] = np.ascontiguousarray(n.data)
    for name, want in checks.items():
        got = dst[idx[name]].cpu().numpy()
        assert got.tobytes() == want.tobytes(), name
        assert fused[idx[name]] == oracle_c.checksum32(want), name
    assert fused[idx["model.norm.weight"]] == oracle.safe_checksum_bytes(checks["model.norm.weight"])

    # idempotence: a second placement over the finished buffers changes nothing
    before = [t.clone() for t in dst[:8]]
    eng.execute_resident(plan, staged, dst)
    assert eng.checksums(plan) == fused
    assert all(torch.equal(a, b) for a, b in zip(before, dst[:8]))

    # the tensor_digest sums accumulated by the placement itself equal a second pass over the finished buffers
    eng.set_fused_digests(True)
    eng.execute_resident(plan, staged, dst)
    assert eng.digests(plan) == eng.digest(dst)
    assert eng.checksums(plan) == fused
    eng.close()


def _check_params_against_oracle(oracle, oracle_c, plan, rv, dst, fused, by_name, names, *, tp, rank, cast=False):
    """Regenerates on the host every checkpoint tensor that writes into the parameters ``names``, runs the
    oracle's loader over them (slice, fuse, stack, cast) and compares bytes and checksums.  Returns the
    regenerated source tensors ``{name: uint8 array of shape + (element size,)}``."""
    from helpers import oracle_place

    sources = sorted({w.tensor for w in plan.writes() if w.param in names})
    host = {n: _host_tensor(by_name[n], SEED) for n in sources}
    weights = [(n, oracle.OTensor(host[n], by_name[n].dtype)) for n in sources]
    want = oracle_place(oracle, None, rv, tp_size=tp, tp_rank=rank, allow_cast=cast, weights=weights, only_params=set(names))
    idx = {p.name: i for i, p in enumerate(plan.params)}
    for name in names:
        got = dst[idx[name]].cpu().numpy()
        assert got.tobytes() == want[name].tobytes(), name
        assert fused[idx[name]] == oracle_c.checksum32(np.frombuffer(want[name].tobytes(), dtype=np.uint8)), name
    return host


def _all_checksums_alone(eng, dst) -> list:
    out = []
    for i in range(0, len(dst), 1024):
        out += eng.checksum32(dst[i:i + 1024])
    return out


def test_llama3_8b_refit_cast_full_size(oracle, oracle_c, tmp_path, mxp):
    """Configuration 3: the resident rank slice refitted from a 32 GB fp32 checkpoint whose values carry
    denormals, infinities and NaNs at 1e-6 density each: slice + round-to-nearest-even cast + checksums in
    one launch (fsdp/adapter.py:203-206, refit/reshard/receiver.py:964-971)."""
    layout = models.Llama()
    tensors = layout.checkpoint(dtype="F32", edge_cases=models.NORMAL_EDGE)
    by_name = {t.name: t for t in tensors}
    synth.write_headers_only(tensors, str(tmp_path), n_shards=8)
    ck = Checkpoint(str(tmp_path))
    assert sum(t.nbytes for t in ck.tensors()) == 32_121_044_992
    rv = layout.rank_view(tp_size=TP, tp_rank=RANK, param_dtype="BF16")
    plan = PlacementPlan(ck, rv.params, tp_size=TP, tp_rank=RANK, stacked_params_mapping=rv.stacked_params_mapping,
                         allow_cast=True)
    totals = plan.totals()
    assert totals["placed_bytes"] == 2_008_031_232 and totals["kernel_algorithmic_bytes"] == 3 * 2_008_031_232
    eng = PlacementEngine(0)
    staged = synth.stage_on_device(ck, tensors, seed=SEED)
    dst = eng.allocate(plan, fill=0x5A)
    eng.execute_resident(plan, staged, dst)
    fused = eng.checksums(plan)
    assert fused == _all_checksums_alone(eng, dst)  # 195 buffers, two independent device passes
    layer = "model.layers.9."
    names = [layer + "self_attn.qkv_proj.weight", layer + "self_attn.o_proj.weight", layer + "mlp.down_proj.weight",
             "model.norm.weight"]
    host = _check_params_against_oracle(oracle, oracle_c, plan, rv, dst, fused, by_name, names, tp=TP, rank=RANK, cast=True)
    # the real edge-case density: at 1e-6 each, ~100 M regenerated elements hold every class
    u = np.concatenate([h.reshape(-1).view("<u4") for h in host.values()])
    mag = u & 0x7FFFFFFF
    counts = {"nan": int((mag > 0x7F800000).sum()), "inf": int((mag == 0x7F800000).sum()),
              "denormal": int(((mag != 0) & (mag < 0x00800000)).sum())}
    assert all(5 <= c <= 2000 for c in counts.values()), (counts, u.size)
    # refit again over the live buffers: same bytes
    eng.execute_resident(plan, staged, dst)
    assert eng.checksums(plan) == fused
    eng.close()


def test_mixtral_layer_expert_stack_real_shapes(oracle, oracle_c, tmp_path, mxp):
    """Configuration 4, one layer at its real shapes: eight experts' w1 / w3 [14336, 4096] fused into
    w13 [8, 28672, 4096], w2 [4096, 14336] stacked into [8, 4096, 14336] (installer.py:695-754)."""
    layout = models.Mixtral(layers=1)
    tensors = layout.checkpoint()
    by_name = {t.name: t for t in tensors}
    synth.write_headers_only(tensors, str(tmp_path), n_shards=2)
    ck = Checkpoint(str(tmp_path))
    rv = layout.rank_view()
    plan = PlacementPlan(ck, rv.params, stacked_params_mapping=rv.stacked_params_mapping, expert_mapping=rv.expert_mapping)
    shapes = {p.name: tuple(p.shape) for p in plan.params}
    pre = "model.layers.0.block_sparse_moe.experts."
    assert shapes[pre + "w13_weight"] == (8, 28672, 4096) and shapes[pre + "w2_weight"] == (8, 4096, 14336)
    eng = PlacementEngine(0)
    staged = synth.stage_on_device(ck, tensors, seed=SEED)
    dst = eng.allocate(plan, fill=0x33)
    eng.execute_resident(plan, staged, dst)
    fused = eng.checksums(plan)
    assert fused == _all_checksums_alone(eng, dst)
    _check_params_against_oracle(oracle, oracle_c, plan, rv, dst, fused, by_name,
                                 [pre + "w13_weight", pre + "w2_weight", "model.layers.0.self_attn.qkv_proj.weight"],
                                 tp=1, rank=0)
    eng.close()


def test_deepseek_v3_layers_real_shapes(oracle, oracle_c, tmp_path, mxp):
    """Configuration 5 at real shapes (three dense layers and one MoE layer of 256 routed experts, TP=8 /
    EP=8): fp8 weights with their fp32 128x128 scale tiles.  o_proj is sliced on K, so its scale tiles are
    a strided column slice ([56, 128] -> [56, 16]: rows of 64 bytes); q_b_proj / kv_b_proj on rows; the
    rank's 32 local experts are stacked with their scale tiles (installer.py:80-83,292-339,695-754)."""
    tp = ep = 8
    rank = 5
    layout = models.DeepSeekV3(layers=4, dense_layers=3)
    tensors = layout.checkpoint()
    by_name = {t.name: t for t in tensors}
    synth.write_headers_only(tensors, str(tmp_path), n_shards=6)
    ck = Checkpoint(str(tmp_path))
    rv = layout.rank_view(tp_size=tp, tp_rank=rank, ep_size=ep, ep_rank=rank)
    plan = PlacementPlan(ck, rv.params, tp_size=tp, tp_rank=rank, stacked_params_mapping=rv.stacked_params_mapping,
                         expert_mapping=rv.expert_mapping)
    shapes = {p.name: tuple(p.shape) for p in plan.params}
    a, m = "model.layers.1.self_attn.", "model.layers.3.mlp."
    assert shapes[a + "o_proj.weight"] == (7168, 2048) and shapes[a + "o_proj.weight_scale_inv"] == (56, 16)
    assert shapes[m + "experts.w13_weight"] == (32, 4096, 7168) and shapes[m + "experts.w13_weight_scale_inv"] == (32, 32, 56)
    assert shapes[m + "experts.w2_weight_scale_inv"] == (32, 56, 16)
    scale_write = [w for w in plan.writes() if w.param == a + "o_proj.weight_scale_inv"]
    assert len(scale_write) == 1 and (scale_write[0].rows, scale_write[0].row_bytes, scale_write[0].src_pitch) == (56, 64, 512)
    eng = PlacementEngine(0)
    staged = synth.stage_on_device(ck, tensors, seed=SEED)
    dst = eng.allocate(plan, fill=0x44)
    eng.execute_resident(plan, staged, dst)
    fused = eng.checksums(plan)
    assert fused == _all_checksums_alone(eng, dst)
    names = [a + "o_proj.weight", a + "o_proj.weight_scale_inv", a + "q_b_proj.weight", a + "q_b_proj.weight_scale_inv",
             a + "kv_b_proj.weight", a + "kv_b_proj.weight_scale_inv", "model.layers.2.mlp.down_proj.weight",
             "model.layers.2.mlp.down_proj.weight_scale_inv", "model.layers.2.mlp.gate_up_proj.weight_scale_inv",
             m + "experts.w13_weight", m + "experts.w13_weight_scale_inv", m + "experts.w2_weight",
             m + "experts.w2_weight_scale_inv", m + "shared_experts.gate_up_proj.weight",
             m + "shared_experts.down_proj.weight_scale_inv"]
    _check_params_against_oracle(oracle, oracle_c, plan, rv, dst, fused, by_name, names, tp=tp, rank=rank)
    eng.close()


def _room_for(n_bytes: int):
    """A directory on a file system with room for ``n_bytes`` of checkpoint files, page cache first; None if none."""
    import os
    import shutil
    import tempfile

    for base in ("/dev/shm", tempfile.gettempdir()):
        try:
            if os.path.isdir(base) and shutil.disk_usage(base).free > n_bytes * 1.2 + (2 << 30):
                return tempfile.mkdtemp(prefix="mxp_fullsize_", dir=base)
        except OSError:
            continue
    return None


def _whole_checkpoint_against_cpu_oracle(layout, tp, ep, rank, n_shards, n_files_expected, placed_expected, oracle, oracle_c, *,
                                         ck_kw=None, cast=False, resident_from_generator=False):
    """Writes a checkpoint's files at full size, places the whole rank share on the CPU with the oracle (numpy planner + C
    executor over the same files) and on the GPU twice - ingested from the files and from the staged copy - and compares
    EVERY parameter buffer byte for byte, every checksum with the oracle's safe_checksum and every digest with the
    oracle's tensor_digest (engines/vllm/refit/installer.py:419-424, tensor_utils.py:27-44, refit/reshard/verify.py:79-155).
    ``resident_from_generator``: the staged copy comes from the device-side generator (the same bytes as the files)
    instead of reading the files back, for checkpoints too large to read twice."""
    import shutil

    from oracle import cpu_path

    tensors = layout.checkpoint(**(ck_kw or {}))
    total = sum(t.nbytes for t in tensors)
    workdir = _room_for(total)
    if workdir is None:
        pytest.skip(f"no file system with room for the {total / 1e9:.1f} GB checkpoint")
    try:
        synth.write_checkpoint(tensors, workdir, n_shards=n_shards, seed=SEED, threads=16)
        ck = Checkpoint(workdir)
        assert len(ck.files()) == n_files_expected and sum(t.nbytes for t in ck.tensors()) == total
        rv = layout.rank_view(tp_size=tp, tp_rank=rank, ep_size=ep, ep_rank=rank % ep, param_dtype="BF16" if cast else None)
        plan = PlacementPlan(ck, rv.params, tp_size=tp, tp_rank=rank, stacked_params_mapping=rv.stacked_params_mapping,
                             expert_mapping=rv.expert_mapping, allow_cast=cast)
        assert plan.totals()["placed_bytes"] == placed_expected
        local_of = {int(r[2]): int(r[4]) for r in (rv.expert_mapping or [])}
        nan_bits = 0x7FC0
        cpu = cpu_path.run(workdir, [(p.name, p.dtype, p.shape) for p in rv.params], tp_size=tp, tp_rank=rank,
                           stacked=rv.stacked_params_mapping,
                           expert_mapping=[r[:4] for r in rv.expert_mapping] if rv.expert_mapping else None,
                           expert_local=(lambda _f, g: local_of.get(g, g)) if rv.expert_mapping else None,
                           allow_cast=cast, nan_bits=nan_bits, threads=16)
        assert cpu["placed_bytes"] == placed_expected
        want = {n: np.frombuffer(t.tobytes(), dtype=np.uint8) for n, t in cpu["params"].items()}
        want_sums = [cpu["checksums"][p.name] for p in plan.params]
        # the C executor's checksums are the oracle's own, checked against the numpy statement on the smaller buffers
        small = [p for p in plan.params if p.nbytes <= (8 << 20)]
        for p in small[:: max(1, len(small) // 200)]:
            assert cpu["checksums"][p.name] == oracle.safe_checksum_bytes(want[p.name]), p.name
        want_digests = [oracle.tensor_digest_bytes(want[p.name]) for p in plan.params]
        eng = PlacementEngine(0, nan_bits=nan_bits)
        eng.set_fused_digests(True)
        for mode in ("ingest", "resident"):
            dst = eng.allocate(plan, fill=0xE7)
            if mode == "ingest":
                stats = eng.execute(plan, dst)
                assert stats["placed_bytes"] == placed_expected
            else:
                if resident_from_generator:
                    staged = synth.stage_on_device(ck, tensors, seed=SEED)
                else:
                    staged = [torch.from_numpy(np.fromfile(f["path"], dtype=np.uint8)).cuda() for f in ck.files()]
                eng.execute_resident(plan, staged, dst)
                del staged
            sums, digests = eng.checksums(plan), eng.digests(plan)
            assert sums == want_sums, (mode, [p.name for p, a, b in zip(plan.params, sums, want_sums) if a != b][:5])
            assert digests == want_digests, (mode, [p.name for p, a, b in zip(plan.params, digests, want_digests) if a != b][:5])
            alone = []
            for i in range(0, len(dst), 1024):
                alone += eng.digest(dst[i:i + 1024])
            assert alone == want_digests  # the stand-alone pass over the finished buffers
            for p, d in zip(plan.params, dst):
                assert np.array_equal(d.view(torch.uint8).reshape(-1).cpu().numpy(), want[p.name]), (mode, p.name)
            del dst
        eng.close()
        plan.close()
        ck.close()
    finally:
        shutil.rmtree(workdir, ignore_errors=True)


def test_gpt2_small_whole_checkpoint_at_real_shapes(oracle, oracle_c, mxp):
    """Configuration 1 at its real shapes: one file, 148 fp16 tensors, 248,879,616 bytes, TP=1 - all buffers."""
    layout, tp, ep, n_shards, _dt, _kind = models.baseline_config(1)
    _whole_checkpoint_against_cpu_oracle(layout, tp, ep, 0, n_shards, 1, 248_879_616, oracle, oracle_c)


def test_llama3_8b_whole_rank_share_against_the_cpu_oracle(oracle, oracle_c, mxp):
    """Configuration 2: the 16 GB checkpoint in 4 shard files, rank 5 of 8 - all 195 buffers byte for byte."""
    layout, tp, ep, n_shards, _dt, _kind = models.baseline_config(2)
    _whole_checkpoint_against_cpu_oracle(layout, tp, ep, RANK, n_shards, 4, 2_008_031_232, oracle, oracle_c)


def test_llama3_8b_refit_whole_rank_share_against_the_cpu_oracle(oracle, oracle_c, mxp):
    """Configuration 3: the 32 GB fp32 checkpoint (denormals, infinities and NaNs at 1e-6 density each) refitted into the
    bf16 rank share - all 195 buffers byte for byte, ingested (PCIe carries fp32, cast in flight) and resident."""
    layout, tp, ep, n_shards, dt, kind = models.baseline_config(3)
    _whole_checkpoint_against_cpu_oracle(layout, tp, ep, RANK, n_shards, 8, 2_008_031_232, oracle, oracle_c,
                                         ck_kw={"dtype": dt, "edge_cases": kind}, cast=True, resident_from_generator=True)


def test_mixtral_two_layers_whole_against_the_cpu_oracle(oracle, oracle_c, mxp):
    """Configuration 4's family at real shapes, two layers: every expert of both layers stacked into w13 [8, 28672, 4096]
    / w2 [8, 4096, 14336], QKV fused - every buffer byte for byte."""
    layout = models.Mixtral(layers=2)
    placed = sum(p.nbytes for p in layout.rank_view().params)
    _whole_checkpoint_against_cpu_oracle(layout, 1, 1, 0, 2, 2, placed, oracle, oracle_c)


def test_deepseek_v3_four_layers_whole_rank_share_against_the_cpu_oracle(oracle, oracle_c, mxp):
    """Configuration 5's family at real shapes (three dense layers and one MoE layer of 256 routed experts, TP=8 / EP=8):
    fp8 weights with their fp32 128x128 scale tiles, the rank's 32 local experts stacked - every buffer of the rank."""
    layout = models.DeepSeekV3(layers=4, dense_layers=3)
    rv = layout.rank_view(tp_size=8, tp_rank=5, ep_size=8, ep_rank=5)
    placed = sum(p.nbytes for p in rv.params)
    _whole_checkpoint_against_cpu_oracle(layout, 8, 8, 5, 6, 6, placed, oracle, oracle_c, resident_from_generator=True)


def test_buffer_beyond_4_gib_wraps_positions_like_the_reference(oracle_c, gpu_engine):
    """A single buffer of 2^32 + 12,345 bytes: checksum positions wrap mod 2^32 exactly as the
    reference's masked int64 weights do (tensor_utils.py:39-42), in the stand-alone checksum,
    in the checksum fused into a copy, and in a digest (which carries no position)."""
    n = (1 << 32) + 12345
    dev = torch.empty(n, dtype=torch.uint8, device="cuda")
    chunk = 1 << 28
    host = np.empty(n, dtype=np.uint8)
    for lo in range(0, n, chunk):  # bytes = (i * 131 + 7) mod 251, built piecewise on both sides
        hi = min(n, lo + chunk)
        idx = torch.arange(lo, hi, dtype=torch.int64, device="cuda")
        dev[lo:hi] = ((idx * 131 + 7) % 251).to(torch.uint8)
        del idx
        host[lo:hi] = ((np.arange(lo, hi, dtype=np.int64) * 131 + 7) % 251).astype(np.uint8)
    want = oracle_c.checksum32(host)
    # the tail beyond 2^32 re-uses positions 0 .. 12,344: the total differs from a non-wrapping sum
    assert want == format((int(oracle_c.checksum32(host[: 1 << 32]), 16) + int(oracle_c.checksum32(host[1 << 32:]), 16)) & 0xFFFFFFFF, "08x")
    assert gpu_engine.checksum32([dev]) == [want]
    out = torch.empty(n, dtype=torch.uint8, device="cuda")
    assert gpu_engine.copy_batch([dev], [out], [n]) == [want]
    assert torch.equal(out[-(1 << 20):], dev[-(1 << 20):]) and torch.equal(out[: 1 << 20], dev[: 1 << 20])
    assert gpu_engine.digest([out]) == gpu_engine.digest([dev])


def test_transposes_beyond_4_gib(gpu_engine, oracle_c):
    """A transposed copy larger than 4 GiB on each side (offsets and tile indices beyond 32 bits):
    transposing twice gives the source back, a strip pulled to the host equals the host transpose,
    and the fused checksum equals the stand-alone checksum of the result."""
    rows, cols = 70_000, 33_000  # 4.62 GB of bf16 per side; neither extent is a tile multiple
    src = torch.empty(rows * cols * 2, dtype=torch.uint8, device="cuda").random_(0, 256)
    mid = torch.empty_like(src)
    c_mid = gpu_engine.permute_copy(src, mid, (rows, cols), (1, 0), 2)
    assert c_mid == gpu_engine.checksum32([mid], [mid.numel()])[0]
    s2 = src.view(torch.int16).view(rows, cols)
    m2 = mid.view(torch.int16).view(cols, rows)
    for r0, c0 in ((0, 0), (rows - 300, cols - 500), (33_333, 17_001)):  # strips around both ends and past 4 GiB
        want = s2[r0:r0 + 300, c0:c0 + 500].cpu().numpy().T
        assert np.array_equal(m2[c0:c0 + 500, r0:r0 + 300].cpu().numpy(), want), (r0, c0)
    back = torch.empty_like(src)
    gpu_engine.permute_copy(mid, back, (cols, rows), (1, 0), 2, checksum=False)
    assert torch.equal(back, src)
    del back, mid
    # the same extents converting fp32 -> bf16 on the way (source 9.2 GB), against torch's device conversion
    f = torch.randn(rows, cols, device="cuda")
    out = torch.empty(cols, rows, dtype=torch.bfloat16, device="cuda")
    gpu_engine.copy_view(f, out, (cols, rows), 2, src_strides=(1, cols), cast=1, checksum=False)
    for c0 in (0, cols - 1000, 20_000):
        assert torch.equal(out[c0:c0 + 1000].view(torch.int16), f[:, c0:c0 + 1000].t().to(torch.bfloat16).contiguous().view(torch.int16)), c0
