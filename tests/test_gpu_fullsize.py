"""Full-size checks (benchmark configuration 2: Llama-3-8B, one TP=8 rank slice, 16 GB
staged in HBM) through properties that do not need the oracle to process 16 GB:

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
    eng.close()


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
