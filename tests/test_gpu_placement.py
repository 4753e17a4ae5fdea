"""End-to-end placement on the GPU (ingest from files and from HBM-staged shards)
against the CPU oracle, on small instances of the five benchmark families."""

import numpy as np
import pytest
import torch

from helpers import cast_setup, make_plan, oracle_place, tiny_layouts
from modelexpress_amd import models, synth

pytestmark = pytest.mark.gpu


def _stage_files(ck, shift=None):
    """Every shard file's bytes in device memory, each `staging_pad` bytes (the address the library
    recommends: data section on a 256-byte boundary) or `shift` bytes past an allocation's start."""
    out = []
    for f in ck.files():
        pad = int(f["staging_pad"]) if shift is None else shift
        host = np.fromfile(f["path"], dtype=np.uint8)
        buf = torch.empty(host.size + pad, dtype=torch.uint8, device="cuda")
        buf[pad:].copy_(torch.from_numpy(host))
        out.append(buf[pad:])
    return out


@pytest.mark.parametrize("name", list(tiny_layouts()))
def test_families_match_oracle(name, gpu_engine, gpu_engine_band, oracle, tmp_path):
    layout, tp, ep, shards, ck_kw = tiny_layouts()[name]
    ck_kw, param_dtype, cast, ratio = cast_setup(ck_kw)
    synth.write_checkpoint(layout.checkpoint(**ck_kw), str(tmp_path), n_shards=shards, seed=7)
    for tp_rank in sorted({0, tp - 1}):
        ep_rank = tp_rank % ep
        rv = layout.rank_view(tp_size=tp, tp_rank=tp_rank, ep_size=ep, ep_rank=ep_rank, param_dtype=param_dtype)
        want = oracle_place(oracle, str(tmp_path), rv, tp_size=tp, tp_rank=tp_rank, allow_cast=cast)
        ck, plan = make_plan(str(tmp_path), rv, tp_size=tp, tp_rank=tp_rank, allow_cast=cast)
        # ingest: contiguous pieces of every size copied straight to their final address; ingest_bounce: every
        # byte through the bounce slot and the kernel; ingest_band: 64 KiB slots, row bands gathered on the device
        # resident_off8: the staged files 8 bytes off the 16-byte grid (any 8-byte aligned address is accepted)
        for mode in ("ingest", "ingest_bounce", "ingest_band", "resident", "resident_off8"):
            eng = gpu_engine_band if mode == "ingest_band" else gpu_engine
            dst = eng.allocate(plan, fill=0xAB)
            if mode.startswith("resident"):
                eng.execute_resident(plan, _stage_files(ck, 8 if mode == "resident_off8" else None), dst)
            else:
                eng.set_direct_placement({"ingest": 1, "ingest_bounce": -1}.get(mode, 0))
                try:
                    stats = eng.execute(plan, dst)
                finally:
                    eng.set_direct_placement(0)
                assert stats["placed_bytes"] == sum(p.nbytes for p in plan.params)
                if mode != "ingest_band":  # packed on the host: nothing but placed bytes (times the cast factor) is read
                    assert stats["file_bytes"] == sum(p.nbytes for p in plan.params) * ratio
            sums = eng.checksums(plan)
            for p, d, s in zip(plan.params, dst, sums):
                assert d.cpu().numpy().tobytes() == want[p.name].tobytes(), (name, mode, tp_rank, p.name)
                assert s == oracle.safe_checksum(want[p.name]), (name, mode, tp_rank, p.name)


# o_proj rows of 2,560 bytes out of a pitch of 81,920: far enough apart that packed rows under direct I/O are
# read one request per row, where the tiny layouts' rows share requests
WIDE_ROWS = (models.Llama(layers=1, hidden=64, ffn=3072, q_heads=512, kv_heads=32, head_dim=80, vocab=256), 32, 1, 2, {})


@pytest.mark.parametrize("name", ["llama_tp4", "llama_f32_refit", "llama_bf16_into_f32", "deepseek_ep", "wide_rows"])
def test_direct_io_ranges_match_oracle(name, oracle, tmp_path, mxp):
    """O_DIRECT mode: every range is widened to 4 KiB blocks (also past the end of the last
    tensor) and boxes start inside the slot; results must not change.  Where the file system
    refuses O_DIRECT the engine falls back to buffered reads of the same widened ranges."""
    from modelexpress_amd.engine import PlacementEngine

    layout, tp, ep, shards, ck_kw = WIDE_ROWS if name == "wide_rows" else tiny_layouts()[name]
    ck_kw, param_dtype, cast, _ratio = cast_setup(ck_kw)
    synth.write_checkpoint(layout.checkpoint(**ck_kw), str(tmp_path), n_shards=shards, seed=9)
    tp_rank = tp - 1
    rv = layout.rank_view(tp_size=tp, tp_rank=tp_rank, ep_size=ep, ep_rank=tp_rank % ep, param_dtype=param_dtype)
    want = oracle_place(oracle, str(tmp_path), rv, tp_size=tp, tp_rank=tp_rank, allow_cast=cast)
    ck, plan = make_plan(str(tmp_path), rv, tp_size=tp, tp_rank=tp_rank, allow_cast=cast)
    # default (strided rows packed by the readers out of large requests), then whole row bands gathered on the device
    for pack in (None, False):
        eng = PlacementEngine(0, ring_slots=3, slot_bytes=1 << 17, reader_threads=2, streams=2, use_o_direct=True,
                              pack_strided_on_host=pack)
        dst = eng.allocate(plan, fill=0x11)
        stats = eng.execute(plan, dst)
        for p, d, s in zip(plan.params, dst, eng.checksums(plan)):
            assert d.cpu().numpy().tobytes() == want[p.name].tobytes(), (pack, p.name)
            assert s == oracle.safe_checksum(want[p.name]), (pack, p.name)
        assert stats["file_bytes"] >= stats["placed_bytes"]  # whole blocks are read
        eng.close()


def test_megatron_interleaved_qkv_refit_on_device(gpu_engine, gpu_engine_band, oracle, tmp_path, mxp):
    """A trainer-native source (fp32, by-KV-group interleaved linear_qkv saved as two row
    shards, fused [gate; up]) placed into a serving rank's bf16 qkv_proj / gate_up_proj:
    de-interleave + TP slice + fuse + cast + checksum in one pass."""
    from safetensors.torch import save_file
    from modelexpress_amd import megatron
    from modelexpress_amd.engine import Checkpoint, ParamSpec, PlacementPlan

    q_heads, kv_heads, head_dim, hidden, ffn, src_tp, dst_tp = 8, 2, 16, 64, 96, 2, 2
    g = torch.Generator().manual_seed(5)
    rows = (q_heads + 2 * kv_heads) * head_dim
    fused = torch.randn(rows, hidden, generator=g)
    fc1 = [torch.randn(2 * ffn // src_tp, hidden, generator=g) for _ in range(src_tp)]
    local = rows // src_tp
    tensors = {f"l0.linear_qkv.rank{r}": fused[r * local:(r + 1) * local].clone() for r in range(src_tp)}
    tensors.update({f"l0.linear_fc1.rank{r}": fc1[r] for r in range(src_tp)})
    save_file(tensors, str(tmp_path / "model.safetensors"))
    virtuals = megatron.qkv_virtuals([(f"l0.linear_qkv.rank{r}", r * local, (r + 1) * local) for r in range(src_tp)],
                                     ("l0.q_proj.weight", "l0.k_proj.weight", "l0.v_proj.weight"), hidden,
                                     head_dim=head_dim, q_heads=q_heads, kv_heads=kv_heads)
    virtuals += megatron.gated_virtuals([(f"l0.linear_fc1.rank{r}", r, src_tp) for r in range(src_tp)],
                                        ("l0.gate_proj.weight", "l0.up_proj.weight"), (hidden,), global_rows=2 * ffn)
    ow = dict(oracle.load_checkpoint(str(tmp_path)))
    weights = [(v.name, oracle.assemble_virtual(v.shape, "F32", [(ow[s], so, do, sh) for s, so, do, sh in v.shards]))
               for v in virtuals]
    ck = Checkpoint(str(tmp_path))
    for rank in range(dst_tp):
        params = [ParamSpec("l0.qkv_proj.weight", "BF16", ((q_heads + 2 * kv_heads) * head_dim // dst_tp, hidden)),
                  ParamSpec("l0.gate_up_proj.weight", "BF16", (2 * ffn // dst_tp, hidden))]
        oparams = {p.name: oracle.OTensor.zeros(p.shape, p.dtype) for p in params}
        oracle.MdlOracle(oparams, dst_tp, rank, allow_cast=True).load_weights(weights)
        plan = PlacementPlan(ck, params, tp_size=dst_tp, tp_rank=rank, virtual_tensors=virtuals, allow_cast=True)
        for eng in (gpu_engine, gpu_engine_band):
            dst = eng.allocate(plan, fill=0x77)
            eng.execute(plan, dst)
            for p, d, s in zip(params, dst, eng.checksums(plan)):
                assert d.cpu().numpy().tobytes() == oparams[p.name].tobytes(), (rank, p.name)
                assert s == oracle.safe_checksum(oparams[p.name])


def test_resident_placement_replays_from_a_hip_graph(gpu_engine, oracle, tmp_path, mxp):
    """The resident step is two kernel launches (accumulator clear by a fill kernel, then
    place_kernel) and no allocation or memset node, so it can be captured.  Every replay is
    checked against the eager result, with eager work and synchronisation between replays."""
    layout, tp, ep, shards, ck_kw = tiny_layouts()["llama_tp4"]
    synth.write_checkpoint(layout.checkpoint(), str(tmp_path), n_shards=shards, seed=31)
    rv = layout.rank_view(tp_size=tp, tp_rank=2)
    ck, plan = make_plan(str(tmp_path), rv, tp_size=tp, tp_rank=2)
    staged = _stage_files(ck)
    dst = gpu_engine.allocate(plan, fill=0)
    gpu_engine.execute_resident(plan, staged, dst)  # eager: also caches the pointer tables
    torch.cuda.synchronize()
    eager_sums = gpu_engine.checksums(plan)
    eager = [d.clone() for d in dst]
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            gpu_engine.execute_resident(plan, staged, dst, stream=torch.cuda.current_stream().cuda_stream)
    for replay in range(3):
        for d in dst:
            d.fill_(replay + 1)  # eager work between replays; also proves the replay rewrites everything
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert gpu_engine.checksums(plan) == eager_sums, replay
        assert all(torch.equal(a, b) for a, b in zip(eager, dst)), replay
    # a replay reads the staged bytes anew: change one source byte and the output follows
    t = [x for x in ck.tensors() if x.name == "model.norm.weight"][0]
    staged[t.file_index][t.file_offset] ^= 0xFF
    graph.replay()
    torch.cuda.synchronize()
    idx = [p.name for p in plan.params].index("model.norm.weight")
    assert gpu_engine.checksums(plan)[idx] != eager_sums[idx]


@pytest.mark.parametrize("side_stream", [False, True])
def test_ingest_waits_for_work_already_queued_on_the_callers_stream(side_stream, gpu_engine, oracle, tmp_path):
    """The engine writes from private streams.  Work the caller queued on its own stream before the call
    (here: a long spin, then fills of every destination) must land BEFORE the placed bytes, as it
    would ahead of ``destination.copy_(source)`` on that stream (installer.py:419-424)."""
    layout, tp, ep, shards, ck_kw = tiny_layouts()["llama_tp4"]
    synth.write_checkpoint(layout.checkpoint(), str(tmp_path), n_shards=shards, seed=41)
    rv = layout.rank_view(tp_size=tp, tp_rank=1)
    want = oracle_place(oracle, str(tmp_path), rv, tp_size=tp, tp_rank=1)
    ck, plan = make_plan(str(tmp_path), rv, tp_size=tp, tp_rank=1)
    dst = gpu_engine.allocate(plan, fill=0)
    gpu_engine.prepare(plan)
    stream = torch.cuda.Stream() if side_stream else torch.cuda.current_stream()
    with torch.cuda.stream(stream):
        torch.cuda._sleep(100_000_000)  # a few hundred milliseconds of queued device time
        for d in dst:
            d.fill_(0xEE)
        gpu_engine.execute(plan, dst)  # the calling thread's current stream is the one waited for
    torch.cuda.synchronize()
    for p, d, s in zip(plan.params, dst, gpu_engine.checksums(plan)):
        assert d.cpu().numpy().tobytes() == want[p.name].tobytes(), p.name
        assert s == oracle.safe_checksum(want[p.name]), p.name


def test_resident_launches_of_one_plan_on_two_streams_do_not_share_tables(gpu_engine, oracle, tmp_path):
    """Double-buffered use: the same plan launched asynchronously into buffer set A on one stream and,
    right away, into set B on another.  The second call rewrites the plan's pointer tables; the first
    launch must still land wholly in A."""
    layout, tp, ep, shards, ck_kw = tiny_layouts()["llama_tp4"]
    synth.write_checkpoint(layout.checkpoint(), str(tmp_path), n_shards=shards, seed=42)
    rv = layout.rank_view(tp_size=tp, tp_rank=3)
    want = oracle_place(oracle, str(tmp_path), rv, tp_size=tp, tp_rank=3)
    ck, plan = make_plan(str(tmp_path), rv, tp_size=tp, tp_rank=3)
    staged = _stage_files(ck)
    sets = [gpu_engine.allocate(plan, fill=0x5A + k) for k in range(4)]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    with torch.cuda.stream(streams[0]):
        torch.cuda._sleep(50_000_000)  # keeps the first launch pending while the second call runs on the host
    for k, dst in enumerate(sets):
        gpu_engine.execute_resident(plan, staged, dst, stream=streams[k % 2].cuda_stream)
    torch.cuda.synchronize()
    for k, dst in enumerate(sets):
        for p, d in zip(plan.params, dst):
            assert d.cpu().numpy().tobytes() == want[p.name].tobytes(), (k, p.name)
    assert gpu_engine.checksums(plan) == [oracle.safe_checksum(want[p.name]) for p in plan.params]


def test_empty_and_scalar_tensors(gpu_engine, gpu_engine_band, oracle, tmp_path, mxp):
    """Zero-element tensors, 0-dim tensors and odd byte counts through the whole path."""
    from safetensors.torch import save_file
    from modelexpress_amd.engine import Checkpoint, ParamSpec, PlacementPlan

    tensors = {"empty.weight": torch.zeros((0, 4)), "scalar.weight": torch.tensor(2.5),
               "odd.weight": torch.arange(7, dtype=torch.uint8), "one.weight": torch.tensor([1.0], dtype=torch.bfloat16),
               "a.q_proj.input_scale": torch.tensor(0.5), "a.k_proj.input_scale": torch.tensor(1.5),
               "a.v_proj.input_scale": torch.tensor(2.5)}
    save_file(tensors, str(tmp_path / "model.safetensors"))
    params = [ParamSpec("empty.weight", "F32", (0, 4)), ParamSpec("scalar.weight", "F32", ()),
              ParamSpec("odd.weight", "U8", (7,)), ParamSpec("one.weight", "BF16", (1,)),
              ParamSpec("a.qkv_proj.input_scale", "F32", (3,))]
    ow = oracle.load_checkpoint(str(tmp_path))
    oparams = {p.name: oracle.OTensor.zeros(p.shape, p.dtype) for p in params}
    oracle.MdlOracle(oparams).load_weights(ow)
    assert oparams["a.qkv_proj.input_scale"].tobytes() == np.array([0.5, 1.5, 2.5], dtype=np.float32).tobytes()
    ck = Checkpoint(str(tmp_path))
    plan = PlacementPlan(ck, params)
    for eng in (gpu_engine, gpu_engine_band):
        dst = eng.allocate(plan, fill=0xEE)
        eng.execute(plan, dst)
        for p, d, s in zip(params, dst, eng.checksums(plan)):
            assert d.cpu().numpy().tobytes() == oparams[p.name].tobytes(), p.name
            assert s == oracle.safe_checksum(oparams[p.name]), p.name
    assert gpu_engine.checksum32([torch.empty(0, dtype=torch.uint8, device="cuda")]) == ["00000000"]


@pytest.mark.parametrize("name", list(tiny_layouts()))
def test_fused_digests_match_oracle(name, oracle, tmp_path, mxp):
    """With fused digests on, the placement kernel accumulates the ``tensor_digest`` sums of what it stores
    (refit/reshard/verify.py:112-150): for every family, every execution mode and the casts, the digest of
    each parameter equals the oracle's digest of the expected bytes and the stand-alone digest of the
    finished buffer; bytes and checksums are unchanged."""
    from modelexpress_amd.engine import PlacementEngine

    layout, tp, ep, shards, ck_kw = tiny_layouts()[name]
    ck_kw, param_dtype, cast, _ratio = cast_setup(ck_kw)
    synth.write_checkpoint(layout.checkpoint(**ck_kw), str(tmp_path), n_shards=shards, seed=17)
    tp_rank = tp - 1
    rv = layout.rank_view(tp_size=tp, tp_rank=tp_rank, ep_size=ep, ep_rank=tp_rank % ep, param_dtype=param_dtype)
    want = oracle_place(oracle, str(tmp_path), rv, tp_size=tp, tp_rank=tp_rank, allow_cast=cast)
    ck, plan = make_plan(str(tmp_path), rv, tp_size=tp, tp_rank=tp_rank, allow_cast=cast)
    for mode, kw in (("ingest", {}), ("ingest_band", dict(ring_slots=3, slot_bytes=1 << 16, pack_strided_on_host=False)), ("resident", {})):
        eng = PlacementEngine(0, **kw)
        dst = eng.allocate(plan, fill=0x5A)
        with pytest.raises(mxp.MxpError, match="did not accumulate digests"):
            eng.execute(plan, dst) if mode != "resident" else eng.execute_resident(plan, _stage_files(ck), dst)
            torch.cuda.synchronize()
            eng.digests(plan)
        eng.set_fused_digests(True)
        for _ in range(2):  # the sums are cleared by every execute
            if mode == "resident":
                eng.execute_resident(plan, _stage_files(ck), dst)
            else:
                eng.execute(plan, dst)
        fused = eng.digests(plan)
        alone = eng.digest(dst, [p.nbytes for p in plan.params])
        sums = eng.checksums(plan)
        for p, d, f, a, s in zip(plan.params, dst, fused, alone, sums):
            assert d.cpu().numpy().tobytes() == want[p.name].tobytes(), (name, mode, p.name)
            assert f == a == oracle.tensor_digest(want[p.name]), (name, mode, p.name)
            assert s == oracle.safe_checksum(want[p.name]), (name, mode, p.name)
        eng.close()


def test_fused_digests_on_odd_sizes_and_narrow_paths(oracle, tmp_path, mxp):
    """Buffers whose size is not a multiple of 4 (ragged bytes), of 4 KiB (tail words) or of 16 (head / tail
    pieces moved by the 4-, 2- and 1-byte paths), a column slice with odd row length, and a narrowing cast with
    an odd element count: the fused digest still equals the oracle's and the stand-alone one."""
    from safetensors.numpy import save_file

    from modelexpress_amd.engine import Checkpoint, ParamSpec, PlacementEngine, PlacementPlan

    rng = np.random.default_rng(5)
    tensors = {
        "u8_ragged": rng.integers(0, 256, 4096 * 3 + 4 * 17 + 3, dtype=np.uint8),   # rows + tail words + 3 ragged bytes
        "u8_tiny": rng.integers(0, 256, 7, dtype=np.uint8),                           # one word + ragged
        "u8_one": rng.integers(0, 256, 1, dtype=np.uint8),
        "f16_odd": rng.integers(0, 1 << 16, 4099, dtype=np.uint16).view(np.float16),  # n % 4 == 2
        "f32_odd": rng.standard_normal(2051).astype(np.float32),                      # cast to bf16: n % 4 == 2
        "cols": rng.integers(0, 256, (37, 52), dtype=np.uint8),                       # TP column slice: 26-byte rows off the 4-byte grid
        "rows": rng.integers(-2 ** 31, 2 ** 31, (6, 1027), dtype=np.int64).astype(np.int32),  # negative words, row slice
    }
    save_file(tensors, str(tmp_path / "model.safetensors"))
    ck = Checkpoint(str(tmp_path))
    params = [ParamSpec("u8_ragged", "U8", (tensors["u8_ragged"].size,)), ParamSpec("u8_tiny", "U8", (7,)), ParamSpec("u8_one", "U8", (1,)),
              ParamSpec("f16_odd", "F16", (4099,)), ParamSpec("f32_odd", "BF16", (2051,)), ParamSpec("cols", "U8", (37, 26)),
              ParamSpec("rows", "I32", (3, 1027))]
    plan = PlacementPlan(ck, params, tp_size=2, tp_rank=1, allow_cast=True)
    want = {"u8_ragged": tensors["u8_ragged"], "u8_tiny": tensors["u8_tiny"], "u8_one": tensors["u8_one"], "f16_odd": tensors["f16_odd"],
            "f32_odd": oracle.cast_f32_bf16_bits(tensors["f32_odd"].view(np.uint32)).astype(np.uint16)}
    want["cols"] = np.ascontiguousarray(tensors["cols"][:, 26:])  # 26-byte rows: 2-byte units
    want["rows"] = np.ascontiguousarray(tensors["rows"][3:])
    eng = PlacementEngine(0)
    eng.set_fused_digests(True)
    dst = eng.allocate(plan, fill=0)
    eng.execute(plan, dst)
    fused, alone = eng.digests(plan), eng.digest(dst, [p.nbytes for p in plan.params])
    for p, d, f, a in zip(plan.params, dst, fused, alone):
        got = d.cpu().numpy().tobytes()
        assert got == np.ascontiguousarray(want[p.name]).tobytes(), p.name
        assert f == a == oracle.tensor_digest_bytes(got), p.name
    eng.close()


@pytest.mark.parametrize("seed", range(40))
def test_random_models_on_the_device(seed, oracle, tmp_path, mxp):
    """The seeded random models of test_planner_random (odd extents down to one element, 0-D to 4-D tensors, TP
    on any axis, fused groups on either axis, premerged pairs, fp32 into bf16) executed on the device, ingest and
    resident, with fused digests: bytes, checksums and digests against the oracle."""
    from test_planner_random import build_random_model, oracle_result

    from modelexpress_amd.engine import Checkpoint, ParamSpec, PlacementEngine, PlacementPlan

    path, params, tp, rank, cast = build_random_model(seed, tmp_path)
    want = oracle_result(oracle, path, params, tp, rank, cast)
    if want is None:
        pytest.skip("the oracle refuses this model (the planner's refusal is checked on the CPU)")
    ck = Checkpoint(str(path))
    plan = PlacementPlan(ck, [ParamSpec(n, dt, tuple(shape)) for n, (dt, shape) in params.items()], tp_size=tp, tp_rank=rank,
                         allow_cast=cast)
    eng = PlacementEngine(0, ring_slots=3, slot_bytes=1 << 16)
    eng.set_fused_digests(True)
    for mode in ("ingest", "resident"):
        dst = eng.allocate(plan, fill=0x3C)
        if mode == "resident":
            eng.execute_resident(plan, _stage_files(ck), dst)
        else:
            eng.execute(plan, dst)
        sums, digests = eng.checksums(plan), eng.digests(plan)
        for p, d, s, g in zip(plan.params, dst, sums, digests):
            assert d.cpu().numpy().tobytes()[: p.nbytes] == want[p.name].tobytes(), (seed, mode, p.name)
            assert s == oracle.safe_checksum(want[p.name]) and g == oracle.tensor_digest(want[p.name]), (seed, mode, p.name)
    eng.close()


@pytest.mark.parametrize("tp", [1, 2])
def test_overlapping_writes_keep_the_later_tensor_on_device(tp, gpu_engine, gpu_engine_band, oracle, tmp_path):
    """A checkpoint with gate_proj, up_proj and a premerged gate_up_proj: tensors installed one after the other
    (engines/vllm/refit/installer.py:419-424) leave the later one's bytes.  The plan settles the order before any
    byte moves, so every execution mode gives the serial result, and the fused checksums are those of the bytes
    that stay."""
    from safetensors.torch import save_file
    from modelexpress_amd.engine import Checkpoint, ParamSpec, PlacementPlan

    g = torch.Generator().manual_seed(11)
    inter, hidden = 192, 96
    tensors = {"mlp.gate_up_proj.weight": torch.randn(2 * inter, hidden, generator=g).to(torch.bfloat16),
               "mlp.up_proj.weight": torch.randn(inter, hidden, generator=g).to(torch.bfloat16),
               "mlp.gate_proj.weight": torch.randn(inter, hidden, generator=g).to(torch.bfloat16),
               "mlp.down_proj.weight": torch.randn(hidden, inter, generator=g).to(torch.bfloat16)}
    save_file(tensors, str(tmp_path / "model.safetensors"))
    ck = Checkpoint(str(tmp_path))
    ow = dict(oracle.load_checkpoint(str(tmp_path)))
    order = [t.name for t in ck.tensors()]
    for rank in range(tp):
        specs = [ParamSpec("mlp.gate_up_proj.weight", "BF16", (2 * inter // tp, hidden)),
                 ParamSpec("mlp.down_proj.weight", "BF16", (hidden, inter // tp))]
        oparams = {p.name: oracle.OTensor.zeros(p.shape, p.dtype) for p in specs}
        oracle.MdlOracle(oparams, tp, rank).load_weights([(n, ow[n]) for n in order])
        plan = PlacementPlan(ck, specs, tp_size=tp, tp_rank=rank)
        assert sum(q["bytes_written"] for q in plan.param_info()) == sum(p.nbytes for p in plan.params)
        for mode in ("ingest", "ingest_bounce", "ingest_band", "resident"):
            eng = gpu_engine_band if mode == "ingest_band" else gpu_engine
            dst = eng.allocate(plan, fill=0xCD)
            if mode == "resident":
                eng.execute_resident(plan, _stage_files(ck), dst)
            else:
                eng.set_direct_placement({"ingest": 1, "ingest_bounce": -1}.get(mode, 0))
                try:
                    eng.execute(plan, dst)
                finally:
                    eng.set_direct_placement(0)
            for p, d, s in zip(plan.params, dst, eng.checksums(plan)):
                assert d.cpu().numpy().tobytes() == oparams[p.name].tobytes(), (tp, rank, mode, p.name)
                assert s == oracle.safe_checksum(oparams[p.name]), (tp, rank, mode, p.name)
