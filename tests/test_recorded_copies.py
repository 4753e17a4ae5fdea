"""Recorded scatter copies (refit/reshard/types.py:57-71) executed on the device: the
reference's own vectors for narrow / transpose / permute op-chains
(tests/test_reshard_refit_slice_plan.py:54-79,155-197) and seeded random chains, against torch's
``dest.as_strided(...).copy_(view)`` on the CPU - the operation the reference performs."""

import numpy as np
import pytest
import torch

from modelexpress_amd.reshard import RecordedCopy, UnsupportedReshard, execute_recorded_copies, replay_view


def _apply(chain, t):
    for op, args, kw in chain:
        t = getattr(t, op)(*args, **dict(kw))
    return t


def test_replay_view_reference_vectors():
    # test_reshard_refit_slice_plan.py:155-197 (transpose, 3-D permute, narrow + transpose)
    assert replay_view((("transpose", (0, 1), ()),), (3, 4)) == (0, (4, 3), (1, 4))
    assert replay_view((("permute", (2, 0, 1), ()),), (2, 3, 4)) == (0, (4, 2, 3), (1, 12, 4))
    assert replay_view((("narrow", (0, 1, 2), ()), ("transpose", (0, 1), ())), (4, 5)) == (5, (5, 2), (1, 5))
    # :54-65 narrow(1, 0, 4) of (4, 8): four runs at source elements 0, 8, 16, 24
    assert replay_view((("narrow", (1, 0, 4), ()),), (4, 8)) == (0, (4, 4), (8, 1))
    assert replay_view((("__getitem__", ((slice(1, 3), slice(None)),), ()),), (4, 6)) == (6, (2, 6), (6, 1))
    # a copy inside the chain detaches the storage (slice_plan.py:155-159); a reshape that merges dims of a
    # non-contiguous view copies as well
    with pytest.raises(UnsupportedReshard, match="not a pure view"):
        replay_view((("transpose", (0, 1), ()), ("contiguous", (), ())), (3, 4))
    with pytest.raises(UnsupportedReshard, match="not a pure view"):
        replay_view((("transpose", (0, 1), ()), ("reshape", (12,), ())), (3, 4))
    with pytest.raises(UnsupportedReshard, match="non-tensor"):
        replay_view((("size", (), ()),), (3, 4))


CASES = [
    # (source shape, op-chain, destination parameter shape, dest_offset, dest_stride or None = contiguous view shape)
    ((3, 4), (("transpose", (0, 1), ()),), (4, 3), 0, None),
    ((2, 3, 4), (("permute", (2, 0, 1), ()),), (4, 2, 3), 0, None),
    ((4, 5), (("narrow", (0, 1, 2), ()), ("transpose", (0, 1), ())), (5, 2), 0, None),
    ((4, 8), (("narrow", (1, 0, 4), ()),), (4, 4), 0, None),
    ((64, 96), (("narrow", (0, 16, 32), ()),), (128, 96), 40 * 96, None),              # k rows of a fused qkv parameter
    ((64, 96), (("narrow", (1, 48, 48), ()),), (64, 100), 3, (100, 1)),                # column block into a wider parameter
    ((256, 192), (("transpose", (0, 1), ()),), (192, 256), 0, None),                   # whole transposed tiles
    ((130, 70), (("transpose", (0, 1), ()),), (70, 200), 50, (200, 1)),                # transposed into a strided region
    ((6, 40, 24), (("permute", (1, 2, 0), ()), ("narrow", (0, 8, 16), ())), (16, 24, 6), 0, None),
    ((32, 48), (("t", (), ()),), (48, 64), 16, (1, 48)),                               # destination strided the other way: a plain row copy
    ((20, 30), (("narrow", (0, 2, 10), ()),), (30, 10), 0, (1, 10)),                   # written transposed: the destination innermost run is the view's dim 0
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", range(len(CASES)))
@pytest.mark.parametrize("dtypes", [(torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32),
                                    (torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32), (torch.uint8, torch.uint8),
                                    (torch.float8_e4m3fn, torch.bfloat16), (torch.float16, torch.bfloat16)])
def test_recorded_copies_match_torch(gpu_engine, case, dtypes):
    src_shape, chain, param_shape, dest_offset, dest_stride = CASES[case]
    src_dt, dst_dt = dtypes
    g = torch.Generator().manual_seed(100 + case)
    if src_dt == torch.uint8:
        src = torch.randint(0, 256, src_shape, dtype=torch.uint8, generator=g)
    else:
        src = (torch.randn(src_shape, generator=g) * 3).to(src_dt)
    view = _apply(chain, src)
    stride = dest_stride if dest_stride is not None else tuple(torch.empty(view.shape).stride())
    want = torch.full(param_shape, 7, dtype=dst_dt)
    want.as_strided(view.shape, stride, dest_offset).copy_(view)
    param = torch.full(param_shape, 7, dtype=dst_dt, device="cuda")
    copy = RecordedCopy("w", chain, "p", dest_offset, tuple(view.shape), tuple(stride), dst_dt)
    n = execute_recorded_copies(gpu_engine, [copy], {"w": src.cuda()}, {"p": param})
    assert n == view.numel() * param.element_size()
    assert torch.equal(param.cpu().view(torch.uint8), want.view(torch.uint8))


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(8))
def test_random_chains_into_one_fused_parameter(gpu_engine, seed):
    """Several sources scattered into disjoint row blocks of one parameter, each through a random
    chain of narrow / transpose / permute; checked against torch on the CPU."""
    rng = np.random.default_rng(700 + seed)
    cols = int(rng.integers(3, 90))
    copies, sources, row = [], {}, 0
    blocks = []
    for k in range(int(rng.integers(2, 6))):
        nd = int(rng.integers(2, 4))
        shape = tuple(int(v) for v in rng.integers(2, 40, nd))
        src = torch.from_numpy(rng.integers(-2 ** 15, 2 ** 15, shape, dtype=np.int16)).view(torch.bfloat16)
        chain = []
        cur = src
        for _ in range(int(rng.integers(1, 4))):
            kind = int(rng.integers(0, 3))
            if kind == 0:
                d = int(rng.integers(0, cur.dim()))
                if cur.shape[d] < 2:
                    continue
                start = int(rng.integers(0, cur.shape[d] - 1))
                size = int(rng.integers(1, cur.shape[d] - start + 1))
                op = ("narrow", (d, start, size), ())
            elif kind == 1:
                a, b = (int(v) for v in rng.choice(cur.dim(), 2, replace=False))
                op = ("transpose", (a, b), ())
            else:
                op = ("permute", tuple(int(v) for v in rng.permutation(cur.dim())), ())
            chain.append(op)
            cur = _apply([op], cur)
        # flatten the leading dims of the view into rows of the fused parameter; keep it when it fits
        view = cur
        rows = int(np.prod(view.shape[:-1]))
        if view.shape[-1] > cols:
            continue
        lead = torch.empty(view.shape[:-1]).stride()
        stride = tuple(int(s) * cols for s in lead) + (1,)
        blocks.append((f"s{k}", tuple(chain), row * cols, tuple(view.shape), stride, view))
        sources[f"s{k}"] = src
        row += rows
    if not blocks:
        pytest.skip("no block fitted")
    want = torch.full((row, cols), 7, dtype=torch.bfloat16)
    for name, chain, off, shape, stride, view in blocks:
        want.as_strided(shape, stride, off).copy_(view)
        copies.append(RecordedCopy(name, chain, "fused", off, shape, stride, torch.bfloat16))
    param = torch.full((row, cols), 7, dtype=torch.bfloat16, device="cuda")
    execute_recorded_copies(gpu_engine, copies, {k: v.cuda() for k, v in sources.items()}, {"fused": param})
    assert torch.equal(param.cpu().view(torch.int16), want.view(torch.int16))


@pytest.mark.gpu
def test_nothing_moves_when_a_copy_cannot_be_resolved(gpu_engine):
    src = torch.arange(12, dtype=torch.float32).reshape(3, 4).cuda()
    param = torch.zeros(4, 3, device="cuda")
    good = RecordedCopy("w", (("transpose", (0, 1), ()),), "p", 0, (4, 3), (3, 1))
    bad = RecordedCopy("w", (("transpose", (0, 1), ()),), "p", 0, (3, 4), (4, 1))  # shape differs from the view
    with pytest.raises(UnsupportedReshard, match="!= resolved view"):
        execute_recorded_copies(gpu_engine, [good, bad], {"w": src}, {"p": param})
    assert float(param.abs().sum()) == 0.0
    with pytest.raises(UnsupportedReshard, match="leaves the parameter"):
        execute_recorded_copies(gpu_engine, [RecordedCopy("w", (), "p", 4, (3, 4), (4, 1))], {"w": src}, {"p": param})
    from modelexpress_amd._lib import MxpError

    with pytest.raises(MxpError, match="overlaps itself"):
        gpu_engine.copy_view(src, param, (3, 4), 4, dst_strides=(1, 1))


@pytest.mark.gpu
@pytest.mark.parametrize("src_dt", [torch.bfloat16, torch.float8_e4m3fn])
def test_mla_absorbed_weights_as_recorded_copies(gpu_engine, src_dt):
    """engines/vllm/refit/receiver.py:244-261 as two recorded copies out of kv_b_proj:
    W_UV = w_uv.transpose(0, 1).to(out_dtype) and W_UK_T = w_uk.permute(1, 2, 0).to(out_dtype),
    with kv_b_proj in bf16 or in fp8 (then the permute goes through the scratch transpose)."""
    H, P, V, L = 16, 128, 128, 512
    g = torch.Generator().manual_seed(5)
    kv_b = (torch.randn(H * (P + V), L, generator=g) * 0.5).to(src_dt)
    view = kv_b.view(H, P + V, L)
    w_uk, w_uv = view.split([P, V], dim=1)
    want_uv = w_uv.transpose(0, 1).to(torch.bfloat16).contiguous()
    want_ukt = w_uk.permute(1, 2, 0).to(torch.bfloat16).contiguous()
    head = ("view", (H, P + V, L), ())
    copies = [
        RecordedCopy("kv_b", (head, ("narrow", (1, P, V), ()), ("transpose", (0, 1), ())), "W_UV", 0, (V, H, L),
                     tuple(want_uv.stride()), torch.bfloat16),
        RecordedCopy("kv_b", (head, ("narrow", (1, 0, P), ()), ("permute", (1, 2, 0), ())), "W_UK_T", 0, (P, L, H),
                     tuple(want_ukt.stride()), torch.bfloat16),
    ]
    params = {"W_UV": torch.zeros(V, H, L, dtype=torch.bfloat16, device="cuda"),
              "W_UK_T": torch.zeros(P, L, H, dtype=torch.bfloat16, device="cuda")}
    ptrs = {k: v.data_ptr() for k, v in params.items()}
    for _ in range(2):  # a second cycle reuses the engine's scratch
        execute_recorded_copies(gpu_engine, copies, {"kv_b": kv_b.cuda()}, params)
    assert torch.equal(params["W_UV"].cpu().view(torch.int16), want_uv.view(torch.int16))
    assert torch.equal(params["W_UK_T"].cpu().view(torch.int16), want_ukt.view(torch.int16))
    assert {k: v.data_ptr() for k, v in params.items()} == ptrs  # written in place: graph-bound addresses are kept


@pytest.mark.gpu
def test_many_transposed_copies_share_launches(gpu_engine):
    """A refit's worth of transposed copies (one W_UK_T per layer, engines/vllm/refit/receiver.py:252-261,
    plus transposed weights of other dtypes) handed over in one call: transposes of one element type run
    as one launch, and every destination matches torch's ``as_strided().copy_()``."""
    g = torch.Generator().manual_seed(5)
    specs = []
    for layer in range(6):  # same shape, same dtype: one group
        specs.append(((8, 24, 40), (("permute", (1, 2, 0), ()),), torch.bfloat16, torch.bfloat16))
    specs += [
        ((130, 70), (("transpose", (0, 1), ()),), torch.bfloat16, torch.bfloat16),      # ragged member of the same group
        ((256, 192), (("transpose", (0, 1), ()),), torch.float32, torch.bfloat16),
        ((65, 33), (("transpose", (0, 1), ()),), torch.float32, torch.bfloat16),
        ((4, 64, 128), (("permute", (1, 2, 0), ()),), torch.float8_e4m3fn, torch.bfloat16),
        ((4, 64, 128), (("permute", (0, 2, 1), ()),), torch.float8_e4m3fn, torch.bfloat16),
        ((96, 48), (("transpose", (0, 1), ()),), torch.bfloat16, torch.float32),
        ((2048, 1024), (("transpose", (0, 1), ()),), torch.bfloat16, torch.bfloat16),   # eight waves per workgroup: its own group
        ((2048, 1024), (("transpose", (0, 1), ()),), torch.bfloat16, torch.bfloat16),
        ((64, 96), (("narrow", (0, 16, 32), ()),), torch.bfloat16, torch.bfloat16),     # a row copy in the same call
        ((7, 9), (("transpose", (0, 1), ()),), torch.float32, torch.float32),           # alone in its group
    ]
    sources, params, wants, copies = {}, {}, {}, []
    for k, (shape, chain, src_dt, dst_dt) in enumerate(specs):
        src = (torch.randn(shape, generator=g) * 3).to(src_dt)
        view = _apply(chain, src)
        stride = tuple(torch.empty(view.shape).stride())
        want = torch.full(tuple(view.shape), 7, dtype=dst_dt)
        want.copy_(view)
        sources[f"w{k}"], wants[f"p{k}"] = src.cuda(), want
        params[f"p{k}"] = torch.full(tuple(view.shape), 7, dtype=dst_dt, device="cuda")
        copies.append(RecordedCopy(f"w{k}", chain, f"p{k}", 0, tuple(view.shape), stride, dst_dt))
    for _ in range(2):  # the descriptor table is reused by the second call
        n = execute_recorded_copies(gpu_engine, copies, sources, params)
        assert n == sum(w.numel() * w.element_size() for w in wants.values())
        for name, want in wants.items():
            assert torch.equal(params[name].cpu().view(torch.uint8), want.view(torch.uint8)), name
        for p in params.values():
            p.fill_(7)


def test_expert_unbind_chain_resolves_to_the_rank_slice():
    # test_reshard_refit_moe_experts.py:127-158: expert 1's up_proj, TP rank 0 of 2, INTER=8, HIDDEN=4 fp32 -
    # unsqueeze(0) / unbind() cancel, the view is this rank's INTER/2 rows from the start of the source
    chain = (("unsqueeze", (0,), ()), ("unbind", (), ()), ("__getitem__", (0,), ()), ("narrow", (0, 0, 4), ()))
    off, shape, stride = replay_view(chain, (8, 4))
    assert (off, shape, stride) == (0, (4, 4), (4, 1))
    assert shape[0] * shape[1] * 4 == 64  # "pulled == INTER_PER_TP * HIDDEN * 4"; rank 0 reads from source byte 0


@pytest.mark.gpu
@pytest.mark.parametrize("inter,hidden,experts,tp", [(8, 4, 2, 2), (768, 2048, 8, 4)])
def test_per_expert_sources_into_fused_w13(gpu_engine, inter, hidden, experts, tp):
    """Per-expert HF sources (``experts.<e>.gate_proj`` / ``up_proj``) scattered into the fused grouped-expert
    buffer ``w13 [local_experts, 2 * inter / tp, hidden]`` through the chain vLLM's expert loader records
    (test_reshard_refit_moe_experts.py:41-78): one copy per (expert, projection), against the loader run on the CPU."""
    per = inter // tp
    g = torch.Generator().manual_seed(3)
    for rank in (0, tp - 1):
        want = torch.full((experts, 2 * per, hidden), 7, dtype=torch.bfloat16)
        sources, copies = {}, []
        for e in range(experts):
            for member, proj in enumerate(("gate_proj", "up_proj")):
                name = f"model.layers.0.mlp.experts.{e}.{proj}.weight"
                src = torch.randn(inter, hidden, generator=g)  # the trainer publishes fp32
                sources[name] = src.cuda()
                want[e].narrow(0, member * per, per).copy_(src.unsqueeze(0).unbind()[0].narrow(0, rank * per, per))
                chain = (("unsqueeze", (0,), ()), ("unbind", (), ()), ("__getitem__", (0,), ()), ("narrow", (0, rank * per, per), ()))
                copies.append(RecordedCopy(name, chain, "w13_weight", (e * 2 * per + member * per) * hidden, (per, hidden), (hidden, 1),
                                           torch.bfloat16))
        param = torch.full((experts, 2 * per, hidden), 7, dtype=torch.bfloat16, device="cuda")
        n = execute_recorded_copies(gpu_engine, copies, sources, {"w13_weight": param})
        assert n == want.numel() * 2
        assert torch.equal(param.cpu().view(torch.int16), want.view(torch.int16)), rank


def _batch_install_plan():
    """test_reshard_refit_batch_install.py:62-160: a 4x6 fp32 source re-sliced into three column blocks
    (q, k, v) and a 4x4 source re-sliced into two row blocks of one buffer - five views over two sources."""
    sources = {"qkv": torch.arange(24, dtype=torch.float32).reshape(4, 6),
               "rows": torch.arange(100, 116, dtype=torch.float32).reshape(4, 4)}
    copies = [RecordedCopy("qkv", (("narrow", (1, start, 2), ()),), name, 0, (4, 2), (2, 1))
              for name, start in (("q", 0), ("k", 2), ("v", 4))]
    copies += [RecordedCopy("rows", (("narrow", (0, start, 2), ()),), "rows", start * 4, (2, 4), (4, 1)) for start in (0, 2)]
    params = {"q": torch.zeros(4, 2), "k": torch.zeros(4, 2), "v": torch.zeros(4, 2), "rows": torch.zeros(4, 4)}
    return sources, copies, params


@pytest.mark.gpu
def test_batch_install_reconstructs_the_expected_values(gpu_engine):
    # test_reshard_refit_batch_install.py:183-196
    sources, copies, params = _batch_install_plan()
    dev = {k: v.cuda() for k, v in params.items()}
    n = execute_recorded_copies(gpu_engine, copies, {k: v.cuda() for k, v in sources.items()}, dev)
    assert n == (24 + 16) * 4
    for name, start in (("q", 0), ("k", 2), ("v", 4)):
        assert torch.equal(dev[name].cpu(), sources["qkv"][:, start:start + 2]), name
    assert torch.equal(dev["rows"].cpu(), sources["rows"])


@pytest.mark.gpu
def test_overlapping_destinations_land_in_plan_order(gpu_engine):
    # test_reshard_refit_batch_install.py:219-238: both row blocks aimed at offset 0 - the later copy wins
    sources, copies, params = _batch_install_plan()
    for c in copies[3:]:
        c.dest_offset = 0
    dev = {k: v.cuda() for k, v in params.items()}
    execute_recorded_copies(gpu_engine, copies, {k: v.cuda() for k, v in sources.items()}, dev)
    assert torch.equal(dev["rows"].cpu()[:2], torch.arange(108, 116, dtype=torch.float32).reshape(2, 4))
    assert torch.equal(dev["rows"].cpu()[2:], torch.zeros(2, 4))


@pytest.mark.gpu
def test_interleaved_column_blocks_of_one_parameter(gpu_engine):
    """Three column blocks written into ONE fused parameter: their spans interleave (the conservative
    test of receiver.py:289-321 calls that overlapping), so they run one after another - same bytes."""
    src = torch.arange(24, dtype=torch.float32).reshape(4, 6).cuda()
    fused = torch.zeros(4, 6, device="cuda")
    copies = [RecordedCopy("qkv", (("narrow", (1, start, 2), ()),), "fused", start, (4, 2), (6, 1)) for start in (4, 0, 2)]
    execute_recorded_copies(gpu_engine, copies, {"qkv": src}, {"fused": fused})
    assert torch.equal(fused, src)


@pytest.mark.gpu
def test_no_copies_is_a_no_op(gpu_engine):
    # test_reshard_refit_batch_install.py:269-284
    assert execute_recorded_copies(gpu_engine, [], {}, {}) == 0


def test_reslice_plan_splits_only_where_spans_meet():
    """The split into calls is decided when the plan is built, on CPU tensors: disjoint row blocks share one
    call; views whose spans meet start a new call at that point, in plan order."""
    from modelexpress_amd.reshard import ReslicePlan

    src = {"w": torch.zeros(8, 4)}
    p = {"p": torch.zeros(8, 4), "q": torch.zeros(8, 4)}
    rows = lambda name, start, off: RecordedCopy("w", (("narrow", (0, start, 2), ()),), name, off, (2, 4), (4, 1))  # noqa: E731
    plan = ReslicePlan([rows("p", 0, 0), rows("p", 2, 8), rows("q", 0, 0), rows("p", 4, 16)], src, p)
    assert plan.batches == [[0, 1, 2, 3]] and plan.bytes == 4 * 2 * 4 * 4
    plan = ReslicePlan([rows("p", 0, 0), rows("p", 2, 8), rows("p", 4, 4), rows("q", 0, 0), rows("p", 6, 8)], src, p)
    assert plan.batches == [[0, 1], [2, 3], [4]]  # copy 2 meets copies 0 and 1; copy 4 meets copy 2
    assert ReslicePlan([], src, p).batches == []


@pytest.mark.gpu
def test_reslice_plan_is_reused_across_steps_and_follows_moved_tensors(gpu_engine):
    """A plan built once serves every step (refit/reshard/receiver.py:787-801): new source values, the same
    addresses; then a parameter that moved; then a source whose shape changed, which is refused."""
    from modelexpress_amd.reshard import ReslicePlan

    g = torch.Generator().manual_seed(8)
    sources = {f"s{k}": torch.randn(64, 48, generator=g).cuda() for k in range(6)}
    param = torch.zeros(6 * 32, 48, dtype=torch.bfloat16, device="cuda")
    copies = [RecordedCopy(f"s{k}", (("narrow", (0, 16, 32), ()),), "fused", k * 32 * 48, (32, 48), (48, 1)) for k in range(6)]
    plan = ReslicePlan(copies, sources, {"fused": param})

    def want():
        return torch.cat([sources[f"s{k}"][16:48] for k in range(6)]).to(torch.bfloat16)

    assert plan.run(gpu_engine, sources, {"fused": param}) == param.numel() * 2
    assert torch.equal(param, want())
    arrays = plan._arrays
    for t in sources.values():
        t.normal_(generator=None)
    plan.run(gpu_engine, sources, {"fused": param})
    assert torch.equal(param, want()) and plan._arrays is arrays  # same addresses: the descriptor arrays are kept
    for t in sources.values():
        t.normal_(generator=None)
    assert plan.replay() == param.numel() * 2 and torch.equal(param, want())  # launches only, same tensors
    moved = torch.zeros_like(param)
    plan.run(gpu_engine, sources, {"fused": moved})
    assert torch.equal(moved, want()) and plan._arrays is not arrays
    sources["s0"] = torch.randn(32, 48).cuda()
    with pytest.raises(UnsupportedReshard, match="changed shape"):
        plan.run(gpu_engine, sources, {"fused": moved})


@pytest.mark.gpu
def test_view_plan_runs_from_a_hip_graph(gpu_engine):
    """``mxp_view_plan_run`` only launches kernels (no allocation, no host copy, no memset node), so a refit's
    re-slice can be recorded into a HIP graph: every replay is checked against the eager result, with eager
    work and synchronisation between replays, for row boxes, a batch of transposes and a converting one."""
    g = torch.Generator().manual_seed(12)
    srcs = [torch.randn(96, 64, generator=g).cuda() for _ in range(5)]
    dsts = [torch.zeros(48, 64, dtype=torch.bfloat16, device="cuda"),      # row box, fp32 -> bf16
            torch.zeros(64, 96, device="cuda"), torch.zeros(64, 96, device="cuda"), torch.zeros(64, 96, device="cuda"),  # transposes
            torch.zeros(64, 96, dtype=torch.bfloat16, device="cuda")]      # converting transpose
    views = [{"src": srcs[0][24:], "dst": dsts[0], "shape": (48, 64), "elem_size": 2, "src_strides": (64, 1), "cast": 1}]
    views += [{"src": srcs[k], "dst": dsts[k], "shape": (64, 96), "elem_size": 4, "src_strides": (1, 64)} for k in (1, 2, 3)]
    views += [{"src": srcs[4], "dst": dsts[4], "shape": (64, 96), "elem_size": 2, "src_strides": (1, 64), "cast": 1}]

    def want():
        return [srcs[0][24:72].to(torch.bfloat16)] + [srcs[k].t().contiguous() for k in (1, 2, 3)] + [srcs[4].t().to(torch.bfloat16).contiguous()]

    from modelexpress_amd import _lib as L

    arr = (L.ViewCopy * len(views))()
    for o, v in zip(arr, views):
        o.src, o.dst, o.ndim, o.elem_size, o.cast = v["src"].data_ptr(), v["dst"].data_ptr(), 2, v["elem_size"], v.get("cast", 0)
        o.contiguous_dst = 1
        for d in range(2):
            o.shape[d], o.src_strides[d] = v["shape"][d], v["src_strides"][d]
    plan = gpu_engine.view_plan(arr, len(views))
    assert plan.bytes == sum(d.numel() * d.element_size() for d in dsts)
    plan.run()
    torch.cuda.synchronize()
    assert all(torch.equal(d, w) for d, w in zip(dsts, want()))
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            plan.run(stream=torch.cuda.current_stream().cuda_stream)
    for step in range(3):
        for s in srcs:
            s.normal_()           # eager work between replays: new source values, same addresses
        for d in dsts:
            d.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(d, w) for d, w in zip(dsts, want())), step
    plan.close()


@pytest.mark.gpu
@pytest.mark.parametrize("tp_size,tp_rank,premerged", [(1, 0, False), (2, 1, False), (4, 3, True)])
def test_decoder_layer_descriptors_replayed_on_the_device(gpu_engine, tp_size, tp_rank, premerged):
    """fp32 trainer tensors into bf16 engine parameters: the descriptors of a decoder layer's loaders (written by
    hand, decoder_layer.py), run on the device and replayed after the sources changed, give the bytes the loaders
    themselves give on the CPU."""
    from decoder_layer import MiniDecoderLayer
    from modelexpress_amd.reshard import ReslicePlan

    hidden, heads, kv_heads, head_dim, inter, vocab = 256, 8, 4, 32, 768, 1000
    shapes = {"q": (heads * head_dim, hidden), "k": (kv_heads * head_dim, hidden), "v": (kv_heads * head_dim, hidden),
              "o_proj": (hidden, heads * head_dim), "down": (hidden, inter), "embed": (vocab, hidden), "c_fc": (hidden, inter), "norm": (hidden,)}
    shapes.update({"gate_up_merged": (2 * inter, hidden)} if premerged else {"gate": (inter, hidden), "up": (inter, hidden)})
    kw = dict(hidden=hidden, heads=heads, kv_heads=kv_heads, head_dim=head_dim, inter=inter, vocab=vocab)
    g = torch.Generator().manual_seed(70 + tp_rank)
    live = MiniDecoderLayer(tp_size, tp_rank, **kw).cuda()
    copies = live.recorded_copies(premerged)
    assert len(copies) == len(shapes) + (1 if premerged else 0)  # the pre-merged source yields two copies
    assert {c.src_name for c in copies} == set(shapes)
    params = dict(live.named_parameters())
    plan = dev = None
    for step in range(2):
        srcs = {n: torch.randn(s, generator=g) * 2 for n, s in shapes.items()}
        truth = MiniDecoderLayer(tp_size, tp_rank, **kw)
        truth.load_weights(list(srcs.items()))
        if step == 0:
            dev = {n: t.cuda() for n, t in srcs.items()}
            plan = ReslicePlan(copies, dev, params)
            plan.run(gpu_engine, dev, params)
        else:
            for n, t in srcs.items():
                dev[n].copy_(t)   # new values at the same addresses
            plan.replay()
        for name, p in truth.named_parameters():
            assert torch.equal(params[name].cpu().view(torch.int16), p.view(torch.int16)), (step, name)
    plan.close()


def test_decoder_layer_descriptors_equal_the_loaders_on_the_cpu():
    """The hand-written descriptors are themselves checked against the loaders, on the CPU, with torch's own
    ``as_strided().copy_()`` (the operation the reference performs per recorded copy)."""
    from decoder_layer import MiniDecoderLayer

    for tp_size, tp_rank, premerged in [(1, 0, False), (2, 1, True), (4, 3, False), (4, 0, True)]:
        kw = dict(hidden=64, heads=8, kv_heads=4, head_dim=8, inter=96, vocab=101)
        shapes = {"q": (64, 64), "k": (32, 64), "v": (32, 64), "o_proj": (64, 64), "down": (64, 96), "embed": (101, 64),
                  "c_fc": (64, 96), "norm": (64,)}
        shapes.update({"gate_up_merged": (192, 64)} if premerged else {"gate": (96, 64), "up": (96, 64)})
        g = torch.Generator().manual_seed(5 + tp_rank)
        srcs = {n: torch.randn(s, generator=g).to(torch.bfloat16) for n, s in shapes.items()}
        truth = MiniDecoderLayer(tp_size, tp_rank, **kw)
        truth.load_weights(list(srcs.items()))
        recon = MiniDecoderLayer(tp_size, tp_rank, **kw)
        params = dict(recon.named_parameters())
        for c in recon.recorded_copies(premerged):
            params[c.param_name].data.as_strided(c.dest_shape, c.dest_stride, c.dest_offset).copy_(_apply(c.op_chain, srcs[c.src_name]))
        for name, p in truth.named_parameters():
            assert torch.equal(params[name].view(torch.int16), p.view(torch.int16)), (tp_size, tp_rank, name)
