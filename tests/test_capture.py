"""Geometry capture (modelexpress_amd/capture.py) against the reference's own cases
(tests/test_reshard_refit_geometry.py, test_reshard_refit_moe_experts.py), then end to end: what the
capture records, executed on the device, must rebuild exactly what the engine's loader builds from the
full tensors (tests/test_reshard_refit_transfer.py:71-125)."""

import pytest
import torch

from modelexpress_amd.capture import CaptureResult, SourceProbe, capture_geometry, summarize_unsupported
from modelexpress_amd.reshard import execute_recorded_copies, replay_view

TP_RANK = 0
_QKV = {"q": (0, 4), "k": (4, 2), "v": (6, 2)}  # (destination row offset, rows) per member


class ToyModel(torch.nn.Module):
    """Destination parameters at their sharded shapes; the loaders narrow the full source down to the shard
    (column-parallel, row-parallel, fused qkv, unsharded) - test_reshard_refit_geometry.py:22-74."""

    def __init__(self, with_bad: bool = False, tp_rank: int = TP_RANK):
        super().__init__()
        self.tp_rank = tp_rank
        self.col = torch.nn.Parameter(torch.empty(4, 4))
        self.col.weight_loader = self._col_loader
        self.row = torch.nn.Parameter(torch.empty(4, 4))
        self.row.weight_loader = self._row_loader
        self.qkv = torch.nn.Parameter(torch.empty(8, 4))
        self.qkv.weight_loader = self._qkv_loader
        self.norm = torch.nn.Parameter(torch.empty(4))
        self.norm.weight_loader = lambda param, loaded: param.data.copy_(loaded)
        if with_bad:
            self.bad = torch.nn.Parameter(torch.empty(4, 4))
            self.bad.weight_loader = self._bad_loader

    def _col_loader(self, param, loaded):
        param.data.copy_(loaded.narrow(0, self.tp_rank * param.shape[0], param.shape[0]))

    def _row_loader(self, param, loaded):
        param.data.copy_(loaded.narrow(1, self.tp_rank * param.shape[1], param.shape[1]))

    def _qkv_loader(self, param, loaded, shard_id):
        off, size = _QKV[shard_id]
        param.data.narrow(0, off, size).copy_(loaded)

    def _bad_loader(self, param, loaded):
        param.data.copy_(loaded * 2)  # arithmetic needs the values: not a view

    def load_weights(self, weights):
        params = dict(self.named_parameters())
        for name, loaded in weights:
            if name in _QKV:
                self.qkv.weight_loader(self.qkv, loaded, name)
            else:
                params[name].weight_loader(params[name], loaded)


def _manifest(with_bad: bool = False):
    f32 = torch.float32
    m = [("col", f32, [8, 4]), ("row", f32, [4, 8]), ("q", f32, [4, 4]), ("k", f32, [2, 4]), ("v", f32, [2, 4]), ("norm", f32, [4])]
    return m + ([("bad", f32, [4, 4])] if with_bad else [])


def test_capture_op_chains_and_dest_offsets():
    # test_reshard_refit_geometry.py:88-110
    with torch.device("meta"):
        model = ToyModel()
    result = capture_geometry(model, _manifest())
    by_src = {c.src_name: c for c in result.copies}
    assert by_src["col"].op_chain == (("narrow", (0, 0, 4), ()),)
    assert by_src["col"].dest_shape == (4, 4) and by_src["col"].dest_offset == 0
    assert by_src["row"].op_chain == (("narrow", (1, 0, 4), ()),) and by_src["row"].dest_shape == (4, 4)
    assert by_src["q"].op_chain == () and by_src["q"].dest_offset == 0
    assert by_src["k"].dest_offset == 16 and by_src["v"].dest_offset == 24
    assert all(by_src[s].param_name == "qkv" for s in ("q", "k", "v"))
    assert by_src["norm"].op_chain == () and by_src["norm"].dest_shape == (4,)
    assert result.unsupported == [] and result.unattributed == 0
    assert not hasattr(model.col.weight_loader, "__wrapped__")  # the loaders are put back as they were


def test_unsupported_op_is_charged_to_its_source_only():
    # :113-140
    with torch.device("meta"):
        model = ToyModel(with_bad=True)
    result = capture_geometry(model, _manifest(with_bad=True))
    by_src = {c.src_name: c for c in result.copies}
    assert result.unsupported == ["bad"] and "bad" not in by_src
    assert by_src["col"].op_chain == (("narrow", (0, 0, 4), ()),)
    assert by_src["q"].dest_offset == 0 and by_src["norm"].op_chain == ()
    assert set(result.unsupported_reasons) == {"bad"}
    reason = result.unsupported_reasons["bad"]
    assert "unsupported op" in reason and "aten.mul" in reason and "'bad'" in reason


def test_summarize_unsupported_groups_by_cause():
    # :143-173
    reasons = {f"model.layers.0.mlp.experts.{i}.gate_proj.weight":
               f"unsupported op aten.index_copy_ on lazy 'model.layers.0.mlp.experts.{i}.gate_proj.weight' (chain=());"
               for i in range(128)}
    reasons["odd"] = "unsupported op aten.mul on lazy 'odd' (chain=());"
    assert summarize_unsupported(reasons) == [("unsupported op aten.index_copy_", 128), ("unsupported op aten.mul", 1)]
    reasons = {f"source-{i}": f"cause-{i} on lazy 'source-{i}'" for i in range(4)}
    assert summarize_unsupported(reasons, limit=None) == [(f"cause-{i}", 1) for i in range(4)]


def test_captured_row_slice_resolves_to_four_runs():
    # :176-198 the row-parallel source (4, 8), columns 0..4: four runs of 16 bytes landing contiguously
    with torch.device("meta"):
        model = ToyModel()
    row = next(c for c in capture_geometry(model, _manifest()).copies if c.src_name == "row")
    off, shape, stride = replay_view(row.op_chain, (4, 8))
    assert (off, shape, stride) == (0, (4, 4), (8, 1)) and row.dest_stride == (4, 1)
    runs = [(off + r * stride[0], r * row.dest_stride[0], shape[1]) for r in range(shape[0])]
    assert len(runs) == 4 and sum(n for _, _, n in runs) * 4 == 64 and [d * 4 for _, d, _ in runs] == [0, 16, 32, 48]


def _plain_default_loader(param, loaded):
    param.data.copy_(loaded)


class DefaultLoaderModel(torch.nn.Module):
    """A parameter with no ``weight_loader`` of its own, loaded through the framework's default (:201-219)."""

    def __init__(self):
        super().__init__()
        self.norm = torch.nn.Parameter(torch.empty(4))

    def load_weights(self, weights):
        params = dict(self.named_parameters())
        for name, loaded in weights:
            getattr(params[name], "weight_loader", _plain_default_loader)(params[name], loaded)


def test_default_loader_param_needs_default_weight_loader():
    # :222-243
    manifest = [("norm", torch.float32, [4])]
    with torch.device("meta"):
        model = DefaultLoaderModel()
    missed = capture_geometry(model, manifest)
    assert missed.copies == [] and missed.unattributed == 1
    with torch.device("meta"):
        model = DefaultLoaderModel()
    got = capture_geometry(model, manifest, default_weight_loader=_plain_default_loader)
    assert [c.src_name for c in got.copies] == ["norm"] and got.copies[0].param_name == "norm"
    assert got.copies[0].op_chain == () and got.copies[0].dest_shape == (4,) and got.unattributed == 0
    assert not hasattr(model.norm, "weight_loader")


HIDDEN, INTER, TP_SIZE, LOCAL_EXPERTS = 4, 8, 2, 2
INTER_PER_TP = INTER // TP_SIZE


class FusedMoEModel(torch.nn.Module):
    """vLLM's expert loader in miniature (test_reshard_refit_moe_experts.py:41-78): per-expert sources go
    through ``unsqueeze(0)`` / ``unbind()`` and a keyword-only ``weight_loader`` into the fused w13 buffer."""

    def __init__(self):
        super().__init__()
        self.w13_weight = torch.nn.Parameter(torch.empty(LOCAL_EXPERTS, 2 * INTER_PER_TP, HIDDEN))
        self.w13_weight.weight_loader = self._expert_loader

    def _expert_loader(self, *, param, loaded_weight, shard_id, expert_id):
        member = 0 if shard_id == "w1" else 1
        dest = param.data[expert_id].narrow(0, member * INTER_PER_TP, INTER_PER_TP)
        dest.copy_(loaded_weight.narrow(0, TP_RANK * INTER_PER_TP, INTER_PER_TP))

    def load_weights(self, weights):
        for name, loaded in weights:
            expert_id = int(name.split(".experts.")[1].split(".")[0])
            shard_id = "w1" if "gate_proj" in name else "w3"
            for local_id, loaded_expert in enumerate(loaded.unsqueeze(0).unbind(), start=expert_id):
                self.w13_weight.weight_loader(param=self.w13_weight, loaded_weight=loaded_expert, shard_id=shard_id,
                                              expert_id=local_id)


def _expert_name(e, proj):
    return f"model.layers.0.mlp.experts.{e}.{proj}.weight"


def test_per_expert_sources_capture_into_the_fused_destination():
    # test_reshard_refit_moe_experts.py:91-158
    manifest = [(_expert_name(e, proj), torch.float32, [INTER, HIDDEN]) for e in range(LOCAL_EXPERTS) for proj in ("gate_proj", "up_proj")]
    with torch.device("meta"):
        model = FusedMoEModel()
    result = capture_geometry(model, manifest)
    assert result.unsupported == [] and result.unsupported_reasons == {} and result.unattributed == 0
    assert len(result.copies) == 2 * LOCAL_EXPERTS and {c.src_name for c in result.copies} == {n for n, _, _ in manifest}
    for c in result.copies:
        assert c.param_name == "w13_weight" and c.dest_shape == (INTER_PER_TP, HIDDEN) and ("unbind", (), ()) in c.op_chain
    first = next(c for c in result.copies if c.src_name == _expert_name(0, "gate_proj"))
    ops = [name for name, _a, _k in first.op_chain]
    assert ops[:3] == ["unsqueeze", "unbind", "__getitem__"] and "narrow" in ops
    up1 = next(c for c in result.copies if c.src_name == _expert_name(1, "up_proj"))
    off, shape, stride = replay_view(up1.op_chain, (INTER, HIDDEN))
    assert off == 0 and shape[0] * shape[1] * 4 == INTER_PER_TP * HIDDEN * 4          # this rank's slice, from the start of the source
    assert up1.dest_offset * 4 == (1 * (2 * INTER_PER_TP) * HIDDEN + INTER_PER_TP * HIDDEN) * 4  # expert 1's upper (w3) half


def test_probe_reports_metadata_without_dispatching():
    p = SourceProbe.for_source("w", torch.bfloat16, (6, 10))
    v = p.narrow(0, 2, 3).t()
    assert v.shape == (10, 3) and v.dtype == torch.bfloat16 and v.dim() == 2 and v.size(0) == 10 and not v.is_contiguous()
    assert v._probe_ops == (("narrow", (0, 2, 3), ()), ("t", (), ()))
    f = torch.narrow(torch.t(p), 1, 1, 4)  # function spellings record the same ops
    assert f.shape == (10, 4) and f._probe_ops == (("t", (), ()), ("narrow", (1, 1, 4), ()))
    assert replay_view(f._probe_ops, (6, 10)) == (10, (10, 4), (1, 10))
    a, b = p.chunk(2, dim=1)
    assert a.shape == (6, 5) and b._probe_ops == (("chunk", (2,), (("dim", 1),)), ("__getitem__", (1,), ()))
    assert isinstance(CaptureResult().copies, list)


@pytest.mark.gpu
@pytest.mark.parametrize("tp_rank", [0, 1])
def test_capture_then_device_execution_rebuilds_the_loaders_result(gpu_engine, tp_rank):
    """test_reshard_refit_transfer.py:71-125: ground truth = the engine's own loader run on the full tensors;
    the reconstruction writes zeroed parameters only through the captured copies, on the device."""
    shapes = {n: tuple(s) for n, _d, s in _manifest()}
    srcs, base = {}, 0
    for name, shape in shapes.items():
        n = 1
        for s in shape:
            n *= s
        srcs[name] = (base + torch.arange(n, dtype=torch.float32)).reshape(shape).contiguous()
        base += n
    truth_model = ToyModel(tp_rank=tp_rank)
    with torch.no_grad():
        truth_model.load_weights(list(srcs.items()))
    with torch.device("meta"):
        twin = ToyModel(tp_rank=tp_rank)
    capture = capture_geometry(twin, _manifest())
    assert capture.unsupported == [] and capture.unattributed == 0
    recon = {n: torch.zeros_like(p, device="cuda") for n, p in truth_model.named_parameters()}
    written = execute_recorded_copies(gpu_engine, capture.copies, {n: t.cuda() for n, t in srcs.items()}, recon)
    assert written == sum(p.numel() * 4 for p in recon.values())
    for name, p in truth_model.named_parameters():
        assert torch.equal(recon[name].cpu(), p.detach()), name


class MiniDecoderLayer(torch.nn.Module):
    """One decoder layer with the loader shapes an inference engine uses: fused QKV with per-member shard ids
    (grouped-query: fewer K/V heads), a merged [gate; up] fed either by two sources or by one pre-merged source
    (``chunk``), row-parallel projections (column slices), a vocabulary-parallel embedding with a padded tail,
    a Conv1D-style weight stored transposed, and a norm loaded by the framework's default loader."""

    def __init__(self, tp_size, tp_rank, hidden=256, heads=8, kv_heads=2, head_dim=32, inter=768, vocab=1000, dtype=torch.bfloat16):
        super().__init__()
        self.tp_size, self.tp_rank = tp_size, tp_rank
        self.q_rows, self.kv_rows = heads * head_dim // tp_size, kv_heads * head_dim // tp_size
        self.inter_local = inter // tp_size
        self.vocab_local = (vocab + tp_size - 1) // tp_size
        self.vocab = vocab
        P = lambda *shape: torch.nn.Parameter(torch.zeros(*shape, dtype=dtype), requires_grad=False)  # noqa: E731
        self.qkv = P(self.q_rows + 2 * self.kv_rows, hidden)
        self.qkv.weight_loader = self._qkv_loader
        self.gate_up = P(2 * self.inter_local, hidden)
        self.gate_up.weight_loader = self._gate_up_loader
        self.o_proj = P(hidden, heads * head_dim // tp_size)
        self.o_proj.weight_loader = self._row_loader
        self.down = P(hidden, self.inter_local)
        self.down.weight_loader = self._row_loader
        self.embed = P(self.vocab_local, hidden)
        self.embed.weight_loader = self._vocab_loader
        self.c_fc = P(self.inter_local, hidden)
        self.c_fc.weight_loader = self._conv1d_loader
        self.norm = P(hidden)

    def _qkv_loader(self, param, loaded, shard_id):
        rows = self.q_rows if shard_id == "q" else self.kv_rows
        offset = {"q": 0, "k": self.q_rows, "v": self.q_rows + self.kv_rows}[shard_id]
        param.data.narrow(0, offset, rows).copy_(loaded.narrow(0, self.tp_rank * rows, rows))

    def _gate_up_loader(self, param, loaded, shard_id=None):
        if shard_id is None:  # one pre-merged [gate; up] source: split, then shard each half
            for k, half in enumerate(loaded.chunk(2, dim=0)):
                self._gate_up_loader(param, half, k)
            return
        n = self.inter_local
        param.data.narrow(0, shard_id * n, n).copy_(loaded.narrow(0, self.tp_rank * n, n))

    def _row_loader(self, param, loaded):
        param.data.copy_(loaded.narrow(1, self.tp_rank * param.shape[1], param.shape[1]))

    def _vocab_loader(self, param, loaded):
        start = self.tp_rank * self.vocab_local
        n = min(self.vocab_local, self.vocab - start)  # the last rank's tail stays as it is
        param.data[:n].copy_(loaded.narrow(0, start, n))

    def _conv1d_loader(self, param, loaded):
        param.data.copy_(loaded.t().narrow(0, self.tp_rank * self.inter_local, self.inter_local))  # stored [in, out]

    def load_weights(self, weights):
        params = dict(self.named_parameters())
        for name, loaded in weights:
            if name in ("q", "k", "v"):
                self.qkv.weight_loader(self.qkv, loaded, name)
            elif name in ("gate", "up"):
                self.gate_up.weight_loader(self.gate_up, loaded, 0 if name == "gate" else 1)
            elif name == "gate_up_merged":
                self.gate_up.weight_loader(self.gate_up, loaded)
            else:
                getattr(params[name], "weight_loader", _plain_default_loader)(params[name], loaded)


@pytest.mark.gpu
@pytest.mark.parametrize("tp_size,tp_rank,premerged", [(1, 0, False), (2, 1, False), (4, 3, True)])
def test_decoder_layer_loaders_captured_and_replayed_on_the_device(gpu_engine, tp_size, tp_rank, premerged):
    """fp32 trainer tensors into bf16 engine parameters through the engine's own loaders: the captured plan,
    run on the device (and replayed after the sources changed), gives the bytes the loaders give on the CPU."""
    from modelexpress_amd.reshard import ReslicePlan

    hidden, heads, kv_heads, head_dim, inter, vocab = 256, 8, 4, 32, 768, 1000
    shapes = {"q": (heads * head_dim, hidden), "k": (kv_heads * head_dim, hidden), "v": (kv_heads * head_dim, hidden),
              "o_proj": (hidden, heads * head_dim), "down": (hidden, inter), "embed": (vocab, hidden), "c_fc": (hidden, inter), "norm": (hidden,)}
    shapes.update({"gate_up_merged": (2 * inter, hidden)} if premerged else {"gate": (inter, hidden), "up": (inter, hidden)})
    kw = dict(hidden=hidden, heads=heads, kv_heads=kv_heads, head_dim=head_dim, inter=inter, vocab=vocab)
    g = torch.Generator().manual_seed(70 + tp_rank)
    with torch.device("meta"):
        twin = MiniDecoderLayer(tp_size, tp_rank, **kw)
    capture = capture_geometry(twin, [(n, torch.float32, list(s)) for n, s in shapes.items()], default_weight_loader=_plain_default_loader)
    assert capture.unsupported == [] and capture.unattributed == 0
    assert len(capture.copies) == len(shapes) + (1 if premerged else 0)  # the pre-merged source yields two copies
    live = MiniDecoderLayer(tp_size, tp_rank, **kw).cuda()
    params = dict(live.named_parameters())
    plan = None
    for step in range(2):
        srcs = {n: torch.randn(s, generator=g) * 2 for n, s in shapes.items()}
        truth = MiniDecoderLayer(tp_size, tp_rank, **kw)
        truth.load_weights(list(srcs.items()))
        dev = {n: t.cuda() for n, t in srcs.items()} if step == 0 else dev
        if step == 0:
            plan = ReslicePlan(capture.copies, dev, params)
            plan.run(gpu_engine, dev, params)
        else:
            for n, t in srcs.items():
                dev[n].copy_(t)   # new values at the same addresses
            plan.replay()
        for name, p in truth.named_parameters():
            assert torch.equal(params[name].cpu().view(torch.int16), p.view(torch.int16)), (step, name)
    plan.close()
