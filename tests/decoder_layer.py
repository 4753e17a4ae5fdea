"""A decoder layer in miniature for the recorded-copy tests, and the list of ``RecordedCopy`` descriptors
(refit/reshard/types.py:57-71: source name, op-chain, parameter, destination offset / shape / stride)
that says, by hand, what each of its loaders does.  The loaders themselves, run on full tensors on the
CPU, are the ground truth the device result is compared with; nothing here records or intercepts them."""

import torch

from modelexpress_amd.reshard import RecordedCopy


def _default_loader(param, loaded):
    param.data.copy_(loaded)


class MiniDecoderLayer(torch.nn.Module):
    """One decoder layer with the loader shapes an inference engine uses: fused QKV with per-member shard ids
    (grouped-query: fewer K/V heads), a merged [gate; up] fed either by two sources or by one pre-merged source
    (``chunk``), row-parallel projections (column slices), a vocabulary-parallel embedding with a padded tail,
    a Conv1D-style weight stored transposed, and a norm loaded by the framework's default loader."""

    def __init__(self, tp_size, tp_rank, hidden=256, heads=8, kv_heads=2, head_dim=32, inter=768, vocab=1000, dtype=torch.bfloat16):
        super().__init__()
        self.tp_size, self.tp_rank, self.hidden = tp_size, tp_rank, hidden
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

    def _vocab_span(self):
        start = self.tp_rank * self.vocab_local
        return start, min(self.vocab_local, self.vocab - start)  # the last rank's tail stays as it is

    def _vocab_loader(self, param, loaded):
        start, n = self._vocab_span()
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
                getattr(params[name], "weight_loader", _default_loader)(params[name], loaded)

    def recorded_copies(self, premerged: bool, dtype=None) -> list:
        """What the loaders above do, written down as descriptors: one per (source, destination view)."""
        h, r = self.hidden, self.tp_rank
        dt = dtype if dtype is not None else self.qkv.dtype
        rows = lambda n: (n, h)  # noqa: E731
        out = []
        for name, n, at in (("q", self.q_rows, 0), ("k", self.kv_rows, self.q_rows), ("v", self.kv_rows, self.q_rows + self.kv_rows)):
            out.append(RecordedCopy(name, (("narrow", (0, r * n, n), ()),), "qkv", at * h, rows(n), (h, 1), dt))
        n = self.inter_local
        if premerged:
            for k in (0, 1):
                chain = (("chunk", (2,), (("dim", 0),)), ("__getitem__", (k,), ()), ("narrow", (0, r * n, n), ()))
                out.append(RecordedCopy("gate_up_merged", chain, "gate_up", k * n * h, rows(n), (h, 1), dt))
        else:
            for k, name in enumerate(("gate", "up")):
                out.append(RecordedCopy(name, (("narrow", (0, r * n, n), ()),), "gate_up", k * n * h, rows(n), (h, 1), dt))
        for name in ("o_proj", "down"):
            cols = getattr(self, name).shape[1]
            out.append(RecordedCopy(name, (("narrow", (1, r * cols, cols), ()),), name, 0, (h, cols), (cols, 1), dt))
        start, n_vocab = self._vocab_span()
        out.append(RecordedCopy("embed", (("narrow", (0, start, n_vocab), ()),), "embed", 0, rows(n_vocab), (h, 1), dt))
        out.append(RecordedCopy("c_fc", (("t", (), ()), ("narrow", (0, r * n, n), ())), "c_fc", 0, rows(n), (h, 1), dt))
        out.append(RecordedCopy("norm", (), "norm", 0, (h,), (1,), dt))
        return out
