"""Checkpoint and rank-parameter tables for the model families the path is measured on.

A ``ModelLayout`` answers two questions with plain data:

* what a Hugging Face style checkpoint of the family contains (``checkpoint()``:
  tensor names, dtypes, shapes in file order) -- used to write seeded synthetic
  checkpoints, and
* what one serving rank allocates for it (``rank_view()``: local parameter names,
  dtypes and shapes, the stacked-parameter mapping and the expert mapping) -- the three
  things the reference's direct loader reads off the engine's model object
  (engines/vllm/refit/installer.py:470-564,773-797).

Dimensions are arguments, so tests build the same families a few kilobytes large.
"""

from __future__ import annotations

from dataclasses import dataclass, field

from .engine import ParamSpec

# synthetic content kinds (mxp_synth_*)
NORMAL, ONES, ZEROS, NORMAL_EDGE, FP8_FINITE, SCALE, NORMAL_EDGE_DENSE = range(7)


@dataclass(frozen=True)
class TensorSpec:
    name: str
    dtype: str
    shape: tuple
    kind: int = NORMAL

    @property
    def nbytes(self) -> int:
        from ._lib import DTYPE_SIZE

        n = DTYPE_SIZE[self.dtype]
        for d in self.shape:
            n *= int(d)
        return n


@dataclass
class RankView:
    params: list  # [ParamSpec]
    stacked_params_mapping: list | None = None
    expert_mapping: list | None = None
    skip_prefixes: tuple = ()


@dataclass
class ModelLayout:
    family: str
    dims: dict = field(default_factory=dict)

    def checkpoint(self, dtype: str | None = None, edge_cases: int | None = None) -> list:
        raise NotImplementedError

    def rank_view(self, tp_size: int = 1, tp_rank: int = 0, ep_size: int = 1, ep_rank: int = 0,
                  param_dtype: str | None = None) -> RankView:
        raise NotImplementedError


def _div(a: int, b: int, what: str) -> int:
    if a % b:
        raise ValueError(f"{what}={a} is not divisible by {b}")
    return a // b


# ----------------------------------------------------------------------------------------
# GPT-2 (already-fused c_attn, Conv1D [in, out] weights): every tensor is a direct copy.
# ----------------------------------------------------------------------------------------
class Gpt2(ModelLayout):
    def __init__(self, layers=12, hidden=768, ffn=3072, vocab=50257, positions=1024, dtype="F16"):
        super().__init__("gpt2", dict(layers=layers, hidden=hidden, ffn=ffn, vocab=vocab, positions=positions,
                                      dtype=dtype))

    def checkpoint(self, dtype=None, edge_cases=None):
        d = self.dims
        dt = dtype or d["dtype"]
        h, f = d["hidden"], d["ffn"]
        out = [TensorSpec("wte.weight", dt, (d["vocab"], h)), TensorSpec("wpe.weight", dt, (d["positions"], h))]
        for i in range(d["layers"]):
            p = f"h.{i}."
            out += [
                TensorSpec(p + "ln_1.weight", dt, (h,), ONES), TensorSpec(p + "ln_1.bias", dt, (h,), ZEROS),
                TensorSpec(p + "attn.c_attn.weight", dt, (h, 3 * h)), TensorSpec(p + "attn.c_attn.bias", dt, (3 * h,), ZEROS),
                TensorSpec(p + "attn.c_proj.weight", dt, (h, h)), TensorSpec(p + "attn.c_proj.bias", dt, (h,), ZEROS),
                TensorSpec(p + "ln_2.weight", dt, (h,), ONES), TensorSpec(p + "ln_2.bias", dt, (h,), ZEROS),
                TensorSpec(p + "mlp.c_fc.weight", dt, (h, f)), TensorSpec(p + "mlp.c_fc.bias", dt, (f,), ZEROS),
                TensorSpec(p + "mlp.c_proj.weight", dt, (f, h)), TensorSpec(p + "mlp.c_proj.bias", dt, (h,), ZEROS),
            ]
        out += [TensorSpec("ln_f.weight", dt, (h,), ONES), TensorSpec("ln_f.bias", dt, (h,), ZEROS)]
        return out

    def rank_view(self, tp_size=1, tp_rank=0, ep_size=1, ep_rank=0, param_dtype=None):
        if tp_size != 1:
            raise ValueError("the GPT-2 table is defined for TP=1")
        return RankView([ParamSpec(t.name, param_dtype or t.dtype, t.shape) for t in self.checkpoint()])


# ----------------------------------------------------------------------------------------
# Llama: q/k/v -> qkv_proj, gate/up -> gate_up_proj, column / row / vocab parallel.
# ----------------------------------------------------------------------------------------
class Llama(ModelLayout):
    def __init__(self, layers=32, hidden=4096, ffn=14336, q_heads=32, kv_heads=8, head_dim=128, vocab=128256,
                 dtype="BF16"):
        super().__init__("llama", dict(layers=layers, hidden=hidden, ffn=ffn, q_heads=q_heads, kv_heads=kv_heads,
                                       head_dim=head_dim, vocab=vocab, dtype=dtype))

    def _attn_ckpt(self, p, dt, kind):
        d = self.dims
        h, hd = d["hidden"], d["head_dim"]
        return [
            TensorSpec(p + "self_attn.q_proj.weight", dt, (d["q_heads"] * hd, h), kind),
            TensorSpec(p + "self_attn.k_proj.weight", dt, (d["kv_heads"] * hd, h), kind),
            TensorSpec(p + "self_attn.v_proj.weight", dt, (d["kv_heads"] * hd, h), kind),
            TensorSpec(p + "self_attn.o_proj.weight", dt, (h, d["q_heads"] * hd), kind),
        ]

    def _attn_params(self, p, dt, tp):
        d = self.dims
        h, hd = d["hidden"], d["head_dim"]
        q = _div(d["q_heads"], tp, "q_heads") * hd
        kv = _div(d["kv_heads"], tp, "kv_heads") * hd
        return [ParamSpec(p + "self_attn.qkv_proj.weight", dt, (q + 2 * kv, h)),
                ParamSpec(p + "self_attn.o_proj.weight", dt, (h, q))]

    def checkpoint(self, dtype=None, edge_cases=None):
        d = self.dims
        dt = dtype or d["dtype"]
        kind = NORMAL if edge_cases is None else edge_cases
        h, f = d["hidden"], d["ffn"]
        out = [TensorSpec("model.embed_tokens.weight", dt, (d["vocab"], h), kind)]
        for i in range(d["layers"]):
            p = f"model.layers.{i}."
            out.append(TensorSpec(p + "input_layernorm.weight", dt, (h,), kind))
            out += self._attn_ckpt(p, dt, kind)
            out.append(TensorSpec(p + "post_attention_layernorm.weight", dt, (h,), kind))
            out += [TensorSpec(p + "mlp.gate_proj.weight", dt, (f, h), kind),
                    TensorSpec(p + "mlp.up_proj.weight", dt, (f, h), kind),
                    TensorSpec(p + "mlp.down_proj.weight", dt, (h, f), kind)]
        out += [TensorSpec("model.norm.weight", dt, (h,), kind), TensorSpec("lm_head.weight", dt, (d["vocab"], h), kind)]
        return out

    def rank_view(self, tp_size=1, tp_rank=0, ep_size=1, ep_rank=0, param_dtype=None):
        d = self.dims
        dt = param_dtype or d["dtype"]
        h = d["hidden"]
        f = _div(d["ffn"], tp_size, "ffn")
        v = _div(d["vocab"], tp_size, "vocab")
        params = [ParamSpec("model.embed_tokens.weight", dt, (v, h))]
        for i in range(d["layers"]):
            p = f"model.layers.{i}."
            params.append(ParamSpec(p + "input_layernorm.weight", dt, (h,)))
            params += self._attn_params(p, dt, tp_size)
            params.append(ParamSpec(p + "post_attention_layernorm.weight", dt, (h,)))
            params += [ParamSpec(p + "mlp.gate_up_proj.weight", dt, (2 * f, h)),
                       ParamSpec(p + "mlp.down_proj.weight", dt, (h, f))]
        params += [ParamSpec("model.norm.weight", dt, (h,)), ParamSpec("lm_head.weight", dt, (v, h))]
        mapping = [("qkv_proj", "q_proj"), ("qkv_proj", "k_proj"), ("qkv_proj", "v_proj"),
                   ("gate_up_proj", "gate_proj"), ("gate_up_proj", "up_proj")]
        return RankView(params, mapping)


# ----------------------------------------------------------------------------------------
# Mixtral: per-expert w1/w3 -> w13_weight[e, half], w2 -> w2_weight[e].
# ----------------------------------------------------------------------------------------
class Mixtral(Llama):
    def __init__(self, layers=32, hidden=4096, ffn=14336, q_heads=32, kv_heads=8, head_dim=128, vocab=32000,
                 experts=8, dtype="BF16"):
        super().__init__(layers, hidden, ffn, q_heads, kv_heads, head_dim, vocab, dtype)
        self.family = "mixtral"
        self.dims["experts"] = experts

    def checkpoint(self, dtype=None, edge_cases=None):
        d = self.dims
        dt = dtype or d["dtype"]
        kind = NORMAL if edge_cases is None else edge_cases
        h, f = d["hidden"], d["ffn"]
        out = [TensorSpec("model.embed_tokens.weight", dt, (d["vocab"], h), kind)]
        for i in range(d["layers"]):
            p = f"model.layers.{i}."
            out.append(TensorSpec(p + "input_layernorm.weight", dt, (h,), kind))
            out += self._attn_ckpt(p, dt, kind)
            out.append(TensorSpec(p + "post_attention_layernorm.weight", dt, (h,), kind))
            out.append(TensorSpec(p + "block_sparse_moe.gate.weight", dt, (d["experts"], h), kind))
            for e in range(d["experts"]):
                q = p + f"block_sparse_moe.experts.{e}."
                out += [TensorSpec(q + "w1.weight", dt, (f, h), kind), TensorSpec(q + "w2.weight", dt, (h, f), kind),
                        TensorSpec(q + "w3.weight", dt, (f, h), kind)]
        out += [TensorSpec("model.norm.weight", dt, (h,), kind), TensorSpec("lm_head.weight", dt, (d["vocab"], h), kind)]
        return out

    def rank_view(self, tp_size=1, tp_rank=0, ep_size=1, ep_rank=0, param_dtype=None):
        d = self.dims
        dt = param_dtype or d["dtype"]
        h = d["hidden"]
        n_exp = d["experts"]
        local_exp = _div(n_exp, ep_size, "experts")
        f = d["ffn"] if ep_size > 1 else _div(d["ffn"], tp_size, "ffn")  # experts are TP-split only without EP
        v = _div(d["vocab"], tp_size, "vocab")
        params = [ParamSpec("model.embed_tokens.weight", dt, (v, h))]
        for i in range(d["layers"]):
            p = f"model.layers.{i}."
            params.append(ParamSpec(p + "input_layernorm.weight", dt, (h,)))
            params += self._attn_params(p, dt, tp_size)
            params.append(ParamSpec(p + "post_attention_layernorm.weight", dt, (h,)))
            params += [ParamSpec(p + "block_sparse_moe.gate.weight", dt, (n_exp, h)),
                       ParamSpec(p + "block_sparse_moe.experts.w13_weight", dt, (local_exp, 2 * f, h)),
                       ParamSpec(p + "block_sparse_moe.experts.w2_weight", dt, (local_exp, h, f))]
        params += [ParamSpec("model.norm.weight", dt, (h,)), ParamSpec("lm_head.weight", dt, (v, h))]
        mapping = [("qkv_proj", "q_proj"), ("qkv_proj", "k_proj"), ("qkv_proj", "v_proj")]
        experts = []
        lo = ep_rank * local_exp
        for e in range(n_exp):
            local = e - lo if lo <= e < lo + local_exp else -1
            experts += [("experts.w13_", f"experts.{e}.w1.", e, "w1", local),
                        ("experts.w2_", f"experts.{e}.w2.", e, "w2", local),
                        ("experts.w13_", f"experts.{e}.w3.", e, "w3", local)]
        return RankView(params, mapping, experts)


# ----------------------------------------------------------------------------------------
# DeepSeek-V3: fp8-e4m3 weights with fp32 128x128 weight_scale_inv tiles, MLA projections,
# routed experts (expert parallel) + shared expert + leading dense layers.
# ----------------------------------------------------------------------------------------
class DeepSeekV3(ModelLayout):
    def __init__(self, layers=61, dense_layers=3, hidden=7168, q_lora=1536, kv_lora=512, heads=128, qk_nope=128,
                 qk_rope=64, v_head=128, routed_experts=256, moe_ffn=2048, dense_ffn=18432, vocab=129280,
                 block=128):
        super().__init__("deepseek_v3", dict(layers=layers, dense_layers=dense_layers, hidden=hidden, q_lora=q_lora,
                                             kv_lora=kv_lora, heads=heads, qk_nope=qk_nope, qk_rope=qk_rope,
                                             v_head=v_head, routed_experts=routed_experts, moe_ffn=moe_ffn,
                                             dense_ffn=dense_ffn, vocab=vocab, block=block))

    def _blocks(self, n: int) -> int:
        b = self.dims["block"]
        return (n + b - 1) // b

    def _q(self, name, shape):
        """A block-quantised weight and its scale tiles."""
        return [TensorSpec(name + ".weight", "F8_E4M3", shape, FP8_FINITE),
                TensorSpec(name + ".weight_scale_inv", "F32", (self._blocks(shape[0]), self._blocks(shape[1])), SCALE)]

    def _qp(self, name, shape):
        return [ParamSpec(name + ".weight", "F8_E4M3", shape),
                ParamSpec(name + ".weight_scale_inv", "F32", (self._blocks(shape[0]), self._blocks(shape[1])))]

    def checkpoint(self, dtype=None, edge_cases=None):
        d = self.dims
        h = d["hidden"]
        qk = d["qk_nope"] + d["qk_rope"]
        out = [TensorSpec("model.embed_tokens.weight", "BF16", (d["vocab"], h))]
        for i in range(d["layers"]):
            p = f"model.layers.{i}."
            out.append(TensorSpec(p + "input_layernorm.weight", "BF16", (h,)))
            out += self._q(p + "self_attn.q_a_proj", (d["q_lora"], h))
            out.append(TensorSpec(p + "self_attn.q_a_layernorm.weight", "BF16", (d["q_lora"],)))
            out += self._q(p + "self_attn.q_b_proj", (d["heads"] * qk, d["q_lora"]))
            out += self._q(p + "self_attn.kv_a_proj_with_mqa", (d["kv_lora"] + d["qk_rope"], h))
            out.append(TensorSpec(p + "self_attn.kv_a_layernorm.weight", "BF16", (d["kv_lora"],)))
            out += self._q(p + "self_attn.kv_b_proj", (d["heads"] * (d["qk_nope"] + d["v_head"]), d["kv_lora"]))
            out += self._q(p + "self_attn.o_proj", (h, d["heads"] * d["v_head"]))
            out.append(TensorSpec(p + "post_attention_layernorm.weight", "BF16", (h,)))
            if i < d["dense_layers"]:
                f = d["dense_ffn"]
                out += self._q(p + "mlp.gate_proj", (f, h)) + self._q(p + "mlp.up_proj", (f, h))
                out += self._q(p + "mlp.down_proj", (h, f))
            else:
                f = d["moe_ffn"]
                out.append(TensorSpec(p + "mlp.gate.weight", "BF16", (d["routed_experts"], h)))
                out.append(TensorSpec(p + "mlp.gate.e_score_correction_bias", "F32", (d["routed_experts"],)))
                for e in range(d["routed_experts"]):
                    q = p + f"mlp.experts.{e}."
                    out += self._q(q + "gate_proj", (f, h)) + self._q(q + "up_proj", (f, h))
                    out += self._q(q + "down_proj", (h, f))
                q = p + "mlp.shared_experts."
                out += self._q(q + "gate_proj", (f, h)) + self._q(q + "up_proj", (f, h)) + self._q(q + "down_proj", (h, f))
        out += [TensorSpec("model.norm.weight", "BF16", (h,)), TensorSpec("lm_head.weight", "BF16", (d["vocab"], h))]
        return out

    def rank_view(self, tp_size=1, tp_rank=0, ep_size=1, ep_rank=0, param_dtype=None):
        d = self.dims
        h = d["hidden"]
        qk = d["qk_nope"] + d["qk_rope"]
        heads = _div(d["heads"], tp_size, "heads")
        v = _div(d["vocab"], tp_size, "vocab")
        local_exp = _div(d["routed_experts"], ep_size, "routed_experts")
        params = [ParamSpec("model.embed_tokens.weight", "BF16", (v, h))]
        for i in range(d["layers"]):
            p = f"model.layers.{i}."
            params.append(ParamSpec(p + "input_layernorm.weight", "BF16", (h,)))
            params += self._qp(p + "self_attn.q_a_proj", (d["q_lora"], h))  # replicated
            params.append(ParamSpec(p + "self_attn.q_a_layernorm.weight", "BF16", (d["q_lora"],)))
            params += self._qp(p + "self_attn.q_b_proj", (heads * qk, d["q_lora"]))  # column parallel
            params += self._qp(p + "self_attn.kv_a_proj_with_mqa", (d["kv_lora"] + d["qk_rope"], h))  # replicated
            params.append(ParamSpec(p + "self_attn.kv_a_layernorm.weight", "BF16", (d["kv_lora"],)))
            params += self._qp(p + "self_attn.kv_b_proj", (heads * (d["qk_nope"] + d["v_head"]), d["kv_lora"]))
            params += self._qp(p + "self_attn.o_proj", (h, heads * d["v_head"]))  # row parallel: K is sliced
            params.append(ParamSpec(p + "post_attention_layernorm.weight", "BF16", (h,)))
            if i < d["dense_layers"]:
                f = _div(d["dense_ffn"], tp_size, "dense_ffn")
                params += self._qp(p + "mlp.gate_up_proj", (2 * f, h)) + self._qp(p + "mlp.down_proj", (h, f))
            else:
                f = d["moe_ffn"]
                fs = _div(f, tp_size, "moe_ffn")
                # routed experts: expert parallel when ep_size > 1 (whole experts), else TP-split
                fe = f if ep_size > 1 else fs
                params.append(ParamSpec(p + "mlp.gate.weight", "BF16", (d["routed_experts"], h)))
                params.append(ParamSpec(p + "mlp.gate.e_score_correction_bias", "F32", (d["routed_experts"],)))
                params += [
                    ParamSpec(p + "mlp.experts.w13_weight", "F8_E4M3", (local_exp, 2 * fe, h)),
                    ParamSpec(p + "mlp.experts.w13_weight_scale_inv", "F32", (local_exp, 2 * self._blocks(fe), self._blocks(h))),
                    ParamSpec(p + "mlp.experts.w2_weight", "F8_E4M3", (local_exp, h, fe)),
                    ParamSpec(p + "mlp.experts.w2_weight_scale_inv", "F32", (local_exp, self._blocks(h), self._blocks(fe))),
                ]
                q = p + "mlp.shared_experts."
                params += self._qp(q + "gate_up_proj", (2 * fs, h)) + self._qp(q + "down_proj", (h, fs))
        params += [ParamSpec("model.norm.weight", "BF16", (h,)), ParamSpec("lm_head.weight", "BF16", (v, h))]
        mapping = [("gate_up_proj", "gate_proj"), ("gate_up_proj", "up_proj")]
        experts = []
        lo = ep_rank * local_exp
        for e in range(d["routed_experts"]):
            local = e - lo if lo <= e < lo + local_exp else -1
            experts += [("experts.w13_", f"experts.{e}.gate_proj.", e, "w1", local),
                        ("experts.w2_", f"experts.{e}.down_proj.", e, "w2", local),
                        ("experts.w13_", f"experts.{e}.up_proj.", e, "w3", local)]
        return RankView(params, mapping, experts)


def baseline_config(index: int) -> tuple:
    """The five benchmark configurations: ``(layout, tp_size, ep_size, n_shards, ckpt_dtype, kind)``."""
    if index == 1:
        return Gpt2(), 1, 1, 1, "F16", None
    if index == 2:
        return Llama(), 8, 1, 4, "BF16", None
    if index == 3:
        return Llama(), 8, 1, 8, "F32", NORMAL_EDGE
    if index == 4:
        return Mixtral(), 1, 1, 19, "BF16", None
    if index == 5:
        return DeepSeekV3(), 8, 8, 163, None, None
    raise ValueError("config index must be 1..5")
