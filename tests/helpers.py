"""Shared test helpers: run the CPU oracle over a checkpoint, interpret a product plan
with numpy, build tiny layouts of the benchmark families."""

from __future__ import annotations

import numpy as np

from modelexpress_amd import models
from modelexpress_amd.engine import Checkpoint, PlacementPlan


def oracle_place(oracle, ckpt_dir: str | None, rv, *, tp_size=1, tp_rank=0, allow_cast=False, nan_bits=0x7FC0,
                 strict_params=True, weights=None, only_params=None):
    """The oracle's parameter buffers for one rank: ``{name: OTensor}``.  ``weights`` (a list of
    ``(name, OTensor)``) stands in for the checkpoint directory; ``only_params`` restricts the rank's
    parameter table to those names (the weights given must then be the ones that write into them)."""
    if weights is None:
        weights = oracle.load_checkpoint(ckpt_dir)
    wanted = [p for p in rv.params if only_params is None or p.name in only_params]
    params = {p.name: oracle.OTensor.zeros(p.shape, p.dtype) for p in wanted}
    skip = tuple(rv.skip_prefixes)
    weights = [(n, t) for n, t in weights if not n.startswith(skip)] if skip else weights
    local_of = {}
    mapping = None
    if rv.expert_mapping:
        mapping = [row[:4] for row in rv.expert_mapping]
        for row in rv.expert_mapping:
            local_of[int(row[2])] = int(row[4]) if len(row) > 4 else int(row[2])

    def expert_local(_fused_name, gid):
        loc = local_of.get(gid, gid)
        return None if loc == -2 else loc

    m = oracle.MdlOracle(params, tp_size, tp_rank, rv.stacked_params_mapping, mapping,
                         expert_local if mapping else None, allow_cast=allow_cast, nan_bits=nan_bits)
    m.load_weights(weights, strict_params=strict_params)
    return params


def make_plan(ckpt_dir: str, rv, *, tp_size=1, tp_rank=0, **kw):
    ck = Checkpoint(ckpt_dir)
    plan = PlacementPlan(ck, rv.params, tp_size=tp_size, tp_rank=tp_rank,
                         stacked_params_mapping=rv.stacked_params_mapping, expert_mapping=rv.expert_mapping,
                         skip_prefixes=rv.skip_prefixes, **kw)
    return ck, plan


def apply_plan_numpy(ck: Checkpoint, plan: PlacementPlan, nan_bits=0x7FC0) -> dict:
    """Interpret the product plan's pitched boxes on the host (checks the planner alone)."""
    files = [np.fromfile(f["path"], dtype=np.uint8) for f in ck.files()]
    tensors = {t.name: t for t in ck.tensors()}
    out = {p.name: np.zeros(p.nbytes, dtype=np.uint8) for p in plan.params}
    for w in plan.writes():
        t = tensors[w.tensor]
        src = files[t.file_index][t.file_offset : t.file_offset + t.nbytes]
        dst = out[w.param]
        src_row = {0: w.row_bytes, 1: w.row_bytes * 2, 4: w.row_bytes * 2, 2: w.row_bytes // 2, 3: w.row_bytes // 2,
                   5: w.row_bytes // 2, 6: w.row_bytes, 7: w.row_bytes}[w.cast]
        for r in range(w.rows):
            s = src[w.src_offset + r * w.src_pitch : w.src_offset + r * w.src_pitch + src_row]
            if w.cast == 1:
                u = s.view("<u4").astype(np.uint64)
                b = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
                b[(u & 0x7FFFFFFF) > 0x7F800000] = nan_bits
                s = b.view(np.uint8)
            elif w.cast == 2:
                s = (s.view("<u2").astype(np.uint32) << 16).view(np.uint8)
            elif w.cast in (3, 4, 5, 6, 7):  # torch is the library the reference converts with
                import torch
                src_t, dst_t = {3: (torch.float16, torch.float32), 4: (torch.float32, torch.float16),
                                5: (torch.float8_e4m3fn, torch.bfloat16), 6: (torch.float16, torch.bfloat16),
                                7: (torch.bfloat16, torch.float16)}[w.cast]
                s = torch.from_numpy(s.copy()).view(src_t).to(dst_t).view(torch.uint8).numpy()
            dst[w.dst_offset + r * w.dst_pitch : w.dst_offset + r * w.dst_pitch + w.row_bytes] = s
    return out


def cast_setup(ck_kw: dict):
    """Splits a ``tiny_layouts`` kwargs dict: ``(checkpoint kwargs, param dtype or None, cast?, source bytes per
    destination byte)``.  An F32 checkpoint without an explicit ``param_dtype`` is the refit into BF16."""
    kw = dict(ck_kw)
    param_dtype = kw.pop("param_dtype", None)
    if param_dtype is None and kw.get("dtype") == "F32":
        param_dtype = "BF16"
    size = {"F32": 4, "BF16": 2, "F16": 2}
    ratio = size[kw.get("dtype") or "BF16"] / size[param_dtype] if param_dtype else 1
    return kw, param_dtype, param_dtype is not None, ratio


def tiny_layouts():
    """Small instances of the five benchmark families: ``name -> (layout, tp, ep, shards, ckpt kwargs)``;
    a ``param_dtype`` among the kwargs asks for a converting placement (see ``cast_setup``)."""
    return {
        "llama_bf16_into_f32": (models.Llama(layers=2, hidden=64, ffn=96, q_heads=8, kv_heads=4, head_dim=8, vocab=256),
                                4, 1, 2, {"dtype": "BF16", "edge_cases": models.NORMAL_EDGE_DENSE, "param_dtype": "F32"}),
        "llama_f16_into_f32": (models.Llama(layers=1, hidden=64, ffn=96, q_heads=8, kv_heads=4, head_dim=8, vocab=256),
                               2, 1, 1, {"dtype": "F16", "edge_cases": models.NORMAL_EDGE_DENSE, "param_dtype": "F32"}),
        "llama_f16_into_bf16": (models.Llama(layers=1, hidden=64, ffn=96, q_heads=8, kv_heads=4, head_dim=8, vocab=256),
                                2, 1, 2, {"dtype": "F16", "param_dtype": "BF16"}),
        "llama_f32_into_f16": (models.Llama(layers=1, hidden=64, ffn=96, q_heads=8, kv_heads=4, head_dim=8, vocab=256),
                               2, 1, 2, {"dtype": "F32", "edge_cases": models.NORMAL_EDGE_DENSE, "param_dtype": "F16"}),
        "gpt2": (models.Gpt2(layers=2, hidden=32, ffn=64, vocab=97, positions=16), 1, 1, 1, {}),
        "llama_tp4": (models.Llama(layers=2, hidden=64, ffn=96, q_heads=8, kv_heads=4, head_dim=8, vocab=256), 4, 1, 3, {}),
        "llama_f32_refit": (models.Llama(layers=2, hidden=64, ffn=96, q_heads=8, kv_heads=4, head_dim=8, vocab=256),
                            4, 1, 2, {"dtype": "F32", "edge_cases": models.NORMAL_EDGE_DENSE}),
        "mixtral": (models.Mixtral(layers=2, hidden=32, ffn=48, q_heads=4, kv_heads=2, head_dim=8, vocab=64, experts=4),
                    1, 1, 3, {}),
        "mixtral_tp2": (models.Mixtral(layers=1, hidden=32, ffn=48, q_heads=4, kv_heads=2, head_dim=8, vocab=64, experts=4),
                        2, 1, 2, {}),
        "deepseek_ep": (models.DeepSeekV3(layers=3, dense_layers=1, hidden=512, q_lora=256, kv_lora=128, heads=4,
                                          qk_nope=128, qk_rope=64, v_head=128, routed_experts=8, moe_ffn=512,
                                          dense_ffn=1024, vocab=512), 2, 2, 4, {}),
    }
