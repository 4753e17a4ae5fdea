"""Refresh of the MLA absorbed weights after ``kv_b_proj`` has been refitted.

``W_UV`` and ``W_UK_T`` are values derived from ``kv_b_proj`` and cached as bare module
attributes; serving graphs hold their addresses, so they are rewritten in place
(modelexpress_rl/inference/engines/vllm/installer.py:251-285;
modelexpress/engines/vllm/refit/receiver.py:229-261).  The reference computes

    kv_b = kv_b_proj.weight.view(num_heads, qk_nope_head_dim + v_head_dim, -1)
    w_uk, w_uv = kv_b.split([qk_nope_head_dim, v_head_dim], dim=1)
    W_UV.copy_(w_uv.transpose(0, 1).to(out_dtype))
    W_UK_T.copy_(w_uk.permute(1, 2, 0).to(out_dtype))

Here both are strided views of ``kv_b_proj.weight`` handed to the engine: ``W_UV`` keeps the
innermost dimension (a row gather), ``W_UK_T`` is a true transpose (the LDS transpose kernel),
each converting to the attribute's dtype on the way, with no intermediate tensor; all layers
of the model go out in one call.
"""

from __future__ import annotations

from typing import Any

from .engine import CAST_CODES, PlacementEngine
from .load_strategy import safetensors_dtype_of


class IncompleteRefit(RuntimeError):
    """The refit ran and still left part of the model unwritten (refit/reshard/types.py:27-35)."""


def update_mla_absorbed_weights(engine: PlacementEngine, model: Any, *, quantized: bool, stream: int = 0) -> int:
    """Recomputes ``W_UV`` / ``W_UK_T`` of every MLA module of ``model`` in place; returns how many
    tensors were rewritten.  A no-op for models without MLA.  ``quantized``: the live ``kv_b_proj`` is
    stored quantized - its values are not the weights, so the refresh is refused as the reference does."""
    views = []
    for _name, module in model.named_modules():
        if not (hasattr(module, "W_UV") or hasattr(module, "W_UK_T")) or not hasattr(module, "kv_b_proj"):
            continue
        if quantized:
            raise IncompleteRefit("MLA derived-weight refresh from a quantized kv_b_proj is unsupported")
        w = module.kv_b_proj.weight
        heads, nope, v_dim = int(module.num_heads), int(module.qk_nope_head_dim), int(module.v_head_dim)
        if w.dim() != 2 or not w.is_contiguous() or w.shape[0] != heads * (nope + v_dim):
            raise IncompleteRefit(f"kv_b_proj.weight of shape {tuple(w.shape)} does not hold {heads} heads of {nope} + {v_dim} rows")
        latent = int(w.shape[1])
        head_stride = (nope + v_dim) * latent
        src_dtype = safetensors_dtype_of(w)
        # (attribute, view shape, source strides of that view in elements, first source element)
        for attr, shape, strides, first in (("W_UV", (v_dim, heads, latent), (latent, head_stride, 1), nope * latent),
                                            ("W_UK_T", (nope, latent, heads), (latent, 1, head_stride), 0)):
            out = getattr(module, attr, None)
            if out is None:
                continue
            if tuple(out.shape) != shape:
                raise IncompleteRefit(f"{attr} has shape {tuple(out.shape)}, the view of kv_b_proj is {shape}")
            dst_dtype = safetensors_dtype_of(out)
            cast = 0
            if dst_dtype != src_dtype:
                cast = CAST_CODES.get((src_dtype, dst_dtype), 0)
                if not cast:
                    raise IncompleteRefit(f"{attr}: no conversion from {src_dtype} to {dst_dtype}")
            views.append({"src": w.data_ptr() + first * w.element_size(), "dst": out.data_ptr(), "shape": shape,
                          "elem_size": out.element_size(), "src_strides": strides,
                          "dst_strides": tuple(int(s) for s in out.stride()), "cast": cast})
    if views:
        engine.copy_views(views, stream=stream)
    return len(views)
