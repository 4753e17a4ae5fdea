"""``update_mla_absorbed_weights``: the reference's refresh of ``W_UV`` / ``W_UK_T`` after a refit
(modelexpress_rl/inference/engines/vllm/installer.py:251-285; tests/test_refit_vllm_installer.py:101-109),
against the same torch expressions evaluated on the CPU."""

import pytest
import torch
from torch import nn

from modelexpress_amd.mla import IncompleteRefit, update_mla_absorbed_weights


def _mla_module(heads, nope, v_dim, latent, w_dtype, out_dtype, device, seed):
    g = torch.Generator().manual_seed(seed)
    m = nn.Module()
    m.kv_b_proj = nn.Linear(latent, heads * (nope + v_dim), bias=False)
    m.kv_b_proj.weight = nn.Parameter((torch.randn(heads * (nope + v_dim), latent, generator=g) * 2).to(w_dtype).to(device),
                                      requires_grad=False)
    m.num_heads, m.qk_nope_head_dim, m.v_head_dim = heads, nope, v_dim
    m.W_UV = torch.full((v_dim, heads, latent), 7, dtype=out_dtype, device=device)
    m.W_UK_T = torch.full((nope, latent, heads), 7, dtype=out_dtype, device=device)
    return m


def test_quantized_kv_b_proj_is_refused_and_plain_models_are_a_no_op():
    # tests/test_refit_vllm_installer.py:101-109: refused before anything is touched (no engine needed)
    model = nn.Module()
    mla = nn.Module()
    mla.kv_b_proj = nn.Linear(1, 1, bias=False)
    mla.W_UV = torch.zeros(1)
    model.add_module("mla", mla)
    with pytest.raises(IncompleteRefit, match="quantized kv_b_proj"):
        update_mla_absorbed_weights(None, model, quantized=True)
    assert update_mla_absorbed_weights(None, nn.Linear(2, 2), quantized=True) == 0  # no MLA module: nothing to refuse


@pytest.mark.gpu
@pytest.mark.parametrize("w_dtype,out_dtype", [(torch.bfloat16, torch.bfloat16), (torch.float32, torch.bfloat16),
                                               (torch.bfloat16, torch.float32), (torch.float16, torch.float16)])
def test_refresh_matches_the_reference_expressions(gpu_engine, w_dtype, out_dtype):
    model = nn.Module()
    shapes = [(16, 128, 128, 512), (4, 64, 32, 96), (3, 20, 12, 40)]  # DeepSeek-like head geometry, then ragged ones
    for k, (heads, nope, v_dim, latent) in enumerate(shapes):
        model.add_module(f"layer{k}", _mla_module(heads, nope, v_dim, latent, w_dtype, out_dtype, "cuda", 50 + k))
    model.add_module("mlp", nn.Linear(4, 4))
    addresses = [(m.W_UV.data_ptr(), m.W_UK_T.data_ptr()) for m in model.children() if hasattr(m, "W_UV")]
    assert update_mla_absorbed_weights(gpu_engine, model, quantized=False) == 2 * len(shapes)
    torch.cuda.synchronize()
    for m, (a_uv, a_ukt) in zip([m for m in model.children() if hasattr(m, "W_UV")], addresses):
        w = m.kv_b_proj.weight.cpu().view(m.num_heads, m.qk_nope_head_dim + m.v_head_dim, -1)
        w_uk, w_uv = w.split([m.qk_nope_head_dim, m.v_head_dim], dim=1)
        want_uv = w_uv.transpose(0, 1).to(out_dtype).contiguous()
        want_ukt = w_uk.permute(1, 2, 0).to(out_dtype).contiguous()
        assert torch.equal(m.W_UV.cpu().view(torch.uint8), want_uv.view(torch.uint8))
        assert torch.equal(m.W_UK_T.cpu().view(torch.uint8), want_ukt.view(torch.uint8))
        assert (m.W_UV.data_ptr(), m.W_UK_T.data_ptr()) == (a_uv, a_ukt)  # rewritten in place: graph-bound addresses kept


@pytest.mark.gpu
def test_refresh_only_the_attributes_a_module_has(gpu_engine):
    m = _mla_module(4, 8, 8, 16, torch.bfloat16, torch.bfloat16, "cuda", 9)
    del m.W_UV
    model = nn.Module()
    model.add_module("attn", m)
    assert update_mla_absorbed_weights(gpu_engine, model, quantized=False) == 1
    w = m.kv_b_proj.weight.cpu().view(4, 16, -1)
    assert torch.equal(m.W_UK_T.cpu(), w[:, :8].permute(1, 2, 0).contiguous())
