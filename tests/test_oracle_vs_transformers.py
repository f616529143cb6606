"""The oracle's layer forward against third-party code that implements the same blocks: the stock
`transformers` sparse MoE blocks, run by transformers itself in fp32 on the CPU.

This pins what no closed form pins: the routing conventions (softmax over all experts then top-k, with and
without renormalisation; Mixtral's renormalised top-k), the per-expert SwiGLU on the dispatched tokens, the
weighted combine and the sigmoid-gated shared expert, as ONE block against an independent implementation.
A dropped renormalisation, a transposed expert matrix, gate and up swapped or a shared expert added before
the scaling each fail it.  (transformers is not the reference: the reference hooks such a module and holds
no arithmetic of its own.)"""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O

transformers = pytest.importorskip("transformers")


def _experts_of(block):
    gu = block.experts.gate_up_proj.detach().float().numpy()      # [E, 2I, H]: gate rows, then up rows
    dn = block.experts.down_proj.detach().float().numpy()         # [E, H, I]
    I = gu.shape[1] // 2
    return [(gu[e, :I], gu[e, I:], dn[e]) for e in range(gu.shape[0])]


def _block_output(block, x):
    with torch.no_grad():
        y = block(torch.from_numpy(x).reshape(1, *x.shape))
    y = y[0] if isinstance(y, tuple) else y
    return y.reshape(x.shape).float().numpy()


@pytest.mark.parametrize("norm", [False, True])
def test_qwen2_moe_block(norm):
    from transformers import Qwen2MoeConfig
    from transformers.models.qwen2_moe.modeling_qwen2_moe import Qwen2MoeSparseMoeBlock
    H, I, I_sh, E, k, T = 64, 32, 48, 8, 3, 11
    cfg = Qwen2MoeConfig(hidden_size=H, moe_intermediate_size=I, shared_expert_intermediate_size=I_sh, num_experts=E,
                         num_experts_per_tok=k, norm_topk_prob=norm)
    torch.manual_seed(3 + int(norm))
    blk = Qwen2MoeSparseMoeBlock(cfg).float().eval()
    with torch.no_grad():
        for p in blk.parameters():
            p.copy_(torch.randn_like(p) * 0.2)
    x = np.random.default_rng(4).standard_normal((T, H)).astype(np.float32)
    want = _block_output(blk, x)
    sh = blk.shared_expert
    got = O.moe_forward(x, blk.gate.weight.detach().numpy(), _experts_of(blk), k,
                        O.MODE_SOFTMAX_TOPK_RENORM if norm else O.MODE_SOFTMAX_TOPK,
                        shared=(sh.gate_proj.weight.detach().numpy(), sh.up_proj.weight.detach().numpy(),
                                sh.down_proj.weight.detach().numpy()),
                        shared_gate=blk.shared_expert_gate.weight.detach().numpy().reshape(-1))
    assert np.abs(got["out"] - want).max() <= 2e-5 * np.abs(want).max()
    # and the routing itself, against torch's own softmax / topk
    p = torch.softmax(torch.from_numpy(x) @ blk.gate.weight.detach().T, dim=-1)
    tw, ti = torch.topk(p, k, dim=-1)
    if norm:
        tw = tw / tw.sum(-1, keepdim=True)
    assert np.array_equal(got["idx"], ti.numpy().astype(np.int32))
    assert np.allclose(got["w"], tw.numpy(), rtol=1e-5, atol=1e-7)


def test_mixtral_block():
    from transformers import MixtralConfig
    from transformers.models.mixtral.modeling_mixtral import MixtralSparseMoeBlock
    H, I, E, k, T = 64, 96, 4, 2, 9
    cfg = MixtralConfig(hidden_size=H, intermediate_size=I, num_local_experts=E, num_experts_per_tok=k)
    torch.manual_seed(5)
    blk = MixtralSparseMoeBlock(cfg).float().eval()
    with torch.no_grad():
        for p in blk.parameters():
            p.copy_(torch.randn_like(p) * 0.2)
    x = np.random.default_rng(6).standard_normal((T, H)).astype(np.float32)
    want = _block_output(blk, x)
    got = O.moe_forward(x, blk.gate.weight.detach().numpy(), _experts_of(blk), k, O.MODE_TOPK_SOFTMAX)
    assert np.abs(got["out"] - want).max() <= 2e-5 * np.abs(want).max()


def test_deepseek_v2_block():
    """DeepSeek-MoE's convention (the bench shape's): softmax over all experts, greedy top-k, no
    renormalisation, two always-on shared experts fused into one MLP that is added unscaled."""
    from transformers import DeepseekV2Config
    from transformers.models.deepseek_v2.modeling_deepseek_v2 import DeepseekV2Moe
    H, I, E, k, T, n_sh = 64, 32, 8, 3, 10, 2
    cfg = DeepseekV2Config(hidden_size=H, moe_intermediate_size=I, n_routed_experts=E, num_experts_per_tok=k,
                           n_shared_experts=n_sh, topk_method="greedy", routed_scaling_factor=1.0, n_group=1, topk_group=1)
    torch.manual_seed(7)
    blk = DeepseekV2Moe(cfg).float().eval()
    with torch.no_grad():
        for p in blk.parameters():
            p.copy_(torch.randn_like(p) * 0.2)
    x = np.random.default_rng(8).standard_normal((T, H)).astype(np.float32)
    want = _block_output(blk, x)
    sh = blk.shared_experts
    got = O.moe_forward(x, blk.gate.weight.detach().numpy(), _experts_of(blk), k, O.MODE_SOFTMAX_TOPK,
                        shared=(sh.gate_proj.weight.detach().numpy(), sh.up_proj.weight.detach().numpy(),
                                sh.down_proj.weight.detach().numpy()))
    assert np.abs(got["out"] - want).max() <= 2e-5 * np.abs(want).max()
