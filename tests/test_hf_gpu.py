"""A stock transformers MoE model with its sparse blocks routed through the engine, against the same
model run by transformers itself (bf16 on the GPU): prefill and cached single-token decode steps."""
import copy

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cuda():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return torch.device("cuda:0")


def _rel(a, b):
    return float((a.float() - b.float()).abs().max() / b.float().abs().max())


def _compare(model, dev, fmt, tol, **cfg):
    from promoe_amd import hf
    torch.manual_seed(0)
    ref = copy.deepcopy(model).to(device=dev, dtype=torch.bfloat16).eval()
    n_blocks = len(hf.find_moe_blocks(model))
    pm = hf.inject_model(model, device=dev, fmt=fmt, max_tokens=64, **cfg)
    model.eval()
    try:
        assert len(hf.find_moe_blocks(ref)) == n_blocks > 0
        # the experts left the module: what stays on the device is the dense part only
        assert sum(p.numel() for p in model.parameters()) < sum(p.numel() for p in ref.parameters())
        ids = torch.randint(0, model.config.vocab_size, (1, 12), device=dev)
        with torch.no_grad():
            a = ref(ids, use_cache=True)
            b = model(ids, use_cache=True)
            errs = [_rel(b.logits, a.logits)]
            pa, pb = a.past_key_values, b.past_key_values
            tok = a.logits[:, -1:].argmax(-1)
            for _ in range(4):                       # cached decode: one token through every sparse block
                a = ref(tok, past_key_values=pa, use_cache=True)
                b = model(tok, past_key_values=pb, use_cache=True)
                errs.append(_rel(b.logits, a.logits))
                pa, pb = a.past_key_values, b.past_key_values
                tok = a.logits[:, -1:].argmax(-1)
        torch.cuda.synchronize()
        print("  logits max-rel-err per forward:", ["%.3e" % e for e in errs], flush=True)
        assert max(errs) <= tol
        c = pm.counters()
        assert c["hit"] + c["miss"] > 0
        return c
    finally:
        pm.close()


def test_qwen2_moe_model_through_the_engine(cuda):
    print("case hf_qwen2_moe", flush=True)
    from transformers import Qwen2MoeConfig, Qwen2MoeForCausalLM
    cfg = Qwen2MoeConfig(vocab_size=128, hidden_size=256, intermediate_size=512, num_hidden_layers=3,
                         num_attention_heads=4, num_key_value_heads=2, moe_intermediate_size=128,
                         shared_expert_intermediate_size=256, num_experts=8, num_experts_per_tok=2,
                         decoder_sparse_step=1, mlp_only_layers=[], norm_topk_prob=False, max_position_embeddings=128)
    torch.manual_seed(1)
    model = Qwen2MoeForCausalLM(cfg)
    c = _compare(model, cuda, "bf16", 3e-2, cache_rate=0.5, cache_policy="lru")
    assert c["miss"] > 0


def test_mixtral_model_through_the_engine_int4(cuda):
    print("case hf_mixtral_int4", flush=True)
    from transformers import MixtralConfig, MixtralForCausalLM
    cfg = MixtralConfig(vocab_size=128, hidden_size=256, intermediate_size=256, num_hidden_layers=2,
                        num_attention_heads=4, num_key_value_heads=2, num_local_experts=4, num_experts_per_tok=2,
                        max_position_embeddings=128)
    torch.manual_seed(2)
    model = MixtralForCausalLM(cfg)
    # int4: the comparison model runs on the dequantised weights the engine holds
    from promoe_amd import hf, quant
    from oracle import moe_oracle as O
    for _, blk in hf.find_moe_blocks(model):
        with torch.no_grad():
            for t in (blk.experts.gate_up_proj, blk.experts.down_proj):
                for e in range(t.shape[0]):
                    w = t[e]
                    if t is blk.experts.gate_up_proj:      # gate and up are quantised as separate matrices
                        half = w.shape[0] // 2
                        for sl in (slice(0, half), slice(half, None)):
                            q = quant.quantize_int4(w[sl].float())
                            w[sl] = torch.from_numpy(O.dequant_int4(q[0], q[1], q[2], w[sl].shape[0], w.shape[1]))
                    else:
                        q = quant.quantize_int4(w.float())
                        w.copy_(torch.from_numpy(O.dequant_int4(q[0], q[1], q[2], w.shape[0], w.shape[1])))
    _compare(model, cuda, "int4", 3e-2, cache_rate=1.0)


@pytest.mark.parametrize("scaling", [1.0, 2.5])
def test_deepseek_model_through_the_engine(cuda, scaling):
    """DeepSeek family (stock transformers DeepseekV2): a dense first layer, then sparse blocks with greedy
    softmax top-k routing and a plain shared expert of two experts' width; half of the experts resident.
    scaling: routed_scaling_factor (it goes into the routed experts' down projections; 2.5 is no power of two)."""
    print(f"case hf_deepseek scaling={scaling}", flush=True)
    from transformers import DeepseekV2Config, DeepseekV2ForCausalLM
    from promoe_amd import hf
    cfg = DeepseekV2Config(vocab_size=128, hidden_size=256, intermediate_size=512, moe_intermediate_size=128,
                           num_hidden_layers=3, num_attention_heads=4, num_key_value_heads=4, n_shared_experts=2,
                           n_routed_experts=8, num_experts_per_tok=2, first_k_dense_replace=1, kv_lora_rank=32,
                           q_lora_rank=None, qk_rope_head_dim=16, qk_nope_head_dim=32, v_head_dim=32, head_dim=16,
                           topk_method="greedy", routed_scaling_factor=scaling, max_position_embeddings=128)
    torch.manual_seed(3)
    model = DeepseekV2ForCausalLM(cfg)
    names = [n for n, _ in hf.find_moe_blocks(model)]
    assert names == ["model.layers.1.mlp", "model.layers.2.mlp"]      # decoder layer i = engine layer i - 1
    c = _compare(model, cuda, "bf16", 3e-2, cache_rate=0.5, cache_policy="lru")
    assert c["miss"] > 0
    assert [blk._layer_id for _, blk in hf.find_moe_blocks(model)] == [0, 1]
