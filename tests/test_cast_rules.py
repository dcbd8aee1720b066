"""Which tensors of an HF-named checkpoint the BF16 -> FP8 converter quantises: the modules the reference builds
with ``Linear.dtype`` (inference/model.py:183, 760; HF names per inference/convert.py:11-30), and nothing else."""
import torch

from dsv3fp8.bf16_cast_fp8 import FP8_MODULES, is_fp8_weight


def test_fp8_layers_are_the_linear_projections():
    w = torch.empty(256, 128, dtype=torch.bfloat16)
    yes = ["model.layers.0.self_attn.q_a_proj.weight", "model.layers.0.self_attn.q_b_proj.weight",
           "model.layers.0.self_attn.q_proj.weight", "model.layers.0.self_attn.kv_a_proj_with_mqa.weight",
           "model.layers.0.self_attn.kv_b_proj.weight", "model.layers.0.self_attn.o_proj.weight",
           "model.layers.0.mlp.gate_proj.weight", "model.layers.0.mlp.up_proj.weight",
           "model.layers.0.mlp.down_proj.weight", "model.layers.7.mlp.experts.255.gate_proj.weight",
           "model.layers.7.mlp.shared_experts.down_proj.weight"]
    no = ["model.embed_tokens.weight", "lm_head.weight", "model.norm.weight",
          "model.layers.0.input_layernorm.weight", "model.layers.0.self_attn.q_a_layernorm.weight",
          "model.layers.7.mlp.gate.weight", "model.layers.7.mlp.gate.e_score_correction_bias",
          "model.layers.0.self_attn.q_a_proj.weight_scale_inv", "model.layers.0.self_attn.o_proj.bias"]
    assert all(is_fp8_weight(n, w) for n in yes)
    assert not any(is_fp8_weight(n, w) for n in no)
    # already-quantised (1-byte) and 1-D tensors are left alone whatever their name
    assert not is_fp8_weight(yes[0], torch.empty(256, 128, dtype=torch.float8_e4m3fn))
    assert not is_fp8_weight(yes[0], torch.empty(256, dtype=torch.bfloat16))
    assert len(FP8_MODULES) == 9
