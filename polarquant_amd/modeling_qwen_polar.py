"""Qwen2 polar-key attention and model shell under the reference's class names
(models/modeling_qwen_polar.py).  Unlike the reference, which expands the whole
code cache to all query heads on every step because its kernel needs a
power-of-two GQA ratio (modeling_qwen_polar.py:65-74), the HIP kernels take
Qwen's ratios (7, 6, 5) natively."""
from .kernel4group import attention_decode_forward_triton_impl  # noqa: F401
from .modeling_common import (  # noqa: F401
    CausalLMOutputWithPast, GenerationConfig, PolarCache, PolarConfig, PolarDecoderLayer, PolarForCausalLM,
    PolarGroupAttention, PolarModel, apply_rotary_pos_emb, generate, repeat_kv, repeat_kv_quant, return_top_p_filtered_indices, sample,
    top_k_top_p_filtering)


class Qwen2PolarGroupAttention(PolarGroupAttention):
    """Qwen2 carries a bias on the q/k/v projections (none on o_proj)."""

    def __init__(self, config, layer_idx=None):
        if not getattr(config, "attention_bias", False):
            import copy
            config = copy.copy(config)
            config.attention_bias = True
        super().__init__(config, layer_idx)


class Qwen2PolarDecoderLayer(PolarDecoderLayer):
    attention_class = Qwen2PolarGroupAttention


class Qwen2PolarModel(PolarModel):
    layer_class = Qwen2PolarDecoderLayer


class Qwen2PolarForCausalLM(PolarForCausalLM):
    model_class = Qwen2PolarModel
