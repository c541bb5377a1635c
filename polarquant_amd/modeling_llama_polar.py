"""Llama polar-key attention and model shell under the reference's class names
(models/modeling_llama_polar.py): LlamaPolarGroupAttention, LlamaPolarMixedGroupAttention, LlamaSnapKVAttention, LlamaPolarDecoderLayer,
LlamaPolarModel, LlamaPolarForCausalLM, generate, sample, top_k_top_p_filtering."""
from .kernel4group import attention_decode_forward_triton_impl  # noqa: F401  (re-exported, as the reference imports it here)
from .modeling_common import (  # noqa: F401
    CausalLMOutputWithPast, GenerationConfig, PolarCache, PolarConfig, PolarDecoderLayer, PolarForCausalLM,
    PolarGroupAttention, PolarMixedGroupAttention, PolarModel, PolarSnapKVAttention, apply_rotary_pos_emb, generate, repeat_kv, repeat_kv_quant, return_top_p_filtered_indices, sample,
    top_k_top_p_filtering)


class LlamaPolarGroupAttention(PolarGroupAttention):
    """q/k/v projections without bias unless config.attention_bias says otherwise (Llama)."""


class LlamaPolarMixedGroupAttention(PolarMixedGroupAttention):
    """Polar keys + 4-bit values (reference: models/modeling_llama_polar.py:160-292)."""


class LlamaSnapKVAttention(PolarSnapKVAttention):
    """SnapKV prompt eviction + polar cache (reference: models/modeling_llama_polar.py:295-443)."""


class LlamaPolarDecoderLayer(PolarDecoderLayer):
    attention_class = LlamaPolarGroupAttention
    mixed_attention_class = LlamaPolarMixedGroupAttention
    snapkv_attention_class = LlamaSnapKVAttention


class LlamaPolarModel(PolarModel):
    layer_class = LlamaPolarDecoderLayer


class LlamaPolarForCausalLM(PolarForCausalLM):
    model_class = LlamaPolarModel
