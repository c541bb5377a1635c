"""Checkpoint directories (polarquant_amd/checkpoint.py): config mapping, sharded safetensors round trip, and the
errors a wrong checkpoint must raise.  Host only: the models are built on the CPU and never run."""
import json
import os

import pytest
import torch

from polarquant_amd import checkpoint as ck
from polarquant_amd.modeling_common import GenerationConfig, PolarConfig
from polarquant_amd.modeling_llama_polar import LlamaPolarForCausalLM
from polarquant_amd.modeling_qwen_polar import Qwen2PolarForCausalLM


def _toy(cls=LlamaPolarForCausalLM, **kw):
    torch.manual_seed(5)
    cfg = PolarConfig(hidden_size=256, num_attention_heads=2, num_key_value_heads=1, num_hidden_layers=2,
                      intermediate_size=128, vocab_size=96, eos_token_id=[7, 9], **kw)
    return cls(cfg)


@pytest.mark.parametrize("shards", [1, 3])
def test_round_trip(tmp_path, shards):
    src = _toy()
    ck.save_pretrained(src, str(tmp_path), shards=shards, generation=GenerationConfig(eos_token_id=[7, 9], top_k=20, top_p=0.9, temperature=0.7))
    if shards > 1:
        assert os.path.exists(tmp_path / "model.safetensors.index.json")
    got = ck.load_pretrained(str(tmp_path), torch.float32, "cpu", rbits=3, tbits=3)
    assert isinstance(got, LlamaPolarForCausalLM) and not got.training
    assert got.config.rbits == 3 and got.config.eos_token_id == [7, 9] and got.config.num_key_value_heads == 1
    want = dict(src.named_parameters())
    for name, p in got.named_parameters():
        assert torch.equal(p, want[name]), name
    gen = ck.load_generation_config(str(tmp_path))
    assert (gen.eos_token_id, gen.top_k, gen.top_p, gen.temperature) == ([7, 9], 20, 0.9, 0.7)
    # the class method the reference's scripts use
    again = LlamaPolarForCausalLM.from_pretrained(str(tmp_path), torch_dtype=torch.bfloat16, device="cpu")
    assert again.lm_head.weight.dtype == torch.bfloat16
    assert torch.equal(again.lm_head.weight, src.lm_head.weight.to(torch.bfloat16))


def test_qwen2_checkpoints_get_biases_and_their_class(tmp_path):
    src = _toy(Qwen2PolarForCausalLM, attention_bias=True)
    ck.save_pretrained(src, str(tmp_path), model_type="qwen2")
    with open(tmp_path / "config.json") as f:
        hf = json.load(f)
    hf.pop("attention_bias")                                  # Qwen2's config.json has no such field
    with open(tmp_path / "config.json", "w") as f:
        json.dump(hf, f)
    got = ck.load_pretrained(str(tmp_path), torch.float32, "cpu")
    assert isinstance(got, Qwen2PolarForCausalLM)
    assert torch.equal(got.model.layers[1].self_attn.k_proj.bias, src.model.layers[1].self_attn.k_proj.bias)


def test_tied_embeddings(tmp_path):
    src = _toy(tie_word_embeddings=True)
    ck.save_pretrained(src, str(tmp_path))
    from safetensors import safe_open
    with safe_open(str(tmp_path / "model.safetensors"), framework="pt") as f:
        assert "lm_head.weight" not in f.keys()
    got = ck.load_pretrained(str(tmp_path), torch.float32, "cpu")
    assert got.lm_head.weight is got.model.embed_tokens.weight
    assert torch.equal(got.lm_head.weight, src.model.embed_tokens.weight)


def test_config_mapping_and_refusals():
    hf = dict(model_type="llama", hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, num_hidden_layers=32,
              intermediate_size=14336, vocab_size=128256, rms_norm_eps=1e-5, rope_theta=5e5, eos_token_id=128009,
              rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                original_max_position_embeddings=8192))
    c = ck.config_from_hf(hf, vbits=4)
    assert c.head_dim == 128 and c.eos_token_id == [128009] and c.vbits == 4 and c.rope_scaling["factor"] == 8.0
    with pytest.raises(ValueError):
        ck.config_from_hf(dict(hf, hidden_size=2048))          # head_dim 64
    with pytest.raises(ValueError):
        ck.config_from_hf(dict(hf, model_type="gpt2"))
    with pytest.raises(TypeError):
        ck.config_from_hf(hf, bits=4)
    with pytest.raises(NotImplementedError):
        ck.config_from_hf(dict(hf, model_type="mistral", sliding_window=4096))
    assert ck.config_from_hf(dict(hf, model_type="mistral", sliding_window=None)).num_key_value_heads == 8
    assert ck.config_from_hf(dict(hf, model_type="qwen2", sliding_window=131072, use_sliding_window=False)).attention_bias


def test_wrong_checkpoints_are_refused(tmp_path):
    from safetensors.torch import load_file, save_file
    src = _toy()
    ck.save_pretrained(src, str(tmp_path))
    state = load_file(str(tmp_path / "model.safetensors"))
    # a missing tensor
    save_file({k: v for k, v in state.items() if k != "model.norm.weight"}, str(tmp_path / "model.safetensors"))
    with pytest.raises(KeyError, match="model.norm.weight"):
        ck.load_pretrained(str(tmp_path), torch.float32, "cpu")
    # a tensor the model has no parameter for
    save_file(dict(state, **{"model.layers.9.mlp.up_proj.weight": torch.zeros(2)}), str(tmp_path / "model.safetensors"))
    with pytest.raises(KeyError, match="layers.9"):
        ck.load_pretrained(str(tmp_path), torch.float32, "cpu")
    # a wrong shape
    save_file(dict(state, **{"model.norm.weight": torch.zeros(3)}), str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError, match="shape"):
        ck.load_pretrained(str(tmp_path), torch.float32, "cpu")
    # an old checkpoint's rotary buffer is ignored
    save_file(dict(state, **{"model.layers.0.self_attn.rotary_emb.inv_freq": torch.zeros(64)}), str(tmp_path / "model.safetensors"))
    ck.load_pretrained(str(tmp_path), torch.float32, "cpu")
    # no safetensors at all (a pickle checkpoint is not read)
    os.remove(tmp_path / "model.safetensors")
    (tmp_path / "pytorch_model.bin").write_bytes(b"")
    with pytest.raises(FileNotFoundError):
        ck.load_pretrained(str(tmp_path), torch.float32, "cpu")


@pytest.mark.parametrize("family", ["llama", "qwen2"])
def test_directories_written_by_transformers_load(tmp_path, family):
    """A checkpoint directory as Hugging Face's own `save_pretrained` writes it (a library, not the reference)."""
    transformers = pytest.importorskip("transformers")
    kw = dict(hidden_size=256, num_attention_heads=2, num_key_value_heads=1, num_hidden_layers=2, intermediate_size=128,
              vocab_size=96, max_position_embeddings=4096, eos_token_id=5)
    scaling = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
               "original_max_position_embeddings": 8192}
    torch.manual_seed(3)
    if family == "llama":
        try:
            cfg = transformers.LlamaConfig(rope_parameters=dict(scaling, rope_theta=5e5), head_dim=128, **kw)
            if getattr(cfg, "rope_parameters", None) is None:
                raise TypeError
        except TypeError:
            cfg = transformers.LlamaConfig(rope_theta=5e5, rope_scaling=scaling, head_dim=128, **kw)
        hf = transformers.LlamaForCausalLM(cfg)
    else:
        hf = transformers.Qwen2ForCausalLM(transformers.Qwen2Config(**kw))
    hf.save_pretrained(str(tmp_path), safe_serialization=True)
    got = ck.load_pretrained(str(tmp_path), torch.float32, "cpu")
    assert type(got).__name__ == ("LlamaPolarForCausalLM" if family == "llama" else "Qwen2PolarForCausalLM")
    want = dict(hf.named_parameters())
    mine = dict(got.named_parameters())
    assert set(mine) == set(want)
    for name, p in mine.items():
        assert torch.equal(p, want[name]), name
    assert got.config.eos_token_id == [5]
    if family == "llama":
        from polarquant_amd.modeling_common import rope_parameters
        theta, sc = rope_parameters(got.config)
        assert theta == 5e5 and sc["rope_type"] == "llama3" and sc["factor"] == 8.0
        assert torch.allclose(got.model.rotary_emb.inv_freq, hf.model.rotary_emb.inv_freq, rtol=1e-6, atol=0)
