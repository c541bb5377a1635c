"""Load a Hugging Face checkpoint directory (config.json + safetensors) into the polar-key models.

The reference gets this from `PreTrainedModel.from_pretrained` (its evaluation scripts call
`LlamaPolarForCausalLM.from_pretrained(path, torch_dtype=torch.bfloat16)`, test4long.py:46-47,
test4gsm8k.py:160); the models here are plain `nn.Module`s whose parameter names are the
checkpoint's, so loading is reading the shards and checking that every name matched.

    model = load_pretrained("/path/to/llama-3.1-8b", rbits=4, tbits=4)
    gen = load_generation_config("/path/to/llama-3.1-8b")

Only safetensors files are read: a pickle checkpoint (`pytorch_model.bin`) is refused.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Dict, Iterable, List, Optional

import torch

from .modeling_common import GenerationConfig, PolarConfig

_ARCH_FIELDS = ("hidden_size", "num_attention_heads", "num_key_value_heads", "num_hidden_layers", "intermediate_size",
                "vocab_size", "rms_norm_eps", "rope_theta", "rope_scaling", "head_dim", "attention_bias", "mlp_bias",
                "tie_word_embeddings")


def _as_id_list(ids) -> List[int]:
    if ids is None:
        return []
    return [int(i) for i in ids] if isinstance(ids, (list, tuple)) else [int(ids)]


def config_from_hf(hf: Dict, **polar_options) -> PolarConfig:
    """PolarConfig from the dict of a checkpoint's config.json.  `polar_options`: the cache fields of PolarConfig
    (rbits, tbits, vbits, snapkv, packed_codes, eager_gpu_codes, cache_capacity)."""
    kind = hf.get("model_type", "llama")
    if kind not in ("llama", "qwen2", "mistral"):
        raise ValueError("polarquant_amd: model_type %r is not one of llama, qwen2, mistral" % (kind,))
    if hf.get("sliding_window") and hf.get("use_sliding_window", kind == "mistral"):
        raise NotImplementedError("polarquant_amd: sliding-window attention is not implemented")
    fields = {k: hf[k] for k in _ARCH_FIELDS if hf.get(k) is not None}
    rp = hf.get("rope_parameters")                          # transformers 5 writes one dict instead of theta + scaling
    if isinstance(rp, dict):
        if rp.get("rope_theta") is not None:
            fields["rope_theta"] = rp["rope_theta"]
        fields["rope_scaling"] = {k: v for k, v in rp.items() if k != "rope_theta"}
    sc = fields.get("rope_scaling")
    if isinstance(sc, dict) and sc.get("rope_type", sc.get("type", "default")) == "default":
        fields.pop("rope_scaling")
    fields.setdefault("num_key_value_heads", fields["num_attention_heads"])
    fields.setdefault("head_dim", fields["hidden_size"] // fields["num_attention_heads"])
    if fields["head_dim"] != 128:
        raise ValueError("polarquant_amd: the polar-key kernels need head_dim 128, the checkpoint has %d" % fields["head_dim"])
    if kind == "qwen2":
        fields["attention_bias"] = True                 # Qwen2 has q/k/v biases and no config field for them
    eos = _as_id_list(hf.get("eos_token_id"))
    if eos:
        fields["eos_token_id"] = eos
    known = {f.name for f in dataclasses.fields(PolarConfig)}
    unknown = set(polar_options) - known
    if unknown:
        raise TypeError("polarquant_amd: unknown PolarConfig options %s" % sorted(unknown))
    return PolarConfig(**fields, **polar_options)


def _shard_files(path: str) -> List[str]:
    index = os.path.join(path, "model.safetensors.index.json")
    if os.path.exists(index):
        with open(index) as f:
            names = sorted(set(json.load(f)["weight_map"].values()))
        return [os.path.join(path, n) for n in names]
    single = os.path.join(path, "model.safetensors")
    if os.path.exists(single):
        return [single]
    raise FileNotFoundError("polarquant_amd: no model.safetensors(.index.json) in %s (pickle checkpoints are not read)" % path)


def load_state(model: torch.nn.Module, shard_files: Iterable[str], dtype: torch.dtype) -> None:
    """Copy the tensors of the shards into `model`'s parameters (cast to `dtype`), shard by shard so that host
    memory holds one shard at a time; every parameter must be found, and every tensor must belong to a parameter
    (rotary `inv_freq` buffers that old checkpoints carry are ignored: they are recomputed)."""
    from safetensors import safe_open
    params = dict(model.named_parameters())
    tied = getattr(model.config, "tie_word_embeddings", False)
    seen = set()
    with torch.no_grad():
        for fn in shard_files:
            with safe_open(fn, framework="pt", device="cpu") as f:
                for name in f.keys():
                    if name.endswith("rotary_emb.inv_freq"):
                        continue
                    if name == "lm_head.weight" and tied:
                        continue
                    if name not in params:
                        raise KeyError("polarquant_amd: %s holds %r, which the model has no parameter for" % (fn, name))
                    t = f.get_tensor(name)
                    p = params[name]
                    if tuple(t.shape) != tuple(p.shape):
                        raise ValueError("polarquant_amd: %r has shape %s in the checkpoint, %s in the model"
                                         % (name, tuple(t.shape), tuple(p.shape)))
                    p.copy_(t.to(dtype))
                    seen.add(name)
    missing = [n for n in params if n not in seen and not (tied and n == "lm_head.weight")]
    if missing:
        raise KeyError("polarquant_amd: the checkpoint has no tensor for %s" % missing[:8])


def load_pretrained(path: str, dtype: torch.dtype = torch.bfloat16, device="cuda:0", model_class=None, **polar_options):
    """-> the polar-key model of the checkpoint in `path`, in eval mode on `device`.  `model_class`: by default
    LlamaPolarForCausalLM (also for Mistral, whose layers are Llama's) or Qwen2PolarForCausalLM by `model_type`."""
    with open(os.path.join(path, "config.json")) as f:
        hf = json.load(f)
    cfg = config_from_hf(hf, **polar_options)
    if model_class is None:
        if hf.get("model_type") == "qwen2":
            from .modeling_qwen_polar import Qwen2PolarForCausalLM as model_class
        else:
            from .modeling_llama_polar import LlamaPolarForCausalLM as model_class
    prev = torch.get_default_dtype()
    torch.set_default_dtype(dtype)
    try:
        with torch.device(device):
            model = model_class(cfg)
    finally:
        torch.set_default_dtype(prev)
    load_state(model, _shard_files(path), dtype)
    return model.eval()


def load_generation_config(path: str) -> GenerationConfig:
    """The fields of generation_config.json that the reference's `sample` reads (models/modeling_llama_polar.py:
    606-619): eos_token_id, top_k, top_p, temperature; config.json's eos_token_id if that file is absent."""
    out: Dict = {}
    for fn in ("config.json", "generation_config.json"):
        full = os.path.join(path, fn)
        if os.path.exists(full):
            with open(full) as f:
                d = json.load(f)
            for k in ("top_k", "top_p", "temperature"):
                if d.get(k) is not None:
                    out[k] = d[k]
            if _as_id_list(d.get("eos_token_id")):
                out["eos_token_id"] = _as_id_list(d["eos_token_id"])
    return GenerationConfig(**out)


def save_pretrained(model: torch.nn.Module, path: str, model_type: str = "llama", shards: int = 1,
                    generation: Optional[GenerationConfig] = None) -> None:
    """Write `model` as a checkpoint directory that `load_pretrained` (and Hugging Face) reads: config.json,
    generation_config.json and `shards` safetensors files with their index."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    c = model.config
    hf = {k: getattr(c, k) for k in _ARCH_FIELDS if getattr(c, k, None) is not None}
    hf.update(model_type=model_type, eos_token_id=_as_id_list(getattr(c, "eos_token_id", None)))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(hf, f, indent=1)
    g = generation or GenerationConfig(eos_token_id=hf["eos_token_id"] or [2])
    with open(os.path.join(path, "generation_config.json"), "w") as f:
        json.dump(dataclasses.asdict(g), f, indent=1)
    tied = getattr(c, "tie_word_embeddings", False)
    state = {k: v.detach().cpu().contiguous() for k, v in model.named_parameters() if not (tied and k == "lm_head.weight")}
    names = list(state)
    if shards <= 1:
        save_file(state, os.path.join(path, "model.safetensors"))
        return
    per = -(-len(names) // shards)
    weight_map = {}
    for i in range(shards):
        part = names[i * per:(i + 1) * per]
        if not part:
            continue
        fn = "model-%05d-of-%05d.safetensors" % (i + 1, shards)
        save_file({k: state[k] for k in part}, os.path.join(path, fn))
        weight_map.update({k: fn for k in part})
    with open(os.path.join(path, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f, indent=1)
