"""Host-side mirror of the reference's polar attention classes and model shell.

Reference interfaces mirrored here (same names, argument meaning, return values):
  * `*PolarGroupAttention.forward(hidden_states, attention_mask=None, past_key_value=None,
    position_embeddings=None, **kwargs) -> (attn_output, past_key_value)` with the 8-tuple cache
    `(key_states_full | None, indices | None, rscale, rmn, tscale, tmn, value_states_full, kv_seq_len)`
    (models/modeling_llama_polar.py:31-157, models/modeling_qwen_polar.py:30-156);
  * `*PolarDecoderLayer`, `*PolarModel`, `*PolarForCausalLM` (modeling_llama_polar.py:447-562);
  * `generate`, `sample`, `top_k_top_p_filtering` (modeling_llama_polar.py:565-666).

Differences that do not show at the interface: the decode branch is ONE fused HIP
launch pair (scores + softmax + P.V, then the split merge) instead of ~12 eager
kernels, and the cache tensors handed back in the tuple are views into a
pre-allocated per-layer arena, so appending a token or a quantized group is O(1)
instead of a torch.cat of the whole cache (reference :86-90,98).  The tuple is a
`PolarCache` (a tuple subclass) that remembers its arena; a plain tuple in the
reference's format is accepted too and is copied into a fresh arena.

The modules are self-contained torch.nn modules whose parameter names match the
HF Llama / Qwen2 checkpoints (model.layers.N.self_attn.q_proj.weight, ...), so a
HF state_dict loads with load_state_dict; they do not import `transformers`.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from .attention import polar_decode_attention, polar_decode_attention_v4
from .quantize import quantize_and_pack_nbit
from .values import quantize_values

GROUP = 128


# ----------------------------------------------------------------------------- config
@dataclass
class PolarConfig:
    hidden_size: int = 4096
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    num_hidden_layers: int = 32
    intermediate_size: int = 14336
    vocab_size: int = 128256
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    rope_scaling: Optional[dict] = None  # HF's dict ("rope_type": "linear" | "llama3", ...), None: plain RoPE
    head_dim: int = 128
    attention_bias: bool = False        # q/k/v bias (Qwen2: True)
    mlp_bias: bool = False
    tie_word_embeddings: bool = False
    eos_token_id: List[int] = field(default_factory=lambda: [128001])
    # polar cache
    rbits: int = 4
    tbits: int = 4
    vbits: int = 16                     # 4: values in 4 bits as well (the Mixed variant); 16: half-precision values
    snapkv: bool = False                # SnapKV prompt eviction in front of the polar cache (batch 1 decode)
    packed_codes: bool = False          # 3/3-bit key codes as packed 6-bit rows (48 instead of 64 bytes per token and head)
    eager_gpu_codes: bool = False       # key codes / metadata as the reference's lines give them on GPU tensors (fp32 wrap,
                                        # device atan2f) instead of on CPU tensors; for caches shared with a GPU-run reference
    cache_capacity: int = 0             # tokens to pre-allocate per layer (0: prompt + 1024, grown by doubling)

    @staticmethod
    def llama3_8b(**kw) -> "PolarConfig":
        return PolarConfig(**kw)

    @staticmethod
    def llama2_7b(**kw) -> "PolarConfig":
        return PolarConfig(num_key_value_heads=32, intermediate_size=11008, vocab_size=32000, rope_theta=1e4,
                           eos_token_id=[2], **kw)

    @staticmethod
    def qwen25_7b(**kw) -> "PolarConfig":
        return PolarConfig(hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, num_hidden_layers=28,
                           intermediate_size=18944, vocab_size=152064, rms_norm_eps=1e-6, rope_theta=1e6,
                           attention_bias=True, eos_token_id=[151645, 151643], **kw)


def _cfg(config, name, default=None):
    return getattr(config, name, default)


# ----------------------------------------------------------------------------- rope helpers (HF conventions)
def rotate_half(x: torch.Tensor) -> torch.Tensor:
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin, unsqueeze_dim: int = 1):
    cos, sin = cos.unsqueeze(unsqueeze_dim), sin.unsqueeze(unsqueeze_dim)
    return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


def project_heads_and_rotate(q_lin, k_lin, cos, sin, n_heads: int, n_kv_heads: int, head_dim: int):
    """The reference's `.view(B, L, heads, d).transpose(1, 2)` on the q / k projections followed by
    `apply_rotary_pos_emb` (models/modeling_llama_polar.py:53-59).  On the GPU, at head_dim 128 in half precision, one
    HIP launch with the same bits as the eager chain of multiplies, negation, concatenation and add."""
    B, L = q_lin.shape[0], q_lin.shape[1]
    if (q_lin.is_cuda and head_dim == 128 and q_lin.dtype in (torch.float16, torch.bfloat16) and cos.dtype == q_lin.dtype
            and cos.dim() == 3 and cos.shape[0] in (1, B) and tuple(cos.shape[1:]) == (L, 128) and not torch.is_grad_enabled()):
        from .decode_ops import rope_qk
        return rope_qk(q_lin, k_lin, cos, sin, n_heads, n_kv_heads)
    q = q_lin.view(B, L, n_heads, head_dim).transpose(1, 2)
    k = k_lin.view(B, L, n_kv_heads, head_dim).transpose(1, 2)
    return apply_rotary_pos_emb(q, k, cos, sin)


def repeat_kv(hidden_states: torch.Tensor, n_rep: int) -> torch.Tensor:
    b, h, s, d = hidden_states.shape
    if n_rep == 1:
        return hidden_states
    return hidden_states[:, :, None, :, :].expand(b, h, n_rep, s, d).reshape(b, h * n_rep, s, d)


def repeat_kv_quant(hidden_states: torch.Tensor, n_rep: int) -> torch.Tensor:
    """(models/modeling_llama_polar.py:23-28) kept for callers that expand the code cache themselves;
    the HIP kernels handle any GQA ratio natively and never need it."""
    b, h, nb, s, d = hidden_states.shape
    if n_rep == 1:
        return hidden_states
    return hidden_states[:, :, None].expand(b, h, n_rep, nb, s, d).reshape(b, h * n_rep, nb, s, d)


def rope_parameters(config):
    """(theta, scaling dict or None) of a PolarConfig or of a HF config of either generation:
    transformers < 5 keeps `rope_theta` / `rope_scaling` as attributes, 5.x one `rope_parameters` dict."""
    theta = getattr(config, "rope_theta", None)
    scaling = getattr(config, "rope_scaling", None)
    rp = getattr(config, "rope_parameters", None)
    if isinstance(rp, dict):
        theta = rp.get("rope_theta", theta)
        scaling = rp
    if isinstance(scaling, dict) and scaling.get("rope_type", scaling.get("type", "default")) == "default":
        scaling = None
    return (10000.0 if theta is None else float(theta)), scaling


class RotaryEmbedding(nn.Module):
    """cos / sin tables as HF's LlamaRotaryEmbedding gives them, which is what the reference's forward receives as
    `position_embeddings` (models/modeling_llama_polar.py:56-59).  Frequency scalings: none, "linear" and "llama3"
    (Llama-3.1's published wavelength-dependent rescaling); any other type is refused."""

    def __init__(self, head_dim: int, base: float, scaling: Optional[dict] = None):
        super().__init__()
        inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
        kind = "default" if not scaling else scaling.get("rope_type", scaling.get("type", "default"))
        if kind == "linear":
            inv_freq = inv_freq / float(scaling["factor"])
        elif kind == "llama3":
            factor, lo, hi = float(scaling["factor"]), float(scaling["low_freq_factor"]), float(scaling["high_freq_factor"])
            old_len = float(scaling["original_max_position_embeddings"])
            wavelen = 2 * math.pi / inv_freq
            scaled = torch.where(wavelen > old_len / lo, inv_freq / factor, inv_freq)
            smooth = (old_len / wavelen - lo) / (hi - lo)
            blended = (1 - smooth) * scaled / factor + smooth * scaled
            medium = ~(wavelen < old_len / hi) & ~(wavelen > old_len / lo)
            inv_freq = torch.where(medium, blended, scaled)
        elif kind != "default":
            raise NotImplementedError("polarquant_amd: rope scaling type %r is not implemented" % (kind,))
        self.register_buffer("inv_freq", inv_freq, persistent=False)

    @torch.no_grad()
    def forward(self, x: torch.Tensor, position_ids: torch.Tensor):
        freqs = position_ids[:, :, None].float() * self.inv_freq[None, None, :].float().to(x.device)
        emb = torch.cat((freqs, freqs), dim=-1)
        return emb.cos().to(x.dtype), emb.sin().to(x.dtype)


class RMSNorm(nn.Module):
    def __init__(self, hidden_size: int, eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps

    def forward(self, x):
        dt = x.dtype
        x = x.float()
        x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
        return self.weight * x.to(dt)


class MLP(nn.Module):
    def __init__(self, config):
        super().__init__()
        h, i, b = config.hidden_size, config.intermediate_size, _cfg(config, "mlp_bias", False)
        self.gate_proj = nn.Linear(h, i, bias=b)
        self.up_proj = nn.Linear(h, i, bias=b)
        self.down_proj = nn.Linear(i, h, bias=b)

    def forward(self, x):
        return self.down_proj(F.silu(self.gate_proj(x)) * self.up_proj(x))


# ----------------------------------------------------------------------------- cache
class _Arena:
    """Pre-allocated per-layer polar KV cache.  codes/meta/v grow by doubling."""

    def __init__(self, B, Nk, dtype, device, capacity_tokens, rbits, tbits, packed=False, eager_gpu=False):
        self.B, self.Nk, self.dtype, self.device = B, Nk, dtype, device
        self.rbits, self.tbits = rbits, tbits
        self.eager_gpu = eager_gpu    # quantize as eager torch does on GPU tensors
        self.packed = packed          # code rows of 48 bytes (packed 6-bit codes) instead of 64
        self.row = 48 if packed else 64
        self.n_groups = self.n_resid = self.kv_len = 0
        self.pos_offset = 0      # tokens the prompt held beyond the cached ones (SnapKV eviction): tuple[-1] = kv_len + pos_offset
        self.kres = torch.zeros(B, Nk, GROUP, 128, dtype=dtype, device=device)
        self._alloc(max(capacity_tokens, GROUP))

    def _alloc(self, cap_tokens):
        gcap = (cap_tokens + GROUP - 1) // GROUP
        vcap = gcap * GROUP + GROUP
        B, Nk, dev, dt = self.B, self.Nk, self.device, self.dtype
        codes = torch.empty(B, Nk, gcap, GROUP, self.row, dtype=torch.uint8, device=dev)
        meta = [torch.empty(B, Nk, gcap, 1, 64, dtype=dt, device=dev) for _ in range(4)]
        v = torch.empty(B, Nk, vcap, 128, dtype=dt, device=dev)
        if self.kv_len:
            codes[:, :, :self.n_groups] = self.codes[:, :, :self.n_groups]
            for new, old in zip(meta, self.meta):
                new[:, :, :self.n_groups] = old[:, :, :self.n_groups]
            v[:, :, :self.kv_len] = self.v[:, :, :self.kv_len]
        self.codes, self.meta, self.v, self.gcap, self.vcap = codes, meta, v, gcap, vcap

    def reserve(self, tokens):
        if tokens > self.vcap or (tokens // GROUP) > self.gcap:
            self._alloc(max(2 * self.vcap, tokens))

    def quantize_into(self, keys):
        """keys [B,Nk,n*128,128] (any strides with unit dim stride) -> groups appended."""
        n = keys.shape[2] // GROUP
        quantize_and_pack_nbit(keys, self.rbits, self.tbits, packed=self.packed, out=(self.codes, *self.meta),
                               group_offset=self.n_groups, eager_gpu=self.eager_gpu)
        self.n_groups += n

    def as_tuple(self) -> "PolarCache":
        kf = self.kres[:, :, :self.n_resid] if self.n_resid else None
        if self.n_groups:
            q5 = [self.codes[:, :, :self.n_groups]] + [m[:, :, :self.n_groups] for m in self.meta]
        else:
            q5 = [None] * 5
        return PolarCache((kf, *q5, self.v[:, :, :self.kv_len], self.kv_len + self.pos_offset), self)


class PolarCache(tuple):
    """The reference's 8-tuple, plus the arena its tensors are views of."""

    def __new__(cls, items, arena):
        obj = super().__new__(cls, items)
        obj.arena = arena
        return obj


_MASK_CACHE = {"src": None, "version": -1, "u8": None}


def _mask_u8(mask: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """attention_mask [B, L] of {0,1} (any dtype) -> uint8, converted once per step, not once per layer.

    The cache entry is recognised by the identity of the mask tensor (and its version counter), and it
    keeps that tensor alive: an address can then not be handed to a different mask while the entry
    exists, which a key made of the address alone would not notice."""
    if mask is None:
        return None
    if mask.dtype == torch.uint8:
        return mask
    if _MASK_CACHE["src"] is not mask or _MASK_CACHE["version"] != mask._version:
        _MASK_CACHE["u8"] = (mask != 0).to(torch.uint8)
        _MASK_CACHE["src"], _MASK_CACHE["version"] = mask, mask._version
    return _MASK_CACHE["u8"]


# ----------------------------------------------------------------------------- attention
class PolarGroupAttention(nn.Module):
    """Polar-key attention with the reference's forward signature and cache tuple."""

    def __init__(self, config, layer_idx: Optional[int] = None):
        super().__init__()
        self.config, self.layer_idx = config, layer_idx
        self.hidden_size = config.hidden_size
        self.num_heads = config.num_attention_heads
        self.head_dim = _cfg(config, "head_dim", None) or self.hidden_size // self.num_heads
        if self.head_dim != 128:
            raise ValueError("polar attention kernels are built for head_dim 128 (64 pairs (d, d+64) per key); "
                             "this configuration has head_dim %d" % self.head_dim)
        self.num_key_value_heads = _cfg(config, "num_key_value_heads", self.num_heads)
        self.num_key_value_groups = self.num_heads // self.num_key_value_heads
        self.is_causal = True
        qkv_bias = _cfg(config, "attention_bias", False)
        self.q_proj = nn.Linear(self.hidden_size, self.num_heads * self.head_dim, bias=qkv_bias)
        self.k_proj = nn.Linear(self.hidden_size, self.num_key_value_heads * self.head_dim, bias=qkv_bias)
        self.v_proj = nn.Linear(self.hidden_size, self.num_key_value_heads * self.head_dim, bias=qkv_bias)
        self.o_proj = nn.Linear(self.num_heads * self.head_dim, self.hidden_size, bias=False)
        # reference :34-37
        self.rbits = _cfg(config, "rbits", 4)
        self.tbits = _cfg(config, "tbits", 4)
        self.group_size = 128
        self.residual_length = 128
        # not in the reference (which stores one byte per pair for every bit width, kernel4group.py:1-3):
        # 3/3-bit codes stored as packed 6-bit rows, indices [B,Nk,Nb,128,48] in the cache tuple
        self.packed_codes = bool(_cfg(config, "packed_codes", False))
        self.eager_gpu_codes = bool(_cfg(config, "eager_gpu_codes", False))
        assert not self.packed_codes or (self.tbits == 3 and self.rbits + self.tbits <= 6), "packed codes: tbits 3, rbits <= 3"
        self.capture = None   # test hook: a list that receives post-RoPE (q, k, v) of every call

    # -- cache plumbing --------------------------------------------------------
    def _new_arena(self, B, dtype, device, tokens):
        cap = _cfg(self.config, "cache_capacity", 0) or (tokens + 1024)
        return _Arena(B, self.num_key_value_heads, dtype, device, max(cap, tokens), self.rbits, self.tbits, self.packed_codes,
                      self.eager_gpu_codes)

    def _arena_of(self, past_key_value, dtype, device) -> _Arena:
        arena = getattr(past_key_value, "arena", None)
        if arena is not None and arena.kv_len + arena.pos_offset == past_key_value[-1]:
            return arena
        # a plain tuple in the reference's format: copy it into a fresh arena
        kf, ind, rs, rm, ts, tm, v, seen = past_key_value
        n = v.shape[2]                       # cached tokens; `seen` may be larger (evicted prompt tokens)
        arena = self._new_arena(v.shape[0], dtype, device, n + 1)
        arena.pos_offset = seen - n
        if ind is not None:
            g = ind.shape[2]
            arena.codes[:, :, :g] = ind
            for dst, src in zip(arena.meta, (rs, rm, ts, tm)):
                dst[:, :, :g] = src
            arena.n_groups = g
        if kf is not None:
            arena.kres[:, :, :kf.shape[2]] = kf
            arena.n_resid = kf.shape[2]
        arena.v[:, :, :n] = v
        arena.kv_len = n
        return arena

    # -- forward (reference :39-133) ---------------------------------------------
    def forward(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                past_key_value=None, position_embeddings: Tuple[torch.Tensor, torch.Tensor] = None, **kwargs):
        bsz, q_len, _ = hidden_states.size()
        value_states = self.v_proj(hidden_states).view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
        cos, sin = position_embeddings
        query_states, key_states = project_heads_and_rotate(self.q_proj(hidden_states), self.k_proj(hidden_states), cos, sin,
                                                            self.num_heads, self.num_key_value_heads, self.head_dim)
        if self.capture is not None:
            self.capture.append((query_states.detach().clone(), key_states.detach().clone(), value_states.detach().clone()))

        # decoding time (:61-101).  A one-token prompt (no cache yet) is a prefill here; the reference takes its
        # decode branch on q_len alone and fails unpacking the missing cache.
        if q_len == 1 and past_key_value is not None:
            arena = self._arena_of(past_key_value, query_states.dtype, query_states.device)
            arena.reserve(arena.kv_len + 1)
            arena.kres[:, :, arena.n_resid] = key_states[:, :, 0]          # :77
            arena.v[:, :, arena.kv_len] = value_states[:, :, 0]            # :98
            arena.n_resid += 1
            arena.kv_len += 1
            attn_output = polar_decode_attention(
                query_states, arena.codes if arena.n_groups else None, *(arena.meta if arena.n_groups else [None] * 4),
                arena.kres, arena.v, arena.n_groups, arena.n_resid, attention_mask=_mask_u8(attention_mask),
                rbits=self.rbits, tbits=self.tbits, sm_scale=1.0 / math.sqrt(self.head_dim))   # :66-99
            if arena.n_resid % self.residual_length == 0:                  # :83-92
                arena.quantize_into(arena.kres)
                arena.n_resid = 0
            past_key_value = arena.as_tuple()                              # :101
        else:            # pre-filling (:102-128)
            assert past_key_value is None
            kv_seq_len = key_states.shape[2]
            attn_output = _prefill_attention(query_states, key_states, value_states, attention_mask,
                                             self.num_key_value_groups, self.is_causal)
            arena = self._new_arena(bsz, key_states.dtype, key_states.device, kv_seq_len + 1)
            residual_length = kv_seq_len % self.residual_length
            n_quant = kv_seq_len - residual_length if kv_seq_len >= self.residual_length else 0
            if n_quant:
                arena.quantize_into(key_states[:, :, :n_quant])            # :124-126 (read in place, strided)
            if kv_seq_len - n_quant:
                arena.kres[:, :, :kv_seq_len - n_quant] = key_states[:, :, n_quant:]
            arena.n_resid = kv_seq_len - n_quant
            arena.v[:, :, :kv_seq_len] = value_states
            arena.kv_len = kv_seq_len
            past_key_value = arena.as_tuple()                              # :128

        attn_output = attn_output.reshape(bsz, q_len, -1).contiguous()
        attn_output = self.o_proj(attn_output)
        return attn_output, past_key_value

    def quantize_and_pack_nbit(self, key_states):
        """(reference :135-157) -> (indices, rscale, rmn, tscale, tmn)."""
        return quantize_and_pack_nbit(key_states, self.rbits, self.tbits, self.group_size)


# ----------------------------------------------------------------------------- Mixed variant: polar keys + 4-bit values
class _MixedArena(_Arena):
    """Per-layer cache of the Mixed variant: polar key groups, 4-bit value rows for the same tokens,
    and a shared 128-token residual window of half-precision keys and values."""

    def __init__(self, B, Nk, dtype, device, capacity_tokens, rbits, tbits, packed=False, eager_gpu=False):
        self.vres = torch.zeros(B, Nk, GROUP, 128, dtype=dtype, device=device)
        super().__init__(B, Nk, dtype, device, capacity_tokens, rbits, tbits, packed, eager_gpu)

    def _alloc(self, cap_tokens):
        gcap = (cap_tokens + GROUP - 1) // GROUP
        B, Nk, dev, dt = self.B, self.Nk, self.device, self.dtype
        codes = torch.empty(B, Nk, gcap, GROUP, self.row, dtype=torch.uint8, device=dev)
        meta = [torch.empty(B, Nk, gcap, 1, 64, dtype=dt, device=dev) for _ in range(4)]
        vcodes = torch.empty(B, Nk, gcap * GROUP, 16, dtype=torch.int32, device=dev)
        vmeta = [torch.empty(B, Nk, gcap * GROUP, 1, dtype=dt, device=dev) for _ in range(2)]
        if self.n_groups:
            g, t = self.n_groups, self.n_groups * GROUP
            codes[:, :, :g] = self.codes[:, :, :g]
            for new, old in zip(meta, self.meta):
                new[:, :, :g] = old[:, :, :g]
            vcodes[:, :, :t] = self.vcodes[:, :, :t]
            for new, old in zip(vmeta, self.vmeta):
                new[:, :, :t] = old[:, :, :t]
        self.codes, self.meta, self.vcodes, self.vmeta, self.gcap = codes, meta, vcodes, vmeta, gcap
        self.v, self.vcap = None, gcap * GROUP + GROUP

    def flush(self):
        """The window holds 128 keys and values: both go to the quantized store together (reference :207-217, :243-250)."""
        quantize_values(self.vres, out=(self.vcodes, *self.vmeta), token_offset=self.n_groups * GROUP)
        self.quantize_into(self.kres)
        self.n_resid = 0

    def as_tuple(self) -> "PolarCache":
        r, g = self.n_resid, self.n_groups
        kf = self.kres[:, :, :r] if r else None
        vf = self.vres[:, :, :r] if r else None
        if g:
            q5 = [self.codes[:, :, :g]] + [m[:, :, :g] for m in self.meta]
            v3 = [self.vcodes[:, :, :g * GROUP]] + [m[:, :, :g * GROUP] for m in self.vmeta]
        else:
            q5, v3 = [None] * 5, [None] * 3
        return PolarCache((kf, *q5, vf, *v3, self.kv_len + self.pos_offset), self)


class PolarMixedGroupAttention(PolarGroupAttention):
    """Polar keys + 4-bit values, the reference's LlamaPolarMixedGroupAttention
    (models/modeling_llama_polar.py:160-292): same forward signature, 11-slot cache tuple
    (key_states_full, indices, rscale, rmn, tscale, tmn, value_states_full, value_states_quant,
    value_scale, value_mn, kv_seq_len)."""

    def __init__(self, config, layer_idx: Optional[int] = None):
        super().__init__(config, layer_idx)
        self.vbits = 4                                                     # :163

    def _new_arena(self, B, dtype, device, tokens):
        cap = _cfg(self.config, "cache_capacity", 0) or (tokens + 1024)
        return _MixedArena(B, self.num_key_value_heads, dtype, device, max(cap, tokens), self.rbits, self.tbits, self.packed_codes,
                           self.eager_gpu_codes)

    def _arena_of(self, past_key_value, dtype, device) -> _MixedArena:
        arena = getattr(past_key_value, "arena", None)
        if arena is not None and arena.kv_len + arena.pos_offset == past_key_value[-1]:
            return arena
        # a plain 11-tuple in the reference's format: copy it into a fresh arena
        kf, ind, rs, rm, ts, tm, vf, vc, vs, vm, n = past_key_value
        assert n == (0 if ind is None else ind.shape[2] * GROUP) + (0 if kf is None else kf.shape[2])
        B = (kf if kf is not None else ind).shape[0]
        arena = self._new_arena(B, dtype, device, n + 1)
        if ind is not None:
            g = ind.shape[2]
            arena.codes[:, :, :g] = ind
            for dst, src in zip(arena.meta, (rs, rm, ts, tm)):
                dst[:, :, :g] = src
            arena.vcodes[:, :, :g * GROUP] = vc
            for dst, src in zip(arena.vmeta, (vs, vm)):
                dst[:, :, :g * GROUP] = src
            arena.n_groups = g
        if kf is not None:
            arena.kres[:, :, :kf.shape[2]] = kf
            arena.vres[:, :, :kf.shape[2]] = vf
            arena.n_resid = kf.shape[2]
        arena.kv_len = n
        return arena

    def forward(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                past_key_value=None, position_embeddings: Tuple[torch.Tensor, torch.Tensor] = None, **kwargs):
        bsz, q_len, _ = hidden_states.size()
        value_states = self.v_proj(hidden_states).view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
        cos, sin = position_embeddings
        query_states, key_states = project_heads_and_rotate(self.q_proj(hidden_states), self.k_proj(hidden_states), cos, sin,
                                                            self.num_heads, self.num_key_value_heads, self.head_dim)
        if self.capture is not None:
            self.capture.append((query_states.detach().clone(), key_states.detach().clone(), value_states.detach().clone()))

        if q_len == 1 and past_key_value is not None:   # decoding time (:185-257); a one-token prompt is a prefill
            arena = self._arena_of(past_key_value, query_states.dtype, query_states.device)
            arena.reserve(arena.kv_len + 1)
            arena.kres[:, :, arena.n_resid] = key_states[:, :, 0]          # :201
            arena.vres[:, :, arena.n_resid] = value_states[:, :, 0]        # :223
            arena.n_resid += 1
            arena.kv_len += 1
            g = arena.n_groups
            attn_output = polar_decode_attention_v4(
                query_states, arena.codes if g else None, *(arena.meta if g else [None] * 4), arena.kres, arena.vres,
                arena.vcodes if g else None, *(arena.vmeta if g else [None] * 2), g, arena.n_resid,
                attention_mask=_mask_u8(attention_mask), rbits=self.rbits, tbits=self.tbits,
                sm_scale=1.0 / math.sqrt(self.head_dim))                   # :189-241
            if arena.n_resid % self.residual_length == 0:                  # :207, :243
                arena.flush()
            past_key_value = arena.as_tuple()                              # :257
        else:            # pre-filling (:258-281)
            assert past_key_value is None
            kv_seq_len = key_states.shape[2]
            attn_output = _prefill_attention(query_states, key_states, value_states, attention_mask,
                                             self.num_key_value_groups, self.is_causal)
            arena = self._new_arena(bsz, key_states.dtype, key_states.device, kv_seq_len + 1)
            residual_length = kv_seq_len % self.residual_length
            n_quant = kv_seq_len - residual_length if kv_seq_len >= self.residual_length else 0
            if n_quant:
                quantize_values(value_states[:, :, :n_quant], out=(arena.vcodes, *arena.vmeta), token_offset=0)   # :275
                arena.quantize_into(key_states[:, :, :n_quant])            # :271
            r = kv_seq_len - n_quant
            if r:
                arena.kres[:, :, :r] = key_states[:, :, n_quant:]
                arena.vres[:, :, :r] = value_states[:, :, n_quant:]
            arena.n_resid, arena.kv_len = r, kv_seq_len
            past_key_value = arena.as_tuple()                              # :281

        attn_output = attn_output.reshape(bsz, q_len, -1).contiguous()
        attn_output = self.o_proj(attn_output)
        return attn_output, past_key_value


# ----------------------------------------------------------------------------- SnapKV prompt eviction + polar cache
class PolarSnapKVAttention(PolarGroupAttention):
    """The reference's LlamaSnapKVAttention (models/modeling_llama_polar.py:295-443): prompts longer
    than max_capacity_prompt keep only the earlier tokens that the last `window_size` queries attend
    to most (pooled, top-k per KV head) plus that window; the kept keys then go through the usual
    polar cache.  Decode is the polar decode step without mask, batch 1 (:327).  The selection runs
    once per prompt with torch ops; the cache and the decode step use the HIP path."""

    def __init__(self, config, layer_idx: Optional[int] = None):
        super().__init__(config, layer_idx)
        self.window_size = 128                                             # :298-300
        self.kernel_size = 7
        self.max_capacity_prompt = 1024 + self.window_size

    def select(self, query_states, key_states):
        """-> indices [B, Nk, max_capacity_prompt - window_size] of the earlier tokens to keep (:398-414)."""
        bsz, ws = query_states.shape[0], self.window_size
        w = torch.matmul(query_states[:, :, -ws:, :], repeat_kv(key_states, self.num_key_value_groups).transpose(2, 3))
        mask = torch.full((ws, ws), torch.finfo(w.dtype).min, device=w.device)
        cond = torch.arange(ws, device=w.device)
        mask.masked_fill_(cond < (cond + 1).view(ws, 1), 0)
        w[:, :, -ws:, -ws:] += mask[None, None, :, :].to(w.dtype)
        w = F.softmax(w, dim=-1, dtype=torch.float32).to(query_states.dtype)
        s = w[:, :, -ws:, :-ws].sum(dim=-2)
        pooled = F.avg_pool1d(s, kernel_size=self.kernel_size, padding=self.kernel_size // 2, stride=1)
        pooled = pooled.view(bsz, self.num_key_value_heads, self.num_key_value_groups, -1).mean(dim=2)
        return pooled.topk(self.max_capacity_prompt - ws, dim=-1).indices

    def forward(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                past_key_value=None, position_embeddings: Tuple[torch.Tensor, torch.Tensor] = None, **kwargs):
        bsz, q_len, _ = hidden_states.size()
        if q_len == 1:
            assert bsz == 1                                                # :327 (no per-sequence mask after eviction)
            return super().forward(hidden_states, None, past_key_value, position_embeddings, **kwargs)
        value_states = self.v_proj(hidden_states).view(bsz, q_len, self.num_key_value_heads, self.head_dim).transpose(1, 2)
        cos, sin = position_embeddings
        query_states, key_states = project_heads_and_rotate(self.q_proj(hidden_states), self.k_proj(hidden_states), cos, sin,
                                                            self.num_heads, self.num_key_value_heads, self.head_dim)
        if self.capture is not None:
            self.capture.append((query_states.detach().clone(), key_states.detach().clone(), value_states.detach().clone()))
        assert past_key_value is None
        kv_seq_len = key_states.shape[2]
        attn_output = _prefill_attention(query_states, key_states, value_states, attention_mask,
                                         self.num_key_value_groups, self.is_causal)
        self.last_selection = None
        if kv_seq_len > self.max_capacity_prompt:                          # :396
            ws = self.window_size
            idx = self.select(query_states, key_states)
            self.last_selection = idx
            idx = idx.unsqueeze(-1).expand(-1, -1, -1, self.head_dim)
            key_states = torch.cat([key_states[:, :, :-ws, :].gather(dim=2, index=idx), key_states[:, :, -ws:, :]], dim=2)
            value_states = torch.cat([value_states[:, :, :-ws, :].gather(dim=2, index=idx), value_states[:, :, -ws:, :]], dim=2)
        kept = key_states.shape[2]
        arena = self._new_arena(bsz, key_states.dtype, key_states.device, kept + 1)
        residual_length = kept % self.residual_length                      # :426
        n_quant = kept - residual_length if kv_seq_len >= self.residual_length else 0
        if n_quant:
            arena.quantize_into(key_states[:, :, :n_quant])
        if kept - n_quant:
            arena.kres[:, :, :kept - n_quant] = key_states[:, :, n_quant:]
        arena.n_resid = kept - n_quant
        arena.v[:, :, :kept] = value_states
        arena.kv_len, arena.pos_offset = kept, kv_seq_len - kept           # the tuple reports the full prompt length (:441)
        attn_output = self.o_proj(attn_output.reshape(bsz, q_len, -1).contiguous())
        return attn_output, arena.as_tuple()


def _prefill_attention(q, k, v, attention_mask, n_rep, is_causal):
    """Causal prompt attention; returns [B, L, N, hd] like the reference's flash-attention call (:106-114).
    `attention_mask` [B, L] of {0,1} marks left padding."""
    B, N, L, hd = q.shape
    if attention_mask is None or bool((attention_mask != 0).all()):
        out = F.scaled_dot_product_attention(q, k, v, is_causal=is_causal and L > 1, enable_gqa=n_rep > 1)
    else:
        keep = (attention_mask != 0)[:, None, None, :]
        causal = torch.ones(L, L, dtype=torch.bool, device=q.device).tril()[None, None]
        m = keep & causal
        m = m | torch.eye(L, dtype=torch.bool, device=q.device)[None, None]   # padded query rows: attend to self
        out = F.scaled_dot_product_attention(q, k, v, attn_mask=m, enable_gqa=n_rep > 1)
    return out.transpose(1, 2)


# ----------------------------------------------------------------------------- model shell
@dataclass
class CausalLMOutputWithPast:
    logits: torch.Tensor = None
    past_key_values: tuple = None


class PolarDecoderLayer(nn.Module):
    attention_class = PolarGroupAttention
    mixed_attention_class = None       # subclasses name their own variants; None falls back to the generic classes
    snapkv_attention_class = None

    def __init__(self, config, layer_idx):
        super().__init__()
        self.config, self.layer_idx = config, layer_idx
        self.hidden_size = config.hidden_size
        # config.vbits == 4 selects the Mixed variant (the reference switches by editing
        # modeling_llama_polar.py:452-453); anything else keeps half-precision values
        mixed = _cfg(config, "vbits", 16) == 4
        cls = (self.mixed_attention_class or PolarMixedGroupAttention) if mixed else self.attention_class
        if _cfg(config, "snapkv", False):       # the reference's third variant (modeling_llama_polar.py:454)
            cls = self.snapkv_attention_class or PolarSnapKVAttention
        self.self_attn = cls(config, layer_idx)
        self.mlp = MLP(config)
        self.input_layernorm = RMSNorm(config.hidden_size, config.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(config.hidden_size, config.rms_norm_eps)

    def forward(self, hidden_states, attention_mask=None, past_key_value=None, position_embeddings=None, **kwargs):
        """-> (hidden_states, present_key_value): pre-norm attention and MLP blocks, each added to its input
        (models/modeling_llama_polar.py:456-486)."""
        x = hidden_states
        attn_out, present = self.self_attn(hidden_states=self.input_layernorm(x), attention_mask=attention_mask,
                                           past_key_value=past_key_value, position_embeddings=position_embeddings, **kwargs)
        x = x + attn_out
        x = x + self.mlp(self.post_attention_layernorm(x))
        return x, present


class PolarModel(nn.Module):
    layer_class = PolarDecoderLayer

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.embed_tokens = nn.Embedding(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList([self.layer_class(config, i) for i in range(config.num_hidden_layers)])
        self.norm = RMSNorm(config.hidden_size, config.rms_norm_eps)
        head_dim = _cfg(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
        self.rotary_emb = RotaryEmbedding(head_dim, *rope_parameters(config))

    def forward(self, input_ids=None, attention_mask=None, past_key_values=None):
        """-> (normed hidden states, tuple of per-layer cache tuples).  Positions continue from the last slot of
        the first layer's cache tuple, the count of tokens seen so far (models/modeling_llama_polar.py:494-521);
        the 2-D padding mask is handed to the layers as it is."""
        n_seen = 0 if past_key_values is None else past_key_values[0][-1]
        x = self.embed_tokens(input_ids)
        positions = torch.arange(n_seen, n_seen + input_ids.shape[1], device=x.device).unsqueeze(0)
        rope = self.rotary_emb(x, positions)
        presents = []
        for i, layer in enumerate(self.layers):
            x, present = layer(x, attention_mask=attention_mask, position_embeddings=rope,
                               past_key_value=None if past_key_values is None else past_key_values[i])
            presents.append(present)
        return self.norm(x), tuple(presents)


class PolarForCausalLM(nn.Module):
    model_class = PolarModel

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.model = self.model_class(config)
        self.lm_head = nn.Linear(config.hidden_size, config.vocab_size, bias=False)
        if _cfg(config, "tie_word_embeddings", False):
            self.lm_head.weight = self.model.embed_tokens.weight

    @property
    def device(self):
        return next(self.parameters()).device

    @classmethod
    def from_pretrained(cls, path, torch_dtype=torch.bfloat16, device="cuda:0", **polar_options):
        """The model of a Hugging Face checkpoint directory (config.json + safetensors), as the reference's
        evaluation scripts obtain it (test4long.py:46-47); `polar_options`: PolarConfig's cache fields."""
        from .checkpoint import load_pretrained
        return load_pretrained(path, torch_dtype, device, model_class=cls, **polar_options)

    def forward(self, input_ids=None, attention_mask=None, past_key_values=None, num_logits_to_keep=0,
                return_dict=True):
        hidden_states, past_key_values = self.model(input_ids=input_ids, attention_mask=attention_mask,
                                                    past_key_values=past_key_values)
        logits = self.lm_head(hidden_states[:, -num_logits_to_keep:, :])
        return CausalLMOutputWithPast(logits=logits, past_key_values=past_key_values)

    def prepare_inputs_for_generation(self, input_ids, past_key_values=None, attention_mask=None, **kwargs):
        """The hook HF's `generate` calls (models/modeling_llama_polar.py:549-560): batch 1 only, the last token
        once a cache exists."""
        if input_ids.size(0) != 1:
            raise NotImplementedError
        return {"input_ids": input_ids[:, -1:] if past_key_values is not None else input_ids,
                "attention_mask": attention_mask, "past_key_values": past_key_values}

    def _prepare_cache_for_generation(self, *args, **kwargs):
        return None                      # the cache is this model's own tuple, never an HF cache object (:562-563)

    def kv_cache_bytes_per_token(self) -> int:
        """Bytes one cached token costs across all layers: 1 code byte per pair, 4 metadata
        halves per (group, pair) amortised over 128 tokens, fp16 V (or 4-bit V with config.vbits == 4)."""
        c = self.config
        nk = _cfg(c, "num_key_value_heads", c.num_attention_heads)
        v_bytes = 128 // 2 + 2 * 2 if _cfg(c, "vbits", 16) == 4 else 128 * 2      # 4-bit codes + half scale and zero-point
        code_bytes = 48 if _cfg(c, "packed_codes", False) else 64
        return c.num_hidden_layers * nk * (code_bytes + 4 * 64 * 2 // 128 + v_bytes)


# ----------------------------------------------------------------------------- generation (reference :565-666)
def top_k_top_p_filtering(logits, top_k: int = 0, top_p: float = 1.0, filter_value: float = -float("Inf"),
                          min_tokens_to_keep: int = 1):
    """Top-k, then nucleus filtering of [rows, vocab] logits, in place (models/modeling_llama_polar.py:565-588).
    Nucleus rule as the reference applies it: in descending order, a token is dropped when the probability mass up
    to and including its predecessor exceeds `top_p`, so the token that crosses the threshold survives; with
    `min_tokens_to_keep` > 1 the predecessors' verdicts of the first `min_tokens_to_keep` places are cleared first."""
    if top_k > 0:
        k = min(max(top_k, min_tokens_to_keep), logits.size(-1))
        kth_largest = logits.topk(k, dim=-1).values[..., -1:]
        logits.masked_fill_(logits < kth_largest, filter_value)
    if top_p < 1.0:
        order = logits.argsort(dim=-1, descending=True)
        over = logits.gather(-1, order).softmax(-1).cumsum(-1) > top_p
        if min_tokens_to_keep > 1:
            over[..., :min_tokens_to_keep] = False
        drop_sorted = torch.zeros_like(over)
        drop_sorted[..., 1:] = over[..., :-1]
        logits.masked_fill_(torch.zeros_like(over).scatter_(-1, order, drop_sorted), filter_value)
    return logits


def return_top_p_filtered_indices(logits, top_p):
    """Boolean mask over the vocabulary of [batch, positions, vocab] logits: True for the tokens nucleus filtering
    keeps, i.e. the most probable ones up to and including the one whose cumulative probability first exceeds
    `top_p` (models/modeling_llama_polar.py:592-606; no caller in the reference)."""
    order = logits.argsort(dim=-1, descending=True)
    over = logits.gather(-1, order).softmax(-1).cumsum(-1) > top_p
    keep_sorted = torch.ones_like(over)
    keep_sorted[..., 1:] = ~over[..., :-1]
    return torch.zeros_like(over).scatter_(-1, order, keep_sorted)


def sample(logits, generation_config, do_sample=False):
    if do_sample:
        logits_ = top_k_top_p_filtering(logits.view(-1, logits.size(-1)) / generation_config.temperature,
                                        top_k=generation_config.top_k, top_p=generation_config.top_p)
        return torch.multinomial(logits_.softmax(-1), num_samples=1)
    return torch.argmax(logits, dim=-1)


@dataclass
class GenerationConfig:
    eos_token_id: List[int] = field(default_factory=lambda: [2])
    top_k: int = 50
    top_p: float = 1.0
    temperature: float = 1.0


def generate(model, input_ids, attention_mask, generation_config, do_sample=False, max_new_tokens=8, graph_decoder=False):
    """The reference's decoding loop (models/modeling_llama_polar.py:622-666): prefill, then one token per step,
    the mask grown by a column of ones; stops early once every sequence has produced a stop token (sequences that
    stopped earlier keep producing tokens until then, as in the reference).  -> LongTensor [B, <= max_new_tokens].
    graph_decoder (not in the reference): the steps after the prompt replay a captured HIP graph on static state
    (`graph_decode.PolarGraphDecoder`) instead of driving the modules launch by launch; logits agree with the
    eager step to rounding, so a near-tie between two tokens may resolve differently."""
    dev = model.device
    n_seq = input_ids.size(0)
    stop_ids = generation_config.eos_token_id
    stop_ids = torch.as_tensor(stop_ids if isinstance(stop_ids, (list, tuple)) else [stop_ids], dtype=torch.long, device=dev)
    produced = torch.zeros((n_seq, max_new_tokens), dtype=torch.long, device=dev)
    finished = torch.zeros((n_seq, 1), dtype=torch.bool, device=dev)
    tokens, cache, n_out = input_ids, None, 0
    decoder = None
    if graph_decoder:
        from .graph_decode import PolarGraphDecoder
        decoder = PolarGraphDecoder(model, max_len=input_ids.size(1) + max_new_tokens + 1)
    with torch.no_grad():
        while n_out < max_new_tokens:
            if decoder is None:
                step_out = model(input_ids=tokens, attention_mask=attention_mask, past_key_values=cache, num_logits_to_keep=1)
                cache, logits = step_out.past_key_values, step_out.logits
            else:
                logits = decoder.prefill(tokens, attention_mask) if n_out == 0 else decoder.step(tokens)
            tokens = sample(logits, generation_config, do_sample=do_sample)
            produced[:, n_out:n_out + 1] = tokens
            n_out += 1
            if attention_mask is not None and decoder is None:
                attention_mask = torch.cat([attention_mask, torch.ones_like(tokens)], dim=-1)
            finished |= torch.isin(tokens, stop_ids)
            if bool(finished.all()):
                break
    return produced[:, :n_out]
