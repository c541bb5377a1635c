"""The un-quantized baseline of the end-to-end decode benchmark: the same model shells, weights, fused
elementwise and linear kernels and captured graph as `PolarGraphDecoder`, but with the keys and values
of every layer cached in the model dtype, which is what the reference's throughput script compares the
polar cache against (benchmark/benchmark_throughput.py:93-113 with the attention of
benchmark/models/modeling_llama_exp.py:39-54: softmax(q K^T / sqrt(d)) V over the whole fp16 cache).

Two attention kernels for that cache, both replayable from a graph (no per-step host state):

  "same_kernel"   this library's fused decode-attention kernel with NO quantized groups: the whole key
                  cache is handed over as its half-precision "residual" keys (q K^T on the matrix cores,
                  rounded to the model dtype as the reference's half-precision matmul output is), slices
                  cut on the device.  The strongest fp16 baseline here: one pass over 512 B per token
                  and KV head.
  "sdpa_splitk"   torch's fused attention (the memory-efficient kernel, which takes a bias) driven as a
                  split-K decode: the cache capacity is cut into S slices that become extra heads
                  (views, no copy), positions beyond the current length are masked by a bias buffer that
                  is refreshed on the device each step, and the S partial outputs are combined by their
                  log-sum-exp.

Benchmark code: nothing in the importable product uses this module.
"""
from __future__ import annotations

import math
from types import SimpleNamespace
from typing import Optional

import torch

from ..attention import _num_cus, new_workspace, polar_decode_attention
from ..graph_decode import PolarGraphDecoder
from ..modeling_common import CausalLMOutputWithPast, _prefill_attention, project_heads_and_rotate


class Fp16KVGraphDecoder(PolarGraphDecoder):
    def __init__(self, model, max_len: int, attention: str = "same_kernel", slices: int = 32, **kw):
        assert attention in ("same_kernel", "sdpa_splitk")
        # the split-K view needs a capacity that divides into `slices` pieces of a multiple of 64 rows
        unit = slices * 64
        max_len = -(-int(max_len) // unit) * unit
        super().__init__(model, max_len, **kw)
        self.attention, self.slices = attention, slices

    # ------------------------------------------------------------------ prompt
    @torch.no_grad()
    def prefill(self, input_ids: torch.Tensor, attention_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        assert attention_mask is None, "the baseline decoder takes unpadded prompts"
        from ..decode_ops import rmsnorm, silu_mul
        model, cfg = self.model, self.cfg
        m = model.model
        dev = input_ids.device
        B, L = input_ids.shape
        assert L + 1 <= self.max_len
        x = m.embed_tokens(input_ids).contiguous()
        dtype = x.dtype
        rope = m.rotary_emb(x, torch.arange(L, device=dev).unsqueeze(0))
        layers = m.layers
        self.arenas = []
        h = rmsnorm(x, layers[0].input_layernorm.weight, layers[0].input_layernorm.variance_epsilon)
        for li, layer in enumerate(layers):
            att = layer.self_attn
            Nk, hd = att.num_key_value_heads, att.head_dim
            v = att.v_proj(h).view(B, L, Nk, hd).transpose(1, 2)
            q, k = project_heads_and_rotate(att.q_proj(h), att.k_proj(h), *rope, att.num_heads, Nk, hd)
            a = _prefill_attention(q, k, v, None, att.num_key_value_groups, True)
            kc = torch.zeros(B, Nk, self.max_len, hd, dtype=dtype, device=dev)
            vc = torch.zeros(B, Nk, self.max_len, hd, dtype=dtype, device=dev)
            kc[:, :, :L] = k
            vc[:, :, :L] = v
            # what the step body reads of an arena: the tensor the new key goes to (row `resid_idx`) and the one the new
            # value goes to (row `pos`); here both are whole caches and both rows are the token's position
            self.arenas.append(SimpleNamespace(kres=kc, v=vc, Nk=Nk, dtype=dtype, kv_len=L, n_resid=L))
            del q, k, v
            a = att.o_proj(a.reshape(B, L, -1).contiguous())
            pn = layer.post_attention_layernorm
            h = rmsnorm(x, pn.weight, pn.variance_epsilon, residual=a, sum_out=x)
            y = layer.mlp.down_proj(silu_mul(layer.mlp.gate_proj(h), layer.mlp.up_proj(h)))
            nn_ = layers[li + 1].input_layernorm if li + 1 < len(layers) else m.norm
            h = rmsnorm(x, nn_.weight, nn_.variance_epsilon, residual=y, sum_out=x)
        logits = model.lm_head(h[:, -1:, :])
        self.B, self.kv_len, self.n_resid = B, L, L
        self.pos = torch.full((1,), L, dtype=torch.int64, device=dev)
        self.resid_idx = self.pos.clone()                      # the key's row is the position as well
        self.n_groups_dev = torch.zeros((B,), dtype=torch.int32, device=dev)
        self.n_resid_dev = torch.full((B,), L + 1, dtype=torch.int32, device=dev)     # keys INCLUDING the new one
        self.ids = torch.zeros((B, 1), dtype=torch.long, device=dev)
        self.mask8 = None
        inv_freq = m.rotary_emb.inv_freq.float().to(dev)
        ang = torch.arange(self.max_len, dtype=torch.float32, device=dev)[:, None] * inv_freq[None, :]
        emb = torch.cat([ang, ang], dim=-1)
        self.cos_table, self.sin_table = emb.cos().to(dtype), emb.sin().to(dtype)
        self.mixed = False
        N, Nk = cfg.num_attention_heads, self.arenas[0].Nk
        # slices cut on the device: a plane is 3 start-up units + one per 64 keys; partial slots for the pieces of the
        # longest plane at the segment length the device will choose
        tiles = -(-self.max_len // 64) + 3
        seg = max(1, -(-tiles * B * Nk // (4 * _num_cus(dev))))
        self.n_splits = -(-tiles // seg) + 2
        self.workspace = new_workspace(B, N, self.n_splits, dev)
        if self.attention == "sdpa_splitk":
            S, per = self.slices, self.max_len // self.slices
            self.col = torch.arange(self.max_len, device=dev).view(1, 1, S, 1, per)
            self.bias = torch.zeros(B, Nk * S, N // Nk, per, dtype=dtype, device=dev)
        self.logits = None
        self.graph = None
        self._fuse_qkv()
        return logits

    # ------------------------------------------------------------------ one token
    def _step_body(self):
        if self.attention == "sdpa_splitk":
            # positions up to and including the new token's are open, the rest of the capacity is closed; one small
            # launch per step, shared by all layers
            B, S = self.B, self.slices
            open_ = self.col <= self.pos
            self.bias.view(B, -1, S, self.bias.shape[2], self.bias.shape[3]).copy_(
                torch.where(open_, 0.0, -30000.0).to(self.bias.dtype).expand(B, self.bias.shape[1] // S, S, self.bias.shape[2], -1))
        return self._step_body_fused()

    def _attend(self, att, ar, q):
        B, N, Nk = self.B, att.num_heads, att.num_key_value_heads
        if self.attention == "same_kernel":
            return polar_decode_attention(q, None, None, None, None, None, ar.kres, ar.v, 0, 0, rbits=att.rbits, tbits=att.tbits,
                                          sm_scale=1.0 / math.sqrt(att.head_dim), n_groups_per_seq=self.n_groups_dev,
                                          n_resid_per_seq=self.n_resid_dev, n_splits=self.n_splits, balanced=True,
                                          workspace=self.workspace)
        S, rep = self.slices, N // Nk
        per = self.max_len // S
        k2, v2 = ar.kres.view(B, Nk * S, per, 128), ar.v.view(B, Nk * S, per, 128)
        q2 = q.view(B, Nk, 1, rep, 128).expand(B, Nk, S, rep, 128).reshape(B, Nk * S, rep, 128)
        o, lse = torch.ops.aten._scaled_dot_product_efficient_attention(q2, k2, v2, self.bias, True)[:2]
        wgt = torch.softmax(lse.view(B, Nk, S, rep).float(), dim=2)
        return (o.view(B, Nk, S, rep, 128).float() * wgt[..., None]).sum(2).to(q.dtype).view(B, N, 1, 128)

    def _flush(self):
        pass                                                   # nothing is ever quantized

    @torch.no_grad()
    def step(self, ids: torch.Tensor) -> torch.Tensor:
        logits = super().step(ids)
        self.n_resid = self.kv_len                             # the "window" is the whole cache and never fills
        return logits

    def cache(self):
        return tuple((ar.kres[:, :, :self.kv_len], ar.v[:, :, :self.kv_len], self.kv_len) for ar in self.arenas)
