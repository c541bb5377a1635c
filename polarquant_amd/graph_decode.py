"""Decode loop captured in a HIP graph.

The reference's decode step is ~40 eager launches per layer driven from Python
(models/modeling_llama_polar.py:61-101, 456-521, 622-666); at batch 8 and a 16k context that
is ~14 ms of launch overhead per token against ~5 ms of GPU work.  `PolarGraphDecoder` runs
the same step — same modules, same weights, same cache arena, same kernels — but with every
per-step scalar (position, residual fill, cache length) held in device memory, so that the
whole step is one captured graph that is replayed per token.  Steps that flush the residual
window into the quantized cache (one in 128) run eagerly.

    dec = PolarGraphDecoder(model, max_len)
    logits = dec.prefill(input_ids)            # eager prompt pass, builds the cache
    for _ in range(n):
        logits = dec.step(next_ids)            # [B, 1, vocab]; graph replay

Left-padding masks are not handled here (use the eager `generate` for padded batches).
"""
from __future__ import annotations

import math
from typing import List, Optional

import torch

from . import _ffi
from .attention import _num_cus, new_workspace, plan_splits, polar_decode_attention, polar_decode_attention_v4
from .modeling_common import GROUP, apply_rotary_pos_emb


class PolarGraphDecoder:
    def __init__(self, model, max_len: int, use_graph: bool = True, fused_ops: bool = True, small_m_gemm: bool = True,
                 fused_prefill: bool = False, fused_qkv_rope: bool = True):
        """fused_ops: run RoPE + cache append, the norms and the MLP activation as one HIP launch each
        (polarquant_amd.decode_ops) instead of the eager modules' chains of elementwise launches.  The
        rotation is bit-identical to the eager ops; the norms and SiLU agree to the dtype's last bit.
        small_m_gemm (with fused_ops, batch <= 16): o_proj, gate/up (with the SiLU product in its epilogue) and
        down_proj through the weight-streaming kernel `decode_ops.linear_small_m` instead of the BLAS library;
        fp32 accumulation in a different order, so logits agree to rounding.
        fused_qkv_rope (with small_m_gemm, batch <= 8): the q|k|v projection, the rotation and the two cache
        appends as one launch, `decode_ops.qkv_rope_append`, bit-identical to the projection followed by the rotation.
        fused_prefill: the prompt pass runs the norms and the MLP activation through the same fused kernels
        instead of the eager modules' elementwise chains (about a sixth of the prompt time); the cache it
        builds and the logits then agree with the eager model to rounding instead of bit for bit."""
        self.fused_ops = fused_ops
        self.small_m_gemm = small_m_gemm
        self.fused_prefill = fused_prefill
        self.fused_qkv_rope = fused_qkv_rope
        self.model = model
        self.cfg = model.config
        self.max_len = int(max_len)
        self.use_graph = use_graph
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.arenas: List = []
        self.kv_len = 0          # host mirrors of the device counters (uniform batch)
        self.n_resid = 0

    # ------------------------------------------------------------------ prompt
    @torch.no_grad()
    def prefill(self, input_ids: torch.Tensor, attention_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        """attention_mask [B, L] of {0, 1}: left padding of the prompt, as the reference's loop takes it
        (models/modeling_llama_polar.py:622-656); the new tokens are always attended to."""
        model, cfg = self.model, self.cfg
        dev = input_ids.device
        B, L = input_ids.shape
        assert L + 1 <= self.max_len
        old = getattr(cfg, "cache_capacity", 0)
        cfg.cache_capacity = self.max_len          # arenas never grow: their addresses are baked into the graph
        try:
            if self.fused_prefill:
                out = self._prefill_fused(input_ids, attention_mask)
            else:
                out = model(input_ids=input_ids, attention_mask=attention_mask, past_key_values=None, num_logits_to_keep=1)
        finally:
            cfg.cache_capacity = old
        self.arenas = [c.arena for c in out.past_key_values]
        a0 = self.arenas[0]
        assert a0.pos_offset == 0, "prompt eviction (SnapKV) is not handled by the graph decoder"
        self.B, self.kv_len, self.n_resid = B, a0.kv_len, a0.n_resid
        dtype = a0.dtype
        # device-side step state
        self.pos = torch.full((1,), self.kv_len, dtype=torch.int64, device=dev)           # position of the next token
        self.resid_idx = torch.full((1,), self.n_resid, dtype=torch.int64, device=dev)    # residual slot to write
        self.n_groups_dev = torch.full((B,), a0.n_groups, dtype=torch.int32, device=dev)
        self.n_resid_dev = torch.full((B,), self.n_resid + 1, dtype=torch.int32, device=dev)  # count INCLUDING the new key
        self.ids = torch.zeros((B, 1), dtype=torch.long, device=dev)
        # static mask over the whole capacity: the prompt's padding, ones for every later position (the
        # kernels read only the columns of tokens that exist, so nothing has to be updated per step)
        self.mask8 = None
        if attention_mask is not None:
            self.mask8 = torch.ones((B, self.max_len), dtype=torch.uint8, device=dev)
            self.mask8[:, :L] = (attention_mask != 0).to(torch.uint8)
        inv_freq = model.model.rotary_emb.inv_freq.float().to(dev)       # same table the eager step multiplies by
        ang = torch.arange(self.max_len, dtype=torch.float32, device=dev)[:, None] * inv_freq[None, :]
        emb = torch.cat([ang, ang], dim=-1)
        self.cos_table, self.sin_table = emb.cos().to(dtype), emb.sin().to(dtype)
        nk = a0.Nk
        self.mixed = hasattr(a0, "vcodes")          # Mixed variant: 4-bit values, shared residual window
        if self.mixed:
            self.n_splits = _ffi.lib().pq_decode_attn_v4_plan(B, cfg.num_attention_heads, nk, max(self.max_len // GROUP, 1), _num_cus(dev))
        else:
            self.n_splits = plan_splits(B, nk, max(self.max_len // GROUP, 1), dev)
        # the captured graph keeps this buffer's address: the decoder owns it, so that no other call can replace it
        self.workspace = new_workspace(B, cfg.num_attention_heads, self.n_splits, dev)
        self.logits = None
        self.graph = None
        if self.fused_ops:
            self._fuse_qkv()
        return out.logits

    def _prefill_fused(self, input_ids, attention_mask):
        """The model's prompt pass with one launch per norm (residual add folded in) and per SiLU * up."""
        from .decode_ops import rmsnorm, silu_mul
        from .modeling_common import CausalLMOutputWithPast
        m = self.model.model
        layers = m.layers
        x = m.embed_tokens(input_ids).contiguous()
        positions = torch.arange(input_ids.shape[1], device=x.device).unsqueeze(0)
        rope = m.rotary_emb(x, positions)
        presents = []
        h = rmsnorm(x, layers[0].input_layernorm.weight, layers[0].input_layernorm.variance_epsilon)
        for li, layer in enumerate(layers):
            a, present = layer.self_attn(hidden_states=h, attention_mask=attention_mask, past_key_value=None,
                                         position_embeddings=rope)
            presents.append(present)
            pn = layer.post_attention_layernorm
            h = rmsnorm(x, pn.weight, pn.variance_epsilon, residual=a.contiguous(), sum_out=x)
            mlp = layer.mlp
            if mlp.gate_proj.bias is None and mlp.up_proj.bias is None:
                y = mlp.down_proj(silu_mul(mlp.gate_proj(h), mlp.up_proj(h)))
            else:
                y = mlp(h)
            nn_ = layers[li + 1].input_layernorm if li + 1 < len(layers) else m.norm
            h = rmsnorm(x, nn_.weight, nn_.variance_epsilon, residual=y, sum_out=x)
        return CausalLMOutputWithPast(logits=self.model.lm_head(h[:, -1:, :]), past_key_values=tuple(presents))

    def _fuse_qkv(self):
        """One projection GEMM instead of three per layer: the q/k/v weights are concatenated once and the
        modules' own parameters re-pointed at slices of the fused tensor (no extra memory; the eager
        modules keep working).  At batch 8 the three small GEMMs are latency-bound (~15 us each whatever
        their size); fused they take about the time of one."""
        for layer in self.model.model.layers:
            att = layer.self_attn
            if getattr(att, "_wqkv", None) is not None:
                continue
            ws = [att.q_proj.weight, att.k_proj.weight, att.v_proj.weight]
            w = torch.cat([p.data for p in ws], dim=0)
            o = 0
            for p in ws:
                n = p.shape[0]
                p.data = w[o:o + n]
                o += n
            att._wqkv, att._bqkv = w, None
            if att.q_proj.bias is not None:
                bs = [att.q_proj.bias, att.k_proj.bias, att.v_proj.bias]
                b = torch.cat([p.data for p in bs], dim=0)
                o = 0
                for p in bs:
                    n = p.shape[0]
                    p.data = b[o:o + n]
                    o += n
                att._bqkv = b

    # ------------------------------------------------------------------ one token
    def _attend(self, att, ar, q):
        common = dict(rbits=att.rbits, tbits=att.tbits, sm_scale=1.0 / math.sqrt(att.head_dim),
                      n_groups_per_seq=self.n_groups_dev, n_resid_per_seq=self.n_resid_dev, n_splits=self.n_splits,
                      attention_mask=self.mask8, workspace=self.workspace)
        if self.mixed:
            return polar_decode_attention_v4(q, ar.codes, *ar.meta, ar.kres, ar.vres, ar.vcodes, *ar.vmeta, 0, 0, **common)
        return polar_decode_attention(q, ar.codes, *ar.meta, ar.kres, ar.v, 0, 0, **common)

    def _step_body_fused(self):
        """The decode step with one launch per elementwise stage: 2 norms (each with the residual add
        folded in), RoPE + append, SiLU * up, plus the GEMMs and the attention, per layer."""
        from .decode_ops import linear_small_m, qkv_rope_append, rmsnorm, rope_append, silu_mul
        model, B = self.model, self.B
        layers = model.model.layers
        x = model.model.embed_tokens(self.ids).contiguous()                 # residual stream [B,1,H], updated in place
        h = rmsnorm(x, layers[0].input_layernorm.weight, layers[0].input_layernorm.variance_epsilon)
        for li, (layer, ar) in enumerate(zip(layers, self.arenas)):
            att, mlp = layer.self_attn, layer.mlp
            nq, nkv = att.num_heads * att.head_dim, att.num_key_value_heads * att.head_dim
            own = self.small_m_gemm and B <= 16 and all(
                w_.is_contiguous() and w_.shape[0] % 16 == 0 and w_.shape[1] % 32 == 0
                for w_ in (att._wqkv, att.o_proj.weight, mlp.gate_proj.weight, mlp.up_proj.weight, mlp.down_proj.weight))
            v_dst, v_row = (ar.vres, self.resid_idx) if self.mixed else (ar.v, self.pos)
            if own and self.fused_qkv_rope and B <= 8 and att._wqkv.shape[1] % 64 == 0:
                # projection, rotation and both appends in one launch (bit-identical to the two below)
                q = qkv_rope_append(h, att._wqkv, att._bqkv, self.cos_table, self.sin_table, self.pos, ar.kres,
                                    self.resid_idx, v_dst, v_row, att.num_heads, att.num_key_value_heads)
            else:
                if own:
                    qkv = linear_small_m(h, att._wqkv, att._bqkv)               # [B,1,(N+2Nk)*128]
                else:
                    qkv = torch.nn.functional.linear(h, att._wqkv, att._bqkv)
                q_lin, k_lin, v_lin = qkv[..., :nq], qkv[..., nq:nq + nkv], qkv[..., nq + nkv:]
                q = rope_append(q_lin, k_lin, v_lin, self.cos_table, self.sin_table, self.pos, ar.kres, self.resid_idx,
                                v_dst, v_row, att.num_heads, att.num_key_value_heads)
            o = self._attend(att, ar, q)
            pn = layer.post_attention_layernorm
            if own and mlp.gate_proj.bias is None and mlp.up_proj.bias is None:
                a = linear_small_m(o.reshape(B, 1, -1), att.o_proj.weight, att.o_proj.bias)
                h = rmsnorm(x, pn.weight, pn.variance_epsilon, residual=a, sum_out=x)
                act = linear_small_m(h, mlp.gate_proj.weight, up_weight=mlp.up_proj.weight)
                m = linear_small_m(act, mlp.down_proj.weight, mlp.down_proj.bias)
            else:
                a = att.o_proj(o.reshape(B, 1, -1))
                h = rmsnorm(x, pn.weight, pn.variance_epsilon, residual=a, sum_out=x)
                # (gate | up as one library GEMM was measured too: no faster than the two, so they stay separate)
                m = mlp.down_proj(silu_mul(mlp.gate_proj(h), mlp.up_proj(h)))
            nn_ = layers[li + 1].input_layernorm if li + 1 < len(layers) else model.model.norm
            h = rmsnorm(x, nn_.weight, nn_.variance_epsilon, residual=m, sum_out=x)
        logits = model.lm_head(h)
        self.pos.add_(1)
        self.resid_idx.add_(1)
        self.n_resid_dev.add_(1)
        return logits

    def _step_body(self):
        """The decode step on the static state; identical arithmetic to the eager modules."""
        if self.fused_ops:
            return self._step_body_fused()
        model = self.model
        x = model.model.embed_tokens(self.ids)
        cos = self.cos_table.index_select(0, self.pos).unsqueeze(0)        # [1,1,128]
        sin = self.sin_table.index_select(0, self.pos).unsqueeze(0)
        B = self.B
        for layer, ar in zip(model.model.layers, self.arenas):
            att = layer.self_attn
            h = layer.input_layernorm(x)
            q = att.q_proj(h).view(B, 1, att.num_heads, att.head_dim).transpose(1, 2)
            k = att.k_proj(h).view(B, 1, att.num_key_value_heads, att.head_dim).transpose(1, 2)
            v = att.v_proj(h).view(B, 1, att.num_key_value_heads, att.head_dim).transpose(1, 2)
            q, k = apply_rotary_pos_emb(q, k, cos, sin)
            ar.kres.index_copy_(2, self.resid_idx, k)
            if self.mixed:
                ar.vres.index_copy_(2, self.resid_idx, v)
                o = polar_decode_attention_v4(q, ar.codes, *ar.meta, ar.kres, ar.vres, ar.vcodes, *ar.vmeta, 0, 0,
                                              rbits=att.rbits, tbits=att.tbits, sm_scale=1.0 / math.sqrt(att.head_dim),
                                              n_groups_per_seq=self.n_groups_dev, n_resid_per_seq=self.n_resid_dev,
                                              n_splits=self.n_splits, attention_mask=self.mask8, workspace=self.workspace)
            else:
                ar.v.index_copy_(2, self.pos, v)
                o = polar_decode_attention(q, ar.codes, *ar.meta, ar.kres, ar.v, 0, 0, rbits=att.rbits, tbits=att.tbits,
                                           sm_scale=1.0 / math.sqrt(att.head_dim), n_groups_per_seq=self.n_groups_dev,
                                           n_resid_per_seq=self.n_resid_dev, n_splits=self.n_splits, attention_mask=self.mask8,
                                           workspace=self.workspace)
            x = x + att.o_proj(o.reshape(B, 1, -1))
            x = x + layer.mlp(layer.post_attention_layernorm(x))
        logits = model.lm_head(model.model.norm(x))
        # advance the device-side counters for the next token
        self.pos.add_(1)
        self.resid_idx.add_(1)
        self.n_resid_dev.add_(1)
        return logits

    def _flush(self):
        """Residual window full (128 keys): quantize it into the next group slot (reference :83-92)."""
        for ar in self.arenas:
            ar.n_resid, ar.kv_len = GROUP, self.kv_len
            if self.mixed:
                ar.flush()
            else:
                ar.quantize_into(ar.kres)
                ar.n_resid = 0
        self.n_resid = 0
        self.resid_idx.zero_()
        self.n_groups_dev.add_(1)
        self.n_resid_dev.fill_(1)

    @torch.no_grad()
    def step(self, ids: torch.Tensor) -> torch.Tensor:
        assert self.kv_len + 1 <= self.max_len, "cache capacity exhausted"
        self.ids.copy_(ids.view(self.B, 1))
        if self.use_graph:
            if self.graph is None:
                # warm up on a side stream (lazy library initialisation must not be captured), then capture;
                # the warm-up steps advance the counters, so they are put back before and after
                state = [t.clone() for t in (self.pos, self.resid_idx, self.n_resid_dev)]
                s = torch.cuda.Stream()
                s.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(s):
                    self._step_body()
                torch.cuda.current_stream().wait_stream(s)
                for t, v in zip((self.pos, self.resid_idx, self.n_resid_dev), state):
                    t.copy_(v)
                self.graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(self.graph):
                    self.logits = self._step_body()
                for t, v in zip((self.pos, self.resid_idx, self.n_resid_dev), state):
                    t.copy_(v)
            self.graph.replay()
            logits = self.logits
        else:
            logits = self._step_body()
        self.kv_len += 1
        self.n_resid += 1
        for ar in self.arenas:
            ar.kv_len, ar.n_resid = self.kv_len, self.n_resid
        if self.n_resid == GROUP:
            self._flush()
        return logits

    def cache(self):
        """The reference-format cache tuples of the current state (one per layer)."""
        return tuple(ar.as_tuple() for ar in self.arenas)
