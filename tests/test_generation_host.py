"""Host logic of the decoding loop (models/modeling_llama_polar.py:565-666 in the reference): top-k / nucleus
filtering against known answers and a plain-loop restatement, and the stopping rule of generate() against a
scripted stand-in model.  No GPU."""
import math
from types import SimpleNamespace

import pytest
import torch

from polarquant_amd.modeling_common import GenerationConfig, generate, sample, top_k_top_p_filtering


def _kept(logits):
    return [sorted(torch.nonzero(torch.isfinite(r)).flatten().tolist()) for r in logits]


def test_nucleus_keeps_the_token_that_crosses_the_threshold():
    probs = torch.tensor([[0.05, 0.5, 0.15, 0.3]])
    assert _kept(top_k_top_p_filtering(probs.log(), top_k=0, top_p=0.7)) == [[1, 3]]        # 0.5, then 0.3 crosses 0.7
    assert _kept(top_k_top_p_filtering(probs.log(), top_k=0, top_p=0.81)) == [[1, 2, 3]]    # 0.8 does not exceed 0.81
    assert _kept(top_k_top_p_filtering(probs.log(), top_k=0, top_p=0.4)) == [[1]]
    assert _kept(top_k_top_p_filtering(probs.log(), top_k=0, top_p=1.0)) == [[0, 1, 2, 3]]


def test_top_k_keeps_ties_with_the_kth_largest_and_clamps_k():
    logits = torch.tensor([[1.0, 3.0, 2.0, 2.0, 0.0]])
    assert _kept(top_k_top_p_filtering(logits.clone(), top_k=2)) == [[1, 2, 3]]      # both 2.0 are "not smaller than the 2nd"
    assert _kept(top_k_top_p_filtering(logits.clone(), top_k=1)) == [[1]]
    assert _kept(top_k_top_p_filtering(logits.clone(), top_k=50)) == [[0, 1, 2, 3, 4]]
    assert _kept(top_k_top_p_filtering(logits.clone(), top_k=1, min_tokens_to_keep=3)) == [[1, 2, 3]]


def _loop_restatement(row, top_k, top_p, min_keep):
    keep = set(range(len(row)))
    if top_k > 0:
        k = min(max(top_k, min_keep), len(row))
        kth = sorted(row, reverse=True)[k - 1]
        keep = {i for i in keep if not row[i] < kth}
    if top_p < 1.0:
        vals = [row[i] if i in keep else -math.inf for i in range(len(row))]
        order = sorted(range(len(row)), key=lambda i: -vals[i])
        m = max(vals)
        z = sum(math.exp(v - m) for v in vals)
        cum, over = 0.0, []
        for i in order:
            cum += math.exp(vals[i] - m) / z
            over.append(cum > top_p)
        if min_keep > 1:
            for j in range(min_keep):
                over[j] = False
        for pos, i in enumerate(order):
            if pos > 0 and over[pos - 1]:
                keep.discard(i)
    return sorted(keep)


@pytest.mark.parametrize("top_k,top_p,min_keep", [(0, 0.9, 1), (5, 0.5, 1), (3, 1.0, 1), (8, 0.3, 4), (0, 0.05, 2)])
def test_filtering_against_a_plain_loop(top_k, top_p, min_keep):
    g = torch.Generator().manual_seed(top_k * 100 + int(top_p * 10))
    logits = torch.randn(6, 17, generator=g, dtype=torch.float64) * 2
    want = [_loop_restatement(r.tolist(), top_k, top_p, min_keep) for r in logits]
    got = top_k_top_p_filtering(logits.clone(), top_k=top_k, top_p=top_p, min_tokens_to_keep=min_keep)
    assert _kept(got) == want
    assert torch.equal(got[torch.isfinite(got)], logits[torch.isfinite(got)])       # survivors keep their values


def test_sample_greedy_and_filtered():
    logits = torch.tensor([[[0.0, 5.0, 1.0]], [[2.0, 0.0, -1.0]]])
    assert sample(logits, GenerationConfig(), do_sample=False).tolist() == [[1], [0]]
    torch.manual_seed(0)
    cfg = GenerationConfig(top_k=1)
    for _ in range(5):      # top_k = 1 leaves one candidate: sampling is then greedy
        assert sample(logits.clone(), cfg, do_sample=True).tolist() == [[1], [0]]


class _Scripted:
    """Stand-in model: sequence b produces script[b][step]; records what generate() passes in."""
    device = torch.device("cpu")

    def __init__(self, script, vocab=10):
        self.script, self.vocab, self.calls = script, vocab, []

    def __call__(self, input_ids, attention_mask, past_key_values, num_logits_to_keep):
        step = 0 if past_key_values is None else past_key_values
        self.calls.append((tuple(input_ids.shape), None if attention_mask is None else tuple(attention_mask.shape), num_logits_to_keep))
        logits = torch.zeros(len(self.script), 1, self.vocab)
        for b, row in enumerate(self.script):
            logits[b, 0, row[step]] = 1.0
        return SimpleNamespace(logits=logits, past_key_values=step + 1)


def test_generate_stops_when_every_sequence_has_stopped_and_keeps_the_stop_token():
    model = _Scripted([[3, 9, 4, 4, 4, 4], [5, 6, 7, 9, 1, 1]])
    out = generate(model, torch.zeros(2, 4, dtype=torch.long), torch.ones(2, 4, dtype=torch.long),
                   GenerationConfig(eos_token_id=[9]), max_new_tokens=6)
    # sequence 0 stops at step 1 and keeps producing; sequence 1 stops at step 3: four columns come back
    assert out.tolist() == [[3, 9, 4, 4], [5, 6, 7, 9]]
    assert model.calls[0] == ((2, 4), (2, 4), 1) and model.calls[1] == ((2, 1), (2, 5), 1) and model.calls[3][1] == (2, 7)


def test_generate_runs_to_the_limit_without_a_stop_token_and_accepts_a_scalar_eos():
    model = _Scripted([[1, 2, 3, 4]])
    out = generate(model, torch.zeros(1, 2, dtype=torch.long), None, GenerationConfig(eos_token_id=7), max_new_tokens=3)
    assert out.tolist() == [[1, 2, 3]] and len(model.calls) == 3 and model.calls[2][1] is None
    assert generate(model, torch.zeros(1, 2, dtype=torch.long), None, GenerationConfig(), max_new_tokens=0).shape == (1, 0)


def test_hf_generation_hook_is_batch_one_and_feeds_the_last_token():
    from polarquant_amd.modeling_common import PolarForCausalLM
    hook = PolarForCausalLM.prepare_inputs_for_generation
    ids = torch.arange(6).view(1, 6)
    first = hook(None, ids, None, torch.ones(1, 6))
    assert first["input_ids"] is ids and first["past_key_values"] is None
    later = hook(None, ids, past_key_values=("cache",), attention_mask=None)
    assert later["input_ids"].tolist() == [[5]] and later["past_key_values"] == ("cache",)
    with pytest.raises(NotImplementedError):
        hook(None, torch.zeros(2, 3, dtype=torch.long))
    assert PolarForCausalLM._prepare_cache_for_generation(None, 1, 2, 3) is None


def test_top_p_keep_mask_matches_the_filter():
    from polarquant_amd.modeling_common import return_top_p_filtered_indices
    probs = torch.tensor([[[0.05, 0.5, 0.15, 0.3], [0.25, 0.25, 0.4, 0.1]]])
    keep = return_top_p_filtered_indices(probs.log(), 0.7)
    assert keep.dtype == torch.bool and keep.tolist() == [[[False, True, False, True], [True, True, True, False]]]
    g = torch.Generator().manual_seed(4)
    logits = torch.randn(2, 3, 19, generator=g, dtype=torch.float64)
    keep = return_top_p_filtered_indices(logits, 0.6)
    filtered = top_k_top_p_filtering(logits.reshape(-1, 19).clone(), top_k=0, top_p=0.6).reshape(2, 3, 19)
    assert torch.equal(keep, torch.isfinite(filtered))


def test_padding_mask_conversion_is_not_fooled_by_a_recycled_address():
    """The uint8 form of the step's attention mask is cached across the layers of one step.  `generate` builds a
    fresh mask tensor per step, and an allocator hands a freed block of the same size straight back: two masks of
    the same shape and address with different padding must each get their own conversion."""
    from polarquant_amd.modeling_common import _mask_u8
    shape = (4, 333)
    first = torch.ones(shape, dtype=torch.int64)
    first[:, :100] = 0
    u_first = _mask_u8(first)
    assert torch.equal(u_first, (first != 0).to(torch.uint8))
    assert _mask_u8(first) is u_first                    # same tensor, same step: converted once
    addr = first.data_ptr()
    recycled = 0
    for pad in (7, 50, 200, 13):
        del first
        first = torch.ones(shape, dtype=torch.int64)     # usually lands on the block just freed
        first[:, :pad] = 0
        recycled += first.data_ptr() == addr
        addr = first.data_ptr()
        assert torch.equal(_mask_u8(first), (first != 0).to(torch.uint8)), pad
    # an in-place edit of the same tensor is seen through its version counter
    first[:, :300] = 0
    assert torch.equal(_mask_u8(first), (first != 0).to(torch.uint8))
    # a uint8 mask passes through untouched
    m8 = torch.ones(shape, dtype=torch.uint8)
    assert _mask_u8(m8) is m8 and _mask_u8(None) is None


def test_the_attention_class_refuses_a_head_dim_the_kernels_are_not_built_for():
    """head_dim is fixed at 128 in the C ABI (PQ_HEAD_DIM); the drop-in classes say so when they are constructed
    instead of failing inside a launch."""
    from polarquant_amd.modeling_common import PolarConfig, PolarGroupAttention
    cfg = PolarConfig(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, num_hidden_layers=1,
                      intermediate_size=128, vocab_size=64, head_dim=64)
    with pytest.raises(ValueError, match="head_dim 128"):
        PolarGroupAttention(cfg, 0)
    PolarGroupAttention(PolarConfig(hidden_size=256, num_attention_heads=2, num_key_value_heads=1, num_hidden_layers=1,
                                    intermediate_size=128, vocab_size=64), 0)
