"""Parity at the full sizes of the benchmark configurations (configs[1], [2], [3]).

The CPU oracle cannot chew through a gigabyte of cache in seconds, so each
full-size case combines (a) the oracle on whole (sequence, KV head) planes picked
from the full problem, and (b) size-independent properties of the full result:
invariance to the context split, to the batch order, chunked == one-shot
quantization, per-sequence == batched for ragged batches.
"""
import math

import pytest
import torch

import bench
from oracle import polar_oracle as po
from polarquant_amd.attention import polar_decode_attention
from polarquant_amd.quantize import quantize_and_pack_nbit

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-2, 1e-3


def _ok(got, ref):
    err = (got.double() - ref.double()).abs()
    return bool((err <= ATOL + RTOL * ref.double().abs()).all()), float(err.max())


def _attn(w, **kw):
    sh = w["shape"]
    args = dict(rbits=sh.rbits, tbits=sh.tbits, n_groups_per_seq=w["groups_per_seq"], n_resid_per_seq=w["resid_per_seq"])
    args.update(kw)
    return polar_decode_attention(w["q"], w["codes"], *w["meta"], w["kres"], w["v"], w["n_groups"], w["n_resid"], **args)


def _oracle_plane(w, b, kvh, n_groups, n_resid):
    """fp64 oracle attention for the `rep` query heads of one (sequence, KV head) plane."""
    sh = w["shape"]
    rep = sh.n_heads // sh.n_kv_heads
    q = w["q"][b:b + 1, kvh * rep:(kvh + 1) * rep].cpu()
    quant = (None,) * 5
    if n_groups:
        quant = [w["codes"][b:b + 1, kvh:kvh + 1, :n_groups].cpu()] + [m[b:b + 1, kvh:kvh + 1, :n_groups].cpu() for m in w["meta"]]
    kres = w["kres"][b:b + 1, kvh:kvh + 1, :n_resid].cpu() if n_resid else None
    v = w["v"][b:b + 1, kvh:kvh + 1, :n_groups * 128 + n_resid].cpu()
    return po.decode_attention_exact(q, kres, *quant, v, None, sh.rbits, sh.tbits)


def test_cfg1_full_size(gpu):
    """configs[1]: batch 16, 32 q / 8 KV heads, context 32768, 4/4 bits."""
    print("building configs[1]", flush=True)
    w = bench.build_workload(1, gpu)
    sh = w["shape"]
    rep = sh.n_heads // sh.n_kv_heads
    out = _attn(w).clone()
    torch.cuda.synchronize()
    assert out.shape == (16, 32, 1, 128) and torch.isfinite(out.float()).all()
    # (a) oracle on three whole planes
    for b, kvh in [(0, 0), (7, 3), (15, 7)]:
        ref = _oracle_plane(w, b, kvh, w["n_groups"], w["n_resid"])
        ok, err = _ok(out[b:b + 1, kvh * rep:(kvh + 1) * rep].cpu(), ref)
        print("plane", b, kvh, "max abs err %.2e" % err, flush=True)
        assert ok
    # (b) the context split must not matter
    for ns in (5, 16, 64):
        other = _attn(w, n_splits=ns)
        ok, err = _ok(other.cpu(), out.cpu())
        assert ok, (ns, err)
    # (c) reversing the batch reverses the output, bit for bit
    flip = lambda t: t.flip(0).contiguous()
    w2 = dict(w, q=flip(w["q"]), codes=flip(w["codes"]), meta=[flip(m) for m in w["meta"]], kres=flip(w["kres"]), v=flip(w["v"]))
    assert torch.equal(_attn(w2).flip(0), out)
    # (d) masking all but the last 1000 tokens == attention over that suffix alone (oracle on one plane)
    L = w["n_groups"] * 128 + w["n_resid"]
    mask = torch.zeros(16, L, dtype=torch.uint8, device=gpu)
    mask[:, -1000:] = 1
    om = _attn(w, attention_mask=mask)
    b, kvh = 3, 5
    qq = w["q"][b:b + 1, kvh * rep:(kvh + 1) * rep].cpu()
    quant = [w["codes"][b:b + 1, kvh:kvh + 1].cpu()] + [m[b:b + 1, kvh:kvh + 1].cpu() for m in w["meta"]]
    ref = po.decode_attention_exact(qq, w["kres"][b:b + 1, kvh:kvh + 1, :1].cpu(), *quant, w["v"][b:b + 1, kvh:kvh + 1].cpu(),
                                    mask[b:b + 1].cpu(), sh.rbits, sh.tbits)
    ok, err = _ok(om[b:b + 1, kvh * rep:(kvh + 1) * rep].cpu(), ref)
    assert ok, err


def test_cfg2_full_size_ragged(gpu):
    """configs[2]: batch 64, 28 q / 4 KV heads (GQA 7), 3/3 bits, per-sequence lengths in [512, 8192]."""
    print("building configs[2]", flush=True)
    w = bench.build_workload(2, gpu)
    sh = w["shape"]
    lens = w["lengths"]
    assert int(lens.min()) >= 512 and int(lens.max()) <= 8192
    out = _attn(w).clone()
    torch.cuda.synchronize()
    assert out.shape == (64, 28, 1, 128) and torch.isfinite(out.float()).all()
    # (a) oracle on whole planes of the shortest, the longest and two other sequences
    order = torch.argsort(lens)
    for b in [int(order[0]), int(order[-1]), int(order[20]), int(order[41])]:
        ng, nr = int(lens[b]) // 128, int(lens[b]) % 128
        for kvh in (0, 3):
            ref = _oracle_plane(w, b, kvh, ng, nr)
            ok, err = _ok(out[b:b + 1, kvh * 7:(kvh + 1) * 7].cpu(), ref)
            print("seq", b, "len", int(lens[b]), "kvh", kvh, "max abs err %.2e" % err, flush=True)
            assert ok
    # (b) every sequence alone (batch of one, uniform counts) == its row in the ragged batch
    for b in [int(order[1]), int(order[33]), int(order[-2])]:
        ng, nr = int(lens[b]) // 128, int(lens[b]) % 128
        alone = polar_decode_attention(w["q"][b:b + 1], w["codes"][b:b + 1], *[m[b:b + 1] for m in w["meta"]],
                                       w["kres"][b:b + 1], w["v"][b:b + 1], ng, nr, rbits=3, tbits=3)
        ok, err = _ok(alone.cpu(), out[b:b + 1].cpu())
        assert ok, err
    # (c) split invariance
    ok, err = _ok(_attn(w, n_splits=7).cpu(), out.cpu())
    assert ok, err


def test_cfg3_full_size_append_and_decode(gpu):
    """configs[3]: batch 1, context 131072: quantize all prompt keys, then one decode step."""
    print("building configs[3]", flush=True)
    w = bench.build_workload(3, gpu, keep_keys=True)
    sh = w["shape"]
    k = w["keys"]                                            # [1,8,131072,128] fp16 on the GPU
    assert k.shape == (1, 8, 131072, 128)
    codes, meta = w["codes"], w["meta"]
    assert int(codes.max()) <= 255
    # (a) append: oracle, bit for bit, on group ranges spread over heads and positions
    for kvh, g0, n in [(0, 0, 8), (3, 500, 8), (7, 1016, 8), (5, 257, 3)]:
        ref = po.quantize_and_pack_nbit(k[:, kvh:kvh + 1, g0 * 128:(g0 + n) * 128].cpu(), 4, 4)
        assert torch.equal(codes[:, kvh:kvh + 1, g0:g0 + n].cpu(), ref[0])
        for m, r in zip(meta, ref[1:]):
            assert bool((m[:, kvh:kvh + 1, g0:g0 + n].cpu().float() == r.float()).all())
    # (b) chunked append (one group at a time into a cache slot, as decode does) == one-shot, via checksums
    kvh = 2
    one = quantize_and_pack_nbit(k[:, kvh:kvh + 1], 4, 4)
    slot = (torch.zeros_like(one[0]), *[torch.zeros_like(m) for m in one[1:]])
    for g in range(0, 1024, 97):
        quantize_and_pack_nbit(k[:, kvh:kvh + 1, g * 128:(g + 1) * 128], 4, 4, out=slot, group_offset=g)
        assert torch.equal(slot[0][:, :, g], one[0][:, :, g])
    assert int(one[0].long().sum()) == int(codes[:, kvh].long().sum())
    # (c) decode over the whole cache: oracle on two planes, and split invariance
    out = _attn(w).clone()
    for kvh in (1, 6):
        ref = _oracle_plane(w, 0, kvh, w["n_groups"], w["n_resid"])
        ok, err = _ok(out[:, kvh * 4:(kvh + 1) * 4].cpu(), ref)
        print("cfg3 plane", kvh, "max abs err %.2e" % err, flush=True)
        assert ok
    for ns in (64, 333):
        ok, err = _ok(_attn(w, n_splits=ns).cpu(), out.cpu())
        assert ok, (ns, err)


def test_cfg1_full_size_with_4bit_values(gpu):
    """configs[1] with the values of the quantized groups in 4 bits (the Mixed variant): the value
    quantizer over 4.2M rows against the oracle on whole planes (bit-exact), the attention against
    the fp64 oracle on whole planes, split invariance, and chunked == one-shot value quantization."""
    from polarquant_amd.attention import polar_decode_attention_v4
    from polarquant_amd.values import quantize_values
    print("building configs[1] + 4-bit values", flush=True)
    w = bench.build_workload(1, gpu)
    sh = w["shape"]
    B, Nk, rep = sh.batch, sh.n_kv_heads, sh.n_heads // sh.n_kv_heads
    L = w["n_groups"] * 128
    vq = quantize_values(w["v"][:, :, :L])
    vres = torch.zeros(B, Nk, 128, 128, dtype=torch.float16, device=gpu)
    vres[:, :, :1] = w["v"][:, :, L:L + 1]
    # chunked quantization into a pre-allocated store == one shot
    store = (torch.empty_like(vq[0]), torch.empty_like(vq[1]), torch.empty_like(vq[2]))
    for t0 in range(0, L, 8192):
        quantize_values(w["v"][:, :, t0:t0 + 8192], out=store, token_offset=t0)
    assert all(torch.equal(a, b) for a, b in zip(store, vq))

    def attn(**kw):
        return polar_decode_attention_v4(w["q"], w["codes"], *w["meta"], w["kres"], vres, *vq, w["n_groups"], 1,
                                         rbits=sh.rbits, tbits=sh.tbits, **kw)
    out = attn().clone()
    torch.cuda.synchronize()
    assert out.shape == (16, 32, 1, 128) and torch.isfinite(out.float()).all()
    for b, kvh in [(0, 0), (9, 2), (15, 7)]:
        v_plane = w["v"][b:b + 1, kvh:kvh + 1, :L].cpu()
        ref_q = po.quantize_values_along_last_dim(v_plane)
        for got, ref in zip(vq, ref_q):
            g = got[b:b + 1, kvh:kvh + 1].cpu()
            assert torch.equal(g if g.dtype == torch.int32 else g.view(torch.int16), ref if ref.dtype == torch.int32 else ref.view(torch.int16))
        q = w["q"][b:b + 1, kvh * rep:(kvh + 1) * rep].cpu()
        quant = [w["codes"][b:b + 1, kvh:kvh + 1].cpu()] + [m[b:b + 1, kvh:kvh + 1].cpu() for m in w["meta"]]
        ref = po.decode_attention_mixed_exact(q, w["kres"][b:b + 1, kvh:kvh + 1, :1].cpu(), *quant,
                                              vres[b:b + 1, kvh:kvh + 1, :1].cpu(), *ref_q)
        ok, err = _ok(out[b:b + 1, kvh * rep:(kvh + 1) * rep].cpu(), ref)
        print("plane", b, kvh, "max abs err %.2e" % err, flush=True)
        assert ok
    for ns in (3, 8, 64):
        ok, err = _ok(attn(n_splits=ns).cpu(), out.cpu())
        assert ok, (ns, err)


def test_cfg4_attention_layer_at_full_width(gpu):
    """configs[4]'s shape for ONE attention layer of the drop-in class (hidden 4096, 32 query / 8 KV heads, bf16,
    batch 8, prompt 16384, then decode steps across nothing but the residual window): the post-RoPE q / k / v the layer
    saw are replayed through the oracle for sequence 0, cache contents bit for bit, outputs within the bf16 band of
    the model test; the other sequences are held to batch invariance (sequence 5 alone == sequence 5 in the batch)."""
    from polarquant_amd.modeling_common import PolarConfig
    from polarquant_amd.modeling_llama_polar import LlamaPolarGroupAttention
    torch.manual_seed(4)
    cfg = PolarConfig.llama3_8b(num_hidden_layers=1)
    att = LlamaPolarGroupAttention(cfg, 0).to(torch.bfloat16).to(gpu)
    att.capture = []
    B, L, steps = 8, 16384, 3
    inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, 128, 2, dtype=torch.float32) / 128))

    def rope(start, n):
        ang = torch.arange(start, start + n, dtype=torch.float32)[:, None] * inv[None]
        emb = torch.cat([ang, ang], -1)[None]
        return emb.cos().to(torch.bfloat16).to(gpu), emb.sin().to(torch.bfloat16).to(gpu)

    g = torch.Generator(device=gpu).manual_seed(44)
    x = torch.randn(B, L + steps, cfg.hidden_size, generator=g, device=gpu).mul_(0.5).to(torch.bfloat16)
    with torch.no_grad():
        _, cache = att(x[:, :L], attention_mask=None, past_key_value=None, position_embeddings=rope(0, L))
        q, k, v = [t[:1].cpu() for t in att.capture[-1]]
        ref_cache = po.prefill_cache(k, v, 4, 4)
        assert cache[-1] == L and cache[1].shape[2] >= L // 128
        for j in (1, 2, 3, 4, 5):                                       # codes and the four metadata tensors of sequence 0
            got, ref = cache[j][:1, :, :L // 128].cpu(), ref_cache[j]
            assert got.shape == ref.shape, j
            assert torch.equal(got, ref) if got.dtype == torch.uint8 else bool((got.float() == ref.float()).all()), "tuple element %d" % j
        o_proj = att.o_proj.weight.detach().float().cpu()
        solo_cache = None
        for i in range(steps):
            out, cache = att(x[:, L + i:L + i + 1], attention_mask=None, past_key_value=cache, position_embeddings=rope(L + i, 1))
            q, k, v = [t[:1].cpu() for t in att.capture[-1]]
            ref_attn, ref_cache = po.decode_step(q, k, v, ref_cache, None, 4, 4)
            ref_out = ref_attn.reshape(1, 1, -1).float() @ o_proj.T
            err = (out[:1].float().cpu() - ref_out).abs().max().item()
            assert err < 2e-2 * max(1.0, ref_out.abs().max().item()), (i, err)
        assert cache[-1] == L + steps
        # batch invariance: sequence 5 on its own gives the bits it gave inside the batch
        att.capture = []
        _, solo_cache = att(x[5:6, :L], attention_mask=None, past_key_value=None, position_embeddings=rope(0, L))
        solo, _ = att(x[5:6, L:L + 1], attention_mask=None, past_key_value=solo_cache, position_embeddings=rope(L, 1))
        _, again = att(x[:, :L], attention_mask=None, past_key_value=None, position_embeddings=rope(0, L))
        batched, _ = att(x[:, L:L + 1], attention_mask=None, past_key_value=again, position_embeddings=rope(L, 1))
        assert torch.equal(solo_cache[1][0, :, :L // 128], again[1][5, :, :L // 128])
        close = (solo[0].float() - batched[5].float()).abs().max().item()
        assert close <= 2e-2 * max(1.0, batched[5].float().abs().max().item()), close


@pytest.mark.parametrize("form", ["pairs", "one_wavefront", "device_cut", "three_slices"])
def test_largest_plane(gpu, form):
    """One (sequence, KV head) plane at the size limit: 2^24 - 256 value rows (4.29 GB of values, 1.07 GB of codes), the
    largest offsets the kernels form.  The context is one block of 7 quantized groups repeated 18 724 times, so every block
    carries the same softmax mass; value dimensions 0..14 hold the binary digits of a token's block number, whose
    attention-weighted mean is then the fraction of blocks with that digit set (a closed form), and the other dimensions
    repeat the block's values, whose result is the oracle's for a single block.  A value row fetched from a wrong offset, a
    slice skipped or read twice, or a group's metadata taken from another group (7 is odd: no power-of-two stride maps a
    block onto itself) moves one or the other."""
    from polarquant_amd import workloads as wl
    print("case", form, flush=True)
    G_BLK, N_BLK = 7, 18724
    n_groups = G_BLK * N_BLK                                  # 131 068 groups = 16 776 704 tokens
    rows, group_cap = (1 << 24) - 256, ((1 << 24) - 256) // 128
    g = torch.Generator().manual_seed(77)
    kb = wl.make_keys(1, 1, G_BLK * 128, 5e5, g, torch.float16)
    quant = po.quantize_and_pack_nbit(kb, 4, 4)
    vb = wl.make_half((1, 1, G_BLK * 128, 128), g, torch.float16)
    vb[..., :16] = 0
    q = wl.make_half((1, 4, 1, 128), g, torch.float16)
    ref_block = po.decode_attention_exact(q, None, *quant, vb, None, 4, 4)          # dimensions 16.. of the expected output
    codes = torch.zeros(1, 1, group_cap, 128, 64, dtype=torch.uint8, device=gpu)
    codes[:, :, :n_groups] = quant[0].to(gpu).repeat(1, 1, N_BLK, 1, 1)
    meta = []
    for m in quant[1:]:
        t = torch.zeros(1, 1, group_cap, 1, 64, dtype=torch.float16, device=gpu)
        t[:, :, :n_groups] = m.to(gpu).repeat(1, 1, N_BLK, 1, 1)
        meta.append(t)
    v = torch.zeros(1, 1, rows, 128, dtype=torch.float16, device=gpu)
    T = n_groups * 128
    v[0, 0, :T, 16:] = vb[0, 0, :, 16:].to(gpu).repeat(N_BLK, 1)
    blk = torch.arange(T, device=gpu) // (G_BLK * 128)
    for d in range(15):
        v[0, 0, :T, d] = ((blk >> d) & 1).to(torch.float16)
    v[0, 0, T:] = float("nan")                               # rows behind the context must not be read as values
    del blk
    want = ref_block.clone().double()
    idx = torch.arange(N_BLK)
    for d in range(15):
        want[..., d] = float(((idx >> d) & 1).double().mean())
    want[..., 15] = 0.0
    kres = torch.zeros(1, 1, 128, 128, dtype=torch.float16, device=gpu)
    kw = dict(rbits=4, tbits=4)
    if form == "one_wavefront":
        kw.update(single_wavefront=True)
    elif form == "device_cut":
        kw.update(n_groups_per_seq=torch.tensor([n_groups], dtype=torch.int32, device=gpu),
                  n_resid_per_seq=torch.tensor([0], dtype=torch.int32, device=gpu))
    elif form == "three_slices":
        kw.update(n_splits=3)
    ng = 0 if form == "device_cut" else n_groups
    out = polar_decode_attention(q.to(gpu), codes, *meta, kres, v, ng, 0, **kw).cpu()
    assert torch.isfinite(out.float()).all()
    ok, emax = _ok(out, want)
    assert ok, emax


@pytest.mark.parametrize("form", ["even", "device_cut"])
def test_largest_plane_with_4bit_values(gpu, form):
    """The same construction for the 4-bit-value kernels at their largest value store (2^24 - 256 rows of packed codes):
    every row has scale 1/15 and zero-point 0, digit dimensions hold code 0 or 15, the others the block's own codes."""
    from polarquant_amd import workloads as wl
    from polarquant_amd.attention import polar_decode_attention_v4
    print("case", form, flush=True)
    G_BLK, N_BLK = 7, 18724
    n_groups = G_BLK * N_BLK
    rows, group_cap = (1 << 24) - 256, ((1 << 24) - 256) // 128
    g = torch.Generator().manual_seed(78)
    kb = wl.make_keys(1, 1, G_BLK * 128, 5e5, g, torch.float16)
    quant = po.quantize_and_pack_nbit(kb, 4, 4)
    q = wl.make_half((1, 4, 1, 128), g, torch.float16)
    TB = G_BLK * 128
    cb = torch.randint(0, 16, (TB, 128), generator=g, dtype=torch.int64)
    cb[:, :16] = 0
    pack = lambda c: (c.reshape(-1, 16, 8) << (4 * torch.arange(8))).sum(-1).to(torch.int32)      # dim 8w + i -> bits [4i, 4i + 4) of word w
    scale_b = torch.full((1, 1, TB, 1), 1.0 / 15.0).half()
    zero_b = torch.zeros(1, 1, TB, 1).half()
    empty = torch.zeros(1, 1, 0, 128, dtype=torch.float16)
    ref_block = po.decode_attention_mixed_exact(q, None, *quant, empty, pack(cb).reshape(1, 1, TB, 16), scale_b, zero_b, None, 4, 4)
    codes = torch.zeros(1, 1, group_cap, 128, 64, dtype=torch.uint8, device=gpu)
    codes[:, :, :n_groups] = quant[0].to(gpu).repeat(1, 1, N_BLK, 1, 1)
    meta = []
    for m in quant[1:]:
        t = torch.zeros(1, 1, group_cap, 1, 64, dtype=torch.float16, device=gpu)
        t[:, :, :n_groups] = m.to(gpu).repeat(1, 1, N_BLK, 1, 1)
        meta.append(t)
    T = n_groups * 128
    # digits of the block number: dims 0..14 are codes 0 / 15 in words 0 and 1 (8 dims per word)
    blk = torch.arange(T, device=gpu) // TB
    vc = torch.full((1, 1, rows, 16), -1, dtype=torch.int32, device=gpu)
    vc[0, 0, :T] = pack(cb).to(gpu).repeat(N_BLK, 1)
    for w in range(2):
        word = torch.zeros(T, dtype=torch.int64, device=gpu)
        for i in range(8):
            d = 8 * w + i
            if d < 15:
                word |= (((blk >> d) & 1) * 15) << (4 * i)
        vc[0, 0, :T, w] = word.to(torch.int32)
    del blk, word
    vs = torch.full((1, 1, rows, 1), float("nan"), dtype=torch.float16, device=gpu)
    vz = torch.full((1, 1, rows, 1), float("nan"), dtype=torch.float16, device=gpu)
    vs[0, 0, :T] = 1.0 / 15.0
    vz[0, 0, :T] = 0.0
    want = ref_block.clone().double()
    idx = torch.arange(N_BLK)
    one = float(torch.tensor(1.0 / 15.0).half()) * 15.0
    for d in range(15):
        want[..., d] = float(((idx >> d) & 1).double().mean()) * one
    want[..., 15] = 0.0
    kres = torch.zeros(1, 1, 128, 128, dtype=torch.float16, device=gpu)
    vres = torch.zeros(1, 1, 128, 128, dtype=torch.float16, device=gpu)
    kw = dict(rbits=4, tbits=4)
    if form == "device_cut":
        kw.update(n_groups_per_seq=torch.tensor([n_groups], dtype=torch.int32, device=gpu),
                  n_resid_per_seq=torch.tensor([0], dtype=torch.int32, device=gpu), balanced=True)
    ng = 0 if form == "device_cut" else n_groups
    out = polar_decode_attention_v4(q.to(gpu), codes, *meta, kres, vres, vc, vs, vz, ng, 0, **kw).cpu()
    assert torch.isfinite(out.float()).all()
    ok, emax = _ok(out, want)
    assert ok, emax


def test_most_planes(gpu):
    """The largest batch the entry points take: 65 520 (sequence, KV head) planes (the limit is 65 535).  Eight different
    sequences repeated 1 023 times and a few more: the quantizer, the score op and the attention must give every replica
    the bits of its original, and the originals must agree with the oracle."""
    from polarquant_amd import workloads as wl
    from polarquant_amd.kernel4group import attention_decode_forward_triton_impl
    B0, Nk, reps = 8, 8, 1023
    B = B0 * reps + 6                                   # 8 190 sequences x 8 KV heads = 65 520 planes
    g = torch.Generator().manual_seed(91)
    k0 = wl.make_keys(B0, Nk, 128 + 5, 5e5, g, torch.float16)
    v0 = wl.make_half((B0, Nk, 128 + 5, 128), g, torch.float16)
    q0 = wl.make_half((B0, Nk, 1, 128), g, torch.float16)
    tile = lambda t: t.to(gpu).repeat(reps + 1, *([1] * (t.dim() - 1)))[:B].contiguous()
    k, v, q = tile(k0), tile(v0), tile(q0)
    quant = quantize_and_pack_nbit(k[:, :, :128], 4, 4)
    ref_quant = po.quantize_and_pack_nbit(k0[:, :, :128].contiguous(), 4, 4)
    for got, ref in zip(quant, ref_quant):
        assert torch.equal(got[:B0].cpu().view(torch.uint8 if got.dtype == torch.uint8 else torch.int16),
                           ref.view(torch.uint8 if ref.dtype == torch.uint8 else torch.int16))
        assert torch.equal(got[B0:2 * B0], got[:B0]) and torch.equal(got[B - B0 - 6:B - 6], got[:B0]) and torch.equal(got[B - 6:], got[:6])
    scores = attention_decode_forward_triton_impl(q, *quant, rbits=4, tbits=4)
    ref_scores = po.decode_scores(q0, *ref_quant, 4, 4)
    assert float((scores[:B0].cpu().double() - ref_scores.double()).abs().max()) <= 2e-5 * float(ref_scores.abs().max())
    assert torch.equal(scores[B - B0 - 6:B - 6], scores[:B0]) and torch.equal(scores[B - 6:], scores[:6])
    kres = torch.zeros(B, Nk, 128, 128, dtype=torch.float16, device=gpu)
    kres[:, :, :5] = k[:, :, 128:]
    out = polar_decode_attention(q, *quant, kres, v, 1, 5, rbits=4, tbits=4)
    ref = po.decode_attention_exact(q0, k0[:, :, 128:], *ref_quant, v0, None, 4, 4)
    ok, emax = _ok(out[:B0].cpu(), ref)
    assert ok, emax
    assert torch.equal(out[B0:2 * B0], out[:B0]) and torch.equal(out[B - B0 - 6:B - 6], out[:B0]) and torch.equal(out[B - 6:], out[:6])
