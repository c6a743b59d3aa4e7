"""What fixes the plain implementation beside the reference's text.

The reference holds no test vectors (it has no tests), so each formula is pinned by a
special case that reduces to a library routine, or by an invariant, chosen so that a
plausible mistake (a wrong sign or pairing, eps or a norm in the wrong place, the wrong
kv head) fails it.
"""
import math

import pytest
import torch

import plain_llama as plain


def test_find_multiple():                       # model.py:16-19
    assert plain.find_multiple(256, 256) == 256
    assert plain.find_multiple(257, 256) == 512
    # derived feed-forward width of the 7B shape, model.py:38-41
    assert plain.config_from_dict(dict(hidden_size=4096, num_attention_heads=32,
                                       num_hidden_layers=1, vocab_size=8))["inter"] == 11008


def test_rms_norm_against_float64_and_eps_place():
    torch.manual_seed(0)
    x = torch.randn(5, 48)
    w = torch.randn(48)
    ref = (x.double() / torch.sqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-5) * w.double())
    assert torch.allclose(plain.rms_norm(x, w, 1e-5).double(), ref, rtol=1e-6, atol=1e-7)
    # eps is inside the root, added to the mean: for a tiny input it dominates
    tiny = torch.full((1, 48), 1e-4)
    out = plain.rms_norm(tiny, torch.ones(48), 1e-2)
    assert torch.allclose(out, tiny / math.sqrt(1e-8 + 1e-2), rtol=1e-5)
    # with w = 1 the mean square of the output is ms / (ms + eps)
    y = plain.rms_norm(x, torch.ones(48), 0.5)
    ms = (x * x).mean(-1)
    assert torch.allclose((y * y).mean(-1), ms / (ms + 0.5), rtol=1e-5)


def test_rope_position_zero_norm_and_relative():
    torch.manual_seed(1)
    hd = 16
    q = torch.randn(6, 2, hd)
    k = torch.randn(6, 2, hd)
    cos0, sin0 = plain.rope_table([0] * 6, hd, 10000.0)
    assert torch.equal(plain.apply_rope(q, cos0, sin0), q)          # position 0 is the identity
    pos = torch.arange(6)
    cos, sin = plain.rope_table(pos, hd, 10000.0)
    qr, kr = plain.apply_rope(q, cos, sin), plain.apply_rope(k, cos, sin)
    # every interleaved pair keeps its norm
    n0 = q.reshape(6, 2, hd // 2, 2).norm(dim=-1)
    n1 = qr.reshape(6, 2, hd // 2, 2).norm(dim=-1)
    assert torch.allclose(n0, n1, rtol=1e-5, atol=1e-6)
    # a shift of all positions leaves every score unchanged: only distances count
    cos_s, sin_s = plain.rope_table(pos + 37, hd, 10000.0)
    qs, ks = plain.apply_rope(q, cos_s, sin_s), plain.apply_rope(k, cos_s, sin_s)
    s0 = torch.einsum("ihd,jhd->hij", qr, kr)
    s1 = torch.einsum("ihd,jhd->hij", qs, ks)
    assert torch.allclose(s0, s1, rtol=1e-4, atol=1e-4)
    # the sign of the rotation: pair (1, 0) at angle a becomes (cos a, sin a)
    x = torch.zeros(1, 1, hd)
    x[0, 0, 0] = 1.0
    c, s = plain.rope_table([3], hd, 10000.0)
    out = plain.apply_rope(x, c, s)
    assert abs(out[0, 0, 0].item() - math.cos(3.0)) < 1e-6
    assert abs(out[0, 0, 1].item() - math.sin(3.0)) < 1e-6


def test_rope_interleaved_on_permuted_rows_equals_half_split():
    """scripts/convert_hf_checkpoint.py:75-81 ties the pair layout to the row permutation:
    interleaved rotation of permuted projections gives the scores of the half-split
    rotation of the unpermuted ones."""
    torch.manual_seed(2)
    H, hd, D, S = 2, 8, 12, 5
    wq, wk = torch.randn(H * hd, D), torch.randn(H * hd, D)
    x = torch.randn(S, D)
    cos, sin = plain.rope_table(torch.arange(S), hd, 10000.0)

    def half_split(v):          # pairs (i, i + hd/2)
        a, b = v[..., : hd // 2], v[..., hd // 2:]
        c, s = cos[:, None, :], sin[:, None, :]
        return torch.cat([a * c - b * s, b * c + a * s], dim=-1)

    q_h = half_split((x @ wq.T).reshape(S, H, hd))
    k_h = half_split((x @ wk.T).reshape(S, H, hd))
    q_i = plain.apply_rope((x @ plain.permute_rows(wq, H, hd).T).reshape(S, H, hd), cos, sin)
    k_i = plain.apply_rope((x @ plain.permute_rows(wk, H, hd).T).reshape(S, H, hd), cos, sin)
    assert torch.allclose(torch.einsum("ihd,jhd->hij", q_h, k_h),
                          torch.einsum("ihd,jhd->hij", q_i, k_i), rtol=1e-4, atol=1e-4)


def test_rope_scaling_branches():               # model.py:244-263
    f = plain.rope_frequencies(128, 500000.0)
    sc = dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=8192)
    g = plain.scale_frequencies(f, sc)
    kept = int((g == f).sum())
    divided = int(torch.isclose(g, f / 8.0, rtol=1e-7).sum())
    assert (kept, 64 - kept - divided, divided) == (29, 6, 29)      # census of the 8B preset
    # factor 1 is the identity
    one = plain.scale_frequencies(f, dict(sc, factor=1.0))
    assert torch.allclose(one, f, rtol=1e-6)
    # continuity at both ends of the blend
    orig = 8192
    for wavelen, expect in ((orig / 4.0, 1.0), (orig / 1.0, 1.0 / 8.0)):
        fr = torch.tensor([2 * math.pi / wavelen * 0.999999, 2 * math.pi / wavelen * 1.000001])
        out = plain.scale_frequencies(fr, sc) / fr
        assert torch.allclose(out, torch.full((2,), expect), rtol=1e-3)
    # the tiny test shape (hd 32, orig 32) hits all three branches
    ft = plain.rope_frequencies(32, 500000.0)
    gt = plain.scale_frequencies(ft, dict(sc, original_max_position_embeddings=32))
    assert gt[0] == ft[0] and torch.isclose(gt[2], ft[2] / 8) and ft[1] / 8 < gt[1] < ft[1]


def test_attention_reduces_to_library_routine():
    torch.manual_seed(3)
    S, H, hd = 9, 4, 16
    q, k, v = torch.randn(S, H, hd), torch.randn(S, H, hd), torch.randn(S, H, hd)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True).transpose(0, 1)
    assert torch.allclose(plain.causal_attention(q, k, v), ref, rtol=1e-5, atol=1e-6)
    # one token: softmax of one score, the output is v
    assert torch.allclose(plain.causal_attention(q[:1], k[:1], v[:1]), v[:1])
    # q = 0: the mean of v over the keys seen so far
    out = plain.causal_attention(torch.zeros_like(q), k, v)
    assert torch.allclose(out[4], v[:5].mean(0), rtol=1e-5, atol=1e-6)
    # causality: a later token does not change earlier outputs
    k2, v2 = k.clone(), v.clone()
    k2[-1] += 1.0
    v2[-1] += 1.0
    assert torch.equal(plain.causal_attention(q, k2, v2)[:-1], plain.causal_attention(q, k, v)[:-1])


def test_gqa_head_mapping_is_repeat_interleave():      # model.py:209-210
    torch.manual_seed(4)
    S, H, G, hd = 5, 6, 2, 8
    q, k, v = torch.randn(S, H, hd), torch.randn(S, G, hd), torch.randn(S, G, hd)
    full = plain.causal_attention(q, k.repeat_interleave(H // G, dim=1),
                                  v.repeat_interleave(H // G, dim=1))
    assert torch.allclose(plain.causal_attention(q, k, v), full)
    wrong = plain.causal_attention(q, k.repeat(1, H // G, 1), v.repeat(1, H // G, 1))
    assert not torch.allclose(full, wrong)


def test_feed_forward():
    torch.manual_seed(5)
    x = torch.randn(4, 10)
    w1, w3, w2 = torch.randn(14, 10), torch.randn(14, 10), torch.randn(10, 14)
    ref = (torch.nn.functional.silu(x @ w1.T) * (x @ w3.T)) @ w2.T
    assert torch.allclose(plain.feed_forward(x, w1, w3, w2), ref, rtol=1e-5, atol=1e-5)
    assert torch.equal(plain.feed_forward(x, w1, torch.zeros_like(w3), w2), torch.zeros(4, 10))
    assert not torch.allclose(plain.feed_forward(x, w3, w1, w2), ref)      # gate is w1, up is w3


def _tiny_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g) * 0.1
    D, H, G, hd, I, V = cfg["dim"], cfg["n_head"], cfg["n_kv"], cfg["head_dim"], cfg["inter"], cfg["vocab"]
    w = {"tok_embeddings.weight": r(V, D), "norm.weight": 1 + r(D), "output.weight": r(V, D)}
    for i in range(cfg["n_layer"]):
        p = f"layers.{i}."
        w[p + "attention.wqkv.weight"] = r((H + 2 * G) * hd, D)
        w[p + "attention.wo.weight"] = r(D, H * hd)
        w[p + "feed_forward.w1.weight"] = r(I, D)
        w[p + "feed_forward.w3.weight"] = r(I, D)
        w[p + "feed_forward.w2.weight"] = r(D, I)
        w[p + "attention_norm.weight"] = 1 + r(D)
        w[p + "ffn_norm.weight"] = 1 + r(D)
    return w


CFG = dict(dim=24, n_layer=2, n_head=3, n_kv=1, head_dim=8, inter=40, vocab=50,
           rope_base=10000.0, eps=1e-5, rope_scaling=None, tie=False)


def test_blocks_are_identity_when_output_projections_vanish():     # model.py:161-164
    w = _tiny_weights(CFG)
    for i in range(CFG["n_layer"]):
        w[f"layers.{i}.attention.wo.weight"].zero_()
        w[f"layers.{i}.feed_forward.w2.weight"].zero_()
    toks = [3, 7, 1, 9]
    x = w["tok_embeddings.weight"][torch.tensor(toks)]
    ref = plain.rms_norm(x, w["norm.weight"], CFG["eps"]) @ w["output.weight"].T
    assert torch.allclose(plain.forward(w, CFG, toks), ref, rtol=1e-6, atol=1e-6)


def test_rope_frequency_ladder_by_hand():                          # model.py:271
    """f_i = base^(-2i/hd): written out for sizes where the powers are plain decimals.  An
    exponent i/hd, (2i+1)/hd or 2i/(hd-2) gives other numbers."""
    assert torch.allclose(plain.rope_frequencies(8, 10000.0),
                          torch.tensor([1.0, 0.1, 0.01, 0.001]), rtol=1e-6)
    assert torch.allclose(plain.rope_frequencies(4, 100.0), torch.tensor([1.0, 0.1]), rtol=1e-6)
    f = plain.rope_frequencies(128, 500000.0).double()
    assert f.numel() == 64 and f[0] == 1.0
    assert torch.allclose(f[1:] / f[:-1], torch.full((63,), 500000.0 ** (-2.0 / 128)).double(), rtol=1e-5)
    assert abs(float(f[-1]) - 500000.0 ** (-126.0 / 128)) < 1e-9
    # the angle of pair i at position p is p * f_i (model.py:274-276): pair 1 of head size 8
    cos, sin = plain.rope_table([5], 8, 10000.0)
    assert abs(float(cos[0, 1]) - math.cos(0.5)) < 1e-6 and abs(float(sin[0, 1]) - math.sin(0.5)) < 1e-6


def test_norms_stand_before_mixer_and_feed_forward():             # model.py:161-164
    """h = x + attention(norm_a(x)), out = h + ffn(norm_f(h)).  With one branch silenced (the
    other one's output projection zero), what the block adds to its input does not change
    when the input is scaled, because the branch sees a normed copy (eps -> 0): with the norm
    behind the branch or behind the sum, it does.  Each branch alone is that part of its own
    norm's rows, which tells the two norm weights apart, and the whole block is the second
    branch on the stream after the first sum."""
    cfg = dict(CFG, eps=1e-12)
    w = _tiny_weights(cfg, 3)
    x = torch.randn(5, cfg["dim"], generator=torch.Generator().manual_seed(4))
    pos = torch.arange(5)
    for silenced in ("layers.0.feed_forward.w2.weight", "layers.0.attention.wo.weight"):
        one = dict(w)
        one[silenced] = torch.zeros_like(w[silenced])
        added = plain.block(x, one, 0, cfg, pos) - x
        assert float(added.abs().max()) > 1e-2
        for c in (0.25, 8.0):
            assert torch.allclose(plain.block(c * x, one, 0, cfg, pos) - c * x, added,
                                  rtol=1e-4, atol=1e-5)
    p = "layers.0."
    only_attn = dict(w)
    only_attn[p + "feed_forward.w2.weight"] = torch.zeros_like(w[p + "feed_forward.w2.weight"])
    a = plain.attention(plain.rms_norm(x, w[p + "attention_norm.weight"], cfg["eps"]),
                        w[p + "attention.wqkv.weight"], w[p + "attention.wo.weight"], cfg, pos)
    assert torch.allclose(plain.block(x, only_attn, 0, cfg, pos) - x, a, rtol=1e-5, atol=1e-6)
    h = x + a
    f = plain.feed_forward(plain.rms_norm(h, w[p + "ffn_norm.weight"], cfg["eps"]),
                           w[p + "feed_forward.w1.weight"], w[p + "feed_forward.w3.weight"],
                           w[p + "feed_forward.w2.weight"])
    assert torch.allclose(plain.block(x, w, 0, cfg, pos), h + f, rtol=1e-5, atol=1e-6)
    swapped = dict(w)
    swapped[p + "attention_norm.weight"], swapped[p + "ffn_norm.weight"] = \
        w[p + "ffn_norm.weight"], w[p + "attention_norm.weight"]
    assert not torch.allclose(plain.block(x, swapped, 0, cfg, pos), h + f, rtol=1e-4, atol=1e-5)


def test_gate_saturates_where_the_first_matrix_is_negative():     # model.py:227
    """silu(w1 x) * (w3 x): a row of w1 that maps x far below zero closes the gate whatever
    w3 gives; a row of w3 far below zero does not."""
    x = torch.ones(1, 4)
    w2 = torch.eye(4)
    closed = plain.feed_forward(x, torch.full((4, 4), -10.0), torch.full((4, 4), 3.0), w2)
    assert float(closed.abs().max()) < 1e-10
    open_ = plain.feed_forward(x, torch.full((4, 4), 3.0), torch.full((4, 4), -10.0), w2)
    assert float(open_.abs().min()) > 100.0


def test_forward_is_causal_and_per_position():
    w = _tiny_weights(CFG, 1)
    a = plain.forward(w, CFG, [3, 7, 1, 9, 4])
    b = plain.forward(w, CFG, [3, 7, 1, 2, 2])
    assert torch.allclose(a[:3], b[:3], rtol=1e-6, atol=1e-6)
    assert not torch.allclose(a[3], b[3])
    assert torch.allclose(plain.forward(w, CFG, [3, 7, 1])[-1], a[2], rtol=1e-5, atol=1e-6)


def test_float64_agrees():
    w = _tiny_weights(CFG, 2)
    a = plain.forward(w, CFG, [1, 2, 3, 4, 5, 6])
    w64 = {k: v.double() for k, v in w.items()}
    b = plain.forward(w64, CFG, [1, 2, 3, 4, 5, 6])
    assert torch.allclose(a.double(), b, rtol=1e-4, atol=1e-5)


def test_sampling_law():                       # generate.py:40-57
    torch.manual_seed(6)
    logits = torch.randn(3, 40)
    p = plain.logits_to_probs(logits, 0.7, 5)
    assert torch.allclose(p.sum(-1), torch.ones(3), rtol=1e-6)
    assert ((p > 0).sum(-1) == 5).all()
    assert torch.equal(plain.logits_to_probs(logits, 1.0, 1).argmax(-1), logits.argmax(-1))
    assert torch.allclose(plain.logits_to_probs(logits, 1.0, 100), torch.softmax(logits, -1))
    near = plain.logits_to_probs(logits, 0.0, None)           # floor 1e-5: near one-hot
    assert torch.equal(near.argmax(-1), logits.argmax(-1)) and (near.max(-1).values > 0.999).all()
    # exponential race draws index i with probability p_i
    probs = torch.tensor([0.5, 0.3, 0.2])
    noise = torch.empty(20000, 3).exponential_(1)
    counts = torch.bincount(plain.sample_with_noise(probs.expand(20000, 3), noise), minlength=3)
    assert torch.allclose(counts / 20000.0, probs, atol=0.015)


def test_noise_generator_known_answers():
    """The tests' own Philox4x32-10 (util.philox4x32_10, with which the GPU tests recompute the
    sampler's noise) against the known answers published with the generator (Random123's
    kat_vectors: counter and key all zeros, all ones)."""
    import util
    got = [int(x[0]) for x in util.philox4x32_10([0], [0], [0], [0], 0, 0)]
    assert got == [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]
    ones = 0xFFFFFFFF
    got = [int(x[0]) for x in util.philox4x32_10([ones], [ones], [ones], [ones], ones, ones)]
    assert got == [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]
    q = util.sampler_noise(1001, seed=7, key=3, pos=12)
    assert q.shape == (1001,) and bool((q > 0).all()) and bool(torch.isfinite(q).all())
    assert abs(float(q.mean()) - 1.0) < 0.1                      # Exp(1)
