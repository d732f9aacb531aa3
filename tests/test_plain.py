"""What fixes the plain implementation beside the reference's text: library routines it must reduce
to, invariants, and examples the reference's own files hold. Each is chosen so that a plausible
mistake (a wrong sign or pairing, a norm in the wrong place, an offset left out) fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_opt
from conftest import TINY_A, TINY_B


def test_layer_norm_is_the_library_routine():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 96, generator=g) * 3 + 2
    w, b = torch.randn(96, generator=g), torch.randn(96, generator=g)
    for eps in (1e-5, 1e-2):
        torch.testing.assert_close(plain_opt.layer_norm(x, w, b, eps), F.layer_norm(x, (96,), w, b, eps))
    y = plain_opt.layer_norm(x, None, None, 1e-5)
    torch.testing.assert_close(y.mean(-1), torch.zeros(7), atol=1e-6, rtol=0)
    var = x.var(-1, unbiased=False)
    torch.testing.assert_close(y.var(-1, unbiased=False), var / (var + 1e-5))      # biased variance, eps inside
    torch.testing.assert_close(plain_opt.layer_norm(x + 5.0, w, b, 1e-5), plain_opt.layer_norm(x, w, b, 1e-5),
                               atol=1e-5, rtol=1e-5)
    # the mean / E[x^2] - mean^2 form of the reference's CPU analogue (pad/layernorm_padded_cpu.py:57-66)
    mean = x.mean(-1, keepdim=True)
    var2 = (x * x).mean(-1, keepdim=True) - mean * mean
    torch.testing.assert_close(y, (x - mean) / torch.sqrt(var2 + 1e-5), atol=1e-5, rtol=1e-5)


def test_linear_and_activations():
    g = torch.Generator().manual_seed(1)
    x, w, b = torch.randn(5, 24, generator=g), torch.randn(40, 24, generator=g), torch.randn(40, generator=g)
    torch.testing.assert_close(plain_opt.linear(x, w, b), F.linear(x, w, b))
    torch.testing.assert_close(plain_opt.linear(x, w), F.linear(x, w))
    z = torch.randn(1000, generator=g) * 3
    torch.testing.assert_close(plain_opt.activation(z, "relu"), F.relu(z))
    torch.testing.assert_close(plain_opt.activation(z, "gelu"), F.gelu(z))
    torch.testing.assert_close(plain_opt.activation(z, "gelu_new"), F.gelu(z, approximate="tanh"))
    r = plain_opt.activation(z, "relu")
    assert torch.equal(plain_opt.activation(r, "relu"), r)
    # the constants of activations.py:25-29
    one = torch.tensor([1.0])
    assert abs(float(plain_opt.activation(one, "gelu_new")) -
               0.5 * (1 + math.tanh(math.sqrt(2 / math.pi) * 1.044715))) < 1e-7


def test_attention_is_library_attention():
    g = torch.Generator().manual_seed(2)
    s, heads, d = 13, 3, 16
    q, k, v = (torch.randn(s, heads * d, generator=g) for _ in range(3))
    got = plain_opt.causal_attention(q, k, v, heads)
    split = lambda t: t.reshape(s, heads, d).transpose(0, 1)   # noqa: E731
    want = F.scaled_dot_product_attention(split(q), split(k), split(v), is_causal=True)
    torch.testing.assert_close(got, want.transpose(0, 1).reshape(s, heads * d), atol=1e-5, rtol=1e-5)
    # token i does not depend on later tokens
    k2, v2 = k.clone(), v.clone()
    k2[8:], v2[8:] = 9.0, -9.0
    assert torch.equal(plain_opt.causal_attention(q, k2, v2, heads)[:8], got[:8])
    # one head of width heads*d is a different function: the split into heads matters
    assert not torch.allclose(plain_opt.causal_attention(q, k, v, 1), got, atol=1e-3)
    # grouped heads: kv head h serves query heads 2h, 2h+1
    kg, vg = k[:, :d], v[:, :d]
    grouped = plain_opt.causal_attention(q[:, :2 * d], kg, vg, 2)
    full = plain_opt.causal_attention(q[:, :2 * d], torch.cat([kg, kg], 1), torch.cat([vg, vg], 1), 2)
    torch.testing.assert_close(grouped, full)
    # a window of the whole length is no window; a window of 1 returns each token's own value
    torch.testing.assert_close(plain_opt.causal_attention(q, k, v, heads, window=s), got)
    torch.testing.assert_close(plain_opt.causal_attention(q, k, v, heads, window=1), v)


def test_two_part_decode_softmax_is_one_softmax():
    g = torch.Generator().manual_seed(3)
    d, n = 16, 21
    q = torch.randn(d, generator=g)
    k, v = torch.randn(n + 1, d, generator=g) * 2, torch.randn(n + 1, d, generator=g)
    got = plain_opt.decode_attention_two_part(q, k[:n], v[:n], k[n], v[n])
    want = torch.softmax(k @ q, 0) @ v
    torch.testing.assert_close(got, want, atol=1e-6, rtol=1e-5)
    # and equals the last row of the whole-sequence form (queries there are scaled inside)
    qs = torch.zeros(n + 1, d)
    qs[n] = q * math.sqrt(d)
    torch.testing.assert_close(plain_opt.causal_attention(qs, k, v, 1)[n], want, atol=1e-6, rtol=1e-5)


def test_positions_read_two_rows_further():
    table = torch.arange(12.0).unsqueeze(1).repeat(1, 3)
    assert plain_opt.learned_positions(table, 4)[:, 0].tolist() == [2.0, 3.0, 4.0, 5.0]
    assert plain_opt.learned_positions(table, 2, start=5)[:, 0].tolist() == [7.0, 8.0]
    w = plain_opt.random_weights(TINY_A, 0)
    toks = [5, 6, 7, 8]
    base = plain_opt.forward_logits(w, TINY_A, toks)
    w2 = dict(w)
    t = w["model.decoder.embed_positions.weight"].clone()
    t[:2] += 100.0                                  # rows 0 and 1 are never read
    w2["model.decoder.embed_positions.weight"] = t
    assert torch.equal(plain_opt.forward_logits(w2, TINY_A, toks), base)
    t = w["model.decoder.embed_positions.weight"].clone()
    t[2] += 1.0                                     # row 2 is position 0
    w2["model.decoder.embed_positions.weight"] = t
    assert not torch.allclose(plain_opt.forward_logits(w2, TINY_A, toks)[0], base[0])


def test_block_orders():
    cfg = dict(TINY_A)
    w = plain_opt.random_weights(cfg, 1)
    x = torch.randn(6, 64, generator=torch.Generator().manual_seed(4))
    # pre-norm with all matrices zero and no bias contribution is the identity
    wz = {k: (torch.zeros_like(v) if ("proj" in k or "fc" in k) else v) for k, v in w.items()}
    torch.testing.assert_close(plain_opt.block(x, wz, cfg, 0), x)
    # post-norm with the same zeros is LN(LN(x)): the norm sits after the sum
    post = dict(cfg, do_layer_norm_before=False)
    p = "model.decoder.layers.0."
    ln = lambda t, n: plain_opt.layer_norm(t, wz[p + n + ".weight"], wz[p + n + ".bias"], 1e-5)   # noqa: E731
    torch.testing.assert_close(plain_opt.block(x, wz, post, 0), ln(ln(x, "self_attn_layer_norm"), "final_layer_norm"))
    # the two orders differ on real weights, and each uses its own norm for its own half
    assert not torch.allclose(plain_opt.block(x, w, cfg, 0), plain_opt.block(x, w, post, 0), atol=1e-3)
    w_swapped = dict(w)
    w_swapped[p + "self_attn_layer_norm.weight"], w_swapped[p + "final_layer_norm.weight"] = \
        w[p + "final_layer_norm.weight"], w[p + "self_attn_layer_norm.weight"]
    assert not torch.allclose(plain_opt.block(x, w, cfg, 0), plain_opt.block(x, w_swapped, cfg, 0), atol=1e-4)


def test_head_tie_projection_and_final_norm():
    for raw in (TINY_A, TINY_B):
        w = plain_opt.random_weights(raw, 2)
        toks = list(range(3, 20))
        logits = plain_opt.forward_logits(w, raw, toks)
        assert logits.shape == (17, raw["vocab_size"])
        # an explicit head equal to the token table changes nothing; another one does
        w2 = dict(w, **{"lm_head.weight": w["model.decoder.embed_tokens.weight"].clone()})
        assert torch.equal(plain_opt.forward_logits(w2, raw, toks), logits)
        w2["lm_head.weight"] = w2["lm_head.weight"] * 2
        torch.testing.assert_close(plain_opt.forward_logits(w2, raw, toks), logits * 2)
        # logits of a prefix are the prefix of the logits (causality of the whole model)
        torch.testing.assert_close(plain_opt.forward_logits(w, raw, toks[:9]), logits[:9], atol=1e-5, rtol=1e-5)
    assert "model.decoder.final_layer_norm.weight" not in plain_opt.random_weights(TINY_B, 0)
    assert "model.decoder.project_in.weight" in plain_opt.random_weights(TINY_B, 0)


def test_top_k_top_p_filter():
    scores = torch.tensor([1.0, 3.0, 2.0, 0.0, 3.0])
    v, i = plain_opt.filter_top_k_top_p(scores, top_k=3)
    assert i.tolist() == [1, 4, 2] and v.tolist() == [3.0, 3.0, 2.0]           # ties: the lower id first
    v, i = plain_opt.filter_top_k_top_p(scores, top_k=10)                        # k clamped to the row
    assert len(i) == 5
    # top-p keeps the first token that crosses p (sampling.py:221-230): probabilities .5 .25 .125 .125
    s = torch.log(torch.tensor([0.125, 0.5, 0.25, 0.125]))
    assert plain_opt.filter_top_k_top_p(s, top_p=0.5)[1].tolist() == [1]        # the first alone reaches .5
    assert plain_opt.filter_top_k_top_p(s, top_p=0.51)[1].tolist() == [1, 2]    # .5 < .51: one more is needed
    assert plain_opt.filter_top_k_top_p(s, top_p=0.76)[1].tolist() == [1, 2, 0]
    assert plain_opt.filter_top_k_top_p(s, top_p=1e-9)[1].tolist() == [1]       # at least one token
    assert plain_opt.filter_top_k_top_p(s, top_k=2, top_p=0.99)[1].tolist() == [1, 2]


def test_draw():
    s = torch.log(torch.tensor([0.125, 0.5, 0.25, 0.125]))
    # inverse CDF in ascending token id: [0, .125) -> 0, [.125, .625) -> 1, [.625, .875) -> 2, rest -> 3
    for u, tok in ((0.0, 0), (0.12, 0), (0.13, 1), (0.62, 1), (0.63, 2), (0.88, 3), (0.999, 3)):
        assert plain_opt.sample_row(s, u) == tok
    assert plain_opt.sample_row(s, 0.999, top_k=1) == 1                          # top_k 1 is argmax
    assert plain_opt.sample_row(s, 0.9, temperature=0.05) == 1                   # temperature -> 0+ is argmax
    assert plain_opt.sample_row(s, 0.9, top_k=2) == 2                            # within the top k only


def test_draw_slack():
    """The yardstick for samplers that round differently: zero for the token `sample_row` draws, the distance
    to the token's stretch for any other, and both numbers of kept tokens count where top-p's sum lies on a
    threshold."""
    s = torch.log(torch.tensor([0.125, 0.5, 0.25, 0.125]))
    assert plain_opt.draw_slack(s, 0.3, 1)[0] == 0.0
    assert abs(plain_opt.draw_slack(s, 0.3, 0)[0]- 0.175) < 1e-6             # token 0 ends at .125
    assert abs(plain_opt.draw_slack(s, 0.3, 2)[0] - 0.325) < 1e-6             # token 2 begins at .625
    assert plain_opt.draw_slack(s, 0.3, 3, top_k=2)[0] == float("inf")         # not kept at all
    assert plain_opt.draw_slack(s, 0.3, 1)[1] == 4 * 2.0 ** -23 + 4 * 2.0 ** -40
    # top-p .75 exactly: tokens 1 and 2 hold .75, so token 0 (first of two at .125, ties to the lower id) may
    # stay or go; with it u = .1 draws token 0, without it token 1; token 3 stays out either way
    assert plain_opt.draw_slack(s, 0.1, 0, top_p=0.75)[0] == 0.0
    assert plain_opt.draw_slack(s, 0.1, 1, top_p=0.75)[0] == 0.0
    assert plain_opt.draw_slack(s, 0.99, 3, top_p=0.75)[0] == float("inf")
    assert plain_opt.draw_slack(s, 0.1, 1, top_p=0.76)[0] > 0.01
    g = torch.Generator().manual_seed(0)
    for t in range(60):
        row = torch.randn(int(torch.randint(2, 2000, (1,), generator=g)), generator=g) * 3
        u = float(torch.rand(1, generator=g))
        k, p, temp, least = [None, 5, 50][t % 3], [None, 0.9, 0.5, 0.05][t % 4], [1.0, 0.3, 1.5][t % 3], [1, 3][t % 2]
        tok = plain_opt.sample_row(row, u, k, p, temp, least)
        slack, bound = plain_opt.draw_slack(row, u, tok, k, p, temp, least)
        assert slack <= bound < 1e-6


def test_philox_known_answers():
    """Known-answer vectors of Philox-4x32-10 (Random123's kat_vectors): counter and key all zero give
    6627e8d5 as the first word; all ones give 408f276d."""
    def first_word(counter4, key2):
        m0, m1, w0, w1, mask = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85, 0xFFFFFFFF
        c, k = list(counter4), list(key2)
        for _ in range(10):
            p0, p1 = m0 * c[0], m1 * c[2]
            c = [((p1 >> 32) ^ c[1] ^ k[0]) & mask, p1 & mask, ((p0 >> 32) ^ c[3] ^ k[1]) & mask, p0 & mask]
            k = [(k[0] + w0) & mask, (k[1] + w1) & mask]
        return c[0]
    assert first_word([0, 0, 0, 0], [0, 0]) == 0x6627E8D5
    assert first_word([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2) == 0x408F276D
    # the function under test is that generator with (counter, 0, 0) and the seed as key
    assert plain_opt.philox_uniform(0, 0) == (0x6627E8D5 >> 8) / (1 << 24)
    us = [plain_opt.philox_uniform(12345, n) for n in range(2000)]
    assert 0.0 <= min(us) and max(us) < 1.0 and abs(sum(us) / 2000 - 0.5) < 0.03
    assert plain_opt.philox_uniform(1, 5) != plain_opt.philox_uniform(2, 5)


def test_greedy_is_argmax_of_the_last_position():
    w = plain_opt.random_weights(TINY_A, 3)
    out = plain_opt.greedy(w, TINY_A, [5, 9, 11], 4)
    assert out[:3] == [5, 9, 11] and len(out) == 7
    assert out[3] == int(plain_opt.forward_logits(w, TINY_A, [5, 9, 11])[-1].argmax())
    assert out[4] == int(plain_opt.forward_logits(w, TINY_A, out[:4])[-1].argmax())


def _constant_norm(w, name, width, value):
    """A norm whose output is the same vector for every token: weight 0, bias `value`."""
    w[name + ".weight"] = torch.zeros(width)
    w[name + ".bias"] = value.clone()


def test_which_norm_feeds_which_half():
    """Pins the composition of a block from outside its own text. A norm with weight 0 and bias c hands the
    same vector c to whatever it feeds. Pre-norm: with `self_attn_layer_norm` made so, every token's query,
    key and value are those of c, attention averages equal values, and the first half adds one and the same
    vector out_proj(v_proj(c)) to every token, which library routines give; with `final_layer_norm` made so
    the second half adds fc2(act(fc1(c))). If the norms were exchanged, or a half read the stream instead of
    its norm, neither would hold."""
    cfg = dict(TINY_A)
    p = "model.decoder.layers.0."
    g = torch.Generator().manual_seed(7)
    x = torch.randn(9, 64, generator=g)
    c = torch.randn(64, generator=g)
    lin = torch.nn.functional.linear
    # the first half
    w = plain_opt.random_weights(cfg, 3)
    _constant_norm(w, p + "self_attn_layer_norm", 64, c)
    for k in ("fc1.weight", "fc2.weight", "fc1.bias", "fc2.bias"):
        w[p + k] = torch.zeros_like(w[p + k])                     # the second half adds nothing
    added = lin(lin(c, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"]),
                w[p + "self_attn.out_proj.weight"], w[p + "self_attn.out_proj.bias"])
    torch.testing.assert_close(plain_opt.block(x, w, cfg, 0), x + added, rtol=1e-5, atol=1e-5)
    # the second half
    w = plain_opt.random_weights(cfg, 3)
    _constant_norm(w, p + "final_layer_norm", 64, c)
    for k in ("q_proj", "k_proj", "v_proj", "out_proj"):
        w[p + f"self_attn.{k}.weight"] = torch.zeros_like(w[p + f"self_attn.{k}.weight"])
        w[p + f"self_attn.{k}.bias"] = torch.zeros_like(w[p + f"self_attn.{k}.bias"])
    added = lin(torch.relu(lin(c, w[p + "fc1.weight"], w[p + "fc1.bias"])), w[p + "fc2.weight"], w[p + "fc2.bias"])
    torch.testing.assert_close(plain_opt.block(x, w, cfg, 0), x + added, rtol=1e-5, atol=1e-5)


def test_post_norm_order_and_no_norm_before_the_head():
    """Post-norm: the stream after the first half is that half's norm, so with that norm constant the second
    half sees c alone and the block's output is norm2(c + ffn(c)) for every token; and with the last block's
    second norm constant the logits are the head of c, nothing in between (no further norm: a post-norm
    model has none before its head)."""
    cfg = dict(TINY_B)
    width = cfg["hidden_size"]
    affine = dict(cfg, layer_norm_elementwise_affine=True)        # so that the norms have parameters to set
    w = plain_opt.random_weights(affine, 4)
    p = "model.decoder.layers.0."
    g = torch.Generator().manual_seed(8)
    x = torch.randn(7, width, generator=g)
    c = torch.randn(width, generator=g)
    lin = torch.nn.functional.linear
    _constant_norm(w, p + "self_attn_layer_norm", width, c)
    inner = torch.nn.functional.gelu(lin(c, w[p + "fc1.weight"]))
    want = torch.nn.functional.layer_norm(c + lin(inner, w[p + "fc2.weight"]), (width,),
                                          w[p + "final_layer_norm.weight"], w[p + "final_layer_norm.bias"],
                                          cfg["layer_norm_eps"])
    got = plain_opt.block(x, w, affine, 0)
    torch.testing.assert_close(got, want.expand_as(got), rtol=1e-5, atol=1e-5)
    # the head
    last = f"model.decoder.layers.{cfg['num_hidden_layers'] - 1}."
    w = plain_opt.random_weights(affine, 4)
    _constant_norm(w, last + "final_layer_norm", width, c)
    logits = plain_opt.forward_logits(w, affine, [5, 9, 300, 4])
    want = lin(lin(c, w["model.decoder.project_out.weight"]), w["model.decoder.embed_tokens.weight"])
    torch.testing.assert_close(logits, want.expand_as(logits), rtol=1e-5, atol=1e-5)


def test_pre_norm_head_norms_the_stream_once():
    """Pre-norm: the logits are head(final_layer_norm(stream)); with that norm constant they are the head of
    c, and with all blocks adding nothing and the norm real they are the head of the normed embedding."""
    cfg = dict(TINY_A)
    w = plain_opt.random_weights(cfg, 5)
    g = torch.Generator().manual_seed(9)
    c = torch.randn(64, generator=g)
    lin = torch.nn.functional.linear
    w1 = dict(w)
    _constant_norm(w1, "model.decoder.final_layer_norm", 64, c)
    logits = plain_opt.forward_logits(w1, cfg, [5, 9, 300])
    torch.testing.assert_close(logits, lin(c, w["model.decoder.embed_tokens.weight"]).expand_as(logits),
                               rtol=1e-5, atol=1e-5)
    wz = {k: (torch.zeros_like(v) if (".layers." in k and ("proj" in k or "fc" in k)) else v) for k, v in w.items()}
    toks = torch.tensor([5, 9, 300])
    x = w["model.decoder.embed_tokens.weight"][toks] + w["model.decoder.embed_positions.weight"][2:5]
    want = lin(torch.nn.functional.layer_norm(x, (64,), w["model.decoder.final_layer_norm.weight"],
                                              w["model.decoder.final_layer_norm.bias"], 1e-5),
               w["model.decoder.embed_tokens.weight"])
    torch.testing.assert_close(plain_opt.forward_logits(wz, cfg, toks.tolist()), want, rtol=1e-5, atol=1e-5)


def test_ngram_ban_by_hand():
    """What pins it beside the reference's text: cases small enough to read. After `1 2 3 1 2` a 3 would
    repeat `1 2 3`; with n = 2 every token that ever followed a 2; with n = 1 every token seen; a sequence
    shorter than n - 1 bans nothing; and the product's own function says the same on random rows."""
    from transformers_neuronx_amd.sampling.sampler import banned_ngram_tokens
    assert plain_opt.banned_by_ngrams([1, 2, 3, 1, 2], 3) == [3]
    assert plain_opt.banned_by_ngrams([1, 2, 3, 1, 2, 4, 2], 2) == [3, 4]
    assert sorted(set(plain_opt.banned_by_ngrams([5, 6, 5], 1))) == [5, 6]
    assert plain_opt.banned_by_ngrams([7], 3) == [] and plain_opt.banned_by_ngrams([7, 8], 3) == []
    assert plain_opt.banned_by_ngrams([7, 8, 9], 4) == []           # the one run of four would need a fourth token
    g = torch.Generator().manual_seed(0)
    for n in (1, 2, 3, 4):
        for _ in range(50):
            row = torch.randint(0, 4, (int(torch.randint(0, 30, (1,), generator=g)),), generator=g).tolist()
            assert sorted(banned_ngram_tokens(row, n)) == sorted(plain_opt.banned_by_ngrams(row, n)), (row, n)
