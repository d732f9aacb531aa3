"""A plain, slow OPT: whole sequences, no cache, no batching, one function per part.

It is written from the formulas in the reference (paths below are relative to
the reference's package folder `src/transformers_neuronx/`) and shares no code with the
package under test. It takes the model as a dict of config.json keys and a dict
of tensors by checkpoint name, and works in any floating dtype (float32 by
default; float64 to tell which of two float32 results is the more exact).

Parts that the reference does not have (post-norm order, project_in/out, no
bias, no affine norm, erf GELU) follow the definitions stated in each function.
"""
import math

import torch


def layer_norm(x, weight, bias, eps):
    """hlo.py:84-105 (`layer_norm`) through hlo.py:51-81 (`batch_norm`, eps default 1e-5):
    per token, mean and biased variance over the hidden axis in float, then
    `(x - mean) / sqrt(var + eps)`, times weight, plus bias. Without affine
    parameters (not in the reference) the last two steps are left out."""
    mean = x.mean(dim=-1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    y = (x - mean) / torch.sqrt(var + eps)
    if weight is not None:
        y = y * weight
    if bias is not None:
        y = y + bias
    return y


def linear(x, weight, bias=None):
    """hlo.py:336-407 (`dot00_add1` and friends) with checkpoint weights `[out, in]`
    (transposes at opt/model.py:100-126): `x @ weight.T + bias`."""
    y = x @ weight.transpose(0, 1)
    if bias is not None:
        y = y + bias
    return y


def activation(x, name):
    """activations.py:43-48 relu = max(x, 0); activations.py:20-40 gelu_new =
    0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))). "gelu" (erf form,
    0.5 x (1 + erf(x / sqrt 2))) is not in the reference; OPT's config names it."""
    if name == "relu":
        return torch.maximum(x, torch.zeros_like(x))
    if name == "gelu_new":
        inner = math.sqrt(2.0 / math.pi) * (x + 0.044715 * x * x * x)
        return 0.5 * x * (1.0 + torch.tanh(inner))
    if name == "gelu":
        return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))
    raise ValueError(name)


def learned_positions(table, n_tokens, offset=2, start=0):
    """opt/model.py:232-244 (`OPTLearnedPositionalEmbedding`, offset 2) with
    decoder.py:562-572 (position = cache id - start id, clamped at 0): row
    `position + 2` of the table for positions start .. start + n - 1."""
    ids = torch.arange(start, start + n_tokens) + offset
    return table[ids]


def causal_attention(q, k, v, n_heads, window=None):
    """opt/model.py:444-521, multi-token branch: `Q / sqrt(d_head)`
    (layers/attention.py:428-437), `S = Q K^T` per head (:440-476), keys `j > i`
    masked out (hlo.py:1030-1042; the reference selects -30000, which after the
    softmax is 0 to float precision, so they are simply left out here), softmax
    in float over keys (hlo.py:880-904), times V (layers/attention.py:707-788).
    `q`, `k`, `v` are `[S, n_heads * d_head]`. `window`, when given, keeps keys
    `j > i - window` only (sliding window of the reference's sparse masks)."""
    s, hidden = q.shape
    d = hidden // n_heads
    n_kv = k.shape[1] // d
    out = torch.zeros_like(q)
    for h in range(n_heads):
        hk = h // (n_heads // n_kv)
        qh = q[:, h * d:(h + 1) * d] / math.sqrt(d)
        kh = k[:, hk * d:(hk + 1) * d]
        vh = v[:, hk * d:(hk + 1) * d]
        for i in range(s):
            lo = 0 if window is None else max(0, i - window + 1)
            scores = kh[lo:i + 1] @ qh[i]
            p = torch.softmax(scores, dim=0)
            out[i, h * d:(h + 1) * d] = p @ vh[lo:i + 1]
    return out


def decode_attention_two_part(q, k_prior, v_prior, k_new, v_new):
    """layers/attention.py:592-704 (`context`) for one head and one new token:
    prior scores over the cache and one active score share a maximum; the
    denominator is the sum of both parts (opt/model.py:483-500). `q` is already
    scaled. Used to pin that this equals one softmax over all keys."""
    sp = k_prior @ q
    sa = (k_new * q).sum()
    m = torch.maximum(sp.max(), sa) if sp.numel() else sa
    pp = torch.exp(sp - m)
    pa = torch.exp(sa - m)
    denom = pp.sum() + pa
    return (pp @ v_prior + pa * v_new) / denom


def attention_part(x, w, prefix, n_heads, bias=True):
    """opt/model.py:444-523: q, k, v projections with bias, attention, output
    projection with bias (layers/attention.py:791-914)."""
    def b(name):
        return w[prefix + name + ".bias"] if bias else None
    q = linear(x, w[prefix + "q_proj.weight"], b("q_proj"))
    k = linear(x, w[prefix + "k_proj.weight"], b("k_proj"))
    v = linear(x, w[prefix + "v_proj.weight"], b("v_proj"))
    c = causal_attention(q, k, v, n_heads)
    return linear(c, w[prefix + "out_proj.weight"], b("out_proj"))


def feed_forward_part(x, w, prefix, act, bias=True):
    """hlo.py:550-559 (`mlp`): fc1 with bias, activation, fc2 with bias."""
    h = linear(x, w[prefix + "fc1.weight"], w[prefix + "fc1.bias"] if bias else None)
    h = activation(h, act)
    return linear(h, w[prefix + "fc2.weight"], w[prefix + "fc2.bias"] if bias else None)


def _norm_params(w, name, affine):
    if not affine:
        return None, None
    return w[name + ".weight"], w[name + ".bias"]


def block(x, w, cfg, i):
    """opt/model.py:351-375: pre-norm order `x = x + Attn(LN(x))`,
    `x = x + FFN(LN(x))`. Post-norm order (`do_layer_norm_before` false; the
    reference refuses it at opt/config.py:23-24) is defined here as
    `x = LN(x + Attn(x))`, `x = LN(x + FFN(x))` with the same tensors."""
    p = f"model.decoder.layers.{i}."
    eps = cfg.get("layer_norm_eps", 1e-5)
    affine = cfg.get("layer_norm_elementwise_affine", True)
    bias = cfg.get("enable_bias", True)
    n1 = _norm_params(w, p + "self_attn_layer_norm", affine)
    n2 = _norm_params(w, p + "final_layer_norm", affine)
    if cfg.get("do_layer_norm_before", True):
        x = x + attention_part(layer_norm(x, *n1, eps), w, p + "self_attn.", cfg["num_attention_heads"], bias)
        x = x + feed_forward_part(layer_norm(x, *n2, eps), w, p, cfg["activation_function"], bias)
    else:
        x = layer_norm(x + attention_part(x, w, p + "self_attn.", cfg["num_attention_heads"], bias), *n1, eps)
        x = layer_norm(x + feed_forward_part(x, w, p, cfg["activation_function"], bias), *n2, eps)
    return x


def embed(tokens, w, cfg):
    """opt/model.py:162-166: token rows plus learned position rows. With
    `word_embed_proj_dim != hidden_size` (read at opt/config.py:34, never used by
    the reference) the token rows go through `project_in` (no bias) first and the
    positions are added in the hidden width."""
    x = w["model.decoder.embed_tokens.weight"][tokens]
    if cfg.get("word_embed_proj_dim", cfg["hidden_size"]) != cfg["hidden_size"]:
        x = linear(x, w["model.decoder.project_in.weight"])
    return x + learned_positions(w["model.decoder.embed_positions.weight"], len(tokens))


def head(x, w, cfg):
    """layers/transformer.py:196-208: final LayerNorm, then logits with the
    `[vocab, width]` head weight, which is the token table when absent
    (opt/model.py:204-205). The final norm exists in pre-norm order only, and not
    when the configuration's `_remove_final_layer_norm` (a key the reference lists,
    opt/gen_random_pretrained.py:114, and never reads) is true: parity unpinned for
    that key; `project_out` (no bias) comes before the head when the widths differ."""
    if cfg.get("do_layer_norm_before", True) and not cfg.get("_remove_final_layer_norm", False):
        g, b = _norm_params(w, "model.decoder.final_layer_norm", cfg.get("layer_norm_elementwise_affine", True))
        x = layer_norm(x, g, b, cfg.get("layer_norm_eps", 1e-5))
    if cfg.get("word_embed_proj_dim", cfg["hidden_size"]) != cfg["hidden_size"]:
        x = linear(x, w["model.decoder.project_out.weight"])
    lm = w.get("lm_head.weight", w["model.decoder.embed_tokens.weight"])
    return linear(x, lm)


def forward_logits(w, cfg, tokens, dtype=torch.float32, layer_order=None):
    """Logits `[S, vocab]` at every position of one whole sequence.
    `layer_order` lists the layers in the order they run (default 0..L-1)."""
    w = {k: v.to(dtype) for k, v in w.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = embed(tokens, w, cfg)
    for i in (range(cfg["num_hidden_layers"]) if layer_order is None else layer_order):
        x = block(x, w, cfg, i)
    return head(x, w, cfg)


def greedy(w, cfg, prompt, n_new, dtype=torch.float32):
    """sampling.py:108-128 (`sample_greedy`): argmax of the last position, append,
    run again (here: the whole sequence again, there being no cache)."""
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward_logits(w, cfg, tokens, dtype)[-1].argmax()))
    return tokens


# ---------------------------------------------------------------- sampling

def filter_top_k_top_p(scores, top_k=None, top_p=None, min_tokens_to_keep=1):
    """sampling.py:199-264 (`top_k_top_p_filtering`) for one row: returns the
    kept `(values, indices)` in descending order of value. Top-k keeps the k
    largest (:210-211, k clamped to the row, :204-205); top-p keeps, of what is
    left, the shortest prefix whose softmax mass reaches `top_p`: the mask
    `cumulative < top_p` shifted right by one (:221-230)."""
    n = scores.numel()
    values, indices = torch.sort(scores.float(), descending=True, stable=True)
    if top_k is not None:
        k = min(max(top_k, min_tokens_to_keep), n)
        values, indices = values[:k], indices[:k]
    if top_p is not None and top_p < 1.0:
        cum = torch.cumsum(torch.softmax(values, dim=-1, dtype=torch.float32), dim=-1)
        mask = cum < top_p
        mask = torch.cat([torch.ones(1, dtype=torch.bool), mask[:-1]])
        mask[:min_tokens_to_keep] = True
        values, indices = values[mask], indices[mask]
    return values, indices


def sample_row(scores, u, top_k=None, top_p=None, temperature=1.0, min_tokens_to_keep=1):
    """sampling.py:337-345: divide by the temperature, filter, softmax over what
    is kept in float (:343), draw one. The draw is by inverse CDF with a given
    uniform `u` in [0, 1) over the kept tokens in ascending order of token id
    (hlo.py:2422-2467 draws by counting `u > cumsum / total` too); the reference's
    host loop uses `torch.multinomial`, whose stream cannot be reproduced, so
    only the distribution is comparable with it."""
    values, indices = filter_top_k_top_p(scores.float() / temperature, top_k, top_p, min_tokens_to_keep)
    order = torch.argsort(indices)
    values, indices = values[order], indices[order]
    probs = torch.softmax(values.double(), dim=-1)
    cum = torch.cumsum(probs, dim=-1)
    pick = int((cum <= u * cum[-1]).sum())
    return int(indices[min(pick, len(indices) - 1)])


def draw_slack(scores, u, token, top_k=None, top_p=None, temperature=1.0, min_tokens_to_keep=1):
    """How far outside `token`'s stretch of the line [0, 1) the drawn point `u` lies, and the bound that float32
    rounding puts on that: `(slack, bound)`, slack 0 where `sample_row` computed without any rounding draws
    `token`. The bound is derived, not chosen: a float32 weight exp(x/T - max/T) is within 2 units of 2^-23
    of the exact one (the library's exponential one, the subtraction another), so a sum of weights divided by
    the whole sum is within 4 * 2^-23 of the exact ratio, whatever the number of tokens; a sampler that adds
    weights as whole numbers of 2^-40 adds 2^-40 a kept token. The same bound decides which numbers of kept
    tokens top-p may arrive at: a token with a mass above it that close to `top_p` may stay or go, and every
    such number is tried (sampling.py:213-249 compares float32 sums, which carry the same rounding)."""
    values, indices = torch.sort(scores.float() / temperature, descending=True, stable=True)
    if top_k is not None:
        k = min(max(top_k, min_tokens_to_keep), values.numel())
        values, indices = values[:k], indices[:k]
    exact = torch.softmax(values.double(), -1)
    n = values.numel()
    bound = 4 * 2.0 ** -23 + n * 2.0 ** -40
    counts = [n]
    if top_p is not None and top_p < 1.0:
        above = torch.cumsum(exact, -1) - exact                    # the mass of the tokens before each one
        fewest = max(int((above < top_p - bound).sum()), min_tokens_to_keep, 1)
        most = max(int((above < top_p + bound).sum()), min_tokens_to_keep, 1)
        counts = list(range(fewest, min(most, n) + 1))
    best = float("inf")
    for count in counts:
        ids, order = torch.sort(indices[:count])
        at = int(torch.searchsorted(ids, token))
        if at >= count or int(ids[at]) != token:
            continue
        mass = exact[:count][order]
        cum = torch.cumsum(mass, -1)
        low, high = float(cum[at] - mass[at]) / float(cum[-1]), float(cum[at]) / float(cum[-1])
        best = min(best, max(low - u, u - high, 0.0))
    return best, bound


def banned_by_ngrams(tokens, n):
    """sampling.py:267-300 for one row: every run of `n` tokens in `tokens` is filed under its first n - 1
    (:275-277); with fewer than n - 1 tokens nothing is banned (:292-294); otherwise the tokens filed under
    the last n - 1 (:284-286) may not come next."""
    tokens = list(tokens)
    if len(tokens) + 1 < n:
        return []
    filed = {}
    for start in range(len(tokens) - n + 1):
        run = tokens[start:start + n]
        filed.setdefault(tuple(run[:-1]), []).append(run[-1])
    return filed.get(tuple(tokens[len(tokens) + 1 - n:]), [])


def philox_uniform(seed, counter):
    """Philox-4x32-10 (Salmon et al., 2011, public algorithm) keyed by the
    request's seed, counter = the request's step; first output word mapped to
    [0, 1) by `(word >> 8) * 2^-24`."""
    m0, m1 = 0xD2511F53, 0xCD9E8D57
    w0, w1 = 0x9E3779B9, 0xBB67AE85
    mask = 0xFFFFFFFF
    c = [counter & mask, (counter >> 32) & mask, 0, 0]
    k = [seed & mask, (seed >> 32) & mask]
    for _ in range(10):
        p0 = m0 * c[0]
        p1 = m1 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & mask, p1 & mask, ((p0 >> 32) ^ c[3] ^ k[1]) & mask, p0 & mask]
        k = [(k[0] + w0) & mask, (k[1] + w1) & mask]
    return (c[0] >> 8) * (1.0 / (1 << 24))


# ---------------------------------------------------------------- weights

def random_weights(cfg, seed, dtype=torch.float32):
    """A set of tensors by checkpoint name (names and shapes:
    opt/gen_random_pretrained.py:49-76) for tests of this file alone: normal with
    the config's init_std; norm weights around one."""
    g = torch.Generator().manual_seed(seed)
    std = cfg.get("init_std", 0.02)
    h, e = cfg["hidden_size"], cfg.get("word_embed_proj_dim", cfg["hidden_size"])
    f, v, p = cfg["ffn_dim"], cfg["vocab_size"], cfg["max_position_embeddings"]
    bias = cfg.get("enable_bias", True)
    affine = cfg.get("layer_norm_elementwise_affine", True)
    w = {}

    def normal(name, *shape, mean=0.0):
        w[name] = (mean + std * torch.randn(*shape, generator=g)).to(dtype)

    def norm(name):
        if affine:
            normal(name + ".weight", h, mean=1.0)
            normal(name + ".bias", h)

    normal("model.decoder.embed_tokens.weight", v, e)
    normal("model.decoder.embed_positions.weight", p + 2, h)
    if e != h:
        normal("model.decoder.project_in.weight", h, e)
        normal("model.decoder.project_out.weight", e, h)
    if cfg.get("do_layer_norm_before", True):
        norm("model.decoder.final_layer_norm")
    for i in range(cfg["num_hidden_layers"]):
        pre = f"model.decoder.layers.{i}."
        for proj in ("q_proj", "k_proj", "v_proj", "out_proj"):
            normal(pre + f"self_attn.{proj}.weight", h, h)
            if bias:
                normal(pre + f"self_attn.{proj}.bias", h)
        norm(pre + "self_attn_layer_norm")
        normal(pre + "fc1.weight", f, h)
        normal(pre + "fc2.weight", h, f)
        if bias:
            normal(pre + "fc1.bias", f)
            normal(pre + "fc2.bias", h)
        norm(pre + "final_layer_norm")
    return w
