"""The bfloat16-only kernels on inputs whose results are exact: no tolerance hides a slip.

The matrix-unit kernels have no float32 form to be compared in, and random inputs let them be compared at a
hundredth only: one key of 2,000 left out, or one step of the inner dimension skipped, passes that. Here the
inputs are small integers and powers of two, so that every product and every sum is exact in float32 and the
result is exact in bfloat16: a product of integers in [-4, 4] (sums below 2^24), and attention whose every
query ties exactly two keys far above all others, so that its output is the mean of two integer value rows.
Everything is compared at 1e-6.
"""
import numpy as np
import pytest
import torch

from test_kernels_gpu import DEV, _make_step, _ops

pytestmark = pytest.mark.gpu

EXACT = dict(rtol=0.0, atol=1e-6)


def _ints(g, *shape, low=-4, high=4):
    return torch.randint(low, high + 1, shape, device=DEV, generator=g).float()


def _apart(pages, pad):
    """The same pages with `pad` elements between one page and the next, as a cache with `page_pad_bytes` lays
    them out; what lies between them is NaN."""
    n = pages.shape[0]
    count = pages[0].numel()
    whole = torch.full((n, count + pad), float("nan"), dtype=pages.dtype, device=pages.device)
    whole[:, :count] = pages.reshape(n, count)
    return whole[:, :count].view(pages.shape)


# ---------------------------------------------------------------- products

def _exact_product(x, w, bias, residual, act, out_dtype):
    y = x.double() @ w.double().t()
    if bias is not None:
        y = y + bias.double()
    if act == "relu":
        y = y.clamp_min(0)
    if residual is not None:
        y = y + residual.double()
    assert float(y.abs().max()) < 2 ** 24
    return y.float().to(out_dtype)


PRODUCT_CASES = [
    # rows, columns, inner size, which way the product goes
    (1, 256, 4096, "few"), (8, 4096, 4096, "few"), (16, 12288, 1024, "few"), (13, 1000, 264, "few"),
    (32, 512, 2048, "few"), (24, 4096, 16384, "few"),
    (40, 4096, 4096, "some"), (64, 1024, 16384, "some"), (128, 256, 2048, "some"), (17, 4096, 4096, "some"),
    (64, 4096, 4096, "library"), (300, 1024, 2048, "library"), (2048, 512, 4096, "library"),
    (256, 1024, 4096, "wide"), (700, 520, 1024, "wide"), (2048, 4096, 1024, "wide"), (130, 264, 136, "wide"),
]


@pytest.mark.parametrize("m,n,k,way", PRODUCT_CASES)
def test_products_of_small_integers_are_exact(m, n, k, way):
    hip, _ = _ops(torch.bfloat16)
    if way == "wide" or way == "few":
        hip.library_rows = 0            # our own kernels at every row count
    if way != "some":
        hip.some_rows = False
    g = torch.Generator(device=DEV).manual_seed(m + 3 * n + 7 * k)
    x, w = _ints(g, m, k).to(torch.bfloat16), _ints(g, n, k).to(torch.bfloat16)
    bias, residual = _ints(g, n, low=-64, high=64), _ints(g, m, n, low=-1000, high=1000)
    pw = hip.prepare_weight(w)
    assert (pw.tiles is not None) == (n % 16 == 0 and k % 128 == 0)
    if way == "some":
        assert hip._some_rows_product(m, n, k, w, pw.tiles, residual, True, False)
    if way == "library":
        assert hip._library_product(m, n, k, w, False)
    for weight in (pw, w):
        # what ends in the residual sum (float32), what a bfloat16 part reads next (with and without ReLU)
        got = hip.linear(x, weight, bias, residual=residual, out_f32=True)
        torch.testing.assert_close(got, _exact_product(x, w, bias, residual, None, torch.float32), **EXACT)
        for act in (None, "relu"):
            got = hip.linear(x, weight, bias, act=act)
            torch.testing.assert_close(got.float(), _exact_product(x, w, bias, None, act, torch.bfloat16).float(), **EXACT)
        got = hip.linear(x, weight, None, out_f32=True)
        torch.testing.assert_close(got, _exact_product(x, w, None, None, None, torch.float32), **EXACT)
    # one weight element changed by one unit of its last place shows: the comparison can fail
    w2 = w.clone()
    w2[n // 2, k - 1] += 1
    x_on = x.clone()
    x_on[:, k - 1] = 1
    got = hip.linear(x_on, hip.prepare_weight(w2), None, out_f32=True)
    want = _exact_product(x_on, w, None, None, None, torch.float32)
    assert float((got - want).abs().max()) == 1.0


@pytest.mark.parametrize("m", [1, 8, 16, 40])
def test_fused_projection_of_small_integers_is_exact(m):
    """The query/key/value projection that scatters its result: queries scaled by a power of two into a dense
    matrix, keys and values into their pages (values transposed inside a page)."""
    hip, _ = _ops(torch.bfloat16)
    heads, kv, hs, ps, k = 4, 2, 64, 16, 512
    g = torch.Generator(device=DEV).manual_seed(m)
    cached = [int(c) for c in torch.randint(0, 60, (m,), generator=torch.Generator().manual_seed(m))]
    num_pages = sum(-(-(c + 1) // ps) for c in cached) + 2
    ctx = _make_step([1] * m, cached, ps, num_pages, seed=m)
    view = ctx.groups["full"]
    n = (heads + 2 * kv) * hs
    x, w, bias = _ints(g, m, k).to(torch.bfloat16), _ints(g, n, k).to(torch.bfloat16), _ints(g, n, low=-64, high=64)
    kp = _apart(torch.full((num_pages, kv, ps, hs), float("nan"), device=DEV, dtype=torch.bfloat16), 8 * m)
    vp = _apart(torch.full((num_pages, kv, hs, ps), float("nan"), device=DEV, dtype=torch.bfloat16), 8 * m)
    q = hip.qkv_project(x, hip.prepare_weight(w), bias, heads, kv, hs, 0.125, ctx, view, kp, vp)
    full = x.double() @ w.double().t() + bias.double()
    torch.testing.assert_close(q.float(), (full[:, :heads * hs] * 0.125).float().to(torch.bfloat16).float(), **EXACT)
    table = view.block_table.cpu()
    for i, c in enumerate(cached):
        page, at = int(table[i, c // ps]), c % ps
        want_k = full[i, heads * hs:(heads + kv) * hs].float().to(torch.bfloat16).float().view(kv, hs)
        want_v = full[i, (heads + kv) * hs:].float().to(torch.bfloat16).float().view(kv, hs)
        torch.testing.assert_close(kp[page, :, at, :].float(), want_k, **EXACT)
        torch.testing.assert_close(vp[page, :, :, at].float(), want_v, **EXACT)
    assert int((~torch.isnan(kp.float())).sum()) == m * kv * hs            # and nothing else was written


@pytest.mark.parametrize("m,own", [(1, True), (8, True), (16, True), (30, True), (64, True), (100, True), (200, True), (40, False),
                                   (300, False)])
@pytest.mark.parametrize("normed", [False, True])
def test_projection_that_turns_pairs_is_exact(m, own, normed):
    """Pairwise tables handed to the projection: element d of every query and key head becomes
    a[p, d] x[d] + b[p, d] x[d ^ 1] at the token's position p, bias added, before the query's scale; values stay.
    Integers throughout, on every way the projection can go: the fused product of few rows (with the tile-ordered
    weight and without), our product of many rows, the library's product with the scatter after it."""
    hip, ref = _ops(torch.bfloat16)
    if own:
        hip.library_rows = 0
    heads, kv, hs, ps, k = 3, 1, 32, 16, 256
    g = torch.Generator(device=DEV).manual_seed(m)
    cached = [int(c) for c in torch.randint(0, 90, (m,), generator=torch.Generator().manual_seed(m))]
    num_pages = sum(-(-(c + 1) // ps) for c in cached) + 2
    ctx = _make_step([1] * m, cached, ps, num_pages, seed=m)
    view = ctx.groups["full"]
    n = (heads + 2 * kv) * hs
    x, w, bias = _ints(g, m, k, low=-2, high=2), _ints(g, n, k, low=-2, high=2).to(torch.bfloat16), _ints(g, n, low=-8, high=8)
    a, b = _ints(g, 100, hs, low=-2, high=2), _ints(g, 100, hs, low=-2, high=2)
    full = x.double() @ w.double().t() + bias.double()
    pos = torch.tensor(cached, device=DEV)
    turned = (heads + kv) * hs
    part = full[:, :turned].reshape(m, -1, hs)
    beside = part.reshape(m, -1, hs // 2, 2).flip(-1).reshape(m, -1, hs)
    part = (a[pos].double()[:, None] * part + b[pos].double()[:, None] * beside).reshape(m, turned)
    want_q = (part[:, :heads * hs] * 0.25).float().to(torch.bfloat16).float()
    want_k = part[:, heads * hs:].float().to(torch.bfloat16).float().view(m, kv, hs)
    want_v = full[:, turned:].float().to(torch.bfloat16).float().view(m, kv, hs)
    for weight in (hip.prepare_weight(w), w):
        kp = _apart(torch.full((num_pages, kv, ps, hs), float("nan"), device=DEV, dtype=torch.bfloat16), 64)
        vp = _apart(torch.full((num_pages, kv, hs, ps), float("nan"), device=DEV, dtype=torch.bfloat16), 64)
        h = x.to(torch.bfloat16)
        if normed:
            # a LayerNorm that changes nothing that matters here cannot be exact: the folded form is compared below
            break
        q = hip.qkv_project(h, weight, bias, heads, kv, hs, 0.25, ctx, view, kp, vp, turn=(a, b))
        torch.testing.assert_close(q.float(), want_q, **EXACT)
        table = view.block_table.cpu()
        for i, c in enumerate(cached):
            page, at = int(table[i, c // ps]), c % ps
            torch.testing.assert_close(kp[page, :, at, :].float(), want_k[i], **EXACT)
            torch.testing.assert_close(vp[page, :, :, at].float(), want_v[i], **EXACT)
    if normed and m <= 32:
        # behind a folded LayerNorm (not exact: against the torch rendition, which applies the same tables)
        gamma, beta = 1 + 0.2 * torch.randn(k, device=DEV, generator=g), 0.3 * torch.randn(k, device=DEV, generator=g)
        xs = torch.randn(m, k, device=DEV, generator=g) * 2 + 3
        wr = (torch.randn(n, k, device=DEV, generator=g) / 16).to(torch.bfloat16)
        pw = hip.prepare_weight(wr)
        assert hip.fold_norm(pw, gamma, beta)
        kp = torch.zeros(num_pages, kv, ps, hs, device=DEV, dtype=torch.bfloat16)
        vp = torch.zeros(num_pages, kv, hs, ps, device=DEV, dtype=torch.bfloat16)
        kp_r, vp_r = kp.clone(), vp.clone()
        q = hip.qkv_project(hip.layernorm_deferred(xs, gamma, beta, 1e-5, torch.bfloat16), pw, bias, heads, kv, hs, 0.25,
                            ctx, view, kp, vp, turn=(a, b))
        h_r = ref.layernorm(xs, gamma, beta, 1e-5, torch.bfloat16, False, True)[1]
        q_r = ref.qkv_project(h_r, wr, bias, heads, kv, hs, 0.25, ctx, view, kp_r, vp_r, turn=(a, b))
        scale = float(q_r.float().abs().max())
        assert float((q.float() - q_r.float()).abs().max()) <= 2e-2 * scale
        assert float((kp.float() - kp_r.float()).abs().max()) <= 2e-2 * float(kp_r.float().abs().max())
        assert torch.equal(kp == 0, kp_r == 0)


# ---------------------------------------------------------------- attention

def _coded_case(heads, kv, hs, ps, runs, cached, window, seed):
    """Pages, queries and the exact result of an attention step in which every (query, head) ties two keys.

    Key j of a request carries its position: dimension b is +1 or -1 by bit b of j; the other dimensions are 1.
    A query is 32 times the code of a key `a` it can see, with one bit left open (0 there), so that `a` and
    the key whose position differs from `a` in that bit score alike, 64 above every other key; on the other
    dimensions it holds small integers, which add the same to every score. Values are integers in [-4, 4].
    Where the partner is a key the query must not see (beyond its own position, or before its window) the
    result is `a`'s value row alone: a mask off by one shows as the mean of two rows."""
    rng = np.random.default_rng(seed)
    totals = [r + c for r, c in zip(runs, cached)]
    bits = max(1, int(max(totals) - 1).bit_length())
    assert bits <= hs
    num_pages = sum(-(-t // ps) for t in totals) + 3
    ctx = _make_step(runs, cached, ps, num_pages, seed=seed)
    table = ctx.groups["full"].block_table.cpu().numpy()
    kp = torch.full((num_pages, kv, ps, hs), float("nan"))
    vp = torch.full((num_pages, kv, hs, ps), float("nan"))
    values = []
    for i, total in enumerate(totals):
        pos = np.arange(total)
        code = np.ones((total, hs), dtype=np.float32)
        for b in range(bits):
            code[:, b] = np.where((pos >> b) & 1, 1.0, -1.0)
        vals = rng.integers(-4, 5, size=(kv, total, hs)).astype(np.float32)
        values.append(vals)
        for j in range(total):
            page, at = int(table[i, j // ps]), j % ps
            kp[page, :, at, :] = torch.from_numpy(code[j])
            vp[page, :, :, at] = torch.from_numpy(vals[:, j, :])
    q = np.zeros((sum(runs), heads, hs), dtype=np.float32)
    want = np.zeros((sum(runs), heads, hs), dtype=np.float32)
    t = 0
    edges = 0
    for i, (run, c) in enumerate(zip(runs, cached)):
        for s in range(run):
            pos = c + s
            low = max(0, pos - window + 1) if window else 0
            for h in range(heads):
                kind = rng.integers(0, 4)
                a = pos if kind == 0 else low if kind == 1 else int(rng.integers(low, pos + 1))
                open_bit = int(rng.integers(0, bits))
                if kind == 0:          # the query's own key, tied with the nearest key after it that the code reaches
                    open_bit = next((b for b in range(bits) if not (pos >> b) & 1), open_bit)
                elif kind == 1 and low > 0:       # the first key of the window, tied with the nearest before it
                    open_bit = next(b for b in range(bits) if (low >> b) & 1)
                partner = a ^ (1 << open_bit)
                row = values[i][h // (heads // kv)]
                if low <= partner <= pos:
                    want[t, h] = (row[a] + row[partner]) / 2
                else:
                    want[t, h] = row[a]
                    edges += partner == pos + 1 or partner == low - 1
                code = np.array([1.0 if (a >> b) & 1 else -1.0 for b in range(bits)], dtype=np.float32) * 32
                code[open_bit] = 0
                q[t, h, :bits] = code
                q[t, h, bits:] = rng.integers(-2, 3, size=hs - bits)
            t += 1
    to = lambda a: torch.from_numpy(a).reshape(a.shape[0], -1).to(DEV).to(torch.bfloat16)    # noqa: E731
    return ctx, to(q), kp.to(DEV).to(torch.bfloat16), vp.to(DEV).to(torch.bfloat16), to(want).float(), edges


CODED_CASES = [
    # heads, kv heads, head size, page size, runs, cached, window
    (2, 2, 128, 64, [700], [0], None),                       # a long prompt: the pipelined kernel, many tiles
    (4, 2, 64, 64, [300, 129], [40, 0], None),               # grouped heads, a run that starts inside a page
    (2, 2, 128, 64, [1, 1, 1], [1999, 255, 256], None),      # decoding over many tiles, at and around a 256 mark
    (3, 1, 64, 16, [1, 1, 200], [1023, 64, 100], None),      # small pages; decoding beside a prompt portion
    (2, 2, 80, 64, [1, 90], [600, 300], None),               # a head size that is no power of two
    (2, 2, 64, 64, [1, 140, 1], [500, 200, 63], 100),        # a window: both of its edges
    (2, 1, 128, 16, [60, 1], [70, 129], 40),
    (1, 1, 256, 16, [33, 1], [0, 200], None),
    (2, 2, 16, 16, [1, 30], [800, 0], None),                 # ten bits of position in a head of sixteen
    # heads that share keys and values are taken together when decoding: a group of 20 (16 and 4), of 8 at the
    # largest head size (one block's worth), of 8 over many tiles, of 5 with a window
    (40, 2, 64, 64, [1, 1], [700, 300], None),
    (24, 3, 256, 16, [1, 3], [300, 10], None),
    (8, 1, 128, 64, [1, 1, 1], [2000, 17, 255], None),
    (10, 2, 96, 32, [1, 1], [400, 90], 70),
]


@pytest.mark.parametrize("case", CODED_CASES)
def test_attention_with_two_tied_keys_is_exact(case):
    heads, kv, hs, ps, runs, cached, window = case
    hip, ref = _ops(torch.bfloat16)
    ctx, q, kp, vp, want, edges = _coded_case(heads, kv, hs, ps, runs, cached, window, seed=hs + len(runs))
    assert edges > 0, "no query of the case has its partner just outside what it may see"
    view = ctx.groups["full"]
    # the construction itself, by the torch rendition of the kernels
    torch.testing.assert_close(ref.attention(q, heads, kv, hs, ctx, view, kp, vp, window).float(), want, **EXACT)
    ways = {"default": {}, "one wave a query": dict(force_plain_attention=True),
            "prompts without staging": dict(prefill_direct=True), "staged, two sets": dict(prefill_direct=6),
            "staged, one set": dict(prefill_direct=7), "pipelined, one set": dict(prefill_direct=2),
            "pipelined, two sets": dict(prefill_direct=3),
            "decoding in many blocks": dict(decode_blocks_wanted=1 << 20), "decoding in one block": dict(decode_blocks_wanted=1),
            "decoding with eight waves": dict(decode_waves=8)}
    for name, settings in ways.items():
        ops = type(hip)(torch.bfloat16, DEV)
        for key, value in settings.items():
            setattr(ops, key, value)
        got = ops.attention(q, heads, kv, hs, ctx, view, kp, vp, window)
        worst = float((got.float() - want).abs().max())
        assert worst <= 1e-6, f"{name}: differs by {worst}"
        # and with the pages some way apart in memory, as the engine's cache lays them out
        got = ops.attention(q, heads, kv, hs, ctx, view, _apart(kp, 136), _apart(vp, 136), window)
        worst = float((got.float() - want).abs().max())
        assert worst <= 1e-6, f"{name}, pages apart: differs by {worst}"
    # the comparison can fail, and pages belong to whom the table says: one more in every value of the first
    # request's pages is one more in every result of that request and nothing in the others'
    pages = view.block_table[0][view.block_table[0] >= 0].long()
    vp[pages] += 1
    moved = hip.attention(q, heads, kv, hs, ctx, view, kp, vp, window).float() - want
    assert float((moved[:runs[0]] - 1).abs().max()) <= 1e-6
    assert len(runs) == 1 or float(moved[runs[0]:].abs().max()) <= 1e-6
