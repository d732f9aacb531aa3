"""Each HIP kernel alone against its plain torch rendition, at sizes other than the engine's."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"

# the planner that an attention mixer brings to every step of its model (the kernels launch by its plan)
from transformers_neuronx_amd.kernels.attention_plan import attention_plan  # noqa: E402
ATTENTION_PLAN = {"attention": attention_plan}


def _ops(dtype):
    from transformers_neuronx_amd.kernels.hip import HipOps
    from transformers_neuronx_amd.kernels.reference import ReferenceOps
    return HipOps(dtype, DEV), ReferenceOps(dtype, DEV)


def _tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width", [(1, 48), (7, 96), (33, 1000), (5, 4096), (3, 5000), (2, 13000)])
def test_layernorm(dtype, rows, width):
    hip, ref = _ops(dtype)
    g = torch.Generator(device=DEV).manual_seed(rows * 1000 + width)
    x = torch.randn(rows, width, device=DEV, generator=g) * 3 + 1.5
    w = torch.randn(width, device=DEV, generator=g)
    b = torch.randn(width, device=DEV, generator=g)
    for weight, bias in ((w, b), (None, None)):
        for eps in (1e-5, 1e-2):
            f_h, c_h = hip.layernorm(x, weight, bias, eps, dtype, True, True)
            f_r, c_r = ref.layernorm(x, weight, bias, eps, dtype, True, True)
            torch.testing.assert_close(f_h, f_r, rtol=2e-5, atol=2e-5)
            torch.testing.assert_close(c_h.float(), c_r.float(), **_tol(dtype))
    # library routine: torch's layer_norm
    f_h, _ = hip.layernorm(x, w, b, 1e-5, dtype, True, False)
    torch.testing.assert_close(f_h, torch.nn.functional.layer_norm(x, (width,), w, b, 1e-5), rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gather_embed_positions_cast(dtype):
    hip, ref = _ops(dtype)
    g = torch.Generator(device=DEV).manual_seed(3)
    table = torch.randn(777, 40, device=DEV, generator=g).to(dtype)
    pos_table = torch.randn(50, 40, device=DEV, generator=g).to(dtype)
    ids = torch.randint(0, 777, (19,), device=DEV, generator=g, dtype=torch.int32)
    pos = torch.randint(0, 47, (19,), device=DEV, generator=g, dtype=torch.int32)
    e_h, e_r = hip.embed(ids, table, dtype), ref.embed(ids, table, dtype)
    assert torch.equal(e_h, e_r)
    for want in (True, False):
        xf_h, xc_h = hip.add_positions(e_h, pos, pos_table, 3, dtype, want)
        xf_r, xc_r = ref.add_positions(e_r, pos, pos_table, 3, dtype, want)
        assert torch.equal(xf_h, xf_r)
        assert (xc_h is None) == (xc_r is None)
        if want:
            assert torch.equal(xc_h, xc_r)
    xf_h, xc_h = hip.to_stream(e_h, dtype, True)
    assert torch.equal(xf_h, e_r.float()) and torch.equal(xc_h, e_r)
    big = torch.randn(100003, device=DEV, generator=g)
    assert torch.equal(hip.cast(big, torch.bfloat16), big.to(torch.bfloat16))
    assert torch.equal(hip.cast(big.to(torch.bfloat16), torch.float32), big.to(torch.bfloat16).float())
    rows = torch.tensor([5, 0, 18, 5], device=DEV, dtype=torch.int32)
    assert torch.equal(hip.gather_rows(xf_h, rows), xf_h[rows.long()])


GEMM_SHAPES = [(1, 16, 8), (3, 50, 24), (8, 96, 96), (17, 1000, 48), (64, 320, 96), (65, 130, 72),
               (130, 257, 136), (300, 96, 320), (5, 4096, 512), (40, 136, 1024), (12, 70, 1000), (16, 33, 264),
               # many rows, whole 64-steps of K: the wide-tile kernel, with tiles that reach beyond M and N
               (128, 264, 64), (257, 1000, 192), (700, 520, 1024), (2048, 256, 128)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
def test_linear(dtype, m, n, k):
    hip, ref = _ops(dtype)
    hip.library_rows = 0        # our own kernels at every row count (the library path has its own test)
    g = torch.Generator(device=DEV).manual_seed(m * 7 + n * 3 + k)
    x = torch.randn(m, k, device=DEV, generator=g).to(dtype)
    w = (torch.randn(n, k, device=DEV, generator=g) / math.sqrt(k)).to(dtype)
    bias = torch.randn(n, device=DEV, generator=g)
    res = torch.randn(m, n, device=DEV, generator=g)
    tol = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    tol32 = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(rtol=1e-3, atol=1e-3)
    for act in (None, "relu", "gelu", "gelu_new"):
        y_h = hip.linear(x, w, bias, act=act)
        y_r = ref.linear(x, w, bias, act=act)
        torch.testing.assert_close(y_h.float(), y_r.float(), **tol)
    y_h = hip.linear(x, w, None, residual=res, out_f32=True)
    y_r = ref.linear(x, w, None, residual=res, out_f32=True)
    torch.testing.assert_close(y_h, y_r, **tol32)
    # library routine
    torch.testing.assert_close(hip.linear(x, w, bias, out_f32=True),
                               torch.nn.functional.linear(x.float(), w.float(), bias), **tol32)
    if dtype == torch.bfloat16:
        # both bfloat16 kernels, whatever the row count
        y_t = hip.linear(x, w, bias, act="relu", residual=res, out_f32=True, force_tiled=True)
        y_r = ref.linear(x, w, bias, act="relu", residual=res, out_f32=True)
        torch.testing.assert_close(y_t, y_r, **tol32)
        if m <= 32:
            # the few-rows kernel with two weight tiles a block, from the row-major weight and from the tile-ordered copy
            y_2 = hip.linear(x, w, bias, act="relu", residual=res, out_f32=True, force_tiled=2)
            torch.testing.assert_close(y_2, y_r, **tol32)
            y_2 = hip.linear(x, hip.prepare_weight(w), bias, act="relu", residual=res, out_f32=True, force_tiled=2)
            torch.testing.assert_close(y_2, y_r, **tol32)


def test_linear_float32_matrix_in_bfloat16_engine():
    hip, ref = _ops(torch.bfloat16)
    g = torch.Generator(device=DEV).manual_seed(11)
    x = torch.randn(9, 64, device=DEV, generator=g).to(torch.bfloat16)
    w = torch.randn(33, 64, device=DEV, generator=g) / 8
    torch.testing.assert_close(hip.linear(x, w, out_f32=True), x.float() @ w.t(), rtol=1e-4, atol=1e-4)


def test_linear_refuses_bad_inner_size():
    hip, _ = _ops(torch.bfloat16)
    x = torch.zeros(4, 12, device=DEV, dtype=torch.bfloat16)
    w = torch.zeros(8, 12, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        hip.linear(x, w)


def _make_step(runs, cached, page_size, num_pages, seed, device=DEV):
    """A step context over requests with `cached[i]` stored tokens and `runs[i]` new ones,
    their pages drawn at random from the pool (so order in memory differs from order in the request)."""
    from transformers_neuronx_amd.engine.batch import StepEntry, build_context
    rng = np.random.default_rng(seed)
    perm = rng.permutation(num_pages).tolist()
    tables, width = [], 0
    for r, c in zip(runs, cached):
        nb = -(-(r + c) // page_size)
        tables.append([perm.pop() for _ in range(nb)])
        width = max(width, nb)
    tab = np.full((len(runs), width + 1), -1, dtype=np.int32)
    for i, t in enumerate(tables):
        tab[i, :len(t)] = t
    entries = [StepEntry(i, [0] * r, []) for i, r in enumerate(runs)]
    return build_context(entries, list(cached), list(range(len(runs))), {"full": tab}, page_size, device, planners=ATTENTION_PLAN)


ATTN_CASES = [
    # heads, kv heads, head size, page size, runs, cached
    (4, 4, 16, 16, [5, 1, 17], [0, 30, 3]),
    (3, 3, 32, 16, [40, 1, 1, 2], [0, 77, 15, 16]),
    (6, 2, 48, 32, [70, 1], [0, 130]),
    (5, 1, 80, 64, [3, 129, 1], [64, 0, 200]),
    (2, 2, 128, 64, [1, 1, 65], [511, 63, 64]),
    (1, 1, 256, 16, [20, 1], [0, 33]),
    # several tiles of one run, starting inside a group of 8 positions and inside a page
    (2, 2, 64, 16, [300, 1, 9], [5, 40, 7]),
    (2, 1, 128, 64, [131, 2], [61, 126]),
    # long decoding runs at head sizes that are no power of two: several tiles a wave, several splits
    (3, 3, 80, 64, [1, 1], [700, 1300]),
    (2, 2, 112, 16, [1, 5], [900, 40]),
    (2, 1, 96, 32, [1, 1, 1], [300, 5, 64]),
    # pages whose size is no power of two: prompts alone (the prompt kernel without LDS staging) and
    # prompts beside decoded tokens (the general kernel)
    (4, 2, 64, 48, [100, 7], [30, 200]),
    (3, 3, 128, 80, [1, 50, 1], [170, 95, 3]),
    (2, 2, 32, 48, [1, 1], [500, 47]),
]


def _fill_cache_and_compare(dtype, heads, kv, hs, ps, runs, cached, window):
    hip, ref = _ops(dtype)
    num_pages = sum(-(-(r + c) // ps) for r, c in zip(runs, cached)) + 3
    g = torch.Generator(device=DEV).manual_seed(heads * 100 + hs)
    # the cache as earlier steps left it: filled by a first step that stores the cached tokens
    kp = torch.full((num_pages, kv, ps, hs), float("nan"), device=DEV, dtype=dtype)
    vp = torch.full((num_pages, kv, hs, ps), float("nan"), device=DEV, dtype=dtype)
    kp_r, vp_r = kp.clone(), vp.clone()
    width = (heads + 2 * kv) * hs
    ctx_all = _make_step([r + c for r, c in zip(runs, cached)], [0] * len(runs), ps, num_pages, seed=hs)
    # same pages, two steps: first the cached part, then the new runs
    tab = ctx_all.groups["full"].block_table.cpu().numpy()
    from transformers_neuronx_amd.engine.batch import StepEntry, build_context
    live = [i for i, c in enumerate(cached) if c > 0]
    bias = torch.randn(width, device=DEV, generator=g) * 0.1
    scale = 1.0 / math.sqrt(hs)
    if live:
        ctx0 = build_context([StepEntry(i, [0] * cached[i], []) for i in live], [0] * len(live), live,
                             {"full": tab[live]}, ps, DEV, planners=ATTENTION_PLAN)
        qkv0 = torch.randn(ctx0.num_tokens, width, device=DEV, generator=g).to(dtype)
        hip.qkv_write(qkv0, bias, heads, kv, hs, scale, ctx0, ctx0.groups["full"], kp, vp)
        ref.qkv_write(qkv0, bias, heads, kv, hs, scale, ctx0, ctx0.groups["full"], kp_r, vp_r)
    ctx = build_context([StepEntry(i, [0] * r, []) for i, r in enumerate(runs)], list(cached),
                        list(range(len(runs))), {"full": tab}, ps, DEV, planners=ATTENTION_PLAN)
    qkv = torch.randn(ctx.num_tokens, width, device=DEV, generator=g).to(dtype)
    q_h = hip.qkv_write(qkv, bias, heads, kv, hs, scale, ctx, ctx.groups["full"], kp, vp)
    q_r = ref.qkv_write(qkv, bias, heads, kv, hs, scale, ctx, ctx.groups["full"], kp_r, vp_r)
    if dtype == torch.bfloat16:
        # values written by tiles (the default for runs of several tokens) and token by token: the same bits
        tokenwise = type(hip)(dtype, DEV)
        tokenwise.value_tiles = False
        kp_t, vp_t = kp_r.clone(), vp_r.clone()      # the reference's pages hold the cached part already
        kp_t.copy_(kp), vp_t.copy_(vp)
        tokenwise.qkv_write(qkv, bias, heads, kv, hs, scale, ctx, ctx.groups["full"], kp_t, vp_t)
        assert torch.equal(torch.nan_to_num(vp_t.float()), torch.nan_to_num(vp.float()))
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(q_h.float(), q_r.float(), **tol)
    # what was written is the same, and nothing else was touched (untouched places are still NaN)
    assert torch.equal(torch.isnan(kp), torch.isnan(kp_r)) and torch.equal(torch.isnan(vp), torch.isnan(vp_r))
    torch.testing.assert_close(torch.nan_to_num(kp.float()), torch.nan_to_num(kp_r.float()), **tol)
    torch.testing.assert_close(torch.nan_to_num(vp.float()), torch.nan_to_num(vp_r.float()), **tol)
    o_h = hip.attention(q_r, heads, kv, hs, ctx, ctx.groups["full"], kp_r, vp_r, window)
    o_r = ref.attention(q_r, heads, kv, hs, ctx, ctx.groups["full"], kp_r, vp_r, window)
    assert not torch.isnan(o_h.float()).any()
    torch.testing.assert_close(o_h.float(), o_r.float(), **tol)
    return ctx, q_r, kp_r, vp_r, o_h


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", ATTN_CASES)
@pytest.mark.parametrize("window", [None, 24])
def test_qkv_write_and_attention(dtype, case, window):
    _fill_cache_and_compare(dtype, *case, window)


def test_attention_is_library_attention_without_cache():
    """One request from position 0, one head group: torch's scaled_dot_product_attention."""
    dtype = torch.float32
    hip, ref = _ops(dtype)
    heads, hs, ps, n = 4, 32, 16, 50
    ctx, q, kp, vp, o = _fill_cache_and_compare(dtype, heads, heads, hs, ps, [n], [0], None)
    tab = ctx.groups["full"].block_table[0, :-(-n // ps)].long()
    keys = kp[tab].permute(1, 0, 2, 3).reshape(heads, -1, hs)[:, :n]
    vals = vp[tab].permute(1, 2, 0, 3).reshape(heads, hs, -1)[:, :, :n].transpose(1, 2)
    qq = q.reshape(n, heads, hs).permute(1, 0, 2)
    want = torch.nn.functional.scaled_dot_product_attention(qq, keys, vals, is_causal=True, scale=1.0)
    torch.testing.assert_close(o, want.permute(1, 0, 2).reshape(n, heads * hs), rtol=1e-5, atol=1e-5)


def test_attention_finds_a_far_key():
    """One key among hundreds carries the value: scale one query and one key so that its score stands out."""
    dtype = torch.bfloat16
    hip, _ = _ops(dtype)
    heads, hs, ps, cached = 2, 64, 16, 700
    num_pages = -(-(cached + 1) // ps) + 2
    ctx = _make_step([1], [cached], ps, num_pages, seed=5)
    view = ctx.groups["full"]
    g = torch.Generator(device=DEV).manual_seed(9)
    kp = (torch.randn(num_pages, heads, ps, hs, device=DEV, generator=g) * 0.1).to(dtype)
    vp = (torch.randn(num_pages, heads, hs, ps, device=DEV, generator=g) * 0.1).to(dtype)
    far = 37
    page = int(view.block_table[0, far // ps])
    direction = torch.randn(hs, device=DEV, generator=g)
    direction /= direction.norm()
    kp[page, :, far % ps, :] = (direction * 40).to(dtype)
    vp[page, :, :, far % ps] = 5.0
    q = (direction * 10).repeat(heads).reshape(1, heads * hs).to(dtype)
    out = hip.attention(q, heads, heads, hs, ctx, view, kp, vp, None)
    torch.testing.assert_close(out.float(), torch.full_like(out, 5.0).float(), rtol=1e-2, atol=1e-2)
    # the window's edge: a query at position `cached` with window w sees keys > cached - w. With
    # w = cached - far the far key is the first one outside, with one more it is the last one inside.
    out_w = hip.attention(q, heads, heads, hs, ctx, view, kp, vp, cached - far)
    assert out_w.float().abs().max() < 1.0
    out_in = hip.attention(q, heads, heads, hs, ctx, view, kp, vp, cached - far + 1)
    torch.testing.assert_close(out_in.float(), torch.full_like(out_in, 5.0).float(), rtol=1e-2, atol=1e-2)
    plain = type(hip)(dtype, DEV)
    plain.force_plain_attention = True
    assert plain.attention(q, heads, heads, hs, ctx, view, kp, vp, cached - far).float().abs().max() < 1.0
    torch.testing.assert_close(plain.attention(q, heads, heads, hs, ctx, view, kp, vp, cached - far + 1).float(),
                               torch.full_like(out_in, 5.0).float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("sets", [2, 3])
@pytest.mark.parametrize("hs", [64, 128])
def test_prompt_attention_when_the_maximum_jumps(sets, hs):
    """The pipelined prompt kernel moves a query's reference maximum only when a score exceeds it by more than
    2^8: a key that stands out by less leaves probabilities above one in play, a key that stands out by much
    more makes all sums so far shrink. Both in the middle of a long prompt, against the torch rendition."""
    dtype = torch.bfloat16
    hip, ref = _ops(dtype)
    hip.prefill_direct = sets
    heads, ps, n = 2, 64, 600
    num_pages = -(-n // ps) + 2
    ctx = _make_step([n], [0], ps, num_pages, seed=21)
    view = ctx.groups["full"]
    g = torch.Generator(device=DEV).manual_seed(33)
    kp = (torch.randn(num_pages, heads, ps, hs, device=DEV, generator=g) * 0.05).to(dtype)
    vp = (torch.randn(num_pages, heads, hs, ps, device=DEV, generator=g) * 0.1).to(dtype)
    direction = torch.randn(hs, device=DEV, generator=g)
    direction /= direction.norm()
    # every query has a component of 2 along `direction`; key 200 has 2 along it (score + 4: e^4, no rescale),
    # key 400 has 10 (score + 20), key 401 has 9.5 (one below the new maximum)
    q = (torch.randn(n, heads, hs, device=DEV, generator=g) * 0.3 + 2 * direction).reshape(n, heads * hs).to(dtype)
    for key, size, value in ((200, 2.0, 1.0), (400, 10.0, -2.0), (401, 9.5, 3.0)):
        page = int(view.block_table[0, key // ps])
        kp[page, :, key % ps, :] = (direction * size).to(dtype)
        vp[page, :, :, key % ps] = value
    got = hip.attention(q, heads, heads, hs, ctx, view, kp, vp, None)
    want = ref.attention(q, heads, heads, hs, ctx, view, kp, vp, None)
    torch.testing.assert_close(got.float(), want.float(), rtol=2e-2, atol=2e-2)
    # queries before key 200 see none of the three, those from 400 on are ruled by keys 400 and 401
    assert got[:200].float().abs().max() < 0.5
    assert (got[450:].float().mean() - (-2 * 0.731 + 3 * 0.269)).abs() < 0.1      # weights e^0 : e^-1


@pytest.mark.parametrize("mode", ["staged", "direct", "plain"])
def test_windowed_attention_over_pages_given_back(mode):
    """A windowed group gives back the pages its queries have passed: their table entries are -1, and the
    first tile of keys a prompt kernel computes can hold such entries beside live pages. What lies in the
    page such an entry is clamped to (here NaN) must not reach the result."""
    dtype = torch.bfloat16
    hip, ref = _ops(dtype)
    if mode == "direct":
        hip.prefill_direct = True
    elif mode == "plain":
        hip.force_plain_attention = True
    heads, kv, hs, ps, window = 2, 1, 64, 16, 40
    runs, cached = [70, 1, 20], [100, 130, 64]
    num_pages = 40
    ctx = _make_step(runs, cached, ps, num_pages - 1, seed=4)
    view = ctx.groups["full"]
    tab = view.block_table.cpu().numpy().copy()
    tab[tab >= 0] += 1                                             # page 0 of the pool is no one's
    for i, c in enumerate(cached):
        gone = max(0, c - window + 1) // ps                        # pages wholly below the first query's window
        tab[i, :gone] = -1
    assert (tab[0, :3] == -1).all() and tab[0, 3] >= 0             # keys 0..47 gone, 48..63 live: one tile
    view.block_table.copy_(torch.from_numpy(tab).to(DEV))
    g = torch.Generator(device=DEV).manual_seed(12)
    kp = torch.randn(num_pages, kv, ps, hs, device=DEV, generator=g).to(dtype)
    vp = torch.randn(num_pages, kv, hs, ps, device=DEV, generator=g).to(dtype)
    q = (torch.randn(ctx.num_tokens, heads * hs, device=DEV, generator=g) / 8).to(dtype)
    want = ref.attention(q, heads, kv, hs, ctx, view, kp, vp, window)
    # every page that no table names holds NaN now, page 0 (where -1 is clamped to) among them
    live = set(tab[tab >= 0].tolist())
    for page in range(num_pages):
        if page not in live:
            kp[page] = float("nan")
            vp[page] = float("nan")
    got = hip.attention(q, heads, kv, hs, ctx, view, kp, vp, window)
    assert not torch.isnan(got.float()).any()
    torch.testing.assert_close(got.float(), want.float(), rtol=2e-2, atol=2e-2)


def test_a_page_size_that_is_no_power_of_two_is_said_once(capfd):
    """Pages of 48 tokens send decoding to the general kernel: correct, several times slower, and said so once."""
    from transformers_neuronx_amd.kernels.hip import HipOps
    hip, ref = _ops(torch.bfloat16)
    HipOps._warned_page_size = False
    ctx = _make_step([1, 1], [100, 47], 48, 8, seed=1)
    g = torch.Generator(device=DEV).manual_seed(2)
    q = torch.randn(2, 2 * 32, device=DEV, generator=g).to(torch.bfloat16)
    kp = torch.randn(8, 2, 48, 32, device=DEV, generator=g).to(torch.bfloat16)
    vp = torch.randn(8, 2, 32, 48, device=DEV, generator=g).to(torch.bfloat16)
    for _ in range(2):
        got = hip.attention(q, 2, 2, 32, ctx, ctx.groups["full"], kp, vp, None)
    torch.testing.assert_close(got.float(), ref.attention(q, 2, 2, 32, ctx, ctx.groups["full"], kp, vp, None).float(),
                               rtol=2e-2, atol=2e-2)
    assert capfd.readouterr().err.count("no power of two") == 1


def test_attention_refuses_bad_head_size():
    hip, _ = _ops(torch.float32)
    ctx = _make_step([1], [0], 16, 2, seed=1)
    q = torch.zeros(1, 24, device=DEV)
    kp = torch.zeros(2, 1, 16, 24, device=DEV)
    vp = torch.zeros(2, 1, 24, 16, device=DEV)
    with pytest.raises(RuntimeError, match="head size"):
        hip.attention(q, 1, 1, 24, ctx, ctx.groups["full"], kp, vp, None)


@pytest.mark.parametrize("vocab", [1000, 50272, 333])
def test_argmax_and_sampling(vocab):
    hip, ref = _ops(torch.float32)
    g = torch.Generator(device=DEV).manual_seed(vocab)
    rows = 24
    logits = torch.randn(rows, vocab, device=DEV, generator=g) * 3
    logits[3, 17] = logits[3, 400 % vocab] = logits[3].max() + 1     # a tie: the lower id wins
    logits[4] = -1 - logits[4].abs()                                  # -0 and +0 tie as well
    logits[4, 7], logits[4, 9] = -0.0, 0.0
    assert torch.equal(hip.argmax(logits), ref.argmax(logits))
    assert int(hip.argmax(logits)[3]) == 17 and int(hip.argmax(logits)[4]) == 7
    temp = torch.tensor([0.0, 1.0, 0.7, 1.3] * 6, device=DEV)
    top_k = torch.tensor([0, 50, 1, 5, 0, vocab + 5] * 4, device=DEV, dtype=torch.int32)
    top_p = torch.tensor([1.0, 1.0, 0.9, 0.5, 0.3, 0.99, 1.0, 0.05] * 3, device=DEV)
    seeds = torch.arange(rows, device=DEV, dtype=torch.int64) * 7919 + 1

    def same_or_on_a_boundary(t_h, t_r, top_p, counters, least=None):
        """Every row is one of 24 different combinations of options, so every row must agree; a draw may
        fall to the neighbouring token only where the random number lies on the boundary between the two
        (within the rounding of the float32 sums), which the plain sampler's own sums show."""
        import plain_opt
        for i in torch.nonzero(t_h != t_r).flatten().tolist():
            assert float(temp[i]) > 0 and int(top_k[i]) != 1, f"row {i} is greedy and differs"
            n = int(counters[i])
            u = 0.5 if n < 0 else plain_opt.philox_uniform(int(seeds[i]), n)
            k = int(top_k[i]) or None
            slack, bound = plain_opt.draw_slack(logits[i].cpu(), u, int(t_h[i]), k, float(top_p[i]), float(temp[i]),
                                                int(least[i]) if least is not None else 1)
            assert slack <= bound, (i, int(t_h[i]), int(t_r[i]), u, slack, bound)

    for step in range(6):
        counters = torch.full((rows,), step, device=DEV, dtype=torch.int64)
        t_h = hip.sample(logits, temp, top_k, top_p, seeds, counters)
        t_r = ref.sample(logits, temp, top_k, top_p, seeds, counters)
        same_or_on_a_boundary(t_h, t_r, top_p, counters)
    # never fewer than `min_keep` tokens, and the constant 0.5 in place of a random number (counter < 0)
    least = torch.tensor([1, 3, 40, 7] * 6, device=DEV, dtype=torch.int32)
    tight_p = torch.full((rows,), 0.01, device=DEV)             # top-p alone would keep one token
    fixed = torch.full((rows,), -1, device=DEV, dtype=torch.int64)
    t_h = hip.sample(logits, temp, top_k, tight_p, seeds, fixed, least)
    t_r = ref.sample(logits, temp, top_k, tight_p, seeds, fixed, least)
    same_or_on_a_boundary(t_h, t_r, tight_p, fixed, least)
    for step in range(4):
        counters = torch.full((rows,), step, device=DEV, dtype=torch.int64)
        t_h = hip.sample(logits, temp, top_k, tight_p, seeds, counters, least)
        t_r = ref.sample(logits, temp, top_k, tight_p, seeds, counters, least)
        same_or_on_a_boundary(t_h, t_r, tight_p, counters, least)


@pytest.mark.parametrize("vocab", [1500, 50272])
def test_sampling_after_a_top_k_with_ties(vocab):
    """Logits in steps of a half, so that the k-th largest value is shared by many tokens (the lower ids stay),
    at numbers of kept tokens around what the kernel gathers (256) and around a wave."""
    import plain_opt
    hip, ref = _ops(torch.float32)
    g = torch.Generator(device=DEV).manual_seed(vocab + 1)
    ks = [2, 63, 64, 65, 255, 256, 257, 1024, vocab - 1, 7]
    rows = 3 * len(ks)
    logits = torch.round(torch.randn(rows, vocab, device=DEV, generator=g) * 4) / 2
    temp = torch.tensor([1.0, 0.6, 1.7] * len(ks), device=DEV)
    top_k = torch.tensor([k for k in ks for _ in range(3)], device=DEV, dtype=torch.int32)
    top_p = torch.tensor([1.0, 0.8, 0.3, 0.97, 0.5] * (rows // 5), device=DEV)
    least = torch.tensor([1, 1, 5, 1, 70, 1] * (rows // 6), device=DEV, dtype=torch.int32)
    seeds = torch.arange(rows, device=DEV, dtype=torch.int64) * 104729 + 5
    for step in (-1, 0, 1, 2, 3):
        counters = torch.full((rows,), step, device=DEV, dtype=torch.int64)
        t_h = hip.sample(logits, temp, top_k, top_p, seeds, counters, least)
        t_r = ref.sample(logits, temp, top_k, top_p, seeds, counters, least)
        for i in range(rows):
            values, indices = plain_opt.filter_top_k_top_p(logits[i].cpu() / float(temp[i]), int(top_k[i]),
                                                           float(top_p[i]), int(least[i]))
            assert int(t_h[i]) in set(indices.tolist()), f"row {i}: token {int(t_h[i])} is outside what the filters keep"
            if int(t_h[i]) != int(t_r[i]):      # only where the random number lies on the boundary between two tokens
                u = 0.5 if step < 0 else plain_opt.philox_uniform(int(seeds[i]), step)
                slack, bound = plain_opt.draw_slack(logits[i].cpu(), u, int(t_h[i]), int(top_k[i]), float(top_p[i]),
                                                    float(temp[i]), int(least[i]))
                assert slack <= bound, (i, int(t_h[i]), int(t_r[i]), u, slack, bound)


@pytest.mark.parametrize("vocab", [32000, 50272, 70001])
def test_sampling_over_thousands_of_kept_tokens(vocab):
    """Low and high temperatures over rows that keep thousands of tokens, where the sums behind a draw run over
    most of the vocabulary: every row draws the plain sampler's token, or one whose stretch of the line the
    drawn point misses by no more than float32 rounding allows (`plain_opt.draw_slack` derives the bound, some
    5e-7; a fast exponential or a multiplication by the reciprocal temperature in the kernel's weights misses
    by 1e-5 to 1e-4 in a few rows of these)."""
    import plain_opt
    hip, _ = _ops(torch.float32)
    rows, differ, fewest = 24, 0, vocab
    for temp_v, scale in ((0.3, 0.36), (1.5, 1.8)):
        for p_v in (0.5, 0.9, 0.99, 1.0):
            g = torch.Generator(device=DEV).manual_seed(vocab + int(temp_v * 10) + int(p_v * 100))
            logits = torch.randn(rows, vocab, device=DEV, generator=g) * scale
            temp = torch.full((rows,), temp_v, device=DEV)
            top_k = torch.zeros(rows, device=DEV, dtype=torch.int32)
            top_p = torch.full((rows,), p_v, device=DEV)
            seeds = torch.arange(rows, device=DEV, dtype=torch.int64) * 7919 + vocab
            host = logits.cpu()
            fewest = min(fewest, len(plain_opt.filter_top_k_top_p(host[0] / temp_v, None, p_v)[0]))
            for c in (0, 1, 2 ** 33):
                counters = torch.full((rows,), c, device=DEV, dtype=torch.int64)
                t_h = hip.sample(logits, temp, top_k, top_p, seeds, counters).tolist()
                for i in range(rows):
                    u = plain_opt.philox_uniform(int(seeds[i]), c)
                    if plain_opt.sample_row(host[i], u, None, p_v, temp_v) != t_h[i]:
                        differ += 1
                        slack, bound = plain_opt.draw_slack(host[i], u, t_h[i], None, p_v, temp_v)
                        assert slack <= bound, (temp_v, p_v, c, i, t_h[i], u, slack, bound)
    assert fewest >= 2000, fewest
    assert differ <= 12, differ          # 576 rows: a draw lands that close to a boundary in a few of them only


def test_sampling_with_logits_that_are_no_numbers():
    """A NaN orders last and has no weight: the draw is the one over the same row with -inf in its place, on
    every way through the kernel, and never lands on it."""
    hip, _ = _ops(torch.float32)
    vocab, rows = 3000, 12
    g = torch.Generator(device=DEV).manual_seed(5)
    clean = torch.randn(rows, vocab, device=DEV, generator=g) * 2
    holes = torch.rand(rows, vocab, device=DEV, generator=g) < 0.05
    holes[:, 0] = True
    clean[holes] = -float("inf")
    dirty = clean.clone()
    dirty[holes] = float("nan")
    temp = torch.tensor([0.0, 1.0, 0.7, 1.3] * 3, device=DEV)
    top_k = torch.tensor([0, 0, 40, 500, 0, 5], device=DEV, dtype=torch.int32).repeat(2)
    top_p = torch.tensor([1.0, 0.9, 0.5, 0.95], device=DEV).repeat(3)
    seeds = torch.arange(rows, device=DEV, dtype=torch.int64) + 77
    for step in range(5):
        counters = torch.full((rows,), step, device=DEV, dtype=torch.int64)
        a = hip.sample(dirty, temp, top_k, top_p, seeds, counters)
        b = hip.sample(clean, temp, top_k, top_p, seeds, counters)
        assert torch.equal(a, b)
        assert not holes[torch.arange(rows, device=DEV), a.long()].any()
    assert torch.equal(hip.argmax(dirty), hip.argmax(clean))


def test_sampling_distribution():
    """Frequencies over many draws follow the softmax over the kept tokens."""
    hip, _ = _ops(torch.float32)
    vocab, n = 64, 20000
    g = torch.Generator(device=DEV).manual_seed(1)
    row = torch.randn(vocab, device=DEV, generator=g) * 2
    logits = row.repeat(n, 1).contiguous()
    temp = torch.full((n,), 0.8, device=DEV)
    top_k = torch.full((n,), 10, device=DEV, dtype=torch.int32)
    top_p = torch.full((n,), 1.0, device=DEV)
    seeds = torch.full((n,), 123, device=DEV, dtype=torch.int64)
    counters = torch.arange(n, device=DEV, dtype=torch.int64)
    toks = hip.sample(logits, temp, top_k, top_p, seeds, counters).long()
    vals, idx = torch.topk(row / 0.8, 10)
    probs = torch.softmax(vals, -1)
    counts = torch.bincount(toks, minlength=vocab).float()
    assert counts.sum() == counts[idx].sum()           # nothing outside the top k
    chi2 = (((counts[idx] - probs * n) ** 2) / (probs * n)).sum().item()
    assert chi2 < 40, chi2                              # 9 degrees of freedom; 40 is far in the tail


FAST_CASES = [
    # heads, kv heads, head size, page size, runs, cached
    (4, 4, 64, 64, [300, 1, 1], [0, 1000, 255]),
    (8, 2, 128, 64, [1, 1, 1, 1], [2047, 100, 0, 640]),
    (4, 4, 128, 16, [129, 40, 1], [77, 0, 300]),
    (2, 1, 256, 32, [1, 200], [500, 31]),
    (3, 3, 32, 16, [1, 1, 2], [0, 1, 0]),
    (2, 2, 16, 64, [1, 260], [900, 3]),
    (2, 2, 96, 16, [150, 33], [10, 0]),
    # long prompts on pages of 64 keys or more at head sizes 64 and 128: the pipelined prompt kernel, whose
    # waves take several whole tiles before the one the positions mask
    (4, 2, 128, 64, [700, 130, 1], [0, 333, 50]),
    (6, 2, 64, 128, [513, 64], [1000, 17]),
    (2, 2, 128, 256, [1000], [37]),
]


@pytest.mark.parametrize("case", FAST_CASES)
@pytest.mark.parametrize("window", [None, 100])
def test_bfloat16_attention_kernels_agree(case, window):
    """The MFMA kernel for prompts and the split kernel for decoding against the torch rendition and
    against the one-wave-per-query kernel, with contexts long enough to split."""
    from transformers_neuronx_amd.kernels.hip import HipOps
    ctx, q, kp, vp, o_fast = _fill_cache_and_compare(torch.bfloat16, *case, window)
    heads, kv, hs = case[:3]
    plain = HipOps(torch.bfloat16, DEV)
    plain.force_plain_attention = True
    o_plain = plain.attention(q, heads, kv, hs, ctx, ctx.groups["full"], kp, vp, window)
    torch.testing.assert_close(o_fast.float(), o_plain.float(), rtol=2e-2, atol=2e-2)
    many = HipOps(torch.bfloat16, DEV)
    many.decode_blocks_wanted = 1 << 20           # as many splits as the contexts allow
    o_many = many.attention(q, heads, kv, hs, ctx, ctx.groups["full"], kp, vp, window)
    torch.testing.assert_close(o_many.float(), o_plain.float(), rtol=2e-2, atol=2e-2)
    direct = HipOps(torch.bfloat16, DEV)
    direct.prefill_direct = True                  # the prompt kernel that reads the pages without staging
    o_direct = direct.attention(q, heads, kv, hs, ctx, ctx.groups["full"], kp, vp, window)
    torch.testing.assert_close(o_direct.float(), o_plain.float(), rtol=2e-2, atol=2e-2)
    # the prompt kernels that stage tiles in LDS with one set of waves a block and with two: 2 and 3 (the
    # pipelined kernel where it applies), 7 and 6 (never the pipelined one)
    for sets in (2, 3, 6, 7):
        forced = HipOps(torch.bfloat16, DEV)
        forced.prefill_direct = sets
        o_forced = forced.attention(q, heads, kv, hs, ctx, ctx.groups["full"], kp, vp, window)
        torch.testing.assert_close(o_forced.float(), o_plain.float(), rtol=2e-2, atol=2e-2)
    wide = HipOps(torch.bfloat16, DEV)
    wide.decode_waves = 8                         # blocks of eight waves
    for wanted in (1 << 20, 1):
        wide.decode_blocks_wanted = wanted
        o_wide = wide.attention(q, heads, kv, hs, ctx, ctx.groups["full"], kp, vp, window)
        torch.testing.assert_close(o_wide.float(), o_plain.float(), rtol=2e-2, atol=2e-2)
    one = HipOps(torch.bfloat16, DEV)
    one.decode_blocks_wanted = 1                  # no split at all
    o_one = one.attention(q, heads, kv, hs, ctx, ctx.groups["full"], kp, vp, window)
    torch.testing.assert_close(o_one.float(), o_plain.float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,hs,ps,runs,cached", [
    (4, 4, 16, 16, [5, 1, 17], [0, 30, 3]), (6, 2, 48, 32, [70, 1], [0, 130]),
    (2, 2, 128, 64, [1, 1, 65, 140], [511, 63, 64, 0]), (3, 1, 80, 16, [1], [4])])
def test_fused_projection_writes_what_the_two_kernels_write(dtype, heads, kv, hs, ps, runs, cached):
    hip, ref = _ops(dtype)
    num_pages = sum(-(-(r + c) // ps) for r, c in zip(runs, cached)) + 2
    ctx = _make_step(runs, cached, ps, num_pages, seed=hs)
    view = ctx.groups["full"]
    width = heads * hs
    total = (heads + 2 * kv) * hs
    g = torch.Generator(device=DEV).manual_seed(hs)
    h = torch.randn(ctx.num_tokens, width, device=DEV, generator=g).to(dtype)
    w = (torch.randn(total, width, device=DEV, generator=g) / math.sqrt(width)).to(dtype)
    bias = torch.randn(total, device=DEV, generator=g) * 0.2
    tol = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    variants = [0] if dtype == torch.float32 else [0, 1, 2]      # 2: two weight tiles a block
    for b in (bias, None):
        kp_r = torch.full((num_pages, kv, ps, hs), float("nan"), device=DEV, dtype=dtype)
        vp_r = torch.full((num_pages, kv, hs, ps), float("nan"), device=DEV, dtype=dtype)
        q_r = ref.qkv_project(h, w, b, heads, kv, hs, 0.3, ctx, view, kp_r, vp_r)
        for variant in variants:
            kp, vp = torch.full_like(kp_r, float("nan")), torch.full_like(vp_r, float("nan"))
            q = hip.qkv_project(h, w, b, heads, kv, hs, 0.3, ctx, view, kp, vp, **({"force_tiled": variant}
                                                                                  if dtype == torch.bfloat16 else {}))
            torch.testing.assert_close(q.float(), q_r.float(), **tol)
            assert torch.equal(torch.isnan(kp), torch.isnan(kp_r)) and torch.equal(torch.isnan(vp), torch.isnan(vp_r))
            torch.testing.assert_close(torch.nan_to_num(kp.float()), torch.nan_to_num(kp_r.float()), **tol)
            torch.testing.assert_close(torch.nan_to_num(vp.float()), torch.nan_to_num(vp_r.float()), **tol)
    # a mixer that only reads another's cache projects queries alone
    q = hip.qkv_project(h, w[:width].contiguous(), bias[:width].contiguous(), heads, 0, hs, 0.3, ctx, view, None, None)
    q_r = ref.qkv_project(h, w[:width].contiguous(), bias[:width].contiguous(), heads, 0, hs, 0.3, ctx, view, None, None)
    torch.testing.assert_close(q.float(), q_r.float(), **tol)


@pytest.mark.parametrize("m,n,k", [(256, 96, 320), (300, 1000, 48), (513, 136, 1024), (17, 4096, 512), (64, 136, 2048),
                                   (2048, 512, 1024)])
def test_library_product_and_own_product_agree(m, n, k):
    """From `library_rows` rows on the plain product goes to the vendor library and our epilogue kernel
    follows; below it, and always when told so, our own tiled kernel does all of it."""
    from transformers_neuronx_amd.kernels.hip import HipOps
    _, ref = _ops(torch.bfloat16)
    lib, own = HipOps(torch.bfloat16, DEV), HipOps(torch.bfloat16, DEV)
    own.library_rows = 0
    g = torch.Generator(device=DEV).manual_seed(m + n)
    x = torch.randn(m, k, device=DEV, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, device=DEV, generator=g) / math.sqrt(k)).to(torch.bfloat16)
    bias = torch.randn(n, device=DEV, generator=g)
    res = torch.randn(m, n, device=DEV, generator=g)
    # (an activation comes before the residual, also where the library, whose own ReLU comes last, makes the product)
    for kwargs in (dict(act="relu"), dict(act="gelu"), dict(residual=res, out_f32=True), dict(bias=None),
                   dict(act="relu", residual=res, out_f32=True), dict(act="gelu_new", residual=res, out_f32=True)):
        b = kwargs.pop("bias", bias)
        want = ref.linear(x, w, b, **kwargs).float()
        for ops in (lib, own):
            torch.testing.assert_close(ops.linear(x, w, b, **kwargs).float(), want, rtol=2e-2, atol=2e-2)
    # the head's float32 output never goes through a bfloat16 product
    torch.testing.assert_close(lib.linear(x, w, None, out_f32=True), ref.linear(x, w, None, out_f32=True),
                               rtol=1e-3, atol=1e-3)
    # nor does the sum with the residual: the library adds bias and residual to its float32 sums itself; with
    # that switched off the product comes back in bfloat16 and our kernel makes the sum
    exact = x.float() @ w.float().t() + res
    torch.testing.assert_close(lib.linear(x, w, None, residual=res, out_f32=True), exact, rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(lib.linear(x, w, bias, residual=res, out_f32=True), exact + bias, rtol=1e-3, atol=1e-3)
    rounded = HipOps(torch.bfloat16, DEV)
    rounded.library_direct = False
    torch.testing.assert_close(rounded.linear(x, w, bias, residual=res, out_f32=True), exact + bias, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("m,n,k", [(1, 64, 128), (8, 4096, 512), (16, 320, 256), (13, 48, 1024), (64, 128, 384),
                                   (8, 8192, 256), (3, 12304, 384), (20, 16400, 128), (1, 50272, 640)])
def test_product_from_the_tile_ordered_copy(m, n, k):
    """The few-rows kernel reading the copy of the weight that is laid out tile after tile. The last four
    matrices have hundreds of tiles: a wave that has no step of its own (K of three steps for four waves), two
    tiles a block with an odd number of tiles, a vocabulary-sized matrix."""
    from transformers_neuronx_amd.kernels.hip import HipOps, tile_order
    hip, ref = _ops(torch.bfloat16)
    hip.library_rows = 0
    g = torch.Generator(device=DEV).manual_seed(m * 31 + n + k)
    x = torch.randn(m, k, device=DEV, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, device=DEV, generator=g) / math.sqrt(k)).to(torch.bfloat16)
    bias = torch.randn(n, device=DEV, generator=g)
    res = torch.randn(m, n, device=DEV, generator=g)
    pw = hip.prepare_weight(w)
    assert pw.tiles is not None and pw.tiles.numel() == w.numel()
    # the copy holds element (n, k) at [n/16][k/128][(k%128)/32][n%16][(k%32)/8][k%8]
    t = tile_order(w)
    for nn, kk in ((0, 0), (17, 5), (n - 1, k - 1), (31, 127 % k)):
        assert t[nn // 16, kk // 128, (kk % 128) // 32, nn % 16, (kk % 32) // 8, kk % 8] == w[nn, kk]
    for act in (None, "relu", "gelu_new"):
        torch.testing.assert_close(hip.linear(x, pw, bias, act=act).float(), ref.linear(x, w, bias, act=act).float(),
                                   rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(hip.linear(x, pw, None, residual=res, out_f32=True),
                               ref.linear(x, w, None, residual=res, out_f32=True), rtol=1e-3, atol=1e-3)
    # bit for bit what the same kernel makes of the plain layout: only the addresses differ
    assert torch.equal(hip.linear(x, pw, bias, out_f32=True), hip.linear(x, w, bias, out_f32=True))
    assert hip.prepare_weight(w[:, :k - 8].contiguous()).tiles is None       # sizes that have no such copy


def test_fused_projection_from_the_tile_ordered_copy():
    hip, ref = _ops(torch.bfloat16)
    heads, kv, hs, ps = 4, 2, 32, 16
    runs, cached = [1, 1, 3], [40, 0, 7]
    num_pages = 8
    ctx = _make_step(runs, cached, ps, num_pages, seed=2)
    view = ctx.groups["full"]
    width, total = 128, (heads + 2 * kv) * hs
    g = torch.Generator(device=DEV).manual_seed(4)
    h = torch.randn(ctx.num_tokens, width, device=DEV, generator=g).to(torch.bfloat16)
    w = (torch.randn(total, width, device=DEV, generator=g) / 11).to(torch.bfloat16)
    bias = torch.randn(total, device=DEV, generator=g) * 0.2
    kp_r = torch.full((num_pages, kv, ps, hs), float("nan"), device=DEV, dtype=torch.bfloat16)
    vp_r = torch.full((num_pages, kv, hs, ps), float("nan"), device=DEV, dtype=torch.bfloat16)
    kp, vp = kp_r.clone(), vp_r.clone()
    q_r = ref.qkv_project(h, w, bias, heads, kv, hs, 0.25, ctx, view, kp_r, vp_r)
    q = hip.qkv_project(h, hip.prepare_weight(w), bias, heads, kv, hs, 0.25, ctx, view, kp, vp)
    torch.testing.assert_close(q.float(), q_r.float(), rtol=2e-2, atol=2e-2)
    assert torch.equal(torch.isnan(kp), torch.isnan(kp_r)) and torch.equal(torch.isnan(vp), torch.isnan(vp_r))
    torch.testing.assert_close(torch.nan_to_num(kp.float()), torch.nan_to_num(kp_r.float()), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(torch.nan_to_num(vp.float()), torch.nan_to_num(vp_r.float()), rtol=2e-2, atol=2e-2)


# ------------------------------------------------------------------ a LayerNorm folded into the product after it

def _float32_norm_then_product(x, gamma, beta, eps, w, bias, act):
    """What the folded product must give, in float32 from the stored (bfloat16) matrix."""
    h = torch.nn.functional.layer_norm(x, (x.shape[1],), gamma, beta, eps)
    y = h @ w.float().T + (bias if bias is not None else 0)
    return torch.relu(y) if act == "relu" else y


@pytest.mark.parametrize("m,n,k", [(1, 48, 128), (8, 12288, 4096), (16, 16384, 4096), (17, 160, 256),
                                   (32, 16384, 4096), (5, 1024, 2048), (2, 4096, 4096), (3, 16, 1152)])
@pytest.mark.parametrize("act", [None, "relu"])
def test_product_of_normalised_rows(m, n, k, act):
    """`linear` on the deferred output of a LayerNorm, with the norm folded into the matrix, against the norm
    and the product in float32: every wave count, tile count and row count of the few-rows kernel. The rows
    carry a common part a hundred times their spread, which the kernel takes out before it rounds."""
    from transformers_neuronx_amd.kernels.hip import DeferredNorm
    hip, _ = _ops(torch.bfloat16)
    g = torch.Generator(device=DEV).manual_seed(m * 7 + n)
    x = torch.randn(m, k, device=DEV, generator=g) * torch.rand(m, 1, device=DEV, generator=g) * 3
    x += torch.randn(m, 1, device=DEV, generator=g) * 100
    gamma = 1 + 0.2 * torch.randn(k, device=DEV, generator=g)
    beta = 0.3 * torch.randn(k, device=DEV, generator=g)
    w = (torch.randn(n, k, device=DEV, generator=g) / k ** 0.5).to(torch.bfloat16)
    bias = torch.randn(n, device=DEV, generator=g) * 0.2
    eps = 1e-5
    pw = hip.prepare_weight(w)
    assert hip.fold_norm(pw, gamma, beta) and pw.tiles is None and pw.folded is not None
    h = hip.layernorm_deferred(x, gamma, beta, eps, torch.bfloat16)
    assert isinstance(h, DeferredNorm)
    got = hip.linear(h, pw, bias, act=act)
    want = _float32_norm_then_product(x, gamma, beta, eps, w, bias, act)
    torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2)
    # and the same through the norm's own kernel and the plain product (another matrix object: not folded)
    plain = hip.linear(hip.layernorm(x, gamma, beta, eps, torch.bfloat16, False, True)[1], hip.prepare_weight(w),
                       bias, act=act)
    torch.testing.assert_close(got.float(), plain.float(), rtol=2e-2, atol=3e-2)
    # a deferred norm that meets a matrix it was not folded into is carried out by its own kernel
    other = hip.linear(h, hip.prepare_weight(w), bias, act=act)
    assert torch.equal(other, plain)


@pytest.mark.parametrize("m,n,k", [(1, 256, 1024), (8, 4096, 4096), (16, 512, 2048)])
def test_product_of_normalised_rows_with_elements_far_from_the_rest(m, n, k):
    """Rows of the kind a residual stream has, a few elements a thousand times the rest, among them the places the
    kernel samples its shift from (the first, the middle and the last element, and more): what the kernel
    subtracts before it rounds to bfloat16 must stay with the bulk of the row, or the rounding of `x - 1000`
    wipes out everything else. Also rows whose common part is fifty times their spread, and both together."""
    hip, _ = _ops(torch.bfloat16)
    g = torch.Generator(device=DEV).manual_seed(m + n + k)
    gamma = 1 + 0.2 * torch.randn(k, device=DEV, generator=g)
    beta = 0.3 * torch.randn(k, device=DEV, generator=g)
    w = (torch.randn(n, k, device=DEV, generator=g) / k ** 0.5).to(torch.bfloat16)
    pw = hip.prepare_weight(w)
    assert hip.fold_norm(pw, gamma, beta)
    step = (k - 1) // 8
    for places, common in (((0, k // 2), 0.0), ((0, k // 2, k - 1), 0.0), ((0, step, 2 * step), 0.0), ((k - 1, 5 * step), 50.0),
                           ((0, 3 * step, 6 * step), 50.0), ((), 50.0), (tuple(range(0, k, 97)), 0.0)):
        x = torch.randn(m, k, device=DEV, generator=g) + common
        for p in places:
            x[:, p] = 1000.0 * (1 if p % 2 == 0 else -1)
        got = hip.linear(hip.layernorm_deferred(x, gamma, beta, 1e-5, torch.bfloat16), pw, None)
        want = _float32_norm_then_product(x, gamma, beta, 1e-5, w, None, None)
        # against the spread of the result: a row's result is small where its few far elements take most of the norm
        scale = float(want.abs().max())
        assert float((got.float() - want).abs().max()) <= 2e-2 * scale, (places, common)


@pytest.mark.parametrize("m,n,k", [(1, 256, 1024), (8, 4096, 4096), (16, 512, 2048), (30, 1024, 512)])
def test_product_after_a_norm_that_only_scales(m, n, k):
    """`center=False`: x / sqrt(mean(x^2) + eps) * weight, alone and folded into the product of few rows and into
    the fused projection's: the mean stays in the rows (here it is as large as their spread)."""
    hip, ref = _ops(torch.bfloat16)
    g = torch.Generator(device=DEV).manual_seed(m + n + k)
    x = torch.randn(m, k, device=DEV, generator=g) * 2 + 1.5
    gamma = 1 + 0.2 * torch.randn(k, device=DEV, generator=g)
    w = (torch.randn(n, k, device=DEV, generator=g) / k ** 0.5).to(torch.bfloat16)
    bias = torch.randn(n, device=DEV, generator=g) * 0.2
    exact = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-3) * gamma
    f_h, c_h = hip.layernorm(x, gamma, None, 1e-3, torch.bfloat16, True, True, center=False)
    torch.testing.assert_close(f_h, exact, rtol=2e-5, atol=2e-5)
    torch.testing.assert_close(c_h.float(), exact, rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(ref.layernorm(x, gamma, None, 1e-3, torch.float32, True, False, center=False)[0], exact,
                               rtol=1e-5, atol=1e-5)
    want = exact @ w.float().T + bias
    pw = hip.prepare_weight(w)
    assert hip.fold_norm(pw, gamma, None, center=False)
    got = hip.linear(hip.layernorm_deferred(x, gamma, None, 1e-3, torch.bfloat16, center=False), pw, bias)
    assert float((got.float() - want).abs().max()) <= 2e-2 * float(want.abs().max())
    # a norm with a mean folded into the same matrix would be another norm: the deferred rows of one do not
    # meet the folded copy of the other, and are normalised by their own kernel
    other = hip.linear(hip.layernorm_deferred(x, gamma, None, 1e-3, torch.bfloat16, center=True), pw, bias)
    centred = torch.nn.functional.layer_norm(x, (k,), gamma, None, 1e-3) @ w.float().T + bias
    assert float((other.float() - centred).abs().max()) <= 2e-2 * float(centred.abs().max())


def test_product_of_normalised_rows_without_weight_and_bias():
    hip, _ = _ops(torch.bfloat16)
    g = torch.Generator(device=DEV).manual_seed(3)
    x = torch.randn(4, 256, device=DEV, generator=g)
    w = (torch.randn(64, 256, device=DEV, generator=g) / 16).to(torch.bfloat16)
    pw = hip.prepare_weight(w)
    assert hip.fold_norm(pw, None, None)
    got = hip.linear(hip.layernorm_deferred(x, None, None, 1e-3, torch.bfloat16), pw, None)
    want = _float32_norm_then_product(x, None, None, 1e-3, w, None, None)
    torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2)


def test_projection_of_normalised_rows_into_the_cache():
    """The fused projection on a deferred LayerNorm: queries, and keys and values in their pages, as from
    the norm's own kernel and the projection after it."""
    hip, ref = _ops(torch.bfloat16)
    heads, kv, hs, ps = 4, 2, 32, 16
    runs, cached = [1, 1, 3, 1], [40, 0, 7, 15]
    num_pages = 10
    ctx = _make_step(runs, cached, ps, num_pages, seed=2)
    view = ctx.groups["full"]
    width, total = 256, (heads + 2 * kv) * hs
    g = torch.Generator(device=DEV).manual_seed(4)
    x = torch.randn(ctx.num_tokens, width, device=DEV, generator=g) * 2 + 5
    gamma = 1 + 0.2 * torch.randn(width, device=DEV, generator=g)
    beta = 0.3 * torch.randn(width, device=DEV, generator=g)
    w = (torch.randn(total, width, device=DEV, generator=g) / 16).to(torch.bfloat16)
    bias = torch.randn(total, device=DEV, generator=g) * 0.2
    kp_r = torch.full((num_pages, kv, ps, hs), float("nan"), device=DEV, dtype=torch.bfloat16)
    vp_r = torch.full((num_pages, kv, hs, ps), float("nan"), device=DEV, dtype=torch.bfloat16)
    kp, vp = kp_r.clone(), vp_r.clone()
    h_r = ref.layernorm(x, gamma, beta, 1e-5, torch.bfloat16, False, True)[1]
    q_r = ref.qkv_project(h_r, w, bias, heads, kv, hs, 0.25, ctx, view, kp_r, vp_r)
    pw = hip.prepare_weight(w)
    assert hip.fold_norm(pw, gamma, beta)
    q = hip.qkv_project(hip.layernorm_deferred(x, gamma, beta, 1e-5, torch.bfloat16), pw, bias, heads, kv, hs, 0.25,
                        ctx, view, kp, vp)
    torch.testing.assert_close(q.float(), q_r.float(), rtol=2e-2, atol=2e-2)
    assert torch.equal(torch.isnan(kp), torch.isnan(kp_r)) and torch.equal(torch.isnan(vp), torch.isnan(vp_r))
    torch.testing.assert_close(torch.nan_to_num(kp.float()), torch.nan_to_num(kp_r.float()), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(torch.nan_to_num(vp.float()), torch.nan_to_num(vp_r.float()), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("m,n,k", [(33, 4096, 512), (48, 64, 128), (64, 2560, 1024), (65, 48, 384), (100, 1040, 640),
                                   (128, 4096, 2048), (7, 16, 128)])
def test_product_of_some_rows(m, n, k):
    """The kernel for 33 to 128 rows (it takes fewer too) against float32 torch: every count of row tiles, shares
    of K that divide its steps unevenly or are cut to what there is, two or three steps in flight (two beyond 64
    rows), weight tiles beyond the last, float32 and bfloat16 results; and `linear`, which sends the
    float32-result products of such row counts there."""
    from transformers_neuronx_amd.kernels.hip import HipOps, _ACT, _code, _ptr, _stream
    hip = HipOps(torch.bfloat16, DEV)
    g = torch.Generator(device=DEV).manual_seed(m + n + k)
    x = torch.randn(m, k, device=DEV, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, device=DEV, generator=g) / math.sqrt(k)).to(torch.bfloat16)
    bias = torch.randn(n, device=DEV, generator=g)
    res = torch.randn(m, n, device=DEV, generator=g)
    pw = hip.prepare_weight(w)
    assert pw.tiles is not None
    space = torch.empty(4 << 20, dtype=torch.float32, device=DEV)
    exact = x.float() @ w.float().t()
    for shares, ahead in ((0, 0), (1, 2), (2, 3), (3, 2), (7, 3), (64, 0)):
        for act, b, r, wide in ((None, bias, res, True), ("relu", bias, None, False), ("gelu", None, res, True),
                                (None, None, None, True)):
            out = torch.full((m, n), float("nan"), device=DEV, dtype=torch.float32 if wide else torch.bfloat16)
            hip.call("gemm", "tnx_gemm_bf16_mid", _ptr(x), _ptr(pw.tiles), _ptr(b), _ptr(r), _ptr(out), _code(out.dtype),
                     _ACT[act], m, n, k, _ptr(space), space.numel(), shares, ahead, _stream())
            want = exact + (b if b is not None else 0)
            want = {None: want, "relu": torch.relu(want), "gelu": torch.nn.functional.gelu(want)}[act]
            want = want + (r if r is not None else 0)
            tol = dict(rtol=1e-3, atol=1e-3) if wide else dict(rtol=2e-2, atol=2e-2)
            torch.testing.assert_close(out.float(), want, **tol)
    # without a workspace the sum over K is not shared out
    out = torch.empty(m, n, device=DEV)
    hip.call("gemm", "tnx_gemm_bf16_mid", _ptr(x), _ptr(pw.tiles), None, None, _ptr(out), _code(out.dtype), 0, m, n, k,
             None, 0, 4, 0, _stream())
    torch.testing.assert_close(out, exact, rtol=1e-3, atol=1e-3)
    if m > 32:
        seen = []
        inner = hip._call
        hip._call = lambda module, fn, *a, **kw: (seen.append(fn), inner(module, fn, *a, **kw))[1]
        got = hip.linear(x, pw, bias, residual=res, out_f32=True)
        assert seen == ["tnx_gemm_bf16_mid"]
        torch.testing.assert_close(got, exact + bias + res, rtol=1e-3, atol=1e-3)
    with pytest.raises(RuntimeError, match="1 to 128 rows"):
        hip.call("gemm", "tnx_gemm_bf16_mid", _ptr(x), _ptr(pw.tiles), None, None, _ptr(out), _code(out.dtype), 0, 129,
                 n, k, None, 0, 0, 0, _stream())


def test_tiles_a_block_of_the_few_rows_product():
    """The choice at the sizes it was measured at (256 compute units): what the fullest unit gets, with the
    reading of `x` counted, and the larger blocks among equals."""
    from transformers_neuronx_amd.kernels.hip import HipOps, library
    hip = HipOps(torch.bfloat16, DEV)
    if hip.compute_units != 256:
        pytest.skip("the cases are those of 256 compute units")
    rule = library("gemm").tnx_gemm_skinny_tiles_per_block
    assert [rule(8, n) for n in (12288, 16384, 4096, 50272)] == [3, 2, 1, 3]          # OPT-6.7B and the head
    assert [rule(8, n) for n in (27648, 9216, 36864)] == [1, 3, 3]                     # OPT-66B
    assert [rule(8, n) for n in (15360, 5120, 20480)] == [2, 2, 1]                     # OPT-13B
    assert rule(16, 20480) == 3 and rule(16, 28672) == 2 and rule(8, 28672) == 1       # 16 rows read twice the `x`
    assert rule(24, 12288) <= 2 and rule(33, 12288) == 1 and rule(8, 288) == 1
    # and the norm is done by the product only where a block takes two tiles or more and the blocks between
    # them read 40 MB of float32 rows at most
    assert hip._norm_in_the_product(8, 12288, 4096) and not hip._norm_in_the_product(8, 27648, 9216)
    assert not hip._norm_in_the_product(9, 12288, 4096)
    assert hip._norm_in_the_product(4, 16384, 4096) and not hip._norm_in_the_product(8, 16384, 4096)
    assert hip._norm_in_the_product(1, 36864, 9216) and not hip._norm_in_the_product(2, 36864, 9216)


def test_which_products_of_some_rows_go_to_our_kernel():
    """The rule of `linear` at the sizes it was measured at (256 compute units): blocks of 64 columns, K shared
    out until every unit has a block at most, taken where three units in four get one."""
    from transformers_neuronx_amd.kernels.hip import HipOps
    hip = HipOps(torch.bfloat16, DEV)
    if hip.compute_units != 256:
        pytest.skip("the cases are those of 256 compute units")
    w = torch.empty(0, dtype=torch.bfloat16)
    res = object()
    rule = lambda m, n, k, r: hip._some_rows_product(m, n, k, w, w, r, True, 0)
    assert rule(24, 4096, 4096, res) and rule(128, 4096, 16384, res)          # 64 column blocks, 4 shares
    assert rule(32, 5120, 20480, res) and rule(128, 7168, 28672, res)         # 80 x 3 and 112 x 2 blocks
    assert not rule(40, 9216, 36864, res) and not rule(64, 9216, 9216, res)   # 144 blocks, and 288 would be ragged
    assert not rule(20, 1024, 1024, res) and rule(40, 1024, 1024, res)        # small: one launch up to 32 rows
    assert rule(17, 50272, 4096, None) and rule(64, 50272, 4096, None) and not rule(65, 50272, 4096, None)
    assert not rule(16, 4096, 4096, res) and not rule(129, 4096, 4096, res)
    assert not hip._some_rows_product(64, 4096, 4096, w, None, res, True, 0)  # no tile-ordered copy
