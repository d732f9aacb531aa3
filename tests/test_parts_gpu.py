"""Each part of a layer alone, on the GPU, against the plain functions."""
import math

import numpy as np
import pytest
import torch

import plain_opt

pytestmark = pytest.mark.gpu
QKVO = ("q_proj", "k_proj", "v_proj", "out_proj")     # the names the tests' tensors carry
DEV = "cuda:0"

# the planner that an attention mixer brings to every step of its model (the kernels launch by its plan)
from transformers_neuronx_amd.kernels.attention_plan import attention_plan  # noqa: E402
ATTENTION_PLAN = {"attention": attention_plan}


def _ops(dtype):
    from transformers_neuronx_amd.kernels.hip import HipOps
    return HipOps(dtype, DEV)


def _tol(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)


def _ctx(runs, cached, page_size, num_pages):
    from test_kernels_gpu import _make_step
    return _make_step(runs, cached, page_size, num_pages, seed=3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("affine,eps", [(True, 1e-5), (False, 1e-3)])
def test_norm_part(dtype, affine, eps):
    from transformers_neuronx_amd.parts import NORMS, PartSpec
    norm = NORMS.build(PartSpec("layer_norm", dict(width=72, eps=eps, affine=affine)))
    assert [d.name for d in norm.param_decls("n")] == (["n.weight", "n.bias"] if affine else [])
    g = torch.Generator(device=DEV).manual_seed(0)
    w, b = torch.randn(72, device=DEV, generator=g), torch.randn(72, device=DEV, generator=g)
    norm.load({"n.weight": w, "n.bias": b}, "n", _ops(dtype), dtype)
    x = torch.randn(9, 72, device=DEV, generator=g) * 2 + 1
    f, c = norm.forward(x, True, True)
    want = plain_opt.layer_norm(x, w if affine else None, b if affine else None, eps)
    torch.testing.assert_close(f, want, atol=2e-5, rtol=2e-5)
    assert c.dtype == dtype
    torch.testing.assert_close(c.float(), want, **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("act,bias", [("relu", True), ("gelu", False), ("gelu_new", True)])
def test_feed_forward_part(dtype, act, bias):
    from transformers_neuronx_amd.parts import FEED_FORWARDS, PartSpec
    ffn = FEED_FORWARDS.build(PartSpec("dense", dict(up_name="fc1", down_name="fc2", width=48, inner=136, activation=act, bias=bias)))
    g = torch.Generator(device=DEV).manual_seed(1)
    t = {"p.fc1.weight": (torch.randn(136, 48, device=DEV, generator=g) / 7).to(dtype),
         "p.fc2.weight": (torch.randn(48, 136, device=DEV, generator=g) / 11).to(dtype),
         "p.fc1.bias": torch.randn(136, device=DEV, generator=g), "p.fc2.bias": torch.randn(48, device=DEV, generator=g)}
    assert len(ffn.param_decls("p.")) == (4 if bias else 2)
    ffn.load(t, "p.", _ops(dtype), dtype)
    h = torch.randn(21, 48, device=DEV, generator=g).to(dtype)
    res = torch.randn(21, 48, device=DEV, generator=g)
    out = ffn.forward(h, None, res)
    w = {k: v.float() for k, v in t.items()}
    want = res + plain_opt.feed_forward_part(h.float(), w, "p.", act, bias)
    assert out.dtype == torch.float32
    torch.testing.assert_close(out, want, **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_position_and_embedding_parts(dtype):
    from transformers_neuronx_amd.parts import EMBEDDINGS, PartSpec
    emb = EMBEDDINGS.build(PartSpec("token_table", dict(
        vocab=90, embed_width=24, width=40, position=PartSpec("learned", dict(width=40, max_positions=30, offset=2)),
        table_name="tok", projection_name="proj", position_name="pos")))
    assert [d.name for d in emb.param_decls()] == ["tok", "proj", "pos.weight"]
    assert [d.shape for d in emb.param_decls()] == [(90, 24), (40, 24), (32, 40)]
    g = torch.Generator(device=DEV).manual_seed(2)
    t = {"tok": torch.randn(90, 24, device=DEV, generator=g).to(dtype),
         "proj": (torch.randn(40, 24, device=DEV, generator=g) / 5).to(dtype),
         "pos.weight": torch.randn(32, 40, device=DEV, generator=g).to(dtype)}
    emb.load(t, "", _ops(dtype), dtype)
    ctx = _ctx([4, 1], [0, 17], 16, 4)
    ctx.token_ids.copy_(torch.tensor([5, 6, 7, 8, 9], dtype=torch.int32))
    s = emb.forward(ctx, True)
    rows = t["tok"].float()[torch.tensor([5, 6, 7, 8, 9])] @ t["proj"].float().t()
    pos = torch.tensor([0, 1, 2, 3, 17]) + 2
    want = rows + t["pos.weight"].float()[pos]
    torch.testing.assert_close(s.x, want, **_tol(dtype))
    assert s.compute.dtype == dtype


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv,hs,bias,window", [(4, 4, 16, True, None), (6, 2, 32, False, None),
                                                      (3, 3, 48, True, 20)])
def test_attention_part_in_two_steps(dtype, heads, kv, hs, bias, window):
    """A request's first 37 tokens in one step and 9 more in the next equal the plain whole-sequence
    attention part; another request shares both steps."""
    from transformers_neuronx_amd.cache.manager import LayerCache
    from transformers_neuronx_amd.engine.batch import StepEntry, build_context
    from transformers_neuronx_amd.parts import MIXERS, PartSpec
    width = heads * hs
    mixer = MIXERS.build(PartSpec("attention", dict(names=QKVO, width=width, num_heads=heads, head_size=hs, num_kv_heads=kv,
                                                    bias=bias, window=window)))
    g = torch.Generator(device=DEV).manual_seed(heads)
    t = {}
    for d in mixer.param_decls("a."):
        scale = 1 / math.sqrt(width) if d.role == "matrix" else 0.3
        t[d.name] = torch.randn(*d.shape, device=DEV, generator=g) * scale
        if d.role == "matrix":
            t[d.name] = t[d.name].to(dtype)
    mixer.load(t, "a.", _ops(dtype), dtype)
    need = mixer.cache_need()
    assert (need.kind, need.kv_heads, need.head_size, need.window) == ("paged", kv, hs, window)
    ps, pages = 16, 8
    cache = LayerCache(0, "full", True,
                       {"k": torch.full((pages, kv, ps, hs), float("nan"), device=DEV, dtype=dtype),
                        "v": torch.full((pages, kv, hs, ps), float("nan"), device=DEV, dtype=dtype)})
    n0, n1, other = 37, 9, 21
    h = (torch.randn(n0 + n1, width, device=DEV, generator=g)).to(dtype)
    ho = (torch.randn(other, width, device=DEV, generator=g)).to(dtype)
    table = np.array([[5, 2, 7], [1, 0, -1]], dtype=np.int32)
    outs = []
    for (a0, a1), (b0, b1), cached in (((0, n0), (0, 11), [0, 0]), ((n0, n0 + n1), (11, other), [n0, 11])):
        ctx = build_context([StepEntry("a", [0] * (a1 - a0), []), StepEntry("b", [0] * (b1 - b0), [])], cached,
                            [0, 1], {"full": table}, ps, DEV, planners=ATTENTION_PLAN)
        hin = torch.cat([h[a0:a1], ho[b0:b1]])
        res = torch.zeros(hin.shape[0], width, device=DEV)
        outs.append(mixer.forward(hin, ctx, cache, res)[:a1 - a0])
    got = torch.cat(outs)
    w = {k: v.float() for k, v in t.items()}

    def lin(x, n):
        return plain_opt.linear(x, w[f"a.{n}.weight"], w.get(f"a.{n}.bias"))
    q, k, v = lin(h.float(), "q_proj"), lin(h.float(), "k_proj"), lin(h.float(), "v_proj")
    want = lin(plain_opt.causal_attention(q.cpu(), k.cpu(), v.cpu(), heads, window=window).to(DEV), "out_proj")
    torch.testing.assert_close(got, want, **_tol(dtype))


def test_a_page_edge_shows(tmp_path):
    """Weights random, inputs made: the key at the last place of a page and the key at the first place of
    the next get scores that stand out in turn; a fault at the edge would pick the wrong value."""
    from transformers_neuronx_amd.engine.batch import StepEntry, build_context
    dtype = torch.float32
    ops = _ops(dtype)
    heads, hs, ps = 1, 16, 16
    kp = torch.zeros(4, 1, ps, hs, device=DEV)
    vp = torch.zeros(4, 1, hs, ps, device=DEV)
    table = np.array([[3, 1, 0]], dtype=np.int32)
    n = 40
    ctx0 = build_context([StepEntry("a", [0] * n, [])], [0], [0], {"full": table}, ps, DEV, planners=ATTENTION_PLAN)
    qkv = torch.zeros(n, 3 * hs, device=DEV)
    for j in range(n):
        qkv[j, hs + (j % hs)] = 1.0 + j / 100.0           # key j points along axis j % 16, a little longer each
        qkv[j, 2 * hs:] = float(j)                         # value j is j
    ops.qkv_write(qkv, None, heads, 1, hs, 1.0, ctx0, ctx0.groups["full"], kp, vp)
    for target in (15, 16, 31, 32, 0, 39):
        ctx = build_context([StepEntry("a", [0], [])], [n], [0], {"full": table}, ps, DEV, planners=ATTENTION_PLAN)
        q = torch.zeros(1, hs, device=DEV)
        q[0, target % hs] = 200.0
        # keys target, target +- 16 share the axis; the longest (latest) wins unless masked: ask for it exactly
        best = max(j for j in range(n) if j % hs == target % hs)
        kq = torch.zeros(1, 3 * hs, device=DEV)
        qq = ops.qkv_write(torch.cat([q, kq[:, :2 * hs]], 1), None, heads, 1, hs, 1.0, ctx, ctx.groups["full"], kp, vp)
        out = ops.attention(qq, heads, 1, hs, ctx, ctx.groups["full"], kp, vp, None)
        assert abs(float(out[0, 0]) - best) < 1e-3, (target, float(out[0, 0]), best)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("order", ["pre_norm", "post_norm"])
def test_block_arrangements(dtype, order):
    """A whole layer through the block part, one request in one step, against the plain block."""
    from transformers_neuronx_amd.cache.manager import LayerCache
    from transformers_neuronx_amd.engine.batch import StepEntry, build_context
    from transformers_neuronx_amd.parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, PartSpec, Stream)
    width, heads, hs, inner, n, ps = 64, 2, 32, 160, 23, 16
    norm = PartSpec("layer_norm", dict(width=width, eps=2e-5, affine=True))
    mixer = MIXERS.build(PartSpec("attention", dict(names=QKVO, width=width, num_heads=heads, head_size=hs)))
    ffn = FEED_FORWARDS.build(PartSpec("dense", dict(up_name="fc1", down_name="fc2", width=width, inner=inner, activation="relu")))
    n1, n2 = NORMS.build(norm), NORMS.build(norm)
    block = BLOCKS.build(PartSpec(order), mixer, ffn, n1, n2)
    named = [(mixer, "model.decoder.layers.0.self_attn."), (ffn, "model.decoder.layers.0."),
             (n1, "model.decoder.layers.0.self_attn_layer_norm"), (n2, "model.decoder.layers.0.final_layer_norm")]
    g = torch.Generator(device=DEV).manual_seed(6)
    t = {}
    for part, prefix in named:
        for d in part.param_decls(prefix):
            v = torch.randn(*d.shape, device=DEV, generator=g) * (0.1 if d.role == "matrix" else 0.3)
            if d.init == "around_one":
                v = v + 1
            t[d.name] = v.to(dtype) if d.role == "matrix" else v
    ops = _ops(dtype)
    for part, prefix in named:
        part.load(t, prefix, ops, dtype)
    cache = LayerCache(0, "full", True, {"k": torch.zeros(3, heads, ps, hs, device=DEV, dtype=dtype),
                                         "v": torch.zeros(3, heads, hs, ps, device=DEV, dtype=dtype)})
    ctx = build_context([StepEntry("a", [0] * n, [])], [0], [0], {"full": np.array([[2, 0]], dtype=np.int32)}, ps, DEV, planners=ATTENTION_PLAN)
    x = torch.randn(n, width, device=DEV, generator=g)
    out = block.forward(Stream(x, ops.cast(x, dtype)), ctx, cache)
    cfg = dict(num_attention_heads=heads, activation_function="relu", do_layer_norm_before=order == "pre_norm",
               layer_norm_eps=2e-5)
    want = plain_opt.block(x.cpu(), {k: v.float().cpu() for k, v in t.items()}, cfg, 0)
    torch.testing.assert_close(out.x.cpu(), want, **_tol(dtype))
    if order == "post_norm":
        assert out.compute is not None and out.compute.dtype == dtype


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("projects,normed", [(False, True), (True, False)])
def test_head_part(dtype, projects, normed):
    from transformers_neuronx_amd.parts import HEADS, PartSpec, Stream
    width, embed, vocab = 64, (40 if projects else 64), 333
    head = HEADS.build(PartSpec("vocab_projection", dict(
        vocab=vocab, embed_width=embed, width=width,
        norm=PartSpec("layer_norm", dict(width=width, eps=1e-5, affine=True)) if normed else None,
        weight_name="lm_head.weight", tied_to="tok", projection_name="proj", norm_name="fn")))
    decls = {d.name: d for d in head.param_decls()}
    assert decls["lm_head.weight"].tied_to == "tok" and ("proj" in decls) == projects and ("fn.weight" in decls) == normed
    g = torch.Generator(device=DEV).manual_seed(8)
    t = {"lm_head.weight": (torch.randn(vocab, embed, device=DEV, generator=g) / 8).to(dtype),
         "proj": (torch.randn(embed, width, device=DEV, generator=g) / 8).to(dtype),
         "fn.weight": torch.randn(width, device=DEV, generator=g) + 1, "fn.bias": torch.randn(width, device=DEV, generator=g)}
    head.load(t, "", _ops(dtype), dtype)
    ctx = _ctx([6, 1], [0, 9], 16, 3)
    ctx.logits_rows = torch.tensor([5, 2, 6], dtype=torch.int32, device=DEV)
    x = torch.randn(7, width, device=DEV, generator=g)
    logits = head.forward(Stream(x, None), ctx)
    rows = x[[5, 2, 6]]
    if normed:
        rows = plain_opt.layer_norm(rows, t["fn.weight"], t["fn.bias"], 1e-5)
    if projects:
        rows = rows @ t["proj"].float().t()
    want = rows @ t["lm_head.weight"].float().t()
    assert logits.dtype == torch.float32 and logits.shape == (3, vocab)
    torch.testing.assert_close(logits, want, **_tol(dtype))
