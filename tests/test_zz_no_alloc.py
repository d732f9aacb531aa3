"""The decode attention's entry point that allocates nothing (`tnx_attention_decode_static`: the partial
results of split keys go through an array the library holds in device memory) against the entry point
that takes the caller's workspace, both called through ctypes: two calls in a row, the second with a
smaller input, so that what the first left in the array must not show."""
import ctypes
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"

# the planner that an attention mixer brings to every step of its model (the kernels launch by its plan)
from transformers_neuronx_amd.kernels.attention_plan import attention_plan  # noqa: E402
ATTENTION_PLAN = {"attention": attention_plan}


def _case(requests, lengths, heads, kv, hs, ps, splits, seed):
    """Decoding requests of the given lengths over pages drawn at random: what both entry points take."""
    from transformers_neuronx_amd.engine.batch import StepEntry, build_context
    rng = np.random.default_rng(seed)
    num_pages = sum(-(-n // ps) for n in lengths) + 5
    perm = rng.permutation(num_pages).tolist()
    width = max(-(-n // ps) for n in lengths) + 1
    tab = np.full((requests, width), -1, dtype=np.int32)
    for i, n in enumerate(lengths):
        for b in range(-(-n // ps)):
            tab[i, b] = perm.pop()
    ctx = build_context([StepEntry(i, [0], []) for i in range(requests)], [n - 1 for n in lengths],
                        list(range(requests)), {"full": tab}, ps, DEV, planners=ATTENTION_PLAN)
    g = torch.Generator(device=DEV).manual_seed(seed)
    kp = torch.randn(num_pages, kv, ps, hs, device=DEV, generator=g).to(torch.bfloat16)
    vp = torch.randn(num_pages, kv, hs, ps, device=DEV, generator=g).to(torch.bfloat16)
    q = (torch.randn(requests, heads * hs, device=DEV, generator=g) / math.sqrt(hs)).to(torch.bfloat16)
    return ctx, q, kp, vp, num_pages


def _both(lib, ctx, q, kp, vp, num_pages, heads, kv, hs, ps, splits, waves):
    view = ctx.groups["full"]
    n = ctx.plan["decode_runs"].numel()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    out_ws = torch.full_like(q, float("nan"))
    part_o = torch.full((n * heads * splits * hs,), float("nan"), dtype=torch.float32, device=DEV)
    part_ml = torch.full((n * heads * splits * 2,), float("nan"), dtype=torch.float32, device=DEV)
    rc = lib.tnx_attention_decode(p(q), p(kp), p(vp), p(ctx.run_start), p(ctx.cached_lens), p(view.block_table),
                                  view.width, ps, num_pages, p(ctx.plan["decode_runs"]), n, p(out_ws), p(part_o), p(part_ml),
                                  heads, kv, hs, 0, splits, waves, p(ctx.plan["longest_decode"]), 0, stream)
    assert rc == 0, lib.tnx_last_error().decode()
    out_st = torch.full_like(q, float("nan"))
    rc = lib.tnx_attention_decode_static(p(q), p(kp), p(vp), p(ctx.run_start), p(ctx.cached_lens),
                                         p(view.block_table), view.width, ps, num_pages, p(ctx.plan["decode_runs"]), n,
                                         p(out_st), heads, kv, hs, 0, splits, waves, p(ctx.plan["longest_decode"]), stream)
    assert rc == 0, lib.tnx_last_error().decode()
    torch.cuda.synchronize()
    return out_ws, out_st


def test_static_scratch_entry_point_matches_the_workspace_one():
    from transformers_neuronx_amd.kernels.hip import HipOps, library
    from transformers_neuronx_amd.kernels.reference import ReferenceOps
    lib = library("attention")
    heads, kv, hs, ps = 6, 2, 64, 16
    # first a larger call (5 requests, 4 splits), then a smaller one (2 requests, 3 splits)
    for requests, lengths, splits, waves, seed in [(5, [700, 33, 1024, 257, 64], 4, 4, 1),
                                                   (2, [300, 129], 3, 8, 2)]:
        ctx, q, kp, vp, num_pages = _case(requests, lengths, heads, kv, hs, ps, splits, seed)
        out_ws, out_st = _both(lib, ctx, q, kp, vp, num_pages, heads, kv, hs, ps, splits, waves)
        assert not torch.isnan(out_st.float()).any()
        assert torch.equal(out_ws, out_st), (requests, splits)
        want = ReferenceOps(torch.bfloat16, DEV).attention(q, heads, kv, hs, ctx, ctx.groups["full"], kp, vp, None)
        torch.testing.assert_close(out_st.float(), want.float(), rtol=2e-2, atol=2e-2)
    # one split needs no partial results at all
    ctx, q, kp, vp, num_pages = _case(2, [40, 90], heads, kv, hs, ps, 1, 3)
    out_ws, out_st = _both(lib, ctx, q, kp, vp, num_pages, heads, kv, hs, ps, 1, 4)
    assert torch.equal(out_ws, out_st)


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    from transformers_neuronx_amd.kernels.hip import library
    lib = library("attention")
    heads, kv, hs, ps = 64, 64, 128, 16
    ctx, q, kp, vp, num_pages = _case(4, [20, 20, 20, 20], 2, 2, 16, ps, 1, 4)
    view = ctx.groups["full"]
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    # 4 requests x 64 heads x 64 splits x 130 floats > 2^20: refused before anything is launched
    rc = lib.tnx_attention_decode_static(p(q), p(kp), p(vp), p(ctx.run_start), p(ctx.cached_lens),
                                         p(view.block_table), view.width, ps, num_pages, p(ctx.plan["decode_runs"]), 4,
                                         p(q), heads, kv, hs, 0, 64, 4, p(ctx.plan["longest_decode"]),
                                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 1
    assert "static array holds" in lib.tnx_last_error().decode()
