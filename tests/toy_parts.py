"""Toy parts, defined outside the package, to show that the framework takes new ones as they are:
a mixer with per-request state of fixed size, and a model whose run order names a layer twice,
lets a layer read another layer's cache, and mixes full and windowed attention."""
import math

import torch

import plain_opt
from transformers_neuronx_amd.parts import (CacheNeed, LayerCall, LayerSpec, Mixer, ModelSpec, ParamDecl, PartSpec,
                                            register_mixer)


QKVO = ("q_proj", "k_proj", "v_proj", "out_proj")     # the names the toy models give their attention tensors


@register_mixer("toy_ema")
class ToyEmaMixer(Mixer):
    """y_t = s_t, s_t = decay * s_{t-1} + (1 - decay) * (h_t W^T), s_{-1} = 0: a running average kept in a
    float32 state slot per request. Written with torch operations: a toy, not a kernel."""

    def __init__(self, width: int, decay: float):
        self.width, self.decay = width, decay

    def cache_need(self):
        return CacheNeed("state", state_shapes=(("ema", (self.width,)),))

    def param_decls(self, prefix):
        return [ParamDecl(prefix + "in.weight", (self.width, self.width))]

    def load(self, tensors, prefix, ops, dtype):
        super().load(tensors, prefix, ops, dtype)
        self.w = tensors[prefix + "in.weight"]

    def forward(self, h, ctx, cache, residual):
        u = self.ops.linear(h, self.w, None, out_f32=True)
        state = cache.state["ema"]
        out = torch.empty_like(u)
        start = 0
        for r in range(ctx.num_requests):
            n, slot = int(ctx.run_lens_host[r]), int(ctx.slots_host[r])
            s = state[slot]
            for t in range(start, start + n):
                s = self.decay * s + (1.0 - self.decay) * u[t]
                out[t] = s
            state[slot] = s
            start += n
        return residual + out


def toy_spec(width=64, heads=4, inner=96, vocab=300, positions=160, window=24, eps=1e-5):
    hs = width // heads
    norm = PartSpec("layer_norm", dict(width=width, eps=eps, affine=True))
    ffn = PartSpec("dense", dict(up_name="fc1", down_name="fc2", width=width, inner=inner, activation="gelu_new", bias=True))

    def layer(i, mixer, block="pre_norm"):
        return LayerSpec(prefix=f"layers.{i}.", block=block, mixer=mixer, feed_forward=ffn, mixer_norm=norm,
                         feed_forward_norm=norm, mixer_name="mix.", feed_forward_name="ffn.",
                         mixer_norm_name="norm1", feed_forward_norm_name="norm2")
    full = PartSpec("attention", dict(names=QKVO, width=width, num_heads=heads, head_size=hs, num_kv_heads=heads // 2))
    windowed = PartSpec("attention", dict(names=QKVO, width=width, num_heads=heads, head_size=hs, window=window))
    reader = PartSpec("attention", dict(names=QKVO, width=width, num_heads=heads, head_size=hs, num_kv_heads=heads // 2,
                                        own_kv=False))
    ema = PartSpec("toy_ema", dict(width=width, decay=0.75))
    layers = (layer(0, full), layer(1, ema), layer(2, windowed), layer(3, reader))
    schedule = (LayerCall(0, cache=0), LayerCall(1), LayerCall(2), LayerCall(3, cache=0, writes=False),
                LayerCall(0), LayerCall(1))
    embedding = PartSpec("token_table", dict(
        vocab=vocab, embed_width=width, width=width,
        position=PartSpec("learned", dict(width=width, max_positions=positions, offset=0)),
        table_name="embed.weight", projection_name=None, position_name="positions"))
    head = PartSpec("vocab_projection", dict(vocab=vocab, embed_width=width, width=width, norm=norm,
                                             weight_name="head.weight", tied_to=None, projection_name=None,
                                             norm_name="final_norm"))
    return ModelSpec(hidden_size=width, vocab_size=vocab, max_positions=positions, embedding=embedding,
                     layers=layers, schedule=schedule, head=head, init_std=0.08)


def toy_plain_logits(w, tokens, width=64, heads=4, window=24, eps=1e-5):
    """The toy model on one whole sequence, from the plain functions."""
    w = {k: v.float() for k, v in w.items()}
    n = len(tokens)
    hs = width // heads
    x = w["embed.weight"][torch.tensor(tokens)] + w["positions.weight"][:n]
    kv_of_first = {}

    def ln(t, name):
        return plain_opt.layer_norm(t, w[name + ".weight"], w[name + ".bias"], eps)

    def ffn(t, p):
        h = plain_opt.activation(plain_opt.linear(t, w[p + "ffn.fc1.weight"], w[p + "ffn.fc1.bias"]), "gelu_new")
        return plain_opt.linear(h, w[p + "ffn.fc2.weight"], w[p + "ffn.fc2.bias"])

    def attn(t, p, kv=None, win=None, remember=False):
        q = plain_opt.linear(t, w[p + "mix.q_proj.weight"], w[p + "mix.q_proj.bias"])
        if kv is None:
            k = plain_opt.linear(t, w[p + "mix.k_proj.weight"], w[p + "mix.k_proj.bias"])
            v = plain_opt.linear(t, w[p + "mix.v_proj.weight"], w[p + "mix.v_proj.bias"])
        else:
            k, v = kv
        if remember:
            kv_of_first["kv"] = (k, v)
        c = plain_opt.causal_attention(q, k, v, heads, window=win)
        return plain_opt.linear(c, w[p + "mix.out_proj.weight"], w[p + "mix.out_proj.bias"])

    def ema(t, p):
        u = plain_opt.linear(t, w[p + "mix.in.weight"])
        s, out = torch.zeros(width), []
        for i in range(n):
            s = 0.75 * s + 0.25 * u[i]
            out.append(s)
        return torch.stack(out)

    order = [(0, "first"), (1, None), (2, None), (3, None), (0, "again"), (1, None)]
    for layer, tag in order:
        p = f"layers.{layer}."
        h = ln(x, p + "norm1")
        if layer == 0:
            x = x + attn(h, p, remember=(tag == "first"))
        elif layer == 1:
            x = x + ema(h, p)
        elif layer == 2:
            x = x + attn(h, p, win=window)
        else:
            x = x + attn(h, p, kv=kv_of_first["kv"])
        x = x + ffn(ln(x, p + "norm2"), p)
    return plain_opt.linear(ln(x, "final_norm"), w["head.weight"])


# ---------------------------------------------------------------- a routed feed-forward, another position encoding

from transformers_neuronx_amd.parts import FeedForward, PositionEncoding, register_feed_forward, register_position  # noqa: E402


@register_feed_forward("toy_routed")
class ToyRoutedFeedForward(FeedForward):
    """Every token goes to the one expert its router names: y = p_e * W2_e relu(W1_e h), e = argmax of the
    router's logits (float32), p_e its softmax probability. Written with torch indexing: a toy."""

    def __init__(self, width: int, inner: int, experts: int):
        self.width, self.inner, self.experts = width, inner, experts

    def param_decls(self, prefix):
        d = [ParamDecl(prefix + "router.weight", (self.experts, self.width), "norm")]      # kept in float32
        for e in range(self.experts):
            d += [ParamDecl(f"{prefix}experts.{e}.up.weight", (self.inner, self.width)),
                  ParamDecl(f"{prefix}experts.{e}.down.weight", (self.width, self.inner))]
        return d

    def load(self, tensors, prefix, ops, dtype):
        super().load(tensors, prefix, ops, dtype)
        self.router = tensors[prefix + "router.weight"].float()
        self.up = [tensors[f"{prefix}experts.{e}.up.weight"] for e in range(self.experts)]
        self.down = [tensors[f"{prefix}experts.{e}.down.weight"] for e in range(self.experts)]

    def forward(self, h, ctx, residual):
        probs = torch.softmax(h.float() @ self.router.t(), dim=-1)
        weight, choice = probs.max(dim=-1)
        out = residual.clone()
        for e in range(self.experts):
            rows = torch.nonzero(choice == e).flatten()
            if rows.numel():
                mid = self.ops.linear(h[rows].contiguous(), self.up[e], None, act="relu")
                y = self.ops.linear(mid, self.down[e], None, out_f32=True)
                out[rows] += weight[rows, None] * y
        return out


@register_position("toy_sinusoid")
class ToySinusoid(PositionEncoding):
    """Fixed sines and cosines of the position, added to the embedded tokens; no parameters."""

    def __init__(self, width: int, base: float):
        self.width, self.base = width, base

    def at_input(self, x, positions, want_compute):
        half = self.width // 2
        freq = self.base ** (-torch.arange(half, device=x.device, dtype=torch.float32) / half)
        angle = positions.float()[:, None] * freq[None, :]
        out = x.float() + torch.cat([torch.sin(angle), torch.cos(angle)], dim=-1)
        return out, (out.to(self.dtype) if want_compute else None)


def toy_spec_routed(width=48, heads=3, inner=40, experts=3, vocab=211, positions=140, eps=1e-4, base=50.0):
    """Two layers: attention with a routed feed-forward (norms after each half), attention with a dense
    one (norms before); sinusoid positions; no norm before the head."""
    hs = width // heads
    norm = PartSpec("layer_norm", dict(width=width, eps=eps, affine=True))
    attention = PartSpec("attention", dict(names=QKVO, width=width, num_heads=heads, head_size=hs))
    routed = PartSpec("toy_routed", dict(width=width, inner=inner, experts=experts))
    dense = PartSpec("dense", dict(up_name="fc1", down_name="fc2", width=width, inner=2 * inner, activation="relu", bias=False))

    def layer(i, ffn, block):
        return LayerSpec(prefix=f"layers.{i}.", block=block, mixer=attention, feed_forward=ffn, mixer_norm=norm,
                         feed_forward_norm=norm, mixer_name="mix.", feed_forward_name="ffn.",
                         mixer_norm_name="norm1", feed_forward_norm_name="norm2")
    embedding = PartSpec("token_table", dict(
        vocab=vocab, embed_width=width, width=width, position=PartSpec("toy_sinusoid", dict(width=width, base=base)),
        table_name="embed.weight", projection_name=None, position_name="positions"))
    head = PartSpec("vocab_projection", dict(vocab=vocab, embed_width=width, width=width, norm=None,
                                             weight_name="head.weight", tied_to="embed.weight",
                                             projection_name=None, norm_name="final_norm"))
    return ModelSpec(hidden_size=width, vocab_size=vocab, max_positions=positions, embedding=embedding,
                     layers=(layer(0, routed, "post_norm"), layer(1, dense, "pre_norm")),
                     schedule=(LayerCall(0), LayerCall(1)), head=head, init_std=0.1)


def toy_routed_plain_logits(w, tokens, width=48, heads=3, experts=3, eps=1e-4, base=50.0):
    w = {k: v.float() for k, v in w.items()}
    n, half = len(tokens), width // 2
    freq = base ** (-torch.arange(half, dtype=torch.float32) / half)
    angle = torch.arange(n, dtype=torch.float32)[:, None] * freq[None, :]
    x = w["embed.weight"][torch.tensor(tokens)] + torch.cat([torch.sin(angle), torch.cos(angle)], dim=-1)

    def ln(t, name):
        return plain_opt.layer_norm(t, w[name + ".weight"], w[name + ".bias"], eps)

    def attn(t, p):
        q, k, v = (plain_opt.linear(t, w[f"{p}mix.{s}_proj.weight"], w[f"{p}mix.{s}_proj.bias"]) for s in "qkv")
        c = plain_opt.causal_attention(q, k, v, heads)
        return plain_opt.linear(c, w[p + "mix.out_proj.weight"], w[p + "mix.out_proj.bias"])

    # layer 0: norms after each half, routed feed-forward
    p = "layers.0."
    x = ln(x + attn(x, p), p + "norm1")
    probs = torch.softmax(x @ w[p + "ffn.router.weight"].t(), dim=-1)
    y = torch.zeros_like(x)
    for t in range(n):
        e = int(probs[t].argmax())
        mid = torch.relu(plain_opt.linear(x[t:t + 1], w[f"{p}ffn.experts.{e}.up.weight"]))
        y[t] = probs[t, e] * plain_opt.linear(mid, w[f"{p}ffn.experts.{e}.down.weight"])[0]
    x = ln(x + y, p + "norm2")
    # layer 1: norms before each half, dense feed-forward without bias
    p = "layers.1."
    x = x + attn(ln(x, p + "norm1"), p)
    h = torch.relu(plain_opt.linear(ln(x, p + "norm2"), w[p + "ffn.fc1.weight"]))
    x = x + plain_opt.linear(h, w[p + "ffn.fc2.weight"])
    return plain_opt.linear(x, w["embed.weight"])


# ---------------------------------------------------------------- an encoding that turns queries and keys, a norm with a kernel of its own

import ctypes  # noqa: E402
import os  # noqa: E402

from transformers_neuronx_amd.parts import Norm, register_norm  # noqa: E402

TOY_KERNEL_SOURCE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "toy_kernels", "toy_norm.hip")


def register_toy_kernels():
    """The toy norm's kernel module: its source and its C signature, registered from outside the package."""
    from transformers_neuronx_amd.kernels import build, hip
    build.register_module("toy_norm", TOY_KERNEL_SOURCE)
    vp, ci, cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
    hip.register_signatures("toy_norm", {"tnx_toy_scale_norm": [vp, vp, cf, vp, vp, ci, ci, ci, vp]})


@register_position("toy_rotation")
class ToyRotation(PositionEncoding):
    """Turns every pair (x[2i], x[2i+1]) of each query and key head by the angle position * base^(-2i/head_size),
    so that a score depends on the distance of query and key only. Torch operations on the device: a toy."""

    def __init__(self, base: float, tables: bool = False, positions: int = 0):
        """`tables`: hand the attention mixer the pairwise form (`pair_tables`) for `positions` positions, which
        the projection applies in its own launch; otherwise `on_query_key` turns the projections with torch."""
        self.base, self.tables, self.positions = base, tables, positions
        self.recordable = bool(tables)

    def load(self, tensors, prefix, ops, dtype):
        super().load(tensors, prefix, ops, dtype)
        self.device = next(iter(tensors.values())).device if tensors else "cpu"

    def pair_tables(self, head_size):
        if not self.tables:
            return None
        freq = self.base ** (-torch.arange(head_size // 2, dtype=torch.float32) * 2 / head_size)
        angle = torch.arange(self.positions, dtype=torch.float32)[:, None] * freq[None, :]
        cos, sin = torch.cos(angle), torch.sin(angle)
        # (x0, x1) -> (x0 cos - x1 sin, x1 cos + x0 sin): a = cos for both, b = -sin for the first, +sin for the second
        a = torch.stack([cos, cos], dim=-1).reshape(self.positions, head_size)
        b = torch.stack([-sin, sin], dim=-1).reshape(self.positions, head_size)
        return a.contiguous().to(self.device), b.contiguous().to(self.device)

    def on_query_key(self, qkv, ctx, num_heads, num_kv_heads, head_size):
        t = qkv.shape[0]
        turned = (num_heads + num_kv_heads) * head_size            # queries and keys; values stay
        x = qkv[:, :turned].float().reshape(t, -1, head_size // 2, 2)
        freq = self.base ** (-torch.arange(head_size // 2, device=qkv.device, dtype=torch.float32) * 2 / head_size)
        angle = ctx.positions.float()[:, None, None] * freq[None, None, :]
        cos, sin = torch.cos(angle), torch.sin(angle)
        out = torch.stack([x[..., 0] * cos - x[..., 1] * sin, x[..., 0] * sin + x[..., 1] * cos], dim=-1)
        return torch.cat([out.reshape(t, turned).to(qkv.dtype), qkv[:, turned:]], dim=1).contiguous()


@register_norm("toy_scale_norm")
class ToyScaleNorm(Norm):
    """y = x * w / sqrt(mean(x^2) + eps). On the HIP backend it runs a kernel of its own, compiled from a
    source under tests/ and reached through `ops.call`; elsewhere torch."""

    recordable = True

    def __init__(self, width: int, eps: float, fold: bool = False):
        """`fold`: where a matrix product alone reads this norm, let the backend fold it into that product (its
        `fold_norm` / `layernorm_deferred` with `center=False`, the norm that only scales) instead of running the
        kernel this part brings."""
        self.width, self.eps, self.fold = width, eps, fold

    def param_decls(self, prefix):
        return [ParamDecl(prefix + ".weight", (self.width,), "vector", "around_one")]

    def fold_into(self, w):
        return self.fold and self.ops.fold_norm(w, self.weight, None, center=False)

    def deferred(self, x):
        return self.ops.layernorm_deferred(x, self.weight, None, self.eps, self.dtype, center=False)

    def load(self, tensors, prefix, ops, dtype):
        super().load(tensors, prefix, ops, dtype)
        self.weight = tensors[prefix + ".weight"]
        if getattr(ops, "name", "") == "hip":
            register_toy_kernels()

    def forward(self, x, want_f32, want_compute):
        if getattr(self.ops, "name", "") != "hip":
            y = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + self.eps) * self.weight
            return (y if want_f32 else None), (y.to(self.dtype) if want_compute else None)
        same = self.dtype == torch.float32
        out_f32 = torch.empty_like(x) if (want_f32 or (want_compute and same)) else None
        out_cd = torch.empty_like(x, dtype=self.dtype) if (want_compute and not same) else None
        ops = self.ops
        ops.call("toy_norm", "tnx_toy_scale_norm", ops.pointer(x), ops.pointer(self.weight), float(self.eps),
                 ops.pointer(out_f32), ops.pointer(out_cd), 1, x.shape[0], x.shape[1], ops.stream())
        return (out_f32 if want_f32 else None), ((out_f32 if same else out_cd) if want_compute else None)


@register_mixer("toy_latent")
class ToyLatentMixer(Mixer):
    """Keeps one small vector per token in pages of its own shape, z_t = h_t W_in^T (a paged cache that is
    no pair of keys and values), and returns the mean of the vectors so far through W_out: y_t = mean_{j<=t}
    z_j W_out^T. Torch operations and a loop over requests: a toy."""

    def __init__(self, width: int, latent: int):
        self.width, self.latent = width, latent

    def cache_need(self):
        return CacheNeed("paged", page_tensors=(("z", ("page", self.latent)),))

    def param_decls(self, prefix):
        return [ParamDecl(prefix + "down.weight", (self.latent, self.width)),
                ParamDecl(prefix + "up.weight", (self.width, self.latent))]

    def load(self, tensors, prefix, ops, dtype):
        super().load(tensors, prefix, ops, dtype)
        self.down, self.up = tensors[prefix + "down.weight"], tensors[prefix + "up.weight"]

    def forward(self, h, ctx, cache, residual):
        z = self.ops.linear(h, self.down, None, out_f32=True)
        pages = cache.pages["z"]                                  # [pages, page_size, latent]
        view = ctx.groups[cache.group]
        table = view.block_table.cpu()
        ps = view.page_size
        means = torch.empty_like(z)
        start = 0
        for r in range(ctx.num_requests):
            n, have = int(ctx.run_lens_host[r]), int(ctx.cached_lens_host[r])
            for i in range(n):                                    # store, token by token
                pos = have + i
                pages[int(table[r, pos // ps]), pos % ps] = z[start + i].to(pages.dtype)
            blocks = [int(b) for b in table[r, :-(-(have + n) // ps)]]
            so_far = pages[blocks].reshape(-1, self.latent)[:have + n].float()
            sums = torch.cumsum(so_far, dim=0)[have:]
            means[start:start + n] = sums / torch.arange(have + 1, have + n + 1, device=z.device)[:, None]
            start += n
        return self.ops.linear(means.to(self.dtype), self.up, None, residual=residual, out_f32=True)


def toy_spec_rotating(width=96, heads=3, kv_heads=1, inner=72, vocab=157, positions=150, eps=1e-3, base=100.0,
                      tables=False, latent_layer=True, fold=False):
    """Attention whose queries and keys are turned by their positions (no encoding at the input), grouped
    heads, between two such layers one whose mixer keeps a paged cache of another shape; a scale-only norm
    with its own kernel, names of its own for every tensor."""
    hs = width // heads
    norm = PartSpec("toy_scale_norm", dict(width=width, eps=eps, fold=fold))
    mixer = PartSpec("attention", dict(width=width, num_heads=heads, head_size=hs, num_kv_heads=kv_heads, bias=False,
                                       names=("wq", "wk", "wv", "wo"),
                                       rotation=PartSpec("toy_rotation", dict(base=base, tables=tables, positions=positions))))
    ffn = PartSpec("dense", dict(width=width, inner=inner, activation="gelu", bias=False, up_name="up", down_name="down"))
    latent = PartSpec("toy_latent", dict(width=width, latent=24))
    layers = tuple(LayerSpec(prefix=f"blocks.{i}.", block="pre_norm", mixer=latent if i == 1 and latent_layer else mixer, feed_forward=ffn,
                             mixer_norm=norm, feed_forward_norm=norm, mixer_name="attn.", feed_forward_name="mlp.",
                             mixer_norm_name="attn_norm", feed_forward_norm_name="mlp_norm") for i in range(3))
    embedding = PartSpec("token_table", dict(vocab=vocab, embed_width=width, width=width, position=PartSpec("none", {}),
                                             table_name="tokens.weight", projection_name=None, position_name=None))
    head = PartSpec("vocab_projection", dict(vocab=vocab, embed_width=width, width=width, norm=norm,
                                             weight_name="out.weight", tied_to=None, projection_name=None,
                                             norm_name="out_norm"))
    return ModelSpec(hidden_size=width, vocab_size=vocab, max_positions=positions, embedding=embedding, layers=layers,
                     schedule=ModelSpec.sequential(3), head=head, init_std=0.1)


def toy_rotating_plain_logits(w, tokens, width=96, heads=3, kv_heads=1, eps=1e-3, base=100.0, first_position=0,
                              latent_layer=True):
    """The rotating toy model on one whole sequence; `first_position` shifts every position (the logits must
    not change: only distances count)."""
    w = {k: v.float() for k, v in w.items()}
    n, hs = len(tokens), width // heads
    x = w["tokens.weight"][torch.tensor(tokens)]
    pos = torch.arange(first_position, first_position + n, dtype=torch.float32)
    freq = base ** (-torch.arange(hs // 2, dtype=torch.float32) * 2 / hs)
    angle = pos[:, None] * freq[None, :]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]

    def norm(t, name):
        return t * torch.rsqrt((t * t).mean(-1, keepdim=True) + eps) * w[name + ".weight"]

    def turn(t, nh):
        t = t.reshape(n, nh, hs // 2, 2)
        return torch.stack([t[..., 0] * cos - t[..., 1] * sin, t[..., 0] * sin + t[..., 1] * cos], -1).reshape(n, nh * hs)

    for i in range(3):
        p = f"blocks.{i}."
        h = norm(x, p + "attn_norm")
        if i == 1 and latent_layer:                 # the layer that keeps a small vector per token and averages them
            z = plain_opt.linear(h, w[p + "attn.down.weight"])
            means = torch.cumsum(z, dim=0) / torch.arange(1, n + 1, dtype=torch.float32)[:, None]
            x = x + plain_opt.linear(means, w[p + "attn.up.weight"])
            h = norm(x, p + "mlp_norm")
            x = x + plain_opt.linear(plain_opt.activation(plain_opt.linear(h, w[p + "mlp.up.weight"]), "gelu"),
                                     w[p + "mlp.down.weight"])
            continue
        q = turn(plain_opt.linear(h, w[p + "attn.wq.weight"]), heads)
        k = turn(plain_opt.linear(h, w[p + "attn.wk.weight"]), kv_heads)
        v = plain_opt.linear(h, w[p + "attn.wv.weight"])
        group = heads // kv_heads
        k = k.reshape(n, kv_heads, hs).repeat_interleave(group, dim=1).reshape(n, width)
        v = v.reshape(n, kv_heads, hs).repeat_interleave(group, dim=1).reshape(n, width)
        x = x + plain_opt.linear(plain_opt.causal_attention(q, k, v, heads), w[p + "attn.wo.weight"])
        h = norm(x, p + "mlp_norm")
        x = x + plain_opt.linear(plain_opt.activation(plain_opt.linear(h, w[p + "mlp.up.weight"]), "gelu"),
                                 w[p + "mlp.down.weight"])
    return plain_opt.linear(norm(x, "out_norm"), w["out.weight"])
