"""Toy parts, defined outside the package, to show that the framework takes new ones as they are:
a mixer with per-request state of fixed size, and a model whose run order names a layer twice,
lets a layer read another layer's cache, and mixes full and windowed attention."""
import math

import torch

import plain_opt
from transformers_neuronx_amd.parts import (CacheNeed, LayerCall, LayerSpec, Mixer, ModelSpec, ParamDecl, PartSpec,
                                            register_mixer)


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
    ffn = PartSpec("dense", dict(width=width, inner=inner, activation="gelu_new", bias=True))

    def layer(i, mixer, block="pre_norm"):
        return LayerSpec(prefix=f"layers.{i}.", block=block, mixer=mixer, feed_forward=ffn, mixer_norm=norm,
                         feed_forward_norm=norm, mixer_name="mix.", feed_forward_name="ffn.",
                         mixer_norm_name="norm1", feed_forward_norm_name="norm2")
    full = PartSpec("attention", dict(width=width, num_heads=heads, head_size=hs, num_kv_heads=heads // 2))
    windowed = PartSpec("attention", dict(width=width, num_heads=heads, head_size=hs, window=window))
    reader = PartSpec("attention", dict(width=width, num_heads=heads, head_size=hs, num_kv_heads=heads // 2,
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
