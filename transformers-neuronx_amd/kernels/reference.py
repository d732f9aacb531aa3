"""A plain torch rendition of every kernel, with the same call signatures.

It is what each HIP kernel is tested against, and it can stand in for the whole
backend (`EngineConfig(kernels="reference")`) to debug the engine on any
device. It is never chosen by itself: the product path is `kernels.hip`.
All arithmetic is done in float32 and rounded once to the output dtype, which
is what the kernels do with their float32 accumulators.
"""
import math
from typing import Optional

import torch


def philox_uniform(seed: int, counter: int) -> float:
    """Philox-4x32-10 keyed by `seed`, counter `counter`; first word -> [0, 1)."""
    m0, m1, w0, w1, mask = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85, 0xFFFFFFFF
    c = [counter & mask, (counter >> 32) & mask, 0, 0]
    k = [seed & mask, (seed >> 32) & mask]
    for _ in range(10):
        p0, p1 = m0 * c[0], m1 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & mask, p1 & mask, ((p0 >> 32) ^ c[3] ^ k[1]) & mask, p0 & mask]
        k = [(k[0] + w0) & mask, (k[1] + w1) & mask]
    return (c[0] >> 8) * (1.0 / (1 << 24))


class ReferenceOps:
    name = "reference"

    def __init__(self, dtype: torch.dtype, device="cpu"):
        self.dtype = dtype
        self.device = torch.device(device)

    # ---------------------------------------------------------------- input end

    def embed(self, token_ids, table, dtype=None, kept_tokens=None):
        """Rows of the token table; an id -1 - k is the token kept in `kept_tokens[k]`."""
        ids = token_ids.long()
        if kept_tokens is not None:
            ids = torch.where(ids < 0, kept_tokens.long()[(-1 - ids).clamp(min=0)], ids)
        return table[ids]

    def send_tokens(self, tokens, kept, ctx):
        self.store_tokens(kept, tokens, ctx)
        return tokens

    def receive_tokens(self, sent):
        return sent.tolist()

    def store_tokens(self, kept, tokens, ctx):
        slots = ctx.slots.long()[ctx.token_request.long()[ctx.logits_rows.long()]]
        kept[slots] = tokens.to(kept.dtype)

    def add_positions(self, src, positions, table, offset, dtype, want_compute):
        x = src.float() + table[(positions + offset).long()].float()
        return x, (x.to(dtype) if want_compute else None)

    def to_stream(self, src, dtype, want_compute):
        x = src.float()
        return x, (x.to(dtype) if want_compute else None)

    # ---------------------------------------------------------------- norms

    def layernorm(self, x, weight, bias, eps, dtype, want_f32, want_compute, center=True):
        """`center=False`: the norm that only scales, x / sqrt(mean(x^2) + eps) (times weight, plus bias)."""
        x = x.float()
        mean = x.mean(-1, keepdim=True) if center else torch.zeros_like(x[:, :1])
        var = ((x - mean) ** 2).mean(-1, keepdim=True)
        y = (x - mean) * torch.rsqrt(var + eps)
        if weight is not None:
            y = y * weight.float()
        if bias is not None:
            y = y + bias.float()
        return (y if want_f32 else None), (y.to(dtype) if want_compute else None)

    # ---------------------------------------------------------------- matrix products

    def layernorm_deferred(self, x, weight, bias, eps, dtype, center=True):
        """The norm's output for a part that only multiplies it; a backend may hand back something a
        product resolves instead (`HipOps.layernorm_deferred`)."""
        return self.layernorm(x, weight, bias, eps, dtype, False, True, center)[1]

    def fold_norm(self, w, weight, bias, center=True) -> bool:
        return False

    def prepare_weight(self, w):
        """Matrices are used as they are here."""
        return w

    @staticmethod
    def activation(y, act):
        if act is None or act == "none":
            return y
        if act == "relu":
            return torch.relu(y)
        if act == "gelu":
            return 0.5 * y * (1.0 + torch.erf(y / math.sqrt(2.0)))
        if act == "gelu_new":
            return 0.5 * y * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (y + 0.044715 * y * y * y)))
        raise ValueError(f"unknown activation {act!r}")

    def linear(self, x, w, bias=None, act=None, residual=None, out_f32=False):
        """`act(x w^T + bias) + residual`, `w` being `[out, in]`. An operand in the
        narrower dtype decides what the other is rounded to, except that a
        float32 matrix keeps the product in float32."""
        if w.dtype == torch.float32:
            xa = x.float()
        else:
            xa = x.to(w.dtype).float()
        y = xa @ w.float().t()
        if bias is not None:
            y = y + bias.float()
        y = self.activation(y, act)
        if residual is not None:
            y = y + residual.float()
        return y if out_f32 else y.to(self.dtype)

    # ---------------------------------------------------------------- attention

    def qkv_project(self, h, w, bias, num_heads, num_kv_write, head_size, scale, ctx, view, k_pages, v_pages, turn=None):
        """The projection to queries, keys and values (`w` holds the three stacked by rows), then
        `qkv_write`."""
        return self.qkv_write(self.linear(h, w, None), bias, num_heads, num_kv_write, head_size, scale, ctx, view,
                              k_pages, v_pages, turn)

    def qkv_write(self, qkv, bias, num_heads, num_kv_write, head_size, scale, ctx, view, k_pages, v_pages, turn=None):
        """Bias, then `turn` = (a, b), float32 `[positions, head_size]`: element d of every query and key head
        of a token at position p becomes a[p, d] x[d] + b[p, d] x[d ^ 1]; then the query scale, and the step's
        keys and values into their pages: page `table[run][position // page_size]`, place `position % page_size`."""
        t = qkv.shape[0]
        y = qkv.float()
        if bias is not None:
            y = y + bias.float()
        nq = num_heads * head_size
        if turn is not None:
            a, b = turn
            turned = nq + num_kv_write * head_size
            at = ctx.positions.long().clamp(0, a.shape[0] - 1)
            x = y[:, :turned].reshape(t, -1, head_size)
            beside = x.reshape(t, -1, head_size // 2, 2).flip(-1).reshape(t, -1, head_size)
            y = torch.cat([(a[at][:, None, :] * x + b[at][:, None, :] * beside).reshape(t, turned), y[:, turned:]], dim=1)
        q = (y[:, :nq] * scale).to(self.dtype)
        if num_kv_write:
            nk = num_kv_write * head_size
            k = y[:, nq:nq + nk].reshape(t, num_kv_write, head_size).to(k_pages.dtype)
            v = y[:, nq + nk:nq + 2 * nk].reshape(t, num_kv_write, head_size).to(v_pages.dtype)
            pos = ctx.positions.long()
            page = view.block_table[ctx.token_request.long(), pos // view.page_size].long()
            if int(page.min()) < 0:
                raise RuntimeError("a token of this step has no page")
            off = pos % view.page_size
            k_pages[page, :, off, :] = k
            v_pages[page, :, :, off] = v
        return q.contiguous()

    def attention(self, q, num_heads, num_kv_heads, head_size, ctx, view, k_pages, v_pages, window=None):
        """For every token: softmax over the keys of its own request at positions
        `<=` its own (`> position - window` with a window), times the values."""
        t = q.shape[0]
        out = torch.empty(t, num_heads * head_size, dtype=torch.float32, device=q.device)
        ps = view.page_size
        group = num_heads // num_kv_heads
        starts = ctx.run_start.tolist()
        for r in range(ctx.num_requests):
            s, e = starts[r], starts[r + 1]
            if e == s:
                continue
            total = int(ctx.cached_lens_host[r]) + (e - s)
            nb = -(-total // ps)
            pages = view.block_table[r, :nb].long().clamp(min=0)
            keys = k_pages[pages].float().permute(1, 0, 2, 3).reshape(num_kv_heads, nb * ps, head_size)[:, :total]
            vals = v_pages[pages].float().permute(1, 2, 0, 3).reshape(num_kv_heads, head_size, nb * ps)[:, :, :total]
            qr = q[s:e].float().reshape(e - s, num_heads, head_size).permute(1, 0, 2)
            keys = keys.repeat_interleave(group, dim=0)
            vals = vals.repeat_interleave(group, dim=0)
            scores = qr @ keys.transpose(1, 2)                       # [heads, run, total]
            pos = ctx.positions[s:e].long().unsqueeze(1)
            j = torch.arange(total, device=q.device).unsqueeze(0)
            allowed = j <= pos
            if window is not None:
                allowed &= j > pos - window
            scores = scores.masked_fill(~allowed.unsqueeze(0), float("-inf"))
            p = torch.softmax(scores, dim=-1)
            o = p @ vals.transpose(1, 2)                             # [heads, run, head_size]
            out[s:e] = o.permute(1, 0, 2).reshape(e - s, num_heads * head_size)
        return out.to(self.dtype)

    # ---------------------------------------------------------------- output end

    def gather_rows(self, x, rows):
        return x[rows.long()]

    def cast(self, x, dtype):
        return x.to(dtype)

    def ban_tokens(self, logits, tokens):
        rows = torch.nonzero(tokens >= 0).flatten()
        logits[rows, tokens[rows].long()] = float("-inf")
        return logits

    def ban_pairs(self, logits, rows, tokens):
        logits[rows.long(), tokens.long()] = float("-inf")
        return logits

    def argmax(self, logits):
        return logits.argmax(dim=-1).to(torch.int32)

    def sample(self, logits, temperature, top_k, top_p, seeds, counters, min_keep=None):
        """One token per row. Row i: logits / temperature[i]; the top_k[i] largest
        are kept (0 keeps all; ties go to the lower token id); of these, in
        descending order, the shortest prefix whose softmax mass reaches
        top_p[i] (>= 1 keeps all); neither keeps fewer than min_keep[i] tokens
        (1 if not given); the draw is by inverse CDF over the kept
        tokens in ascending order of token id with the uniform number
        `philox_uniform(seeds[i], counters[i])`, or 0.5 for a counter below zero.
        temperature 0 is argmax."""
        m, v = logits.shape
        out = torch.empty(m, dtype=torch.int32)
        for i in range(m):
            row = logits[i].float().cpu()
            temp = float(temperature[i])
            if temp == 0.0:
                out[i] = int(row.argmax())
                continue
            row = row / temp
            values, indices = torch.sort(row, descending=True, stable=True)
            least = max(1, int(min_keep[i])) if min_keep is not None else 1
            k = int(top_k[i])
            if k > 0:
                k = max(k, least)
            if 0 < k < v:
                values, indices = values[:k], indices[:k]
            p = float(top_p[i])
            if p < 1.0:
                cum = torch.cumsum(torch.softmax(values, -1, dtype=torch.float32), -1)
                keep = torch.cat([torch.ones(1, dtype=torch.bool), (cum < p)[:-1]])
                keep[:least] = True
                values, indices = values[keep], indices[keep]
            order = torch.argsort(indices)
            values, indices = values[order], indices[order]
            w = torch.exp(values - values.max()).double()
            cum = torch.cumsum(w, -1)
            u = 0.5 if int(counters[i]) < 0 else philox_uniform(int(seeds[i]), int(counters[i]))
            pick = int((cum <= u * float(cum[-1])).sum())
            out[i] = int(indices[min(pick, len(indices) - 1)])
        return out.to(logits.device)

    def synchronize(self):
        if self.device.type == "cuda":
            torch.cuda.synchronize(self.device)
