"""Input and output ends of the decoder."""
from typing import Dict, List, Optional

import torch

from .base import (EMBEDDINGS, HEADS, NORMS, POSITIONS, Part, Stream, register_embedding, register_head)
from .spec import ParamDecl, PartSpec


@register_embedding("token_table")
class TokenEmbedding(Part):
    """Token rows `[vocab, embed_width]`, a projection to the hidden width when the
    two differ (no bias), then the position encoding's input step (reference:
    opt/model.py:162-166; the projection is read by no reference code path,
    opt/config.py:34)."""

    recordable = True

    def __init__(self, vocab: int, embed_width: int, width: int, position: PartSpec,
                 table_name: str, projection_name: Optional[str], position_name: str):
        self.vocab, self.embed_width, self.width = vocab, embed_width, width
        self.table_name, self.projection_name, self.position_name = table_name, projection_name, position_name
        self.position = POSITIONS.build(position)
        self.projects = embed_width != width

    def param_decls(self, prefix: str = "") -> List[ParamDecl]:
        d = [ParamDecl(self.table_name, (self.vocab, self.embed_width), "table")]
        if self.projects:
            d.append(ParamDecl(self.projection_name, (self.width, self.embed_width)))
        return d + self.position.param_decls(self.position_name)

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.table = tensors[self.table_name]
        self.projection = ops.prepare_weight(tensors[self.projection_name]) if self.projects else None
        self.position.load(tensors, self.position_name, ops, dtype)

    def forward(self, ctx, want_compute: bool) -> Stream:
        x = self.ops.embed(ctx.token_ids, self.table, self.dtype, ctx.kept_tokens)
        if self.projects:
            x = self.ops.linear(x, self.projection, None)
        xf, xc = self.position.at_input(x, ctx.positions, want_compute)
        return Stream(xf, xc)


@register_head("vocab_projection")
class VocabHead(Part):
    """Rows that need logits are picked first, then an optional norm, an optional
    projection to the embedding width (no bias) and the `[vocab, width]` matrix,
    which is the token table when the checkpoint holds no head of its own
    (reference: layers/transformer.py:196-208, row selection :298-333; tie
    opt/model.py:204-205). Logits are float32."""

    recordable = True

    def __init__(self, vocab: int, embed_width: int, width: int, norm: Optional[PartSpec],
                 weight_name: str, tied_to: Optional[str], projection_name: Optional[str], norm_name: str):
        self.vocab, self.embed_width, self.width = vocab, embed_width, width
        self.norm = NORMS.build(norm) if norm is not None else None
        self.weight_name, self.tied_to = weight_name, tied_to
        self.projection_name, self.norm_name = projection_name, norm_name
        self.projects = embed_width != width

    def param_decls(self, prefix: str = "") -> List[ParamDecl]:
        d = [ParamDecl(self.weight_name, (self.vocab, self.embed_width), "matrix", tied_to=self.tied_to)]
        if self.projects:
            d.append(ParamDecl(self.projection_name, (self.embed_width, self.width)))
        if self.norm is not None:
            d += self.norm.param_decls(self.norm_name)
        return d

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.weight = ops.prepare_weight(tensors[self.weight_name])
        self.projection = ops.prepare_weight(tensors[self.projection_name]) if self.projects else None
        if self.norm is not None:
            self.norm.load(tensors, self.norm_name, ops, dtype)

    def forward(self, stream: Stream, ctx):
        if ctx.logits_rows.numel() == 0:      # a step of prompt portions alone: nothing is asked of the head
            return torch.empty(0, self.vocab, dtype=torch.float32, device=stream.x.device)
        rows = self.ops.gather_rows(stream.x, ctx.logits_rows)
        if self.norm is not None:
            _, h = self.norm.forward(rows, False, True)
        else:
            h = self.ops.cast(rows, self.dtype)
        if self.projects:
            h = self.ops.linear(h, self.projection, None)
        return self.ops.linear(h, self.weight, None, out_f32=True)
