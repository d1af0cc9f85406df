"""Pre-norm residual block: ``x += mixer(norm1(x)); x += ffn(norm2(x))``
(/root/reference/src/torchlet/v10_triton_paged_gqa/layer/transformer_block.py:37-40).

The additions are deferred: a branch's output is left ``pending`` on the stream and the
next norm (the block's second one, the next block's first one, or the model's final one)
adds it in 32-bit while it normalises.

The other arrangement built here puts the norm after the sum: ``x <- norm1(alpha * x + mixer(x))``, then
``x <- norm2(alpha * x + ffn(x))``; the sublayers read the normed stream itself, and the sum and the norm are one
kernel that leaves the stream in 32-bit and, for the products that read it next, in the activation dtype.
"""
from __future__ import annotations

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Block, Stream, join_name, under


@BLOCKS.register("prenorm_residual")
class PreNormBlock(Block):
    graph_safe = True       # the arrangement itself; its four parts answer for themselves

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.mixer_norm = NORMS.build(spec.mixer_norm, dtype, device)
        self.mixer = MIXERS.build(spec.mixer, dtype, device)
        self.ffn_norm = NORMS.build(spec.ffn_norm, dtype, device)
        self.ffn = FEED_FORWARDS.build(spec.ffn, dtype, device)
        self._children = {
            spec.mixer_norm_name: self.mixer_norm,
            spec.mixer_name: self.mixer,
            spec.ffn_norm_name: self.ffn_norm,
            spec.ffn_name: self.ffn,
        }

    def parts(self):
        yield self
        for part in self._children.values():
            yield from part.parts()

    def weight_specs(self):
        return {join_name(name, k): v for name, part in self._children.items() for k, v in part.weight_specs().items()}

    def load_weights(self, tensors):
        for name, part in self._children.items():
            part.load_weights(under(tensors, name))

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        # a part that says it takes a norm that has not run yet (``takes_lazy_norm``) may get one, see LazyNorm
        h = (self.mixer_norm.lazy(stream) if getattr(self.mixer, "takes_lazy_norm", False) else None) or self.mixer_norm.forward(stream)
        stream.pending = self.mixer.forward(h, ctx, cache)
        h = (self.ffn_norm.lazy(stream) if getattr(self.ffn, "takes_lazy_norm", False) else None) or self.ffn_norm.forward(stream)
        stream.pending = self.ffn.forward(h, ctx)
        return stream


@BLOCKS.register("postnorm_residual")
class PostNormBlock(Block):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.alpha = float(spec.alpha)
        self.mixer = MIXERS.build(spec.mixer, dtype, device)
        self.mixer_norm = NORMS.build(spec.mixer_norm, dtype, device)
        self.ffn = FEED_FORWARDS.build(spec.ffn, dtype, device) if spec.ffn is not None else None
        self.ffn_norm = NORMS.build(spec.ffn_norm, dtype, device) if spec.ffn is not None else None
        self._children = {spec.mixer_norm_name: self.mixer_norm, spec.mixer_name: self.mixer}
        if self.ffn is not None:
            self._children.update({spec.ffn_norm_name: self.ffn_norm, spec.ffn_name: self.ffn})

    parts = PreNormBlock.parts
    weight_specs = PreNormBlock.weight_specs
    load_weights = PreNormBlock.load_weights

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        h = stream.normed
        if h is None:                # the first block reads the embedding rows
            h = stream.residual if self.dtype == stream.residual.dtype else stream.residual.to(self.dtype)
        stream.pending = self.mixer.forward(h, ctx, cache)
        h = self.mixer_norm.renorm(stream, self.alpha)
        if self.ffn is not None:
            stream.pending = self.ffn.forward(h, ctx)
            h = self.ffn_norm.renorm(stream, self.alpha)
        stream.normed = h
        return stream
