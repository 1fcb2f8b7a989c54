"""Pre-norm residual arrangement: h += mixer(norm(h)); h += feed_forward(norm(h))
(worker/src/inference/qwen2/model.py:279-290). Each sub-layer's output is left pending
on the stream; the next norm adds it while it reads the stream."""

from __future__ import annotations

from .base import Block, ResidualStream, StepContext, register_part


class PreNormResidual(Block):
    CHILDREN = {"mixer_norm": "norm", "mixer": "mixer", "feed_forward_norm": "norm", "feed_forward": "feed_forward"}

    def forward(self, ops, stream: ResidualStream, ctx: StepContext, cache, writes_cache: bool) -> None:
        normed = self.mixer_norm.of_stream(ops, stream, ctx.act_dtype)
        stream.pending = self.mixer.forward(ops, normed, ctx, cache["mixer"], writes_cache)
        normed = self.feed_forward_norm.of_stream(ops, stream, ctx.act_dtype)
        stream.pending = self.feed_forward.forward(ops, normed, ctx)


register_part("block", "prenorm_residual", PreNormResidual)
