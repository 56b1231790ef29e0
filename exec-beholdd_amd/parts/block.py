"""The arrangement of parts in a layer.

Pre-norm residual block: h = h + Mixer(Norm(h)); h = h + FeedForward(Norm(h))
(crates/beholdd-model/src/qwen3moe/forward.rs:1022-1414).  The residual `hidden` is float32
and is updated in place; the mixer and the feed-forward add into it.
"""

from __future__ import annotations

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, graph_rows_allowed


class PreNormBlock:
    def __init__(self, mixer_norm, mixer, feed_forward_norm, feed_forward):
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.feed_forward_norm, self.feed_forward = feed_forward_norm, feed_forward

    def parts(self):
        return [self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward]

    @property
    def graph_safe(self):
        return all(getattr(part, "graph_safe", False) for part in self.parts())

    @property
    def graph_safe_rows(self):
        return graph_rows_allowed(self.parts())

    def tensor_specs(self):
        return [spec for part in self.parts() for spec in part.tensor_specs()]

    def load(self, get):
        for part in self.parts():
            part.load(get)

    def prepare(self, kernels):
        for part in self.parts():
            if hasattr(part, "prepare"):
                part.prepare(kernels)

    def working_bytes(self, step) -> int:
        """Everything the four parts allocate, as if nothing were freed before the layer ends."""
        total = 0
        for norm, consumer in ((self.mixer_norm, self.mixer), (self.feed_forward_norm, self.feed_forward)):
            if hasattr(norm, "working_bytes"):
                total += norm.working_bytes(step)
            if hasattr(consumer, "working_bytes"):
                total += consumer.working_bytes(step)
        return total

    def unaccounted_parts(self) -> list:
        return [type(part).__name__ for part in self.parts() if not hasattr(part, "working_bytes")]

    def cache_need(self):
        return self.mixer.cache_need()

    @staticmethod
    def _joined(producer, norm, consumer):
        """The request to hand `producer` so that its last product prepares `norm` for `consumer`, or None."""
        if (getattr(producer, "prepares_next_norm", False) and getattr(consumer, "takes_prepared_input", False)
                and hasattr(norm, "request")):
            reader = PreNormBlock._reader(norm, consumer)
            return norm.request(reader) if reader is not None else norm.request()
        return None

    @staticmethod
    def _reader(norm, consumer):
        """The product of `consumer` that alone reads what `norm` writes, if both parts say so."""
        return getattr(consumer, "input_reader", None) if getattr(norm, "serves_reader", False) else None

    @staticmethod
    def _normed(ctx, norm, consumer, hidden):
        reader = PreNormBlock._reader(norm, consumer)
        return norm.forward(ctx, hidden, reader=reader) if reader is not None else norm.forward(ctx, hidden)

    def entry_request(self, producer):
        """What the part that runs before this block (`producer`) may prepare of this block's first norm."""
        return self._joined(producer, self.mixer_norm, self.mixer)

    def forward(self, ctx, hidden, cache, prepared=None, next_block=None):
        """One layer.  `prepared`: the mixer's input if the block before has prepared it already;
        `next_block`: the block that runs after this one, whose first norm this block's feed-forward
        may prepare.  Returns that prepared input, or None."""
        x = prepared if prepared is not None else self._normed(ctx, self.mixer_norm, self.mixer, hidden)
        request = self._joined(self.mixer, self.feed_forward_norm, self.feed_forward)
        if request is not None:
            x = self.mixer.forward(ctx, x, hidden, cache, then_norm=request)
        else:
            self.mixer.forward(ctx, x, hidden, cache)
            x = None
        if x is None:
            x = self._normed(ctx, self.feed_forward_norm, self.feed_forward, hidden)
        request = next_block.entry_request(self.feed_forward) if hasattr(next_block, "entry_request") else None
        if request is not None:
            return self.feed_forward.forward(ctx, x, hidden, then_norm=request)
        self.feed_forward.forward(ctx, x, hidden)
        return None


@BLOCKS.register("pre_norm")
def _build_pre_norm(config, layer_index, prefix, kinds, shared):
    norm = NORMS.get(kinds.norm)
    return PreNormBlock(
        norm(config, config.hidden, prefix + "input_layernorm.weight", shared),
        MIXERS.get(kinds.mixer)(config, layer_index, prefix, shared),
        norm(config, config.hidden, prefix + "post_attention_layernorm.weight", shared),
        FEED_FORWARDS.get(kinds.feed_forward)(config, layer_index, prefix, shared))
