"""How a layer's parts are arranged."""
from __future__ import annotations

from typing import Dict

from .base import LayerCache, ParamSpec, Part, ResidualStream, StepContext, TensorSource


class PreNormBlock(Part):
    """h += mixer(norm1(h)); h += ffn(norm2(h))
    (reference: src/SharpInference.Engine/ForwardPass.cs:1557-1561, 1690-1714).

    The additions are folded into the norm that follows them (see ResidualStream), so a block
    leaves its feed-forward output pending for the next block's first norm.  A feed-forward that
    has ``forward_from_stream(stream, norm, ctx)`` is handed the stream and the second norm instead
    of normalised rows (it must leave the stream as the norm would have).  Names of the four
    parts in the weight file are arguments."""

    def __init__(self, norm1: Part, mixer: Part, norm2: Part, ffn: Part, names=None):
        self.norm1, self.mixer, self.norm2, self.ffn = norm1, mixer, norm2, ffn
        self.names = dict(names or {"norm1": "input_layernorm.", "mixer": "self_attn.",
                                    "norm2": "post_attention_layernorm.", "ffn": "feed_forward."})

    def _children(self):
        return ((self.names["norm1"], self.norm1), (self.names["mixer"], self.mixer),
                (self.names["norm2"], self.norm2), (self.names["ffn"], self.ffn))

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        out: Dict[str, ParamSpec] = {}
        for name, part in self._children():
            out.update(part.param_specs(prefix + name))
        return out

    def load(self, prefix: str, source: TensorSource) -> None:
        for name, part in self._children():
            part.load(prefix + name, source)

    def step_planners(self):
        out = []
        for _, part in self._children():
            out.extend(getattr(part, "step_planners", tuple)())
        return out

    def cache_spec(self):
        spec = getattr(self.mixer, "cache_spec", None)
        return spec() if spec else None

    def decode_graph_safe(self) -> bool:
        """Can a decode step through this block be captured into a graph?  Paged attention can; a
        mixer with state of its own says so itself (``graph_safe``)."""
        from ..cache.spec import StateSpec

        return not isinstance(self.cache_spec(), StateSpec) or bool(getattr(self.mixer, "graph_safe", False))

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: LayerCache) -> None:
        n = self.norm1.forward(stream, ctx.act_dtype)
        stream.pending = self.mixer.forward(n, ctx, cache)
        from_stream = getattr(self.ffn, "forward_from_stream", None)
        if from_stream is not None:    # a feed-forward that may fuse the norm with work of its own
            stream.pending = from_stream(stream, self.norm2, ctx)
        else:
            n = self.norm2.forward(stream, ctx.act_dtype)
            stream.pending = self.ffn.forward(n, ctx)
