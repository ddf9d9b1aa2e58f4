"""The pre-norm arrangement of a layer: norm, mixer, residual, norm,
feed-forward, residual (reference: model/mod.rs:84-136).

The residual stream is 32-bit.  A block receives the stream and the previous
block's output that has not been added yet, adds it inside its first norm, and
returns its own feed-forward output unadded, so that every residual sum is
fused with the norm that follows it.  With few rows the fusion goes the other
way: a part that can adds its output into the stream as the last stage of its
product kernel and the norm becomes the first stage of the next product.
"""

from __future__ import annotations

import torch

from ..errors import ConfigError
from .norm import PendingNorm
from .registry import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, lookup, prefixed, register_block, scoped)


class PreNormBlock:
    NAMES = {"norm1": "input_layernorm", "mixer": "self_attn", "norm2": "post_attention_layernorm",
             "feed_forward": "mlp"}

    @classmethod
    def names_of(cls, layer) -> dict:
        """The name parts of the members' tensors: this architecture's, or the layer spec's own."""
        given = getattr(layer, "names", None) or {}
        unknown = sorted(set(given) - set(cls.NAMES))
        if unknown:
            raise ConfigError(f"a layer names members that this arrangement does not have: {unknown}")
        return {**cls.NAMES, **given}

    @classmethod
    def declare(cls, layer, hidden: int) -> list:
        norm = lookup(NORMS, layer.norm.kind, "norm")
        mixer = lookup(MIXERS, layer.mixer.kind, "mixer")
        ffn = lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward")
        n = cls.names_of(layer)
        return (prefixed(norm.declare(layer.norm, hidden), n["norm1"])
                + prefixed(mixer.declare(layer.mixer, hidden), n["mixer"])
                + prefixed(norm.declare(layer.norm, hidden), n["norm2"])
                + prefixed(ffn.declare(layer.feed_forward, hidden), n["feed_forward"]))

    def __init__(self, layer, hidden: int, params: dict, dtype, device, shared: dict):
        n = self.names = self.names_of(layer)
        norm = lookup(NORMS, layer.norm.kind, "norm")
        self.dtype = dtype
        self.norm1 = norm(layer.norm, hidden, scoped(params, n["norm1"]), dtype, device)
        self.mixer = lookup(MIXERS, layer.mixer.kind, "mixer")(
            layer.mixer, hidden, scoped(params, n["mixer"]), dtype, device, shared)
        self.norm2 = norm(layer.norm, hidden, scoped(params, n["norm2"]), dtype, device)
        self.feed_forward = lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward")(
            layer.feed_forward, hidden, scoped(params, n["feed_forward"]), dtype, device, shared)

    @property
    def graph_safe(self) -> bool:
        """Whether a step through this block may be captured as a HIP graph: a part that
        reads device values on the host, or allocates by data, sets ``graph_safe = False``."""
        return getattr(self.mixer, "graph_safe", True) and getattr(self.feed_forward, "graph_safe", True)

    @property
    def first_norm(self):
        """The norm this block applies to the stream first: the block before may leave its work behind."""
        return self.norm1

    @staticmethod
    def _room(norm, resid):
        """Room for ``norm`` handed forward over the rows of ``resid``, where the norm has such a thing."""
        make = getattr(norm, "handoff", None)
        return make(resid.shape[0], resid.device) if make is not None else None

    def forward(self, resid, delta, ctx):
        """``delta``: what the block before has not added to the stream yet, or None.  Returns this
        block's own unadded output, or None when the feed-forward added it itself."""
        if ctx.trace is not None:
            return self._forward_recorded(resid, delta, ctx)
        mixer_fuses = getattr(self.mixer, "fuses", False)
        ffn_fuses = getattr(self.feed_forward, "fuses", False)
        half = self.dtype == torch.bfloat16
        if delta is None and mixer_fuses:
            # every sum is in the stream already (and the product that added the last may have left this norm's work)
            x = PendingNorm(self.norm1, resid, self.dtype, handed=getattr(ctx, "handed", None))
        else:
            x = self.norm1.apply(resid, delta, self.dtype)
        ctx.residual = resid if mixer_fuses else None
        # a mixer that adds into the stream may leave the second norm's work behind ...
        ctx.hand = self._room(self.norm2, resid) if half and mixer_fuses and ffn_fuses else None
        mixed = self.mixer.forward(x, ctx)
        left, ctx.residual, ctx.hand = ctx.hand, None, None
        if mixed is None and ffn_fuses:
            x = PendingNorm(self.norm2, resid, self.dtype, handed=left)
        else:
            x = self.norm2.apply(resid, mixed, self.dtype)
        if ffn_fuses:
            # ... and a feed-forward that does, the next layer's first norm's
            after = getattr(ctx, "norm_after", None)
            if half and after is not None and getattr(self.feed_forward, "hands_forward", False):
                room = self._room(after, resid)
                out = self.feed_forward.forward(x, residual=resid, hand=room)
                ctx.handed_out = room if out is None and room is not None and room.filled else None
                return out
            return self.feed_forward.forward(x, residual=resid)
        return self.feed_forward.forward(x)

    def _forward_recorded(self, resid, delta, ctx):
        """The same layer with every module's output recorded under its name: nothing is fused, so
        every norm runs as a kernel and no part adds into the stream itself.  A part whose class sets
        ``records = True`` takes the recorder (``ctx.trace`` for a mixer, ``trace=`` for a feed-forward)
        and records what happens inside it."""
        n, trace = self.names, ctx.trace
        x = self.norm1.apply(resid, delta, self.dtype)
        trace.record(f"{n['norm1']}.out", x)
        ctx.trace = trace.child(n["mixer"]) if getattr(self.mixer, "records", False) else None
        mixed = self.mixer.forward(x, ctx)
        ctx.trace = trace
        trace.record(f"{n['mixer']}.out", mixed)
        x = self.norm2.apply(resid, mixed, self.dtype)
        trace.record(f"{n['norm2']}.out", x)
        if getattr(self.feed_forward, "records", False):
            out = self.feed_forward.forward(x, trace=trace.child(n["feed_forward"]))
        else:
            out = self.feed_forward.forward(x)
        trace.record(f"{n['feed_forward']}.out", out)
        return out


register_block("pre_norm", PreNormBlock)
