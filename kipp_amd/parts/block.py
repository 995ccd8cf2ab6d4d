"""Block arrangements: how the parts of one layer are put together.

Interface of a block:

    roles: tuple of (role, category) the arrangement needs in LayerSpec.parts
    forward(x, pending, batch, cache, state) -> (x, pending)
        x        float32 [tokens, hidden], the residual stream (updated in place)
        pending  a delta not yet added to x (or None); the block adds it inside
                 its first norm and hands its own last delta on the same way,
                 so that residual add and norm are one kernel.  A delta may
                 be a product that the runtime has not launched yet
                 (`Runtime.linear(..., defer=True)`), and a norm may leave its
                 scale to the product that follows (`ScaledRows`): the block
                 settles either for a part that does not declare it takes it
                 (`fuses_products` of a norm, `takes_scaled_rows` of a mixer
                 or feed-forward).
"""
from __future__ import annotations

from .base import build_part, register


@register("block", "pre_norm")
class PreNormBlock:
    """x += mixer(mixer_norm(x)); x += ffn(ffn_norm(x))
    (/root/reference/docs/ARCHITECTURE.md:77-92)."""

    roles = (("mixer_norm", "norm"), ("mixer", "mixer"), ("ffn_norm", "norm"), ("ffn", "feed_forward"))

    def __init__(self, layer_spec, runtime):
        self.rt = runtime
        self.parts = {role: build_part(cat, layer_spec.part(role), runtime) for role, cat in self.roles}
        self.mixer = self.parts["mixer"]
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self.parts.values())

    def forward(self, x, pending, batch, cache, state):
        act = self.rt.act_dtype
        norm1, norm2 = self.parts["mixer_norm"], self.parts["ffn_norm"]
        rt, ffn = self.rt, self.parts["ffn"]
        if pending is not None and not getattr(norm1, "fuses_products", False):
            pending = rt.settle(pending)
        h = norm1.forward(x, act) if pending is None else norm1.add_forward(x, pending, act)
        if not getattr(self.mixer, "takes_scaled_rows", False):
            h = rt.rows_of(h)
        delta = self.mixer.forward(h, batch, cache, state)
        if not getattr(norm2, "fuses_products", False):
            delta = rt.settle(delta)
        h = norm2.add_forward(x, delta, act)
        if not getattr(ffn, "takes_scaled_rows", False):
            h = rt.rows_of(h)
        return x, ffn.forward(h, batch)


@register("block", "post_norm")
class PostNormBlock:
    """The norm after the sum: x = mixer_norm(a x + mixer(x)); x = ffn_norm(a x + ffn(x)), a = the layer's
    `residual_scale`.  The sublayers read x itself, so the float32 residual stream is what the norms write; under
    bfloat16 the norm's kernel writes the same rows once more in bfloat16 for the products that follow (kept in the
    step's cache for the next block of this kind, which would otherwise cast x again).  Nothing is left pending."""

    roles = (("mixer_norm", "norm"), ("mixer", "mixer"), ("ffn_norm", "norm"), ("ffn", "feed_forward"))

    def __init__(self, layer_spec, runtime):
        self.rt = runtime
        self.alpha = float(layer_spec.residual_scale)
        self.parts = {role: build_part(cat, layer_spec.part(role), runtime) for role, cat in self.roles}
        self.mixer = self.parts["mixer"]
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self.parts.values())

    def _rows(self, x, batch):
        """x in the type the products read."""
        import torch
        if self.rt.act_dtype == torch.float32:
            return x
        kept = batch.step_cache.get("residual_rows")
        if kept is not None and kept[0] is x:
            return kept[1]
        return self.rt.ops.cast(x, self.rt.empty(x.shape, self.rt.act_dtype))

    def forward(self, x, pending, batch, cache, state):
        rt = self.rt
        if pending is not None:
            rt.ops.residual_add(x, rt.settle(pending))
        h = self._rows(x, batch)
        h = self.parts["mixer_norm"].post_forward(x, self.mixer.forward(h, batch, cache, state), self.alpha, rt.act_dtype)
        if "ffn" in self.parts:
            h = self.parts["ffn_norm"].post_forward(x, self.parts["ffn"].forward(h, batch), self.alpha, rt.act_dtype)
        batch.step_cache["residual_rows"] = (x, h)
        return x, None


@register("block", "post_norm_mixer")
class PostNormMixerBlock(PostNormBlock):
    """The first half of the post-norm arrangement alone: a layer without a feed-forward."""

    roles = (("mixer_norm", "norm"), ("mixer", "mixer"))


@register("block", "sandwich_norm")
class SandwichNormBlock:
    """A norm in front of a sublayer and another on its result: x += a mixer_post_norm(mixer(mixer_norm(x)));
    x += a ffn_post_norm(ffn(ffn_norm(x))), a = the layer's `residual_scale`.  A sublayer's result is handed on as a
    `NormedDelta`: the norm in front of the next sublayer (this block's or the next one's) norms it, adds it and norms
    the new residual in one kernel."""

    roles = (("mixer_norm", "norm"), ("mixer", "mixer"), ("mixer_post_norm", "norm"),
             ("ffn_norm", "norm"), ("ffn", "feed_forward"), ("ffn_post_norm", "norm"))

    def __init__(self, layer_spec, runtime):
        self.rt = runtime
        self.alpha = float(layer_spec.residual_scale)
        self.parts = {role: build_part(cat, layer_spec.part(role), runtime) for role, cat in self.roles}
        self.mixer = self.parts["mixer"]
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self.parts.values())

    def _sublayer(self, x, pending, norm, post_norm, run):
        from .norm import NormedDelta
        rt, act = self.rt, self.rt.act_dtype
        if pending is not None and not getattr(norm, "fuses_products", False):
            pending = rt.settle(pending)
        h = rt.rows_of(norm.forward(x, act) if pending is None else norm.add_forward(x, pending, act))
        return NormedDelta(rt, rt.settle(run(h)), post_norm, self.alpha)

    def forward(self, x, pending, batch, cache, state):
        p = self.parts
        pending = self._sublayer(x, pending, p["mixer_norm"], p["mixer_post_norm"], lambda h: self.mixer.forward(h, batch, cache, state))
        if "ffn" in p:
            pending = self._sublayer(x, pending, p["ffn_norm"], p["ffn_post_norm"], lambda h: p["ffn"].forward(h, batch))
        return x, pending


@register("block", "sandwich_norm_mixer")
class SandwichNormMixerBlock(SandwichNormBlock):
    """The first half of the sandwich arrangement alone: a layer without a feed-forward."""

    roles = (("mixer_norm", "norm"), ("mixer", "mixer"), ("mixer_post_norm", "norm"))


@register("block", "parallel")
class ParallelBlock:
    """One norm whose output both sublayers read: h = mixer_norm(x); x += mixer(h) + ffn(h).  The mixer's result is added
    at once (a weighted sum of deltas term by term, where it lies); the feed-forward's is handed on and added inside the next
    block's norm."""

    roles = (("mixer_norm", "norm"), ("mixer", "mixer"), ("ffn", "feed_forward"))

    def __init__(self, layer_spec, runtime):
        self.rt = runtime
        self.parts = {role: build_part(cat, layer_spec.part(role), runtime) for role, cat in self.roles}
        self.mixer = self.parts["mixer"]
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in self.parts.values())

    def forward(self, x, pending, batch, cache, state):
        rt, norm = self.rt, self.parts["mixer_norm"]
        if pending is not None and not getattr(norm, "fuses_products", False):
            pending = rt.settle(pending)
        h = norm.forward(x, rt.act_dtype) if pending is None else norm.add_forward(x, pending, rt.act_dtype)
        h = rt.rows_of(h)       # two readers: the rows are finished once
        delta = self.mixer.forward(h, batch, cache, state)
        if hasattr(delta, "add_to"):
            delta.add_to(x)
        else:
            rt.ops.residual_add(x, rt.settle(delta))
        if "ffn" not in self.parts:
            return x, None
        return x, self.parts["ffn"].forward(h, batch)


@register("block", "parallel_mixer")
class ParallelMixerBlock(ParallelBlock):
    """The parallel arrangement without a feed-forward."""

    roles = (("mixer_norm", "norm"), ("mixer", "mixer"))
