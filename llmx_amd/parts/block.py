"""The arrangements of a layer's parts.

"prenorm": x += mixer(norm(x)); x += ffn(norm(x)) with the residual x in float32: the arrangement of
/root/reference/src/model/arch/minimax_m3.hpp:247-287 (norm, mixer joined into the residual, norm, feed-forward joined).
"parallel": x += s1 * mixer(norm1(x)) + s2 * ffn(norm2(x)) with both norms of the same x, learned factors s1, s2 a
coordinate (or constants), and an optional per-layer token input after the sum; without a second norm both sublayers read
norm1's rows.
"outnorm": x += norm1(mixer(x)); x += norm2(ffn(x)): the sublayers read the residual itself and only their results are
normed.
"sandwich": x += norm1b(mixer(norm1(x))); x += norm2b(ffn(norm2(x))): a norm on both sides of each sublayer.
"""

from __future__ import annotations

import torch

from .. import ops
from .base import BuildContext, LayerCache, Mixer, Part, build_part, register
from .norm import RMSNorm
from .spec import BlockSpec, TensorSpec


class PreNormBlock:
    graph_safe = True   # see Part.graph_safe

    def __init__(self, spec: BlockSpec, ctx: BuildContext):
        self.mixer_norm = build_part("norm", spec.mixer_norm, ctx)
        self.mixer = build_part("mixer", spec.mixer, ctx)
        self.ffn_norm = build_part("norm", spec.ffn_norm, ctx)
        self.ffn = build_part("feed_forward", spec.ffn, ctx)

    def parts(self):
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.ffn]

    @staticmethod
    def normed(step, norm, part, x):
        """(h, h32) for `part`: the norm's description where the norm has one and the part carries it out in its own
        products for this step (a step of very few rows, where a norm kernel of its own costs more than its work);
        otherwise the norm runs here."""
        later = norm.deferred(x)
        if later is not None and part.takes_deferred_norm(step):
            return later, later
        T, E = x.shape
        h = step.buf("block.h", (T, E), step.act_dtype)
        h32 = step.buf("block.h32", (T, E), torch.float32) if part.wants_f32_input else None
        norm.forward(step, x, h, h32)
        return h, h32

    def forward(self, step, x: torch.Tensor, cache: LayerCache) -> None:
        h, h32 = self.normed(step, self.mixer_norm, self.mixer, x)
        self.mixer.forward(step, h, x, True, cache, h32)
        h, h32 = self.normed(step, self.ffn_norm, self.ffn, x)
        self.ffn.forward(step, h, x, True, h32)


class LayerScale(Part):
    """One learned factor a coordinate on a part's result.  params: width; optional (True: nothing applies it, and it is
    listed only when the file holds it).  Tensor: the prefix itself, (width,)."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.width = int(params["width"])
        self.optional = bool(params.get("optional", False))
        self.weight = None

    def tensor_specs(self, available):
        if self.optional and self.prefix not in available:
            return []
        return [TensorSpec(self.prefix, (self.width,), "norm")]

    def load(self, tensors):
        self.weight = tensors.get(self.prefix) if self.optional else tensors[self.prefix]


class ConstantScale(Part):
    """One number on a part's result, a constant of the model.  params: value.  No tensor."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.value = float(params["value"])
        self.weight = None


class ParallelBlock:
    """x += s1 * mixer(norm1(x)) + s2 * ffn(norm2(x)), both of the same x, then an optional token input that reads the
    new x.  The slots: mixer_norm, mixer, ffn_norm, ffn (a feed-forward without a norm of its own reads the mixer's normed
    rows: one norm for both sublayers); in `extra`: "mixer_scale" and "ffn_scale" (family "scale": a factor a coordinate, or
    a constant, on each result before the sum, optional) and "token_input" (family "token_input", optional).  Two RMS norms
    with one eps are one pass over x with two gains."""
    graph_safe = True

    def __init__(self, spec: BlockSpec, ctx: BuildContext):
        self.mixer_norm = build_part("norm", spec.mixer_norm, ctx)
        self.mixer = build_part("mixer", spec.mixer, ctx)
        self.ffn_norm = build_part("norm", spec.ffn_norm, ctx) if spec.ffn_norm is not None else None
        self.ffn = build_part("feed_forward", spec.ffn, ctx) if spec.ffn is not None else None
        built = {}
        for slot, family in (("mixer_scale", "scale"), ("ffn_scale", "scale"), ("token_input", "token_input")):
            if slot in spec.extra:
                got_family, part = spec.extra[slot]
                if got_family != family:
                    raise ValueError(f"parallel block: {slot} is a part of family {family!r}, not {got_family!r}")
                built[slot] = build_part(family, part, ctx)
        unknown = set(spec.extra) - {"mixer_scale", "ffn_scale", "token_input"}
        if unknown:
            raise ValueError(f"parallel block: no slot named {sorted(unknown)}")
        self.mixer_scale = built.get("mixer_scale")
        self.ffn_scale = built.get("ffn_scale")
        # without a feed-forward its norm and scale run nowhere; they may still be listed (as optional parts) for files that hold them
        self._idle = [p for p in (self.ffn_norm, self.ffn_scale) if p is not None] if self.ffn is None else []
        if self.ffn is None:
            self.ffn_norm = self.ffn_scale = None
        self.token_input = built.get("token_input")
        a, b = self.mixer_norm, self.ffn_norm
        self._shared_norm = self.ffn is not None and self.ffn_norm is None
        self._one_pass = isinstance(a, RMSNorm) and not self._shared_norm and (b is None or (isinstance(b, RMSNorm) and b.eps == a.eps and b.width == a.width))
        scales = [s for s in (self.mixer_scale, self.ffn_scale) if s is not None]
        self._constants = bool(scales) and all(isinstance(s, ConstantScale) for s in scales)
        if scales and not self._constants and any(isinstance(s, ConstantScale) for s in scales):
            raise ValueError("parallel block: both scales are constants or both are factors a coordinate")
        if self._constants and self.token_input is not None:
            raise ValueError("parallel block: a token input goes with factors a coordinate")
        if self.ffn is not None and self.ffn.wants_f32_input:
            self._one_pass = False

    def parts(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn, self.mixer_scale, self.ffn_scale, self.token_input)
                if p is not None] + self._idle

    def forward(self, step, x: torch.Tensor, cache: LayerCache) -> None:
        T, E = x.shape
        act = step.act_dtype
        h1 = step.buf("block.h", (T, E), act)
        h2 = step.buf("block.h2", (T, E), act) if self.ffn is not None and not self._shared_norm else None
        # a feed-forward whose router reads unrounded rows gets them from its norm
        h32 = step.buf("block.h32", (T, E), torch.float32) if self.ffn is not None and self.ffn.wants_f32_input else None
        if self._shared_norm:
            self.mixer_norm.forward(step, x, h1, h32)
            h2 = h1
        elif self._one_pass:
            ops.rmsnorm_pair(x, self.mixer_norm.weight, self.ffn_norm.weight if h2 is not None else None, self.mixer_norm.eps, h1, h2)
        else:
            self.mixer_norm.forward(step, x, h1)
            if h2 is not None:
                self.ffn_norm.forward(step, x, h2, h32)
        y1 = step.buf("block.y1", (T, E), torch.float32)
        self.mixer.forward(step, h1, y1, False, cache)
        y2 = None
        if self.ffn is not None:
            y2 = step.buf("block.y2", (T, E), torch.float32)
            self.ffn.forward(step, h2, y2, False, h32)
        if self._constants:
            ops.combine_rows(x, y1, self.mixer_scale.value if self.mixer_scale else 1.0, None, y2, self.ffn_scale.value if self.ffn_scale else 1.0,
                             accumulate=True)
            return
        copy = step.buf("block.x_act", (T, E), act) if self.token_input is not None else None
        ops.scale_add(x, y1, self.mixer_scale.weight if self.mixer_scale else None, y2, self.ffn_scale.weight if self.ffn_scale else None, copy)
        if self.token_input is not None:
            self.token_input.forward(step, x, copy)


class OutNormBlock:
    """x += mixer_norm(mixer(x)); x += ffn_norm(ffn(x)), the feed-forward (with its norm) optional.  The sublayers read x
    itself: in the serving path its rounded copy, which the join before them writes on its way (`add_into(..., copy)`), so
    that only a model's first layer needs a launch for it; the router of a routed feed-forward still gets the unrounded
    rows.  The norms are parts of the "norm" family that have `add_into` (x += norm(y))."""
    graph_safe = True

    def __init__(self, spec: BlockSpec, ctx: BuildContext):
        if (spec.ffn is None) != (spec.ffn_norm is None):
            raise ValueError("outnorm block: a feed-forward comes with its norm, and a norm with its feed-forward")
        self.mixer_norm = build_part("norm", spec.mixer_norm, ctx)
        self.mixer = build_part("mixer", spec.mixer, ctx)
        self.ffn_norm = build_part("norm", spec.ffn_norm, ctx) if spec.ffn_norm is not None else None
        self.ffn = build_part("feed_forward", spec.ffn, ctx) if spec.ffn is not None else None
        for n in (self.mixer_norm, self.ffn_norm):
            if n is not None and not hasattr(n, "add_into"):
                raise ValueError(f"outnorm block: the norm {n.kind!r} cannot join a result into the residual (no add_into)")
        if spec.extra:
            raise ValueError(f"outnorm block: no slot named {sorted(spec.extra)}")

    def parts(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def forward(self, step, x: torch.Tensor, cache: LayerCache) -> None:
        T, E = x.shape
        exact = step.act_dtype == torch.float32
        if exact:
            h = x                                   # the sublayers write elsewhere, so they may read the residual in place
        else:
            h = step.buf("block.x_act", (T, E), step.act_dtype)
            fresh = step.shared("outnorm.copy", dict)       # which run-order entry the copy was written for
            if fresh.get("for") != step.run_index:
                ops.cast_rows(x, h)
        y = step.buf("block.y", (T, E), torch.float32)
        self.mixer.forward(step, h, y, False, cache, x if self.mixer.wants_f32_input else None)
        last = self.ffn is None
        self.mixer_norm.add_into(step, x, y, None if exact else h)
        if not last:
            self.ffn.forward(step, h, y, False, x if self.ffn.wants_f32_input else None)
            self.ffn_norm.add_into(step, x, y, None if exact else h)
        if not exact:
            step.shared("outnorm.copy", dict)["for"] = step.run_index + 1


class SandwichBlock:
    """x += mixer_post(mixer(mixer_norm(x))); x += ffn_post(ffn(ffn_norm(x))): a norm before and a norm after each
    sublayer, the feed-forward (with both its norms) optional.  The slots: mixer_norm, mixer, ffn_norm, ffn; in `extra`:
    "mixer_post" and "ffn_post" (family "norm", parts that have `add_into`: x += norm(y))."""
    graph_safe = True

    def __init__(self, spec: BlockSpec, ctx: BuildContext):
        if (spec.ffn is None) != (spec.ffn_norm is None) or (spec.ffn is None) != ("ffn_post" not in spec.extra):
            raise ValueError("sandwich block: a feed-forward comes with both its norms, and the norms with their feed-forward")
        unknown = set(spec.extra) - {"mixer_post", "ffn_post"}
        if unknown or "mixer_post" not in spec.extra:
            raise ValueError(f"sandwich block: the extra slots are mixer_post and ffn_post, not {sorted(spec.extra)}")
        for slot, (family, _) in spec.extra.items():
            if family != "norm":
                raise ValueError(f"sandwich block: {slot} is a part of family 'norm', not {family!r}")
        self.mixer_norm = build_part("norm", spec.mixer_norm, ctx)
        self.mixer = build_part("mixer", spec.mixer, ctx)
        self.mixer_post = build_part("norm", spec.extra["mixer_post"][1], ctx)
        self.ffn_norm = build_part("norm", spec.ffn_norm, ctx) if spec.ffn_norm is not None else None
        self.ffn = build_part("feed_forward", spec.ffn, ctx) if spec.ffn is not None else None
        self.ffn_post = build_part("norm", spec.extra["ffn_post"][1], ctx) if spec.ffn is not None else None
        for n in (self.mixer_post, self.ffn_post):
            if n is not None and not hasattr(n, "add_into"):
                raise ValueError(f"sandwich block: the norm {n.kind!r} cannot join a result into the residual (no add_into)")
        # RMS norms on both sides of the join before the feed-forward: one launch joins the mixer's result and norms the new rows
        self._join_then_norm = (self.ffn is not None and isinstance(self.mixer_post, RMSNorm) and isinstance(self.ffn_norm, RMSNorm)
                                and self.mixer_post.width == self.ffn_norm.width)

    def parts(self):
        return [p for p in (self.mixer_norm, self.mixer, self.mixer_post, self.ffn_norm, self.ffn, self.ffn_post) if p is not None]

    def forward(self, step, x: torch.Tensor, cache: LayerCache) -> None:
        T, E = x.shape
        y = step.buf("block.y", (T, E), torch.float32)
        h, h32 = PreNormBlock.normed(step, self.mixer_norm, self.mixer, x)
        self.mixer.forward(step, h, y, False, cache, h32)
        if self.ffn is None:
            self.mixer_post.add_into(step, x, y)
            return
        if self._join_then_norm and not (self.ffn_norm.deferred(x) is not None and self.ffn.takes_deferred_norm(step)):
            h = step.buf("block.h", (T, E), step.act_dtype)
            h32 = step.buf("block.h32", (T, E), torch.float32) if self.ffn.wants_f32_input else None
            self.mixer_post.add_into_then_norm(step, x, y, self.ffn_norm, h, h32)
        else:
            self.mixer_post.add_into(step, x, y)
            h, h32 = PreNormBlock.normed(step, self.ffn_norm, self.ffn, x)
        self.ffn.forward(step, h, y, False, h32)
        self.ffn_post.add_into(step, x, y)


register("block", "prenorm", PreNormBlock)
register("block", "sandwich", SandwichBlock)
register("block", "outnorm", OutNormBlock)
register("block", "parallel", ParallelBlock)
register("scale", "layer_scale", LayerScale)
register("scale", "constant", ConstantScale)
