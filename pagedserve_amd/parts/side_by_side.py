"""Two mixers that read the same input, their results normed and averaged."""

import torch

from ..ops import kernels
from ..weights.loader import VECTOR, ParamSpec
from .base import Mixer
from .registry import MIXERS, build_part, register_mixer


@register_mixer("side_by_side")
class SideBySide(Mixer):
    """``out = (rms_norm(left(x)) * w_left + rms_norm(right(x)) * w_right) / 2``: both mixers read
    the same rows, each result is RMS-normed over the model width with a plain weight of its own.

    ``left`` and ``right`` are ``PartSpec`` records of any mixer kinds.  Each child keeps a cache
    entry of its own kind (``cache_spec`` is the pair; the view of a call carries one child view
    per mixer), and its parameters live under ``left.`` / ``right.``.  The children add their
    results into two float scratch rows that are clear between calls; one launch norms both, adds
    their mean into ``residual`` and clears them again."""

    accepts_pending_norm = False

    def __init__(self, width: int, dtype, left, right, norm_eps: float):
        self.width = width
        self.dtype = dtype
        self.norm_eps = float(norm_eps)
        self.left = build_part(MIXERS, "mixer (left)", left, width=width, dtype=dtype)
        self.right = build_part(MIXERS, "mixer (right)", right, width=width, dtype=dtype)
        self.children = (("left", self.left), ("right", self.right))

    @property
    def graph_safe(self):
        return all(getattr(child, "graph_safe", False) for _, child in self.children)

    @property
    def query_tile(self):
        sizes = set()
        for _, child in self.children:
            asked = getattr(child, "query_tile", None)
            if asked:
                sizes.update(asked if isinstance(asked, (tuple, list)) else (asked,))
        return tuple(sorted(sizes))

    def set_position(self, position):
        self.position = position
        for _, child in self.children:
            child.set_position(position)

    def parameters(self):
        params = {}
        for prefix, child in self.children:
            for name, spec in child.parameters().items():
                params[f"{prefix}.{name}"] = spec
            params[f"{prefix}_scale"] = ParamSpec((self.width,), VECTOR)
        return params

    def bind(self, tensors):
        for prefix, child in self.children:
            child.bind({name: tensors[f"{prefix}.{name}"] for name in child.parameters()})
        self.left_scale = tensors["left_scale"]
        self.right_scale = tensors["right_scale"]

    def cache_spec(self):
        return tuple(child.cache_spec() for _, child in self.children)

    def forward(self, x, residual, ctx, cache):
        tokens = ctx.tokens
        # float rows that are clear whenever no call is under way: made cleared, and cleared again
        # by the launch that reads them
        workspace = ctx.workspace
        workspace.rows("side_left", self.width, torch.float32, cleared=True)
        workspace.rows("side_right", self.width, torch.float32, cleared=True)
        a = workspace.first_rows("side_left", self.width, torch.float32, tokens)
        b = workspace.first_rows("side_right", self.width, torch.float32, tokens)
        views = cache.children
        self.left.forward(x, a, ctx, views[0])
        self.right.forward(x, b, ctx, views[1])
        kernels.pair_norm_mix(a, b, self.left_scale, self.right_scale, self.norm_eps, 0.5, residual,
                              tokens, self.width)
