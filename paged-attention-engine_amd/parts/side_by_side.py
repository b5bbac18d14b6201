"""Two mixers side by side: both read the same input, and the result is
left_scale * left(h) + right_scale * right(h).

The two are ordinary mixers built from their own specs, with their tensors below `left.` and `right.` of
this mixer's prefix.  What they keep is kept for both under this mixer's stop: at most one of them may keep
pages (the other state only), and their state tensors' names must differ.  The sum is not formed here: the
two outputs are returned as `BranchTerms` with their factors, and the kernel that next norms the stream adds
them into the float32 residual.
"""

from __future__ import annotations

from .base import MIXERS, BranchTerms, Part, build_part, register_mixer


def _as_tuple(spec):
    if spec is None:
        return ()
    return tuple(spec) if isinstance(spec, (tuple, list)) else (spec,)


@register_mixer("side_by_side")
class SideBySide(Part):
    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.left is None or spec.right is None:
            raise ValueError("two mixers side by side need both of their specs")
        self.left = build_part(MIXERS, "mixer", spec.left, dtype, device)
        self.right = build_part(MIXERS, "mixer", spec.right, dtype, device)
        if self.left.paged_spec() is not None and self.right.paged_spec() is not None:
            raise ValueError("of two mixers side by side only one may keep pages")
        names = [one.name for side in (self.left, self.right) for one in _as_tuple(side.state_spec())]
        if len(set(names)) != len(names):
            raise ValueError(f"two mixers side by side keep state under the same name: {names}")

    def inner_parts(self):
        return [self.left, self.right]

    @property
    def graph_safe(self) -> bool:
        return self.left.graph_safe and self.right.graph_safe

    @property
    def graph_max_rows(self):
        limits = [side.graph_max_rows for side in (self.left, self.right) if side.graph_max_rows is not None]
        return min(limits) if limits else None

    def paged_spec(self):
        return self.left.paged_spec() or self.right.paged_spec()

    def state_spec(self):
        specs = _as_tuple(self.left.state_spec()) + _as_tuple(self.right.state_spec())
        return specs or None

    def tensors(self, prefix):
        s = self.spec
        return {**self.left.tensors(prefix + s.left_prefix), **self.right.tensors(prefix + s.right_prefix)}

    def bind(self, prefix, weights):
        s = self.spec
        self.left.bind(prefix + s.left_prefix, weights)
        self.right.bind(prefix + s.right_prefix, weights)

    def forward(self, ctx, x):
        s = self.spec
        terms = BranchTerms()
        for side, factor in ((self.left, s.left_scale), (self.right, s.right_scale)):
            y = side.forward(ctx, x)
            if isinstance(y, BranchTerms):
                terms.extend((t, factor * f) for t, f in y)
            else:
                terms.append((y, factor))
        return terms
