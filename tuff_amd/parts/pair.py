"""Two mixers side by side on the same input:
    y = coef * (norm_l(left(h)) + norm_r(right(h))),   norm(z) = z / sqrt(mean(z^2) + eps) * w
each output normed over the model width with a plain weight of its own before the two are summed (coef 1/2:
their mean).  The two may be any mixers; what they keep per request lies side by side in the cache (the left
one's declarations, then the right one's).
"""
from __future__ import annotations

import torch

from ..csrc import ops
from .base import MIXERS, Mixer, Runtime, WeightDecl, cache_specs_of


@MIXERS.register("pair")
class PairMixer(Mixer):
    def __init__(self, hidden_size: int, left: Mixer, right: Mixer, eps: float, *, names: dict[str, str], coef: float = 0.5):
        """names: checkpoint names of 'left_norm' and 'right_norm' [d], the weights of the two outputs' norms."""
        self.d, self.left, self.right, self.eps, self.coef = int(hidden_size), left, right, float(eps), float(coef)
        self.names = dict(names)
        self._left_specs, self._left_several = cache_specs_of(left)
        self._right_specs, self._right_several = cache_specs_of(right)

    @property
    def graph_safe(self):
        return self.left.graph_safe and self.right.graph_safe

    @property
    def records_portions(self):
        return self.left.records_portions and self.right.records_portions

    def weight_decls(self):
        return (self.left.weight_decls() + self.right.weight_decls()
                + [WeightDecl(self.names["left_norm"], (self.d,), "norm"), WeightDecl(self.names["right_norm"], (self.d,), "norm")])

    def kernel_modules(self):
        return ["postnorm", "elementwise"] + self.left.kernel_modules() + self.right.kernel_modules()

    def token_inputs(self):
        return self.left.token_inputs() + self.right.token_inputs()

    def cache_spec(self):
        both = self._left_specs + self._right_specs
        return both if both else None

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        self.left.bind(weights, rt)
        self.right.bind(weights, rt)
        self.w_left = weights[self.names["left_norm"]].float().contiguous()
        self.w_right = weights[self.names["right_norm"]].float().contiguous()

    @staticmethod
    def _views(views: tuple, several: bool):
        return views if several else (views[0] if views else None)

    def forward(self, h, ctx, cache, residual, write_cache: bool = True) -> None:
        views = tuple(cache) if cache is not None else ()
        n = len(self._left_specs)
        T = h.shape[0]
        # what the two add their outputs into, cleared by one kernel
        ab = torch.empty(2, T, self.d, dtype=torch.float32, device=residual.device)
        ops.fill_u32(ab, 0)
        for mixer, out, v, several in ((self.left, ab[0], views[:n], self._left_several),
                                       (self.right, ab[1], views[n:], self._right_several)):
            kw = {"next_norm": None} if mixer.adds_once_through_linear else {}
            mixer.forward(h, ctx, self._views(v, several), out, write_cache, **kw)
        ops.normed_mean2(ab[0], self.w_left, ab[1], self.w_right, residual, eps=self.eps, coef=self.coef)
