"""Norms of the residual stream, in float32.

RMSNorm: y = x / sqrt(mean(x^2) + eps) * w (src/lfm25_gpu.cu:235,244); with offset c the stored weight
lies around zero and y = x / sqrt(mean(x^2) + eps) * (c + w).
DynamicTanh: y = tanh(alpha x) w + b with a learned scalar alpha; no mean, no variance.
LayerNorm: y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w, a weight and no bias.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..csrc import ops
from .base import NORMS, Norm, Runtime, WeightDecl


class PendingNorm:
    """An RMSNorm that has not run yet: the float32 rows, the weight and eps.  A projection that
    can apply the norm inside its own kernel takes it as it is; anything else calls tensor(),
    which runs the norm kernel once."""

    def __init__(self, norm: "RMSNorm", x: torch.Tensor, rows: Optional[torch.Tensor], pre=None):
        self.norm, self.x, self.rows = norm, x, rows
        self.pre = pre            # (xw, ss) left by the product that last added into x, or None
        self._tensor: Optional[torch.Tensor] = None

    @property
    def shape(self):
        n = self.x.shape[0] if self.rows is None else self.rows.shape[0]
        return (n, self.norm.dim)

    @property
    def dtype(self):
        return self.norm.rt.dtype

    def tensor(self) -> torch.Tensor:
        if self._tensor is None:
            self._tensor = self.norm.forward(self.x, self.rows)
        return self._tensor


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True
    records_portions = True

    def __init__(self, dim: int, eps: float, name: str, aliases: tuple = (), offset: float = 0.0):
        """offset: added to the stored weight (a checkpoint that keeps its norm weights around zero: offset 1)."""
        self.dim, self.eps, self.name, self.aliases = int(dim), float(eps), name, tuple(aliases)
        self.offset = float(offset)
        self.weight: Optional[torch.Tensor] = None

    def weight_decls(self):
        return [WeightDecl(self.name, (self.dim,), "normal" if self.offset else "norm", aliases=self.aliases)]

    def kernel_modules(self):
        return ["elementwise"]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        self.weight = weights[self.name]
        if self.offset:
            # the sum is float32 whatever the stored type: every kernel that takes this norm reads the sum
            self.weight = (self.weight.float() + self.offset).contiguous()
        self.weight_f32 = self.weight if self.weight.dtype == torch.float32 else self.weight.float()

    def pending(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> PendingNorm:
        """The norm of x as a PendingNorm, for consumers that say they accept one."""
        pre = self.take_announced(x)
        return PendingNorm(self, x, rows, pre if rows is None else None)

    def take_announced(self, x: torch.Tensor):
        """(xw, ss) if the product that last added into x announced them, else None; either way nothing stays."""
        ready, self._ready = getattr(self, "_ready", None), None
        return ready[1:] if ready is not None and ready[0] is x else None

    def announce_operand(self, x: torch.Tensor, xw: torch.Tensor, ss: torch.Tensor) -> None:
        """Called by the product that has just added into x and, in the same kernel, written
        xw = bf16(x * weight) and the per-tile sums of squares ss: the next pending(x) carries them."""
        self._ready = (x, xw, ss)

    def forget(self) -> None:
        """Drops what announce_operand() left, if nobody asked for it (end of a step)."""
        self._ready = None

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.shape[0]
        out = self.rt.empty(n, self.dim)
        ops.rmsnorm(x, self.weight, out, self.eps, rows)
        return out


@NORMS.register("dyt")
class DynamicTanh(Norm):
    """y = tanh(alpha * x) * w + b: an element-wise squashing in place of a norm; it reads no statistics of
    the row, so it has no eps.  names: checkpoint names of 'weight' [d], 'bias' [d] and 'alpha' (a scalar)."""
    graph_safe = True
    records_portions = True

    def __init__(self, dim: int, *, names: dict[str, str]):
        self.dim, self.names = int(dim), dict(names)

    def weight_decls(self):
        return [WeightDecl(self.names["weight"], (self.dim,), "norm"),
                WeightDecl(self.names["bias"], (self.dim,), "normal"),
                WeightDecl(self.names["alpha"], (), "norm", alt_shapes=((1,),))]

    def kernel_modules(self):
        return ["elementwise"]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        self.weight_f32 = weights[self.names["weight"]].float().contiguous()
        self.bias_f32 = weights[self.names["bias"]].float().contiguous()
        self.alpha_f32 = weights[self.names["alpha"]].float().reshape(1).contiguous()

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.shape[0]
        out = self.rt.empty(n, self.dim)
        ops.dyt(x, self.weight_f32, self.bias_f32, self.alpha_f32, out, rows)
        return out


@NORMS.register("layernorm")
class LayerNorm(Norm):
    """y = (x - mean(x)) / sqrt(var(x) + eps) * w with var the mean of the squared deviations; a weight [d] and no
    bias.  Statistics and result are formed in float32 and rounded once to the compute type."""
    graph_safe = True
    records_portions = True

    def __init__(self, dim: int, eps: float, name: str):
        self.dim, self.eps, self.name = int(dim), float(eps), name

    def weight_decls(self):
        return [WeightDecl(self.name, (self.dim,), "norm")]

    def kernel_modules(self):
        return ["postnorm"]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        self.weight_f32 = weights[self.name].float().contiguous()

    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.shape[0]
        out = self.rt.empty(n, self.dim)
        ops.scale_add_layer_norm(x, next_w=self.weight_f32, eps=self.eps, h_out=out, rows=rows)
        return out
