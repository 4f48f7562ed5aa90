"""Arrangements of parts around the residual stream.

PreNormBlock is the reference's layer (src/lfm25_engine.c:370-419):
    x += mixer(norm1(x));  x += ffn(norm2(x))
with the residual stream x in float32.  A feed-forward of None leaves out the second half.

ParallelBlock has one norm whose output both sublayers read:
    h = norm(x);  x += mixer(h) + ffn(h)

SandwichBlock norms a sublayer on both sides:
    x += m * norm1b(mixer(norm1(x)));  x += m * norm2b(ffn(norm2(x)))

LayerScaleBlock is the pre-norm layer whose sublayers' outputs are scaled per channel before they join the stream:
    x += ls1 * mixer(norm1(x));  x += ls2 * ffn(norm2(x))

HyperConnectionBlock is the pre-norm layer over several residual streams: a sublayer reads a weighted sum
of the streams and its output goes back into all of them through a mixing matrix.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..csrc import ops
from .base import BLOCKS, Block, FeedForward, Mixer, Norm, Runtime, WeightDecl
from .norm import LayerNorm, RMSNorm


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Optional[Norm] = None,
                 ffn: Optional[FeedForward] = None):
        if (norm2 is None) != (ffn is None):
            raise ValueError("norm2 and ffn go together")
        self.norm1, self.mixer, self.norm2, self.ffn = norm1, mixer, norm2, ffn

    def _parts(self):
        return [p for p in (self.norm1, self.mixer, self.norm2, self.ffn) if p is not None]

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self._parts())

    @property
    def records_portions(self):
        return all(p.records_portions for p in self._parts())

    def weight_decls(self):
        return [d for p in self._parts() for d in p.weight_decls()]

    def kernel_modules(self):
        return [m for p in self._parts() for m in p.kernel_modules()]

    def token_inputs(self):
        return [t for p in self._parts() for t in p.token_inputs()]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        for p in self._parts():
            p.bind(weights, rt)

    takes_next_norm = True

    def first_norm_consumer(self):
        """(norm, part that consumes it) at the head of the block, for the block before this one."""
        return self.norm1, self.mixer

    def forward(self, x, ctx, cache, write_cache: bool = True, next_norm=None) -> None:
        """next_norm: (norm, consumer) that will read x right after this block, or None."""
        h = self._normed(self.norm1, x, self.mixer)
        after = self._hand_over(self.mixer, (self.norm2, self.ffn) if self.ffn is not None else next_norm)
        self.mixer.forward(h, ctx, cache, x, write_cache, **after)
        if self.ffn is not None:
            h = self._normed(self.norm2, x, self.ffn)
            after = self._hand_over(self.ffn, next_norm)
            self.ffn.forward(h, ctx, x, **after)

    def forget(self) -> None:
        """End of a step: drops what a product left for a norm that never asked for it."""
        for n in (self.norm1, self.norm2):
            if hasattr(n, "forget"):
                n.forget()

    @staticmethod
    def _hand_over(producer, nxt) -> dict:
        """The keyword that tells the producer's last projection which norm reads x next: only if
        producer, norm and the norm's consumer all know how (else nothing is passed and the norm
        runs as a kernel of its own)."""
        if not producer.adds_once_through_linear:
            return {}
        ok = (nxt is not None and hasattr(nxt[0], "announce_operand") and nxt[1] is not None
              and nxt[1].accepts_pending_norm)
        return {"next_norm": nxt[0] if ok else None}

    @staticmethod
    def _normed(norm, x, consumer):
        """The norm of x for `consumer`: left pending if both sides know how (the consumer's first
        projection then runs the norm inside its kernel), else computed now."""
        if consumer.accepts_pending_norm and hasattr(norm, "pending"):
            return norm.pending(x)
        return norm.forward(x)


@BLOCKS.register("parallel")
class ParallelBlock(Block):
    """x <- x + mixer(h) + ffn(h) with h = norm(x): mixer and feed-forward read the same normed rows and
    both add into the float32 stream.  ffn None: the mixer alone."""

    def __init__(self, norm: Norm, mixer: Mixer, ffn: Optional[FeedForward] = None):
        self.norm, self.mixer, self.ffn = norm, mixer, ffn

    def _parts(self):
        return [p for p in (self.norm, self.mixer, self.ffn) if p is not None]

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self._parts())

    @property
    def records_portions(self):
        return all(p.records_portions for p in self._parts())

    def weight_decls(self):
        return [d for p in self._parts() for d in p.weight_decls()]

    def kernel_modules(self):
        return [m for p in self._parts() for m in p.kernel_modules()]

    def token_inputs(self):
        return [t for p in self._parts() for t in p.token_inputs()]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        for p in self._parts():
            p.bind(weights, rt)

    def forward(self, x, ctx, cache, write_cache: bool = True) -> None:
        h = self.norm.forward(x)            # computed before either sublayer touches x
        kw = {"next_norm": None} if self.mixer.adds_once_through_linear else {}
        self.mixer.forward(h, ctx, cache, x, write_cache, **kw)
        if self.ffn is not None:
            kw = {"next_norm": None} if self.ffn.adds_once_through_linear else {}
            self.ffn.forward(h, ctx, x, **kw)


@BLOCKS.register("sandwich")
class SandwichBlock(Block):
    """x <- x + mult * after1(mixer(before1(x))), then x <- x + mult * after2(ffn(before2(x))): every sublayer is
    normed before and after.  ffn None: the mixer's sublayer alone.  The four norms are RMS norms (they run inside
    one kernel, ops.post_norm_add, which norms a sublayer's output, adds it into the stream and reads the next
    sublayer's input with its norm; the next sublayer may be the next block's first, so forward() takes what the
    block before left (`carry`) and is told who reads next (`next_read`))."""
    carries_norm = True

    def __init__(self, before1: Norm, mixer: Mixer, after1: Norm, before2: Optional[Norm] = None,
                 ffn: Optional[FeedForward] = None, after2: Optional[Norm] = None, *, mult: float = 1.0):
        if not ((before2 is None) == (ffn is None) == (after2 is None)):
            raise ValueError("before2, ffn and after2 go together")
        for n in (before1, after1, before2, after2):
            if n is not None and not isinstance(n, RMSNorm):
                raise ValueError("the norms of a sandwich block are RMS norms (they run inside the block's kernel)")
        self.before1, self.mixer, self.after1 = before1, mixer, after1
        self.before2, self.ffn, self.after2 = before2, ffn, after2
        self.mult = float(mult)

    def _parts(self):
        return [p for p in (self.before1, self.mixer, self.after1, self.before2, self.ffn, self.after2) if p is not None]

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self._parts())

    @property
    def records_portions(self):
        return all(p.records_portions for p in self._parts())

    def weight_decls(self):
        return [d for p in self._parts() for d in p.weight_decls()]

    def kernel_modules(self):
        return ["postnorm", "elementwise"] + [m for p in self._parts() for m in p.kernel_modules()]

    def token_inputs(self):
        return [t for p in self._parts() for t in p.token_inputs()]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        for p in self._parts():
            p.bind(weights, rt)

    def first_read(self):
        """(norm weight float32 [d], eps): what the block before needs to prepare this block's first input."""
        return self.before1.weight_f32, self.before1.eps

    def forward(self, x, ctx, cache, write_cache: bool = True, carry=None, next_read=None, y=None, extra=None):
        """x float32 [T, d], in place.  carry: before1(x) where the block before left it (None: computed here).
        next_read: (norm weight, eps) of whoever reads x next; that norm of the new x is returned (None: nothing is
        read and None returned).  y: float32 [T, d] of zeros that the sublayers add into (left zero again); None:
        made here.  extra: float32 [T, d] that joins x after the block's last sublayer, before next_read's norm."""
        T, d = x.shape
        if carry is None:
            carry = self.before1.forward(x)
        if y is None:
            y = torch.empty(T, d, dtype=torch.float32, device=x.device)
            ops.fill_u32(y, 0)
        kw = {"next_norm": None} if self.mixer.adds_once_through_linear else {}
        self.mixer.forward(carry, ctx, cache, y, write_cache, **kw)
        if self.ffn is None:
            return self._join(x, y, self.after1, next_read, extra)
        # (a feed-forward that adds a bias to its output: the kernel that clears y leaves the bias there instead)
        bias = getattr(self.ffn, "output_bias", None)
        h = self._join(x, y, self.after1, (self.before2.weight_f32, self.before2.eps), None, y_next=bias)
        kw = {"next_norm": None} if self.ffn.adds_once_through_linear else {}
        if bias is not None:
            kw["bias_preloaded"] = True
        self.ffn.forward(h, ctx, y, **kw)
        return self._join(x, y, self.after2, next_read, extra)

    def _join(self, x, y, after, read, extra, y_next=None):
        h = None
        kw = {}
        if read is not None:
            h = self.rt.empty(*x.shape)
            kw = dict(next_w=read[0], next_eps=read[1], h_out=h)
        ops.post_norm_add(x, y=y, w=after.weight_f32, eps=after.eps, mult=self.mult, extra=extra, clear_y=True, y_next=y_next, **kw)
        return h


@BLOCKS.register("layer_scale")
class LayerScaleBlock(Block):
    """x <- x + ls1 * mixer(norm1(x)), then x <- x + ls2 * ffn(norm2(x)): pre-norm with a learned scale per channel
    ('layer scale') on each sublayer's output.  ffn None: the mixer's sublayer alone.  The norms are layer norms (they
    run inside one kernel, ops.scale_add_layer_norm, which scales a sublayer's output, adds it into the stream and
    reads the next sublayer's input with its norm; the next sublayer may be the next block's first, so forward()
    takes what the block before left (`carry`) and is told who reads next (`next_read`)).  names: checkpoint names
    'ls1' [d] and, with a feed-forward, 'ls2' [d]."""
    carries_norm = True

    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Optional[Norm] = None, ffn: Optional[FeedForward] = None, *,
                 names: dict[str, str]):
        if (norm2 is None) != (ffn is None):
            raise ValueError("norm2 and ffn go together")
        for n in (norm1, norm2):
            if n is not None and not isinstance(n, LayerNorm):
                raise ValueError("the norms of a layer-scale block are layer norms (they run inside the block's kernel)")
        self.norm1, self.mixer, self.norm2, self.ffn = norm1, mixer, norm2, ffn
        self.names = dict(names)

    def _parts(self):
        return [p for p in (self.norm1, self.mixer, self.norm2, self.ffn) if p is not None]

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self._parts())

    @property
    def records_portions(self):
        return all(p.records_portions for p in self._parts())

    def weight_decls(self):
        decls = [d for p in self._parts() for d in p.weight_decls()]
        decls.append(WeightDecl(self.names["ls1"], (self.norm1.dim,), "norm"))
        if self.ffn is not None:
            decls.append(WeightDecl(self.names["ls2"], (self.norm1.dim,), "norm"))
        return decls

    def kernel_modules(self):
        return ["postnorm", "elementwise"] + [m for p in self._parts() for m in p.kernel_modules()]

    def token_inputs(self):
        return [t for p in self._parts() for t in p.token_inputs()]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        for p in self._parts():
            p.bind(weights, rt)
        self.ls1 = weights[self.names["ls1"]].float().contiguous()
        self.ls2 = weights[self.names["ls2"]].float().contiguous() if self.ffn is not None else None

    def first_read(self):
        """(norm weight float32 [d], eps): what the block before needs to prepare this block's first input."""
        return self.norm1.weight_f32, self.norm1.eps

    def forward(self, x, ctx, cache, write_cache: bool = True, carry=None, next_read=None, y=None, extra=None):
        """x float32 [T, d], in place.  carry: norm1(x) where the block before left it (None: computed here).
        next_read: (norm weight, eps) of whoever reads x next; that norm of the new x is returned (None: nothing is
        read and None returned).  y: float32 [T, d] of zeros that the sublayers add into (left zero again); None:
        made here."""
        if extra is not None:
            raise ValueError("a layer-scale block adds nothing but its sublayers to the stream")
        T, d = x.shape
        if carry is None:
            carry = self.norm1.forward(x)
        if y is None:
            y = torch.empty(T, d, dtype=torch.float32, device=x.device)
            ops.fill_u32(y, 0)
        kw = {"next_norm": None} if self.mixer.adds_once_through_linear else {}
        self.mixer.forward(carry, ctx, cache, y, write_cache, **kw)
        if self.ffn is None:
            return self._join(x, y, self.ls1, next_read)
        h = self._join(x, y, self.ls1, (self.norm2.weight_f32, self.norm2.eps))
        kw = {"next_norm": None} if self.ffn.adds_once_through_linear else {}
        self.ffn.forward(h, ctx, y, **kw)
        return self._join(x, y, self.ls2, next_read)

    def _join(self, x, y, ls, read):
        h = None
        kw = {}
        if read is not None:
            h = self.rt.empty(*x.shape)
            kw = dict(next_w=read[0], eps=read[1], h_out=h)
        ops.scale_add_layer_norm(x, y=y, ls=ls, clear_y=True, **kw)
        return h


@BLOCKS.register("hyper")
class HyperConnectionBlock(Block):
    """A pre-norm layer over S residual streams xs [S, T, d] instead of one.  For sublayer q (1: the mixer, 2: the
    feed-forward) with its three tensors in_q [S], mix_q [S, S] (indexed [from, to]) and out_q [S]:
        u = sum_s in_q[s] xs[s];   y = sublayer(norm_q(u));   xs[r] <- sum_s mix_q[s, r] xs[s] + out_q[r] y
    (all streams at once, from the old values).  ffn None: the mixer's sublayer alone.

    One kernel writes a sublayer's output into the streams and reads the next sublayer's input with its norm
    (ops.hc_step); the next sublayer may be the next block's first, so forward() takes what the block before left
    (`carry`) and is told who reads next (`next_read`).  names: checkpoint names 'in1', 'mix1', 'out1' and, with
    a feed-forward, 'in2', 'mix2', 'out2'."""
    multi_stream = True

    def __init__(self, streams: int, norm1: Norm, mixer: Mixer, norm2: Optional[Norm] = None,
                 ffn: Optional[FeedForward] = None, *, names: dict[str, str]):
        if (norm2 is None) != (ffn is None):
            raise ValueError("norm2 and ffn go together")
        self.S = int(streams)
        if self.S < 1:
            raise ValueError("at least one stream")
        for n in (norm1, norm2):
            if n is not None and not isinstance(n, RMSNorm):
                raise ValueError("the norms of a hyper-connection block are RMS norms (they run inside the streams' kernel)")
        self.norm1, self.mixer, self.norm2, self.ffn = norm1, mixer, norm2, ffn
        self.names = dict(names)

    def _parts(self):
        return [p for p in (self.norm1, self.mixer, self.norm2, self.ffn) if p is not None]

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self._parts())

    @property
    def records_portions(self):
        return all(p.records_portions for p in self._parts())

    def weight_decls(self):
        S = self.S
        decls = [d for p in self._parts() for d in p.weight_decls()]
        for q in ("1", "2") if self.ffn is not None else ("1",):
            decls += [WeightDecl(self.names["in" + q], (S,), f"around:{1.0 / S}"),
                      WeightDecl(self.names["out" + q], (S,), "norm"),
                      WeightDecl(self.names["mix" + q], (S, S), "identity")]
        return decls

    def kernel_modules(self):
        return ["hyper", "elementwise"] + [m for p in self._parts() for m in p.kernel_modules()]

    def token_inputs(self):
        return [t for p in self._parts() for t in p.token_inputs()]

    def bind(self, weights, rt: Runtime):
        self.rt = rt
        for p in self._parts():
            p.bind(weights, rt)
        f32 = lambda name: weights[self.names[name]].to(torch.float32).contiguous()
        self.hc = {q: (f32("in" + q), f32("mix" + q), f32("out" + q)) for q in (("1", "2") if self.ffn is not None else ("1",))}

    def first_read(self):
        """(in [S], norm weight float32 [d], eps): what the block before needs to prepare this block's first input."""
        return self.hc["1"][0], self.norm1.weight_f32, self.norm1.eps

    def forward(self, xs, ctx, cache, write_cache: bool = True, carry=None, next_read=None, y=None):
        """xs float32 [S, T, d], in place.  carry: norm1(u) of this block's first sublayer where the block before
        left it (None: computed here).  next_read: (in, norm weight or None, eps) of whoever reads the streams
        next; the result of that read is returned (the normed rows in the compute type, or, without a norm weight,
        the plain weighted sum in float32); None: nothing is read.  y: float32 [T, d] of zeros that the sublayers add
        into (the kernel that mixes it into the streams leaves it zero again); None: made here."""
        S, T, d = xs.shape
        if S != self.S:
            raise ValueError(f"{S} streams handed to a block of {self.S}")
        if carry is None:
            carry = self.rt.empty(T, d)
            in1, w1, eps1 = self.first_read()
            ops.hc_step(xs, in_w=in1, norm_w=w1, eps=eps1, h_out=carry)
        if y is None:
            y = torch.empty(T, d, dtype=torch.float32, device=xs.device)
            ops.fill_u32(y, 0)
        kw = {"next_norm": None} if self.mixer.adds_once_through_linear else {}
        self.mixer.forward(carry, ctx, cache, y, write_cache, **kw)
        _, mix1, out1 = self.hc["1"]
        if self.ffn is None:
            return self._write_and_read(xs, y, mix1, out1, next_read)
        in2, mix2, out2 = self.hc["2"]
        h = self._write_and_read(xs, y, mix1, out1, (in2, self.norm2.weight_f32, self.norm2.eps))
        kw = {"next_norm": None} if self.ffn.adds_once_through_linear else {}
        self.ffn.forward(h, ctx, y, **kw)
        return self._write_and_read(xs, y, mix2, out2, next_read)

    def _write_and_read(self, xs, y, mix, out_w, read):
        T, d = y.shape
        if read is None:
            ops.hc_step(xs, y=y, mix=mix, out_w=out_w, clear_y=True)
            return None
        in_w, norm_w, eps = read
        if norm_w is None:
            u = torch.empty(T, d, dtype=torch.float32, device=xs.device)
            ops.hc_step(xs, y=y, mix=mix, out_w=out_w, in_w=in_w, u_out=u, clear_y=True)
            return u
        h = self.rt.empty(T, d)
        ops.hc_step(xs, y=y, mix=mix, out_w=out_w, in_w=in_w, norm_w=norm_w, eps=eps, h_out=h, clear_y=True)
        return h
