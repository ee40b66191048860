"""Arrangement of norms, mixer and feed-forward in a block.

``prenorm`` (/root/reference/core/src/model/emit.cpp:436-459 without the
optional post-norms): x += mixer(norm(x)); x += ffn(norm(x)).  Mixer and
feed-forward add their result into the float32 residual stream themselves,
which lets their last projection fuse the addition (and a multiplier of the
branch, the ``out_scale`` of their specs).  A block may have no feed-forward:
it is then the first sublayer alone.  With ``input_taps`` the mixer reads h + conv(h) in place of
h = norm(x): a causal convolution over time on every channel of the normed stream (taps
[width, input_taps], the last on the current token, zeros before the sequence's start), whose last
input_taps - 1 inputs are per-sequence state of the block.

``outnorm``: the sublayers read the stream as it is and the norm sits on what they give back:
x += norm(mixer(x)); x += norm(ffn(x)).  The mixer and the feed-forward hand their result over
(``produce``) and one pass sums its slices, norms it, adds it into the stream and leaves the new
stream in the activation type for the sublayer that reads it next.

``parallel``: both sublayers read the same stream, each through a norm of its own, and their results
join it together: x += mixer(norm1(x)) + ffn(norm2(x)).  One pass norms the stream for both (the root
mean square is the same, the weights differ); the mixer and the feed-forward then add into the stream
one after the other.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import Branch, Part, StateSpec, register_part
from .spec import PartSpec, TensorSpec


def prenorm_block_spec(mixer_norm: PartSpec, mixer: PartSpec, ffn_norm: PartSpec = None, ffn: PartSpec = None,
                       input_conv_name: str = None, input_taps: int = 0, width: int = 0) -> PartSpec:
    """``input_conv_name``: the tensor [width, input_taps] of the convolution over time that the
    mixer's input passes (h + conv(h))."""
    parts = {"mixer_norm": mixer_norm, "mixer": mixer}
    if ffn is not None:
        if ffn_norm is None:
            raise ValueError("a block with a feed-forward needs the norm before it")
        parts.update(ffn_norm=ffn_norm, ffn=ffn)
    params, tensors = {}, {}
    if input_conv_name is not None:
        if input_taps < 2 or width <= 0:
            raise ValueError("a convolution on the mixer's input needs at least two taps and the stream's width")
        params = {"input_taps": int(input_taps), "width": int(width)}
        tensors = {"input_conv": TensorSpec(input_conv_name, (width, input_taps), init=(0.0, 0.1))}
    return PartSpec("block", "prenorm", params, tensors, parts)


@register_part("block", "prenorm")
class PreNormBlock(Part):
    category = "block"

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        self.mixer_norm = parts["mixer_norm"]
        self.first_norm = self.mixer_norm      # what the block before may apply in its last pass
        self.mixer = parts["mixer"]
        self.ffn_norm = parts.get("ffn_norm")
        self.ffn = parts.get("ffn")              # None: the block is its mixer's sublayer alone
        self.input_taps = int(spec.params.get("input_taps", 0) or 0)
        self.input_conv = tensors.get("input_conv") if self.input_taps else None
        if self.input_taps and self.input_taps > ops.time_conv_max_taps():
            raise ValueError(f"{self.input_taps} taps are more than the convolution kernel's {ops.time_conv_max_taps()}")

    def state_specs(self):
        """The last taps - 1 inputs of the convolution on the mixer's input, a row of the stream's width each."""
        if not self.input_taps:
            return {}
        return {"input_conv": StateSpec((self.input_taps - 1, int(self.spec.params["width"])), torch.float32)}

    def forward(self, x, ctx, binding, h=None, next_norm=None):
        """Run the block on the residual stream ``x`` in place.  ``h`` is mixer_norm(x) when the
        previous block has already computed it; ``next_norm`` is the norm the next block starts
        with.  Returns next_norm(x) when the feed-forward's last pass produced it, else None.
        Mixers and feed-forwards that can apply a norm in their last pass say so with
        ``fuses_norm``; the others are simply followed by the norm."""
        act = self.rt.act_dtype
        if h is None:
            h = self.mixer_norm.forward(x, act)
        if self.input_conv is not None:
            h = ops.time_conv(h, self.input_conv, None, binding.states["block.input_conv"], ctx, act, residual=True)
        f = None
        after = self.ffn_norm if self.ffn is not None else next_norm     # the norm that follows the mixer
        if getattr(self.mixer, "fuses_norm", False):
            f = self.mixer.forward(h, x, ctx, binding, then_norm=after)
        else:
            self.mixer.forward(h, x, ctx, binding)
        trace = getattr(ctx, "trace", None)
        if trace is not None:
            trace("after_mixer", x)
        if self.ffn is None:
            return f
        if f is None:
            f = self.ffn_norm.forward(x, act)
        out = None
        if getattr(self.ffn, "fuses_norm", False):
            out = self.ffn.forward(f, x, ctx, then_norm=next_norm)
        else:
            self.ffn.forward(f, x, ctx)
        if trace is not None:
            trace("after_ffn", x)
        return out


def outnorm_block_spec(mixer_norm: PartSpec, mixer: PartSpec, ffn_norm: PartSpec = None, ffn: PartSpec = None) -> PartSpec:
    parts = {"mixer_norm": mixer_norm, "mixer": mixer}
    if ffn is not None:
        if ffn_norm is None:
            raise ValueError("a block with a feed-forward needs the norm after it")
        parts.update(ffn_norm=ffn_norm, ffn=ffn)
    return PartSpec("block", "outnorm", {}, {}, parts)


class StreamAsItIs:
    """What a block that reads the stream itself names as its ``first_norm``: no norm, the stream
    in the activation type.  A block before it that cannot produce that in its last pass is simply
    followed by the conversion."""
    fusable = False
    weight = None

    def forward(self, x, out_dtype, rows=None):
        if rows is not None:
            raise ValueError("the stream as it is has no picked rows")
        return ops.cast(x, out_dtype)


@register_part("block", "outnorm")
class OutNormBlock(Part):
    category = "block"

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        self.mixer_norm = parts["mixer_norm"]
        self.first_norm = StreamAsItIs()
        self.mixer = parts["mixer"]
        self.ffn_norm = parts.get("ffn_norm")
        self.ffn = parts.get("ffn")
        for part, what in ((self.mixer, "mixer"), (self.ffn, "feed-forward")):
            if part is not None and not hasattr(part, "produce"):
                raise ValueError(f"a block that norms outputs needs a {what} that hands its result over (produce)")
        for n in (self.mixer_norm, self.ffn_norm):
            if n is not None and (getattr(n, "groups", 1) != 1 or not hasattr(n, "eps")):
                raise ValueError("a block that norms outputs takes RMS norms over whole rows")

    def _join(self, x, y, norm, copy_dtype):
        """x += norm(y); the new stream in ``copy_dtype`` (x itself when that is float32)."""
        b = y if isinstance(y, Branch) else Branch(y)
        return ops.norm_add(x, b.part, norm.weight, norm.eps, getattr(norm, "offset", 0.0), copy_dtype,
                            part_weights=b.part_weights, extra=b.extra, extra_weights=b.extra_weights, by_row=b.by_row)

    def forward(self, x, ctx, binding, h=None, next_norm=None):
        """Run the block on the residual stream ``x`` in place.  ``h``: the stream in the activation
        type when the block before has left it.  Returns the stream in the activation type when the
        next block reads it as it is, else None."""
        act = self.rt.act_dtype
        if h is None:
            left = (getattr(ctx, "shared", None) or {}).pop("stream", None)      # the embedding's own copy of what it made
            h = left[1] if left is not None and left[0] is x and left[1].dtype == act else ops.cast(x, act)
        last = self.ffn is None
        want = act if not last or isinstance(next_norm, StreamAsItIs) else None
        h = self._join(x, self.mixer.produce(h, ctx, binding), self.mixer_norm, want)
        trace = getattr(ctx, "trace", None)
        if trace is not None:
            trace("after_mixer", x)
        if last:
            return h
        want = act if isinstance(next_norm, StreamAsItIs) else None
        h = self._join(x, self.ffn.produce(h, ctx), self.ffn_norm, want)
        if trace is not None:
            trace("after_ffn", x)
        return h


def parallel_block_spec(mixer_norm: PartSpec, mixer: PartSpec, ffn_norm: PartSpec = None, ffn: PartSpec = None) -> PartSpec:
    parts = {"mixer_norm": mixer_norm, "mixer": mixer}
    if ffn is not None:
        if ffn_norm is None:
            raise ValueError("a block with a feed-forward needs the norm before it")
        parts.update(ffn_norm=ffn_norm, ffn=ffn)
    return PartSpec("block", "parallel", {}, {}, parts)


@register_part("block", "parallel")
class ParallelBlock(Part):
    category = "block"

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        self.mixer_norm = parts["mixer_norm"]
        self.mixer = parts["mixer"]
        self.ffn_norm = parts.get("ffn_norm")
        self.ffn = parts.get("ffn")              # None: the block is its mixer's branch alone
        # with two branches the block norms for both in one pass of its own; alone, the mixer's norm is what
        # the block before may apply in its last pass
        self.first_norm = self.mixer_norm if self.ffn is None else None
        a, b = self.mixer_norm, self.ffn_norm
        # one pass for both norms when they are RMS norms over whole rows with the same eps and plain weights
        self.one_pass = b is not None and all(
            getattr(n, "fusable", False) and getattr(n, "groups", 1) == 1 and hasattr(n, "eps") for n in (a, b)) \
            and a.eps == b.eps and (a.weight is None) == (b.weight is None) \
            and (a.weight is None or a.weight.dtype == b.weight.dtype)

    def forward(self, x, ctx, binding, h=None, next_norm=None):
        """Run the block on the residual stream ``x`` in place.  ``h`` is mixer_norm(x) when the block
        before has already computed it.  Returns next_norm(x) when the last pass produced it, else None.
        Both branches are normed before either result joins the stream."""
        act = self.rt.act_dtype
        f = None
        if self.ffn is not None:
            if h is None and self.one_pass:
                h, f = ops.rmsnorm_pair(x, self.mixer_norm.weight, self.ffn_norm.weight, self.mixer_norm.eps, act)
            else:
                f = self.ffn_norm.forward(x, act)
        if h is None:
            h = self.mixer_norm.forward(x, act)
        last = self.ffn is None
        if getattr(self.mixer, "fuses_norm", False):
            out = self.mixer.forward(h, x, ctx, binding, then_norm=next_norm if last else None)
        else:
            out = self.mixer.forward(h, x, ctx, binding)
        trace = getattr(ctx, "trace", None)
        if trace is not None:
            trace("after_mixer", x)
        if last:
            return out
        out = None
        if getattr(self.ffn, "fuses_norm", False):
            out = self.ffn.forward(f, x, ctx, then_norm=next_norm)
        else:
            self.ffn.forward(f, x, ctx)
        if trace is not None:
            trace("after_ffn", x)
        return out
