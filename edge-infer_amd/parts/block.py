"""Arrangements of norm, mixer and feed-forward in one layer."""
from __future__ import annotations

import torch

from ..csrc import lib
from ..weights.loader import ParamSpec
from .base import StateRequest
from .registry import lookup


class PreNormBlock:
    """x += mixer(norm1(x)); x += feed_forward(norm2(x)).
    runtime/include/execution/decoder.hpp:119-168 of the reference.  The second
    addition is left pending: the next block's first norm (or the model's final
    norm) performs it while reading the row.  A layer may have no feed-forward (then it has
    no second norm either, and the mixer's output is what is left pending)."""

    parts = ("norm1", "mixer", "norm2", "ffn")
    capture_safe = True      # nothing of its own besides its parts' kernels

    def members(self):
        """The parts this block is made of, in the order in which they run."""
        return tuple(part for part in (self.norm1, self.mixer, self.norm2, self.ffn)
                     if part is not None)

    @classmethod
    def _owners(cls, layer_spec):
        norm_cls = lookup("norm", layer_spec.norm.kind)
        owners = [("norm1", norm_cls, layer_spec.norm),
                  ("mixer", lookup("mixer", layer_spec.mixer.kind), layer_spec.mixer)]
        if layer_spec.feed_forward is not None:
            owners += [("norm2", norm_cls, layer_spec.norm),
                       ("ffn", lookup("feed_forward", layer_spec.feed_forward.kind),
                        layer_spec.feed_forward)]
        return owners

    @classmethod
    def parameters(cls, layer_spec, hidden):
        params = {}
        for prefix, owner, spec in cls._owners(layer_spec):
            for name, param in owner.parameters(spec, hidden).items():
                params[f"{prefix}.{name}"] = param
        if layer_spec.feed_forward is None:
            # a checkpoint may still hold the second norm of a layer without a feed-forward;
            # it is taken and has no use
            norm_cls = lookup("norm", layer_spec.norm.kind)
            for name, param in norm_cls.parameters(layer_spec.norm, hidden).items():
                params[f"norm2.{name}"] = ParamSpec(param.shape, init=param.init, optional=True)
        return params

    @classmethod
    def mixer_spec(cls, layer_spec):
        return layer_spec.mixer

    @classmethod
    def kernel_libraries(cls, layer_spec, dtype):
        """The kernel libraries its parts say they run (a part without the method says none)."""
        names = []
        for _, owner, spec in cls._owners(layer_spec):
            ask = getattr(owner, "kernel_libraries", None)
            if ask is not None:
                names.extend(ask(spec, dtype))
        return tuple(names)

    def __init__(self, layer_spec, hidden, params, dtype, device, positions):
        def sub(prefix):
            return {name[len(prefix) + 1:]: tensor for name, tensor in params.items()
                    if name.startswith(prefix + ".")}
        norm_cls = lookup("norm", layer_spec.norm.kind)
        mixer_cls = lookup("mixer", layer_spec.mixer.kind)
        self.norm1 = norm_cls(layer_spec.norm, hidden, sub("norm1"), dtype, device)
        self.mixer = mixer_cls(layer_spec.mixer, hidden, sub("mixer"), dtype, device,
                               positions=positions)
        self.norm2 = self.ffn = None
        if layer_spec.feed_forward is not None:
            ffn_cls = lookup("feed_forward", layer_spec.feed_forward.kind)
            self.norm2 = norm_cls(layer_spec.norm, hidden, sub("norm2"), dtype, device)
            self.ffn = ffn_cls(layer_spec.feed_forward, hidden, sub("ffn"), dtype, device)

    def forward(self, ctx, residual, pending, entry):
        h = self.norm1.add_norm(ctx, residual, pending, "block.h")
        ctx.release(pending)             # added into the residual: its storage is free
        a = self.mixer.forward(ctx, h, entry)
        ctx.release(h)
        if self.ffn is None:
            return a
        h2 = self.norm2.add_norm(ctx, residual, a, "block.h")
        ctx.release(a)
        out = self.ffn.forward(ctx, h2)
        ctx.release(h2)
        return out


class OutputNormBlock:
    """x += norm1(mixer(x)); x += norm2(feed_forward(x)): the sublayers read the residual
    stream itself and each norm sits on its sublayer's output.  A layer may have no
    feed-forward (then it has no second norm either).

    The stream is float32; a sublayer's products read it in the step's storage type.  In
    float32 that is the stream itself; in bfloat16 the norm kernel that adds a sublayer's
    output also writes the rounded rows for the next reader (two buffers in turn, since a
    reader's copy is still live while the next one is written), and only a model's first
    layer needs a cast kernel of its own.  The block returns no pending delta: everything is
    added when it returns."""

    capture_safe = True      # nothing of its own besides its parts' kernels and the cast
    CAST_NOTE = "outnorm.cast"     # ctx.notes: (stream rows in the storage type, index of its buffer)

    def members(self):
        return tuple(part for part in (self.mixer, self.norm1, self.ffn, self.norm2)
                     if part is not None)

    @classmethod
    def _owners(cls, layer_spec):
        norm_cls = lookup("norm", layer_spec.norm.kind)
        owners = [("mixer", lookup("mixer", layer_spec.mixer.kind), layer_spec.mixer),
                  ("norm1", norm_cls, layer_spec.norm)]
        if layer_spec.feed_forward is not None:
            owners += [("ffn", lookup("feed_forward", layer_spec.feed_forward.kind),
                        layer_spec.feed_forward),
                       ("norm2", norm_cls, layer_spec.norm)]
        return owners

    @classmethod
    def parameters(cls, layer_spec, hidden):
        params = {}
        for prefix, owner, spec in cls._owners(layer_spec):
            for name, param in owner.parameters(spec, hidden).items():
                params[f"{prefix}.{name}"] = param
        if layer_spec.feed_forward is None:
            # a checkpoint may still hold the second norm of a layer without a feed-forward;
            # it is taken and has no use
            norm_cls = lookup("norm", layer_spec.norm.kind)
            for name, param in norm_cls.parameters(layer_spec.norm, hidden).items():
                params[f"norm2.{name}"] = ParamSpec(param.shape, init=param.init, optional=True)
        return params

    @classmethod
    def mixer_spec(cls, layer_spec):
        return layer_spec.mixer

    @classmethod
    def kernel_libraries(cls, layer_spec, dtype):
        names = ["rowwise"]
        for _, owner, spec in cls._owners(layer_spec):
            ask = getattr(owner, "kernel_libraries", None)
            if ask is not None:
                names.extend(ask(spec, dtype))
        return tuple(names)

    def __init__(self, layer_spec, hidden, params, dtype, device, positions):
        def sub(prefix):
            return {name[len(prefix) + 1:]: tensor for name, tensor in params.items()
                    if name.startswith(prefix + ".")}
        norm_cls = lookup("norm", layer_spec.norm.kind)
        if not hasattr(norm_cls, "norm_add"):
            raise ValueError(f"norm kind '{layer_spec.norm.kind}' cannot sit on a sublayer's output")
        self.mixer = lookup("mixer", layer_spec.mixer.kind)(
            layer_spec.mixer, hidden, sub("mixer"), dtype, device, positions=positions)
        self.norm1 = norm_cls(layer_spec.norm, hidden, sub("norm1"), dtype, device)
        self.ffn = self.norm2 = None
        if layer_spec.feed_forward is not None:
            self.ffn = lookup("feed_forward", layer_spec.feed_forward.kind)(
                layer_spec.feed_forward, hidden, sub("ffn"), dtype, device)
            self.norm2 = norm_cls(layer_spec.norm, hidden, sub("norm2"), dtype, device)
        self.narrow = dtype != torch.float32

    def _stream_rows(self, ctx, residual):
        """The stream as the products read it, and which of the two cast buffers holds it."""
        if not self.narrow:
            return residual, 0
        held = ctx.notes.pop(self.CAST_NOTE, None)
        if held is not None:
            return held
        rows = ctx.buffer("outnorm.x0", tuple(residual.shape))
        lib.cast_rows(residual, rows)
        return rows, 0

    def forward(self, ctx, residual, pending, entry):
        if pending is not None:
            raise ValueError("outnorm: a delta of the block before is still pending; this "
                             "arrangement follows only blocks that add everything themselves")
        x, index = self._stream_rows(ctx, residual)
        a = self.mixer.forward(ctx, x, entry)
        if self.narrow:
            ctx.release(x)
        x = self.norm1.norm_add(ctx, residual, a, f"outnorm.x{1 - index}" if self.narrow else None)
        ctx.release(a)
        index = 1 - index
        if self.ffn is not None:
            f = self.ffn.forward(ctx, residual if x is None else x)
            if self.narrow:
                ctx.release(x)
            x = self.norm2.norm_add(ctx, residual, f,
                                    f"outnorm.x{1 - index}" if self.narrow else None)
            ctx.release(f)
            index = 1 - index
        if self.narrow:
            ctx.notes[self.CAST_NOTE] = (x, index)
        return None


class SandwichBlock:
    """x += s * norm1b(mixer(norm1(x))); x += s * norm2b(feed_forward(norm2(x))): a norm before
    and a norm after every sublayer, and a multiplier s (`residual_scale`) on what is added.  A
    layer may have no feed-forward (then it has no second pair of norms either).

    Options of the layer spec: `layer_scale`: what a sublayer adds is also multiplied, element
    by element, by a learned vector (`scale1` for the mixer, `scale2` for the feed-forward);
    `input_conv` T > 0: what a sublayer reads, h = norm(x), becomes h + conv(h), a causal
    convolution over time on every channel with a learned filter [width, T] (`conv1.weight`,
    `conv2.weight`); the last T - 1 inputs of both sublayers are state of the sequence, which
    the block keeps under the run's own cache id (`own_cache_request`), so a prompt may come
    whole, in portions or token by token.

    The multipliers are folded into the float32 weights (and biases) of the norms on the
    outputs when the block is built.  The norm on the mixer's output, the addition and the feed-forward's input
    norm are one kernel; everything is added when the block returns, so it returns no pending
    delta and follows only blocks that do the same."""

    capture_safe = True      # nothing of its own besides its parts' kernels

    def members(self):
        return tuple(part for part in (self.norm1, self.mixer, self.norm1b, self.norm2, self.ffn,
                                       self.norm2b) if part is not None)

    @classmethod
    def _owners(cls, layer_spec):
        norm_cls = lookup("norm", layer_spec.norm.kind)
        owners = [("norm1", norm_cls, layer_spec.norm),
                  ("mixer", lookup("mixer", layer_spec.mixer.kind), layer_spec.mixer),
                  ("norm1b", norm_cls, layer_spec.norm)]
        if layer_spec.feed_forward is not None:
            owners += [("norm2", norm_cls, layer_spec.norm),
                       ("ffn", lookup("feed_forward", layer_spec.feed_forward.kind),
                        layer_spec.feed_forward),
                       ("norm2b", norm_cls, layer_spec.norm)]
        return owners

    @classmethod
    def parameters(cls, layer_spec, hidden):
        params = {}
        for prefix, owner, spec in cls._owners(layer_spec):
            for name, param in owner.parameters(spec, hidden).items():
                params[f"{prefix}.{name}"] = param
        if layer_spec.feed_forward is None:
            # a checkpoint may still hold the second pair of norms of a layer without a
            # feed-forward; they are taken and have no use
            norm_cls = lookup("norm", layer_spec.norm.kind)
            for prefix in ("norm2", "norm2b"):
                for name, param in norm_cls.parameters(layer_spec.norm, hidden).items():
                    params[f"{prefix}.{name}"] = ParamSpec(param.shape, init=param.init,
                                                           optional=True)
        both = layer_spec.feed_forward is not None
        if getattr(layer_spec, "layer_scale", False):
            params["scale1"] = ParamSpec((hidden,), init="uniform", low=0.5, high=1.5)
            params["scale2"] = ParamSpec((hidden,), init="uniform", low=0.5, high=1.5,
                                         optional=not both)
        taps = getattr(layer_spec, "input_conv", 0)
        if taps:
            params["conv1.weight"] = ParamSpec((hidden, taps), scale=0.3)
            params["conv2.weight"] = ParamSpec((hidden, taps), scale=0.3, optional=not both)
        return params

    CONV_STATE = "input_conv"      # the name of the block's state under the run's own cache id

    @classmethod
    def own_cache_request(cls, layer_spec):
        """What a run of this layer keeps for itself, whichever cache entry its mixer uses:
        the last taps - 1 inputs of both convolutions, [2, taps - 1, width] floats a sequence
        (two versions: a step reads one and writes the other)."""
        taps = getattr(layer_spec, "input_conv", 0)
        if taps <= 1:
            return None
        return {cls.CONV_STATE: StateRequest(shape=(2 * (taps - 1) * cls._width_of(layer_spec),),
                                             two_versions=True)}

    @staticmethod
    def _width_of(layer_spec):
        width = getattr(layer_spec, "width", None)
        if width is None:
            raise ValueError("sandwich: a layer with an input convolution must name the model's "
                             "width (LayerSpec.width)")
        return int(width)

    @classmethod
    def mixer_spec(cls, layer_spec):
        return layer_spec.mixer

    @classmethod
    def kernel_libraries(cls, layer_spec, dtype):
        names = ["rowwise"]
        if getattr(layer_spec, "input_conv", 0):
            names.append("input_conv")
        for _, owner, spec in cls._owners(layer_spec):
            ask = getattr(owner, "kernel_libraries", None)
            if ask is not None:
                names.extend(ask(spec, dtype))
        return tuple(names)

    def __init__(self, layer_spec, hidden, params, dtype, device, positions):
        def sub(prefix):
            return {name[len(prefix) + 1:]: tensor for name, tensor in params.items()
                    if name.startswith(prefix + ".")}
        norm_cls = lookup("norm", layer_spec.norm.kind)
        if not hasattr(norm_cls, "norm_add"):
            raise ValueError(f"norm kind '{layer_spec.norm.kind}' cannot sit on a sublayer's output")
        scale = float(layer_spec.residual_scale)
        layer_scale = getattr(layer_spec, "layer_scale", False)

        def after(prefix, vector_name):
            """The norm on a sublayer's output, with the multipliers in its weight."""
            norm = norm_cls(layer_spec.norm, hidden, sub(prefix), dtype, device)
            factor = None if scale == 1.0 else scale
            if layer_scale:
                vector = params[vector_name].to(device=device, dtype=torch.float32)
                factor = vector if factor is None else vector * factor
            if factor is not None:
                if hasattr(norm, "scale_by"):
                    norm.scale_by(factor)
                else:
                    norm.weight = (norm.weight * factor).contiguous()
            return norm
        self.norm1 = norm_cls(layer_spec.norm, hidden, sub("norm1"), dtype, device)
        self.mixer = lookup("mixer", layer_spec.mixer.kind)(
            layer_spec.mixer, hidden, sub("mixer"), dtype, device, positions=positions)
        self.norm1b = after("norm1b", "scale1")
        self.norm2 = self.ffn = self.norm2b = None
        if layer_spec.feed_forward is not None:
            self.norm2 = norm_cls(layer_spec.norm, hidden, sub("norm2"), dtype, device)
            self.ffn = lookup("feed_forward", layer_spec.feed_forward.kind)(
                layer_spec.feed_forward, hidden, sub("ffn"), dtype, device)
            self.norm2b = after("norm2b", "scale2")
        # one kernel for the norm on the mixer's output, the addition and the next norm: two
        # plain RMS norms of one eps, or norms that bring such a kernel themselves
        self.fused = all(hasattr(norm, "weight") and hasattr(norm, "eps")
                         and not getattr(norm, "centred", False)
                         for norm in (self.norm1b, self.norm2) if norm is not None)
        self.fused_own = (self.norm2 is not None and hasattr(self.norm1b, "norm_add_then")
                          and type(self.norm1b) is type(self.norm2))
        self.hidden = hidden
        self.taps = int(getattr(layer_spec, "input_conv", 0))
        self.conv1 = self.conv2 = None
        if self.taps:
            # (kept tap by tap, [taps, width]: neighbouring channels' weights are neighbours)
            self.conv1 = params["conv1.weight"].to(device=device, dtype=torch.float32).t().contiguous()
            if self.ffn is not None:
                self.conv2 = params["conv2.weight"].to(device=device, dtype=torch.float32).t().contiguous()

    def _conv_in_norm(self, ctx, entry, part, norm):
        """What the norm kernel needs to take the convolution of sublayer `part` in itself, or
        None where it cannot: in a step whose sequences bring one token each, a row's taps are
        its own sequence's state, so the norm that makes the row can add them."""
        widths = getattr(norm, "conv_widths", 0)
        if not (self.taps and ctx.decode and widths and self.hidden % widths == 0):
            return None
        state = seq_in = seq_out = None
        if self.taps > 1:
            state = ctx.cache.state((entry.own_id, self.CONV_STATE))
            seq_in, seq_out = ctx.meta.seq_state_in, ctx.meta.seq_state_out
        return (self.conv1 if part == 0 else self.conv2, state, part, 2, seq_in, seq_out)

    def _convolved(self, ctx, h, entry, part):
        """h + conv(h) for sublayer `part` (0: the mixer, 1: the feed-forward)."""
        meta = ctx.meta
        out = ctx.buffer("block.hc", tuple(h.shape))
        state = seq_in = seq_out = None
        if self.taps > 1:
            state = ctx.cache.state((entry.own_id, self.CONV_STATE))
            seq_in, seq_out = meta.seq_state_in, meta.seq_state_out
        lib.input_conv(h, self.conv1 if part == 0 else self.conv2, state, part, 2, meta.row_pos,
                       meta.row_seq, seq_in, seq_out, meta.seq_start, meta.seq_count,
                       meta.seq_row0, out)
        ctx.release(h)
        return out

    def forward(self, ctx, residual, pending, entry):
        if pending is not None:
            raise ValueError("sandwich: a delta of the block before is still pending; this "
                             "arrangement follows only blocks that add everything themselves")
        conv = self._conv_in_norm(ctx, entry, 0, self.norm1)
        h = self.norm1.add_norm(ctx, residual, None, "block.h", write_residual=False,
                                **({} if conv is None else {"conv": conv}))
        if self.taps and conv is None:
            h = self._convolved(ctx, h, entry, 0)
        # a sublayer that can leave its last product's bias to the norm kernel behind it does
        a, a_bias = (self.mixer.forward(ctx, h, entry, bias_later=True)
                     if getattr(self.mixer, "bias_later", False)
                     else (self.mixer.forward(ctx, h, entry), None))
        ctx.release(h)
        if self.ffn is None:
            self.norm1b.norm_add(ctx, residual, a, bias=a_bias)
            ctx.release(a)
            return None
        conv = None
        if self.fused:
            h2 = ctx.buffer("block.h", tuple(residual.shape))
            lib.norm_add_norm(residual, a, self.norm1b.weight, self.norm2.weight, self.norm2.eps, h2,
                              bias=a_bias)
        else:
            conv = self._conv_in_norm(ctx, entry, 1, self.norm2)
            more = {} if conv is None else {"conv": conv}
            if self.fused_own:
                h2 = self.norm1b.norm_add_then(ctx, residual, a, self.norm2, "block.h", bias=a_bias,
                                               **more)
            else:
                self.norm1b.norm_add(ctx, residual, a, bias=a_bias)
                h2 = self.norm2.add_norm(ctx, residual, None, "block.h", write_residual=False,
                                         **more)
        ctx.release(a)
        if self.taps and conv is None:
            h2 = self._convolved(ctx, h2, entry, 1)
        f, f_bias = (self.ffn.forward(ctx, h2, bias_later=True)
                     if getattr(self.ffn, "bias_later", False)
                     else (self.ffn.forward(ctx, h2), None))
        ctx.release(h2)
        self.norm2b.norm_add(ctx, residual, f, bias=f_bias)
        ctx.release(f)
        return None
