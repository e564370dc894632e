"""Arrangements of norm, mixer and feed-forward in one layer."""
from __future__ import annotations

import torch

from ..csrc import lib
from ..weights.loader import ParamSpec
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

    The multiplier is folded into the float32 weights of the norms on the outputs when the
    block is built.  The norm on the mixer's output, the addition and the feed-forward's input
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
        scale = float(layer_spec.residual_scale)

        def after(prefix):
            """The norm on a sublayer's output, with the multiplier in its weight."""
            norm = norm_cls(layer_spec.norm, hidden, sub(prefix), dtype, device)
            if scale != 1.0:
                norm.weight = (norm.weight * scale).contiguous()
            return norm
        self.norm1 = norm_cls(layer_spec.norm, hidden, sub("norm1"), dtype, device)
        self.mixer = lookup("mixer", layer_spec.mixer.kind)(
            layer_spec.mixer, hidden, sub("mixer"), dtype, device, positions=positions)
        self.norm1b = after("norm1b")
        self.norm2 = self.ffn = self.norm2b = None
        if layer_spec.feed_forward is not None:
            self.norm2 = norm_cls(layer_spec.norm, hidden, sub("norm2"), dtype, device)
            self.ffn = lookup("feed_forward", layer_spec.feed_forward.kind)(
                layer_spec.feed_forward, hidden, sub("ffn"), dtype, device)
            self.norm2b = after("norm2b")
        # the fused kernel takes two plain RMS norms of one eps
        self.fused = all(hasattr(norm, "weight") and hasattr(norm, "eps")
                         for norm in (self.norm1b, self.norm2) if norm is not None)

    def forward(self, ctx, residual, pending, entry):
        if pending is not None:
            raise ValueError("sandwich: a delta of the block before is still pending; this "
                             "arrangement follows only blocks that add everything themselves")
        h = self.norm1.add_norm(ctx, residual, None, "block.h", write_residual=False)
        # a sublayer that can leave its last product's bias to the norm kernel behind it does
        a, a_bias = (self.mixer.forward(ctx, h, entry, bias_later=True)
                     if getattr(self.mixer, "bias_later", False)
                     else (self.mixer.forward(ctx, h, entry), None))
        ctx.release(h)
        if self.ffn is None:
            self.norm1b.norm_add(ctx, residual, a, bias=a_bias)
            ctx.release(a)
            return None
        if self.fused:
            h2 = ctx.buffer("block.h", tuple(residual.shape))
            lib.norm_add_norm(residual, a, self.norm1b.weight, self.norm2.weight, self.norm2.eps, h2,
                              bias=a_bias)
        else:
            self.norm1b.norm_add(ctx, residual, a, bias=a_bias)
            h2 = self.norm2.add_norm(ctx, residual, None, "block.h", write_residual=False)
        ctx.release(a)
        f, f_bias = (self.ffn.forward(ctx, h2, bias_later=True)
                     if getattr(self.ffn, "bias_later", False)
                     else (self.ffn.forward(ctx, h2), None))
        ctx.release(h2)
        self.norm2b.norm_add(ctx, residual, f, bias=f_bias)
        ctx.release(f)
        return None
