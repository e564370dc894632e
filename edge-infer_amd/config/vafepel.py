"""Typed configuration of the Vafepel decoder, read from config.json keys.

A Vafepel model is a list of pre-norm layers, x += mixer(norm1(x)); x += ff(norm2(x)), each
with a mixer of its own kind and sizes and an optional feed-forward that is dense or a mixture
of experts.  The embedding rows pass an RMS norm; the head is the embedding table, and its
logits are multiplied by `logit_scale` and capped by `logit_softcap`.  config.json:

    architecture    "Vafepel"
    vocab, width    sizes of the table and of the stream
    norm.eps        eps of every RMS norm
    logit_scale     multiplier of the logits (absent: 1)
    logit_softcap   c: logits <- c tanh(logits / c) (absent or null: no cap)
    layers[i]       type     "attention" | "mamba2"
                    mixer    attention: heads, kv_heads, dim, vdim, scale, mask {size} (absent:
                                        every earlier position), rot {base, dims, scaling {factor,
                                        low, high, original}} (rot absent: no rotation; scaling
                                        absent: plain frequencies), v_mix
                             mamba2:    heads, vdim, state, groups, conv, norm_groups
                    mlp      null, or {kind: "dense", ff, limit},
                             or {kind: "moe", expert {ff}, router {experts, top}}

Mixers: `attention` is grouped-query attention with a per-head RMS norm of queries and keys, a
rotation of the first rot.dims elements of every head, a sliding window, a learned sink per
head in the softmax's denominator, values mixed with those of the first value-mixing layer,
and a sigmoid gate on the concatenated heads (`parts.attention.Attention` with those options);
`mamba2` is the state-space mixer `parts.ssm.StateSpace`.  Checkpoint names: `embed`,
`embed.norm`, `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.*`, `l<i>.mlp.*`, `final.norm`.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .specs import (AttentionSpec, FrequencyScaling, GatedMLPSpec, LayerSpec, ModelSpec, NormSpec,
                    PositionSpec, RoutedMLPSpec, StateSpaceSpec, default_schedule)

ARCHITECTURE = "Vafepel"
# constants the design fixes
SWISH_ALPHA = 1.702            # of the dense feed-forward's gate: g sigmoid(1.702 g)
MAX_POSITIONS = 1 << 30        # no table of positions: a sequence is as long as the cache allows


class VafepelConfigError(ValueError):
    pass


def _int(source: Mapping[str, Any], key: str, where: str, least: int = 1) -> int:
    if key not in source:
        raise VafepelConfigError(f"config.json: {where} lacks '{key}'")
    value = source[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) or int(value) != value \
            or value < least or value > 2**31 - 1:
        raise VafepelConfigError(f"config.json: {where}.{key} must be an integer of at least "
                                 f"{least}, got {value!r}")
    return int(value)


def _number(source: Mapping[str, Any], key: str, where: str) -> float:
    if key not in source:
        raise VafepelConfigError(f"config.json: {where} lacks '{key}'")
    value = source[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(value) \
            or value <= 0:
        raise VafepelConfigError(f"config.json: {where}.{key} must be a positive number, "
                                 f"got {value!r}")
    return float(value)


def _object(source: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    value = source.get(key)
    if not isinstance(value, dict):
        raise VafepelConfigError(f"config.json: {where} lacks the object '{key}'")
    return value


def _optional_object(source, key, where):
    value = source.get(key)
    if value is not None and not isinstance(value, dict):
        raise VafepelConfigError(f"config.json: {where}.{key} must be an object")
    return value


def _known_keys(source: Mapping[str, Any], known, where: str) -> None:
    """Options this decoder does not implement are refused, never ignored."""
    extra = sorted(set(source) - set(known))
    if extra:
        raise VafepelConfigError(f"config.json: {where} has keys this decoder does not know: {extra}")


@dataclass(frozen=True)
class VafepelAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]                    # mask.size; None: every earlier position
    rot_base: Optional[float]                # None: no rotation
    rot_dims: int
    rot_scaling: Optional[Tuple[float, float, float, float]]    # factor, low, high, original
    v_mix: bool

    type = "attention"

    @classmethod
    def from_dict(cls, source, where):
        _known_keys(source, ("heads", "kv_heads", "dim", "vdim", "scale", "mask", "rot", "v_mix"),
                    where)
        window = None
        mask = _optional_object(source, "mask", where)
        if mask is not None:
            _known_keys(mask, ("size",), where + ".mask")
            if mask.get("size") is not None:          # (a mask without a size masks nothing)
                window = _int(mask, "size", where + ".mask")
        rot = _optional_object(source, "rot", where)
        base, dims, scaling = None, 0, None
        if rot is not None:
            _known_keys(rot, ("base", "dims", "scaling"), where + ".rot")
            base = _number(rot, "base", where + ".rot")
            dims = _int(rot, "dims", where + ".rot", least=2)
            stretch = _optional_object(rot, "scaling", where + ".rot")
            if stretch is not None:
                _known_keys(stretch, ("factor", "low", "high", "original"), where + ".rot.scaling")
                scaling = tuple(_number(stretch, key, where + ".rot.scaling")
                                for key in ("factor", "low", "high", "original"))
                if scaling[2] <= scaling[1]:
                    raise VafepelConfigError(f"config.json: {where}.rot.scaling.high must be "
                                             "above low")
        v_mix = source.get("v_mix", False)
        if not isinstance(v_mix, bool):
            raise VafepelConfigError(f"config.json: {where}.v_mix must be true or false")
        mixer = cls(heads=_int(source, "heads", where), kv_heads=_int(source, "kv_heads", where),
                    dim=_int(source, "dim", where), vdim=_int(source, "vdim", where),
                    scale=_number(source, "scale", where), window=window, rot_base=base,
                    rot_dims=dims, rot_scaling=scaling, v_mix=v_mix)
        if mixer.heads % mixer.kv_heads:
            raise VafepelConfigError(f"config.json: {where}.heads must be a multiple of kv_heads")
        if mixer.rot_dims % 2 or mixer.rot_dims > mixer.dim:
            raise VafepelConfigError(f"config.json: {where}.rot.dims must be even and at most dim")
        return mixer

    def to_dict(self):
        out = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
               "scale": self.scale, "v_mix": self.v_mix, "vdim": self.vdim}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        if self.rot_base is not None:
            out["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_scaling is not None:
                out["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"),
                                                 self.rot_scaling))
        return out


@dataclass(frozen=True)
class VafepelStateSpace:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    type = "mamba2"

    @classmethod
    def from_dict(cls, source, where):
        _known_keys(source, ("heads", "vdim", "state", "groups", "conv", "norm_groups"), where)
        mixer = cls(heads=_int(source, "heads", where), vdim=_int(source, "vdim", where),
                    state=_int(source, "state", where), groups=_int(source, "groups", where),
                    conv=_int(source, "conv", where),
                    norm_groups=_int(source, "norm_groups", where))
        if mixer.heads % mixer.groups:
            raise VafepelConfigError(f"config.json: {where}.heads must be a multiple of groups")
        if (mixer.heads * mixer.vdim) % mixer.norm_groups:
            raise VafepelConfigError(f"config.json: {where}.norm_groups must divide heads * vdim")
        return mixer

    def to_dict(self):
        return {"conv": self.conv, "groups": self.groups, "heads": self.heads,
                "norm_groups": self.norm_groups, "state": self.state, "vdim": self.vdim}


MIXERS = {"attention": VafepelAttention, "mamba2": VafepelStateSpace}


@dataclass(frozen=True)
class VafepelDense:
    ff: int
    limit: float

    kind = "dense"

    def to_dict(self):
        return {"ff": self.ff, "kind": "dense", "limit": self.limit}


@dataclass(frozen=True)
class VafepelExperts:
    ff: int
    experts: int
    top: int

    kind = "moe"

    def to_dict(self):
        return {"expert": {"ff": self.ff}, "kind": "moe",
                "router": {"experts": self.experts, "top": self.top}}


def _feed_forward(mlp, where):
    if mlp is None:
        return None
    if not isinstance(mlp, dict):
        raise VafepelConfigError(f"config.json: {where} must be an object or null")
    kind = mlp.get("kind")
    if kind == "dense":
        _known_keys(mlp, ("kind", "ff", "limit"), where)
        return VafepelDense(ff=_int(mlp, "ff", where), limit=_number(mlp, "limit", where))
    if kind == "moe":
        _known_keys(mlp, ("kind", "expert", "router"), where)
        expert = _object(mlp, "expert", where)
        router = _object(mlp, "router", where)
        _known_keys(expert, ("ff",), where + ".expert")
        _known_keys(router, ("experts", "top"), where + ".router")
        made = VafepelExperts(ff=_int(expert, "ff", where + ".expert"),
                              experts=_int(router, "experts", where + ".router"),
                              top=_int(router, "top", where + ".router"))
        if made.top > made.experts:
            raise VafepelConfigError(f"config.json: {where}.router.top is above its experts")
        return made
    raise VafepelConfigError(f"config.json: {where}.kind must be 'dense' or 'moe', got {kind!r}")


@dataclass(frozen=True)
class VafepelLayer:
    mixer: object                # one of the two mixer configurations
    mlp: object                  # VafepelDense, VafepelExperts or None

    @classmethod
    def from_dict(cls, source, where):
        if not isinstance(source, dict):
            raise VafepelConfigError(f"config.json: {where} must be an object")
        _known_keys(source, ("type", "mixer", "mlp"), where)
        kind = source.get("type")
        if kind not in MIXERS:
            raise VafepelConfigError(f"config.json: {where}.type must be one of {sorted(MIXERS)}, "
                                     f"got {kind!r}")
        mixer = MIXERS[kind].from_dict(_object(source, "mixer", where), where + ".mixer")
        return cls(mixer=mixer, mlp=_feed_forward(source.get("mlp"), where + ".mlp"))

    def to_dict(self):
        return {"mixer": self.mixer.to_dict(),
                "mlp": None if self.mlp is None else self.mlp.to_dict(),
                "type": self.mixer.type}


@dataclass(frozen=True)
class VafepelConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[VafepelLayer, ...]
    logit_scale: float = 1.0
    logit_softcap: Optional[float] = None

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "VafepelConfig":
        # (keys of the top level that the decoder does not know are a file's own notes; inside
        # a layer an unknown key would change what is computed, and is refused)
        norm = _object(source, "norm", "the top level")
        _known_keys(norm, ("eps",), "norm")
        layers = source.get("layers")
        if not isinstance(layers, list) or not layers:
            raise VafepelConfigError("config.json: 'layers' must be a list of at least one layer")
        config = cls(vocab=_int(source, "vocab", "the top level"),
                     width=_int(source, "width", "the top level"),
                     norm_eps=_number(norm, "eps", "norm"),
                     layers=tuple(VafepelLayer.from_dict(layer, f"layers[{index}]")
                                  for index, layer in enumerate(layers)),
                     logit_scale=(1.0 if source.get("logit_scale") is None
                                  else _number(source, "logit_scale", "the top level")),
                     logit_softcap=(None if source.get("logit_softcap") in (None, 0, 0.0, False)
                                    else _number(source, "logit_softcap", "the top level")))
        widths = {layer.mixer.kv_heads * layer.mixer.vdim for layer in config.layers
                  if isinstance(layer.mixer, VafepelAttention) and layer.mixer.v_mix}
        if len(widths) > 1:
            raise VafepelConfigError("config.json: layers that mix values must have values of one "
                                     f"width, got {sorted(widths)}")
        return config

    def to_dict(self) -> dict:
        """config.json content that `from_dict` reads back to an equal object."""
        return {"architecture": ARCHITECTURE, "layers": [layer.to_dict() for layer in self.layers],
                "logit_scale": self.logit_scale, "logit_softcap": self.logit_softcap,
                "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}

    # ------------------------------------------------------------------
    def _mixer_spec(self, mixer, value_mix):
        if isinstance(mixer, VafepelStateSpace):
            return StateSpaceSpec(n_heads=mixer.heads, head_dim=mixer.vdim, state=mixer.state,
                                  groups=mixer.groups, conv_taps=mixer.conv,
                                  norm_parts=mixer.norm_groups, norm_eps=self.norm_eps)
        if mixer.rot_base is None:
            position = PositionSpec(kind="none")
        else:
            scaling = None if mixer.rot_scaling is None else FrequencyScaling(*mixer.rot_scaling)
            position = PositionSpec(kind="rope_half", theta=mixer.rot_base, dim=mixer.rot_dims,
                                    scaling=scaling)
        return AttentionSpec(n_heads=mixer.heads, n_kv_heads=mixer.kv_heads, head_dim=mixer.dim,
                             value_dim=mixer.vdim, qk_norm=True, qk_norm_eps=self.norm_eps,
                             qkv_bias=False, o_bias=False, scale=mixer.scale, window=mixer.window,
                             sink=True, position=position, value_mix=value_mix, output_gate=True)

    def _feed_forward_spec(self, mlp):
        if mlp is None:
            return None
        if isinstance(mlp, VafepelDense):
            return GatedMLPSpec(intermediate_size=mlp.ff, activation="clamped_swish", bias=False,
                                limit=mlp.limit, alpha=SWISH_ALPHA)
        return RoutedMLPSpec(n_experts=mlp.experts, top=mlp.top, intermediate_size=mlp.ff)

    def model_spec(self) -> ModelSpec:
        norm = NormSpec(kind="rmsnorm", eps=self.norm_eps)
        layers, source_seen = [], False
        for layer in self.layers:
            value_mix = None
            if isinstance(layer.mixer, VafepelAttention):
                # the first layer that mixes values is the source of the others; a layer that
                # mixes nothing may still hold the weight, which then has no use
                value_mix = "off"
                if layer.mixer.v_mix:
                    value_mix = "mix" if source_seen else "source"
                    source_seen = True
            layers.append(LayerSpec(block="prenorm", norm=norm,
                                    mixer=self._mixer_spec(layer.mixer, value_mix),
                                    feed_forward=self._feed_forward_spec(layer.mlp)))
        spec = ModelSpec(architecture=ARCHITECTURE, vocab_size=self.vocab, hidden_size=self.width,
                         layers=tuple(layers), schedule=default_schedule(len(layers)),
                         final_norm=norm, tie_word_embeddings=True,
                         max_position_embeddings=MAX_POSITIONS, bos_token_id=None,
                         eos_token_id=None, embedding_norm=norm, logit_scale=self.logit_scale,
                         logit_softcap=self.logit_softcap)
        spec.validate()
        return spec

    # ------------------------------------------------------------------
    _MIXER_NAMES = {
        "attention": {
            "q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v",
            "q_norm.weight": "q.norm", "k_norm.weight": "k.norm", "sink": "sink",
            "value_mix": "vmix", "gate_proj.weight": "g", "o_proj.weight": "o",
        },
        "mamba2": {
            "in_proj.weight": "in", "conv.weight": "conv", "conv.bias": "conv.b",
            "dt_bias": "dt_bias", "a_log": "A_log", "skip": "D", "out_norm.weight": "norm",
            "o_proj.weight": "o",
        },
    }
    _DENSE_NAMES = {"gate_proj.weight": "gate", "up_proj.weight": "up", "down_proj.weight": "down"}

    def checkpoint_name(self, parameter: str) -> str:
        """Name of a model parameter in the checkpoint."""
        top = {"embed.weight": "embed", "embed_norm.weight": "embed.norm",
               "final_norm.weight": "final.norm", "head.weight": "head", "head.bias": "head.b"}
        if parameter in top:
            return top[parameter]
        parts = parameter.split(".", 3)
        if parts[0] == "layers" and len(parts) == 4 and parts[1].isdigit() \
                and int(parts[1]) < len(self.layers):
            index, part, rest = int(parts[1]), parts[2], parts[3]
            if part in ("norm1", "norm2") and rest == "weight":
                return f"l{index}.{part}"
            if part == "mixer":
                table = self._MIXER_NAMES[self.layers[index].mixer.type]
                if rest in table:
                    return f"l{index}.mix.{table[rest]}"
            if part == "ffn":
                if rest in self._DENSE_NAMES:
                    return f"l{index}.mlp.{self._DENSE_NAMES[rest]}"
                if rest == "router.weight":
                    return f"l{index}.mlp.router"
                pieces = rest.split(".")        # experts.<e>.<gate|up|down>_proj.weight
                if len(pieces) == 4 and pieces[0] == "experts" and pieces[1].isdigit() \
                        and ".".join(pieces[2:]) in self._DENSE_NAMES:
                    return f"l{index}.mlp.e{pieces[1]}.{self._DENSE_NAMES['.'.join(pieces[2:])]}"
        raise KeyError(f"Vafepel has no checkpoint tensor for parameter '{parameter}'")
