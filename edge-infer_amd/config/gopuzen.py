"""Typed configuration of the Gopuzen decoder, read from config.json keys.

A Gopuzen model is a list of layers with a layer norm (weight and bias) before and after
every sublayer, x += ls1 * norm1b(mixer(c1(norm1(x)))); x += ls2 * norm2b(ff(c2(norm2(x)))):
ls1 and ls2 are learned vectors, c1 and c2 short causal convolutions over time that are added
to what they read, h + conv(h).  The embedding rows are multiplied by a constant; the model
ends with a layer norm and a head of its own.  config.json:

    architecture     "Gopuzen"
    vocab, width     sizes of the table and of the stream
    norm.eps         eps of every norm
    embedding.scale  multiplier of the embedding rows
    canon.taps       taps of the input convolutions
    layers[i]        type     "parallel" | "attention"
                     mixer    parallel:  left  {heads, kv_heads, dim, vdim, scale,
                                                q_temp {coef, every}}
                                         right {heads, dim, vdim, decay [heads]}
                              attention: heads, kv_heads, dim, vdim, scale, mask {size, pool},
                                         rot {base, dims}, kv_from
                     mlp      null, or {kind: "dense", ff},
                              or {kind: "moe", expert {ff}, router {experts, top, identity}}

Mixers: `parallel` is softmax attention without a rotation, whose queries grow with the
position (`parts.attention.Attention` with `query_temperature`), beside linear attention with
a fixed decay per head (`parts.linear_attention.LinearAttention`), joined by
`parts.parallel.ParallelMixer`; `attention` rotates neighbouring pairs of the first rot.dims
elements of a head, sees a window of tokens and the pooled blocks before it, gates every head,
and may read the keys and values of an earlier layer (`kv_from`).  Checkpoint names: `embed`,
`l<i>.norm1|norm1b|norm2|norm2b` (+ `.b`), `l<i>.ls1|ls2`, `l<i>.canon1|canon2`,
`l<i>.mix.*`, `l<i>.mlp.*`, `final.norm` (+ `.b`), `head`.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .specs import (AttentionSpec, GatedMLPSpec, LayerSpec, LinearAttentionSpec, ModelSpec,
                    NormSpec, ParallelSpec, PositionSpec, RoutedMLPSpec, ScheduleEntry)

ARCHITECTURE = "Gopuzen"
MAX_POSITIONS = 1 << 30        # no table of positions: a sequence is as long as the cache allows


class GopuzenConfigError(ValueError):
    pass


def _int(source: Mapping[str, Any], key: str, where: str, least: int = 1) -> int:
    if key not in source:
        raise GopuzenConfigError(f"config.json: {where} lacks '{key}'")
    value = source[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) or int(value) != value \
            or value < least or value > 2**31 - 1:
        raise GopuzenConfigError(f"config.json: {where}.{key} must be an integer of at least "
                                 f"{least}, got {value!r}")
    return int(value)


def _number(source: Mapping[str, Any], key: str, where: str, positive: bool = True) -> float:
    if key not in source:
        raise GopuzenConfigError(f"config.json: {where} lacks '{key}'")
    value = source[key]
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(value) \
            or (positive and value <= 0):
        raise GopuzenConfigError(f"config.json: {where}.{key} must be a "
                                 f"{'positive ' if positive else ''}number, got {value!r}")
    return float(value)


def _object(source: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    value = source.get(key)
    if not isinstance(value, dict):
        raise GopuzenConfigError(f"config.json: {where} lacks the object '{key}'")
    return value


def _optional_object(source, key, where):
    value = source.get(key)
    if value is not None and not isinstance(value, dict):
        raise GopuzenConfigError(f"config.json: {where}.{key} must be an object")
    return value


def _known_keys(source: Mapping[str, Any], known, where: str) -> None:
    """Options this decoder does not implement are refused, never ignored."""
    extra = sorted(set(source) - set(known))
    if extra:
        raise GopuzenConfigError(f"config.json: {where} has keys this decoder does not know: {extra}")


@dataclass(frozen=True)
class GopuzenSoftmax:
    """The softmax half of a parallel mixer."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    q_temp: Optional[Tuple[float, int]]          # (coef, every); None: queries as they are

    @classmethod
    def from_dict(cls, source, where):
        _known_keys(source, ("heads", "kv_heads", "dim", "vdim", "scale", "q_temp"), where)
        temp = _optional_object(source, "q_temp", where)
        q_temp = None
        if temp is not None:
            _known_keys(temp, ("coef", "every"), where + ".q_temp")
            q_temp = (_number(temp, "coef", where + ".q_temp", positive=False),
                      _int(temp, "every", where + ".q_temp"))
        made = cls(heads=_int(source, "heads", where), kv_heads=_int(source, "kv_heads", where),
                   dim=_int(source, "dim", where), vdim=_int(source, "vdim", where),
                   scale=_number(source, "scale", where), q_temp=q_temp)
        if made.heads % made.kv_heads:
            raise GopuzenConfigError(f"config.json: {where}.heads must be a multiple of kv_heads")
        return made

    def to_dict(self):
        out = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
               "scale": self.scale, "vdim": self.vdim}
        if self.q_temp is not None:
            out["q_temp"] = {"coef": self.q_temp[0], "every": self.q_temp[1]}
        return out


@dataclass(frozen=True)
class GopuzenLightning:
    """The linear-attention half of a parallel mixer."""
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    @classmethod
    def from_dict(cls, source, where):
        _known_keys(source, ("heads", "dim", "vdim", "decay"), where)
        heads = _int(source, "heads", where)
        decay = source.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or any(
                isinstance(d, bool) or not isinstance(d, (int, float)) or not math.isfinite(d)
                for d in decay):
            raise GopuzenConfigError(f"config.json: {where}.decay must be a list of {heads} numbers")
        return cls(heads=heads, dim=_int(source, "dim", where), vdim=_int(source, "vdim", where),
                   decay=tuple(float(d) for d in decay))

    def to_dict(self):
        return {"decay": list(self.decay), "dim": self.dim, "heads": self.heads, "vdim": self.vdim}


@dataclass(frozen=True)
class GopuzenParallel:
    left: GopuzenSoftmax
    right: GopuzenLightning

    type = "parallel"

    @classmethod
    def from_dict(cls, source, where):
        _known_keys(source, ("left", "right"), where)
        return cls(left=GopuzenSoftmax.from_dict(_object(source, "left", where), where + ".left"),
                   right=GopuzenLightning.from_dict(_object(source, "right", where),
                                                    where + ".right"))

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass(frozen=True)
class GopuzenAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]                    # mask.size; None: every earlier position
    pool: Optional[int]                      # mask.pool
    rot_base: Optional[float]                # None: no rotation
    rot_dims: int
    kv_from: Optional[int]                   # the layer whose keys and values this one reads

    type = "attention"

    @classmethod
    def from_dict(cls, source, where):
        _known_keys(source, ("heads", "kv_heads", "dim", "vdim", "scale", "mask", "rot", "kv_from"),
                    where)
        window = pool = None
        mask = _optional_object(source, "mask", where)
        if mask is not None:
            _known_keys(mask, ("size", "pool"), where + ".mask")
            window = _int(mask, "size", where + ".mask")
            if mask.get("pool") is not None:
                pool = _int(mask, "pool", where + ".mask")
        rot = _optional_object(source, "rot", where)
        base, dims = None, 0
        if rot is not None:
            _known_keys(rot, ("base", "dims"), where + ".rot")
            base = _number(rot, "base", where + ".rot")
            dims = _int(rot, "dims", where + ".rot", least=2)
        kv_from = None if source.get("kv_from") is None else _int(source, "kv_from", where, least=0)
        made = cls(heads=_int(source, "heads", where), kv_heads=_int(source, "kv_heads", where),
                   dim=_int(source, "dim", where), vdim=_int(source, "vdim", where),
                   scale=_number(source, "scale", where), window=window, pool=pool,
                   rot_base=base, rot_dims=dims, kv_from=kv_from)
        if made.heads % made.kv_heads:
            raise GopuzenConfigError(f"config.json: {where}.heads must be a multiple of kv_heads")
        if made.rot_dims % 2 or made.rot_dims > made.dim:
            raise GopuzenConfigError(f"config.json: {where}.rot.dims must be even and at most dim")
        return made

    def to_dict(self):
        out = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
               "scale": self.scale, "vdim": self.vdim}
        if self.window is not None:
            out["mask"] = {"size": self.window}
            if self.pool is not None:
                out["mask"]["pool"] = self.pool
        if self.rot_base is not None:
            out["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


MIXERS = {"parallel": GopuzenParallel, "attention": GopuzenAttention}


@dataclass(frozen=True)
class GopuzenDense:
    ff: int

    kind = "dense"

    def to_dict(self):
        return {"ff": self.ff, "kind": "dense"}


@dataclass(frozen=True)
class GopuzenExperts:
    ff: int
    experts: int
    top: int
    identity: int

    kind = "moe"

    def to_dict(self):
        return {"expert": {"ff": self.ff}, "kind": "moe",
                "router": {"experts": self.experts, "identity": self.identity, "top": self.top}}


def _feed_forward(mlp, where):
    if mlp is None:
        return None
    if not isinstance(mlp, dict):
        raise GopuzenConfigError(f"config.json: {where} must be an object or null")
    kind = mlp.get("kind")
    if kind == "dense":
        _known_keys(mlp, ("kind", "ff"), where)
        return GopuzenDense(ff=_int(mlp, "ff", where))
    if kind == "moe":
        _known_keys(mlp, ("kind", "expert", "router"), where)
        expert = _object(mlp, "expert", where)
        router = _object(mlp, "router", where)
        _known_keys(expert, ("ff",), where + ".expert")
        _known_keys(router, ("experts", "top", "identity"), where + ".router")
        made = GopuzenExperts(ff=_int(expert, "ff", where + ".expert"),
                              experts=_int(router, "experts", where + ".router"),
                              top=_int(router, "top", where + ".router"),
                              identity=(0 if router.get("identity") is None else
                                        _int(router, "identity", where + ".router", least=0)))
        if made.top > made.experts + made.identity:
            raise GopuzenConfigError(f"config.json: {where}.router.top is above its outputs")
        return made
    raise GopuzenConfigError(f"config.json: {where}.kind must be 'dense' or 'moe', got {kind!r}")


@dataclass(frozen=True)
class GopuzenLayer:
    mixer: object                # one of the two mixer configurations
    mlp: object                  # GopuzenDense, GopuzenExperts or None

    @classmethod
    def from_dict(cls, source, where):
        if not isinstance(source, dict):
            raise GopuzenConfigError(f"config.json: {where} must be an object")
        _known_keys(source, ("type", "mixer", "mlp"), where)
        kind = source.get("type")
        if kind not in MIXERS:
            raise GopuzenConfigError(f"config.json: {where}.type must be one of {sorted(MIXERS)}, "
                                     f"got {kind!r}")
        mixer = MIXERS[kind].from_dict(_object(source, "mixer", where), where + ".mixer")
        return cls(mixer=mixer, mlp=_feed_forward(source.get("mlp"), where + ".mlp"))

    def to_dict(self):
        return {"mixer": self.mixer.to_dict(),
                "mlp": None if self.mlp is None else self.mlp.to_dict(),
                "type": self.mixer.type}


@dataclass(frozen=True)
class GopuzenConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    canon_taps: int
    layers: Tuple[GopuzenLayer, ...]

    architecture = ARCHITECTURE

    @classmethod
    def from_dict(cls, source: Mapping[str, Any]) -> "GopuzenConfig":
        # (keys of the top level that the decoder does not know are a file's own notes; inside
        # a layer an unknown key would change what is computed, and is refused)
        norm = _object(source, "norm", "the top level")
        _known_keys(norm, ("eps",), "norm")
        embedding = _object(source, "embedding", "the top level")
        _known_keys(embedding, ("scale",), "embedding")
        canon = _object(source, "canon", "the top level")
        _known_keys(canon, ("taps",), "canon")
        layers = source.get("layers")
        if not isinstance(layers, list) or not layers:
            raise GopuzenConfigError("config.json: 'layers' must be a list of at least one layer")
        config = cls(vocab=_int(source, "vocab", "the top level"),
                     width=_int(source, "width", "the top level"),
                     norm_eps=_number(norm, "eps", "norm"),
                     embedding_scale=_number(embedding, "scale", "embedding", positive=False),
                     canon_taps=_int(canon, "taps", "canon"),
                     layers=tuple(GopuzenLayer.from_dict(layer, f"layers[{index}]")
                                  for index, layer in enumerate(layers)))
        for index, layer in enumerate(config.layers):
            mixer = layer.mixer
            source_index = getattr(mixer, "kv_from", None)
            if source_index is None:
                continue
            where = f"layers[{index}].mixer.kv_from"
            if source_index >= index:
                raise GopuzenConfigError(f"config.json: {where} must name an earlier layer")
            other = config.layers[source_index].mixer
            if not isinstance(other, GopuzenAttention) or other.kv_from is not None:
                raise GopuzenConfigError(f"config.json: {where} must name an attention layer "
                                         "with keys and values of its own")
            if (other.kv_heads, other.dim, other.vdim, other.rot_base, other.rot_dims) != \
                    (mixer.kv_heads, mixer.dim, mixer.vdim, mixer.rot_base, mixer.rot_dims):
                raise GopuzenConfigError(f"config.json: {where}: the two layers' key and value "
                                         "heads and rotations differ")
        return config

    def to_dict(self) -> dict:
        """config.json content that `from_dict` reads back to an equal object."""
        return {"architecture": ARCHITECTURE, "canon": {"taps": self.canon_taps},
                "embedding": {"scale": self.embedding_scale},
                "layers": [layer.to_dict() for layer in self.layers],
                "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}

    # ------------------------------------------------------------------
    def _cache_span(self, index: int) -> Optional[int]:
        """What layer `index`'s cache must keep for the layers that read it: None if its own
        mask says enough, 0 (everything) if a reader has no mask, else the widest need."""
        own = self.layers[index].mixer
        users = [own] + [layer.mixer for layer in self.layers
                         if getattr(layer.mixer, "kv_from", None) == index]
        if len(users) == 1:
            return None
        if any(user.window is None for user in users):
            return 0
        return max(max(user.window, user.pool or 1) for user in users)

    def _attention_spec(self, index: int, mixer: GopuzenAttention) -> AttentionSpec:
        position = PositionSpec(kind="none") if mixer.rot_base is None else \
            PositionSpec(kind="rope_pairs", theta=mixer.rot_base, dim=mixer.rot_dims)
        return AttentionSpec(n_heads=mixer.heads, n_kv_heads=mixer.kv_heads, head_dim=mixer.dim,
                             value_dim=mixer.vdim, qkv_bias=False, o_bias=False, scale=mixer.scale,
                             window=mixer.window, pool=mixer.pool, position=position,
                             output_gate="head", shared_kv=mixer.kv_from is not None,
                             cache_span=None if mixer.kv_from is not None
                             else self._cache_span(index))

    def _mixer_spec(self, index: int, mixer):
        if isinstance(mixer, GopuzenAttention):
            return self._attention_spec(index, mixer)
        left, right = mixer.left, mixer.right
        return ParallelSpec(
            branches=(AttentionSpec(n_heads=left.heads, n_kv_heads=left.kv_heads,
                                    head_dim=left.dim, value_dim=left.vdim, qkv_bias=False,
                                    o_bias=False, scale=left.scale,
                                    position=PositionSpec(kind="none"),
                                    query_temperature=left.q_temp),
                      LinearAttentionSpec(n_heads=right.heads, key_dim=right.dim,
                                          value_dim=right.vdim, decay=right.decay,
                                          norm_eps=self.norm_eps)),
            names=("left", "right"), norm_eps=self.norm_eps)

    def _feed_forward_spec(self, mlp):
        if mlp is None:
            return None
        if isinstance(mlp, GopuzenDense):
            return GatedMLPSpec(intermediate_size=mlp.ff, activation="silu", bias=True)
        return RoutedMLPSpec(n_experts=mlp.experts, top=mlp.top, intermediate_size=mlp.ff,
                             scoring="softmax_all", correction=True, identity=mlp.identity)

    def model_spec(self) -> ModelSpec:
        norm = NormSpec(kind="layernorm", eps=self.norm_eps)
        layers, schedule = [], []
        for index, layer in enumerate(self.layers):
            layers.append(LayerSpec(block="sandwich", norm=norm,
                                    mixer=self._mixer_spec(index, layer.mixer),
                                    feed_forward=self._feed_forward_spec(layer.mlp),
                                    layer_scale=True, input_conv=self.canon_taps,
                                    width=self.width))
            source = getattr(layer.mixer, "kv_from", None)
            schedule.append(ScheduleEntry(layer=index, cache=index) if source is None else
                            ScheduleEntry(layer=index, cache=source, writes_cache=False,
                                          own=index))
        spec = ModelSpec(architecture=ARCHITECTURE, vocab_size=self.vocab, hidden_size=self.width,
                         layers=tuple(layers), schedule=tuple(schedule), final_norm=norm,
                         tie_word_embeddings=False, max_position_embeddings=MAX_POSITIONS,
                         bos_token_id=None, eos_token_id=None,
                         embedding_scale=self.embedding_scale)
        spec.validate()
        return spec

    # ------------------------------------------------------------------
    _ATTENTION_NAMES = {"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v",
                        "gate_proj.weight": "g", "o_proj.weight": "o"}
    _LIGHTNING_NAMES = {"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v",
                        "gate_proj.weight": "g", "out_norm.weight": "norm", "o_proj.weight": "o"}
    _DENSE_NAMES = {"gate_proj.weight": "gate", "up_proj.weight": "up", "down_proj.weight": "down",
                    "gate_proj.bias": "gate.b", "up_proj.bias": "up.b", "down_proj.bias": "down.b"}
    _BLOCK_NAMES = {"scale1": "ls1", "scale2": "ls2", "conv1.weight": "canon1",
                    "conv2.weight": "canon2"}

    def checkpoint_name(self, parameter: str) -> str:
        """Name of a model parameter in the checkpoint."""
        top = {"embed.weight": "embed", "final_norm.weight": "final.norm",
               "final_norm.bias": "final.norm.b", "head.weight": "head", "head.bias": "head.b"}
        if parameter in top:
            return top[parameter]
        parts = parameter.split(".", 3)
        if parts[0] == "layers" and len(parts) >= 3 and parts[1].isdigit() \
                and int(parts[1]) < len(self.layers):
            index, part = int(parts[1]), parts[2]
            rest = parts[3] if len(parts) == 4 else ""
            tail = ".".join(parts[2:])
            if tail in self._BLOCK_NAMES:
                return f"l{index}.{self._BLOCK_NAMES[tail]}"
            if part in ("norm1", "norm1b", "norm2", "norm2b") and rest in ("weight", "bias"):
                return f"l{index}.{part}" + ("" if rest == "weight" else ".b")
            if part == "mixer":
                if isinstance(self.layers[index].mixer, GopuzenAttention):
                    if rest in self._ATTENTION_NAMES:
                        return f"l{index}.mix.{self._ATTENTION_NAMES[rest]}"
                else:
                    side, _, inner = rest.partition(".")
                    if side in ("left_out", "right_out") and inner == "weight":
                        return f"l{index}.mix.{side[:-4]}.out"
                    table = {"left": self._ATTENTION_NAMES, "right": self._LIGHTNING_NAMES}.get(side)
                    if table is not None and inner in table:
                        return f"l{index}.mix.{side}.{table[inner]}"
            if part == "ffn":
                if rest in self._DENSE_NAMES:
                    return f"l{index}.mlp.{self._DENSE_NAMES[rest]}"
                if rest == "router.weight":
                    return f"l{index}.mlp.router"
                if rest == "router.correction":
                    return f"l{index}.mlp.correction"
                pieces = rest.split(".")        # experts.<e>.<gate|up|down>_proj.weight
                if len(pieces) == 4 and pieces[0] == "experts" and pieces[1].isdigit() \
                        and ".".join(pieces[2:]) in self._DENSE_NAMES:
                    return f"l{index}.mlp.e{pieces[1]}.{self._DENSE_NAMES['.'.join(pieces[2:])]}"
        raise KeyError(f"Gopuzen has no checkpoint tensor for parameter '{parameter}'")
