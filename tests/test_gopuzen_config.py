"""The Gopuzen configuration: what config.json gives, the spec it becomes, the checkpoint's
names, what is refused and what may be absent (no GPU)."""
import copy

import pytest

from gopuzen_helpers import CONFIGS, tensor_shapes


def config_of(raw):
    from edge_infer_amd.config import GopuzenConfig
    return GopuzenConfig.from_dict(raw)


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_round_trip_and_spec(name):
    from edge_infer_amd.config.specs import (AttentionSpec, GatedMLPSpec, LinearAttentionSpec,
                                             ParallelSpec, RoutedMLPSpec)
    raw = CONFIGS[name]
    cfg = config_of(raw)
    assert config_of(cfg.to_dict()) == cfg
    spec = cfg.model_spec()
    assert spec.embedding_scale == raw["embedding"]["scale"] and not spec.tie_word_embeddings
    assert spec.final_norm.kind == "layernorm" and spec.final_norm.eps == raw["norm"]["eps"]
    for index, (layer, made) in enumerate(zip(raw["layers"], spec.layers)):
        assert made.block == "sandwich" and made.layer_scale and made.norm.kind == "layernorm"
        assert made.input_conv == raw["canon"]["taps"] and made.width == raw["width"]
        mixer = layer["mixer"]
        if layer["type"] == "parallel":
            assert isinstance(made.mixer, ParallelSpec) and made.mixer.names == ("left", "right")
            left, right = made.mixer.branches
            assert isinstance(left, AttentionSpec) and isinstance(right, LinearAttentionSpec)
            assert (left.n_heads, left.n_kv_heads, left.head_dim, left.v_dim, left.scale) == \
                tuple(mixer["left"][k] for k in ("heads", "kv_heads", "dim", "vdim", "scale"))
            temp = mixer["left"].get("q_temp")
            assert left.query_temperature == (None if temp is None else (temp["coef"], temp["every"]))
            assert left.position.kind == "none" and left.window is None and not left.output_gate
            assert right.decay == tuple(mixer["right"]["decay"])
            assert (right.n_heads, right.key_dim, right.value_dim) == \
                tuple(mixer["right"][k] for k in ("heads", "dim", "vdim"))
        else:
            assert isinstance(made.mixer, AttentionSpec) and made.mixer.output_gate == "head"
            mask = mixer.get("mask") or {}
            assert made.mixer.window == mask.get("size") and made.mixer.pool == mask.get("pool")
            assert made.mixer.shared_kv == ("kv_from" in mixer)
            rot = mixer.get("rot")
            assert made.mixer.position.kind == ("none" if rot is None else "rope_pairs")
            entry = spec.schedule[index]
            if "kv_from" in mixer:
                assert (entry.cache, entry.writes_cache, entry.own) == (mixer["kv_from"], False, index)
            else:
                assert (entry.cache, entry.writes_cache, entry.own_id) == (index, True, index)
        mlp = layer["mlp"]
        if mlp is None:
            assert made.feed_forward is None
        elif mlp["kind"] == "dense":
            assert isinstance(made.feed_forward, GatedMLPSpec) and made.feed_forward.bias is True
            assert made.feed_forward.intermediate_size == mlp["ff"]
        else:
            ffn = made.feed_forward
            assert isinstance(ffn, RoutedMLPSpec) and ffn.scoring == "softmax_all" and ffn.correction
            assert (ffn.n_experts, ffn.top, ffn.identity) == \
                (mlp["router"]["experts"], mlp["router"]["top"], mlp["router"]["identity"])


def test_what_a_shared_cache_keeps():
    """A layer whose keys other layers read keeps what the widest of their masks needs; all of
    it when a reader has no mask."""
    from edge_infer_amd.cache.storage import CacheLayout
    spec = config_of(CONFIGS["C"]).model_spec()
    assert spec.layers[1].mixer.cache_span == 0          # layer 3 reads it without a mask
    layout = CacheLayout(spec)
    windows = {request.window for request, entries in layout.kv_groups if 1 in entries}
    assert windows == {None}
    spec = config_of(CONFIGS["A"]).model_spec()
    assert spec.layers[1].mixer.cache_span == 33 and spec.layers[2].mixer.cache_span is None
    layout = CacheLayout(spec)
    assert {request.window for request, entries in layout.kv_groups if 1 in entries} == {33}
    # the pooled blocks are every layer's own, one entry a block
    strides = {cache_id: request.stride for request, entries in layout.kv_groups
               for cache_id in entries if isinstance(cache_id, tuple) and cache_id[1] == "pool"}
    assert strides == {(1, "pool"): 5, (2, "pool"): 7}
    # pooled blocks larger than their window: the cache keeps a block's worth
    spec = config_of(CONFIGS["D"]).model_spec()
    layout = CacheLayout(spec)
    assert {request.window for request, entries in layout.kv_groups if 0 in entries} == {130}


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_checkpoint_names_and_shapes(name):
    from edge_infer_amd.engine.model import expected_parameters
    cfg = config_of(CONFIGS[name])
    expected = expected_parameters(cfg.model_spec(), cfg.checkpoint_name)
    shapes = {key: shape for key, (shape, _) in tensor_shapes(CONFIGS[name]).items()}
    needed = {ck: tuple(param.shape) for ck, param in expected.values() if not param.optional}
    optional = {ck for ck, param in expected.values() if param.optional}
    assert needed == {key: tuple(shape) for key, shape in shapes.items() if key not in optional}


def test_registry_finds_the_architecture():
    from edge_infer_amd.config import GopuzenConfig, resolve_architecture
    assert resolve_architecture({"architecture": "Gopuzen"}).config_class is GopuzenConfig
    assert resolve_architecture({"model_type": "gopuzen"}).config_class is GopuzenConfig


def changed(path, value):
    raw = copy.deepcopy(CONFIGS["A"])
    at = raw
    for key in path[:-1]:
        at = at[key]
    if value is KeyError:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    return raw


@pytest.mark.parametrize("path, value, message", [
    (("layers", 0, "type"), "mamba2", "type must be one of"),
    (("layers", 0, "mixer", "right", "decay"), [0.5, 0.9], "decay must be a list of 3"),
    (("layers", 0, "mixer", "left", "heads"), 5, "multiple of kv_heads"),
    (("layers", 0, "mixer", "left", "rot"), {"base": 10.0, "dims": 4}, "does not know"),
    (("layers", 1, "mixer", "rot", "dims"), 7, "even and at most dim"),
    (("layers", 1, "mixer", "mask", "size"), KeyError, "lacks 'size'"),
    (("layers", 2, "mixer", "kv_from"), 2, "earlier layer"),
    (("layers", 2, "mixer", "kv_from"), 0, "attention layer with keys"),
    (("layers", 2, "mixer", "dim"), 32, "heads and rotations differ"),
    (("layers", 1, "mlp", "router", "top"), 9, "above its outputs"),
    (("layers", 0, "mlp", "kind"), "relu", "must be 'dense' or 'moe'"),
    (("canon",), KeyError, "lacks the object 'canon'"),
    (("embedding", "scale"), "big", "must be a number"),
    (("layers", 1, "mixer", "sink"), True, "does not know"),
])
def test_refusals(path, value, message):
    from edge_infer_amd.config.gopuzen import GopuzenConfigError
    with pytest.raises(GopuzenConfigError, match=message):
        config_of(changed(path, value))


def test_what_may_be_absent():
    raw = changed(("layers", 1, "mixer", "mask"), {"size": 9})      # a window without blocks
    assert config_of(raw).model_spec().layers[1].mixer.pool is None
    raw = changed(("layers", 1, "mlp", "router"), {"experts": 5, "top": 2})
    assert config_of(raw).model_spec().layers[1].feed_forward.identity == 0
    raw = changed(("layers", 0, "mixer", "left", "q_temp"), KeyError)
    assert config_of(raw).model_spec().layers[0].mixer.branches[0].query_temperature is None


def test_a_strided_cache_group_counts_blocks():
    from edge_infer_amd.cache.allocator import PagePool, SequencePages
    pages = SequencePages(PagePool(8), 2, stride=5)
    pages.open(0)
    assert pages.pages_needed(0, 4) == 0 and pages.pages_needed(0, 5) == 1
    assert pages.pages_needed(0, 5 * 64) == 1 and pages.pages_needed(0, 5 * 64 + 5) == 2
    pages.grow(0, 5 * 64 + 5)
    assert len(pages.row(0)) == 2
    pages.trim(0, 5 * 64 + 5)                # nothing is ever given back before the end
    assert pages.held() == 2
    pages.close(0)
    assert pages.pool.n_free == 8
