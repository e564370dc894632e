"""The Vafepel configuration: what config.json keys become, what is refused, the names of the
checkpoint's tensors, and which layer is the source of the mixed values.  Runs without a GPU."""
import copy
import json

import pytest

import plain_vafepel as plain
from vafepel_helpers import CONFIGS, TWINS, tensor_shapes


def config_class():
    from edge_infer_amd.config import VafepelConfig
    return VafepelConfig


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_round_trip_and_spec(name):
    from edge_infer_amd.config.specs import (AttentionSpec, GatedMLPSpec, RoutedMLPSpec,
                                             StateSpaceSpec)
    raw = CONFIGS[name]
    cfg = config_class().from_dict(raw)
    assert config_class().from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    spec = cfg.model_spec()
    assert spec.tie_word_embeddings and spec.embedding_norm is not None
    assert spec.logit_scale == raw.get("logit_scale", 1.0)
    assert spec.logit_softcap == raw.get("logit_softcap")
    source_seen = False
    for layer, made in zip(raw["layers"], spec.layers):
        assert made.block == "prenorm" and made.norm.eps == raw["norm"]["eps"]
        m = layer["mixer"]
        if layer["type"] == "attention":
            assert isinstance(made.mixer, AttentionSpec)
            a = made.mixer
            assert (a.n_heads, a.n_kv_heads, a.head_dim, a.v_dim) == \
                (m["heads"], m["kv_heads"], m["dim"], m["vdim"])
            assert a.window == (m["mask"]["size"] if "mask" in m else None)
            assert a.scale == m["scale"] and a.sink and a.output_gate and a.qk_norm
            if "rot" in m:
                assert a.position.kind == "rope_half" and a.position.dim == m["rot"]["dims"]
                assert (a.position.scaling is None) == ("scaling" not in m["rot"])
            else:
                assert a.position.kind == "none"
            if m["v_mix"]:
                assert a.value_mix == ("mix" if source_seen else "source")
                source_seen = True
            else:
                assert a.value_mix == "off"
        else:
            assert isinstance(made.mixer, StateSpaceSpec)
            s = made.mixer
            assert (s.n_heads, s.head_dim, s.state, s.groups, s.conv_taps, s.norm_parts) == \
                (m["heads"], m["vdim"], m["state"], m["groups"], m["conv"], m["norm_groups"])
        mlp = layer["mlp"]
        if mlp is None:
            assert made.feed_forward is None
        elif mlp["kind"] == "dense":
            assert isinstance(made.feed_forward, GatedMLPSpec)
            assert made.feed_forward.activation == "clamped_swish"
            assert made.feed_forward.limit == mlp["limit"] and made.feed_forward.alpha == 1.702
        else:
            assert isinstance(made.feed_forward, RoutedMLPSpec)
            assert (made.feed_forward.n_experts, made.feed_forward.top,
                    made.feed_forward.intermediate_size) == \
                (mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"])


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_checkpoint_names_and_shapes(name):
    from edge_infer_amd.engine.model import expected_parameters
    for raw in (CONFIGS[name], TWINS[name]):
        cfg = config_class().from_dict(raw)
        expected = expected_parameters(cfg.model_spec(), cfg.checkpoint_name)
        shapes = tensor_shapes(raw)
        required = {ckpt for path, (ckpt, param) in expected.items()
                    if not param.optional and path != "head.weight"}
        known = {ckpt for _, (ckpt, _) in expected.items()}
        assert required <= set(shapes) <= known
        for _, (ckpt, param) in expected.items():
            if ckpt in shapes:
                assert tuple(param.shape) == tuple(shapes[ckpt][0]), ckpt


def test_registry_finds_the_architecture():
    from edge_infer_amd.config import resolve_architecture
    assert resolve_architecture({"architecture": "Vafepel"}).config_class is config_class()
    assert resolve_architecture({"model_type": "vafepel"}).config_class is config_class()


def test_frequencies_as_the_plain_function():
    import torch
    from edge_infer_amd.parts.rope import scaled_frequencies
    cfg = config_class().from_dict(CONFIGS["A"])
    position = cfg.model_spec().layers[0].mixer.position
    want = plain.rotary_frequencies(CONFIGS["A"]["layers"][0]["mixer"]["rot"])
    assert torch.allclose(scaled_frequencies(position), want, rtol=1e-13, atol=0)


def edit(raw, path, value):
    out = copy.deepcopy(raw)
    node = out
    for key in path[:-1]:
        node = node[key]
    if value is KeyError:
        del node[path[-1]]
    else:
        node[path[-1]] = value
    return out


@pytest.mark.parametrize("path, value, message", [
    (("layers", 0, "type"), "conv", "type must be one of"),
    (("layers", 0, "mixer", "heads"), 7, "multiple of kv_heads"),
    (("layers", 0, "mixer", "rot", "dims"), 7, "even"),
    (("layers", 0, "mixer", "rot", "dims"), 18, "at most dim"),
    (("layers", 0, "mixer", "bias"), True, "does not know"),
    (("layers", 0, "mixer", "rot", "scaling", "kind"), "yarn", "does not know"),
    (("layers", 0, "mixer", "scale"), KeyError, "lacks 'scale'"),
    (("layers", 0, "mixer", "v_mix"), 1, "true or false"),
    (("layers", 0, "mlp", "kind"), "sparse", "'dense' or 'moe'"),
    (("layers", 0, "mlp", "limit"), KeyError, "lacks 'limit'"),
    (("layers", 1, "mixer", "groups"), 3, "multiple of groups"),
    (("layers", 1, "mixer", "norm_groups"), 5, "norm_groups must divide"),
    (("layers", 1, "mlp", "router", "top"), 9, "above its experts"),
    (("layers", 2, "mixer", "vdim"), 8, "values of one width"),
    (("norm",), KeyError, "lacks the object 'norm'"),
    (("vocab",), 0, "at least 1"),
    (("logit_softcap",), -1.0, "positive number"),
])
def test_refusals(path, value, message):
    from edge_infer_amd.config.vafepel import VafepelConfigError
    with pytest.raises(VafepelConfigError, match=message):
        config_class().from_dict(edit(CONFIGS["A"], path, value))


def test_what_may_be_absent():
    """No window, no rotation, no rescaling, no feed-forward, no scale and no cap of the logits
    are all configurations; a layer that mixes no values may say so or say nothing."""
    raw = edit(CONFIGS["B"], ("layers", 0, "mixer", "v_mix"), KeyError)
    cfg = config_class().from_dict(raw)
    spec = cfg.model_spec()
    assert spec.logit_scale == 1.0 and spec.logit_softcap is None
    assert [layer.mixer.value_mix for layer in spec.layers if hasattr(layer.mixer, "value_mix")] \
        == ["off", "off", "off"]
    assert spec.layers[1].feed_forward is None and spec.layers[2].mixer.position.kind == "none"
    assert spec.layers[3].mixer.window is None
    raw = edit(edit(CONFIGS["A"], ("layers", 0, "mixer", "mask", "size"), None), ("logit_softcap",), 0)
    spec = config_class().from_dict(raw).model_spec()
    assert spec.layers[0].mixer.window is None and spec.logit_softcap is None
