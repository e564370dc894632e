"""Small Vafepel configurations and weights for the tests.

The configurations differ from each other in every size and option: key and value head sizes
that differ or are equal (64 and 64 take the matrix-core attention kernels in bfloat16), group
ratios 1, 2, 3 and 4, windows below, at and just above the cache's page of 64 tokens and none
at all, rotations of a part of the head, of the whole head and none, with and without
rescaled frequencies, value mixing whose source is the first layer, a later layer, or no
layer, state sizes that are and are not multiples of the scan's 16 rows, 1 to 4 groups,
convolutions of 1 to 5 taps, norms in 1 to 4 parts, layers without a feed-forward, dense
feed-forwards with small and large limits, 3 to 70 experts of which 1 to 4 are chosen, logits
with and without scale and cap.  The weights are drawn so that signals are of order one
(N(0, 0.02) matrices would make every softmax flat and every state tiny, and hide a wrong key
or a lost state); they are rounded to bfloat16, so that both precisions and the oracle see
the same numbers.
"""
import json
from pathlib import Path

import torch


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def attention(heads, kv_heads, dim, vdim, scale, window, rot, v_mix, mlp):
    """rot: None, or (base, dims) or (base, dims, (factor, low, high, original))."""
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
             "v_mix": v_mix}
    if window is not None:
        mixer["mask"] = {"size": window}
    if rot is not None:
        mixer["rot"] = {"base": rot[0], "dims": rot[1]}
        if len(rot) > 2:
            mixer["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), rot[2]))
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def mamba(heads, vdim, state, groups, conv, norm_groups, mlp):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state,
                                        "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}, "mlp": mlp}


def model(vocab, width, eps, logit_scale, softcap, layers):
    out = {"architecture": "Vafepel", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "layers": layers}
    if logit_scale is not None:
        out["logit_scale"] = logit_scale
    if softcap is not None:
        out["logit_softcap"] = softcap
    return out


CONFIG_A = model(211, 64, 1e-5, 0.5, 12.0, [
    attention(6, 3, 16, 24, 0.3, 20, (10000.0, 8, (4.0, 1.0, 4.0, 64)), True, dense(96, 1.5)),
    mamba(4, 12, 16, 2, 4, 2, moe(40, 6, 2)),
    attention(3, 3, 16, 24, 0.25, 70, (500.0, 16), True, moe(24, 5, 3)),
    attention(12, 3, 32, 24, 0.2, None, (1e6, 2), True, None),
    mamba(2, 20, 24, 1, 3, 1, dense(80, 7.0))])
# values as wide as keys and head size 64: the matrix-core attention kernels in bfloat16;
# windows of exactly a page and of one token more; no layer mixes values; one expert chosen
CONFIG_B = model(97, 128, 1e-6, None, None, [
    attention(4, 2, 64, 64, 0.125, 64, (10000.0, 64), False, moe(48, 3, 1)),
    mamba(8, 16, 32, 4, 2, 4, None),
    attention(8, 2, 64, 64, 0.1, 65, None, False, dense(160, 3.0)),
    attention(2, 2, 64, 64, 0.15, None, (2000.0, 32, (8.0, 1.0, 2.0, 128)), False, moe(64, 4, 2))])
# a state-space layer first; the source of the mixed values is the third layer, after an
# attention layer that mixes nothing; more experts than a wave has lanes
CONFIG_C = model(150, 96, 1e-6, 0.7, None, [
    mamba(3, 32, 128, 1, 5, 3, moe(16, 70, 4)),
    attention(4, 4, 24, 8, 0.2, 33, (100.0, 24), False, None),
    attention(2, 1, 48, 40, 0.15, 3, (10000.0, 12), True, dense(56, 0.5)),
    mamba(6, 8, 8, 3, 1, 1, None),
    attention(10, 1, 8, 40, 0.4, 100, None, True, moe(32, 8, 2))])
# sizes that are multiples of nothing: no vector kernel and no few-rows product applies
CONFIG_D = model(101, 50, 1e-5, None, 9.0, [
    attention(6, 2, 10, 7, 0.3, 7, (3000.0, 6, (2.0, 1.0, 3.0, 16)), True, moe(13, 3, 2)),
    mamba(5, 6, 19, 5, 4, 5, dense(30, 2.0)),
    attention(2, 2, 12, 7, 0.3, 130, (50.0, 12), True, None)])
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C, "D": CONFIG_D}


def dense_twin(cfg):
    """`cfg` with every routed feed-forward replaced by a dense one.  A router chooses by the
    order of its logits, which any rounding may change where two of them nearly tie, and one
    token routed otherwise changes the rows after it as well; comparisons in bfloat16 over
    whole requests therefore run on models that route nothing."""
    twin = json.loads(json.dumps(cfg))
    for layer in twin["layers"]:
        mlp = layer["mlp"]
        if mlp is not None and mlp["kind"] == "moe":
            layer["mlp"] = dense(mlp["expert"]["ff"] * mlp["router"]["top"], 2.5)
    return twin


TWINS = {name: dense_twin(cfg) for name, cfg in CONFIGS.items()}


def tensor_shapes(cfg):
    """name -> (shape, law) of every tensor of a model of `cfg`."""
    w = cfg["width"]
    out = {"embed": ((cfg["vocab"], w), "table"), "embed.norm": ((w,), "norm"),
           "final.norm": ((w,), "norm")}
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}."
        out[p + "norm1"] = ((w,), "norm")
        if layer["type"] == "attention":
            q, k, v = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            o = m["heads"] * m["vdim"]
            out[p + "mix.q"] = ((q, w), "matrix")
            out[p + "mix.k"] = ((k, w), "matrix")
            out[p + "mix.v"] = ((v, w), "matrix")
            out[p + "mix.q.norm"] = ((m["dim"],), "head_norm")
            out[p + "mix.k.norm"] = ((m["dim"],), "head_norm")
            out[p + "mix.vmix"] = ((), "mix")
            out[p + "mix.sink"] = ((m["heads"],), "sink")
            out[p + "mix.g"] = ((o, w), "matrix")
            out[p + "mix.o"] = ((w, o), "matrix")
        else:
            inner = m["heads"] * m["vdim"]
            channels = inner + 2 * m["groups"] * m["state"]
            out[p + "mix.in"] = ((inner + channels + m["heads"], w), "matrix")
            out[p + "mix.conv"] = ((channels, m["conv"]), "filter")
            out[p + "mix.conv.b"] = ((channels,), "bias")
            out[p + "mix.dt_bias"] = ((m["heads"],), "step")
            out[p + "mix.A_log"] = ((m["heads"],), "rate")
            out[p + "mix.D"] = ((m["heads"],), "norm")
            out[p + "mix.norm"] = ((inner,), "norm")
            out[p + "mix.o"] = ((w, inner), "matrix")
        mlp = layer["mlp"]
        if mlp is None:
            continue
        out[p + "norm2"] = ((w,), "norm")
        if mlp["kind"] == "dense":
            ff = mlp["ff"]
            out[p + "mlp.gate"] = ((ff, w), "wide")
            out[p + "mlp.up"] = ((ff, w), "wide")
            out[p + "mlp.down"] = ((w, ff), "matrix")
        else:
            ff = mlp["expert"]["ff"]
            out[p + "mlp.router"] = ((mlp["router"]["experts"], w), "router")
            for e in range(mlp["router"]["experts"]):
                out[p + f"mlp.e{e}.gate"] = ((ff, w), "wide")
                out[p + f"mlp.e{e}.up"] = ((ff, w), "wide")
                out[p + f"mlp.e{e}.down"] = ((w, ff), "matrix")
    return out


def sharp_weights(cfg, seed, long_memory=False, head_norm=1.6):
    """Tensors of order-one signal, bfloat16.  `long_memory`: the state-space layers forget
    slowly, so that a token far back still shows in the logits.  `head_norm`: the mean of the
    query and key norms' weights; above 1 the scores spread and single keys stand out."""
    g = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, (shape, law) in tensor_shapes(cfg).items():
        if law == "matrix":
            value = torch.randn(shape, generator=g) / shape[1] ** 0.5
        elif law == "wide":       # pre-activations that reach past the limits now and then
            value = torch.randn(shape, generator=g) * 1.6 / shape[1] ** 0.5
        elif law == "router":     # logits far enough apart that few choices are close calls
            value = torch.randn(shape, generator=g) * 6.0 / shape[1] ** 0.5
        elif law == "table":
            value = torch.randn(shape, generator=g)
        elif law == "norm":
            value = 1.0 + (torch.rand(shape, generator=g) * 0.4 - 0.2)
        elif law == "head_norm":
            value = head_norm + (torch.rand(shape, generator=g) * 0.4 - 0.2)
        elif law == "bias":
            value = torch.randn(shape, generator=g) * 0.3
        elif law == "filter":
            value = torch.randn(shape, generator=g) * 0.6
        elif law == "sink":
            value = torch.rand(shape, generator=g) * 3.0 - 1.0
        elif law == "mix":
            value = torch.rand(shape, generator=g) * 0.5 + 0.2
        elif law == "step":
            value = torch.rand(shape, generator=g) * 3.0 - 3.5
        elif law == "rate":
            value = (torch.rand(shape, generator=g) - 7.0 if long_memory
                     else torch.rand(shape, generator=g) * 3.0 - 2.5)
        tensors[name] = value.to(torch.bfloat16)
    return tensors


def write_folder(path, cfg, tensors):
    from safetensors.torch import save_file
    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg, indent=1))
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(path / "model.safetensors"))
    return path


def ids(vocab, count, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=g).tolist()
