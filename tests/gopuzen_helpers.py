"""Small Gopuzen configurations and weights for the tests.

The configurations differ from each other in every size and option: key and value head sizes
that differ or are equal (64 and 64 take the matrix-core attention kernels in bfloat16 where the
options allow them), group ratios 1 to 8, windows below, at and just above the cache's page of
64 tokens, pooled blocks smaller and larger than their window and of one token, layers that
read an earlier layer's keys with a mask of their own or none, rotations of a part of the head, of the
whole head and none, queries with and without a temperature, linear attention with key heads
of 12 to 160 elements and value heads that need one to three column tiles, decays of 1 and
near 0, convolutions of 1 to 5 taps, layers without a feed-forward, 3 to 70 experts of which 1
to 4 are chosen with 0 to 5 identity experts.  The weights are drawn so that signals are of
order one (N(0, 0.02) matrices would make every softmax flat and every state tiny, and hide a
wrong key or a lost state); they are rounded to bfloat16, so that both precisions and the
oracle see the same numbers.
"""
import json
from pathlib import Path

import torch


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, identity):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "identity": identity}}


def parallel(left, right, mlp):
    """left: (heads, kv_heads, dim, vdim, scale, q_temp or None); right: (heads, dim, vdim,
    decays)."""
    heads, kv_heads, dim, vdim, scale, q_temp = left
    softmax = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if q_temp is not None:
        softmax["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    r_heads, r_dim, r_vdim, decay = right
    return {"type": "parallel",
            "mixer": {"left": softmax, "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim,
                                                 "decay": list(decay)}}, "mlp": mlp}


def attention(heads, kv_heads, dim, vdim, scale, mask, rot, mlp, kv_from=None):
    """mask: None, (size,) or (size, pool); rot: None or (base, dims)."""
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if mask is not None:
        mixer["mask"] = {"size": mask[0]}
        if len(mask) > 1:
            mixer["mask"]["pool"] = mask[1]
    if rot is not None:
        mixer["rot"] = {"base": rot[0], "dims": rot[1]}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def model(vocab, width, eps, embedding_scale, taps, layers):
    return {"architecture": "Gopuzen", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": embedding_scale}, "canon": {"taps": taps}, "layers": layers}


CONFIG_A = model(211, 64, 1e-5, 3.0, 3, [
    parallel((6, 3, 16, 24, 0.3, (0.4, 16)), (3, 12, 24, (0.5, 0.9, 0.99)), dense(96)),
    attention(4, 2, 16, 8, 0.25, (20, 5), (10000.0, 8), moe(40, 5, 2, 2)),
    attention(4, 2, 16, 8, 0.3, (33, 7), (10000.0, 8), None, kv_from=1),
    parallel((4, 4, 8, 8, 0.35, None), (2, 32, 72, (1.0, 0.7)), moe(24, 6, 3, 1)),
    attention(12, 3, 32, 24, 0.2, None, None, dense(80))])
# head size 64 with values as wide as keys: the matrix-core kernels in bfloat16 for the softmax
# half; a window of exactly a page with blocks of a page, and one of a token more with blocks
# of one token; one tap; one expert chosen; no identity expert
CONFIG_B = model(97, 128, 1e-6, 1.0, 1, [
    attention(4, 2, 64, 64, 0.125, (64, 64), (10000.0, 64), moe(48, 3, 1, 0)),
    parallel((8, 2, 64, 64, 0.125, (0.2, 64)), (4, 64, 64, (0.95, 0.9, 0.8, 0.999)), None),
    attention(8, 2, 64, 64, 0.1, (65, 1), (500.0, 32), dense(160), kv_from=None),
    attention(8, 2, 64, 64, 0.15, (10,), (500.0, 32), moe(64, 4, 2, 3), kv_from=2)])
# key heads of 160 elements in the linear half (the widest register tile), pooled blocks larger
# than their window, a reader whose mask is wider than its source's and one without a mask,
# five taps, more router outputs than a wave has lanes
CONFIG_C = model(150, 96, 1e-6, 0.5, 5, [
    parallel((2, 1, 48, 40, 0.15, (0.3, 3)), (1, 160, 136, (0.97,)), moe(16, 65, 4, 5)),
    attention(8, 1, 24, 40, 0.2, (3, 8), (100.0, 24), None),
    attention(8, 1, 24, 40, 0.2, (40, 6), (100.0, 24), dense(56), kv_from=1),
    attention(8, 1, 24, 40, 0.25, None, (100.0, 24), moe(32, 8, 2, 0), kv_from=1),
    parallel((3, 3, 24, 8, 0.2, None), (5, 16, 16, (0.1, 0.5, 0.9, 0.99, 0.999)), dense(40))])
# sizes that are multiples of nothing: no vector kernel and no few-rows product applies
CONFIG_D = model(101, 50, 1e-5, 7.0, 2, [
    attention(6, 2, 10, 7, 0.3, (7, 3), (3000.0, 6), moe(13, 3, 2, 1)),
    parallel((5, 5, 6, 9, 0.4, (0.3, 5)), (3, 7, 11, (0.8, 0.9, 0.95)), dense(30)),
    attention(6, 2, 10, 7, 0.3, (130, 20), (3000.0, 6), None, kv_from=0)])
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C, "D": CONFIG_D}


def dense_twin(cfg):
    """`cfg` with every routed feed-forward replaced by a dense one.  A router chooses by the
    order of its scores, which any rounding may change where two of them nearly tie, and one
    token routed otherwise changes the rows after it as well; comparisons in bfloat16 over
    whole requests therefore run on models that route nothing."""
    twin = json.loads(json.dumps(cfg))
    for layer in twin["layers"]:
        mlp = layer["mlp"]
        if mlp is not None and mlp["kind"] == "moe":
            layer["mlp"] = dense(mlp["expert"]["ff"] * mlp["router"]["top"])
    return twin


TWINS = {name: dense_twin(cfg) for name, cfg in CONFIGS.items()}


def tensor_shapes(cfg):
    """name -> (shape, law) of every tensor of a model of `cfg`."""
    w = cfg["width"]
    taps = cfg["canon"]["taps"]
    out = {"embed": ((cfg["vocab"], w), "table"), "final.norm": ((w,), "norm"),
           "final.norm.b": ((w,), "bias"), "head": ((cfg["vocab"], w), "matrix")}

    def softmax(p, m, shared=False, gate=False):
        # queries and keys of such a size that the scores' spread is about 3 whatever the
        # head's size and the mixer's scale
        law = ("query", (3.0 / (m["dim"] ** 0.5 * m["scale"])) ** 0.5)
        out[p + "q"] = ((m["heads"] * m["dim"], w), law)
        if not shared:
            out[p + "k"] = ((m["kv_heads"] * m["dim"], w), law)
            out[p + "v"] = ((m["kv_heads"] * m["vdim"], w), "matrix")
        if gate:
            out[p + "g"] = ((m["heads"], w), "matrix")
        out[p + "o"] = ((w, m["heads"] * m["vdim"]), "matrix")
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}."
        for which in ("norm1", "norm1b"):
            out[p + which] = ((w,), "norm")
            out[p + which + ".b"] = ((w,), "bias")
        out[p + "ls1"] = ((w,), "norm")
        out[p + "canon1"] = ((w, taps), "filter")
        if layer["type"] == "attention":
            softmax(p + "mix.", m, shared=m.get("kv_from") is not None, gate=True)
        else:
            softmax(p + "mix.left.", m["left"])
            r = m["right"]
            out[p + "mix.right.q"] = ((r["heads"] * r["dim"], w), "matrix")
            out[p + "mix.right.k"] = ((r["heads"] * r["dim"], w), "matrix")
            out[p + "mix.right.v"] = ((r["heads"] * r["vdim"], w), "matrix")
            out[p + "mix.right.g"] = ((r["heads"] * r["vdim"], w), "matrix")
            out[p + "mix.right.norm"] = ((r["heads"] * r["vdim"],), "norm")
            out[p + "mix.right.o"] = ((w, r["heads"] * r["vdim"]), "matrix")
            out[p + "mix.left.out"] = ((w,), "norm")
            out[p + "mix.right.out"] = ((w,), "norm")
        mlp = layer["mlp"]
        if mlp is None:
            continue
        for which in ("norm2", "norm2b"):
            out[p + which] = ((w,), "norm")
            out[p + which + ".b"] = ((w,), "bias")
        out[p + "ls2"] = ((w,), "norm")
        out[p + "canon2"] = ((w, taps), "filter")
        if mlp["kind"] == "dense":
            ff = mlp["ff"]
            for name, shape in (("gate", (ff, w)), ("up", (ff, w)), ("down", (w, ff))):
                out[p + "mlp." + name] = (shape, "matrix")
                out[p + "mlp." + name + ".b"] = ((shape[0],), "bias")
        else:
            ff, router = mlp["expert"]["ff"], mlp["router"]
            outputs = router["experts"] + router.get("identity", 0)
            out[p + "mlp.router"] = ((outputs, w), "router")
            out[p + "mlp.correction"] = ((outputs,), "correction")
            for e in range(router["experts"]):
                out[p + f"mlp.e{e}.gate"] = ((ff, w), "matrix")
                out[p + f"mlp.e{e}.up"] = ((ff, w), "matrix")
                out[p + f"mlp.e{e}.down"] = ((w, ff), "matrix")
    return out


def sharp_weights(cfg, seed, query_gain=1.0):
    """Tensors of order-one signal, bfloat16.  The query and key matrices of the softmax mixers
    are drawn so that the scores spread by about 3 (single keys stand out, and a key that is
    left out or read twice moves the logits by far more than any tolerance); `query_gain`
    multiplies them further."""
    g = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, (shape, law) in tensor_shapes(cfg).items():
        if isinstance(law, tuple):    # ("query", gain)
            value = torch.randn(shape, generator=g) * law[1] * query_gain / shape[1] ** 0.5
        elif law == "matrix":
            value = torch.randn(shape, generator=g) / shape[1] ** 0.5
        elif law == "router":     # scores far enough apart that few choices are close calls
            value = torch.randn(shape, generator=g) * 4.0 / shape[1] ** 0.5
        elif law == "correction":     # of the size of a score's spread, so that it changes choices
            value = torch.randn(shape, generator=g) * 0.3 / shape[0]
        elif law == "table":
            value = torch.randn(shape, generator=g)
        elif law == "norm":
            value = 1.0 + (torch.rand(shape, generator=g) * 0.4 - 0.2)
        elif law == "bias":
            value = torch.randn(shape, generator=g) * 0.2
        elif law == "filter":
            value = torch.randn(shape, generator=g) * 0.4
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
