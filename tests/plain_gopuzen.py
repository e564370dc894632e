"""A plain, slow implementation of the Gopuzen decoder used only as the oracle of the tests.

Whole sequences from position 0, no cache, token-by-token recurrences, one function per
mechanism, float64 arithmetic on the CPU.  Nothing here imports the product package.  A
model is a dictionary `cfg` (the content of its config.json) and a dictionary of tensors
under their checkpoint names.

Notation: T tokens, W the model's width; matrices are stored [out, in].
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def f64(t):
    return t.to(F64)


def linear(x, weight, bias=None):
    y = f64(x) @ f64(weight).T
    return y if bias is None else y + f64(bias)


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


# ---------------------------------------------------------------------------- norms
def rms_norm(x, weight, eps):
    """y = x / sqrt(mean(x^2) + eps) * w over the last axis."""
    x = f64(x)
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * f64(weight)


def layer_norm(x, weight, bias, eps):
    """y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b over the last axis."""
    x = f64(x)
    centred = x - x.mean(dim=-1, keepdim=True)
    return centred / torch.sqrt((centred * centred).mean(dim=-1, keepdim=True) + eps) \
        * f64(weight) + f64(bias)


# ---------------------------------------------------------------------------- input convolution
def input_convolution(h, taps_weight):
    """h [T, W], taps_weight [W, taps]: y_t = h_t + sum_j w[:, j] h_(t - taps + 1 + j), rows
    before the sequence's start being zero."""
    h = f64(h)
    w = f64(taps_weight)
    taps = w.shape[1]
    out = h.clone()
    for t in range(h.shape[0]):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


# ---------------------------------------------------------------------------- rotation
def rotate_neighbours(x, positions, rot):
    """x [T, heads, dim]: elements (2i, 2i + 1), i < dims / 2, of every head turn by the angle
    position * base^(-2i / dims); the rest pass."""
    if not rot:
        return x
    dims = int(rot["dims"])
    out = x.clone()
    for i in range(dims // 2):
        f = float(rot["base"]) ** (-2.0 * i / dims)
        angle = f64(positions) * f
        cos, sin = torch.cos(angle)[:, None], torch.sin(angle)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * cos - v * sin
        out[..., 2 * i + 1] = v * cos + u * sin
    return out


# ---------------------------------------------------------------------------- attention
def softmax_attention(q, k, v, scale, visible):
    """q [T, H, d], k [S, G, d], v [S, G, e]; head h reads kv head h // (H / G); `visible(i)`
    gives the indices into k and v that query row i sees.  Returns [T, H, e]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for i in range(T):
        seen = visible(i)
        for h in range(H):
            g = h // (H // G)
            scores = (k[seen, g] @ q[i, h]) * scale
            weights = torch.softmax(scores, dim=0)
            out[i, h] = (weights[:, None] * v[seen, g]).sum(dim=0)
    return out


def query_temperature(positions, q_temp):
    """1 + coef ln(floor((p + 1) / every) + 1) for every position p."""
    steps = torch.div(positions.to(torch.int64) + 1, int(q_temp["every"]), rounding_mode="floor")
    return 1.0 + float(q_temp["coef"]) * torch.log(f64(steps) + 1.0)


def pooled_window_attention(q, k, v, scale, window, pool):
    """Position i sees the tokens j with 0 <= i - j < window and, for every block b of `pool`
    tokens with b pool + pool - 1 <= i - window, one key and value that are the block's means;
    tokens and blocks share one softmax."""
    T = q.shape[0]
    blocks = T // pool
    k_all, v_all = k, v
    if blocks:
        k_mean = k[:blocks * pool].reshape(blocks, pool, *k.shape[1:]).mean(dim=1)
        v_mean = v[:blocks * pool].reshape(blocks, pool, *v.shape[1:]).mean(dim=1)
        k_all, v_all = torch.cat([k, k_mean]), torch.cat([v, v_mean])

    def visible(i):
        seen = list(range(max(0, i - window + 1), i + 1))
        seen += [T + b for b in range(blocks) if b * pool + pool - 1 <= i - window]
        return seen
    return softmax_attention(q, k_all, v_all, scale, visible)


def causal_attention(h, tensors, prefix, mixer, positions):
    """The softmax half of the parallel mixer: no rotation, queries with a temperature that
    grows with the position, every earlier key visible."""
    H, G = int(mixer["heads"]), int(mixer["kv_heads"])
    d, e = int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q = linear(h, tensors[prefix + "q"]).reshape(T, H, d)
    k = linear(h, tensors[prefix + "k"]).reshape(T, G, d)
    v = linear(h, tensors[prefix + "v"]).reshape(T, G, e)
    if mixer.get("q_temp"):
        q = q * query_temperature(positions, mixer["q_temp"])[:, None, None]
    out = softmax_attention(q, k, v, float(mixer["scale"]), lambda i: list(range(i + 1)))
    return linear(out.reshape(T, H * e), tensors[prefix + "o"])


def attention_mixer(h, tensors, prefix, mixer, positions, shared):
    """The mixer 'attention': rotated queries and keys, a window with pooled blocks before it,
    a sigmoid gate per head.  `shared`: (k, v) of the layer whose keys and values this layer
    uses, or None.  Returns (output [T, W], (k, v) as cached)."""
    H, G = int(mixer["heads"]), int(mixer["kv_heads"])
    d, e = int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q = rotate_neighbours(linear(h, tensors[prefix + "q"]).reshape(T, H, d), positions,
                          mixer.get("rot"))
    if shared is None:
        k = rotate_neighbours(linear(h, tensors[prefix + "k"]).reshape(T, G, d), positions,
                              mixer.get("rot"))
        v = linear(h, tensors[prefix + "v"]).reshape(T, G, e)
    else:
        k, v = shared
    mask = mixer.get("mask")
    if mask and mask.get("pool") is not None:
        out = pooled_window_attention(q, k, v, float(mixer["scale"]), int(mask["size"]),
                                      int(mask["pool"]))
    elif mask:
        size = int(mask["size"])
        out = softmax_attention(q, k, v, float(mixer["scale"]),
                                lambda i: list(range(max(0, i - size + 1), i + 1)))
    else:
        out = softmax_attention(q, k, v, float(mixer["scale"]), lambda i: list(range(i + 1)))
    gate = sigmoid(linear(h, tensors[prefix + "g"]))              # [T, H]
    out = out * gate[:, :, None]
    return linear(out.reshape(T, H * e), tensors[prefix + "o"]), (k, v)


# ---------------------------------------------------------------------------- linear attention
def decayed_linear_attention(q, k, v, decay):
    """q, k [T, H, d], v [T, H, e], decay [H]: S_t = decay_h S_(t-1) + k_t v_t^T and
    o_t = S_t^T q_t, with S_(-1) = 0.  Returns [T, H, e]."""
    T, H, d = q.shape
    e = v.shape[2]
    state = torch.zeros(H, d, e, dtype=F64)
    out = torch.zeros(T, H, e, dtype=F64)
    for t in range(T):
        state = state * decay[:, None, None] + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hde,hd->he", state, q[t])
    return out


def lightning_mixer(h, tensors, prefix, mixer, eps):
    H, d, e = int(mixer["heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q = silu(linear(h, tensors[prefix + "q"])).reshape(T, H, d)
    k = silu(linear(h, tensors[prefix + "k"])).reshape(T, H, d)
    v = silu(linear(h, tensors[prefix + "v"])).reshape(T, H, e)
    decay = torch.tensor([float(x) for x in mixer["decay"]], dtype=F64)
    out = decayed_linear_attention(q, k, v, decay).reshape(T, H * e)
    out = rms_norm(out, tensors[prefix + "norm"], eps) * sigmoid(linear(h, tensors[prefix + "g"]))
    return linear(out, tensors[prefix + "o"])


def parallel_mixer(h, tensors, prefix, mixer, eps, positions):
    """Half the sum of the two mixers' outputs, each RMS-normed over the width first."""
    left = causal_attention(h, tensors, prefix + "left.", mixer["left"], positions)
    right = lightning_mixer(h, tensors, prefix + "right.", mixer["right"], eps)
    return 0.5 * (rms_norm(left, tensors[prefix + "left.out"], eps)
                  + rms_norm(right, tensors[prefix + "right.out"], eps))


# ---------------------------------------------------------------------------- feed-forwards
def dense_feed_forward(h, tensors, prefix):
    gate = linear(h, tensors[prefix + "gate"], tensors[prefix + "gate.b"])
    up = linear(h, tensors[prefix + "up"], tensors[prefix + "up.b"])
    return linear(silu(gate) * up, tensors[prefix + "down"], tensors[prefix + "down.b"])


def route(h, tensors, prefix, router):
    """(chosen experts [T, top], their weights [T, top], all scores [T, E + I]): the scores
    are the softmax over all router outputs; the choice is by score plus correction, the
    weights are the scores themselves."""
    scores = torch.softmax(linear(h, tensors[prefix + "router"]), dim=-1)
    choice = scores + f64(tensors[prefix + "correction"])
    chosen = torch.topk(choice, int(router["top"]), dim=-1).indices
    return chosen, torch.gather(scores, 1, chosen), scores


def choice_margins(h, tensors, prefix, router):
    """For every row the gap between the last chosen and the first unchosen choice score,
    relative to the larger of the two: a rounding that is larger may choose otherwise (what a
    rounding does to a score grows with the score)."""
    scores = torch.softmax(linear(h, tensors[prefix + "router"]), dim=-1)
    choice = torch.sort(scores + f64(tensors[prefix + "correction"]), dim=-1, descending=True).values
    top = int(router["top"])
    if top >= choice.shape[1]:
        return torch.full((choice.shape[0],), float("inf"), dtype=F64)
    larger = torch.maximum(choice[:, top - 1].abs(), choice[:, top].abs()).clamp_min(1e-30)
    return (choice[:, top - 1] - choice[:, top]) / larger


def routed_feed_forward(h, tensors, prefix, mlp, margins=None):
    router = mlp["router"]
    experts = int(router["experts"])
    chosen, weights, _ = route(h, tensors, prefix, router)
    if margins is not None:
        margins.append(choice_margins(h, tensors, prefix, router))
    h = f64(h)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), weights[t]):
            if e >= experts:                      # an identity expert
                out[t] += w * h[t]
                continue
            name = f"{prefix}e{e}."
            mid = silu(linear(h[t], tensors[name + "gate"])) * linear(h[t], tensors[name + "up"])
            out[t] += w * linear(mid, tensors[name + "down"])
    return out


# ---------------------------------------------------------------------------- the model
def forward(cfg, tensors, tokens, layer_outputs=None, margins=None):
    """Logits [T, vocab] of one sequence of token ids from position 0.  `layer_outputs`: a
    list that receives the stream after every layer; `margins`: a list that receives, for
    every routed feed-forward, the rows' choice margins."""
    eps = float(cfg["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.int64)
    positions = torch.arange(tokens.shape[0])
    x = f64(tensors["embed"])[tokens] * float(cfg["embedding"]["scale"])
    kept = {}
    for index, layer in enumerate(cfg["layers"]):
        name = f"l{index}."

        def norm(which, rows):
            return layer_norm(rows, tensors[name + which], tensors[name + which + ".b"], eps)
        h = input_convolution(norm("norm1", x), tensors[name + "canon1"])
        mixer = layer["mixer"]
        if layer["type"] == "parallel":
            a = parallel_mixer(h, tensors, name + "mix.", mixer, eps, positions)
        elif layer["type"] == "attention":
            source = mixer.get("kv_from")
            a, kept[index] = attention_mixer(h, tensors, name + "mix.", mixer, positions,
                                             None if source is None else kept[int(source)])
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        x = x + norm("norm1b", a) * f64(tensors[name + "ls1"])
        mlp = layer.get("mlp")
        if mlp is not None:
            h = input_convolution(norm("norm2", x), tensors[name + "canon2"])
            if mlp["kind"] == "dense":
                f = dense_feed_forward(h, tensors, name + "mlp.")
            else:
                f = routed_feed_forward(h, tensors, name + "mlp.", mlp, margins)
            x = x + norm("norm2b", f) * f64(tensors[name + "ls2"])
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    x = layer_norm(x, tensors["final.norm"], tensors["final.norm.b"], eps)
    return linear(x, tensors["head"])


def clear_rows(cfg, tensors, tokens, margin, carry=True):
    """(logits, mask of the positions whose logits no routing decision closer than `margin`
    can have touched).  `carry`: a close call at a position also touches every later one (the
    caches and states carry it on)."""
    margins = []
    logits = forward(cfg, tensors, tokens, margins=margins)
    clear = torch.ones(logits.shape[0], dtype=torch.bool)
    for rows in margins:
        clear &= rows >= margin
    if carry and not bool(clear.all()):
        first = int((~clear).nonzero()[0])
        clear[first:] = False
    return logits, clear
