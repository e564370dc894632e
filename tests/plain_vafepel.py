"""A plain, slow implementation of the Vafepel decoder used only as the oracle of the tests.

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


def rms_norm(x, weight, eps):
    """y = x / sqrt(mean(x^2) + eps) * w over the last axis."""
    x = f64(x)
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * f64(weight)


def linear(x, weight):
    return f64(x) @ f64(weight).T


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 40.0, x, torch.log1p(torch.exp(torch.clamp(x, max=40.0))))


# ---------------------------------------------------------------------------- rotation
def rotary_frequencies(rot):
    """f_i = base^(-2i / dims), i < dims / 2, then the piecewise rescaling of long wavelengths:
    with l = 2 pi / f, f stays where l < original / high, becomes f / factor where
    l > original / low, and in between a blend (1 - s) f / factor + s f with
    s = (original / l - low) / (high - low)."""
    dims = int(rot["dims"])
    f = [float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)]
    scaling = rot.get("scaling")
    if scaling:
        factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
        original = float(scaling["original"])
        out = []
        for fi in f:
            wavelength = 2.0 * math.pi / fi
            if wavelength < original / high:
                out.append(fi)
            elif wavelength > original / low:
                out.append(fi / factor)
            else:
                s = (original / wavelength - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = out
    return torch.tensor(f, dtype=F64)


def rotate(x, positions, rot):
    """x [T, heads, dim]: the first rot.dims elements of every head are rotated in pairs
    (i, i + dims/2) by the angle position * f_i; the rest pass."""
    if not rot:
        return x
    dims = int(rot["dims"])
    half = dims // 2
    angle = f64(positions)[:, None] * rotary_frequencies(rot)[None, :]      # [T, half]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# ---------------------------------------------------------------------------- attention
def sink_window_attention(q, k, v, scale, window, sink):
    """q [T, H, d], k [T, G, d], v [T, G, e]; head h reads kv head h // (H / G).  Position i sees
    j with 0 <= i - j < window (None: every j <= i).  The softmax's denominator also holds
    exp(sink_h) (None: no such term).  Returns [T, H, e]."""
    T, H, d = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = 0 if window is None else max(0, i - window + 1)
            scores = (k[lo:i + 1, g] @ q[i, h]) * scale
            top = scores.max()
            if sink is not None:
                top = torch.maximum(top, sink[h])
            weights = torch.exp(scores - top)
            denominator = weights.sum()
            if sink is not None:
                denominator = denominator + torch.exp(sink[h] - top)
            out[i, h] = (weights[:, None] * v[lo:i + 1, g]).sum(dim=0) / denominator
    return out


def attention_mixer(h, tensors, prefix, mixer, eps, positions, first_values):
    """The attention mixer of one layer on the normed rows h [T, W].  `first_values`: the
    values [T, G, e] of the first layer that mixes values, or None if this is that layer (or
    the layer does not mix).  Returns (output [T, W], this layer's values before mixing)."""
    H, G = int(mixer["heads"]), int(mixer["kv_heads"])
    d, e = int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q = linear(h, tensors[prefix + "q"]).reshape(T, H, d)
    k = linear(h, tensors[prefix + "k"]).reshape(T, G, d)
    v = linear(h, tensors[prefix + "v"]).reshape(T, G, e)
    q = rms_norm(q, tensors[prefix + "q.norm"], eps)
    k = rms_norm(k, tensors[prefix + "k.norm"], eps)
    q = rotate(q, positions, mixer.get("rot"))
    k = rotate(k, positions, mixer.get("rot"))
    raw_values = v
    if mixer.get("v_mix") and first_values is not None:
        lam = f64(tensors[prefix + "vmix"])
        v = (1.0 - lam) * v + lam * first_values
    mask = mixer.get("mask")
    window = None if not mask else int(mask["size"])
    sink = f64(tensors[prefix + "sink"]) if prefix + "sink" in tensors else None
    o = sink_window_attention(q, k, v, float(mixer["scale"]), window, sink).reshape(T, H * e)
    if prefix + "g" in tensors:
        o = o * sigmoid(linear(h, tensors[prefix + "g"]))
    return linear(o, tensors[prefix + "o"]), raw_values


# ---------------------------------------------------------------------------- mamba2
def causal_conv(x, weight, bias):
    """y[t, c] = b[c] + sum_j w[c, j] x[t - (J - 1) + j, c], zeros before the start."""
    x, w = f64(x), f64(weight)
    T, C = x.shape
    J = w.shape[1]
    padded = torch.cat([torch.zeros(J - 1, C, dtype=F64), x], dim=0)
    y = f64(bias)[None, :].repeat(T, 1)
    for j in range(J):
        y = y + padded[j:j + T] * w[:, j]
    return y


def ssm_recurrence(x, B, C, dt, a, D):
    """One head: x [T, P], B, C [T, N], dt [T], a = exp(A_log) > 0, D a number.
    S_t = exp(-a dt_t) S_{t-1} + dt_t B_t x_t^T;  y_t = S_t^T C_t + D x_t."""
    T, P = x.shape
    N = B.shape[1]
    S = torch.zeros(N, P, dtype=F64)
    y = torch.zeros(T, P, dtype=F64)
    for t in range(T):
        S = torch.exp(-a * dt[t]) * S + dt[t] * torch.outer(B[t], x[t])
        y[t] = S.T @ C[t] + D * x[t]
    return y


def grouped_rms_norm(y, weight, parts, eps):
    """y [T, I] cut into `parts` equal parts, each divided by its own root mean square."""
    T, I = y.shape
    cut = y.reshape(T, parts, I // parts)
    cut = cut / torch.sqrt((cut * cut).mean(dim=-1, keepdim=True) + eps)
    return cut.reshape(T, I) * f64(weight)


def mamba2_mixer(h, tensors, prefix, mixer, eps):
    heads, P, N = int(mixer["heads"]), int(mixer["vdim"]), int(mixer["state"])
    G = int(mixer["groups"])
    inner = heads * P
    T = h.shape[0]
    proj = linear(h, tensors[prefix + "in"])
    z = proj[:, :inner]
    xbc = proj[:, inner:2 * inner + 2 * G * N]
    dt = proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, tensors[prefix + "conv"], tensors[prefix + "conv.b"]))
    x = xbc[:, :inner].reshape(T, heads, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + f64(tensors[prefix + "dt_bias"]))
    a = torch.exp(f64(tensors[prefix + "A_log"]))
    D = f64(tensors[prefix + "D"])
    y = torch.zeros(T, heads, P, dtype=F64)
    for head in range(heads):
        g = head // (heads // G)
        y[:, head] = ssm_recurrence(x[:, head], B[:, g], C[:, g], dt[:, head], a[head], D[head])
    y = y.reshape(T, inner) * silu(z)
    y = grouped_rms_norm(y, tensors[prefix + "norm"], int(mixer["norm_groups"]), eps)
    return linear(y, tensors[prefix + "o"])


# ---------------------------------------------------------------------------- feed-forward
def clamped_feed_forward(h, tensors, prefix, limit):
    g = torch.clamp(linear(h, tensors[prefix + "gate"]), max=limit)
    u = torch.clamp(linear(h, tensors[prefix + "up"]), min=-limit, max=limit)
    return linear(g * sigmoid(1.702 * g) * (u + 1.0), tensors[prefix + "down"])


def routed_feed_forward(h, tensors, prefix, experts, top, margins=None):
    """Every token runs its `top` experts with the largest router logits, weighted by the
    softmax over those logits alone.  `margins` (optional, a list) receives, per token, the gap
    between the smallest chosen logit and the largest one that was not chosen."""
    logits = linear(h, tensors[prefix + "router"])
    T = h.shape[0]
    out = torch.zeros(T, tensors[prefix + "e0.down"].shape[0], dtype=F64)
    if margins is not None:
        ordered = torch.sort(logits, dim=1, descending=True).values
        margins.append(ordered[:, top - 1] - ordered[:, top] if top < experts
                       else torch.full((T,), float("inf"), dtype=F64))
    for t in range(T):
        chosen = torch.topk(logits[t], top).indices
        weights = torch.softmax(logits[t][chosen], dim=0)
        for weight, expert in zip(weights, chosen.tolist()):
            name = f"{prefix}e{expert}."
            x = f64(h[t])
            act = silu(linear(x, tensors[name + "gate"])) * linear(x, tensors[name + "up"])
            out[t] += weight * linear(act, tensors[name + "down"])
    return out


def feed_forward(h, tensors, prefix, mlp, margins=None):
    if mlp["kind"] == "dense":
        return clamped_feed_forward(h, tensors, prefix, float(mlp["limit"]))
    return routed_feed_forward(h, tensors, prefix, int(mlp["router"]["experts"]),
                               int(mlp["router"]["top"]), margins)


# ---------------------------------------------------------------------------- the model
def forward(cfg, tensors, tokens, streams=None, margins=None):
    """Logits [T, vocab] (float64) of one sequence from position 0.  `streams`: a list that
    receives the residual stream after every layer; `margins`: a list that receives, for every
    routed feed-forward, each token's gap between its last chosen and its first unchosen
    router logit (a token whose gap is tiny may be routed otherwise by any rounding)."""
    eps = float(cfg["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.shape[0]
    positions = torch.arange(T)
    x = rms_norm(f64(tensors["embed"])[tokens], tensors["embed.norm"], eps)
    first_values = None
    for index, layer in enumerate(cfg["layers"]):
        prefix = f"l{index}."
        h = rms_norm(x, tensors[prefix + "norm1"], eps)
        if layer["type"] == "attention":
            mixes = bool(layer["mixer"].get("v_mix"))
            out, raw = attention_mixer(h, tensors, prefix + "mix.", layer["mixer"], eps, positions,
                                       first_values if mixes else None)
            if mixes and first_values is None:
                first_values = raw
        elif layer["type"] == "mamba2":
            out = mamba2_mixer(h, tensors, prefix + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        x = x + out
        if layer.get("mlp"):
            h = rms_norm(x, tensors[prefix + "norm2"], eps)
            x = x + feed_forward(h, tensors, prefix + "mlp.", layer["mlp"], margins)
        if streams is not None:
            streams.append(x.clone())
    h = rms_norm(x, tensors["final.norm"], eps)
    logits = linear(h, tensors["embed"]) * float(cfg.get("logit_scale", 1.0))
    cap = cfg.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return logits


def clear_rows(cfg, tensors, tokens, least, carry=False):
    """(logits, mask): the logits of `forward`, and at which positions no routing decision was
    closer than `least`; with `carry`, no decision up to and including them (a choice that a
    rounding flips at one token also reaches the tokens after it, through the mixers, if far
    more weakly)."""
    margins = []
    logits = forward(cfg, tensors, tokens, margins=margins)
    clear = torch.ones(logits.shape[0], dtype=torch.bool)
    for gaps in margins:
        clear &= (torch.cummin(gaps, dim=0).values if carry else gaps) > least
    return logits, clear


def greedy(cfg, tensors, prompt, count):
    sequence = list(prompt)
    for _ in range(count):
        sequence.append(int(forward(cfg, tensors, sequence)[-1].argmax()))
    return sequence[len(prompt):]
