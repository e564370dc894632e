"""Gopuzen models of drawn sizes against the plain implementation: every size, option and the
order of the layers come from a seeded generator, so that nothing rests on the sizes of the
hand-made configurations.  Per model: whole prompts, a prompt cut into portions, a batch of
unequal requests decoded together, in float32; and the twin that routes nothing in bfloat16."""
import random

import pytest
import torch

import plain_gopuzen as plain
from helpers import assert_close_bf16, assert_close_f32
from gopuzen_helpers import (attention, dense, dense_twin, ids, model, moe, parallel,
                             sharp_weights, write_folder)

pytestmark = pytest.mark.gpu
SEEDS = list(range(40))


def drawn_config(seed):
    rng = random.Random(3000 + seed)
    width = rng.choice([32, 40, 64, 72, 96, 128, 256])
    vocab = rng.randint(20, 300)
    layers, sources = [], []          # sources: (index, layer) of attention layers with own keys
    for index in range(rng.randint(1, 6)):
        kind = rng.random()
        if kind < 0.25:
            mlp = None
        elif kind < 0.6:
            mlp = dense(rng.choice([16, 24, 56, 64, 100, 128]))
        else:
            experts = rng.choice([2, 3, 4, 8, 16, 33])
            identity = rng.choice([0, 0, 1, 2, 4])
            mlp = moe(rng.choice([8, 24, 64, 96, 128]), experts,
                      rng.randint(1, min(experts + identity, 4)), identity)
        if rng.random() < 0.5:
            kv_heads = rng.choice([1, 2, 3, 4])
            heads = kv_heads * rng.choice([1, 2, 4, 5])
            dim = rng.choice([8, 16, 24, 32, 64, 64, 128])
            vdim = dim if rng.random() < 0.4 else rng.choice([8, 16, 32, 48, 64])
            q_temp = None if rng.random() < 0.3 else (rng.choice([0.1, 0.3, 0.5]), rng.choice([1, 4, 16, 50]))
            r_heads = rng.choice([1, 2, 3, 4, 6])
            r_dim = rng.choice([4, 8, 16, 32, 48, 64, 128])
            r_vdim = rng.choice([8, 16, 24, 32, 64, 72, 128])
            decay = [rng.choice([1.0, 0.999, 0.97, 0.9, 0.6, 0.2]) for _ in range(r_heads)]
            layers.append(parallel((heads, kv_heads, dim, vdim, rng.choice([0.1, 0.125, 0.25, 0.4]), q_temp),
                                   (r_heads, r_dim, r_vdim, decay), mlp))
            continue
        if sources and rng.random() < 0.4:       # reads an earlier layer's keys, with a mask of its own
            source, other = rng.choice(sources)
            m = other["mixer"]
            kv_heads, dim, vdim = m["kv_heads"], m["dim"], m["vdim"]
            rot = None if "rot" not in m else (m["rot"]["base"], m["rot"]["dims"])
            kv_from = source
        else:
            kv_heads = rng.choice([1, 2, 3, 4])
            dim = rng.choice([8, 16, 24, 32, 64, 64, 128])
            vdim = dim if rng.random() < 0.5 else rng.choice([8, 16, 32, 48, 64])
            rot = None
            if rng.random() < 0.8:
                rot = (rng.choice([100.0, 10000.0, 250000.0]),
                       rng.choice([d for d in (2, 4, 8, 16, 32, dim) if d <= dim]))
            kv_from = None
        heads = kv_heads * rng.choice([1, 2, 4, 5])
        window = rng.choice([None, 1, 2, 17, 63, 64, 65, 100])
        mask = None
        if window is not None:
            mask = (window,) if rng.random() < 0.2 else (window, rng.choice([1, 2, 5, 12, 16, 64, 70]))
        layer = attention(heads, kv_heads, dim, vdim, rng.choice([0.1, 0.125, 0.25, 0.4]), mask, rot,
                          mlp, kv_from=kv_from)
        if kv_from is None:
            sources.append((index, layer))
        layers.append(layer)
    return model(vocab, width, rng.choice([1e-5, 1e-6]), rng.choice([1.0, 0.5, 4.0, 16.0]),
                 rng.choice([1, 2, 3, 4]), layers)


def run_all(cfg, tensors, dtype, folder, margin):
    import edge_infer_amd as ei
    vocab = cfg["vocab"]
    requests = [ids(vocab, n, 50 + n) for n in (150, 1, 37)]
    refs = [plain.clear_rows(cfg, tensors, r, margin, carry=True) for r in requests]
    model_ = ei.load_model(write_folder(folder, cfg, tensors), dtype=dtype)
    session = ei.Session(model_, max_tokens=64 * 8, max_seqs=3)

    def close(got, want, clear, what):
        if clear.sum() == 0:
            return
        got, want = got[clear.to(got.device)], want[clear]
        if dtype == "float32":
            assert_close_f32(got, want, what)
        else:
            # (bfloat16's roundings add up like a random walk over the layers: the bound of the
            # hand-made models, which have four or five, grows with the root of the depth)
            deeper = max(1.0, len(cfg["layers"]) / 5.0) ** 0.5
            assert_close_bf16(got, want, what, rms_rel=4e-2 * deeper, max_rel=12e-2 * deeper)
    # whole, and in portions
    slot = session.begin()
    close(session.step([(slot, requests[0], list(range(150)))]), *refs[0], "whole")
    session.end(slot)
    slot = session.begin()
    rows, at = [], 0
    for take in (2, 3, 60, 1, 70, 14):
        rows.append(session.step([(slot, requests[0][at:at + take], list(range(take)))]))
        at += take
    close(torch.cat(rows), *refs[0], "portions")
    session.end(slot)
    # a batch of unequal requests that start together and are decoded together
    slots = [session.begin() for _ in requests]
    cuts = [max(1, len(r) - 12) for r in requests]
    got = [[] for _ in requests]
    logits = session.step([(slots[i], requests[i][:cuts[i]], [cuts[i] - 1]) for i in range(3)])
    for i in range(3):
        got[i].append(logits[i:i + 1])
    at = list(cuts)
    live = [i for i in range(3) if at[i] < len(requests[i])]
    while live:
        logits = session.step([(slots[i], [requests[i][at[i]]], [0]) for i in live])
        for row, i in enumerate(live):
            got[i].append(logits[row:row + 1])
            at[i] += 1
        live = [i for i in live if at[i] < len(requests[i])]
    for i in range(3):
        want, clear = refs[i]
        close(torch.cat(got[i]), want[cuts[i] - 1:], clear[cuts[i] - 1:], f"request {i} of the batch")
    session.cache.check()


@pytest.mark.parametrize("seed", SEEDS)
def test_drawn_model_in_float32(seed, tmp_path):
    cfg = drawn_config(seed)
    run_all(cfg, sharp_weights(cfg, seed=seed), "float32", tmp_path / "m", 1e-4)


@pytest.mark.parametrize("seed", SEEDS)
def test_drawn_twin_in_bfloat16(seed, tmp_path):
    cfg = dense_twin(drawn_config(seed))
    run_all(cfg, sharp_weights(cfg, seed=seed), "bfloat16", tmp_path / "m", 0.05)
