"""The mechanisms of the Vafepel layers alone, each against its plain function: the row-wise
kernels (the norm on the stream itself, the output gate, scaled and capped logits, the clamped
swish), the store kernel (norms, rotation from rescaled frequencies at far positions, values of
their own width, values mixed across layers), attention with keys made to stand out just
inside and just outside the window and far back, and a sink that weighs, the state-space
mixer's kernels and the mixer in portions, token by token, in batches and with slots used
again, the router's choices (ties included) and the experts."""
import math

import pytest
import torch

import plain_vafepel as plain
from helpers import assert_close_bf16, assert_close_f32

pytestmark = pytest.mark.gpu
DEV = "cuda"
HIDDEN, VOCAB, EPS = 48, 31, 1e-5


def one_layer(mixer, ffn=None):
    from edge_infer_amd.config.specs import LayerSpec, ModelSpec, NormSpec, default_schedule
    norm = NormSpec(eps=EPS)
    return ModelSpec(architecture="test", vocab_size=VOCAB, hidden_size=HIDDEN,
                     layers=(LayerSpec(block="prenorm", norm=norm, mixer=mixer, feed_forward=ffn),),
                     schedule=default_schedule(1), final_norm=norm, tie_word_embeddings=False,
                     max_position_embeddings=1 << 20, bos_token_id=None, eos_token_id=None)


def params_for(spec, seed):
    """Order-one parameters by parameter path, float32 values that bfloat16 holds exactly."""
    from edge_infer_amd.engine.model import model_parameters
    g = torch.Generator().manual_seed(seed)
    out = {}
    for path, param in model_parameters(spec).items():
        if param.optional and not path.endswith("value_mix"):
            continue
        shape = tuple(param.shape)
        if param.init == "norm":
            value = 1 + 0.2 * (torch.rand(shape, generator=g) - 0.5)
        elif param.init == "uniform":
            value = param.low + (param.high - param.low) * torch.rand(shape, generator=g)
        elif len(shape) == 2:
            value = torch.randn(shape, generator=g) / shape[1] ** 0.5
        else:
            value = torch.randn(shape, generator=g) * 0.5
        out[path] = value.to(torch.bfloat16).float()
    return out


def session_for(spec, params, dtype="float32", max_tokens=1024, max_seqs=4):
    from edge_infer_amd.engine import DecoderModel, Session
    model = DecoderModel(spec, params, dtype, DEV)
    return model, Session(model, max_tokens=max_tokens, max_seqs=max_seqs, graphs=False)


def run_part(session, part, pieces):
    """`pieces`: (slot, start, x rows) per sequence of one step; the part's output rows."""
    from edge_infer_amd.config.specs import ScheduleEntry
    from edge_infer_amd.engine.batch import SeqStep
    seqs = [SeqStep(slot=slot, start=start, tokens=[0] * x.shape[0]) for slot, start, x in pieces]
    session.cache.grow([(s.slot, s.start + s.count) for s in seqs])
    ctx, _ = session.context_for(seqs)
    rows = torch.cat([x for _, _, x in pieces]).contiguous().to(DEV).to(session.dtype)
    out = part.forward(ctx, rows, ScheduleEntry(0, 0))
    if out.dim() == 3:
        out = out.sum(0)
    out = out.float().clone()
    session.cache.commit([(s.slot, s.start + s.count) for s in seqs])
    return out


def in_cuts(session, part, x, cuts, slot=None):
    """The rows of `x` through the part in steps of the given sizes, as one sequence."""
    own = slot is None
    slot = session.begin() if own else slot
    rows, at = [], 0
    for take in cuts:
        rows.append(run_part(session, part, [(slot, at, x[at:at + take])]))
        at += take
    assert at == x.shape[0]
    if own:
        session.end(slot)
    return torch.cat(rows)


def mixer_tensors(params, names):
    """The mixer's parameters under the oracle's (checkpoint) names."""
    pre = "layers.0.mixer."
    return {"m." + names[k[len(pre):]]: v for k, v in params.items()
            if k.startswith(pre) and k[len(pre):] in names}


# -- row-wise kernels -------------------------------------------------------------------
@pytest.mark.parametrize("width", [48, 1000, 4100])
def test_norm_on_the_stream_itself(width):
    from edge_infer_amd.csrc import lib
    torch.manual_seed(width)
    x = torch.randn(7, width, device=DEV) * 3
    w = 1 + 0.1 * torch.randn(width, device=DEV)
    want = plain.rms_norm(x.cpu(), w.cpu(), 1e-3)
    lib.norm_rows(x, w, 1e-3)
    assert_close_f32(x, want, "norm_rows")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("slices", [1, 3])
def test_output_gate(dtype, slices):
    """out *= sigmoid(columns of the fused projection), also from float32 slices."""
    from edge_infer_amd.csrc import lib
    torch.manual_seed(3)
    rows, width, first, stride = 9, 40, 56, 112
    out = torch.randn(rows, width, device=DEV).to(dtype)
    if slices > 1:
        proj = torch.randn(slices, rows, stride, device=DEV)
        gate = proj.sum(0)
    else:
        proj = (torch.randn(rows, stride, device=DEV) * 2).to(dtype)
        gate = proj.float()
    want = out.double().cpu() * plain.sigmoid(gate[:, first:first + width].double().cpu())
    lib.gate_rows(proj, first, out)
    if dtype == torch.float32:
        assert_close_f32(out, want, "gate_rows")
    else:
        assert_close_bf16(out, want, "gate_rows")


def test_scaled_and_capped_logits():
    from edge_infer_amd.csrc import lib
    torch.manual_seed(4)
    x = torch.randn(5, 333, device=DEV) * 20
    want = 9.0 * torch.tanh(x.double().cpu() * 2.5 / 9.0)
    capped = x.clone()
    lib.scale_cap(capped, 2.5, 9.0)
    assert_close_f32(capped, want, "scale and cap")


def test_scale_alone():
    from edge_infer_amd.csrc import lib
    x = torch.linspace(-50, 50, 1001, device=DEV).reshape(1, -1).contiguous()
    want = x.double().cpu() * 0.3
    lib.scale_cap(x, 0.3, None)
    assert_close_f32(x, want, "scale alone")


@pytest.mark.parametrize("inter, strip", [(24, 0), (32, 16), (50, 0)])
def test_clamped_swish(inter, strip):
    """g = min(gate, limit), u = clamp(up, -limit, limit): g sigmoid(alpha g) (u + 1); values far
    beyond the limits on both sides."""
    from edge_infer_amd.csrc import lib
    torch.manual_seed(inter)
    rows, limit, alpha = 6, 1.25, 1.702
    gate = torch.randn(rows, inter) * 3
    up = torch.randn(rows, inter) * 3
    g = gate.double().clamp(max=limit)
    want = g * plain.sigmoid(alpha * g) * (up.double().clamp(-limit, limit) + 1.0)
    if strip:
        both = torch.stack([gate.reshape(rows, -1, strip), up.reshape(rows, -1, strip)], dim=2)
        both = both.reshape(rows, 2 * inter)
    else:
        both = torch.cat([gate, up], dim=1)
    out = torch.empty(rows, inter, device=DEV)
    lib.swiglu(both.to(DEV).contiguous(), out, strip, "clamped_swish", limit=limit, alpha=alpha)
    assert_close_f32(out, want, "clamped swish")
    assert (gate > limit).any() and (up < -limit).any() and (up > limit).any()


# -- the store kernel ---------------------------------------------------------------------
def test_rescaled_frequencies_follow_the_three_cases():
    from edge_infer_amd.config.specs import FrequencyScaling, PositionSpec
    from edge_infer_amd.parts.rope import scaled_frequencies
    rot = {"base": 10000.0, "dims": 32, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0,
                                                     "original": 256}}
    spec = PositionSpec(kind="rope_half", theta=10000.0, dim=32,
                        scaling=FrequencyScaling(8.0, 1.0, 4.0, 256.0))
    got, want = scaled_frequencies(spec), plain.rotary_frequencies(rot)
    assert torch.allclose(got, want, rtol=1e-12, atol=0)
    plainf = plain.rotary_frequencies({"base": 10000.0, "dims": 32})
    kept = (want == plainf).sum().item()
    divided = torch.isclose(want, plainf / 8.0, rtol=1e-12).sum().item()
    assert kept >= 2 and divided >= 2 and kept + divided < 16      # all three cases occur


@pytest.mark.parametrize("heads, kv_heads, dim, vdim, rot_dims", [
    (4, 2, 16, 24, 8), (3, 3, 10, 7, 10), (2, 1, 72, 8, 2), (5, 1, 12, 40, 0),
    # sizes that take the kernel's form in 16-byte pieces (the rows then go on by 16 columns)
    (4, 2, 64, 32, 16), (2, 2, 128, 128, 64), (3, 1, 24, 40, 0), (6, 3, 48, 8, 48)])
@pytest.mark.parametrize("slices", [1, 2])
def test_store_kernel(heads, kv_heads, dim, vdim, rot_dims, slices):
    """Queries out, keys and values in their pages: per-head norms, rotation of the first
    rot_dims elements at positions up to a million, values mixed with an earlier layer's, from
    rows that go on after the values (by 13 columns, or by 16 where all sizes are multiples
    of 8)."""
    from edge_infer_amd.csrc import lib
    torch.manual_seed(heads * 100 + dim)
    n_pages, tail = 10, (16 if dim % 8 == 0 and vdim % 8 == 0 else 13)
    qw, kw, vw = heads * dim, kv_heads * dim, kv_heads * vdim
    far = torch.tensor([0, 1, 63, 64, 65, 130, 1000000, 99999, 255, 300])     # the rows' positions
    n = far.numel()
    proj = torch.randn(slices, n, qw + kw + vw + tail)
    q_norm, k_norm = 1 + 0.3 * torch.randn(dim), 1 + 0.3 * torch.randn(dim)
    freqs = None
    rot = None
    if rot_dims:
        rot = {"base": 300.0, "dims": rot_dims,
               "scaling": {"factor": 3.0, "low": 1.0, "high": 5.0, "original": 40}}
        freqs = plain.rotary_frequencies(rot).to(DEV)
    rows = proj.double().sum(0)
    q = plain.rotate(plain.rms_norm(rows[:, :qw].reshape(n, heads, dim), q_norm, EPS), far, rot)
    k = plain.rotate(plain.rms_norm(rows[:, qw:qw + kw].reshape(n, kv_heads, dim), k_norm, EPS), far, rot)
    v = rows[:, qw + kw:qw + kw + vw].reshape(n, kv_heads, vdim)
    first = torch.randn(n, vw)
    # one sequence; the pages its rows fall into lie in a shuffled order among the few pages
    # the test holds
    table_width = int(far.max()) // 64 + 1
    page_table = torch.zeros(1, table_width, dtype=torch.int32)
    for index, logical in enumerate(sorted({int(p) // 64 for p in far})):
        page_table[0, logical] = (index * 3 + 2) % n_pages
    slot_of = [(int(page_table[0, int(far[r]) // 64]), int(far[r]) % 64) for r in range(n)]
    assert len(set(slot_of)) == n
    for mode, lam in ((0, None), (1, None), (2, 0.3125)):
        k_pages = torch.zeros(n_pages, kv_heads, 64, dim, device=DEV)
        v_pages = torch.zeros(n_pages, kv_heads, 64, vdim, device=DEV)
        q_out = torch.empty(n, qw, device=DEV)
        v_first = first.clone().to(DEV)
        lib.head_store(proj.to(DEV) if slices > 1 else proj[0].contiguous().to(DEV) * 1.0,
                       q_norm.to(DEV), k_norm.to(DEV), EPS, freqs, far.int().to(DEV),
                       torch.zeros(n, dtype=torch.int32, device=DEV), page_table.to(DEV), q_out,
                       k_pages, v_pages, heads, kv_heads, dim, vdim, v_first=v_first, v_mode=mode,
                       v_lambda=None if lam is None else torch.tensor([lam], device=DEV))
        if slices == 1:      # (the single slice is the first one alone)
            single = proj[0].double()
            q = plain.rotate(plain.rms_norm(single[:, :qw].reshape(n, heads, dim), q_norm, EPS), far, rot)
            k = plain.rotate(plain.rms_norm(single[:, qw:qw + kw].reshape(n, kv_heads, dim), k_norm, EPS), far, rot)
            v = single[:, qw + kw:qw + kw + vw].reshape(n, kv_heads, vdim)
        assert_close_f32(q_out, q.reshape(n, qw), f"queries, mode {mode}")
        got_k = torch.stack([k_pages[p, :, s] for p, s in slot_of])
        got_v = torch.stack([v_pages[p, :, s] for p, s in slot_of])
        assert_close_f32(got_k, k, f"keys, mode {mode}")
        want_v = v if mode != 2 else (1 - lam) * v + lam * first.double().reshape(n, kv_heads, vdim)
        assert_close_f32(got_v, want_v, f"values, mode {mode}")
        if mode == 1:
            assert_close_f32(v_first, v.reshape(n, vw), "the values kept for later layers")
        else:
            assert torch.equal(v_first.cpu(), first)
        assert k_pages.abs().sum().item() == pytest.approx(got_k.abs().sum().item(), rel=1e-5)


# -- attention ----------------------------------------------------------------------------
ATTENTION_NAMES = {"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v",
                   "q_norm.weight": "q.norm", "k_norm.weight": "k.norm", "sink": "sink",
                   "value_mix": "vmix", "gate_proj.weight": "g", "o_proj.weight": "o"}


def attention_spec(rot=None, **kw):
    from edge_infer_amd.config.specs import AttentionSpec, FrequencyScaling, PositionSpec
    position = PositionSpec(kind="none")
    if rot is not None:
        stretch = rot.get("scaling")
        position = PositionSpec(kind="rope_half", theta=rot["base"], dim=rot["dims"],
                                scaling=None if stretch is None else FrequencyScaling(
                                    stretch["factor"], stretch["low"], stretch["high"],
                                    stretch["original"]))
    return AttentionSpec(qk_norm=True, qk_norm_eps=EPS, qkv_bias=False, o_bias=False, sink=True,
                         output_gate=True, value_mix="off", position=position, **kw)


def plain_attention(params, spec, rot, x, start=0):
    mixer = {"heads": spec.n_heads, "kv_heads": spec.n_kv_heads, "dim": spec.head_dim,
             "vdim": spec.v_dim, "scale": spec.scale, "v_mix": False}
    if spec.window is not None:
        mixer["mask"] = {"size": spec.window}
    if rot is not None:
        mixer["rot"] = rot
    out, _ = plain.attention_mixer(x, mixer_tensors(params, ATTENTION_NAMES), "m.", mixer, EPS,
                                   torch.arange(start, start + x.shape[0]), None)
    return out


@pytest.mark.parametrize("shape", [
    dict(n_heads=4, n_kv_heads=2, head_dim=16, value_dim=24, window=20, scale=0.3),
    dict(n_heads=6, n_kv_heads=1, head_dim=10, value_dim=6, window=None, scale=0.4),
    dict(n_heads=2, n_kv_heads=2, head_dim=64, value_dim=64, window=70, scale=0.15),
    dict(n_heads=8, n_kv_heads=2, head_dim=64, value_dim=64, window=None, scale=0.125)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_alone(shape, dtype):
    """Whole, in portions down to two tokens and token by token; head size 64 with values as
    wide takes the matrix-core kernels in bfloat16."""
    rot = {"base": 200.0, "dims": min(shape["head_dim"], 12),
           "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 32}}
    mixer = attention_spec(rot=rot, **shape)
    spec = one_layer(mixer)
    params = params_for(spec, seed=5)
    model, session = session_for(spec, params, dtype)
    part = model.layers[0].mixer
    torch.manual_seed(8)
    T = 150
    x = torch.randn(T, HIDDEN).to(torch.bfloat16).float()
    want = plain_attention(params, mixer, rot, x.double())
    for cuts in ([T], [2] * 10 + [T - 20], [63, 2, 65, 20], [T - 40] + [1] * 40):
        got = in_cuts(session, part, x, cuts)
        if dtype == "float32":
            assert_close_f32(got, want, f"attention {shape}, cuts {cuts[:3]}")
        else:
            assert_close_bf16(got, want, f"attention {shape}, cuts {cuts[:3]}", rms_rel=2e-2,
                              max_rel=4e-2)


@pytest.mark.parametrize("dtype, dim", [("float32", 16), ("bfloat16", 64), ("bfloat16", 16)])
@pytest.mark.parametrize("window", [5, 64, 65, 100])
def test_keys_that_stand_out_at_the_windows_edge(window, dtype, dim):
    """The key just outside the window of the last position is made to dominate (its input is
    a multiple of the query's, and the keys are made with the queries' matrix and norm, so its
    score is a large positive number): the engine must not see it.  Then the key just inside.
    In prompts, in portions that end at the edge, and decoded."""
    mixer = attention_spec(n_heads=2, n_kv_heads=2, head_dim=dim, value_dim=dim if dim == 64 else 8,
                           window=window, scale=0.5 if dim == 16 else 0.2)
    spec = one_layer(mixer)
    params = params_for(spec, seed=9)
    pre = "layers.0.mixer."
    params[pre + "k_proj.weight"] = params[pre + "q_proj.weight"].clone()
    params[pre + "k_norm.weight"] = params[pre + "q_norm.weight"].clone()
    model, session = session_for(spec, params, dtype)
    part = model.layers[0].mixer
    torch.manual_seed(6)
    T = 180
    base = (0.3 * torch.randn(T, HIDDEN)).to(torch.bfloat16).float()
    for offset, seen in ((window, False), (window - 1, True)):
        x = base.clone()
        x[T - 1 - offset] = 4.0 * x[T - 1]
        x = x.to(torch.bfloat16).float()
        want = plain_attention(params, mixer, None, x.double())
        calm = x.clone()
        calm[T - 1 - offset] = base[T - 1 - offset]
        quiet = plain_attention(params, mixer, None, calm.double())
        moved = (want[-1] - quiet[-1]).abs().max().item() / want[-1].abs().max().item()
        assert (moved > 0.1) == seen, f"the test's key does not stand out as meant ({moved:.2e})"
        for cuts in ([T], [T - 1, 1], [T - offset - 1, 1, offset], [T - 30] + [1] * 30):
            got = in_cuts(session, part, x, cuts)
            what = f"window {window}, key at distance {offset}, cuts {cuts[:3]}"
            if dtype == "float32":
                assert_close_f32(got, want, what)
            else:
                assert_close_bf16(got, want, what, rms_rel=2e-2, max_rel=4e-2)


def test_a_far_key_among_hundreds_and_the_sink():
    """Position 3 of 700 repeats the last position's input and the layer has no window, so that
    key takes a weight that shows; with the sink left out, or the far key, the oracle's own
    output moves by much more than the tolerance."""
    rot = {"base": 1e8, "dims": 4}
    mixer = attention_spec(rot=rot, n_heads=2, n_kv_heads=1, head_dim=16, value_dim=12, window=None,
                           scale=0.6)
    spec = one_layer(mixer)
    params = params_for(spec, seed=13)
    pre = "layers.0.mixer."
    params[pre + "k_proj.weight"] = params[pre + "q_proj.weight"][:16].clone()
    params[pre + "k_norm.weight"] = params[pre + "q_norm.weight"].clone()
    params[pre + "sink"] = torch.tensor([9.0, 9.0])
    model, session = session_for(spec, params, max_tokens=1024)
    part = model.layers[0].mixer
    torch.manual_seed(10)
    T = 700
    x = torch.randn(T, HIDDEN).to(torch.bfloat16).float()
    x[3] = x[T - 1]
    want = plain_attention(params, mixer, rot, x.double())
    other = x.clone()
    other[3] = x[4]
    moved = (plain_attention(params, mixer, rot, other.double())[-1] - want[-1]).abs().max() / want[-1].abs().max()
    assert moved > 0.05, f"the far key does not show ({moved:.2e})"
    no_sink = dict(params)
    no_sink[pre + "sink"] = torch.tensor([-30.0, -30.0])
    moved = (plain_attention(no_sink, mixer, rot, x.double())[-1] - want[-1]).abs().max() / want[-1].abs().max()
    assert moved > 0.05, f"the sink does not show ({moved:.2e})"
    for cuts in ([T], [T - 1, 1], [2, 2, 300, T - 304 - 40] + [1] * 40):
        got = in_cuts(session, part, x, cuts)
        assert_close_f32(got, want, f"far key, cuts {cuts[:4]}")


# -- the state-space mixer ------------------------------------------------------------------
SSM_NAMES = {"in_proj.weight": "in", "conv.weight": "conv", "conv.bias": "conv.b",
             "dt_bias": "dt_bias", "a_log": "A_log", "skip": "D", "out_norm.weight": "norm",
             "o_proj.weight": "o"}


def ssm_spec(**kw):
    from edge_infer_amd.config.specs import StateSpaceSpec
    return StateSpaceSpec(norm_eps=EPS, **kw)


def plain_ssm(params, spec, x):
    mixer = {"heads": spec.n_heads, "vdim": spec.head_dim, "state": spec.state,
             "groups": spec.groups, "conv": spec.conv_taps, "norm_groups": spec.norm_parts}
    return plain.mamba2_mixer(x, mixer_tensors(params, SSM_NAMES), "m.", mixer, EPS)


@pytest.mark.parametrize("shape", [
    dict(n_heads=4, head_dim=12, state=16, groups=2, conv_taps=4, norm_parts=2),
    dict(n_heads=3, head_dim=5, state=19, groups=1, conv_taps=1, norm_parts=1),
    dict(n_heads=6, head_dim=40, state=130, groups=3, conv_taps=7, norm_parts=4),
    dict(n_heads=2, head_dim=300, state=8, groups=2, conv_taps=2, norm_parts=3),
    dict(n_heads=2, head_dim=8, state=1024, groups=1, conv_taps=3, norm_parts=1),
    dict(n_heads=4, head_dim=16, state=272, groups=2, conv_taps=4, norm_parts=2)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_state_space_mixer_alone(shape, dtype):
    """Whole, in portions shorter than the convolution and down to two tokens, token by token."""
    mixer = ssm_spec(**shape)
    spec = one_layer(mixer)
    params = params_for(spec, seed=15)
    model, session = session_for(spec, params, dtype)
    part = model.layers[0].mixer
    torch.manual_seed(18)
    T = 120
    x = torch.randn(T, HIDDEN).to(torch.bfloat16).float()
    want = plain_ssm(params, mixer, x.double())
    for cuts in ([T], [2, 1, 2, 3, 16, 17, T - 41], [T - 30] + [1] * 30, [1, T - 1]):
        got = in_cuts(session, part, x, cuts)
        if dtype == "float32":
            assert_close_f32(got, want, f"state space {shape}, cuts {cuts[:4]}")
        else:
            assert_close_bf16(got, want, f"state space {shape}, cuts {cuts[:4]}", rms_rel=2e-2,
                              max_rel=5e-2)


def test_state_space_in_batches_with_slots_used_again():
    """Three sequences of unequal lengths advance together, one ends and its slot is taken by a
    new sequence, whose state starts at zero whatever the slot held."""
    mixer = ssm_spec(n_heads=4, head_dim=8, state=24, groups=2, conv_taps=3, norm_parts=2)
    spec = one_layer(mixer)
    params = params_for(spec, seed=16)
    model, session = session_for(spec, params, max_seqs=3)
    part = model.layers[0].mixer
    torch.manual_seed(19)
    xs = [torch.randn(n, HIDDEN).to(torch.bfloat16).float() for n in (70, 9, 33, 50)]
    wants = [plain_ssm(params, mixer, x.double()) for x in xs]
    slots = [session.begin() for _ in range(3)]
    got = [[], [], [], []]
    out = run_part(session, part, [(slots[0], 0, xs[0][:40]), (slots[1], 0, xs[1][:9]),
                                   (slots[2], 0, xs[2][:1])])
    got[0].append(out[:40]); got[1].append(out[40:49]); got[2].append(out[49:])
    session.end(slots[1])
    again = session.begin()
    assert again == slots[1]
    out = run_part(session, part, [(slots[2], 1, xs[2][1:33]), (again, 0, xs[3][:2]),
                                   (slots[0], 40, xs[0][40:41])])
    got[2].append(out[:32]); got[3].append(out[32:34]); got[0].append(out[34:])
    for t in range(41, 70):
        out = run_part(session, part, [(slots[0], t, xs[0][t:t + 1]), (again, t - 39, xs[3][t - 39:t - 38])])
        got[0].append(out[:1]); got[3].append(out[1:])
    out = run_part(session, part, [(again, 31, xs[3][31:])])
    got[3].append(out)
    for index in range(4):
        assert_close_f32(torch.cat(got[index]), wants[index], f"sequence {index}")


def test_state_space_kernels_one_by_one():
    """The convolution with its tail, the scan with a state that is carried, and the gated norm
    in parts, each against its own plain function."""
    from edge_infer_amd.csrc import lib
    torch.manual_seed(21)
    shape = lib.SsmShape(heads=3, groups=1, head_dim=6, state=20, taps=4)
    n, first = 11, 5          # a sequence's rows 5..10 follow rows 0..4 of an earlier step
    proj = torch.randn(n, shape.proj_width)
    conv_w, conv_b = torch.randn(shape.channels, 4) * 0.5, torch.randn(shape.channels) * 0.2
    a_log, dt_bias, skip = torch.rand(3) - 1.0, torch.rand(3) - 2.0, 1 + 0.2 * torch.randn(3)
    xbc = proj[:, shape.inner:shape.inner + shape.channels].double()
    conv_want = plain.silu(plain.causal_conv(xbc, conv_w, conv_b))
    x = conv_want[:, :shape.inner].reshape(n, 3, 6)
    B, C = conv_want[:, shape.inner:shape.inner + 20], conv_want[:, shape.inner + 20:]
    dt = plain.softplus(proj[:, -3:].double() + dt_bias.double())
    y_want = torch.stack([plain.ssm_recurrence(x[:, h], B, C, dt[:, h], torch.exp(a_log[h].double()),
                                               skip[h].double()) for h in range(3)], dim=1)
    state = torch.zeros(4, shape.state_floats, device=DEV)      # rows 0/1: the two versions
    meta = lambda *v: torch.tensor(v, dtype=torch.int32, device=DEV)
    conv = torch.empty(n, shape.channels, device=DEV)
    y = torch.empty(n, shape.inner, device=DEV)
    pieces = ((0, first, 0, 1), (first, n - first, 1, 0))       # (row0, count, version in, version out)
    for row0, count, v_in, v_out in pieces:
        part = proj[row0:row0 + count].contiguous().to(DEV)
        pos = torch.arange(row0, row0 + count, dtype=torch.int32, device=DEV)
        seq = torch.zeros(count, dtype=torch.int32, device=DEV)
        lib.ssm_conv(part, conv_w.to(DEV), conv_b.to(DEV), state, shape, pos, seq, meta(v_in),
                     meta(v_out), meta(row0), meta(count), meta(0), conv[row0:row0 + count])
        lib.ssm_scan(conv[row0:row0 + count], part, a_log.to(DEV), dt_bias.to(DEV), skip.to(DEV),
                     state, shape, meta(v_in), meta(v_out), meta(count), meta(0), y[row0:row0 + count])
    assert_close_f32(conv, conv_want, "convolution over two steps")
    assert_close_f32(y, y_want.reshape(n, -1), "scan over two steps")
    tail = state[0, shape.inner * shape.state:].reshape(3, shape.channels)
    assert_close_f32(tail, xbc[-3:], "the tail after the last step")
    norm_w = 1 + 0.2 * torch.randn(shape.inner)
    out = torch.empty(n, shape.inner, device=DEV)
    lib.ssm_out(y, proj.to(DEV), norm_w.to(DEV), EPS, shape, 3, torch.zeros(n, dtype=torch.int32, device=DEV), out)
    gated = y_want.reshape(n, -1) * plain.silu(proj[:, :shape.inner].double())
    assert_close_f32(out, plain.grouped_rms_norm(gated, norm_w, 3, EPS), "gate, then the norm in parts")


# -- the routed feed-forward --------------------------------------------------------------------
@pytest.mark.parametrize("experts, top, width", [(6, 2, 48), (70, 4, 100), (3, 1, 50), (5, 5, 64),
                                                 (130, 7, 33)])
def test_the_router_chooses_the_largest_logits(experts, top, width):
    from edge_infer_amd.csrc import lib
    torch.manual_seed(experts)
    rows = 37
    x = torch.randn(rows, width)
    router = torch.randn(experts, width)
    logits = x.double() @ router.double().T
    order = torch.sort(logits, dim=1, descending=True)
    expert = torch.empty(rows, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(rows, top, device=DEV)
    row_seq = torch.zeros(rows, dtype=torch.int32, device=DEV)
    row_seq[5] = -1                           # a padding row
    lib.moe_route(x.to(DEV), router.to(DEV), row_seq, expert, weight)
    keep = [r for r in range(rows) if r != 5]
    assert torch.equal(expert.cpu()[keep].long(), order.indices[keep, :top])
    assert_close_f32(weight[keep], torch.softmax(order.values[keep, :top], dim=1), "weights of the chosen")
    assert weight[5].abs().sum().item() == 0


def test_of_equal_logits_the_lower_index_is_chosen():
    from edge_infer_amd.csrc import lib
    x = torch.ones(2, 8)
    router = torch.zeros(9, 8)
    router[[2, 4, 7]] = 0.5          # three equal largest logits; all others equal too
    expert = torch.empty(2, 5, dtype=torch.int32, device=DEV)
    weight = torch.empty(2, 5, device=DEV)
    lib.moe_route(x.to(DEV), router.to(DEV), None, expert, weight)
    assert expert.cpu().tolist() == [[2, 4, 7, 0, 1]] * 2


@pytest.mark.parametrize("experts, top, inter, width, rows", [
    (6, 2, 40, 48, 21), (9, 3, 13, 50, 21), (4, 1, 96, 64, 21), (5, 2, 128, 64, 3),
    (3, 2, 192, 128, 700), (12, 3, 64, 192, 77), (4, 2, 256, 512, 5), (6, 1, 512, 256, 40), (4, 2, 256, 512, 2), (5, 3, 768, 256, 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_experts_of_a_rows_choice(experts, top, inter, width, rows, dtype):
    """The experts' kernels on the router kernel's own choice, against the plain expert run on
    that choice (so that no close call of the router enters).  In bfloat16, widths that are
    multiples of 64 take the grouped products on the matrix cores: tiles of 32 places for few
    rows, of 128 for many, experts with no row at all, tiles that an expert fills in part."""
    from edge_infer_amd.csrc import lib
    torch.manual_seed(inter)
    x = torch.randn(rows, width).to(torch.bfloat16).float()
    router = torch.randn(experts, width)
    gate, up = (torch.randn(experts, inter, width) / width ** 0.5 for _ in range(2))
    down = torch.randn(experts, width, inter) / inter ** 0.5
    gate, up, down = (t.to(torch.bfloat16).float() for t in (gate, up, down))
    expert = torch.empty(rows, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(rows, top, device=DEV)
    xd = x.to(DEV).to(dtype)
    lib.moe_route(xd, router.to(DEV), None, expert, weight)
    act = torch.empty(rows * top, inter, device=DEV, dtype=dtype)
    out = torch.empty(rows, width, device=DEV)
    matrices = [t.to(DEV).to(dtype) for t in (gate, up, down)]
    if lib.moe_grouped_supported(dtype, width, inter, experts):
        pairs = rows * top
        order = torch.empty(2 * pairs + experts + 1, dtype=torch.int32, device=DEV)
        sums = torch.empty(pairs, width, device=DEV)
        lib.moe_experts_grouped(xd, *matrices, expert, weight, order[:pairs], order[pairs:2 * pairs],
                                order[2 * pairs:], act, sums, out)
        assert sorted(order[:pairs].tolist()) == list(range(pairs))
    else:
        assert dtype == torch.float32 or width % 64 or inter % 64
        lib.moe_experts(xd, *matrices, expert, weight, act, out)
    want = torch.zeros(rows, width, dtype=torch.float64)
    for r in range(rows):
        for k in range(top):
            e = int(expert[r, k])
            h = plain.silu(gate[e].double() @ x[r].double()) * (up[e].double() @ x[r].double())
            want[r] += weight[r, k].item() * (down[e].double() @ h)
    if dtype == torch.float32:
        assert_close_f32(out, want, "experts")
    else:
        assert_close_bf16(out, want, "experts")


def test_routed_feed_forward_in_a_layer():
    """The part through the block: router, experts and the weighted sum against the plain
    function, on rows whose routing is no close call."""
    from edge_infer_amd.config.specs import RoutedMLPSpec
    ffn = RoutedMLPSpec(n_experts=7, top=3, intermediate_size=20)
    spec = one_layer(ssm_spec(n_heads=2, head_dim=8, state=8, groups=1, conv_taps=2, norm_parts=1), ffn)
    params = params_for(spec, seed=23)
    model, session = session_for(spec, params)
    part = model.layers[0].ffn
    torch.manual_seed(24)
    x = torch.randn(60, HIDDEN).to(torch.bfloat16).float()
    tensors = {"f.router": params["layers.0.ffn.router.weight"]}
    for e in range(7):
        for name in ("gate", "up", "down"):
            tensors[f"f.e{e}.{name}"] = params[f"layers.0.ffn.experts.{e}.{name}_proj.weight"]
    margins = []
    want = plain.routed_feed_forward(x.double(), tensors, "f.", 7, 3, margins)
    clear = margins[0] > 1e-4
    from edge_infer_amd.engine.batch import SeqStep
    slot = session.begin()
    seqs = [SeqStep(slot=slot, start=0, tokens=[0] * 60)]
    session.cache.grow([(slot, 60)])
    ctx, _ = session.context_for(seqs)
    got = part.forward(ctx, x.to(DEV)).float()
    assert clear.sum() > 50
    assert_close_f32(got[clear.to(DEV)], want[clear], "routed feed-forward")
