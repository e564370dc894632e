"""The mechanisms of the Gopuzen layers alone, each against its plain function: the layer norm
in its three places, the mean of normed branches, the input convolution whole, in portions and
token by token with its state carried and slots used again, the linear-attention recurrence
and its read-out, the router's scores with their correction and the identity experts, and the
attention part's options: queries that grow with the position, the rotation of neighbouring
pairs, one gate a head, keys made to stand out just inside and just outside the window and
the pooled blocks, a far key among hundreds, and a layer that reads another layer's keys."""
import math

import pytest
import torch

import plain_gopuzen as plain
from helpers import assert_close_bf16, assert_close_f32

pytestmark = pytest.mark.gpu
DEV = "cuda"
HIDDEN, VOCAB, EPS = 48, 31, 1e-5


def exact(shape, generator, scale=1.0):
    """Random float32 values that bfloat16 holds exactly."""
    return (torch.randn(shape, generator=generator) * scale).to(torch.bfloat16).float()


# -- norms ------------------------------------------------------------------------------------
@pytest.mark.parametrize("width", [48, 50, 1000, 4100])
@pytest.mark.parametrize("slices", [0, 1, 5, 11])
def test_layer_norm_in_its_three_places(width, slices):
    """Before a sublayer (with a delta still to add, and gathered rows), on a sublayer's
    output, and both in one pass; deltas as one tensor or as float32 slices."""
    from edge_infer_amd.csrc import lib
    g = torch.Generator().manual_seed(width + slices)
    rows = 7
    residual = exact((rows, width), g)
    shape = (rows, width) if slices == 0 else (slices, rows, width)
    delta = exact(shape, g, 0.7)
    summed = delta if slices == 0 else delta.double().sum(0)
    w1, b1, w2, b2 = (exact((width,), g) for _ in range(4))
    bias = exact((width,), g, 0.3)
    # before a sublayer: rows 5, 0, 3 take their delta and are normed (-1: a padding row); the
    # other rows are not touched
    res = residual.clone().to(DEV)
    pick = torch.tensor([5, 0, -1, 3], dtype=torch.int32, device=DEV)
    out = torch.empty(4, width, device=DEV)
    lib.stream_norm(res, delta.to(DEV), out, w_next=w2.to(DEV), b_next=b2.to(DEV), eps=EPS,
                    centred=True, rows=pick)
    added = residual.double() + summed
    assert_close_f32(res[[5, 0, 3]], added[[5, 0, 3]], "stream after the addition")
    assert torch.equal(res[[1, 2, 4, 6]].cpu(), residual[[1, 2, 4, 6]])
    want = plain.layer_norm(added[[5, 0, 3]], w2, b2, EPS)
    assert_close_f32(out[[0, 1, 3]], want, "gathered rows")
    assert out[2].abs().max().item() == 0.0
    # on a sublayer's output (with a bias that the product left to this kernel)
    res = residual.clone().to(DEV)
    lib.stream_norm(res, delta.to(DEV), None, w_after=w1.to(DEV), b_after=b1.to(DEV), eps=EPS,
                    centred=True, delta_bias=bias.to(DEV))
    after = residual.double() + plain.layer_norm(summed + bias.double(), w1, b1, EPS)
    assert_close_f32(res, after, "stream after the norm on the output")
    # both in one pass, into bfloat16 rows
    res = residual.clone().to(DEV)
    out = torch.empty(rows, width, device=DEV, dtype=torch.bfloat16)
    lib.stream_norm(res, delta.to(DEV), out, w_after=w1.to(DEV), b_after=b1.to(DEV),
                    w_next=w2.to(DEV), b_next=b2.to(DEV), eps=EPS, centred=True,
                    delta_bias=bias.to(DEV))
    assert_close_f32(res, after, "stream after the fused pass")
    assert_close_bf16(out, plain.layer_norm(after, w2, b2, EPS), "fused rows")
    # no delta at all: the stream is only read
    out = torch.empty(rows, width, device=DEV)
    lib.stream_norm(res, None, out, w_next=w2.to(DEV), b_next=b2.to(DEV), eps=EPS, centred=True,
                    write_residual=False)
    assert_close_f32(out, plain.layer_norm(after, w2, b2, EPS), "norm alone")
    # and the same kernel without the mean
    lib.stream_norm(res, None, out, w_next=w2.to(DEV), eps=EPS, centred=False, write_residual=False)
    assert_close_f32(out, plain.rms_norm(after, w2, EPS), "rms norm alone")


@pytest.mark.parametrize("width, rows", [(48, 3), (50, 2), (2048, 1), (2048, 600)])
def test_mean_of_normed_branches(width, rows):
    from edge_infer_amd.csrc import lib
    g = torch.Generator().manual_seed(width)
    one = exact((3, rows, width), g)                       # float32 slices
    two = exact((rows, width), g, 5.0)                     # one bfloat16 tensor
    w1, w2 = exact((width,), g), exact((width,), g)
    out = torch.empty(rows, width, device=DEV)
    lib.norm_mean([one.to(DEV), two.to(DEV).to(torch.bfloat16)], [w1.to(DEV), w2.to(DEV)], EPS, out)
    want = 0.5 * (plain.rms_norm(one.double().sum(0), w1, EPS) + plain.rms_norm(two, w2, EPS))
    assert_close_f32(out, want, "mean of two branches")
    lib.norm_mean([two.to(DEV)], [w2.to(DEV)], EPS, out)
    assert_close_f32(out, plain.rms_norm(two, w2, EPS), "one branch")


# -- the input convolution ----------------------------------------------------------------------
class ConvRig:
    """Drives `lib.input_conv` as a session would: state rows of two versions a slot, the
    step's metadata on the device."""

    def __init__(self, slots, taps, width, parts=2):
        self.slots, self.taps, self.width, self.parts = slots, taps, width, parts
        self.state = torch.zeros(2 * (slots + 1), parts * max(taps - 1, 0) * width, device=DEV)
        self.version = [0] * slots
        self.length = [0] * slots

    def reset(self, slot):
        self.length[slot] = 0
        self.state[slot].zero_()
        self.state[self.slots + 1 + slot].zero_()

    def step(self, pieces, weight, part, dtype):
        """pieces: (slot, rows [n, width]); returns the convolved rows of every piece."""
        from edge_infer_amd.csrc import lib
        row_pos, row_seq, seq_in, seq_out, start, count, row0 = [], [], [], [], [], [], []
        at = 0
        for index, (slot, x) in enumerate(pieces):
            n = x.shape[0]
            row_pos += list(range(self.length[slot], self.length[slot] + n))
            row_seq += [index] * n
            v = self.version[slot]
            seq_in.append(v * (self.slots + 1) + slot)
            seq_out.append((1 - v) * (self.slots + 1) + slot)
            start.append(self.length[slot])
            count.append(n)
            row0.append(at)
            at += n

        def i32(values):
            return torch.tensor(values, dtype=torch.int32, device=DEV)
        h = torch.cat([x for _, x in pieces]).to(DEV).to(dtype).contiguous()
        out = torch.empty_like(h)
        lib.input_conv(h, weight.t().contiguous().to(DEV), self.state if self.taps > 1 else None,
                       part, self.parts,
                       i32(row_pos), i32(row_seq), i32(seq_in), i32(seq_out), i32(start),
                       i32(count), i32(row0), out)
        return out.float().cpu()

    def commit(self, pieces):
        for slot, x in pieces:
            self.version[slot] ^= 1
            self.length[slot] += x.shape[0]


@pytest.mark.parametrize("taps, width", [(3, 48), (1, 50), (2, 7), (5, 64), (4, 2048)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_input_convolution(taps, width, dtype):
    """Whole, in portions down to one token (shorter than the filter), two sequences side by
    side, both sublayers' parts of the state, and a slot that is used again."""
    g = torch.Generator().manual_seed(taps * 100 + width)
    w = [exact((width, taps), g, 0.5) for _ in range(2)]
    xs = [exact((40, width), g), exact((23, width), g)]
    want = [[plain.input_convolution(x, w[part]).float() for x in xs] for part in range(2)]
    tol = dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=3e-2, rtol=2e-2)
    rig = ConvRig(slots=3, taps=taps, width=width)
    for cuts in ([40], [1, 1, 1, 2, 3, 32], [taps, 40 - taps], [39, 1]):
        for slot in range(3):
            rig.reset(slot)
        at = 0
        for take in cuts:
            # sequence 0 in slot 2 takes `take` rows, sequence 1 in slot 0 at most as many
            other = min(take, 23 - min(at, 23))
            pieces = [(2, xs[0][at:at + take])] + ([(0, xs[1][at:at + other])] if other else [])
            for part in range(2):
                got = rig.step(pieces, w[part], part, dtype)
                torch.testing.assert_close(got[:take], want[part][0][at:at + take], **tol)
                if other:
                    torch.testing.assert_close(got[take:], want[part][1][at:at + other], **tol)
            rig.commit(pieces)
            at += take


# -- linear attention ---------------------------------------------------------------------------
@pytest.mark.parametrize("heads, key_dim, value_dim, seqs", [
    (3, 12, 20, 2), (2, 32, 72, 1), (1, 160, 136, 3), (5, 16, 16, 1), (8, 128, 64, 40),
    (4, 64, 128, 70), (2, 256, 16, 1), (3, 7, 11, 2)])
def test_linear_attention_recurrence(heads, key_dim, value_dim, seqs):
    """`la_scan` and `la_out` against the token-by-token recurrence: several sequences of
    unequal lengths in one step, then each continued in portions and token by token from the
    carried state (few sequences take the kernel's narrow column tiles, many the wide ones)."""
    from edge_infer_amd.csrc import lib
    g = torch.Generator().manual_seed(heads * key_dim + value_dim)
    decay = torch.tensor([1.0, 0.5, 0.9, 0.99, 0.999, 0.97, 0.8, 0.3][:heads])
    width = heads * (2 * key_dim + 2 * value_dim)
    lengths = [30 + 5 * (s % 4) for s in range(seqs)]
    projections = [exact((n, width), g) for n in lengths]
    norm_w = exact((heads * value_dim,), g)

    def reference(proj):
        n = proj.shape[0]
        q = plain.silu(proj[:, :heads * key_dim].double()).reshape(n, heads, key_dim)
        k = plain.silu(proj[:, heads * key_dim:2 * heads * key_dim].double()).reshape(n, heads, key_dim)
        v = plain.silu(proj[:, 2 * heads * key_dim:2 * heads * key_dim + heads * value_dim].double())
        o = plain.decayed_linear_attention(q, k, v.reshape(n, heads, value_dim), decay.double())
        o = o.reshape(n, heads * value_dim)
        gate = proj[:, 2 * heads * key_dim + heads * value_dim:].double()
        return o, plain.rms_norm(o, norm_w, EPS) * plain.sigmoid(gate)
    wants = [reference(p) for p in projections]
    floats = lib.la_state_floats(heads, key_dim, value_dim)
    state = torch.zeros(2 * (seqs + 1), floats, device=DEV)
    version = [0] * seqs

    def i32(values):
        return torch.tensor(values, dtype=torch.int32, device=DEV)

    def step(taken):
        """taken: (sequence, first row, rows); the raw read-outs and the gated rows."""
        rows = torch.cat([projections[s][a:a + n] for s, a, n in taken]).to(DEV).contiguous()
        total = rows.shape[0]
        o_raw = torch.empty(total, heads * value_dim, device=DEV)
        row0, at = [], 0
        for _, _, n in taken:
            row0.append(at)
            at += n
        scanned, activated = rows, total % 2 == 0
        if activated:       # (q, k and v activated aside, as a prompt step of many rows does)
            scanned = torch.empty(total, heads * (2 * key_dim + value_dim), device=DEV)
            lib.la_activate(rows, scanned)
        lib.la_scan(scanned, decay.to(DEV), state,
                    i32([version[s] * (seqs + 1) + s for s, _, _ in taken]),
                    i32([(1 - version[s]) * (seqs + 1) + s for s, _, _ in taken]),
                    i32([n for _, _, n in taken]), i32(row0), o_raw, heads, key_dim, value_dim,
                    activated=activated)
        out = torch.empty(total, heads * value_dim, device=DEV)
        lib.la_out(o_raw, rows, 2 * heads * key_dim + heads * value_dim, norm_w.to(DEV), EPS, None, out)
        for s, _, _ in taken:
            version[s] ^= 1
        return o_raw, out
    # the first 20 rows of every sequence in one step, then portions, then tokens
    o_raw, out = step([(s, 0, 20) for s in range(seqs)])
    for s in range(seqs):
        assert_close_f32(o_raw[20 * s:20 * s + 20], wants[s][0][:20], f"read-out of sequence {s}")
        assert_close_f32(out[20 * s:20 * s + 20], wants[s][1][:20], f"gated rows of sequence {s}")
    o_raw, out = step([(s, 20, 2) for s in range(seqs)])
    assert_close_f32(out[2 * (seqs - 1):], wants[seqs - 1][1][20:22], "a portion of two tokens")
    for t in range(22, 30):
        o_raw, out = step([(s, t, 1) for s in range(seqs)])
    for s in range(seqs):
        assert_close_f32(out[s:s + 1], wants[s][1][29:30], f"token 29 of sequence {s}")
    longer = [s for s in range(seqs) if lengths[s] > 30]
    if longer:
        o_raw, out = step([(s, 30, lengths[s] - 30) for s in longer])
        assert_close_f32(o_raw[:lengths[longer[0]] - 30], wants[longer[0]][0][30:], "the rest")


# -- the router and the experts ------------------------------------------------------------------
@pytest.mark.parametrize("experts, identity, top, width", [(5, 2, 2, 48), (65, 5, 4, 96),
                                                           (3, 0, 1, 50), (8, 3, 3, 64)])
def test_router_scores_with_correction(experts, identity, top, width):
    from edge_infer_amd.csrc import lib
    g = torch.Generator().manual_seed(experts)
    outputs = experts + identity
    x = exact((40, width), g)
    tensors = {"r.router": exact((outputs, width), g, 3.0 / width ** 0.5),
               "r.correction": exact((outputs,), g, 0.3 / outputs)}
    chosen, weights, scores = plain.route(x, tensors, "r.", {"top": top})
    expert = torch.empty(40, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(40, top, device=DEV)
    lib.moe_route(x.to(DEV), tensors["r.router"].to(DEV), None, expert, weight,
                  scoring="softmax_all", correction=tensors["r.correction"].to(DEV))
    assert expert.cpu().tolist() == chosen.tolist()
    assert_close_f32(weight, weights, "the chosen scores, not renormalised")
    assert (weights.sum(-1) < 1.0 - 1e-6).any()
    # without the correction the order is the scores' own
    lib.moe_route(x.to(DEV), tensors["r.router"].to(DEV), None, expert, weight, scoring="softmax_all")
    assert expert.cpu().tolist() == torch.topk(scores, top, dim=-1).indices.tolist()


@pytest.mark.parametrize("experts, identity, top, inter, width, rows, dtype", [
    (5, 2, 2, 40, 48, 9, "float32"), (4, 3, 3, 64, 64, 50, "bfloat16"),
    (4, 3, 3, 64, 64, 300, "bfloat16"), (3, 1, 4, 13, 50, 6, "float32")])
def test_identity_experts_add_the_row_itself(experts, identity, top, inter, width, rows, dtype):
    """The routed feed-forward part on rows whose choices hold identity experts (every row
    chooses one, by a large correction), through the pair-at-a-time kernels and the grouped
    matrix-core ones."""
    from edge_infer_amd.config.specs import RoutedMLPSpec
    from edge_infer_amd.parts import RoutedMLP
    g = torch.Generator().manual_seed(inter)
    outputs = experts + identity
    spec = RoutedMLPSpec(n_experts=experts, top=top, intermediate_size=inter,
                         scoring="softmax_all", correction=True, identity=identity)
    tensors = {"f.router": exact((outputs, width), g, 2.0 / width ** 0.5),
               "f.correction": exact((outputs,), g, 0.02)}
    tensors["f.correction"][experts] = 2.0          # the first identity expert is always chosen
    for e in range(experts):
        tensors[f"f.e{e}.gate"] = exact((inter, width), g, width ** -0.5)
        tensors[f"f.e{e}.up"] = exact((inter, width), g, width ** -0.5)
        tensors[f"f.e{e}.down"] = exact((width, inter), g, inter ** -0.5)
    params = {"router.weight": tensors["f.router"], "router.correction": tensors["f.correction"]}
    for e in range(experts):
        for name in ("gate", "up", "down"):
            params[f"experts.{e}.{name}_proj.weight"] = tensors[f"f.e{e}.{name}"]
    part = RoutedMLP(spec, width, params, torch.float32 if dtype == "float32" else torch.bfloat16, DEV)
    assert part.grouped == (dtype == "bfloat16")
    x = exact((rows, width), g)
    mlp = {"router": {"experts": experts, "top": top, "identity": identity}}
    want = plain.routed_feed_forward(x, tensors, "f.", mlp)

    class Context:
        class meta:
            row_seq = torch.zeros(rows, dtype=torch.int32, device=DEV)

        @staticmethod
        def buffer(name, shape, kind=None):
            return torch.empty(shape, device=DEV, dtype=kind or part.w_gate.dtype)

        @staticmethod
        def release(*buffers):
            pass
    got = part.forward(Context, x.to(DEV).to(part.w_gate.dtype))
    if dtype == "float32":
        assert_close_f32(got, want, "identity experts")
    else:
        assert_close_bf16(got, want, "identity experts, grouped")


# -- the attention part's options -----------------------------------------------------------------
def one_layer(*mixers):
    """A model of pre-norm layers without feed-forwards, one a mixer; a mixer with `shared_kv`
    reads the first layer's cache."""
    from edge_infer_amd.config.specs import LayerSpec, ModelSpec, NormSpec, ScheduleEntry
    norm = NormSpec(eps=EPS)
    schedule = tuple(ScheduleEntry(layer=i, cache=0, writes_cache=False, own=i)
                     if getattr(m, "shared_kv", False) else ScheduleEntry(layer=i, cache=i)
                     for i, m in enumerate(mixers))
    return ModelSpec(architecture="test", vocab_size=VOCAB, hidden_size=HIDDEN,
                     layers=tuple(LayerSpec(block="prenorm", norm=norm, mixer=m, feed_forward=None)
                                  for m in mixers),
                     schedule=schedule, final_norm=norm, tie_word_embeddings=False,
                     max_position_embeddings=1 << 20, bos_token_id=None, eos_token_id=None)


def params_for(spec, seed, gain=1.0):
    from edge_infer_amd.engine.model import model_parameters
    g = torch.Generator().manual_seed(seed)
    out = {}
    for path, param in model_parameters(spec).items():
        if param.optional:
            continue
        shape = tuple(param.shape)
        if param.init == "norm":
            value = 1 + 0.2 * (torch.rand(shape, generator=g) - 0.5)
        elif len(shape) == 2:
            value = torch.randn(shape, generator=g) / shape[1] ** 0.5
            if path.endswith("q_proj.weight") or path.endswith("k_proj.weight"):
                value = value * gain
        else:
            value = torch.randn(shape, generator=g) * 0.5
        out[path] = value.to(torch.bfloat16).float()
    return out


def session_for(spec, params, dtype="float32", max_tokens=1024, max_seqs=4):
    from edge_infer_amd.engine import DecoderModel, Session
    model = DecoderModel(spec, params, dtype, DEV)
    return model, Session(model, max_tokens=max_tokens, max_seqs=max_seqs, graphs=False)


def run_parts(session, parts, pieces):
    """`pieces`: (slot, start, x rows) per sequence of one step; every part's output rows (the
    parts are the layers' mixers, run in order on the same rows)."""
    from edge_infer_amd.engine.batch import SeqStep
    seqs = [SeqStep(slot=slot, start=start, tokens=[0] * x.shape[0]) for slot, start, x in pieces]
    session.cache.grow([(s.slot, s.start + s.count) for s in seqs])
    ctx, _ = session.context_for(seqs)
    rows = torch.cat([x for _, _, x in pieces]).contiguous().to(DEV).to(session.dtype)
    outs = []
    for part, entry in zip(parts, session.model.spec.schedule):
        out = part.forward(ctx, rows, entry)
        outs.append((out.sum(0) if out.dim() == 3 else out).float().clone())
    session.cache.commit([(s.slot, s.start + s.count) for s in seqs])
    return outs


def in_cuts(session, parts, x, cuts):
    slot = session.begin()
    rows, at = [[] for _ in parts], 0
    for take in cuts:
        for kept, out in zip(rows, run_parts(session, parts, [(slot, at, x[at:at + take])])):
            kept.append(out)
        at += take
    assert at == x.shape[0]
    session.end(slot)
    return [torch.cat(kept) for kept in rows]


NAMES = {"q_proj.weight": "q", "k_proj.weight": "k", "v_proj.weight": "v", "gate_proj.weight": "g",
         "o_proj.weight": "o"}


def tensors_of(params, layer):
    pre = f"layers.{layer}.mixer."
    return {"m." + NAMES[k[len(pre):]]: v for k, v in params.items()
            if k.startswith(pre) and k[len(pre):] in NAMES}


def window_spec(heads, kv_heads, dim, vdim, scale, window, pool, rot, shared=False):
    from edge_infer_amd.config.specs import AttentionSpec, PositionSpec
    position = PositionSpec(kind="none") if rot is None else \
        PositionSpec(kind="rope_pairs", theta=rot[0], dim=rot[1])
    return AttentionSpec(n_heads=heads, n_kv_heads=kv_heads, head_dim=dim, value_dim=vdim,
                         qkv_bias=False, o_bias=False, scale=scale, window=window, pool=pool,
                         position=position, output_gate="head", shared_kv=shared)


def plain_window(params, layer, spec, x, shared=None):
    mixer = {"heads": spec.n_heads, "kv_heads": spec.n_kv_heads, "dim": spec.head_dim,
             "vdim": spec.v_dim, "scale": spec.scale}
    if spec.window is not None:
        mixer["mask"] = {"size": spec.window}
        if spec.pool is not None:
            mixer["mask"]["pool"] = spec.pool
    if spec.position.kind != "none":
        mixer["rot"] = {"base": spec.position.theta, "dims": spec.position.dim}
    return plain.attention_mixer(x, tensors_of(params, layer), "m.", mixer,
                                 torch.arange(x.shape[0]), shared)


@pytest.mark.parametrize("shape", [
    dict(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, window=20, pool=5, rot=(100.0, 8)),
    dict(heads=6, kv_heads=1, dim=10, vdim=6, scale=0.4, window=None, pool=None, rot=(50.0, 10)),
    dict(heads=2, kv_heads=2, dim=64, vdim=64, scale=0.15, window=70, pool=64, rot=(1e4, 32)),
    dict(heads=8, kv_heads=2, dim=64, vdim=64, scale=0.125, window=3, pool=8, rot=None),
    dict(heads=4, kv_heads=1, dim=128, vdim=128, scale=0.09, window=64, pool=1, rot=(1e4, 128))])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_attention_with_pooled_blocks_alone(shape, dtype):
    """Whole, in portions down to two tokens and token by token; head sizes 64 and 128 with
    values as wide take the matrix-core kernels in bfloat16, beside which the pooled blocks are
    gathered by the generic kernel."""
    mixer = window_spec(**shape)
    spec = one_layer(mixer)
    params = params_for(spec, seed=5, gain=1.5)
    model, session = session_for(spec, params, dtype)
    part = model.layers[0].mixer
    assert part.pooled_aside == (dtype == "bfloat16" and shape["dim"] >= 64 and shape["pool"] is not None)
    torch.manual_seed(8)
    T = 150
    x = torch.randn(T, HIDDEN).to(torch.bfloat16).float()
    want, _ = plain_window(params, 0, mixer, x.double())
    for cuts in ([T], [2] * 10 + [T - 20], [63, 2, 65, 20], [T - 40] + [1] * 40):
        got, = in_cuts(session, [part], x, cuts)
        if dtype == "float32":
            assert_close_f32(got, want, f"attention {shape}, cuts {cuts[:3]}")
        else:
            assert_close_bf16(got, want, f"attention {shape}, cuts {cuts[:3]}", rms_rel=2e-2,
                              max_rel=4e-2)


@pytest.mark.parametrize("dim, heads, kv_heads", [(64, 8, 2), (128, 4, 1), (64, 3, 3)])
def test_pooled_blocks_beside_the_matrix_core_kernel_whose_waves_take_whole_pages(dim, heads, kv_heads):
    """A prompt of few blocks lets two waves share every page's keys; one of many blocks gives
    a wave the whole page.  The second form is asked for here on a short prompt (the oracle
    walks every pair of positions), with the pooled slice and the gate taken in at its end."""
    mixer = window_spec(heads, kv_heads, dim, dim, 0.15, 40, 6, (1e4, dim // 2))
    spec = one_layer(mixer)
    params = params_for(spec, seed=17, gain=1.5)
    model, session = session_for(spec, params, "bfloat16")
    part = model.layers[0].mixer
    assert part.pooled_aside
    part.prefill_key_ways = lambda counts: 1
    torch.manual_seed(3)
    T = 200
    x = torch.randn(T, HIDDEN).to(torch.bfloat16).float()
    want, _ = plain_window(params, 0, mixer, x.double())
    for cuts in ([T], [70, 130], [T - 3, 1, 1, 1]):
        got, = in_cuts(session, [part], x, cuts)
        assert_close_bf16(got, want, f"one wave a page, cuts {cuts}", rms_rel=2e-2, max_rel=4e-2)


@pytest.mark.parametrize("dtype, dim", [("float32", 16), ("bfloat16", 64), ("bfloat16", 16)])
@pytest.mark.parametrize("window, pool", [(5, 3), (64, 64), (65, 7), (100, 12), (6, 16)])
def test_keys_that_stand_out_at_the_edges_of_window_and_blocks(window, pool, dtype, dim):
    """A key is made to dominate the last position's softmax (its input is a multiple of the
    query's, and the keys are made with the queries' matrix): the last token inside the window
    shows; the first token outside it shows only when its whole block lies outside (then
    through the block's mean), and a token of a block that the window still touches must not
    show at all.  In prompts, in portions that end at the edge, and decoded."""
    mixer = window_spec(2, 2, dim, dim if dim == 64 else 8, 0.5 if dim == 16 else 0.2, window, pool, None)
    spec = one_layer(mixer)
    params = params_for(spec, seed=9)
    pre = "layers.0.mixer."
    params[pre + "k_proj.weight"] = params[pre + "q_proj.weight"].clone()
    model, session = session_for(spec, params, dtype)
    part = model.layers[0].mixer
    torch.manual_seed(6)
    T = 180
    last = T - 1
    base = (0.3 * torch.randn(T, HIDDEN)).to(torch.bfloat16).float()
    seen_blocks = (last - window + 1) // pool              # blocks wholly before the window
    cases = [(last - window + 1, True),                    # the oldest token of the window
             (seen_blocks * pool - 1, True)]               # the newest token of a seen block
    if (last - window + 1) % pool:                         # a token that has left the window
        cases.append((last - window, False))               # while its block is not seen yet
    for place, seen in cases:
        x = base.clone()
        x[place] = (4.0 if place > last - window else 4.0 * pool) * x[last]
        x = x.to(torch.bfloat16).float()
        want, _ = plain_window(params, 0, mixer, x.double())
        quiet, _ = plain_window(params, 0, mixer, base.double())
        moved = (want[-1] - quiet[-1]).abs().max().item() / want[-1].abs().max().item()
        assert (moved > 0.1) == seen, f"the key at {place} does not stand out as meant ({moved:.2e})"
        for cuts in ([T], [T - 1, 1], [place + 1, T - place - 1], [T - 30] + [1] * 30):
            got, = in_cuts(session, [part], x, cuts)
            what = f"window {window}, pool {pool}, key at {place}, cuts {cuts[:3]}"
            if dtype == "float32":
                assert_close_f32(got, want, what)
            else:
                assert_close_bf16(got, want, what, rms_rel=2e-2, max_rel=4e-2)


def test_a_far_key_among_hundreds_and_a_growing_query():
    """Position 3 of 700 repeats the last position's input and the mixer sees every key, so
    that key takes a weight that shows; the queries' temperature, which is 1 for the first
    positions and about 2.4 at the end, shows as well."""
    from edge_infer_amd.config.specs import AttentionSpec, PositionSpec
    mixer = AttentionSpec(n_heads=2, n_kv_heads=1, head_dim=16, value_dim=12, qkv_bias=False,
                          o_bias=False, scale=0.6, position=PositionSpec(kind="none"),
                          query_temperature=(0.3, 7))
    spec = one_layer(mixer)
    params = params_for(spec, seed=13)
    pre = "layers.0.mixer."
    params[pre + "k_proj.weight"] = params[pre + "q_proj.weight"][:16].clone()
    model, session = session_for(spec, params, max_tokens=1024)
    part = model.layers[0].mixer
    torch.manual_seed(10)
    T = 700
    x = (0.5 * torch.randn(T, HIDDEN)).to(torch.bfloat16).float()
    x[3] = x[T - 1]
    left = {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 12, "scale": 0.6,
            "q_temp": {"coef": 0.3, "every": 7}}

    def reference(rows, temp=True):
        m = dict(left) if temp else {k: v for k, v in left.items() if k != "q_temp"}
        return plain.causal_attention(rows.double(), tensors_of(params, 0), "m.", m,
                                      torch.arange(rows.shape[0]))
    want = reference(x)
    other = x.clone()
    other[3] = x[4]
    moved = (reference(other)[-1] - want[-1]).abs().max() / want[-1].abs().max()
    assert moved > 0.05, f"the far key does not show ({moved:.2e})"
    moved = (reference(x, temp=False)[-1] - want[-1]).abs().max() / want[-1].abs().max()
    assert moved > 0.05, f"the temperature does not show ({moved:.2e})"
    assert torch.equal(reference(x, temp=False)[:6], want[:6])       # floor(6 / 7) = 0
    for cuts in ([T], [T - 1, 1], [2, 2, 300, T - 304 - 40] + [1] * 40):
        got, = in_cuts(session, [part], x, cuts)
        assert_close_f32(got, want, f"far key, cuts {cuts[:4]}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_that_reads_another_layers_keys(dtype):
    """The second mixer has no key and value projections: it meets the first one's cached keys
    (after their rotation) and values with queries, a window, blocks and a gate of its own; the
    first one's cache keeps what the wider of the two masks needs."""
    first = window_spec(4, 2, 64, 64, 0.15, 10, 4, (500.0, 32))
    second = window_spec(4, 2, 64, 64, 0.2, 90, 9, (500.0, 32), shared=True)
    import dataclasses
    first = dataclasses.replace(first, cache_span=90)
    spec = one_layer(first, second)
    params = params_for(spec, seed=21, gain=1.5)
    model, session = session_for(spec, params, dtype)
    parts = [layer.mixer for layer in model.layers]
    assert "k_proj.weight" not in type(parts[1]).parameters(second, HIDDEN)
    torch.manual_seed(4)
    T = 200
    x = torch.randn(T, HIDDEN).to(torch.bfloat16).float()
    want_first, kept = plain_window(params, 0, first, x.double())
    want_second, _ = plain_window(params, 1, second, x.double(), shared=kept)
    for cuts in ([T], [70, 2, 64, 64], [T - 50] + [1] * 50):
        got_first, got_second = in_cuts(session, parts, x, cuts)
        for got, want, what in ((got_first, want_first, "own keys"), (got_second, want_second, "shared keys")):
            if dtype == "float32":
                assert_close_f32(got, want, f"{what}, cuts {cuts[:3]}")
            else:
                assert_close_bf16(got, want, f"{what}, cuts {cuts[:3]}", rms_rel=2e-2, max_rel=4e-2)
    session.cache.check()


@pytest.mark.parametrize("taps, width", [(3, 48), (1, 64), (4, 2048)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_decode_steps_convolution_inside_the_norm_kernel(taps, width, dtype):
    """A step whose sequences bring one token each: the norm kernel adds the taps itself.  The
    rows it writes and the state it leaves are, bit for bit, those of the norm followed by the
    convolution kernel, token after token, for three sequences side by side."""
    from edge_infer_amd.csrc import lib
    g = torch.Generator().manual_seed(taps + width)
    w = exact((width, taps), g, 0.5).t().contiguous().to(DEV)
    weight, bias = exact((width,), g).to(DEV), exact((width,), g).to(DEV)
    seqs, floats = 3, 2 * max(taps - 1, 0) * width
    states = [torch.zeros(2 * (seqs + 1), max(floats, 1), device=DEV) for _ in range(2)]

    def i32(values):
        return torch.tensor(values, dtype=torch.int32, device=DEV)
    version = 0
    for token in range(7):
        residual = exact((seqs, width), g, 2.0).to(DEV)
        seq_in = i32([version * (seqs + 1) + s for s in range(seqs)])
        seq_out = i32([(1 - version) * (seqs + 1) + s for s in range(seqs)])
        # apart: the norm, then the convolution of the step's rows
        h = torch.empty(seqs, width, device=DEV, dtype=dtype)
        lib.stream_norm(residual, None, h, w_next=weight, b_next=bias, eps=EPS, centred=True,
                        write_residual=False)
        apart = torch.empty_like(h)
        lib.input_conv(h, w, states[0] if taps > 1 else None, 1, 2, i32([token] * seqs),
                       i32(list(range(seqs))), seq_in, seq_out, i32([token] * seqs), i32([1] * seqs),
                       i32(list(range(seqs))), apart)
        # in one kernel
        fused = torch.empty_like(h)
        lib.stream_norm(residual, None, fused, w_next=weight, b_next=bias, eps=EPS, centred=True,
                        write_residual=False,
                        conv=(w, states[1] if taps > 1 else None, 1, 2, seq_in, seq_out))
        assert torch.equal(fused, apart), f"token {token}"
        if taps > 1:
            assert torch.equal(states[0], states[1]), f"state after token {token}"
        version ^= 1
