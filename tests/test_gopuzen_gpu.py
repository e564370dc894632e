"""The Gopuzen decoder in the engine against the plain implementation (`plain_gopuzen`), in
float32 and bfloat16: whole prompts, the stream after every layer, prompts then tokens one by
one, portions down to two tokens, batches of unequal requests with slots and pages used
again, long decoding over window edges, block edges and page borders, the first tokens of a
sequence, a token far back, greedy generation through the entry point, the framework's own
random-weights folder and the replay program.

A routed feed-forward chooses experts by the order of its scores, so any rounding may choose
otherwise where two scores nearly tie, and a token routed otherwise changes the rows after it
as well.  The oracle reports every token's margin.  In float32 the comparisons leave out the
positions from the first margin below 1e-4 on.  In bfloat16 whole requests run on the
configurations' twins that route nothing (`dense_twin`), and the routed configurations are
compared up to their first close call."""
import json

import pytest
import torch

import plain_gopuzen as plain
from helpers import assert_close_bf16, assert_close_f32
from gopuzen_helpers import CONFIGS, TWINS, ids, sharp_weights, tensor_shapes, write_folder

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
NAMES = ["A", "B", "C", "D"]
LENGTHS = {"A": [150, 1, 49, 75], "B": [210, 2, 101, 64], "C": [200, 3, 130, 65],
           "D": [140, 1, 5, 66]}
# bfloat16 engine against the float64 oracle on these order-one weights with raised queries
# and keys: root-mean-square error relative to the logits' root-mean-square, and largest
# error relative to the largest logit
BF16_RMS, BF16_MAX = 4e-2, 12e-2
MARGIN = {"float32": 1e-4, "bfloat16": 0.05}


def config_of(name, dtype):
    """The configuration a test of `dtype` runs: the routed one, or in bfloat16 its twin."""
    return CONFIGS[name] if dtype == "float32" else TWINS[name]


def close(dtype, actual, expected, what, clear=None):
    if clear is not None:
        assert clear.sum().item() >= 0.5 * clear.numel(), f"{what}: too few clear positions"
        actual, expected = actual[clear.to(actual.device)], expected[clear]
    if dtype == "float32":
        return assert_close_f32(actual, expected, what)
    return assert_close_bf16(actual, expected, what, rms_rel=BF16_RMS, max_rel=BF16_MAX)


@pytest.fixture(scope="module")
def weights():
    """name -> dtype -> tensors of the configuration that `dtype` runs."""
    return {name: {dtype: sharp_weights(config_of(name, dtype), seed=20 + i) for dtype in DTYPES}
            for i, name in enumerate(NAMES)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory, weights):
    root = tmp_path_factory.mktemp("gopuzen")
    return {(name, dtype): write_folder(root / f"{name}_{dtype}", config_of(name, dtype),
                                        weights[name][dtype])
            for name in NAMES for dtype in DTYPES}


@pytest.fixture(scope="module")
def models(folders):
    import edge_infer_amd as ei
    cache = {}

    def get(name, dtype, routed=False):
        """The model a test of `dtype` runs; `routed`: the routed configuration in bfloat16."""
        key = (name, dtype, routed)
        if key not in cache:
            folder = folders[(name, "float32")] if routed else folders[(name, dtype)]
            cache[key] = ei.load_model(folder, dtype=dtype)
        return cache[key]
    return get


def requests_for(name, seed=5):
    return [ids(CONFIGS[name]["vocab"], n, seed + i) for i, n in enumerate(LENGTHS[name])]


@pytest.fixture(scope="module")
def references(weights):
    """name -> dtype -> [(logits, clear positions) of every request]."""
    out = {}
    for name in NAMES:
        out[name] = {dtype: [plain.clear_rows(config_of(name, dtype), weights[name][dtype], r,
                                              MARGIN[dtype], carry=True)
                             for r in requests_for(name)] for dtype in DTYPES}
    return out


@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_bfloat16_with_routing_up_to_the_first_close_call(models, weights, name):
    """The routed configurations in bfloat16, whole and decoded from graphs: every position
    before the first routing decision that bfloat16 could take otherwise (a gap of less than a
    twentieth of the score; C, which chooses 4 of 70 outputs, meets one within a few tokens)."""
    import edge_infer_amd as ei
    cfg, tensors = CONFIGS[name], weights[name]["float32"]
    session = ei.Session(models(name, "bfloat16", routed=True), max_tokens=512)
    compared = 0
    for seed in range(10):
        request = ids(cfg["vocab"], 70, 300 + seed)
        ref, clear = plain.clear_rows(cfg, tensors, request, MARGIN["bfloat16"], carry=True)
        rows = int(clear.sum())
        if rows < 8:
            continue
        slot = session.begin()
        cut = rows // 2
        got = [session.step([(slot, request[:cut], list(range(cut)))])]
        got += [session.step([(slot, [token], [0])]) for token in request[cut:rows]]
        session.end(slot)
        assert_close_bf16(torch.cat(got), ref[:rows], f"{name} routed, {rows} positions",
                          rms_rel=BF16_RMS, max_rel=BF16_MAX)
        compared += rows
    assert compared >= 20, f"{name}: only {compared} positions before close calls"


# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts(models, references, name, dtype):
    import edge_infer_amd as ei
    session = ei.Session(models(name, dtype), max_tokens=512)
    for request, (ref, clear) in zip(requests_for(name), references[name][dtype]):
        slot = session.begin()
        logits = session.step([(slot, request, list(range(len(request))))])
        close(dtype, logits, ref, f"{name} {dtype} whole {len(request)}", clear)
        session.end(slot)
    session.cache.check()


@pytest.mark.parametrize("name", ["A", "C"])
def test_the_stream_after_every_layer(models, weights, name):
    import edge_infer_amd as ei
    model = models(name, "float32")
    request = requests_for(name)[2]
    kept = []
    _, clear = plain.clear_rows(CONFIGS[name], weights[name]["float32"], request, 1e-4)
    plain.forward(CONFIGS[name], weights[name]["float32"], request, layer_outputs=kept)
    seen = []
    originals = [layer.forward for layer in model.layers]
    try:
        for layer, original in zip(model.layers, originals):
            def watched(ctx, residual, pending, entry, original=original):
                out = original(ctx, residual, pending, entry)
                assert out is None            # the arrangement adds everything itself
                seen.append(residual.clone())
                return out
            layer.forward = watched
        session = ei.Session(model, max_tokens=256, graphs=False)
        session.step([(session.begin(), request, [])])
    finally:
        for layer in model.layers:
            del layer.forward
    assert len(seen) == len(kept) == len(CONFIGS[name]["layers"])
    for index, (got, want) in enumerate(zip(seen, kept)):
        assert_close_f32(got[clear.to(got.device)], want[clear], f"stream after layer {index}")


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_tokens_one_by_one(models, references, name, dtype, graphs):
    """The decoded tokens pass window edges, block edges and a page border (64, 128)."""
    import edge_infer_amd as ei
    session = ei.Session(models(name, dtype), max_tokens=512, graphs=graphs)
    for request, (ref, clear) in zip(requests_for(name), references[name][dtype]):
        cut = max(1, len(request) - 60)
        slot = session.begin()
        rows = [session.step([(slot, request[:cut], [cut - 1])])]
        rows += [session.step([(slot, [token], [0])]) for token in request[cut:]]
        close(dtype, torch.cat(rows), ref[cut - 1:], f"{name} {dtype} tail of {len(request)}",
              clear[cut - 1:])
        session.end(slot)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("sizes", [(2, 2, 3, 2), (1, 5, 64, 2, 7), (63, 2, 65), (20, 100, 3)])
def test_portions(models, references, name, dtype, sizes):
    """A prompt cut into portions (the given sizes in turn, down to two tokens and one): every
    position's logits are those of the whole prompt."""
    import edge_infer_amd as ei
    session = ei.Session(models(name, dtype), max_tokens=512)
    request, (ref, clear) = requests_for(name)[0], references[name][dtype][0]
    slot = session.begin()
    rows, at, turn = [], 0, 0
    while at < len(request):
        take = min(sizes[turn % len(sizes)], len(request) - at)
        rows.append(session.step([(slot, request[at:at + take], list(range(take)))]))
        at, turn = at + take, turn + 1
    close(dtype, torch.cat(rows), ref, f"{name} {dtype} portions {sizes}", clear)
    session.end(slot)


def test_float32_logits_do_not_depend_on_the_cut(models, references):
    """Whole, in portions and token by token: the same float32 logits, up to the rounding of a
    few sums that the kernels take in another order for another number of rows (half the
    bound against the oracle)."""
    import edge_infer_amd as ei
    model = models("A", "float32")
    request = requests_for("A")[0][:100]
    clear = references["A"]["float32"][0][1][:100].to("cuda")
    session = ei.Session(model, max_tokens=512)

    def run(sizes):
        slot = session.begin()
        rows, at = [], 0
        for take in sizes:
            rows.append(session.step([(slot, request[at:at + take], list(range(take)))]))
            at += take
        session.end(slot)
        return torch.cat(rows)[clear]
    whole = run([100])
    for sizes in ([37, 63], [2] * 50, [99, 1], [1] * 100):
        got = run(sizes)
        assert (got - whole).abs().max().item() <= 1e-5 * whole.abs().max().item(), sizes


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_batches_of_unequal_requests_with_slots_and_pages_used_again(models, references, name, dtype):
    """Requests of unequal lengths start together and are decoded together; the shorter end
    earlier and their slots, pages and state rows go back; a second and a third batch then run
    in what was freed (the cache has room for little more than one batch)."""
    import edge_infer_amd as ei
    requests, refs = requests_for(name), references[name][dtype]
    tail = 20
    session = ei.Session(models(name, dtype), max_tokens=64 * 12, max_seqs=4)
    for batch in ([0, 1, 2, 3], [3, 2, 0], [1, 0, 3, 2]):
        slots = {i: session.begin() for i in batch}
        cuts = {i: max(1, len(requests[i]) - tail) for i in batch}
        got = {i: [] for i in batch}
        logits = session.step([(slots[i], requests[i][:cuts[i]], [cuts[i] - 1]) for i in batch])
        for row, i in enumerate(batch):
            got[i].append(logits[row:row + 1])
        at = dict(cuts)
        live = [i for i in batch if at[i] < len(requests[i])]
        for i in batch:
            if i not in live:
                session.end(slots[i])
        while live:
            logits = session.step([(slots[i], [requests[i][at[i]]], [0]) for i in live])
            for row, i in enumerate(live):
                got[i].append(logits[row:row + 1])
                at[i] += 1
            for i in [i for i in live if at[i] == len(requests[i])]:
                session.end(slots[i])
                live.remove(i)
        for i in batch:
            ref, clear = refs[i]
            if clear[cuts[i] - 1:].sum() == 0:     # (a request of one token that is a close call)
                continue
            actual, expected = torch.cat(got[i]), ref[cuts[i] - 1:]
            keep = clear[cuts[i] - 1:]
            close(dtype, actual[keep.to(actual.device)], expected[keep],
                  f"{name} {dtype} request {i} in batch {batch}")
        session.cache.check()
    assert session.cache.slots.n_free == 4
    assert all(pool.n_free == pool.n_pages for pool in session.cache.kv_pools)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_long_decoding_from_the_first_token(models, weights, name, dtype):
    """One token, then 299 more one by one, from graphs: every window's and block's edge and
    four page borders are passed while decoding, and the states are carried 300 times."""
    import edge_infer_amd as ei
    cfg = config_of(name, dtype)
    request = ids(cfg["vocab"], 300, 77)
    ref, clear = plain.clear_rows(cfg, weights[name][dtype], request, MARGIN[dtype], carry=True)
    if dtype == "float32" and clear.sum() < 200:    # compare up to the first call that is closer still
        clear = plain.clear_rows(cfg, weights[name][dtype], request, 2e-5, carry=True)[1]
    session = ei.Session(models(name, dtype), max_tokens=320)
    slot = session.begin()
    rows = [session.step([(slot, [token], [0])]) for token in request]
    close(dtype, torch.cat(rows), ref, f"{name} {dtype} 300 tokens one by one", clear)
    if session.graphs:     # (D in bfloat16 has products of odd widths, which the library multiplies)
        assert session.graph_replays > 250
    else:
        assert (name, dtype) == ("D", "bfloat16")


@pytest.mark.parametrize("graphs", [True, False])
def test_a_failed_step_leaves_the_state_as_it_was(models, references, graphs):
    """The linear-attention state and the convolutions' inputs have two versions a slot: a step
    that fails after its layers have run (here the head raises, once in a prompt portion and
    once in a decode step) has written the other version only, so the same step again gives
    what a run without the failure gives."""
    import edge_infer_amd as ei
    model = models("A", "float32")
    request, (ref, clear) = requests_for("A")[0], references["A"]["float32"][0]
    session = ei.Session(model, max_tokens=512, graphs=graphs)
    assert session.cache.two_versions and all(c is None for c in session.cache._state_copies)
    slot = session.begin()
    rows = [session.step([(slot, request[:40], list(range(40)))])]
    whole = type(model).logits
    failures = []

    def failing(self, ctx, hidden):
        if not failures:
            failures.append(ctx.n_rows)
            raise RuntimeError("forced failure after the layers have run")
        return whole(self, ctx, hidden)
    try:
        type(model).logits = failing
        with pytest.raises(RuntimeError, match="forced failure"):
            session.step([(slot, request[40:90], list(range(50)))])
        assert session.length(slot) == 40
        rows.append(session.step([(slot, request[40:90], list(range(50)))]))
        failures.clear()       # (the first decode step: the one that runs eagerly before a graph is made)
        with pytest.raises(RuntimeError, match="forced failure"):
            session.step([(slot, request[90:91], [0])])
        for t in range(90, 100):
            rows.append(session.step([(slot, request[t:t + 1], [0])]))
    finally:
        type(model).logits = whole
    close("float32", torch.cat(rows), ref[:100], "after failed steps", clear[:100])


@pytest.mark.parametrize("name", ["A", "C"])
def test_a_token_far_back_shows(tmp_path, name):
    """Two prompts that differ in their third token alone still differ at position 400, by far
    more than the tolerance (through the linear attention's heads that forget slowly or not at
    all, and through the softmax halves, which see every key), and the engine follows the
    oracle for both, whole, in portions and decoded."""
    import edge_infer_amd as ei
    cfg = TWINS[name]
    tensors = sharp_weights(cfg, seed=31)
    model = ei.load_model(write_folder(tmp_path / "far", cfg, tensors), dtype="float32")
    base = ids(cfg["vocab"], 401, 3)
    other = list(base)
    other[2] = (base[2] + 1) % cfg["vocab"]
    refs = [plain.forward(cfg, tensors, r)[-1:] for r in (base, other)]
    gap = (refs[0] - refs[1]).abs().max().item() / refs[0].abs().max().item()
    assert gap > 1e-3, f"the test's weights do not carry the third token to the end ({gap:.1e})"
    session = ei.Session(model, max_tokens=1024)
    for request, ref in zip((base, other), refs):
        slot = session.begin()
        close("float32", session.step([(slot, request, [400])]), ref, "far token, whole")
        session.end(slot)
        slot = session.begin()
        session.step([(slot, request[:130], [])])
        session.step([(slot, request[130:390], [])])
        for token in request[390:400]:
            session.step([(slot, [token], [])])
        close("float32", session.step([(slot, request[400:], [0])]), ref, "far token, decoded")
        session.end(slot)


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_entry_point(models, weights, name):
    """`Session.generate_batch` (the scheduler, sampler and step function together) gives the
    oracle's greedy tokens in float32."""
    import edge_infer_amd as ei
    cfg = CONFIGS[name]
    prompts = [ids(cfg["vocab"], n, 40 + n) for n in (5, 1, 30)]
    session = ei.Session(models(name, "float32"), max_tokens=512, max_seqs=3)
    got = session.generate_batch(prompts, max_new_tokens=12, temperature=0.0)
    for prompt, tokens in zip(prompts, got):
        sequence = list(prompt)
        for token in tokens:
            logits, clear = plain.clear_rows(cfg, weights[name]["float32"], sequence, 1e-5)
            if not clear[-1]:
                break                       # a routing decision within float32's reach
            logits = logits[-1]
            best = logits.argmax().item()
            if token != best:       # only a tie within float32's reach may differ
                assert (logits[best] - logits[token]).item() <= 2e-5 * logits.abs().max().item()
            sequence.append(token)
        assert len(tokens) == 12


def test_model_type_through_the_python_entry(folders, weights):
    from edge_infer_amd.api import Model
    model = Model.from_pretrained(folders[("A", "float32")], "gopuzen_fp32")
    session = model.new_session(capacity=128, max_batch=2)
    prompt = ids(CONFIGS["A"]["vocab"], 9, 1)
    tokens = session.generate(prompt, None, max_length=len(prompt) + 4, temperature=0.0)
    logits = plain.forward(CONFIGS["A"], weights["A"]["float32"], prompt)[-1]
    assert tokens[0] == logits.argmax().item() and len(tokens) == 4
    with pytest.raises(ValueError, match="names the family"):
        Model.from_pretrained(folders[("A", "float32")], "qwen3_bf16")


def test_random_weights_folder_of_the_framework(tmp_path):
    """`write_model_folder` writes a Gopuzen folder that reads back to the same configuration
    and runs; its tensors carry the checkpoint's names."""
    import edge_infer_amd as ei
    from safetensors.torch import load_file
    cfg = ei.config.GopuzenConfig.from_dict(CONFIGS["C"])
    folder = ei.write_model_folder(tmp_path / "random", cfg, seed=2)
    assert ei.read_config(folder)[1] == cfg
    tensors = load_file(str(folder / "model.safetensors"))
    shapes = {k: shape for k, (shape, _) in tensor_shapes(CONFIGS["C"]).items()}
    assert set(tensors) <= set(shapes)       # (what has no use is left out)
    assert all(tuple(v.shape) == tuple(shapes[k]) for k, v in tensors.items())
    model = ei.load_model(folder, dtype="float32")
    session = ei.Session(model, max_tokens=128)
    slot = session.begin()
    request = ids(CONFIGS["C"]["vocab"], 70, 9)
    logits = session.step([(slot, request, list(range(70)))])
    raw = json.loads((folder / "config.json").read_text())
    ref, clear = plain.clear_rows(raw, tensors, request, 1e-5, carry=True)
    assert clear.sum() >= 10
    close("float32", logits[clear.to(logits.device)], ref[clear], "random folder")


def test_the_replay_program_runs_a_gopuzen_folder(folders, weights, tmp_path):
    """`bin/trace_run` chooses the model class by config.json and writes the step's logits."""
    import subprocess
    import sys
    from pathlib import Path
    import numpy as np
    root = Path(__file__).resolve().parents[1]
    cfg, tensors = TWINS["A"], weights["A"]["bfloat16"]
    vocab = cfg["vocab"]
    one, two = ids(vocab, 30, 8), ids(vocab, 12, 9)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": one[:28], "want": [0, 27]},
                                     {"id": "y", "tokens": two[:11], "want": [10]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": one[28:29], "want": []},
                                     {"id": "y", "tokens": two[11:], "want": [0]}], "end": ["y"]},
             {"step": 2, "entries": [{"id": "x", "tokens": one[29:], "want": [0]}], "end": ["x"]}]
    done = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model",
                           str(folders[("A", "bfloat16")]), "--dtype", "float32", "--out", str(tmp_path),
                           "--max-tokens", "64"], input="\n".join(json.dumps(s) for s in steps),
                          capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [l for l in done.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    ref_one = plain.forward(cfg, tensors, one)
    ref_two = plain.forward(cfg, tensors, two)
    first = torch.from_numpy(np.fromfile(tmp_path / "0.f32", dtype="<f4").reshape(3, vocab))
    second = torch.from_numpy(np.fromfile(tmp_path / "1.f32", dtype="<f4").reshape(1, vocab))
    last = torch.from_numpy(np.fromfile(tmp_path / "2.f32", dtype="<f4").reshape(1, vocab))
    assert_close_f32(first, torch.cat([ref_one[[0, 27]], ref_two[[10]]]), "replayed prompts")
    assert_close_f32(second, ref_two[11:], "replayed token of the short request")
    assert_close_f32(last, ref_one[29:], "replayed token")
