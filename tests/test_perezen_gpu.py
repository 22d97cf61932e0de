"""The Perezen design through the framework: replayed traces (whole prompts, decoding, portions, mixed batches with pages and
state slots used again) against the plain implementation, generation through the entry point and the scheduler, and weights made
so that a far key, a chunk's edge, a borrowed key or a lost state shows in the logits."""

import copy
import json
import subprocess
import sys

import numpy as np
import pytest

import plain_gpt2
import plain_perezen as plain
import replay
from conftest import random_tokens
from perezen_cases import CASES, attention_layer, mlstm_layer, model

pytestmark = pytest.mark.gpu


def sharpen(config, weights, factor=4.0):
    """Random projections give nearly uniform softmaxes, under which a wrong key or page hardly moves a logit. Queries and keys are
    normed, which undoes a scaled matrix: the queries' gain vectors are scaled up instead, so that attention weights differ by
    orders of magnitude."""
    for index, layer in enumerate(config["layers"]):
        name = f"l{index}.mix.q.norm"
        if name in weights:
            weights[name] = plain_gpt2.round_to_bf16(weights[name] * factor)
    return weights


@pytest.fixture(scope="module")
def perezen_dirs(tmp_path_factory):
    out = {}
    for seed, (name, config) in enumerate(CASES.items()):
        weights = sharpen(config, plain.random_weights(config, 60 + seed))
        folder = plain.write_model_dir(tmp_path_factory.mktemp(f"perezen_{name}"), config, weights)
        out[name] = (folder, copy.deepcopy(config), weights)
    return out


def requests_for(config, lengths, seed=700):
    return {f"r{i}": random_tokens(seed + i, n, config["vocab"]) for i, n in enumerate(lengths)}


def plain_logits(config, weights, requests, bf16):
    w = plain.as_float64(weights)
    return {name: plain.forward(config, w, tokens, round_to=plain_gpt2.stored_as_bf16 if bf16 else None) for name, tokens in requests.items()}


LENGTHS = {"mixed": [5, 130, 64, 65, 1, 200, 33], "odd": [67, 2, 130, 31], "wide": [3, 150, 64, 17, 129, 260], "large": [150, 70, 3, 97]}
MODES = {"whole": replay.whole, "tail": replay.prefill_then_decode, "chunked": replay.chunked, "mixed": replay.mixed}
# sums in another order than numpy's, and positions at which a matrix memory's normaliser or a head's difference of two maps passes
# close to zero, which multiply every rounding before them
TOLERANCE = {"float32": dict(atol=1e-3, rtol=2e-4)}


def check(got, config, weights, requests, dtype):
    """32-bit: every logit of every position within the tolerance. bfloat16: the engine rounds at other places than the plain
    implementation does when it rounds what a bfloat16 run stores, so the two are not compared with each other but each with exact
    arithmetic, position by position (largest difference of a position's logits): the engine's distance may be three times the
    plain bfloat16 run's at nine positions in ten, one and a half times in the median and in the root mean square over all
    positions, and ten times anywhere. A wrong key, page, slot or state moves the logits of every position behind it by tens of
    times the noise, and shows at once in the 32-bit run of the same trace."""
    exact = plain_logits(config, weights, requests, False)
    if dtype == "float32":
        atol, rtol = TOLERANCE[dtype]["atol"], TOLERANCE[dtype]["rtol"]
        for name, rows in exact.items():
            assert set(got[name]) == set(range(len(rows))), name
            share = np.array([(np.abs(got[name][p].astype(np.float64) - rows[p]) / (atol + rtol * np.abs(rows[p]))).max() for p in range(len(rows))])
            assert share.max() <= 5.0 and (share > 1.0).sum() <= max(1, len(rows) // 100), f"request {name!r}: position {int(share.argmax())} is {share.max():.2f} times the tolerance off, {(share > 1.0).sum()} positions beyond it"
        return
    rounded = plain_logits(config, weights, requests, True)
    noise, error = [], []
    for name, rows in exact.items():
        assert set(got[name]) == set(range(len(rows))), name
        noise.append(np.abs(rounded[name] - rows).max(axis=1))
        error.append(np.abs(np.stack([got[name][p] for p in range(len(rows))]).astype(np.float64) - rows).max(axis=1))
    noise, error = np.concatenate(noise), np.concatenate(error)
    ratio = error / (noise + 0.02 * np.median(noise) + 1e-3)
    assert np.quantile(ratio, 0.9) <= 3.0 and np.median(ratio) <= 1.5 and ratio.max() <= 10.0, (np.quantile(ratio, 0.9), np.median(ratio), ratio.max(), int(ratio.argmax()))
    assert np.sqrt((error ** 2).mean()) <= 1.5 * np.sqrt((noise ** 2).mean()) + 1e-3, "rms error against rms noise"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("name", list(CASES))
def test_replay_matches_plain(perezen_dirs, tmp_path, name, mode, dtype):
    folder, config, weights = perezen_dirs[name]
    requests = requests_for(config, LENGTHS[name])
    collector = MODES[mode](requests)
    for page_size in ((None, 16) if mode == "mixed" and dtype == "float32" else (None,)):
        # exactly the pages that are needed and four state slots: they are used again (16: many pages a request, borders everywhere)
        outputs = replay.run_trace(folder, dtype, collector.steps, tmp_path / f"out{page_size}", replay.peak_tokens(collector, page_size or 64), page_size=page_size)
        check(collector.gather(outputs), config, weights, requests, dtype)


def test_replay_hands_out_the_stream_after_every_layer(perezen_dirs, tmp_path):
    folder, config, weights = perezen_dirs["mixed"]
    requests = requests_for(config, [40, 9])
    collector = replay.chunked(requests, sizes=(7, 2, 16))
    replay.run_trace(folder, "float32", collector.steps, tmp_path / "out", replay.peak_tokens(collector), hidden_out=tmp_path / "hidden")
    layers = {name: [] for name in requests}
    for name, tokens in requests.items():
        plain.forward(config, plain.as_float64(weights), tokens, layers_out=layers[name])
    fed = {}
    for step in collector.steps:
        for e in step["entries"]:   # one request a step
            start, n = fed.get(e["id"], 0), len(e["tokens"])
            for index in range(len(config["layers"])):
                rows = np.fromfile(tmp_path / "hidden" / f"{step['step']}.{index}.f32", dtype="<f4").reshape(n, config["width"])
                np.testing.assert_allclose(rows, layers[e["id"]][index][start : start + n], atol=2e-4, rtol=2e-4, err_msg=f"step {step['step']} layer {index}")
            fed[e["id"]] = start + n


def hot_key_model(chunk, borrowed_chunk=None):
    """Layers whose mixers are all that tells a logit from another: no feed-forward. ``borrowed_chunk``: a second layer that reads the
    first one's keys and values through chunks of its own size."""
    layers = [attention_layer(heads=2, kv_heads=1, dim=16, vdim=16, scale=1.0, diff=0.3, chunk=chunk, rot=(8, 1000.0), ff=None)]
    if borrowed_chunk is not None:
        layers.append(attention_layer(heads=2, kv_heads=1, dim=16, vdim=16, scale=1.0, diff=0.3, chunk=borrowed_chunk or None, rot=(8, 1000.0), kv_from=0, ff=None))
    return model(layers, width=32, vocab=50, max_positions=400)


def plant_hot_key(weights, prefixes, token=7, heads=2, dim=16, element=12):
    """Makes every first-map query look for ``token``: column 0 of the embedding is 1 for every token and column 1 is 3 for ``token``
    alone (0 elsewhere), and the position table is silent there; one element of every head's first map, beyond the rotated ones, reads
    column 0 in the queries and column 1 in the keys, and their gains are large. The key of ``token`` then outscores every other key
    of map 1 for every query that sees it, while map 2 stays as random as it was. ``prefixes``: the first names the layer that
    keeps the keys, the others borrow them."""
    embed, pos = weights["embed"].copy(), weights["pos"].copy()
    embed[:, 0], embed[:, 1] = 1.0, 0.0
    embed[token, 1] = 3.0
    pos[:, :2] = 0.0
    weights["embed"], weights["pos"] = embed, pos
    for number, prefix in enumerate(prefixes):
        names = ["q"] + (["k"] if number == 0 else [])
        for name in names:
            w, gain = weights[prefix + name].copy(), weights[prefix + name + ".norm"].copy()
            w[:, :2] = 0.0
            n_heads = heads if name == "q" else 1
            for head in range(n_heads):
                row = head * 2 * dim + element           # map 1 of the head
                w[row] = 0.0
                w[row, 0 if name == "q" else 1] = 4.0 if name == "q" else 2.0
            gain[element] = 6.0
            weights[prefix + name] = plain_gpt2.round_to_bf16(w.astype(np.float32))
            weights[prefix + name + ".norm"] = plain_gpt2.round_to_bf16(gain.astype(np.float32))
            weights[prefix + name + ".b"] = np.zeros_like(weights[prefix + name + ".b"])
        # no layer writes into the two columns, so that a layer behind the first still finds them as the embedding left them
        o = weights[prefix + "o"].copy()
        o[:2] = 0.0
        weights[prefix + "o"] = o
    return weights


@pytest.mark.parametrize("chunk,borrowed", [(70, None), (64, None), (70, 100), (40, 0)])
def test_a_key_just_inside_and_just_outside_a_chunk_in_prompts_and_in_decoding(tmp_path, chunk, borrowed):
    # Token 7 appears once; every other token is drawn from 10..49, and every query's first map looks for token 7 (plant_hot_key).
    # The queries up to the end of the hot token's chunk see it, the first query of the next chunk does not: the logits at those
    # places are checked in whole prompts, in token-by-token decoding and in portions, with the hot token at a page's and a chunk's
    # first and last place; taking the token away moves the logits inside the chunk by far more than the tolerance, and those
    # outside it not at all. With a second layer that borrows the keys, its own chunks (longer, or none at all) decide what it sees.
    config = hot_key_model(chunk, borrowed)
    prefixes = ["l0.mix."] + (["l1.mix."] if borrowed is not None else [])
    weights = plant_hot_key(plain.random_weights(config, 77), prefixes)
    rng = np.random.default_rng(3)
    folder = plain.write_model_dir(tmp_path / "model", config, weights)
    widest = max(chunk, borrowed or 0) if borrowed != 0 else 150
    requests = {}
    for at in (0, 63, 64, chunk - 1, chunk, 2 * chunk - 1):
        tokens = rng.integers(10, 50, size=at + widest + 8).tolist()
        tokens[at] = 7
        requests[f"hot{at}"] = tokens
    for dtype in ("float32", "bfloat16"):
        for mode in ("whole", "tail", "chunked"):
            collector = MODES[mode](requests)
            outputs = replay.run_trace(folder, dtype, collector.steps, tmp_path / f"{dtype}{mode}", replay.peak_tokens(collector))
            check(collector.gather(outputs), config, weights, requests, dtype)
    w = plain.as_float64(weights)
    for at in (0, chunk - 1, chunk):
        tokens = requests[f"hot{at}"]
        without = list(tokens)
        without[at] = 11
        moved = np.abs(plain.forward(config, w, without) - plain.forward(config, w, tokens)).max(axis=1)
        def end_of(size):
            return len(tokens) if not size else (at // size + 1) * size
        last_seen = max(end_of(chunk), end_of(borrowed) if borrowed is not None else 0)
        assert moved[min(end_of(chunk), len(tokens)) - 1] > 100 * TOLERANCE["float32"]["atol"], (at, moved[end_of(chunk) - 1])
        if borrowed is not None:
            assert moved[last_seen - 1] > 100 * TOLERANCE["float32"]["atol"], (at, last_seen, moved[last_seen - 1])
        if last_seen < len(tokens):
            assert moved[last_seen:].max() < 1e-9, (at, last_seen)


def test_a_state_slot_that_is_used_again_starts_from_zero(tmp_path):
    # matrix memories only, one live request at a time in a cache with a single slot: what the request before left in the slot would
    # show in every logit of the next one
    config = model([mlstm_layer(heads=2, dim=8, vdim=8, ff=None), mlstm_layer(heads=1, dim=16, vdim=8, cap=None, ff=24)], width=32, vocab=40)
    weights = plain.random_weights(config, 9)
    folder = plain.write_model_dir(tmp_path / "model", config, weights)
    requests = requests_for(config, [30, 30, 7, 30])
    collector = replay.chunked(requests, sizes=(5, 1, 1, 9))
    out_dir = tmp_path / "out"
    done = subprocess.run([sys.executable, str(replay.ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32", "--out", str(out_dir),
                           "--max-tokens", "64", "--max-requests", "1"], input="".join(json.dumps(s) + "\n" for s in collector.steps), capture_output=True,
                          text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    outputs = {s["step"]: np.fromfile(out_dir / f"{s['step']}.f32", dtype="<f4").reshape(-1, config["vocab"]) for s in collector.steps}
    check(collector.gather(outputs), config, weights, requests, "float32")


def test_the_weight_of_the_second_map_and_the_scale_of_the_logits_show(tmp_path):
    # the four vectors that make the second map's weight, `diff` and `logit_scale` each move the logits
    config = model([attention_layer(heads=2, kv_heads=2, dim=8, vdim=8, chunk=None, rot=None, diff=0.2, ff=None)], width=32, vocab=40, logit_scale=1.0)
    base = plain.random_weights(config, 5)
    requests = requests_for(config, [20, 3])
    logits = {}
    for name in ("base", "lq2", "diff", "scale"):
        weights, changed = dict(base), copy.deepcopy(config)
        if name == "lq2":
            weights["l0.mix.lq2"] = plain_gpt2.round_to_bf16((base["l0.mix.lk2"] * 8.0).astype(np.float32))
        if name == "diff":
            changed["layers"][0]["mixer"]["diff"] = 0.6
        if name == "scale":
            changed["logit_scale"] = 2.5
        folder = plain.write_model_dir(tmp_path / name, changed, weights)
        collector = replay.whole(requests)
        got = collector.gather(replay.run_trace(folder, "float32", collector.steps, tmp_path / f"out_{name}", 128))
        check(got, changed, weights, requests, "float32")
        logits[name] = got
    for name in ("lq2", "diff"):
        assert np.abs(logits[name]["r0"][19] - logits["base"]["r0"][19]).max() > 1e-2, name
    np.testing.assert_allclose(logits["scale"]["r0"][19], 2.5 * logits["base"]["r0"][19], rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_through_the_engine_and_its_scheduler(perezen_dirs, dtype):
    from mini_llm_amd.engine.engine import Engine, EngineOptions

    folder, config, weights = perezen_dirs["mixed"]
    prompts = [random_tokens(9, 5, config["vocab"]), random_tokens(10, 70, config["vocab"]), [3], random_tokens(11, 31, config["vocab"])]
    # few pages: four requests of up to 70 + 24 tokens do not all fit at once, so pages and slots are given back and used again
    with Engine(folder, EngineOptions(dtype=dtype, max_sessions=4, max_length=256, max_tokens=256)) as engine:
        generated = engine.generate(prompts, max_new_tokens=24)
        with engine.open_session() as session:
            first = session.prefill(prompts[1])
    w = plain.as_float64(weights)
    rnd = plain_gpt2.stored_as_bf16 if dtype == "bfloat16" else None
    for prompt, new in zip(prompts, generated):
        assert len(new) == 24
        logits = plain.forward(config, w, list(prompt) + list(new), round_to=rnd)
        for k, token in enumerate(new):   # greedy: the plain implementation's own choice, unless the two lie within rounding
            row = logits[len(prompt) - 1 + k]
            assert row[token] >= row.max() - (2e-4 if dtype == "float32" else 0.5), (prompt[:3], k, token, int(row.argmax()))
    want = plain.forward(config, w, prompts[1])[-1]
    if dtype == "float32":
        np.testing.assert_allclose(first, want, **TOLERANCE["float32"])
    else:
        assert want[int(np.argmax(first))] >= want.max() - 3.0


def test_the_command_line_completes_greedily(perezen_dirs):
    folder, config, weights = perezen_dirs["odd"]
    prompt = random_tokens(12, 9, config["vocab"])
    done = subprocess.run([sys.executable, str(replay.ROOT / "bin" / "complete"), "--model", str(folder), "--dtype", "float32", "--temperature", "0",
                           "--max-new-tokens", "12", "--max-length", "128", "--tokens", ",".join(map(str, prompt))], capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    new = [int(t) for t in done.stdout.strip().split(",")]
    logits = plain.forward(config, plain.as_float64(weights), prompt + new)
    assert len(new) == 12
    for k, token in enumerate(new):
        row = logits[len(prompt) - 1 + k]
        assert row[token] >= row.max() - 2e-4, (k, token, int(row.argmax()))


def test_long_decoding_from_captured_steps(perezen_dirs):
    # 380 decoded tokens, one by one, from captured steps: past five pages, past the edges of every chunk, the matrix memory moved on
    # 380 times, up to the last row of the position table
    from mini_llm_amd.engine.engine import Engine, EngineOptions

    folder, config, weights = perezen_dirs["wide"]
    prompt = random_tokens(4, 3, config["vocab"])
    with Engine(folder, EngineOptions(dtype="float32", max_sessions=2, max_tokens=1024)) as engine:
        new = engine.generate([prompt], max_new_tokens=380)[0]
    assert len(new) == 380
    logits = plain.forward(config, plain.as_float64(weights), prompt + new)
    wrong = [k for k, token in enumerate(new) if logits[len(prompt) - 1 + k][token] < logits[len(prompt) - 1 + k].max() - 5e-4]
    assert not wrong, wrong[:5]


def test_the_position_table_bounds_a_sequence(perezen_dirs):
    # a prompt too long for the new tokens to fit is cut from the left; the last new token then sits on the table's last row
    from mini_llm_amd.engine.engine import Engine, EngineOptions

    folder, config, weights = perezen_dirs["odd"]   # 300 positions
    prompt = random_tokens(5, 290, config["vocab"])
    with Engine(folder, EngineOptions(dtype="float32", max_sessions=2)) as engine:
        new = engine.generate([prompt], max_new_tokens=50)[0]
    assert len(new) == 50
    kept = prompt[-250:]
    logits = plain.forward(config, plain.as_float64(weights), kept + new)
    assert len(kept + new) == config["max_positions"]
    wrong = [k for k, token in enumerate(new) if logits[len(kept) - 1 + k][token] < logits[len(kept) - 1 + k].max() - 5e-4]
    assert not wrong, wrong[:5]


def test_config_json_round_trip_and_random_weights(tmp_path):
    from mini_llm_amd.config import config_from_dict
    from mini_llm_amd.engine.engine import Engine, EngineOptions
    from mini_llm_amd.weights import write_model_dir

    config = config_from_dict(CASES["mixed"])
    folder = write_model_dir(config, 3, tmp_path / "random")
    plain_config = json.loads((folder / "config.json").read_text())
    assert plain_config["layers"][2]["mixer"]["kv_from"] == 0 and plain_config["layers"][2]["mixer"]["mask"] == {"size": 100}
    weights = plain_gpt2.read_safetensors(folder / "model.safetensors")
    assert set(weights) == set(plain.tensor_shapes(plain_config))
    with Engine(folder, EngineOptions(dtype="float32", max_sessions=2, max_length=64)) as engine:
        got = engine.forward_last([1, 2, 3, 4, 5])
    np.testing.assert_allclose(got, plain.forward(plain_config, plain.as_float64(weights), [1, 2, 3, 4, 5])[-1], atol=2e-4, rtol=2e-4)
