"""The Dizizen design through the framework: replayed traces (whole prompts, decoding, portions, mixed batches with pages used again)
against the plain implementation, generation through the entry point and the scheduler, and weights made so that a far key, a key at
a page's border or a lost page shows in the logits."""

import copy
import json
import subprocess
import sys

import numpy as np
import pytest

import plain_dizizen as plain
import plain_gpt2
import replay
from conftest import random_tokens
from dizizen_cases import CASES, layer, model

pytestmark = pytest.mark.gpu


def sharpen(config, weights, factor=4.0):
    """Random projections give nearly uniform softmaxes, under which a wrong key or page hardly moves a logit: the query matrices and
    their biases are scaled up, so that attention weights differ by orders of magnitude."""
    for index in range(len(config["layers"])):
        for name in (f"l{index}.mix.q", f"l{index}.mix.q.b"):
            weights[name] = plain_gpt2.round_to_bf16(weights[name] * factor)
    return weights


@pytest.fixture(scope="module")
def dizizen_dirs(tmp_path_factory):
    out = {}
    for seed, (name, config) in enumerate(CASES.items()):
        weights = sharpen(config, plain.random_weights(config, 80 + seed))
        folder = plain.write_model_dir(tmp_path_factory.mktemp(f"dizizen_{name}"), config, weights)
        out[name] = (folder, copy.deepcopy(config), weights)
    return out


def requests_for(config, lengths, seed=900):
    return {f"r{i}": random_tokens(seed + i, n, config["vocab"]) for i, n in enumerate(lengths)}


def plain_logits(config, weights, requests, bf16):
    w = plain.as_float64(weights)
    return {name: plain.forward(config, w, tokens, round_to=plain_gpt2.stored_as_bf16 if bf16 else None) for name, tokens in requests.items()}


LENGTHS = {"mixed": [5, 130, 64, 65, 1, 200, 33], "odd": [67, 2, 130, 31], "wide": [3, 150, 64, 17, 129, 260], "large": [150, 70, 3, 97]}
MODES = {"whole": replay.whole, "tail": replay.prefill_then_decode, "chunked": replay.chunked, "mixed": replay.mixed}
TOLERANCE = {"float32": dict(atol=3e-4, rtol=2e-4)}   # sums in another order than numpy's


def check(got, config, weights, requests, dtype):
    """32-bit: every logit of every position within the tolerance (one position in a hundred may be up to five times off: a router whose
    two candidates lie within rounding of each other picks the other one). bfloat16: the engine rounds at other places than the plain
    implementation does when it rounds what a bfloat16 run stores, so the two are not compared with each other but each with exact
    arithmetic, position by position (largest difference of a position's logits): the engine's distance may be three times the plain
    bfloat16 run's at nine positions in ten, one and a half times in the median and in the root mean square, and ten times, at all but
    one position in fifty: where two experts' choice scores lie within a bfloat16 rounding of the router's input, either run may pick
    either, which moves that position's logits by an expert's whole share. A wrong key, page or slot moves the logits of every
    position behind it by tens of times the noise, and shows at once in the 32-bit run of the same trace."""
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
    assert np.quantile(ratio, 0.9) <= 3.0 and np.median(ratio) <= 1.5 and np.quantile(ratio, 0.98) <= 10.0, (np.quantile(ratio, 0.9), np.median(ratio), ratio.max(), int(ratio.argmax()))
    usual = np.argsort(ratio)[: int(np.ceil(0.98 * len(ratio)))]   # without the positions at which a router's pick fell the other way
    assert np.sqrt((error[usual] ** 2).mean()) <= 1.5 * np.sqrt((noise[usual] ** 2).mean()) + 1e-3, "rms error against rms noise"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("name", list(CASES))
def test_replay_matches_plain(dizizen_dirs, tmp_path, name, mode, dtype):
    folder, config, weights = dizizen_dirs[name]
    requests = requests_for(config, LENGTHS[name])
    collector = MODES[mode](requests)
    for page_size in ((None, 16) if mode == "mixed" and dtype == "float32" else (None,)):
        # exactly the pages that are needed: they are used again (16: many pages a request, borders everywhere)
        outputs = replay.run_trace(folder, dtype, collector.steps, tmp_path / f"out{page_size}", replay.peak_tokens(collector, page_size or 64), page_size=page_size)
        check(collector.gather(outputs), config, weights, requests, dtype)


def test_replay_hands_out_the_stream_after_every_layer(dizizen_dirs, tmp_path):
    folder, config, weights = dizizen_dirs["mixed"]
    requests = requests_for(config, [40, 9])
    collector = replay.chunked(requests, sizes=(7, 2, 16))
    replay.run_trace(folder, "float32", collector.steps, tmp_path / "out", replay.peak_tokens(collector), hidden_out=tmp_path / "hidden")
    layers = {name: [] for name in requests}
    for name, tokens in requests.items():
        plain.forward(config, plain.as_float64(weights), tokens, streams=layers[name])
    fed = {}
    for step in collector.steps:
        for e in step["entries"]:   # one request a step
            start, n = fed.get(e["id"], 0), len(e["tokens"])
            for index in range(len(config["layers"])):
                rows = np.fromfile(tmp_path / "hidden" / f"{step['step']}.{index}.f32", dtype="<f4").reshape(n, config["width"])
                np.testing.assert_allclose(rows, layers[e["id"]][index][start : start + n], atol=2e-4, rtol=2e-4, err_msg=f"step {step['step']} layer {index}")
            fed[e["id"]] = start + n


def hot_key_model(borrowed=False):
    """Layers whose mixers are all that tells a logit from another: no feed-forward. ``borrowed``: a second layer that reads the first
    one's keys and values."""
    layers = [layer(heads=2, kv_heads=1, dim=16, vdim=16, scale=1.0, rot=(8, 1000.0), mlp=None)]
    if borrowed:
        layers.append(layer(heads=2, kv_heads=1, dim=16, vdim=16, scale=1.0, rot=(8, 1000.0), kv_from=0, mlp=None))
    return model(layers, width=32, vocab=50, mult=1.0, embedding_scale=4.0)


def plant_hot_key(config, weights, prefixes, token=7, heads=2, dim=16, element=12):
    """Makes every query look for ``token``: column 0 of the embedding is the same for every token and column 1 is large for ``token``
    alone (0 elsewhere); one element of every head, beyond the rotated ones, reads column 0 in the queries and column 1 in the keys.
    The key of ``token`` then outscores every other key for every query that sees it. ``prefixes``: the first names the layer that
    keeps the keys, the others borrow them."""
    scale = float(config["embedding"]["scale"])
    embed = weights["embed"].copy()
    embed[:, 0], embed[:, 1] = 1.0 / scale, 0.0
    embed[token, 1] = 3.0 / scale
    weights["embed"] = plain_gpt2.round_to_bf16(embed.astype(np.float32))
    for number, prefix in enumerate(prefixes):
        for name in ["q"] + (["k"] if number == 0 else []):
            w, b = weights[prefix + name].copy(), weights[prefix + name + ".b"].copy()
            w[:, :2] = 0.0
            for head in range(heads if name == "q" else 1):
                row = head * dim + element
                w[row], b[row] = 0.0, 0.0
                w[row, 0 if name == "q" else 1] = 6.0 if name == "q" else 3.0
            weights[prefix + name] = plain_gpt2.round_to_bf16(w.astype(np.float32))
            weights[prefix + name + ".b"] = plain_gpt2.round_to_bf16(b.astype(np.float32))
        # no layer writes into the two columns, so that a layer behind the first still finds them as the embedding left them
        o, ob = weights[prefix + "o"].copy(), weights[prefix + "o.b"].copy()
        o[:2], ob[:2] = 0.0, 0.0
        weights[prefix + "o"], weights[prefix + "o.b"] = o, ob
        layer_prefix = prefix[: -len("mix.")]
        weights[layer_prefix + "norm1"] = np.zeros_like(weights[layer_prefix + "norm1"])
    return weights


@pytest.mark.parametrize("borrowed", [False, True])
def test_a_far_key_and_keys_at_page_borders_in_prompts_and_in_decoding(tmp_path, borrowed):
    # Token 7 appears once; every other token is drawn from 10..49, and every query looks for token 7 (plant_hot_key). The hot token sits
    # at a sequence's first place, at a page's last and first place, and hundreds of tokens before the places that are asked for; the
    # logits are checked in whole prompts, in token-by-token decoding and in portions. Taking the token away moves the logits of every
    # place behind it by far more than the tolerance, and those before it not at all.
    config = hot_key_model(borrowed)
    prefixes = ["l0.mix."] + (["l1.mix."] if borrowed else [])
    weights = plant_hot_key(config, plain.random_weights(config, 77), prefixes)
    rng = np.random.default_rng(3)
    folder = plain.write_model_dir(tmp_path / "model", config, weights)
    requests = {}
    for at, length in ((0, 70), (63, 80), (64, 140), (127, 200), (128, 131), (5, 420), (2, 3)):
        tokens = rng.integers(10, 50, size=length).tolist()
        tokens[at] = 7
        requests[f"hot{at}"] = tokens
    for dtype in ("float32", "bfloat16"):
        for mode in ("whole", "tail", "chunked"):
            collector = MODES[mode](requests)
            outputs = replay.run_trace(folder, dtype, collector.steps, tmp_path / f"{dtype}{mode}", replay.peak_tokens(collector))
            check(collector.gather(outputs), config, weights, requests, dtype)
    w = plain.as_float64(weights)
    for at in (0, 64, 5):
        tokens = requests[f"hot{at}"]
        without = list(tokens)
        without[at] = 11
        moved = np.abs(plain.forward(config, w, without) - plain.forward(config, w, tokens)).max(axis=1)
        assert moved[-1] > 100 * TOLERANCE["float32"]["atol"] and moved[at + 1 :].min() > 30 * TOLERANCE["float32"]["atol"], (at, moved[-1], moved[at + 1 :].min())
        assert at == 0 or moved[:at].max() < 1e-9, at


def test_every_constant_of_the_design_shows(tmp_path):
    # the multiplier of the residual sum, the embedding's scale, the limit of the gate unit and the experts that hand their input on each
    # move the logits, and the framework follows
    base_config = CASES["mixed"]
    base = plain.random_weights(base_config, 5)
    requests = requests_for(base_config, [20, 3])
    logits = {}
    for name in ("base", "mult", "scale", "limit", "top"):
        changed = copy.deepcopy(base_config)
        if name == "mult":
            changed["residual_mult"] = 0.9
        if name == "scale":
            changed["embedding"]["scale"] = 3.0
        if name == "limit":
            changed["layers"][0]["mlp"]["limit"] = 0.2
        if name == "top":
            changed["layers"][1]["mlp"]["router"]["top"] = 1
        folder = plain.write_model_dir(tmp_path / name, changed, base)
        collector = replay.whole(requests)
        got = collector.gather(replay.run_trace(folder, "float32", collector.steps, tmp_path / f"out_{name}", 128))
        check(got, changed, base, requests, "float32")
        logits[name] = got
    for name in ("mult", "scale", "limit", "top"):
        assert np.abs(logits[name]["r0"][19] - logits["base"]["r0"][19]).max() > 1e-2, name


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_through_the_engine_and_its_scheduler(dizizen_dirs, dtype):
    from mini_llm_amd.engine.engine import Engine, EngineOptions

    folder, config, weights = dizizen_dirs["mixed"]
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


def test_the_command_line_completes_greedily(dizizen_dirs):
    folder, config, weights = dizizen_dirs["odd"]
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


def test_long_decoding_from_captured_steps(dizizen_dirs):
    # 400 decoded tokens, one by one, from captured steps: past six pages, every value turned by its own position and every sum turned back
    from mini_llm_amd.engine.engine import Engine, EngineOptions

    folder, config, weights = dizizen_dirs["wide"]
    prompt = random_tokens(4, 3, config["vocab"])
    with Engine(folder, EngineOptions(dtype="float32", max_sessions=2, max_length=512, max_tokens=1024)) as engine:
        new = engine.generate([prompt], max_new_tokens=400)[0]
    assert len(new) == 400
    logits = plain.forward(config, plain.as_float64(weights), prompt + new)
    wrong = [k for k, token in enumerate(new) if logits[len(prompt) - 1 + k][token] < logits[len(prompt) - 1 + k].max() - 5e-4]
    assert not wrong, wrong[:5]


def test_config_json_round_trip_and_random_weights(tmp_path):
    from mini_llm_amd.config import config_from_dict
    from mini_llm_amd.engine.engine import Engine, EngineOptions
    from mini_llm_amd.weights import write_model_dir

    config = config_from_dict(CASES["mixed"])
    folder = write_model_dir(config, 3, tmp_path / "random")
    plain_config = json.loads((folder / "config.json").read_text())
    assert plain_config["layers"][2]["mixer"]["kv_from"] == 0 and plain_config["layers"][1]["mlp"]["router"]["groups"] == {"count": 4, "keep": 2}
    weights = plain_gpt2.read_safetensors(folder / "model.safetensors")
    assert set(weights) == set(plain.tensor_shapes(plain_config))
    with Engine(folder, EngineOptions(dtype="float32", max_sessions=2, max_length=64)) as engine:
        got = engine.forward_last([1, 2, 3, 4, 5])
    np.testing.assert_allclose(got, plain.forward(plain_config, plain.as_float64(weights), [1, 2, 3, 4, 5])[-1], atol=3e-4, rtol=3e-4)
