"""The Perezen configuration, its registry entry, the tensors, cache groups and state its model declares, and the plain
implementation's own mechanisms against each other (no GPU)."""

import copy

import numpy as np
import pytest

import plain_perezen as plain
from perezen_cases import CASES, attention_layer, mlstm_layer, model
from mini_llm_amd.config import ConfigError, PerezenConfig, config_from_dict
from mini_llm_amd.engine.loading import build_model


@pytest.mark.parametrize("name", list(CASES))
def test_round_trip_tensor_names_cache_and_state(name):
    raw = CASES[name]
    config = config_from_dict(raw)
    assert isinstance(config, PerezenConfig) and config_from_dict(config.to_dict()) == config
    built = build_model(config, "float32")
    assert {n: tuple(s.shape) for n, s in built.named_tensor_specs().items()} == plain.tensor_shapes(raw)
    # pages for every attention layer with keys and values of its own; a layer that borrows has none, and is scheduled onto its source's
    own = [i for i, layer in enumerate(raw["layers"]) if layer["type"] == "attention" and layer["mixer"].get("kv_from") is None]
    assert sorted(layer for group in built.cache_groups() for layer in group.layers) == own
    for group in built.cache_groups():
        for layer in group.layers:
            mixer = raw["layers"][layer]["mixer"]
            assert group.n_kv_heads == 2 * mixer["kv_heads"]       # a key head for each of the two maps
            assert group.head_size == -(-max(mixer["dim"], mixer["vdim"]) // 16) * 16
            assert group.window is None                            # a borrower with larger chunks, or none, may look further back
    for index, (call, layer) in enumerate(zip(built.schedule, raw["layers"])):
        source = layer["mixer"].get("kv_from")
        if layer["type"] == "attention":
            assert (call.cache, call.write_cache) == ((index, True) if source is None else (source, False))
    state = built.state_needs()
    for index, layer in enumerate(raw["layers"]):
        m = layer["mixer"]
        if layer["type"] == "mlstm":
            assert state[index].shape == (m["heads"] * (m["dim"] * m["vdim"] + m["dim"] + 1),)
        else:
            assert index not in state
    assert built.all_graph_safe() and built.max_positions() == raw["max_positions"]
    # every layer but the last knows the norm that reads its output next
    assert all(a._following is b.norm_1 for a, b in zip(built.blocks, built.blocks[1:])) and built.blocks[-1]._following is None


def test_what_the_configuration_refuses():
    def broken(change, match):
        bad = copy.deepcopy(CASES["mixed"])
        change(bad)
        with pytest.raises(ConfigError, match=match):
            config_from_dict(bad)

    broken(lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "divide")
    broken(lambda c: c["layers"][0].update(type="convolution"), "unknown type")
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims")
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims")
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(base=0.0), "rot.base")
    broken(lambda c: c["layers"][2]["mixer"].update(kv_from=1), "kv_from")          # a matrix memory keeps no keys
    broken(lambda c: c["layers"][2]["mixer"].update(kv_from=2), "kv_from")          # not itself
    broken(lambda c: c["layers"][6]["mixer"].update(kv_from=2), "kv_from")          # not a layer that borrows
    broken(lambda c: c["layers"][2]["mixer"].update(vdim=32), "other heads or sizes")
    broken(lambda c: c["layers"][0]["mixer"].update(dim=4096), "wider")
    broken(lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "size")
    broken(lambda c: c["layers"][1]["mixer"].update(gate_cap=0.0), "gate_cap")
    broken(lambda c: c["layers"][1].update(mlp={"kind": "routed", "ff": 8}), "mlp.kind")
    broken(lambda c: c.update(norm={"eps": 0.0}), "eps")
    with pytest.raises(ConfigError):
        config_from_dict({"architecture": "Perezen", "layers": []})


def test_what_config_json_leaves_out_is_off():
    raw = model([attention_layer(chunk=None, rot=None, ff=None), mlstm_layer(cap=None)])
    del raw["logit_scale"]
    config = config_from_dict(raw)
    assert config.logit_scale == 1.0 and config.layers[0].mixer.chunk is None and config.layers[0].mixer.rot is None
    assert config.layers[0].ff is None and config.layers[1].mixer.gate_cap is None
    built = build_model(config, "float32")
    assert built.blocks[0].mixer.rotary is None and built.blocks[0].mixer.chunk is None and built.blocks[0].feed_forward is None


def test_rotation_frequencies_of_the_part_are_the_plain_ones():
    for raw in CASES.values():
        built = build_model(config_from_dict(raw), "float32")
        for index, layer in enumerate(raw["layers"]):
            if layer["type"] != "attention":
                continue
            rot, part = layer["mixer"].get("rot"), built.blocks[index].mixer.rotary
            if rot:
                assert part.pairing == "half" and part.dims == rot["dims"]
                np.testing.assert_allclose(part.values, float(rot["base"]) ** (-2.0 * np.arange(rot["dims"] // 2) / rot["dims"]), rtol=1e-13)
            else:
                assert part is None


# -- the plain implementation's mechanisms against each other ---------------------------------------------------------------
def test_rotation_of_halves():
    rng = np.random.default_rng(2)
    x = rng.normal(0, 1, (5, 2, 12))
    turned = plain.rotate_halves(x, [0, 1, 2, 3, 100], 8, 100.0)
    np.testing.assert_allclose(turned[0], x[0])                                           # position 0 turns nothing
    np.testing.assert_allclose(turned[..., 8:], x[..., 8:])                               # beyond the rotated elements nothing turns
    np.testing.assert_allclose(turned[..., 1] ** 2 + turned[..., 5] ** 2, x[..., 1] ** 2 + x[..., 5] ** 2)   # elements 1 and 1 + 4 are a pair
    assert np.abs(turned[1:, :, 0] ** 2 + turned[1:, :, 1] ** 2 - x[1:, :, 0] ** 2 - x[1:, :, 1] ** 2).max() > 1e-3   # neighbours are not
    # the pair (1, 0) at position p with frequency 1 (element 0 of any base) becomes (cos p, sin p)
    unit = np.zeros((1, 1, 8))
    unit[0, 0, 0] = 1.0
    got = plain.rotate_halves(unit, [3], 8, 50.0)[0, 0]
    np.testing.assert_allclose([got[0], got[4]], [np.cos(3.0), np.sin(3.0)])
    a = plain.rotate_halves(x[:1], [7], 12, 50.0)[0, 0] @ plain.rotate_halves(x[1:2], [4], 12, 50.0)[0, 0]
    b = plain.rotate_halves(x[:1], [13], 12, 50.0)[0, 0] @ plain.rotate_halves(x[1:2], [10], 12, 50.0)[0, 0]
    np.testing.assert_allclose(a, b)                                                      # scores depend on the distance alone


def test_chunks_are_counted_from_the_start_of_the_sequence():
    rng = np.random.default_rng(3)
    q, k, v = rng.normal(0, 1, (11, 2, 4)), rng.normal(0, 1, (11, 1, 4)), rng.normal(0, 1, (11, 1, 3))
    seen = plain.chunked_attention(q, k, v, 0.5, size=4)
    k2, v2 = k.copy(), v.copy()
    k2[:8], v2[:8] = 9.0, 9.0
    np.testing.assert_allclose(plain.chunked_attention(q, k2, v2, 0.5, size=4)[8:], seen[8:])   # positions 8..10 see 8.. alone
    np.testing.assert_allclose(seen[8], np.broadcast_to(v[8, 0], (2, 3)))                        # the first of a chunk sees itself
    assert np.abs(plain.chunked_attention(q, k2, v2, 0.5, size=5)[8] - seen[8]).max() > 1e-3    # chunks of five: 8 sees 5..8
    np.testing.assert_allclose(plain.chunked_attention(q, k, v, 0.5, size=100), plain.chunked_attention(q, k, v, 0.5, size=None))
    assert [plain.chunk_start(i, 4) for i in (0, 3, 4, 7, 8)] == [0, 0, 4, 4, 8] and plain.chunk_start(9, None) == 0


def test_the_difference_of_two_maps():
    rng = np.random.default_rng(4)
    T, H, G, dim, vdim = 7, 2, 1, 4, 6
    q, k, v = rng.normal(0, 1, (T, H, 2, dim)), rng.normal(0, 1, (T, G, 2, dim)), rng.normal(0, 1, (T, G, vdim))
    a1 = plain.chunked_attention(q[:, :, 0], k[:, :, 0], v, 0.7)
    a2 = plain.chunked_attention(q[:, :, 1], k[:, :, 1], v, 0.7)
    got = plain.differential_attention(q, k, v, 0.7, None, 0.3, 0.25, 1e-6)
    np.testing.assert_allclose(got, plain.rms_unit(a1 - 0.3 * a2, 1e-6) * 0.75)
    # without the second map a head is its first map's result, brought to unit size
    np.testing.assert_allclose(plain.differential_attention(q, k, v, 0.7, None, 0.0, 0.25, 1e-6), plain.rms_unit(a1, 1e-6) * 0.75)
    # map 1 and map 2 are not interchangeable, and both read the same values
    swapped = plain.differential_attention(q[:, :, ::-1], k[:, :, ::-1], v, 0.7, None, 0.3, 0.25, 1e-6)
    assert np.abs(swapped - got).max() > 1e-2
    lq1, lk1, lq2, lk2 = rng.normal(0, 0.5, (4, dim))
    assert np.isclose(plain.difference_weight(lq1, lk1, lq2, lk2, 0.4), np.exp(lq1 @ lk1) - np.exp(lq2 @ lk2) + 0.4)


def test_the_matrix_memory_is_attention_with_decaying_weights_and_goes_on_from_its_state():
    rng = np.random.default_rng(0)
    T, dim, vdim = 40, 6, 5
    q, k, v = rng.normal(0, 1, (T, 1, dim)), rng.normal(0, 1, (T, 1, dim)), rng.normal(0, 1, (T, 1, vdim))
    gi, gf = rng.normal(0, 2, (T, 1)), plain.log_sigmoid(rng.normal(2, 2, (T, 1)))
    got = plain.matrix_memory(q, k, v, gi, gf)[:, 0]
    F = np.cumsum(gf[:, 0])
    for t in range(T):
        reach = F[t] - F[: t + 1] + gi[: t + 1, 0]
        m = max(F[t], reach.max())     # the maximum starts at 0 and decays with the gates: F[t] is what is left of it
        w = np.exp(reach - m) * (k[: t + 1, 0] @ q[t, 0])
        np.testing.assert_allclose(got[t], (w @ v[: t + 1, 0]) / (max(abs(w.sum()), np.exp(-m)) + 1e-6), rtol=1e-9, atol=1e-12)
    state = [(np.zeros((dim, vdim)), np.zeros(dim), 0.0)]
    parts = [plain.matrix_memory(q[a:b], k[a:b], v[a:b], gi[a:b], gf[a:b], state) for a, b in ((0, 13), (13, 14), (14, 40))]
    np.testing.assert_allclose(np.concatenate(parts)[:, 0], got, rtol=1e-12)
    assert 4.9 < plain.capped(np.array(15.0), 5.0) < 5.0 and plain.capped(np.array(0.01), 5.0) == pytest.approx(0.01, rel=1e-4)
    assert plain.capped(np.array(100.0), None) == 100.0


def test_the_plain_model_norms_before_and_behind_every_branch():
    raw = model([mlstm_layer(heads=1, dim=4, vdim=4, ff=8), attention_layer(heads=2, kv_heads=1, dim=4, vdim=4, chunk=3, rot=(2, 10.0), ff=None),
                 attention_layer(heads=2, kv_heads=1, dim=4, vdim=4, chunk=None, rot=(2, 10.0), kv_from=1, ff=8)], width=8, vocab=11, logit_scale=3.0)
    weights = plain.as_float64(plain.random_weights(raw, 3))
    layers = []
    tokens = [1, 2, 3, 4, 5]
    logits = plain.forward(raw, weights, tokens, layers_out=layers)
    assert logits.shape == (5, 11) and len(layers) == 3
    again = plain.forward(raw, weights, [1, 2, 3, 4, 9])
    np.testing.assert_allclose(again[:4], logits[:4])       # a later token changes nothing before it
    x0 = weights["embed"][tokens] + weights["pos"][:5]
    branch = plain.mlstm_mixer(plain.rms_unit(x0, 1e-5) * weights["l0.norm1"], raw["layers"][0]["mixer"], weights, "l0.mix.", 1e-5)
    x1 = x0 + plain.rms_unit(branch, 1e-5) * weights["l0.norm1b"]
    ff = plain.gated_feed_forward(plain.rms_unit(x1, 1e-5) * weights["l0.norm2"], weights, "l0.mlp.")
    np.testing.assert_allclose(layers[0], x1 + plain.rms_unit(ff, 1e-5) * weights["l0.norm2b"])
    final = plain.rms_unit(layers[2], 1e-5) * weights["final.norm"]
    np.testing.assert_allclose(logits, 3.0 * final @ weights["head"].T)
    # the layer that borrows reads layer 1's keys as they were kept: with keys of its own it would need tensors it does not have
    assert "l2.mix.k" not in weights and "l2.mix.v" not in weights
    kept = {}
    h1 = plain.rms_unit(layers[0], 1e-5) * weights["l1.norm1"]
    plain.attention_mixer(h1, np.arange(5), raw["layers"][1]["mixer"], weights, "l1.mix.", 1e-5, kept, 1)
    k, v = plain.attention_keys_values(h1, np.arange(5), raw["layers"][1]["mixer"], weights, "l1.mix.", 1e-5)
    np.testing.assert_allclose(kept[1][0], k)
    np.testing.assert_allclose(kept[1][1], v)
    assert plain.greedy(raw, weights, [1, 2], 3)[:2] == plain.greedy(raw, weights, [1, 2], 2)
