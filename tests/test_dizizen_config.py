"""The Dizizen configuration, its registry entry, the tensors and cache groups its model declares, and the plain implementation's own
mechanisms against each other (no GPU)."""

import copy

import numpy as np
import pytest

import plain_dizizen as plain
from dizizen_cases import CASES, dense, layer, model, moe
from mini_llm_amd.config import ConfigError, DizizenConfig, config_from_dict
from mini_llm_amd.engine.loading import build_model


@pytest.mark.parametrize("name", list(CASES))
def test_round_trip_tensor_names_and_cache(name):
    raw = CASES[name]
    config = config_from_dict(raw)
    assert isinstance(config, DizizenConfig) and config_from_dict(config.to_dict()) == config
    built = build_model(config, "float32")
    assert {n: tuple(s.shape) for n, s in built.named_tensor_specs().items()} == plain.tensor_shapes(raw)
    # pages for every layer with keys and values of its own; a layer that borrows has none, and is scheduled onto its source's
    own = [i for i, entry in enumerate(raw["layers"]) if entry["mixer"].get("kv_from") is None]
    assert sorted(i for group in built.cache_groups() for i in group.layers) == own
    for group in built.cache_groups():
        for i in group.layers:
            mixer = raw["layers"][i]["mixer"]
            assert group.n_kv_heads == mixer["kv_heads"] and group.window is None
            assert group.head_size == -(-max(mixer["dim"], mixer["vdim"]) // 16) * 16
    for index, (call, entry) in enumerate(zip(built.schedule, raw["layers"])):
        source = entry["mixer"].get("kv_from")
        assert (call.cache, call.write_cache) == ((index, True) if source is None else (source, False))
    assert built.state_needs() == {} and built.all_graph_safe() and built.max_positions() is None
    # every layer but the last knows the norm that reads its sum next
    assert all(a._following is b.norm_1 for a, b in zip(built.blocks, built.blocks[1:])) and built.blocks[-1]._following is None


def test_what_config_json_leaves_out():
    raw = model([layer(mlp=moe(experts=4, top=2)), layer(mlp=None)])
    config = config_from_dict(raw)
    routed = config.layers[0].mlp
    assert (routed.identity, routed.groups, routed.keep, routed.shared_ff) == (0, 1, 1, None)
    assert config.layers[1].mlp is None
    names = set(build_model(config, "float32").named_tensor_specs())
    assert "l0.mlp.shared.up" not in names and "l1.ls2" not in names and "l1.rg2" not in names and "l1.ls1" in names


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
    broken(lambda c: c["layers"][0]["mixer"].update(vdim=15), "pairs")
    broken(lambda c: c["layers"][2]["mixer"].update(kv_from=2), "kv_from")          # not itself
    broken(lambda c: c["layers"][3]["mixer"].update(kv_from=2), "kv_from")          # not a layer that borrows
    broken(lambda c: c["layers"][2]["mixer"].update(kv_from=1), "other heads")      # other sizes
    broken(lambda c: c["layers"][0]["mlp"].update(kind="conv"), "mlp.kind")
    broken(lambda c: c["layers"][0]["mlp"].update(limit=0.0), "limit")
    broken(lambda c: c["layers"][1]["mlp"]["router"].update(top=5), "picked")        # two kept groups of two
    broken(lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=3), "groups")
    broken(lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(keep=5), "groups")
    broken(lambda c: c.pop("residual_mult"), "residual_mult")
    broken(lambda c: c.pop("embedding"), "embedding")
    broken(lambda c: c["norm"].update(eps=0.0), "eps")


# -- the plain mechanisms against each other ---------------------------------------------------------------------------------------
def test_rotation_pairs_halves_and_goes_by_distance():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(1, 1, 12))
    turned = plain.rotate_halves(x, [5], 8, 100.0)
    np.testing.assert_allclose(turned[..., 8:], x[..., 8:])                      # beyond the rotated elements nothing moves
    a = 5 * 100.0 ** (-2.0 * 1 / 8)                                              # pair 1 is (element 1, element 5)
    np.testing.assert_allclose(turned[0, 0, 1], x[0, 0, 1] * np.cos(a) - x[0, 0, 5] * np.sin(a))
    np.testing.assert_allclose(turned[0, 0, 5], x[0, 0, 5] * np.cos(a) + x[0, 0, 1] * np.sin(a))
    q, k = rng.normal(size=(1, 1, 8)), rng.normal(size=(1, 1, 8))
    near = plain.rotate_halves(q, [7], 8, 50.0)[0, 0] @ plain.rotate_halves(k, [3], 8, 50.0)[0, 0]
    far = plain.rotate_halves(q, [1007], 8, 50.0)[0, 0] @ plain.rotate_halves(k, [1003], 8, 50.0)[0, 0]
    np.testing.assert_allclose(near, far, atol=1e-9)
    np.testing.assert_allclose(plain.rotate_halves(turned, [5], 8, 100.0, sign=-1.0), x, atol=1e-12)


def test_turned_values_enter_a_sum_by_their_distance():
    # a head's sum over values turned by their own position, turned back by the query's: every value turned by (j - i)
    rng = np.random.default_rng(1)
    T, vdim, base = 9, 6, 30.0
    q, k, v = rng.normal(size=(T, 1, 4)), rng.normal(size=(T, 1, 4)), rng.normal(size=(T, 1, vdim))
    positions = np.arange(T) + 40
    kept = plain.rotate_halves(v, positions, vdim, base)
    out = plain.rotate_halves(plain.causal_attention(q, k, kept, 0.5), positions, vdim, base, sign=-1.0)
    for i in range(T):
        s = (k[: i + 1, 0] @ q[i, 0]) * 0.5
        w = np.exp(s - s.max())
        w /= w.sum()
        want = sum(w[j] * plain.rotate_halves(v[j : j + 1], [j - i], vdim, base)[0, 0] for j in range(i + 1))
        np.testing.assert_allclose(out[i, 0], want, atol=1e-12)
    # and it is not the plain sum: the turn shows
    assert np.abs(out - plain.causal_attention(q, k, v, 0.5)).max() > 0.1


def test_the_clamped_gate_unit():
    g, u = np.array([-3.0, 0.5, 2.0, 9.0]), np.array([-7.0, 0.25, 0.9, 4.0])
    got = plain.clamped_gate_unit(g, u, 1.0)
    gc, uc = np.array([-3.0, 0.5, 1.0, 1.0]), np.array([-1.0, 0.25, 0.9, 1.0])     # the gate is cut from above only, the other half on both sides
    np.testing.assert_allclose(got, gc / (1.0 + np.exp(-1.702 * gc)) * (uc + 1.0))
    assert got[0] == 0.0                                                           # u = -1 silences a unit whatever its gate


def test_the_router_picks_inside_the_best_groups_and_weighs_by_the_scores():
    z = np.log(np.array([[0.30, 0.05, 0.25, 0.24, 0.10, 0.06]]))
    none = np.zeros(6)
    # one group: the three largest scores, weights their shares of the three
    w = plain.route(z, none, 3, 1, 1)[0]
    np.testing.assert_allclose(w, np.array([0.30, 0, 0.25, 0.24, 0, 0]) / 0.79)
    # three groups of two, one kept: the group of the best score, so its weak neighbour is picked although four scores are larger
    w = plain.route(z, none, 2, 3, 1)[0]
    np.testing.assert_allclose(w, np.array([0.30, 0.05, 0, 0, 0, 0]) / 0.35)
    # the correction moves the choice, not the weights: expert 5 is lifted into the pick, and weighs by its small score
    w = plain.route(z, np.array([0, 0, 0, 0, 0, 0.3]), 2, 1, 1)[0]
    np.testing.assert_allclose(w, np.array([0.30, 0, 0, 0, 0, 0.06]) / 0.36)
    # corrections below zero: experts outside the kept groups count as minus infinity, not as zero, so a negative choice score inside a kept
    # group still wins over them
    w = plain.route(z, np.array([0.0, -0.5, -1.0, -1.0, -1.0, -1.0]), 2, 3, 1)[0]
    np.testing.assert_allclose(w, np.array([0.30, 0.05, 0, 0, 0, 0]) / 0.35)


def test_experts_that_hand_their_input_on_and_the_shared_expert():
    rng = np.random.default_rng(2)
    width = 8
    mlp = moe(experts=2, identity=2, top=2, ff=4, shared=6)
    tensors = {f"m.e{e}.{n}": rng.normal(size=(4, width) if n == "up" else (width, 4)) for e in range(2) for n in ("up", "down")}
    tensors.update({"m.shared.up": rng.normal(size=(6, width)), "m.shared.down": rng.normal(size=(width, 6)), "m.correction": np.zeros(4)})
    h = rng.normal(size=(3, width))
    shared = plain.squared_relu_expert(h, tensors["m.shared.up"], tensors["m.shared.down"])
    # a router that always picks the two experts without tensors: their weights sum to one, so the routed part is h itself
    tensors["m.router"] = np.zeros((4, width))
    tensors["m.correction"] = np.array([0.0, 0.0, 1.0, 1.0])
    np.testing.assert_allclose(plain.routed_feed_forward(h, mlp, tensors, "m."), h + shared, atol=1e-12)
    # and one that always picks the two with matrices, equally
    tensors["m.correction"] = np.array([1.0, 1.0, 0.0, 0.0])
    both = sum(0.5 * plain.squared_relu_expert(h, tensors[f"m.e{e}.up"], tensors[f"m.e{e}.down"]) for e in range(2))
    np.testing.assert_allclose(plain.routed_feed_forward(h, mlp, tensors, "m."), both + shared, atol=1e-12)


def test_the_layer_norms_once_and_adds_both_branches():
    raw = model([layer(heads=2, kv_heads=1, dim=8, vdim=8, mlp=dense(ff=12, limit=2.0))], width=16, vocab=20, mult=0.25)
    w = plain.as_float64(plain.random_weights(raw, 3))
    x = np.random.default_rng(4).normal(size=(5, 16))
    h = plain.centred_rms_norm(x, w["l0.norm1"], 1e-5)
    np.testing.assert_allclose(h, x / np.sqrt((x * x).mean(axis=1, keepdims=True) + 1e-5) * (1.0 + w["l0.norm1"]))
    a = plain.attention_mixer(h, np.arange(5), raw["layers"][0]["mixer"], w, "l0.mix.", {}, 0)
    b = plain.dense_feed_forward(h, raw["layers"][0]["mlp"], w, "l0.mlp.")
    g1 = plain.sigmoid(h @ w["l0.rg1"].T + w["l0.rg1.b"])
    g2 = plain.sigmoid(h @ w["l0.rg2"].T + w["l0.rg2.b"])
    want = x + 0.25 * (a * w["l0.ls1"] * g1 + b * w["l0.ls2"] * g2)
    np.testing.assert_allclose(plain.layer_forward(x, np.arange(5), raw, w, 0, {}), want, atol=1e-12)


def test_a_layer_that_borrows_reads_the_keys_as_they_are_kept():
    # the borrowing layer's result depends on the source's key and value matrices and not on any of its own
    raw = model([layer(mlp=None), layer(kv_from=0, mlp=None)], width=32, vocab=30)
    w = plain.as_float64(plain.random_weights(raw, 5))
    assert "l1.mix.k" not in w and "l1.mix.v" not in w
    tokens = list(range(12))
    base = plain.forward(raw, w, tokens)
    changed = dict(w)
    changed["l0.mix.v"] = w["l0.mix.v"] * 1.5
    only_first = copy.deepcopy(raw)
    only_first["layers"] = raw["layers"][:1]
    moved_alone = np.abs(plain.forward(only_first, changed, tokens) - plain.forward(only_first, w, tokens)).max()
    assert np.abs(plain.forward(raw, changed, tokens) - base).max() > 0 and moved_alone > 0


def test_greedy_generation_is_prefix_stable():
    raw = CASES["mixed"]
    w = plain.as_float64(plain.random_weights(raw, 6))
    new = plain.greedy(raw, w, [3, 1, 4], 5)
    assert plain.greedy(raw, w, [3, 1, 4] + new[:2], 3) == new[2:]


def test_the_gates_and_the_router_ride_in_the_attention_input_product():
    # bound on the host (nothing runs there): the attention's fused input matrix holds q, k, v, then the block's two gate matrices, then
    # the router's rows, and the biases lie beside their rows
    import torch

    from mini_llm_amd.weights import bind_tensors

    raw = CASES["mixed"]
    built = build_model(config_from_dict(raw), "float32")
    weights = plain.random_weights(raw, 11)
    bind_tensors(built, {name: torch.tensor(value) for name, value in weights.items()}, "cpu")
    width = raw["width"]
    for index, (block, entry) in enumerate(zip(built.blocks, raw["layers"])):
        mixer, m = block.mixer, entry["mixer"]
        own = m["heads"] * m["dim"] + (0 if "kv_from" in m else m["kv_heads"] * (m["dim"] + m["vdim"]))
        gates_at, gates_n = mixer._carried_at["gates"]
        assert gates_at == own and gates_n >= (2 if entry["mlp"] else 1) * width and block.gates is None
        fused, bias = mixer.w_in.numpy(), mixer.b_in.numpy()
        np.testing.assert_array_equal(fused[: m["heads"] * m["dim"]], weights[f"l{index}.mix.q"])
        np.testing.assert_array_equal(fused[gates_at : gates_at + width], weights[f"l{index}.rg1"])
        np.testing.assert_array_equal(bias[gates_at : gates_at + width], weights[f"l{index}.rg1.b"])
        np.testing.assert_array_equal(bias[: m["heads"] * m["dim"]], weights[f"l{index}.mix.q.b"])
        if entry["mlp"]:
            np.testing.assert_array_equal(fused[gates_at + width : gates_at + 2 * width], weights[f"l{index}.rg2"])
            np.testing.assert_array_equal(bias[gates_at + width : gates_at + 2 * width], weights[f"l{index}.rg2.b"])
        routed = (entry["mlp"] or {}).get("kind") == "moe"
        assert ("feed_forward" in mixer._carried_at) == routed == block._feed_forward_rides
        if routed:
            at, n = mixer._carried_at["feed_forward"]
            outputs = weights[f"l{index}.mlp.router"].shape[0]
            assert at == gates_at + gates_n and n >= outputs
            np.testing.assert_array_equal(fused[at : at + outputs], weights[f"l{index}.mlp.router"])
            assert not bias[at : at + n].any() and not fused[at + outputs : at + n].any()
