"""A plain, slow implementation of the Dizizen design: numpy, float64, whole sequences, no cache, no batching. One function per
mechanism; the framework's parts and kernels are compared with these.

A model is (config, tensors): ``config`` the dictionary that config.json holds, ``tensors`` name -> float64 array. The stream starts
as token row * embedding.scale. A layer norms the stream once, h = norm1(x), hands h to its mixer and to its feed-forward side by side,
and adds both results: x <- x + m (ls1 * sigmoid(rg1 h + b1) * mixer(h) + ls2 * sigmoid(rg2 h + b2) * ff(h)), m = residual_mult.
Logits = head . final_norm(x).

``round_to`` (optional, a function array -> array) is applied where a bfloat16 run stores something in bfloat16: the inputs of
matrix products and what lies in the cache. None: exact arithmetic."""

from __future__ import annotations

import numpy as np

QUICK_SIGMOID = 1.702   # the constant of the dense feed-forward's activation g * sigmoid(1.702 g)
WEIGHT_FLOOR = 1e-20    # joins the sum the chosen experts' scores are divided by


def _same(x):
    return x


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def product(x, w, rnd=_same, bias=None):
    """Rows of x times W^T (W stored [out, in]), plus a bias."""
    y = rnd(x) @ rnd(w).T
    return y if bias is None else y + bias


def centred_rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * (1 + w): the gain is stored around zero."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * (1.0 + w)


# -- rotation -----------------------------------------------------------------------------------------------------------
def pair_frequencies(dims: int, base: float):
    return float(base) ** (-2.0 * np.arange(dims // 2) / dims)


def rotate_halves(x, positions, dims: int, base: float, sign: float = 1.0):
    """x: [tokens, heads, size]. Of the first ``dims`` elements of the last axis, element i and element i + dims/2 make a pair
    (u, v) that becomes (u cos a - v sin a, v cos a + u sin a), a = sign * position * base^(-2i/dims); the rest stays."""
    if not dims:
        return x.copy()
    half = dims // 2
    angles = sign * np.asarray(positions, dtype=np.float64)[:, None] * pair_frequencies(dims, base)[None, :]
    c, s = np.cos(angles)[:, None, :], np.sin(angles)[:, None, :]
    out = x.copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# -- attention ----------------------------------------------------------------------------------------------------------
def causal_attention(q, k, v, scale):
    """q: [T, H, dim], k: [T, G, dim], v: [T, G, vdim] -> [T, H, vdim]; query i sees every key j <= i; an ordinary softmax."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            s = (k[: i + 1, g] @ q[i, h]) * scale
            w = np.exp(s - s.max())
            out[i, h] = (w / w.sum()) @ v[: i + 1, g]
    return out


def kept_keys_values(h, positions, mixer: dict, tensors: dict, prefix: str, rnd=_same):
    """What a layer keeps of its input rows: keys after their rotation [T, G, dim], and values turned by their own position over
    all vdim elements [T, G, vdim]."""
    G, dim, vdim = int(mixer["kv_heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    rot = mixer["rot"]
    k = product(h, tensors[prefix + "k"], rnd, tensors[prefix + "k.b"]).reshape(T, G, dim)
    k = rotate_halves(k, positions, int(rot["dims"]), float(rot["base"]))
    v = product(h, tensors[prefix + "v"], rnd, tensors[prefix + "v.b"]).reshape(T, G, vdim)
    v = rotate_halves(v, positions, vdim, float(rot["base"]))
    return rnd(k), rnd(v)


def attention_mixer(h, positions, mixer: dict, tensors: dict, prefix: str, kept: dict, layer: int, rnd=_same):
    """Attention over rows h [T, width]. ``kept``: layer -> (keys, values) of the layers before; a layer with ``kv_from`` takes
    another layer's, any other leaves its own there. Every head's sum over the (turned) values is turned back by the query's
    position before the output product."""
    H, dim, vdim = int(mixer["heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    rot = mixer["rot"]
    q = product(h, tensors[prefix + "q"], rnd, tensors[prefix + "q.b"]).reshape(T, H, dim)
    q = rnd(rotate_halves(q, positions, int(rot["dims"]), float(rot["base"])))
    source = mixer.get("kv_from")
    if source is None:
        kept[layer] = kept_keys_values(h, positions, mixer, tensors, prefix, rnd)
        source = layer
    k, v = kept[source]
    mixed = causal_attention(q, k, v, float(mixer["scale"]))
    mixed = rotate_halves(mixed, positions, vdim, float(rot["base"]), sign=-1.0)
    return product(mixed.reshape(T, H * vdim), tensors[prefix + "o"], rnd, tensors[prefix + "o.b"])


# -- feed-forwards ------------------------------------------------------------------------------------------------------
def clamped_gate_unit(g, u, limit):
    """min(g, limit) * sigmoid(1.702 min(g, limit)) * (clamp(u, -limit, limit) + 1)."""
    g = np.minimum(g, limit)
    u = np.clip(u, -limit, limit)
    return g * sigmoid(QUICK_SIGMOID * g) * (u + 1.0)


def dense_feed_forward(h, mlp: dict, tensors: dict, prefix: str, rnd=_same):
    limit = float(mlp["limit"])
    g = product(h, tensors[prefix + "gate"], rnd, tensors[prefix + "gate.b"])
    u = product(h, tensors[prefix + "up"], rnd, tensors[prefix + "up.b"])
    return product(clamped_gate_unit(g, u, limit), tensors[prefix + "down"], rnd, tensors[prefix + "down.b"])


def squared_relu_expert(h, up, down, rnd=_same):
    a = np.maximum(product(h, up, rnd), 0.0)
    return product(a * a, down, rnd)


def route(z, correction, top: int, groups: int, keep: int):
    """z: [T, E] router logits over all experts (identity experts last) -> [T, E] weights, zero for the experts not chosen.
    Scores are a softmax over all experts; the choice goes by score + correction, inside the ``keep`` groups (of ``groups`` equal
    groups of neighbours) whose best choice score is largest; the weights are the chosen experts' scores over their sum."""
    T, E = z.shape
    s = np.exp(z - z.max(axis=1, keepdims=True))
    s = s / s.sum(axis=1, keepdims=True)
    choice = s + correction[None, :]
    weights = np.zeros((T, E))
    size = E // groups
    for t in range(T):
        c = choice[t].copy()
        best = c.reshape(groups, size).max(axis=1)
        kept_groups = np.argsort(-best, kind="stable")[:keep]
        allowed = np.zeros(E, dtype=bool)
        for g in kept_groups:
            allowed[g * size : (g + 1) * size] = True
        c[~allowed] = -np.inf
        chosen = np.argsort(-c, kind="stable")[:top]
        weights[t, chosen] = s[t, chosen] / (s[t, chosen].sum() + WEIGHT_FLOOR)
    return weights


def routed_feed_forward(h, mlp: dict, tensors: dict, prefix: str, rnd=_same):
    router = mlp["router"]
    experts, identity, top = int(router["experts"]), int(router.get("identity", 0)), int(router["top"])
    groups = router.get("groups") or {"count": 1, "keep": 1}
    z = product(h, tensors[prefix + "router"], rnd)
    weights = route(z, tensors[prefix + "correction"], top, int(groups["count"]), int(groups["keep"]))
    out = np.zeros_like(h)
    for e in range(experts):
        rows = np.nonzero(weights[:, e])[0]
        if len(rows):
            out[rows] += weights[rows, e, None] * squared_relu_expert(h[rows], tensors[f"{prefix}e{e}.up"], tensors[f"{prefix}e{e}.down"], rnd)
    for e in range(experts, experts + identity):
        out += weights[:, e, None] * rnd(h)
    if mlp.get("shared"):
        out += squared_relu_expert(h, tensors[prefix + "shared.up"], tensors[prefix + "shared.down"], rnd)
    return out


def feed_forward(h, mlp, tensors, prefix, rnd=_same):
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return dense_feed_forward(h, mlp, tensors, prefix, rnd)
    if mlp["kind"] == "moe":
        return routed_feed_forward(h, mlp, tensors, prefix, rnd)
    raise ValueError(mlp["kind"])


# -- layer and model ----------------------------------------------------------------------------------------------------
def gated_scaled(branch, h, tensors, scale_name, gate_name, rnd=_same):
    """branch * layer scale * sigmoid(W h + b)."""
    return branch * tensors[scale_name] * sigmoid(product(h, tensors[gate_name], rnd, tensors[gate_name + ".b"]))


def layer_forward(x, positions, config: dict, tensors: dict, index: int, kept: dict, rnd=_same):
    layer = config["layers"][index]
    p = f"l{index}."
    h = centred_rms_norm(x, tensors[p + "norm1"], float(config["norm"]["eps"]))
    total = gated_scaled(attention_mixer(h, positions, layer["mixer"], tensors, p + "mix.", kept, index, rnd), h, tensors, p + "ls1", p + "rg1", rnd)
    ff = feed_forward(h, layer.get("mlp"), tensors, p + "mlp.", rnd)
    if ff is not None:
        total = total + gated_scaled(ff, h, tensors, p + "ls2", p + "rg2", rnd)
    return x + float(config["residual_mult"]) * total


def forward(config: dict, tensors: dict, tokens, round_to=None, streams: list | None = None):
    """Logits [T, vocab] of one whole sequence; ``streams`` collects the stream after every layer."""
    rnd = round_to or _same
    tokens = np.asarray(tokens)
    positions = np.arange(len(tokens))
    x = rnd(tensors["embed"])[tokens] * float(config["embedding"]["scale"])
    kept = {}
    for index in range(len(config["layers"])):
        x = layer_forward(x, positions, config, tensors, index, kept, rnd)
        if streams is not None:
            streams.append(x.copy())
    x = centred_rms_norm(x, tensors["final.norm"], float(config["norm"]["eps"]))
    return product(x, tensors["head"], rnd)


def tensor_shapes(config: dict) -> dict:
    """name -> shape of every tensor a model of this configuration has."""
    width, vocab = int(config["width"]), int(config["vocab"])
    shapes = {"embed": (vocab, width), "final.norm": (width,), "head": (vocab, width)}
    for index, layer in enumerate(config["layers"]):
        p, mixer, mlp = f"l{index}.", layer["mixer"], layer.get("mlp")
        H, G, dim, vdim = (int(mixer[key]) for key in ("heads", "kv_heads", "dim", "vdim"))
        shapes[p + "norm1"] = (width,)
        for n in ("1", "2") if mlp is not None else ("1",):
            shapes.update({p + "ls" + n: (width,), p + "rg" + n: (width, width), p + "rg" + n + ".b": (width,)})
        shapes.update({p + "mix.q": (H * dim, width), p + "mix.q.b": (H * dim,), p + "mix.o": (width, H * vdim), p + "mix.o.b": (width,)})
        if mixer.get("kv_from") is None:
            shapes.update({p + "mix.k": (G * dim, width), p + "mix.k.b": (G * dim,), p + "mix.v": (G * vdim, width), p + "mix.v.b": (G * vdim,)})
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            ff = int(mlp["ff"])
            shapes.update({p + "mlp.gate": (ff, width), p + "mlp.gate.b": (ff,), p + "mlp.up": (ff, width), p + "mlp.up.b": (ff,),
                           p + "mlp.down": (width, ff), p + "mlp.down.b": (width,)})
        else:
            router = mlp["router"]
            outputs = int(router["experts"]) + int(router.get("identity", 0))
            shapes.update({p + "mlp.router": (outputs, width), p + "mlp.correction": (outputs,)})
            ff = int(mlp["expert"]["ff"])
            for e in range(int(router["experts"])):
                shapes.update({p + f"mlp.e{e}.up": (ff, width), p + f"mlp.e{e}.down": (width, ff)})
            if mlp.get("shared"):
                ff = int(mlp["shared"]["ff"])
                shapes.update({p + "mlp.shared.up": (ff, width), p + "mlp.shared.down": (width, ff)})
    return shapes


def greedy(config: dict, tensors: dict, prompt, n_new: int, round_to=None) -> list:
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward(config, tensors, tokens, round_to)[-1].argmax()))
    return tokens[len(prompt):]


# -- random models for the tests ------------------------------------------------------------------------------------------
def random_weights(config: dict, seed: int) -> dict:
    """Weights whose activations stay of order one and whose every mechanism moves the logits: matrices ~ N(0, 1/in) (the router's
    larger, so that its scores differ), norm gains around zero, layer scales around one, biases of order one, corrections of the size
    of the scores. The embedding is drawn so that its rows times embedding.scale are of order one. float32 arrays holding bfloat16
    values (as files hold them)."""
    import plain_gpt2

    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        last = name.rsplit(".", 1)[-1]
        if last in ("norm", "norm1"):
            value = rng.normal(0.0, 0.1, shape)
        elif last in ("ls1", "ls2"):
            value = rng.normal(1.0, 0.3, shape)
        elif last == "correction":
            value = rng.normal(0.0, 0.5 / shape[0], shape)
        elif last == "b":
            value = rng.normal(0.0, 0.3, shape)
        elif name == "embed":
            value = rng.normal(0.0, 1.0 / float(config["embedding"]["scale"]), shape)
        elif last == "router":
            value = rng.normal(0.0, 2.0 * shape[1] ** -0.5, shape)
        else:
            value = rng.normal(0.0, shape[1] ** -0.5, shape)
        out[name] = plain_gpt2.round_to_bf16(np.asarray(value, dtype=np.float32))
    return out


def as_float64(weights: dict) -> dict:
    return {name: np.asarray(value, dtype=np.float64) for name, value in weights.items()}


def write_model_dir(path, config: dict, weights: dict):
    import json
    from pathlib import Path

    import plain_gpt2

    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(config, indent=1))
    plain_gpt2.write_safetensors(path / "model.safetensors", {k: np.asarray(v, dtype=np.float32) for k, v in weights.items()}, bf16=True)
    return path
