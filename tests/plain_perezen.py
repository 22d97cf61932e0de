"""A plain, slow implementation of the Perezen design: numpy, float64, whole sequences, token by token where the design is
recurrent, no cache, no batching. One function per mechanism; the framework's parts and kernels are compared with these.

A model is (config, tensors): ``config`` the dictionary that config.json holds, ``tensors`` name -> float64 array. The stream starts
as token row + position row. A layer is x <- x + norm1b(mixer(norm1(x))), then, if it has a feed-forward, x <- x +
norm2b(ff(norm2(x))): a norm in front of every branch and one on its output. Logits = head . final_norm(x) * logit_scale.

``round_to`` (optional, a function array -> array) is applied where a bfloat16 run stores something in bfloat16: the inputs of
matrix products and what lies in the cache. None: exact arithmetic."""

from __future__ import annotations

import numpy as np


def _same(x):
    return x


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def product(x, w, rnd=_same, bias=None):
    """Rows of x times W^T (W stored [out, in]), plus a bias."""
    y = rnd(x) @ rnd(w).T
    return y if bias is None else y + bias


# -- rotation -----------------------------------------------------------------------------------------------------------
def rotate_halves(x, positions, dims: int, base: float):
    """x: [tokens, ..., dim]. Of the first ``dims`` elements of the last axis, element i and element i + dims/2 make a pair that
    turns by position * base^(-2i/dims); what lies beyond ``dims`` stays."""
    if not dims:
        return x
    half = dims // 2
    f = float(base) ** (-2.0 * np.arange(half) / dims)
    angles = np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (half,)
    c, s = np.cos(angles).reshape(shape), np.sin(angles).reshape(shape)
    out = x.copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# -- attention inside chunks of the sequence ----------------------------------------------------------------------------
def chunk_start(i: int, size) -> int:
    """The first key that query i sees: the start of its chunk of ``size`` positions (None: position 0)."""
    return 0 if not size else (i // int(size)) * int(size)


def chunked_attention(q, k, v, scale, size=None):
    """q: [T, H, dim], k: [T, G, dim], v: [T, G, vdim] -> [T, H, vdim]. Query i sees the keys j <= i of its own chunk, chunks
    counted from position 0; an ordinary softmax over them."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = chunk_start(i, size)
            s = (k[lo : i + 1, g] @ q[i, h]) * scale
            w = np.exp(s - s.max())
            out[i, h] = (w / w.sum()) @ v[lo : i + 1, g]
    return out


def difference_weight(lq1, lk1, lq2, lk2, diff):
    """The one number of a layer by which the second map is subtracted."""
    return float(np.exp(np.sum(lq1 * lk1)) - np.exp(np.sum(lq2 * lk2)) + diff)


def differential_attention(q, k, v, scale, size, lam, diff, eps):
    """q: [T, H, 2, dim], k: [T, G, 2, dim] (two maps a head), v: [T, G, vdim]. Each map is an attention of its own over the
    same values; a head's result is a1 - lam * a2, divided by its root mean square, times (1 - diff)."""
    a1 = chunked_attention(q[:, :, 0], k[:, :, 0], v, scale, size)
    a2 = chunked_attention(q[:, :, 1], k[:, :, 1], v, scale, size)
    return rms_unit(a1 - lam * a2, eps) * (1.0 - diff)


def attention_keys_values(h, positions, mixer: dict, tensors: dict, prefix: str, eps: float, rnd=_same):
    """What a layer keeps of its input rows h: keys after norm and rotation [T, G, 2, dim] and values [T, G, vdim], as stored."""
    G, dim, vdim = int(mixer["kv_heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    k = product(h, tensors[prefix + "k"], rnd, tensors[prefix + "k.b"]).reshape(T, G, 2, dim)
    k = rms_unit(k, eps) * tensors[prefix + "k.norm"]
    rot = mixer.get("rot")
    if rot:
        k = rotate_halves(k, positions, int(rot["dims"]), float(rot["base"]))
    v = product(h, tensors[prefix + "v"], rnd, tensors[prefix + "v.b"]).reshape(T, G, vdim)
    return rnd(k), rnd(v)


def attention_mixer(h, positions, mixer: dict, tensors: dict, prefix: str, eps: float, kept: dict, layer: int, rnd=_same):
    """The differential attention mixer over rows h [T, width]. ``kept``: layer -> (keys, values) of the layers before; a layer with
    ``kv_from`` takes another layer's, any other leaves its own there."""
    H, dim = int(mixer["heads"]), int(mixer["dim"])
    T = h.shape[0]
    q = product(h, tensors[prefix + "q"], rnd, tensors[prefix + "q.b"]).reshape(T, H, 2, dim)
    q = rms_unit(q, eps) * tensors[prefix + "q.norm"]
    rot = mixer.get("rot")
    if rot:
        q = rotate_halves(q, positions, int(rot["dims"]), float(rot["base"]))
    q = rnd(q)
    source = mixer.get("kv_from")
    if source is None:
        kept[layer] = attention_keys_values(h, positions, mixer, tensors, prefix, eps, rnd)
        source = layer
    k, v = kept[int(source)]
    diff = float(mixer["diff"])
    lam = difference_weight(tensors[prefix + "lq1"], tensors[prefix + "lk1"], tensors[prefix + "lq2"], tensors[prefix + "lk2"], diff)
    size = (mixer.get("mask") or {}).get("size")
    heads = differential_attention(q, k, v, float(mixer["scale"]), size, lam, diff, eps)
    gated = heads.reshape(T, -1) * sigmoid(product(h, tensors[prefix + "g"], rnd))
    return product(gated, tensors[prefix + "o"], rnd)


# -- the matrix memory, token by token ----------------------------------------------------------------------------------
def capped(z, cap):
    return z if not cap else cap * np.tanh(z / cap)


def matrix_memory(q, k, v, log_in, log_forget, state=None):
    """q, k: [T, H, dim] (q already scaled), v: [T, H, vdim], log gates [T, H] -> [T, H, vdim]. Per head a matrix S, a vector n and
    a running maximum m, all zero at the start (``state``: a list per head of [S, n, m] to go on from, moved on in place)."""
    T, H, dim = q.shape
    vdim = v.shape[2]
    out = np.zeros((T, H, vdim))
    for h in range(H):
        S, n, m = (np.zeros((dim, vdim)), np.zeros(dim), 0.0) if state is None else state[h]
        for t in range(T):
            m_new = max(log_forget[t, h] + m, log_in[t, h])
            keep, take = np.exp(log_forget[t, h] + m - m_new), np.exp(log_in[t, h] - m_new)
            S = keep * S + take * np.outer(k[t, h], v[t, h])
            n = keep * n + take * k[t, h]
            m = m_new
            out[t, h] = (S.T @ q[t, h]) / (max(abs(n @ q[t, h]), np.exp(-m)) + 1e-6)
        if state is not None:
            state[h] = (S, n, m)
    return out


def mlstm_mixer(h, mixer: dict, tensors: dict, prefix: str, eps: float, rnd=_same):
    H, dim, vdim = int(mixer["heads"]), int(mixer["dim"]), int(mixer["vdim"])
    cap = mixer.get("gate_cap")
    T = h.shape[0]
    q = product(h, tensors[prefix + "q"], rnd).reshape(T, H, dim) * dim ** -0.5
    k = product(h, tensors[prefix + "k"], rnd).reshape(T, H, dim)
    v = product(h, tensors[prefix + "v"], rnd).reshape(T, H, vdim)
    log_in = capped(product(h, tensors[prefix + "i"], rnd, tensors[prefix + "i.b"]), cap)
    log_forget = log_sigmoid(capped(product(h, tensors[prefix + "f"], rnd, tensors[prefix + "f.b"]), cap))
    heads = rms_unit(matrix_memory(q, k, v, log_in, log_forget), eps).reshape(T, H * vdim)
    gated = heads * tensors[prefix + "norm"] * sigmoid(product(h, tensors[prefix + "g"], rnd))
    return product(gated, tensors[prefix + "o"], rnd)


# -- feed-forward, layers, model ----------------------------------------------------------------------------------------
def gated_feed_forward(h, tensors: dict, prefix: str, rnd=_same):
    inner = silu(product(h, tensors[prefix + "gate"], rnd)) * product(h, tensors[prefix + "up"], rnd)
    return product(inner, tensors[prefix + "down"], rnd)


def forward(config: dict, tensors: dict, tokens, round_to=None, layers_out: list | None = None):
    """Logits [T, vocab] of one sequence from position 0. ``layers_out``: a list that receives the stream after every layer."""
    rnd = round_to or _same
    eps = float(config["norm"]["eps"])
    tokens = np.asarray(tokens)
    positions = np.arange(len(tokens))
    x = tensors["embed"][tokens] + tensors["pos"][positions]
    kept: dict = {}
    for index, layer in enumerate(config["layers"]):
        p = f"l{index}."
        h = rms_unit(x, eps) * tensors[p + "norm1"]
        if layer["type"] == "attention":
            branch = attention_mixer(h, positions, layer["mixer"], tensors, p + "mix.", eps, kept, index, rnd)
        elif layer["type"] == "mlstm":
            branch = mlstm_mixer(h, layer["mixer"], tensors, p + "mix.", eps, rnd)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        x = x + rms_unit(branch, eps) * tensors[p + "norm1b"]
        if layer.get("mlp") is not None:
            h = rms_unit(x, eps) * tensors[p + "norm2"]
            x = x + rms_unit(gated_feed_forward(h, tensors, p + "mlp.", rnd), eps) * tensors[p + "norm2b"]
        if layers_out is not None:
            layers_out.append(x.copy())
    x = rms_unit(x, eps) * tensors["final.norm"]
    return product(x, tensors["head"], rnd) * float(config.get("logit_scale", 1.0))


def tensor_shapes(config: dict) -> dict:
    """name -> shape of every tensor a model of this configuration has."""
    width, vocab = int(config["width"]), int(config["vocab"])
    shapes = {"embed": (vocab, width), "pos": (int(config["max_positions"]), width), "final.norm": (width,), "head": (vocab, width)}
    for index, layer in enumerate(config["layers"]):
        p, mixer = f"l{index}.", layer["mixer"]
        shapes[p + "norm1"] = shapes[p + "norm1b"] = (width,)
        if layer["type"] == "attention":
            H, G, dim, vdim = (int(mixer[key]) for key in ("heads", "kv_heads", "dim", "vdim"))
            shapes.update({p + "mix.q": (H * 2 * dim, width), p + "mix.q.b": (H * 2 * dim,), p + "mix.q.norm": (dim,),
                           p + "mix.g": (H * vdim, width), p + "mix.o": (width, H * vdim)})
            shapes.update({p + f"mix.{name}": (dim,) for name in ("lq1", "lk1", "lq2", "lk2")})
            if mixer.get("kv_from") is None:
                shapes.update({p + "mix.k": (G * 2 * dim, width), p + "mix.k.b": (G * 2 * dim,), p + "mix.k.norm": (dim,),
                               p + "mix.v": (G * vdim, width), p + "mix.v.b": (G * vdim,)})
        else:
            H, dim, vdim = (int(mixer[key]) for key in ("heads", "dim", "vdim"))
            shapes.update({p + "mix.q": (H * dim, width), p + "mix.k": (H * dim, width), p + "mix.v": (H * vdim, width),
                           p + "mix.g": (H * vdim, width), p + "mix.o": (width, H * vdim), p + "mix.norm": (H * vdim,),
                           p + "mix.i": (H, width), p + "mix.i.b": (H,), p + "mix.f": (H, width), p + "mix.f.b": (H,)})
        if layer.get("mlp") is not None:
            ff = int(layer["mlp"]["ff"])
            shapes[p + "norm2"] = shapes[p + "norm2b"] = (width,)
            shapes.update({p + "mlp.gate": (ff, width), p + "mlp.up": (ff, width), p + "mlp.down": (width, ff)})
    return shapes


def greedy(config: dict, tensors: dict, prompt, n_new: int, round_to=None) -> list:
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(forward(config, tensors, tokens, round_to)[-1].argmax()))
    return tokens[len(prompt):]


# -- random models for the tests ------------------------------------------------------------------------------------------
def random_weights(config: dict, seed: int) -> dict:
    """Weights whose activations stay of order one: matrices ~ N(0, 1/in), gains around one, biases of order one, forget biases well
    above zero, the four vectors of the second map's weight small. float32 arrays holding bfloat16 values (as files hold them)."""
    import plain_gpt2

    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        last = name.rsplit(".", 1)[-1]
        if name.endswith(".f.b"):
            value = rng.normal(3.0, 0.5, shape)
        elif last in ("lq1", "lk1", "lq2", "lk2"):
            value = rng.normal(0.0, 0.25, shape)
        elif last in ("norm", "norm1", "norm2", "norm1b", "norm2b"):
            value = 1.0 + rng.normal(0.0, 0.1, shape)
        elif last == "b":
            value = rng.normal(0.0, 0.3, shape)
        elif name == "embed":
            value = rng.normal(0.0, 1.0, shape)
        elif name == "pos":
            value = rng.normal(0.0, 0.3, shape)
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
