"""Each mechanism of the Dizizen design alone: the kernel (or the part) against the plain function of tests/plain_dizizen.py."""

import numpy as np
import pytest
import torch

import plain_dizizen as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def kernels():
    from mini_llm_amd.ops import kernels

    return kernels


def gpu(array, dtype=torch.float32):
    return torch.tensor(np.asarray(array), dtype=torch.float32).to(dtype).cuda().contiguous()


def ints(values):
    return torch.tensor(np.asarray(values), dtype=torch.int32).cuda()


def rounded(array, dtype):
    return torch.tensor(np.asarray(array), dtype=torch.float32).to(dtype).to(torch.float32).numpy().astype(np.float64)


def tol(dtype):
    return dict(atol=3e-5, rtol=3e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def frequencies(dims, base):
    return torch.tensor(plain.pair_frequencies(dims, base), dtype=torch.float64).cuda() if dims else None


def rotate_neighbours(x, positions, dims, base, sign=1.0):
    """The other pairing: element 2m with element 2m + 1."""
    out = x.copy()
    angles = sign * np.asarray(positions, dtype=np.float64)[:, None] * plain.pair_frequencies(dims, base)[None, :]
    c, s = np.cos(angles)[:, None, :], np.sin(angles)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("own_keys", [True, False])
@pytest.mark.parametrize("pairing", ["half", "neighbours"])
@pytest.mark.parametrize("lead", [3, 4])   # columns in front of the queries: with 4 the heads start on 16 bytes, and whole fours take the kernel for them
@pytest.mark.parametrize("dim,vdim,heads,kv_heads,rot_dims,v_dims", [(16, 16, 4, 2, 8, 16), (24, 8, 3, 3, 24, 8), (8, 40, 2, 1, 0, 40), (64, 64, 6, 2, 32, 64),
                                                                     (10, 6, 3, 1, 4, 6), (128, 192, 2, 1, 128, 192), (20, 12, 5, 5, 6, 4), (32, 48, 4, 4, 16, 48)])
def test_rows_are_rotated_and_values_are_kept_turned(dtype, own_keys, pairing, lead, dim, vdim, heads, kv_heads, rot_dims, v_dims):
    k = kernels()
    rng = np.random.default_rng(dim + vdim)
    rows, page_size, n_pages = 9, 4, 8
    head_size = -(-max(dim, vdim) // 16) * 16
    qw, kw, vw = heads * dim, kv_heads * dim, kv_heads * vdim
    fused = rng.normal(0, 2, (rows, lead + qw + kw + vw + 8 - lead)).astype(np.float32).astype(np.float64)   # [columns of something else | q | k | v | more]
    positions = np.array([0, 1, 2, 63, 64, 65, 500, 1100, 7])
    slots = np.array([5, 4, 31, -1, 0, 1, 2, 3, 17])
    base, v_base = 300.0, 40.0
    k_pages = torch.full((n_pages, kv_heads, page_size, head_size), 7.0, dtype=dtype).cuda()
    v_pages = torch.full((n_pages, kv_heads, page_size, head_size), 7.0, dtype=dtype).cuda()
    q = k.map_rows(gpu(fused), lead, lead + qw if own_keys else None, lead + qw + kw if own_keys else None, None, None, 1.0, frequencies(rot_dims, base), rot_dims,
                   ints(positions), ints(slots), k_pages, v_pages, heads, kv_heads, 1, dim, vdim, v_frequencies=frequencies(v_dims, v_base), v_rot_dims=v_dims,
                   v_pairing=pairing)
    want_q = plain.rotate_halves(fused[:, lead : lead + qw].reshape(rows, heads, dim), positions, rot_dims, base)
    got_q = q.float().cpu().numpy().reshape(rows, heads, head_size)
    np.testing.assert_allclose(got_q[..., :dim], rounded(want_q, dtype), **tol(dtype))
    assert not got_q[..., dim:].any()
    kp, vp = k_pages.float().cpu().numpy(), v_pages.float().cpu().numpy()
    if not own_keys:
        assert (kp == 7.0).all() and (vp == 7.0).all()
        return
    want_k = plain.rotate_halves(fused[:, lead + qw : lead + qw + kw].reshape(rows, kv_heads, dim), positions, rot_dims, base)
    v = fused[:, lead + qw + kw : lead + qw + kw + vw].reshape(rows, kv_heads, vdim)
    want_v = plain.rotate_halves(v, positions, v_dims, v_base) if pairing == "half" else rotate_neighbours(v, positions, v_dims, v_base)
    written = set()
    for row, slot in enumerate(slots):
        if slot < 0:
            continue
        page, place = divmod(slot, page_size)
        written.add((page, place))
        np.testing.assert_allclose(kp[page, :, place, :dim], rounded(want_k[row], dtype), **tol(dtype))
        np.testing.assert_allclose(vp[page, :, place, :vdim], rounded(want_v[row], dtype), **tol(dtype))
        assert not kp[page, :, place, dim:].any() and not vp[page, :, place, vdim:].any()
    for page in range(n_pages):
        for place in range(page_size):
            if (page, place) not in written:   # a padding row stores nothing
                assert (kp[page, :, place] == 7.0).all() and (vp[page, :, place] == 7.0).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pairing", ["half", "neighbours"])
@pytest.mark.parametrize("spare", [5, 8])   # columns behind the heads: with 8 the rows lie whole fours apart
@pytest.mark.parametrize("heads,in_size,out_size,dims", [(4, 16, 16, 16), (3, 48, 36, 36), (2, 64, 40, 8), (5, 32, 12, 0), (2, 192, 192, 192), (1, 16, 6, 6), (6, 64, 64, 64)])
def test_heads_are_turned_back_by_the_rows_position(dtype, pairing, spare, heads, in_size, out_size, dims):
    k = kernels()
    rng = np.random.default_rng(in_size + out_size)
    rows = 7
    x = rng.normal(0, 1, (rows, heads, in_size)).astype(np.float32).astype(np.float64)
    wide = np.concatenate([x.reshape(rows, -1), np.zeros((rows, spare))], axis=1)   # rows with something behind the heads: strided
    positions = np.array([0, 1, 63, 64, 999, 1500, 3])
    for sign in (1.0, -1.0):
        got = k.turn_heads(gpu(wide)[:, : heads * in_size], frequencies(dims, 77.0), dims, ints(positions), heads, in_size, out_size, sign=sign, pairing=pairing,
                           out_dtype=dtype)
        turn = plain.rotate_halves if pairing == "half" else rotate_neighbours
        want = turn(x[..., :out_size], positions, dims, 77.0, sign=sign) if dims else x[..., :out_size]
        np.testing.assert_allclose(got.float().cpu().numpy().reshape(rows, heads, out_size), rounded(want, dtype), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inner,limit,alpha,shift", [(8, 1.0, 1.702, 1.0), (33, 0.4, 1.702, 1.0), (256, 7.0, 1.0, 0.0), (50, None, 1.0, 0.0), (1, 2.5, 0.5, -1.0)])
def test_the_gate_unit_clamps_its_halves(dtype, inner, limit, alpha, shift):
    k = kernels()
    rng = np.random.default_rng(inner)
    both = rounded(rng.normal(0, 2.0, (6, 2 * inner)), dtype)
    both[0, 0], both[0, inner] = 50.0, -50.0    # far beyond any limit
    got = k.gate_unit(gpu(both, dtype), limit, alpha, shift).float().cpu().numpy()
    g = np.minimum(both[:, :inner], np.inf if limit is None else limit)
    u = np.clip(both[:, inner:], -(np.inf if limit is None else limit), np.inf if limit is None else limit)
    want = g * plain.sigmoid(alpha * g) * (u + shift)
    if (limit, alpha, shift) == (1.0, 1.702, 1.0):
        np.testing.assert_allclose(want, plain.clamped_gate_unit(both[:, :inner], both[:, inner:], 1.0))
    np.testing.assert_allclose(got, rounded(want, dtype), **tol(dtype))


@pytest.mark.parametrize("experts,top,groups,keep", [(6, 3, 1, 1), (6, 2, 3, 1), (8, 3, 4, 2), (10, 3, 2, 1), (12, 4, 3, 2), (1, 1, 1, 1), (64, 6, 8, 3),
                                                    (130, 7, 5, 2), (4, 2, 2, 1), (9, 9, 1, 1)])
def test_the_router_against_the_plain_choice(experts, top, groups, keep):
    k = kernels()
    rng = np.random.default_rng(experts * 7 + top)
    rows = 37
    z = rng.normal(0, 1.5, (rows, experts)).astype(np.float32).astype(np.float64)
    for correction in (None, rng.normal(0, 0.2, experts).astype(np.float32).astype(np.float64), -1.0 - rng.random(experts).astype(np.float32).astype(np.float64)):
        padded = np.concatenate([z, np.full((rows, 3), 99.0)], axis=1)   # the sums lie in rows with other columns behind them
        got = k.route(gpu(padded)[:, :experts], experts, top, correction=None if correction is None else gpu(correction), n_groups=groups, keep=keep,
                      floor=1e-20).cpu().numpy()
        want = plain.route(z, np.zeros(experts) if correction is None else correction, top, groups, keep)
        assert ((got != 0) == (want != 0)).all(), np.argwhere((got != 0) != (want != 0))[:3]
        assert ((got != 0).sum(axis=1) == top).all()
        np.testing.assert_allclose(got, want, atol=1e-6, rtol=1e-5)
        np.testing.assert_allclose(got.sum(axis=1), 1.0, atol=1e-5)


def test_the_router_breaks_ties_by_the_smaller_index():
    k = kernels()
    z = np.zeros((2, 6))
    got = k.route(gpu(z), 6, 2, n_groups=3, keep=2).cpu().numpy()
    np.testing.assert_allclose(got, [[0.5, 0.5, 0, 0, 0, 0]] * 2)


def build_routed(mlp, width, seed, dtype):
    """A RoutedExperts part with random tensors bound as the loader would bind them, and the same tensors for the plain function."""
    from mini_llm_amd.parts import make_part

    router = mlp["router"]
    groups = router.get("groups") or {"count": 1, "keep": 1}
    part = make_part("feed_forward", "routed_experts", width=width, n_experts=router["experts"], ff=mlp["expert"]["ff"], top=router["top"],
                     n_identity=router.get("identity", 0), n_groups=groups["count"], keep=groups["keep"], correction=True,
                     shared_ff=(mlp.get("shared") or {}).get("ff"), floor=1e-20)
    rng = np.random.default_rng(seed)
    tensors, bound = {}, {}
    for name, spec in part.tensor_specs().items():
        scale = 0.3 / spec.shape[0] if name == "correction" else (2.0 if name == "router" else 1.0) * spec.shape[-1] ** -0.5
        value = rounded(rng.normal(0, scale, spec.shape), torch.bfloat16)
        tensors["m." + name] = value
        bound[name] = gpu(value, torch.float32 if spec.role == "vector" else dtype)
    part.bind(bound)
    return part, tensors


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 5, 70, 300])
@pytest.mark.parametrize("case", ["groups", "plain", "identity", "one"])
def test_routed_experts_against_the_plain_sum_over_the_picked(dtype, rows, case):
    from dizizen_cases import moe

    mlp = {"groups": moe(experts=6, identity=2, top=3, groups=(4, 2), ff=16, shared=24), "plain": moe(experts=5, top=2, ff=24),
           "identity": moe(experts=2, identity=4, top=3, groups=(2, 2), ff=40, shared=8), "one": moe(experts=1, top=1, ff=12, shared=50)}[case]
    width = 48
    part, tensors = build_routed(mlp, width, rows + len(case), dtype)
    h = rounded(np.random.default_rng(rows).normal(0, 1, (rows, width)), dtype)
    got = part.forward(gpu(h, dtype), None).cpu().numpy()
    rnd = (lambda x: rounded(x, dtype)) if dtype == torch.bfloat16 else None
    want = plain.routed_feed_forward(h, mlp, tensors, "m.", rnd or (lambda x: x))
    scale = np.abs(want).max()
    np.testing.assert_allclose(got, want, atol=(3e-5 if dtype == torch.float32 else 3e-2) * scale, rtol=0)
    # with a residual the sum is taken inside
    stream = np.random.default_rng(1).normal(0, 1, (rows, width)).astype(np.float32)
    with_stream = part.forward(gpu(h, dtype), gpu(stream)).cpu().numpy()
    np.testing.assert_allclose(with_stream, got + stream, atol=1e-4 * max(scale, 1.0), rtol=0)
    # for a block that takes the sums itself: the partial products of the down product, and the share of the experts that hand h on behind them
    part.sums_later = True
    later = part.forward(gpu(h, dtype), None)
    assert later.bias is None and later.rows.dim() == 3 and later.rows.shape[0] >= (2 if mlp["router"].get("identity") else 1)
    np.testing.assert_allclose(later.rows.cpu().numpy().astype(np.float64).sum(axis=0), got, atol=1e-4 * max(scale, 1.0), rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,rows", [(16, 1), (100, 5), (192, 70), (2500, 3)])
def test_the_sum_of_two_branches_side_by_side(dtype, width, rows):
    k = kernels()
    rng = np.random.default_rng(width + rows)
    f = lambda *shape: rng.normal(0, 1, shape).astype(np.float32)
    x, a, b = f(rows, width), f(3, rows, width), f(rows, width)
    a_bias, b_bias, s1, s2, gates, gain = f(width), f(width), f(width), f(width), f(rows, 2 * width + 7), f(width) * 0.1
    sig = plain.sigmoid
    x64, a64 = x.astype(np.float64), a.astype(np.float64).sum(axis=0)
    # everything: partial products, biases, scales, gates, and the norm of the layer behind
    got, normed = k.branch_join(gpu(x), gpu(a), gpu(b), a_bias=gpu(a_bias), b_bias=gpu(b_bias), scale_a=gpu(s1), scale_b=gpu(s2), gates=gpu(gates)[:, 3:],
                                gate_a_at=0, gate_b_at=width + 2, mult=0.3, next_weight=gpu(gain), one_plus=True, eps=1e-6, out_dtype=dtype)
    want = x64 + 0.3 * ((a64 + a_bias) * s1 * sig(gates[:, 3 : 3 + width].astype(np.float64)) + (b.astype(np.float64) + b_bias) * s2 * sig(gates[:, 5 + width : 5 + 2 * width].astype(np.float64)))
    np.testing.assert_allclose(got.cpu().numpy(), want, atol=2e-5, rtol=2e-5)
    np.testing.assert_allclose(normed.float().cpu().numpy(), rounded(plain.centred_rms_norm(want, gain.astype(np.float64), 1e-6), dtype), **tol(dtype))
    # a plain gain, one branch, nothing else
    got, normed = k.branch_join(gpu(x), gpu(b), mult=1.5, next_weight=gpu(gain), one_plus=False, eps=1e-3, out_dtype=dtype)
    want = x64 + 1.5 * b
    np.testing.assert_allclose(got.cpu().numpy(), want, atol=2e-5, rtol=2e-5)
    np.testing.assert_allclose(normed.float().cpu().numpy(), rounded(want / np.sqrt((want ** 2).mean(axis=1, keepdims=True) + 1e-3) * gain, dtype), **tol(dtype))
    # no norm behind: the sum alone
    got = k.branch_join(gpu(x), gpu(a[0]), gpu(b), scale_b=gpu(s2), mult=1.0)
    np.testing.assert_allclose(got.cpu().numpy(), x64 + a[0] + b.astype(np.float64) * s2, atol=2e-5, rtol=2e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [3, 40])
def test_the_clamped_gated_feed_forward_part(dtype, rows):
    from mini_llm_amd.parts import make_part

    width, inner, limit = 40, 56, 0.7
    part = make_part("feed_forward", "clamped_gated_mlp", width=width, inner=inner, limit=limit, alpha=1.702, shift=1.0, biases=True)
    rng = np.random.default_rng(rows)
    tensors, bound = {}, {}
    for name, spec in part.tensor_specs().items():
        value = rounded(rng.normal(0, 0.3 if name.endswith(".b") else spec.shape[-1] ** -0.5, spec.shape), torch.bfloat16)
        tensors["m." + name] = value
        placed = gpu(value, torch.float32 if spec.role == "vector" else dtype)
        bound[name] = k_pack(placed) if spec.role == "matrix" else placed
    part.bind(bound)
    h = rounded(rng.normal(0, 1.5, (rows, width)), dtype)
    rnd = (lambda x: rounded(x, dtype)) if dtype == torch.bfloat16 else (lambda x: x)
    want = plain.dense_feed_forward(h, {"kind": "dense", "ff": inner, "limit": limit}, tensors, "m.", rnd)
    got = part.forward(gpu(h, dtype), None).cpu().numpy()
    np.testing.assert_allclose(got, want, atol=(3e-5 if dtype == torch.float32 else 3e-2) * np.abs(want).max(), rtol=0)
    part.sums_later = True   # for a block that takes the sums itself
    later = part.forward(gpu(h, dtype), None)
    total = later.rows.cpu().numpy().astype(np.float64)
    total = (total.sum(axis=0) if total.ndim == 3 else total) + later.bias.cpu().numpy()
    np.testing.assert_allclose(total, got, atol=1e-4 * np.abs(want).max(), rtol=0)


def k_pack(matrix):
    return kernels().pack_matrix(matrix)
