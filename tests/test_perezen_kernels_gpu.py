"""Each mechanism of the Perezen design alone: the kernel against the plain function of tests/plain_perezen.py."""

import numpy as np
import pytest
import torch

import plain_perezen as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
MAPS = 2


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


def as_attention_heads(x, heads, kv_heads):
    """[T, heads, maps, d] in the design's order -> the order the paged kernels get: head (g * maps + m) * R + r for query head g R + r."""
    T, _, maps, d = x.shape
    R = heads // kv_heads
    return x.reshape(T, kv_heads, R, maps, d).transpose(0, 1, 3, 2, 4).reshape(T, heads * maps, d)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("own_keys", [True, False])
@pytest.mark.parametrize("dim,vdim,heads,kv_heads,rot_dims", [(16, 16, 4, 2, 8), (24, 8, 3, 3, 24), (8, 40, 2, 1, 0), (64, 64, 6, 2, 32), (10, 6, 3, 1, 4),
                                                              (128, 192, 2, 1, 128), (20, 12, 5, 5, 6)])
def test_map_rows_norm_rotate_and_store(dtype, own_keys, dim, vdim, heads, kv_heads, rot_dims):
    k = kernels()
    rng = np.random.default_rng(dim + vdim)
    rows, page_size, n_pages, eps = 9, 4, 8, 1e-5
    head_size = -(-max(dim, vdim) // 16) * 16
    qw, kw, vw = heads * MAPS * dim, kv_heads * MAPS * dim, kv_heads * vdim
    # [3 columns of something else | q | k | v | 5 more]
    fused = rng.normal(0, 2, (rows, 3 + qw + kw + vw + 5)).astype(np.float32).astype(np.float64)
    qg, kg = rng.normal(1, 0.2, dim), rng.normal(1, 0.2, dim)
    positions = np.array([0, 1, 2, 63, 64, 65, 500, 1100, 7])
    slots = np.array([5, 4, 31, -1, 0, 1, 2, 3, 17])
    base = 300.0
    frequencies = torch.tensor(base ** (-2.0 * np.arange(rot_dims // 2) / rot_dims), dtype=torch.float64).cuda() if rot_dims else None
    k_pages = torch.full((n_pages, kv_heads * MAPS, page_size, head_size), 7.0, dtype=dtype).cuda()
    v_pages = torch.full_like(k_pages, 7.0)
    q = k.map_rows(gpu(fused), 3, 3 + qw if own_keys else None, 3 + qw + kw if own_keys else None, gpu(qg), gpu(kg) if own_keys else None, eps, frequencies,
                   rot_dims, ints(positions), ints(slots), k_pages, v_pages, heads, kv_heads, MAPS, dim, vdim)
    want_q = plain.rotate_halves(plain.rms_unit(fused[:, 3 : 3 + qw].reshape(rows, heads, MAPS, dim), eps) * qg, positions, rot_dims, base)
    got_q = q.float().cpu().numpy().reshape(rows, heads * MAPS, head_size)
    np.testing.assert_allclose(got_q[:, :, :dim], as_attention_heads(want_q, heads, kv_heads), **tol(dtype))   # (angles in 64-bit: position 1,100 is as good as 1)
    assert (got_q[:, :, dim:] == 0).all()
    kp, vp = k_pages.float().cpu().numpy(), v_pages.float().cpu().numpy()
    if not own_keys:
        assert (kp == 7).all() and (vp == 7).all()    # a layer that borrows stores nothing
        return
    want_k = plain.rotate_halves(plain.rms_unit(fused[:, 3 + qw : 3 + qw + kw].reshape(rows, kv_heads, MAPS, dim), eps) * kg, positions, rot_dims, base)
    want_v = fused[:, 3 + qw + kw : 3 + qw + kw + vw].reshape(rows, kv_heads, vdim)
    for row, slot in enumerate(slots):
        if slot < 0:
            continue
        page, offset = divmod(int(slot), page_size)
        np.testing.assert_allclose(kp[page, :, offset, :dim], want_k[row].reshape(kv_heads * MAPS, dim), **tol(dtype))
        for m in range(MAPS):   # the value head under each of its maps
            np.testing.assert_allclose(vp[page, m::MAPS, offset, :vdim], want_v[row], **tol(dtype))
        assert (kp[page, :, offset, dim:] == 0).all() and (vp[page, :, offset, vdim:] == 0).all()
    assert (kp[6] == 7).all() and (vp[5] == 7).all()   # pages no slot names are left alone


def test_map_rows_norms_every_map_of_every_head_by_itself():
    # one map far larger than the other three: each is brought to unit size by itself, with the one gain vector they share
    k = kernels()
    q = np.concatenate([np.full((1, 8), 10.0), np.full((1, 8), 0.1), np.full((1, 8), -3.0), np.full((1, 8), 1.0)], axis=1)
    pages = torch.zeros((1, 2, 4, 16)).cuda()
    got = k.map_rows(gpu(q), 0, None, None, gpu(np.full(8, 2.0)), None, 1e-9, None, 0, ints([0]), ints([0]), pages, pages.clone(), 2, 1, MAPS, 8, 8)
    got = got.cpu().numpy().reshape(4, 16)
    np.testing.assert_allclose(got[:, :8], np.array([2.0, -2.0, 2.0, 2.0])[:, None] * np.ones((4, 8)), rtol=1e-5)   # heads (g, m, r): h0m0, h1m0, h0m1, h1m1
    assert (got[:, 8:] == 0).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("vdim,heads,kv_heads", [(16, 4, 2), (8, 3, 3), (40, 2, 1), (64, 6, 2), (6, 3, 1), (192, 2, 1), (256, 1, 1)])
def test_map_difference_subtracts_norms_and_gates(dtype, vdim, heads, kv_heads):
    k = kernels()
    rng = np.random.default_rng(vdim)
    rows, eps, lam, diff = 11, 1e-5, 0.37, 0.2
    head_size = -(-vdim // 16) * 16 + (16 if vdim % 32 == 8 else 0)    # also heads with more room than the values need
    a = rounded(rng.normal(0, 1, (rows, heads, MAPS, head_size)), dtype)
    gate = rng.normal(0, 2, (rows, 4 + heads * vdim)).astype(np.float32).astype(np.float64)
    want = plain.rms_unit(a[:, :, 0, :vdim] - lam * a[:, :, 1, :vdim], eps) * (1.0 - diff)
    maps_out = gpu(as_attention_heads(a, heads, kv_heads).reshape(rows, -1), dtype)
    got = k.map_difference(maps_out, gpu(gate)[:, 4:], lam, eps, heads, kv_heads, vdim, head_size, scale=1.0 - diff)
    np.testing.assert_allclose(got.float().cpu().numpy(), (want * plain.sigmoid(gate[:, 4:].reshape(rows, heads, vdim))).reshape(rows, -1), **tol(dtype))
    got = k.map_difference(maps_out, None, lam, eps, heads, kv_heads, vdim, head_size, scale=1.0 - diff)
    np.testing.assert_allclose(got.float().cpu().numpy(), want.reshape(rows, -1), **tol(dtype))
    # 32-bit maps into rows of the compute type: nothing is rounded before the difference
    got = k.map_difference(maps_out.float(), None, lam, eps, heads, kv_heads, vdim, head_size, scale=1.0 - diff, out_dtype=dtype)
    assert got.dtype == dtype
    np.testing.assert_allclose(got.float().cpu().numpy(), want.reshape(rows, -1), **tol(dtype))


def test_two_maps_that_nearly_cancel_keep_their_difference_in_32_bit():
    # a1 and lam a2 agree to three digits: rounded to bfloat16 first, their difference would be noise
    k = kernels()
    rng = np.random.default_rng(8)
    rows, heads, vdim, lam = 5, 2, 32, 0.5
    a2 = rng.normal(0, 1, (rows, heads, vdim))
    a1 = lam * a2 + 1e-3 * rng.normal(0, 1, (rows, heads, vdim))
    a = np.stack([a1, a2], axis=2).astype(np.float32).astype(np.float64)
    want = plain.rms_unit(a[:, :, 0] - lam * a[:, :, 1], 1e-12)
    got = k.map_difference(gpu(as_attention_heads(a, heads, 1).reshape(rows, -1)), None, lam, 1e-12, heads, 1, vdim, vdim, out_dtype=torch.bfloat16)
    np.testing.assert_allclose(got.float().cpu().numpy(), want.reshape(rows, -1), atol=2e-2, rtol=2e-2)


def paged(keys, values, page_size, head_size, dtype, order):
    """Keys and values [T, G, d] of one request in pages taken in ``order``; returns (k_pages, v_pages, block table)."""
    T, G, _ = keys.shape
    n_blocks = -(-T // page_size)
    k_pages = torch.zeros((max(order) + 1, G, page_size, head_size), dtype=dtype).cuda()
    v_pages = torch.zeros_like(k_pages)
    for b in range(n_blocks):
        rows = slice(b * page_size, min(T, (b + 1) * page_size))
        n = rows.stop - rows.start
        k_pages[order[b], :, :n, : keys.shape[2]] = gpu(keys[rows], dtype).transpose(0, 1)
        v_pages[order[b], :, :n, : values.shape[2]] = gpu(values[rows], dtype).transpose(0, 1)
    return k_pages, v_pages, ints([order[:n_blocks]])


def every_way(k, rows, k_pages, v_pages, table, T, common, want, dtype, portion_from=90, singles=()):
    """The whole prompt at once, then a portion over cached keys, then rows one by one and in short portions; each with the result in
    the pages' type and in 32-bit."""
    for wide in (False, True):
        def run(q_rows, *args, **kwargs):
            got = k.paged_attention(q_rows, *args, wide_out=wide, **kwargs, **common)
            assert got.dtype == (torch.float32 if wide else dtype)
            return got.float().cpu().numpy()

        got = run(rows, k_pages, v_pages, ints(np.zeros(T)), ints(np.arange(T)), table, max_q_len=T, max_len=T, q_starts=ints([0, T]), context_lens=ints([0]))
        np.testing.assert_allclose(got, want, **tol(dtype))
        n = T - portion_from
        got = run(rows[portion_from:], k_pages, v_pages, ints(np.zeros(n)), ints(np.arange(portion_from, T)), table, max_q_len=n, max_len=T,
                  q_starts=ints([0, n]), context_lens=ints([portion_from]))
        np.testing.assert_allclose(got, want[portion_from:], **tol(dtype))
        for at, n in singles:
            got = run(rows[at : at + n], k_pages, v_pages, ints(np.zeros(n)), ints(np.arange(at, at + n)), table, max_q_len=n, max_len=T,
                      q_starts=ints([0, n]), context_lens=ints([at]))
            np.testing.assert_allclose(got, want[at : at + n], err_msg=f"rows {at}..{at + n - 1}", **tol(dtype))
        # no queries' starts given: the general kernel, a wave a (row, head)
        got = run(rows, k_pages, v_pages, ints(np.zeros(T)), ints(np.arange(T)), table)
        np.testing.assert_allclose(got, want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("head_size,heads,kv_heads,chunk", [(64, 4, 2, 40), (32, 2, 1, 16), (48, 3, 3, 70), (16, 2, 2, 5), (128, 2, 1, 64), (160, 1, 1, 33),
                                                            (64, 2, 2, 1), (96, 2, 1, 149), (64, 8, 2, 1000)])
def test_attention_inside_chunks_in_prompts_and_in_decoding(dtype, head_size, heads, kv_heads, chunk):
    k = kernels()
    rng = np.random.default_rng(head_size + chunk)
    T, page_size = 150, 16
    q = rounded(rng.normal(0, 1.5, (T, heads, head_size)), dtype)
    keys = rounded(rng.normal(0, 1.5, (T, kv_heads, head_size)), dtype)
    values = rounded(rng.normal(0, 1, (T, kv_heads, head_size)), dtype)
    scale = head_size ** -0.5 * 2.0
    want = plain.chunked_attention(q, keys, values, scale, chunk).reshape(T, heads * head_size)
    if chunk < T:
        assert np.abs(want - plain.chunked_attention(q, keys, values, scale, None).reshape(T, -1)).max() > 0.05
    k_pages, v_pages, table = paged(keys, values, page_size, head_size, dtype, list(rng.permutation(12)))
    rows = gpu(q.reshape(T, heads * head_size), dtype)
    common = dict(n_heads=heads, n_kv_heads=kv_heads, head_size=head_size, scale=scale, chunk=chunk)
    edges = [(e + d, 1) for e in range(chunk, T, max(chunk, 37)) for d in (-1, 0, 1) if 0 <= e + d < T]    # the last row of a chunk, the first of the next, one more
    every_way(k, rows, k_pages, v_pages, table, T, common, want, dtype,
              singles=[(T - 1, 1), (T - 5, 5), (3, 1), (64, 2), (0, 1)] + edges + [(max(0, e - 3), min(6, T - max(0, e - 3))) for e in range(chunk, T, max(chunk, 53))])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk,at", [(40, 40), (40, 79), (64, 64), (64, 63), (100, 0), (33, 66)])
def test_a_key_that_outscores_all_others_is_seen_inside_its_chunk_only(dtype, chunk, at):
    # among random keys a missing or an extra one hardly moves a softmax: one key is made ten times the others' size along the
    # direction every query looks in, with a value far from the others, so that the rows that see it return that value
    k = kernels()
    rng = np.random.default_rng(chunk + at)
    T, page_size, heads, head_size = 210, 16, 2, 32
    q = rng.normal(0, 0.3, (T, heads, head_size))
    keys = rng.normal(0, 0.3, (T, 1, head_size))
    values = rng.normal(0, 0.1, (T, 1, head_size))
    q[:, :, 5], keys[at, 0, 5], values[at, 0] = 4.0, 8.0, 50.0
    q, keys, values = rounded(q, dtype), rounded(keys, dtype), rounded(values, dtype)
    want = plain.chunked_attention(q, keys, values, 1.0, chunk).reshape(T, heads * head_size)
    end = (at // chunk + 1) * chunk
    assert (want[at:end] > 49).all() and np.abs(want[end:]).max() < 1 and (at == 0 or np.abs(want[:at]).max() < 1)
    k_pages, v_pages, table = paged(keys, values, page_size, head_size, dtype, list(rng.permutation(16)))
    rows = gpu(q.reshape(T, -1), dtype)
    common = dict(n_heads=heads, n_kv_heads=1, head_size=head_size, scale=1.0, chunk=chunk)
    every_way(k, rows, k_pages, v_pages, table, T, common, want, dtype, portion_from=max(1, at - 3),
              singles=[(at, 1), (end - 1, 1), (end, 1), (end - 2, 4), (max(0, at - 2), 5)] + ([(at - 1, 1)] if at else []))


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_long_chunk_in_runs_of_keys(dtype):
    # one row over a chunk of 2,500 keys that starts at 3,000: the split-key kernel cuts the chunk's keys, not the sequence's, into runs
    k = kernels()
    rng = np.random.default_rng(1)
    T, page_size, heads, head_size, chunk = 5500, 64, 2, 64, 3000
    keys, values = rounded(rng.normal(0, 1, (T, 1, head_size)), dtype), rounded(rng.normal(0, 1, (T, 1, head_size)), dtype)
    q = rounded(rng.normal(0, 1, (1, heads, head_size)), dtype)
    keys[2999, 0], values[2999, 0] = 3.0 * q[0, 0], 40.0    # the last key of the chunk before: it would win if it were seen
    k_pages, v_pages, table = paged(keys, values, page_size, head_size, dtype, list(range(86)))
    scores = np.einsum("hd,td->ht", q[0], keys[3000:, 0]) * 0.2
    w = np.exp(scores - scores.max(axis=1, keepdims=True))
    want = (w @ values[3000:, 0]) / w.sum(axis=1)[:, None]
    got = k.paged_attention(gpu(q.reshape(1, -1), dtype), k_pages, v_pages, ints([0]), ints([T - 1]), table, heads, 1, head_size, 0.2, max_q_len=1, max_len=T,
                            q_starts=ints([0, 1]), context_lens=ints([T - 1]), chunk=chunk)
    np.testing.assert_allclose(got.float().cpu().numpy().reshape(heads, head_size), want, **(dict(atol=2e-5, rtol=2e-4) if dtype == torch.float32 else tol(dtype)))


def test_a_window_and_chunks_together_are_refused():
    k = kernels()
    pages = torch.zeros((2, 1, 16, 16)).cuda()
    with pytest.raises(k.OperandError, match="window or by chunks"):
        k.paged_attention(gpu(np.zeros((1, 16))), pages, pages.clone(), ints([0]), ints([0]), ints([[0]]), 1, 1, 16, 1.0, window=4, chunk=4)


def test_learned_positions_join_the_token_rows_unscaled():
    k = kernels()
    rng = np.random.default_rng(5)
    table, pos = rng.normal(0, 1, (20, 24)), rng.normal(0, 1, (50, 24))
    tokens, positions = np.array([3, 19, 0, 3]), np.array([0, 49, 7, 1])
    for dtype in DTYPES:
        got = k.embed(ints(tokens), ints(positions), gpu(table, dtype), gpu(pos, dtype))
        np.testing.assert_allclose(got.float().cpu().numpy(), rounded(table, dtype)[tokens] + rounded(pos, dtype)[positions], atol=1e-6)
        assert got.dtype == torch.float32    # the stream is 32-bit whatever the tables are


@pytest.mark.parametrize("width", [5, 64, 100, 768, 2048, 2500])
def test_the_norm_behind_a_branch_and_the_norm_in_front_of_the_next_from_one_kernel(width):
    from mini_llm_amd.parts import make_part

    rng = np.random.default_rng(width)
    stream, branch = rng.normal(0, 2, (7, width)), rng.normal(0, 3, (7, width))
    w, w_next = rng.normal(1, 0.3, width), rng.normal(1, 0.3, width)
    total = stream + plain.rms_unit(branch, 1e-5) * w
    behind, ahead = (make_part("norm", "rmsnorm", width=width, eps=1e-5, tensor_name="") for _ in range(2))
    behind.bind({"": gpu(w)})
    ahead.bind({"": gpu(w_next)})
    for dtype in DTYPES:
        got = behind.forward_added(gpu(stream), gpu(branch), then=ahead, out_dtype=dtype)    # (rows of 2,500 take two launches)
        assert got.norm is ahead and got.rows.dtype == dtype
        np.testing.assert_allclose(got.stream.cpu().numpy(), total, atol=2e-5, rtol=2e-5)
        np.testing.assert_allclose(got.rows.float().cpu().numpy(), plain.rms_unit(total, 1e-5) * w_next, **tol(dtype))
    # the branch as the partial products of a product cut along K
    parts = rng.normal(0, 1, (4, 7, width))
    got = behind.forward_added(gpu(stream), gpu(parts), then=ahead, out_dtype=torch.float32)
    total = stream + plain.rms_unit(parts.sum(axis=0), 1e-5) * w
    np.testing.assert_allclose(got.stream.cpu().numpy(), total, atol=2e-5, rtol=2e-5)
    np.testing.assert_allclose(got.rows.cpu().numpy(), plain.rms_unit(total, 1e-5) * w_next, atol=3e-5, rtol=3e-5)
    np.testing.assert_allclose(behind.forward_added(gpu(stream), gpu(parts)).cpu().numpy(), total, atol=2e-5, rtol=2e-5)
