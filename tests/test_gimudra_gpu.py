"""Gimudra on the GPU against the plain implementation: every mechanism's kernel alone, then
whole models cut every way (whole prompts, token by token, portions down to two tokens, mixed
batches over pages and slots that are used again), long decoding, and greedy generation
through the engine."""
import math

import numpy as np
import pytest
import torch

from tests.gimudra_helpers import CONFIGS, make_folder, read_folder, tokens
from tests.helpers import rows_within
from tests.plain import gimudra as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32_BOUND = 2e-4   # of a row's largest |logit|
BF16_BOUND = 1e-1
ROUTER_MARGIN = 0.008  # in bfloat16, choices between corrected scores (each below one) closer than this are accidents of rounding


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.kernels import ops as module

    return module


@pytest.fixture(scope="module")
def tmp(tmp_path_factory):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return tmp_path_factory.mktemp("gimudra")


def i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


def dev(array, dtype=torch.float32):
    return torch.tensor(np.asarray(array), dtype=dtype, device=DEV)


def close(got, want, bound, what=""):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want)
    err = np.abs(got - want).max() / max(np.abs(want).max(), 1e-30)
    assert err <= bound, f"{what}: off by {err:.2e} of the largest value"


def rounded(array, dtype):
    """What a tensor of ``dtype`` holds of these numbers, as float64."""
    return torch.tensor(np.asarray(array)).to(dtype).double().numpy()


# ---- mechanisms alone ---------------------------------------------------------------------------
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [40, 300, 7, 1024, 5000])
def test_token_shift_in_portions_of_two_requests_over_reused_slots(ops, width, out_dtype):
    rng = np.random.default_rng(width)
    shift = rng.uniform(-0.5, 1.5, size=width)
    shift[:2] = (0.0, 1.0)  # the input itself; the previous input alone
    seqs = {0: rng.normal(size=(150, width)), 1: rng.normal(size=(31, width))}
    f32 = lambda a: rounded(a, torch.float32)
    want = {s: plain.token_shift(f32(h), f32(shift)) for s, h in seqs.items()}
    state = torch.full((3, width), 5.0, device=DEV)  # as slots that were used before
    state[[0, 2]] = 0.0  # what handing out a slot does
    slot, pos, got = {0: 2, 1: 0}, {0: 0, 1: 0}, {0: [], 1: []}
    plan = [{0: 1}, {0: 2, 1: 1}, {1: 2, 0: 1}, {0: 70, 1: 1}, {1: 3}, {0: 1, 1: 24}, {0: 65}, {0: 10}]
    for step in plan:
        rows = list(step)
        h = dev(np.concatenate([seqs[s][pos[s]: pos[s] + step[s]] for s in rows]))
        starts = np.concatenate([[0], np.cumsum([step[s] for s in rows])])
        out = ops.token_shift(h, dev(shift), state, i32(starts), i32(slot[s] for s in rows), rows=len(rows),
                              max_count=max(step.values()), out_dtype=out_dtype)
        assert out.dtype == out_dtype
        out = out.float().cpu().numpy()
        for r, s in enumerate(rows):
            got[s].append(out[starts[r]: starts[r + 1]])
            pos[s] += step[s]
    for s in seqs:
        g = np.concatenate(got[s])
        assert len(g) == len(want[s])
        if out_dtype == torch.float32:
            assert np.abs(g - want[s]).max() < 1e-5, s
        else:  # one rounding of the float32 result
            assert np.array_equal(g, rounded(g, torch.bfloat16)) and np.abs(g - want[s]).max() < 2.0 ** -7 * np.abs(want[s]).max()
        assert np.array_equal(g[0, :2], rounded([seqs[s][0, 0], 0.0], out_dtype).astype(np.float32))  # zeros before the first
    assert float((state[1] - 5.0).abs().max()) == 0.0  # nobody's slot is left alone
    for s in seqs:  # the state is the last input as it came, not as it left
        assert np.array_equal(state[slot[s]].cpu().numpy(), seqs[s][-1].astype(np.float32))


@pytest.mark.parametrize("delta_dtype, out_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                                     (torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("dim, parts, total", [(64, 1, 3), (200, 4, 6), (2560, 1, 9), (7, 2, 2), (5000, 1, 4)])
def test_depth_mix_keeps_every_result_and_hands_on_their_mix(ops, dim, parts, total, delta_dtype, out_dtype):
    """A step's layers one after the other: the sum with the scaled and biased output, the result
    among the streams, the mix of all streams so far and its norm."""
    if parts > 1 and delta_dtype != torch.float32:
        pytest.skip("partial sums are float32")
    rng = np.random.default_rng(dim + total)
    rows = 5
    streams = torch.full((total, rows, dim), float("nan"), device=DEV)
    first = rng.normal(size=(rows, dim)) * 2
    streams[0] = dev(first)
    resid = dev(first)
    plain_streams, x = [rounded(first, torch.float32)], rounded(first, torch.float32)
    for index in range(1, total):
        delta = rounded(rng.normal(size=(parts, rows, dim)), delta_dtype)
        scale, bias, gain = rng.normal(size=dim), rng.normal(size=dim), rng.normal(size=dim)
        coeff = rng.normal(size=index + 1)
        use_bias, use_scale, use_gain = index % 2 == 1, index % 3 != 2, index != 2
        d = delta.sum(0) + (rounded(bias, torch.float32) if use_bias else 0.0)
        result = x + d * (rounded(scale, torch.float32) if use_scale else 1.0)
        plain_streams.append(result)
        x = plain.depth_mix(plain_streams, rounded(coeff, torch.float32))
        out = ops.depth_mix(resid, dev(delta if parts > 1 else delta[0], delta_dtype), streams, index, dev(coeff),
                            delta_scale=dev(scale) if use_scale else None, delta_bias=dev(bias) if use_bias else None,
                            gain=dev(gain) if use_gain else None, eps=1e-3, out_dtype=out_dtype)
        bound = 2e-5 * max(1.0, np.abs(x).max())
        assert np.abs(streams[index].cpu().numpy() - result).max() < bound, index
        assert np.abs(resid.cpu().numpy() - x).max() < bound, index
        if use_gain:
            want = plain.rms_norm(x, rounded(gain, torch.float32), 1e-3)
            close(out.float().cpu().numpy(), want, 2e-5 if out_dtype == torch.float32 else 8e-3, f"norm of mix {index}")
        else:
            assert out is None
    assert np.array_equal(streams[0].cpu().numpy(), first.astype(np.float32))


@pytest.mark.parametrize("dim", [6, 176, 5, 1000])
def test_position_vectors_of_sines_and_cosines(ops, dim):
    positions = [0, 1, 2, 63, 64, 1000, 4097, 3, 0]
    freq = dev(10000.0 ** (-np.arange(0, dim, 2, dtype=np.float64) / dim))
    x = torch.full((len(positions), dim), 0.25, device=DEV)
    ops.add_sinusoid(x, i32(positions), freq)
    want = plain.sinusoid(5000, dim)[positions] + 0.25
    got = x.cpu().numpy()
    assert np.abs(got[[0, 1, 2, 7, 8]] - want[[0, 1, 2, 7, 8]]).max() < 1e-6
    assert np.abs(got - want).max() < 1e-3  # a float32 angle of thousands of radians
    assert np.array_equal(got[0], got[8])


def planted_case(rng, n, heads, groups, dim, vdim, planted):
    """Queries, keys and values of one request of ``n`` tokens in which the keys ``planted`` lie
    along one direction that every query has a large share of: whoever sees one of them gives it
    nearly all of its weight, so a mask that is one key off shows in the output."""
    u = rng.normal(size=dim)
    u /= np.linalg.norm(u)
    q = 0.3 * rng.normal(size=(n, heads, dim)) + 3.0 * u
    k = 0.3 * rng.normal(size=(n, groups, dim))
    for j, strength in planted:
        k[j] += strength * u
    return q, k, rng.normal(size=(n, groups, vdim))


def plain_biased_attention(q, k, v, visible, scale, r1, r2):
    n, heads, _ = q.shape
    groups = k.shape[1]
    bias = plain.distance_bias(r1, r2, n)
    out = np.zeros((n, heads, v.shape[2]))
    for h in range(heads):
        g = h // (heads // groups)
        out[:, h] = plain.softmax_masked(q[:, h] @ k[:, g].T * scale - bias[h], visible) @ v[:, g]
    return out


@pytest.mark.parametrize("size", [37, 64, 129, 1, 300, None])
@pytest.mark.parametrize("dtype, heads, groups, dim, vdim, page", [
    (torch.float32, 4, 2, 16, 24, 16), (torch.float32, 3, 1, 12, 20, 16), (torch.bfloat16, 6, 3, 20, 6, 16),
    (torch.bfloat16, 4, 2, 64, 72, 32), (torch.bfloat16, 8, 4, 64, 48, 64), (torch.bfloat16, 16, 1, 16, 8, 64),
    (torch.bfloat16, 3, 3, 128, 128, 64), (torch.bfloat16, 5, 5, 40, 36, 96)])
def test_attention_with_a_bias_by_log_distance_at_the_edges_of_chunks_and_pages(ops, size, dtype, heads, groups, dim, vdim, page):
    """Keys planted at both sides of a chunk's edge, at a page's first and last slot and far back;
    every query position of a 300-token request, as a prompt and token by token, on the general
    kernel and (bfloat16, pages of a multiple of 32) on the matrix cores.  The bias is large enough
    to move weight between near and far keys; some queries are zero, so that it alone decides."""
    rng = np.random.default_rng((size or 0) * 7 + dim + heads)
    n, scale = 300, 0.4
    edge = size if size is not None and size < n else 100
    planted = [(0, 5.0), (page - 1, 6.0), (page, 7.0), (edge - 1, 8.0), (min(edge, n - 1), 9.0),
               (2 * edge if 2 * edge < n else 5, 10.0), (n - 2 - edge if n - 2 - edge > 0 else 7, 11.0)]
    q, k, v = planted_case(rng, n, heads, groups, dim, vdim, planted)
    q[150:170] = 0.0
    q, k, v = rounded(q, dtype), rounded(k, dtype), rounded(v, dtype)
    r1 = rounded(rng.uniform(0.0, 3.0, size=heads), torch.float32)
    r2 = rounded(rng.uniform(0.05, 4.0, size=heads), torch.float32)
    r1[0] = 0.0  # one head without a bias
    want = plain_biased_attention(q, k, v, plain.chunk_mask(n, size), scale, r1, r2)
    pages = -(-n // page)
    order = rng.permutation(pages + 3)[:pages]  # the request's pages lie scattered in a larger pool
    k_cache = torch.full((pages + 3, page, groups, dim), float("nan"), dtype=dtype)
    v_cache = torch.full((pages + 3, page, groups, vdim), float("nan"), dtype=dtype)
    slots = np.array([order[p // page] * page + p % page for p in range(n)])
    k_cache.view(-1, groups, dim)[slots] = torch.tensor(k).to(dtype)
    v_cache.view(-1, groups, vdim)[slots] = torch.tensor(v).to(dtype)
    k_cache, v_cache, qd = k_cache.to(DEV), v_cache.to(DEV), torch.tensor(q).to(dtype).to(DEV)
    table = i32(order).view(1, pages)
    log_bias = dev(np.stack([r1, r2]))
    bound = 3e-5 if dtype == torch.float32 else 2e-2
    positions = i32(range(n))
    rows = torch.zeros(n, dtype=torch.int32, device=DEV)
    got = ops.paged_attention(qd, k_cache.nan_to_num(1e4), v_cache.nan_to_num(1e4), table, rows, positions, page_size=page,
                              scale=scale, window=None, chunk=size, log_bias=log_bias)
    close(got.float().cpu().numpy(), want, bound, "general kernel")
    # the second half alone over the cached first, as queries that are a slice of wider rows
    wide = torch.zeros((n - 143, heads * dim + 24), dtype=dtype, device=DEV)
    wide[:, : heads * dim] = qd[143:].reshape(n - 143, -1)
    qv = wide.as_strided((n - 143, heads, dim), (wide.stride(0), dim, 1))
    got = ops.paged_attention(qv, k_cache.nan_to_num(1e4), v_cache.nan_to_num(1e4), table, rows[143:], positions[143:],
                              page_size=page, scale=scale, window=None, chunk=size, log_bias=log_bias)
    close(got.float().cpu().numpy(), want[143:], bound, "general kernel, a portion")
    span = size if size is not None else ops.SINK_MAX_BIAS + 1
    if not ops.attention_sink_ok(dtype, head_dim=dim, v_dim=vdim, page_size=page, bucket_len=span):
        assert dtype == torch.float32 or page % 32 or size is None
        return
    # the matrix cores: the bias as a table by distance, values transposed inside their pages
    distance = np.arange(span, dtype=np.float64)
    bias = dev(-r1[:, None] * np.log(1.0 + r2[:, None] * distance[None]))
    vt = v_cache.permute(0, 2, 3, 1).contiguous()  # NaN where no token lies
    for first in (0, 143):
        count = n - first
        tiles = [(a, min(32, count - a), 0, first + a) for a in range(0, count, 32)]
        tiles = i32(np.array(tiles[::-1]).reshape(-1)).view(-1, 4)
        got = ops.attention_sink(qv if first else qd, k_cache, vt, table, tiles, None, page_size=page, scale=scale,
                                 bias=bias, sink=False, chunk=size).float().cpu().numpy()
        assert not np.isnan(got).any()
        close(got, want[first:], bound, f"matrix cores, a prompt from {first}")
    # single tokens: every position a "request" of its own on the same pages
    many = i32(order).view(1, pages).repeat(n, 1).contiguous()
    for cuts in (1, 2, 8):
        got = ops.attention_sink(qd, k_cache, vt, many, None, positions, page_size=page, scale=scale, bias=bias,
                                 sink=False, cuts=cuts, chunk=size).float().cpu().numpy()
        assert not np.isnan(got).any()
        close(got, want, bound, f"matrix cores, single tokens, {cuts} cuts")


def test_a_far_key_among_hundreds_carries_the_output_despite_the_bias(ops):
    """Without chunks every earlier key counts: one key 500 tokens back whose score stands out takes
    nearly all the weight although the bias by distance is against it, in prompts and single tokens."""
    rng = np.random.default_rng(11)
    n, heads, groups, dim, vdim, page, scale = 520, 2, 1, 32, 16, 16, 0.5
    q, k, v = planted_case(rng, n, heads, groups, dim, vdim, [(13, 14.0)])
    r1, r2 = np.array([1.5, 0.5]), np.array([2.0, 0.1])
    want = plain_biased_attention(q, k, v, plain.chunk_mask(n, None), scale, r1, r2)
    assert np.abs(want[-1, 0] - v[13, 0]).max() < 0.05 and np.abs(want[12, 0] - v[13, 0]).max() > 0.3
    pages = -(-n // page)
    k_cache = torch.zeros((pages, page, groups, dim))
    v_cache = torch.zeros((pages, page, groups, vdim))
    k_cache.view(-1, groups, dim)[:n] = torch.tensor(k)
    v_cache.view(-1, groups, vdim)[:n] = torch.tensor(v)
    table = i32(range(pages)).view(1, pages)
    got = ops.paged_attention(dev(q), k_cache.to(DEV), v_cache.to(DEV), table, torch.zeros(n, dtype=torch.int32, device=DEV),
                              i32(range(n)), page_size=page, scale=scale, window=None, chunk=None,
                              log_bias=dev(np.stack([r1, r2])))
    close(got.cpu().numpy(), want, 3e-5, "every position")
    last = ops.paged_attention(dev(q[-1:]), k_cache.to(DEV), v_cache.to(DEV), table, i32([0]), i32([n - 1]), page_size=page,
                               scale=scale, window=None, chunk=None, log_bias=dev(np.stack([r1, r2])))
    close(last.cpu().numpy(), want[-1:], 3e-5, "the last token alone")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, groups, dim, vdim, page, transposed", [(4, 2, 16, 24, 16, True), (3, 1, 12, 20, 32, True),
                                                                         (6, 2, 64, 72, 64, True), (2, 2, 8, 8, 16, False)])
def test_biases_join_the_projections_before_the_one_rounding(ops, dtype, heads, groups, dim, vdim, page, transposed):
    rng = np.random.default_rng(dim + vdim)
    n, pages = 45, 5
    qs, ks, vs = heads * dim, groups * dim, groups * vdim
    sums = rng.normal(size=(n, qs + ks + vs + 8)) * 3  # rows wider than q, k and v together
    bias = rng.normal(size=qs + ks + vs)
    # the float32 sum, then one rounding to the cache's type
    want = (torch.tensor(sums[:, : qs + ks + vs], dtype=torch.float32) + torch.tensor(bias, dtype=torch.float32)).to(dtype).double().numpy()
    slots = rng.permutation(pages * page)[:n]
    k_cache = torch.full((pages, page, groups, dim), 9.0, dtype=dtype, device=DEV)
    v_shape = (pages, groups, vdim, page) if transposed else (pages, page, groups, vdim)
    v_cache = torch.full(v_shape, 9.0, dtype=dtype, device=DEV)
    wide = dev(sums)
    q = ops.qkv_bias_store(wide[:, : qs + ks + vs], dev(bias), k_cache, v_cache, i32(slots), q_size=qs, k_size=ks, v_size=vs,
                           out_dtype=dtype, store=True, v_transposed=transposed)
    assert q.dtype == dtype and np.array_equal(q.double().cpu().numpy(), want[:, :qs])
    got_k = k_cache.view(-1, ks)[torch.tensor(slots, device=DEV)].double().cpu().numpy()
    assert np.array_equal(got_k, want[:, qs: qs + ks])
    if transposed:
        got_v = v_cache.permute(0, 3, 1, 2).reshape(-1, vs)[torch.tensor(slots, device=DEV)].double().cpu().numpy()
    else:
        got_v = v_cache.view(-1, vs)[torch.tensor(slots, device=DEV)].double().cpu().numpy()
    assert np.array_equal(got_v, want[:, qs + ks:])
    assert int((k_cache == 9.0).sum()) >= (pages * page - n) * ks - 5  # other slots are left alone
    # a run that stores nothing: the queries alone
    q = ops.qkv_bias_store(wide[:, :qs], dev(bias[:qs]), None, None, None, q_size=qs, k_size=ks, v_size=vs, out_dtype=dtype,
                           store=False)
    assert np.array_equal(q.double().cpu().numpy(), want[:, :qs])


def test_a_gated_activation_and_a_residual_sum_take_their_biases_and_scales(ops):
    rng = np.random.default_rng(2)
    gu, bias = rng.normal(size=(9, 2 * 37)) * 2, rng.normal(size=2 * 37)
    z = rounded(gu, torch.float32) + rounded(bias, torch.float32)
    got = ops.gated_act(dev(gu), alpha=1.0, offset=0.0, limit=0.0, bias=dev(bias))
    assert np.abs(got.cpu().numpy() - plain.silu(z[:, :37]) * z[:, 37:]).max() < 1e-5
    resid, delta = rng.normal(size=(6, 100)), rng.normal(size=(6, 100))
    scale, down_bias, gain = rng.normal(size=100), rng.normal(size=100), rng.normal(size=100)
    x = resid + (delta + down_bias) * scale
    r = dev(resid)
    out = ops.add_normed_rmsnorm(r, dev(delta), dev(gain), 1e-4, torch.float32, delta_scale=dev(scale), delta_bias=dev(down_bias))
    assert np.abs(r.cpu().numpy() - x).max() < 1e-5
    assert np.abs(out.cpu().numpy() - plain.rms_norm(x, gain, 1e-4)).max() < 1e-4
    r = dev(resid)
    out = ops.add_normed_rmsnorm(r, dev(delta), dev(gain), 1e-4, torch.float32, delta_scale=dev(scale), row_idx=i32([4, 1]))
    assert np.abs(out.cpu().numpy() - plain.rms_norm(resid + delta * scale, gain, 1e-4)[[4, 1]]).max() < 1e-4
    assert np.array_equal(r.cpu().numpy(), resid.astype(np.float32))


def router_of(experts, identity, top, count, keep, scale):
    return {"experts": experts, "identity": identity, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}}


@pytest.mark.parametrize("experts, identity, top, count, keep", [
    (10, 6, 4, 4, 3), (5, 1, 2, 3, 2), (4, 0, 4, 1, 1), (2, 3, 2, 5, 5), (8, 0, 1, 4, 1), (60, 4, 6, 8, 3),
    (300, 84, 32, 12, 5), (1, 1, 1, 2, 1), (6, 6, 4, 6, 4), (3, 0, 3, 3, 3)])
def test_routing_by_corrected_scores_inside_the_best_groups(ops, experts, identity, top, count, keep):
    rng = np.random.default_rng(experts * 7 + identity)
    outputs, n = experts + identity, 61
    logits = (rng.normal(size=(n, outputs)) * 2.0).astype(np.float32)
    # corrections as large as the scores, most of them below zero: barred outputs must lose to negative ones
    correction = (rng.normal(size=outputs) / outputs - 0.7 / outputs).astype(np.float32)
    router = router_of(experts, identity, top, count, keep, 2.5)
    weights = {"router": np.eye(outputs), "correction": correction.astype(np.float64)}
    chosen, chosen_w, margin = plain.route(logits.astype(np.float64), weights, "", router)
    got_e, got_w, got_id = ops.route_scored(dev(logits), dev(correction), n_experts=experts, top=top, groups=count,
                                            keep=keep, scale=2.5)
    got_e, got_w = got_e.cpu().numpy(), got_w.cpu().numpy()
    assert (got_id is None) == (identity == 0)
    clear = margin > 1e-6
    assert clear.mean() > 0.9
    for t in np.flatnonzero(clear):
        assert got_e[t].tolist() == chosen[t], (t, got_e[t], chosen[t])  # in the order of the corrected scores
        want_w = np.array([0.0 if e >= experts else w for e, w in zip(chosen[t], chosen_w[t])])
        assert np.abs(got_w[t] - want_w).max() < 1e-6 * 2.5
        if identity:
            want_id = sum(w for e, w in zip(chosen[t], chosen_w[t]) if e >= experts)
            assert abs(float(got_id[t]) - want_id) < 1e-6 * 2.5
    # without a correction the scores themselves choose
    got_e, _w, _i = ops.route_scored(dev(logits), None, n_experts=experts, top=top, groups=count, keep=keep)
    weights["correction"] = np.zeros(outputs)
    chosen, _, margin = plain.route(logits.astype(np.float64), weights, "", router)
    for t in np.flatnonzero(margin > 1e-6):
        assert got_e[t].tolist() == chosen[t]


def test_routing_among_equals_takes_the_lower_index_and_bars_groups_by_their_best(ops):
    # six outputs in three pairs; every score 1/6; corrections in eighths (exact sums)
    correction = np.array([-0.5, -0.5, -0.875, -0.75, 0.0, 0.0], dtype=np.float32)
    logits = np.zeros((2, 6), dtype=np.float32)
    got_e, got_w, got_id = ops.route_scored(dev(logits), dev(correction), n_experts=4, top=3, groups=3, keep=2, scale=3.0)
    # pair 1 is barred (its best -0.75 + 1/6 is the lowest): of the rest 4, 5 (equal: the lower first), then 0 before 1
    assert got_e.cpu().numpy().tolist() == [[4, 5, 0]] * 2
    assert np.allclose(got_w.cpu().numpy(), [[0.0, 0.0, 0.5]] * 2) and np.allclose(got_id.cpu().numpy(), [1.0, 1.0])
    # all groups kept: the barred pair's -0.75 is not chosen either (lower than -0.5), but with top 5 it is
    got_e, _, _ = ops.route_scored(dev(logits), dev(correction), n_experts=4, top=5, groups=3, keep=3)
    assert got_e.cpu().numpy().tolist() == [[4, 5, 0, 1, 3]] * 2
    # two groups kept and all four of their outputs wanted
    got_e, _, _ = ops.route_scored(dev(logits), dev(correction), n_experts=4, top=4, groups=3, keep=2)
    assert got_e.cpu().numpy().tolist() == [[4, 5, 0, 1]] * 2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width, experts, identity, top, ff, count, keep", [
    (64, 5, 1, 2, 24, 3, 2), (48, 3, 0, 1, 32, 1, 1), (512, 6, 2, 4, 520, 4, 3), (100, 4, 0, 4, 7, 2, 2),
    (128, 8, 4, 4, 64, 4, 3), (160, 2, 6, 3, 80, 8, 5), (64, 1, 3, 4, 16, 2, 2),
    (128, 6, 2, 4, 4608, 4, 3)])  # the last: a token's hidden activations take more than 64 KB of LDS
def test_mixture_with_identity_experts_against_the_plain_one(ops, dtype, width, experts, identity, top, ff, count, keep):
    from pylon_amd.config.specs import MixtureFeedForwardSpec
    from pylon_amd.parts import build_part

    rng = np.random.default_rng(width + ff + identity)
    outputs = experts + identity
    spec = MixtureFeedForwardSpec(hidden_size=width, n_experts=experts, top=top, expert_size=ff, shared_size=None,
                                  shared_gate=False, router_bias=True, expert_act="relu2", scoring="softmax_all",
                                  n_identity=identity, groups=count, groups_kept=keep, route_scale=1.75)
    part = build_part("feed_forward", spec, dtype=dtype, device=DEV)
    w = {"f.router": rng.normal(size=(outputs, width)) * 0.3, "f.correction": rng.normal(size=outputs) / outputs}
    for e in range(experts):
        w[f"f.e{e}.up"], w[f"f.e{e}.down"] = rng.normal(size=(ff, width)) * 0.2, rng.normal(size=(width, ff)) * 0.2
    w = {k: rounded(a, torch.float32 if k == "f.correction" else dtype) for k, a in w.items()}  # what the part will hold
    p = part.params
    p["router"][:] = dev(w["f.router"], dtype)
    p["router_bias"][:] = dev(w["f.correction"])
    for e in range(experts):
        p["up"][e * ff: (e + 1) * ff] = dev(w[f"f.e{e}.up"], dtype)
        p["down"][e * width: (e + 1) * width] = dev(w[f"f.e{e}.down"], dtype)
    mlp = {"router": router_of(experts, identity, top, count, keep, 1.75)}
    for n in (1, 5, 70, 150, 400):  # the products change kernels with the row count (from 256 tokens: sorted by expert)
        h = torch.tensor(rng.normal(size=(n, width)), dtype=dtype)
        margins = []
        want = plain.mixture(h.double().numpy(), w, "f.", mlp, margins)
        clear = margins[0] > 1e-5
        assert clear.mean() > 0.9
        got = part.forward(h.to(DEV), None)
        assert got.dtype == torch.float32 and got.shape == (n, width)
        close(got.cpu().numpy()[clear], want[clear], 2e-5 if dtype == torch.float32 else 3e-2, f"{n} tokens")
        if n == 70:  # a token's result does not depend on its neighbours in the step
            alone = part.forward(h[3:4].to(DEV), None)
            if dtype == torch.float32:
                assert np.abs(alone.cpu().numpy() - got[3:4].cpu().numpy()).max() <= 2e-5 * np.abs(want).max()


@pytest.mark.parametrize("tokens_n", [300, 400])
def test_experts_sorted_by_expert_pass_over_identities_at_tile_edges(ops, tokens_n):
    """The matrix-core path against the token-by-token kernels on routings made by hand: an expert
    nobody chose, experts with exactly one tile, one pair more, one pair, many identities, and the rest."""
    rng = np.random.default_rng(tokens_n)
    width, ff, experts, top = 72, 40, 5, 2
    pairs = tokens_n * top
    tile = 128 if pairs // experts >= 128 else 64
    counts = [0, tile, tile + 1, 1, 0, 90, 33]  # the last two: identities (choices 5 and 6)
    counts[4] = pairs - sum(counts)
    flat = np.repeat(np.arange(experts + 2), counts)
    rng.shuffle(flat)
    chosen = flat.reshape(tokens_n, top)
    weights = rng.uniform(0.1, 1.0, size=(tokens_n, top)).astype(np.float32)
    identity = (weights * (chosen >= experts)).sum(axis=1).astype(np.float32)
    weights[chosen >= experts] = 0.0
    x = torch.tensor(rng.normal(size=(tokens_n, width)), dtype=torch.bfloat16, device=DEV)
    up = torch.tensor(rng.normal(size=(experts * ff, width)) * 0.2, dtype=torch.bfloat16, device=DEV)
    down = torch.tensor(rng.normal(size=(experts * width, ff)) * 0.2, dtype=torch.bfloat16, device=DEV)
    e, w, ident = i32(chosen.reshape(-1)).view(tokens_n, top), dev(weights), dev(identity)
    hidden = ops.expert_gate_up(x, up, e, n_experts=experts, ff=ff, act="relu2")
    want = ops.expert_down(hidden, down, e, w, n_experts=experts, width=width, identity_x=x, identity_weight=ident)
    got = ops.experts_grouped(x, up, down, e, w, n_experts=experts, ff=ff, act="relu2", identity_weight=ident)
    close(got.cpu().numpy(), want.double().cpu().numpy(), 2e-2, "sorted by expert")
    # and against the rule itself, in float64
    xs, ups, downs = x.double().cpu().numpy(), up.double().cpu().numpy(), down.double().cpu().numpy()
    ref = identity[:, None] * xs
    for t in range(tokens_n):
        for s in range(top):
            c = chosen[t, s]
            if c < experts:
                mid = rounded(np.maximum(ups[c * ff: (c + 1) * ff] @ xs[t], 0.0) ** 2, torch.bfloat16)
                ref[t] += weights[t, s] * (downs[c * width: (c + 1) * width] @ mid)
    close(want.double().cpu().numpy(), ref, 1e-2, "token by token")


# ---- whole models ---------------------------------------------------------------------------------
class Case:
    def __init__(self, tmp, name, dtype, lengths, seed=3):
        self.folder = make_folder(tmp, name, dtype=dtype, seed=seed)
        self.cfg, self.weights = read_folder(self.folder)
        self.requests = {f"r{i}": tokens(self.cfg["vocab"], n, 50 + i) for i, n in enumerate(lengths)}
        self.want, self.clear = {}, {}
        for rid, toks in self.requests.items():
            margins = []
            self.want[rid] = plain.forward(self.cfg, self.weights, toks, margins=margins)
            # In bfloat16 a router's choice between two nearly equal scores is an accident of
            # rounding: positions at which some router's margin is that small are not compared.
            closest = np.min(margins, axis=0) if margins else np.full(len(toks), np.inf)
            self.clear[rid] = closest >= (1e-6 if dtype == "float32" else ROUTER_MARGIN)
        self.dtype = dtype
        self.bound = F32_BOUND if dtype == "float32" else BF16_BOUND

    def runner(self, page_size=16, num_pages=40, max_requests=3):
        from pylon_amd.engine import Runner

        return Runner.from_folder(self.folder, dtype=self.dtype, page_size=page_size, num_pages=num_pages,
                                  max_requests=max_requests)

    def check(self, rid, got, label):
        clear = self.clear[rid][: len(got)]
        assert clear.mean() >= getattr(self, "least_clear", 0.3), "too few positions with clear routing to compare"
        assert np.isfinite(got).all()
        if not clear.any():
            return
        got, want = got[clear], self.want[rid][: len(got)][clear]
        ok, worst, frac = rows_within(got, want, self.bound if self.dtype == "float32" else 3 * self.bound)
        assert ok, f"{label}: request {rid}, position {np.flatnonzero(clear)[worst]} is off by {frac:.2e} of its largest logit"
        if self.dtype != "float32":
            # A choice that rounding did flip at an unclear position also moves the positions that look
            # back at it: a few may be further off than rounding alone explains, none by much.
            over = np.abs(got - want).max(axis=1) > self.bound * np.abs(want).max(axis=1)
            assert over.mean() <= 0.05, f"{label}: request {rid}: {over.sum()} of {len(over)} positions are off by more than {self.bound}"


def run_plan(runner, case, plan):
    """``plan``: steps ``{request: tokens to feed}``; 0 closes a request.  Returns logits per request."""
    from pylon_amd.engine import StepEntry

    live, pos = {}, {rid: 0 for rid in case.requests}
    got = {rid: [] for rid in case.requests}
    for step in plan:
        entries = []
        for rid, size in step.items():
            if size == 0:
                runner.close(live.pop(rid))
                continue
            if rid not in live:
                live[rid] = runner.open(rid)
            chunk = case.requests[rid][pos[rid]: pos[rid] + size]
            entries.append((rid, StepEntry(live[rid], chunk, list(range(len(chunk))))))
            pos[rid] += len(chunk)
        if entries:
            logits = runner.step([e for _, e in entries]).cpu().numpy()
            cursor = 0
            for rid, e in entries:
                got[rid].append(logits[cursor: cursor + len(e.tokens)])
                cursor += len(e.tokens)
        runner.manager.check()
    for seq in live.values():
        runner.close(seq)
    return {rid: np.concatenate(parts) for rid, parts in got.items() if parts}, pos


@pytest.mark.parametrize("name, page", [("P", 16), ("Q", 16), ("R", 16), ("S", 32)])
def test_the_stream_after_every_layer(tmp, name, page):
    """What every layer hands on (the mix of all results so far), in float32, for a whole prompt and
    for the same tokens in two portions."""
    from pylon_amd.engine import StepEntry

    case = Case(tmp, name, "float32", (45,))
    runner = case.runner(page_size=page, num_pages=8)
    kept = []

    def watch(norm):
        def wrapped(resid, delta, *, row_idx=None, inner=norm.add_forward):
            out = inner(resid, delta, row_idx=row_idx)
            if delta is not None:
                kept.append(resid.cpu().numpy().copy())  # the norm's kernel has left the mix there
            return out
        norm.add_forward = wrapped

    for block in runner.model.blocks[1:]:
        watch(block.mixer_norm)
    watch(runner.model.final_norm)
    toks = case.requests["r0"]
    _, want = plain.forward(case.cfg, case.weights, toks, keep_layers=True)
    seq = runner.open("a")
    runner.step([StepEntry(seq, toks, [0])])
    runner.close(seq)
    assert len(kept) == len(want) == len(case.cfg["layers"])
    for layer, (got, ref) in enumerate(zip(kept, want)):
        assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max(), f"layer {layer}"
    kept.clear()
    seq = runner.open("b")
    runner.step([StepEntry(seq, toks[:19], [0])])
    runner.step([StepEntry(seq, toks[19:], [0])])
    for layer, ref in enumerate(want):
        got = np.concatenate([kept[layer], kept[len(want) + layer]])
        assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max(), f"layer {layer}, two portions"


@pytest.mark.parametrize("name, dtype, page", [("P", "float32", 16), ("Q", "float32", 16), ("R", "float32", 16),
                                                ("S", "float32", 32), ("R", "bfloat16", 16), ("P", "bfloat16", 16),
                                                ("Q", "bfloat16", 32), ("Q", "bfloat16", 64), ("S", "bfloat16", 64),
                                                ("P", "bfloat16", 64)])
def test_whole_token_by_token_and_in_portions(tmp, name, dtype, page):
    """Pages of 16 tokens run the general attention kernel, pages of 32 and 64 the matrix-core one
    where the heads' sizes allow it."""
    case = Case(tmp, name, dtype, (71, 38))
    runner = case.runner(page_size=page, num_pages=640 // page)
    whole, _ = run_plan(runner, case, [{"r0": 71}, {"r0": 0, "r1": 38}])
    for rid, got in whole.items():
        case.check(rid, got, "whole")
    single, _ = run_plan(runner, case, [{"r1": 1} for _ in range(38)])
    case.check("r1", single["r1"], "token by token")
    cut, _ = run_plan(runner, case, [{"r0": n} for n in (2, 3, 2, 17, 1, 1, 30, 2, 13)])
    case.check("r0", cut["r0"], "portions")
    if dtype == "float32":  # how a request is cut moves nothing but the order of a product's sums
        assert np.abs(cut["r0"] - whole["r0"]).max() <= 2e-5 * np.abs(whole["r0"]).max()
        assert np.abs(single["r1"] - whole["r1"]).max() <= 2e-5 * np.abs(whole["r1"]).max()


@pytest.mark.parametrize("name, dtype, page", [("P", "float32", 16), ("Q", "float32", 16), ("S", "float32", 16),
                                                ("R", "bfloat16", 16), ("Q", "bfloat16", 32), ("S", "bfloat16", 32)])
def test_mixed_batches_over_pages_and_slots_that_are_used_again(tmp, name, dtype, page):
    case = Case(tmp, name, dtype, (60, 45, 33, 20))
    pages = 9 if page == 16 else 6  # room for 144 (or 192) tokens: never all four requests at once
    runner = case.runner(page_size=page, num_pages=pages, max_requests=3)
    plan = [{"r0": 20}, {"r0": 1, "r1": 30}, {"r0": 2, "r1": 1, "r2": 5}, {"r0": 1, "r1": 1, "r2": 1},
            {"r0": 20, "r1": 13, "r2": 2}, {"r1": 0, "r0": 1, "r2": 1}, {"r3": 17, "r0": 15, "r2": 24},
            {"r2": 0, "r0": 0, "r3": 1}, {"r3": 2}]
    got, pos = run_plan(runner, case, plan)
    assert pos == {"r0": 60, "r1": 45, "r2": 33, "r3": 20}
    for rid, logits in got.items():
        case.check(rid, logits, "mixed")
    alone, _ = run_plan(runner, case, [{"r3": 20}])
    if dtype == "float32":
        assert np.abs(alone["r3"] - got["r3"]).max() <= 2e-5 * np.abs(alone["r3"]).max()
    assert runner.manager.free_pages == pages and runner.manager.slots.free_slots == 3


@pytest.mark.parametrize("name, dtype, pages", [("Q", "float32", 4), ("Q", "bfloat16", 4), ("R", "float32", 8)])
def test_long_decoding_after_a_prompt(tmp, name, dtype, pages):
    """420 tokens, 320 of them one by one.  Q's chunks of 50 and 128 never need more than 4 pages of
    64, because the pages a chunk has left behind go back while the request runs; R keeps them all."""
    case = Case(tmp, name, dtype, (420,))
    runner = case.runner(page_size=64, num_pages=pages, max_requests=2)
    got, _ = run_plan(runner, case, [{"r0": 100}] + [{"r0": 1}] * 320)
    case.check("r0", got["r0"], "long decoding")
    assert runner.manager.free_pages == pages


def test_requests_do_not_see_what_a_freed_slot_or_page_held(tmp):
    """The same request, alone in a fresh runner and after others have used every page and slot."""
    case = Case(tmp, "P", "float32", (50, 64, 64))
    fresh, _ = run_plan(case.runner(num_pages=8, max_requests=2), case, [{"r0": 50}])
    runner = case.runner(num_pages=8, max_requests=2)
    for tensor in runner.manager.slots.tensors.values():
        tensor.fill_(float("nan"))
    for group in runner.manager.groups:
        for cache in list(group.k.values()) + [v for v in group.v.values() if v is not None]:
            cache.fill_(float("nan"))
    used, _ = run_plan(runner, case, [{"r1": 64, "r2": 64}, {"r1": 0, "r2": 0}, {"r0": 25}, {"r0": 25}])
    assert np.abs(used["r0"] - fresh["r0"]).max() <= 2e-5 * np.abs(fresh["r0"]).max()


def test_the_first_tokens_of_a_sequence_start_from_nothing(tmp):
    """Position 0 sees itself alone and is shifted towards zeros: its logits are those of a
    one-token request, whatever follows it and whatever ran in its slot before."""
    case = Case(tmp, "Q", "float32", (9, 30))
    runner = case.runner(num_pages=8, max_requests=1)
    first, _ = run_plan(runner, case, [{"r1": 30}, {"r1": 0}, {"r0": 1}])
    want = plain.forward(case.cfg, case.weights, case.requests["r0"][:1])
    assert np.abs(first["r0"] - want).max() <= F32_BOUND * np.abs(want).max()
    assert np.abs(case.want["r0"][0] - want[0]).max() <= 1e-9 * np.abs(want).max()


@pytest.mark.parametrize("name, dtype, graphs, page", [("P", "float32", False, 16), ("Q", "float32", True, 16),
                                                         ("R", "bfloat16", True, 16), ("Q", "bfloat16", True, 32),
                                                         ("S", "bfloat16", True, 64)])
def test_greedy_generation_through_the_engine(tmp, name, dtype, graphs, page):
    from pylon_amd.engine.engine import Engine
    from pylon_amd.sampling import Sampling

    folder = make_folder(tmp, name, dtype=dtype, seed=8)
    cfg, weights = read_folder(folder)
    prompts = [tokens(cfg["vocab"], n, 70 + n) for n in (3, 19, 41)]
    engine = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=384 // page, max_batch_size=3,
                                prefill_chunk_size=16, cuda_graphs=graphs)
    try:
        results = engine.generate(prompts, Sampling(max_new_tokens=12, temperature=0.0))
    finally:
        engine.close()
    slack = 1e-4 if dtype == "float32" else 5e-2
    for prompt, result in zip(prompts, results):
        assert len(result.output_ids) == 12
        sequence = list(prompt)
        for produced in result.output_ids:
            row = plain.forward(cfg, weights, sequence)[-1]
            assert produced == int(row.argmax()) or row.max() - row[produced] <= slack * np.abs(row).max(), \
                (prompt[:3], result.output_ids)
            sequence.append(produced)


def draw_config(seed: int):
    """A configuration drawn over what config.json allows: any order of layers with and without
    keys and values of their own, heads and sizes in steps of 8 and a few odd ones, chunks that are no
    multiple of anything, every shape of router."""
    rng = np.random.default_rng(4000 + seed)
    width = int(rng.choice([48, 64, 96, 136, 160, 256]))
    layers, owners = [], []
    for index in range(int(rng.integers(2, 7))):
        borrow = owners and rng.random() < 0.45
        if borrow:
            lender = int(rng.choice(owners))
            m = dict(layers[lender]["mixer"])
            m.pop("kv_from", None)
            m["kv_from"] = lender
            m["scale"] = float(rng.uniform(0.05, 0.4))
            if rng.random() < 0.3:
                m["mask"] = {"size": int(rng.integers(3, 200))}
        else:
            kv_heads = int(rng.integers(1, 4))
            dim = int(rng.choice([8, 16, 24, 32, 40, 64, 96, 128, 12]))
            m = {"heads": kv_heads * int(rng.choice([1, 2, 3, 4, 8])), "kv_heads": kv_heads, "dim": dim,
                 "vdim": int(rng.choice([4, 8, 20, 32, 48, 64, 80, 128, 10])), "scale": float(rng.uniform(0.05, 0.4)),
                 "mask": {"size": int(rng.choice([int(rng.integers(3, 200)), 32, 64, 128, 1000]))}}
            owners.append(index)
        kind = rng.random()
        if kind < 0.15:
            mlp = None
        elif kind < 0.4:
            mlp = {"kind": "dense", "ff": 2 * int(rng.integers(8, 80))}
        else:
            count = int(rng.choice([1, 2, 3, 4, 6]))
            per_group = int(rng.integers(1, 5))
            outputs = count * per_group
            identity = int(rng.integers(0, outputs))  # at least one expert
            keep = int(rng.integers(1, count + 1))
            top = int(rng.integers(1, min(keep * per_group, 8) + 1))
            mlp = {"kind": "moe", "expert": {"ff": 8 * int(rng.integers(1, 12))},
                   "router": {"experts": outputs - identity, "identity": identity, "top": top,
                              "scale": float(rng.uniform(0.5, 3.0)), "groups": {"count": count, "keep": keep}}}
        layers.append({"type": "attention", "mixer": m, "mlp": mlp})
    config = {"architecture": "Gimudra", "vocab": int(rng.integers(90, 700)), "width": width,
              "norm": {"eps": float(10 ** rng.uniform(-7, -4))}, "embedding": {"scale": float(rng.uniform(0.3, 3.0))},
              "layers": layers}
    return config, (int(rng.integers(1, 40)), int(rng.integers(60, 200)), int(rng.integers(200, 330)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(10))
def test_a_configuration_drawn_at_random_matches_the_plain_model(tmp, seed, dtype):
    """Pages of 64 and four slots, as the replay program has them: each request whole, the longest with
    its tail token by token, then all three side by side in portions over a pool too small for them
    to have pages to spare."""
    config, lengths = draw_config(seed)
    case = Case.__new__(Case)
    case.folder = make_folder(tmp, f"drawn{seed}", dtype=dtype, seed=seed, config=config)
    case.cfg, case.weights = read_folder(case.folder)
    case.requests = {f"r{i}": tokens(case.cfg["vocab"], n, 90 + i) for i, n in enumerate(lengths)}
    case.want, case.clear = {}, {}
    for rid, toks in case.requests.items():
        margins = []
        case.want[rid] = plain.forward(case.cfg, case.weights, toks, margins=margins)
        closest = np.min(margins, axis=0) if margins else np.full(len(toks), np.inf)
        if dtype == "float32":
            case.clear[rid] = closest >= 1e-6
        else:
            # These routers are steep: bfloat16 rounding of their inputs moves scores by a hundredth, a
            # flipped choice changes the token's whole feed-forward output, and the shift and the
            # attention carry that to every later token.  Only the positions before the first
            # unclear choice are held to the plain model; float32 holds them all.
            unclear = np.flatnonzero(closest < 0.03)
            case.clear[rid] = np.arange(len(toks)) < (unclear[0] if len(unclear) else len(toks))
    case.dtype, case.bound = dtype, F32_BOUND if dtype == "float32" else BF16_BOUND
    case.least_clear = 0.0
    if sum(int(c.sum()) for c in case.clear.values()) < 40:
        pytest.skip("too few positions with clear routing in this draw")
    pages = sum(-(-n // 64) for n in lengths)
    runner = case.runner(page_size=64, num_pages=pages, max_requests=4)
    whole, _ = run_plan(runner, case, [{"r0": lengths[0]}, {"r0": 0, "r1": lengths[1]}, {"r1": 0, "r2": lengths[2]}])
    for rid, got in whole.items():
        case.check(rid, got, f"whole (seed {seed})")
    tail, _ = run_plan(runner, case, [{"r2": lengths[2] - 70}] + [{"r2": 1}] * 70)
    case.check("r2", tail["r2"], f"decoded tail (seed {seed})")
    plan, left = [], dict(zip(("r0", "r1", "r2"), lengths))
    sizes = iter(np.random.default_rng(seed).choice([1, 2, 3, 7, 31, 64, 65, 100], size=200).tolist())
    while any(left.values()):
        step = {}
        for rid in left:
            if left[rid]:
                step[rid] = min(left[rid], next(sizes))
                left[rid] -= step[rid]
        plan.append(step)
    mixed, _ = run_plan(runner, case, plan)
    for rid, got in mixed.items():
        case.check(rid, got, f"portions side by side (seed {seed})")
        if dtype == "float32":
            assert np.abs(got - whole[rid]).max() <= 2e-5 * np.abs(whole[rid]).max(), (seed, rid)
    assert runner.manager.free_pages == pages
