"""Tukarax on the GPU against the plain implementation: every mechanism's kernel alone, then
whole models cut every way (whole prompts, token by token, portions down to two tokens, mixed
batches over pages and slots that are used again), long decoding, and greedy generation
through the engine."""
import math

import numpy as np
import pytest
import torch

from tests.helpers import rows_within
from tests.plain import tukarax as plain
from tests.tukarax_helpers import CONFIGS, make_folder, read_folder, tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32_BOUND = 2e-4   # of a row's largest |logit|
BF16_BOUND = 1e-1
ROUTER_MARGIN = 0.1  # in bfloat16, choices between router outputs closer than this share of the largest are accidents of rounding


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
    return tmp_path_factory.mktemp("tukarax")


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


# ---- the delta rule ------------------------------------------------------------------------------

def plain_delta_outputs(q, k, v, gate, b, a, a_log, dt_bias, norm_w, heads, kv_heads, dim, vdim, eps):
    """From conv'd q, k, v rows: unit vectors, beta, decay, the recurrence, the head norm and the gate."""
    n = q.shape[0]
    q = q.reshape(n, kv_heads, dim)
    k = k.reshape(n, kv_heads, dim)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * dim ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    rep = heads // kv_heads
    q, k = np.repeat(q, rep, axis=1), np.repeat(k, rep, axis=1)
    beta = plain.sigmoid(b)
    decay = np.exp(-np.exp(a_log) * plain.softplus(a + dt_bias))
    o = plain.delta_rule(q, k, v.reshape(n, heads, vdim), beta, decay)
    o = plain.rms_norm(o, norm_w, eps) * plain.silu(gate).reshape(n, heads, vdim)
    return o.reshape(n, heads * vdim)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, kv_heads, dim, vdim", [(4, 2, 12, 20), (2, 2, 32, 32), (2, 1, 128, 128), (3, 1, 64, 128),
                                                        (2, 2, 256, 64), (1, 1, 100, 24), (2, 1, 6, 4), (1, 1, 256, 256),
                                                        (5, 5, 1, 1), (2, 2, 48, 200)])
def test_delta_rule_in_portions_of_two_requests_over_reused_slots(ops, heads, kv_heads, dim, vdim, out_dtype):
    """Two requests of 41 and 23 tokens in portions of changing size (single tokens among them, more
    than a piece of sixteen too), in slots that held other numbers before; decays close to one, so
    that a state lost between two portions is missed."""
    rng = np.random.default_rng(heads * 1000 + dim + vdim)
    lengths = {"x": 41, "y": 23}
    qk, vv = kv_heads * dim, heads * vdim
    data = {}
    for rid, n in lengths.items():
        data[rid] = dict(qkv=rng.normal(size=(n, 2 * qk + vv)), gate=rng.normal(size=(n, vv)),
                         b=rng.normal(size=(n, heads)) * 2, a=rng.normal(size=(n, heads)) * 2)
    a_log, dt_bias = rng.uniform(-4.0, -1.0, heads), rng.normal(size=heads)
    norm_w = 1.0 + 0.3 * rng.normal(size=vdim)
    eps = 1e-5
    want = {rid: plain_delta_outputs(d["qkv"][:, :qk], d["qkv"][:, qk: 2 * qk], d["qkv"][:, 2 * qk:], d["gate"], d["b"],
                                     d["a"], a_log, dt_bias, norm_w, heads, kv_heads, dim, vdim, eps)
            for rid, d in data.items()}
    state = torch.full((3, heads, vdim, dim), 9.0, device=DEV)
    slots = {"x": 2, "y": 0}
    for slot in slots.values():
        state[slot].zero_()  # what the manager does when it hands a slot out
    plan = [{"x": 5}, {"x": 1, "y": 2}, {"y": 1}, {"x": 18, "y": 1}, {"x": 1}, {"y": 19, "x": 16}]
    # a head's columns dealt to several workgroups where they divide (the norm then in a second kernel)
    groups = max([g for g in (2, 4, 8, 16) if vdim % g == 0 and vdim // g >= 4] + [1])
    pos = {rid: 0 for rid in lengths}
    got = {rid: [] for rid in lengths}
    pad = 3  # the projection's rows are wider than what the kernel reads
    for step in plan:
        rows, qkv_rows, proj_rows, starts = [], [], [], [0]
        for rid, count in step.items():
            d, p = data[rid], pos[rid]
            qkv_rows.append(d["qkv"][p: p + count])
            proj_rows.append(np.concatenate([np.zeros((count, pad)), d["gate"][p: p + count], d["b"][p: p + count],
                                             d["a"][p: p + count]], axis=1))
            rows.append(rid)
            starts.append(starts[-1] + count)
            pos[rid] += count
        out = ops.delta_rule(dev(np.concatenate(qkv_rows)), dev(np.concatenate(proj_rows)), state, dev(a_log), dev(dt_bias),
                             dev(norm_w), i32(starts), i32(slots[r] for r in rows), rows=len(rows), heads=heads,
                             kv_heads=kv_heads, dim=dim, vdim=vdim, gate_off=pad, beta_off=pad + vv,
                             decay_off=pad + vv + heads, eps=eps, unit_eps=1e-6, q_scale=dim ** -0.5, out_dtype=out_dtype,
                             col_groups=groups if len(step) % 2 else 1,  # the two ways in turns over one state,
                             chunked=pos["x"] % 2 == 0)                  # and sixteen tokens at a time or one
        out = out.float().cpu().numpy()
        for i, rid in enumerate(rows):
            got[rid].append(out[starts[i]: starts[i + 1]])
    assert pos == lengths
    assert float(state[1].min()) == 9.0  # nobody's slot
    for rid in lengths:
        close(np.concatenate(got[rid]), want[rid], 2e-4 if out_dtype == torch.float32 else 1e-2, rid)


def test_delta_rule_keeps_what_it_wrote_far_back(ops):
    """With a decay of one and orthogonal unit keys the state answers token 3's key with token 3's
    value 300 tokens later, in a prompt and token by token."""
    n, dim, vdim = 320, 64, 8
    rng = np.random.default_rng(3)
    keys = np.zeros((n, dim))
    keys[np.arange(n), np.arange(n) % (dim - 1) + 1] = 1.0  # never direction 0 ...
    keys[3] = 0.0
    keys[3, 0] = 1.0                                         # ... except token 3
    values = rng.normal(size=(n, vdim))
    queries = np.zeros((n, dim))
    queries[-1, 0] = 1.0
    qkv = np.concatenate([queries, keys, values], axis=1)
    proj = np.concatenate([np.full((n, vdim), 30.0), np.full((n, 1), 30.0), np.full((n, 1), -60.0)], axis=1)  # gate ~x, beta 1, decay 1
    args = dict(heads=1, kv_heads=1, dim=dim, vdim=vdim, gate_off=0, beta_off=vdim, decay_off=vdim + 1, eps=1e-6,
                unit_eps=1e-6, q_scale=1.0, out_dtype=torch.float32)
    want = values[3] / np.sqrt((values[3] ** 2).mean() + 1e-6) * 30.0
    state = torch.zeros((1, 1, vdim, dim), device=DEV)
    for chunked in (False, True):
        state.zero_()
        out = ops.delta_rule(dev(qkv), dev(proj), state, dev([0.0]), dev([0.0]), dev(np.ones(vdim)), i32([0, n]), i32([0]),
                             rows=1, chunked=chunked, **args)
        close(out[-1].cpu().numpy(), want, 1e-4, f"whole, chunked {chunked}")
    state.zero_()
    for t in range(n):
        out = ops.delta_rule(dev(qkv[t: t + 1]), dev(proj[t: t + 1]), state, dev([0.0]), dev([0.0]), dev(np.ones(vdim)),
                             i32([0, 1]), i32([0]), rows=1, **args)
    close(out[-1].cpu().numpy(), want, 1e-4, "token by token")


@pytest.mark.parametrize("taps, width", [(3, 70), (2, 300), (5, 7), (1, 40), (8, 513)])
def test_convolution_with_activation_on_a_slice_of_wider_rows(ops, taps, width):
    rng = np.random.default_rng(taps * 100 + width)
    lengths = {"x": 37, "y": 9}
    data = {rid: rng.normal(size=(n, width + 5)) for rid, n in lengths.items()}
    w = rng.normal(size=(width, taps))
    want = {rid: plain.silu(plain.causal_conv(d[:, :width], w)) for rid, d in data.items()}
    state = torch.full((3, max(taps - 1, 1), width), 5.0, device=DEV)
    slots = {"x": 1, "y": 2}
    for slot in slots.values():
        state[slot].zero_()
    got, pos = {rid: [] for rid in lengths}, {rid: 0 for rid in lengths}
    for step in [{"x": 2}, {"x": 1, "y": 4}, {"x": 20, "y": 1}, {"y": 1, "x": 1}, {"x": 13, "y": 3}]:
        rows, parts, starts = [], [], [0]
        for rid, count in step.items():
            parts.append(data[rid][pos[rid]: pos[rid] + count])
            pos[rid] += count
            rows.append(rid)
            starts.append(starts[-1] + count)
        h = dev(np.concatenate(parts))
        out = ops.short_conv(h[:, :width], dev(w), state if taps > 1 else None, i32(starts), i32(slots[r] for r in rows),
                             rows=len(rows), max_count=max(step.values()), out_dtype=torch.float32, mode="silu")
        out = out.cpu().numpy()
        for i, rid in enumerate(rows):
            got[rid].append(out[starts[i]: starts[i + 1]])
    for rid in lengths:
        close(np.concatenate(got[rid]), want[rid], 1e-5, rid)


# ---- q/k preparation -----------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, kv_heads, dim, rot_dims, neighbours, per_head, keyed, factor", [
    (4, 2, 12, 6, True, True, True, 1.0), (2, 1, 64, 32, True, True, True, 1.0), (3, 3, 10, 10, False, False, False, 1.2079),
    (6, 2, 64, 64, False, False, False, 1.3), (2, 2, 128, 64, True, True, True, 1.0), (4, 1, 24, 0, False, True, True, 1.0)])
def test_head_norms_both_pairings_a_factor_on_the_rotation_and_values_that_are_the_keys(
        ops, heads, kv_heads, dim, rot_dims, neighbours, per_head, keyed, factor, dtype):
    rng = np.random.default_rng(heads + dim)
    n, vdim = 9, dim if keyed else 7
    positions = np.array([0, 1, 2, 63, 64, 65, 1000, 4097, 5])
    q_size, k_size, v_size = heads * dim, kv_heads * dim, 0 if keyed else kv_heads * vdim
    extra = 5  # a gate's columns behind q, k and v
    rows = rounded(rng.normal(size=(n, q_size + k_size + v_size + extra)), dtype)
    qw, kw = 1 + 0.3 * rng.normal(size=dim), 1 + 0.3 * rng.normal(size=dim)
    eps = 1e-5
    q, k = rows[:, :q_size].reshape(n, heads, dim), rows[:, q_size: q_size + k_size].reshape(n, kv_heads, dim)
    v = k.copy() if keyed else rows[:, q_size + k_size: q_size + k_size + v_size].reshape(n, kv_heads, vdim)
    if per_head:
        q, k = plain.rms_norm(q, qw, eps), plain.rms_norm(k, kw, eps)
    if rot_dims:
        freq = 10000.0 ** (-2.0 * np.arange(rot_dims // 2) / rot_dims)
        angle = positions[:, None] * freq.astype(np.float32)[None, :].astype(np.float64)
        c, s = (np.cos(angle) * factor)[:, None, :], (np.sin(angle) * factor)[:, None, :]

        def turn(x):
            out = x.copy()
            if neighbours:
                a, b = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
                out[..., 0:rot_dims:2], out[..., 1:rot_dims:2] = a * c - b * s, b * c + a * s
            else:
                a, b = x[..., : rot_dims // 2], x[..., rot_dims // 2: rot_dims]
                out[..., : rot_dims // 2], out[..., rot_dims // 2: rot_dims] = a * c - b * s, b * c + a * s
            return out
        q, k = turn(q), turn(k)
    slots = [3, 0, 7, 8, 1, 15, 2, 9, 4]
    k_cache = torch.zeros((1, 16, kv_heads, dim), dtype=dtype, device=DEV)
    v_cache = torch.zeros((1, 16, kv_heads, vdim), dtype=dtype, device=DEV)
    q_out = torch.empty((n, heads, dim), dtype=dtype, device=DEV)
    ops.qkv_prepare_wide(dev(rows, dtype), q_out, k_cache, v_cache, n_heads=heads, n_kv_heads=kv_heads, head_dim=dim,
                         v_dim=vdim, q_weight=dev(qw) if per_head else None, k_weight=dev(kw) if per_head else None, eps=eps,
                         inv_freq=dev(10000.0 ** (-2.0 * np.arange(rot_dims // 2) / rot_dims)) if rot_dims else None,
                         rot_dim=rot_dims, interleaved=neighbours, positions=i32(positions), slot_map=i32(slots),
                         store_kv=True, per_head=per_head, rot_scale=factor, values_from_keys=keyed)
    bound = 3e-5 if dtype == torch.float32 else 1e-2
    # at position 4097 a float32 angle is good to a few 1e-4
    close(q_out.float().cpu().numpy()[:6], q[:6], bound, "q")
    close(q_out.float().cpu().numpy(), q, max(bound, 2e-3), "q far out")
    close(k_cache.float().cpu().numpy()[0, slots][:6], k[:6], bound, "k")
    assert np.array_equal(v_cache.float().cpu().numpy()[0, slots], v)  # copied as they are


# ---- attention with capped scores and a learned sink ------------------------------------------------

def planted_case(rng, n, heads, groups, dim, vdim, planted):
    """Keys among which the planted positions stand out along a direction that every query has a
    large share of."""
    direction = rng.normal(size=dim)
    direction /= np.linalg.norm(direction)
    q = rng.normal(size=(n, heads, dim)) + 4.0 * direction
    k = rng.normal(size=(n, groups, dim)) * 0.5
    for j in planted:
        k[j] += 6.0 * direction
    v = rng.normal(size=(n, groups, vdim))
    return q, k, v


@pytest.mark.parametrize("size", [37, 64, 129, 1, 300, None])
@pytest.mark.parametrize("dtype, heads, groups, dim, vdim, page", [
    (torch.float32, 4, 2, 12, 20, 16), (torch.float32, 2, 1, 64, 64, 64), (torch.bfloat16, 6, 2, 64, 64, 64),
    (torch.bfloat16, 3, 3, 32, 48, 32)])
def test_attention_with_a_cap_and_a_sink_at_the_edges_of_chunks_and_pages(ops, size, dtype, heads, groups, dim, vdim, page):
    """A 300-token request whose planted keys lie at position 0, at a page's last and first slot, just
    inside and just outside the chunk of many queries, and far back; pages scattered over a pool
    whose other slots hold NaN; whole, and as a portion over a cached first part."""
    rng = np.random.default_rng(17 + (size or 0))
    n = 300
    planted = sorted({0, page - 1, page, 2 * page, 150, 151} | ({size - 1, size, 2 * size} if size and 2 * size < n else set()))
    q, k, v = planted_case(rng, n, heads, groups, dim, vdim, planted)
    q, k, v = rounded(q, dtype), rounded(k, dtype), rounded(v, dtype)
    scale, cap = 0.3, 4.0
    sink = rng.normal(size=heads) * 3.0
    want = plain.softmax_attention(q, k, v, scale, plain.visible(n, size), cap, sink)
    pages = -(-n // page)
    pool = pages + 5
    order = rng.permutation(pool)[:pages]
    k_cache = torch.full((pool, page, groups, dim), float("nan"), dtype=dtype, device=DEV)
    v_cache = torch.full((pool, page, groups, vdim), float("nan"), dtype=dtype, device=DEV)
    slots = np.array([order[j // page] * page + j % page for j in range(n)])
    k_cache.view(-1, groups, dim)[torch.tensor(slots, device=DEV)] = dev(k, dtype)
    v_cache.view(-1, groups, vdim)[torch.tensor(slots, device=DEV)] = dev(v, dtype)
    table = i32(order).view(1, -1)
    bound = 2e-5 if dtype == torch.float32 else 2e-2
    for first in (0, 143):
        out = ops.paged_attention(dev(q[first:], dtype), k_cache, v_cache, table, i32([0] * (n - first)), i32(range(first, n)),
                                  page_size=page, window=None, chunk=size, scale=scale, softcap=cap, sink_logit=dev(sink))
        close(out.float().cpu().numpy(), want[first:], bound, f"from {first}")
    if dtype == torch.bfloat16:
        # the matrix-core kernel over the same pages, the values transposed inside them: prompt tiles of up
        # to 32 tokens from position 0 and from 143, then every position as a single token with its keys
        # in one piece and cut over 2 and 8 workgroups
        v_t = v_cache.view(pool, page, groups, vdim).permute(0, 2, 3, 1).contiguous()
        for first in (0, 143):
            tiles = i32(x for a in range(first, n, 32) for x in (a - first, min(32, n - a), 0, a)).view(-1, 4)
            out = ops.attention_sink(dev(q[first:], dtype), k_cache, v_t, table, tiles, None, page_size=page, scale=scale,
                                     bias=None, sink=True, chunk=size, softcap=cap, sink_logit=dev(sink))
            close(out.float().cpu().numpy(), want[first:], bound, f"matrix cores from {first}")
        for cuts in (1, 2, 8):
            out = ops.attention_sink(dev(q, dtype), k_cache, v_t, table.expand(n, -1).contiguous(), None, i32(range(n)),
                                     page_size=page, scale=scale, bias=None, sink=True, cuts=cuts, chunk=size,
                                     softcap=cap, sink_logit=dev(sink))
            close(out.float().cpu().numpy(), want, bound, f"single tokens, {cuts} cuts")
    # the cap and the sink matter in this case: without either the result is another
    bare = plain.softmax_attention(q, k, v, scale, plain.visible(n, size), None, sink)
    assert np.abs(bare - want).max() > 0.05
    bare = plain.softmax_attention(q, k, v, scale, plain.visible(n, size), cap, None)
    assert np.abs(bare - want).max() > 0.05


def test_a_sink_that_takes_all_the_weight_and_one_that_takes_none(ops):
    rng = np.random.default_rng(1)
    n, heads, dim = 20, 2, 16
    q, k, v = rng.normal(size=(n, heads, dim)), rng.normal(size=(n, 1, dim)), rng.normal(size=(n, 1, dim))
    k_cache, v_cache = dev(k).view(1, n, 1, dim).contiguous(), dev(v).view(1, n, 1, dim).contiguous()
    k_cache = torch.cat([k_cache, torch.zeros((1, 32 - n, 1, dim), device=DEV)], dim=1)
    v_cache = torch.cat([v_cache, torch.zeros((1, 32 - n, 1, dim), device=DEV)], dim=1)
    sink = np.array([60.0, -60.0])
    out = ops.paged_attention(dev(q), k_cache, v_cache, i32([0]).view(1, 1), i32([0] * n), i32(range(n)), page_size=32,
                              window=None, scale=0.25, sink_logit=dev(sink)).cpu().numpy()
    want = plain.softmax_attention(q, k, v, 0.25, plain.visible(n, None), None, sink)
    assert np.abs(out[:, 0]).max() < 1e-12 and np.abs(want[:, 0]).max() < 1e-12
    close(out[:, 1], want[:, 1], 2e-5)


def test_gates_on_heads_and_elements_and_the_weighted_sum_of_two_mixers(ops):
    rng = np.random.default_rng(2)
    n, heads, vdim = 7, 3, 10
    for dtype in (torch.float32, torch.bfloat16):
        x = rounded(rng.normal(size=(n, heads * vdim)), dtype)
        wide = rounded(rng.normal(size=(n, 4 + heads * vdim)), dtype)
        got = ops.sigmoid_gate_(dev(x, dtype), dev(wide, dtype)[:, 4: 4 + heads], per=vdim).float().cpu().numpy()
        want = (x.reshape(n, heads, vdim) * plain.sigmoid(wide[:, 4: 4 + heads])[:, :, None]).reshape(n, -1)
        close(got, want, 1e-6 if dtype == torch.float32 else 5e-3, "per head")
        got = ops.sigmoid_gate_(dev(x, dtype), dev(wide, dtype)[:, 4:], per=1).float().cpu().numpy()
        close(got, x * plain.sigmoid(wide[:, 4:]), 1e-6 if dtype == torch.float32 else 5e-3, "per element")
    a, b = rng.normal(size=(3, n, 12)), rounded(rng.normal(size=(n, 12)), torch.bfloat16)
    got = ops.scaled_sum(dev(a), 1.2, dev(b, torch.bfloat16), -0.5).cpu().numpy()
    close(got, 1.2 * a.sum(0) - 0.5 * b, 1e-6)
    got = ops.scaled_sum(dev(a[0]), 0.3, dev(a[1:]), 2.0).cpu().numpy()
    close(got, 0.3 * a[0] + 2.0 * a[1:].sum(0), 1e-6)


# ---- the mixture ---------------------------------------------------------------------------------

@pytest.mark.parametrize("experts, top", [(5, 2), (16, 1), (4, 4), (70, 8), (1, 1)])
def test_routing_by_sigmoid_scores(ops, experts, top):
    rng = np.random.default_rng(experts)
    logits = rng.normal(size=(33, experts)) * 3
    chosen, weights, _ = ops.route_top(dev(logits), None, n_experts=experts, top=top, shared_gate=False, scoring="sigmoid")
    scores = plain.sigmoid(logits.astype(np.float32).astype(np.float64))
    order = np.argsort(-scores, axis=-1, kind="stable")[:, :top]
    assert np.array_equal(chosen.cpu().numpy(), order)
    close(weights.cpu().numpy(), np.take_along_axis(scores, order, axis=-1), 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width, experts, top, ff", [(40, 5, 2, 16), (64, 8, 1, 24), (128, 4, 4, 64), (96, 9, 3, 40)])
def test_mixture_with_weights_on_the_inputs_against_the_plain_one(ops, dtype, width, experts, top, ff):
    """1 to 400 tokens: the token-by-token kernels, and from 33 bfloat16 tokens on the sorted path."""
    from pylon_amd.config.specs import MixtureFeedForwardSpec
    from pylon_amd.parts.mixture import MixtureFeedForward

    rng = np.random.default_rng(width + experts)
    spec = MixtureFeedForwardSpec(hidden_size=width, n_experts=experts, top=top, expert_size=ff, shared_size=None,
                                  shared_gate=False, router_bias=False, scoring="sigmoid", weight_on_input=True)
    part = MixtureFeedForward(spec, dtype=dtype, device=DEV)
    w = {"router": rounded(rng.normal(size=(experts, width)) * 0.4, dtype)}
    gate_up, down = [], []
    for e in range(experts):
        w[f"e{e}.gate"], w[f"e{e}.up"] = (rounded(rng.normal(size=(ff, width)) * 0.3, dtype) for _ in range(2))
        w[f"e{e}.down"] = rounded(rng.normal(size=(width, ff)) * 0.3, dtype)
        gate_up += [w[f"e{e}.gate"], w[f"e{e}.up"]]
        down.append(w[f"e{e}.down"])
    part.params["router"].copy_(dev(w["router"], dtype))
    part.params["gate_up"].copy_(dev(np.concatenate(gate_up), dtype))
    part.params["down"].copy_(dev(np.concatenate(down), dtype))
    for n in (1, 7, 32, 33, 130, 400):
        h = rounded(rng.normal(size=(n, width)), dtype)
        margins = []
        want = plain.mixture(h, {"router": {"top": top}}, w, "", margins)
        got = part.forward(dev(h, dtype), None).cpu().numpy()
        clear = margins[0] > (1e-5 if dtype == torch.float32 else 0.05)
        assert clear.mean() > 0.5 or n == 1
        close(got[clear], want[clear], 1e-4 if dtype == torch.float32 else 3e-2, f"{n} tokens")
        alone = part.forward(dev(h[:1], dtype), None).cpu().numpy()
        if n <= 32 or dtype == torch.float32:
            assert np.array_equal(alone[0], got[0])  # a token's result does not depend on the batch


# ---- whole models --------------------------------------------------------------------------------

def clear_tokens(cfg, weights, count, seed, margin=2 * ROUTER_MARGIN):
    """A request drawn token by token so that no router of the plain model has a close call at any
    position (a position's routing depends on the tokens up to it only): a drawn token whose
    position would have one is drawn again."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        for _attempt in range(40):
            candidate = out + [int(rng.integers(0, cfg["vocab"]))]
            margins = []
            plain.forward(cfg, weights, candidate, margins=margins)
            if not margins or min(m[-1] for m in margins) >= margin:
                break
        out = candidate
    return out


class Case:
    def __init__(self, tmp, name, dtype, lengths, seed=3, config=None, pick=None):
        self.folder = make_folder(tmp, name, dtype=dtype, seed=seed, config=config)
        self.cfg, self.weights = read_folder(self.folder)
        # bfloat16 requests of up to a hundred tokens are drawn so that every position's routing is clear
        pick = (dtype != "float32" and max(lengths) <= 100) if pick is None else pick
        if pick:
            self.requests = {f"r{i}": clear_tokens(self.cfg, self.weights, n, 50 + i) for i, n in enumerate(lengths)}
        else:
            self.requests = {f"r{i}": tokens(self.cfg["vocab"], n, 50 + i) for i, n in enumerate(lengths)}
        self.want, self.clear = {}, {}
        for rid, toks in self.requests.items():
            margins = []
            self.want[rid] = plain.forward(self.cfg, self.weights, toks, margins=margins)
            closest = np.min(margins, axis=0) if margins else np.full(len(toks), np.inf)
            if dtype == "float32":
                self.clear[rid] = closest >= 1e-5
            else:
                # In bfloat16 a router's choice between two nearly equal scores is an accident of rounding,
                # and a flipped choice reaches every later token through the state and the attention: only
                # the positions before the first unclear choice are held to the plain model.
                unclear = np.flatnonzero(closest < ROUTER_MARGIN)
                self.clear[rid] = np.arange(len(toks)) < (unclear[0] if len(unclear) else len(toks))
        self.dtype = dtype
        self.bound = F32_BOUND if dtype == "float32" else BF16_BOUND

    def runner(self, page_size=16, num_pages=40, max_requests=3):
        from pylon_amd.engine import Runner

        return Runner.from_folder(self.folder, dtype=self.dtype, page_size=page_size, num_pages=num_pages,
                                  max_requests=max_requests)

    def check(self, rid, got, label):
        clear = self.clear[rid][: len(got)]
        assert np.isfinite(got).all()
        if not clear.any():
            return
        got, want = got[clear], self.want[rid][: len(got)][clear]
        if self.dtype == "float32":
            ok, worst, frac = rows_within(got, want, self.bound)
            assert ok, f"{label}: request {rid}, position {np.flatnonzero(clear)[worst]} is off by {frac:.2e} of its largest logit"
            return
        # bfloat16: the stream that a deep layer's router reads has been rounded many times, and a choice
        # that looked clear in the plain model may still fall the other way; such a position, and a few
        # that look back at it, are further off than rounding alone explains.  One position in twenty-five
        # may be, none by more than six times the bound.
        off = np.abs(got - want).max(axis=1) / np.abs(want).max(axis=1)
        assert off.max() <= 6 * self.bound, f"{label}: request {rid}, position {np.flatnonzero(clear)[off.argmax()]} is off by {off.max():.2e}"
        assert (off > self.bound).sum() <= max(1, len(off) // 25), \
            f"{label}: request {rid}: {(off > self.bound).sum()} of {len(off)} positions are off by more than {self.bound}"

    def compared(self):
        return sum(int(c.sum()) for c in self.clear.values())


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


@pytest.mark.parametrize("name, page", [("A", 16), ("B", 64), ("C", 16), ("D", 32)])
def test_the_stream_after_every_layer(tmp, name, page):
    """The residual stream after every layer, in float32, for a whole prompt and in two portions."""
    from pylon_amd.engine import StepEntry

    case = Case(tmp, name, "float32", (45,))
    runner = case.runner(page_size=page, num_pages=8)
    kept = []

    def watch(norm):
        def wrapped(resid, delta, *, row_idx=None, inner=norm.add_forward):
            out = inner(resid, delta, row_idx=row_idx)
            if row_idx is None:
                kept.append(resid.cpu().numpy().copy())  # the norm's kernel has left the sum there
            else:
                from pylon_amd.parts.base import summed
                kept.append((resid + summed(delta)).cpu().numpy())
            return out
        norm.add_forward = wrapped

    for block in runner.model.blocks[1:]:
        watch(block.mixer_norm)
    watch(runner.model.final_norm)
    toks = case.requests["r0"]
    want = []
    plain.forward(case.cfg, case.weights, toks, streams=want)
    seq = runner.open("a")
    runner.step([StepEntry(seq, toks, list(range(len(toks))))])
    runner.close(seq)
    assert len(kept) == len(want) == len(case.cfg["layers"])
    for layer, (got, ref) in enumerate(zip(kept, want)):
        assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max(), f"layer {layer}"
    kept.clear()
    seq = runner.open("b")
    runner.step([StepEntry(seq, toks[:19], list(range(19)))])
    runner.step([StepEntry(seq, toks[19:], list(range(len(toks) - 19)))])
    for layer, ref in enumerate(want):
        got = np.concatenate([kept[layer], kept[len(want) + layer]])
        assert np.abs(got - ref).max() <= 1e-4 * np.abs(ref).max(), f"layer {layer}, two portions"


@pytest.mark.parametrize("name, dtype, page", [("A", "float32", 16), ("B", "float32", 16), ("C", "float32", 16),
                                                ("D", "float32", 32), ("A", "bfloat16", 16), ("B", "bfloat16", 64),
                                                ("B", "bfloat16", 32), ("C", "bfloat16", 64), ("D", "bfloat16", 64),
                                                ("C", "float32", 64), ("E", "float32", 64), ("E", "bfloat16", 64)])
def test_whole_token_by_token_and_in_portions(tmp, name, dtype, page):
    """Pages of 16 tokens run the general attention kernel everywhere; with pages of 32 and 64 the
    left mixers with heads of 64 or 128 run on the matrix cores."""
    case = Case(tmp, name, dtype, (71, 38))
    assert case.compared() >= 100
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


@pytest.mark.parametrize("name, dtype, page", [("A", "float32", 16), ("B", "float32", 16), ("D", "float32", 16),
                                                ("C", "bfloat16", 16), ("B", "bfloat16", 32), ("D", "bfloat16", 64)])
def test_mixed_batches_over_pages_and_slots_that_are_used_again(tmp, name, dtype, page):
    case = Case(tmp, name, dtype, (60, 45, 33, 20))
    pages = {16: 9, 32: 6, 64: 4}[page]  # never room for all four requests at once
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


@pytest.mark.parametrize("name, dtype", [("B", "float32"), ("B", "bfloat16"), ("A", "float32")])
def test_long_decoding_after_a_prompt(tmp, name, dtype):
    """420 tokens, 320 of them one by one: the state goes through hundreds of single steps, chunks of
    50 and 128 positions (or 7 and 5) pass by, and the pages a chunk has left go back."""
    case = Case(tmp, name, dtype, (420,))
    runner = case.runner(page_size=64, num_pages=7, max_requests=2)
    got, _ = run_plan(runner, case, [{"r0": 100}] + [{"r0": 1}] * 320)
    case.check("r0", got["r0"], "long decoding")
    assert runner.manager.free_pages == 7


def test_requests_do_not_see_what_a_freed_slot_or_page_held(tmp):
    """The same request, alone in a fresh runner and after others have used every page and slot."""
    case = Case(tmp, "A", "float32", (50, 64, 64))
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
    """Position 0 sees itself alone, its convolution reads zeros and its state starts empty: its
    logits are those of a one-token request, whatever follows it and whatever ran in its slot before."""
    case = Case(tmp, "D", "float32", (9, 30))
    runner = case.runner(num_pages=8, max_requests=1)
    first, _ = run_plan(runner, case, [{"r1": 30}, {"r1": 0}, {"r0": 1}])
    want = plain.forward(case.cfg, case.weights, case.requests["r0"][:1])
    assert np.abs(first["r0"] - want).max() <= F32_BOUND * np.abs(want).max()
    two, _ = run_plan(runner, case, [{"r0": 2}])
    assert np.abs(two["r0"] - case.want["r0"][:2]).max() <= F32_BOUND * np.abs(want).max()


def test_a_long_request_whole_and_with_its_tail_decoded(tmp):
    """700 tokens over eleven pages of 64: the left mixer looks back over all of them, the state has
    gone through all of them."""
    case = Case(tmp, "C", "float32", (700,))
    runner = case.runner(page_size=64, num_pages=12, max_requests=1)
    whole, _ = run_plan(runner, case, [{"r0": 700}])
    case.check("r0", whole["r0"], "whole")
    tail, _ = run_plan(runner, case, [{"r0": 650}] + [{"r0": 1}] * 50)
    case.check("r0", tail["r0"], "tail decoded")


@pytest.mark.parametrize("name, dtype, graphs, page", [("A", "float32", False, 16), ("B", "float32", True, 16),
                                                         ("C", "bfloat16", True, 64), ("B", "bfloat16", True, 32),
                                                         ("D", "bfloat16", True, 64)])
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
            margins = []
            row = plain.forward(cfg, weights, sequence, margins=margins)[-1]
            if dtype != "float32" and margins and np.min(margins) < ROUTER_MARGIN:
                break  # a router's close call somewhere before: from here on rounding decides
            assert produced == int(row.argmax()) or row.max() - row[produced] <= slack * np.abs(row).max(), \
                (prompt[:3], result.output_ids)
            sequence.append(produced)


@pytest.mark.parametrize("name, dtype", [("B", "float32"), ("D", "float32"), ("B", "bfloat16")])
def test_the_replay_program_as_a_user_runs_it(tmp, tmp_path, name, dtype):
    """``bin/trace_run`` as a subprocess over pages of 64 and four slots: up to four live requests,
    portions of some beside single tokens of others, pages and slots used again; the logits files
    against the plain model."""
    import json
    import os
    import subprocess
    import sys
    from pathlib import Path

    from tests import traces

    root = Path(__file__).resolve().parent.parent
    case = Case(tmp, name, dtype, (5, 90, 64, 33, 70, 1), seed=11)
    steps = traces.mixed(case.requests, seed=7)
    out = tmp_path / "out"
    proc = subprocess.Popen(
        [sys.executable, str(root / "bin" / "trace_run"), "--model", str(case.folder), "--dtype", dtype,
         "--out", str(out), "--max-tokens", str(traces.peak_tokens(steps))],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, cwd=str(tmp_path),
        env=dict(os.environ, PYTHONUNBUFFERED="1"))
    try:
        for step in steps:
            proc.stdin.write(json.dumps(step) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {step['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    vocab = case.cfg["vocab"]
    outputs = {}
    for step in steps:
        wanted = sum(len(e["want"]) for e in step["entries"])
        if wanted:
            outputs[step["step"]] = np.fromfile(out / f"{step['step']}.f32", dtype="<f4").reshape(wanted, vocab)
    got = traces.collect(steps, outputs, vocab)
    for rid in case.requests:
        assert len(got[rid]) == len(case.requests[rid])
        case.check(rid, np.asarray(got[rid]), "replayed")


def draw_config(seed: int):
    """A configuration drawn over what config.json allows: layers in any order, heads and sizes in
    steps of 8 and a few odd ones, chunks that are no multiple of anything, with and without
    stretched frequencies, caps, feed-forwards."""
    rng = np.random.default_rng(7000 + seed)
    width = int(rng.choice([48, 64, 96, 136, 160, 256]))

    def rot(dim, scaled):
        if rng.random() < 0.15:
            return None
        dims = int(rng.choice([d for d in (2, 4, 8, 16, 32, 64, 128, dim) if d <= dim and d % 2 == 0]))
        out = {"base": float(rng.choice([100.0, 1.0e4, 5.0e5, 1.0e6])), "dims": dims}
        if scaled and rng.random() < 0.7:
            out["scaling"] = {"factor": float(rng.choice([2.0, 8.0, 32.0])), "original": float(rng.choice([16, 64, 2048])),
                              "fast": float(rng.choice([4.0, 32.0])), "slow": float(rng.choice([1.0, 2.0]))}
        return out

    layers = []
    for _ in range(int(rng.integers(2, 6))):
        if rng.random() < 0.5:
            kv_heads = int(rng.integers(1, 4))
            dim = int(rng.choice([8, 16, 24, 32, 40, 64, 96, 128, 12]))
            m = {"heads": kv_heads * int(rng.choice([1, 2, 3, 4, 8])), "kv_heads": kv_heads, "dim": dim,
                 "vdim": int(rng.choice([4, 8, 20, 32, 48, 64, 80, 128, 10])), "scale": float(rng.uniform(0.05, 0.4)),
                 "mask": {"size": int(rng.choice([int(rng.integers(3, 200)), 32, 64, 128, 1000]))},
                 "softcap": float(rng.choice([2.0, 15.0, 50.0]))}
            r = rot(dim, True)
            if r is not None:
                m["rot"] = r
            kind = "attention"
        else:
            kv_heads = int(rng.integers(1, 3))
            dim = int(rng.choice([16, 24, 64, 128, 12, 32]))
            left = {"heads": kv_heads * int(rng.choice([1, 2, 4])), "kv_heads": kv_heads, "dim": dim, "vdim": dim,
                    "scale": float(rng.uniform(0.05, 0.3))}
            r = rot(dim, False)
            if r is not None:
                left["rot"] = r
            qk_heads = int(rng.integers(1, 3))
            right = {"heads": qk_heads * int(rng.choice([1, 2, 3])), "kv_heads": qk_heads,
                     "dim": int(rng.choice([8, 20, 32, 64, 128])), "vdim": int(rng.choice([8, 12, 32, 64, 128])),
                     "conv": int(rng.integers(1, 6))}
            m = {"left": left, "right": right, "left_scale": float(rng.uniform(0.3, 1.5)),
                 "right_scale": float(rng.uniform(0.3, 1.5))}
            kind = "parallel"
        mlp = None
        if rng.random() > 0.15:
            experts = int(rng.integers(1, 12))
            mlp = {"kind": "moe", "expert": {"ff": 8 * int(rng.integers(1, 12))},
                   "router": {"experts": experts, "top": int(rng.integers(1, min(experts, 4) + 1))}}
        layers.append({"type": kind, "mixer": m, "mlp": mlp})
    config = {"architecture": "Tukarax", "vocab": int(rng.integers(90, 700)), "width": width,
              "norm": {"eps": float(10 ** rng.uniform(-7, -4))}, "layers": layers}
    return config, (int(rng.integers(1, 40)), int(rng.integers(60, 200)), int(rng.integers(200, 330)))


@pytest.mark.parametrize("seed, dtype", [(seed, "float32") for seed in range(8)] + [(seed, "bfloat16") for seed in range(4)])
def test_a_configuration_drawn_at_random_matches_the_plain_model(tmp, seed, dtype):
    """Pages of 64 and four slots: each request whole, the longest with its tail token by token, then
    all three side by side in portions over a pool too small for them to have pages to spare."""
    config, lengths = draw_config(seed)
    if dtype != "float32":
        # shorter requests, drawn token by token so that every position's routing is clear
        lengths = (lengths[0], min(lengths[1], 70), min(lengths[2], 100))
    case = Case(tmp, f"drawn{seed}", dtype, lengths, seed=seed, config=config, pick=dtype != "float32")
    if case.compared() < 40:
        pytest.skip("too few positions with clear routing in this draw")
    pages = sum(-(-n // 64) for n in lengths)
    runner = case.runner(page_size=64, num_pages=pages, max_requests=4)
    whole, _ = run_plan(runner, case, [{"r0": lengths[0]}, {"r0": 0, "r1": lengths[1]}, {"r1": 0, "r2": lengths[2]}])
    for rid, got in whole.items():
        case.check(rid, got, f"whole (seed {seed})")
    tail, _ = run_plan(runner, case, [{"r2": lengths[2] - 70}] + [{"r2": 1}] * 70)
    assert len(tail["r2"]) == lengths[2]
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
