"""Tukarax on the CPU: its configuration, its specs, its tensors, what its runs ask of the
cache manager, and the plain implementation held to a few closed forms."""
import copy
import math

import numpy as np
import pytest
import torch

from tests.plain import tukarax as plain
from tests.tukarax_helpers import CONFIGS, TUKARAX_A, TUKARAX_B, TUKARAX_D, make_folder, read_folder


def test_config_json_selects_the_architecture_and_round_trips():
    from pylon_amd.config.registry import resolve

    for raw in CONFIGS.values():
        arch = resolve(raw)
        assert arch.name == "Tukarax"
        cfg = arch.parse_config(raw)
        assert arch.parse_config(arch.config_to_json(cfg)) == cfg
    cfg = resolve(TUKARAX_A).parse_config(TUKARAX_A)
    assert cfg.layers[1].mlp is None and cfg.layers[0].mlp.top == 2 and cfg.layers[0].mlp.experts == 5
    assert cfg.layers[0].mixer.right.conv == 2 and cfg.layers[0].mixer.left_scale == 0.7
    assert cfg.layers[1].mixer.rot.scaling == (4.0, 16.0, 4.0, 1.0) and cfg.layers[1].mixer.softcap == 3.0
    assert cfg.layers[3].mixer.left.rot is None and cfg.layers[2].mixer.softcap is None


def test_layers_become_specs_of_parts_that_other_designs_can_use():
    from pylon_amd.config.registry import resolve
    from pylon_amd.config.specs import AttentionSpec, DeltaRuleSpec, ParallelMixerSpec

    arch = resolve(TUKARAX_A)
    spec = arch.model_spec(arch.parse_config(TUKARAX_A))
    assert [(e.layer, e.cache) for e in spec.schedule] == [(0, None), (1, None), (2, None), (3, None)]
    first = spec.layers[0].mixer
    assert isinstance(first, ParallelMixerSpec) and (first.left_scale, first.right_scale) == (0.7, 1.6)
    left, right = first.left, first.right
    assert isinstance(left, AttentionSpec) and left.values_from_keys and left.output_gate == "element"
    assert left.qk_norm and left.qk_norm_over == "head" and left.qk_norm_eps == 2e-5 and left.position.interleaved
    assert not left.sink and left.softcap is None and left.chunk is None and left.gate_size == 4 * 12
    assert isinstance(right, DeltaRuleSpec) and (right.n_heads, right.n_kv_heads, right.head_dim, right.v_head_dim,
                                                 right.conv_taps, right.norm_eps) == (4, 2, 12, 20, 2, 2e-5)
    att = spec.layers[1].mixer
    assert (att.n_heads, att.n_kv_heads, att.head_dim, att.value_dim, att.scale, att.chunk, att.softcap) == \
        (4, 2, 12, 20, 0.4, 7, 3.0)
    assert att.sink and att.output_gate == "head" and att.gate_size == 4 and not att.position.interleaved
    assert att.position.scaling.factor == 4.0 and not att.qk_norm
    ff = spec.layers[0].feed_forward
    assert (ff.scoring, ff.weight_on_input, ff.n_experts, ff.top, ff.expert_size, ff.router_bias) == \
        ("sigmoid", True, 5, 2, 16, False)
    assert spec.layers[1].feed_forward is None and spec.layers[1].feed_forward_norm is None
    assert spec.layers[3].mixer.left.position.kind == "none"


def _changed(path, value):
    def change(raw):
        node = raw
        for key in path[:-1]:
            node = node[key]
        if value is KeyError:
            del node[path[-1]]
        else:
            node[path[-1]] = value
    return change


@pytest.mark.parametrize("change, message", [
    (_changed(("layers", 0, "type"), "retention"), "unknown layer type"),
    (_changed(("layers", 1, "mixer", "kv_heads"), 3), "divisible"),
    (_changed(("layers", 0, "mixer", "right", "kv_heads"), 3), "divisible"),
    (_changed(("layers", 0, "mixer", "left", "vdim"), 16), "the values are the keys"),
    (_changed(("layers", 0, "mixer", "left", "softcap"), 5.0), "caps no score"),
    (_changed(("layers", 1, "mixer", "rot", "dims"), 14), "rot.dims"),
    (_changed(("layers", 1, "mixer", "rot", "dims"), 5), "rot.dims"),
    (_changed(("layers", 1, "mixer", "rot", "scaling", "slow"), KeyError), "lacks required keys"),
    (_changed(("layers", 0, "mlp", "router", "top"), 6), "exceeds"),
    (_changed(("layers", 0, "mlp", "kind"), "dense"), "unknown feed-forward kind"),
    (_changed(("layers", 0, "mixer", "right", "conv"), KeyError), "lacks required keys"),
    (_changed(("norm",), KeyError), "lacks required keys"),
    (_changed(("layers",), []), "no layers"),
])
def test_bad_configurations_are_refused(change, message):
    from pylon_amd.config.registry import resolve

    raw = copy.deepcopy(TUKARAX_A)
    change(raw)
    with pytest.raises(ValueError, match=message):
        resolve(raw).parse_config(raw)


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_a_written_folder_loads_into_every_parameter(tmp_path, name):
    from pylon_amd.config.registry import load_model_config
    from pylon_amd.engine.model import Model
    from pylon_amd.weights.loader import load_weights

    folder = make_folder(tmp_path, name)
    arch, cfg = load_model_config(folder)
    model = Model(arch.model_spec(cfg), dtype=torch.float32, device="cpu")
    for _path, owner, pname in model.named_params():
        owner.params[pname].fill_(float("nan"))
    assert load_weights(model, arch, cfg, folder, strict=True) == []
    for path, owner, pname in model.named_params():
        assert not torch.isnan(owner.params[pname]).any(), path
    _cfg, weights = read_folder(folder)
    if name == "A":
        same = lambda tensor, name: np.array_equal(tensor.numpy(), weights[name].astype(np.float32))  # noqa: E731
        side = model.blocks[0].mixer
        assert side.left.params["qkv"].shape == (48 + 24 + 48, 40)  # q, k, the gate: no value projection
        assert same(side.left.params["qkv"][48: 72], "l0.mix.left.k") and same(side.left.params["qkv"][72:], "l0.mix.left.g")
        assert same(side.left.params["q_norm"], "l0.mix.left.q.norm") and side.left.params["k_norm"].shape == (12,)
        right = side.right
        assert right.params["proj"].shape == (24 + 24 + 80 + 80 + 4 + 4, 40) and right.params["conv"].shape == (128, 2)
        assert same(right.params["proj"][48: 128], "l0.mix.right.v") and same(right.params["proj"][128: 208], "l0.mix.right.g")
        assert same(right.params["proj"][208: 212], "l0.mix.right.b") and same(right.params["proj"][212:], "l0.mix.right.a")
        assert same(right.params["conv"][24: 48], "l0.mix.right.k.conv") and same(right.params["a_log"], "l0.mix.right.A_log")
        att = model.blocks[1].mixer
        assert att.params["qkv"].shape == (48 + 24 + 40 + 4, 40) and same(att.params["qkv"][112:], "l1.mix.g")
        assert same(att.params["sink"], "l1.mix.sink") and same(att.params["qkv"][72: 112], "l1.mix.v")
        ff = model.blocks[0].feed_forward
        assert ff.params["router"].shape == (5, 40) and "router_bias" not in ff.params
        assert same(ff.params["gate_up"][3 * 32 + 16: 4 * 32], "l0.mlp.e3.up") and same(ff.params["down"][80: 120], "l0.mlp.e2.down")
        assert model.blocks[1].feed_forward is None


def test_a_folder_that_lacks_a_tensor_or_holds_one_too_many_is_refused(tmp_path):
    from safetensors.torch import load_file, save_file

    from pylon_amd.config.registry import load_model_config
    from pylon_amd.engine.model import Model
    from pylon_amd.weights.loader import WeightsError, load_weights

    folder = make_folder(tmp_path, "A")
    arch, cfg = load_model_config(folder)
    tensors = load_file(str(folder / "model.safetensors"))
    assert "l0.mix.left.v" not in tensors and "l1.norm2" not in tensors and "l3.mix.left.q.norm" in tensors
    sink = tensors.pop("l1.mix.sink")
    tensors["l0.mix.left.v"] = sink
    save_file(tensors, str(folder / "model.safetensors"))
    model = Model(arch.model_spec(cfg), dtype=torch.float32, device="cpu")
    with pytest.raises(WeightsError) as error:
        load_weights(model, arch, cfg, folder, strict=True)
    assert "l1.mix.sink" in str(error.value) and "l0.mix.left.v" in str(error.value)


def test_runs_ask_for_keys_values_a_state_and_a_window_of_the_convolution():
    from pylon_amd.cache.manager import CacheManager
    from pylon_amd.config.registry import resolve
    from pylon_amd.engine.model import Model
    from pylon_amd.parts.base import KVRequirement, StateRequirement

    arch = resolve(TUKARAX_D)
    model = Model(arch.model_spec(arch.parse_config(TUKARAX_D)), dtype=torch.float32, device="cpu")
    needs = model.cache_requirements()
    # a convolution of one tap keeps no window; the state is kept transposed (a column of S contiguous)
    assert needs[0] == (KVRequirement(2, 24), StateRequirement((2, 64, 256), torch.float32, name="delta"))
    assert needs[1] == KVRequirement(2, 40, None, v_head_dim=72, chunk=64)
    assert needs[2] == (KVRequirement(2, 128), StateRequirement((3, 24, 40), torch.float32, name="delta"),
                        StateRequirement((7, 2 * 3 * 40 + 3 * 24), torch.float32, name="delta_conv"))
    manager = CacheManager(needs, dtype=torch.float32, page_size=16, num_pages=6, max_requests=2, device="cpu")
    seq = manager.open("a")
    assert set(manager.view(2).states) == {"delta", "delta_conv"} and set(manager.view(0).states) == {"delta"}
    # a slot that is handed out again starts from zeros
    for tensor in manager.slots.tensors.values():
        tensor.fill_(7.0)
    manager.close(seq)
    again = manager.open("b")
    for key, tensor in manager.slots.tensors.items():
        assert float(tensor[again.slot].abs().max()) == 0.0, key


def test_the_chunked_layer_gives_back_the_pages_its_chunk_has_left():
    from pylon_amd.parts.base import KVRequirement

    need = KVRequirement(2, 40, None, v_head_dim=72, chunk=64)
    assert need.bounded and need.span == 64
    assert [need.first_needed(n) for n in (0, 63, 64, 65, 200)] == [0, 0, 64, 64, 192]


def test_stretched_frequencies_follow_the_ramp_between_fast_and_slow_pairs():
    from pylon_amd.config.specs import PositionSpec, RotaryScalingSpec
    from pylon_amd.parts.position import scaled_frequencies

    for base, dims, scaling in ((1.0e6, 32, (8.0, 64, 16.0, 2.0)), (5000.0, 12, (4.0, 16, 4.0, 1.0)),
                                (1.0e4, 8, (2.0, 32, 8.0, 1.0)), (1.0e4, 64, (40.0, 4096, 32.0, 1.0)), (50.0, 6, (1.0, 8, 2.0, 1.0))):
        spec = PositionSpec(kind="rope", theta=base, rotary_dim=dims, scaling=RotaryScalingSpec(*scaling))
        freq, factor = scaled_frequencies(spec)
        want, want_factor = plain.rotary_frequencies({"base": base, "dims": dims, "scaling": dict(zip(
            ("factor", "original", "fast", "slow"), scaling))})
        assert np.allclose(freq.double().numpy(), want, rtol=1e-6, atol=0.0) and abs(factor - want_factor) < 1e-12
    # by hand: base 16, four pairs, original length 2 pi * 16: pair i makes 16 / 16^(i/4) = 16, 8, 4, 2 turns;
    # fast 8 -> lo = 1, slow 2 -> hi = 3: pair 0 and 1 as they are, pair 2 half-way, pair 3 stretched
    got, factor = plain.rotary_frequencies({"base": 16.0, "dims": 8, "scaling": {"factor": 4.0, "original": 2 * math.pi * 16,
                                                                                 "fast": 8.0, "slow": 2.0}})
    f = 16.0 ** (-np.arange(4) / 4.0)
    assert np.allclose(got, [f[0], f[1], f[2] * (0.5 / 4 + 0.5), f[3] / 4]) and abs(factor - (0.1 * math.log(4.0) + 1)) < 1e-12


def test_plain_rotation_pairs_halves_or_neighbours_and_leaves_the_rest():
    x = np.arange(2 * 1 * 6, dtype=np.float64).reshape(2, 1, 6) + 1.0
    rot = {"base": 100.0, "dims": 4}
    halves, neighbours = plain.rotate(x, rot, False), plain.rotate(x, rot, True)
    assert np.array_equal(halves[0], x[0]) and np.array_equal(neighbours[..., 4:], x[..., 4:])  # position 0; beyond dims
    a0, a1 = 1.0, 100.0 ** -0.5  # position 1 times the two frequencies
    u, v = x[1, 0, 0], x[1, 0, 2]
    assert np.allclose(halves[1, 0, [0, 2]], [u * math.cos(a0) - v * math.sin(a0), v * math.cos(a0) + u * math.sin(a0)])
    u, v = x[1, 0, 2], x[1, 0, 3]
    assert np.allclose(neighbours[1, 0, [2, 3]], [u * math.cos(a1) - v * math.sin(a1), v * math.cos(a1) + u * math.sin(a1)])


def test_plain_mask_counts_chunks_from_position_zero():
    seen = plain.visible(7, 3)
    assert seen[5].tolist() == [False, False, False, True, True, True, False]
    assert seen[3].tolist() == [False, False, False, True, False, False, False]
    assert plain.visible(4, None)[3].all()


def test_plain_softmax_with_a_sink_and_a_cap():
    q = np.zeros((1, 1, 2))
    k = np.ones((1, 1, 2))
    v = np.full((1, 1, 3), 5.0)
    # one key of score 0 and a sink of ln 3: the key keeps a quarter of the weight
    out = plain.softmax_attention(q, k, v, 1.0, plain.visible(1, None), None, np.array([math.log(3.0)]))
    assert np.allclose(out, 1.25)
    # two keys with scores 100 and 0 capped at 1: weights e^tanh(100) : e^0
    q = np.array([[[0.0]], [[10.0]]])
    k = np.array([[[0.0]], [[10.0]]])
    v = np.array([[[0.0]], [[1.0]]])
    out = plain.softmax_attention(q, k, v, 1.0, plain.visible(2, None), 1.0, None)
    assert np.allclose(out[1, 0, 0], math.e / (math.e + 1.0), rtol=1e-9)


def test_plain_delta_rule_writes_before_it_reads_and_forgets_by_its_decay():
    # one head, dim 2, vdim 1: with beta 1 and unit keys the state answers a key with its value
    q = np.array([[[1.0, 0.0]], [[1.0, 0.0]], [[0.0, 1.0]]])
    k = np.array([[[1.0, 0.0]], [[0.0, 1.0]], [[1.0, 0.0]]])
    v = np.array([[[3.0]], [[5.0]], [[7.0]]])
    ones = np.ones((3, 1))
    out = plain.delta_rule(q, k, v, ones, ones)
    assert np.allclose(out[:, 0, 0], [3.0, 3.0, 5.0])  # the first read-out sees the first write
    half = plain.delta_rule(q, k, v, ones, 0.5 * ones)
    assert np.allclose(half[:, 0, 0], [3.0, 1.5, 2.5])
    # beta 0.5 moves the stored value half-way towards the new one
    again = plain.delta_rule(q[:2] * 0 + [1.0, 0.0], k[:2] * 0 + [1.0, 0.0], v[:2], 0.5 * ones[:2], ones[:2])
    assert np.allclose(again[:, 0, 0], [1.5, 1.5 + 0.5 * (5.0 - 1.5)])


def test_plain_convolution_weighs_the_current_token_with_its_last_tap():
    x = np.array([[1.0], [10.0], [100.0]])
    assert np.allclose(plain.causal_conv(x, np.array([[0.0, 0.0, 2.0]]))[:, 0], [2.0, 20.0, 200.0])
    assert np.allclose(plain.causal_conv(x, np.array([[3.0, 0.0, 0.0]]))[:, 0], [0.0, 0.0, 3.0])


def test_plain_experts_run_on_their_weighted_inputs():
    rng = np.random.default_rng(0)
    h = rng.normal(size=(3, 4))
    w = {"router": np.array([[5.0, 0, 0, 0], [0, 5.0, 0, 0], [0, 0, 0, 0.0]])}
    for e in range(3):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = rng.normal(size=(2, 4)), rng.normal(size=(2, 4)), rng.normal(size=(4, 2))
    chosen, weights, margin = plain.route(h, w["router"], 2)
    scores = plain.sigmoid(h @ w["router"].T)
    for t in range(3):
        assert set(chosen[t]) == set(np.argsort(-scores[t])[:2]) and np.allclose(weights[t], np.sort(scores[t])[::-1][:2])
    assert (margin > 0).all() and weights.sum(axis=1).max() > 1.0  # not renormalised
    out = plain.mixture(h, {"router": {"top": 2}}, w, "")
    t = 0
    want = sum(w[f"e{e}.down"] @ (plain.silu(w[f"e{e}.gate"] @ (a * h[t])) * (w[f"e{e}.up"] @ (a * h[t])))
               for e, a in zip(chosen[t], weights[t]))
    assert np.allclose(out[t], want)


def test_plain_forward_in_two_cuts_agrees_on_the_common_positions(tmp_path):
    folder = make_folder(tmp_path, "A")
    cfg, weights = read_folder(folder)
    toks = list(range(3, 40))
    whole = plain.forward(cfg, weights, toks)
    assert np.allclose(plain.forward(cfg, weights, toks[:21]), whole[:21], atol=1e-9)
    streams = []
    plain.forward(cfg, weights, toks, streams=streams)
    assert len(streams) == len(cfg["layers"]) and streams[0].shape == (len(toks), cfg["width"])
    for name in ("B",):
        cfg, weights = read_folder(make_folder(tmp_path, name))
        assert np.isfinite(plain.forward(cfg, weights, toks)).all()
    assert TUKARAX_B["layers"][1]["mixer"]["right"]["heads"] == 4
