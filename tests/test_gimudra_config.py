"""Gimudra on the CPU: its configuration, its specs, its tensors, what its runs ask of the
cache manager, and the plain implementation held to a few closed forms."""
import copy
import math

import numpy as np
import pytest
import torch

from tests.gimudra_helpers import CONFIGS, GIMUDRA_P, GIMUDRA_Q, GIMUDRA_R, make_folder, read_folder
from tests.plain import gimudra as plain


def test_config_json_selects_the_architecture_and_round_trips():
    from pylon_amd.config.registry import resolve

    for raw in CONFIGS.values():
        arch = resolve(raw)
        assert arch.name == "Gimudra"
        cfg = arch.parse_config(raw)
        assert arch.parse_config(arch.config_to_json(cfg)) == cfg
    cfg = resolve(GIMUDRA_P).parse_config(GIMUDRA_P)
    assert cfg.layers[1].mixer.kv_from == 0 and cfg.layers[2].mlp is None and cfg.layers[0].mlp.ff == 24
    assert (cfg.layers[1].mlp.experts, cfg.layers[1].mlp.identity, cfg.layers[1].mlp.groups,
            cfg.layers[1].mlp.groups_kept, cfg.layers[1].mlp.scale) == (5, 1, 3, 2, 1.5)


def test_layers_become_specs_and_a_schedule_that_borrows_keys_and_values():
    from pylon_amd.config.registry import resolve

    arch = resolve(GIMUDRA_P)
    spec = arch.model_spec(arch.parse_config(GIMUDRA_P))
    assert [(e.layer, e.cache) for e in spec.schedule] == [(0, None), (1, 0), (2, None), (3, 0)]
    assert [layer.mixer.own_kv for layer in spec.layers] == [True, False, True, False]
    # layers 0, 1 and 3 read one cache with chunks of 7 and of 9: it keeps every token; layer 2's own does not
    assert [layer.mixer.cache_bounded for layer in spec.layers] == [False, False, True, False]
    att = spec.layers[1].mixer
    assert (att.n_heads, att.n_kv_heads, att.head_dim, att.v_head_dim, att.scale, att.chunk) == (4, 2, 12, 20, 0.4, 7)
    assert att.bias_form == "log" and att.qkv_bias and not att.sink and att.window is None
    assert [layer.depth_mix for layer in spec.layers] == [(1, 5), (2, 5), (3, 5), (4, 5)]
    assert all(layer.sublayer_scale and layer.input_conv.kind == "token_shift" for layer in spec.layers)
    assert spec.layers[2].feed_forward is None and spec.layers[2].feed_forward_norm is None
    assert spec.layers[0].feed_forward.bias and spec.layers[0].feed_forward.intermediate_size == 24
    moe = spec.layers[1].feed_forward
    assert (moe.n_experts, moe.n_identity, moe.top, moe.groups, moe.groups_kept, moe.route_scale) == (5, 1, 2, 3, 2, 1.5)
    assert moe.expert_act == "relu2" and moe.scoring == "softmax_all" and moe.shared_size is None
    assert spec.embedding_scale == 1.7 and spec.stream_parts[0].kind == "sinusoid" and not spec.tie_word_embeddings
    # layers of Q that share a cache all have its chunks: the cache lets go what a chunk has left behind
    spec_q = arch.model_spec(arch.parse_config(GIMUDRA_Q))
    assert all(layer.mixer.cache_bounded for layer in spec_q.layers)
    spec_r = arch.model_spec(arch.parse_config(GIMUDRA_R))
    assert spec_r.layers[0].mixer.chunk is None and spec_r.layers[1].mixer.chunk == 1000


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][1]["mixer"].update(kv_from=1), "earlier layer"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=1), "no keys and values of its own"),
    (lambda c: c["layers"][3]["mixer"].update(vdim=24), "heads differ"),
    (lambda c: c["layers"][0].update(type="window"), "unknown layer type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "divisible"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "lacks required keys"),
    (lambda c: c.pop("norm"), "lacks required keys"),
    (lambda c: c["layers"][1]["mlp"].update(kind="routed"), "feed-forward kind"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "exceeds"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(groups={"count": 4, "keep": 2}), "equal groups"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(groups={"count": 3, "keep": 4}), "equal groups"),
    (lambda c: c["layers"][0]["mixer"].update(mask={"size": 0}), "positive integer"),
    (lambda c: c.update(layers=[]), "no layers"),
])
def test_bad_configurations_are_refused(change, message):
    from pylon_amd.config.registry import resolve

    config = copy.deepcopy(GIMUDRA_P)
    change(config)
    with pytest.raises(ValueError, match=message):
        resolve(config).parse_config(config)


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
    if name == "P":
        first, second = model.blocks[0], model.blocks[1]
        assert np.array_equal(first.mixer.params["qkv"][:48].numpy(), weights["l0.mix.q"].astype(np.float32))
        assert np.array_equal(first.mixer.params["qkv"][48 + 24:].numpy(), weights["l0.mix.v"].astype(np.float32))
        assert np.array_equal(first.mixer.params["qkv_bias"][48: 48 + 24].numpy(), weights["l0.mix.k.b"].astype(np.float32))
        assert second.mixer.params["qkv"].shape == (48, 40) and second.mixer.params["qkv_bias"].shape == (48,)
        assert np.array_equal(second.mixer.params["log_bias"].numpy(),
                              np.concatenate([weights["l1.mix.r1"], weights["l1.mix.r2"]]).astype(np.float32))
        assert second.feed_forward.params["router"].shape == (6, 40) and second.feed_forward.params["router_bias"].shape == (6,)
        assert second.feed_forward.params["up"].shape == (5 * 16, 40) and second.feed_forward.params["down"].shape == (5 * 40, 16)
        assert np.array_equal(second.feed_forward.params["down"][3 * 40: 4 * 40].numpy(), weights["l1.mlp.e3.down"].astype(np.float32))
        assert [model.blocks[i].params["depth_coeff"].shape[0] for i in range(4)] == [2, 3, 4, 5]
        assert "feed_forward_scale" not in model.blocks[2].params and "mixer_scale" in model.blocks[2].params
        assert np.array_equal(first.input_conv.params["weight"].numpy(), weights["l0.shift"].astype(np.float32))


def test_a_folder_that_lacks_a_tensor_or_holds_one_too_many_is_refused(tmp_path):
    from safetensors.torch import load_file, save_file

    from pylon_amd.config.registry import load_model_config
    from pylon_amd.engine.model import Model
    from pylon_amd.weights.loader import load_weights

    folder = make_folder(tmp_path, "P")
    arch, cfg = load_model_config(folder)
    tensors = load_file(str(folder / "model.safetensors"))
    assert "l1.mix.k" not in tensors and "l2.norm2" not in tensors and "l2.ls2" not in tensors
    lost = dict(tensors)
    lost.pop("l1.mlp.correction")
    save_file(lost, str(folder / "model.safetensors"))
    model = Model(arch.model_spec(cfg), dtype=torch.float32, device="cpu")
    with pytest.raises(Exception, match="correction|router_bias"):
        load_weights(model, arch, cfg, folder, strict=True)


def test_runs_ask_for_keys_values_and_the_last_input_of_the_shift():
    from pylon_amd.cache import CacheManager
    from pylon_amd.config.registry import resolve
    from pylon_amd.engine.model import Model
    from pylon_amd.parts import KVRequirement, StateRequirement

    arch = resolve(GIMUDRA_P)
    model = Model(arch.model_spec(arch.parse_config(GIMUDRA_P)), dtype=torch.float32, device="cpu")
    needs = model.cache_requirements()
    shift = StateRequirement((40,), torch.float32, "shift")
    assert len(needs) == 4
    assert needs[0] == (KVRequirement(2, 12, None, v_head_dim=20), shift)  # read with two sizes of chunks: unbounded
    assert needs[1] == shift and needs[3] == shift  # borrowed keys and values, a shift of their own
    assert needs[2] == (KVRequirement(1, 10, None, v_head_dim=6, chunk=5), shift)
    manager = CacheManager(needs, page_size=16, num_pages=6, max_requests=2, dtype=torch.float32)
    view = manager.view(1)
    assert view.k is None and view.states["shift"].shape == (2, 40)
    assert manager.view(0).states["shift"].data_ptr() != view.states["shift"].data_ptr()
    # a slot that is handed out again starts from zero in every run's state
    seq = manager.open("a")
    for tensor in manager.slots.tensors.values():
        tensor[seq.slot].fill_(7.0)
    manager.close(seq)
    again = manager.open("b")
    assert again.slot == seq.slot
    assert all(float(tensor[again.slot].abs().max()) == 0.0 for tensor in manager.slots.tensors.values())
    manager.check()


# ---- the plain implementation against closed forms --------------------------------------------
def test_plain_position_vector_alternates_sine_and_cosine_of_one_angle():
    out = plain.sinusoid(3, 6)
    assert np.allclose(out[0], [0, 1, 0, 1, 0, 1])
    for i in range(3):
        angle = 2 * 10000.0 ** (-2 * i / 6)
        assert np.allclose(out[2, 2 * i: 2 * i + 2], [math.sin(angle), math.cos(angle)])
    odd = plain.sinusoid(2, 5)  # the last element of an odd width is a sine without its cosine
    assert np.allclose(odd[1, 4], math.sin(10000.0 ** (-4 / 5)))


def test_plain_token_shift_reads_the_previous_input_as_it_was():
    h = np.array([[1.0, 10.0], [2.0, 20.0], [4.0, 40.0]])
    out = plain.token_shift(h, np.array([0.5, 1.0]))
    assert np.array_equal(out, [[0.5, 0.0], [1.5, 10.0], [3.0, 20.0]])


def test_plain_mask_counts_chunks_from_position_zero():
    seen = plain.chunk_mask(7, 3)
    assert [int(r.sum()) for r in seen] == [1, 2, 3, 1, 2, 3, 1]
    assert seen[5, 3] and not seen[5, 2] and not seen[3, 2] and not seen[2, 3]
    assert [int(r.sum()) for r in plain.chunk_mask(4, None)] == [1, 2, 3, 4]


def test_plain_bias_by_distance_is_taken_off_and_grows_with_the_logarithm():
    bias = plain.distance_bias(np.array([2.0, 0.0]), np.array([0.5, 3.0]), 4)
    assert bias.shape == (2, 4, 4) and np.allclose(bias[1], 0.0) and np.allclose(np.diag(bias[0]), 0.0)
    assert np.allclose(bias[0, 3, 0], 2.0 * math.log(1 + 0.5 * 3)) and bias[0, 0, 3] == 0.0
    # two equal keys: the nearer one gets the larger weight, by exactly the bias
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 1, "scale": 1.0}
    zero = np.zeros((1, 2))
    weights = {"q": np.zeros((2, 2)), "q.b": np.zeros(2), "r1": np.array([1.0]), "r2": np.array([1.0]), "o": np.eye(1)}
    kv = (np.zeros((2, 1, 2)), np.array([[[1.0]], [[0.0]]]))
    out = plain.attention(np.vstack([zero, zero]), weights, "", m, kv)
    assert np.allclose(out[1, 0], 0.5 / (0.5 + 1.0))  # exp(-log 2) against exp(0)


def _router(experts, identity, top, count, keep, scale=1.0):
    return {"experts": experts, "identity": identity, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}}


def test_plain_router_chooses_by_corrected_scores_and_weighs_by_the_scores():
    z = np.log(np.array([[0.4, 0.3, 0.2, 0.1]]))
    weights = {"router": z, "correction": np.array([-0.35, 0.0, 0.0, 0.25])}
    chosen, w, gap = plain.route(np.array([[1.0]]), {"router": z.T, "correction": weights["correction"]}, "",
                                 _router(4, 0, 2, 1, 1, 2.0))
    assert chosen == [[3, 1]] and np.allclose(w, [[0.2, 0.6]]) and np.isclose(gap[0], 0.3 - 0.2)


def test_plain_router_bars_groups_although_their_corrected_scores_are_larger_than_negative_ones():
    # groups {0,1} {2,3} {4,5}: the corrected scores of group 0 are negative, yet it is among the two
    # best groups when group 1's best is lower still; a barred output never wins over a negative one
    z = np.log(np.array([[0.30, 0.05, 0.10, 0.15, 0.25, 0.15]]))
    correction = np.array([-0.5, -0.5, -0.9, -0.9, 0.0, 0.0])
    chosen, w, _ = plain.route(np.array([[1.0]]), {"router": z.T, "correction": correction}, "", _router(4, 2, 3, 3, 2))
    assert chosen == [[4, 5, 0]]  # 3 and 2 are barred (-0.75, -0.8 < -0.2), then 0 (-0.2) before 1 (-0.45)
    assert np.allclose(w, [[0.25, 0.15, 0.30]])


def test_plain_identity_experts_hand_on_their_input():
    h = np.array([[1.0, -2.0]])
    weights = {"router": np.array([[0.0, 0.0], [5.0, 0.0]]), "correction": np.zeros(2),
               "e0.up": np.ones((3, 2)), "e0.down": np.ones((2, 3))}
    mlp = {"router": _router(1, 1, 1, 1, 1, 3.0)}
    s = 1.0 / (1.0 + math.exp(-5.0))
    assert np.allclose(plain.mixture(h, weights, "", mlp), 3.0 * s * h)
    # and a plain expert squares what is above zero
    weights["router"] = np.array([[5.0, 0.0], [0.0, 0.0]])
    weights["e0.up"] = np.array([[1.0, 0.0], [0.0, 1.0], [2.0, 0.0]])
    assert np.allclose(plain.mixture(h, weights, "", mlp), 3.0 * s * np.array([5.0, 5.0]))


def test_plain_depth_mix_weighs_every_earlier_result():
    streams = [np.full((1, 2), 1.0), np.full((1, 2), 10.0), np.full((1, 2), 100.0)]
    assert np.array_equal(plain.depth_mix(streams, np.array([1.0, 2.0, 3.0])), [[321.0, 321.0]])


def test_plain_forward_in_two_cuts_agrees_on_the_common_positions(tmp_path):
    folder = make_folder(tmp_path, "P")
    cfg, weights = read_folder(folder)
    toks = list(np.random.default_rng(1).integers(0, cfg["vocab"], 30))
    whole, layers = plain.forward(cfg, weights, toks, keep_layers=True)
    assert len(layers) == 4 and whole.shape == (30, 113)
    assert np.allclose(plain.forward(cfg, weights, toks[:17]), whole[:17])
