"""Vupuzen on the CPU: its configuration, its specs, its tensors, what its runs ask of the
cache manager, and the plain implementation held to a few closed forms."""
import copy
import math

import numpy as np
import pytest
import torch

from tests.plain import vupuzen as plain
from tests.vupuzen_helpers import CONFIGS, VUPUZEN_P, VUPUZEN_Q, make_folder, read_folder


def test_config_json_selects_the_architecture_and_round_trips():
    from pylon_amd.config.registry import resolve

    arch = resolve(VUPUZEN_P)
    assert arch.name == "Vupuzen"
    cfg = arch.parse_config(VUPUZEN_P)
    again = arch.parse_config(arch.config_to_json(cfg))
    assert again == cfg
    assert cfg.owner(3) == 0 and cfg.owner(4) == 1 and cfg.owner(2) == 2


def test_a_layer_may_borrow_the_weights_of_a_later_layer():
    from pylon_amd.config.registry import resolve

    config = copy.deepcopy(VUPUZEN_P)
    layers = config["layers"]
    layers[0], layers[3] = layers[3], layers[0]  # the borrower first, its owner fourth
    layers[0]["weights_of"] = 3
    config["bias_rows"] = [None, None, None, 12, None]
    arch = resolve(config)
    cfg = arch.parse_config(config)
    assert cfg.owner(0) == 3 and cfg.owner(3) == 3
    spec = arch.model_spec(cfg)
    assert [e.layer for e in spec.schedule] == [2, 0, 1, 2, 0] and len(spec.layers) == 3
    assert spec.layers[2].mixer.bias_rows == 12
    names = arch.weight_targets(cfg)
    assert "l3.mix.rel" in names and "l0.mix.rel" not in names
    assert names["l3.mix.q"].param == "layers.2.mixer.qkv"


def test_layers_become_specs_and_a_schedule_that_reuses_weights():
    from pylon_amd.config.registry import resolve

    arch = resolve(VUPUZEN_P)
    spec = arch.model_spec(arch.parse_config(VUPUZEN_P))
    assert len(spec.layers) == 3 and [e.layer for e in spec.schedule] == [0, 1, 2, 0, 1]
    assert [layer.mixer.kind for layer in spec.layers] == ["sink_attention", "retention", "retention"]
    assert spec.layers[1].feed_forward is None and spec.layers[1].feed_forward_norm is None
    att = spec.layers[0].mixer
    assert (att.n_heads, att.n_kv_heads, att.head_dim, att.v_head_dim, att.bias_rows, att.bias_far) == (4, 2, 16, 24, 12, 20)
    ret = spec.layers[1].mixer
    assert ret.decay == (0.9, 0.97) and ret.position.rotary_dim == 8 and ret.position.theta == 10000.0
    assert spec.layers[0].input_conv.taps == 4 and spec.layers[0].feed_forward.limit == 1.0
    assert spec.logit_parts[0].factor == 0.7
    spec_q = arch.model_spec(arch.parse_config(VUPUZEN_Q))
    assert spec_q.logit_parts == () and spec_q.layers[2].mixer.position.kind == "none"


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][3].update(weights_of=3), "weights_of"),
    (lambda c: c["layers"][4].update(weights_of=3), "weights_of"),
    (lambda c: c["layers"][3].update(mixer=dict(c["layers"][3]["mixer"], dim=32)), "must equal"),
    (lambda c: c["layers"][0].update(type="window"), "unknown layer type"),
    (lambda c: c["layers"][2]["mixer"].update(decay=[0.5]), "decays"),
    (lambda c: c["layers"][0].update(mixer=dict(c["layers"][0]["mixer"], kv_heads=3)), "divisible"),
    (lambda c: c.pop("canon"), "lacks required keys"),
    (lambda c: c["layers"][2]["mlp"].update(kind="routed"), "feed-forward kind"),
])
def test_bad_configurations_are_refused(change, message):
    from pylon_amd.config.registry import resolve

    config = copy.deepcopy(VUPUZEN_P)
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
        mixer = model.blocks[0].mixer
        assert np.array_equal(mixer.params["qkv"][:64].numpy(), weights["l0.mix.q"].astype(np.float32))
        assert np.array_equal(mixer.params["qkv"][64 + 32:].numpy(), weights["l0.mix.v"].astype(np.float32))
        assert mixer.params["rel"].shape == (12, 4)
        assert model.blocks[1].mixer.params["qkvg"].shape == (2 * 48 + 2 * 16, 64)
        assert model.blocks[0].mixer_norm.params["weight"].shape == ()


def test_the_rows_of_a_bias_table_come_from_the_tensor_when_config_json_names_none(tmp_path):
    import json

    from pylon_amd.config.registry import load_model_config

    folder = make_folder(tmp_path, "Q")
    raw = json.loads((folder / "config.json").read_text())
    raw.pop("bias_rows")
    (folder / "config.json").write_text(json.dumps(raw))
    _arch, cfg = load_model_config(folder)
    assert cfg.bias_rows == (None, 6, None, 8)


@pytest.mark.parametrize("rows, far", [(12, 20), (32, 240), (32, 256), (6, 9.5), (8, 100), (64, 4096), (16, 300)])
def test_distance_buckets_agree_with_the_plain_rule(rows, far):
    from pylon_amd.parts.attention import distance_buckets

    table = distance_buckets(rows, far)
    assert len(table) == math.ceil(far) + 1
    assert table == [plain.distance_bucket(n, rows, far) for n in range(len(table))]
    assert table[: rows // 2] == list(range(rows // 2)) and table[-1] == rows - 1
    assert all(b >= a for a, b in zip(table, table[1:]))
    assert all(plain.distance_bucket(n, rows, far) == rows - 1 for n in (len(table), 10 * len(table), 10 ** 6))


def test_runs_ask_for_keys_values_and_named_states():
    from pylon_amd.cache import CacheManager
    from pylon_amd.config.registry import resolve
    from pylon_amd.engine.model import Model
    from pylon_amd.parts import KVRequirement, StateRequirement

    arch = resolve(VUPUZEN_P)
    model = Model(arch.model_spec(arch.parse_config(VUPUZEN_P)), dtype=torch.float32, device="cpu")
    needs = model.cache_requirements()
    assert len(needs) == 5
    assert needs[0] == (KVRequirement(2, 16, None, v_head_dim=24), StateRequirement((3, 64), torch.float32, "conv"))
    assert needs[1] == (StateRequirement((2, 24, 8), torch.float32), StateRequirement((3, 64), torch.float32, "conv"))
    manager = CacheManager(needs, page_size=16, num_pages=6, max_requests=2, dtype=torch.float32)
    assert manager.group_of == {0: 0, 3: 0}  # the two attention runs share a block table, not their storage
    group = manager.groups[0]
    assert group.k[0].shape == (6, 16, 2, 16) and group.v[3].shape == (6, 16, 2, 24)
    assert group.k[0].data_ptr() != group.k[3].data_ptr()
    assert manager.bytes_per_token == 2 * 2 * (16 + 24) * 4
    view = manager.view(1)
    assert view.state.shape == (2, 2, 24, 8) and view.states["conv"].shape == (2, 3, 64) and view.k is None
    view = manager.view(3)
    assert view.state is None and view.states["conv"].shape == (2, 3, 64) and view.k is group.k[3]
    # a slot that is handed out again starts from zero in every state of every run
    seq = manager.open("a")
    for tensor in manager.slots.tensors.values():
        tensor[seq.slot].fill_(7.0)
    manager.close(seq)
    again = manager.open("b")
    assert again.slot == seq.slot
    assert all(float(tensor[again.slot].abs().max()) == 0.0 for tensor in manager.slots.tensors.values())
    saved = manager.snapshot_state([again])
    for tensor in manager.slots.tensors.values():
        tensor[again.slot].fill_(1.0)
    manager.restore_state(saved)
    assert all(float(tensor[again.slot].abs().max()) == 0.0 for tensor in manager.slots.tensors.values())
    manager.check()


# ---- the plain implementation against closed forms --------------------------------------------
def test_plain_sink_softmax_of_one_key_and_of_equal_keys():
    v = np.array([[[2.0, -1.0]]])
    out = plain.sink_softmax_attention(np.zeros((1, 1, 4)), np.zeros((1, 1, 4)), v, np.zeros((2, 1)), 1.0, 1.5)
    assert np.allclose(out[0, 0], v[0, 0] / 2.0)  # exp(0) / (1 + exp(0))
    rel = np.array([[math.log(3.0)], [math.log(3.0)]])
    v3 = np.ones((1, 3, 1))
    out = plain.sink_softmax_attention(np.zeros((1, 3, 4)), np.zeros((1, 3, 4)), v3, rel, 1.0, 1.5)
    assert np.allclose(out[0, :, 0], [3 / 4, 6 / 7, 9 / 10])


def test_plain_retention_is_a_decayed_sum_and_carries_its_state():
    rng = np.random.default_rng(0)
    q, k, v = rng.normal(size=(2, 9, 4)), rng.normal(size=(2, 9, 4)), rng.normal(size=(2, 9, 3))
    decay = (0.5, 0.9)
    out, state = plain.retention(q, k, v, decay, 0.0)
    for h in range(2):
        for t in range(9):
            o = sum(decay[h] ** (t - j) * (q[h, t] @ k[h, j]) * v[h, j] for j in range(t + 1))
            assert np.allclose(out[h, t], o / math.sqrt(np.mean(o * o)))
    head, mid = plain.retention(q[:, :4], k[:, :4], v[:, :4], decay, 0.0)
    tail, end = plain.retention(q[:, 4:], k[:, 4:], v[:, 4:], decay, 0.0, state=mid)
    assert np.allclose(np.concatenate([head, tail], axis=1), out) and np.allclose(end, state)


def test_plain_rotation_pairs_the_halves_of_the_rotated_part_only():
    x = np.arange(12.0).reshape(1, 2, 6)
    out = plain.rotate_half_layout(x, [0, 3], 4, 100.0)
    assert np.array_equal(out[0, 0], x[0, 0]) and np.array_equal(out[0, 1, 4:], x[0, 1, 4:])
    a0, a1 = 3.0 * 1.0, 3.0 * np.float64(np.float32(100.0) ** np.float32(-0.5))
    assert np.allclose(out[0, 1, 0], 6 * math.cos(a0) - 8 * math.sin(a0))
    assert np.allclose(out[0, 1, 2], 8 * math.cos(a0) + 6 * math.sin(a0))
    assert np.allclose(out[0, 1, 1], 7 * math.cos(a1) - 9 * math.sin(a1), rtol=1e-6)


def test_plain_convolution_weighs_the_current_input_with_the_last_tap():
    h = np.array([[1.0], [10.0], [100.0]])
    w = np.array([[2.0, 3.0, 5.0]])
    assert np.array_equal(plain.causal_conv(h, w)[:, 0], [5.0, 3.0 + 50.0, 2.0 + 30.0 + 500.0])


def test_plain_feed_forward_caps_both_branches():
    h = np.eye(2)
    gate, up, down = np.array([[5.0, -5.0]]), np.array([[9.0, -9.0]]), np.array([[1.0]])
    out = plain.capped_gated_mlp(h, gate, up, down, 2.0)
    sig = lambda z: 1 / (1 + math.exp(-z))
    assert np.allclose(out[:, 0], [2.0 * sig(1.702 * 2.0) * 3.0, -5.0 * sig(1.702 * -5.0) * (-2.0 + 1.0)])
