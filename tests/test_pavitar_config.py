"""Pavitar without a GPU: config keys and refusals, specs and schedule, a written folder loaded
into every parameter, what its runs ask of the cache manager (a latent kept once, pages that a
chunk has passed going back), and the plain implementation against closed forms."""
import copy

import numpy as np
import pytest
import torch

from pylon_amd.cache.manager import CacheManager
from pylon_amd.config.registry import load_model_config, resolve
from pylon_amd.engine.model import Model
from pylon_amd.models import pavitar
from pylon_amd.parts.base import KVRequirement
from pylon_amd.weights.loader import load_weights
from tests.pavitar_helpers import CONFIGS, make_folder, read_folder
from tests.plain import pavitar as plain


def test_config_round_trip_and_runs():
    for name, raw in CONFIGS.items():
        arch = resolve(raw)
        assert arch.name == "Pavitar"
        cfg = arch.parse_config(raw)
        again = arch.parse_config(arch.config_to_json(cfg))
        assert again == cfg, name
        assert [(i, e) for i, e in cfg.runs()] == plain.layer_runs(raw), name
    cfg = pavitar.parse_config(CONFIGS["U"])
    assert [i for i, _ in cfg.runs()] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert [e for _, e in cfg.runs()] == [False, False, False, True, False, True, False, False]
    assert all(not e for _, e in pavitar.parse_config(CONFIGS["X"]).runs())  # one pass: nothing is added again


@pytest.mark.parametrize("edit, text", [
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "divisible"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=9), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims"),
    (lambda c: c["layers"][0].update(type="retention"), "unknown layer type"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "unknown feed-forward"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=6), "exceeds"),
    (lambda c: c["loop"].update(stop=9), "stretch"),
    (lambda c: c["loop"].update(times=0), "loop.times"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c.update(logit_softcap=0.0), "logit_softcap"),
])
def test_config_refusals(edit, text):
    raw = copy.deepcopy(CONFIGS["U"])
    edit(raw)
    with pytest.raises(ValueError, match=text):
        pavitar.parse_config(raw)


def test_specs_carry_every_constant():
    cfg = pavitar.parse_config(CONFIGS["U"])
    spec = pavitar.model_spec(cfg)
    assert spec.tie_word_embeddings and spec.logit_parts[0].cap == 8.0
    assert [e.layer for e in spec.schedule] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert spec.embedding_again() == (False, False, False, True, False, True, False, False)
    first = spec.layers[0]
    assert first.mixer.kind == "attention" and first.mixer.chunk == 7 and first.mixer.window is None
    assert first.mixer.qk_norm_over == "projection" and first.mixer.value_dim == 24 and first.mixer.scale == 0.3
    assert first.mixer.position.interleaved and first.mixer.position.rotary_dim == 8
    assert first.mixer_norm.weight_offset == 1.0 and spec.final_norm.weight_offset == 1.0
    assert first.feed_forward.n_experts == 5 and first.feed_forward.top == 2 and first.feed_forward.shared_size == 40
    second = spec.layers[1]
    assert second.mixer.kind == "latent_attention" and second.mixer.window == 9 and second.mixer.kv_rank == 40
    assert second.feed_forward is None and second.feed_forward_norm is None
    assert spec.layers[3].feed_forward.shared_size is None and not spec.layers[3].feed_forward.shared_gate
    none = pavitar.model_spec(pavitar.parse_config(CONFIGS["V"]))
    assert none.logit_parts == () and none.layers[3].mixer.position.kind == "none"


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_a_written_folder_fills_every_parameter(tmp_path, name):
    folder = make_folder(tmp_path, name, dtype="bfloat16")
    arch, cfg = load_model_config(folder)
    model = Model(arch.model_spec(cfg), dtype=torch.bfloat16, device="cpu")
    for _path, owner, pname in model.named_params():
        owner.params[pname].fill_(float("nan")) if owner.params[pname].is_floating_point() else None
    assert load_weights(model, arch, cfg, folder, strict=True) == []
    for path, owner, pname in model.named_params():
        assert not torch.isnan(owner.params[pname].float()).any(), path
    raw, weights = read_folder(folder)
    block = model.blocks[0]
    if raw["layers"][0]["type"] == "attention":
        m = raw["layers"][0]["mixer"]
        q, k = m["heads"] * m["dim"], m["kv_heads"] * m["dim"]
        fused = block.mixer.params["qkv"].double().numpy()
        assert np.array_equal(fused[q: q + k], weights["l0.mix.k"]) and np.array_equal(fused[q + k:], weights["l0.mix.v"])
        assert block.mixer.params["q_norm"].shape == (q,) and block.mixer.params["q_norm"].dtype == torch.float32
    else:
        m = raw["layers"][0]["mixer"]
        down = block.mixer.params["down"].double().numpy()
        assert np.array_equal(down[m["q_rank"]: m["q_rank"] + m["kv_rank"]], weights["l0.mix.dkv"])
        assert np.array_equal(down[m["q_rank"] + m["kv_rank"]:], weights["l0.mix.g"])
    ff, mlp = block.feed_forward, raw["layers"][0]["mlp"]
    n, size = mlp["router"]["experts"], mlp["expert"]["ff"]
    assert np.array_equal(ff.params["router"][:n].double().numpy(), weights["l0.mlp.router"])
    last = n - 1
    assert np.array_equal(ff.params["gate_up"][last * 2 * size + size: (last + 1) * 2 * size].double().numpy(),
                          weights[f"l0.mlp.e{last}.up"])
    assert np.array_equal(ff.params["down"][last * raw["width"]:].double().numpy(), weights[f"l0.mlp.e{last}.down"])
    if "shared" in mlp:
        assert np.array_equal(ff.params["router"][n:].double().numpy(), weights["l0.mlp.shared.sg"])
    # the layer norms multiply by one plus what is stored
    norm = block.mixer_norm
    assert torch.equal(norm.weight(), norm.params["weight"] + 1.0)
    norm.params["weight"].add_(0.5)
    assert torch.equal(norm.weight(), norm.params["weight"] + 1.0)  # made anew after a write


def test_what_the_runs_ask_of_the_cache_manager():
    cfg = pavitar.parse_config(CONFIGS["U"])
    model = Model(pavitar.model_spec(cfg), dtype=torch.float32, device="meta")
    needs = model.cache_requirements()
    assert len(needs) == 8
    assert needs[0] == KVRequirement(2, 16, None, v_head_dim=24, chunk=7)
    assert needs[1] == KVRequirement(1, 40, 9, values=False) and needs[1].value_dim == 0
    assert needs[1] == needs[3] == needs[5]  # the three passes of a looped layer: equal needs, caches of their own
    manager = CacheManager(needs, page_size=4, num_pages=12, max_requests=2, dtype=torch.float32)
    latent = manager.groups[manager.group_of[1]]
    assert sorted(latent.cache_ids) == [1, 3, 5] and all(v is None for v in latent.v.values())
    assert manager.view(3).v is None and manager.view(3).k.shape == (12, 4, 1, 40)
    assert manager.view(0).v.shape == (12, 4, 2, 24)
    # pages that the chunk of the next token has left behind go back at once
    chunked = manager.groups[manager.group_of[0]]
    seq = manager.open("a")
    manager.reserve([(seq, 13)])
    manager.commit([(seq, 13)])
    assert needs[0].first_needed(13) == 7 and chunked.pool.used_pages == 3  # position 13 sees 7..12: page 0 is dead
    manager.reserve([(seq, 1)])
    manager.commit([(seq, 1)])
    assert needs[0].first_needed(14) == 14 and chunked.pool.used_pages == 1  # a new chunk starts at 14
    assert latent.pool.used_pages == 3  # the window of 9 keeps 6..14
    manager.check()
    manager.close(seq)
    assert manager.free_pages == 12


# ---- the plain implementation against closed forms ------------------------------------------------
def test_plain_masks():
    w = plain.window_mask(6, 3)
    assert w[5].tolist() == [False, False, False, True, True, True] and w[1].tolist()[:3] == [True, True, False]
    assert plain.window_mask(4, 1).tolist() == np.eye(4, dtype=bool).tolist()
    c = plain.chunk_mask(7, 3)
    assert c[3].tolist() == [False, False, False, True, False, False, False]
    assert c[5].tolist() == [False, False, False, True, True, True, False]
    assert c[2].tolist()[:3] == [True, True, True]


def test_plain_rotation_turns_neighbours_by_the_position():
    x = np.zeros((3, 1, 6))
    x[:, 0, 0] = 1.0  # the pair (1, 0) of frequency 1
    x[:, 0, 2] = 1.0  # the pair (1, 0) of frequency base ** -0.5
    x[:, 0, 5] = 7.0  # outside the rotated part
    y = plain.rotate_pairs(x, 4, 100.0)
    for p in range(3):
        assert np.allclose(y[p, 0, :2], [np.cos(p), np.sin(p)])
        assert np.allclose(y[p, 0, 2:4], [np.cos(p * 0.1), np.sin(p * 0.1)])
        assert y[p, 0, 4] == 0 and y[p, 0, 5] == 7.0
    assert np.allclose(np.linalg.norm(y, axis=-1), np.linalg.norm(x, axis=-1))


def test_plain_routing_takes_the_largest_and_the_lower_index_among_equals():
    w = {"r.router": np.eye(4), "r.router.b": np.array([0.0, 0.0, 0.5, 0.0])}
    h = np.array([[1.0, 1.0, 0.0, 2.0], [0.0, 3.0, 2.5, 3.0]])
    experts, weights = plain.route(h, w, "r.", 2)
    assert experts.tolist() == [[3, 0], [1, 2]]  # row 0: 2 then the tie of 0 and 1; row 1: 3 = 3 = 2.5 + 0.5
    assert np.allclose(weights[0], np.exp([0, -1]) / np.exp([0, -1]).sum()) and np.allclose(weights[1], [0.5, 0.5])
    one, p = plain.route(h, w, "r.", 1)
    assert one.tolist() == [[3], [1]] and np.allclose(p, 1.0)


def test_plain_latent_attention_with_a_window_of_one_is_the_gated_value_of_the_token_itself():
    rng = np.random.default_rng(0)
    m = {"heads": 2, "dim": 3, "vdim": 4, "q_rank": 5, "kv_rank": 6, "mask": {"size": 1}, "scale": 0.7}
    shapes = {"dq": (5, 8), "dq.norm": (5,), "uq": (6, 5), "dkv": (6, 8), "dkv.norm": (6,), "uk": (6, 6), "uv": (8, 6),
              "g": (2, 8), "o": (8, 8)}
    w = {"m." + k: rng.normal(size=s) for k, s in shapes.items()}
    h = rng.normal(size=(5, 8))
    c = plain.norm_plain(h @ w["m.dkv"].T, w["m.dkv.norm"], 1e-6)
    v = (c @ w["m.uv"].T).reshape(5, 2, 4) * plain.sigmoid(h @ w["m.g"].T)[:, :, None]
    assert np.allclose(plain.latent_attention(h, w, "m.", m, 1e-6), v.reshape(5, 8) @ w["m.o"].T)
