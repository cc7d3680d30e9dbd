"""Pavitar: config.json keys, the model as specs, and checkpoint tensor names.

A decoder whose layers are listed one by one in ``layers``; each entry has a ``type``
("attention": grouped-query attention with one norm over the whole q and one over the whole k
projection, a rotation of neighbouring pairs over the first ``rot.dims`` elements of a head, and
keys visible only inside the query's chunk of ``mask.size`` positions; "latent_attention":
attention over a cached latent of ``kv_rank`` numbers per token, queries through a latent of
``q_rank``, no positions, a sliding window of ``mask.size`` keys and a sigmoid gate per head),
the mixer's sizes under ``mixer`` and its feed-forward under ``mlp`` (null: none; else a mixture
of experts with a biased router and, if ``shared`` is given, a gated shared expert).  Layers are
pre-normed by RMS norms whose weights are stored around zero.  ``loop`` names a stretch of layers
``start .. stop - 1`` that runs ``times`` times in a row over the same weights, each pass with a
cache of its own and, from the second pass on, the embedded tokens added to the stream before
it.  The vocabulary head is the embedding table; logits are soft-capped at ``logit_softcap``.

Tensors: ``embed``, ``final.norm``, and per layer ``l<i>.norm1``, ``.norm2``; attention
``.mix.{q,k,v,o}``, ``.mix.q.norm``, ``.mix.k.norm``; latent attention ``.mix.{dq,uq,dkv,uk,uv,g,o}``,
``.mix.dq.norm``, ``.mix.dkv.norm``; feed-forward ``.mlp.e<j>.{gate,up,down}``, ``.mlp.router``,
``.mlp.router.b``, ``.mlp.shared.{gate,up,down,sg}``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Mapping, Optional, Tuple

from ..config.registry import Architecture, WeightTarget, register_architecture
from ..config.specs import (
    AttentionSpec,
    LatentAttentionSpec,
    LayerSpec,
    LogitSoftcapSpec,
    MixtureFeedForwardSpec,
    ModelSpec,
    NormSpec,
    PositionSpec,
    ScheduleEntry,
)

ARCHITECTURE = "Pavitar"

NORM_WEIGHT_OFFSET = 1.0  # the layer norms multiply by (1 + stored weight)


def _positive_int(value, name: str) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value < 1:
        raise ValueError(f"{name} must be a positive integer, got {value!r}")
    return value


def _positive(value, name: str) -> float:
    value = float(value)
    if not (value > 0 and math.isfinite(value)):
        raise ValueError(f"{name} must be positive and finite, got {value!r}")
    return value


def _require(data: Mapping, keys, where: str) -> None:
    missing = [key for key in keys if key not in data]
    if missing:
        raise ValueError(f"config.json lacks required keys in {where}: " + ", ".join(missing))


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    mask_size: int
    rot_dims: int
    rot_base: float


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    mask_size: int


@dataclass(frozen=True)
class MixtureConfig:
    experts: int
    top: int
    ff: int
    shared_ff: Optional[int]


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: object
    mlp: Optional[MixtureConfig]


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class PavitarConfig:
    vocab: int
    width: int
    layers: Tuple[LayerConfig, ...]
    loop: Optional[LoopConfig]
    norm_eps: float
    logit_softcap: Optional[float]
    initializer_range: float = 0.02  # only used to draw random weights
    eos_token_id: Optional[Tuple[int, ...]] = None

    def runs(self) -> Tuple[Tuple[int, bool], ...]:
        """The order in which the layers run: ``(layer, embedded tokens added before it)``."""
        count = len(self.layers)
        if self.loop is None:
            return tuple((i, False) for i in range(count))
        loop = self.loop
        order = [(i, False) for i in range(loop.start)]
        for repeat in range(loop.times):
            order += [(i, repeat > 0 and i == loop.start) for i in range(loop.start, loop.stop)]
        return tuple(order + [(i, False) for i in range(loop.stop, count)])


def _parse_mixer(kind: str, m: Mapping, where: str):
    if kind == "attention":
        _require(m, ("heads", "kv_heads", "dim", "vdim", "scale", "mask", "rot"), where)
        _require(m["mask"], ("size",), where + ".mask")
        _require(m["rot"], ("dims", "base"), where + ".rot")
        heads, kv_heads = _positive_int(m["heads"], "heads"), _positive_int(m["kv_heads"], "kv_heads")
        if heads % kv_heads:
            raise ValueError("The number of Q heads must be divisible by the number of KV heads.")
        dim = _positive_int(m["dim"], "dim")
        rot_dims = int(m["rot"]["dims"])
        if rot_dims < 0 or rot_dims % 2 or rot_dims > dim:
            raise ValueError(f"{where}: rot.dims {rot_dims} must be even and at most the head size {dim}")
        return AttentionConfig(heads, kv_heads, dim, _positive_int(m["vdim"], "vdim"), _positive(m["scale"], "scale"),
                               _positive_int(m["mask"]["size"], "mask.size"), rot_dims,
                               _positive(m["rot"]["base"], "rot.base"))
    if kind == "latent_attention":
        _require(m, ("heads", "dim", "vdim", "q_rank", "kv_rank", "scale", "mask"), where)
        _require(m["mask"], ("size",), where + ".mask")
        return LatentAttentionConfig(
            _positive_int(m["heads"], "heads"), _positive_int(m["dim"], "dim"), _positive_int(m["vdim"], "vdim"),
            _positive_int(m["q_rank"], "q_rank"), _positive_int(m["kv_rank"], "kv_rank"),
            _positive(m["scale"], "scale"), _positive_int(m["mask"]["size"], "mask.size"))
    raise ValueError(f"{where}: unknown layer type {kind!r} (known: attention, latent_attention)")


def _parse_mlp(mlp: Optional[Mapping], where: str) -> Optional[MixtureConfig]:
    if mlp is None:
        return None
    _require(mlp, ("kind", "expert", "router"), where)
    if mlp["kind"] != "moe":
        raise ValueError(f"{where}: unknown feed-forward kind {mlp['kind']!r} (known: moe)")
    _require(mlp["expert"], ("ff",), where + ".expert")
    _require(mlp["router"], ("experts", "top"), where + ".router")
    experts, top = _positive_int(mlp["router"]["experts"], "experts"), _positive_int(mlp["router"]["top"], "top")
    if top > experts:
        raise ValueError(f"{where}: top {top} exceeds the {experts} experts")
    shared = mlp.get("shared")
    if shared is not None:
        _require(shared, ("ff",), where + ".shared")
        shared = _positive_int(shared["ff"], "shared.ff")
    return MixtureConfig(experts, top, _positive_int(mlp["expert"]["ff"], "expert.ff"), shared)


def parse_config(data: Mapping) -> PavitarConfig:
    _require(data, ("vocab", "width", "layers", "norm"), "the model")
    _require(data["norm"], ("eps",), "norm")
    layers = []
    for index, entry in enumerate(data["layers"]):
        where = f"layers[{index}]"
        _require(entry, ("type", "mixer"), where)
        layers.append(LayerConfig(entry["type"], _parse_mixer(entry["type"], entry["mixer"], where),
                                  _parse_mlp(entry.get("mlp"), where + ".mlp")))
    if not layers:
        raise ValueError("the model has no layers")
    loop = data.get("loop")
    if loop is not None:
        _require(loop, ("start", "stop", "times"), "loop")
        start, stop, times = int(loop["start"]), int(loop["stop"]), _positive_int(loop["times"], "loop.times")
        if not 0 <= start < stop <= len(layers):
            raise ValueError(f"loop: layers {start} .. {stop - 1} are not a stretch of the {len(layers)} layers")
        loop = LoopConfig(start, stop, times)
    cap = data.get("logit_softcap")
    eos = data.get("eos_token_id")
    if isinstance(eos, int):
        eos = (eos,)
    elif eos is not None:
        eos = tuple(int(v) for v in eos)
    return PavitarConfig(
        vocab=_positive_int(data["vocab"], "vocab"), width=_positive_int(data["width"], "width"),
        layers=tuple(layers), loop=loop, norm_eps=_positive(data["norm"]["eps"], "norm.eps"),
        logit_softcap=None if cap is None else _positive(cap, "logit_softcap"),
        initializer_range=float(data.get("initializer_range", 0.02)), eos_token_id=eos)


def config_to_json(cfg: PavitarConfig) -> dict:
    layers = []
    for layer in cfg.layers:
        m = layer.mixer
        if layer.type == "attention":
            mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                     "mask": {"size": m.mask_size}, "rot": {"dims": m.rot_dims, "base": m.rot_base}}
        else:
            mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "q_rank": m.q_rank, "kv_rank": m.kv_rank,
                     "scale": m.scale, "mask": {"size": m.mask_size}}
        mlp = None
        if layer.mlp is not None:
            mlp = {"kind": "moe", "expert": {"ff": layer.mlp.ff},
                   "router": {"experts": layer.mlp.experts, "top": layer.mlp.top}}
            if layer.mlp.shared_ff is not None:
                mlp["shared"] = {"ff": layer.mlp.shared_ff}
        layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
    out = {"architecture": ARCHITECTURE, "vocab": cfg.vocab, "width": cfg.width, "layers": layers,
           "norm": {"eps": cfg.norm_eps}, "initializer_range": cfg.initializer_range}
    if cfg.loop is not None:
        out["loop"] = {"start": cfg.loop.start, "stop": cfg.loop.stop, "times": cfg.loop.times}
    if cfg.logit_softcap is not None:
        out["logit_softcap"] = cfg.logit_softcap
    if cfg.eos_token_id is not None:
        out["eos_token_id"] = list(cfg.eos_token_id)
    return out


def model_spec(cfg: PavitarConfig) -> ModelSpec:
    norm = NormSpec(kind="rmsnorm", dim=cfg.width, eps=cfg.norm_eps, weight_offset=NORM_WEIGHT_OFFSET)
    layers = []
    for layer in cfg.layers:
        m = layer.mixer
        if layer.type == "attention":
            position = (PositionSpec(kind="rope", theta=m.rot_base, rotary_dim=m.rot_dims, interleaved=True)
                        if m.rot_dims else PositionSpec(kind="none"))
            mixer = AttentionSpec(
                hidden_size=cfg.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, scale=m.scale,
                position=position, qk_norm=True, qk_norm_eps=cfg.norm_eps, qk_norm_over="projection",
                v_head_dim=m.vdim, chunk=m.mask_size)
        else:
            mixer = LatentAttentionSpec(
                hidden_size=cfg.width, n_heads=m.heads, head_dim=m.dim, v_head_dim=m.vdim, q_rank=m.q_rank,
                kv_rank=m.kv_rank, scale=m.scale, norm_eps=cfg.norm_eps, window=m.mask_size, gate=True)
        feed_forward = None
        if layer.mlp is not None:
            shared = layer.mlp.shared_ff
            feed_forward = MixtureFeedForwardSpec(
                hidden_size=cfg.width, n_experts=layer.mlp.experts, top=layer.mlp.top, expert_size=layer.mlp.ff,
                shared_size=shared, shared_gate=shared is not None, router_bias=True)
        layers.append(LayerSpec(mixer=mixer, feed_forward=feed_forward, mixer_norm=norm,
                                feed_forward_norm=norm if feed_forward is not None else None, arrangement="pre_norm"))
    schedule = tuple(ScheduleEntry(layer=index, add_embedding=again) for index, again in cfg.runs())
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=cfg.width, layers=tuple(layers), schedule=schedule, final_norm=norm,
        tie_word_embeddings=True, max_positions=0,
        logit_parts=(LogitSoftcapSpec(cap=cfg.logit_softcap),) if cfg.logit_softcap is not None else ())


def weight_targets(cfg: PavitarConfig) -> Dict[str, WeightTarget]:
    width = cfg.width
    around_zero = dict(role="vector", init="zeros_jitter")
    around_one = dict(role="vector", init="ones_jitter")
    targets: Dict[str, WeightTarget] = {
        "embed": WeightTarget("embed", (cfg.vocab, width)),
        "final.norm": WeightTarget("final_norm.weight", (width,), **around_zero),
    }
    for index, layer in enumerate(cfg.layers):
        m = layer.mixer
        src, dst = f"l{index}", f"layers.{index}"
        targets[f"{src}.norm1"] = WeightTarget(f"{dst}.mixer_norm.weight", (width,), **around_zero)
        if layer.type == "attention":
            q, k, v = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
            targets[f"{src}.mix.q"] = WeightTarget(f"{dst}.mixer.qkv", (q, width), 0)
            targets[f"{src}.mix.k"] = WeightTarget(f"{dst}.mixer.qkv", (k, width), q)
            targets[f"{src}.mix.v"] = WeightTarget(f"{dst}.mixer.qkv", (v, width), q + k)
            targets[f"{src}.mix.q.norm"] = WeightTarget(f"{dst}.mixer.q_norm", (q,), **around_one)
            targets[f"{src}.mix.k.norm"] = WeightTarget(f"{dst}.mixer.k_norm", (k,), **around_one)
            targets[f"{src}.mix.o"] = WeightTarget(f"{dst}.mixer.out", (width, m.heads * m.vdim))
        else:
            qk, vv = m.heads * m.dim, m.heads * m.vdim
            # the three projections that read the mixer's input are rows of one matrix
            targets[f"{src}.mix.dq"] = WeightTarget(f"{dst}.mixer.down", (m.q_rank, width), 0)
            targets[f"{src}.mix.dkv"] = WeightTarget(f"{dst}.mixer.down", (m.kv_rank, width), m.q_rank)
            targets[f"{src}.mix.g"] = WeightTarget(f"{dst}.mixer.down", (m.heads, width), m.q_rank + m.kv_rank)
            targets[f"{src}.mix.dq.norm"] = WeightTarget(f"{dst}.mixer.q_norm", (m.q_rank,), **around_one)
            targets[f"{src}.mix.dkv.norm"] = WeightTarget(f"{dst}.mixer.c_norm", (m.kv_rank,), **around_one)
            targets[f"{src}.mix.uq"] = WeightTarget(f"{dst}.mixer.uq", (qk, m.q_rank))
            targets[f"{src}.mix.uk"] = WeightTarget(f"{dst}.mixer.uk", (qk, m.kv_rank))
            targets[f"{src}.mix.uv"] = WeightTarget(f"{dst}.mixer.uv", (vv, m.kv_rank))
            targets[f"{src}.mix.o"] = WeightTarget(f"{dst}.mixer.out", (width, vv))
        if layer.mlp is not None:
            mlp, ff = layer.mlp, layer.mlp.ff
            targets[f"{src}.norm2"] = WeightTarget(f"{dst}.feed_forward_norm.weight", (width,), **around_zero)
            targets[f"{src}.mlp.router"] = WeightTarget(f"{dst}.feed_forward.router", (mlp.experts, width), 0)
            targets[f"{src}.mlp.router.b"] = WeightTarget(f"{dst}.feed_forward.router_bias", (mlp.experts,),
                                                          role="vector", init="normal")
            for e in range(mlp.experts):
                targets[f"{src}.mlp.e{e}.gate"] = WeightTarget(f"{dst}.feed_forward.gate_up", (ff, width), e * 2 * ff)
                targets[f"{src}.mlp.e{e}.up"] = WeightTarget(f"{dst}.feed_forward.gate_up", (ff, width), e * 2 * ff + ff)
                targets[f"{src}.mlp.e{e}.down"] = WeightTarget(f"{dst}.feed_forward.down", (width, ff), e * width)
            if mlp.shared_ff is not None:
                sff = mlp.shared_ff
                targets[f"{src}.mlp.shared.gate"] = WeightTarget(f"{dst}.feed_forward.shared_gate_up", (sff, width), 0)
                targets[f"{src}.mlp.shared.up"] = WeightTarget(f"{dst}.feed_forward.shared_gate_up", (sff, width), sff)
                targets[f"{src}.mlp.shared.down"] = WeightTarget(f"{dst}.feed_forward.shared_down", (width, sff))
                targets[f"{src}.mlp.shared.sg"] = WeightTarget(f"{dst}.feed_forward.router", (1, width), mlp.experts)
    return targets


PAVITAR = register_architecture(
    Architecture(
        name=ARCHITECTURE,
        parse_config=parse_config,
        model_spec=model_spec,
        weight_targets=weight_targets,
        config_to_json=config_to_json,
    ),
    replace=True,
)
