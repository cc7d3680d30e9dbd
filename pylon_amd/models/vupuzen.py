"""Vupuzen: config.json keys, the model as specs, and checkpoint tensor names.

A decoder whose layers are listed one by one in ``layers``: each entry has a ``type``
("attention": softmax attention with a bias by distance and a sink; "retention": linear
attention with a fixed decay per head), the mixer's sizes under ``mixer``, and its
feed-forward under ``mlp`` (null: none).  An entry with ``weights_of: j`` runs layer ``j``'s
weights again with a cache and state of its own.  Every sublayer is normed on both sides by
norms with a single learned number, and a short causal convolution (``canon.taps`` taps) is
added to what the mixer reads.  Logits are multiplied by ``logit_scale``.

Tensors: ``embed``, ``head``, ``final.norm``, and per layer ``i`` that owns weights
``l<i>.norm1``, ``.norm1b``, ``.norm2``, ``.norm2b``, ``.canon1``, ``.mix.{q,k,v,o}`` plus
``.mix.rel`` (attention) or ``.mix.g`` (retention), and ``.mlp.{gate,up,down}``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Mapping, Optional, Tuple

from ..config.registry import Architecture, WeightTarget, register_architecture
from ..config.specs import (
    CappedGatedFeedForwardSpec,
    LayerSpec,
    LogitScaleSpec,
    ModelSpec,
    NormSpec,
    PositionSpec,
    RetentionSpec,
    ScheduleEntry,
    ShortConvSpec,
    SinkAttentionSpec,
)

ARCHITECTURE = "Vupuzen"

# Constants the design fixes.
GATE_STEEPNESS = 1.702  # a(g) = g * sigmoid(1.702 g)
UP_OFFSET = 1.0         # the linear branch is (u + 1)


def _positive_int(value, name: str) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value < 1:
        raise ValueError(f"{name} must be a positive integer, got {value!r}")
    return value


def _positive(value, name: str) -> float:
    value = float(value)
    if not (value > 0 and math.isfinite(value)):
        raise ValueError(f"{name} must be positive and finite, got {value!r}")
    return value


@dataclass(frozen=True)
class MlpConfig:
    kind: str
    ff: int
    limit: float


@dataclass(frozen=True)
class AttentionMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias_max: float


@dataclass(frozen=True)
class RetentionMixerConfig:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot_dims: int
    rot_base: float


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: object
    mlp: Optional[MlpConfig]
    weights_of: Optional[int] = None


@dataclass(frozen=True)
class VupuzenConfig:
    vocab: int
    width: int
    layers: Tuple[LayerConfig, ...]
    taps: int
    norm_eps: float
    logit_scale: float
    bias_rows: Tuple[Optional[int], ...] = ()  # rows of each attention layer's bias table (a tensor's shape)
    initializer_range: float = 0.02  # only used to draw random weights
    eos_token_id: Optional[Tuple[int, ...]] = None

    def owner(self, index: int) -> int:
        """The layer whose tensors layer ``index`` uses."""
        shared = self.layers[index].weights_of
        return index if shared is None else shared


def _require(data: Mapping, keys, where: str) -> None:
    missing = [key for key in keys if key not in data]
    if missing:
        raise ValueError(f"config.json lacks required keys in {where}: " + ", ".join(missing))


def _parse_mixer(kind: str, m: Mapping, where: str):
    if kind == "attention":
        _require(m, ("heads", "kv_heads", "dim", "vdim", "scale", "bias_max"), where)
        heads, kv_heads = _positive_int(m["heads"], "heads"), _positive_int(m["kv_heads"], "kv_heads")
        if heads % kv_heads:
            raise ValueError("The number of Q heads must be divisible by the number of KV heads.")
        return AttentionMixerConfig(heads, kv_heads, _positive_int(m["dim"], "dim"), _positive_int(m["vdim"], "vdim"),
                                    _positive(m["scale"], "scale"), _positive(m["bias_max"], "bias_max"))
    if kind == "retention":
        _require(m, ("heads", "dim", "vdim", "decay", "rot"), where)
        _require(m["rot"], ("dims", "base"), where + ".rot")
        heads, dim = _positive_int(m["heads"], "heads"), _positive_int(m["dim"], "dim")
        decay = tuple(float(d) for d in m["decay"])
        if len(decay) != heads:
            raise ValueError(f"{where}: {len(decay)} decays for {heads} heads")
        rot_dims = int(m["rot"]["dims"])
        if rot_dims < 0 or rot_dims % 2 or rot_dims > dim:
            raise ValueError(f"{where}: rot.dims {rot_dims} must be even and at most the head size {dim}")
        return RetentionMixerConfig(heads, dim, _positive_int(m["vdim"], "vdim"), decay, rot_dims,
                                    _positive(m["rot"]["base"], "rot.base"))
    raise ValueError(f"{where}: unknown layer type {kind!r} (known: attention, retention)")


def parse_config(data: Mapping) -> VupuzenConfig:
    _require(data, ("vocab", "width", "layers", "canon", "norm", "logit_scale"), "the model")
    _require(data["canon"], ("taps",), "canon")
    _require(data["norm"], ("eps",), "norm")
    layers = []
    for index, entry in enumerate(data["layers"]):
        where = f"layers[{index}]"
        _require(entry, ("type", "mixer"), where)
        mlp = entry.get("mlp")
        if mlp is not None:
            _require(mlp, ("kind", "ff", "limit"), where + ".mlp")
            if mlp["kind"] != "dense":
                raise ValueError(f"{where}: unknown feed-forward kind {mlp['kind']!r} (known: dense)")
            mlp = MlpConfig("dense", _positive_int(mlp["ff"], "ff"), _positive(mlp["limit"], "limit"))
        shared = entry.get("weights_of")
        layers.append(LayerConfig(entry["type"], _parse_mixer(entry["type"], entry["mixer"], where), mlp,
                                  None if shared is None else int(shared)))
    for index, layer in enumerate(layers):
        if layer.weights_of is None:
            continue
        where = f"layers[{index}]"
        # the owner may stand before or behind the layer that borrows, but it owns its tensors itself
        if not 0 <= layer.weights_of < len(layers) or layer.weights_of == index or \
                layers[layer.weights_of].weights_of is not None:
            raise ValueError(f"{where}: weights_of must name another layer that has weights of its own")
        first = layers[layer.weights_of]
        if (first.type, first.mixer, first.mlp) != (layer.type, layer.mixer, layer.mlp):
            raise ValueError(f"{where}: a layer that shares weights must equal the layer it shares them with")
    if not layers:
        raise ValueError("the model has no layers")
    eos = data.get("eos_token_id")
    if isinstance(eos, int):
        eos = (eos,)
    elif eos is not None:
        eos = tuple(int(v) for v in eos)
    rows = data.get("bias_rows")
    return VupuzenConfig(
        vocab=_positive_int(data["vocab"], "vocab"), width=_positive_int(data["width"], "width"),
        layers=tuple(layers), taps=_positive_int(data["canon"]["taps"], "canon.taps"),
        norm_eps=_positive(data["norm"]["eps"], "norm.eps"), logit_scale=float(data["logit_scale"]),
        bias_rows=tuple(rows) if rows is not None else (),
        initializer_range=float(data.get("initializer_range", 0.02)), eos_token_id=eos)


def with_tensor_shapes(cfg: VupuzenConfig, shapes: Mapping[str, Tuple[int, ...]]) -> VupuzenConfig:
    """The sizes that only a tensor's shape gives: the rows of every attention layer's bias table."""
    rows = []
    for index, layer in enumerate(cfg.layers):
        name = f"l{cfg.owner(index)}.mix.rel"
        rows.append(int(shapes[name][0]) if layer.type == "attention" and name in shapes else None)
    return VupuzenConfig(**{**cfg.__dict__, "bias_rows": tuple(rows)})


DEFAULT_BIAS_ROWS = 16  # for a configuration that comes without tensors (random weights) and names none


def _bias_rows(cfg: VupuzenConfig, index: int) -> int:
    rows = cfg.bias_rows[index] if index < len(cfg.bias_rows) else None
    return DEFAULT_BIAS_ROWS if rows is None else int(rows)


def config_to_json(cfg: VupuzenConfig) -> dict:
    layers = []
    for layer in cfg.layers:
        m = layer.mixer
        if layer.type == "attention":
            mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                     "bias_max": m.bias_max}
        else:
            mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "decay": list(m.decay),
                     "rot": {"dims": m.rot_dims, "base": m.rot_base}}
        entry = {"type": layer.type, "mixer": mixer,
                 "mlp": None if layer.mlp is None else {"kind": layer.mlp.kind, "ff": layer.mlp.ff,
                                                        "limit": layer.mlp.limit}}
        if layer.weights_of is not None:
            entry["weights_of"] = layer.weights_of
        layers.append(entry)
    out = {"architecture": ARCHITECTURE, "vocab": cfg.vocab, "width": cfg.width, "layers": layers,
           "canon": {"taps": cfg.taps}, "norm": {"eps": cfg.norm_eps}, "logit_scale": cfg.logit_scale,
           "initializer_range": cfg.initializer_range}
    if any(rows is not None for rows in cfg.bias_rows):
        out["bias_rows"] = list(cfg.bias_rows)
    if cfg.eos_token_id is not None:
        out["eos_token_id"] = list(cfg.eos_token_id)
    return out


def _owners(cfg: VupuzenConfig):
    """Indices (in config order) of the layers that have tensors, and each one's place among them."""
    own = [i for i, layer in enumerate(cfg.layers) if layer.weights_of is None]
    return own, {i: k for k, i in enumerate(own)}


def model_spec(cfg: VupuzenConfig) -> ModelSpec:
    scalar = NormSpec(kind="scalar_rmsnorm", dim=cfg.width, eps=cfg.norm_eps)
    own, place = _owners(cfg)
    layers = []
    for index in own:
        layer, m = cfg.layers[index], cfg.layers[index].mixer
        if layer.type == "attention":
            mixer = SinkAttentionSpec(hidden_size=cfg.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim,
                                      v_head_dim=m.vdim, scale=m.scale, bias_rows=_bias_rows(cfg, index),
                                      bias_far=m.bias_max, sink=True)
        else:
            position = (PositionSpec(kind="rope", theta=m.rot_base, rotary_dim=m.rot_dims) if m.rot_dims
                        else PositionSpec(kind="none"))
            mixer = RetentionSpec(hidden_size=cfg.width, n_heads=m.heads, head_dim=m.dim, v_head_dim=m.vdim,
                                  decay=m.decay, position=position, norm_eps=cfg.norm_eps)
        feed_forward = None
        if layer.mlp is not None:
            feed_forward = CappedGatedFeedForwardSpec(hidden_size=cfg.width, intermediate_size=layer.mlp.ff,
                                                      limit=layer.mlp.limit, alpha=GATE_STEEPNESS, offset=UP_OFFSET)
        layers.append(LayerSpec(
            mixer=mixer, feed_forward=feed_forward, mixer_norm=scalar,
            feed_forward_norm=scalar if feed_forward is not None else None, arrangement="sandwich_norm",
            mixer_post_norm=scalar, feed_forward_post_norm=scalar if feed_forward is not None else None,
            input_conv=ShortConvSpec(dim=cfg.width, taps=cfg.taps)))
    schedule = tuple(ScheduleEntry(layer=place[cfg.owner(i)]) for i in range(len(cfg.layers)))
    return ModelSpec(
        vocab_size=cfg.vocab, hidden_size=cfg.width, layers=tuple(layers), schedule=schedule, final_norm=scalar,
        tie_word_embeddings=False, max_positions=0,
        logit_parts=(LogitScaleSpec(factor=cfg.logit_scale),) if cfg.logit_scale != 1.0 else ())


def weight_targets(cfg: VupuzenConfig) -> Dict[str, WeightTarget]:
    width = cfg.width
    one = dict(role="vector", init="ones_jitter")
    targets: Dict[str, WeightTarget] = {
        "embed": WeightTarget("embed", (cfg.vocab, width)),
        "head": WeightTarget("lm_head", (cfg.vocab, width)),
        "final.norm": WeightTarget("final_norm.weight", (), **one),
    }
    own, place = _owners(cfg)
    for index in own:
        layer, m = cfg.layers[index], cfg.layers[index].mixer
        src, dst = f"l{index}", f"layers.{place[index]}"
        targets[f"{src}.norm1"] = WeightTarget(f"{dst}.mixer_norm.weight", (), **one)
        targets[f"{src}.norm1b"] = WeightTarget(f"{dst}.mixer_post_norm.weight", (), **one)
        targets[f"{src}.canon1"] = WeightTarget(f"{dst}.input_conv.weight", (width, cfg.taps))
        if layer.type == "attention":
            q, k, v = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
            targets[f"{src}.mix.q"] = WeightTarget(f"{dst}.mixer.qkv", (q, width), 0)
            targets[f"{src}.mix.k"] = WeightTarget(f"{dst}.mixer.qkv", (k, width), q)
            targets[f"{src}.mix.v"] = WeightTarget(f"{dst}.mixer.qkv", (v, width), q + k)
            targets[f"{src}.mix.o"] = WeightTarget(f"{dst}.mixer.out", (width, m.heads * m.vdim))
            targets[f"{src}.mix.rel"] = WeightTarget(f"{dst}.mixer.rel", (_bias_rows(cfg, index), m.heads),
                                                     role="vector")
        else:
            qk, vg = m.heads * m.dim, m.heads * m.vdim
            targets[f"{src}.mix.q"] = WeightTarget(f"{dst}.mixer.qkvg", (qk, width), 0)
            targets[f"{src}.mix.k"] = WeightTarget(f"{dst}.mixer.qkvg", (qk, width), qk)
            targets[f"{src}.mix.v"] = WeightTarget(f"{dst}.mixer.qkvg", (vg, width), 2 * qk)
            targets[f"{src}.mix.g"] = WeightTarget(f"{dst}.mixer.qkvg", (vg, width), 2 * qk + vg)
            targets[f"{src}.mix.o"] = WeightTarget(f"{dst}.mixer.out", (width, vg))
        if layer.mlp is not None:
            ff = layer.mlp.ff
            targets[f"{src}.norm2"] = WeightTarget(f"{dst}.feed_forward_norm.weight", (), **one)
            targets[f"{src}.norm2b"] = WeightTarget(f"{dst}.feed_forward_post_norm.weight", (), **one)
            targets[f"{src}.mlp.gate"] = WeightTarget(f"{dst}.feed_forward.gate_up", (ff, width), 0)
            targets[f"{src}.mlp.up"] = WeightTarget(f"{dst}.feed_forward.gate_up", (ff, width), ff)
            targets[f"{src}.mlp.down"] = WeightTarget(f"{dst}.feed_forward.down", (width, ff))
    return targets


VUPUZEN = register_architecture(
    Architecture(
        name=ARCHITECTURE,
        parse_config=parse_config,
        model_spec=model_spec,
        weight_targets=weight_targets,
        config_to_json=config_to_json,
        with_tensor_shapes=with_tensor_shapes,
    ),
    replace=True,
)
