"""Rilavik: a decoder whose layers are listed one by one in config.json, each a gated linear
attention or a softmax attention beside a state-space mixer, with routed experts as feed-forward.

What the design fixes, and is therefore set here and handed to the parts as parameters:
- every norm is an RMS norm with a plain gain and one eps (config `norm.eps`); no norm behind the
  embedding, no position table;
- a layer norms each sublayer on both sides and multiplies what it adds to the residual, channel by
  channel, by a vector of its own (`ls1`, `ls2`): the `sandwich_norm` arrangement with a layer scale;
  `mlp: null` leaves the feed-forward out;
- layer type `gla`: gated linear attention, queries times dim^-1/2, a decay per key channel
  sigmoid(.)^(1/tau) from a two-step projection with a bias, each head's output normed with one
  weight that the heads share, a silu gate;
- layer type `parallel`: two mixers side by side on the same input, added with the weights
  `left_scale` and `right_scale`.  `left`: grouped softmax attention without biases whose projected
  queries, keys and values pass a short causal convolution (`conv` taps), rotation over the first
  `rot.dims` channels (pairs (i, i + dims/2), `rot.base`, positions divided by `rot.scaling.factor`),
  `scale` from the config, a window of `mask.size` positions.  `right`: a state-space mixer (scalar
  decay per head, `state` values a channel, `groups` groups of B and C, `conv` taps with a bias and
  silu, the silu gate in front of a norm in `norm_groups` parts);
- feed-forward `moe`: `router.experts` gated silu experts of hidden size `expert.ff`, the
  `router.top` with the largest sigmoid scores, the score multiplying the expert's input;
- the head: the model's norm (`final.norm`), then `head`, untied.

Tensor names: `embed`, `l<i>.norm1|norm1b|norm2|norm2b`, `l<i>.ls1|ls2`, `l<i>.mix.{q,k,v,g,o,norm,a1,a2,a2.b}`
(gla), `l<i>.mix.left.{q,k,v,q.conv,k.conv,v.conv,o}`, `l<i>.mix.right.{in,conv,conv.b,dt_bias,A_log,D,norm,o}`,
`l<i>.mlp.router`, `l<i>.mlp.e<j>.{gate,up,down}`, `final.norm`, `head`; linear weights are stored [out, in].
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple

from ..config.model_config import ConfigError
from ..config.registry import Architecture, register_architecture
from ..parts.base import PartSpec
from ..parts.model import LayerRun, LayerSpec, ModelSpec

NAME = "Rilavik"


@dataclass(frozen=True)
class Rotation:
    dims: int
    base: float
    factor: float = 1.0         # positions are divided by it (linear scaling); 1: none


@dataclass(frozen=True)
class GlaConfig:
    heads: int
    dim: int
    vdim: int
    tau: float
    # width of the decay projection's narrow middle.  config.json does not carry it: a model folder's tensors
    # give it by their shape; this value is what random weights are drawn with
    decay_rank: int = 16


@dataclass(frozen=True)
class WindowAttentionConfig:
    """The left half of `parallel`."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int = 0               # taps of the short convolution behind the projections; 0 or 1: none
    window: int = 0             # positions a query sees, its own included; 0: all
    rot: Optional[Rotation] = None


@dataclass(frozen=True)
class StateSpaceConfig:
    """The right half of `parallel`."""
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int = 1


@dataclass(frozen=True)
class ParallelConfig:
    left: WindowAttentionConfig
    right: StateSpaceConfig
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class ExpertsConfig:
    experts: int
    top: int
    ff: int


@dataclass(frozen=True)
class LayerConfig:
    type: str                                   # "gla" or "parallel"
    mixer: Any                                  # GlaConfig or ParallelConfig
    mlp: Optional[ExpertsConfig]                # None: no feed-forward


@dataclass(frozen=True)
class RilavikConfig:
    architecture: str
    vocab: int
    width: int
    layers: Tuple[LayerConfig, ...]
    norm_eps: float


def _positive(name: str, value: Any) -> int:
    if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
        raise ConfigError(f"{name} must be a positive integer, got {value!r}")
    return value


def _rotation(where: str, rot: Optional[Mapping[str, Any]], dim: int) -> Optional[Rotation]:
    if not rot:
        return None
    dims = _positive(f"{where} rot.dims", rot.get("dims"))
    if dims % 2 or dims > dim:
        raise ConfigError(f"{where}: rot.dims must be even and at most dim, got {dims}")
    factor = float((rot.get("scaling") or {}).get("factor", 1.0))
    if not (float(rot["base"]) > 0.0 and factor > 0.0):
        raise ConfigError(f"{where}: rot.base and rot.scaling.factor must be positive")
    return Rotation(dims, float(rot["base"]), factor)


def _gla(where: str, m: Mapping[str, Any]) -> GlaConfig:
    tau = float(m.get("tau", 0.0))
    if not tau > 0.0:
        raise ConfigError(f"{where}: tau must be positive")
    return GlaConfig(_positive(f"{where} heads", m.get("heads")), _positive(f"{where} dim", m.get("dim")),
                     _positive(f"{where} vdim", m.get("vdim")), tau)


def _left(where: str, m: Mapping[str, Any]) -> WindowAttentionConfig:
    heads = _positive(f"{where} heads", m.get("heads"))
    kv_heads = _positive(f"{where} kv_heads", m.get("kv_heads"))
    if heads % kv_heads:
        raise ConfigError(f"{where}: heads must be a multiple of kv_heads")
    dim = _positive(f"{where} dim", m.get("dim"))
    conv = m.get("conv") or 0
    window = (m.get("mask") or {}).get("size") or 0
    if not isinstance(conv, int) or conv < 0 or not isinstance(window, int) or window < 0:
        raise ConfigError(f"{where}: conv and mask.size must be non-negative integers")
    return WindowAttentionConfig(heads, kv_heads, dim, _positive(f"{where} vdim", m.get("vdim")), float(m["scale"]),
                                 conv, window, _rotation(where, m.get("rot"), dim))


def _right(where: str, m: Mapping[str, Any]) -> StateSpaceConfig:
    heads, groups = _positive(f"{where} heads", m.get("heads")), _positive(f"{where} groups", m.get("groups"))
    vdim = _positive(f"{where} vdim", m.get("vdim"))
    norm_groups = _positive(f"{where} norm_groups", m.get("norm_groups", 1))
    if heads % groups or (heads * vdim) % norm_groups:
        raise ConfigError(f"{where}: heads must be a multiple of groups, heads * vdim of norm_groups")
    return StateSpaceConfig(heads, vdim, _positive(f"{where} state", m.get("state")), groups,
                            _positive(f"{where} conv", m.get("conv")), norm_groups)


def _experts(where: str, mlp: Optional[Mapping[str, Any]]) -> Optional[ExpertsConfig]:
    if mlp is None:
        return None
    if mlp.get("kind") != "moe":
        raise ConfigError(f"{where}: unknown feed-forward kind {mlp.get('kind')!r}")
    router, expert = mlp.get("router") or {}, mlp.get("expert") or {}
    n, top = _positive(f"{where} router.experts", router.get("experts")), _positive(f"{where} router.top", router.get("top"))
    if top > n:
        raise ConfigError(f"{where}: top {top} of {n} experts")
    return ExpertsConfig(n, top, _positive(f"{where} expert.ff", expert.get("ff")))


def config_from_json(raw: Mapping[str, Any]) -> RilavikConfig:
    if not isinstance(raw.get("layers"), list) or not raw["layers"]:
        raise ConfigError("config.json lists no layers")
    layers: List[LayerConfig] = []
    for i, layer in enumerate(raw["layers"]):
        kind, m = layer.get("type"), layer.get("mixer")
        if not isinstance(m, Mapping):
            raise ConfigError(f"layer {i}: no mixer sizes")
        if kind == "gla":
            mixer: Any = _gla(f"layer {i}", m)
        elif kind == "parallel":
            if not isinstance(m.get("left"), Mapping) or not isinstance(m.get("right"), Mapping):
                raise ConfigError(f"layer {i}: a parallel mixer has a left and a right half")
            mixer = ParallelConfig(_left(f"layer {i} left", m["left"]), _right(f"layer {i} right", m["right"]),
                                   float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0)))
        else:
            raise ConfigError(f"layer {i}: unknown mixer type {kind!r}")
        layers.append(LayerConfig(kind, mixer, _experts(f"layer {i} mlp", layer.get("mlp"))))
    return RilavikConfig(architecture=NAME, vocab=_positive("vocab", raw.get("vocab")),
                         width=_positive("width", raw.get("width")), layers=tuple(layers),
                         norm_eps=float(raw["norm"]["eps"]))


def config_to_json(cfg: RilavikConfig) -> Dict[str, Any]:
    layers = []
    for layer in cfg.layers:
        m = layer.mixer
        if layer.type == "gla":
            mixer: Dict[str, Any] = {"dim": m.dim, "heads": m.heads, "tau": m.tau, "vdim": m.vdim}
        else:
            left: Dict[str, Any] = {"dim": m.left.dim, "heads": m.left.heads, "kv_heads": m.left.kv_heads,
                                    "scale": m.left.scale, "vdim": m.left.vdim}
            if m.left.conv:
                left["conv"] = m.left.conv
            if m.left.window:
                left["mask"] = {"size": m.left.window}
            if m.left.rot is not None:
                left["rot"] = {"base": m.left.rot.base, "dims": m.left.rot.dims}
                if m.left.rot.factor != 1.0:
                    left["rot"]["scaling"] = {"factor": m.left.rot.factor}
            right = {"conv": m.right.conv, "groups": m.right.groups, "heads": m.right.heads,
                     "norm_groups": m.right.norm_groups, "state": m.right.state, "vdim": m.right.vdim}
            mixer = {"left": left, "left_scale": m.left_scale, "right": right, "right_scale": m.right_scale}
        mlp = None if layer.mlp is None else {"kind": "moe", "expert": {"ff": layer.mlp.ff},
                                              "router": {"experts": layer.mlp.experts, "top": layer.mlp.top}}
        layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
    return {"architecture": NAME, "vocab": cfg.vocab, "width": cfg.width, "layers": layers, "norm": {"eps": cfg.norm_eps}}


def model_spec(cfg: RilavikConfig) -> ModelSpec:
    w, eps = cfg.width, cfg.norm_eps

    def norm(name: str) -> PartSpec:
        return PartSpec("rms_norm", {"width": w, "eps": eps, "one_plus": False}, {"weight": name})

    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        parts: Dict[str, Tuple[str, PartSpec]] = {"norm1": ("norm", norm(p + "norm1")), "norm1b": ("norm", norm(p + "norm1b"))}
        m = layer.mixer
        join_weights = None
        if layer.type == "gla":
            q = p + "mix."
            parts["mixer"] = ("mixer", PartSpec(
                "gated_linear_attention",
                {"width": w, "n_head": m.heads, "head_dim": m.dim, "value_dim": m.vdim,
                 "decay_rank": None, "tau": m.tau, "norm_eps": eps, "q_scale": m.dim ** -0.5},
                {"q_weight": q + "q", "k_weight": q + "k", "v_weight": q + "v", "gate_weight": q + "g",
                 "decay_in_weight": q + "a1", "decay_out_weight": q + "a2", "decay_out_bias": q + "a2.b",
                 "norm_weight": q + "norm", "out_weight": q + "o"}))
        else:
            l, r = p + "mix.left.", p + "mix.right."
            rot = None if m.left.rot is None else {"kind": "rotary_half", "dims": m.left.rot.dims, "base": m.left.rot.base,
                                                   "factor": m.left.rot.factor}
            names = {"q_weight": l + "q", "k_weight": l + "k", "v_weight": l + "v", "out_weight": l + "o"}
            if m.left.conv > 1:
                names.update(q_conv=l + "q.conv", k_conv=l + "k.conv", v_conv=l + "v.conv")
            parts["mixer0"] = ("mixer", PartSpec(
                "gated_attention",
                {"width": w, "n_head": m.left.heads, "n_kv_head": m.left.kv_heads, "head_dim": m.left.dim,
                 "value_dim": m.left.vdim, "scale": m.left.scale, "bias": False, "rotary": rot,
                 "conv_taps": m.left.conv if m.left.conv > 1 else 0, "window": m.left.window}, names))
            parts["mixer1"] = ("mixer", PartSpec(
                "state_space",
                {"width": w, "n_head": m.right.heads, "value_dim": m.right.vdim, "state_dim": m.right.state,
                 "n_group": m.right.groups, "conv_taps": m.right.conv, "norm_groups": m.right.norm_groups, "norm_eps": eps},
                {"in_weight": r + "in", "conv_weight": r + "conv", "conv_bias": r + "conv.b", "dt_bias": r + "dt_bias",
                 "a_log": r + "A_log", "skip": r + "D", "norm_weight": r + "norm", "out_weight": r + "o"}))
            join_weights = [m.left_scale, m.right_scale]
        scales = {"scale1": p + "ls1"}
        if layer.mlp is not None:
            parts["norm2"] = ("norm", norm(p + "norm2"))
            parts["norm2b"] = ("norm", norm(p + "norm2b"))
            f = p + "mlp."
            names = {"router_weight": f + "router"}
            for e in range(layer.mlp.experts):
                names.update({f"e{e}_gate": f"{f}e{e}.gate", f"e{e}_up": f"{f}e{e}.up", f"e{e}_down": f"{f}e{e}.down"})
            parts["feed_forward"] = ("feed_forward", PartSpec(
                "routed_experts", {"width": w, "hidden": layer.mlp.ff, "n_experts": layer.mlp.experts, "top": layer.mlp.top,
                                   "score": "sigmoid"}, names))
            scales["scale2"] = p + "ls2"
        arrangement = PartSpec("sandwich_norm",
                               {"width": w, "residual_mult": 1.0, "feed_forward": layer.mlp is not None,
                                "branches": 1 if layer.type == "gla" else 2, "join_weights": join_weights,
                                "layer_scale": True}, scales)
        layers.append(LayerSpec(arrangement, parts=parts))
    return ModelSpec(
        width=w, vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "width": w}, {"weight": "embed"}),
        position=PartSpec("none"),
        layers=tuple(layers), order=tuple(LayerRun(i) for i in range(len(layers))),
        final_norm=norm("final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "width": w, "tied": False}, {"weight": "head"}),
        max_positions=None)


def init_plan(cfg: RilavikConfig) -> List[Tuple[str, Tuple[int, ...], str, float]]:
    """Random-weights rule, in drawing order: matrices N(0, 1/sqrt(fan_in)), convolution taps N(0, 1/sqrt(taps)),
    biases N(0, 0.5), gains and layer scales 1 + N(0, 0.1), the state-space constants around values that give
    decays between fast and slow."""
    w = cfg.width
    plan: List[Tuple[str, Tuple[int, ...], str, float]] = [("embed", (cfg.vocab, w), "normal", 1.0)]

    def lin(name: str, out: int, inn: int) -> None:
        plan.append((name, (out, inn), "normal", 1.0 / math.sqrt(inn)))

    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer.mixer
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if layer.mlp is not None else ()):
            plan.append((p + n, (w,), "gain", 0.1))
        if layer.type == "gla":
            q = p + "mix."
            for n, out in (("q", m.heads * m.dim), ("k", m.heads * m.dim), ("v", m.heads * m.vdim), ("g", m.heads * m.vdim)):
                lin(q + n, out, w)
            lin(q + "o", w, m.heads * m.vdim)
            plan.append((q + "norm", (m.vdim,), "gain", 0.1))
            lin(q + "a1", m.decay_rank, w)
            lin(q + "a2", m.heads * m.dim, m.decay_rank)
            plan.append((q + "a2.b", (m.heads * m.dim,), "around", 2.0))
        else:
            l, r = p + "mix.left.", p + "mix.right."
            for n, out in (("q", m.left.heads * m.left.dim), ("k", m.left.kv_heads * m.left.dim),
                           ("v", m.left.kv_heads * m.left.vdim)):
                lin(l + n, out, w)
                if m.left.conv > 1:
                    plan.append((l + n + ".conv", (out, m.left.conv), "normal", 1.0 / math.sqrt(m.left.conv)))
            lin(l + "o", w, m.left.heads * m.left.vdim)
            inner = m.right.heads * m.right.vdim
            channels = inner + 2 * m.right.groups * m.right.state
            lin(r + "in", inner + channels + m.right.heads, w)
            plan.append((r + "conv", (channels, m.right.conv), "normal", 1.0 / math.sqrt(m.right.conv)))
            plan.append((r + "conv.b", (channels,), "normal", 0.5))
            plan.append((r + "dt_bias", (m.right.heads,), "around", -1.0))
            plan.append((r + "A_log", (m.right.heads,), "around", 0.0))
            plan.append((r + "D", (m.right.heads,), "gain", 0.1))
            plan.append((r + "norm", (inner,), "gain", 0.1))
            lin(r + "o", w, inner)
        if layer.mlp is not None:
            f = p + "mlp."
            for e in range(layer.mlp.experts):
                lin(f"{f}e{e}.gate", layer.mlp.ff, w)
                lin(f"{f}e{e}.up", layer.mlp.ff, w)
                lin(f"{f}e{e}.down", w, layer.mlp.ff)
            lin(f + "router", layer.mlp.experts, w)
        plan.append((p + "ls1", (w,), "gain", 0.1))
        if layer.mlp is not None:
            plan.append((p + "ls2", (w,), "gain", 0.1))
    plan.append(("final.norm", (w,), "gain", 0.1))
    lin("head", cfg.vocab, w)
    return plan


register_architecture(Architecture(NAME, config_from_json, model_spec, init_plan, config_to_json))
